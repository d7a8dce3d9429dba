// Fused learned-optimizer step for MI355X (gfx950): the C ABI of include/pylo_mi355.h.
//
// Pipeline of one ELO-CELO2 step over all tensors of a plan (6 launches, no host sync):
//   k_p0 (pass 0)   row / column sums of g^2 per tile, sum g^2 and clamp flag per block     4 B/elem
//   k_gnorm         global gradient norm, clamp flag
//   k_p0 (pass 1)   exits at once unless some |g| exceeded the clamp: redoes the sums exactly
//   k_v0a           fac_r / fac_c EMAs per 64 vector entries, partial sums of their statistics
//   k_v0b           row / column factor tables; the 12 row-only / column-only feature channels
//                   normalised and folded into 8-float first-layer terms per row / column
//   k_celo2_elem    one launch, items ordered slab by slab (k_celo2.h):
//     statistics    sum of squares of the 18 per-element channels (accumulators advanced in
//                   registers, nothing written); AdamW tensors are fully updated here      24 B/elem
//     fold          per tensor, by its last statistics block: normalisation scales folded into the
//                   first-layer weights
//     apply         accumulators advanced and written, features, MLP, step_out             44 B/elem
//   (PYLO_MI355_SLAB_ELEMS=0: k_celo2_stats, k_stat_segsum, k_celo2_fold, k_celo2_apply as launches
//   of their own, each over all tensors)
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "k_celo2.h"
#include "k_gradstats.h"
#include "k_adafac.h"
#include "k_single.h"
#include "k_velo.h"
#include "k_celo2_slices.h"
#include "k_ns.h"
#include "k_ns_hf.h"
#include "k_slice_finish.h"
#include "k_cast.h"
#include "pylo_common.h"
#include "pylo_mi355_bench.h"

// =============================================================================================
// Host side: plan construction and the C ABI
// =============================================================================================
using namespace pylo;

namespace {

thread_local std::string g_err;

int fail(const std::string& m) {
  g_err = m;
  return 1;
}

#define HIP_TRY(expr)                                                                    \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) return fail(std::string(#expr) + ": " + hipGetErrorString(e_)); \
  } while (0)

size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }
long long round4(long long x) { return (x + 3) / 4 * 4; }

// (dc, dr): index of the 2nd-largest and largest dim, ties keep index order
// (pylo/optim/CELO2_naive.py:42-47); VeLO swaps an equal pair except 4-D (0,1)
// (pylo/optim/velo_cuda.py:121-131).
bool factored_dims(int kind, const PyloTensorShape& s, int* dc, int* dr) {
  if (s.ndim < 2) return false;
  std::vector<int> order(s.ndim);
  for (int i = 0; i < s.ndim; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return s.shape[x] < s.shape[y]; });
  int a = order[s.ndim - 2], b = order[s.ndim - 1];
  if (kind == PYLO_KIND_VELO && s.shape[a] == s.shape[b] && !(s.ndim == 4 && a == 0 && b == 1)) std::swap(a, b);
  *dc = a;
  *dr = b;
  return true;
}

// One group of matrices of the split-fp16 Newton-Schulz kernels: its ranges in the job tables.
struct NsGroup {
  int gram0, n_gram, poly0, n_poly, upd0, n_upd, upd40, n_upd4, split0, n_split, split_max_m;
  int list0, n_list;       // its matrices (ns_list)
  int sitem0, n_sitems;    // its tiles of the pass that splits the raw steps into planes
  int fitem0, n_fitems;    // its blocks of the pass that sums the squares of A (chain length per matrix)
  int fin0, n_fin;         // its blocks of the finishing pass
  int unit0, n_units;      // ... and their units
};
// One batch of matrices: those whose operand planes share the plane workspace at one time.
struct NsBatch { int mat0, n_mats, group0, n_groups; long long plane_elems; };

struct Layout {
  std::vector<Item> mx_items;   // ELO-CELO2: statistics and apply items in slab order (k_celo2_elem)
  size_t off_mx_items = 0, off_sync = 0;
  size_t off_newsum = 0, off_piv = 0, off_wmix = 0;   // VeLO: sums carried to the next step, pivots, un-folded MLPs
  // ELO-CELO2: Newton-Schulz on the 2-D tensors (k_ns.h)
  std::vector<NsMat> ns_mats;
  std::vector<NsItem> ns_gram, ns_poly, ns_upd;
  std::vector<NsItem> ns_upd4;        // split-fp16 kernels: update jobs with 256-column tiles
  std::vector<NsGroup> ns_groups;     // split-fp16 kernels: ranges of the job tables, one per group of matrices
  std::vector<NsBatch> ns_batches;    // split-fp16 kernels: batches of matrices that run one after another
  std::vector<int> ns_split;          // matrices whose Gram product is split (k_ns_gram_reduce)
  std::vector<long long> ns_xalt;     // per tensor: offset of its second X buffer, -1 without one
  std::vector<int> ns_of_tensor;      // per tensor: index into ns_mats, -1
  std::vector<int> ns_group_of_tensor;  // split-fp16 kernels, per tensor: its group (index into ns_groups), -1
  std::vector<int> ns_list;           // the groups' matrices, group after group
  int fin_rest0 = 0, n_fin_rest = 0, unit_rest0 = 0, n_unit_rest = 0;   // finishing pass: what belongs to no group
  size_t off_ns_list = 0;
  // ELO-CELO2: tensors with more than two dims, finished per slice of the last two dims (k_slice_finish.h)
  std::vector<SliceMat> slice_mats;
  // blocks of the lane-owned slices (in registers: 1 x 1, 3 x 3, 5 x 5, 7 x 7; in LDS: up to 12, 28, 64 KB a wave),
  // of the wave-owned and of the block-owned ones
  std::vector<Item> slice_items_l[kSliceLaneSets], slice_items_w, slice_items_b;
  std::vector<int> slice_of_tensor;   // per tensor: index into slice_mats, -1
  std::vector<FinUnit> fin_units;     // ELO-CELO2 finishing pass: what each normaliser runs over
  size_t off_fin_units = 0;
  int slice_lds_l[kSliceLaneSets] = {}, slice_lds_w = 0, slice_lds_b = 0;
  size_t off_slice_mats = 0, off_slice_items_l[kSliceLaneSets] = {}, off_slice_items_w = 0, off_slice_items_b = 0;
  int ns_max_m = 0;
  std::vector<Item> ns_flag_items;    // split-fp16 kernels: {matrix, chunk of its A} of k_ns_hf_chain_sumsq, group after group
  int ns_fpart_total = 0;
  size_t off_ns_flags = 0, off_ns_fpart = 0, off_ns_flag_items = 0;
  // Newton-Schulz on the fp16 matrix pipe (two-way split operands): tables of their own
  bool ns_hf = false;
  std::vector<NsHfMat> nsb_mats;
  std::vector<NsTileItem> nsb_split_items;
  size_t off_nsb_mats = 0, off_nsb_split_items = 0, off_ns_pw = 0, off_ns_upd4 = 0;
  long long nsb_plane_elems = 0;
  size_t off_ns_mats = 0, off_ns_gram = 0, off_ns_poly = 0, off_ns_upd = 0, off_ns_split = 0, off_ns_xalt = 0,
         off_ns_scale = 0, off_ns_ws = 0;
  // tensors whose grad / param are not fp32 (PYLO_F_STORE_*): fp32 staging, pieces of the cast kernels
  bool typed = false;
  std::vector<StageOfs> stage_ofs;
  std::vector<Item> cast_items;
  long long stage_floats = 0;
  size_t off_dyn_user = 0, off_stage_ofs = 0, off_cast_items = 0, off_stage = 0;
  std::vector<TDesc> descs;
  std::vector<Item> sl_lane_items;    // ELO-CELO2: blocks of k_celo2_slices_lane, the classes of slice length one after another
  std::vector<Item> sl_lane_cls[kSliceLaneClasses];
  int sl_lane_n[kSliceLaneClasses] = {}, sl_lane_lds[kSliceLaneClasses] = {};   // a launch per class: LDS sized for its longest slice
  size_t off_sl_lane_items = 0;
  std::vector<Item> p0_items, nd_items, sl_items, seg_items, el_items, ap_items, pp_items, ga_items, fin_items, v0a_items, v0b_items;
  std::vector<int> fac_list;
  std::vector<int> dc, dr;
  int H = 8;  // width of the first MLP layer (terms per row / column)
  int Tpad = 0;
  bool global_norm = false;  // AdafacLO kind: every tensor has P0 items, the call may clip by global norm
  bool tensor_norm = false;  // ... or every tensor by its own norm (PYLO_F_TENSOR_NORM)
  size_t off_descs, off_dyn, off_p0_items, off_nd_items, off_sl_items, off_seg_items, off_segtot, off_el_items, off_ap_items, off_pp_items, off_ga_items, off_fin_items, off_finpart, off_finscale, off_tscale, off_v0a_items, off_v0b_items, off_fac_list,
      off_part, off_gsq, off_flag, off_globals, off_fac, off_term, off_v0part, off_bscale, off_stats, off_wfold,
      off_chan_ms, off_totals, off_xfeat, off_lossfeat, off_xT, off_mixbuf, off_pmax, off_canon, off_frac, total;
};

int first_layer_width(int kind) { return kind == PYLO_KIND_CELO2 ? 8 : kind == PYLO_KIND_VELO ? 4 : 32; }

// The hidden layers of ELO-CELO2 run as lane-local 4x4x1 fp32 outer products on the matrix pipe and
// wide 2-D tensors are walked column-resident; PYLO_MI355_VALU_MLP=1 in the environment keeps the
// earlier all-VALU kernels over linear chunks (same results up to rounding; for A/B measurements).
bool env_matrix_pipe() {
  const char* v = std::getenv("PYLO_MI355_VALU_MLP");
  return !(v && v[0] == '1');
}

// AdafacLO's element MLP on the fp16 matrix instructions (two-plane operands); PYLO_MI355_ADAFAC_F32=1 keeps
// the fp32 matrix instructions.
bool env_adafac_hf() {
  const char* v = std::getenv("PYLO_MI355_ADAFAC_F32");
  return !(v && v[0] == '1');
}

// Elements per slab of the fused element pass of ELO-CELO2 (k_celo2_elem).  While the apply items of one
// slab run, the statistics items of the third slab after it do, with the slabs between them resident
// as well: four slabs of 24 bytes per element plus the 20 bytes per element the apply items write
// must fit the 256 MB memory-side cache (measured on the GPT-2-small set: 1.2 M elements 1.51 ms a step,
// 2.4 M 1.48, 3.6 M 1.48, 4.8 M 1.72).  PYLO_MI355_SLAB_ELEMS=0 in the environment (read at plan
// creation) runs each pass over all tensors as a launch of its own instead.
long long env_slab_elems() {
  const char* v = std::getenv("PYLO_MI355_SLAB_ELEMS");
  if (v && v[0]) return std::atoll(v);
  return 2400000;
}
// Slabs of statistics items between a slab's statistics and its apply items (measured: ELO-CELO2 on the
// GPT-2-small set 1.49 / 1.48 ms a step with 2 / 3, VeLO on the ViT-B/16 set 1.06 / 1.00 / 1.04 ms with 1 / 2 / 3).
int env_slab_depth(int kind) {
  const char* v = std::getenv("PYLO_MI355_SLAB_DEPTH");
  return (v && v[0]) ? std::max(1, std::atoi(v)) : (kind == PYLO_KIND_VELO ? 2 : 3);
}
long long env_keep_elems() {   // largest tensor whose inputs are still expected in the cache when its apply items run
  const char* v = std::getenv("PYLO_MI355_KEEP_ELEMS");
  return (v && v[0]) ? std::atoll(v) : 8000000;
}

int tile_rows_for(int kind) {
  const char* v = std::getenv("PYLO_MI355_TILE_ROWS");
  if (kind == PYLO_KIND_CELO2 && v && v[0] && std::atoi(v) > 0) return std::atoi(v);
  return kTileRows;
}

// Items of k_celo2_elem.  Slabs are runs of whole tensors, last tensors first (their gradients are what
// k_p0 read last).  A tensor too large to stay cached is streamed: its statistics items are cut into
// slab-sized pieces (so that the apply items of the slabs before it keep their place two pieces behind),
// and its apply items follow its last piece, last item first: they start on what was read last.
void build_elem_items(Layout& L, int T, int kind) {
  struct Piece { int st0, st1, ap0, ap1; bool keep; };   // statistics items [st0, st1); apply items [ap0, ap1) or none
  const long long cap = env_slab_elems(), keep_max = env_keep_elems();
  if (cap <= 0) return;
  std::vector<Piece> pieces;
  long long elems = 0;
  int el_hi = -1, el_lo = -1;
  auto close = [&]() {
    if (el_hi > el_lo) pieces.push_back(Piece{el_lo, el_hi, el_lo, el_hi, true});
    el_hi = el_lo = -1;
    elems = 0;
  };
  for (int t = T - 1; t >= 0; --t) {
    const TDesc& d = L.descs[t];
    if (d.nblk == 0) continue;
    if (d.n > keep_max) {
      close();
      const long long per_item = std::max<long long>(d.n / d.nblk, 1);
      const int step = (int)std::max<long long>(cap / per_item, 1);
      for (int i = d.blk0; i < d.blk0 + d.nblk; i += step) {
        const int e = std::min(i + step, d.blk0 + d.nblk);
        const bool last = e == d.blk0 + d.nblk;
        pieces.push_back(Piece{i, e, last ? d.blk0 : 0, last ? d.blk0 + d.nblk : 0, false});
      }
      continue;
    }
    if (elems > 0 && elems + d.n > cap) close();
    if (el_hi < 0) el_hi = d.blk0 + d.nblk;
    el_lo = d.blk0;   // tensors are visited in descending order: the run grows downwards
    elems += d.n;
  }
  close();
  const int np = (int)pieces.size(), depth = env_slab_depth(kind);
  auto push = [&](int i0, int i1, bool apply, bool keep) {
    const int n0 = (int)L.mx_items.size();
    for (int i = i0; i < i1; ++i) {
      Item it = L.el_items[i];
      if (apply && L.descs[it.tensor].mode == kModeFlat) continue;   // AdamW tensors are finished by their statistics items
      it.b = i;
      it.c = apply ? kElemApply : (keep ? kElemKeep : 0);
      L.mx_items.push_back(it);
    }
    if (apply && !keep) std::reverse(L.mx_items.begin() + n0, L.mx_items.end());
  };
  for (int k = 0; k < np + depth; ++k) {
    if (k < np) push(pieces[k].st0, pieces[k].st1, false, pieces[k].keep);
    if (k >= depth) push(pieces[k - depth].ap0, pieces[k - depth].ap1, true, pieces[k - depth].keep);
  }
}

// PYLO_MI355_NS_F32=1 keeps the Newton-Schulz products on the fp32 matrix instructions (k_ns.h) instead of
// the split-fp16 ones (k_ns_hf.h); read at plan creation.
bool env_ns_xcd() {
  const char* e = getenv("PYLO_MI355_NS_XCD");
  return !(e && e[0] == '0');
}

// PYLO_MI355_NS_GROUPS: into how many groups (streams) the matrices of a plan are dealt, 1 to 4; read at plan creation.
int env_ns_groups() {
  const char* e = getenv("PYLO_MI355_NS_GROUPS");
  const int g = e ? atoi(e) : 4;
  return std::max(1, std::min(g, 4));
}

// PYLO_MI355_NS_WORKSPACE_MB: what the operand planes of the matrices that are orthogonalised at one time may take
// (in fp16 elements here); read at plan creation.
long long env_ns_budget_elems() {
  const char* e = getenv("PYLO_MI355_NS_WORKSPACE_MB");
  const long long mb = e ? atoll(e) : 8192;
  return std::max(1ll, mb) * (1ll << 20) / 2;
}

// How the Newton-Schulz iterations share their products over the long dim (k_ns_hf.h): a chain of L iterations takes
// one Gram product, one update and 4 L - 3 products of m x m matrices.  PYLO_MI355_NS_CHAINS="2,3" gives the chain
// lengths in order (they must add up to the iteration count, else the default applies); PYLO_MI355_NS_PAIRS=0 means
// chains of one: one Gram product and one update per iteration, as the formula is written.  Read when the products
// are enqueued.
std::vector<int> ns_chains(int iters) {
  std::vector<int> out;
  const char* p = getenv("PYLO_MI355_NS_PAIRS");
  if (p && p[0] == '0') {
    out.assign(iters, 1);
    return out;
  }
  if (const char* e = getenv("PYLO_MI355_NS_CHAINS")) {
    int sum = 0;
    for (const char* c = e; *c;) {
      const int v = atoi(c);
      if (v < 1) break;
      out.push_back(v);
      sum += v;
      while (*c && *c != ',') ++c;
      if (*c == ',') ++c;
    }
    if (sum == iters) return out;
    out.clear();
  }
  // default: pairs (five iterations: 2, 2, 1).  Longer chains are faster and less accurate: "3,2" takes the
  // GPT-2-small step from 6.4 to 5.7 ms and stays at the formula's own fp32 error on most inputs, but reaches 1e-4
  // of the result's RMS (against 1.3e-5 for pairs) on matrices with a dominant direction over a flat rest.
  for (int left = iters; left > 0;) {
    const int l = std::min(left, 2);
    out.push_back(l);
    left -= l;
  }
  return out;
}

// PYLO_MI355_NS_ADAPTIVE=1: a first chain of three iterations for the matrices whose spectrum allows it
// (k_ns_hf_chain_flag), pairs for the others -- unless the environment fixes the chains (PYLO_MI355_NS_CHAINS,
// PYLO_MI355_NS_PAIRS=0).  Off by default: raw steps with a direction that holds more than 8 % of their squared norm
// never qualify (an untrained MLP's steps, with their common offset, are such), and the test costs 0.04 ms a step.
// Read when the products are enqueued.
bool ns_adaptive() {
  const char* a = getenv("PYLO_MI355_NS_ADAPTIVE");
  if (!(a && a[0] == '1')) return false;
  const char* p = getenv("PYLO_MI355_NS_PAIRS");
  if (p && p[0] == '0') return false;
  const char* c = getenv("PYLO_MI355_NS_CHAINS");
  return !(c && c[0]);
}

// The planes of the Newton-Schulz products are fp16 numbers: every matrix is stored times a power of two that puts its
// largest possible entry at 12 000 .. 24 000 (the format ends at 65 504), so that the second plane keeps its bits on
// entries five decades smaller.  No entry exceeds the matrix's largest singular value, and those follow from the
// coefficients alone: X0 has unit Frobenius norm, so its singular values lie in [0, 1], and every iteration maps
// sigma to sigma p(sigma^2), p(l) = c2 l^2 + c1 l + c0.  Bounds over all iterations, from a grid of starting values:
// X (sigma), A = X X^T (sigma^2), B' = p(A), T = A B', and the products of k consecutive B' (q[k], k >= 1).
struct NsExps {
  int x, a, b, t;
  std::vector<int> q;
};
inline float pow2(int e) { return std::ldexp(1.0f, e); }
NsExps ns_plane_exps(float c0, float c1, float c2, int iters) {
  constexpr int kGrid = 2048;
  const int n = std::max(iters, 1);
  double bx = 1.0, ba = 1.0, bb = std::fabs((double)c0), bt = 0.0;
  std::vector<double> bq(n + 1, 0.0), pv(n);
  for (int g = 0; g <= kGrid; ++g) {
    double sig = (double)g / kGrid;
    for (int t = 0; t < n; ++t) {
      const double l = sig * sig, pl = (double)c2 * l * l + (double)c1 * l + (double)c0;
      pv[t] = std::fabs(pl);
      ba = std::max(ba, l);
      bb = std::max(bb, pv[t]);
      bt = std::max(bt, l * pv[t]);
      sig *= pl;
      bx = std::max(bx, std::fabs(sig));
    }
    for (int t0 = 0; t0 < n; ++t0) {
      double prod = 1.0;
      for (int k = 1; t0 + k <= n; ++k) {
        prod *= pv[t0 + k - 1];
        bq[k] = std::max(bq[k], prod);
      }
    }
  }
  auto exp_of = [](double bound) {
    if (!(bound > 0.0) || !std::isfinite(bound)) return -60;   // (coefficients that diverge: nothing to keep)
    const int e = (int)std::floor(std::log2(30000.0 / (1.25 * bound)));
    return std::max(-60, std::min(e, 14));
  };
  NsExps ex;
  ex.x = exp_of(bx); ex.a = exp_of(ba); ex.b = exp_of(bb); ex.t = exp_of(bt);
  ex.q.resize(n + 1);
  for (int k = 1; k <= n; ++k) ex.q[k] = exp_of(bq[k]);
  ex.q[0] = ex.b;
  return ex;
}

// PYLO_MI355_SLICES_LDS=0: the short slices of ELO-CELO2 tensors with more than two dims stay on the kernel that reads
// them straight from memory, twice (k_celo2_slices); read at plan creation.
bool env_slices_lds() {
  const char* e = getenv("PYLO_MI355_SLICES_LDS");
  return !(e && e[0] == '0');
}

bool env_ns_hf() {
  const char* e = getenv("PYLO_MI355_NS_F32");
  return !(e && e[0] == '1');
}

// Workgroups go to the eight XCDs in turn (block b runs on XCD b % 8) and every XCD has an L2 of its own:
// tile jobs that read the same operands should share an XCD.  `units` are runs of jobs that belong together
// (count, work per job); the run sequence is cut into eight stretches of about equal work, stretch x becomes
// the jobs 8 i + x.  Stretches are filled up with jobs that do nothing (mat = -1).
constexpr int kXcds = 8;
void xcd_interleave(std::vector<NsItem>& items, const std::vector<std::pair<int, long long>>& units) {
  long long total = 0;
  for (const auto& u : units) total += u.first * u.second;
  std::vector<std::vector<NsItem>> lane(kXcds);
  long long done = 0;
  size_t pos = 0;
  int x = 0;
  for (const auto& u : units) {
    // a unit goes to the stretch in which its middle falls
    const long long mid = done + u.first * u.second / 2;
    x = std::max(x, (int)std::min<long long>(kXcds - 1, total > 0 ? mid * kXcds / total : 0));
    for (int i = 0; i < u.first; ++i) lane[x].push_back(items[pos + i]);
    pos += u.first;
    done += u.first * u.second;
  }
  size_t longest = 0;
  for (const auto& l : lane) longest = std::max(longest, l.size());
  std::vector<NsItem> out;
  out.reserve(longest * kXcds);
  for (size_t i = 0; i < longest; ++i)
    for (int q = 0; q < kXcds; ++q) out.push_back(i < lane[q].size() ? lane[q][i] : NsItem{-1, 0, 0, 0, 0, -1});
  items.swap(out);
}

// Newton-Schulz tables: every 2-D MLP tensor (the fp32 kernels: those whose rows (C) and whose smaller dim are
// multiples of 4).  `ws_floats` returns the floats of workspace behind off_ns_ws.
void build_ns_tables(Layout& L, const PyloTensorShape* shapes, int T, long long& ws_floats) {
  ws_floats = 0;
  L.ns_xalt.assign(T, -1);
  L.ns_of_tensor.assign(T, -1);
  L.ns_group_of_tensor.assign(T, -1);
  auto take = [&](long long n) { const long long o = ws_floats; ws_floats += (n + 63) / 64 * 64; return o; };
  for (int t = 0; t < T; ++t) {
    const TDesc& d = L.descs[t];
    if (d.n == 0 || (shapes[t].flags & PYLO_F_NO_ORTHOGONALIZE)) continue;
    // two dims; or more, as one matrix per slice of the last two, where the per-slice launches do not take the
    // slices (k_slice_finish.h) -- the split-fp16 kernels only, whose tables carry a matrix's place in its tensor
    const bool slices = d.mode == kModeFacND && L.ns_hf && L.slice_of_tensor[t] < 0;
    if (d.mode != kModeFac2D && !slices) continue;
    const int R = slices ? (int)shapes[t].shape[shapes[t].ndim - 2] : d.R0;
    const int C = slices ? (int)shapes[t].shape[shapes[t].ndim - 1] : d.C0;
    // the fp32 kernels load 16 bytes at a time along the contiguous dim of X, A and B'
    if (!L.ns_hf && (C % 4 != 0 || std::min(R, C) % 4 != 0)) continue;
    const int n_sl = slices ? (int)(d.n / ((long long)R * C)) : 1;
    for (int sl = 0; sl < n_sl; ++sl) {
    NsMat mt{};
    mt.tensor = t;
    mt.unit = sl;        // the finishing pass's tables come later: build_fin_tables adds the tensor's first unit
    mt.elem_off = (long long)sl * R * C;
    mt.R = R; mt.C = C;
    mt.tall = R > C;
    mt.m = std::min(R, C);
    const int K = mt.tall ? mt.R : mt.C;
    mt.n_slabs = K >= kNsSplitMin ? (K + kNsSlabK - 1) / kNsSlabK : 1;
    mt.slab_k = kNsSlabK;
    mt.off_x1 = take((long long)R * C);
    mt.off_a = take((long long)mt.m * mt.m);
    mt.off_b = take((long long)mt.m * mt.m);
    mt.off_part = mt.n_slabs > 1 ? take((long long)mt.n_slabs * mt.m * mt.m) : 0;
    const int q = (int)L.ns_mats.size();
    if (sl == 0) {
      L.ns_of_tensor[t] = q;
      L.ns_xalt[t] = mt.off_x1;
    }
    L.ns_max_m = std::max(L.ns_max_m, mt.m);
    const int nt = (mt.m + kNsTile - 1) / kNsTile;
    for (int tm = 0; tm < nt; ++tm)
      for (int tn = tm; tn < nt; ++tn) {
        if (mt.n_slabs > 1) {
          for (int sb = 0; sb < mt.n_slabs; ++sb)
            L.ns_gram.push_back(NsItem{q, tm, tn, sb * kNsSlabK, std::min(K, (sb + 1) * kNsSlabK), sb});
        } else {
          L.ns_gram.push_back(NsItem{q, tm, tn, 0, K, -1});
        }
        L.ns_poly.push_back(NsItem{q, tm, tn, 0, mt.m, -1});
      }
    const int ni = ((mt.tall ? mt.R : mt.m) + kNsTile - 1) / kNsTile, nj = ((mt.tall ? mt.m : mt.C) + kNsTile - 1) / kNsTile;
    for (int tm = 0; tm < ni; ++tm)
      for (int tn = 0; tn < nj; ++tn) L.ns_upd.push_back(NsItem{q, tm, tn, 0, mt.m, -1});
    if (mt.n_slabs > 1) L.ns_split.push_back(q);
    L.ns_mats.push_back(mt);
    }
  }
  if (L.ns_hf) {
    // A plan with few matrices (a convolutional net's one classifier, a small MLP) has fewer Gram tile jobs than the
    // part has CUs, each a long reduction: split them along it, up to eight ways, until there are two jobs a CU.
    {
      long long jobs = 0;
      for (const NsMat& f : L.ns_mats) {
        const long long nt = (f.m + kNsTile - 1) / kNsTile;
        jobs += nt * (nt + 1) / 2 * f.n_slabs;
      }
      if (jobs > 0 && jobs < kNsFewJobs) {
        const int ways = (int)std::min<long long>(8, (kNsFewJobs + jobs - 1) / jobs);
        for (NsMat& f : L.ns_mats) {
          if (f.n_slabs > 1) continue;
          const int K = f.tall ? f.R : f.C;
          const int sk = std::max(256, ((K + ways - 1) / ways + 15) / 16 * 16);
          if ((K + sk - 1) / sk > 1) {
            f.slab_k = sk;
            f.n_slabs = (K + sk - 1) / sk;
          }
        }
      }
    }
    // same matrices, operands as fp16 planes; the item tables are rebuilt for the uniform (n x m) orientation
    L.ns_gram.clear(); L.ns_poly.clear(); L.ns_upd.clear(); L.ns_upd4.clear();
    ws_floats = 0;
    long long pw = 0;
    auto take_p = [&](long long n) { const long long o = pw; pw += (n + 63) / 64 * 64; return o; };
    auto up = [](int x, int q) { return (x + q - 1) / q * q; };
    auto up16 = [&](int x) { return up(x, kHfBK); };
    // Planes and fp32 matrices of every matrix.  The planes are only live during a matrix's own products, so
    // the matrices are cut into batches (in tensor order) whose planes fit PYLO_MI355_NS_WORKSPACE_MB (8192 by
    // default); the batches run one after another in the same memory.  A plan whose matrices fit in one batch
    // has its planes' padding zeroed once, at plan creation; with several batches every batch starts by zeroing
    // the region (one fill at HBM write speed: the padding of one batch's planes lies in another's data).
    const long long budget = env_ns_budget_elems();
    long long pw_max = 0, ws_max = 0;
    std::vector<int> batch_of;
    L.ns_batches.clear();
    NsBatch batch{};
    auto mats_of_tensor = [&](size_t q) {
      size_t e = q;
      while (e < L.ns_mats.size() && L.ns_mats[e].tensor == L.ns_mats[q].tensor) ++e;
      return (long long)(e - q);
    };
    for (size_t q = 0; q < L.ns_mats.size(); ++q) {
      const NsMat& f = L.ns_mats[q];
      NsHfMat b{};
      b.tensor = f.tensor; b.R = f.R; b.C = f.C; b.m = f.m; b.n = std::max(f.R, f.C); b.tall = f.tall;
      b.pad_m = up16(b.m);
      b.pad_n = up16(b.n);
      // update tiles of 256 columns where that does not compute much more padding than tiles of 128 would
      const bool wide_tiles = up(b.m, 256) <= 1.06 * up(b.m, 128);
      b.rows_m = up(b.m, wide_tiles ? 256 : kNsTile);
      b.rows_n = up(b.n, kNsTile);
      b.lda = up(b.m, 4);
      b.n_slabs = f.n_slabs;
      b.p_stride = ((long long)kNsPl * b.rows_m * b.pad_m + 63) / 64 * 64;
      // (the matrices of one tensor -- the slices of one with more than two dims -- stay in one batch)
      const bool first_of_tensor = q == 0 || L.ns_mats[q - 1].tensor != f.tensor;
      const long long need = ((long long)kNsPl * b.rows_m * b.pad_n + 2ll * kNsPl * b.rows_n * b.pad_m + kNsBufs * b.p_stride + 4 * 64) *
                             (first_of_tensor ? mats_of_tensor(q) : 1);
      if (pw > 0 && first_of_tensor && pw + need > budget) {   // this tensor opens the next batch
        batch.plane_elems = pw;
        L.ns_batches.push_back(batch);
        batch = NsBatch{};
        batch.mat0 = (int)q;
        pw = 0;
        ws_floats = 0;
      }
      b.off_xs = take_p((long long)kNsPl * b.rows_m * b.pad_n);
      b.off_xl[0] = take_p((long long)kNsPl * b.rows_n * b.pad_m);
      b.off_xl[1] = take_p((long long)kNsPl * b.rows_n * b.pad_m);
      b.off_p = take_p(kNsBufs * b.p_stride);
      b.off_a = take((long long)b.m * b.lda);
      b.off_part = b.n_slabs > 1 ? take((long long)b.n_slabs * b.m * b.lda) : 0;
      b.elem_off = f.elem_off;
      L.ns_mats[q].off_a = b.off_a;   // the fp32 tables stay consistent for k_ns_scale (tensor index only)
      L.nsb_mats.push_back(b);
      batch_of.push_back((int)L.ns_batches.size());
      batch.n_mats = (int)q + 1 - batch.mat0;
      pw_max = std::max(pw_max, pw);
      ws_max = std::max(ws_max, ws_floats);
    }
    if (batch.n_mats > 0) {
      batch.plane_elems = pw;
      L.ns_batches.push_back(batch);
    }
    pw = pw_max;
    ws_floats = ws_max;
    L.nsb_plane_elems = pw;
    std::fill(L.ns_xalt.begin(), L.ns_xalt.end(), -1);   // the result always replaces the raw step
    // Groups of matrices.  The products of one matrix depend on each other, those of different matrices do not:
    // each group runs its chain of launches on a stream of its own, so that the blocks of one group's launch
    // fill the CUs that the tail of the other's leaves idle.  Matrices are dealt to the groups heaviest first.
    L.ns_groups.clear();
    L.ns_split.clear();
    L.ns_list.clear();
    L.nsb_split_items.clear();
    L.ns_flag_items.clear();
    L.ns_fpart_total = 0;
    for (NsBatch& bt : L.ns_batches) {
    const int n_groups = std::min<int>(env_ns_groups(), std::max(bt.n_mats / 8, 1));
    std::vector<std::vector<int>> members(n_groups);
    {
      // (tensor by tensor: the slices of a tensor with more than two dims share a group, which also finishes it)
      struct Run { int q0, q1; double work; };
      std::vector<Run> runs;
      for (int q = bt.mat0; q < bt.mat0 + bt.n_mats; ++q) {
        const NsHfMat& b = L.nsb_mats[q];
        // (five iterations in pairs: three Gram products on the upper blocks and three updates, eleven m x m products)
        const double w = (double)b.m * b.m * (4.6 * b.n + 5.9 * b.m);
        if (!runs.empty() && L.nsb_mats[runs.back().q0].tensor == b.tensor) { runs.back().q1 = q + 1; runs.back().work += w; }
        else runs.push_back(Run{q, q + 1, w});
      }
      std::stable_sort(runs.begin(), runs.end(), [](const Run& x, const Run& y) { return x.work > y.work; });
      std::vector<double> load(n_groups, 0.0);
      for (const Run& r : runs) {
        const int g = (int)(std::min_element(load.begin(), load.end()) - load.begin());
        for (int q = r.q0; q < r.q1; ++q) members[g].push_back(q);
        load[g] += r.work;
      }
      for (auto& mm : members) std::sort(mm.begin(), mm.end());   // neighbours in memory stay neighbours in the tables
    }
    bt.group0 = (int)L.ns_groups.size();
    bt.n_groups = n_groups;
    for (int g = 0; g < n_groups; ++g) {
      // job runs that read the same operands: per matrix (slab), and finer, per row of tiles, for sets of few matrices
      std::vector<std::pair<int, long long>> gram_units, poly_units, upd_units, upd4_units, gram_rows, poly_rows;
      std::vector<NsItem> gram, poly, upd, upd4;
      NsGroup grp{};
      grp.split0 = (int)L.ns_split.size();
      grp.list0 = (int)L.ns_list.size();
      grp.sitem0 = (int)L.nsb_split_items.size();
      grp.fitem0 = (int)L.ns_flag_items.size();
      for (int q : members[g]) {
        {
          NsHfMat& bw = L.nsb_mats[q];
          bw.fpart0 = L.ns_fpart_total;
          bw.n_fpart = (int)(((long long)bw.m * bw.m + kNsFlagChunk - 1) / kNsFlagChunk);
          L.ns_fpart_total += bw.n_fpart;
          for (int c = 0; c < bw.n_fpart; ++c) L.ns_flag_items.push_back(Item{q, c, 0, 0});
        }
        const NsHfMat& b = L.nsb_mats[q];
        L.ns_list.push_back(q);
        L.ns_group_of_tensor[b.tensor] = (int)L.ns_groups.size();
        for (int tr = 0; tr < (b.R + 63) / 64; ++tr)
          for (int tc = 0; tc < (b.C + 63) / 64; ++tc) L.nsb_split_items.push_back(NsTileItem{q, tr, tc});
        const bool wide_tiles = b.rows_m % 256 == 0 && up(b.m, 256) <= 1.06 * up(b.m, 128);
        const int nt = (b.m + kNsTile - 1) / kNsTile, n_upper = nt * (nt + 1) / 2;
        // Gram: the tiles of one matrix (of one slab of it) read the same rows of Xs; Poly: the same A
        for (int sl = 0; sl < b.n_slabs; ++sl) {
          const int slab_k = L.ns_mats[q].slab_k;
          const int k0 = b.n_slabs > 1 ? sl * slab_k : 0;
          const int k1 = b.n_slabs > 1 ? up16(std::min(b.n, (sl + 1) * slab_k)) : up16(b.n);
          for (int tm = 0; tm < nt; ++tm)
            for (int tn = tm; tn < nt; ++tn) gram.push_back(NsItem{q, tm, tn, k0, k1, b.n_slabs > 1 ? sl : -1});
          gram_units.push_back({n_upper, (long long)(k1 - k0)});
          for (int tm = 0; tm < nt; ++tm) gram_rows.push_back({nt - tm, (long long)(k1 - k0)});
        }
        for (int tm = 0; tm < nt; ++tm)
          for (int tn = tm; tn < nt; ++tn) poly.push_back(NsItem{q, tm, tn, 0, up16(b.m), -1});
        poly_units.push_back({n_upper, (long long)up16(b.m)});
        for (int tm = 0; tm < nt; ++tm) poly_rows.push_back({nt - tm, (long long)up16(b.m)});
        // Update: the tiles of one row block read the same rows of Xl, all of them the same B'
        const int ni = (b.n + kNsTile - 1) / kNsTile, ntu = wide_tiles ? (b.m + 255) / 256 : nt;
        std::vector<NsItem>& u = wide_tiles ? upd4 : upd;
        std::vector<std::pair<int, long long>>& units = wide_tiles ? upd4_units : upd_units;
        for (int tm = 0; tm < ni; ++tm) {
          for (int tn = 0; tn < ntu; ++tn) u.push_back(NsItem{q, tm, tn, 0, up16(b.m), -1});
          units.push_back({ntu, (long long)up16(b.m)});
        }
        if (b.n_slabs > 1) {
          L.ns_split.push_back(q);
          grp.split_max_m = std::max(grp.split_max_m, b.m);
        }
      }
      if (env_ns_xcd()) {
        // with fewer runs than a few per XCD the stretches would be uneven: take the finer runs, or leave the order
        auto pick = [](std::vector<NsItem>& items, const std::vector<std::pair<int, long long>>& coarse,
                       const std::vector<std::pair<int, long long>>& fine) {
          if (coarse.size() >= 4 * kXcds) xcd_interleave(items, coarse);
          else if (fine.size() >= 4 * kXcds) xcd_interleave(items, fine);
        };
        pick(gram, gram_units, gram_rows);
        pick(poly, poly_units, poly_rows);
        pick(upd, upd_units, upd_units);
        pick(upd4, upd4_units, upd4_units);
      }
      auto append = [](std::vector<NsItem>& all, const std::vector<NsItem>& part, int& first, int& count) {
        first = (int)all.size();
        count = (int)part.size();
        all.insert(all.end(), part.begin(), part.end());
      };
      append(L.ns_gram, gram, grp.gram0, grp.n_gram);
      append(L.ns_poly, poly, grp.poly0, grp.n_poly);
      append(L.ns_upd, upd, grp.upd0, grp.n_upd);
      append(L.ns_upd4, upd4, grp.upd40, grp.n_upd4);
      grp.n_split = (int)L.ns_split.size() - grp.split0;
      grp.n_list = (int)L.ns_list.size() - grp.list0;
      grp.n_sitems = (int)L.nsb_split_items.size() - grp.sitem0;
      grp.n_fitems = (int)L.ns_flag_items.size() - grp.fitem0;
      L.ns_groups.push_back(grp);
    }
    }
    return;
  }
  // longest jobs first: the launch ends when its last block does
  auto longer = [](const NsItem& x, const NsItem& y) { return x.k1 - x.k0 > y.k1 - y.k0; };
  std::stable_sort(L.ns_gram.begin(), L.ns_gram.end(), longer);
  std::stable_sort(L.ns_poly.begin(), L.ns_poly.end(), longer);
  std::stable_sort(L.ns_upd.begin(), L.ns_upd.end(), longer);
}

// ELO-CELO2 tensors with more than two dims on the MLP path: the slices of their last two dims, where one fits the
// LDS of the lanes that would own it (k_slice_finish.h).
void build_slice_tables(Layout& L, const PyloTensorShape* shapes, int T) {
  L.slice_of_tensor.assign(T, -1);
  L.slice_mats.clear(); L.slice_items_w.clear(); L.slice_items_b.clear();
  for (int k = 0; k < kSliceLaneSets; ++k) { L.slice_items_l[k].clear(); L.slice_lds_l[k] = 0; }
  L.slice_lds_w = L.slice_lds_b = 0;
  for (int t = 0; t < T; ++t) {
    const TDesc& d = L.descs[t];
    const PyloTensorShape& sh = shapes[t];
    if (d.mode != kModeFacND || d.n == 0 || sh.ndim < 3) continue;
    SliceMat sm{};
    sm.tensor = t;
    sm.R = (int)sh.shape[sh.ndim - 2];
    sm.C = (int)sh.shape[sh.ndim - 1];
    sm.slices = d.n / ((long long)sm.R * sm.C);
    sm.no_orth = (sh.flags & PYLO_F_NO_ORTHOGONALIZE) != 0;
    if (!slice_geometry(sm)) continue;
    const int per_block = sm.lanes == 1 ? 64 : 256 / sm.lanes;
    const long long blocks = (sm.slices + per_block - 1) / per_block;
    if (blocks >= (1ll << 31)) continue;
    const int q = (int)L.slice_mats.size();
    L.slice_of_tensor[t] = q;
    // lane-owned slices: one launch per register size, and per LDS size class of the others (a wave's LDS share
    // decides how many waves a CU holds)
    int set = 0;
    if (sm.lanes == 1) {
      const long long need = slice_lane_lds(sm.m, sm.n);
      set = slice_in_registers(sm.m, sm.n) ? sm.m / 2 : need <= 12 * 1024 ? 4 : need <= 28 * 1024 ? 5 : 6;
    }
    std::vector<Item>& items = sm.lanes == 1 ? L.slice_items_l[set] : sm.lanes == 256 ? L.slice_items_b : L.slice_items_w;
    int& lds = sm.lanes == 1 ? L.slice_lds_l[set] : sm.lanes == 256 ? L.slice_lds_b : L.slice_lds_w;
    lds = std::max(lds, sm.lanes == 1 ? (int)slice_lane_lds(sm.m, sm.n) : (int)sizeof(float) * sm.per_floats * per_block);
    for (long long b = 0; b < blocks; ++b) items.push_back(Item{q, (int)b, 0, 0});
    L.slice_mats.push_back(sm);
  }
}

// Units and blocks of ELO-CELO2's finishing pass (after Newton-Schulz): a unit is what one normaliser runs over, cut
// into linear 8192-element blocks.  MLP tensors of up to two dims are one unit; a tensor with more dims whose slices
// the per-slice launches do not take (k_slice_finish.h) is one unit per slice of its last two dims.  The tables
// hold the tensors of each group of Newton-Schulz matrices together (a group finishes its own tensors on its own
// stream), then the tensors of no group.
int build_fin_tables(Layout& L, const PyloTensorShape* shapes, int T) {
  L.fin_units.clear(); L.fin_items.clear();
  auto add = [&](int t) {
    TDesc& d = L.descs[t];
    d.fin_unit0 = (int)L.fin_units.size();
    d.fin_units = 0;
    if (d.mode == kModeFlat || d.n == 0) return;
    long long slices = 1, len = d.n;
    if (d.mode == kModeFacND) {
      if (L.slice_of_tensor[t] >= 0) return;
      len = shapes[t].shape[shapes[t].ndim - 2] * shapes[t].shape[shapes[t].ndim - 1];
      slices = d.n / len;
    }
    for (long long sl = 0; sl < slices; ++sl) {
      FinUnit u{};
      u.tensor = t;
      u.off = sl * len;
      u.n = len;
      u.vec = len % 4 == 0;
      u.blk0 = (int)L.fin_items.size();
      const int unit = (int)L.fin_units.size();
      for (long long c = 0; c * kFinElems < len; ++c) L.fin_items.push_back(Item{unit, (int)c, 0, 0});
      u.nblk = (int)L.fin_items.size() - u.blk0;
      L.fin_units.push_back(u);
    }
    d.fin_units = (int)slices;
  };
  for (size_t g = 0; g < L.ns_groups.size(); ++g) {
    NsGroup& grp = L.ns_groups[g];
    grp.fin0 = (int)L.fin_items.size();
    grp.unit0 = (int)L.fin_units.size();
    for (int t = 0; t < T; ++t)
      if (L.ns_group_of_tensor[t] == (int)g) add(t);
    grp.n_fin = (int)L.fin_items.size() - grp.fin0;
    grp.n_units = (int)L.fin_units.size() - grp.unit0;
    if (L.fin_items.size() >= (1u << 30)) return fail("plan: too many blocks in the finishing pass");
  }
  L.fin_rest0 = (int)L.fin_items.size();
  L.unit_rest0 = (int)L.fin_units.size();
  for (int t = 0; t < T; ++t)
    if (L.ns_group_of_tensor[t] < 0) add(t);
  L.n_fin_rest = (int)L.fin_items.size() - L.fin_rest0;
  L.n_unit_rest = (int)L.fin_units.size() - L.unit_rest0;
  if (L.fin_items.size() >= (1u << 30)) return fail("plan: too many blocks in the finishing pass");
  for (NsMat& m : L.ns_mats) m.unit += L.descs[m.tensor].fin_unit0;
  return 0;
}

int build_layout(int kind, const PyloTensorShape* shapes, int T, Layout& L, int velo_hidden) {
  if (kind != PYLO_KIND_CELO2 && kind != PYLO_KIND_VELO && kind != PYLO_KIND_ADAFAC)
    return fail("plan: unknown optimizer kind");
  if (T <= 0 || shapes == nullptr) return fail("plan: no tensors");
  L.H = first_layer_width(kind);
  L.descs.assign(T, TDesc{});
  L.dc.assign(T, -1);
  L.dr.assign(T, -1);
  long long part = 0, fac = 0, term = 0;
  const int H = L.H;
  L.tensor_norm = (shapes[0].flags & PYLO_F_TENSOR_NORM) != 0;
  L.global_norm = (shapes[0].flags & PYLO_F_GLOBAL_NORM) != 0 || L.tensor_norm;
  for (int t = 0; t < T; ++t) {
    const PyloTensorShape& s = shapes[t];
    if (s.ndim < 0 || s.ndim > PYLO_MAX_DIMS) return fail("plan: bad ndim");
    long long n = 1;
    int rank = 0;
    for (int i = 0; i < s.ndim; ++i) {
      if (s.shape[i] < 0) return fail("plan: negative dim");
      n *= s.shape[i];
      rank += s.shape[i] > 1;
    }
    if (n >= (1ll << 31)) return fail("plan: tensors of 2^31 or more elements are not supported");
    TDesc& d = L.descs[t];
    d.n = n;
    d.gscale = 1.0f;
    if ((s.flags & (PYLO_F_NAN_TO_NUM | PYLO_F_WD_PRESTEP | PYLO_F_GLOBAL_NORM | PYLO_F_TENSOR_NORM)) &&
        kind != PYLO_KIND_ADAFAC)
      return fail("plan: PYLO_F_NAN_TO_NUM / PYLO_F_WD_PRESTEP / PYLO_F_GLOBAL_NORM / PYLO_F_TENSOR_NORM belong to "
                  "AdafacLO plans");
    if (((s.flags & PYLO_F_TENSOR_NORM) != 0) != L.tensor_norm)
      return fail("plan: PYLO_F_TENSOR_NORM must be set on every tensor of the plan or on none");
    if (L.tensor_norm && (s.flags & (PYLO_F_GLOBAL_NORM | PYLO_F_NAN_TO_NUM)))
      return fail("plan: PYLO_F_TENSOR_NORM does not combine with PYLO_F_GLOBAL_NORM or PYLO_F_NAN_TO_NUM");
    if (!L.tensor_norm && ((s.flags & PYLO_F_GLOBAL_NORM) != 0) != L.global_norm)
      return fail("plan: PYLO_F_GLOBAL_NORM must be set on every tensor of the plan or on none");
    d.own_norm = L.tensor_norm ? 1 : 0;
    d.nan0 = (s.flags & PYLO_F_NAN_TO_NUM) != 0;
    d.store = (s.flags & PYLO_F_STORE_MASK) >> 8;
    L.stage_ofs.push_back(StageOfs{-1, -1});
    if (d.store != kStoreF32 && n > 0) {
      const long long pitch = (n + 63) / 64 * 64;
      L.stage_ofs.back() = StageOfs{L.stage_floats, L.stage_floats + pitch};
      L.stage_floats += 2 * pitch;
      for (long long c = 0; c * kCastElems < n; ++c) L.cast_items.push_back(Item{t, (int)c, 0, 0});
      L.typed = true;
    }
    d.wd_prestep = (s.flags & PYLO_F_WD_PRESTEP) != 0;
    d.fac_slot = -1;
    d.rank = rank < 4 ? rank : 4;
    int dc = -1, dr = -1;
    const bool can_factor = factored_dims(kind, s, &dc, &dr);
    if (kind == PYLO_KIND_CELO2) {
      const bool adam = (s.flags & (PYLO_F_ADAM | PYLO_F_ADAM_INDEP)) != 0;
      d.adam_indep = (s.flags & PYLO_F_ADAM_INDEP) != 0;
      if (adam) d.mode = kModeFlat;
      else if (!can_factor) d.mode = kModeVec;  // the MLP on a tensor with fewer than two dims
      else d.mode = s.ndim == 2 ? kModeFac2D : kModeFacND;
      if (d.mode == kModeVec) d.slice_len = (int)std::max<long long>(n, 1);
      if (d.mode == kModeFacND) d.slice_len = (int)std::max<long long>(s.shape[s.ndim - 2] * s.shape[s.ndim - 1], 1);
    } else {
      d.mode = !can_factor ? kModeVec : (s.ndim == 2 ? kModeFac2D : kModeFacND);
    }
    // Geometry is laid out over the dims that matter: dims of size 1 other than the two factored ones
    // change neither strides nor sums, so a (O, I, 1, 1) convolution kernel or a (1, 1, C) token is a
    // plain 2-D tensor for the kernels (vectorised loads, column-resident walk).  Not for CELO2, whose
    // normalisers run over slices of the last two dims as given.
    PyloTensorShape e = s;
    int edc = dc, edr = dr;
    if (can_factor && kind != PYLO_KIND_CELO2 && n > 0) {
      e.ndim = 0;
      for (int i = 0; i < s.ndim; ++i) {
        if (s.shape[i] == 1 && i != dc && i != dr) continue;
        if (i == dc) edc = e.ndim;
        if (i == dr) edr = e.ndim;
        e.shape[e.ndim++] = s.shape[i];
      }
      d.mode = e.ndim == 2 ? kModeFac2D : kModeFacND;
    }
    if (d.mode == kModeFlat || d.mode == kModeVec) {
      d.vec = (n % 4 == 0) ? 4 : 1;
    } else {
      L.dc[t] = dc;
      L.dr[t] = dr;
      if (d.mode == kModeFac2D) {
        d.R0 = (int)e.shape[0];
        d.C0 = (int)e.shape[1];
        d.vec = (d.C0 % 4 == 0) ? 4 : 1;
        d.vec0_is_r = (edr == 1) ? 1 : 0;  // vector 0 (indexed by dim 0) results from summing over dim 1
        d.len[0] = d.R0; d.len[1] = d.C0;
        d.sumlen[0] = d.C0; d.sumlen[1] = d.R0;
        d.n_strips = (d.R0 + kP0Rows - 1) / kP0Rows;
        d.n_colblk = (d.C0 + 64 * d.vec - 1) / (64 * d.vec);
        d.npart[0] = d.n_colblk; d.npart[1] = d.n_strips;
      } else {
        d.vec = 1;
        d.vec0_is_r = 1;
        const int rem[2] = {edr, edc};  // the dim each vector lost
        for (int w = 0; w < 2; ++w) {
          long long stride = 1;
          for (int i = rem[w] + 1; i < e.ndim; ++i) stride *= e.shape[i];
          d.nd_size[w] = (int)e.shape[rem[w]];
          d.nd_stride[w] = (int)stride;
          d.nd_div_blk[w] = make_fastdiv((unsigned)std::max<long long>(e.shape[rem[w]] * stride, 1));
          d.nd_div_st[w] = make_fastdiv((unsigned)std::max<long long>(stride, 1));
          d.len[w] = d.nd_size[w] > 0 ? (int)(n / d.nd_size[w]) : 0;
          d.sumlen[w] = d.nd_size[w];
          d.npart[w] = std::max(1, (d.nd_size[w] + kNdX - 1) / kNdX);
        }
        // the dc axis as it sits inside the row vector (the tensor without dim dr)
        d.rcm_size = d.nd_size[1];
        d.rcm_stride = edc > edr ? d.nd_stride[1] : d.nd_stride[1] / std::max(d.nd_size[0], 1);
      }
      for (int w = 0; w < 2; ++w) {
        d.pitch[w] = (int)round4(d.len[w]);
        d.part_off[w] = part;
        part += round4((long long)d.npart[w] * d.len[w]);
        d.fac_off[w] = fac;              // [entry][4]
        fac += (long long)d.len[w] * 4;
        d.term_off[w] = term;            // [entry][H]
        term += round4((long long)d.len[w] * H);
      }
      if (n > 0) {
        d.fac_slot = (int)L.fac_list.size();
        L.fac_list.push_back(t);
        for (int w = 0; w < 2; ++w) {
          d.v0a_first[w] = (int)L.v0a_items.size();
          for (int c = 0; c * kV0aEnt < d.len[w]; ++c) L.v0a_items.push_back(Item{t, c, w, 0});
          d.v0a_n[w] = (int)L.v0a_items.size() - d.v0a_first[w];
          for (int c = 0; c * kV0bEnt < d.len[w]; ++c) L.v0b_items.push_back(Item{t, c, w, 0});
          if (d.mode == kModeFacND)
            for (int c = 0; c * kV0aEnt < d.len[w]; ++c)
              for (int q = 0; q < d.npart[w]; ++q) L.nd_items.push_back(Item{t, c, w, q});
        }
      }
    }
    const long long chunk = (long long)kThreads * d.vec * kElemIters;
    // P0 items: tiles of 2-D factored tensors; flat chunks only where a global norm is needed
    // (CELO2's AdamW tensors, every other tensor of a PYLO_F_GLOBAL_NORM plan)
    d.p0_first = (int)L.p0_items.size();
    if (n > 0) {
      if (d.mode == kModeFac2D) {
        for (int st = 0; st < d.n_strips; ++st)
          for (int cb = 0; cb < d.n_colblk; ++cb) L.p0_items.push_back(Item{t, st, cb, 0});
      } else if (kind == PYLO_KIND_CELO2 || L.global_norm) {
        for (long long c = 0; c * chunk < n; ++c) L.p0_items.push_back(Item{t, (int)c, 0, 0});
      }
    }
    d.p0_n = (int)L.p0_items.size() - d.p0_first;
    d.blk0 = (int)L.el_items.size();
    const bool wide = d.mode == kModeFac2D && n > 0 && env_matrix_pipe();
    if (kind == PYLO_KIND_CELO2 && (d.mode == kModeFacND || d.mode == kModeVec)) {
      // one pass per slice of the last two dims (k_celo2_slices): 256 slices a block, or 4
      const long long n_slices = n / d.slice_len, per = d.slice_len <= kSliceLaneMax ? kThreads : kWaves;
      if (n_slices >= (1ll << 31)) return fail("plan: too many slices");
      if (d.mode == kModeFacND && d.slice_len <= kSliceLaneMax && env_slices_lds()) {
        // short slices of a tensor with more than two dims: 64 a block, staged through LDS (k_celo2_slices_lane)
        int cls = 0;
        while (d.slice_len > kSliceLaneClassMax[cls]) ++cls;
        for (long long s0 = 0; s0 < n_slices && n > 0; s0 += 64 * slice_lane_groups(d.slice_len))
          L.sl_lane_cls[cls].push_back(Item{t, (int)s0, 0, 0});
        L.sl_lane_lds[cls] = std::max(L.sl_lane_lds[cls], (int)sizeof(float) * 6 * d.slice_len * kSlicePitchF);
      } else
      for (long long s0 = 0; s0 < n_slices && n > 0; s0 += per) L.sl_items.push_back(Item{t, (int)s0, 0, 0});
    } else if (wide && d.C0 % kTileCols == 0) {
      d.tile_nct = d.C0 / kTileCols;
      d.tile_rows = tile_rows_for(kind);
      d.tile_ntask = d.tile_nct * ((d.R0 + d.tile_rows - 1) / d.tile_rows);
      for (int b = 0; b * 4 < d.tile_ntask; ++b) L.el_items.push_back(Item{t, b, 0, 0});
    } else {
      for (long long c = 0; c * chunk < n; ++c) L.el_items.push_back(Item{t, (int)c, 0, 0});
    }
    d.nblk = (int)L.el_items.size() - d.blk0;
    if (d.nblk > kSegMin) {  // two-stage reduction of the statistics partials (k_stat_segsum)
      d.seg0 = (int)L.seg_items.size();
      for (int r = 0; r < d.nblk; r += kSegRows) L.seg_items.push_back(Item{t, r, std::min(kSegRows, d.nblk - r), 0});
      d.nseg = (int)L.seg_items.size() - d.seg0;
    }
    // blocks of AdafacLO's apply pass: one column per lane where the tensor allows it (ap_items,
    // k_adafac_apply_tile), linear chunks otherwise (ga_items, k_adafac_apply)
    if (kind == PYLO_KIND_ADAFAC) {
      // an (O, I, k, ..) tensor factored over its two leading dims (convolution kernels) is the matrix (O, I * P)
      // for this pass, P = product of the trailing dims (pp_items)
      bool periodic = false;
      if (d.mode == kModeFacND && n > 0 && env_matrix_pipe() && env_adafac_hf() && e.ndim >= 3 &&
          ((edr == 0 && edc == 1) || (edr == 1 && edc == 0))) {
        long long P = 1;
        for (int i = 2; i < e.ndim; ++i) P *= e.shape[i];
        if ((e.shape[1] * P) % 64 == 0) {
          periodic = true;
          d.aper = (int)P;
          d.aper_col = edr == 0 ? 0 : 1;   // vector 0 lost dim edr: it is indexed by the column if that dim is O
          d.R0 = (int)e.shape[0];
          d.C0 = (int)(e.shape[1] * P);
        }
      }
      if ((wide && d.C0 % 64 == 0) || periodic) {
        d.atile_nct = d.C0 / 64;
        if (d.tile_rows == 0) d.tile_rows = tile_rows_for(kind);
        d.atile_ntask = d.atile_nct * ((d.R0 + d.tile_rows - 1) / d.tile_rows);
        for (int b = 0; b * 4 < d.atile_ntask; ++b) (periodic ? L.pp_items : L.ap_items).push_back(Item{t, b, 0, 0});
      } else {
        for (long long c = 0; c * chunk < n; ++c) L.ga_items.push_back(Item{t, (int)c, 0, 0});
      }
    }
  }
  if (kind == PYLO_KIND_CELO2 || kind == PYLO_KIND_VELO) build_elem_items(L, T, kind);
  long long ns_floats = 0;
  if (kind == PYLO_KIND_CELO2) {
    L.ns_hf = env_ns_hf();
    build_slice_tables(L, shapes, T);
    build_ns_tables(L, shapes, T, ns_floats);
    if (int rc = build_fin_tables(L, shapes, T)) return rc;
  }
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off = align_up(off + std::max<size_t>(bytes, 16));
    return o;
  };
  const size_t nfac = std::max<size_t>(L.fac_list.size(), 1);
  L.off_descs = take(sizeof(TDesc) * T);
  L.off_dyn = take(sizeof(PyloTensorArgs) * T);
  L.off_dyn_user = L.typed ? take(sizeof(PyloTensorArgs) * T) : L.off_dyn;
  L.off_stage_ofs = take(L.typed ? sizeof(StageOfs) * T : 0);
  L.off_cast_items = take(sizeof(Item) * L.cast_items.size());
  L.off_stage = take(sizeof(float) * (size_t)L.stage_floats);
  L.off_p0_items = take(sizeof(Item) * L.p0_items.size());
  L.off_nd_items = take(sizeof(Item) * L.nd_items.size());
  L.off_sl_items = take(sizeof(Item) * L.sl_items.size());
  for (int c = 0; c < kSliceLaneClasses; ++c) {
    L.sl_lane_n[c] = (int)L.sl_lane_cls[c].size();
    L.sl_lane_items.insert(L.sl_lane_items.end(), L.sl_lane_cls[c].begin(), L.sl_lane_cls[c].end());
    L.sl_lane_cls[c] = std::vector<Item>();
  }
  L.off_sl_lane_items = take(sizeof(Item) * L.sl_lane_items.size());
  L.off_seg_items = take(sizeof(Item) * L.seg_items.size());
  L.off_segtot = take(sizeof(double) * kStatW * L.seg_items.size());
  L.off_el_items = take(sizeof(Item) * L.el_items.size());
  L.off_ap_items = take(sizeof(Item) * L.ap_items.size());
  L.off_pp_items = take(sizeof(Item) * L.pp_items.size());
  L.off_ga_items = take(sizeof(Item) * L.ga_items.size());
  L.off_fin_items = take(sizeof(Item) * L.fin_items.size());
  L.off_finpart = take(sizeof(double) * L.fin_items.size());
  L.off_finscale = take(sizeof(float) * L.fin_units.size());
  L.off_fin_units = take(sizeof(FinUnit) * L.fin_units.size());
  L.off_v0a_items = take(sizeof(Item) * L.v0a_items.size());
  L.off_v0b_items = take(sizeof(Item) * L.v0b_items.size());
  L.off_fac_list = take(sizeof(int) * nfac);
  L.off_part = take(sizeof(float) * part);
  L.off_gsq = take(sizeof(double) * L.p0_items.size());
  L.off_flag = take(sizeof(int) * L.p0_items.size());
  L.off_globals = take(sizeof(Globals));
  L.off_tscale = take(sizeof(float) * (L.tensor_norm ? T : 0));
  L.off_fac = take(sizeof(float) * fac);
  L.off_term = take(sizeof(float) * term);
  L.off_v0part = take(sizeof(double) * kNV0 * L.v0a_items.size());
  L.off_bscale = take(sizeof(BScale) * nfac);
  L.off_stats = take(sizeof(double) * kStatW * L.el_items.size());
  L.off_wfold = take(sizeof(float) * (kind == PYLO_KIND_CELO2 ? kC2Fold * nfac
                                      : kind == PYLO_KIND_VELO ? (size_t)kVFold * T : (size_t)kAFold * T));
  L.off_chan_ms = take(sizeof(float) * kNStat * nfac);
  L.off_totals = take(sizeof(double) * kStatW * T);
  L.Tpad = (T + kGateBT - 1) / kGateBT * kGateBT;
  L.off_xfeat = take(sizeof(float) * kXW * T);
  L.off_lossfeat = take(sizeof(float) * 16);
  L.off_xT = take(kind == PYLO_KIND_VELO ? sizeof(float) * 2 * (size_t)velo_hidden * L.Tpad : 0);
  L.off_mixbuf = take(kind == PYLO_KIND_VELO ? sizeof(float) * 2 * (size_t)velo_hidden * T : 0);
  L.off_pmax = take(kind == PYLO_KIND_VELO ? sizeof(float) * (size_t)velo_hidden * ((T + kMixRows - 1) / kMixRows) : 0);
  L.off_canon = take(kind == PYLO_KIND_VELO ? sizeof(float) * kVCanon * (size_t)T : 0);
  L.off_frac = take(kind == PYLO_KIND_VELO ? sizeof(float) * 9 * PYLO_MAX_GROUPS : 0);
  L.off_mx_items = take(sizeof(Item) * L.mx_items.size());
  // (VeLO: behind the counters, the guard of the carried sums: flag address, padding, T doubles -- k_velo.h)
  L.off_sync = take(sizeof(int) * (size_t)((2 * T + 3) & ~3) + (kind == PYLO_KIND_VELO ? 16 + sizeof(double) * (size_t)T : 0));
  L.off_newsum = take(kind == PYLO_KIND_VELO ? sizeof(double) * kNewSumW * L.el_items.size() : 0);
  L.off_piv = take(kind == PYLO_KIND_VELO ? sizeof(float) * 4 * (size_t)T : 0);
  L.off_wmix = take(kind == PYLO_KIND_VELO ? sizeof(float) * 160 * (size_t)T : 0);
  if (kind == PYLO_KIND_CELO2) {
    L.off_ns_mats = take(sizeof(NsMat) * L.ns_mats.size());
    L.off_ns_gram = take(sizeof(NsItem) * L.ns_gram.size());
    L.off_ns_poly = take(sizeof(NsItem) * L.ns_poly.size());
    L.off_ns_upd = take(sizeof(NsItem) * L.ns_upd.size());
    L.off_ns_upd4 = take(sizeof(NsItem) * L.ns_upd4.size());
    L.off_ns_split = take(sizeof(int) * L.ns_split.size());
    L.off_ns_xalt = take(sizeof(long long) * (size_t)T);
    L.off_ns_scale = take(sizeof(float) * L.ns_mats.size());
    L.off_ns_flags = take(sizeof(int) * L.ns_mats.size());
    L.off_ns_fpart = take(sizeof(float) * (size_t)L.ns_fpart_total);
    L.off_ns_flag_items = take(sizeof(Item) * L.ns_flag_items.size());
    L.off_ns_ws = take(sizeof(float) * (size_t)ns_floats);
    L.off_nsb_mats = take(sizeof(NsHfMat) * L.nsb_mats.size());
    L.off_nsb_split_items = take(sizeof(NsTileItem) * L.nsb_split_items.size());
    L.off_ns_list = take(sizeof(int) * L.ns_list.size());
    L.off_ns_pw = take(sizeof(hbits) * (size_t)L.nsb_plane_elems);
    L.off_slice_mats = take(sizeof(SliceMat) * L.slice_mats.size());
    for (int k = 0; k < kSliceLaneSets; ++k) L.off_slice_items_l[k] = take(sizeof(Item) * L.slice_items_l[k].size());
    L.off_slice_items_w = take(sizeof(Item) * L.slice_items_w.size());
    L.off_slice_items_b = take(sizeof(Item) * L.slice_items_b.size());
  }
  L.total = off;
  return 0;
}

constexpr int kStageSlots = PYLO_ARG_TABLES;
constexpr int kVeloHiddenMax = 1024;  // workspace is sized for LSTM widths up to this

}  // namespace

struct PyloPlan {
  int kind = 0, T = 0;
  Layout L;
  char* ws = nullptr;
  PyloTensorArgs* stage[kStageSlots] = {nullptr, nullptr, nullptr, nullptr};
  hipEvent_t ev[kStageSlots] = {nullptr, nullptr, nullptr, nullptr};
  bool ev_used[kStageSlots] = {false, false, false, false};
  bool handed[kStageSlots] = {false, false, false, false};  // given to the caller by plan_arg_table
  int slot = 0;
  PyloDeviceSteps dsteps = {nullptr, 0.0, 0.0, 1.0};
  std::vector<PyloTensorArgs> last;
  size_t last_dst = 0;   // where `last` was copied to
  bool have_last = false;
  bool mlp_on_matrix_pipe = true;  // env_matrix_pipe() when the plan was created
  bool adafac_hf = true;           // AdafacLO's element MLP on the fp16 matrix instructions (PYLO_MI355_ADAFAC_F32=1: fp32 ones)
  // optional per-launch timing (pylo_mi355_plan_timing_begin/end)
  std::vector<hipEvent_t> tev;
  int t_steps_max = 0, t_steps = 0, t_per_step = 0;
  bool timing = false;
  // VeLO: the LSTM's input sums were left by the previous step's apply items (see k_velo_elem); false
  // until a step has run and after pylo_mi355_plan_invalidate_statistics
  bool stats_carried = false;
  // the guard of those sums: 1 + tensor in pinned host memory that the kernel writes straight into when it catches a
  // mismatch (nothing is copied on the steps that find none; pylo_mi355_plan_invalidate_statistics clears it), and
  // its address as the device sees it
  int* stale_host = nullptr;
  int* stale_dev = nullptr;
  hipStream_t side = nullptr;            // the LSTM runs next to the gradient sums on a stream of the plan's own
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  // ELO-CELO2: the Newton-Schulz chains of the groups of matrices after the first run on streams of the plan's own
  hipStream_t ns_side[3] = {nullptr, nullptr, nullptr};
  hipEvent_t ns_fork = nullptr, ns_join[3] = {nullptr, nullptr, nullptr};
  // the per-slice finishing launches next to the matrices' products, where the groups leave a hardware queue free
  hipStream_t slice_side = nullptr;
  hipEvent_t slice_fork = nullptr, slice_join = nullptr;

  template <class Tp>
  Tp* at(size_t off) const { return reinterpret_cast<Tp*>(ws + off); }
};

extern "C" {

int pylo_mi355_abi_version(void) { return PYLO_MI355_ABI_VERSION; }

const char* pylo_mi355_last_error(void) { return g_err.c_str(); }

int pylo_mi355_plan_workspace_bytes(int kind, const PyloTensorShape* shapes, int n_tensors, size_t* bytes_out) {
  if (!bytes_out) return fail("workspace_bytes: null output");
  Layout L;
  if (int rc = build_layout(kind, shapes, n_tensors, L, kVeloHiddenMax)) return rc;
  *bytes_out = L.total;
  return 0;
}

int pylo_mi355_plan_create(int kind, const PyloTensorShape* shapes, int n_tensors, void* workspace,
                           size_t workspace_bytes, void* stream, PyloPlan** plan_out) {
  if (!plan_out) return fail("plan_create: null output");
  *plan_out = nullptr;
  PyloPlan* P = new PyloPlan();
  P->kind = kind;
  P->T = n_tensors;
  P->mlp_on_matrix_pipe = env_matrix_pipe();
  P->adafac_hf = env_adafac_hf();
  if (int rc = build_layout(kind, shapes, n_tensors, P->L, kVeloHiddenMax)) { delete P; return rc; }
  if (workspace == nullptr || workspace_bytes < P->L.total) { delete P; return fail("plan_create: workspace too small"); }
  if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0) { delete P; return fail("plan_create: workspace must be 256-byte aligned"); }
  P->ws = static_cast<char*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Layout& L = P->L;
  auto up = [&](size_t off, const void* src, size_t bytes) -> hipError_t {
    if (bytes == 0) return hipSuccess;
    return hipMemcpyAsync(P->ws + off, src, bytes, hipMemcpyHostToDevice, s);
  };
  hipError_t e = hipSuccess;
  if (e == hipSuccess) e = up(L.off_descs, L.descs.data(), sizeof(TDesc) * L.descs.size());
  if (e == hipSuccess) e = up(L.off_p0_items, L.p0_items.data(), sizeof(Item) * L.p0_items.size());
  if (e == hipSuccess && L.typed) e = up(L.off_stage_ofs, L.stage_ofs.data(), sizeof(StageOfs) * L.stage_ofs.size());
  if (e == hipSuccess) e = up(L.off_cast_items, L.cast_items.data(), sizeof(Item) * L.cast_items.size());
  if (e == hipSuccess) e = up(L.off_nd_items, L.nd_items.data(), sizeof(Item) * L.nd_items.size());
  if (e == hipSuccess) e = up(L.off_sl_items, L.sl_items.data(), sizeof(Item) * L.sl_items.size());
  if (e == hipSuccess) e = up(L.off_sl_lane_items, L.sl_lane_items.data(), sizeof(Item) * L.sl_lane_items.size());
  if (e == hipSuccess) e = up(L.off_seg_items, L.seg_items.data(), sizeof(Item) * L.seg_items.size());
  if (e == hipSuccess) e = up(L.off_el_items, L.el_items.data(), sizeof(Item) * L.el_items.size());
  if (e == hipSuccess) e = up(L.off_ap_items, L.ap_items.data(), sizeof(Item) * L.ap_items.size());
  if (e == hipSuccess) e = up(L.off_pp_items, L.pp_items.data(), sizeof(Item) * L.pp_items.size());
  if (e == hipSuccess) e = up(L.off_ga_items, L.ga_items.data(), sizeof(Item) * L.ga_items.size());
  if (e == hipSuccess) e = up(L.off_fin_items, L.fin_items.data(), sizeof(Item) * L.fin_items.size());
  if (e == hipSuccess) e = up(L.off_fin_units, L.fin_units.data(), sizeof(FinUnit) * L.fin_units.size());
  if (e == hipSuccess) e = up(L.off_fac_list, L.fac_list.data(), sizeof(int) * L.fac_list.size());
  if (e == hipSuccess) e = up(L.off_v0a_items, L.v0a_items.data(), sizeof(Item) * L.v0a_items.size());
  if (e == hipSuccess) e = up(L.off_v0b_items, L.v0b_items.data(), sizeof(Item) * L.v0b_items.size());
  if (e == hipSuccess) e = up(L.off_mx_items, L.mx_items.data(), sizeof(Item) * L.mx_items.size());
  if (e == hipSuccess) e = up(L.off_ns_mats, L.ns_mats.data(), sizeof(NsMat) * L.ns_mats.size());
  if (e == hipSuccess) e = up(L.off_ns_gram, L.ns_gram.data(), sizeof(NsItem) * L.ns_gram.size());
  if (e == hipSuccess) e = up(L.off_ns_poly, L.ns_poly.data(), sizeof(NsItem) * L.ns_poly.size());
  if (e == hipSuccess) e = up(L.off_ns_upd, L.ns_upd.data(), sizeof(NsItem) * L.ns_upd.size());
  if (e == hipSuccess) e = up(L.off_ns_upd4, L.ns_upd4.data(), sizeof(NsItem) * L.ns_upd4.size());
  if (e == hipSuccess) e = up(L.off_ns_split, L.ns_split.data(), sizeof(int) * L.ns_split.size());
  if (e == hipSuccess && kind == PYLO_KIND_CELO2) e = up(L.off_ns_xalt, L.ns_xalt.data(), sizeof(long long) * L.ns_xalt.size());
  if (e == hipSuccess) e = up(L.off_nsb_mats, L.nsb_mats.data(), sizeof(NsHfMat) * L.nsb_mats.size());
  if (e == hipSuccess) e = up(L.off_nsb_split_items, L.nsb_split_items.data(), sizeof(NsTileItem) * L.nsb_split_items.size());
  if (e == hipSuccess) e = up(L.off_ns_list, L.ns_list.data(), sizeof(int) * L.ns_list.size());
  if (e == hipSuccess) e = up(L.off_ns_flag_items, L.ns_flag_items.data(), sizeof(Item) * L.ns_flag_items.size());
  if (e == hipSuccess) e = up(L.off_slice_mats, L.slice_mats.data(), sizeof(SliceMat) * L.slice_mats.size());
  for (int k = 0; k < kSliceLaneSets; ++k)
    if (e == hipSuccess) e = up(L.off_slice_items_l[k], L.slice_items_l[k].data(), sizeof(Item) * L.slice_items_l[k].size());
  if (e == hipSuccess) e = up(L.off_slice_items_w, L.slice_items_w.data(), sizeof(Item) * L.slice_items_w.size());
  if (e == hipSuccess) e = up(L.off_slice_items_b, L.slice_items_b.data(), sizeof(Item) * L.slice_items_b.size());
  // the padding of the operand planes is read by the products and written by nobody: zero, once
  if (e == hipSuccess && L.nsb_plane_elems > 0)
    e = hipMemsetAsync(P->ws + L.off_ns_pw, 0, sizeof(hbits) * (size_t)L.nsb_plane_elems, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  for (int i = 0; i < kStageSlots && e == hipSuccess; ++i) {
    e = hipHostMalloc(reinterpret_cast<void**>(&P->stage[i]), (sizeof(PyloTensorArgs) * n_tensors + 15) / 16 * 16,
                      hipHostMallocDefault);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->ev[i], hipEventDisableTiming);
  }
  if (e == hipSuccess && kind == PYLO_KIND_VELO) {
    e = hipHostMalloc(reinterpret_cast<void**>(&P->stale_host), 64, hipHostMallocMapped);
    if (e == hipSuccess) P->stale_host[0] = P->stale_host[1] = 0;
    if (e == hipSuccess) e = hipHostGetDevicePointer(reinterpret_cast<void**>(&P->stale_dev), P->stale_host, 0);
    if (e == hipSuccess) {   // its address, where the kernels look for it (behind the counters of `sync`)
      const long long addr = reinterpret_cast<long long>(P->stale_dev);
      e = hipMemcpyAsync(P->ws + L.off_sync + sizeof(int) * (size_t)((2 * n_tensors + 3) & ~3), &addr, sizeof(addr),
                         hipMemcpyHostToDevice, s);
      if (e == hipSuccess) e = hipStreamSynchronize(s);
    }
  }
  if (e == hipSuccess && kind == PYLO_KIND_VELO && !P->L.mx_items.empty()) {
    e = hipStreamCreateWithFlags(&P->side, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->ev_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->ev_join, hipEventDisableTiming);
  }
  size_t ns_streams = 0;
  for (const NsBatch& bt : L.ns_batches) ns_streams = std::max<size_t>(ns_streams, bt.n_groups);
  for (size_t g = 1; g < ns_streams && e == hipSuccess; ++g) {
    if (g == 1) e = hipEventCreateWithFlags(&P->ns_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&P->ns_side[g - 1], hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->ns_join[g - 1], hipEventDisableTiming);
  }
  bool plan_has_slices = !L.slice_items_w.empty() || !L.slice_items_b.empty();
  for (const auto& v : L.slice_items_l) plan_has_slices = plan_has_slices || !v.empty();
  if (e == hipSuccess && plan_has_slices && ns_streams >= 1 && ns_streams <= 3) {   // main + groups + this one <= 4 queues
    e = hipStreamCreateWithFlags(&P->slice_side, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->slice_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->slice_join, hipEventDisableTiming);
  }
  if (e != hipSuccess) {
    pylo_mi355_plan_destroy(P);
    return fail(std::string("plan_create: ") + hipGetErrorString(e));
  }
  *plan_out = P;
  return 0;
}

int pylo_mi355_plan_destroy(PyloPlan* P) {
  if (!P) return 0;
  for (hipEvent_t e : P->tev) (void)hipEventDestroy(e);
  if (P->ev_fork) (void)hipEventDestroy(P->ev_fork);
  if (P->ev_join) (void)hipEventDestroy(P->ev_join);
  if (P->side) (void)hipStreamDestroy(P->side);
  if (P->stale_host) (void)hipHostFree(P->stale_host);
  if (P->ns_fork) (void)hipEventDestroy(P->ns_fork);
  if (P->slice_fork) (void)hipEventDestroy(P->slice_fork);
  if (P->slice_join) (void)hipEventDestroy(P->slice_join);
  if (P->slice_side) (void)hipStreamDestroy(P->slice_side);
  for (int g = 0; g < 3; ++g) {
    if (P->ns_join[g]) (void)hipEventDestroy(P->ns_join[g]);
    if (P->ns_side[g]) (void)hipStreamDestroy(P->ns_side[g]);
  }
  for (int i = 0; i < kStageSlots; ++i) {
    if (P->ev[i]) (void)hipEventDestroy(P->ev[i]);
    if (P->stage[i]) (void)hipHostFree(P->stage[i]);
  }
  delete P;
  return 0;
}

static const char* kCelo2Launches[] = {"k_p0(sums)", "k_gnorm", "k_p0(exact)", "k_v0a", "k_v0b",
                                       "k_celo2_stats", "k_celo2_fold", "k_celo2_apply"};
static const char* kCelo2FusedLaunches[] = {"k_p0(sums)", "k_gnorm", "k_p0(exact)", "k_v0a", "k_v0b",
                                            "k_celo2_elem", "k_celo2_slices"};
static const char* kVeloLaunches[] = {"k_p0(sums)", "k_p0_nd", "k_v0a", "k_v0b", "k_velo_stats",
                                      "k_lo_reduce", "k_velo_mix", "k_velo_gates", "k_velo_heads", "k_terms",
                                      "k_velo_apply"};

static const char* kVeloFusedLaunches[] = {"k_p0(sums) | LSTM", "k_v0a", "k_v0b", "k_terms", "k_velo_elem"};
static const char* kAdafacLaunches[] = {"k_p0(sums)", "k_p0_nd", "k_v0a", "k_adafac_bias", "k_v0b", "k_adafac_stats",
                                        "k_lo_reduce", "k_adafac_fold", "k_adafac_apply"};

int pylo_mi355_plan_num_launches(const PyloPlan* P) {
  if (!P) return -1;
  const int n_celo2 = P->L.mx_items.empty() ? (int)(sizeof(kCelo2Launches) / sizeof(kCelo2Launches[0]))
                                            : (int)(sizeof(kCelo2FusedLaunches) / sizeof(kCelo2FusedLaunches[0]));
  const int n_velo = P->L.mx_items.empty() ? (int)(sizeof(kVeloLaunches) / sizeof(kVeloLaunches[0]))
                                           : (int)(sizeof(kVeloFusedLaunches) / sizeof(kVeloFusedLaunches[0]));
  constexpr int n_adafac = sizeof(kAdafacLaunches) / sizeof(kAdafacLaunches[0]);
  return P->kind == PYLO_KIND_CELO2 ? n_celo2 : P->kind == PYLO_KIND_VELO ? n_velo : P->kind == PYLO_KIND_ADAFAC ? n_adafac : -1;
}

const char* pylo_mi355_plan_launch_name(const PyloPlan* P, int launch) {
  if (!P || launch < 0 || launch >= pylo_mi355_plan_num_launches(P)) return "";
  return P->kind == PYLO_KIND_CELO2 ? (P->L.mx_items.empty() ? kCelo2Launches[launch] : kCelo2FusedLaunches[launch])
         : P->kind == PYLO_KIND_VELO ? (P->L.mx_items.empty() ? kVeloLaunches[launch] : kVeloFusedLaunches[launch])
                                     : kAdafacLaunches[launch];
}

int pylo_mi355_plan_timing_begin(PyloPlan* P, int max_steps) {
  if (!P || max_steps <= 0) return fail("timing_begin: bad argument");
  const int per = pylo_mi355_plan_num_launches(P) + 1;
  for (hipEvent_t e : P->tev) (void)hipEventDestroy(e);
  P->tev.assign((size_t)per * max_steps, nullptr);
  for (auto& e : P->tev) HIP_TRY(hipEventCreate(&e));
  P->t_steps_max = max_steps;
  P->t_steps = 0;
  P->t_per_step = per;
  P->timing = true;
  return 0;
}

int pylo_mi355_plan_timing_end(PyloPlan* P, float* ms_out, int capacity, int* steps_out) {
  if (!P || !ms_out || !steps_out) return fail("timing_end: bad argument");
  P->timing = false;
  const int nl = P->t_per_step - 1;
  const int steps = P->t_steps;
  if (capacity < steps * nl) return fail("timing_end: output too small");
  if (steps > 0) HIP_TRY(hipEventSynchronize(P->tev[(size_t)steps * P->t_per_step - 1]));
  for (int s = 0; s < steps; ++s)
    for (int k = 0; k < nl; ++k) {
      float ms = 0.0f;
      HIP_TRY(hipEventElapsedTime(&ms, P->tev[(size_t)s * P->t_per_step + k], P->tev[(size_t)s * P->t_per_step + k + 1]));
      ms_out[s * nl + k] = ms;
    }
  *steps_out = steps;
  return 0;
}

int pylo_mi355_plan_arg_table(PyloPlan* P, int slot, PyloTensorArgs** table_out) {
  if (!P || !table_out || slot < 0 || slot >= kStageSlots) return fail("plan_arg_table: bad argument");
  // a staged copy out of this slot may still be pending on the device
  if (P->ev_used[slot]) HIP_TRY(hipEventSynchronize(P->ev[slot]));
  P->handed[slot] = true;
  *table_out = P->stage[slot];
  return 0;
}

int pylo_mi355_plan_device_steps(PyloPlan* P, const PyloDeviceSteps* steps) {
  if (!P) return fail("plan_device_steps: null plan");
  if (!steps || !steps->counters) {
    P->dsteps = PyloDeviceSteps{nullptr, 0.0, 0.0, 1.0};
    return 0;
  }
  if (reinterpret_cast<uintptr_t>(steps->counters) % 4 != 0) return fail("plan_device_steps: misaligned counters");
  if (P->kind == PYLO_KIND_VELO && !(steps->num_steps > 0.0)) return fail("plan_device_steps: num_steps must be positive");
  P->dsteps = *steps;
  return 0;
}

int pylo_mi355_plan_factored_dims(const PyloPlan* P, int tensor, int* dc, int* dr) {
  if (!P || tensor < 0 || tensor >= P->T || !dc || !dr) return fail("factored_dims: bad argument");
  *dc = P->L.dc[tensor];
  *dr = P->L.dr[tensor];
  return 0;
}

}  // extern "C"

namespace {

// Copies the per-step argument table to the device through a ring of pinned slots; skipped when
// the table is byte-identical to the one already resident.
// The per-step argument table goes from pinned host memory to the workspace with a small kernel on
// the launch stream: an async memcpy on the same stream costs a hand-over to the copy engine and back
// (about 0.1 ms of idle GPU between two steps), a kernel reading 10 KB over the host link does not.
__global__ __launch_bounds__(256) void k_copy_args(const uint4* __restrict__ src, uint4* __restrict__ dst, int n16) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n16; i += gridDim.x * 256) dst[i] = src[i];
}

// `dst_off`: where the table goes, the records the kernels read (off_dyn) or, for a step of a plan with
// tensors of other storage types, the caller's records that k_stage_args copies from (off_dyn_user).
int upload_args(PyloPlan* P, const PyloTensorArgs* args, hipStream_t s, size_t dst_off) {
  const size_t bytes = sizeof(PyloTensorArgs) * P->T;
  static_assert(sizeof(PyloTensorArgs) % 8 == 0, "argument records are copied in 16-byte pieces");
  const int n16 = (int)((bytes + 15) / 16);
  const dim3 grid(std::min(64, (n16 + 255) / 256));
  for (int j = 0; j < kStageSlots; ++j) {
    if (args != P->stage[j]) continue;
    // one of the plan's own pinned tables: read in place when the kernel runs (a graph replay sees the
    // table as it is then); nothing on the host side depends on earlier calls
    void* src_dev = nullptr;
    HIP_TRY(hipHostGetDevicePointer(&src_dev, P->stage[j], 0));
    hipLaunchKernelGGL(k_copy_args, grid, dim3(256), 0, s, static_cast<const uint4*>(src_dev),
                       reinterpret_cast<uint4*>(P->ws + dst_off), n16);
    P->have_last = false;
    return 0;
  }
  if (P->have_last && P->last_dst == dst_off && std::memcmp(P->last.data(), args, bytes) == 0) return 0;
  int i = -1;
  for (int k = 0; k < kStageSlots && i < 0; ++k) {
    const int c = (P->slot + k) % kStageSlots;
    if (!P->handed[c]) i = c;
  }
  if (i < 0) return fail("step: every argument table of the plan has been handed out; call with one of them");
  P->slot = (i + 1) % kStageSlots;
  if (P->ev_used[i]) HIP_TRY(hipEventSynchronize(P->ev[i]));
  std::memcpy(P->stage[i], args, bytes);
  void* src_dev = nullptr;
  HIP_TRY(hipHostGetDevicePointer(&src_dev, P->stage[i], 0));
  hipLaunchKernelGGL(k_copy_args, grid, dim3(256), 0, s,
                     static_cast<const uint4*>(src_dev), reinterpret_cast<uint4*>(P->ws + dst_off), n16);
  HIP_TRY(hipEventRecord(P->ev[i], s));
  P->ev_used[i] = true;
  P->last.assign(args, args + P->T);
  P->last_dst = dst_off;
  P->have_last = true;
  return 0;
}

// Step of a plan with tagged tensors: the records the kernels read are the caller's with grad / param of the
// tagged tensors redirected into the staging, which is filled here.  `what`: 1 gradient, 2 parameter, 3 both.
void stage_in(PyloPlan* P, hipStream_t s, int what) {
  const Layout& L = P->L;
  if (!L.typed) return;
  hipLaunchKernelGGL(k_stage_args, dim3((P->T + 255) / 256), dim3(256), 0, s, P->T, P->at<TDesc>(L.off_descs),
                     P->at<PyloTensorArgs>(L.off_dyn_user), P->at<PyloTensorArgs>(L.off_dyn),
                     P->at<StageOfs>(L.off_stage_ofs), P->at<float>(L.off_stage));
  hipLaunchKernelGGL(k_cast_in, dim3((unsigned)L.cast_items.size()), dim3(kThreads), 0, s, P->at<TDesc>(L.off_descs),
                     P->at<PyloTensorArgs>(L.off_dyn_user), P->at<Item>(L.off_cast_items),
                     P->at<StageOfs>(L.off_stage_ofs), P->at<float>(L.off_stage), what);
}

void stage_out(PyloPlan* P, hipStream_t s, int flat_only) {
  const Layout& L = P->L;
  if (!L.typed) return;
  hipLaunchKernelGGL(k_cast_out, dim3((unsigned)L.cast_items.size()), dim3(kThreads), 0, s, P->at<TDesc>(L.off_descs),
                     P->at<PyloTensorArgs>(L.off_dyn_user), P->at<Item>(L.off_cast_items),
                     P->at<StageOfs>(L.off_stage_ofs), P->at<float>(L.off_stage), flat_only);
}

// Step counters kept on the device: advances them and writes what the host otherwise supplies per
// step into the device copy of the argument table (bias corrections, AdafacLO's counter) or into
// the VeLO time-feature buffer.  One thread per tensor (VeLO: per group).
__global__ __launch_bounds__(256) void k_advance_steps(int kind, int T, const TDesc* __restrict__ descs,
                                                       PyloTensorArgs* __restrict__ dyn, PyloDeviceSteps ds,
                                                       float* __restrict__ frac_out) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (kind == PYLO_KIND_VELO) {
    if (t >= PYLO_MAX_GROUPS) return;
    const float ts[9] = {0.03f, 0.1f, 0.2f, 0.4f, 0.6f, 0.8f, 0.9f, 1.0f, 1.1f};
    const int c = ds.counters[t];
    const float x = (float)((double)c / ds.num_steps);
#pragma unroll
    for (int q = 0; q < 9; ++q) frac_out[t * 9 + q] = tanhf((x - ts[q]) * 10.0f);
    ds.counters[t] = c + 1;
    return;
  }
  if (t >= T) return;
  const bool has_grad = dyn[t].grad != nullptr;
  if (kind == PYLO_KIND_ADAFAC) {
    if (!has_grad) return;
    const int c = ds.counters[t];
    dyn[t].bc1 = (float)c;
    ds.counters[t] = c + 1;
    return;
  }
  // CELO2 kind: a per-parameter counter (independent AdamW moments) sits a step out with its tensor,
  // the others count the calls like the reference's per-group counter
  if (descs[t].adam_indep && !has_grad) return;
  const int c = ds.counters[t] + 1;
  ds.counters[t] = c;
  if (descs[t].mode != kModeFlat) return;
  dyn[t].bc1 = (float)(1.0 - pow(ds.beta1, (double)c));
  dyn[t].bc2 = (float)(1.0 - pow(ds.beta2, (double)c));
}

void advance_steps(PyloPlan* P, hipStream_t s) {
  if (!P->dsteps.counters) return;
  const int n = P->kind == PYLO_KIND_VELO ? PYLO_MAX_GROUPS : P->T;
  hipLaunchKernelGGL(k_advance_steps, dim3((n + 255) / 256), dim3(256), 0, s, P->kind, P->T,
                     P->at<TDesc>(P->L.off_descs), P->at<PyloTensorArgs>(P->L.off_dyn), P->dsteps,
                     P->kind == PYLO_KIND_VELO ? P->at<float>(P->L.off_frac) : nullptr);
}

int check_args(const PyloPlan* P, const PyloTensorArgs* args, bool need_all_grads) {
  for (int t = 0; t < P->T; ++t) {
    const TDesc& d = P->L.descs[t];
    const PyloTensorArgs& a = args[t];
    const std::string at = " at tensor " + std::to_string(t);
    if (a.grad == nullptr) {
      // an empty tensor has no gradient buffer to point to; its LSTM row sees zero statistics
      if (need_all_grads && d.n > 0) return fail("step: every tensor needs a gradient" + at);
      continue;
    }
    if (d.n == 0) continue;
    if (!a.param || !a.mom || !a.rms) return fail("step: null param/mom/rms pointer" + at);
    const bool factored = d.mode == kModeFac2D || d.mode == kModeFacND;
    if (factored && (!a.fac_r || !a.fac_c)) return fail("step: null fac_r/fac_c pointer" + at);
    if ((factored || d.mode == kModeVec) && P->kind == PYLO_KIND_CELO2 && !a.step_out)
      return fail("step: null step_out pointer" + at);
    if (d.mode == kModeVec && !a.fac_v) return fail("step: null fac_v pointer" + at);
    if (a.group < 0 || a.group >= PYLO_MAX_GROUPS) return fail("step: group index out of range" + at);
    const uintptr_t m = reinterpret_cast<uintptr_t>(a.grad) | reinterpret_cast<uintptr_t>(a.param) |
                        reinterpret_cast<uintptr_t>(a.mom) | reinterpret_cast<uintptr_t>(a.rms) |
                        reinterpret_cast<uintptr_t>(a.fac_r) | reinterpret_cast<uintptr_t>(a.fac_c) |
                        reinterpret_cast<uintptr_t>(a.fac_v) | reinterpret_cast<uintptr_t>(a.step_out);
    if (m % (d.vec == 4 ? 16 : 4) != 0) return fail("step: misaligned pointer (16 bytes needed)" + at);
    const uintptr_t gp = reinterpret_cast<uintptr_t>(a.grad) | reinterpret_cast<uintptr_t>(a.param);
    if (d.store != kStoreF32 && gp % 16 != 0)
      return fail("step: grad / param of a tensor with a storage type tag must be 16-byte aligned" + at);
  }
  return 0;
}

// The sums of g^2 of a globally clipped 2-D tensor are taken on the raw gradient and scaled afterwards;
// that is exact unless some scaled element lies beyond the tensor's clamp, in which case a second
// pass redoes them (k_p0, pass 1).  The scaled gradient is bounded by the global norm times the scale,
// i.e. by clip_norm, so with clip_norm below clip_val (1.0 against 1000 by default) the second pass can
// never be needed and is not launched.  Tensors whose NaNs are replaced always keep it.
bool exact_pass_possible(const PyloPlan* P, const PyloTensorArgs* args) {
  for (int t = 0; t < P->T; ++t) {
    const PyloTensorArgs& a = args[t];
    if (a.grad == nullptr || !(a.clip_norm > 0.0f)) continue;
    if (P->L.descs[t].nan0) return true;
    if (a.clip_val > 0.0f && !(a.clip_norm <= 0.99f * a.clip_val)) return true;
  }
  return false;
}

struct Marks {  // per-launch HIP events when timing is on
  PyloPlan* P;
  hipStream_t s;
  hipEvent_t* ev;
  int mark = 0;
  Marks(PyloPlan* P_, hipStream_t s_) : P(P_), s(s_) {
    const bool timed = P->timing && P->t_steps < P->t_steps_max;
    ev = timed ? &P->tev[(size_t)P->t_steps * P->t_per_step] : nullptr;
  }
  hipError_t operator()() { return ev ? hipEventRecord(ev[mark++], s) : hipSuccess; }
  void done() { if (ev) P->t_steps++; }
};

}  // namespace

extern "C" int pylo_mi355_celo2_step(PyloPlan* P, const PyloTensorArgs* args, const PyloDecays* decays,
                                     const float* mlp, void* stream) {
  if (!P || !args || !decays || !mlp) return fail("celo2_step: null argument");
  if (P->kind != PYLO_KIND_CELO2) return fail("celo2_step: plan is not a CELO2 plan");
  if (int rc = check_args(P, args, false)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = upload_args(P, args, s, P->L.off_dyn_user)) return rc;
  stage_in(P, s, 3);
  advance_steps(P, s);
  const Layout& L = P->L;
  const TDesc* descs = P->at<TDesc>(L.off_descs);
  const PyloTensorArgs* dyn = P->at<PyloTensorArgs>(L.off_dyn);
  const Item* p0_items = P->at<Item>(L.off_p0_items);
  const Item* el_items = P->at<Item>(L.off_el_items);
  const Item* v0a_items = P->at<Item>(L.off_v0a_items);
  const Item* v0b_items = P->at<Item>(L.off_v0b_items);
  const Item* nd_items = P->at<Item>(L.off_nd_items);
  const Item* sl_items = P->at<Item>(L.off_sl_items);
  const int n_nd = (int)L.nd_items.size(), n_sl = (int)L.sl_items.size();
  const int* fac_list = P->at<int>(L.off_fac_list);
  float* part = P->at<float>(L.off_part);
  double* gsq = P->at<double>(L.off_gsq);
  int* flag = P->at<int>(L.off_flag);
  Globals* gl = P->at<Globals>(L.off_globals);
  float* fac_tab = P->at<float>(L.off_fac);
  float* term_tab = P->at<float>(L.off_term);
  double* v0part = P->at<double>(L.off_v0part);
  BScale* bscale = P->at<BScale>(L.off_bscale);
  double* stats = P->at<double>(L.off_stats);
  float* wfold = P->at<float>(L.off_wfold);
  float* chan_ms = P->at<float>(L.off_chan_ms);
  const int n_p0 = (int)L.p0_items.size(), n_el = (int)L.el_items.size(), n_fac = (int)L.fac_list.size();
  const int n_v0a = (int)L.v0a_items.size(), n_v0b = (int)L.v0b_items.size();
  const PyloDecays dec = *decays;
  Marks mark(P, s);

  const bool exact_pass = exact_pass_possible(P, args);
  HIP_TRY(mark());
  if (n_p0 > 0)
    hipLaunchKernelGGL(k_p0, dim3(n_p0), dim3(kThreads), 0, s, descs, dyn, p0_items, part, gsq, flag, gl, 0,
                       (const Item*)nullptr, n_p0);
  HIP_TRY(mark());
  hipLaunchKernelGGL(k_gnorm, dim3(1), dim3(kThreads), 0, s, gsq, flag, n_p0, gl, exact_pass ? 1 : 0,
                     P->at<int>(L.off_sync), 2 * P->T);
  HIP_TRY(mark());
  if (n_p0 > 0 && exact_pass)
    hipLaunchKernelGGL(k_p0, dim3(n_p0), dim3(kThreads), 0, s, descs, dyn, p0_items, part, gsq, flag, gl, 1,
                       (const Item*)nullptr, n_p0);
  if (n_nd > 0) hipLaunchKernelGGL(k_p0_nd, dim3(n_nd), dim3(kThreads), 0, s, descs, dyn, nd_items, part, gl);
  HIP_TRY(mark());
  if (n_v0a > 0)
    hipLaunchKernelGGL(k_v0a, dim3(n_v0a), dim3(kV0aThreads), 0, s, descs, dyn, v0a_items, part, gl, dec, v0part);
  HIP_TRY(mark());
  if (n_v0b > 0)
    hipLaunchKernelGGL(k_v0b<8>, dim3(n_v0b), dim3(kThreads), 0, s, descs, dyn, v0b_items, v0part, 1e-9f, mlp,
                       mlp + 240, 0, fac_tab, term_tab, bscale);
  HIP_TRY(mark());
  const int n_mx = (int)L.mx_items.size();
  if (n_mx > 0) {
    const Item* mx_items = P->at<Item>(L.off_mx_items);
    int* sync = P->at<int>(L.off_sync);
    if (P->mlp_on_matrix_pipe)
      hipLaunchKernelGGL(k_celo2_elem<true>, dim3(n_mx), dim3(kThreads), 0, s, descs, dyn, mx_items, fac_tab, term_tab,
                         gl, dec, mlp, wfold, chan_ms, stats, sync, P->T);
    else
      hipLaunchKernelGGL(k_celo2_elem<false>, dim3(n_mx), dim3(kThreads), 0, s, descs, dyn, mx_items, fac_tab, term_tab,
                         gl, dec, mlp, wfold, chan_ms, stats, sync, P->T);
    HIP_TRY(mark());
  } else {
    if (n_el > 0) hipLaunchKernelGGL(k_celo2_stats, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac_tab, gl, dec, stats);
    HIP_TRY(mark());
    const Item* seg_items = P->at<Item>(L.off_seg_items);
    double* seg_tot = P->at<double>(L.off_segtot);
    const int n_seg = (int)L.seg_items.size();
    if (n_seg > 0) hipLaunchKernelGGL(k_stat_segsum, dim3(n_seg), dim3(kThreads), 0, s, descs, seg_items, stats, seg_tot);
    if (n_fac > 0)
      hipLaunchKernelGGL(k_celo2_fold, dim3(n_fac), dim3(kFoldThreads), 0, s, descs, dyn, fac_list, stats, seg_tot, mlp, wfold,
                         chan_ms);
    HIP_TRY(mark());
    if (n_el > 0) {
      if (P->mlp_on_matrix_pipe)
        hipLaunchKernelGGL(k_celo2_apply<true>, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac_tab,
                           term_tab, gl, dec, wfold);
      else
        hipLaunchKernelGGL(k_celo2_apply<false>, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac_tab,
                           term_tab, gl, dec, wfold);
    }
  }
  if (n_sl > 0)
    hipLaunchKernelGGL(k_celo2_slices, dim3(n_sl), dim3(kThreads), 0, s, descs, dyn, sl_items, fac_tab, gl, dec, mlp);
  for (int c = 0, at = 0; c < kSliceLaneClasses; at += L.sl_lane_n[c], ++c)
    if (L.sl_lane_n[c] > 0)
      hipLaunchKernelGGL(k_celo2_slices_lane, dim3((unsigned)L.sl_lane_n[c]), dim3(64), L.sl_lane_lds[c], s, descs, dyn,
                         P->at<Item>(L.off_sl_lane_items) + at, fac_tab, gl, dec, mlp);
  HIP_TRY(mark());
  mark.done();
  stage_out(P, s, 1);   // only the AdamW tensors were updated
  HIP_TRY(hipGetLastError());
  return 0;
}

namespace {

// The split-fp16 product kernels take their LDS as dynamic shared memory; tiles of 256 columns need more than
// the 64 KB a kernel may have without asking.
int ns_hf_lds_once() {
  static std::mutex mu;
  static std::vector<int> done;   // devices on which the attribute has been set
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (int d : done)
    if (d == dev) return 0;
  HIP_TRY(hipFuncSetAttribute((const void*)k_ns_hf_gemm<kNsGram, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(2)));
  HIP_TRY(hipFuncSetAttribute((const void*)k_ns_hf_gemm<kNsPoly, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(2)));
  HIP_TRY(hipFuncSetAttribute((const void*)k_ns_hf_gemm<kNsProd, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(2)));
  HIP_TRY(hipFuncSetAttribute((const void*)k_ns_hf_gemm<kNsProdA, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(2)));
  HIP_TRY(hipFuncSetAttribute((const void*)k_ns_hf_gemm<kNsUpdate, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(2)));
  HIP_TRY(hipFuncSetAttribute((const void*)k_ns_hf_gemm<kNsUpdate, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(4)));
  done.push_back(dev);
  return 0;
}

int slice_lds_once() {
  static std::mutex mu;
  static std::vector<int> done;
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (int d : done)
    if (d == dev) return 0;
  HIP_TRY(hipFuncSetAttribute((const void*)k_celo2_slice_finish<true>, hipFuncAttributeMaxDynamicSharedMemorySize, kSliceLdsBlock));
  done.push_back(dev);
  return 0;
}

__global__ __launch_bounds__(256) void k_ns_zero(u32x4* __restrict__ p, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) p[i] = u32x4{0u, 0u, 0u, 0u};
}

// Newton-Schulz (ns_iters > 0, on the tensors flagged PYLO_ARG_ORTHOGONALIZE) and the finishing pass.
int finish_impl(PyloPlan* P, const PyloTensorArgs* args, const float* coeffs, int ns_iters, float ns_eps, void* stream,
                const char* who) {
  const std::string w(who);
  if (!P || P->kind != PYLO_KIND_CELO2) return fail(w + ": not an ELO-CELO2 plan");
  if (!args) return fail(w + ": null argument");
  const Layout& L = P->L;
  bool any_ns = false, any_slices = false;
  for (int t = 0; t < P->T; ++t) {
    const TDesc& d = L.descs[t];
    const PyloTensorArgs& a = args[t];
    if (a.grad == nullptr || d.mode == kModeFlat || d.n == 0) continue;
    const std::string at = " (tensor " + std::to_string(t) + ")";
    if (!a.param || !a.step_out) return fail(w + ": null param/step_out pointer" + at);
    const uintptr_t m = reinterpret_cast<uintptr_t>(a.param) | reinterpret_cast<uintptr_t>(a.step_out);
    if (d.mode == kModeFacND && L.slice_of_tensor[t] >= 0) {
      if (reinterpret_cast<uintptr_t>(a.step_out) % 4 != 0 || reinterpret_cast<uintptr_t>(a.param) % (d.store != 0 ? 2 : 4) != 0)
        return fail(w + ": misaligned pointer" + at);
      if (coeffs && (a.flags & PYLO_ARG_ORTHOGONALIZE) && L.slice_mats[L.slice_of_tensor[t]].no_orth)
        return fail(w + ": PYLO_ARG_ORTHOGONALIZE on a tensor whose shape carries PYLO_F_NO_ORTHOGONALIZE" + at);
      any_slices = true;
      continue;
    }
    const bool vec = d.fin_units > 0 && L.fin_units[d.fin_unit0].vec;
    if (m % (vec ? 16 : 4) != 0) return fail(w + ": misaligned pointer" + at);
    if (coeffs && ns_iters == 0 && (a.flags & PYLO_ARG_ORTHOGONALIZE))
      return fail(w + ": PYLO_ARG_ORTHOGONALIZE with ns_iters = 0 on a tensor that the tiled products orthogonalise "
                  "(the division by the norm alone is the caller's)" + at);
    if (ns_iters > 0 && (a.flags & PYLO_ARG_ORTHOGONALIZE)) {
      if (L.ns_of_tensor[t] < 0) return fail(w + ": PYLO_ARG_ORTHOGONALIZE on a tensor the library cannot orthogonalise" + at);
      any_ns = true;
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // the caller's records as they are: the update kernel reads and writes the parameter in its storage type
  if (int rc = upload_args(P, args, s, L.off_dyn)) return rc;
  const TDesc* descs = P->at<TDesc>(L.off_descs);
  const PyloTensorArgs* dyn = P->at<PyloTensorArgs>(L.off_dyn);
  const Item* fin_items = P->at<Item>(L.off_fin_items);
  const FinUnit* units = P->at<FinUnit>(L.off_fin_units);
  double* fin_part = P->at<double>(L.off_finpart);
  float* fin_scale = P->at<float>(L.off_finscale);
  const int n_fin = (int)L.fin_items.size();
  // The per-slice launches touch only their own tensors: next to the matrices' chains of products they run on a stream
  // of their own (forked from and joined into the caller's like the groups').
  const bool slices_aside = any_slices && any_ns && L.ns_hf && P->slice_side != nullptr;
  if (any_slices) {
    // tensors with more than two dims: everything per slice, in LDS (k_slice_finish.h)
    if (int rc = slice_lds_once()) return rc;
    hipStream_t caller = s;
    if (slices_aside) {
      HIP_TRY(hipEventRecord(P->slice_fork, caller));
      HIP_TRY(hipStreamWaitEvent(P->slice_side, P->slice_fork, 0));
    }
    hipStream_t s = slices_aside ? P->slice_side : caller;
    const SliceMat* smats = P->at<SliceMat>(L.off_slice_mats);
    const float c0 = coeffs ? coeffs[0] : 0.0f, c1 = coeffs ? coeffs[1] : 0.0f, c2 = coeffs ? coeffs[2] : 0.0f;
    const int orth_call = coeffs != nullptr;
    auto lanes = [&](auto kern, int set) {
      if (!L.slice_items_l[set].empty())
        hipLaunchKernelGGL(kern, dim3((unsigned)L.slice_items_l[set].size()), dim3(64), L.slice_lds_l[set], s, smats,
                           P->at<Item>(L.off_slice_items_l[set]), descs, dyn, orth_call, ns_iters, ns_eps, c0, c1, c2);
    };
    lanes(k_celo2_slice_finish_lane<1>, 0);
    lanes(k_celo2_slice_finish_lane<3>, 1);
    lanes(k_celo2_slice_finish_lane<5>, 2);
    lanes(k_celo2_slice_finish_lane<7>, 3);
    for (int set = 4; set < kSliceLaneSets; ++set) lanes(k_celo2_slice_finish_lane<0>, set);
    if (!L.slice_items_w.empty())
      hipLaunchKernelGGL(k_celo2_slice_finish<false>, dim3((unsigned)L.slice_items_w.size()), dim3(256), L.slice_lds_w, s,
                         smats, P->at<Item>(L.off_slice_items_w), descs, dyn, orth_call, ns_iters, ns_eps, c0, c1, c2);
    if (!L.slice_items_b.empty())
      hipLaunchKernelGGL(k_celo2_slice_finish<true>, dim3((unsigned)L.slice_items_b.size()), dim3(256), L.slice_lds_b, s,
                         smats, P->at<Item>(L.off_slice_items_b), descs, dyn, orth_call, ns_iters, ns_eps, c0, c1, c2);
    if (slices_aside) HIP_TRY(hipEventRecord(P->slice_join, P->slice_side));
  }
  if (n_fin == 0) {
    HIP_TRY(hipGetLastError());
    return 0;
  }
  // sum of squares, per-unit scale and update over a range of the finishing pass's blocks and units
  auto finish_range = [&](hipStream_t st, int fin0, int nf, int unit0, int nu, const long long* x_alt, const float* ws) {
    if (nf == 0) return;
    hipLaunchKernelGGL(k_celo2_sumsq, dim3(nf), dim3(kThreads), 0, st, units, dyn, fin_items + fin0, fin_part + fin0, x_alt, ws);
    hipLaunchKernelGGL(k_celo2_finscale, dim3(nu), dim3(kThreads), 0, st, units + unit0, dyn, fin_part, fin_scale + unit0);
    hipLaunchKernelGGL(k_celo2_update, dim3(nf), dim3(kThreads), 0, st, units, descs, dyn, fin_items + fin0, fin_scale, x_alt, ws);
  };
  if (!any_ns) {
    finish_range(s, 0, n_fin, 0, (int)L.fin_units.size(), nullptr, nullptr);
  } else if (L.ns_hf) {
    // The split-fp16 kernels.  Every group of matrices is a chain of its own from the norms of its raw steps to the
    // update of its parameters, on a stream of its own (the first group on the caller's): the memory-bound ends of
    // one chain run under the matrix products of the others.
    const NsMat* mats = P->at<NsMat>(L.off_ns_mats);
    const NsItem* gram = P->at<NsItem>(L.off_ns_gram);
    const NsItem* poly = P->at<NsItem>(L.off_ns_poly);
    const NsItem* upd = P->at<NsItem>(L.off_ns_upd);
    const NsItem* upd4 = P->at<NsItem>(L.off_ns_upd4);
    const int* split = P->at<int>(L.off_ns_split);
    const int* list = P->at<int>(L.off_ns_list);
    float* scale = P->at<float>(L.off_ns_scale);
    float* ns_ws = P->at<float>(L.off_ns_ws);
    const NsHfMat* bmats = P->at<NsHfMat>(L.off_nsb_mats);
    const NsTileItem* sitems = P->at<NsTileItem>(L.off_nsb_split_items);
    hbits* pw = P->at<hbits>(L.off_ns_pw);
    if (int rc = ns_hf_lds_once()) return rc;
    finish_range(s, L.fin_rest0, L.n_fin_rest, L.unit_rest0, L.n_unit_rest, nullptr, nullptr);   // tensors of no group
    const bool several = L.ns_batches.size() > 1;
    const float c0 = coeffs[0], c1 = coeffs[1], c2 = coeffs[2];
    const std::vector<int> chains = ns_chains(ns_iters);
    const NsExps ex = ns_plane_exps(c0, c1, c2, ns_iters);
    // chain lengths chosen per matrix on the device: an odd iteration count of three or more, nothing given in the environment
    const bool adaptive = ns_adaptive() && ns_iters >= 3 && (ns_iters & 1);
    int* chain_flags = P->at<int>(L.off_ns_flags);
    float* chain_part = P->at<float>(L.off_ns_fpart);
    const Item* flag_items = P->at<Item>(L.off_ns_flag_items);
    const float chain_tau2 = (16.0f / 196.0f) * (16.0f / 196.0f);
    for (const NsBatch& bt : L.ns_batches) {
      // the planes' padding: zero from plan creation on when one batch has the memory to itself
      if (several) {
        const size_t n16 = (size_t)bt.plane_elems * sizeof(hbits) / 16;
        hipLaunchKernelGGL(k_ns_zero, dim3((unsigned)std::min<size_t>((n16 + 255) / 256, 1u << 16)), dim3(256), 0, s,
                           reinterpret_cast<u32x4*>(pw), n16);
      }
      const int n_groups = bt.n_groups;
      auto stream_of = [&](int g) { return g == 0 ? s : P->ns_side[g - 1]; };
      if (n_groups > 1) {
        HIP_TRY(hipEventRecord(P->ns_fork, s));
        for (int g = 1; g < n_groups; ++g) HIP_TRY(hipStreamWaitEvent(P->ns_side[g - 1], P->ns_fork, 0));
      }
      for (int g = 0; g < n_groups; ++g) {
        // ||raw|| per matrix (the finishing pass's sums of squares, taken on the raw steps), then the planes
        const NsGroup& G = L.ns_groups[bt.group0 + g];
        hipStream_t sg = stream_of(g);
        if (G.n_fin > 0)
          hipLaunchKernelGGL(k_celo2_sumsq, dim3(G.n_fin), dim3(kThreads), 0, sg, units, dyn, fin_items + G.fin0,
                             fin_part + G.fin0, (const long long*)nullptr, (const float*)nullptr);
        if (G.n_list > 0)
          hipLaunchKernelGGL(k_ns_scale, dim3(G.n_list), dim3(256), 0, sg, mats, list + G.list0, G.n_list, units, fin_part,
                             ns_eps, scale);
        if (G.n_sitems > 0)
          hipLaunchKernelGGL(k_ns_hf_split, dim3((unsigned)G.n_sitems), dim3(256), 0, sg, bmats, sitems + G.sitem0, dyn,
                             (const float*)scale, pw, pow2(ex.x));
      }
      // The launch sequence of one group (every group runs the same one on its own tables), then its launches,
      // interleaved over the groups so that every stream is fed in turn.
      enum OpKind { kOpGram, kOpFlag, kOpPoly, kOpProd, kOpProdA, kOpUpdate };
      struct Op { OpKind kind; NsBufs b; int par, last; NsPick pick; };
      std::vector<Op> ops;
      const NsPick all{nullptr, kNsAll, 0, 0, 0.0f};
      int par = 0;   // which Xl buffer the next update reads
      // A is buffer A throughout; B' of the latest iteration in `bprev`, the product of all B' so far in `q`
      // (`nq` of them); eb[]: the exponent of the scale of the planes in each buffer
      int bprev = kNsBufB, q = kNsBufB, nq = 1;
      int eb[kNsBufs] = {};
      // the accumulators of a product of planes with exponents e1 and e2, and planes out with exponent ed
      auto bufs = [&](int s1, int s2, int d, int e1, int e2, int ed) {
        if (d >= 0) eb[d] = ed;
        return NsBufs{s1, s2, d < 0 ? 0 : d, pow2(-(e1 + e2)), pow2(ed)};
      };
      auto extend = [&](NsPick pk) {   // one more iteration into the chain: A <- B' A B', the next B', Q <- B' Q
        int free_buf[2], nf = 0;
        for (int b : {kNsBufB, kNsBufT, kNsBufC})
          if (b != bprev && b != q && nf < 2) free_buf[nf++] = b;
        const int t = free_buf[0];
        ops.push_back(Op{kOpProd, bufs(kNsBufA, bprev, t, ex.a, eb[bprev], ex.t), par, 0, pk});
        ops.push_back(Op{kOpProdA, bufs(bprev, t, kNsBufA, eb[bprev], ex.t, ex.a), par, 0, pk});
        ops.push_back(Op{kOpPoly, bufs(kNsBufA, kNsBufA, t, ex.a, ex.a, ex.b), par, 0, pk});
        const int qn = q == bprev ? free_buf[1] : bprev;   // (the old B' is done with)
        ++nq;
        ops.push_back(Op{kOpProd, bufs(t, q, qn, ex.b, eb[q], ex.q[std::min<size_t>(nq, ex.q.size() - 1)]), par, 0, pk});
        bprev = t;
        q = qn;
      };
      auto open_chain = [&](NsPick pk) {   // Gram product and the first B'
        ops.push_back(Op{kOpGram, bufs(0, 0, kNsBufA, ex.x, ex.x, ex.a), par, 0, pk});
        ops.push_back(Op{kOpPoly, bufs(kNsBufA, kNsBufA, kNsBufB, ex.a, ex.a, ex.b), par, 0, pk});
        bprev = q = kNsBufB;
        nq = 1;
      };
      auto update = [&](int last, NsPick pk) {   // X <- Q X
        ops.push_back(Op{kOpUpdate, bufs(q, 0, -1, ex.x, eb[q], ex.x), par, last, pk});
        par ^= 1;
      };
      if (adaptive) {
        // First chain: two iterations for every matrix, a third for those whose flag says so (k_ns_hf_chain_flag),
        // then pairs for all -- the last of them is the end for the flagged ones -- and one iteration more for the others.
        const NsPick longer{chain_flags, kNsLongOnly, 0, 0, 0.0f}, shorter{chain_flags, kNsShortOnly, 0, 0, 0.0f};
        const int n_pairs = (ns_iters - 3) / 2;
        open_chain(all);
        ops.push_back(Op{kOpFlag, NsBufs{0, 0, 0, 0.0f, 0.0f}, par, 0, all});
        extend(all);
        const int q_short = q, e_short = eb[q];
        extend(longer);
        update(n_pairs == 0, NsPick{chain_flags, kNsBoth, q_short, 0, pow2(-(ex.x + e_short))});
        for (int p = 0; p < n_pairs; ++p) {
          open_chain(all);
          extend(all);
          update(p == n_pairs - 1, NsPick{chain_flags, kNsBoth, q, 0, pow2(-(ex.x + eb[q]))});
        }
        open_chain(shorter);
        update(1, shorter);
      } else {
        int done = 0;
        for (size_t ch = 0; ch < chains.size(); ++ch) {
          // a chain of iterations: one Gram product, 4 len - 3 products of m x m matrices and one update (k_ns_hf.h)
          done += chains[ch];
          open_chain(all);
          for (int j = 1; j < chains[ch]; ++j) extend(all);
          update(done == ns_iters, all);
        }
      }
      for (const Op& op : ops)
        for (int g = 0; g < n_groups; ++g) {
          const NsGroup& G = L.ns_groups[bt.group0 + g];
          hipStream_t sg = stream_of(g);
          auto small = [&](auto kern) {
            if (G.n_poly > 0)
              hipLaunchKernelGGL(kern, dim3(G.n_poly), dim3(256), hf_gemm_lds(2), sg, bmats, poly + G.poly0, dyn, ns_ws, pw,
                                 op.par, op.last, op.b, c0, c1, c2, op.pick);
          };
          switch (op.kind) {
            case kOpGram:
              if (G.n_gram > 0)
                hipLaunchKernelGGL((k_ns_hf_gemm<kNsGram, 2>), dim3(G.n_gram), dim3(256), hf_gemm_lds(2), sg, bmats,
                                   gram + G.gram0, dyn, ns_ws, pw, op.par, op.last, op.b, c0, c1, c2, op.pick);
              if (G.n_split > 0)
                hipLaunchKernelGGL(k_ns_hf_gram_reduce, dim3(((size_t)G.split_max_m * G.split_max_m + 255) / 256, G.n_split),
                                   dim3(256), 0, sg, bmats, split + G.split0, dyn, ns_ws, pw, op.pick, op.b.out_scale);
              break;
            case kOpFlag:
              if (G.n_list > 0) {
                hipLaunchKernelGGL(k_ns_hf_chain_sumsq, dim3(G.n_fitems), dim3(256), 0, sg, bmats, flag_items + G.fitem0, dyn,
                                   (const float*)ns_ws, chain_part);
                hipLaunchKernelGGL(k_ns_hf_chain_flag, dim3(G.n_list), dim3(64), 0, sg, bmats, list + G.list0, dyn,
                                   (const float*)chain_part, chain_tau2, chain_flags);
              }
              break;
            case kOpPoly: small(k_ns_hf_gemm<kNsPoly, 2>); break;
            case kOpProd: small(k_ns_hf_gemm<kNsProd, 2>); break;
            case kOpProdA: small(k_ns_hf_gemm<kNsProdA, 2>); break;
            case kOpUpdate:
              if (G.n_upd4 > 0)
                hipLaunchKernelGGL((k_ns_hf_gemm<kNsUpdate, 4>), dim3(G.n_upd4), dim3(256), hf_gemm_lds(4), sg, bmats,
                                   upd4 + G.upd40, dyn, ns_ws, pw, op.par, op.last, op.b, c0, c1, c2, op.pick);
              if (G.n_upd > 0)
                hipLaunchKernelGGL((k_ns_hf_gemm<kNsUpdate, 2>), dim3(G.n_upd), dim3(256), hf_gemm_lds(2), sg, bmats,
                                   upd + G.upd0, dyn, ns_ws, pw, op.par, op.last, op.b, c0, c1, c2, op.pick);
              break;
          }
        }
      for (int g = 0; g < n_groups; ++g) {
        const NsGroup& G = L.ns_groups[bt.group0 + g];
        finish_range(stream_of(g), G.fin0, G.n_fin, G.unit0, G.n_units, nullptr, nullptr);
      }
      for (int g = 1; g < n_groups; ++g) {
        HIP_TRY(hipEventRecord(P->ns_join[g - 1], P->ns_side[g - 1]));
        HIP_TRY(hipStreamWaitEvent(s, P->ns_join[g - 1], 0));
      }
    }
  } else {
    // The fp32 matrix instructions: one chain for all matrices.
    const NsMat* mats = P->at<NsMat>(L.off_ns_mats);
    const NsItem* gram = P->at<NsItem>(L.off_ns_gram);
    const NsItem* poly = P->at<NsItem>(L.off_ns_poly);
    const NsItem* upd = P->at<NsItem>(L.off_ns_upd);
    const int* split = P->at<int>(L.off_ns_split);
    float* scale = P->at<float>(L.off_ns_scale);
    float* ns_ws = P->at<float>(L.off_ns_ws);
    const int n_mats = (int)L.ns_mats.size(), n_gram = (int)L.ns_gram.size(), n_poly = (int)L.ns_poly.size(),
              n_upd = (int)L.ns_upd.size(), n_split = (int)L.ns_split.size();
    // ||raw||: the finishing pass's sums of squares, taken on the raw steps
    hipLaunchKernelGGL(k_celo2_sumsq, dim3(n_fin), dim3(kThreads), 0, s, units, dyn, fin_items, fin_part,
                       (const long long*)nullptr, (const float*)nullptr);
    hipLaunchKernelGGL(k_ns_scale, dim3(n_mats), dim3(256), 0, s, mats, (const int*)nullptr, n_mats, units, fin_part, ns_eps,
                       scale);
    for (int it = 0; it < ns_iters; ++it) {
      const int first = it == 0, par = it & 1;
      hipLaunchKernelGGL(k_ns_gemm<kNsGram>, dim3(n_gram), dim3(256), 0, s, mats, gram, dyn, ns_ws, scale, first, par,
                         coeffs[0], coeffs[1], coeffs[2]);
      if (n_split > 0)
        hipLaunchKernelGGL(k_ns_gram_reduce, dim3(((size_t)L.ns_max_m * L.ns_max_m + 255) / 256, n_split), dim3(256), 0, s,
                           mats, split, dyn, ns_ws);
      hipLaunchKernelGGL(k_ns_gemm<kNsPoly>, dim3(n_poly), dim3(256), 0, s, mats, poly, dyn, ns_ws, scale, first, par,
                         coeffs[0], coeffs[1], coeffs[2]);
      hipLaunchKernelGGL(k_ns_gemm<kNsUpdate>, dim3(n_upd), dim3(256), 0, s, mats, upd, dyn, ns_ws, scale, first, par,
                         coeffs[0], coeffs[1], coeffs[2]);
    }
    // an odd number of iterations leaves the result in the second buffer
    const long long* x_alt = (ns_iters & 1) ? P->at<long long>(L.off_ns_xalt) : nullptr;
    finish_range(s, 0, n_fin, 0, (int)L.fin_units.size(), x_alt, ns_ws);
  }
  if (slices_aside) HIP_TRY(hipStreamWaitEvent(s, P->slice_join, 0));
  HIP_TRY(hipGetLastError());
  return 0;
}

}  // namespace

extern "C" int pylo_mi355_celo2_finish(PyloPlan* P, const PyloTensorArgs* args, void* stream) {
  return finish_impl(P, args, nullptr, 0, 0.0f, stream, "celo2_finish");
}

extern "C" int pylo_mi355_celo2_orthogonalize_finish(PyloPlan* P, const PyloTensorArgs* args, const float* ns_coeffs,
                                                     int ns_iters, float ns_eps, void* stream) {
  if (ns_iters < 0 || (ns_iters > 0 && !ns_coeffs)) return fail("celo2_orthogonalize_finish: bad Newton-Schulz arguments");
  return finish_impl(P, args, ns_coeffs, ns_iters, ns_eps, stream, "celo2_orthogonalize_finish");
}

extern "C" int pylo_mi355_plan_finish_supported(const PyloPlan* P, int tensor) {
  if (!P || tensor < 0 || tensor >= P->T || P->kind != PYLO_KIND_CELO2) return 0;
  return P->L.descs[tensor].mode == kModeFlat ? 0 : 1;
}

extern "C" int pylo_mi355_plan_orthogonalize_supported(const PyloPlan* P, int tensor) {
  if (!P || tensor < 0 || tensor >= P->T || P->kind != PYLO_KIND_CELO2) return 0;
  if (P->L.slice_of_tensor[tensor] >= 0) return P->L.slice_mats[P->L.slice_of_tensor[tensor]].no_orth ? 0 : 2;
  return P->L.ns_of_tensor[tensor] >= 0 ? 1 : 0;
}

extern "C" int pylo_mi355_velo_step(PyloPlan* P, const PyloTensorArgs* args, const PyloDecays* decays,
                                    const PyloVeloNets* nets, const PyloVeloStep* step, void* stream) {
  if (!P || !args || !decays || !nets || !step) return fail("velo_step: null argument");
  if (P->kind != PYLO_KIND_VELO) return fail("velo_step: plan is not a VeLO plan");
  const int H = nets->hidden, K = nets->n_bank, T = P->T;
  if (H <= 0 || H % 64 != 0 || H > kVeloHiddenMax) return fail("velo_step: LSTM width must be a multiple of 64, at most 1024");
  if (K <= 0 || K > 4096) return fail("velo_step: bank size out of range");
  if (!nets->mix2_wt || !nets->mix2_b || !nets->fmix_wt || !nets->fmix_b || !nets->lstm_wt || !nets->lstm_b ||
      !nets->ctrl_wt || !nets->ctrl_b || !nets->lr_w || !nets->lr_b || !nets->bank)
    return fail("velo_step: null weight pointer");
  if (!step->lstm_h || !step->lstm_c || !step->loss_means || !step->loss_running_min || !step->loss_decays ||
      !step->loss_iteration || !step->loss)
    return fail("velo_step: null state pointer");
  if (int rc = check_args(P, args, true)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = upload_args(P, args, s, P->L.off_dyn_user)) return rc;
  stage_in(P, s, 3);
  advance_steps(P, s);
  // the sums the apply items carry over are taken on the fp32 parameter they write; the next step starts
  // from that value rounded to the tensor's storage type
  if (P->L.typed) P->stats_carried = false;
  const Layout& L = P->L;
  const TDesc* descs = P->at<TDesc>(L.off_descs);
  const PyloTensorArgs* dyn = P->at<PyloTensorArgs>(L.off_dyn);
  const Item* p0_items = P->at<Item>(L.off_p0_items);
  const Item* nd_items = P->at<Item>(L.off_nd_items);
  const Item* el_items = P->at<Item>(L.off_el_items);
  const Item* v0a_items = P->at<Item>(L.off_v0a_items);
  const Item* v0b_items = P->at<Item>(L.off_v0b_items);
  float* part = P->at<float>(L.off_part);
  double* gsq = P->at<double>(L.off_gsq);
  int* flag = P->at<int>(L.off_flag);
  Globals* gl = P->at<Globals>(L.off_globals);
  float* fac_tab = P->at<float>(L.off_fac);
  float* term_tab = P->at<float>(L.off_term);
  double* v0part = P->at<double>(L.off_v0part);
  BScale* bscale = P->at<BScale>(L.off_bscale);
  double* stats = P->at<double>(L.off_stats);
  float* wfold = P->at<float>(L.off_wfold);
  double* totals = P->at<double>(L.off_totals);
  float* xfeat = P->at<float>(L.off_xfeat);
  float* xT = P->at<float>(L.off_xT);
  float* canon = P->at<float>(L.off_canon);
  float* mixbuf = P->at<float>(L.off_mixbuf);
  const int n_p0 = (int)L.p0_items.size(), n_nd = (int)L.nd_items.size(), n_el = (int)L.el_items.size();
  const int n_v0a = (int)L.v0a_items.size(), n_v0b = (int)L.v0b_items.size();
  const PyloDecays dec = *decays;
  VeloStep vs;
  std::memcpy(vs.frac, step->frac, sizeof(vs.frac));
  vs.frac_dev = P->dsteps.counters ? P->at<float>(L.off_frac) : nullptr;
  Marks mark(P, s);
  float* piv = P->at<float>(L.off_piv);
  double* newsum = P->at<double>(L.off_newsum);
  float* wmix = P->at<float>(L.off_wmix);
  const LossState ls{step->loss_means, step->loss_running_min, step->loss_decays, step->loss_iteration, step->loss};
  const int n_chunks = (T + kMixRows - 1) / kMixRows;
  float* pmax = n_chunks > 1 ? P->at<float>(L.off_pmax) : nullptr;
  const size_t heads_lds = sizeof(float) * (H + K + 160 + 32 + 16 + 4 * (size_t)std::max(K, 160));
  // The LSTM from the tensors' 30 input features on: input mixing across tensors, cell, heads.
  auto lstm = [&](hipStream_t q, const double* tot, bool timed) {
    if (pmax != nullptr)
      hipLaunchKernelGGL(k_velo_colmax, dim3(H / 64, n_chunks), dim3(kThreads), 0, q, (const float*)mixbuf, T, H, pmax);
    hipLaunchKernelGGL(k_velo_mix, dim3(H / 64, L.Tpad / kGateBT), dim3(kThreads), 0, q, (const float*)mixbuf, T, L.Tpad, H,
                       (const float*)pmax, n_chunks, step->lstm_h, xT, ls);
    if (timed) (void)mark();
    hipLaunchKernelGGL(k_velo_gates, dim3((L.Tpad / kGateBT) * (H / kGateU)), dim3(kThreads), 0, q, xT, T, L.Tpad, H,
                       nets->lstm_wt, nets->lstm_b, step->lstm_h, step->lstm_c);
    if (timed) (void)mark();
    hipLaunchKernelGGL(k_velo_heads, dim3(T), dim3(kFoldThreads), heads_lds, q, descs, T, H, K, step->lstm_h,
                       nets->ctrl_wt, nets->ctrl_b, nets->lr_w, nets->lr_b, nets->bank, tot, canon, wfold,
                       step->controls_out, step->lr_mult_out, wmix);
    if (timed) (void)mark();
  };
  // clip_norm is 0 for VeLO tensors: k_p0 clamps directly; its norm / flag outputs are not used
  // no global norm to wait for: the N-D tensors' sums ride in the tail blocks of the same launch
  auto gradient_sums = [&]() {
    if (n_p0 + n_nd > 0)
      hipLaunchKernelGGL(k_p0, dim3(n_p0 + n_nd), dim3(kThreads), 0, s, descs, dyn, p0_items, part, gsq, flag, gl, 0,
                         nd_items, n_p0);
  };
  auto factor_tables = [&]() {
    if (n_v0a > 0)
      hipLaunchKernelGGL(k_v0a, dim3(n_v0a), dim3(kV0aThreads), 0, s, descs, dyn, v0a_items, part, gl, dec, v0part);
    HIP_TRY(mark());
    if (n_v0b > 0)
      hipLaunchKernelGGL(k_v0b<4>, dim3(n_v0b), dim3(kThreads), 0, s, descs, dyn, v0b_items, v0part, 1e-5f,
                         (const float*)nullptr, (const float*)nullptr, 0, fac_tab, term_tab, bscale);
    HIP_TRY(mark());
    return 0;
  };
  const int n_mx = (int)L.mx_items.size();
  HIP_TRY(mark());
  if (n_mx > 0 && P->stats_carried) {
    // The LSTM's inputs are sums over the parameters and accumulators as they stand before the step: the
    // previous step's apply items left them.  It runs next to the gradient sums, on the plan's own stream.
    HIP_TRY(hipEventRecord(P->ev_fork, s));
    HIP_TRY(hipStreamWaitEvent(P->side, P->ev_fork, 0));
    hipLaunchKernelGGL(k_velo_feat, dim3(T), dim3(kFoldThreads), 0, P->side, descs, dyn, T, (const double*)newsum, piv, ls, vs,
                       xfeat, H, nets->mix2_wt, nets->mix2_b, nets->fmix_wt, nets->fmix_b, mixbuf, P->at<int>(L.off_sync));
    lstm(P->side, nullptr, false);
    HIP_TRY(hipEventRecord(P->ev_join, P->side));
    gradient_sums();
    HIP_TRY(mark());
    if (int rc = factor_tables()) return rc;
    HIP_TRY(hipStreamWaitEvent(s, P->ev_join, 0));
    if (n_v0b > 0)
      hipLaunchKernelGGL(k_terms<4>, dim3(n_v0b), dim3(kThreads), 0, s, descs, dyn, v0b_items, bscale, canon, kVCanon, term_tab);
    HIP_TRY(mark());
    hipLaunchKernelGGL(k_velo_elem, dim3(n_mx), dim3(kThreads), 0, s, descs, dyn, P->at<Item>(L.off_mx_items), fac_tab, term_tab,
                       dec, (const float*)wmix, wfold, stats, (const float*)piv, newsum, P->at<int>(L.off_sync), T);
    HIP_TRY(mark());
    mark.done();
    stage_out(P, s, 0);
    HIP_TRY(hipGetLastError());
    return 0;
  }
  // Each pass as a launch of its own: the first step of a plan, a step after its carried sums were
  // invalidated, and every step with PYLO_MI355_SLAB_ELEMS=0.
  gradient_sums();
  HIP_TRY(mark());
  if (n_mx == 0) HIP_TRY(mark());
  if (int rc = factor_tables()) return rc;
  if (n_el > 0) hipLaunchKernelGGL(k_velo_stats, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac_tab, dec, stats);
  if (n_mx == 0) HIP_TRY(mark());
  const Item* seg_items = P->at<Item>(L.off_seg_items);
  double* seg_tot = P->at<double>(L.off_segtot);
  const int n_seg = (int)L.seg_items.size();
  if (n_seg > 0) hipLaunchKernelGGL(k_stat_segsum, dim3(n_seg), dim3(kThreads), 0, s, descs, seg_items, stats, seg_tot);
  hipLaunchKernelGGL(k_lo_reduce, dim3(T), dim3(kFoldThreads), 0, s, descs, dyn, T, stats, seg_tot, totals, ls, vs, xfeat,
                     H, nets->mix2_wt, nets->mix2_b, nets->fmix_wt, nets->fmix_b, mixbuf, piv);
  if (n_mx == 0) HIP_TRY(mark());
  lstm(s, totals, n_mx == 0);   // the LSTM's launches have intervals of their own only in the launch list without k_velo_elem
  if (n_v0b > 0)
    hipLaunchKernelGGL(k_terms<4>, dim3(n_v0b), dim3(kThreads), 0, s, descs, dyn, v0b_items, bscale, canon, kVCanon, term_tab);
  HIP_TRY(mark());
  if (n_el > 0)
    hipLaunchKernelGGL(k_velo_apply, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac_tab, term_tab, dec, wfold,
                       (const float*)piv, newsum);
  HIP_TRY(mark());
  mark.done();
  stage_out(P, s, 0);
  HIP_TRY(hipGetLastError());
  P->stats_carried = n_mx > 0;
  return 0;
}

extern "C" int pylo_mi355_plan_invalidate_statistics(PyloPlan* P) {
  if (!P) return fail("plan_invalidate_statistics: null plan");
  P->stats_carried = false;
  if (P->stale_host) *static_cast<volatile int*>(P->stale_host) = 0;   // what the guard found before this call no longer counts
  return 0;
}

extern "C" int pylo_mi355_plan_statistics_stale(const PyloPlan* P) {
  if (!P || !P->stale_host) return 0;
  return *static_cast<const volatile int*>(P->stale_host);
}

extern "C" int pylo_mi355_adafac_step(PyloPlan* P, const PyloTensorArgs* args, const PyloDecays* decays,
                                      const float* net, float step, void* stream) {
  if (!P || !args || !decays || !net) return fail("adafac_step: null argument");
  if (P->kind != PYLO_KIND_ADAFAC) return fail("adafac_step: plan is not an AdafacLO plan");
  if (int rc = check_args(P, args, false)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = upload_args(P, args, s, P->L.off_dyn_user)) return rc;
  stage_in(P, s, 3);
  advance_steps(P, s);
  const Layout& L = P->L;
  const TDesc* descs = P->at<TDesc>(L.off_descs);
  const PyloTensorArgs* dyn = P->at<PyloTensorArgs>(L.off_dyn);
  const Item* p0_items = P->at<Item>(L.off_p0_items);
  const Item* nd_items = P->at<Item>(L.off_nd_items);
  const Item* el_items = P->at<Item>(L.off_el_items);
  const Item* v0a_items = P->at<Item>(L.off_v0a_items);
  const Item* v0b_items = P->at<Item>(L.off_v0b_items);
  float* part = P->at<float>(L.off_part);
  double* gsq = P->at<double>(L.off_gsq);
  int* flag = P->at<int>(L.off_flag);
  Globals* gl = P->at<Globals>(L.off_globals);
  float* fac_tab = P->at<float>(L.off_fac);
  float* term_tab = P->at<float>(L.off_term);
  double* v0part = P->at<double>(L.off_v0part);
  BScale* bscale = P->at<BScale>(L.off_bscale);
  double* stats = P->at<double>(L.off_stats);
  float* wfold = P->at<float>(L.off_wfold);
  double* totals = P->at<double>(L.off_totals);
  float* bias_eff = P->at<float>(L.off_xfeat);  // [T][32]; the LSTM feature buffer is unused by this kind
  const int n_p0 = (int)L.p0_items.size(), n_nd = (int)L.nd_items.size(), n_el = (int)L.el_items.size();
  const int n_v0a = (int)L.v0a_items.size(), n_v0b = (int)L.v0b_items.size();
  const int T = P->T;
  const PyloDecays dec = *decays;
  VeloStep vs;
  std::memset(&vs, 0, sizeof(vs));
  Marks mark(P, s);

  // ELO's global-norm clipping (ELO_cuda.py:153-161): the norm, then the exact sums where an element
  // is not a fixed point of the conditioning.  Plain AdafacLO steps skip both launches.
  bool clips = false;
  for (int t = 0; t < T; ++t) clips = clips || (args[t].grad != nullptr && args[t].clip_norm > 0.0f);
  if (clips && !L.global_norm)
    return fail("adafac_step: clip_norm > 0 needs a plan built with PYLO_F_GLOBAL_NORM or PYLO_F_TENSOR_NORM");
  if (clips && L.tensor_norm)
    for (int t = 0; t < T; ++t)
      if (args[t].grad != nullptr && args[t].clip_norm > 0.0f && args[t].clip_val != 0.0f)
        return fail("adafac_step: a tensor clipped by its own norm (PYLO_F_TENSOR_NORM) takes no clip_val");
  HIP_TRY(mark());
  // without global-norm clipping the N-D tensors' sums ride in the tail blocks of the first launch
  const int n_tail = clips ? 0 : n_nd;
  if (n_p0 + n_tail > 0)
    hipLaunchKernelGGL(k_p0, dim3(n_p0 + n_tail), dim3(kThreads), 0, s, descs, dyn, p0_items, part, gsq, flag, gl, 0,
                       nd_items, n_p0);
  if (clips && L.tensor_norm) {
    // every tensor against its own norm (AdafacLO_naive.py:199-200): no clamp on such tensors, no exact pass
    hipLaunchKernelGGL(k_tnorm, dim3(T), dim3(kThreads), 0, s, descs, dyn, gsq, gl, P->at<float>(L.off_tscale));
  } else if (clips) {
    const bool exact_pass = exact_pass_possible(P, args);
    hipLaunchKernelGGL(k_gnorm, dim3(1), dim3(kThreads), 0, s, gsq, flag, n_p0, gl, exact_pass ? 1 : 0, (int*)nullptr, 0);
    if (n_p0 > 0 && exact_pass)
      hipLaunchKernelGGL(k_p0, dim3(n_p0), dim3(kThreads), 0, s, descs, dyn, p0_items, part, gsq, flag, gl, 1,
                         (const Item*)nullptr, n_p0);
  }
  HIP_TRY(mark());
  if (n_nd > 0 && clips) hipLaunchKernelGGL(k_p0_nd, dim3(n_nd), dim3(kThreads), 0, s, descs, dyn, nd_items, part, gl);
  HIP_TRY(mark());
  if (n_v0a > 0)
    hipLaunchKernelGGL(k_v0a, dim3(n_v0a), dim3(kV0aThreads), 0, s, descs, dyn, v0a_items, part, gl, dec, v0part);
  HIP_TRY(mark());
  hipLaunchKernelGGL(k_adafac_bias, dim3(T), dim3(64), 0, s, net, P->dsteps.counters ? -1.0f : step, dyn, bias_eff);
  HIP_TRY(mark());
  if (n_v0b > 0)
    hipLaunchKernelGGL(k_v0b<kAH>, dim3(n_v0b), dim3(kThreads), 0, s, descs, dyn, v0b_items, v0part, 1e-5f,
                       net + kAW1, (const float*)bias_eff, kAH, fac_tab, term_tab, bscale);
  HIP_TRY(mark());
  if (n_el > 0) hipLaunchKernelGGL(k_adafac_stats, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac_tab, dec, stats, gl);
  HIP_TRY(mark());
  const Item* seg_items = P->at<Item>(L.off_seg_items);
  double* seg_tot = P->at<double>(L.off_segtot);
  const int n_seg = (int)L.seg_items.size();
  if (n_seg > 0) hipLaunchKernelGGL(k_stat_segsum, dim3(n_seg), dim3(kThreads), 0, s, descs, seg_items, stats, seg_tot);
  hipLaunchKernelGGL(k_lo_reduce, dim3(T), dim3(kFoldThreads), 0, s, descs, dyn, T, stats, seg_tot, totals, LossState{}, vs,
                     (float*)nullptr, 0, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr,
                     (const float*)nullptr, (float*)nullptr, (float*)nullptr);
  HIP_TRY(mark());
  hipLaunchKernelGGL(k_adafac_fold, dim3(T), dim3(kThreads), 0, s, descs, dyn, totals, net, wfold);
  HIP_TRY(mark());
  const Item* ap_items = P->at<Item>(L.off_ap_items);
  const Item* ga_items = P->at<Item>(L.off_ga_items);
  const Item* pp_items = P->at<Item>(L.off_pp_items);
  const int n_ap = (int)L.ap_items.size(), n_ga = (int)L.ga_items.size(), n_pp = (int)L.pp_items.size();
  if (n_ga > 0)
    hipLaunchKernelGGL(k_adafac_apply, dim3(n_ga), dim3(kThreads), 0, s, descs, dyn, ga_items, fac_tab, term_tab, dec,
                       wfold, net, (const float*)bias_eff, gl);
  if (n_pp > 0)
    hipLaunchKernelGGL((k_adafac_apply_tile<true, true>), dim3(n_pp), dim3(kThreads), 0, s, descs, dyn, pp_items, fac_tab,
                       term_tab, dec, wfold, net, gl);
  if (n_ap > 0) {
    if (P->adafac_hf)
      hipLaunchKernelGGL(k_adafac_apply_tile<true>, dim3(n_ap), dim3(kThreads), 0, s, descs, dyn, ap_items, fac_tab,
                         term_tab, dec, wfold, net, gl);
    else
      hipLaunchKernelGGL(k_adafac_apply_tile<false>, dim3(n_ap), dim3(kThreads), 0, s, descs, dyn, ap_items, fac_tab,
                         term_tab, dec, wfold, net, gl);
  }
  HIP_TRY(mark());
  mark.done();
  stage_out(P, s, 0);
  HIP_TRY(hipGetLastError());
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Single-tensor calls with the reference's argument lists
// ---------------------------------------------------------------------------------------------
namespace {

// Geometry as the reference launchers derive it from the parameter tensor (celo2_kernel.cu:306-312):
// sizes and strides of dims dr / dc of a contiguous tensor.
int single_geometry(const char* who, const int64_t* shape, int ndim, int dc, int dr, int vector_like, SingleArgs& a) {
  const std::string w(who);
  if (ndim < 0 || ndim > PYLO_MAX_DIMS || (ndim > 0 && !shape)) return fail(w + ": bad shape");
  long long n = 1;
  for (int i = 0; i < ndim; ++i) {
    if (shape[i] < 0) return fail(w + ": negative dim");
    n *= shape[i];
    if (n >= (1LL << 31)) return fail(w + ": tensors of 2^31 elements or more are not supported");
  }
  a.n = (int)n;
  a.vector_like = vector_like ? 1 : 0;
  if (vector_like) {
    a.num_rows = a.num_cols = a.n;
    a.row_stride = a.col_stride = 1;
    return 0;
  }
  if (dc < 0 || dr < 0 || dc >= ndim || dr >= ndim || dc == dr) return fail(w + ": dc / dr are not two dims of the tensor");
  auto stride = [&](int d) {
    long long st = 1;
    for (int i = d + 1; i < ndim; ++i) st *= shape[i];
    return (int)st;
  };
  a.num_rows = (int)shape[dr];
  a.num_cols = (int)shape[dc];
  a.row_stride = stride(dr);
  a.col_stride = stride(dc);
  if (a.n > 0) {   // then every dim is at least 1
    a.stride_r = a.n / a.num_rows;
    a.stride_c = a.n / a.num_cols;
    a.div_rblock = make_fastdiv((unsigned)a.num_rows * (unsigned)a.row_stride);
    a.div_rstride = make_fastdiv((unsigned)a.row_stride);
    a.div_cblock = make_fastdiv((unsigned)a.num_cols * (unsigned)a.col_stride);
    a.div_cstride = make_fastdiv((unsigned)a.col_stride);
  }
  return 0;
}

template <int F>
int single_check(const char* who, const SingleArgs& a) {
  if (a.n == 0) return 0;
  if (!a.g || !a.p || !a.m || !a.v || !a.fac_r || !a.fac_c || !a.row_factor || !a.second_moment || !a.w_in ||
      !a.b_in || !a.w_h || !a.b_h || !a.w_out || !a.b_out || (!a.vector_like && !a.col_factor) ||
      (F == kFamCelo2 && !a.step_out))
    return fail(std::string(who) + ": null pointer");
  return 0;
}

template <int F, int ST>
void single_enqueue(const SingleArgs& a, int blocks, hipStream_t s) {
  hipLaunchKernelGGL((k_single_moment<F, ST>), dim3(blocks), dim3(kSingleThreads), 0, s, a);
  hipLaunchKernelGGL((k_single_apply<F, ST>), dim3(blocks), dim3(kSingleThreads), 0, s, a);
}

// `dtype`: PYLO_F_STORE_* of every array but `second_moment` (the reference's scalar_t)
template <int F>
int single_launch(const char* who, const SingleArgs& a, void* stream, int dtype = PYLO_F_STORE_F32) {
  if (dtype & ~PYLO_F_STORE_MASK) return fail(std::string(who) + ": dtype must be one of PYLO_F_STORE_*");
  if (a.n == 0) return 0;
  if (int rc = single_check<F>(who, a)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int blocks = std::min((a.n + kSingleThreads - 1) / kSingleThreads, kSingleMaxBlocks);
  switch (dtype >> 8) {
    case kStoreF16: single_enqueue<F, kStoreF16>(a, blocks, s); break;
    case kStoreBF16: single_enqueue<F, kStoreBF16>(a, blocks, s); break;
    case kStoreF64: single_enqueue<F, kStoreF64>(a, blocks, s); break;
    default: single_enqueue<F, kStoreF32>(a, blocks, s);
  }
  HIP_TRY(hipGetLastError());
  return 0;
}

}  // namespace

extern "C" int pylo_mi355_celo2_kernel(const float* g, const float* p, const float* m, const float* v,
                                       const float* fac_r, const float* fac_c, const float* row_factor,
                                       const float* col_factor, float* second_moment, const float* w_in,
                                       const float* b_in, const float* w_h, const float* b_h, const float* w_out,
                                       const float* b_out, float* step_out, float exp_mult, const int64_t* shape,
                                       int ndim, int dc, int dr, int vector_like, void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("celo2_kernel", shape, ndim, dc, dr, vector_like, a)) return rc;
  a.g = g; a.p = const_cast<float*>(p); a.m = m; a.v = v; a.fac_r = fac_r; a.fac_c = fac_c;
  a.row_factor = row_factor; a.col_factor = col_factor; a.second_moment = second_moment;
  a.w_in = w_in; a.b_in = b_in; a.w_h = w_h; a.b_h = b_h; a.w_out = w_out; a.b_out = b_out;
  a.step_out = step_out; a.exp_mult = exp_mult;
  return single_launch<kFamCelo2>("celo2_kernel", a, stream);
}

extern "C" int pylo_mi355_learned_optimizer_kernel(const float* g, float* p, const float* m, const float* v,
                                                   const float* fac_r, const float* fac_c, const float* row_factor,
                                                   const float* col_factor, float* second_moment,
                                                   const float* input_weights, const float* input_bias,
                                                   const float* hidden_weights, const float* hidden_bias,
                                                   const float* output_weights, const float* output_bias, float lr,
                                                   float step_mult, float exp_mult, float epsilon, float step,
                                                   float weight_decay, const int64_t* shape, int ndim, int dc, int dr,
                                                   int vector_like, void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("learned_optimizer_kernel", shape, ndim, dc, dr, vector_like, a)) return rc;
  a.g = g; a.p = p; a.m = m; a.v = v; a.fac_r = fac_r; a.fac_c = fac_c;
  a.row_factor = row_factor; a.col_factor = col_factor; a.second_moment = second_moment;
  a.w_in = input_weights; a.b_in = input_bias; a.w_h = hidden_weights; a.b_h = hidden_bias;
  a.w_out = output_weights; a.b_out = output_bias;
  a.lr = lr; a.step_mult = step_mult; a.exp_mult = exp_mult; a.epsilon = epsilon; a.step = step;
  a.weight_decay = weight_decay;
  return single_launch<kFamLo>("learned_optimizer_kernel", a, stream);
}

extern "C" int pylo_mi355_velo_kernel_simple(const float* grad, float* param, const float* momentum, const float* rms,
                                             const float* row_factor, const float* col_factor,
                                             const float* fac_vec_row, const float* fac_vec_col, float* second_moment,
                                             const float* input_weights, const float* input_bias,
                                             const float* hidden_weights, const float* hidden_bias,
                                             const float* output_weights, const float* output_bias, float lr,
                                             float step_mult, float exp_mult, float epsilon, float weight_decay,
                                             const int64_t* shape, int ndim, int dc, int dr, int vector_like,
                                             void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("velo_kernel_simple", shape, ndim, dc, dr, vector_like, a)) return rc;
  a.g = grad; a.p = param; a.m = momentum; a.v = rms; a.fac_r = fac_vec_row; a.fac_c = fac_vec_col;
  a.row_factor = row_factor; a.col_factor = col_factor; a.second_moment = second_moment;
  a.w_in = input_weights; a.b_in = input_bias; a.w_h = hidden_weights; a.b_h = hidden_bias;
  a.w_out = output_weights; a.b_out = output_bias;
  a.lr = lr; a.step_mult = step_mult; a.exp_mult = exp_mult; a.epsilon = epsilon; a.weight_decay = weight_decay;
  return single_launch<kFamVelo>("velo_kernel_simple", a, stream);
}

// The same three calls for arrays of another element type (the reference's AT_DISPATCH_FLOATING_TYPES_AND_HALF
// over p.scalar_type(), celo2_kernel.cu:314,328, learned_optimizer.cu:338,364, velo_kernel.cu:405,427): every
// array but `second_moment` holds elements of `dtype`.
#define PYLO_AS_F(x) static_cast<const float*>(x)
extern "C" int pylo_mi355_celo2_kernel_typed(int dtype, const void* g, const void* p, const void* m, const void* v,
                                             const void* fac_r, const void* fac_c, const void* row_factor,
                                             const void* col_factor, float* second_moment, const void* w_in,
                                             const void* b_in, const void* w_h, const void* b_h, const void* w_out,
                                             const void* b_out, void* step_out, float exp_mult, const int64_t* shape,
                                             int ndim, int dc, int dr, int vector_like, void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("celo2_kernel", shape, ndim, dc, dr, vector_like, a)) return rc;
  a.g = PYLO_AS_F(g); a.p = const_cast<float*>(PYLO_AS_F(p)); a.m = PYLO_AS_F(m); a.v = PYLO_AS_F(v);
  a.fac_r = PYLO_AS_F(fac_r); a.fac_c = PYLO_AS_F(fac_c);
  a.row_factor = PYLO_AS_F(row_factor); a.col_factor = PYLO_AS_F(col_factor); a.second_moment = second_moment;
  a.w_in = PYLO_AS_F(w_in); a.b_in = PYLO_AS_F(b_in); a.w_h = PYLO_AS_F(w_h); a.b_h = PYLO_AS_F(b_h);
  a.w_out = PYLO_AS_F(w_out); a.b_out = PYLO_AS_F(b_out);
  a.step_out = static_cast<float*>(step_out); a.exp_mult = exp_mult;
  return single_launch<kFamCelo2>("celo2_kernel", a, stream, dtype);
}

extern "C" int pylo_mi355_learned_optimizer_kernel_typed(int dtype, const void* g, void* p, const void* m, const void* v,
                                                         const void* fac_r, const void* fac_c, const void* row_factor,
                                                         const void* col_factor, float* second_moment,
                                                         const void* input_weights, const void* input_bias,
                                                         const void* hidden_weights, const void* hidden_bias,
                                                         const void* output_weights, const void* output_bias, float lr,
                                                         float step_mult, float exp_mult, float epsilon, float step,
                                                         float weight_decay, const int64_t* shape, int ndim, int dc,
                                                         int dr, int vector_like, void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("learned_optimizer_kernel", shape, ndim, dc, dr, vector_like, a)) return rc;
  a.g = PYLO_AS_F(g); a.p = static_cast<float*>(p); a.m = PYLO_AS_F(m); a.v = PYLO_AS_F(v);
  a.fac_r = PYLO_AS_F(fac_r); a.fac_c = PYLO_AS_F(fac_c);
  a.row_factor = PYLO_AS_F(row_factor); a.col_factor = PYLO_AS_F(col_factor); a.second_moment = second_moment;
  a.w_in = PYLO_AS_F(input_weights); a.b_in = PYLO_AS_F(input_bias); a.w_h = PYLO_AS_F(hidden_weights);
  a.b_h = PYLO_AS_F(hidden_bias); a.w_out = PYLO_AS_F(output_weights); a.b_out = PYLO_AS_F(output_bias);
  a.lr = lr; a.step_mult = step_mult; a.exp_mult = exp_mult; a.epsilon = epsilon; a.step = step;
  a.weight_decay = weight_decay;
  return single_launch<kFamLo>("learned_optimizer_kernel", a, stream, dtype);
}

extern "C" int pylo_mi355_velo_kernel_simple_typed(int dtype, const void* grad, void* param, const void* momentum,
                                                   const void* rms, const void* row_factor, const void* col_factor,
                                                   const void* fac_vec_row, const void* fac_vec_col,
                                                   float* second_moment, const void* input_weights,
                                                   const void* input_bias, const void* hidden_weights,
                                                   const void* hidden_bias, const void* output_weights,
                                                   const void* output_bias, float lr, float step_mult, float exp_mult,
                                                   float epsilon, float weight_decay, const int64_t* shape, int ndim,
                                                   int dc, int dr, int vector_like, void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("velo_kernel_simple", shape, ndim, dc, dr, vector_like, a)) return rc;
  a.g = PYLO_AS_F(grad); a.p = static_cast<float*>(param); a.m = PYLO_AS_F(momentum); a.v = PYLO_AS_F(rms);
  a.fac_r = PYLO_AS_F(fac_vec_row); a.fac_c = PYLO_AS_F(fac_vec_col);
  a.row_factor = PYLO_AS_F(row_factor); a.col_factor = PYLO_AS_F(col_factor); a.second_moment = second_moment;
  a.w_in = PYLO_AS_F(input_weights); a.b_in = PYLO_AS_F(input_bias); a.w_h = PYLO_AS_F(hidden_weights);
  a.b_h = PYLO_AS_F(hidden_bias); a.w_out = PYLO_AS_F(output_weights); a.b_out = PYLO_AS_F(output_bias);
  a.lr = lr; a.step_mult = step_mult; a.exp_mult = exp_mult; a.epsilon = epsilon; a.weight_decay = weight_decay;
  return single_launch<kFamVelo>("velo_kernel_simple", a, stream, dtype);
}
#undef PYLO_AS_F

// ---------------------------------------------------------------------------------------------
// celo2_kernel for callers that cannot allocate: the per-channel sums live in the library's own
// device array instead of a caller-supplied `second_moment`
// ---------------------------------------------------------------------------------------------
namespace {

constexpr int kScratchFloats = 64;   // 30 channel sums, padded to one 256-byte line
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices];   // device address of `scratch` per GPU, resolved on first use
std::mutex g_scratch_mu;

// The array's name is a host-side stand-in, not a device address: each GPU holds its own copy at its
// own address, looked up once per device with that device current.
int scratch_on_current_device(float** out) {
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail("celo2_kernel_noalloc: device index out of range");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail("celo2_kernel_noalloc: no device address for the scratch array");
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// a fill kernel rather than a memset node: callers may record the call into a HIP graph
__global__ __launch_bounds__(64) void k_scratch_clear(float* __restrict__ s) { s[threadIdx.x] = 0.0f; }

}  // namespace

extern "C" int pylo_mi355_celo2_kernel_noalloc(const float* g, const float* p, const float* m, const float* v,
                                               const float* fac_r, const float* fac_c, const float* row_factor,
                                               const float* col_factor, const float* w_in, const float* b_in,
                                               const float* w_h, const float* b_h, const float* w_out,
                                               const float* b_out, float* step_out, float exp_mult,
                                               const int64_t* shape, int ndim, int dc, int dr, int vector_like,
                                               void* stream) {
  SingleArgs a{};
  if (int rc = single_geometry("celo2_kernel_noalloc", shape, ndim, dc, dr, vector_like, a)) return rc;
  float* sums = nullptr;
  if (int rc = scratch_on_current_device(&sums)) return rc;
  a.g = g; a.p = const_cast<float*>(p); a.m = m; a.v = v; a.fac_r = fac_r; a.fac_c = fac_c;
  a.row_factor = row_factor; a.col_factor = col_factor; a.second_moment = sums;
  a.w_in = w_in; a.b_in = b_in; a.w_h = w_h; a.b_h = b_h; a.w_out = w_out; a.b_out = b_out;
  a.step_out = step_out; a.exp_mult = exp_mult;
  if (a.n == 0) return 0;
  if (int rc = single_check<kFamCelo2>("celo2_kernel_noalloc", a)) return rc;
  // the array keeps the previous call's sums: they start at zero on every call
  hipLaunchKernelGGL(k_scratch_clear, dim3(1), dim3(kScratchFloats), 0, static_cast<hipStream_t>(stream), sums);
  return single_launch<kFamCelo2>("celo2_kernel_noalloc", a, stream);
}

// ---------------------------------------------------------------------------------------------
// Bare streaming kernel (benchmark instrumentation): the rate the memory system gives an access mix
// ---------------------------------------------------------------------------------------------
namespace {

template <int R, int W, bool NT>
__global__ __launch_bounds__(kThreads) void k_stream_probe(const float* __restrict__ in, float* __restrict__ out,
                                                           size_t n) {
  constexpr int kIters = 8;
  const size_t base = (size_t)blockIdx.x * kThreads * 4 * kIters;
  for (int it = 0; it < kIters; ++it) {
    const size_t i = base + ((size_t)it * kThreads + threadIdx.x) * 4;
    if (i >= n) break;
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const gv4f* p = (const gv4f*)(in + (size_t)r * n + i);
      acc += NT ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int w = 0; w < W; ++w) {
      gv4f* p = (gv4f*)(out + (size_t)w * n + i);
      const v4f v = acc * (float)(w + 1);
      if (NT) __builtin_nontemporal_store(v, p);
      else *p = v;
    }
    if (W == 0 && acc.x == 123.456f) out[0] = acc.y;   // keeps the loads of a read-only mix alive
  }
}

template <int R, int W>
void stream_launch(const float* in, float* out, size_t n, bool nt, hipStream_t s) {
  const unsigned grid = (unsigned)((n + (size_t)kThreads * 4 * 8 - 1) / ((size_t)kThreads * 4 * 8));
  if (nt) hipLaunchKernelGGL((k_stream_probe<R, W, true>), dim3(grid), dim3(kThreads), 0, s, in, out, n);
  else hipLaunchKernelGGL((k_stream_probe<R, W, false>), dim3(grid), dim3(kThreads), 0, s, in, out, n);
}

}  // namespace

extern "C" int pylo_mi355_stream_probe(const float* in, float* out, size_t n, int reads, int writes, int nontemporal,
                                       void* stream) {
  if (!in || !out || n == 0 || n % 4 != 0) return fail("stream_probe: null pointer or n not a multiple of 4");
  if ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) % 16 != 0)
    return fail("stream_probe: 16-byte alignment needed");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool nt = nontemporal != 0;
  if (reads == 6 && writes == 5) stream_launch<6, 5>(in, out, n, nt, s);
  else if (reads == 6 && writes == 0) stream_launch<6, 0>(in, out, n, nt, s);
  else if (reads == 6 && writes == 1) stream_launch<6, 1>(in, out, n, nt, s);
  else if (reads == 1 && writes == 1) stream_launch<1, 1>(in, out, n, nt, s);
  else if (reads == 1 && writes == 0) stream_launch<1, 0>(in, out, n, nt, s);
  else if (reads == 1 && writes == 5) stream_launch<1, 5>(in, out, n, nt, s);
  else return fail("stream_probe: reads must be 1 or 6, writes 0, 1 or 5");
  HIP_TRY(hipGetLastError());
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Bare matrix-pipe kernel (benchmark instrumentation): what the fp16 matrix instructions deliver for the
// instruction mix of the Newton-Schulz update product, with parts of its data path taken away
// ---------------------------------------------------------------------------------------------
namespace {

// The main loop of k_ns_hf_gemm<kNsUpdate, 4> (128 x 256 outputs, three v_mfma_f32_32x32x16_f16 per pair of
// 32 x 32 blocks and 16 reduction steps) over synthetic planes.  MODE 0: as in the product (operands staged
// from memory into LDS every 16 steps); 1: the first stage is staged once and read from LDS in every step (no
// global loads, no barriers); 2: the first stage's fragments stay in registers (matrix instructions only).
template <int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_matrix_probe(
    const hbits* __restrict__ X, int rows_x, const hbits* __restrict__ B, int rows_b, int K, float* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) char lds_[];
  PYLO_LDS char* lds = (PYLO_LDS char*)lds_;
  constexpr int WN = 4, RB = 64 * WN, SA = 128 * kNsRowB;
  const int nj = rows_b / RB, i0 = (blockIdx.x / nj) * 128, j0 = (blockIdx.x % nj) * RB;
  v16f acc[2][WN];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const HfPlanes PX{X, rows_x}, PB{B, rows_b};
  if (MODE == 0) {
    hf_tile_product<WN>(PX, i0, PB, j0, 0, K, lds, acc);
  } else if (MODE == 4) {
    hf_tile_product_direct<WN>(PX, i0, PB, j0, 0, K, lds, acc);
  } else {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wi = (wave >> 1) * 64, wj = (wave & 1) * 32 * WN;
    const int kg = lane >> 5, lo = lane & 31;
    int offa[128 * kNsRowPc / 256], offb[RB * kNsRowPc / 256];
    hf_stage_offsets<128>(wave, lane, offa);
    hf_stage_offsets<RB>(wave, lane, offb);
    hf_stage_issue<128>((const char*)X + (size_t)i0 * kNsRowB, offa, lds, wave);
    hf_stage_issue<RB>((const char*)B + (size_t)j0 * kNsRowB, offb, lds + SA, wave);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    const int sw = 16 * (kg ^ ((lo >> 2) & 3));
    const int oa = (wi + lo) * kNsRowB + sw, ob = SA + (wj + lo) * kNsRowB + sw;
    f16x8 a[2][kNsPl], b[WN][kNsPl];
    for (int k = 0; k < K; k += kHfBK) {
      if (MODE == 1 || k == 0) {
#pragma unroll
        for (int q = 0; q < kNsPl; ++q) {
#pragma unroll
          for (int i = 0; i < 2; ++i) a[i][q] = __builtin_bit_cast(f16x8, *(const luint4*)(lds + ((oa + i * 32 * kNsRowB) ^ (q * 32))));
#pragma unroll
          for (int j = 0; j < WN; ++j) b[j][q] = __builtin_bit_cast(f16x8, *(const luint4*)(lds + ((ob + j * 32 * kNsRowB) ^ (q * 32))));
        }
      }
#pragma unroll
      for (int term = 0; term < 3; ++term) {
        constexpr int pa[3] = {1, 0, 0}, pb[3] = {0, 1, 0};
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
#pragma unroll
          for (int hj = 0; hj < WN; ++hj)
            acc[hi][hj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[hi][pa[term]], b[hj][pb[term]], acc[hi][hj], 0, 0, 0);
      }
      if (MODE == 1) asm volatile("" ::: "memory");   // the fragments are read again in the next step
    }
  }
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = sum;
}

// MODE 3: the same loop with tiles of 256 x 256 outputs by 512 threads (4 x 2 waves of 64 x 128): two thirds of the
// bytes staged per product.
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void k_matrix_probe_wide(
    const hbits* __restrict__ X, int rows_x, const hbits* __restrict__ B, int rows_b, int K, float* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) char lds_[];
  PYLO_LDS char* lds = (PYLO_LDS char*)lds_;
  constexpr int WN = 4;
  const int nj = rows_b / 256, i0 = (blockIdx.x / nj) * 256, j0 = (blockIdx.x % nj) * 256;
  v16f acc[2][WN];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const HfPlanes PX{X, rows_x}, PB{B, rows_b};
  hf_tile_product<WN, 8>(PX, i0, PB, j0, 0, K, lds, acc);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
  out[(size_t)blockIdx.x * 512 + threadIdx.x] = sum;
}

}  // namespace

extern "C" int pylo_mi355_matrix_probe(const void* x_planes, int rows_x, const void* b_planes, int rows_b, int k_steps,
                                       int mode, float* out, void* stream) {
  if (!x_planes || !b_planes || !out) return fail("matrix_probe: null pointer");
  if (rows_x <= 0 || rows_x % 128 != 0 || rows_b <= 0 || rows_b % 256 != 0 || k_steps <= 0 || k_steps % 16 != 0)
    return fail("matrix_probe: rows_x must be a multiple of 128, rows_b of 256, k_steps of 16");
  if (mode < 0 || mode > 4) return fail("matrix_probe: mode must be 0 .. 4");
  if (mode == 3 && rows_x % 256 != 0) return fail("matrix_probe: mode 3 takes rows_x in multiples of 256");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned grid = (unsigned)(rows_x / 128) * (unsigned)(rows_b / 256);
  static std::mutex mu;
  {
    std::lock_guard<std::mutex> lock(mu);
    HIP_TRY(hipFuncSetAttribute((const void*)k_matrix_probe<0>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(4)));
    HIP_TRY(hipFuncSetAttribute((const void*)k_matrix_probe<1>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(4)));
    HIP_TRY(hipFuncSetAttribute((const void*)k_matrix_probe<2>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(4)));
    HIP_TRY(hipFuncSetAttribute((const void*)k_matrix_probe_wide, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 512 * kNsRowB));
    HIP_TRY(hipFuncSetAttribute((const void*)k_matrix_probe<4>, hipFuncAttributeMaxDynamicSharedMemorySize, hf_gemm_lds(4)));
  }
  const hbits* X = static_cast<const hbits*>(x_planes);
  const hbits* B = static_cast<const hbits*>(b_planes);
  if (mode == 0) hipLaunchKernelGGL(k_matrix_probe<0>, dim3(grid), dim3(256), hf_gemm_lds(4), s, X, rows_x, B, rows_b, k_steps, out);
  else if (mode == 1) hipLaunchKernelGGL(k_matrix_probe<1>, dim3(grid), dim3(256), hf_gemm_lds(4), s, X, rows_x, B, rows_b, k_steps, out);
  else if (mode == 2) hipLaunchKernelGGL(k_matrix_probe<2>, dim3(grid), dim3(256), hf_gemm_lds(4), s, X, rows_x, B, rows_b, k_steps, out);
  else if (mode == 3) hipLaunchKernelGGL(k_matrix_probe_wide, dim3(grid / 2), dim3(512), 2 * 512 * kNsRowB, s, X, rows_x, B, rows_b, k_steps, out);
  else hipLaunchKernelGGL(k_matrix_probe<4>, dim3(grid), dim3(256), 2 * 256 * kNsRowB, s, X, rows_x, B, rows_b, k_steps, out);
  HIP_TRY(hipGetLastError());
  return 0;
}
