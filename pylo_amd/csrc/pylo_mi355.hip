// Fused learned-optimizer step for MI355X (gfx950): the C ABI of include/pylo_mi355.h.
//
// Pipeline of one ELO-CELO2 step over all tensors of a plan (8 launches, no host sync):
//   k_p0 (pass 0)   row / column sums of g^2 per tile, sum g^2 and clamp flag per block     4 B/elem
//   k_gnorm         global gradient norm, clamp flag
//   k_p0 (pass 1)   exits at once unless some |g| exceeded the clamp: redoes the sums exactly
//   k_v0a           fac_r / fac_c EMAs per 64 vector entries, partial sums of their statistics
//   k_v0b           row / column factor tables; the 12 row-only / column-only feature channels
//                   normalised and folded into 8-float first-layer terms per row / column
//   k_celo2_stats   sum of squares of the 18 per-element channels (accumulators advanced in
//                   registers, nothing written); AdamW tensors are fully updated here      24 B/elem
//   k_celo2_fold    per tensor: normalisation scales folded into the first-layer weights
//   k_celo2_apply   accumulators advanced and written, features, MLP, step_out             44 B/elem
#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#include "k_celo2.h"
#include "k_gradstats.h"
#include "pylo_common.h"

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

struct Layout {
  std::vector<TDesc> descs;
  std::vector<Item> p0_items, el_items, v0a_items, v0b_items;
  std::vector<int> fac_list;
  std::vector<int> dc, dr;
  int H = 8;  // width of the first MLP layer (terms per row / column)
  size_t off_descs, off_dyn, off_p0_items, off_el_items, off_v0a_items, off_v0b_items, off_fac_list,
      off_rowpart, off_colpart, off_gsq, off_flag, off_globals, off_fac0, off_fac1, off_term0, off_term1,
      off_v0part, off_bscale, off_stats, off_wfold, off_chan_ms, total;
};

int build_layout(int kind, const PyloTensorShape* shapes, int T, Layout& L) {
  if (kind != PYLO_KIND_CELO2) return fail("plan: only PYLO_KIND_CELO2 is implemented");
  if (T <= 0 || shapes == nullptr) return fail("plan: no tensors");
  L.descs.assign(T, TDesc{});
  L.dc.assign(T, -1);
  L.dr.assign(T, -1);
  long long rowpart = 0, colpart = 0, fac0 = 0, fac1 = 0, term0 = 0, term1 = 0;
  const int H = L.H;
  for (int t = 0; t < T; ++t) {
    const PyloTensorShape& s = shapes[t];
    if (s.ndim < 0 || s.ndim > PYLO_MAX_DIMS) return fail("plan: bad ndim");
    long long n = 1;
    for (int i = 0; i < s.ndim; ++i) {
      if (s.shape[i] < 0) return fail("plan: negative dim");
      n *= s.shape[i];
    }
    if (n >= (1ll << 31)) return fail("plan: tensors of 2^31 or more elements are not supported");
    TDesc& d = L.descs[t];
    d.n = n;
    d.fac_slot = -1;
    const bool adam = (s.flags & PYLO_F_ADAM) != 0 || s.ndim < 2;
    if (kind == PYLO_KIND_CELO2 && s.ndim < 2 && !(s.flags & PYLO_F_ADAM))
      return fail("plan: CELO2 tensors with fewer than 2 dims must carry PYLO_F_ADAM");
    if (adam) {
      d.mode = kModeFlat;
      d.vec = (n % 4 == 0) ? 4 : 1;
    } else {
      if (s.ndim != 2) return fail("plan: CELO2 tensors with more than 2 dims are not supported yet");
      int dc, dr;
      factored_dims(kind, s, &dc, &dr);
      L.dc[t] = dc;
      L.dr[t] = dr;
      d.mode = kModeFac2D;
      d.R0 = (int)s.shape[0];
      d.C0 = (int)s.shape[1];
      d.vec = (d.C0 % 4 == 0) ? 4 : 1;
      d.r_is_dim0 = (dr == 1) ? 1 : 0;
      d.len_r = d.r_is_dim0 ? d.R0 : d.C0;
      d.len_c = d.r_is_dim0 ? d.C0 : d.R0;
      d.n_strips = (d.R0 + kP0Rows - 1) / kP0Rows;
      d.n_colblk = (d.C0 + 64 * d.vec - 1) / (64 * d.vec);
      d.rowpart_off = rowpart;
      d.colpart_off = colpart;
      rowpart += (long long)d.n_colblk * d.R0;
      colpart += (long long)d.n_strips * d.C0;
      d.C0r = (d.C0 + 3) / 4 * 4;
      d.fac0_off = fac0;
      d.fac1_off = fac1;
      d.term0_off = term0;
      d.term1_off = term1;
      fac0 += (long long)d.R0 * 4;
      fac1 += 3ll * d.C0r;
      term0 += (long long)d.R0 * H;
      term1 += (long long)H * d.C0r;
      d.fac_slot = -1;
      if (n > 0) {
        d.fac_slot = (int)L.fac_list.size();
        L.fac_list.push_back(t);
        for (int which = 0; which < 2; ++which) {
          const int len = which ? d.C0 : d.R0;
          d.v0a_first[which] = (int)L.v0a_items.size();
          for (int c = 0; c * kV0aEnt < len; ++c) L.v0a_items.push_back(Item{t, c, which, 0});
          d.v0a_n[which] = (int)L.v0a_items.size() - d.v0a_first[which];
          for (int c = 0; c * kV0bEnt < len; ++c) L.v0b_items.push_back(Item{t, c, which, 0});
        }
      }
    }
    // P0 items
    if (n > 0) {
      if (d.mode == kModeFac2D) {
        for (int st = 0; st < d.n_strips; ++st)
          for (int cb = 0; cb < d.n_colblk; ++cb) L.p0_items.push_back(Item{t, st, cb, 0});
      } else {
        const long long chunk = (long long)kThreads * d.vec * kElemIters;
        for (long long c = 0; c * chunk < n; ++c) L.p0_items.push_back(Item{t, (int)c, 0, 0});
      }
    }
    // element items
    const long long chunk = (long long)kThreads * d.vec * kElemIters;
    d.blk0 = (int)L.el_items.size();
    for (long long c = 0; c * chunk < n; ++c) L.el_items.push_back(Item{t, (int)c, 0, 0});
    d.nblk = (int)L.el_items.size() - d.blk0;
  }
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off = align_up(off + bytes);
    return o;
  };
  const size_t nfac = std::max<size_t>(L.fac_list.size(), 1);
  L.off_descs = take(sizeof(TDesc) * T);
  L.off_dyn = take(sizeof(PyloTensorArgs) * T);
  L.off_p0_items = take(sizeof(Item) * std::max<size_t>(L.p0_items.size(), 1));
  L.off_el_items = take(sizeof(Item) * std::max<size_t>(L.el_items.size(), 1));
  L.off_v0a_items = take(sizeof(Item) * std::max<size_t>(L.v0a_items.size(), 1));
  L.off_v0b_items = take(sizeof(Item) * std::max<size_t>(L.v0b_items.size(), 1));
  L.off_fac_list = take(sizeof(int) * nfac);
  L.off_rowpart = take(sizeof(float) * std::max<long long>(rowpart, 1));
  L.off_colpart = take(sizeof(float) * std::max<long long>(colpart, 1));
  L.off_gsq = take(sizeof(double) * std::max<size_t>(L.p0_items.size(), 1));
  L.off_flag = take(sizeof(int) * std::max<size_t>(L.p0_items.size(), 1));
  L.off_globals = take(sizeof(Globals));
  L.off_fac0 = take(sizeof(float) * std::max<long long>(fac0, 4));
  L.off_fac1 = take(sizeof(float) * std::max<long long>(fac1, 4));
  L.off_term0 = take(sizeof(float) * std::max<long long>(term0, 4));
  L.off_term1 = take(sizeof(float) * std::max<long long>(term1, 4));
  L.off_v0part = take(sizeof(double) * kNV0 * std::max<size_t>(L.v0a_items.size(), 1));
  L.off_bscale = take(sizeof(BScale) * nfac);
  L.off_stats = take(sizeof(double) * kNStat * std::max<size_t>(L.el_items.size(), 1));
  L.off_wfold = take(sizeof(float) * kC2Fold * nfac);
  L.off_chan_ms = take(sizeof(float) * kNStat * nfac);
  L.total = off;
  return 0;
}

constexpr int kStageSlots = 4;

}  // namespace

struct PyloPlan {
  int kind = 0, T = 0;
  Layout L;
  char* ws = nullptr;
  PyloTensorArgs* stage[kStageSlots] = {nullptr, nullptr, nullptr, nullptr};
  hipEvent_t ev[kStageSlots] = {nullptr, nullptr, nullptr, nullptr};
  bool ev_used[kStageSlots] = {false, false, false, false};
  int slot = 0;
  std::vector<PyloTensorArgs> last;
  bool have_last = false;
  // optional per-launch timing (pylo_mi355_plan_timing_begin/end)
  std::vector<hipEvent_t> tev;
  int t_steps_max = 0, t_steps = 0, t_per_step = 0;
  bool timing = false;

  template <class Tp>
  Tp* at(size_t off) const { return reinterpret_cast<Tp*>(ws + off); }
};

extern "C" {

int pylo_mi355_abi_version(void) { return PYLO_MI355_ABI_VERSION; }

const char* pylo_mi355_last_error(void) { return g_err.c_str(); }

int pylo_mi355_plan_workspace_bytes(int kind, const PyloTensorShape* shapes, int n_tensors, size_t* bytes_out) {
  if (!bytes_out) return fail("workspace_bytes: null output");
  Layout L;
  if (int rc = build_layout(kind, shapes, n_tensors, L)) return rc;
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
  if (int rc = build_layout(kind, shapes, n_tensors, P->L)) { delete P; return rc; }
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
  if (e == hipSuccess) e = up(L.off_el_items, L.el_items.data(), sizeof(Item) * L.el_items.size());
  if (e == hipSuccess) e = up(L.off_fac_list, L.fac_list.data(), sizeof(int) * L.fac_list.size());
  if (e == hipSuccess) e = up(L.off_v0a_items, L.v0a_items.data(), sizeof(Item) * L.v0a_items.size());
  if (e == hipSuccess) e = up(L.off_v0b_items, L.v0b_items.data(), sizeof(Item) * L.v0b_items.size());
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  for (int i = 0; i < kStageSlots && e == hipSuccess; ++i) {
    e = hipHostMalloc(reinterpret_cast<void**>(&P->stage[i]), sizeof(PyloTensorArgs) * n_tensors, hipHostMallocDefault);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&P->ev[i], hipEventDisableTiming);
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
  for (int i = 0; i < kStageSlots; ++i) {
    if (P->ev[i]) (void)hipEventDestroy(P->ev[i]);
    if (P->stage[i]) (void)hipHostFree(P->stage[i]);
  }
  delete P;
  return 0;
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

int pylo_mi355_plan_num_launches(const PyloPlan* P) {
  if (!P) return -1;
  return P->kind == PYLO_KIND_CELO2 ? 8 : -1;
}

const char* pylo_mi355_plan_launch_name(const PyloPlan* P, int launch) {
  static const char* celo2[] = {"k_p0(sums)", "k_gnorm", "k_p0(exact)", "k_v0a", "k_v0b",
                                "k_celo2_stats", "k_celo2_fold", "k_celo2_apply"};
  if (!P || launch < 0 || launch >= pylo_mi355_plan_num_launches(P)) return "";
  return celo2[launch];
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
int upload_args(PyloPlan* P, const PyloTensorArgs* args, hipStream_t s) {
  const size_t bytes = sizeof(PyloTensorArgs) * P->T;
  if (P->have_last && std::memcmp(P->last.data(), args, bytes) == 0) return 0;
  const int i = P->slot;
  P->slot = (P->slot + 1) % kStageSlots;
  if (P->ev_used[i]) HIP_TRY(hipEventSynchronize(P->ev[i]));
  std::memcpy(P->stage[i], args, bytes);
  HIP_TRY(hipMemcpyAsync(P->ws + P->L.off_dyn, P->stage[i], bytes, hipMemcpyHostToDevice, s));
  HIP_TRY(hipEventRecord(P->ev[i], s));
  P->ev_used[i] = true;
  P->last.assign(args, args + P->T);
  P->have_last = true;
  return 0;
}

int check_args(const PyloPlan* P, const PyloTensorArgs* args) {
  for (int t = 0; t < P->T; ++t) {
    const TDesc& d = P->L.descs[t];
    const PyloTensorArgs& a = args[t];
    if (a.grad == nullptr || d.n == 0) continue;
    if (!a.param || !a.mom || !a.rms) return fail("step: null param/mom/rms pointer at tensor " + std::to_string(t));
    if (d.mode == kModeFac2D && (!a.fac_r || !a.fac_c || !a.step_out))
      return fail("step: null fac_r/fac_c/step_out pointer at tensor " + std::to_string(t));
    const uintptr_t m = reinterpret_cast<uintptr_t>(a.grad) | reinterpret_cast<uintptr_t>(a.param) |
                        reinterpret_cast<uintptr_t>(a.mom) | reinterpret_cast<uintptr_t>(a.rms) |
                        reinterpret_cast<uintptr_t>(a.fac_r) | reinterpret_cast<uintptr_t>(a.fac_c) |
                        reinterpret_cast<uintptr_t>(a.step_out);
    if (m % 16 != 0) return fail("step: pointers must be 16-byte aligned (tensor " + std::to_string(t) + ")");
  }
  return 0;
}

}  // namespace

extern "C" int pylo_mi355_celo2_step(PyloPlan* P, const PyloTensorArgs* args, const PyloDecays* decays,
                                     const float* mlp, void* stream) {
  if (!P || !args || !decays || !mlp) return fail("celo2_step: null argument");
  if (P->kind != PYLO_KIND_CELO2) return fail("celo2_step: plan is not a CELO2 plan");
  if (int rc = check_args(P, args)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = upload_args(P, args, s)) return rc;
  const Layout& L = P->L;
  const TDesc* descs = P->at<TDesc>(L.off_descs);
  const PyloTensorArgs* dyn = P->at<PyloTensorArgs>(L.off_dyn);
  const Item* p0_items = P->at<Item>(L.off_p0_items);
  const Item* el_items = P->at<Item>(L.off_el_items);
  const int* fac_list = P->at<int>(L.off_fac_list);
  float* rowpart = P->at<float>(L.off_rowpart);
  float* colpart = P->at<float>(L.off_colpart);
  double* gsq = P->at<double>(L.off_gsq);
  int* flag = P->at<int>(L.off_flag);
  Globals* gl = P->at<Globals>(L.off_globals);
  const Item* v0a_items = P->at<Item>(L.off_v0a_items);
  const Item* v0b_items = P->at<Item>(L.off_v0b_items);
  float* fac0 = P->at<float>(L.off_fac0);
  float* fac1 = P->at<float>(L.off_fac1);
  float* term0 = P->at<float>(L.off_term0);
  float* term1 = P->at<float>(L.off_term1);
  double* v0part = P->at<double>(L.off_v0part);
  BScale* bscale = P->at<BScale>(L.off_bscale);
  const int n_v0a = (int)L.v0a_items.size(), n_v0b = (int)L.v0b_items.size();
  double* stats = P->at<double>(L.off_stats);
  float* wfold = P->at<float>(L.off_wfold);
  float* chan_ms = P->at<float>(L.off_chan_ms);
  const int n_p0 = (int)L.p0_items.size(), n_el = (int)L.el_items.size(), n_fac = (int)L.fac_list.size();
  const PyloDecays dec = *decays;

  const bool timed = P->timing && P->t_steps < P->t_steps_max;
  hipEvent_t* ev = timed ? &P->tev[(size_t)P->t_steps * P->t_per_step] : nullptr;
  int mark = 0;
#define PYLO_MARK() do { if (timed) HIP_TRY(hipEventRecord(ev[mark++], s)); } while (0)
  PYLO_MARK();
  if (n_p0 > 0) hipLaunchKernelGGL(k_p0, dim3(n_p0), dim3(kThreads), 0, s, descs, dyn, p0_items, rowpart, colpart, gsq, flag, gl, 0);
  PYLO_MARK();
  hipLaunchKernelGGL(k_gnorm, dim3(1), dim3(kThreads), 0, s, gsq, flag, n_p0, gl);
  PYLO_MARK();
  if (n_p0 > 0) hipLaunchKernelGGL(k_p0, dim3(n_p0), dim3(kThreads), 0, s, descs, dyn, p0_items, rowpart, colpart, gsq, flag, gl, 1);
  PYLO_MARK();
  if (n_v0a > 0)
    hipLaunchKernelGGL(k_v0a, dim3(n_v0a), dim3(kThreads), 0, s, descs, dyn, v0a_items, rowpart, colpart, gl, dec, v0part);
  PYLO_MARK();
  if (n_v0b > 0)
    hipLaunchKernelGGL(k_v0b<8>, dim3(n_v0b), dim3(kThreads), 0, s, descs, dyn, v0b_items, v0part, 1e-9f, mlp,
                       mlp + 240, fac0, fac1, term0, term1, bscale);
  PYLO_MARK();
  if (n_el > 0) hipLaunchKernelGGL(k_celo2_stats, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac0, fac1, gl, dec, stats);
  PYLO_MARK();
  if (n_fac > 0) hipLaunchKernelGGL(k_celo2_fold, dim3(n_fac), dim3(kFoldThreads), 0, s, descs, dyn, fac_list, stats, mlp, wfold, chan_ms);
  PYLO_MARK();
  if (n_el > 0)
    hipLaunchKernelGGL(k_celo2_apply, dim3(n_el), dim3(kThreads), 0, s, descs, dyn, el_items, fac0, fac1, term0, term1,
                       gl, dec, wfold);
  PYLO_MARK();
#undef PYLO_MARK
  if (timed) P->t_steps++;
  HIP_TRY(hipGetLastError());
  return 0;
}
