// Shared host/device definitions of the fused learned-optimizer step (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "pylo_mi355.h"

namespace pylo {

// ---- launch geometry ---------------------------------------------------------------------
constexpr int kThreads = 256;   // 4 waves of 64 lanes
constexpr int kWaves = 4;
constexpr int kP0Rows = 128;    // rows of one row/column-sum tile; tile columns = 64 * vec
constexpr int kElemIters = 8;   // an element chunk is kThreads * vec * kElemIters elements
constexpr int kTileV = 2;       // column-resident walk: a wave owns 64 * kTileV columns ...
constexpr int kTileCols = 64 * kTileV;
constexpr int kTileRows = 16;   // ... and walks this many rows of them (TDesc::tile_rows; ELO-CELO2 plans may choose fewer)
constexpr int kNStat = 18;      // feature channels that vary per element (the other 12 are
                                // functions of the row or of the column only)
constexpr int kV0aEnt = 64;     // vector entries per k_v0a block
constexpr int kV0bEnt = 1024;   // vector entries per k_v0b block
constexpr int kNV0 = 9;         // partial sums per k_v0a block
constexpr int kV0aThreads = 256;   // groups of 64 lanes share the partial rows of 64 entries
constexpr int kFoldThreads = 1024;
constexpr int kRcmSlots = 1024; // slices of an N-D row vector whose row_col_mean one k_v0b block tabulates
constexpr int kNdX = 64;        // elements of the summed dim one k_p0_nd block covers (one partial row)

// Per-element channels, as indices into the reference's 30-channel order
// (pylo/csrc/celo2_kernel.cu:86-124): g, clip(g), p, m0..2, rms, m_k*rs, rs, g*rf_k*cf_k, g*rs,
// [15..26 depend on the row or column only], m_k*rf_k*cf_k.
__host__ __device__ constexpr int stat_channel(int c) { return c < 15 ? c : c + 12; }

// Folded per-tensor MLP weights for CELO2 (floats): w1[18][8] | w_h[8][8] | b_h[8] | w_out[8][2] | b_out[2]
// folded per-tensor weights: W1 (18,8) | WH (8,8) | bH 8 | WO (8,4: two outputs, two zeros) | bO 4 (same padding)
constexpr int kC2W1 = 0, kC2WH = 144, kC2BH = 208, kC2WO = 216, kC2BO = 248, kC2Fold = 256;

// ---- plan tables (device copies live in the caller's workspace) -----------------------------
// kModeFlat   no factored statistics, no MLP: CELO2 tensors routed to AdamW
// kModeFac2D  2-D factored tensor, tiled fast path
// kModeFacND  >2-D factored tensor (any two dims), generic indexing, dword accesses
// kModeVec    VeLO / AdafacLO tensor with fewer than 2 dims: per-element accumulator fac_v
enum : int { kModeFlat = 0, kModeFac2D = 1, kModeFacND = 2, kModeVec = 3 };

// A factored tensor owns two statistics vectors.  2-D: vector 0 is indexed by the dim-0
// coordinate (sums over dim 1), vector 1 by the dim-1 coordinate.  N-D: vector 0 is the tensor
// with the largest dim removed (the reference's fac_vec_row), vector 1 with the 2nd-largest removed.
// Division of an element index (< 2^31) by a divisor fixed for the launch or the plan: q = (n * m) >> (31 + s) with
// s = ceil(log2 d), m = floor(2^(31+s) / d) + 1 < 2^32, exact for every n < 2^31 (the error of m is at
// most d / 2^(31+s) per unit of n).  s < 0 marks d == 1.  Four of these per element replace four integer
// divisions of some twenty instructions each.
struct FastDiv {
  unsigned m;
  int s;
  unsigned d;
};
__host__ inline FastDiv make_fastdiv(unsigned d) {
  FastDiv f{0u, -1, d};
  if (d <= 1) return f;
  int s = 0;
  while ((1ull << s) < d) ++s;
  f.s = s;
  f.m = (unsigned)((1ull << (31 + s)) / d + 1);
  return f;
}
__device__ __forceinline__ unsigned fd_div(unsigned n, const FastDiv& f) {
  return f.s < 0 ? n : (__umulhi(n, f.m) >> (f.s - 1));
}

struct TDesc {
  long long n;
  int mode;
  int vec;          // 4: 128-bit accesses (2-D with C0 % 4 == 0, flat/vec with n % 4 == 0); 1: dword
  int R0, C0;       // 2-D: sizes of dim 0 / dim 1
  int vec0_is_r;    // vector 0 carries fac_r / row_factor (else fac_c / col_factor)
  int len[2];       // entries of vector 0 / 1
  int sumlen[2];    // elements summed into one entry
  int npart[2];     // partial rows to add up per entry (2-D: column blocks / strips; N-D: 1)
  int pitch[2];     // len rounded up to 4
  int nd_size[2];   // N-D: size and stride of the dim removed from vector 0 / 1;
  int nd_stride[2]; //      entry = (idx / (size*stride)) * stride + idx % stride
  FastDiv nd_div_blk[2], nd_div_st[2];  // the two divisors of that formula per vector, as multiply-and-shift
  int rcm_size;     // N-D: size of the 2nd-largest dim and its stride inside the row vector; row_col_mean
  int rcm_stride;   //      is the mean over that axis, one value per slice (2-D: one value per tensor)
  int n_strips, n_colblk;
  int blk0, nblk;   // range of element-chunk blocks (rows of the statistics partials)
  int seg0, nseg;   // tensors with many rows: their rows are first summed in segments of kSegRows (k_stat_segsum)
  int fac_slot;     // index among factored tensors, -1 otherwise
  int rank;         // number of dims larger than 1 (VeLO's rank one-hot feature)
  long long part_off[2];  // floats, partial sums of g^2
  long long fac_off[2];   // floats, factor tables [entry][4] (three decays + padding: one 16-byte access per entry)
  long long term_off[2];  // floats, first-layer terms [entry][H]
  int v0a_first[2], v0a_n[2];  // k_v0a blocks of vector 0 / 1
  // Column-resident walk (wide 2-D tensors, C0 % kTileCols == 0): wave task w covers columns
  // [ (w % tile_nct) * kTileCols, +kTileCols ) of rows [ (w / tile_nct) * tile_rows, +tile_rows );
  // element block a holds tasks 4a .. 4a+3.  tile_nct == 0: linear chunks instead.
  int tile_nct, tile_ntask, tile_rows;
  // AdafacLO's apply pass walks one column per lane (its 32-wide MLP leaves no registers for two):
  // same scheme with 64 columns per wave task; apply block a holds tasks 4a .. 4a+3.
  int atile_nct, atile_ntask;
  // ... and an (O, I, k, ..) tensor whose factored dims are the two leading ones is walked the same way as the
  // matrix (O, I * P), P = product of the trailing dims: one vector is indexed by the matrix column, the other by
  // (row, column mod P).  aper = P (0: not walked so), aper_col = which vector the column indexes; R0 / C0 hold
  // the matrix view.
  int aper, aper_col;
  int adam_indep;          // kModeFlat: AdamW on the tensor's own two moments instead of mom[0] / rms
  int fin_unit0, fin_units;  // ELO-CELO2 finishing pass: the tensor's units (FinUnit)
  int slice_len;           // CELO2, N-D or fewer than two dims: elements per slice of the last two dims (or n)
  int nan0;                // gradients pass through torch.nan_to_num (PYLO_F_NAN_TO_NUM)
  int wd_prestep;          // p -= lr * (step + wd * p) against the pre-step parameter (PYLO_F_WD_PRESTEP)
  int store;               // storage type of the caller's grad / param buffers (kStore*, k_cast.h); 0 = fp32
  int own_norm;            // clip_norm bounds the tensor's own gradient norm (PYLO_F_TENSOR_NORM), not the call's
  int p0_first, p0_n;      // the tensor's blocks of the first statistics launch (rows of its sum-of-squares partials)
  float gscale;            // 1 in the plan; AdafacLO-family kernels overwrite their copy with the clip scale
};

// Field of vector 0 or 1 chosen at run time.  Indexing the by-value descriptor with a run-time
// index would force the whole struct into scratch memory; a select keeps it in registers.
template <class T>
__device__ __forceinline__ T pick(const T (&a)[2], int w) { return w ? a[1] : a[0]; }

// ELO-CELO2 finishing pass: what one normaliser runs over -- a whole tensor, or one slice of the last two dims of a
// tensor with more dims.
struct FinUnit {
  int tensor;
  int blk0, nblk;   // range of 8192-element blocks (rows of the pass's partial sums)
  int vec;          // 16-byte accesses: off and n multiples of 4
  long long off;    // elements from the tensor's start
  long long n;
};

struct Item {
  int tensor;
  int a;  // P0: strip (or flat chunk); element kernels: chunk; V0 / N-D sums: chunk of entries
  int b;  // P0: column block; V0 / N-D sums: vector 0 or 1
  int c;  // N-D sums: chunk of the summed dim (= partial row)
};

// Width of one row of statistics partials (doubles): sum of squares per feature channel in the
// reference's 30-channel order, then the per-tensor LSTM input sums of VeLO taken over the
// accumulators *before* the update: sum m_k (30..32), sum m_k^2 (33..35), sum rms (36), sum rms^2 (37).
constexpr int kStatW = 40;
constexpr int kSegRows = 256;   // rows of statistics partials one k_stat_segsum block adds up
constexpr int kSegMin = 1024;   // tensors with more rows than this are reduced in two stages

// Where a per-tensor reduction finds the tensor's rows: its segment sums if it has any, else its partials.
__device__ __forceinline__ const double* stat_rows(const TDesc& d, const double* stats_part, const double* seg_tot,
                                                   int& n_rows) {
  if (d.nseg > 0) { n_rows = d.nseg; return seg_tot + (size_t)d.seg0 * kStatW; }
  n_rows = d.nblk;
  return stats_part + (size_t)d.blk0 * kStatW;
}

constexpr int kSumM = 30, kSumMM = 33, kSumR = 36, kSumRR = 37;

struct Globals {
  float gnorm;  // ||all grads||_2
  int flag;     // some |g| exceeded clip_val on a tensor whose sums were taken un-clamped
  const float* tscale;  // plans with per-tensor norm clipping: the clip factor of every tensor (k_tnorm)
};

// Item::c of the fused element pass of ELO-CELO2 (k_celo2_elem)
constexpr int kElemApply = 1;   // apply item (else statistics item); Item::b is the row of the statistics partials
constexpr int kElemKeep = 2;    // statistics item whose inputs the apply pass re-reads from the memory-side cache
constexpr int kSpinLimit = 2000000;   // polls of a tensor's "folded weights ready" flag before a block gives up

// Per factored tensor, written by k_v0b: normalisation scales of the 12 broadcast channels in the
// reference's channel order 15..26 (fac_r_k, fac_c_k, rsqrt(fac_r_k+1e-8), rsqrt(fac_c_k+1e-8)).
struct BScale {
  float s[12];
  float rcm[3];
  float pad_;
};

// ---- device helpers ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum over the wave without the LDS crossbar (six DPP adds); the total is valid in lane 63 only.
__device__ __forceinline__ float wave_sum_to_last(float v) {
  auto dpp = [](float x, int ctrl, int row_mask) {
    int r;
    switch (ctrl) {  // the control word must be an immediate
      case 0xB1: r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false); break;   // quad_perm [1,0,3,2]
      case 0x4E: r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false); break;   // quad_perm [2,3,0,1]
      case 0x141: r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false); break; // row_half_mirror
      case 0x140: r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false); break; // row_mirror
      case 0x142: r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xA, 0xF, false); break; // row_bcast:15 into rows 1, 3
      default: r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x143, 0xC, 0xF, false); break;    // row_bcast:31 into rows 2, 3
    }
    (void)row_mask;
    return __builtin_bit_cast(float, r);
  };
  v += dpp(v, 0xB1, 0xF);
  v += dpp(v, 0x4E, 0xF);
  v += dpp(v, 0x141, 0xF);
  v += dpp(v, 0x140, 0xF);
  v += dpp(v, 0x142, 0xA);
  v += dpp(v, 0x143, 0xC);
  return v;
}

// DPP moves with the control word as a template argument (it must be an immediate).
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}

// Four values per lane (one per row u) -> per 16-lane group, lane 4q + u holds the sum of row u over
// the group's 16 lanes (q = 0..3 all hold it).  Fourteen VALU instructions instead of four full
// wave reductions; lane-pair exchanges first, so every lane ends up owning one row.
__device__ __forceinline__ float reduce4_rows16(float a0, float a1, float a2, float a3) {
  const int lane = threadIdx.x & 63;
  const bool b0 = lane & 1, b1 = lane & 2;
  const float k01 = b0 ? a1 : a0, s01 = b0 ? a0 : a1;
  const float k23 = b0 ? a3 : a2, s23 = b0 ? a2 : a3;
  const float p01 = k01 + dpp_mov<0xB1>(s01);  // quad_perm [1,0,3,2]
  const float p23 = k23 + dpp_mov<0xB1>(s23);
  const float k = b1 ? p23 : p01, s = b1 ? p01 : p23;
  float v = k + dpp_mov<0x4E>(s);              // quad_perm [2,3,0,1]: lane%4 = u holds row u of its quad
  v += dpp_mov<0x124>(v);                      // row_ror:4
  v += dpp_mov<0x128>(v);                      // row_ror:8
  return v;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// torch.clamp semantics (NaN propagates); c <= 0 disables the clamp.  Branch-free: the bound is a
// wave-uniform select that the compiler hoists out of element loops.
__device__ __forceinline__ float clampf(float x, float c) {
  const float hi = c > 0.0f ? c : __builtin_inff();
  return x < -hi ? -hi : (x > hi ? hi : x);
}

// clip_norm / max(norm, clip_norm); 1 when clipping is off (ELO_CELO2_naive.py:126-135).
__device__ __forceinline__ float clip_scale(float gnorm, float clip_norm) {
  if (!(clip_norm > 0.0f)) return 1.0f;
  float denom = fmaxf(gnorm, clip_norm);
  return denom > 0.0f ? clip_norm / denom : 1.0f;
}

// Factor on tensor t's gradient from norm clipping: by the norm of all gradients of the call, or, on tensors
// flagged PYLO_F_TENSOR_NORM, by the tensor's own (k_tnorm has left the factor in gl->tscale).
__device__ __forceinline__ float grad_scale(const TDesc& d, const PyloTensorArgs& a, const Globals* gl, int t) {
  if (!(a.clip_norm > 0.0f)) return 1.0f;
  return d.own_norm ? gl->tscale[t] : clip_scale(gl->gnorm, a.clip_norm);
}

// The descriptor copy of a kernel carries the tensor's clip factor for cond_grad.
__device__ __forceinline__ void set_grad_scale(TDesc& d, const PyloTensorArgs& a, const Globals* gl, int t) {
  d.gscale = grad_scale(d, a, gl, t);
}

// The gradient as the optimizer sees it (ELO_naive.py:141-146): scaled by the global-norm clip factor,
// NaN -> 0 where the tensor asks for torch.nan_to_num (its clip_val is FLT_MAX then, which maps
// +-inf as torch does), clamped to +-clip_val.
__device__ __forceinline__ float cond_grad(float raw, float scale, float clip_val, int nan0) {
  float x = raw * scale;
  if (nan0) x = (x == x) ? x : 0.0f;
  return clampf(x, clip_val);
}

// 1/sqrt(x) for x in the normal range (callers add an epsilon >= 1e-9 first): v_rsq_f32, 1 ulp.
__device__ __forceinline__ float rsq(float x) { return __builtin_amdgcn_rsqf(x); }

// Tensor pointers come out of a table in memory, so the compiler cannot infer their address
// space; these casts say "global" and turn flat_load/flat_store into global_load/global_store.
typedef __attribute__((address_space(1))) float gfloat;
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) v4f gv4f;
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(1))) v2f gv2f;

template <int V>
__device__ __forceinline__ void load_vec(const float* p, float (&x)[V]) {
  if constexpr (V == 4) {
    const v4f t = *(const gv4f*)(p);
    x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
  } else if constexpr (V == 2) {
    const v2f t = *(const gv2f*)(p);
    x[0] = t.x; x[1] = t.y;
  } else {
    x[0] = *(const gfloat*)(p);
  }
}

template <int V>
__device__ __forceinline__ void store_vec(float* p, const float (&x)[V]) {
  if constexpr (V == 4) {
    v4f t;
    t.x = x[0]; t.y = x[1]; t.z = x[2]; t.w = x[3];
    *(gv4f*)(p) = t;
  } else if constexpr (V == 2) {
    v2f t;
    t.x = x[0]; t.y = x[1];
    *(gv2f*)(p) = t;
  } else {
    *(gfloat*)(p) = x[0];
  }
}

// The same through a wave-uniform base and a 32-bit byte offset per lane: one scalar base register
// pair plus one offset VGPR per access instead of a 64-bit address per lane.
typedef __attribute__((address_space(1))) char gchar;

template <int V>
__device__ __forceinline__ void load_vec_o(const float* sbase, unsigned byte_off, float (&x)[V]) {
  const gchar* p = (const gchar*)sbase + byte_off;
  if constexpr (V == 4) {
    const v4f t = *(const gv4f*)p;
    x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
  } else if constexpr (V == 2) {
    const v2f t = *(const gv2f*)p;
    x[0] = t.x; x[1] = t.y;
  } else {
    x[0] = *(const gfloat*)p;
  }
}

template <int V>
__device__ __forceinline__ void store_vec_o(float* sbase, unsigned byte_off, const float (&x)[V]) {
  gchar* p = (gchar*)sbase + byte_off;
  if constexpr (V == 4) {
    v4f t;
    t.x = x[0]; t.y = x[1]; t.z = x[2]; t.w = x[3];
    *(gv4f*)p = t;
  } else if constexpr (V == 2) {
    v2f t;
    t.x = x[0]; t.y = x[1];
    *(gv2f*)p = t;
  } else {
    *(gfloat*)p = x[0];
  }
}

// Streaming variants: the data is not needed again before it would be evicted anyway.
template <int V>
__device__ __forceinline__ void load_vec_nt(const float* sbase, unsigned byte_off, float (&x)[V]) {
  const gchar* p = (const gchar*)sbase + byte_off;
  if constexpr (V == 4) {
    const v4f t = __builtin_nontemporal_load((const gv4f*)p);
    x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
  } else if constexpr (V == 2) {
    const v2f t = __builtin_nontemporal_load((const gv2f*)p);
    x[0] = t.x; x[1] = t.y;
  } else {
    x[0] = __builtin_nontemporal_load((const gfloat*)p);
  }
}

template <int V>
__device__ __forceinline__ void store_vec_nt(float* sbase, unsigned byte_off, const float (&x)[V]) {
  gchar* p = (gchar*)sbase + byte_off;
  if constexpr (V == 4) {
    v4f t;
    t.x = x[0]; t.y = x[1]; t.z = x[2]; t.w = x[3];
    __builtin_nontemporal_store(t, (gv4f*)p);
  } else if constexpr (V == 2) {
    v2f t;
    t.x = x[0]; t.y = x[1];
    __builtin_nontemporal_store(t, (gv2f*)p);
  } else {
    __builtin_nontemporal_store(x[0], (gfloat*)p);
  }
}

__device__ __forceinline__ float4 load_f4(const float* p) {
  const v4f t = *(const gv4f*)(p);
  return make_float4(t.x, t.y, t.z, t.w);
}

__device__ __forceinline__ void store_f4(float* p, float a, float b, float c, float d) {
  v4f t;
  t.x = a; t.y = b; t.z = c; t.w = d;
  *(gv4f*)(p) = t;
}

// D(4x4, 16 blocks) += A(4x1) B(1x4) per block, fp32.  Lane l = 4*block + j holds B[j] (src1) and the
// column D[0..3][j] (4 VGPRs); with cbsz = 4 the four A values are taken from lanes 4*abid .. 4*abid+3
// of src0 for every block.  Used as a lane-local FMA engine: B = a value of the lane's own element,
// A = four weights, D = four hidden units of the lane's own element -- nothing crosses lanes except
// the weights.  `abid` must be a compile-time constant after unrolling.
__device__ __forceinline__ v4f mfma_w4(float wreg, float b, v4f c, int abid) {
  switch (abid & 15) {
    case 0: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 0, 0);
    case 1: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 1, 0);
    case 2: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 2, 0);
    case 3: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 3, 0);
    case 4: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 4, 0);
    case 5: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 5, 0);
    case 6: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 6, 0);
    case 7: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 7, 0);
    case 8: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 8, 0);
    case 9: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 9, 0);
    case 10: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 10, 0);
    case 11: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 11, 0);
    case 12: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 12, 0);
    case 13: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 13, 0);
    case 14: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 14, 0);
    default: return __builtin_amdgcn_mfma_f32_4x4x1f32(wreg, b, c, 4, 15, 0);
  }
}

// max(x, 0) for finite x as one median-of-three (no NaN-quieting pre-pass as fmaxf needs; written
// with a compiler builtin so the hazard recogniser sees an ordinary VALU instruction after an MFMA)
__device__ __forceinline__ float relu(float x) { return __builtin_amdgcn_fmed3f(x, 0.0f, 3.0e38f); }

// ---- values handed from one running block to another (the fused element pass of ELO-CELO2) -------
// Ordinary loads and stores go through an L2 that is private to each of the eight XCDs, so a value
// written by a block on one XCD is not seen by a block on another before the kernel ends.  Agent-scope
// atomics are performed at the memory side, which all XCDs share.  A producer writes its values with
// atomic exchanges, whose returned old values it waits for (then the writes have been performed), and
// only then announces them with a counter or flag, again an atomic; a consumer reads with atomic loads.
// No fence is used: a release fence writes back the XCD's whole L2 and costs microseconds per block.
__device__ __forceinline__ void coh_store_wait(float* p, float v) {
  const float old = __hip_atomic_exchange(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  asm volatile("" ::"v"(old) : "memory");   // the old value has arrived: the exchange has been performed
}
__device__ __forceinline__ void coh_store_wait(double* p, double v) {
  const unsigned long long old = __hip_atomic_exchange(reinterpret_cast<unsigned long long*>(p),
                                                       __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
  asm volatile("" ::"v"(old) : "memory");
}
__device__ __forceinline__ float coh_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ double coh_load(const double* p) {
  return __builtin_bit_cast(double, __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ int coh_load(const int* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Makes the compiler forget what it knows about a (wave-uniform) pointer, so loads through it
// are re-issued where they are written instead of being hoisted out of the enclosing loop; the
// result points to memory that is read-only for the life of the kernel (scalar loads).
typedef __attribute__((address_space(4))) float cfloat;
__device__ __forceinline__ const cfloat* launder(const float* p) {
  asm volatile("" : "+s"(p));
  return (const cfloat*)p;
}

// N consecutive floats at a wave-uniform address, through the scalar cache into SGPRs.  The memory
// must not be written by the running kernel.
template <int N>
__device__ __forceinline__ void load_uniform(const float* p, float (&x)[N]) {
  const cfloat* q = (const cfloat*)p;
#pragma unroll
  for (int i = 0; i < N; ++i) x[i] = q[i];
}

}  // namespace pylo
