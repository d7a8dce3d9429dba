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
constexpr int kNStat = 18;      // feature channels that vary per element (the other 12 are
                                // functions of the row or of the column only)
constexpr int kTabW = 12;       // floats per row/column table entry: 3 factors, pad, 8 MLP terms
constexpr int kV0Threads = 1024;
constexpr int kNV0Sums = 15;

// Per-element channels, as indices into the reference's 30-channel order
// (pylo/csrc/celo2_kernel.cu:86-124): g, clip(g), p, m0..2, rms, m_k*rs, rs, g*rf_k*cf_k, g*rs,
// [15..26 depend on the row or column only], m_k*rf_k*cf_k.
__host__ __device__ constexpr int stat_channel(int c) { return c < 15 ? c : c + 12; }

// Folded per-tensor MLP weights for CELO2 (floats): w1[18][8] | w_h[8][8] | b_h[8] | w_out[8][2] | b_out[2]
constexpr int kC2W1 = 0, kC2WH = 144, kC2BH = 208, kC2WO = 216, kC2BO = 232, kC2Fold = 240;

// ---- plan tables (device copies live in the caller's workspace) -----------------------------
enum : int { kModeFlat = 0, kModeFac2D = 1 };

struct TDesc {
  long long n;
  int mode;        // kModeFlat: no factored statistics (CELO2 AdamW tensors); kModeFac2D: 2-D factored
  int vec;         // 4: 128-bit loads (row length % 4 == 0); 1: dword loads
  int R0, C0;      // sizes of dim 0 / dim 1
  int r_is_dim0;   // fac_r / row_factor are indexed by the dim-0 coordinate (largest dim is dim 1)
  int len_r, len_c;
  int n_strips, n_colblk;
  long long rowpart_off, colpart_off;  // floats
  long long rtab_off, ctab_off;        // table entries
  int blk0, nblk;  // range of element-chunk blocks (rows of the statistics partials)
  int fac_slot;    // index among factored tensors
  int pad_;
};

struct Item {
  int tensor;
  int a;  // P0: strip (or flat chunk); element kernels: chunk
  int b;  // P0: column block
  int pad_;
};

struct Globals {
  float gnorm;  // ||all grads||_2
  int flag;     // some |g| exceeded clip_val on a tensor whose sums were taken un-clamped
};

// ---- device helpers ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// torch.clamp semantics (NaN propagates); c <= 0 disables the clamp.
__device__ __forceinline__ float clampf(float x, float c) {
  return (c > 0.0f) ? (x < -c ? -c : (x > c ? c : x)) : x;
}

// clip_norm / max(norm, clip_norm); 1 when clipping is off (ELO_CELO2_naive.py:126-135).
__device__ __forceinline__ float clip_scale(float gnorm, float clip_norm) {
  if (!(clip_norm > 0.0f)) return 1.0f;
  float denom = fmaxf(gnorm, clip_norm);
  return denom > 0.0f ? clip_norm / denom : 1.0f;
}

template <int V>
struct VecT;
template <>
struct VecT<4> {
  using type = float4;
};
template <>
struct VecT<1> {
  using type = float;
};

template <int V>
__device__ __forceinline__ void load_vec(const float* __restrict__ p, float (&x)[V]) {
  if constexpr (V == 4) {
    float4 t = *reinterpret_cast<const float4*>(p);
    x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
  } else {
    x[0] = *p;
  }
}

template <int V>
__device__ __forceinline__ void store_vec(float* __restrict__ p, const float (&x)[V]) {
  if constexpr (V == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
  } else {
    *p = x[0];
  }
}

}  // namespace pylo
