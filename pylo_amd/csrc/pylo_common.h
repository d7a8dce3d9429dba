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
constexpr int kV0aEnt = 64;     // vector entries per k_v0a block
constexpr int kV0bEnt = 1024;   // vector entries per k_v0b block
constexpr int kNV0 = 9;         // partial sums per k_v0a block
constexpr int kFoldThreads = 1024;

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
  int C0r;         // C0 rounded up to a multiple of 4 (row pitch of the dim-1 tables)
  int r_is_dim0;   // fac_r / row_factor are indexed by the dim-0 coordinate (largest dim is dim 1)
  int len_r, len_c;
  int n_strips, n_colblk;
  int blk0, nblk;  // range of element-chunk blocks (rows of the statistics partials)
  int fac_slot;    // index among factored tensors
  long long rowpart_off, colpart_off;  // floats
  long long fac0_off, fac1_off;        // floats: dim-0 factors [R0][4], dim-1 factors [3][C0r]
  long long term0_off, term1_off;      // floats: dim-0 terms [R0][H], dim-1 terms [H][C0r]
  int v0a_first[2], v0a_n[2];          // k_v0a blocks of the dim-0 / dim-1 vector
};

struct Item {
  int tensor;
  int a;  // P0: strip (or flat chunk); element kernels: chunk; V0: chunk
  int b;  // P0: column block; V0: 0 = dim-0 vector, 1 = dim-1 vector
  int pad_;
};

struct Globals {
  float gnorm;  // ||all grads||_2
  int flag;     // some |g| exceeded clip_val on a tensor whose sums were taken un-clamped
};

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

// 1/sqrt(x) for x in the normal range (callers add an epsilon >= 1e-9 first): v_rsq_f32, 1 ulp.
__device__ __forceinline__ float rsq(float x) { return __builtin_amdgcn_rsqf(x); }

// Tensor pointers come out of a table in memory, so the compiler cannot infer their address
// space; these casts say "global" and turn flat_load/flat_store into global_load/global_store.
typedef __attribute__((address_space(1))) float gfloat;
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) v4f gv4f;

template <int V>
__device__ __forceinline__ void load_vec(const float* p, float (&x)[V]) {
  if constexpr (V == 4) {
    const v4f t = *(const gv4f*)(p);
    x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
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
  } else {
    *(gfloat*)(p) = x[0];
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

// Makes the compiler forget what it knows about a (wave-uniform) pointer, so loads through it
// are re-issued where they are written instead of being hoisted out of the enclosing loop; the
// result points to memory that is read-only for the life of the kernel (scalar loads).
typedef __attribute__((address_space(4))) float cfloat;
__device__ __forceinline__ const cfloat* launder(const float* p) {
  asm volatile("" : "+s"(p));
  return (const cfloat*)p;
}

}  // namespace pylo
