// ELO-CELO2, tensors with more than two dims: Newton-Schulz, normaliser and parameter update per slice of the
// last two dims, one launch for all such tensors.
//
// The reference orthogonalises and normalises such a tensor slice by slice (orthogonalize_via_newton_schulz
// works "over the last two dims", pylo/optim/CELO2_naive.py:59-73; the normaliser's axes are the last two,
// pylo/optim/ELO_CELO2_naive.py:231-235): a convolution kernel (O, I, kh, kw) is O * I matrices of kh x kw.
// These slices are small and many, the opposite of the matrices that the tiled matrix-pipe products serve,
// so a slice is held in LDS by the lanes that own it from the raw step to the parameter update:
//     X = raw / (||raw||_F + eps)                                  (tall slices transposed, as the reference does)
//     ns_iters times:  A = X X^T;  B' = c2 A A + c1 A + c0 I;  X <- B' X      (fp32 FMA, sums in index order)
//     param <- param - lr * (X * rsqrt(1e-9 + mean(X^2)) * step_mult + weight_decay * param)
// A slice is owned by one lane (small slices: 3 x 3, 5 x 5, 7 x 7 convolution kernels; a wave holds 64 of them,
// element f of every slice in one LDS row, so the loops over i, j, k are the wave's own and every access is
// conflict-free), by one wave, or by the whole block, whichever is the smallest whose LDS share holds X twice
// and two m x m matrices; lanes of one wave need no barrier between the phases, only the ordering of their own
// LDS accesses.  HBM traffic is the raw step once and the parameter once each way; nothing is written back
// to the raw step.
#pragma once
#include "k_cast.h"
#include "pylo_common.h"

namespace pylo {

struct SliceMat {
  int tensor;          // index into the argument table
  int R, C;            // a slice is R x C, row-major, contiguous
  int m, n;            // min and max of the two
  int tall;            // R > C: X is the slice transposed
  int lanes;           // lanes per slice: 1, 64 or 256
  int ldx, lda;        // wave / block: row pitches in LDS (odd, against bank conflicts)
  int per_floats;      // wave / block: LDS floats of one slice, 2 ldx m + 2 lda m + lanes
  int no_orth;         // the shape carries PYLO_F_NO_ORTHOGONALIZE
  long long slices;
};

constexpr int kSliceLdsWave = 64 * 1024;     // LDS of a block whose slices are owned by lanes or by waves
constexpr int kSliceLdsBlock = 128 * 1024;   // ... by the whole block (needs the function attribute)
constexpr int kSlicePitch = 65;              // lane-owned slices: floats between two elements of one slice
constexpr int kSliceLaneSets = 7;            // launches of lane-owned slices: four register sizes, three LDS sizes

// Square slices of these sizes are kept in registers (k_celo2_slice_finish_lane<M>).
inline bool slice_in_registers(int m, int n) { return m == n && (m == 1 || m == 3 || m == 5 || m == 7); }

// LDS bytes of a wave of lane-owned slices: X, X', A, B' element by element, and one scale per slice (X alone
// when the slices are worked on in registers).
inline long long slice_lane_lds(int m, int n) {
  return ((slice_in_registers(m, n) ? 1ll * m * n : 2ll * m * n + 2ll * m * m) * kSlicePitch + 64) * 4;
}

// Lanes per slice and LDS pitches; false when a slice does not fit.
inline bool slice_geometry(SliceMat& s) {
  s.m = s.R < s.C ? s.R : s.C;
  s.n = s.R < s.C ? s.C : s.R;
  s.tall = s.R > s.C;
  s.ldx = s.n | 1;
  s.lda = s.m | 1;
  const long long base = 2ll * s.ldx * s.m + 2ll * s.lda * s.m;
  if (slice_lane_lds(s.m, s.n) <= kSliceLdsWave) s.lanes = 1;
  else if ((base + 64) * 4 * 4 <= kSliceLdsWave) s.lanes = 64;
  else if ((base + 256) * 4 <= kSliceLdsBlock) s.lanes = 256;
  else return false;
  s.per_floats = (int)base + s.lanes;
  return true;
}

// Newton-Schulz on one M x M slice held in a lane's registers (the common convolution kernels: every loop unrolled,
// A and B' symmetric so only their upper halves are computed).
template <int M>
__device__ __forceinline__ void slice_lane_iterate(float (&x)[M * M], int ns_iters, float c0, float c1, float c2) {
  for (int t = 0; t < ns_iters; ++t) {
    float A[M * M], B[M * M], y[M * M];
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
      for (int j = i; j < M; ++j) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < M; ++k) s = fmaf(x[i * M + k], x[j * M + k], s);
        A[i * M + j] = A[j * M + i] = s;
      }
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
      for (int j = i; j < M; ++j) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < M; ++k) s = fmaf(A[i * M + k], A[k * M + j], s);
        B[i * M + j] = B[j * M + i] = fmaf(c2, s, c1 * A[i * M + j]) + (i == j ? c0 : 0.0f);
      }
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
      for (int k = 0; k < M; ++k) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < M; ++j) s = fmaf(B[i * M + j], x[j * M + k], s);
        y[i * M + k] = s;
      }
#pragma unroll
    for (int f = 0; f < M * M; ++f) x[f] = y[f];
  }
}

// One lane per slice; items[b] = {slice table row, b}: block b (one wave) takes slices 64 b .. 64 b + 63.
// M > 0: the slices are M x M and live in registers between the load and the store (LDS only turns the wave's
// contiguous elements into one slice per lane and back); M == 0: any m x n, the slice stays in LDS.
template <int M>
__global__ __launch_bounds__(64) void k_celo2_slice_finish_lane(const SliceMat* __restrict__ mats,
                                                                const Item* __restrict__ items,
                                                                const TDesc* __restrict__ descs,
                                                                const PyloTensorArgs* __restrict__ dyn, int orth_call,
                                                                int ns_iters, float ns_eps, float c0, float c1, float c2) {
  extern __shared__ float slice_lds[];
  constexpr int S = kSlicePitch;
  const Item it = items[blockIdx.x];
  const SliceMat mt = mats[it.tensor];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr) return;
  const int store = descs[mt.tensor].store;
  const int lane = threadIdx.x;
  const int m = M > 0 ? M : mt.m, n = M > 0 ? M : mt.n, C = M > 0 ? M : mt.C, mn = m * n, mm = m * m;
  const bool tall = M > 0 ? false : mt.tall != 0;
  const long long s0 = (long long)it.a * 64;
  const long long left = mt.slices - s0;
  const int live = left < 64 ? (int)left : 64;
  const int total = live * mn;             // the wave's slices are contiguous in memory
  const long long e0 = s0 * mn;
  float* X = slice_lds;
  float* Y = X + mn * S;
  float* A = M > 0 ? X : Y + mn * S;
  float* B = A + mm * S;
  float* scl = M > 0 ? X + mn * S : B + mm * S;
  const bool orth = orth_call && (a.flags & PYLO_ARG_ORTHOGONALIZE);
  // memory order in; element (i, k) of slice s at X[(i n + k) S + s]
  for (int idx = lane; idx < total; idx += 64) {
    const int sl = idx / mn, e = idx - sl * mn, r = e / C, c = e - r * C;
    X[(tall ? c * n + r : r * n + c) * S + sl] = *(const gfloat*)(a.step_out + e0 + idx);
  }
  __syncthreads();
  bool in_y = false;
  if (lane < live) {
    float* x = X + lane;
    if constexpr (M > 0) {
      float v[M * M];
#pragma unroll
      for (int f = 0; f < M * M; ++f) v[f] = x[f * S];
      if (orth) {
        float ss = 0.0f;
#pragma unroll
        for (int f = 0; f < M * M; ++f) ss = fmaf(v[f], v[f], ss);
        const float sc = 1.0f / (sqrtf(ss) + ns_eps);
#pragma unroll
        for (int f = 0; f < M * M; ++f) v[f] *= sc;
        slice_lane_iterate<M>(v, ns_iters, c0, c1, c2);
      }
      float ss = 0.0f;
#pragma unroll
      for (int f = 0; f < M * M; ++f) ss = fmaf(v[f], v[f], ss);
#pragma unroll
      for (int f = 0; f < M * M; ++f) x[f * S] = v[f];
      scl[lane] = rsq(1e-9f + ss / (float)mn);
    } else {
      float* y = Y + lane;
      float* pa = A + lane;
      float* pb = B + lane;
      if (orth) {
        float ss = 0.0f;
        for (int f = 0; f < mn; ++f) ss = fmaf(x[f * S], x[f * S], ss);
        const float sc = 1.0f / (sqrtf(ss) + ns_eps);
        for (int f = 0; f < mn; ++f) x[f * S] *= sc;
        for (int t = 0; t < ns_iters; ++t) {
          for (int i = 0; i < m; ++i)                 // A = X X^T, symmetric
            for (int j = i; j < m; ++j) {
              float s = 0.0f;
              for (int k = 0; k < n; ++k) s = fmaf(x[(i * n + k) * S], x[(j * n + k) * S], s);
              pa[(i * m + j) * S] = s;
              pa[(j * m + i) * S] = s;
            }
          for (int i = 0; i < m; ++i)                 // B' = c2 A A + c1 A + c0 I, symmetric
            for (int j = i; j < m; ++j) {
              float s = 0.0f;
              for (int k = 0; k < m; ++k) s = fmaf(pa[(i * m + k) * S], pa[(k * m + j) * S], s);
              s = fmaf(c2, s, c1 * pa[(i * m + j) * S]) + (i == j ? c0 : 0.0f);
              pb[(i * m + j) * S] = s;
              pb[(j * m + i) * S] = s;
            }
          for (int i = 0; i < m; ++i)                 // X' = B' X
            for (int k = 0; k < n; ++k) {
              float s = 0.0f;
              for (int j = 0; j < m; ++j) s = fmaf(pb[(i * m + j) * S], x[(j * n + k) * S], s);
              y[(i * n + k) * S] = s;
            }
          float* t2 = x; x = y; y = t2;
        }
      }
      float ss = 0.0f;
      for (int f = 0; f < mn; ++f) ss = fmaf(x[f * S], x[f * S], ss);
      scl[lane] = rsq(1e-9f + ss / (float)mn);
    }
  }
  if (M == 0) in_y = orth && (ns_iters & 1);
  __syncthreads();
  const float* xf = in_y ? Y : X;
  const float rm = a.step_mult, wd = a.weight_decay, nlr = -a.lr;
  for (int idx = lane; idx < total; idx += 64) {
    const int sl = idx / mn, e = idx - sl * mn, r = e / C, c = e - r * C;
    const float v = xf[(tall ? c * n + r : r * n + c) * S + sl] * scl[sl];
    if (store != 0) {
      const float q = load_stored(a.param, e0 + idx, store);
      store_stored(a.param, e0 + idx, store, fmaf(nlr, v * rm + wd * q, q));
    } else {
      gfloat* p = (gfloat*)(a.param + e0 + idx);
      const float q = *p;
      *p = fmaf(nlr, v * rm + wd * q, q);
    }
  }
}

template <bool BLOCK>
__device__ __forceinline__ void slice_sync() {
  if (BLOCK) __syncthreads();
  else __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // LDS accesses of one wave complete in order
}

// out(i, j) = sum over k < len of P[i pi + k pk] Q[j qj + k qk] for the `count` outputs e = i * cols + j, dealt to
// the lanes of a slice four at a time (four independent sums in flight per lane).
template <typename F>
__device__ __forceinline__ void slice_products(const float* P, int pi, int pk, const float* Q, int qj, int qk, int len,
                                               int cols, int count, int gl, int lanes, F&& out) {
  for (int e0 = gl; e0 < count; e0 += 4 * lanes) {
    const float* p[4];
    const float* q[4];
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = e0 + u * lanes < count ? e0 + u * lanes : count - 1;   // past the end: a repeat, not stored
      const int i = e / cols, j = e - i * cols;
      p[u] = P + i * pi;
      q[u] = Q + j * qj;
    }
    for (int k = 0; k < len; ++k) {
#pragma unroll
      for (int u = 0; u < 4; ++u) s[u] = fmaf(p[u][k * pk], q[u][k * qk], s[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = e0 + u * lanes;
      if (e < count) out(e / cols, e - (e / cols) * cols, s[u]);
    }
  }
}

// Sum over the lanes of a slice, the same value on every lane, added in lane order.
template <bool BLOCK>
__device__ __forceinline__ float slice_sum(float* red, int lanes, int gl, float v) {
  slice_sync<BLOCK>();   // the last reads of `red`
  red[gl] = v;
  slice_sync<BLOCK>();
  float s = 0.0f;
  for (int j = 0; j < lanes; j += 4) s += (red[j] + red[j + 1]) + (red[j + 2] + red[j + 3]);
  return s;
}

// One wave or the whole block per slice; items[b] = {slice table row, first group of slices}: a block takes
// 256 / lanes consecutive slices.
// `orth_call`: the call is the one that orthogonalises (flags are honoured); ns_iters may be 0 (division by
// the norm only, as the reference does).
template <bool BLOCK>
__global__ __launch_bounds__(256) void k_celo2_slice_finish(const SliceMat* __restrict__ mats,
                                                            const Item* __restrict__ items,
                                                            const TDesc* __restrict__ descs,
                                                            const PyloTensorArgs* __restrict__ dyn, int orth_call,
                                                            int ns_iters, float ns_eps, float c0, float c1, float c2) {
  extern __shared__ float slice_lds[];
  const Item it = items[blockIdx.x];
  const SliceMat mt = mats[it.tensor];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr) return;
  const int store = descs[mt.tensor].store;
  const int lanes = BLOCK ? 256 : 64;
  const int gl = threadIdx.x % lanes, grp = threadIdx.x / lanes;
  const long long sl = (long long)it.a * (256 / lanes) + grp;
  if (!BLOCK && sl >= mt.slices) return;   // whole groups of lanes; no block-wide barrier on this path
  const int m = mt.m, n = mt.n, C = mt.C, ldx = mt.ldx, lda = mt.lda, mn = m * n, mm = m * m;
  const bool tall = mt.tall != 0;
  float* X = slice_lds + (size_t)grp * mt.per_floats;
  float* Y = X + ldx * m;
  float* A = Y + ldx * m;
  float* B = A + lda * m;
  float* red = B + lda * m;
  const long long e0 = sl * mn;
  const float* raw = a.step_out + e0;
  const bool orth = orth_call && (a.flags & PYLO_ARG_ORTHOGONALIZE);

  // the raw slice, memory order in, (m x n) in LDS
  float ss = 0.0f;
  for (int e = gl; e < mn; e += lanes) {
    const float v = *(const gfloat*)(raw + e);
    const int r = e / C, c = e - r * C;
    X[tall ? c * ldx + r : r * ldx + c] = v;
    ss = fmaf(v, v, ss);
  }
  if (orth) {
    const float sc = 1.0f / (sqrtf(slice_sum<BLOCK>(red, lanes, gl, ss)) + ns_eps);
    for (int e = gl; e < mn; e += lanes) {   // a lane scales what it wrote
      const int r = e / C, c = e - r * C;
      X[tall ? c * ldx + r : r * ldx + c] *= sc;
    }
    for (int t = 0; t < ns_iters; ++t) {
      slice_sync<BLOCK>();
      slice_products(X, ldx, 1, X, ldx, 1, n, m, mm, gl, lanes, [&](int i, int j, float s) { A[i * lda + j] = s; });   // A = X X^T
      slice_sync<BLOCK>();
      slice_products(A, lda, 1, A, 1, lda, m, m, mm, gl, lanes, [&](int i, int j, float s) {                            // B' = c2 A A + c1 A + c0 I
        B[i * lda + j] = fmaf(c2, s, c1 * A[i * lda + j]) + (i == j ? c0 : 0.0f);
      });
      slice_sync<BLOCK>();
      slice_products(B, lda, 1, X, 1, ldx, m, n, mn, gl, lanes, [&](int i, int k, float s) { Y[i * ldx + k] = s; });   // X' = B' X
      float* t2 = X; X = Y; Y = t2;
    }
    slice_sync<BLOCK>();
    ss = 0.0f;
    for (int e = gl; e < mn; e += lanes) {
      const int r = e / C, c = e - r * C;
      const float v = X[tall ? c * ldx + r : r * ldx + c];
      ss = fmaf(v, v, ss);
    }
  }
  const float ms = slice_sum<BLOCK>(red, lanes, gl, ss) / (float)mn;
  const float sc = rsq(1e-9f + ms), rm = a.step_mult, wd = a.weight_decay, nlr = -a.lr;
  for (int e = gl; e < mn; e += lanes) {
    const int r = e / C, c = e - r * C;
    const float v = X[tall ? c * ldx + r : r * ldx + c];
    if (store != 0) {
      const float q = load_stored(a.param, e0 + e, store);
      store_stored(a.param, e0 + e, store, fmaf(nlr, (v * sc) * rm + wd * q, q));
    } else {
      gfloat* p = (gfloat*)(a.param + e0 + e);
      const float q = *p;
      *p = fmaf(nlr, (v * sc) * rm + wd * q, q);
    }
  }
}

}  // namespace pylo
