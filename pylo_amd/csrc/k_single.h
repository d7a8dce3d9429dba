// Single-tensor kernels behind the entry points that keep the argument lists of the reference's three
// extension functions (celo2_cuda_kernel.celo2_kernel, cuda_lo.learned_optimizer_kernel,
// velo_cuda_kernel.velo_kernel_simple): the caller has already updated the accumulators and formed
// row_factor / col_factor; one launch adds the per-channel sums of squared features into
// `second_moment`, a second one normalises, runs the MLP and writes the step or the parameter.
// These are the compatibility path for per-tensor callers; the multi-tensor plans are the fast path.
#pragma once

#include "pylo_common.h"
#include "k_cast.h"

namespace pylo {

enum { kFamCelo2 = 0, kFamLo = 1, kFamVelo = 2 };

template <int F> struct Fam;
// CELO2: 30 channels, 30 -> 8 -> 8 -> 3, weights stored (in, out)          (celo2_kernel.cu:33-40,214-219)
template <> struct Fam<kFamCelo2> { static constexpr int NSTAT = 30, NIN = 30, H = 8, NOUT = 3; static constexpr bool in_major = true; };
// AdafacLO / ELO: 28 channels + 11 time features, 39 -> 32 -> 32 -> 2, (out, in)   (learned_optimizer.cu:10-13)
template <> struct Fam<kFamLo> { static constexpr int NSTAT = 28, NIN = 39, H = 32, NOUT = 2; static constexpr bool in_major = false; };
// VeLO: 30 channels, 30 -> 4 -> 4 -> 3, (out, in)                                   (velo_kernel.cu:10-13)
template <> struct Fam<kFamVelo> { static constexpr int NSTAT = 30, NIN = 30, H = 4, NOUT = 3; static constexpr bool in_major = false; };

// Every array except `second_moment` holds elements of the call's element type (float unless the typed
// entry points say otherwise; the reference instantiates its kernels for float, double and half and passes
// all of them as scalar_t, celo2_kernel.cu:314-347): the members are typed float* and read through ld<ST>.
struct SingleArgs {
  const float *g, *m, *v, *fac_r, *fac_c, *row_factor, *col_factor;
  float* p;              // read by every family; updated in place by the lo / velo families
  float* second_moment;  // NSTAT floats, accumulated into (the caller zeroes it)
  const float *w_in, *b_in, *w_h, *b_h, *w_out, *b_out;
  float* step_out;       // celo2 only
  int n, num_rows, num_cols, row_stride, col_stride, vector_like;
  int stride_r, stride_c;                        // decay strides of the row / column vectors
  FastDiv div_rblock, div_rstride, div_cblock, div_cstride;   // num_rows*row_stride, row_stride, num_cols*col_stride, col_stride
  float lr, step_mult, exp_mult, epsilon, step, weight_decay;
};

constexpr int kSingleThreads = 256;
constexpr int kSingleMaxBlocks = 2048;

// Offsets of element idx into the row vectors (row_factor, fac_r: the tensor's shape with the largest
// dim dr removed) and the column vectors (col_factor, fac_c: dim dc removed), and their decay strides.
// For tensors of up to two dims this is the reference's `col_idx + k * num_cols` / `row_idx + k * num_rows`
// (celo2_kernel.cu:67-84, learned_optimizer.cu:55-72); with more dims it is velo_kernel.cu:109-120:
//   ofs_row = (idx / (num_rows * row_stride)) * row_stride + idx % row_stride, likewise for columns.
struct FacOfs { int r, c, stride_r, stride_c; };
__device__ __forceinline__ FacOfs fac_offsets(const SingleArgs& a, int idx) {
  FacOfs o;
  if (a.vector_like) {
    o.r = o.c = idx;
    o.stride_r = o.stride_c = a.n;
  } else {
    const unsigned u = (unsigned)idx;
    o.stride_r = a.stride_r;
    o.stride_c = a.stride_c;
    o.r = (int)(fd_div(u, a.div_rblock) * (unsigned)a.row_stride + (u - fd_div(u, a.div_rstride) * (unsigned)a.row_stride));
    o.c = (int)(fd_div(u, a.div_cblock) * (unsigned)a.col_stride + (u - fd_div(u, a.div_cstride) * (unsigned)a.col_stride));
  }
  return o;
}

// Element i of an array of the call's element type ST (kStore*), widened to float as the reference's
// static_cast<float> does (celo2_kernel.cu:70-75), and the narrowing store (celo2_kernel.cu:280).
template <int ST>
__device__ __forceinline__ float ld(const float* base, size_t i) {
  if constexpr (ST == kStoreF32) return base[i];
  else return load_stored(base, (long long)i, ST);
}
template <int ST>
__device__ __forceinline__ void st(float* base, size_t i, float x) {
  if constexpr (ST == kStoreF32) base[i] = x;
  else store_stored(base, (long long)i, ST, x);
}

template <int F, int ST>
__device__ __forceinline__ void single_features(const SingleArgs& a, int idx, float (&f)[Fam<F>::NSTAT]) {
  const FacOfs o = fac_offsets(a, idx);
  const float g = ld<ST>(a.g, idx), p = ld<ST>(a.p, idx);
  const float m0 = ld<ST>(a.m, idx), m1 = ld<ST>(a.m, idx + (size_t)a.n), m2 = ld<ST>(a.m, idx + 2 * (size_t)a.n);
  const float v = ld<ST>(a.v, idx);
  const bool vl = a.vector_like != 0;
  const float rf0 = ld<ST>(a.row_factor, o.r), rf1 = ld<ST>(a.row_factor, o.r + (size_t)o.stride_r),
              rf2 = ld<ST>(a.row_factor, o.r + 2 * (size_t)o.stride_r);
  const float cf0 = vl ? 1.0f : ld<ST>(a.col_factor, o.c), cf1 = vl ? 1.0f : ld<ST>(a.col_factor, o.c + (size_t)o.stride_c),
              cf2 = vl ? 1.0f : ld<ST>(a.col_factor, o.c + 2 * (size_t)o.stride_c);
  if constexpr (F == kFamLo) {
    // learned_optimizer.cu:34-98
    const float rs = rsq(v + a.epsilon);
    f[0] = g; f[1] = p; f[2] = m0; f[3] = m1; f[4] = m2; f[5] = v;
    f[6] = m0 * rs; f[7] = m1 * rs; f[8] = m2 * rs; f[9] = rs;
    f[10] = rf0 * cf0 * g; f[11] = rf1 * cf1 * g; f[12] = rf2 * cf2 * g;
    const float r0 = ld<ST>(a.fac_r, o.r), r1 = ld<ST>(a.fac_r, o.r + (size_t)o.stride_r), r2 = ld<ST>(a.fac_r, o.r + 2 * (size_t)o.stride_r);
    const float c0 = ld<ST>(a.fac_c, o.c), c1 = ld<ST>(a.fac_c, o.c + (size_t)o.stride_c), c2 = ld<ST>(a.fac_c, o.c + 2 * (size_t)o.stride_c);
    f[13] = r0; f[14] = r1; f[15] = r2; f[16] = c0; f[17] = c1; f[18] = c2;
    f[19] = rsq(r0 + 1e-8f); f[20] = rsq(r1 + 1e-8f); f[21] = rsq(r2 + 1e-8f);
    f[22] = rsq(c0 + 1e-8f); f[23] = rsq(c1 + 1e-8f); f[24] = rsq(c2 + 1e-8f);
    f[25] = rf0 * cf0 * m0; f[26] = rf1 * cf1 * m1; f[27] = rf2 * cf2 * m2;
  } else {
    // celo2_kernel.cu:48-125 (rsqrt epsilon fixed at 1e-8), velo_kernel.cu:72-164 (epsilon argument)
    const float rs = rsq(v + (F == kFamCelo2 ? 1e-8f : a.epsilon));
    f[0] = g; f[1] = fminf(fmaxf(g, -0.1f), 0.1f); f[2] = p; f[3] = m0; f[4] = m1; f[5] = m2; f[6] = v;
    f[7] = m0 * rs; f[8] = m1 * rs; f[9] = m2 * rs; f[10] = rs;
    f[11] = g * rf0 * cf0; f[12] = g * rf1 * cf1; f[13] = g * rf2 * cf2;
    f[14] = g * rs;
    if (F == kFamCelo2 && vl) {   // only the first nine feature groups exist for a vector-like tensor
#pragma unroll
      for (int c = 15; c < 30; ++c) f[c] = 0.0f;
      return;
    }
    const float r0 = ld<ST>(a.fac_r, o.r), r1 = ld<ST>(a.fac_r, o.r + (size_t)o.stride_r), r2 = ld<ST>(a.fac_r, o.r + 2 * (size_t)o.stride_r);
    const float c0 = ld<ST>(a.fac_c, o.c), c1 = ld<ST>(a.fac_c, o.c + (size_t)o.stride_c), c2 = ld<ST>(a.fac_c, o.c + 2 * (size_t)o.stride_c);
    f[15] = r0; f[16] = r1; f[17] = r2; f[18] = c0; f[19] = c1; f[20] = c2;
    f[21] = rsq(r0 + 1e-8f); f[22] = rsq(r1 + 1e-8f); f[23] = rsq(r2 + 1e-8f);
    f[24] = rsq(c0 + 1e-8f); f[25] = rsq(c1 + 1e-8f); f[26] = rsq(c2 + 1e-8f);
    f[27] = m0 * rf0 * cf0; f[28] = m1 * rf1 * cf1; f[29] = m2 * rf2 * cf2;
  }
}

// second_moment[c] += sum over the elements of feature_c^2: per-thread and per-wave sums, then one
// float atomic per channel and block, as the reference does (celo2_kernel.cu:129-199).
template <int F, int ST>
__global__ __launch_bounds__(kSingleThreads) void k_single_moment(SingleArgs a) {
  constexpr int NS = Fam<F>::NSTAT;
  float acc[NS];
#pragma unroll
  for (int c = 0; c < NS; ++c) acc[c] = 0.0f;
  for (long long i = (long long)blockIdx.x * kSingleThreads + threadIdx.x; i < a.n;
       i += (long long)gridDim.x * kSingleThreads) {
    float f[NS];
    single_features<F, ST>(a, (int)i, f);
#pragma unroll
    for (int c = 0; c < NS; ++c) acc[c] = fmaf(f[c], f[c], acc[c]);
  }
  __shared__ float s[kSingleThreads / 64][NS];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int c = 0; c < NS; ++c) {
    const float t = wave_sum(acc[c]);
    if (lane == 0) s[wave][c] = t;
  }
  __syncthreads();
  if (threadIdx.x < NS) {
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < kSingleThreads / 64; ++w) t += s[w][threadIdx.x];
    atomicAdd(a.second_moment + threadIdx.x, t);
  }
}

// The MLP of one element on normalised features; WP is the pointer type the weights are read through.
template <int F, class WP>
__device__ __forceinline__ void single_mlp(const float (&f)[Fam<F>::NSTAT], const float* b1, WP w1, WP w2, WP w3, WP bh,
                                           WP bo, float (&out)[Fam<F>::NOUT]) {
  using Fm = Fam<F>;
  constexpr int NS = Fm::NSTAT, NIN = Fm::NIN, H = Fm::H, NO = Fm::NOUT;
  float h0[H], h1[H];
  if constexpr (Fm::in_major) {
#pragma unroll
    for (int j = 0; j < H; ++j) h0[j] = b1[j];
#pragma unroll
    for (int k = 0; k < NS; ++k)
#pragma unroll
      for (int j = 0; j < H; ++j) h0[j] = fmaf(f[k], w1[k * H + j], h0[j]);
#pragma unroll
    for (int j = 0; j < H; ++j) { h0[j] = fmaxf(h0[j], 0.0f); h1[j] = bh[j]; }
#pragma unroll
    for (int k = 0; k < H; ++k)
#pragma unroll
      for (int j = 0; j < H; ++j) h1[j] = fmaf(h0[k], w2[k * H + j], h1[j]);
#pragma unroll
    for (int j = 0; j < NO; ++j) out[j] = bo[j];
#pragma unroll
    for (int k = 0; k < H; ++k) {
      const float hk = fmaxf(h1[k], 0.0f);
#pragma unroll
      for (int j = 0; j < NO; ++j) out[j] = fmaf(hk, w3[k * NO + j], out[j]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < H; ++j) {
      float acc = b1[j];
#pragma unroll
      for (int k = 0; k < NS; ++k) acc = fmaf(f[k], w1[j * NIN + k], acc);
      h0[j] = fmaxf(acc, 0.0f);
    }
#pragma unroll
    for (int j = 0; j < H; ++j) {
      float acc = bh[j];
#pragma unroll
      for (int k = 0; k < H; ++k) acc = fmaf(h0[k], w2[j * H + k], acc);
      h1[j] = fmaxf(acc, 0.0f);
    }
#pragma unroll
    for (int j = 0; j < NO; ++j) {
      float acc = bo[j];
#pragma unroll
      for (int k = 0; k < H; ++k) acc = fmaf(h1[k], w3[j * H + k], acc);
      out[j] = acc;
    }
  }
}

// Normalise by rsqrt(second_moment / n + eps), MLP, output.  The weights are the same for every lane:
// float weights are read through the scalar cache into SGPRs where they are used (the pointer is laundered
// once per element so that the loads stay inside the loop instead of being hoisted into a register file they
// do not fit), which leaves the vector pipe with the multiply-adds only; weights of another element type are
// widened into LDS once per block and read from there.  AdafacLO's eleven time features are the same for
// every element and go into the first bias, once per block.
template <int F, int ST>
__global__ __launch_bounds__(kSingleThreads) void k_single_apply(SingleArgs a) {
  using Fm = Fam<F>;
  constexpr int NS = Fm::NSTAT, NIN = Fm::NIN, H = Fm::H, NO = Fm::NOUT;
  constexpr int kW1 = 0, kW2 = NIN * H, kW3 = kW2 + H * H, kBH = kW3 + H * NO, kBO = kBH + H, kWTot = kBO + NO;
  __shared__ float s_norm[NS];
  __shared__ float b1[H];
  __shared__ float wl[ST == kStoreF32 ? 1 : kWTot];
  const int tid = threadIdx.x;
  const float nf = (float)a.n;
  if (tid < NS) s_norm[tid] = rsq(a.second_moment[tid] / nf + (F == kFamCelo2 ? 1e-9f : 1e-5f));
  if (tid < H) {
    float b = ld<ST>(a.b_in, tid);
    if constexpr (F == kFamLo) {   // tanh(step / ts - 1), learned_optimizer.cu:27-32
      const float ts[11] = {1.f, 3.f, 10.f, 30.f, 100.f, 300.f, 1000.f, 3000.f, 10000.f, 30000.f, 100000.f};
#pragma unroll
      for (int q = 0; q < 11; ++q) b = fmaf(tanhf(a.step / ts[q] - 1.0f), ld<ST>(a.w_in, tid * NIN + NS + q), b);
    }
    b1[tid] = b;
  }
  if constexpr (ST != kStoreF32) {
    for (int i = tid; i < NIN * H; i += kSingleThreads) wl[kW1 + i] = ld<ST>(a.w_in, i);
    for (int i = tid; i < H * H; i += kSingleThreads) wl[kW2 + i] = ld<ST>(a.w_h, i);
    for (int i = tid; i < H * NO; i += kSingleThreads) wl[kW3 + i] = ld<ST>(a.w_out, i);
    for (int i = tid; i < H; i += kSingleThreads) wl[kBH + i] = ld<ST>(a.b_h, i);
    for (int i = tid; i < NO; i += kSingleThreads) wl[kBO + i] = ld<ST>(a.b_out, i);
  }
  __syncthreads();
  const float pscale = F == kFamVelo ? sqrtf(a.second_moment[2] / nf + 1e-9f) : 1.0f;   // channel 2 is p

  for (long long i = (long long)blockIdx.x * kSingleThreads + tid; i < a.n; i += (long long)gridDim.x * kSingleThreads) {
    float f[NS];
    single_features<F, ST>(a, (int)i, f);
    const float p_old = f[F == kFamLo ? 1 : 2];
#pragma unroll
    for (int k = 0; k < NS; ++k) f[k] *= s_norm[k];
    float out[NO];
    if constexpr (ST == kStoreF32)
      single_mlp<F>(f, b1, launder(a.w_in), launder(a.w_h), launder(a.w_out), launder(a.b_h), launder(a.b_out), out);
    else
      single_mlp<F, const float*>(f, b1, wl + kW1, wl + kW2, wl + kW3, wl + kBH, wl + kBO, out);
    const float step = out[0] * expf(out[1] * a.exp_mult);
    if constexpr (F == kFamCelo2) {
      st<ST>(a.step_out, i, step);                             // celo2_kernel.cu:280; p is left untouched
    } else if constexpr (F == kFamLo) {
      st<ST>(a.p, i, p_old - a.lr * (step * a.step_mult));    // learned_optimizer.cu:296-299
    } else {
      float pn = p_old - a.lr * (pscale * step * a.step_mult); // velo_kernel.cu:352-362
      if (a.weight_decay > 0.0f) pn = pn - a.weight_decay * a.lr * pn;
      st<ST>(a.p, i, pn);
    }
  }
}

}  // namespace pylo
