// ELO-CELO2 / CELO2 MLP tensors whose feature normalisers are not tensor-wide: tensors with more
// than two dims (the naive class normalises every feature over the last two dims only,
// ELO_CELO2_naive.py:217-218, so each slice of the last two dims has its own 30 normalisers) and
// tensors with fewer than two dims on the MLP path (use_adamw_for_1d=False: per-element Adafactor
// accumulator, the first nine feature groups only, :166-169,180-191).  The row / column vectors of an
// N-D tensor still span the whole tensor and come from the P0 / V0 passes; everything after that is
// local to a slice, so one pass does statistics, MLP and the accumulator writes.
//
// A slice is walked twice (sum of squares, then apply) by one lane when it is short (conv kernels:
// 9 .. 32 elements) and by one wave otherwise.  These tensors are small in the models this path
// serves (patch embeddings, conv kernels, biases); the kernel is written for correctness on any
// shape, not for the bandwidth roofline.
#pragma once

#include "k_velo.h"

namespace pylo {

constexpr int kSliceLaneMax = 32;  // slices up to this length are walked by a single lane
// raw CELO2 MLP block: w_in (30,8) | b_in 8 | w_h (8,8) | b_h 8 | w_out (8,3) | b_out 3, all (in, out)
constexpr int kC2RawBI = 240, kC2RawWH = 248, kC2RawBH = 312, kC2RawWO = 320, kC2RawBO = 344;

// Accumulators of element idx advanced, and its feature channels in the reference's 30-channel order.
template <bool VEC>
__device__ __forceinline__ void slice_element(const TDesc& d, const PyloTensorArgs& a, long long idx,
                                              const EmaConsts& e, const PyloDecays& dec,
                                              const float* __restrict__ fac_tab, float (&f)[30], float (&m)[3],
                                              float& rms, float (&fv)[3]) {
  float f18[kNStat];
  if constexpr (VEC) {
    const long long n = d.n;
    const float g = cond_grad(*(const gfloat*)(a.grad + idx), d.gscale, a.clip_val, d.nan0);
    const float p = *(const gfloat*)(a.param + idx);
    rms = *(const gfloat*)(a.rms + idx);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      m[k] = *(const gfloat*)(a.mom + k * n + idx);
      fv[k] = *(const gfloat*)(a.fac_v + k * n + idx);
    }
    vec_update(e, dec, g, m, rms, fv);
    float rf[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) rf[k] = rsq(fmaxf(fv[k] + 1e-9f, 1e-9f));
    lo_features(g, p, m, rms, rf, 1e-8f, f18);
#pragma unroll
    for (int c = 0; c < 15; ++c) f[c] = f18[c];
#pragma unroll
    for (int c = 15; c < 30; ++c) f[c] = 0.0f;
  } else {
    ElemIn<1> x;
    lo_load<1, true>(d, a, idx, fac_tab, x);
    ema_update(e, x.g[0], x.m[0], x.rms[0]);
    lo_features(x.g[0], x.p[0], x.m[0], x.rms[0], x.rfcf[0], 1e-8f, f18);
#pragma unroll
    for (int c = 0; c < 15; ++c) f[c] = f18[c];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const float fr = *(const gfloat*)(a.fac_r + (size_t)k * d.len[0] + x.i0);  // vector 0 is the row vector
      const float fc = *(const gfloat*)(a.fac_c + (size_t)k * d.len[1] + x.i1);
      f[15 + k] = fr;
      f[18 + k] = fc;
      f[21 + k] = rsq(fr + 1e-8f);
      f[24 + k] = rsq(fc + 1e-8f);
      f[27 + k] = f18[15 + k];
      m[k] = x.m[0][k];
    }
    rms = x.rms[0];
  }
}

// direction * exp(magnitude * exp_mult) from the normalised features (ELO_CELO2_naive.py:219-229)
template <int NC>
__device__ __forceinline__ float slice_mlp(const float (&f)[30], const float (&s)[30], const cfloat* w, float exp_mult) {
  float h0[8], h1[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) h0[j] = w[kC2RawBI + j];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const float x = f[c] * s[c];
#pragma unroll
    for (int j = 0; j < 8; ++j) h0[j] = fmaf(x, w[c * 8 + j], h0[j]);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) h1[j] = w[kC2RawBH + j];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float hk = fmaxf(h0[k], 0.0f);
#pragma unroll
    for (int j = 0; j < 8; ++j) h1[j] = fmaf(hk, w[kC2RawWH + k * 8 + j], h1[j]);
  }
  float o0 = w[kC2RawBO + 0], o1 = w[kC2RawBO + 1];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float hk = fmaxf(h1[k], 0.0f);
    o0 = fmaf(hk, w[kC2RawWO + k * 3 + 0], o0);
    o1 = fmaf(hk, w[kC2RawWO + k * 3 + 1], o1);
  }
  return o0 * expf(o1 * exp_mult);
}

// One slice: elements first + j for j = j0, j0 + dj, ... < S.  LANE: the lane owns the slice (no
// reduction across lanes); else the 64 lanes of the wave share it.
template <bool VEC, bool LANE>
__device__ __forceinline__ void slice_run(const TDesc& d, const PyloTensorArgs& a, long long first, int S,
                                          const EmaConsts& e, const PyloDecays& dec,
                                          const float* __restrict__ fac_tab, const cfloat* w) {
  constexpr int NC = VEC ? 15 : 30;
  const int j0 = LANE ? 0 : (threadIdx.x & 63), dj = LANE ? 1 : 64;
  float acc[30];
#pragma unroll
  for (int c = 0; c < 30; ++c) acc[c] = 0.0f;
  for (int j = j0; j < S; j += dj) {
    float f[30], m[3], rms, fv[3];
    slice_element<VEC>(d, a, first + j, e, dec, fac_tab, f, m, rms, fv);
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = fmaf(f[c], f[c], acc[c]);
  }
  float s[30];
#pragma unroll
  for (int c = 0; c < 30; ++c) {
    const float tot = (LANE || c >= NC) ? acc[c] : wave_sum(acc[c]);
    s[c] = rsq(1e-9f + tot / (float)S);
  }
  const long long n = d.n;
  for (int j = j0; j < S; j += dj) {
    const long long idx = first + j;
    float f[30], m[3], rms, fv[3];
    slice_element<VEC>(d, a, idx, e, dec, fac_tab, f, m, rms, fv);
    const float step = slice_mlp<NC>(f, s, w, a.exp_mult);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      *(gfloat*)(a.mom + k * n + idx) = m[k];
      if constexpr (VEC) *(gfloat*)(a.fac_v + k * n + idx) = fv[k];
    }
    *(gfloat*)(a.rms + idx) = rms;
    *(gfloat*)(a.step_out + idx) = step;
  }
}

// Item: tensor, first slice of the block.  A block covers 256 slices (one per lane) or 4 (one per wave).
__global__ __launch_bounds__(kThreads) void k_celo2_slices(const TDesc* __restrict__ descs,
                                                           const PyloTensorArgs* __restrict__ dyn,
                                                           const Item* __restrict__ items,
                                                           const float* __restrict__ fac_tab,
                                                           const Globals* __restrict__ gl, PyloDecays dec,
                                                           const float* __restrict__ mlp) {
  const Item it = items[blockIdx.x];
  TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  set_grad_scale(d, a, gl, it.tensor);
  const EmaConsts e = make_ema(dec);
  const cfloat* w = launder(mlp);
  const int S = d.slice_len;
  const long long n_slices = d.n / S;
  const bool vec = d.mode == kModeVec;
  if (S <= kSliceLaneMax) {
    const long long sl = (long long)it.a + threadIdx.x;
    if (sl >= n_slices) return;
    if (vec) slice_run<true, true>(d, a, sl * S, S, e, dec, fac_tab, w);
    else slice_run<false, true>(d, a, sl * S, S, e, dec, fac_tab, w);
  } else {
    const long long sl = (long long)it.a + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (sl >= n_slices) return;
    if (vec) slice_run<true, false>(d, a, sl * S, S, e, dec, fac_tab, w);
    else slice_run<false, false>(d, a, sl * S, S, e, dec, fac_tab, w);
  }
}

}  // namespace pylo
