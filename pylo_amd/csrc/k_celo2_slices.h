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
constexpr int kSliceLaneClasses = 4;   // of slice length, for the kernel that stages such slices through LDS
constexpr int kSliceLaneClassMax[kSliceLaneClasses] = {4, 9, 16, kSliceLaneMax};
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

// What an element of a tensor with more than two dims reads of the factored statistics: the products of the table
// (row and column) and the two accumulators themselves, three decays each.  Gathered apart from the arithmetic so
// that a walk over a slice can have the next element's loads in flight while it works on this one.
struct SliceFac { float4 fa, fb; float fr[3], fc[3]; };
__device__ __forceinline__ SliceFac slice_gather_nd(const TDesc& d, const PyloTensorArgs& a, long long idx,
                                                    const float* __restrict__ fac_tab) {
  const unsigned u = (unsigned)idx;
  const unsigned s0 = (unsigned)d.nd_stride[0], s1 = (unsigned)d.nd_stride[1];
  const int i0 = (int)(fd_div(u, d.nd_div_blk[0]) * s0 + (u - fd_div(u, d.nd_div_st[0]) * s0));
  const int i1 = (int)(fd_div(u, d.nd_div_blk[1]) * s1 + (u - fd_div(u, d.nd_div_st[1]) * s1));
  SliceFac x;
  x.fa = load_f4(fac_tab + d.fac_off[0] + (size_t)i0 * 4);
  x.fb = load_f4(fac_tab + d.fac_off[1] + (size_t)i1 * 4);
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    x.fr[k] = *(const gfloat*)(a.fac_r + (size_t)k * d.len[0] + i0);  // vector 0 is the row vector
    x.fc[k] = *(const gfloat*)(a.fac_c + (size_t)k * d.len[1] + i1);
  }
  return x;
}

// The feature channels of one element of a tensor with more than two dims from its inputs and accumulators as
// they stand after this step's update (what slice_element computes after loading and updating them).
__device__ __forceinline__ void slice_features_nd(const SliceFac& x, float g, float p, const float (&m)[3], float rms,
                                                  float (&f)[30]) {
  const float rfcf[3] = {x.fa.x * x.fb.x, x.fa.y * x.fb.y, x.fa.z * x.fb.z};
  float f18[kNStat];
  lo_features(g, p, m, rms, rfcf, 1e-8f, f18);
#pragma unroll
  for (int c = 0; c < 15; ++c) f[c] = f18[c];
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    f[15 + k] = x.fr[k];
    f[18 + k] = x.fc[k];
    f[21 + k] = rsq(x.fr[k] + 1e-8f);
    f[24 + k] = rsq(x.fc[k] + 1e-8f);
    f[27 + k] = f18[15 + k];
  }
}

// The raw MLP block as the lane-local matrix instruction wants it (mfma_w4: four weights of one input from four
// neighbouring lanes): 96 groups of four floats in six registers a lane.  w_in, b_in, w_h, b_h are already rows of
// eight = two groups; a row of w_out (three outputs) and b_out become a group each, padded with a zero.
constexpr int kC2GrpBI = 60, kC2GrpWH = 62, kC2GrpBH = 78, kC2GrpWO = 80, kC2GrpBO = 88;
__device__ __forceinline__ void slice_mlp_weights(const float* __restrict__ mlp, float (&wreg)[6]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const int q = 64 * r + lane, g = q >> 2, j = q & 3;
    int src = q;                                   // w_in | b_in | w_h | b_h: as stored
    if (g >= kC2GrpBO) src = g == kC2GrpBO && j < 3 ? kC2RawBO + j : -1;
    else if (g >= kC2GrpWO) src = j < 3 ? kC2RawWO + 3 * (g - kC2GrpWO) + j : -1;
    wreg[r] = src >= 0 ? *(const gfloat*)(mlp + src) : 0.0f;
  }
}

// direction * exp(magnitude * exp_mult) from the normalised features, on the matrix pipe: every lane of the wave
// must get here (lanes without an element pass zeros and drop the result).
__device__ __forceinline__ float slice_mlp_mfma(const float (&f)[30], const float (&s)[30], const float (&wreg)[6],
                                                float exp_mult) {
  const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
  v4f ha = mfma_w4(wreg[kC2GrpBI / 16], 1.0f, zero, kC2GrpBI % 16);
  v4f hb = mfma_w4(wreg[(kC2GrpBI + 1) / 16], 1.0f, zero, (kC2GrpBI + 1) % 16);
#pragma unroll
  for (int c = 0; c < 30; ++c) {
    const float x = f[c] * s[c];
    ha = mfma_w4(wreg[(2 * c) / 16], x, ha, (2 * c) % 16);
    hb = mfma_w4(wreg[(2 * c + 1) / 16], x, hb, (2 * c + 1) % 16);
  }
  v4f ga = mfma_w4(wreg[kC2GrpBH / 16], 1.0f, zero, kC2GrpBH % 16);
  v4f gb = mfma_w4(wreg[(kC2GrpBH + 1) / 16], 1.0f, zero, (kC2GrpBH + 1) % 16);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float hk = fmaxf(k < 4 ? ha[k] : hb[k - 4], 0.0f);
    ga = mfma_w4(wreg[(kC2GrpWH + 2 * k) / 16], hk, ga, (kC2GrpWH + 2 * k) % 16);
    gb = mfma_w4(wreg[(kC2GrpWH + 2 * k + 1) / 16], hk, gb, (kC2GrpWH + 2 * k + 1) % 16);
  }
  v4f o = mfma_w4(wreg[kC2GrpBO / 16], 1.0f, zero, kC2GrpBO % 16);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float hk = fmaxf(k < 4 ? ga[k] : gb[k - 4], 0.0f);
    o = mfma_w4(wreg[(kC2GrpWO + k) / 16], hk, o, (kC2GrpWO + k) % 16);
  }
  return o[0] * expf(o[1] * exp_mult);
}

// Short slices of tensors with more than two dims (convolution kernels: 1 .. 32 elements a slice), one lane per
// slice, 64 consecutive slices per block (one wave).  The wave's slices are contiguous in every array: gradient,
// parameter and accumulators come in with coalesced loads, through LDS ([element of the slice][slice], pitch 65: the
// lanes' walks over their own slices are conflict-free), the accumulators are updated there on the first walk, the
// second walk leaves the raw step in the gradient's place, and everything goes out coalesced.  Every input is read
// once and every output written once.  A block takes several such groups of 64 slices one after another when the
// slices are very short (the set-up of a block is some hundreds of instructions, as much as the walk over a few
// elements).  Item: tensor, first slice of the block.
constexpr int kSlicePitchF = 65;
__host__ __device__ constexpr int slice_lane_groups(int S) { return S <= 2 ? 8 : S <= 4 ? 4 : S <= 9 ? 2 : 1; }
__global__ __launch_bounds__(64) void k_celo2_slices_lane(const TDesc* __restrict__ descs,
                                                          const PyloTensorArgs* __restrict__ dyn,
                                                          const Item* __restrict__ items,
                                                          const float* __restrict__ fac_tab,
                                                          const Globals* __restrict__ gl, PyloDecays dec,
                                                          const float* __restrict__ mlp) {
  extern __shared__ float sl_lds[];
  constexpr int P = kSlicePitchF;
  const Item it = items[blockIdx.x];
  TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  set_grad_scale(d, a, gl, it.tensor);
  const EmaConsts e = make_ema(dec);
  const int S = d.slice_len, lane = threadIdx.x;
  const long long n = d.n, n_slices = n / S;
  float* Lg = sl_lds;
  float* Lp = Lg + S * P;
  float* Lm0 = Lp + S * P;
  float* Lm1 = Lm0 + S * P;
  float* Lm2 = Lm1 + S * P;
  float* Lr = Lm2 + S * P;
  // idx / S for idx < 64 * S <= 2048 without the integer division: the half keeps the product 0.5 / S away from
  // the integers, the rounding of a float product of this size is some 1e-4 at most
  const float inv_s = 1.0f / (float)S;
  float wreg[6];
  slice_mlp_weights(mlp, wreg);
  if (S == 1) {
    // A slice is an element (1 x 1 kernels): nothing to stage, every lane takes its own element, and the next
    // group's loads are in flight under this group's arithmetic.  Lanes past the end work on the block's first element
    // and store nothing.
    struct In { float g, p, m[3], r; SliceFac fac; };
    auto fetch = [&](long long idx) {
      In x;
      x.g = *(const gfloat*)(a.grad + idx);
      x.p = *(const gfloat*)(a.param + idx);
      x.m[0] = *(const gfloat*)(a.mom + idx);
      x.m[1] = *(const gfloat*)(a.mom + n + idx);
      x.m[2] = *(const gfloat*)(a.mom + 2 * n + idx);
      x.r = *(const gfloat*)(a.rms + idx);
      x.fac = slice_gather_nd(d, a, idx, fac_tab);
      return x;
    };
    const long long b0 = it.a;
    In cur = fetch(b0 + lane < n ? b0 + lane : b0);
    for (int grp = 0; grp < slice_lane_groups(1); ++grp) {
      const long long idx = b0 + 64 * grp + lane;
      if (b0 + 64 * grp >= n) break;
      const bool mine = idx < n;
      const long long nidx = idx + 64;
      const In nxt = fetch(grp + 1 < slice_lane_groups(1) && nidx < n ? nidx : b0);
      const float g = cond_grad(cur.g, d.gscale, a.clip_val, d.nan0);
      float m[3] = {cur.m[0], cur.m[1], cur.m[2]}, rms = cur.r, f[30], sc[30];
      ema_update(e, g, m, rms);
      slice_features_nd(cur.fac, g, cur.p, m, rms, f);
#pragma unroll
      for (int c = 0; c < 30; ++c) sc[c] = rsq(1e-9f + f[c] * f[c]);
      const float step = slice_mlp_mfma(f, sc, wreg, a.exp_mult);
      if (mine) {
        *(gfloat*)(a.mom + idx) = m[0];
        *(gfloat*)(a.mom + n + idx) = m[1];
        *(gfloat*)(a.mom + 2 * n + idx) = m[2];
        *(gfloat*)(a.rms + idx) = rms;
        *(gfloat*)(a.step_out + idx) = step;
      }
      cur = nxt;
    }
    return;
  }
  for (int grp = 0; grp < slice_lane_groups(S); ++grp) {
    const long long s0 = (long long)it.a + 64 * grp, left = n_slices - s0;
    if (left <= 0) break;
    const int live = left < 64 ? (int)left : 64, total = live * S;
    const long long e0 = s0 * S;
    for (int idx = lane; idx < total; idx += 64) {
      const int sl = (int)(((float)idx + 0.5f) * inv_s), pos = (idx - sl * S) * P + sl;
      const long long gi = e0 + idx;
      Lg[pos] = cond_grad(*(const gfloat*)(a.grad + gi), d.gscale, a.clip_val, d.nan0);
      Lp[pos] = *(const gfloat*)(a.param + gi);
      Lm0[pos] = *(const gfloat*)(a.mom + gi);
      Lm1[pos] = *(const gfloat*)(a.mom + n + gi);
      Lm2[pos] = *(const gfloat*)(a.mom + 2 * n + gi);
      Lr[pos] = *(const gfloat*)(a.rms + gi);
    }
    __syncthreads();
    {
      // every lane walks a slice (the matrix instructions of the MLP want the whole wave): lanes past the last slice
      // walk the first one again and write nothing
      const bool mine = lane < live;
      const int col = mine ? lane : 0;
      const long long first = e0 + (long long)col * S;
      float acc[30], f[30];
#pragma unroll
      for (int c = 0; c < 30; ++c) acc[c] = 0.0f;
      SliceFac fac = slice_gather_nd(d, a, first, fac_tab);
      for (int j = 0; j < S; ++j) {
        // the next element's loads before this one's arithmetic; the last round fetches the second walk's first
        const SliceFac nxt = slice_gather_nd(d, a, first + (j + 1 < S ? j + 1 : 0), fac_tab);
        const int pos = j * P + col;
        float m[3] = {Lm0[pos], Lm1[pos], Lm2[pos]}, rms = Lr[pos];
        const float g = Lg[pos];
        ema_update(e, g, m, rms);
        if (mine) { Lm0[pos] = m[0]; Lm1[pos] = m[1]; Lm2[pos] = m[2]; Lr[pos] = rms; }
        slice_features_nd(fac, g, Lp[pos], m, rms, f);
        fac = nxt;
#pragma unroll
        for (int c = 0; c < 30; ++c) acc[c] = fmaf(f[c], f[c], acc[c]);
      }
      float sc[30];
#pragma unroll
      for (int c = 0; c < 30; ++c) sc[c] = rsq(1e-9f + acc[c] * inv_s);   // the mean by the reciprocal, not thirty divisions
      for (int j = 0; j < S; ++j) {
        const int pos = j * P + col;
        if (S > 1) {   // a slice of one element still has its features from the first walk
          const SliceFac nxt = slice_gather_nd(d, a, first + (j + 1 < S ? j + 1 : 0), fac_tab);
          const float m[3] = {Lm0[pos], Lm1[pos], Lm2[pos]};
          slice_features_nd(fac, Lg[pos], Lp[pos], m, Lr[pos], f);
          fac = nxt;
        }
        const float step = slice_mlp_mfma(f, sc, wreg, a.exp_mult);
        if (mine) Lg[pos] = step;
      }
    }
    __syncthreads();
    for (int idx = lane; idx < total; idx += 64) {
      const int sl = (int)(((float)idx + 0.5f) * inv_s), pos = (idx - sl * S) * P + sl;
      const long long gi = e0 + idx;
      *(gfloat*)(a.mom + gi) = Lm0[pos];
      *(gfloat*)(a.mom + n + gi) = Lm1[pos];
      *(gfloat*)(a.mom + 2 * n + gi) = Lm2[pos];
      *(gfloat*)(a.rms + gi) = Lr[pos];
      *(gfloat*)(a.step_out + gi) = Lg[pos];
    }
    __syncthreads();   // the next group's loads overwrite what the stores above read
  }
}

// Item: tensor, first slice of the block.  A block covers 256 slices (one per lane) or 4 (one per wave)."
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
