// AdafacLO (small_fc_lopt): element kernels.  28 normalised features + 11 time features,
// 39 -> 32 -> 32 -> 2 MLP, parameter updated in place (pylo/optim/AdafacLO_naive.py:187-311).
//
// The 28 features are the VeLO channel set without clip(g) and g*rsqrt(rms); they are kept in the
// same 30-channel numbering so the statistics machinery is shared.  The 11 time features are the
// same for every element of a step and are folded into the first-layer bias.
#pragma once

#include "k_velo.h"

namespace pylo {

// Host-packed network (floats), all (in, out):
//   w1 (30,32) rows in the 30-channel order (rows 1 and 14 zero) | b1 32 | w_time (11,32) |
//   w_h (32,32) | b_h 32 | w_o (32,2) | b_o 2
#ifndef PYLO_ADAFAC_WAVES
#define PYLO_ADAFAC_WAVES 3
#endif
constexpr int kAH = 32;
constexpr int kAW1 = 0, kAB1 = 960, kAWT = 992, kAWH = 1344, kABH = 2368, kAWO = 2400, kABO = 2464, kANet = 2466;
constexpr int kAFold = 992;  // per-tensor first-layer rows scaled by the channel normalisers, then the 30 normalisers themselves

__host__ __device__ constexpr bool adafac_channel(int c) { return c != 1 && c != 14; }

// b_eff = b1 + w_time^T tanh(step / ts - 1)   (AdafacLO_naive.py:81-87,226)
// One block per tensor: `step` >= 0 is the counter of every tensor, a negative `step` takes each
// tensor's own counter from its argument record (bc1; AdafacLO_cuda.py:304-305,400 keeps one per parameter).
__global__ __launch_bounds__(64) void k_adafac_bias(const float* __restrict__ net, float step,
                                                    const PyloTensorArgs* __restrict__ dyn,
                                                    float* __restrict__ bias_all) {
  const float ts[11] = {1.f, 3.f, 10.f, 30.f, 100.f, 300.f, 1000.f, 3000.f, 10000.f, 30000.f, 100000.f};
  const int j = threadIdx.x;
  if (j >= kAH) return;
  if (step < 0.0f) step = dyn[blockIdx.x].bc1;
  float* bias_eff = bias_all + (size_t)blockIdx.x * kAH;
  float acc = net[kAB1 + j];
#pragma unroll
  for (int q = 0; q < 11; ++q) acc = fmaf(tanhf(step / ts[q] - 1.0f), net[kAWT + q * kAH + j], acc);
  bias_eff[j] = acc;
}

template <int V, bool ND>
__device__ __forceinline__ void adafac_stats_fac(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                 const EmaConsts& e, const float* __restrict__ fac_tab, VeloAcc& acc) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
#pragma unroll 2
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= d.n) break;
    ElemIn<V> x;
    lo_load<V, ND>(d, a, idx, fac_tab, x);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ema_update(e, x.g[v], x.m[v], x.rms[v]);
      float f[kNStat];
      lo_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.rfcf[v], 1e-6f, f);
#pragma unroll
      for (int c = 0; c < kNStat; ++c)
        if (adafac_channel(stat_channel(c))) acc.ch[stat_channel(c)] = fmaf(f[c], f[c], acc.ch[stat_channel(c)]);
    }
  }
}

// Column-resident walk of one wave task (wide 2-D tensors), as in VeLO's statistics pass.
__device__ __forceinline__ void adafac_stats_tile(const TDesc& d, const PyloTensorArgs& a, int task,
                                                  const EmaConsts& e, const float* __restrict__ fac_tab,
                                                  VeloAcc& acc) {
  constexpr int V = kTileV;
  const TileTask tk(d, task);
  const float* f0 = fac_tab + d.fac_off[0];
  const float* f1 = fac_tab + d.fac_off[1];
  float fb[V][4];
#pragma unroll
  for (int v = 0; v < V; ++v) load_vec_o<4>(f1 + v * 4, tk.col * 16u, fb[v]);
  const unsigned lo = (threadIdx.x & 63) * (V * 4u);
  const float *g = a.grad + tk.first, *p = a.param + tk.first, *m0 = a.mom + tk.first,
              *m1 = a.mom + d.n + tk.first, *m2 = a.mom + 2 * d.n + tk.first, *rms = a.rms + tk.first;
  const float* fr = f0 + (size_t)tk.r0 * 4;
#pragma unroll 2
  for (int r = tk.r0; r < tk.r1; ++r) {
    float xg[V], xp[V], x0[V], x1[V], x2[V], xr[V], fa[4];
    load_vec_nt<V>(g, lo, xg);
    load_vec_nt<V>(p, lo, xp);
    load_vec_nt<V>(m0, lo, x0);
    load_vec_nt<V>(m1, lo, x1);
    load_vec_nt<V>(m2, lo, x2);
    load_vec_nt<V>(rms, lo, xr);
    load_uniform<4>(fr, fa);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const float gg = cond_grad(xg[v], d.gscale, a.clip_val, d.nan0);
      float m[3] = {x0[v], x1[v], x2[v]};
      float rr = xr[v];
      ema_update(e, gg, m, rr);
      const float rfcf[3] = {fa[0] * fb[v][0], fa[1] * fb[v][1], fa[2] * fb[v][2]};
      float f[kNStat];
      lo_features(gg, xp[v], m, rr, rfcf, 1e-6f, f);
#pragma unroll
      for (int c = 0; c < kNStat; ++c)
        if (adafac_channel(stat_channel(c))) acc.ch[stat_channel(c)] = fmaf(f[c], f[c], acc.ch[stat_channel(c)]);
    }
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0; fr += 4;
  }
}

template <int V>
__device__ __forceinline__ void adafac_stats_vec(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                 const EmaConsts& e, const PyloDecays& dec, VeloAcc& acc) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= d.n) break;
    VecIn<V> x;
    vec_load<V>(d, a, idx, x);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      vec_update(e, dec, x.g[v], x.m[v], x.rms[v], x.v[v]);
      float f[30];
      vec_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.v[v], 1e-6f, f);
#pragma unroll
      for (int c = 0; c < 30; ++c)
        if (adafac_channel(c)) acc.ch[c] = fmaf(f[c], f[c], acc.ch[c]);
    }
  }
}

__global__ __launch_bounds__(kThreads) void k_adafac_stats(const TDesc* __restrict__ descs,
                                                           const PyloTensorArgs* __restrict__ dyn,
                                                           const Item* __restrict__ items,
                                                           const float* __restrict__ fac_tab, PyloDecays dec,
                                                           double* __restrict__ stats_part,
                                                           const Globals* __restrict__ gl) {
  __shared__ float red[kWaves][30];
  const Item it = items[blockIdx.x];
  TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  set_grad_scale(d, a, gl, it.tensor);
  const EmaConsts e = make_ema(dec);
  VeloAcc acc;
#pragma unroll
  for (int c = 0; c < 30; ++c) acc.ch[c] = 0.0f;
  if (d.tile_nct > 0) {
    const int task = it.a * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (task < d.tile_ntask) adafac_stats_tile(d, a, task, e, fac_tab, acc);
  } else if (d.mode == kModeFac2D) {
    if (d.vec == 4) adafac_stats_fac<4, false>(d, a, it.a, e, fac_tab, acc);
    else adafac_stats_fac<1, false>(d, a, it.a, e, fac_tab, acc);
  } else if (d.mode == kModeFacND) {
    adafac_stats_fac<1, true>(d, a, it.a, e, fac_tab, acc);
  } else {
    if (d.vec == 4) adafac_stats_vec<4>(d, a, it.a, e, dec, acc);
    else adafac_stats_vec<1>(d, a, it.a, e, dec, acc);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int c = 0; c < 30; ++c) {
    const float s = wave_sum(acc.ch[c]);
    if (lane == 0) red[wave][c] = s;
  }
  __syncthreads();
  if (threadIdx.x < kStatW) {
    const int c = threadIdx.x;
    stats_part[(size_t)blockIdx.x * kStatW + c] =
        c < 30 ? ((double)red[0][c] + (double)red[1][c]) + ((double)red[2][c] + (double)red[3][c]) : 0.0;
  }
}

// Per tensor: first-layer rows scaled by rsqrt(1e-5 + mean f_c^2) (AdafacLO_naive.py:90-92,301).
__global__ __launch_bounds__(kThreads) void k_adafac_fold(const TDesc* __restrict__ descs,
                                                          const PyloTensorArgs* __restrict__ dyn,
                                                          const double* __restrict__ totals,
                                                          const float* __restrict__ net, float* __restrict__ wfold) {
  __shared__ float sc[32];
  const int t = blockIdx.x;
  const TDesc d = descs[t];
  if (dyn[t].grad == nullptr) return;
  if (threadIdx.x < 30) {
    const double n = (double)(d.n > 0 ? d.n : 1);
    sc[threadIdx.x] = rsq(1e-5f + (float)(totals[(size_t)t * kStatW + threadIdx.x] / n));
  }
  __syncthreads();
  float* w = wfold + (size_t)t * kAFold;
  for (int i = threadIdx.x; i < 30 * kAH; i += kThreads) w[i] = net[kAW1 + i] * sc[i / kAH];
  if (threadIdx.x < 32) w[30 * kAH + threadIdx.x] = threadIdx.x < 30 ? sc[threadIdx.x] : 0.0f;
}

// Parameter update from the unit step direction * exp(magnitude * exp_mult).  AdafacLO
// (AdafacLO_naive.py:305-310): p -= lr * step_mult * step, then p -= wd * lr * p on the updated value.
// ELO (ELO_naive.py:236-237): p -= lr * (step + wd * p) against the pre-step parameter.
__device__ __forceinline__ float adafac_update(const TDesc& d, const PyloTensorArgs& a, float unit_step, float p) {
  const float step = unit_step * a.step_mult;
  if (d.wd_prestep) return fmaf(step + a.weight_decay * p, -a.lr, p);
  p = fmaf(step, -a.lr, p);
  if (a.weight_decay > 0.0f) p = fmaf(p, -(a.weight_decay * a.lr), p);
  return p;
}

// One element per lane: 16 (factored) or 28 (non-factored) scaled features -> 32 -> 32 -> 2.
// Weights are wave-uniform and come through the scalar cache, one input row at a time.
template <int NF>
__device__ __forceinline__ float adafac_mlp(const float (&f)[NF], const int (&row)[NF], float (&h)[kAH],
                                            const float* wfold_t, const float* net, const TDesc& d,
                                            const PyloTensorArgs& a, float p) {
  const cfloat* w1 = launder(wfold_t);
  const cfloat* nw = launder(net);
#pragma unroll
  for (int c = 0; c < NF; ++c) {
#pragma unroll
    for (int j = 0; j < kAH; ++j) h[j] = fmaf(f[c], w1[row[c] * kAH + j], h[j]);
  }
  float h1[kAH];
#pragma unroll
  for (int j = 0; j < kAH; ++j) h1[j] = nw[kABH + j];
#pragma unroll
  for (int k = 0; k < kAH; ++k) {
    const float hk = fmaxf(h[k], 0.0f);
#pragma unroll
    for (int j = 0; j < kAH; ++j) h1[j] = fmaf(hk, nw[kAWH + k * kAH + j], h1[j]);
  }
  float o0 = nw[kABO + 0], o1 = nw[kABO + 1];
#pragma unroll
  for (int k = 0; k < kAH; ++k) {
    const float hk = fmaxf(h1[k], 0.0f);
    o0 = fmaf(hk, nw[kAWO + k * 2 + 0], o0);
    o1 = fmaf(hk, nw[kAWO + k * 2 + 1], o1);
  }
  return adafac_update(d, a, o0 * expf(o1 * a.exp_mult), p);
}

template <bool ND>
__device__ __forceinline__ void adafac_apply_fac(const TDesc& d, const PyloTensorArgs& a, long long base,
                                                 long long count, const EmaConsts& e,
                                                 const float* __restrict__ fac_tab, const float* __restrict__ term_tab,
                                                 const float* wfold_t, const float* net) {
  const long long n = d.n;
  for (long long off = threadIdx.x; off < count; off += kThreads) {
    const long long idx = base + off;
    if (idx >= n) break;
    ElemIn<1> x;
    if constexpr (ND) {
      lo_load<1, true>(d, a, idx, fac_tab, x);
    } else {  // 2-D, one element per lane
      x.g[0] = cond_grad(*(const gfloat*)(a.grad + idx), d.gscale, a.clip_val, d.nan0);
      x.p[0] = *(const gfloat*)(a.param + idx);
      x.m[0][0] = *(const gfloat*)(a.mom + idx);
      x.m[0][1] = *(const gfloat*)(a.mom + n + idx);
      x.m[0][2] = *(const gfloat*)(a.mom + 2 * n + idx);
      x.rms[0] = *(const gfloat*)(a.rms + idx);
      const unsigned u = (unsigned)idx;
      x.i0 = (int)(u / (unsigned)d.C0);
      x.i1 = (int)(u - (unsigned)x.i0 * (unsigned)d.C0);
      const float4 fa = load_f4(fac_tab + d.fac_off[0] + (size_t)x.i0 * 4);
      const float4 fb = load_f4(fac_tab + d.fac_off[1] + (size_t)x.i1 * 4);
      x.rfcf[0][0] = fa.x * fb.x;
      x.rfcf[0][1] = fa.y * fb.y;
      x.rfcf[0][2] = fa.z * fb.z;
    }
    float h[1][kAH];
    lo_terms<1, ND, kAH>(d, x, term_tab, h);
    ema_update(e, x.g[0], x.m[0], x.rms[0]);
    float f18[kNStat];
    lo_features(x.g[0], x.p[0], x.m[0], x.rms[0], x.rfcf[0], 1e-6f, f18);
    // the 16 per-element channels AdafacLO uses, and their rows in the 30-channel order
    const float f[16] = {f18[0], f18[2], f18[3], f18[4], f18[5], f18[6], f18[7], f18[8], f18[9], f18[10],
                         f18[11], f18[12], f18[13], f18[15], f18[16], f18[17]};
    const int row[16] = {0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 27, 28, 29};
    const float pn = adafac_mlp<16>(f, row, h[0], wfold_t, net, d, a, x.p[0]);
    *(gfloat*)(a.mom + idx) = x.m[0][0];
    *(gfloat*)(a.mom + n + idx) = x.m[0][1];
    *(gfloat*)(a.mom + 2 * n + idx) = x.m[0][2];
    *(gfloat*)(a.rms + idx) = x.rms[0];
    *(gfloat*)(a.param + idx) = pn;
  }
}

__device__ __forceinline__ void adafac_apply_vec(const TDesc& d, const PyloTensorArgs& a, long long base,
                                                 long long count, const EmaConsts& e, const PyloDecays& dec,
                                                 const float* wfold_t, const float* net, const float* bias_eff) {
  const long long n = d.n;
  for (long long off = threadIdx.x; off < count; off += kThreads) {
    const long long idx = base + off;
    if (idx >= n) break;
    VecIn<1> x;
    vec_load<1>(d, a, idx, x);
    vec_update(e, dec, x.g[0], x.m[0], x.rms[0], x.v[0]);
    float f30[30];
    vec_features(x.g[0], x.p[0], x.m[0], x.rms[0], x.v[0], 1e-6f, f30);
    float f[28];
    int row[28];
    {
      int q = 0;
#pragma unroll
      for (int c = 0; c < 30; ++c)
        if (adafac_channel(c)) { f[q] = f30[c]; row[q] = c; ++q; }
    }
    float h[kAH];
#pragma unroll
    for (int j = 0; j < kAH; ++j) h[j] = bias_eff[j];
    const float pn = adafac_mlp<28>(f, row, h, wfold_t, net, d, a, x.p[0]);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      *(gfloat*)(a.mom + k * n + idx) = x.m[0][k];
      *(gfloat*)(a.fac_v + k * n + idx) = x.v[0][k];
    }
    *(gfloat*)(a.rms + idx) = x.rms[0];
    *(gfloat*)(a.param + idx) = pn;
  }
}

// Row of the 30-channel first layer that per-element channel c (0..15) of a factored tensor uses:
// {0, 2..13, 27, 28, 29}.
__device__ __forceinline__ int adafac_elem_row(int c) { return c == 0 ? 0 : (c <= 12 ? c + 1 : c + 14); }

// The apply pass over one wave task of the column-resident walk (one column per lane).  The
// 16 -> 32 -> 32 -> 2 element MLP runs as v_mfma_f32_16x16x4_f32 products with the *elements* as the
// N dimension: D(16 units x 16 elements) += A(16 units x 4 inputs) B(4 inputs x 16 elements).
// Operand layouts (lane = 16 q + e): A holds unit e, input q; B holds input q of element e; D holds
// units 4q..4q+3 of element e.  The D layout of one layer is a valid B layout of the next (input
// slot (q, r) = unit 16 b + 4 q + r), so activations never move between lanes; only the 16 features
// of the 64 elements a wave holds (one element per lane) are regrouped once per row through LDS
// into four groups of 16 elements.  Per row of 64 elements: 32 + 64 MFMAs for the two layers; the
// output layer's per-lane partial products are summed over q with two cross-lane moves each.
// 1 536 matrix FMAs + 64 VALU FMAs per element, bound by the fp32 matrix rate.
// Row pitch of the feature exchange buffer: 64 elements plus 16 floats, so that the four lane groups
// of a read (rows 4c'+q, q = 0..3, same 16 columns) fall into different LDS banks; with a pitch of 64
// they collided and every read took twice as long.
constexpr int kXPitch = 80;
__device__ __forceinline__ v4f mfma16(float a, float b, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void adafac_apply_tile(const TDesc& d, const PyloTensorArgs& a, int task,
                                                  const EmaConsts& e, const float* __restrict__ fac_tab,
                                                  const float* __restrict__ term_tab, const float* wfold_t,
                                                  const float* net, float* xch /* LDS [16][kXPitch] of this wave */) {
  const TileTask tk(d, task, d.atile_nct, 1);
  const int lane = threadIdx.x & 63, q = lane >> 4, el = lane & 15;
  // A operands: first layer [b][c'] (inputs 4c'+q), hidden layer [bo][b][r] (input 16b+4q+r)
  float a1[2][4], a2[2][2][4], wo[2][4][2];
  v4f bh[2];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
      a1[b][c] = *(const gfloat*)(wfold_t + adafac_elem_row(4 * c + q) * kAH + 16 * b + el);
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
#pragma unroll
      for (int r = 0; r < 4; ++r) a2[b][bi][r] = *(const gfloat*)(net + kAWH + (16 * bi + 4 * q + r) * kAH + 16 * b + el);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      bh[b][r] = *(const gfloat*)(net + kABH + 16 * b + 4 * q + r);
      wo[b][r][0] = *(const gfloat*)(net + kAWO + (16 * b + 4 * q + r) * 2 + 0);
      wo[b][r][1] = *(const gfloat*)(net + kAWO + (16 * b + 4 * q + r) * 2 + 1);
    }
  }
  const cfloat* nw = launder(net);
  const float bo0 = nw[kABO + 0], bo1 = nw[kABO + 1];
  const float exp_scale = a.exp_mult * 1.44269504088896341f;
  float fb[4];
  load_vec_o<4>(fac_tab + d.fac_off[1], tk.col * 16u, fb);
  // column terms of element (16 g + el), units 16 b + 4 q ..: one voffset, immediates per (g, b)
  const float* tcol = term_tab + d.term_off[1];
  const unsigned tcol_off = ((tk.col - lane + el) * kAH + 4 * q) * 4u;
  const unsigned trow_off = 4 * q * 4u;
  const unsigned lo = lane * 4u;
  float* xw = xch + lane;                 // feature c of this lane's element goes to xch[c][lane]
  const float* xr = xch + q * kXPitch + el;  // input 4c'+q of element 16g+el is xch[4c'+q][16g+el]
  const float* g = a.grad + tk.first;
  float *p = a.param + tk.first, *m0 = a.mom + tk.first, *m1 = a.mom + d.n + tk.first,
        *m2 = a.mom + 2 * d.n + tk.first, *rms = a.rms + tk.first;
  const float* fr = fac_tab + d.fac_off[0] + (size_t)tk.r0 * 4;
  const float* tr = term_tab + d.term_off[0] + (size_t)tk.r0 * kAH;
  for (int r = tk.r0; r < tk.r1; ++r) {
    float xg[1], xp[1], x0[1], x1[1], x2[1], xr_[1], fa[4];
    load_vec_nt<1>(g, lo, xg);
    load_vec_nt<1>(p, lo, xp);
    load_vec_nt<1>(m0, lo, x0);
    load_vec_nt<1>(m1, lo, x1);
    load_vec_nt<1>(m2, lo, x2);
    load_vec_nt<1>(rms, lo, xr_);
    load_uniform<4>(fr, fa);
    float ta[2][4];
#pragma unroll
    for (int b = 0; b < 2; ++b) load_vec_o<4>(tr + 16 * b, trow_off, ta[b]);
    const float gg = cond_grad(xg[0], d.gscale, a.clip_val, d.nan0);
    float m[3] = {x0[0], x1[0], x2[0]};
    ema_update(e, gg, m, xr_[0]);
    x0[0] = m[0]; x1[0] = m[1]; x2[0] = m[2];
    store_vec_nt<1>(m0, lo, x0);
    store_vec_nt<1>(m1, lo, x1);
    store_vec_nt<1>(m2, lo, x2);
    store_vec_nt<1>(rms, lo, xr_);
    const float rfcf[3] = {fa[0] * fb[0], fa[1] * fb[1], fa[2] * fb[2]};
    float f18[kNStat];
    lo_features(gg, xp[0], m, xr_[0], rfcf, 1e-6f, f18);
    const float f[16] = {f18[0], f18[2], f18[3], f18[4], f18[5], f18[6], f18[7], f18[8], f18[9], f18[10],
                         f18[11], f18[12], f18[13], f18[15], f18[16], f18[17]};
#pragma unroll
    for (int c = 0; c < 16; ++c) xw[c * kXPitch] = f[c];
    float o0 = 0.0f, o1 = 0.0f;
    // two groups of 16 elements at a time: four independent accumulator chains
#pragma unroll
    for (int gP = 0; gP < 4; gP += 2) {
      v4f h[2][2], g2[2][2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          float tb[4];
          load_vec_o<4>(tcol + (16 * (gP + u)) * kAH + 16 * b, tcol_off, tb);
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) h[u][b][rr] = ta[b][rr] + tb[rr];
        }
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const float bv = xr[(4 * c) * kXPitch + 16 * (gP + u)];
          h[u][0] = mfma16(a1[0][c], bv, h[u][0]);
          h[u][1] = mfma16(a1[1][c], bv, h[u][1]);
        }
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) { g2[u][0] = bh[0]; g2[u][1] = bh[1]; }
#pragma unroll
      for (int bi = 0; bi < 2; ++bi) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const float hv = relu(h[u][bi][rr]);
            g2[u][0] = mfma16(a2[0][bi][rr], hv, g2[u][0]);
            g2[u][1] = mfma16(a2[1][bi][rr], hv, g2[u][1]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float p0 = 0.0f, p1 = 0.0f;
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const float gv = relu(g2[u][b][rr]);
            p0 = fmaf(gv, wo[b][rr][0], p0);
            p1 = fmaf(gv, wo[b][rr][1], p1);
          }
        }
        // sum of the per-lane partial products over the four lane groups q (lanes el, el+16, el+32, el+48)
        p0 += __shfl_xor(p0, 16, 64);
        p1 += __shfl_xor(p1, 16, 64);
        p0 += __shfl_xor(p0, 32, 64);
        p1 += __shfl_xor(p1, 32, 64);
        if (q == gP + u) { o0 = p0; o1 = p1; }
      }
    }
    o0 += bo0;
    o1 += bo1;
    float pn[1];
    pn[0] = adafac_update(d, a, o0 * __builtin_amdgcn_exp2f(o1 * exp_scale), xp[0]);
    store_vec_o<1>(p, lo, pn);
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0;
    fr += 4; tr += kAH;
  }
}

// ---- the same pass with the element MLP on the fp16 matrix instructions at fp32 accuracy ----------------
// An fp32 number within fp16's range is, to 2^-23 of its size, the sum of two fp16 numbers taken by rounding
// (h = fp16(x), l = fp16(x - h): v_cvt_pk_f16_f32 converts and packs two values in one instruction), and a product
// of two such sums is the three products h h, h l, l h, each exact in fp32, plus l l (2^-24 of |x y|), which is
// dropped with the remainders: about 2^-22 of a product, unbiased -- below the rounding of the fp32 accumulation.
// Range: fp16 ends at 65 504 and resolves 6e-8 absolutely at its lower end, so the operands must be of order one.
// The hidden values and the weights are; the raw features are not (a second moment of 1e-12 next to its
// reciprocal root of 1e6), which is why this variant does not use the first-layer rows folded with the channel
// normalisers: it multiplies each feature by its normaliser (unit second moment over the tensor afterwards, so
// no feature exceeds sqrt(n) < 46 341 in a tensor of n < 2^31 elements; sixteen multiplications an element) and
// takes the first layer's rows as they are.  The hidden values are clamped at 65 000 by the instruction that is
// their ReLU anyway (one as large takes normalised features of 1e4 and more, i.e. a single outlier in a tensor
// of 1e8 elements).
// Three v_mfma_f32_32x32x16_f16 per fp32 product leave 18 matrix instructions per row of 64 elements where the
// fp32 instructions need 96 and three bf16 planes needed 36; the split costs 3.25 vector instructions a value
// (two conversions and a subtraction per value, a packing conversion per pair and plane) where three bf16
// planes cost 5.5, in a kernel that is bound by exactly these instructions: splitting the 16 features and the
// 2 x 16 hidden values a lane holds.
//
// Layouts (lane = 32 half + e): units are the M dimension, elements the N dimension, inputs the K
// dimension.  A operand: lane holds reduction slots 8 half .. 8 half + 7 of unit e.  B operand: lane holds
// slots 8 half .. + 7 of element e of the group (two groups of 32 elements per wave row; a lane owns element
// 32 half + e, i.e. the lanes of one half own one group).  D: lane holds units 8 j + 4 half + i (j, i = 0..3)
// of element e.
// First layer: slot = input.  A lane has all 16 features of its own element and needs, per group, half of the
// features of element e of that group: lanes e and e + 32 trade the halves the other needs, eight
// v_permlane32_swap on the fp32 values (lanes 32..63 of the first operand change places with lanes 0..31 of the
// second), before the split.
// Hidden layer: which hidden unit a reduction slot stands for is free as long as both operands agree, so slot
// 8 half + 4 q + i of step s is unit 8 (2 s + q) + 4 half + i: exactly the sixteen units the lane holds in D
// after the first layer.  The hidden values never leave their lane; nothing goes through LDS.
typedef _Float16 ah16x8 __attribute__((ext_vector_type(8)));
typedef float av16f __attribute__((ext_vector_type(16)));
typedef unsigned int au32x4 __attribute__((ext_vector_type(4)));

// two values -> one dword of each plane (`a` in the lower halves), by rounding (v_cvt_pk_f16_f32)
typedef float af32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 ah16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void hf2_split2(float a, float b, unsigned& h, unsigned& l) {
  const ah16x2 hh = __builtin_convertvector(af32x2{a, b}, ah16x2);
  const ah16x2 ll = __builtin_convertvector(af32x2{a - (float)hh[0], b - (float)hh[1]}, ah16x2);
  h = __builtin_bit_cast(unsigned, hh);
  l = __builtin_bit_cast(unsigned, ll);
}

// eight values (consecutive inputs of a matrix operand) as two planes of eight fp16
__device__ __forceinline__ void hf2_pack8(const float (&x)[8], au32x4 (&pl)[2]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    unsigned h, l;
    hf2_split2(x[2 * i], x[2 * i + 1], h, l);
    pl[0][i] = h;
    pl[1][i] = l;
  }
}

// lanes 32..63 of `a` change places with lanes 0..31 of `b`
__device__ __forceinline__ void half_swap(unsigned& a, unsigned& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}

// acc += W (two planes) x act (two planes), smallest terms first
__device__ __forceinline__ av16f hf2_mfma(const au32x4 (&w)[2], const au32x4 (&x)[2], av16f acc) {
  constexpr int pw[3] = {1, 0, 0}, px[3] = {0, 1, 0};
#pragma unroll
  for (int t = 0; t < 3; ++t)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(ah16x8, w[pw[t]]), __builtin_bit_cast(ah16x8, x[px[t]]),
                                                 acc, 0, 0, 0);
  return acc;
}

// PER: the tensor is an (O, I, k, ..) one walked as the matrix (O, I * P) (TDesc::aper): the vector that is not
// indexed by the column has an entry per (row, column mod P), so a lane fetches the row's factor and first-layer
// terms for its own columns (one per element group) instead of sharing one entry with the wave.
template <bool PER>
__device__ __forceinline__ void adafac_apply_tile_hf(const TDesc& d, const PyloTensorArgs& a, int task,
                                                     const EmaConsts& e, const float* __restrict__ fac_tab,
                                                     const float* __restrict__ term_tab, const float* wfold_t,
                                                     const float* net) {
  const TileTask tk(d, task, d.atile_nct, 1);
  const int lane = threadIdx.x & 63, half = lane >> 5, el = lane & 31;
  // A operands: first layer (unit el, inputs 8 half ..), hidden layer per reduction step s (slot 8 half + 4 q + i:
  // hidden unit 8 (2 s + q) + 4 half + i)
  au32x4 w1[2], w2[2][2];
  {
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = *(const gfloat*)(net + kAW1 + adafac_elem_row(8 * half + i) * kAH + el);
    hf2_pack8(x, w1);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        x[i] = *(const gfloat*)(net + kAWH + (8 * (2 * s + (i >> 2)) + 4 * half + (i & 3)) * kAH + el);
      hf2_pack8(x, w2[s]);
    }
  }
  // the normalisers of the sixteen features an element brings itself (the first layer's rows are not folded here)
  float fsc[16];
  {
    const cfloat* sc = launder(wfold_t + 30 * kAH);
#pragma unroll
    for (int c = 0; c < 16; ++c) fsc[c] = sc[adafac_elem_row(c)];
  }
  // what belongs to the units this lane holds in D: hidden bias, output weights
  av16f bh;
  float wo[16][2];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int unit = 8 * (r >> 2) + 4 * half + (r & 3);
    bh[r] = *(const gfloat*)(net + kABH + unit);
    wo[r][0] = *(const gfloat*)(net + kAWO + unit * 2 + 0);
    wo[r][1] = *(const gfloat*)(net + kAWO + unit * 2 + 1);
  }
  const cfloat* nw = launder(net);
  const float bo0 = nw[kABO + 0], bo1 = nw[kABO + 1];
  const float exp_scale = a.exp_mult * 1.44269504088896341f;
  const int cv = PER ? d.aper_col : 1, pv = 1 - cv;   // the vector the column indexes, and the other one
  const int per = PER ? d.aper : 1;
  float fb[4];
  load_vec_o<4>(fac_tab + pick(d.fac_off, cv), tk.col * 16u, fb);
  // column terms of element e of group g (column: the wave's first + 32 g + e), units 8 j + 4 half ..: one
  // offset per lane, immediates per (g, j); row terms likewise from the row's table entry
  const float* tcol = term_tab + pick(d.term_off, cv);
  const unsigned tcol_off = ((tk.col - lane + el) * kAH + 4 * half) * 4u;
  // row side: byte offsets of the lane's entries relative to the row's first (zero unless PER)
  unsigned fa_off = 0, trow_off[2] = {4 * half * 4u, 4 * half * 4u};
  if constexpr (PER) {
    fa_off = (tk.col % (unsigned)per) * 16u;
#pragma unroll
    for (int gq = 0; gq < 2; ++gq) trow_off[gq] += ((tk.col - lane + 32 * gq + el) % (unsigned)per) * (kAH * 4u);
  }
  const unsigned lo = lane * 4u;
  const float* g = a.grad + tk.first;
  float *p = a.param + tk.first, *m0 = a.mom + tk.first, *m1 = a.mom + d.n + tk.first,
        *m2 = a.mom + 2 * d.n + tk.first, *rms = a.rms + tk.first;
  const float* fr = fac_tab + pick(d.fac_off, pv) + (size_t)tk.r0 * 4 * per;
  const float* tr = term_tab + pick(d.term_off, pv) + (size_t)tk.r0 * kAH * per;
  // Everything a row reads from memory.  The loop keeps one row in flight: the loads of row r + 1 are issued
  // before row r is worked on (a wave shares its SIMD with one other wave only, too few to cover a memory round
  // trip per row otherwise).
  struct RowIn { float g[1], p[1], m0[1], m1[1], m2[1], rms[1], fa[4], ta[PER ? 2 : 1][4][4]; };
  auto fetch = [&](RowIn& x, long long eo, const float* fr_, const float* tr_) {
    load_vec_nt<1>(g + eo, lo, x.g);
    load_vec_nt<1>(p + eo, lo, x.p);
    load_vec_nt<1>(m0 + eo, lo, x.m0);
    load_vec_nt<1>(m1 + eo, lo, x.m1);
    load_vec_nt<1>(m2 + eo, lo, x.m2);
    load_vec_nt<1>(rms + eo, lo, x.rms);
    if constexpr (PER) load_vec_o<4>(fr_, fa_off, x.fa);
    else load_uniform<4>(fr_, x.fa);
#pragma unroll
    for (int gq = 0; gq < (PER ? 2 : 1); ++gq)
#pragma unroll
      for (int j = 0; j < 4; ++j) load_vec_o<4>(tr_ + 8 * j, trow_off[gq], x.ta[gq][j]);
  };
  RowIn cur;
  fetch(cur, 0, fr, tr);
  for (int r = tk.r0; r < tk.r1; ++r) {
    RowIn nxt;
    {   // past the last row: the same row again, discarded
      const bool more = r + 1 < tk.r1;
      fetch(nxt, more ? d.C0 : 0, fr + (more ? 4 * per : 0), tr + (more ? kAH * per : 0));
    }
    float xg[1] = {cur.g[0]}, xp[1] = {cur.p[0]}, x0[1] = {cur.m0[0]}, x1[1] = {cur.m1[0]}, x2[1] = {cur.m2[0]},
          xr_[1] = {cur.rms[0]};
    const float (&fa)[4] = cur.fa;
    const float (&ta)[PER ? 2 : 1][4][4] = cur.ta;
    const float gg = cond_grad(xg[0], d.gscale, a.clip_val, d.nan0);
    float m[3] = {x0[0], x1[0], x2[0]};
    ema_update(e, gg, m, xr_[0]);
    x0[0] = m[0]; x1[0] = m[1]; x2[0] = m[2];
    store_vec_nt<1>(m0, lo, x0);
    store_vec_nt<1>(m1, lo, x1);
    store_vec_nt<1>(m2, lo, x2);
    store_vec_nt<1>(rms, lo, xr_);
    const float rfcf[3] = {fa[0] * fb[0], fa[1] * fb[1], fa[2] * fb[2]};
    float f18[kNStat];
    lo_features(gg, xp[0], m, xr_[0], rfcf, 1e-6f, f18);
    float flo[8] = {f18[0], f18[2], f18[3], f18[4], f18[5], f18[6], f18[7], f18[8]};
    float fhi[8] = {f18[9], f18[10], f18[11], f18[12], f18[13], f18[15], f18[16], f18[17]};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      flo[i] *= fsc[i];
      fhi[i] *= fsc[8 + i];
    }
    // B operands of the first layer: after the swap flo serves group 0 (lanes 0..31: their own inputs 0..7,
    // lanes 32..63: inputs 8..15 of the element 32 lanes below), fhi group 1
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      unsigned u = __float_as_uint(flo[i]), v = __float_as_uint(fhi[i]);
      half_swap(u, v);
      flo[i] = __uint_as_float(u);
      fhi[i] = __uint_as_float(v);
    }
    au32x4 xb[2][2];
    hf2_pack8(flo, xb[0]);
    hf2_pack8(fhi, xb[1]);
    // The two groups of 32 elements go through the layers a phase apart, so that the matrix instructions of one
    // have the vector work of the other to run under: first layer of both, then per group split -> hidden layer,
    // then the output layer (on the vector pipe) of both.
    av16f h[2];
#pragma unroll
    for (int gq = 0; gq < 2; ++gq) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float tb[4];
        load_vec_o<4>(tcol + (32 * gq) * kAH + 8 * j, tcol_off, tb);
#pragma unroll
        for (int i = 0; i < 4; ++i) h[gq][4 * j + i] = ta[PER ? gq : 0][j][i] + tb[i];
      }
      h[gq] = hf2_mfma(w1, xb[gq], h[gq]);
    }
    av16f g2[2];
#pragma unroll
    for (int gq = 0; gq < 2; ++gq) {
      // hidden values of the units this lane holds -> planes, four units (two dwords) per block j
      unsigned hp[2][4][2];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i)
          hf2_split2(__builtin_amdgcn_fmed3f(h[gq][4 * j + 2 * i], 0.0f, 65000.0f),
                     __builtin_amdgcn_fmed3f(h[gq][4 * j + 2 * i + 1], 0.0f, 65000.0f), hp[0][j][i], hp[1][j][i]);
      // blocks 2 s and 2 s + 1 are the lane's eight slots of reduction step s as they stand
      g2[gq] = bh;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        au32x4 hb[2];
#pragma unroll
        for (int q = 0; q < 2; ++q)
          hb[q] = au32x4{hp[q][2 * s2][0], hp[q][2 * s2][1], hp[q][2 * s2 + 1][0], hp[q][2 * s2 + 1][1]};
        g2[gq] = hf2_mfma(w2[s2], hb, g2[gq]);
      }
    }
    float part[2][2];
#pragma unroll
    for (int gq = 0; gq < 2; ++gq) {
      float p0 = 0.0f, p1 = 0.0f;
#pragma unroll
      for (int r2 = 0; r2 < 16; ++r2) {
        const float gv = relu(g2[gq][r2]);
        p0 = fmaf(gv, wo[r2][0], p0);
        p1 = fmaf(gv, wo[r2][1], p1);
      }
      part[gq][0] = p0;
      part[gq][1] = p1;
    }
    // a lane's element belongs to group `half`; its other 16 units sit 32 lanes away
    unsigned a0 = __float_as_uint(part[0][0]), b0 = __float_as_uint(part[1][0]);
    unsigned a1 = __float_as_uint(part[0][1]), b1 = __float_as_uint(part[1][1]);
    half_swap(a0, b0);
    half_swap(a1, b1);
    const float o0 = (__uint_as_float(a0) + __uint_as_float(b0)) + bo0;
    const float o1 = (__uint_as_float(a1) + __uint_as_float(b1)) + bo1;
    float pn[1];
    pn[0] = adafac_update(d, a, o0 * __builtin_amdgcn_exp2f(o1 * exp_scale), xp[0]);
    store_vec_o<1>(p, lo, pn);
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0;
    fr += 4 * per; tr += kAH * per;
    cur = nxt;
  }
}

__global__ __launch_bounds__(kThreads) void k_adafac_apply(const TDesc* __restrict__ descs,
                                                           const PyloTensorArgs* __restrict__ dyn,
                                                           const Item* __restrict__ items,
                                                           const float* __restrict__ fac_tab,
                                                           const float* __restrict__ term_tab, PyloDecays dec,
                                                           const float* __restrict__ wfold,
                                                           const float* __restrict__ net,
                                                           const float* __restrict__ bias_eff,
                                                           const Globals* __restrict__ gl) {
  const Item it = items[blockIdx.x];
  TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  set_grad_scale(d, a, gl, it.tensor);
  const EmaConsts e = make_ema(dec);
  const float* w = wfold + (size_t)it.tensor * kAFold;
  const long long count = (long long)kThreads * d.vec * kElemIters;
  const long long base = (long long)it.a * count;
  if (d.mode == kModeFac2D) adafac_apply_fac<false>(d, a, base, count, e, fac_tab, term_tab, w, net);
  else if (d.mode == kModeFacND) adafac_apply_fac<true>(d, a, base, count, e, fac_tab, term_tab, w, net);
  else adafac_apply_vec(d, a, base, count, e, dec, w, net, bias_eff + (size_t)it.tensor * kAH);
}

// The apply pass for tensors walked column-resident (items hold four wave tasks each).  BF: the element MLP on
// the fp16 matrix instructions (two-plane operands), else on the fp32 ones.
template <bool BF, bool PER = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(BF ? 2 : PYLO_ADAFAC_WAVES)))
void k_adafac_apply_tile(const TDesc* __restrict__ descs, const PyloTensorArgs* __restrict__ dyn,
                         const Item* __restrict__ items, const float* __restrict__ fac_tab,
                         const float* __restrict__ term_tab, PyloDecays dec, const float* __restrict__ wfold,
                         const float* __restrict__ net, const Globals* __restrict__ gl) {
  const Item it = items[blockIdx.x];
  TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  set_grad_scale(d, a, gl, it.tensor);
  __shared__ float xch[BF ? 1 : kWaves][BF ? 1 : 16 * kXPitch];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int task = it.a * 4 + wave;
  if (task >= d.atile_ntask) return;
  static_assert(BF || !PER, "tensors with more than two dims are walked by the fp16 variant only");
  if constexpr (BF)
    adafac_apply_tile_hf<PER>(d, a, task, make_ema(dec), fac_tab, term_tab, wfold + (size_t)it.tensor * kAFold, net);
  else
    adafac_apply_tile(d, a, task, make_ema(dec), fac_tab, term_tab, wfold + (size_t)it.tensor * kAFold, net, xch[wave]);
}

}  // namespace pylo
