// VeLO: element kernels (statistics / apply for factored 2-D, factored N-D and non-factored
// tensors), the per-tensor reduction with the LSTM input features, and the per-tensor LSTM that
// emits each tensor's MLP weights.
#pragma once

#include "k_celo2.h"
#include "k_gradstats.h"
#include "pylo_common.h"

namespace pylo {

// Folded per-tensor weights (floats): first layer rows scaled by the channel normalisers
// (18 per-element rows for factored tensors, all 30 rows for non-factored ones), (in, out).
// W1 (30,4) | b1 4 | WH (4,4) | bH 4 | WO (4,4: two outputs, two zeros) | bO 4 (same padding) |
// param_scale | lr_mult; padded to three 64-float registers for the matrix-pipe path
constexpr int kVW1 = 0, kVB1 = 120, kVWH = 124, kVBH = 140, kVWO = 144, kVBO = 160, kVPS = 164, kVLR = 165,
              kVFold = 192;
constexpr int kVCanon = 128;   // per-tensor un-scaled first layer (30,4) + bias 4, for k_terms
constexpr int kVBank = 159;    // floats per bank entry: W_in (4,30) | b_in 4 | W_h (4,4) | b_h 4 | W_out (3,4) | b_out 3
constexpr int kXW = 32;        // row pitch of the LSTM input features (30 used)
constexpr int kGateBT = 8;     // tensors per k_velo_gates block

struct LossState {             // by-value kernel argument: the caller's loss accumulators (PyloVeloStep)
  float* means;
  float* running_min;
  const float* decays;
  int* iteration;
  const float* loss;
};

struct VeloStep {              // by-value kernel argument: scalars of one step
  float frac[PYLO_MAX_GROUPS][9];
  const float* frac_dev;       // the same table in device memory when the step counters live there, else null
};

// ---------------------------------------------------------------------------------------------
// element access for factored tensors, 2-D fast path (V consecutive elements of one row) or
// generic N-D (V == 1)
// ---------------------------------------------------------------------------------------------
template <int V, bool ND>
__device__ __forceinline__ void lo_load(const TDesc& d, const PyloTensorArgs& a, long long idx,
                                        const float* __restrict__ fac_tab, ElemIn<V>& x) {
  if constexpr (!ND) {
    load_elems<V>(d, a, idx, d.gscale, fac_tab + d.fac_off[0], fac_tab + d.fac_off[1], x);
  } else {
    const long long n = d.n;
    x.g[0] = cond_grad(*(const gfloat*)(a.grad + idx), d.gscale, a.clip_val, d.nan0);
    x.p[0] = *(const gfloat*)(a.param + idx);
    x.m[0][0] = *(const gfloat*)(a.mom + idx);
    x.m[0][1] = *(const gfloat*)(a.mom + n + idx);
    x.m[0][2] = *(const gfloat*)(a.mom + 2 * n + idx);
    x.rms[0] = *(const gfloat*)(a.rms + idx);
    const unsigned u = (unsigned)idx;
    const unsigned s0 = (unsigned)d.nd_stride[0], s1 = (unsigned)d.nd_stride[1];
    x.i0 = (int)(fd_div(u, d.nd_div_blk[0]) * s0 + (u - fd_div(u, d.nd_div_st[0]) * s0));
    x.i1 = (int)(fd_div(u, d.nd_div_blk[1]) * s1 + (u - fd_div(u, d.nd_div_st[1]) * s1));
    const float4 fa = load_f4(fac_tab + d.fac_off[0] + (size_t)x.i0 * 4);
    const float4 fb = load_f4(fac_tab + d.fac_off[1] + (size_t)x.i1 * 4);
    x.rfcf[0][0] = fa.x * fb.x;
    x.rfcf[0][1] = fa.y * fb.y;
    x.rfcf[0][2] = fa.z * fb.z;
  }
}

// h[v][j] = term0[j] + term1[j] of the element's row / column
template <int V, bool ND, int H>
__device__ __forceinline__ void lo_terms(const TDesc& d, const ElemIn<V>& x, const float* __restrict__ term_tab,
                                         float (&h)[V][H]) {
  if constexpr (!ND) {
    static_assert(H % 4 == 0, "term tables are read four floats at a time");
    const float* t0 = term_tab + d.term_off[0] + (size_t)x.i0 * H;
    const float* t1 = term_tab + d.term_off[1] + (size_t)x.i1 * H;
#pragma unroll
    for (int q = 0; q < H / 4; ++q) {
      const float4 ta = load_f4(t0 + q * 4);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float4 tb = load_f4(t1 + v * H + q * 4);
        h[v][q * 4 + 0] = ta.x + tb.x; h[v][q * 4 + 1] = ta.y + tb.y;
        h[v][q * 4 + 2] = ta.z + tb.z; h[v][q * 4 + 3] = ta.w + tb.w;
      }
    }
  } else {
    static_assert(H % 4 == 0, "term tables are read four floats at a time");
    const float* t0 = term_tab + d.term_off[0] + (size_t)x.i0 * H;
    const float* t1 = term_tab + d.term_off[1] + (size_t)x.i1 * H;
#pragma unroll
    for (int q = 0; q < H / 4; ++q) {
      const float4 ta = load_f4(t0 + q * 4), tb = load_f4(t1 + q * 4);
      h[0][q * 4 + 0] = ta.x + tb.x; h[0][q * 4 + 1] = ta.y + tb.y;
      h[0][q * 4 + 2] = ta.z + tb.z; h[0][q * 4 + 3] = ta.w + tb.w;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// statistics pass
// ---------------------------------------------------------------------------------------------
struct VeloAcc {
  float ch[30];   // sum of squares per channel (factored tensors fill the 18 per-element ones)
  // The LSTM's variance features are taken over the accumulators before the update.  Their sums are
  // shifted by a pivot per tensor (its first element): sum (m_k - c_k), sum (m_k - c_k)^2, sum (rms - c_r),
  // sum (rms - c_r)^2.  Plain sums of m and m^2 cancel catastrophically where the spread is small
  // against the mean -- a one-element tensor has variance exactly 0 in the reference, and the rounding
  // of its m^2, scaled by 1 / mean p^2, used to land far above the feature's clamp at exp(-5).
  float lstm[8];
  float piv[4];   // c_0, c_1, c_2, c_r
};

// First element of each accumulator of a tensor (0 for an empty one); the same for every block.
__device__ __forceinline__ void lstm_pivots(const TDesc& d, const PyloTensorArgs& a, float (&piv)[4]) {
  if (d.n > 0) {
    piv[0] = *(const gfloat*)(a.mom);
    piv[1] = *(const gfloat*)(a.mom + d.n);
    piv[2] = *(const gfloat*)(a.mom + 2 * d.n);
    piv[3] = *(const gfloat*)(a.rms);
  } else {
    piv[0] = piv[1] = piv[2] = piv[3] = 0.0f;
  }
}

// What the apply pass adds up over the values it WRITES, for the LSTM features of the next step (they are
// that step's "accumulators before the update"): sum p^2, then the shifted sums as in VeloAcc::lstm.  The
// pivots are the tensor's first elements AFTER this step's update -- what the next step finds there --
// which every block derives for itself from the first elements before the update (kept per tensor by the
// kernel that formed the LSTM's inputs, since the apply pass overwrites them while it runs) and the
// tensor's first gradient element; they are wave-uniform and live in scalar registers.
constexpr int kNewSumW = 10;    // doubles per row of those partial sums (9 used)
struct NewSums {
  float v[9];
  float piv[4];
  __device__ __forceinline__ void clear(const TDesc& d, const PyloTensorArgs& a, const EmaConsts& e,
                                        const float* __restrict__ old_first) {
#pragma unroll
    for (int c = 0; c < 9; ++c) v[c] = 0.0f;
    float of[4];
    load_uniform<4>(old_first, of);
    const float g0 = d.n > 0 ? cond_grad(*(const cfloat*)a.grad, d.gscale, a.clip_val, d.nan0) : 0.0f;
    float m[3] = {of[0], of[1], of[2]};
    float r = of[3];
    ema_update(e, g0, m, r);
    auto uniform = [](float x) {   // the value is the same in every lane: keep it in a scalar register
      return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
    };
    piv[0] = uniform(m[0]);
    piv[1] = uniform(m[1]);
    piv[2] = uniform(m[2]);
    piv[3] = uniform(r);
  }
  __device__ __forceinline__ void add(float p_new, const float (&m)[3], float rms) {
    v[0] = fmaf(p_new, p_new, v[0]);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const float dm = m[k] - piv[k];
      v[1 + k] += dm;
      v[4 + k] = fmaf(dm, dm, v[4 + k]);
    }
    const float dr = rms - piv[3];
    v[7] += dr;
    v[8] = fmaf(dr, dr, v[8]);
  }
};

__device__ __forceinline__ void lstm_sums(const float (&m)[3], float rms, VeloAcc& acc) {
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const float dm = m[k] - acc.piv[k];
    acc.lstm[k] += dm;
    acc.lstm[3 + k] = fmaf(dm, dm, acc.lstm[3 + k]);
  }
  const float dr = rms - acc.piv[3];
  acc.lstm[6] += dr;
  acc.lstm[7] = fmaf(dr, dr, acc.lstm[7]);
}

template <int V, bool ND>
__device__ __forceinline__ void velo_stats_fac(const TDesc& d, const PyloTensorArgs& a, int chunk,
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
      lstm_sums(x.m[v], x.rms[v], acc);
      ema_update(e, x.g[v], x.m[v], x.rms[v]);
      float f[kNStat];
      lo_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.rfcf[v], 1e-6f, f);
#pragma unroll
      for (int c = 0; c < kNStat; ++c) acc.ch[stat_channel(c)] = fmaf(f[c], f[c], acc.ch[stat_channel(c)]);
    }
  }
}

// Column-resident walk of one wave task (wide 2-D tensors): column factors in registers, row
// factors through the scalar cache, six streams per row.
// KEEP: plain loads, which leave the lines in the memory-side cache for the apply items that follow
// (k_velo_elem); otherwise non-temporal loads (see celo2_stats_tile).
template <bool KEEP>
__device__ __forceinline__ void velo_stats_tile(const TDesc& d, const PyloTensorArgs& a, int task,
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
    if constexpr (KEEP) {
      load_vec_o<V>(g, lo, xg);
      load_vec_o<V>(p, lo, xp);
      load_vec_o<V>(m0, lo, x0);
      load_vec_o<V>(m1, lo, x1);
      load_vec_o<V>(m2, lo, x2);
      load_vec_o<V>(rms, lo, xr);
    } else {
      load_vec_nt<V>(g, lo, xg);
      load_vec_nt<V>(p, lo, xp);
      load_vec_nt<V>(m0, lo, x0);
      load_vec_nt<V>(m1, lo, x1);
      load_vec_nt<V>(m2, lo, x2);
      load_vec_nt<V>(rms, lo, xr);
    }
    load_uniform<4>(fr, fa);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const float gg = clampf(xg[v], a.clip_val);
      float m[3] = {x0[v], x1[v], x2[v]};
      float rr = xr[v];
      lstm_sums(m, rr, acc);
      ema_update(e, gg, m, rr);
      const float rfcf[3] = {fa[0] * fb[v][0], fa[1] * fb[v][1], fa[2] * fb[v][2]};
      float f[kNStat];
      lo_features(gg, xp[v], m, rr, rfcf, 1e-6f, f);
#pragma unroll
      for (int c = 0; c < kNStat; ++c) acc.ch[stat_channel(c)] = fmaf(f[c], f[c], acc.ch[stat_channel(c)]);
    }
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0; fr += 4;
  }
}

// Non-factored tensor: the 30 channels of one element (Velo_naive.py:60-68,439-451,478-488).
// m, rms, v are the accumulators after this step's update; fm_eps is added to v under the
// power -1/2 of the last group (0 for VeLO, 1e-6 for AdafacLO).
__device__ __forceinline__ void vec_features(float g, float p, const float (&m)[3], float rms,
                                             const float (&v)[3], float fm_eps, float (&f)[30]) {
  const float rs = rsq(rms + 1e-6f);
  f[0] = g;
  f[1] = fminf(fmaxf(g, -0.1f), 0.1f);
  f[2] = p;
  f[6] = rms;
  f[10] = rs;
  f[14] = g * rs;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    f[3 + k] = m[k];
    f[7 + k] = m[k] * rs;
    f[11 + k] = g * rsq(fmaxf(v[k] + 1e-9f, 1e-9f));
    f[15 + k] = v[k];
    f[18 + k] = v[k];
    const float q = rsq(v[k] + 1e-8f);
    f[21 + k] = q;
    f[24 + k] = q;
    f[27 + k] = m[k] * rsq(v[k] + fm_eps);
  }
}

template <int V>
struct VecIn {
  float g[V], p[V], m[V][3], rms[V], v[V][3];
};

template <int V>
__device__ __forceinline__ void vec_load(const TDesc& d, const PyloTensorArgs& a, long long idx, VecIn<V>& x) {
  const long long n = d.n;
  float t[3][V], u[3][V];
  load_vec<V>(a.grad + idx, x.g);
  load_vec<V>(a.param + idx, x.p);
  load_vec<V>(a.rms + idx, x.rms);
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    load_vec<V>(a.mom + k * n + idx, t[k]);
    load_vec<V>(a.fac_v + k * n + idx, u[k]);
  }
#pragma unroll
  for (int v = 0; v < V; ++v) {
    x.g[v] = cond_grad(x.g[v], d.gscale, a.clip_val, d.nan0);
#pragma unroll
    for (int k = 0; k < 3; ++k) { x.m[v][k] = t[k][v]; x.v[v][k] = u[k][v]; }
  }
}

__device__ __forceinline__ void vec_update(const EmaConsts& e, const PyloDecays& dec, float g, float (&m)[3],
                                           float& rms, float (&v)[3]) {
  ema_update(e, g, m, rms);
  const float q = g * g + 1e-30f;
#pragma unroll
  for (int k = 0; k < 3; ++k) v[k] = dec.beta_fac[k] * v[k] + (1.0f - dec.beta_fac[k]) * q;
}

template <int V>
__device__ __forceinline__ void velo_stats_vec(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                               const EmaConsts& e, const PyloDecays& dec, VeloAcc& acc) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= d.n) break;
    VecIn<V> x;
    vec_load<V>(d, a, idx, x);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      lstm_sums(x.m[v], x.rms[v], acc);
      vec_update(e, dec, x.g[v], x.m[v], x.rms[v], x.v[v]);
      float f[30];
      vec_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.v[v], 0.0f, f);
#pragma unroll
      for (int c = 0; c < 30; ++c) acc.ch[c] = fmaf(f[c], f[c], acc.ch[c]);
    }
  }
}

// One block of the statistics pass (channel sums and, when nobody carried them over, the LSTM's sums).
// Returns after a barrier with the four waves' sums in `red`.
template <bool LSTM_SUMS, bool KEEP>
__device__ __forceinline__ void velo_stats_block(const TDesc& d, const PyloTensorArgs& a, const Item& it,
                                                 const float* __restrict__ fac_tab, const PyloDecays& dec,
                                                 float (*red)[38]) {
  const EmaConsts e = make_ema(dec);
  VeloAcc acc;
#pragma unroll
  for (int c = 0; c < 30; ++c) acc.ch[c] = 0.0f;
#pragma unroll
  for (int c = 0; c < 8; ++c) acc.lstm[c] = 0.0f;
  lstm_pivots(d, a, acc.piv);
  if (d.tile_nct > 0) {
    const int task = it.a * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (task < d.tile_ntask) velo_stats_tile<KEEP>(d, a, task, e, fac_tab, acc);
  } else if (d.mode == kModeFac2D) {
    if (d.vec == 4) velo_stats_fac<4, false>(d, a, it.a, e, fac_tab, acc);
    else velo_stats_fac<1, false>(d, a, it.a, e, fac_tab, acc);
  } else if (d.mode == kModeFacND) {
    velo_stats_fac<1, true>(d, a, it.a, e, fac_tab, acc);
  } else {
    if (d.vec == 4) velo_stats_vec<4>(d, a, it.a, e, dec, acc);
    else velo_stats_vec<1>(d, a, it.a, e, dec, acc);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int c = 0; c < 30; ++c) {
    const float s = wave_sum(acc.ch[c]);
    if (lane == 0) red[wave][c] = s;
  }
  if (LSTM_SUMS) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const float s = wave_sum(acc.lstm[c]);
      if (lane == 0) red[wave][30 + c] = s;
    }
  }
  __syncthreads();
}

__global__ __launch_bounds__(kThreads) void k_velo_stats(const TDesc* __restrict__ descs,
                                                         const PyloTensorArgs* __restrict__ dyn,
                                                         const Item* __restrict__ items,
                                                         const float* __restrict__ fac_tab, PyloDecays dec,
                                                         double* __restrict__ stats_part) {
  __shared__ float red[kWaves][38];
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  velo_stats_block<true, false>(d, a, it, fac_tab, dec, red);
  if (threadIdx.x < 38) {
    const int c = threadIdx.x;
    stats_part[(size_t)blockIdx.x * kStatW + c] =
        ((double)red[0][c] + (double)red[1][c]) + ((double)red[2][c] + (double)red[3][c]);
  }
}

// ---------------------------------------------------------------------------------------------
// loss features (Velo_naive.py:147-175): 10 EMAs of the clipped loss, updated in place
// ---------------------------------------------------------------------------------------------
// One step of the loss accumulators (Velo_naive.py:129-175), by a whole block (its first wave works, the
// others keep the barriers): ten EMAs of the loss clipped to twice the largest corrected mean, their running
// minima, the iteration counter, and the nine features clamp((cm_i - rmin_i) / max(1e-8, cm_{i+1} - rmin_i) - 1,
// +-1), zero while iteration <= 2, left in feat_s[0..8].  write == false only reads the state: every block of
// k_lo_reduce derives the features that way, and one block of the launch after it advances the state.
__device__ __forceinline__ void loss_step(float* __restrict__ means, float* __restrict__ running_min,
                                          const float* __restrict__ decays, int* __restrict__ iteration,
                                          const float* __restrict__ loss_p, bool write, float* cor_s /*10*/,
                                          float* rmin_s /*10*/, float* feat_s /*9*/) {
  const int dI = threadIdx.x;
  int it = 0;
  if (dI < 64) {
    it = *iteration;
    const float loss = *loss_p;
    float cor = -INFINITY, dec = 0.0f, mean = 0.0f, pw = 0.0f;
    if (dI < 10) {
      dec = decays[dI];
      mean = means[dI];
      pw = powf(dec, (float)(it + 1));
      cor = mean / (1.0f - pw);
    }
    float mx = cor;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float approx_max = (it == 0) ? loss : mx;
    const float l = fminf(fabsf(approx_max) * 2.0f, loss);
    if (dI < 10) {
      const float m2 = mean * dec + l * (1.0f - dec);
      const float cor2 = m2 / (1.0f - pw);
      const float rmin = fminf(running_min[dI], cor2);
      if (write) {
        means[dI] = m2;
        running_min[dI] = rmin;
      }
      cor_s[dI] = cor2;
      rmin_s[dI] = rmin;
    }
  }
  __syncthreads();
  if (write && dI == 0) *iteration = it + 1;
  if (dI < 9) {
    const float den = fmaxf(1e-8f, cor_s[dI + 1] - rmin_s[dI]);
    float f = (cor_s[dI] - rmin_s[dI]) / den - 1.0f;
    f = fminf(fmaxf(f, -1.0f), 1.0f);
    feat_s[dI] = (it + 1 <= 2) ? f * 0.0f : f;
  }
  __syncthreads();
}

// ---------------------------------------------------------------------------------------------
// per-tensor totals of the statistics partials, then (VeLO) the 30 LSTM input features of the
// tensor (Velo_naive.py:178-206), written to row T-1-t (the reference flips the tensor order).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float clip_log_abs10(double v) {
  const float x = (float)v;
  return 0.5f * fminf(fmaxf(logf(1e-8f + fabsf(x * 10.0f)), -5.0f), 5.0f);
}

// Feature q of the 30 LSTM inputs of one tensor from its totals (Velo_naive.py:178-206).
// piv_in: the pivots the totals were shifted by when they are not the tensor's first elements as they stand
// (totals carried over from the previous step's apply pass), else null.
__device__ __forceinline__ float lo_lstm_feature(const TDesc& d, const PyloTensorArgs& a, const double* tot,
                                                 const float* __restrict__ lossfeat, const VeloStep& st, int q,
                                                 const float* piv_in = nullptr) {
  const double n = (double)(d.n > 0 ? d.n : 1);

  const float nu = rsq(fmaxf((float)(tot[2] / n), 1e-9f));
  const double nu2 = (double)nu * (double)nu;
  float val;
  if (q < 9) {
    val = st.frac_dev ? st.frac_dev[a.group * 9 + q] : st.frac[a.group][q];
  } else if (q < 18) {
    val = lossfeat[q - 9];
  } else {
    // totals are of the accumulators shifted by the tensor's pivots (VeloAcc)
    float piv[4];
    if (piv_in != nullptr) { piv[0] = piv_in[0]; piv[1] = piv_in[1]; piv[2] = piv_in[2]; piv[3] = piv_in[3]; }
    else lstm_pivots(d, a, piv);
    const double dr = tot[kSumR] / n;
    const double mean_r = (double)piv[3] + dr;
    if (q == 18) {
      val = clip_log_abs10((double)nu * mean_r);
    } else if (q < 24) {
      val = (q - 19 == d.rank) ? 1.0f : 0.0f;
    } else {
      const int k = (q - 24) % 3;
      const double dm = tot[kSumM + k] / n;
      const double mean_m = (double)(k == 0 ? piv[0] : k == 1 ? piv[1] : piv[2]) + dm;
      if (q < 27) {
        val = clip_log_abs10(nu2 * (tot[kSumMM + k] / n - dm * dm));
      } else {  // the reference subtracts mean_m (not mean_rms) from rms here (Velo_naive.py:198):
                // mean (rms - mean_m)^2 = var(rms) + (mean_rms - mean_m)^2
        const double var_r = tot[kSumRR] / n - dr * dr;
        val = clip_log_abs10(nu2 * (var_r + (mean_r - mean_m) * (mean_r - mean_m)));
      }
    }
  }
  return val;
}


// Row T-1-t of the LSTM input: the tensor's 30 features from its totals and its share of the input mixing
// (VeLO_RNN.py:110-122): relu(mix2 x) and final_mix x for every hidden unit; the maximum over rows and the sum
// follow in k_velo_mix.  Afterwards the tensor's pivots for the sums its apply pass will take are stored
// (its accumulators' first elements as they stand now; the apply pass overwrites them while it runs).
__device__ __forceinline__ void velo_row_features(const TDesc& d, const PyloTensorArgs& a, int t, int T,
                                                  const double* tot, const float* piv_in, float* __restrict__ piv_out,
                                                  const LossState& ls, const VeloStep& st, float* __restrict__ xfeat,
                                                  int H, const float* __restrict__ w2t, const float* __restrict__ b2,
                                                  const float* __restrict__ wft, const float* __restrict__ bf,
                                                  float* __restrict__ mixbuf, float* xs) {
  const int row = T - 1 - t;
  __shared__ float cor_s[10], rmin_s[10], lossfeat[9];
  loss_step(ls.means, ls.running_min, ls.decays, ls.iteration, ls.loss, false, cor_s, rmin_s, lossfeat);
  if (threadIdx.x < 30) xs[threadIdx.x] = lo_lstm_feature(d, a, tot, lossfeat, st, threadIdx.x, piv_in);
  __syncthreads();
  if (piv_out != nullptr && threadIdx.x == 0) {
    float pv[4];
    lstm_pivots(d, a, pv);
#pragma unroll
    for (int q = 0; q < 4; ++q) piv_out[(size_t)t * 4 + q] = pv[q];
  }
  if (threadIdx.x < 30) xfeat[(size_t)row * kXW + threadIdx.x] = xs[threadIdx.x];
  for (int i = threadIdx.x; i < 2 * H; i += kFoldThreads) {
    const int u = i < H ? i : i - H;
    const float* w = i < H ? w2t : wft;
    float acc = i < H ? b2[u] : bf[u];
#pragma unroll
    for (int k = 0; k < 30; ++k) acc = fmaf(xs[k], w[k * H + u], acc);
    mixbuf[((size_t)(i < H ? 0 : 1) * T + row) * H + u] = i < H ? fmaxf(acc, 0.0f) : acc;
  }
}

__global__ __launch_bounds__(kFoldThreads) void k_lo_reduce(const TDesc* __restrict__ descs,
                                                        const PyloTensorArgs* __restrict__ dyn, int T,
                                                        const double* __restrict__ stats_part,
                                                        const double* __restrict__ seg_tot,
                                                        double* __restrict__ totals,
                                                        LossState ls, VeloStep st,
                                                        float* __restrict__ xfeat, int H,
                                                        const float* __restrict__ w2t, const float* __restrict__ b2,
                                                        const float* __restrict__ wft, const float* __restrict__ bf,
                                                        float* __restrict__ mixbuf /* [2][T][H]: relu(mix2 x), final_mix x */,
                                                        float* __restrict__ piv_out /* [T][4], VeLO: see velo_row_features */) {
  constexpr int G = kFoldThreads / kStatW;  // 25 groups x 40 sums = 1000 threads
  __shared__ double part[G][kStatW];
  __shared__ double tot[kStatW];
  __shared__ float xs[32];
  const int t = blockIdx.x;
  const TDesc d = descs[t];
  const PyloTensorArgs a = dyn[t];
  const int c = threadIdx.x % kStatW, gI = threadIdx.x / kStatW;
  if (gI < G) {
    double s = 0.0;
    if (a.grad != nullptr && c < 38) {
      int n_rows;
      const double* rows = stat_rows(d, stats_part, seg_tot, n_rows);
#pragma unroll 16
      for (int b = gI; b < n_rows; b += G) s += rows[(size_t)b * kStatW + c];
    }
    part[gI][c] = s;
  }
  __syncthreads();
  if (threadIdx.x < kStatW) {
    double s = 0.0;
    for (int g2 = 0; g2 < G; ++g2) s += part[g2][threadIdx.x];
    tot[threadIdx.x] = s;
    totals[(size_t)t * kStatW + threadIdx.x] = s;
  }
  __syncthreads();
  if (xfeat == nullptr) return;
  velo_row_features(d, a, t, T, tot, nullptr, piv_out, ls, st, xfeat, H, w2t, b2, wft, bf, mixbuf, xs);
}

// Behind the 2 T counters and flags of `sync` (rounded up to 16 bytes) the workspace holds the guard of the carried
// sums: the address of the plan's flag in pinned host memory, then per tensor the sum of p^2 that the LSTM of the
// current step was fed.
__device__ __forceinline__ long long* velo_guard_base(int* sync, int T) {
  return reinterpret_cast<long long*>(sync + ((2 * T + 3) & ~3));
}
__device__ __forceinline__ int* velo_guard_flag(int* sync, int T) { return reinterpret_cast<int*>(velo_guard_base(sync, T)[0]); }
__device__ __forceinline__ double* velo_guard_sums(int* sync, int T) { return reinterpret_cast<double*>(velo_guard_base(sync, T) + 2); }

// The same from the sums the previous step's apply pass left (rows of kNewSumW doubles per element
// block, shifted by the tensor's first elements as that pass wrote them, i.e. as they stand now): the
// LSTM does not wait for this step's statistics pass.
__global__ __launch_bounds__(kFoldThreads) void k_velo_feat(const TDesc* __restrict__ descs,
                                                            const PyloTensorArgs* __restrict__ dyn, int T,
                                                            const double* __restrict__ newsum_part,
                                                            float* __restrict__ piv, LossState ls, VeloStep st,
                                                            float* __restrict__ xfeat, int H,
                                                            const float* __restrict__ w2t, const float* __restrict__ b2,
                                                            const float* __restrict__ wft, const float* __restrict__ bf,
                                                            float* __restrict__ mixbuf, int* __restrict__ sync) {
  constexpr int G = kFoldThreads / kNewSumW;
  __shared__ double part[G][kNewSumW];
  __shared__ double tot[kStatW];
  __shared__ float xs[32];
  const int t = blockIdx.x;
  const TDesc d = descs[t];
  const PyloTensorArgs a = dyn[t];
  const int c = threadIdx.x % kNewSumW, gI = threadIdx.x / kNewSumW;
  if (gI < G) {
    double s = 0.0;
    const double* rows = newsum_part + (size_t)d.blk0 * kNewSumW;
    for (int b0 = gI; b0 < d.nblk; b0 += 16 * G) {
      double v[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int b = b0 + q * G;
        v[q] = b < d.nblk ? rows[(size_t)b * kNewSumW + c] : 0.0;
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) s += v[q];
    }
    part[gI][c] = s;
  }
  if (threadIdx.x < kStatW) tot[threadIdx.x] = 0.0;
  // the tensor's counter and flag of the fused element pass that follows (k_velo_elem) start at zero
  if (threadIdx.x == 0) { sync[t] = 0; sync[T + t] = 0; }
  __syncthreads();
  if (threadIdx.x < 9) {
    double s = 0.0;
    for (int g2 = 0; g2 < G; ++g2) s += part[g2][threadIdx.x];
    const int q = threadIdx.x;   // 0: sum p^2 | 1..3: m | 4..6: m^2 | 7: rms | 8: rms^2
    tot[q == 0 ? 2 : q < 4 ? kSumM + q - 1 : q < 7 ? kSumMM + q - 4 : q == 7 ? kSumR : kSumRR] = s;
    if (q == 0) velo_guard_sums(sync, T)[t] = s;   // the statistics items of this step hold it against the sum they take themselves
  }
  __syncthreads();
  velo_row_features(d, a, t, T, tot, nullptr, piv, ls, st, xfeat, H, w2t, b2, wft, bf, mixbuf, xs);
}

// ---------------------------------------------------------------------------------------------
// LSTM (VeLO_RNN.py:43-66,110-135).  All weights are pre-transposed to (in, out) by the host.
// Rows are in the reference's order r = T-1-t.
// ---------------------------------------------------------------------------------------------
// Maximum of relu(mix2 x) over a chunk of rows: many tensors only (T > kMixRows), so that the blocks of
// k_velo_mix do not each walk every row.  Block (x, y): 64 hidden units, rows y*kMixRows .. +kMixRows.
constexpr int kMixRows = 256;
__device__ __forceinline__ float mix_colmax(const float* __restrict__ m2, int r0, int r1, int H, int u,
                                            float (*mx_s)[64]) {
  const int lane = threadIdx.x & 63, grp = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float mx = 0.0f;  // relu output is >= 0
#pragma unroll 8
  for (int r = r0 + grp; r < r1; r += kWaves) mx = fmaxf(mx, m2[(size_t)r * H + u]);
  mx_s[grp][lane] = mx;
  __syncthreads();
  return fmaxf(fmaxf(mx_s[0][lane], mx_s[1][lane]), fmaxf(mx_s[2][lane], mx_s[3][lane]));
}

__global__ __launch_bounds__(kThreads) void k_velo_colmax(const float* __restrict__ mixbuf, int T, int H,
                                                          float* __restrict__ pmax /* [chunks][H] */) {
  __shared__ float mx_s[kWaves][64];
  const int u = blockIdx.x * 64 + (threadIdx.x & 63);
  const int r0 = blockIdx.y * kMixRows;
  const float v = mix_colmax(mixbuf, r0, min(T, r0 + kMixRows), H, u, mx_s);
  if (threadIdx.x < 64) pmax[(size_t)blockIdx.y * H + u] = v;
}

// x' = final_mix(x) + max_r relu(mix2(x));  xT[u][r] = x'[r][u], xT[H+u][r] = h[r][u].  The per-row
// products are in mixbuf (written by k_lo_reduce).  Block (x, y): 64 hidden units (one per lane) and
// the 8 rows 8y .. 8y+7, two per wave; the maximum over all rows is taken by every block itself, or
// from the per-chunk maxima of k_velo_colmax when there are many rows.
__global__ __launch_bounds__(kThreads) void k_velo_mix(const float* __restrict__ mixbuf, int T, int Tpad, int H,
                                                       const float* __restrict__ pmax, int n_chunks,
                                                       const float* __restrict__ h_state, float* __restrict__ xT,
                                                       LossState ls) {
  __shared__ float mx_s[kWaves][64];
  // every block of k_lo_reduce has read the loss accumulators by now: one block advances them
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    __shared__ float cor_s[10], rmin_s[10], feat_s[9];
    loss_step(ls.means, ls.running_min, ls.decays, ls.iteration, ls.loss, true, cor_s, rmin_s, feat_s);
  }
  const int lane = threadIdx.x & 63, grp = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int u = blockIdx.x * 64 + lane;  // H is a multiple of 64
  const float* fm = mixbuf + (size_t)T * H;
  const float v = pmax != nullptr ? mix_colmax(pmax, 0, n_chunks, H, u, mx_s) : mix_colmax(mixbuf, 0, T, H, u, mx_s);
#pragma unroll
  for (int q = 0; q < kGateBT / kWaves; ++q) {
    const int r = blockIdx.y * kGateBT + q * kWaves + grp;  // < Tpad
    float acc = 0.0f, hv = 0.0f;
    if (r < T) {
      acc = fm[(size_t)r * H + u] + v;
      hv = h_state[(size_t)r * H + u];
    }
    xT[(size_t)u * Tpad + r] = acc;
    xT[(size_t)(H + u) * Tpad + r] = hv;
  }
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

// gates = [x', h] W^T + b in chunks i, g, f, o;  c = sig(f+1) c + sig(i) tanh(g);  h = sig(o) tanh(c)
// Block = 16 hidden units x 16 slices of the 2H-long contraction, 8 tensors; the slices are added
// in LDS in a fixed order.  (A block streams its units' weights with a fixed number of bytes in flight:
// 16 units a block instead of 32 halves the bytes per block and doubles the blocks, 416 for 256 CUs.)  The weights arrive with the four gates of a unit adjacent, wt[k][u][4],
// so a thread fetches its unit's four gate weights of one input with a single 16-byte load; the
// inputs of the block's 8 tensors (32 B per k, the same for every unit) are staged in LDS once and
// read back as broadcasts, which leaves the weight stream as the only vector-memory traffic of the
// loop.  Blocks are numbered so that the blocks one XCD receives (block id modulo 8) share their
// unit blocks: each XCD's L2 then holds its 1/8 of the 8 MB weight matrix instead of all of it.
constexpr int kGateU = 16, kGateS = 16;
__global__ __launch_bounds__(kThreads) void k_velo_gates(const float* __restrict__ xT, int T, int Tpad, int H,
                                                         const float* __restrict__ wt /*(2H, H, 4)*/,
                                                         const float* __restrict__ b /*4H*/,
                                                         float* __restrict__ h_state, float* __restrict__ c_state) {
  // x tile [2H][8] during the loop (2H <= 2048: 64 KB would not fit, so it is staged in two halves),
  // then the partial sums [kGateS][4 * kGateBT][kGateU]
  constexpr int kHalf = 1024;
  __shared__ float lds[kGateS * 4 * kGateBT * kGateU];
  static_assert(kHalf * kGateBT <= kGateS * 4 * kGateBT * kGateU, "x tile must fit the reduction buffer");
  static_assert(8 * kGateS <= 128 && kHalf % (8 * kGateS) == 0,
                "a batch of eight weight loads per slice must divide 2H for every H that is a multiple of 64");
  const int ul = threadIdx.x % kGateU, sl = threadIdx.x / kGateU;
  const int n_ub = H / kGateU;
  int ub, rb;
  if (n_ub % 8 == 0) {
    const int per = n_ub / 8, xcd = blockIdx.x % 8, j = blockIdx.x / 8;
    ub = xcd * per + j % per;
    rb = j / per;
  } else {
    ub = blockIdx.x % n_ub;
    rb = blockIdx.x / n_ub;
  }
  const int u = ub * kGateU + ul;
  const int r0 = rb * kGateBT;
  float acc[4][kGateBT];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int t = 0; t < kGateBT; ++t) acc[g][t] = 0.0f;
  const int K2 = 2 * H;
  for (int k0 = 0; k0 < K2; k0 += kHalf) {
    const int kn = min(kHalf, K2 - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < kn * 2; i += kThreads) {  // 2 float4 per k
      const int k = i >> 1, h4 = (i & 1) * 4;
      *(float4*)(lds + k * kGateBT + h4) = load_f4(xT + (size_t)(k0 + k) * Tpad + r0 + h4);
    }
    __syncthreads();
    // eight weight loads are issued before the first is used: the loop is bound by how many bytes a
    // block keeps in flight, not by arithmetic (kn is a multiple of 8 * kGateS: H is a multiple of 64)
    for (int kb = sl; kb < kn; kb += 8 * kGateS) {
      float4 wv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) wv[i] = load_f4(wt + ((size_t)(k0 + kb + i * kGateS) * H + u) * 4);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int k = kb + i * kGateS;
        const float w[4] = {wv[i].x, wv[i].y, wv[i].z, wv[i].w};
        const float4 xa = *(const float4*)(lds + k * kGateBT), xb = *(const float4*)(lds + k * kGateBT + 4);
        const float xv[kGateBT] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
        for (int t = 0; t < kGateBT; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g) acc[g][t] = fmaf(xv[t], w[g], acc[g][t]);
      }
    }
  }
  __syncthreads();
  float (*red)[4 * kGateBT][kGateU] = reinterpret_cast<float (*)[4 * kGateBT][kGateU]>(lds);
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int t = 0; t < kGateBT; ++t) red[sl][g * kGateBT + t][ul] = acc[g][t];
  __syncthreads();
  // thread (ul, sl), sl < 8, finishes tensor t = sl of unit ul
  const int t = sl, r = r0 + t;
  if (sl < kGateBT && r < T) {
    float gate[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float s = b[g * H + u];
#pragma unroll
      for (int q = 0; q < kGateS; ++q) s += red[q][g * kGateBT + t][ul];
      gate[g] = s;
    }
    const float c_old = c_state[(size_t)r * H + u];
    const float c_new = sigmoidf_(gate[2] + 1.0f) * c_old + sigmoidf_(gate[0]) * tanhf(gate[1]);
    c_state[(size_t)r * H + u] = c_new;
    h_state[(size_t)r * H + u] = sigmoidf_(gate[3]) * tanhf(c_new);
  }
}

// Entry i of a tensor's folded weight block (layout at the top of this file) from its un-scaled MLP `wm`
// (a bank entry's layout, kVBank floats), the channel normalisers sc[30], param_scale and lr_mult.
// Entries the layout leaves unused read as zero.
__device__ __forceinline__ float velo_fold_entry(const TDesc& d, const float* wm, const float* sc, float pscale,
                                                 float lr_mult, int i) {
  const bool factored = d.mode == kModeFac2D || d.mode == kModeFacND;
  if (i < kVB1) {
    const int k = i / 4, j = i % 4;
    if (factored) return k < kNStat ? wm[j * 30 + stat_channel(k)] * sc[stat_channel(k)] : 0.0f;
    return wm[j * 30 + k] * sc[k];
  }
  if (i < kVWH) return wm[120 + (i - kVB1)];
  if (i < kVBH) return wm[124 + ((i - kVWH) % 4) * 4 + (i - kVWH) / 4];   // (in, out)
  if (i < kVWO) return wm[140 + (i - kVBH)];
  if (i < kVBO) return ((i - kVWO) % 4) < 2 ? wm[144 + ((i - kVWO) % 4) * 4 + (i - kVWO) / 4] : 0.0f;   // [k][j], j < 2 used
  if (i < kVPS) return (i - kVBO) < 2 ? wm[156 + (i - kVBO)] : 0.0f;
  if (i == kVPS) return pscale;
  if (i == kVLR) return lr_mult;
  return 0.0f;
}

// One block per tensor row r: controls = h Wc^T + bc, lr_mult = h.wlr + blr, the tensor's MLP =
// 100 * mean_i(control_i * bank_i) (VeLO_MLP.py:92-126), then the weight blocks the element
// kernels read: un-scaled first layer for k_terms, and the folded block (first-layer rows scaled
// by rsqrt(1e-5 + mean f_c^2), param_scale = sqrt(mean p^2 + 1e-9), lr_mult).
__global__ __launch_bounds__(kFoldThreads) void k_velo_heads(const TDesc* __restrict__ descs, int T, int H, int K,
                                                             const float* __restrict__ h_state,
                                                             const float* __restrict__ wct /*(H,K)*/,
                                                             const float* __restrict__ bc, const float* __restrict__ wlr,
                                                             const float* __restrict__ blr,
                                                             const float* __restrict__ bank /*(K,159)*/,
                                                             const double* __restrict__ totals,
                                                             float* __restrict__ canon, float* __restrict__ wfold,
                                                             float* __restrict__ controls_out,
                                                             float* __restrict__ lr_mult_out,
                                                             float* __restrict__ wmix) {
  // totals == nullptr: the channel sums of this step are not known yet (the LSTM runs ahead of the
  // statistics pass); the tensor's un-scaled MLP (159 floats) and lr_mult go to wmix[t][160] and the
  // folded block is written later, by the tensor's last statistics block (k_velo_elem)
  // Both contractions (controls over the H hidden units, the bank mix over the K controls) are cut
  // into four slices that run side by side and are added in a fixed order; eight loads are issued
  // before the first is used, since a block is bound by the bytes it keeps in flight.
  constexpr int kSl = 4;
  extern __shared__ float smem[];  // hs[H] | ctrl[K] | wm[160] | sc[32] | red[16] | part[kSl][max(K,160)]
  float* hs = smem;
  float* ctrl = hs + H;
  float* wm = ctrl + K;
  float* sc = wm + 160;
  float* red = sc + 32;
  float* part = red + 16;
  const int pitch = K > 160 ? K : 160;
  const int r = blockIdx.x;
  const int t = T - 1 - r;
  const TDesc d = descs[t];
  for (int u = threadIdx.x; u < H; u += kFoldThreads) hs[u] = h_state[(size_t)r * H + u];
  __syncthreads();
  for (int i = threadIdx.x; i < K * kSl; i += kFoldThreads) {
    const int j = i % K, sl = i / K;
    const int u0 = sl * (H / kSl), u1 = u0 + H / kSl;  // H is a multiple of 64
    float acc = 0.0f;
    for (int u = u0; u < u1; u += 8) {
      float w[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) w[q] = wct[(size_t)(u + q) * K + j];
#pragma unroll
      for (int q = 0; q < 8; ++q) acc = fmaf(hs[u + q], w[q], acc);
    }
    part[sl * pitch + j] = acc;
  }
  {
    float s = 0.0f;
    for (int u = threadIdx.x; u < H; u += kFoldThreads) s = fmaf(hs[u], wlr[u], s);
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  }
  if (threadIdx.x < 30 && totals != nullptr) {
    const double n = (double)(d.n > 0 ? d.n : 1);
    sc[threadIdx.x] = rsq(1e-5f + (float)(totals[(size_t)t * kStatW + threadIdx.x] / n));
  }
  __syncthreads();
  for (int j = threadIdx.x; j < K; j += kFoldThreads) {
    const float acc = bc[j] + ((part[j] + part[pitch + j]) + (part[2 * pitch + j] + part[3 * pitch + j]));
    ctrl[j] = acc;
    if (controls_out != nullptr) controls_out[(size_t)r * K + j] = acc;
  }
  float lr_mult = blr[0];
  {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < kFoldThreads / 64; ++w) s += red[w];
    lr_mult += s;
  }
  __syncthreads();
  const int Kq = (K + kSl - 1) / kSl;
  for (int i = threadIdx.x; i < 160 * kSl; i += kFoldThreads) {
    const int q = i % 160, sl = i / 160;
    float acc = 0.0f;
    if (q < kVBank) {
      const int i0 = sl * Kq, i1 = min(K, i0 + Kq);
      int c = i0;
      for (; c + 8 <= i1; c += 8) {
        float b8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) b8[e] = bank[(size_t)(c + e) * kVBank + q];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = fmaf(ctrl[c + e], b8[e], acc);
      }
      for (; c < i1; ++c) acc = fmaf(ctrl[c], bank[(size_t)c * kVBank + q], acc);
    }
    part[sl * pitch + q] = acc;
  }
  __syncthreads();
  for (int q = threadIdx.x; q < kVBank; q += kFoldThreads) {
    const float acc = (part[q] + part[pitch + q]) + (part[2 * pitch + q] + part[3 * pitch + q]);
    wm[q] = (acc / (float)K) * 100.0f;
  }
  __syncthreads();
  float* cn = canon + (size_t)t * kVCanon;
  for (int i = threadIdx.x; i < 124; i += kFoldThreads) cn[i] = i < 120 ? wm[(i % 4) * 30 + i / 4] : wm[i];
  if (threadIdx.x == 0 && lr_mult_out != nullptr) lr_mult_out[r] = lr_mult;
  if (totals == nullptr) {
    float* o = wmix + (size_t)t * 160;
    for (int i = threadIdx.x; i < 160; i += kFoldThreads) o[i] = i < kVBank ? wm[i] : lr_mult;
    return;
  }
  const double n = (double)(d.n > 0 ? d.n : 1);
  const float pscale = sqrtf((float)(totals[(size_t)t * kStatW + 2] / n) + 1e-9f);
  for (int i = threadIdx.x; i < kVFold; i += kFoldThreads) {
    const float v = velo_fold_entry(d, wm, sc, pscale, lr_mult, i);
    if (i < kVLR + 1) wfold[(size_t)t * kVFold + i] = v;
  }
}

// ---------------------------------------------------------------------------------------------
// apply pass: accumulators advanced and written, features, 30->4->4->3 MLP,
//   p <- p - lr * lr_mult * param_scale * o0 * exp(o1 * exp_mult) * step_mult;  p <- p - wd*lr*p
// (Velo_naive.py:491-502)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float velo_update(float p, const float (&h1)[4], const cfloat* w, const PyloTensorArgs& a) {
  float o0 = w[kVBO + 0], o1 = w[kVBO + 1];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float hk = fmaxf(h1[k], 0.0f);
    o0 = fmaf(hk, w[kVWO + k * 4 + 0], o0);
    o1 = fmaf(hk, w[kVWO + k * 4 + 1], o1);
  }
  float step = w[kVPS] * ((o0 * expf(o1 * a.exp_mult)) * a.step_mult);
  step = w[kVLR] * step;
  p = fmaf(step, -a.lr, p);
  if (a.weight_decay > 0.0f) p = fmaf(p, -(a.weight_decay * a.lr), p);
  return p;
}

__device__ __forceinline__ void velo_hidden(const float (&h0)[4], const cfloat* w, float (&h1)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) h1[j] = w[kVBH + j];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float hk = fmaxf(h0[k], 0.0f);
#pragma unroll
    for (int j = 0; j < 4; ++j) h1[j] = fmaf(hk, w[kVWH + k * 4 + j], h1[j]);
  }
}

template <int V, bool ND>
__device__ __forceinline__ void velo_apply_fac(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                               const EmaConsts& e, const float* __restrict__ fac_tab,
                                               const float* __restrict__ term_tab, const float* wbase, NewSums& ns) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  const long long n = d.n;
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= n) break;
    ElemIn<V> x;
    lo_load<V, ND>(d, a, idx, fac_tab, x);
    float h[V][4];
    lo_terms<V, ND, 4>(d, x, term_tab, h);
    float f[V][kNStat], m0[V], m1[V], m2[V], pn[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ema_update(e, x.g[v], x.m[v], x.rms[v]);
      m0[v] = x.m[v][0]; m1[v] = x.m[v][1]; m2[v] = x.m[v][2];
      lo_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.rfcf[v], 1e-6f, f[v]);
    }
    const cfloat* w = launder(wbase);
#pragma unroll
    for (int c = 0; c < kNStat; ++c) {
      float wc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) wc[j] = w[kVW1 + c * 4 + j];
#pragma unroll
      for (int v = 0; v < V; ++v) {
#pragma unroll
        for (int j = 0; j < 4; ++j) h[v][j] = fmaf(f[v][c], wc[j], h[v][j]);
      }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
      float h1[4];
      velo_hidden(h[v], w, h1);
      pn[v] = velo_update(x.p[v], h1, w, a);
      ns.add(pn[v], x.m[v], x.rms[v]);
    }
    store_vec<V>(a.mom + idx, m0);
    store_vec<V>(a.mom + n + idx, m1);
    store_vec<V>(a.mom + 2 * n + idx, m2);
    store_vec<V>(a.rms + idx, x.rms);
    store_vec<V>(a.param + idx, pn);
  }
}

// The apply pass over one wave task of the column-resident walk, with the 30->4->4->2 MLP as
// lane-local 4x4x1 fp32 outer products on the matrix pipe: weight group v (four consecutive floats
// of the folded block) sits in lanes 4*(v%16).. of register v/16; biases enter as a rank-1 update
// with the constant 1.
__device__ __forceinline__ void velo_apply_tile(const TDesc& d, const PyloTensorArgs& a, int task,
                                                const EmaConsts& e, const float* __restrict__ fac_tab,
                                                const float* __restrict__ term_tab, const float* wbase, NewSums& ns,
                                                bool coh) {
  // coh: the folded block was written by another block of the running kernel (see coh_store_wait)
  constexpr int V = kTileV;
  const TileTask tk(d, task);
  const int lane = threadIdx.x & 63;
  float wreg[3];
#pragma unroll
  for (int r = 0; r < 3; ++r) wreg[r] = coh ? coh_load(wbase + r * 64 + lane) : *(const gfloat*)(wbase + r * 64 + lane);
  // param_scale and lr_mult sit in floats 164 / 165 of the block, i.e. in lanes 36 / 37 of register 2
  const float pscale = __shfl(wreg[2], kVPS - 128, 64), lr_mult = __shfl(wreg[2], kVLR - 128, 64);
  const float exp_scale = a.exp_mult * 1.44269504088896341f;
  constexpr int gWH = kVWH / 4, gBH = kVBH / 4, gWO = kVWO / 4, gBO = kVBO / 4;
  const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
  const float* f0 = fac_tab + d.fac_off[0];
  const float* f1 = fac_tab + d.fac_off[1];
  const float* t0 = term_tab + d.term_off[0];
  const float* t1 = term_tab + d.term_off[1];
  float fb[V][4], tb[V][4];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    load_vec_o<4>(f1 + v * 4, tk.col * 16u, fb[v]);
    load_vec_o<4>(t1 + v * 4, tk.col * 16u, tb[v]);
  }
  const unsigned lo = lane * (V * 4u);
  const float* g = a.grad + tk.first;
  float *p = a.param + tk.first, *m0 = a.mom + tk.first, *m1 = a.mom + d.n + tk.first,
        *m2 = a.mom + 2 * d.n + tk.first, *rms = a.rms + tk.first;
  const float* fr = f0 + (size_t)tk.r0 * 4;
  const float* tr = t0 + (size_t)tk.r0 * 4;
  const float wd_lr = a.weight_decay * a.lr;
  for (int r = tk.r0; r < tk.r1; ++r) {
    float xg[V], xp[V], x0[V], x1[V], x2[V], xr[V], fa[4], ta[4];
    load_vec_nt<V>(g, lo, xg);
    load_vec_nt<V>(p, lo, xp);
    load_vec_nt<V>(m0, lo, x0);
    load_vec_nt<V>(m1, lo, x1);
    load_vec_nt<V>(m2, lo, x2);
    load_vec_nt<V>(rms, lo, xr);
    load_uniform<4>(fr, fa);
    load_uniform<4>(tr, ta);
    float f[V][kNStat];
    v4f h[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const float gg = clampf(xg[v], a.clip_val);
      float m[3] = {x0[v], x1[v], x2[v]};
      ema_update(e, gg, m, xr[v]);
      x0[v] = m[0]; x1[v] = m[1]; x2[v] = m[2];
      const float rfcf[3] = {fa[0] * fb[v][0], fa[1] * fb[v][1], fa[2] * fb[v][2]};
      lo_features(gg, xp[v], m, xr[v], rfcf, 1e-6f, f[v]);
#pragma unroll
      for (int j = 0; j < 4; ++j) h[v][j] = ta[j] + tb[v][j];
    }
    store_vec_nt<V>(m0, lo, x0);
    store_vec_nt<V>(m1, lo, x1);
    store_vec_nt<V>(m2, lo, x2);
    store_vec_nt<V>(rms, lo, xr);
#pragma unroll
    for (int c = 0; c < kNStat; ++c) {
#pragma unroll
      for (int v = 0; v < V; ++v) h[v] = mfma_w4(wreg[c / 16], f[v][c], h[v], c % 16);
    }
    v4f g2[V], o[V];
#pragma unroll
    for (int v = 0; v < V; ++v) g2[v] = mfma_w4(wreg[gBH / 16], 1.0f, zero, gBH % 16);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int v = 0; v < V; ++v) g2[v] = mfma_w4(wreg[(gWH + k) / 16], relu(h[v][k]), g2[v], (gWH + k) % 16);
    }
#pragma unroll
    for (int v = 0; v < V; ++v) o[v] = mfma_w4(wreg[gBO / 16], 1.0f, zero, gBO % 16);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int v = 0; v < V; ++v) o[v] = mfma_w4(wreg[(gWO + k) / 16], relu(g2[v][k]), o[v], (gWO + k) % 16);
    }
    float pn[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      float step = pscale * ((o[v][0] * __builtin_amdgcn_exp2f(o[v][1] * exp_scale)) * a.step_mult);
      step = lr_mult * step;
      float q = fmaf(step, -a.lr, xp[v]);
      if (a.weight_decay > 0.0f) q = fmaf(q, -wd_lr, q);
      pn[v] = q;
      const float mm[3] = {x0[v], x1[v], x2[v]};
      ns.add(q, mm, xr[v]);
    }
    store_vec_o<V>(p, lo, pn);
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0;
    fr += 4; tr += 4;
  }
}

template <int V>
__device__ __forceinline__ void velo_apply_vec(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                               const EmaConsts& e, const PyloDecays& dec, const float* wbase,
                                               NewSums& ns) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  const long long n = d.n;
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= n) break;
    VecIn<V> x;
    vec_load<V>(d, a, idx, x);
    const cfloat* w = launder(wbase);
    float pn[V], mo[3][V], vo[3][V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      vec_update(e, dec, x.g[v], x.m[v], x.rms[v], x.v[v]);
      float f[30];
      vec_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.v[v], 0.0f, f);
      float h0[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) h0[j] = w[kVB1 + j];
#pragma unroll
      for (int c = 0; c < 30; ++c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) h0[j] = fmaf(f[c], w[kVW1 + c * 4 + j], h0[j]);
      }
      float h1[4];
      velo_hidden(h0, w, h1);
      pn[v] = velo_update(x.p[v], h1, w, a);
      ns.add(pn[v], x.m[v], x.rms[v]);
#pragma unroll
      for (int k = 0; k < 3; ++k) { mo[k][v] = x.m[v][k]; vo[k][v] = x.v[v][k]; }
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      store_vec<V>(a.mom + k * n + idx, mo[k]);
      store_vec<V>(a.fac_v + k * n + idx, vo[k]);
    }
    store_vec<V>(a.rms + idx, x.rms);
    store_vec<V>(a.param + idx, pn);
  }
}

// One block of the apply pass; its sums over the written values go to row `row` of newsum_part.
__device__ __forceinline__ void velo_apply_block(const TDesc& d, const PyloTensorArgs& a, const Item& it,
                                                 const float* __restrict__ fac_tab,
                                                 const float* __restrict__ term_tab, const PyloDecays& dec,
                                                 const float* __restrict__ wfold, const float* __restrict__ piv,
                                                 double* __restrict__ newsum_part, int row, bool coh, float (*red)[9]) {
  const EmaConsts e = make_ema(dec);
  const float* w = wfold + (size_t)it.tensor * kVFold;
  NewSums ns;
  ns.clear(d, a, e, piv + (size_t)it.tensor * 4);
  if (d.tile_nct > 0) {
    const int task = it.a * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (task < d.tile_ntask) velo_apply_tile(d, a, task, e, fac_tab, term_tab, w, ns, coh);
  } else if (d.mode == kModeFac2D) {
    if (d.vec == 4) velo_apply_fac<4, false>(d, a, it.a, e, fac_tab, term_tab, w, ns);
    else velo_apply_fac<1, false>(d, a, it.a, e, fac_tab, term_tab, w, ns);
  } else if (d.mode == kModeFacND) {
    velo_apply_fac<1, true>(d, a, it.a, e, fac_tab, term_tab, w, ns);
  } else {
    if (d.vec == 4) velo_apply_vec<4>(d, a, it.a, e, dec, w, ns);
    else velo_apply_vec<1>(d, a, it.a, e, dec, w, ns);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int c = 0; c < 9; ++c) {
    const float sc = wave_sum(ns.v[c]);
    if (lane == 0) red[wave][c] = sc;
  }
  __syncthreads();
  if (threadIdx.x < 9) {
    const int c = threadIdx.x;
    newsum_part[(size_t)row * kNewSumW + c] =
        ((double)red[0][c] + (double)red[1][c]) + ((double)red[2][c] + (double)red[3][c]);
  }
}

// Apply pass as a launch of its own.
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) void k_velo_apply(const TDesc* __restrict__ descs,
                                                         const PyloTensorArgs* __restrict__ dyn,
                                                         const Item* __restrict__ items,
                                                         const float* __restrict__ fac_tab,
                                                         const float* __restrict__ term_tab, PyloDecays dec,
                                                         const float* __restrict__ wfold,
                                                         const float* __restrict__ piv,
                                                         double* __restrict__ newsum_part) {
  __shared__ float red[kWaves][9];
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  velo_apply_block(d, a, it, fac_tab, term_tab, dec, wfold, piv, newsum_part, (int)blockIdx.x, false, red);
}

// ---------------------------------------------------------------------------------------------
// The fused element pass of VeLO: statistics, weight folding and apply items of every tensor in ONE
// launch, ordered slab by slab, exactly as k_celo2_elem does it (see there for the ordering, the
// hand-over between running blocks and why a wait ends).  It needs the tensors' MLPs before it starts,
// i.e. an LSTM that does not depend on this step's statistics pass: the LSTM's inputs are sums over the
// parameters and accumulators as they stand BEFORE the step, which are the values the previous step's
// apply items wrote and summed up on the way (NewSums, k_velo_feat).  The tensor's last statistics
// block folds this step's channel normalisers, param_scale and lr_mult into the block the apply
// items read.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) void k_velo_elem(const TDesc* __restrict__ descs,
                                                        const PyloTensorArgs* __restrict__ dyn,
                                                        const Item* __restrict__ items,
                                                        const float* __restrict__ fac_tab,
                                                        const float* __restrict__ term_tab, PyloDecays dec,
                                                        const float* __restrict__ wmix, float* __restrict__ wfold,
                                                        double* __restrict__ stats_part, const float* __restrict__ piv,
                                                        double* __restrict__ newsum_part, int* __restrict__ sync,
                                                        int n_tensors) {
  __shared__ float red[kWaves][38];
  __shared__ double part[kThreads / 30][30];
  __shared__ float sc[30];
  __shared__ int s_flag;
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  if (it.c & kElemApply) {
    if (threadIdx.x == 0) {
      const int* ready = sync + n_tensors + it.tensor;
      int ok = coh_load(ready);
      for (int spin = 0; !ok && spin < kSpinLimit; ++spin) {
        __builtin_amdgcn_s_sleep(16);
        ok = coh_load(ready);
      }
      s_flag = ok;
    }
    __syncthreads();
    if (s_flag) {
      velo_apply_block(d, a, it, fac_tab, term_tab, dec, wfold, piv, newsum_part, it.b, true,
                       reinterpret_cast<float(*)[9]>(&red[0][0]));
    } else {
      // gave up waiting (see k_celo2_elem): NaN parameters for this block's elements rather than a hang
      const float nan = __builtin_nanf("");
      if (d.tile_nct > 0) {
        const int task = it.a * 4 + (threadIdx.x >> 6);
        if (task < d.tile_ntask) {
          const TileTask tk(d, task);
          for (int r = tk.r0; r < tk.r1; ++r)
            for (int v = 0; v < kTileV; ++v) a.param[(size_t)r * d.C0 + tk.col + v] = nan;
        }
      } else {
        const long long chunk = (long long)kThreads * d.vec * kElemIters, base = (long long)it.a * chunk;
        for (long long i = base + threadIdx.x; i < base + chunk && i < d.n; i += kThreads) a.param[i] = nan;
      }
    }
    return;
  }
  // the LSTM's sums were carried over: nobody reads them here
  if (it.c & kElemKeep) velo_stats_block<false, true>(d, a, it, fac_tab, dec, red);
  else velo_stats_block<false, false>(d, a, it, fac_tab, dec, red);
  if (threadIdx.x < 30) {
    const int c = threadIdx.x;
    coh_store_wait(stats_part + (size_t)it.b * kStatW + c,
                   ((double)red[0][c] + (double)red[1][c]) + ((double)red[2][c] + (double)red[3][c]));
  }
  __syncthreads();
  if (threadIdx.x == 0)
    s_flag = __hip_atomic_fetch_add(sync + it.tensor, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == d.nblk - 1;
  __syncthreads();
  if (!s_flag) return;
  // the tensor's last statistics block: channel sums in row order, then the folded block
  constexpr int G = kThreads / 30;
  const int c = threadIdx.x % 30, gI = threadIdx.x / 30;
  if (gI < G) {
    const double* rows = stats_part + (size_t)d.blk0 * kStatW;
    double s = 0.0;
    for (int b0 = gI; b0 < d.nblk; b0 += 16 * G) {
      double v[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int b = b0 + q * G;
        v[q] = b < d.nblk ? coh_load(rows + (size_t)b * kStatW + c) : 0.0;
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) s += v[q];
    }
    part[gI][c] = s;
  }
  __syncthreads();
  __shared__ float pscale_s;
  if (threadIdx.x < 30) {
    double s = 0.0;
    for (int g2 = 0; g2 < G; ++g2) s += part[g2][threadIdx.x];
    const double n = (double)(d.n > 0 ? d.n : 1);
    sc[threadIdx.x] = rsq(1e-5f + (float)(s / n));
    if (threadIdx.x == 2) {   // channel 2 is the parameter
      // The LSTM of this step was fed the sum of p^2 that the previous step's apply items carried over; `s` is
      // the same sum over the parameter as it stands now.  They differ (beyond the rounding of two summation
      // orders) only if somebody else wrote the parameter in between without the plan being told: the
      // tensor's step is poisoned (a NaN param_scale multiplies it) and the plan's flag raised rather than a
      // step taken on stale statistics.  The flag is pinned host memory (a system-scope store of 1 + tensor).
      // Both addresses are found behind the counters of `sync` rather than passed as arguments: the kernel's
      // scalar registers are spilled as it is, and three more live arguments cost its hot loops 7 %.
      const double carried = velo_guard_sums(sync, n_tensors)[it.tensor];
      const bool ok = fabs(s - carried) <= 1e-3 * fmax(fabs(s), fabs(carried));
      pscale_s = ok ? sqrtf((float)(s / n) + 1e-9f) : __builtin_nanf("");
      if (!ok) __hip_atomic_store(velo_guard_flag(sync, n_tensors), it.tensor + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
  __syncthreads();
  const float* wm = wmix + (size_t)it.tensor * 160;
  if (threadIdx.x < kVFold)
    coh_store_wait(wfold + (size_t)it.tensor * kVFold + threadIdx.x,
                   velo_fold_entry(d, wm, sc, pscale_s, wm[kVBank], threadIdx.x));
  __syncthreads();   // every folded weight has been performed
  if (threadIdx.x == 0) __hip_atomic_store(sync + n_tensors + it.tensor, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pylo
