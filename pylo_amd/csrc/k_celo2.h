// ELO-CELO2 / CELO2 element kernels: statistics pass, weight folding, apply pass.
#pragma once

#include "pylo_common.h"
#include "k_cast.h"

#ifndef PYLO_STATS_UNROLL
#define PYLO_STATS_UNROLL 2   // rows of the statistics walk whose loads are issued together
#endif

namespace pylo {

struct EmaConsts {
  float bm[3], obm[3];  // momentum decays and 1-decay
  float br, obr;        // rms
};

__device__ __forceinline__ EmaConsts make_ema(const PyloDecays& dec) {
  EmaConsts e;
#pragma unroll
  for (int k = 0; k < 3; ++k) { e.bm[k] = dec.beta_m[k]; e.obm[k] = 1.0f - dec.beta_m[k]; }
  e.br = dec.beta_rms;
  e.obr = 1.0f - dec.beta_rms;
  return e;
}

// acc <- beta*acc + (1-beta)*new, each product and the sum rounded (ELO_CELO2_naive.py:145,149)
__device__ __forceinline__ void ema_update(const EmaConsts& e, float g, float (&m)[3], float& rms) {
#pragma unroll
  for (int k = 0; k < 3; ++k) m[k] = m[k] * e.bm[k] + e.obm[k] * g;
  rms = rms * e.br + e.obr * (g * g);
}

// The 18 per-element channels (ELO_CELO2_naive.py:180-215); rs = rsqrt(rms + eps_rs), rfcf_k =
// row_factor_k * col_factor_k of the element's row and column.
__device__ __forceinline__ void lo_features(float g, float p, const float (&m)[3], float rms,
                                            const float (&rfcf)[3], float eps_rs, float (&f)[kNStat]) {
  const float rs = rsq(rms + eps_rs);
  f[0] = g;
  f[1] = fminf(fmaxf(g, -0.1f), 0.1f);
  f[2] = p;
  f[3] = m[0]; f[4] = m[1]; f[5] = m[2];
  f[6] = rms;
  f[7] = m[0] * rs; f[8] = m[1] * rs; f[9] = m[2] * rs;
  f[10] = rs;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    f[11 + k] = g * rfcf[k];
    f[15 + k] = m[k] * rfcf[k];
  }
  f[14] = g * rs;
}

// AdamW over the shared mom[0] / rms accumulators (ELO_CELO2_naive.py:296-302).
template <int V>
__device__ __forceinline__ void celo2_adam_chunk(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                 float scale, const EmaConsts& e) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  const long long n = d.n;
#pragma unroll 2
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= n) break;
    float g[V], p[V], m0[V], m1[V], m2[V], r[V];
    load_vec<V>(a.grad + idx, g);
    load_vec<V>(a.param + idx, p);
    load_vec<V>(a.mom + idx, m0);
    load_vec<V>(a.mom + n + idx, m1);
    load_vec<V>(a.mom + 2 * n + idx, m2);
    load_vec<V>(a.rms + idx, r);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const float gg = clampf(g[v] * scale, a.clip_val);
      float m[3] = {m0[v], m1[v], m2[v]};
      ema_update(e, gg, m, r[v]);
      m0[v] = m[0]; m1[v] = m[1]; m2[v] = m[2];
      const float mh = m[0] / a.bc1;
      const float vh = r[v] / a.bc2;
      const float upd = mh / (sqrtf(vh) + 1e-8f);
      p[v] = fmaf(upd + a.weight_decay * p[v], -a.lr, p[v]);
    }
    store_vec<V>(a.mom + idx, m0);
    store_vec<V>(a.mom + n + idx, m1);
    store_vec<V>(a.mom + 2 * n + idx, m2);
    store_vec<V>(a.rms + idx, r);
    store_vec<V>(a.param + idx, p);
  }
}

// AdamW with the tensor's own moments (CELO2_cuda.py:234-253): a.mom = exp_avg, a.rms = exp_avg_sq.
template <int V>
__device__ __forceinline__ void celo2_adam_indep_chunk(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                       float scale, const PyloDecays& dec) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  const long long n = d.n;
  const float b1 = dec.adam_beta1, ob1 = 1.0f - dec.adam_beta1, b2 = dec.adam_beta2, ob2 = 1.0f - dec.adam_beta2;
#pragma unroll 2
  for (int it = 0; it < kElemIters; ++it) {
    const long long idx = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (idx >= n) break;
    float g[V], p[V], m[V], v[V];
    load_vec<V>(a.grad + idx, g);
    load_vec<V>(a.param + idx, p);
    load_vec<V>(a.mom + idx, m);
    load_vec<V>(a.rms + idx, v);
#pragma unroll
    for (int q = 0; q < V; ++q) {
      const float gg = clampf(g[q] * scale, a.clip_val);
      m[q] = m[q] * b1 + ob1 * gg;
      v[q] = v[q] * b2 + (ob2 * gg) * gg;
      const float mh = m[q] / a.bc1;
      const float vh = v[q] / a.bc2;
      const float upd = mh / (sqrtf(vh) + dec.adam_eps);
      p[q] = fmaf(upd + a.weight_decay * p[q], -a.lr, p[q]);
    }
    store_vec<V>(a.mom + idx, m);
    store_vec<V>(a.rms + idx, v);
    store_vec<V>(a.param + idx, p);
  }
}

// One vector of V consecutive elements (same dim-0 index i0, dim-1 indices i1..i1+V-1).
template <int V>
struct ElemIn {
  float g[V], p[V], m[V][3], rms[V];
  float rfcf[V][3];
  int i0, i1;
};

template <int V>
__device__ __forceinline__ void load_elems(const TDesc& d, const PyloTensorArgs& a, long long idx,
                                           float scale, const float* f0, const float* f1, ElemIn<V>& x) {
  const long long n = d.n;
  float m0[V], m1[V], m2[V];
  load_vec<V>(a.grad + idx, x.g);
  load_vec<V>(a.param + idx, x.p);
  load_vec<V>(a.mom + idx, m0);
  load_vec<V>(a.mom + n + idx, m1);
  load_vec<V>(a.mom + 2 * n + idx, m2);
  load_vec<V>(a.rms + idx, x.rms);
  const unsigned u = (unsigned)idx;  // n < 2^31
  x.i0 = (int)(u / (unsigned)d.C0);
  x.i1 = (int)(u - (unsigned)x.i0 * (unsigned)d.C0);
  const float4 fa = load_f4(f0 + (size_t)x.i0 * 4);
#pragma unroll
  for (int v = 0; v < V; ++v) {
    const float4 fb = load_f4(f1 + (size_t)(x.i1 + v) * 4);
    x.g[v] = cond_grad(x.g[v], scale, a.clip_val, d.nan0);
    x.m[v][0] = m0[v]; x.m[v][1] = m1[v]; x.m[v][2] = m2[v];
    x.rfcf[v][0] = fa.x * fb.x;
    x.rfcf[v][1] = fa.y * fb.y;
    x.rfcf[v][2] = fa.z * fb.z;
  }
}

// Position of a lane inside one chunk of consecutive elements of a 2-D tensor: element
// offset from the chunk's first element, row and column.  Advancing by a whole block stride costs
// three or four instructions (no division); every access is "uniform base + 32-bit lane offset".
// V = elements per lane and access, VC = the tensor's vector width (which fixes the chunk size).
template <int V, int VC = V>
struct Cursor {
  static constexpr int kChunkElems = kThreads * VC * kElemIters;
  static constexpr int kIters = kElemIters * VC / V;
  unsigned off, i0, i1;  // lane's vector: element offset in the chunk, row, column
  unsigned lim;          // elements of the chunk that exist
  unsigned C0, sq, sr;   // row length; block stride = sq rows + sr columns
  unsigned c_i0, c_i1;   // coordinates of the chunk's first element (always valid)

  __device__ __forceinline__ Cursor(const TDesc& d, long long base) {
    off = threadIdx.x * V;
    const long long left = d.n - base;
    lim = left < (long long)kChunkElems ? (unsigned)left : (unsigned)kChunkElems;
    C0 = (unsigned)d.C0;
    const unsigned ub = (unsigned)base;  // n < 2^31
    c_i0 = ub / C0;
    c_i1 = ub - c_i0 * C0;
    const unsigned q = off / C0;
    i0 = c_i0 + q;
    i1 = c_i1 + (off - q * C0);
    if (i1 >= C0) { i1 -= C0; ++i0; }
    constexpr unsigned step = kThreads * V;
    sq = step / C0;
    sr = step - sq * C0;
  }
  __device__ __forceinline__ bool live() const { return off < lim; }
  __device__ __forceinline__ void advance() {
    off += kThreads * V;
    i0 += sq;
    i1 += sr;
    if (i1 >= C0) { i1 -= C0; ++i0; }
  }
};

// Base pointers of one chunk (all wave-uniform).
struct ChunkPtrs {
  const float *g, *p;
  float *m0, *m1, *m2, *rms, *out;
  __device__ __forceinline__ ChunkPtrs(const TDesc& d, const PyloTensorArgs& a, long long base) {
    g = a.grad + base; p = a.param + base;
    m0 = a.mom + base; m1 = a.mom + d.n + base; m2 = a.mom + 2 * d.n + base;
    rms = a.rms + base; out = a.step_out + base;
  }
};

// eight consecutive floats of row i of a table with eight floats per row
__device__ __forceinline__ void load_row8(const float* tab, unsigned i, float (&t)[8]) {
  float lo[4], hi[4];
  load_vec_o<4>(tab, i * 32u, lo);
  load_vec_o<4>(tab + 4, i * 32u, hi);
#pragma unroll
  for (int j = 0; j < 4; ++j) { t[j] = lo[j]; t[4 + j] = hi[j]; }
}

// load_elems through a cursor; (off, i0, i1) are the lane's (possibly substituted) coordinates.
template <int V>
__device__ __forceinline__ void load_elems_at(const TDesc& d, const PyloTensorArgs& a, const ChunkPtrs& cp,
                                              unsigned off, unsigned i0, unsigned i1, float scale,
                                              const float* f0, const float* f1, ElemIn<V>& x) {
  float m0[V], m1[V], m2[V];
  const unsigned bo = off * 4u;
  load_vec_o<V>(cp.g, bo, x.g);
  load_vec_o<V>(cp.p, bo, x.p);
  load_vec_o<V>(cp.m0, bo, m0);
  load_vec_o<V>(cp.m1, bo, m1);
  load_vec_o<V>(cp.m2, bo, m2);
  load_vec_o<V>(cp.rms, bo, x.rms);
  x.i0 = (int)i0;
  x.i1 = (int)i1;
  float fa[4];
  load_vec_o<4>(f0, i0 * 16u, fa);
#pragma unroll
  for (int v = 0; v < V; ++v) {
    float fb[4];
    load_vec_o<4>(f1 + v * 4, i1 * 16u, fb);
    x.g[v] = clampf(x.g[v] * scale, a.clip_val);
    x.m[v][0] = m0[v]; x.m[v][1] = m1[v]; x.m[v][2] = m2[v];
    x.rfcf[v][0] = fa[0] * fb[0];
    x.rfcf[v][1] = fa[1] * fb[1];
    x.rfcf[v][2] = fa[2] * fb[2];
  }
}

template <int V>
__device__ __forceinline__ void celo2_stats_chunk(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                  float scale, const EmaConsts& e, const float* f0,
                                                  const float* f1, float (&acc)[kNStat]) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  Cursor<V> cur(d, base);
  const ChunkPtrs cp(d, a, base);
#pragma unroll 2
  for (int it = 0; it < kElemIters; ++it, cur.advance()) {
    if (!cur.live()) break;
    ElemIn<V> x;
    load_elems_at<V>(d, a, cp, cur.off, cur.i0, cur.i1, scale, f0, f1, x);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ema_update(e, x.g[v], x.m[v], x.rms[v]);
      float f[kNStat];
      lo_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.rfcf[v], 1e-8f, f);
#pragma unroll
      for (int c = 0; c < kNStat; ++c) acc[c] = fmaf(f[c], f[c], acc[c]);
    }
  }
}

// Geometry of one wave task of the column-resident walk: V columns per lane, nct column tiles.
struct TileTask {
  int r0, r1;          // rows
  unsigned col;        // the lane's first column
  long long first;     // element index of (r0, first column of the wave)
  __device__ __forceinline__ TileTask(const TDesc& d, int task, int nct, int V) {
    const int ct = task % nct, rr = task / nct;
    r0 = rr * d.tile_rows;
    r1 = r0 + d.tile_rows < d.R0 ? r0 + d.tile_rows : d.R0;
    col = (unsigned)ct * (64 * V) + (threadIdx.x & 63) * V;
    first = (long long)r0 * d.C0 + (long long)ct * (64 * V);
  }
  __device__ __forceinline__ TileTask(const TDesc& d, int task) : TileTask(d, task, d.tile_nct, kTileV) {}
};

// Statistics of one wave task: the column factors stay in registers, the row factors arrive through
// the scalar cache, and the only per-row vector memory traffic is the six streams.
// KEEP: plain loads, which leave the lines in the memory-side cache for the apply items that follow a
// few thousand blocks later (k_celo2_elem); otherwise non-temporal loads, the faster way to stream
// data that will have been evicted before anyone reads it again.
template <bool KEEP>
__device__ __forceinline__ void celo2_stats_tile(const TDesc& d, const PyloTensorArgs& a, int task, float scale,
                                                 const EmaConsts& e, const float* f0, const float* f1,
                                                 float (&acc)[kNStat]) {
  constexpr int V = kTileV;
  const TileTask tk(d, task);
  float fb[V][4];
#pragma unroll
  for (int v = 0; v < V; ++v) load_vec_o<4>(f1 + v * 4, tk.col * 16u, fb[v]);
  const unsigned lo = (threadIdx.x & 63) * (V * 4u);
  const float *g = a.grad + tk.first, *p = a.param + tk.first, *m0 = a.mom + tk.first,
              *m1 = a.mom + d.n + tk.first, *m2 = a.mom + 2 * d.n + tk.first, *rms = a.rms + tk.first;
  const float* fr = f0 + (size_t)tk.r0 * 4;
#pragma unroll PYLO_STATS_UNROLL
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
      const float gg = clampf(xg[v] * scale, a.clip_val);
      float m[3] = {x0[v], x1[v], x2[v]};
      float rr = xr[v];
      ema_update(e, gg, m, rr);
      const float rfcf[3] = {fa[0] * fb[v][0], fa[1] * fb[v][1], fa[2] * fb[v][2]};
      float f[kNStat];
      lo_features(gg, xp[v], m, rr, rfcf, 1e-8f, f);
#pragma unroll
      for (int c = 0; c < kNStat; ++c) acc[c] = fmaf(f[c], f[c], acc[c]);
    }
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0; fr += 4;
  }
}

// One block of the statistics pass: sum of squares of the 18 per-element channels over the block's
// elements, with the accumulators advanced in registers only (nothing is written back); an AdamW tensor
// is updated completely instead.  Returns true when `red` holds the four waves' sums (after a barrier).
template <bool KEEP>
__device__ __forceinline__ bool celo2_stats_block(const TDesc& d, const PyloTensorArgs& a, const Item& it,
                                                  const float* __restrict__ fac_tab, const Globals* __restrict__ gl,
                                                  const PyloDecays& dec, float (*red)[kNStat]) {
  const float scale = clip_scale(gl->gnorm, a.clip_norm);
  const EmaConsts e = make_ema(dec);
  if (d.mode == kModeFlat) {
    if (d.adam_indep) {
      if (d.vec == 4) celo2_adam_indep_chunk<4>(d, a, it.a, scale, dec);
      else celo2_adam_indep_chunk<1>(d, a, it.a, scale, dec);
    } else {
      if (d.vec == 4) celo2_adam_chunk<4>(d, a, it.a, scale, e);
      else celo2_adam_chunk<1>(d, a, it.a, scale, e);
    }
    return false;
  }
  float acc[kNStat];
#pragma unroll
  for (int c = 0; c < kNStat; ++c) acc[c] = 0.0f;
  const float* f0 = fac_tab + d.fac_off[0];
  const float* f1 = fac_tab + d.fac_off[1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (d.tile_nct > 0) {
    const int task = it.a * 4 + __builtin_amdgcn_readfirstlane(wave);
    if (task < d.tile_ntask) celo2_stats_tile<KEEP>(d, a, task, scale, e, f0, f1, acc);
  } else if (d.vec == 4) {
    celo2_stats_chunk<4>(d, a, it.a, scale, e, f0, f1, acc);
  } else {
    celo2_stats_chunk<1>(d, a, it.a, scale, e, f0, f1, acc);
  }
#pragma unroll
  for (int c = 0; c < kNStat; ++c) {
    const float s = wave_sum(acc[c]);
    if (lane == 0) red[wave][c] = s;
  }
  __syncthreads();
  return true;
}

__device__ __forceinline__ double stats_block_total(const float (*red)[kNStat], int c) {
  return ((double)red[0][c] + (double)red[1][c]) + ((double)red[2][c] + (double)red[3][c]);
}

// Statistics pass as a launch of its own (each pass over all tensors; the fused element pass,
// k_celo2_elem, is the default).
__global__ __launch_bounds__(kThreads) void k_celo2_stats(const TDesc* __restrict__ descs,
                                                          const PyloTensorArgs* __restrict__ dyn,
                                                          const Item* __restrict__ items,
                                                          const float* __restrict__ fac_tab,
                                                          const Globals* __restrict__ gl, PyloDecays dec,
                                                          double* __restrict__ stats_part) {
  __shared__ float red[kWaves][kNStat];
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  if (!celo2_stats_block<false>(d, a, it, fac_tab, gl, dec, red)) return;
  if (threadIdx.x < kNStat)
    stats_part[(size_t)blockIdx.x * kStatW + stat_channel(threadIdx.x)] = stats_block_total(red, threadIdx.x);
}

// Per factored tensor: s_c = rsqrt(1e-9 + mean f_c^2) folded into the first-layer rows of the 18
// per-element channels; the remaining layers are copied behind them so the apply pass reads one
// contiguous block per tensor.  NT threads; `rows` are n_rows rows of kStatW doubles, added in a fixed
// order.  COH: the rows were written by other blocks of the running kernel and the results are for
// such blocks (see coh_store_wait).
template <int NT, bool COH>
__device__ __forceinline__ void celo2_fold_tensor(const TDesc& d, const double* __restrict__ rows, int n_rows,
                                                  const float* __restrict__ mlp, float* __restrict__ w,
                                                  float* __restrict__ chan_ms, double (*part)[kNStat],
                                                  float* scale_c) {
  constexpr int G = NT / kNStat;
  const int c = threadIdx.x % kNStat, gI = threadIdx.x / kNStat;
  if (gI < G) {
    double s = 0.0;
    if constexpr (COH) {
      // every load is a round trip to the memory side: sixteen are in flight before the first is added
      for (int b0 = gI; b0 < n_rows; b0 += 16 * G) {
        double v[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          const int b = b0 + q * G;
          v[q] = b < n_rows ? coh_load(rows + (size_t)b * kStatW + stat_channel(c)) : 0.0;
        }
#pragma unroll
        for (int q = 0; q < 16; ++q) s += v[q];
      }
    } else {
#pragma unroll 16
      for (int b = gI; b < n_rows; b += G) s += rows[(size_t)b * kStatW + stat_channel(c)];
    }
    part[gI][c] = s;
  }
  __syncthreads();
  if (threadIdx.x < kNStat) {
    double s = 0.0;
    for (int g2 = 0; g2 < G; ++g2) s += part[g2][threadIdx.x];
    const float ms = (float)(s / (double)d.n);
    chan_ms[(size_t)d.fac_slot * kNStat + threadIdx.x] = ms;
    scale_c[threadIdx.x] = rsq(1e-9f + ms);
  }
  __syncthreads();
  const float* w_in = mlp;                  // (30,8)
  const float* w_h = mlp + 240 + 8;         // (8,8)
  const float* b_h = w_h + 64;              // 8
  const float* w_out = b_h + 8;             // (8,3)
  const float* b_out = w_out + 24;          // 3
  for (int i = threadIdx.x; i < kC2Fold; i += NT) {
    float v;
    if (i < kC2WH) v = w_in[stat_channel(i / 8) * 8 + i % 8] * scale_c[i / 8];
    else if (i < kC2BH) v = w_h[i - kC2WH];
    else if (i < kC2WO) v = b_h[i - kC2BH];
    else if (i < kC2BO) v = ((i - kC2WO) % 4) < 2 ? w_out[((i - kC2WO) / 4) * 3 + ((i - kC2WO) % 4)] : 0.0f;
    else v = (i - kC2BO) < 2 ? b_out[i - kC2BO] : 0.0f;
    if constexpr (COH) coh_store_wait(w + i, v);
    else w[i] = v;
  }
}

__global__ __launch_bounds__(kFoldThreads) void k_celo2_fold(const TDesc* __restrict__ descs,
                                                             const PyloTensorArgs* __restrict__ dyn,
                                                             const int* __restrict__ fac_list,
                                                             const double* __restrict__ stats_part,
                                                             const double* __restrict__ seg_tot,
                                                             const float* __restrict__ mlp,
                                                             float* __restrict__ wfold, float* __restrict__ chan_ms) {
  __shared__ double part[kFoldThreads / kNStat][kNStat];
  __shared__ float scale_c[kNStat];
  const int t = fac_list[blockIdx.x];
  const TDesc d = descs[t];
  if (dyn[t].grad == nullptr) return;
  int n_rows;
  const double* rows = stat_rows(d, stats_part, seg_tot, n_rows);
  celo2_fold_tensor<kFoldThreads, false>(d, rows, n_rows, mlp, wfold + (size_t)d.fac_slot * kC2Fold, chan_ms, part, scale_c);
}

template <int V>
__device__ __forceinline__ void celo2_apply_chunk(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                  float scale, const EmaConsts& e, const float* f0,
                                                  const float* f1, const float* t0, const float* t1,
                                                  const float* wbase) {
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
  const bool use_exp = a.exp_mult != 0.0f;
  Cursor<V> cur(d, base);
  const ChunkPtrs cp(d, a, base);
  for (int it = 0; it < kElemIters; ++it, cur.advance()) {
    if (!cur.live()) break;
    ElemIn<V> x;
    load_elems_at<V>(d, a, cp, cur.off, cur.i0, cur.i1, scale, f0, f1, x);
    float f[V][kNStat], h[V][8];
    float m0[V], m1[V], m2[V];
    {
      float ta[8];
      load_row8(t0, cur.i0, ta);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        float tb[8];
        load_row8(t1 + v * 8, cur.i1, tb);
#pragma unroll
        for (int j = 0; j < 8; ++j) h[v][j] = ta[j] + tb[j];
      }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ema_update(e, x.g[v], x.m[v], x.rms[v]);
      m0[v] = x.m[v][0]; m1[v] = x.m[v][1]; m2[v] = x.m[v][2];
      lo_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.rfcf[v], 1e-8f, f[v]);
    }
    store_vec_o<V>(cp.m0, cur.off * 4u, m0);
    store_vec_o<V>(cp.m1, cur.off * 4u, m1);
    store_vec_o<V>(cp.m2, cur.off * 4u, m2);
    store_vec_o<V>(cp.rms, cur.off * 4u, x.rms);
    // The weights are wave-uniform: they are fetched through the scalar cache into SGPRs one input
    // row at a time and shared by the P elements processed together (channel-outer loop order).
    constexpr int P = V >= 2 ? 2 : 1;
    float out[V];
#pragma unroll
    for (int v0 = 0; v0 < V; v0 += P) {
      const cfloat* w = launder(wbase);
#pragma unroll
      for (int c = 0; c < kNStat; ++c) {
        float wc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) wc[j] = w[kC2W1 + c * 8 + j];
#pragma unroll
        for (int v = v0; v < v0 + P; ++v) {
#pragma unroll
          for (int j = 0; j < 8; ++j) h[v][j] = fmaf(f[v][c], wc[j], h[v][j]);
        }
      }
      float h1[P][8];
#pragma unroll
      for (int q = 0; q < P; ++q) {
#pragma unroll
        for (int j = 0; j < 8; ++j) { h[v0 + q][j] = fmaxf(h[v0 + q][j], 0.0f); h1[q][j] = w[kC2BH + j]; }
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        float wk[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) wk[j] = w[kC2WH + k * 8 + j];
#pragma unroll
        for (int q = 0; q < P; ++q) {
#pragma unroll
          for (int j = 0; j < 8; ++j) h1[q][j] = fmaf(h[v0 + q][k], wk[j], h1[q][j]);
        }
      }
#pragma unroll
      for (int q = 0; q < P; ++q) {
        float o0 = w[kC2BO + 0], o1 = w[kC2BO + 1];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float hk = fmaxf(h1[q][k], 0.0f);
          o0 = fmaf(hk, w[kC2WO + k * 4 + 0], o0);
          o1 = fmaf(hk, w[kC2WO + k * 4 + 1], o1);
        }
        out[v0 + q] = use_exp ? o0 * expf(o1 * a.exp_mult) : o0;
      }
    }
    store_vec_o<V>(cp.out, cur.off * 4u, out);
  }
}

#ifndef PYLO_MFMA_V
#define PYLO_MFMA_V 2
#endif
#ifndef PYLO_APPLY_WAVES
#define PYLO_APPLY_WAVES 4
#endif
constexpr int kMfmaV = PYLO_MFMA_V;   // elements per lane and iteration on the matrix-pipe path

// The same pass with the three layers on the matrix pipe (128-bit-aligned tensors only).  The folded
// weight block is 63 groups of four consecutive floats; lane l of register r holds float r*64 + l,
// so group v sits in lanes 4*(v%16).. of register v/16 and is selected with abid = v % 16.  Four
// VGPRs hold every weight.  Biases enter as a rank-1 update with the constant 1.
template <int V, bool COH>
__device__ __forceinline__ void celo2_apply_chunk_mfma(const TDesc& d, const PyloTensorArgs& a, int chunk,
                                                       float scale, const EmaConsts& e, const float* f0,
                                                       const float* f1, const float* t0, const float* t1,
                                                       const float* wbase) {
  const long long base = (long long)chunk * (kThreads * 4 * kElemIters);   // chunks are sized for vec == 4
  const bool use_exp = a.exp_mult != 0.0f;
  const float exp_scale = a.exp_mult * 1.44269504088896341f;
  const int lane = threadIdx.x & 63;
  float wreg[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) wreg[r] = COH ? coh_load(wbase + r * 64 + lane) : *(const gfloat*)(wbase + r * 64 + lane);
  constexpr int gWH = kC2WH / 4, gBH = kC2BH / 4, gWO = kC2WO / 4, gBO = kC2BO / 4;
  const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
  Cursor<V, 4> cur(d, base);
  const ChunkPtrs cp(d, a, base);
  for (int it = 0; it < Cursor<V, 4>::kIters; ++it, cur.advance()) {
    // no early exit: every lane of the wave must reach the matrix instructions; lanes past the end
    // work on the chunk's first element and store nothing
    const bool live = cur.live();
    const unsigned off = live ? cur.off : 0u, i0 = live ? cur.i0 : cur.c_i0, i1 = live ? cur.i1 : cur.c_i1;
    ElemIn<V> x;
    load_elems_at<V>(d, a, cp, off, i0, i1, scale, f0, f1, x);
    v4f ha[V], hb[V];
    {
      float ta[8];
      load_row8(t0, i0, ta);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        float tb[8];
        load_row8(t1 + v * 8, i1, tb);
#pragma unroll
        for (int j = 0; j < 4; ++j) { ha[v][j] = ta[j] + tb[j]; hb[v][j] = ta[4 + j] + tb[4 + j]; }
      }
    }
    float f[V][kNStat], m0[V], m1[V], m2[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ema_update(e, x.g[v], x.m[v], x.rms[v]);
      m0[v] = x.m[v][0]; m1[v] = x.m[v][1]; m2[v] = x.m[v][2];
      lo_features(x.g[v], x.p[v], x.m[v], x.rms[v], x.rfcf[v], 1e-8f, f[v]);
    }
    if (live) {
      store_vec_o<V>(cp.m0, off * 4u, m0);
      store_vec_o<V>(cp.m1, off * 4u, m1);
      store_vec_o<V>(cp.m2, off * 4u, m2);
      store_vec_o<V>(cp.rms, off * 4u, x.rms);
    }
    // layer 1: 18 rank-1 updates per half (hidden units 0-3 / 4-7)
#pragma unroll
    for (int c = 0; c < kNStat; ++c) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        ha[v] = mfma_w4(wreg[(2 * c) / 16], f[v][c], ha[v], (2 * c) % 16);
        hb[v] = mfma_w4(wreg[(2 * c + 1) / 16], f[v][c], hb[v], (2 * c + 1) % 16);
      }
    }
    // layer 2: bias, then 8 rank-1 updates per half
    v4f ga[V], gb[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ga[v] = mfma_w4(wreg[gBH / 16], 1.0f, zero, gBH % 16);
      gb[v] = mfma_w4(wreg[(gBH + 1) / 16], 1.0f, zero, (gBH + 1) % 16);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float hk = relu(k < 4 ? ha[v][k] : hb[v][k - 4]);
        ga[v] = mfma_w4(wreg[(gWH + 2 * k) / 16], hk, ga[v], (gWH + 2 * k) % 16);
        gb[v] = mfma_w4(wreg[(gWH + 2 * k + 1) / 16], hk, gb[v], (gWH + 2 * k + 1) % 16);
      }
    }
    // layer 3: the two outputs sit in elements 0 and 1 of the accumulator
    v4f o[V];
#pragma unroll
    for (int v = 0; v < V; ++v) o[v] = mfma_w4(wreg[gBO / 16], 1.0f, zero, gBO % 16);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float hk = relu(k < 4 ? ga[v][k] : gb[v][k - 4]);
        o[v] = mfma_w4(wreg[(gWO + k) / 16], hk, o[v], (gWO + k) % 16);
      }
    }
    float out[V];
#pragma unroll
    for (int v = 0; v < V; ++v)
      out[v] = use_exp ? o[v][0] * __builtin_amdgcn_exp2f(o[v][1] * exp_scale) : o[v][0];
    if (live) store_vec_o<V>(cp.out, off * 4u, out);
  }
}

// The matrix-pipe apply pass over one wave task of the column-resident walk: column factors and
// column terms stay in registers, row factors and row terms arrive through the scalar cache.
template <bool COH>
__device__ __forceinline__ void celo2_apply_tile(const TDesc& d, const PyloTensorArgs& a, int task, float scale,
                                                 const EmaConsts& e, const float* f0, const float* f1,
                                                 const float* t0, const float* t1, const float* wbase) {
  constexpr int V = kTileV;
  const TileTask tk(d, task);
  const bool use_exp = a.exp_mult != 0.0f;
  const float exp_scale = a.exp_mult * 1.44269504088896341f;
  const int lane = threadIdx.x & 63;
  float wreg[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) wreg[r] = COH ? coh_load(wbase + r * 64 + lane) : *(const gfloat*)(wbase + r * 64 + lane);
  constexpr int gWH = kC2WH / 4, gBH = kC2BH / 4, gWO = kC2WO / 4, gBO = kC2BO / 4;
  const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
  float fb[V][4], tb[V][8];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    load_vec_o<4>(f1 + v * 4, tk.col * 16u, fb[v]);
    load_row8(t1 + v * 8, tk.col, tb[v]);
  }
  const unsigned lo = lane * (V * 4u);
  const float *g = a.grad + tk.first, *p = a.param + tk.first;
  float *m0 = a.mom + tk.first, *m1 = a.mom + d.n + tk.first, *m2 = a.mom + 2 * d.n + tk.first,
        *rms = a.rms + tk.first, *out = a.step_out + tk.first;
  const float* fr = f0 + (size_t)tk.r0 * 4;
  const float* tr = t0 + (size_t)tk.r0 * 8;
  for (int r = tk.r0; r < tk.r1; ++r) {
    float xg[V], xp[V], x0[V], x1[V], x2[V], xr[V], fa[4], ta[8];
    load_vec_nt<V>(g, lo, xg);
    load_vec_nt<V>(p, lo, xp);
    load_vec_nt<V>(m0, lo, x0);
    load_vec_nt<V>(m1, lo, x1);
    load_vec_nt<V>(m2, lo, x2);
    load_vec_nt<V>(rms, lo, xr);
    load_uniform<4>(fr, fa);
    load_uniform<8>(tr, ta);
    float f[V][kNStat];
    v4f ha[V], hb[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const float gg = clampf(xg[v] * scale, a.clip_val);
      float m[3] = {x0[v], x1[v], x2[v]};
      ema_update(e, gg, m, xr[v]);
      x0[v] = m[0]; x1[v] = m[1]; x2[v] = m[2];
      const float rfcf[3] = {fa[0] * fb[v][0], fa[1] * fb[v][1], fa[2] * fb[v][2]};
      lo_features(gg, xp[v], m, xr[v], rfcf, 1e-8f, f[v]);
#pragma unroll
      for (int j = 0; j < 4; ++j) { ha[v][j] = ta[j] + tb[v][j]; hb[v][j] = ta[4 + j] + tb[v][4 + j]; }
    }
    store_vec_nt<V>(m0, lo, x0);
    store_vec_nt<V>(m1, lo, x1);
    store_vec_nt<V>(m2, lo, x2);
    store_vec_nt<V>(rms, lo, xr);
#pragma unroll
    for (int c = 0; c < kNStat; ++c) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        ha[v] = mfma_w4(wreg[(2 * c) / 16], f[v][c], ha[v], (2 * c) % 16);
        hb[v] = mfma_w4(wreg[(2 * c + 1) / 16], f[v][c], hb[v], (2 * c + 1) % 16);
      }
    }
    v4f ga[V], gb[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      ga[v] = mfma_w4(wreg[gBH / 16], 1.0f, zero, gBH % 16);
      gb[v] = mfma_w4(wreg[(gBH + 1) / 16], 1.0f, zero, (gBH + 1) % 16);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float hk = relu(k < 4 ? ha[v][k] : hb[v][k - 4]);
        ga[v] = mfma_w4(wreg[(gWH + 2 * k) / 16], hk, ga[v], (gWH + 2 * k) % 16);
        gb[v] = mfma_w4(wreg[(gWH + 2 * k + 1) / 16], hk, gb[v], (gWH + 2 * k + 1) % 16);
      }
    }
    v4f o[V];
#pragma unroll
    for (int v = 0; v < V; ++v) o[v] = mfma_w4(wreg[gBO / 16], 1.0f, zero, gBO % 16);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float hk = relu(k < 4 ? ga[v][k] : gb[v][k - 4]);
        o[v] = mfma_w4(wreg[(gWO + k) / 16], hk, o[v], (gWO + k) % 16);
      }
    }
    float res[V];
#pragma unroll
    for (int v = 0; v < V; ++v)
      res[v] = use_exp ? o[v][0] * __builtin_amdgcn_exp2f(o[v][1] * exp_scale) : o[v][0];
    store_vec_nt<V>(out, lo, res);
    g += d.C0; p += d.C0; m0 += d.C0; m1 += d.C0; m2 += d.C0; rms += d.C0; out += d.C0;
    fr += 4; tr += 8;
  }
}

// One block of the apply pass: accumulators advanced and written, features, MLP, raw step.
// COH: the tensor's folded weights were written by another block of the running kernel.
template <bool MFMA, bool COH>
__device__ __forceinline__ void celo2_apply_block(const TDesc& d, const PyloTensorArgs& a, const Item& it,
                                                  const float* __restrict__ fac_tab,
                                                  const float* __restrict__ term_tab, const Globals* __restrict__ gl,
                                                  const PyloDecays& dec, const float* __restrict__ wfold) {
  const float scale = clip_scale(gl->gnorm, a.clip_norm);
  const EmaConsts e = make_ema(dec);
  const float* w = wfold + (size_t)d.fac_slot * kC2Fold;
  if (MFMA && d.tile_nct > 0) {
    const int task = it.a * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (task < d.tile_ntask)
      celo2_apply_tile<COH>(d, a, task, scale, e, fac_tab + d.fac_off[0], fac_tab + d.fac_off[1],
                            term_tab + d.term_off[0], term_tab + d.term_off[1], w);
  } else if (MFMA && d.vec == 4)
    celo2_apply_chunk_mfma<kMfmaV, COH>(d, a, it.a, scale, e, fac_tab + d.fac_off[0], fac_tab + d.fac_off[1],
                                        term_tab + d.term_off[0], term_tab + d.term_off[1], w);
  else if (d.vec == 4)
    celo2_apply_chunk<4>(d, a, it.a, scale, e, fac_tab + d.fac_off[0], fac_tab + d.fac_off[1],
                         term_tab + d.term_off[0], term_tab + d.term_off[1], w);
  else
    celo2_apply_chunk<1>(d, a, it.a, scale, e, fac_tab + d.fac_off[0], fac_tab + d.fac_off[1],
                         term_tab + d.term_off[0], term_tab + d.term_off[1], w);
}

// Apply pass as a launch of its own (see k_celo2_stats).
template <bool MFMA>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PYLO_APPLY_WAVES))) void k_celo2_apply(const TDesc* __restrict__ descs,
                                                          const PyloTensorArgs* __restrict__ dyn,
                                                          const Item* __restrict__ items,
                                                          const float* __restrict__ fac_tab,
                                                          const float* __restrict__ term_tab,
                                                          const Globals* __restrict__ gl, PyloDecays dec,
                                                          const float* __restrict__ wfold) {
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  if (d.mode == kModeFlat) return;
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  celo2_apply_block<MFMA, false>(d, a, it, fac_tab, term_tab, gl, dec, wfold);
}

// ---------------------------------------------------------------------------------------------
// The fused element pass: statistics, weight folding and apply pass of every tensor in ONE launch.
//
// The plan orders the items slab by slab (a slab is a run of whole tensors of a few million elements):
//   stats(slab 0) stats(slab 1) stats(slab 2) apply(slab 0) stats(slab 3) apply(slab 1) ...
// Blocks are dispatched in index order, so at any time the GPU works on the statistics of one slab
// and on the apply items of the slab two before it, whose six input streams (24 of the apply pass's 44
// bytes per element) are then still in the 256 MB memory-side cache: they are read from HBM once
// instead of twice.  A launch per slab and pass does not get there: a slab fills a fraction of the
// GPU, and every launch boundary drains it.
//
// What makes one launch possible is a hand-over between running blocks, per tensor:
//   - a statistics block leaves its row of partial sums with coh_store_wait and then counts itself in
//     (sync[t], an agent-scope atomic); the block that completes the count folds the tensor's weights
//     (rows added in index order, whichever block comes last: results stay bit-reproducible), leaves
//     them the same way and raises sync[T + t];
//   - an apply block polls that flag first.  Every block it can be waiting for has a lower index, was
//     therefore dispatched earlier and waits for nothing itself, so the wait ends; the plan puts two
//     slabs of statistics items (hundreds of blocks, tens of microseconds) between a tensor's last
//     statistics item and its first apply item, so it rarely begins.  A block that has polled
//     kSpinLimit times (seconds) gives up and writes NaN steps, which no caller can overlook,
//     rather than hang the GPU.
// k_gnorm zeroes `sync` before every launch.
// ---------------------------------------------------------------------------------------------
template <bool MFMA>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PYLO_APPLY_WAVES))) void k_celo2_elem(
    const TDesc* __restrict__ descs, const PyloTensorArgs* __restrict__ dyn, const Item* __restrict__ items,
    const float* __restrict__ fac_tab, const float* __restrict__ term_tab, const Globals* __restrict__ gl,
    PyloDecays dec, const float* __restrict__ mlp, float* __restrict__ wfold, float* __restrict__ chan_ms,
    double* __restrict__ stats_part, int* __restrict__ sync, int n_tensors) {
  __shared__ float red[kWaves][kNStat];
  __shared__ double part[kThreads / kNStat][kNStat];
  __shared__ float scale_c[kNStat];
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
      celo2_apply_block<MFMA, true>(d, a, it, fac_tab, term_tab, gl, dec, wfold);
    } else {
      // gave up: NaN steps for this block's elements (tile items: the wave tasks' rows; else the chunk)
      const float nan = __builtin_nanf("");
      if (d.tile_nct > 0) {
        const int task = it.a * 4 + (threadIdx.x >> 6);
        if (task < d.tile_ntask) {
          const TileTask tk(d, task);
          for (int r = tk.r0; r < tk.r1; ++r)
            for (int v = 0; v < kTileV; ++v) a.step_out[(size_t)r * d.C0 + tk.col + v] = nan;
        }
      } else {
        const long long chunk = (long long)kThreads * d.vec * kElemIters, base = (long long)it.a * chunk;
        for (long long i = base + threadIdx.x; i < base + chunk && i < d.n; i += kThreads) a.step_out[i] = nan;
      }
    }
    return;
  }
  const bool counted = (it.c & kElemKeep) ? celo2_stats_block<true>(d, a, it, fac_tab, gl, dec, red)
                                          : celo2_stats_block<false>(d, a, it, fac_tab, gl, dec, red);
  if (!counted) return;
  if (threadIdx.x < kNStat)
    coh_store_wait(stats_part + (size_t)it.b * kStatW + stat_channel(threadIdx.x), stats_block_total(red, threadIdx.x));
  __syncthreads();   // every row entry of this block has been performed
  if (threadIdx.x == 0)
    s_flag = __hip_atomic_fetch_add(sync + it.tensor, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == d.nblk - 1;
  __syncthreads();
  if (!s_flag) return;
  // the tensor's last statistics block: fold its weights
  celo2_fold_tensor<kThreads, true>(d, stats_part + (size_t)d.blk0 * kStatW, d.nblk, mlp,
                                    wfold + (size_t)d.fac_slot * kC2Fold, chan_ms, part, scale_c);
  __syncthreads();   // every folded weight has been performed
  if (threadIdx.x == 0) __hip_atomic_store(sync + n_tensors + it.tensor, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------------
// Finishing pass of ELO-CELO2 (after Newton-Schulz): x = step_out,
//   step = x * rsqrt(1e-9 + mean x^2) * rmsmult;  p <- p - lr * (step + wd * p)
// (CELO2_naive.py:54-56, ELO_CELO2_cuda.py:294-296).  Linear 8192-element blocks.
// ---------------------------------------------------------------------------------------------
constexpr int kFinElems = kThreads * 4 * kElemIters;

// Where the finishing pass finds a tensor's step: `step_out`, or -- for a tensor the same call has
// orthogonalised with an odd number of Newton-Schulz iterations -- the second X buffer in the workspace
// (x_alt[tensor] floats into `ws`; x_alt == nullptr: always `step_out`).
__device__ __forceinline__ const float* fin_source(const PyloTensorArgs& a, int tensor, const long long* x_alt,
                                                   const float* ws) {
  if (x_alt != nullptr && (a.flags & PYLO_ARG_ORTHOGONALIZE) && x_alt[tensor] >= 0) return ws + x_alt[tensor];
  return a.step_out;
}

__global__ __launch_bounds__(kThreads) void k_celo2_sumsq(const FinUnit* __restrict__ units,
                                                          const PyloTensorArgs* __restrict__ dyn,
                                                          const Item* __restrict__ items,
                                                          double* __restrict__ fin_part,
                                                          const long long* __restrict__ x_alt,
                                                          const float* __restrict__ ws) {
  __shared__ float red[kWaves];
  const Item it = items[blockIdx.x];
  const FinUnit u = units[it.tensor];
  const PyloTensorArgs a = dyn[u.tensor];
  if (a.grad == nullptr) return;
  const long long base = (long long)it.a * kFinElems;
  const long long left = u.n - base;
  const unsigned lim = left < (long long)kFinElems ? (unsigned)left : (unsigned)kFinElems;
  const float* x = fin_source(a, u.tensor, x_alt, ws) + u.off + base;
  float s = 0.0f;
  if (u.vec) {
#pragma unroll
    for (int i = 0; i < kElemIters; ++i) {
      const unsigned off = (i * kThreads + threadIdx.x) * 4u;
      if (off < lim) {
        float v[4];
        load_vec_nt<4>(x, off * 4u, v);
        s += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
      }
    }
  } else {
    for (unsigned off = threadIdx.x; off < lim; off += kThreads) {
      const float v = *(const gfloat*)(x + off);
      s = fmaf(v, v, s);
    }
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0)
    fin_part[blockIdx.x] = ((double)red[0] + (double)red[1]) + ((double)red[2] + (double)red[3]);
}

__global__ __launch_bounds__(kThreads) void k_celo2_finscale(const FinUnit* __restrict__ units,
                                                             const PyloTensorArgs* __restrict__ dyn,
                                                             const double* __restrict__ fin_part,
                                                             float* __restrict__ fin_scale) {
  __shared__ double red[kWaves];
  const int t = blockIdx.x;  // one block per unit: a tensor, or a slice of the last two dims of one with more
  const FinUnit d = units[t];
  if (dyn[d.tensor].grad == nullptr || d.nblk == 0) return;
  double s = 0.0;
#pragma unroll 8
  for (int b = threadIdx.x; b < d.nblk; b += kThreads) s += fin_part[d.blk0 + b];
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float ms = (float)(((red[0] + red[1]) + (red[2] + red[3])) / (double)d.n);
    fin_scale[t] = rsq(1e-9f + ms);
  }
}

__global__ __launch_bounds__(kThreads) void k_celo2_update(const FinUnit* __restrict__ units,
                                                           const TDesc* __restrict__ descs,
                                                           const PyloTensorArgs* __restrict__ dyn,
                                                           const Item* __restrict__ items,
                                                           const float* __restrict__ fin_scale,
                                                           const long long* __restrict__ x_alt,
                                                           const float* __restrict__ ws) {
  const Item it = items[blockIdx.x];
  const FinUnit u = units[it.tensor];
  const PyloTensorArgs a = dyn[u.tensor];
  if (a.grad == nullptr) return;
  const int store = descs[u.tensor].store;
  const long long base = u.off + (long long)it.a * kFinElems;
  const long long left = u.n - (long long)it.a * kFinElems;
  const unsigned lim = left < (long long)kFinElems ? (unsigned)left : (unsigned)kFinElems;
  const float* x = fin_source(a, u.tensor, x_alt, ws) + base;
  float* p = a.param + base;
  const float sc = fin_scale[it.tensor], rm = a.step_mult, wd = a.weight_decay, nlr = -a.lr;
  if (store != 0) {
    // the parameter in its storage type (fp16, bf16, fp64): widened, updated in fp32, rounded to nearest-even
    for (unsigned off = threadIdx.x; off < lim; off += kThreads) {
      const float v = *(const gfloat*)(x + off), q = load_stored(a.param, base + off, store);
      store_stored(a.param, base + off, store, fmaf(nlr, (v * sc) * rm + wd * q, q));
    }
    return;
  }
  if (u.vec) {
#pragma unroll
    for (int i = 0; i < kElemIters; ++i) {
      const unsigned off = (i * kThreads + threadIdx.x) * 4u;
      if (off < lim) {
        float v[4], q[4];
        load_vec_nt<4>(x, off * 4u, v);
        load_vec_o<4>(p, off * 4u, q);
#pragma unroll
        for (int j = 0; j < 4; ++j) q[j] = fmaf(nlr, (v[j] * sc) * rm + wd * q[j], q[j]);
        store_vec_o<4>(p, off * 4u, q);
      }
    }
  } else {
    for (unsigned off = threadIdx.x; off < lim; off += kThreads) {
      const float v = *(const gfloat*)(x + off), q = *(const gfloat*)(p + off);
      *(gfloat*)(p + off) = fmaf(nlr, (v * sc) * rm + wd * q, q);
    }
  }
}

}  // namespace pylo
