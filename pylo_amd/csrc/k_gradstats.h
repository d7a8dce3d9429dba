// Gradient statistics shared by the three optimizers: row / column sums of g^2 (P0), the global
// gradient norm, and the Adafactor row / column vectors with everything derived from them (V0).
#pragma once

#include "pylo_common.h"

namespace pylo {

// =============================================================================================
// P0: row / column sums of g^2 for 2-D factored tensors; sum g^2 and clamp flag for everything
// =============================================================================================
// |x|; NaN counts as infinity on tensors whose NaNs are replaced (fmaxf alone would drop it), so
// that the flag for the exact pass is raised.
__device__ __forceinline__ float abs_or_inf(float x, int nan0) {
  const float ax = fabsf(x);
  return (nan0 && ax != ax) ? __builtin_inff() : ax;
}

template <int V, bool exact>
__device__ __forceinline__ void p0_factored(const TDesc& d, const float* g, int strip, int cb,
                                            float scale, float clipv, int nan0, float* __restrict__ rowpart,
                                            float* __restrict__ colpart, float* lds_col, float* lds_row,
                                            float& gsq, float& amax) {
  constexpr int TC = 64 * V;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int C0 = d.C0, R0 = d.R0;
  const int r0 = strip * kP0Rows;
  const int r1 = min(R0, r0 + kP0Rows);
  const int c = cb * TC + lane * V;
  const bool in = c < C0;  // V == 4 implies C0 % 4 == 0, so the whole vector is in or out
  float col[V];
#pragma unroll
  for (int v = 0; v < V; ++v) col[v] = 0.0f;
  // Four rows per wave and trip (rows rb, rb+4, rb+8, rb+12): the loads are independent and issued
  // together, and the four row sums are reduced jointly.  lds_row is [wave][trip][16-lane group][u].
  // The next trip's loads are issued before this trip's values are worked on (eight 16-byte loads a lane in
  // flight).  Measured, it does not change the pass's time inside a step (0.125 ms where a bare streaming kernel
  // reads the same bytes in 0.07 - 0.08 ms): what holds it back there is the write-back of the lines that the
  // kernels before it left dirty, not the bytes it has in flight.
  const float* gc = g + (in ? c : 0);
  auto load_trip = [&](int rb, float (&x)[4][V]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int r = rb + u * kWaves;
      load_vec<V>(gc + (size_t)(r < r1 ? r : rb) * C0, x[u]);
    }
  };
  int trip = 0;
  float x[4][V], xn[4][V];
  if (r0 + wave < r1) load_trip(r0 + wave, x);
  for (int rb = r0 + wave; rb < r1; rb += 4 * kWaves, ++trip) {
    const bool more = rb + 4 * kWaves < r1;
    if (more) load_trip(rb + 4 * kWaves, xn);
    float rs[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool live = in && rb + u * kWaves < r1;
      float sq[V];
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float raw = live ? x[u][v] : 0.0f;
        amax = fmaxf(amax, abs_or_inf(raw, nan0));
        if (exact) gsq = fmaf(raw, raw, gsq);
        const float y = exact ? cond_grad(raw, scale, clipv, nan0) : raw;
        sq[v] = y * y;
        col[v] += sq[v];
      }
      if constexpr (V == 4) rs[u] = (sq[0] + sq[1]) + (sq[2] + sq[3]);
      else rs[u] = sq[0];
      if (!exact) gsq += rs[u];
    }
    const float tot = reduce4_rows16(rs[0], rs[1], rs[2], rs[3]);
    if ((lane & 12) == 0) lds_row[((wave * (kP0Rows / 16) + trip) * 4 + (lane >> 4)) * 4 + (lane & 3)] = tot;
    if (more) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int v = 0; v < V; ++v) x[u][v] = xn[u][v];
    }
  }
#pragma unroll
  for (int v = 0; v < V; ++v) lds_col[wave * TC + lane * V + v] = col[v];
  __syncthreads();
  for (int j = threadIdx.x; j < TC; j += kThreads) {
    const float s = ((lds_col[j] + lds_col[TC + j]) + lds_col[2 * TC + j]) + lds_col[3 * TC + j];
    const int cc = cb * TC + j;
    if (cc < C0) colpart[(size_t)strip * C0 + cc] = s;
  }
  for (int j = threadIdx.x; j < r1 - r0; j += kThreads) {
    // row r0 + j was handled by wave j % 4 in trip (j / 4) / 4 as its row u = (j / 4) % 4
    const int w = j % kWaves, q = j / kWaves;
    const float* t = lds_row + ((w * (kP0Rows / 16) + q / 4) * 4) * 4 + (q % 4);
    rowpart[(size_t)cb * R0 + r0 + j] = (t[0] + t[4]) + (t[8] + t[12]);
  }
}

template <int V>
__device__ __forceinline__ void p0_flat(const TDesc& d, const float* g, int chunk, float& gsq, float& amax) {
  const int nan0 = d.nan0;
  const long long base = (long long)chunk * (kThreads * V * kElemIters);
#pragma unroll
  for (int it = 0; it < kElemIters; ++it) {
    const long long e = base + (long long)(it * kThreads + threadIdx.x) * V;
    if (e < d.n) {
      float x[V];
      load_vec<V>(g + e, x);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        gsq = fmaf(x[v], x[v], gsq);
        amax = fmaxf(amax, abs_or_inf(x[v], nan0));
      }
    }
  }
}

// Sums of g^2 of a tensor with more than two dims over one of its two factored dims, one block per
// (chunk of 64 entries, slab of kNdX positions along the removed dim); used by k_p0_nd and, when no
// global norm has to be known first, by the tail blocks of k_p0.  `lds` holds kWaves * 64 floats.
__device__ __forceinline__ void p0_nd_block(const TDesc* __restrict__ descs, const PyloTensorArgs* __restrict__ dyn,
                                            const Item it, float* __restrict__ part,
                                            const Globals* __restrict__ gl, float* lds) {
  static_assert(kV0aEnt == 64, "one lane per entry");
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  const int w = it.b;
  const int e = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int i = it.a * kV0aEnt + e;
  const int X = pick(d.nd_size, w), sX = pick(d.nd_stride, w);
  const float scale = grad_scale(d, a, gl, it.tensor);
  float s = 0.0f;
  if (i < pick(d.len, w)) {
    const long long base = (long long)(i / sX) * X * sX + (i % sX);
    const int x0 = it.c * kNdX + grp * (kNdX / kWaves);
    const int x1 = min(X, x0 + kNdX / kWaves);
    for (int x = x0; x < x1; ++x) {
      const float g = cond_grad(*(const gfloat*)(a.grad + base + (long long)x * sX), scale, a.clip_val, d.nan0);
      s = fmaf(g, g, s);
    }
  }
  lds[grp * kV0aEnt + e] = s;
  __syncthreads();
  if (grp == 0 && i < pick(d.len, w))
    part[pick(d.part_off, w) + (size_t)it.c * pick(d.len, w) + i] =
        ((lds[e] + lds[kV0aEnt + e]) + lds[2 * kV0aEnt + e]) + lds[3 * kV0aEnt + e];
}

// pass 0: tensors with clip_norm > 0 are summed raw (the scale factors out of g^2) and flag
//         elements beyond the clamp; tensors without global-norm clipping are clamped directly.
// pass 1: only if the flag was raised: redo clip_norm > 0 tensors with scale and clamp applied.
__global__ __launch_bounds__(kThreads) void k_p0(const TDesc* __restrict__ descs,
                                                 const PyloTensorArgs* __restrict__ dyn,
                                                 const Item* __restrict__ items, float* __restrict__ part,
                                                 double* __restrict__ gsq_part, int* __restrict__ flag_part,
                                                 const Globals* __restrict__ gl, int pass,
                                                 const Item* __restrict__ nd_items, int n_main) {
  __shared__ float lds_col[kWaves * 256];
  __shared__ float lds_row[kWaves * (kP0Rows / 16) * 16];
  __shared__ float lds_red[kWaves];
  __shared__ int lds_flag[kWaves];
  // blocks past the main items: the N-D tensors' sums, when the launcher appended them (it does when
  // no tensor is clipped by the global norm, which they would have to wait for)
  if ((int)blockIdx.x >= n_main) {
    p0_nd_block(descs, dyn, nd_items[blockIdx.x - n_main], part, gl, lds_col);
    return;
  }
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  const bool clip_on = a.clip_norm > 0.0f;
  if (pass == 1 && (!clip_on || d.mode != kModeFac2D || gl->flag == 0)) return;
  float gsq = 0.0f, amax = 0.0f;
  if (a.grad != nullptr) {
    if (d.mode == kModeFac2D) {
      const bool exact = (pass == 1) || !clip_on;
      const float scale = (pass == 1) ? grad_scale(d, a, gl, it.tensor) : 1.0f;
      float* p0r = part + d.part_off[0];
      float* p0c = part + d.part_off[1];
      if (d.vec == 4 && exact) p0_factored<4, true>(d, a.grad, it.a, it.b, scale, a.clip_val, d.nan0, p0r, p0c, lds_col, lds_row, gsq, amax);
      else if (d.vec == 4) p0_factored<4, false>(d, a.grad, it.a, it.b, scale, a.clip_val, d.nan0, p0r, p0c, lds_col, lds_row, gsq, amax);
      else if (exact) p0_factored<1, true>(d, a.grad, it.a, it.b, scale, a.clip_val, d.nan0, p0r, p0c, lds_col, lds_row, gsq, amax);
      else p0_factored<1, false>(d, a.grad, it.a, it.b, scale, a.clip_val, d.nan0, p0r, p0c, lds_col, lds_row, gsq, amax);
    } else {
      if (d.vec == 4) p0_flat<4>(d, a.grad, it.a, gsq, amax);
      else p0_flat<1>(d, a.grad, it.a, gsq, amax);
    }
  }
  if (pass == 1) return;
  gsq = wave_sum(gsq);
  // some element lies beyond the clamp (fmaxf drops NaNs, which therefore never raise the flag)
  const int flag = __any(a.clip_val > 0.0f && !(amax <= a.clip_val)) ? 1 : 0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { lds_red[wave] = gsq; lds_flag[wave] = flag; }
  __syncthreads();
  if (threadIdx.x == 0) {
    gsq_part[blockIdx.x] = ((double)lds_red[0] + (double)lds_red[1]) + ((double)lds_red[2] + (double)lds_red[3]);
    flag_part[blockIdx.x] = (clip_on && (lds_flag[0] | lds_flag[1] | lds_flag[2] | lds_flag[3])) ? 1 : 0;
  }
}

// use_flags == 0: the caller has shown that no element can exceed its clamp after scaling (the scaled
// gradient is bounded by clip_norm), so the exact pass never runs and the flags are ignored.
__global__ __launch_bounds__(kThreads) void k_gnorm(const double* __restrict__ gsq_part,
                                                    const int* __restrict__ flag_part, int nblk,
                                                    Globals* __restrict__ gl, int use_flags,
                                                    int* __restrict__ sync, int n_sync) {
  __shared__ double red[kWaves];
  __shared__ int fred[kWaves];
  // the counters and flags of the fused element pass that follows (k_celo2_elem) start at zero
  for (int i = threadIdx.x; i < n_sync; i += kThreads) sync[i] = 0;
  double s = 0.0;
  int f = 0;
  // sixteen partials are fetched before the first is added: the one block is bound by load latency
  for (int i0 = threadIdx.x; i0 < nblk; i0 += 16 * kThreads) {
    double sv[16];
    int fv[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int i = i0 + q * kThreads;
      sv[q] = i < nblk ? gsq_part[i] : 0.0;
      fv[q] = i < nblk ? flag_part[i] : 0;
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) { s += sv[q]; f |= fv[q]; }
  }
  s = wave_sum(s);
  f = __any(f) ? 1 : 0;
  if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = s; fred[threadIdx.x >> 6] = f; }
  __syncthreads();
  if (threadIdx.x == 0) {
    gl->gnorm = (float)sqrt((red[0] + red[1]) + (red[2] + red[3]));
    gl->flag = use_flags ? (fred[0] | fred[1] | fred[2] | fred[3]) : 0;
  }
}

// Per-tensor norm clipping (PYLO_F_TENSOR_NORM; AdafacLO_naive.py:199-200 calls torch.nn.utils.clip_grad_norm_
// on each parameter by itself): one block per tensor adds up the tensor's sum-of-squares partials in a fixed
// order and leaves  min(1, clip_norm / (norm + 1e-6))  in tscale[t], torch's clip coefficient.  Such tensors
// carry no clamp (the launcher checks), so the exact pass never runs: flag = 0.
__global__ __launch_bounds__(kThreads) void k_tnorm(const TDesc* __restrict__ descs,
                                                    const PyloTensorArgs* __restrict__ dyn,
                                                    const double* __restrict__ gsq_part, Globals* __restrict__ gl,
                                                    float* __restrict__ tscale) {
  __shared__ double red[kWaves];
  const int t = blockIdx.x;
  if (t == 0 && threadIdx.x == 0) {
    gl->gnorm = 0.0f;
    gl->flag = 0;
    gl->tscale = tscale;
  }
  const int first = descs[t].p0_first, n = descs[t].p0_n;
  const float clip = dyn[t].clip_norm;
  double s = 0.0;
  for (int i0 = threadIdx.x; i0 < n; i0 += 16 * kThreads) {
    double sv[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int i = i0 + q * kThreads;
      sv[q] = i < n ? gsq_part[first + i] : 0.0;
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) s += sv[q];
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float norm = (float)sqrt((red[0] + red[1]) + (red[2] + red[3]));
    const float c = clip / (norm + 1e-6f);
    tscale[t] = clip > 0.0f ? (c > 1.0f ? 1.0f : c) : 1.0f;   // a NaN norm gives a NaN factor, as torch.clamp does
  }
}

// =============================================================================================
// Sums of g^2 over one dim of an N-D tensor (any two factored dims): a block takes 64 entries of
// the statistics vector and 64 positions of the removed dim and writes one partial row; k_v0a adds
// the partial rows up.  Small tensors only (conv kernels, cls tokens); runs after the global norm is
// known and takes the sums of the conditioned gradient directly.
// =============================================================================================
__global__ __launch_bounds__(kThreads) void k_p0_nd(const TDesc* __restrict__ descs,
                                                    const PyloTensorArgs* __restrict__ dyn,
                                                    const Item* __restrict__ items, float* __restrict__ part,
                                                    const Globals* __restrict__ gl) {
  __shared__ float lds[kWaves * kV0aEnt];
  p0_nd_block(descs, dyn, items[blockIdx.x], part, gl, lds);
}

// =============================================================================================
// First stage of the per-tensor reduction of the statistics partials, for tensors with thousands
// of rows: one block adds up kSegRows rows, so that the per-tensor block that follows (one block,
// hence one CU's bandwidth) reads a few dozen rows instead of thousands.  Fixed order throughout.
// Item: tensor, first row (relative to the tensor's rows), number of rows.
// =============================================================================================
__global__ __launch_bounds__(kThreads) void k_stat_segsum(const TDesc* __restrict__ descs,
                                                          const Item* __restrict__ items,
                                                          const double* __restrict__ stats_part,
                                                          double* __restrict__ seg_tot) {
  constexpr int G = kThreads / kStatW;  // 6 groups x 40 channels
  __shared__ double part[G][kStatW];
  const Item it = items[blockIdx.x];
  const int blk0 = descs[it.tensor].blk0 + it.a;
  const int c = threadIdx.x % kStatW, gI = threadIdx.x / kStatW;
  if (gI < G) {
    double s = 0.0;
    for (int b0 = gI; b0 < it.b; b0 += 16 * G) {
      double v[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int b = b0 + q * G;
        v[q] = b < it.b ? stats_part[(size_t)(blk0 + b) * kStatW + c] : 0.0;
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) s += v[q];
    }
    part[gI][c] = s;
  }
  __syncthreads();
  if (threadIdx.x < kStatW) {
    double s = 0.0;
#pragma unroll
    for (int g2 = 0; g2 < G; ++g2) s += part[g2][threadIdx.x];
    seg_tot[(size_t)blockIdx.x * kStatW + threadIdx.x] = s;
  }
}

// =============================================================================================
// V0a: one block per 64 entries of a statistics vector.  Finishes the sums of g^2 over the
// partials, advances the three Adafactor accumulators (ELO_CELO2_naive.py:152-160) and leaves
// per-block partial sums of  f, f^2, rsqrt(f+1e-8)^2  per decay.
// =============================================================================================
__global__ __launch_bounds__(kV0aThreads) void k_v0a(const TDesc* __restrict__ descs,
                                                  const PyloTensorArgs* __restrict__ dyn,
                                                  const Item* __restrict__ items,
                                                  const float* __restrict__ part,
                                                  const Globals* __restrict__ gl, PyloDecays dec,
                                                  double* __restrict__ v0part) {
  constexpr int G = kV0aThreads / 64;
  __shared__ double lds[G][kV0aEnt];
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  const int which = it.b;
  const int len = pick(d.len, which);
  const int npart = pick(d.npart, which);
  const float* pp = part + pick(d.part_off, which);
  const int e = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int i = it.a * kV0aEnt + e;
  const int k = grp;  // after the sums: waves 0..2 take one decay each
  // everything the second half needs from memory is requested before the partial sums are read, so that
  // the block pays one memory round trip instead of two (kernels start with cold caches)
  const bool is_r = (which == 0) == (d.vec0_is_r != 0);
  float* fac = is_r ? a.fac_r : a.fac_c;
  float fac_old = 0.0f;
  if (k < 3 && i < len) fac_old = *(const gfloat*)(fac + (size_t)k * len + i);
  double s2 = 1.0;
  if (a.clip_norm > 0.0f && gl->flag == 0 && d.mode == kModeFac2D) {  // other modes sum the scaled gradient
    const float sc = grad_scale(d, a, gl, it.tensor);
    s2 = (double)sc * (double)sc;
  }
  {
    double s = 0.0;
    if (i < len) {
#pragma unroll 8
      for (int q = grp; q < npart; q += G) s += (double)*(const gfloat*)(pp + (size_t)q * len + i);
    }
    lds[grp][e] = s;
  }
  __syncthreads();
  if (k >= 3) return;
  double s_f = 0.0, s_ff = 0.0, s_rr = 0.0;
  if (i < len) {
    double S = 0.0;
#pragma unroll
    for (int q = 0; q < G; ++q) S += lds[q][e];
    const float q = (float)(s2 * S / (double)pick(d.sumlen, which)) + 1e-30f;
    const float beta = dec.beta_fac[k];
    const float f = beta * fac_old + (1.0f - beta) * q;
    fac[(size_t)k * len + i] = f;
    const float rq = rsq(f + 1e-8f);
    s_f = (double)f;
    s_ff = (double)f * (double)f;
    s_rr = (double)rq * (double)rq;
  }
  s_f = wave_sum(s_f);
  s_ff = wave_sum(s_ff);
  s_rr = wave_sum(s_rr);
  if (e == 0) {
    double* o = v0part + (size_t)blockIdx.x * kNV0 + k * 3;
    o[0] = s_f; o[1] = s_ff; o[2] = s_rr;
  }
}

// Where entry i of vector `which` of tensor d lives in the factor / term tables.
__device__ __forceinline__ size_t fac_index(const TDesc& d, int which, int k, int i) {
  return (size_t)pick(d.fac_off, which) + (size_t)i * 4 + k;   // [entry][4]: one 16-byte access per entry
}
template <int H>
__device__ __forceinline__ size_t term_index(const TDesc& d, int which, int j, int i) {
  return (size_t)pick(d.term_off, which) + (size_t)i * H + j;   // [entry][H]
}

// Row_factor / col_factor of one entry, and the two normalised broadcast features it carries
// (accumulator value and rsqrt(value + 1e-8)).  ELO_CELO2_naive.py:161-164,202-213
// rcm: row_col_mean per decay; s0 / s1: normalisation scales of the vector's two broadcast channels.
// (They arrive as plain arrays: indexing a BScale held in registers with `is_r ? k : 3 + k` makes the
// compiler move the struct to LDS, 64 bytes a thread with bank conflicts on every access.)
// fv: the entry's three accumulator values (fac[k * len + i]), loaded by the caller.
__device__ __forceinline__ void vector_entry(const TDesc& d, bool is_r, const float* fac, int len, int i,
                                             const float (&fv)[3], const float (&rcm3)[3], const float (&s0)[3],
                                             const float (&s1)[3], float (&fct)[3], float (&x0)[3], float (&x1)[3],
                                             const float* rcm_slices = nullptr, int slice = 0) {
  float rcm[3] = {rcm3[0], rcm3[1], rcm3[2]};
  if (is_r && d.mode == kModeFacND) {  // mean over the dc axis of this entry's slice of fac_r
    if (rcm_slices != nullptr) {       // the block has it in its per-slice table
#pragma unroll
      for (int k = 0; k < 3; ++k) rcm[k] = rcm_slices[k * kRcmSlots + slice];
    } else {
      const int sz = d.rcm_size, st = d.rcm_stride;
      const int base = (i / (sz * st)) * (sz * st) + i % st;
      double s[3] = {0.0, 0.0, 0.0};
      // sixteen positions of all three decays are requested before any is added (addresses clamped,
      // values past the end dropped afterwards, so that the loads stay unconditional)
      for (int xb = 0; xb < sz; xb += 16) {
        float v[3][16];
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
          for (int q = 0; q < 16; ++q)
            v[k][q] = *(const gfloat*)(fac + (size_t)k * len + base + (size_t)min(xb + q, sz - 1) * st);
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
          for (int q = 0; q < 16; ++q) s[k] += xb + q < sz ? (double)v[k][q] : 0.0;
      }
#pragma unroll
      for (int k = 0; k < 3; ++k) rcm[k] = (float)(s[k] / (double)sz);
    }
  }
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const float f = fv[k];
    fct[k] = is_r ? rsq(fmaxf(f / (rcm[k] + 1e-9f), 1e-9f)) : rsq(fmaxf(f, 1e-9f));
    x0[k] = f * s0[k];
    x1[k] = rsq(f + 1e-8f) * s1[k];
  }
}

// First-layer contribution of the channels an entry carries: t_j = (bias_j) + sum_k x0_k w[ch_f+k][j]
// + x1_k w[ch_q+k][j], with w (30, H) row-major (in, out).
template <int H>
__device__ __forceinline__ void vector_terms(const TDesc& d, int which, bool is_r, int i, const float (&x0)[3],
                                             const float (&x1)[3], const float* __restrict__ w1,
                                             const float* __restrict__ b1, float* __restrict__ term) {
  const int ch_f = is_r ? 15 : 18, ch_q = is_r ? 21 : 24;
  // The weight rows are the same for every lane: eight outputs at a time they arrive as a few wide
  // scalar loads (w1 and b1 are not written by the running kernel).
  static_assert(H % 4 == 0, "first-layer width");
  constexpr int JB = H < 8 ? H : 8;
#pragma unroll
  for (int j0 = 0; j0 < H; j0 += JB) {
    float wf[3][JB], wq[3][JB], bb[JB];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      load_uniform<JB>(w1 + (ch_f + k) * H + j0, wf[k]);
      load_uniform<JB>(w1 + (ch_q + k) * H + j0, wq[k]);
    }
    load_uniform<JB>(b1 + j0, bb);
    float tv[JB];
#pragma unroll
    for (int j = 0; j < JB; ++j) {
      float t = (which == 0) ? bb[j] : 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        t = fmaf(x0[k], wf[k][j], t);
        t = fmaf(x1[k], wq[k][j], t);
      }
      tv[j] = t;
    }
    // [entry][H]: the entry's outputs are adjacent, 16 bytes a store
#pragma unroll
    for (int j = 0; j < JB; j += 4)
      *(float4*)(term + term_index<H>(d, which, j0 + j, i)) = make_float4(tv[j], tv[j + 1], tv[j + 2], tv[j + 3]);
  }
}

// =============================================================================================
// V0b: one block per 1024 entries of a statistics vector.  Reduces the V0a partials of its
// tensor into the normalisation scales of the 12 broadcast channels and row_col_mean (BScale),
// writes the factor tables and, when first-layer weights are given (shared by all tensors), the
// per-row / per-column MLP terms: the 12 feature channels that depend on the row or on the column
// only are normalised and pushed through the first layer once per row / column instead of once
// per element.  The bias goes into the terms of vector 0.
// =============================================================================================
template <int H>
__global__ __launch_bounds__(kThreads) void k_v0b(const TDesc* __restrict__ descs,
                                                  const PyloTensorArgs* __restrict__ dyn,
                                                  const Item* __restrict__ items,
                                                  const double* __restrict__ v0part, float norm_eps,
                                                  const float* __restrict__ w1, const float* __restrict__ b1,
                                                  int b1_stride /* floats between the tensors' biases, 0: shared */,
                                                  float* __restrict__ fac_tab, float* __restrict__ term_tab,
                                                  BScale* __restrict__ bscale) {
  constexpr int G = 14;  // 14 groups x 18 (vector, slot) pairs = 252 threads
  __shared__ double red[G][2 * kNV0];
  __shared__ double tot[2 * kNV0];
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  // the entries' accumulator values are requested before the reduction below waits on its own loads:
  // one memory round trip for the block instead of two (kernels start with cold caches)
  constexpr int kPer = kV0bEnt / kThreads;
  const int which = it.b;
  const bool is_r = (which == 0) == (d.vec0_is_r != 0);
  const int len = pick(d.len, which);
  const float* fac = is_r ? a.fac_r : a.fac_c;
  const int i_end = min(len, (it.a + 1) * kV0bEnt);
  float fpre[kPer][3];
#pragma unroll
  for (int q = 0; q < kPer; ++q) {
    const int i = it.a * kV0bEnt + q * kThreads + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 3; ++k) fpre[q][k] = i < i_end ? *(const gfloat*)(fac + (size_t)k * len + i) : 0.0f;
  }
  {
    const int pair = threadIdx.x % (2 * kNV0), gI = threadIdx.x / (2 * kNV0);
    if (gI < G) {
      const int vecI = pair / kNV0, slot = pair % kNV0;
      double s = 0.0;
      const int nb = vecI ? d.v0a_n[1] : d.v0a_n[0], first = vecI ? d.v0a_first[1] : d.v0a_first[0];
      // up to 32 partial rows per thread requested at once (same order of addition as a plain loop): a
      // vector of tens of thousands of entries has hundreds of rows, and every batch is a memory round trip
      for (int b0 = gI; b0 < nb; b0 += 32 * G) {
        double v[32];
#pragma unroll
        for (int q = 0; q < 32; ++q) {
          const int b = b0 + q * G;
          v[q] = b < nb ? v0part[(size_t)(first + b) * kNV0 + slot] : 0.0;
        }
#pragma unroll
        for (int q = 0; q < 32; ++q) s += v[q];
      }
      red[gI][pair] = s;
    }
    __syncthreads();
    if (threadIdx.x < 2 * kNV0) {
      double s = 0.0;
      for (int g2 = 0; g2 < G; ++g2) s += red[g2][threadIdx.x];
      tot[threadIdx.x] = s;
    }
    __syncthreads();
  }
  const int rI = d.vec0_is_r ? 0 : 1, cI = 1 - rI;
  const double* tr = tot + rI * kNV0;
  const double* tc = tot + cI * kNV0;
  // means as sum * (1 / len): one double division per vector instead of nine
  const double inv_r = 1.0 / (double)d.len[rI], inv_c = 1.0 / (double)d.len[cI];
  if (which == 0 && it.a == 0 && threadIdx.x == 0) {  // the tensor's scales, for k_terms
    BScale bs;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      bs.rcm[k] = (float)(tr[k * 3 + 0] * inv_r);
      bs.s[k] = rsq(norm_eps + (float)(tr[k * 3 + 1] * inv_r));        // fac_r_k
      bs.s[3 + k] = rsq(norm_eps + (float)(tc[k * 3 + 1] * inv_c));    // fac_c_k
      bs.s[6 + k] = rsq(norm_eps + (float)(tr[k * 3 + 2] * inv_r));    // rsqrt(fac_r_k + 1e-8)
      bs.s[9 + k] = rsq(norm_eps + (float)(tc[k * 3 + 2] * inv_c));    // rsqrt(fac_c_k + 1e-8)
    }
    bs.pad_ = 0.0f;
    bscale[d.fac_slot] = bs;
  }
  // this block's vector: its own sums sit at tot + which * kNV0
  const double* own = tot + which * kNV0;
  const double inv_own = 1.0 / (double)pick(d.len, which);
  float rcm3[3], s0[3], s1[3];
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    rcm3[k] = (float)(tr[k * 3 + 0] * inv_r);
    s0[k] = rsq(norm_eps + (float)(own[k * 3 + 1] * inv_own));
    s1[k] = rsq(norm_eps + (float)(own[k * 3 + 2] * inv_own));
  }
  // N-D row vector: row_col_mean is a mean over the dc axis inside the vector, one value per slice
  // (o, r) of its [o][dc][r] view.  The slices this block's entries belong to are reduced once, here,
  // into a table in LDS (a thread per slice while the axis is short, a wave per slice otherwise; fixed
  // order either way) instead of once per entry, which costs the axis length in loads per entry.
  __shared__ float rcm_tab[3 * kRcmSlots];
  const float* rcm_slices = nullptr;
  int o_first = 0;
  if (is_r && d.mode == kModeFacND) {
    const int sz = d.rcm_size, st = d.rcm_stride, blk = sz * st;
    const int i0 = it.a * kV0bEnt;
    o_first = i0 / blk;
    const int count = ((i_end - 1) / blk - o_first + 1) * st;
    if (count <= kRcmSlots) {
      const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      if (sz < 64) {
        for (int sl = threadIdx.x; sl < count; sl += kThreads) {
          const int base = (o_first + sl / st) * blk + sl % st;
          double sk[3] = {0.0, 0.0, 0.0};
          for (int xb = 0; xb < sz; xb += 16) {
            float v[3][16];
#pragma unroll
            for (int k = 0; k < 3; ++k)
#pragma unroll
              for (int q = 0; q < 16; ++q)
                v[k][q] = *(const gfloat*)(fac + (size_t)k * len + base + (size_t)min(xb + q, sz - 1) * st);
#pragma unroll
            for (int k = 0; k < 3; ++k)
#pragma unroll
              for (int q = 0; q < 16; ++q) sk[k] += xb + q < sz ? (double)v[k][q] : 0.0;
          }
#pragma unroll
          for (int k = 0; k < 3; ++k) rcm_tab[k * kRcmSlots + sl] = (float)(sk[k] / (double)sz);
        }
      } else {
        for (int sl = wave; sl < count; sl += kWaves) {
          const int base = (o_first + sl / st) * blk + sl % st;
          double sk[3] = {0.0, 0.0, 0.0};
          for (int x = lane; x < sz; x += 64)
#pragma unroll
            for (int k = 0; k < 3; ++k) sk[k] += (double)*(const gfloat*)(fac + (size_t)k * len + base + (size_t)x * st);
#pragma unroll
          for (int k = 0; k < 3; ++k) {
            const double t = wave_sum(sk[k]);
            if (lane == 0) rcm_tab[k * kRcmSlots + sl] = (float)(t / (double)sz);
          }
        }
      }
      __syncthreads();
      rcm_slices = rcm_tab;
    }
  }
#pragma unroll
  for (int q = 0; q < kPer; ++q) {
    const int i = it.a * kV0bEnt + q * kThreads + threadIdx.x;
    if (i >= i_end) break;
    float fct[3], x0[3], x1[3];
    int slice = 0;
    if (rcm_slices != nullptr) {
      const int st = d.rcm_stride, blk = d.rcm_size * st;
      slice = (i / blk - o_first) * st + i % st;
    }
    vector_entry(d, is_r, fac, len, i, fpre[q], rcm3, s0, s1, fct, x0, x1, rcm_slices, slice);
    *(float4*)(fac_tab + fac_index(d, which, 0, i)) = make_float4(fct[0], fct[1], fct[2], 0.0f);
    if (w1 != nullptr) vector_terms<H>(d, which, is_r, i, x0, x1, w1, b1 + (size_t)it.tensor * b1_stride, term_tab);
  }
}

// First-layer terms with per-tensor weights that only exist after k_v0b has run (VeLO: the LSTM
// emits them).  w1 / b1 are per-tensor blocks `w_stride` floats apart, (30, H) then (H).
template <int H>
__global__ __launch_bounds__(kThreads) void k_terms(const TDesc* __restrict__ descs,
                                                    const PyloTensorArgs* __restrict__ dyn,
                                                    const Item* __restrict__ items,
                                                    const BScale* __restrict__ bscale,
                                                    const float* __restrict__ w1_all, int w_stride,
                                                    float* __restrict__ term_tab) {
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = dyn[it.tensor];
  if (a.grad == nullptr) return;
  const float* w1 = w1_all + (size_t)it.tensor * w_stride;
  const float* b1 = w1 + 30 * H;
  const int which = it.b;
  const bool is_r = (which == 0) == (d.vec0_is_r != 0);
  const int len = pick(d.len, which);
  const float* fac = is_r ? a.fac_r : a.fac_c;
  // the tensor's scales, written by k_v0b: wave-uniform, through the scalar cache
  const BScale* bs = bscale + d.fac_slot;
  float rcm3[3], s0[3], s1[3];
  load_uniform<3>(bs->rcm, rcm3);
  load_uniform<3>(bs->s + (is_r ? 0 : 3), s0);
  load_uniform<3>(bs->s + (is_r ? 6 : 9), s1);
  for (int i = it.a * kV0bEnt + threadIdx.x; i < min(len, (it.a + 1) * kV0bEnt); i += kThreads) {
    float fct[3], x0[3], x1[3], fv[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) fv[k] = *(const gfloat*)(fac + (size_t)k * len + i);
    vector_entry(d, is_r, fac, len, i, fv, rcm3, s0, s1, fct, x0, x1);
    vector_terms<H>(d, which, is_r, i, x0, x1, w1, b1, term_tab);
  }
}

}  // namespace pylo
