// Newton-Schulz orthogonalisation of ELO-CELO2's raw steps (pylo/optim/CELO2_naive.py:59-73) as fp32
// matrix-pipe kernels of our own, for every 2-D tensor of a plan at once.
//
// One iteration on X (R x C, m = min(R, C)) is three products,
//     A  = X X^T            (or X^T X when X is tall)        m x m, symmetric
//     B' = c2 A A + c1 A + c0 I                               m x m, symmetric
//     X <- B' X             (or X B')
// i.e. c0 X + (c1 A + c2 A A) X with the scalings riding on the small matrices.  A and B' are
// symmetric: only the tiles on and above the diagonal are computed and each is stored twice (29 % of
// the step's FLOPs on a GPT-2-small set).  The first iteration takes X = raw / (||raw|| + eps) by
// scaling A with s^2 and the new X with s, so the raw step is never rewritten.  Every product of every
// tensor is one launch over a table of tile jobs (k_ns_gemm<OP>): three or four launches per iteration
// however many tensors there are; the Gram product of a very tall matrix is cut along its reduction into
// slabs whose partial tiles k_ns_gram_reduce adds in a fixed order.
//
// Tile job: 128 x 128 outputs by 256 threads = 2 x 2 waves of 64 x 64 = 2 x 2 v_mfma_f32_32x32x2_f32
// accumulators; operands staged through LDS 16 reduction steps at a time, double buffered, k-major
// ([k][row]) so that an MFMA operand is one conflict-free ds_read_b32 per lane.
#pragma once

#include "pylo_common.h"

namespace pylo {

constexpr int kNsTile = 128;     // output tile edge
constexpr int kNsBK = 16;        // reduction steps per stage
constexpr int kNsLd = kNsTile + 4;   // LDS row pitch in floats (16-byte aligned rows)
constexpr int kNsSlabK = 2048;   // reduction length of one slab of a split Gram product
constexpr int kNsSplitMin = 8192;   // Gram products with a reduction at least this long are split
constexpr int kNsFewJobs = 512;     // a plan with fewer Gram tile jobs than this splits them further (two per CU)

enum : int { kNsGram = 0, kNsPoly = 1, kNsUpdate = 2 };

struct NsMat {
  int tensor;          // index into the argument table (raw step pointer, flags)
  int unit;            // the finishing pass's unit whose sum of squares is this matrix's (FinUnit)
  int R, C, m, tall;   // X is R x C row-major; m = min(R, C); tall: R > C
  int n_slabs;         // > 1: the Gram product is split along its reduction
  int slab_k;          // reduction length of one slab
  long long off_x1;    // floats into the workspace: the second X buffer (R x C)
  long long off_a;     // A (m x m)
  long long off_b;     // B' (m x m)
  long long off_part;  // split Gram product: n_slabs partial matrices (m x m each), else unused
  long long elem_off;  // elements from the tensor's raw step to this matrix (split-fp16 kernels: a slice of a tensor with more dims)
};

struct NsItem {
  int mat;
  int tm, tn;    // output tile
  int k0, k1;    // reduction range
  int slab;      // Gram: slab index (partial matrix) when the product is split, else -1
};

typedef float v16f __attribute__((ext_vector_type(16)));
// LDS pointers carry their address space explicitly: a generic pointer chosen at run time between the
// two stages compiles to flat loads, which also wait on the global prefetch in flight
typedef __attribute__((address_space(3))) float lfloat;
typedef __attribute__((address_space(3))) v4f lv4f;

constexpr int kArgOrthogonalize = PYLO_ARG_ORTHOGONALIZE;

// One operand tile (kNsBK reduction steps x 128 rows/columns) from global memory into registers.
// KMAJOR: the operand is stored [k][o] (o contiguous): thread t takes k = t / 32 (+8), o = 4 (t % 32) ..+3.
// else:   the operand is stored [o][k] (k contiguous): thread t takes o = t / 4 (+64), k = 4 (t % 4) ..+3.
// Elements outside [0, n_o) x [k_lo, k_hi) read as zero (n_o and the contiguous extent are multiples of 4).
template <bool KMAJOR>
__device__ __forceinline__ void ns_load_tile(const float* __restrict__ src, int ld, int o0, int n_o, int k0,
                                             int k_hi, v4f (&reg)[2]) {
  const int t = threadIdx.x;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    int k, o;
    if (KMAJOR) { k = k0 + (t >> 5) + 8 * h; o = o0 + 4 * (t & 31); }
    else { o = o0 + (t >> 2) + 64 * h; k = k0 + 4 * (t & 3); }
    const bool in = o < n_o && k < k_hi;
    const float* p = KMAJOR ? src + (size_t)k * ld + o : src + (size_t)o * ld + k;
    reg[h] = in ? *(const gv4f*)p : v4f{0.0f, 0.0f, 0.0f, 0.0f};
  }
}

// ... and from the registers into an LDS stage laid out [k][o] with pitch kNsLd.
template <bool KMAJOR>
__device__ __forceinline__ void ns_store_tile(lfloat* lds, const v4f (&reg)[2]) {
  const int t = threadIdx.x;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (KMAJOR) {
      *(lv4f*)(lds + ((t >> 5) + 8 * h) * kNsLd + 4 * (t & 31)) = reg[h];
    } else {
      const int o = (t >> 2) + 64 * h, k = 4 * (t & 3);
      lds[(k + 0) * kNsLd + o] = reg[h].x;
      lds[(k + 1) * kNsLd + o] = reg[h].y;
      lds[(k + 2) * kNsLd + o] = reg[h].z;
      lds[(k + 3) * kNsLd + o] = reg[h].w;
    }
  }
}

// acc[hi][hj] += A-tile x B-tile over [k0, k1).  A rows i0.., B rows j0.. ("rows" = output index of the
// operand).  AK / BK: the operand is stored k-major.
template <bool AK, bool BK>
__device__ __forceinline__ void ns_tile_product(const float* __restrict__ A, int lda, int i0, int n_i,
                                                const float* __restrict__ B, int ldb, int j0, int n_j, int k0,
                                                int k1, lfloat* lds, v16f (&acc)[2][2]) {
  constexpr int kStage = 2 * kNsBK * kNsLd;   // floats of one stage: the A tile, then the B tile
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wi = (wave >> 1) * 64, wj = (wave & 1) * 64;
  const int kr = lane >> 5, lo = lane & 31;
  v4f ra[2], rb[2];
  ns_load_tile<AK>(A, lda, i0, n_i, k0, k1, ra);
  ns_load_tile<BK>(B, ldb, j0, n_j, k0, k1, rb);
  ns_store_tile<AK>(lds, ra);
  ns_store_tile<BK>(lds + kNsBK * kNsLd, rb);
  __syncthreads();
  int cur = 0;   // offset of the stage being read
  for (int k = k0; k < k1; k += kNsBK) {
    const bool more = k + kNsBK < k1;
    if (more) {
      ns_load_tile<AK>(A, lda, i0, n_i, k + kNsBK, k1, ra);
      ns_load_tile<BK>(B, ldb, j0, n_j, k + kNsBK, k1, rb);
    }
    const lfloat* a = lds + cur + kr * kNsLd + wi + lo;
    const lfloat* b = lds + cur + kNsBK * kNsLd + kr * kNsLd + wj + lo;
#pragma unroll
    for (int kk = 0; kk < kNsBK; kk += 2) {
      const float a0 = a[kk * kNsLd], a1 = a[kk * kNsLd + 32];
      const float b0 = b[kk * kNsLd], b1 = b[kk * kNsLd + 32];
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    }
    if (more) {
      ns_store_tile<AK>(lds + (kStage - cur), ra);
      ns_store_tile<BK>(lds + (kStage - cur) + kNsBK * kNsLd, rb);
    }
    __syncthreads();
    cur = kStage - cur;
  }
}

// Row and column of accumulator register r of sub-tile (hi, hj) of this lane's wave, inside the tile.
__device__ __forceinline__ int ns_acc_row(int hi, int r) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  return (wave >> 1) * 64 + hi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}
__device__ __forceinline__ int ns_acc_col(int hj) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  return (wave & 1) * 64 + hj * 32 + (lane & 31);
}

// One launch = one product of one Newton-Schulz iteration, for every tensor.
//   kNsGram    A (or a slab's partial matrix) = alpha X X^T / X^T X, tiles tm <= tn, stored twice unless partial
//   kNsPoly    B' = c2 A A + c1 A + c0 I, tiles tm <= tn, stored twice
//   kNsUpdate  X_out = alpha B' X_in / X_in B'
// alpha is s^2 / s in the first iteration (s = 1 / (||raw|| + eps), scale[mat]) and 1 afterwards.
// `par`: X_in is the raw step (0) or the second buffer (1); X_out is the other.
template <int OP>
__global__ __launch_bounds__(256) void k_ns_gemm(const NsMat* __restrict__ mats, const NsItem* __restrict__ items,
                                                 const PyloTensorArgs* __restrict__ dyn, float* __restrict__ ws,
                                                 const float* __restrict__ scale, int first, int par, float c0,
                                                 float c1, float c2) {
  __shared__ __attribute__((aligned(16))) float lds_[4 * kNsBK * kNsLd];
  lfloat* lds = (lfloat*)lds_;
  const NsItem it = items[blockIdx.x];
  const NsMat mt = mats[it.mat];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  float* x0 = a.step_out;
  float* x1 = ws + mt.off_x1;
  const float* xin = par ? x1 : x0;
  float* xout = par ? x0 : x1;
  float* A = ws + mt.off_a;
  float* B = ws + mt.off_b;
  const int m = mt.m;
  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const int i0 = it.tm * kNsTile, j0 = it.tn * kNsTile;
  float* out;
  int ldo, n_i, n_j;
  float alpha = 1.0f;
  if (OP == kNsGram) {
    if (mt.tall) ns_tile_product<true, true>(xin, mt.C, i0, m, xin, mt.C, j0, m, it.k0, it.k1, lds, acc);
    else ns_tile_product<false, false>(xin, mt.C, i0, m, xin, mt.C, j0, m, it.k0, it.k1, lds, acc);
    out = it.slab >= 0 ? ws + mt.off_part + (size_t)it.slab * m * m : A;
    ldo = m; n_i = m; n_j = m;
    if (first) { const float s = scale[it.mat]; alpha = s * s; }
  } else if (OP == kNsPoly) {
    ns_tile_product<true, true>(A, m, i0, m, A, m, j0, m, it.k0, it.k1, lds, acc);
    out = B; ldo = m; n_i = m; n_j = m;
  } else {
    if (mt.tall) {   // X_out (R x m) = X_in B'
      ns_tile_product<false, true>(xin, mt.C, i0, mt.R, B, m, j0, m, it.k0, it.k1, lds, acc);
      n_i = mt.R; n_j = m;
    } else {         // X_out (m x C) = B' X_in
      ns_tile_product<true, true>(B, m, i0, m, xin, mt.C, j0, mt.C, it.k0, it.k1, lds, acc);
      n_i = m; n_j = mt.C;
    }
    out = xout; ldo = mt.C;
    if (first) alpha = scale[it.mat];
  }
  const bool mirror = OP != kNsUpdate && it.slab < 0 && it.tm != it.tn;
#pragma unroll
  for (int hi = 0; hi < 2; ++hi)
#pragma unroll
    for (int hj = 0; hj < 2; ++hj) {
      const int col = j0 + ns_acc_col(hj);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = i0 + ns_acc_row(hi, 4 * q);   // rows row .. row + 3
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float x = acc[hi][hj][4 * q + r] * alpha;
          if (OP == kNsPoly) {
            const bool in = row + r < n_i && col < n_j;
            const float aij = in ? A[(size_t)(row + r) * m + col] : 0.0f;
            x = c2 * x + c1 * aij + ((row + r) == col ? c0 : 0.0f);
          }
          v[r] = x;
        }
        if (col < n_j) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (row + r < n_i) out[(size_t)(row + r) * ldo + col] = v[r];
          // the mirrored tile: four consecutive columns of row `col` (n_i is a multiple of 4)
          if (mirror && row < n_i) *(gv4f*)(out + (size_t)col * ldo + row) = v4f{v[0], v[1], v[2], v[3]};
        }
      }
    }
}

// A = sum over the slabs' partial matrices, in slab order.  The partials hold the tiles on and above the
// diagonal only; a thread adds up one element of such a tile (eight slabs' values in flight at a time)
// and writes it to A twice, as (i, j) and as (j, i).  blockIdx.y: matrix; blockIdx.x: 256 elements of
// the m x m index space, of which the threads below the diagonal tiles have nothing to do.
__global__ __launch_bounds__(256) void k_ns_gram_reduce(const NsMat* __restrict__ mats, const int* __restrict__ split_mats,
                                                        const PyloTensorArgs* __restrict__ dyn, float* __restrict__ ws) {
  const NsMat mt = mats[split_mats[blockIdx.y]];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  const int m = mt.m;
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long long)m * m) return;
  const int i = (int)(e / m), j = (int)(e - (long long)i * m);
  if (i / kNsTile > j / kNsTile) return;
  const size_t mm = (size_t)m * m;
  const float* p = ws + mt.off_part + (size_t)i * m + j;
  float s = 0.0f;
  for (int q0 = 0; q0 < mt.n_slabs; q0 += 8) {
    float v[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) v[q] = q0 + q < mt.n_slabs ? *(const gfloat*)(p + (size_t)(q0 + q) * mm) : 0.0f;
#pragma unroll
    for (int q = 0; q < 8; ++q) s += v[q];
  }
  float* A = ws + mt.off_a;
  A[(size_t)i * m + j] = s;
  if (i / kNsTile != j / kNsTile) A[(size_t)j * m + i] = s;
}

// s = 1 / (||raw|| + eps) per matrix from the per-block sums of squares of the finishing pass's first kernel.
// (`list`: the matrices of the launch, one block each; nullptr: matrices 0 .. n_mats - 1)
__global__ __launch_bounds__(256) void k_ns_scale(const NsMat* __restrict__ mats, const int* __restrict__ list, int n_mats,
                                                  const FinUnit* __restrict__ units, const double* __restrict__ fin_part,
                                                  float eps, float* __restrict__ scale) {
  __shared__ double red[4];
  if ((int)blockIdx.x >= n_mats) return;
  const int q = list ? list[blockIdx.x] : (int)blockIdx.x;
  const FinUnit d = units[mats[q].unit];
  double s = 0.0;
  for (int b = threadIdx.x; b < d.nblk; b += 256) s += fin_part[d.blk0 + b];
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) scale[q] = 1.0f / ((float)sqrt((red[0] + red[1]) + (red[2] + red[3])) + eps);
}

}  // namespace pylo
