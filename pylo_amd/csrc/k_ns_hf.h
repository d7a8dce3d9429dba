// Newton-Schulz products at fp32 accuracy on the fp16 matrix pipe.
//
// An fp32 number times a power of two is, to 2^-22 of its size, the sum of two fp16 numbers: x s = h + l with
// h = fp16(x s), l = fp16(x s - h) (11 + 11 significand bits), as long as h does not overflow (|x s| < 65 504) and l
// does not fall off the format's lower end (fp16 keeps subnormals down to 2^-24 and the matrix instructions take
// them as they are: l is exact to 2^-25 absolutely, i.e. entries below 1/8 lose relative, not absolute, accuracy).
// A product of two such numbers is four fp16 products; the smallest (l l, 2^-22 |x y|) is dropped with the
// remainders.  The other three are exact in fp32 and are accumulated in fp32 by v_mfma_f32_32x32x16_f16, which does
// sixteen times the multiply-adds of v_mfma_f32_32x32x2_f32 per instruction slot: three of them replace eight fp32
// instructions' worth of work.  An operand carries 23 significant bits where fp32 has 24: a product of the iteration
// is off by about 6e-8 of its entries' RMS, a quarter of what the fp32 accumulation of a reduction over 256 .. 4096
// terms adds anyway (a plain fp32 GEMM: 2.5e-7), but each entry of the result carries 1 .. 3e-7 of its own size where
// an fp32 product carries 6e-8.  With the reference's coefficients, which multiply rounding by up to 3.44 an
// iteration, the result is as far from the fp64 formula as the fp32 torch products are (0.4 .. 0.9 times, tests); with
// polynomials that do not amplify (1.5 x - 0.5 x^3, 2 x - x^3) it is 3 .. 12 times further, 1e-5 of its RMS at most.
// The scales: no entry of a matrix exceeds its largest singular value, and the singular values of everything the
// iteration forms follow from the coefficients alone once X0 has unit Frobenius norm (the host walks a grid of
// starting values through sigma -> sigma p(sigma^2), ns_plane_exps): X and A = X X^T stay below 1.5, B' = p(A)
// below c0, products of k such B' below c0^k.  Every kind of matrix gets the power of two that puts its bound at
// 12 000 .. 24 000; a product's accumulators are scaled back by the reciprocal of its operands' scales (exact) and
// what it writes is scaled by its own.  A value outside its bound -- there should be none -- is clamped, not made
// an infinity.
//
// Operands therefore live as *planes*: two fp16 matrices (h, l) with the reduction index contiguous,
// written by the kernel that produces the matrix (never converted inside a product's main loop).
// With X of m x n or n x m (m the smaller dim), Xs = X as [m][n] and Xl = X as [n][m]:
//     A   = Xs Xs^T                      (reduction over n; symmetric, tiles on and above the diagonal)
//     B'  = c2 A A + c1 A + c0 I         (reduction over m; symmetric)
//     Xl' = Xl B'                        (reduction over m), written as planes of Xl' and of Xs' = Xl'^T,
//                                         or as fp32 in the tensor's own layout after the last iteration
// for wide and tall matrices alike (B' is symmetric, so (B' X)^T = X^T B').
//
// Two iterations can share the two products over the long dim.  Every B'_t is a polynomial in A_t, so it
// commutes with A_t and is symmetric, and A_{t+1} = X_{t+1} X_{t+1}^T = B'_t A_t B'_t needs no X:
//     A_t (Gram), B'_t = p(A_t) (Poly), T = A_t B'_t (Prod), A_{t+1} = B'_t T (ProdA), B'_{t+1} = p(A_{t+1}) (Poly),
//     Q = B'_{t+1} B'_t (Prod), X_{t+2} = Q X_t (Update)
// i.e. four products of m^3 / 2 multiply-adds in place of one Gram product (m^2 n / 2) and one update (m^2 n).
// What it costs in accuracy is bounded whatever the spectrum of X: A_t as computed is off by eps ||A_t|| in
// absolute terms, which A_{t+1} = B'_t A_t B'_t inherits relative to its small eigenvalues -- they grow by
// p(0)^2 = c0^2 in the step, so the error of p(A_{t+1}) in those directions is c1 c0^2 eps sigma_max^2, about
// 12 times that of p of a freshly formed Gram matrix and about 1e-6 of B' itself; a second chained step
// multiplies it by c0^2 again, which is why pairs are the default and the next pair starts from a Gram product
// of the X it was handed.  The host enqueues chains of any length L (one Gram product, 4 L - 3 products of
// m x m matrices rotating through four plane buffers, one update): PYLO_MI355_NS_CHAINS="3,2" in the environment
// trades accuracy for time (up to 1e-4 of the result's RMS on a dominant direction over a flat rest, where pairs
// are at 1.3e-5), PYLO_MI355_NS_PAIRS=0 keeps one Gram product and one update per iteration.
//
// Tile job: 128 x 128 (Gram, Poly, narrow updates) or 128 x 256 outputs (updates with m > 128) by 256 threads =
// 2 x 2 waves of 64 x 64 / 64 x 128 = 2 x 2 / 2 x 4 accumulators of 32 x 32; 16 reduction steps per stage,
// double buffered in LDS (32 / 48 KB), staged from global memory straight into LDS (global_load_lds_dwordx4: no
// staging registers, no LDS store instructions), one 16-byte read per lane, plane and 32-row block per stage.
// The planes are allocated with their rows rounded up to whole tiles and the padding holds zeros, so the main
// loop has no bounds checks; any two dims are taken (the raw step is read and the result written per element
// where the tensor's rows are not 16-byte aligned).
#pragma once

#include <type_traits>

#include "k_ns.h"

namespace pylo {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short hbits;   // one number of a plane in memory (an fp16)
constexpr int kNsPl = 2;                      // planes per matrix
constexpr int kNsRowB = 32 * kNsPl;           // bytes of one row in a block of 16 reduction steps
constexpr int kNsRowPc = 2 * kNsPl;           // the same in 16-byte pieces
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) u32x4 luint4;

constexpr int kHfBK = 16;                     // reduction steps per stage
// LDS of a tile job with 64 WN columns: two stages of (128 + 64 WN) rows x 2 planes x 32 bytes
constexpr int hf_gemm_lds(int wn) { return 2 * (128 + 64 * wn) * kNsRowB; }

// Planes of one matrix with `rows` rows and a (padded) reduction length: stored in blocks of 16 reduction
// steps, [k / 16][row][plane][k % 16], so that the 128 rows x 3 planes x 16 steps a tile job stages at a
// time are 12 KB of consecutive memory (whole cache lines; with row-major planes a stage was 32 bytes
// out of every row and each 128-byte line was fetched from L2 four times).
struct HfPlanes {
  const hbits* base;
  int rows;   // rows allocated (a multiple of the tiles' rows; rows past the matrix hold zeros)
};

// element offset of (row, k) in plane 0; plane 1 is 16 elements further
__device__ __forceinline__ size_t hf_off(int rows, int row, int k) {
  return ((size_t)(k >> 4) * rows + row) * (16 * kNsPl) + (k & 15);
}

struct NsHfMat {
  int tensor;
  int R, C, m, n, tall;      // X is R x C row-major; m = min, n = max; tall: R > C
  int pad_m, pad_n;          // m and n rounded up to the 16 reduction steps of a stage (the padding holds zeros)
  int rows_m, rows_n;        // rows allocated for the planes whose rows are the m / n index (whole tiles)
  int lda;                   // row pitch of the fp32 A and of the partial matrices: m rounded up to 4
  int n_slabs;
  long long off_xs;          // elements (hbits) into the plane workspace: planes of Xs (m rows, reduction n)
  long long off_xl[2];       // planes of Xl (n rows, reduction m), two buffers (a product reads one and writes the other)
  long long off_p, p_stride; // planes of the m x m matrices (m rows, reduction m): buffer b at off_p + b p_stride
  long long off_a;           // floats into the fp32 workspace: A (m x m)
  long long off_part;        // floats: partial matrices of a split Gram product
  long long elem_off;        // elements from the tensor's raw step to this matrix (a slice of a tensor with more dims)
  int fpart0, n_fpart;       // its partial sums of squares of A (k_ns_hf_chain_sumsq): first, count
};

// the m x m plane buffers, and the two products on planes in and planes out (k_ns_hf_gemm's OP, after
// kNsGram / kNsPoly / kNsUpdate)
enum : int { kNsBufA = 0, kNsBufB = 1, kNsBufT = 2, kNsBufC = 3, kNsBufs = 4 };
enum : int { kNsProd = 3, kNsProdA = 4 };
// operand and result buffers of an m x m product (the update's B' is s1); what turns the accumulators into the
// product's values (the reciprocal of the operands' plane scales) and the scale of the planes written
struct NsBufs { int s1, s2, d; float acc_scale, out_scale; };

// x (already times its plane scale) = h + l + what is left below 2^-22 |x|.  The clamp never acts on a matrix
// within the bounds the scales were chosen for; it keeps a stray value from becoming an infinity.
__device__ __forceinline__ void hf_split(float x, hbits& h, hbits& l) {
  const float c = __builtin_amdgcn_fmed3f(x, -65000.0f, 65000.0f);
  x = x == x ? c : x;   // (the median of three takes a NaN for the smallest: keep it a NaN)
  const _Float16 hb = (_Float16)x;
  const _Float16 lb = (_Float16)(x - (float)hb);
  h = __builtin_bit_cast(hbits, hb);
  l = __builtin_bit_cast(hbits, lb);
}

// A stage of one operand in LDS: [row][plane][half], 64 bytes a row, as in memory, except that the four
// 16-byte pieces of a row are permuted: piece s of row r sits in slot s ^ ((r / 4) % 4), so that sixteen
// consecutive rows, read one piece each by sixteen lanes, touch sixteen different 16-byte bank groups (rows 4
// apart would share them).
// A wave-wide load instruction moves 64 consecutive 16-byte pieces of the stage from global memory into LDS
// (the hardware puts lane l's piece at the instruction's LDS base + 16 l); the permutation is done on the global
// side: lane l fetches the piece whose place in LDS it fills.  ROWS x 4 pieces = ROWS x 4 / 256 instructions
// per thread; `off[]` holds the lane's byte offsets into the stage in memory (they do not change with k).
#define PYLO_LDS __attribute__((address_space(3)))
#define PYLO_GLB __attribute__((address_space(1)))

// (NW: waves of the block)
template <int ROWS, int NW = 4>
__device__ __forceinline__ void hf_stage_offsets(int wave, int lane, int (&off)[ROWS * kNsRowPc / (64 * NW)]) {
#pragma unroll
  for (int j = 0; j < ROWS * kNsRowPc / (64 * NW); ++j) {
    const int p = (j * NW + wave) * 64 + lane;
    off[j] = (p ^ ((p >> 4) & 3)) * 16;   // row p / 4: its four pieces permuted by (row / 4) % 4
  }
}

template <int ROWS, int NW = 4>
__device__ __forceinline__ void hf_stage_issue(const char* g, const int (&off)[ROWS * kNsRowPc / (64 * NW)], PYLO_LDS char* lds, int wave) {
#pragma unroll
  for (int j = 0; j < ROWS * kNsRowPc / (64 * NW); ++j)
    __builtin_amdgcn_global_load_lds((const PYLO_GLB void*)(g + off[j]), (PYLO_LDS void*)(lds + (j * NW + wave) * 1024), 16, 0, 0);
}

// acc[hi][hj] += (rows i0.. of P1) x (rows j0.. of P2)^T over the reduction range [k0, k1) (multiples of 16);
// 128 rows of P1, 64 WN rows of P2.  LDS: two stages of (128 + 64 WN) x 64 bytes.
// `compute` (the same for all lanes of a wave): false for a wave whose values nobody needs -- it stages and meets the
// barriers, and leaves the matrix pipe to the other waves of its SIMD.
template <int WN, int NW = 4>
__device__ __forceinline__ void hf_tile_product(const HfPlanes& P1, int i0, const HfPlanes& P2, int j0, int k0, int k1,
                                                PYLO_LDS char* lds, v16f (&acc)[2][WN], bool compute = true) {
  constexpr int RA = 32 * NW, RB = 64 * WN, SA = RA * kNsRowB, STAGE = SA + RB * kNsRowB;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wi = (wave >> 1) * 64, wj = (wave & 1) * 32 * WN;
  const int kg = lane >> 5, lo = lane & 31;
  int offa[RA * kNsRowPc / (64 * NW)], offb[RB * kNsRowPc / (64 * NW)];
  hf_stage_offsets<RA, NW>(wave, lane, offa);
  hf_stage_offsets<RB, NW>(wave, lane, offb);
  const char* ga = (const char*)P1.base + ((size_t)(k0 >> 4) * P1.rows + i0) * kNsRowB;
  const char* gb = (const char*)P2.base + ((size_t)(k0 >> 4) * P2.rows + j0) * kNsRowB;
  const size_t sa = (size_t)P1.rows * kNsRowB, sb = (size_t)P2.rows * kNsRowB;
  // a diagonal tile of X X^T or A A: both operands are the same 128 rows, staged once
  const bool same = WN == 2 && P1.base == P2.base && i0 == j0;
  hf_stage_issue<RA, NW>(ga, offa, lds, wave);
  if (!same) hf_stage_issue<RB, NW>(gb, offb, lds + SA, wave);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  // the lane's rows are lo, lo + 32, ..: all with the same (row / 4) % 4; plane q, half kg is piece 2 q + kg
  const int sw = 16 * (kg ^ ((lo >> 2) & 3));
  const int oa = (wi + lo) * kNsRowB + sw, ob = (same ? 0 : SA) + (wj + lo) * kNsRowB + sw;
  int cur = 0;
  for (int k = k0; k < k1; k += kHfBK) {
    if (k + kHfBK < k1) {
      ga += sa;
      gb += sb;
      hf_stage_issue<RA, NW>(ga, offa, lds + (STAGE - cur), wave);
      if (!same) hf_stage_issue<RB, NW>(gb, offb, lds + (STAGE - cur) + SA, wave);
    }
    if (compute) {
      f16x8 a[2][kNsPl], b[WN][kNsPl];
#pragma unroll
      for (int q = 0; q < kNsPl; ++q) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          a[i][q] = __builtin_bit_cast(f16x8, *(const luint4*)(lds + cur + ((oa + i * 32 * kNsRowB) ^ (q * 32))));
#pragma unroll
        for (int j = 0; j < WN; ++j)
          b[j][q] = __builtin_bit_cast(f16x8, *(const luint4*)(lds + cur + ((ob + j * 32 * kNsRowB) ^ (q * 32))));
      }
      // smallest terms first: l h, h l, h h
#pragma unroll
      for (int term = 0; term < 3; ++term) {
        constexpr int pa[3] = {1, 0, 0}, pb[3] = {0, 1, 0};
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
#pragma unroll
          for (int hj = 0; hj < WN; ++hj)
            acc[hi][hj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[hi][pa[term]], b[hj][pb[term]], acc[hi][hj], 0, 0, 0);
      }
    }
    // the loads into the other stage have landed (they are counted like any other vector-memory load) and
    // every wave has read this one
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    cur = STAGE - cur;
  }
}

// The same product with the first operand's fragments loaded straight from memory into registers, two steps ahead (a
// lane's fragment of a row is 16 consecutive bytes of the planes): only the second operand goes through LDS, 48 KB
// of LDS traffic a step and block instead of 73.  128 rows of P1 (by 256 threads), 64 WN rows of P2; LDS: two
// stages of 64 WN x 64 bytes.  Benchmark instrumentation only (pylo_mi355_matrix_probe, mode 4): the bare loop is
// 8 - 12 % faster this way on one large operand, the update product inside whole steps (four groups of matrices on
// four streams) 2.5 % slower.
template <int WN>
__device__ __forceinline__ void hf_tile_product_direct(const HfPlanes& P1, int i0, const HfPlanes& P2, int j0, int k0, int k1,
                                                       PYLO_LDS char* lds, v16f (&acc)[2][WN]) {
  constexpr int RB = 64 * WN, STAGE = RB * kNsRowB;
  typedef PYLO_GLB u32x4 gu32x4;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wi = (wave >> 1) * 64, wj = (wave & 1) * 32 * WN;
  const int kg = lane >> 5, lo = lane & 31;
  int offb[RB * kNsRowPc / 256];
  hf_stage_offsets<RB>(wave, lane, offb);
  const char* ga = (const char*)P1.base + ((size_t)(k0 >> 4) * P1.rows + i0 + wi + lo) * kNsRowB + 16 * kg;
  const char* gb = (const char*)P2.base + ((size_t)(k0 >> 4) * P2.rows + j0) * kNsRowB;
  const size_t sa = (size_t)P1.rows * kNsRowB, sb = (size_t)P2.rows * kNsRowB;
  u32x4 an[2][2][kNsPl];   // the fragments of this step and the next (slot = step % 2), refilled for two steps on
  auto fetch_a = [&](auto slot, const char* g) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < kNsPl; ++q) an[slot.value][i][q] = *(const gu32x4*)(g + i * 32 * kNsRowB + q * 32);
  };
  typedef std::integral_constant<int, 0> S0;
  typedef std::integral_constant<int, 1> S1;
  hf_stage_issue<RB>(gb, offb, lds, wave);
  fetch_a(S0(), ga);
  if (k0 + kHfBK < k1) fetch_a(S1(), ga + sa);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  const int ob = (wj + lo) * kNsRowB + 16 * (kg ^ ((lo >> 2) & 3));
  int cur = 0;
  ga += sa;
  auto step = [&](auto slot, int k) {
    f16x8 a[2][kNsPl], b[WN][kNsPl];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < kNsPl; ++q) a[i][q] = __builtin_bit_cast(f16x8, an[slot.value][i][q]);
    const bool more_b = k + kHfBK < k1, more_a = k + 2 * kHfBK < k1;
    if (more_b) {
      gb += sb;
      hf_stage_issue<RB>(gb, offb, lds + (STAGE - cur), wave);
    }
    if (more_a) {
      ga += sa;
      fetch_a(slot, ga);
    }
#pragma unroll
    for (int q = 0; q < kNsPl; ++q)
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[j][q] = __builtin_bit_cast(f16x8, *(const luint4*)(lds + cur + ((ob + j * 32 * kNsRowB) ^ (q * 32))));
#pragma unroll
    for (int term = 0; term < 3; ++term) {
      constexpr int pa[3] = {1, 0, 0}, pb[3] = {0, 1, 0};
#pragma unroll
      for (int hi = 0; hi < 2; ++hi)
#pragma unroll
        for (int hj = 0; hj < WN; ++hj)
          acc[hi][hj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[hi][pa[term]], b[hj][pb[term]], acc[hi][hj], 0, 0, 0);
    }
    // the second operand's next stage has landed and every wave has read this one; the fragments just asked for
    // (the newest loads: loads complete in order) may still be on their way.  The bare barrier: a __syncthreads()
    // would wait for them too.
    if (more_a) __builtin_amdgcn_s_waitcnt((2 * kNsPl) | (7 << 4));   // vmcnt <= 4, lgkmcnt 0
    else __builtin_amdgcn_s_waitcnt(7 << 4);                            // vmcnt 0, lgkmcnt 0
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    cur = STAGE - cur;
  };
  for (int k = k0; k < k1; k += 2 * kHfBK) {
    step(S0(), k);
    if (k + kHfBK < k1) step(S1(), k + kHfBK);
  }
}

// one value (times its plane scale already) into both planes
__device__ __forceinline__ void hf_store1(hbits* base, int rows, int row, int k, float v) {
  hbits h, l;
  hf_split(v, h, l);
  hbits* p = base + hf_off(rows, row, k);
  p[0] = h;
  p[16] = l;
}

// The block's 128 x 64 WN values (accumulator layout) times `scale` into planes, in one or both orientations, every
// value split once.
//   D   planes whose reduction index is the tile's column index: through the wave's own LDS patch
//       ([row][plane][32 WN columns], 2 bytes each), 16 rows at a time; the wave reads the patch back as
//       16-byte pieces in the order the planes have in memory ([16 columns][row][plane][half]: 64 pieces for the
//       patch's 16 rows, one a lane).
//   D4  (when not null) planes whose reduction index is the tile's row index: four consecutive rows of a
//       lane are four consecutive reduction indices, one 8-byte store per plane straight from the registers.
// Only the lanes of one wave meet in a patch and a wave's LDS instructions execute in order, so the passes
// need no barrier, just the compiler kept from moving the reads over the writes.
template <int WN>
__device__ __forceinline__ void hf_store_planes(PYLO_LDS char* lds, const v16f (&acc)[2][WN], hbits* __restrict__ D,
                                                int rows_total, int i0, int j0, int n_rows, int n_cols,
                                                hbits* __restrict__ D4, int rows4, float scale) {
  constexpr int kPlane = 64 * WN + 16;        // bytes: 32 WN columns x 2 + 16 (bank spread)
  constexpr int kRow = kNsPl * kPlane, kWave = 16 * kRow;
  typedef PYLO_LDS hbits lbf;
  typedef unsigned long long u64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  PYLO_LDS char* patch = lds + wave * kWave;
  const int wi = i0 + (wave >> 1) * 64, wj = j0 + (wave & 1) * 32 * WN;   // origin of the wave's values
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int hi = pass >> 1, half = pass & 1;   // rows 32 hi + 16 half .. + 15 of the wave's 64
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // the patch is free: the previous pass has read it
#pragma unroll
    for (int hj = 0; hj < WN; ++hj)
#pragma unroll
      for (int g4 = 0; g4 < 2; ++g4) {
        hbits h[4], l[4];
        const int col_l = 32 * hj + (lane & 31);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          hf_split(acc[hi][hj][8 * half + 4 * g4 + r] * scale, h[r], l[r]);
          lbf* q = (lbf*)(patch + (8 * g4 + 4 * (lane >> 5) + r) * kRow + col_l * 2);
          q[0] = h[r];
          q[kPlane / 2] = l[r];
        }
        if (D4 != nullptr) {
          const int row = wi + 32 * hi + 16 * half + 8 * g4 + 4 * (lane >> 5), col = wj + col_l;
          if (col < n_cols && row < n_rows) {   // values past n_rows are zeros, into the padding
            hbits* p = D4 + hf_off(rows4, col, row);
            *(u64*)p = (u64)h[0] | (u64)h[1] << 16 | (u64)h[2] << 32 | (u64)h[3] << 48;
            *(u64*)(p + 16) = (u64)l[0] | (u64)l[1] << 16 | (u64)l[2] << 32 | (u64)l[3] << 48;
          }
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    const int row_w0 = wi + 32 * hi + 16 * half;
#pragma unroll
    for (int c = 0; c < 2 * WN; ++c) {     // 16 columns = one block of the planes' layout
      const int col = wj + 16 * c;
      if (col >= n_cols) continue;
      hbits* dst = D + hf_off(rows_total, row_w0, col);
      const int row_l = lane >> 2, plane = (lane >> 1) & 1, hf = lane & 1;   // piece `lane` of [row][plane][half]
      if (row_w0 + row_l >= n_rows) continue;
      const u32x4 w = *(const luint4*)(patch + row_l * kRow + plane * kPlane + (16 * c + 8 * hf) * 2);
      *(u32x4*)(dst + (size_t)lane * 8) = w;
    }
  }
}

// One launch = one product of one iteration, for every tensor (see the head of this file).
//   kNsGram    A = Xs Xs^T as fp32 and planes, both halves; a slab of a split product: fp32 partial tile only
//   kNsPoly    c2 A A + c1 A + c0 I as planes (buffer bufs.d), both halves; A: buffer kNsBufA and its fp32 copy
//   kNsProd    (buffer s1) (buffer s2) as planes (buffer d), both halves
//   kNsProdA   the same, into buffer d and into the fp32 copy of A
//   kNsUpdate  Xl' = Xl (buffer s1): planes of Xl' (buffer 1 - par) and Xs', or fp32 X in place of the raw step (`last`)
// WN: the tile has 64 WN columns (Gram and Poly: 2; updates: 2 or 4, a table of jobs each).
// Registers: 64 / 128 accumulator registers plus what the epilogues need; tiles of 256 columns are held to two
// waves per SIMD (256 registers: left alone the epilogue takes 296 and a CU runs one job at a time).
// Which matrices a launch is for, when the chain length is chosen per matrix (k_ns_hf_chain_flag): all of them; those
// whose first chain is the longer one; the others; or all, the others with another first operand buffer and `last`.
enum : int { kNsAll = 0, kNsLongOnly = 1, kNsShortOnly = 2, kNsBoth = 3 };
struct NsPick {
  const int* flags;
  int sel, s1_short, last_short;
  float acc_scale_short;   // with s1_short: that buffer's planes have a scale of their own
};

template <int OP, int WN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WN == 4 ? 2 : 3))) void k_ns_hf_gemm(const NsHfMat* __restrict__ mats, const NsItem* __restrict__ items,
                                                    const PyloTensorArgs* __restrict__ dyn, float* __restrict__ ws,
                                                    hbits* __restrict__ pw, int par, int last, NsBufs bufs, float c0,
                                                    float c1, float c2, NsPick pick) {
  extern __shared__ __attribute__((aligned(16))) char lds_[];
  PYLO_LDS char* lds = (PYLO_LDS char*)lds_;
  const NsItem it = items[blockIdx.x];
  if (it.mat < 0) return;   // a filler job
  if (pick.sel != kNsAll) {
    const bool longer = pick.flags[it.mat] != 0;
    if ((pick.sel == kNsLongOnly && !longer) || (pick.sel == kNsShortOnly && longer)) return;
    if (pick.sel == kNsBoth && !longer) {
      bufs.s1 = pick.s1_short;
      bufs.acc_scale = pick.acc_scale_short;
      last = pick.last_short;
    }
  }
  const NsHfMat mt = mats[it.mat];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  const int m = mt.m, n = mt.n, lda = mt.lda;
  v16f acc[2][WN];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const int i0 = it.tm * kNsTile, j0 = it.tn * 64 * WN;
  // A tile on the diagonal of a symmetric product: the 64 x 64 quadrant below the diagonal is the mirror image of the
  // one above it, which its own wave (wave 1) writes to both places; wave 2 computes and stores nothing.
  const int wave_u = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool diag = OP != kNsUpdate && WN == 2 && it.tm == it.tn;
  const bool idle = diag && wave_u == 2;
  if (OP == kNsGram) {
    const HfPlanes X{pw + mt.off_xs, mt.rows_m};
    hf_tile_product<WN>(X, i0, X, j0, it.k0, it.k1, lds, acc, !idle);
  } else if (OP == kNsPoly) {
    const HfPlanes A{pw + mt.off_p, mt.rows_m};
    hf_tile_product<WN>(A, i0, A, j0, it.k0, it.k1, lds, acc, !idle);
  } else if (OP == kNsUpdate) {
    const HfPlanes X{pw + (par ? mt.off_xl[1] : mt.off_xl[0]), mt.rows_n};   // no run-time index: the struct stays in registers
    const HfPlanes B{pw + mt.off_p + bufs.s1 * mt.p_stride, mt.rows_m};
    hf_tile_product<WN>(X, i0, B, j0, it.k0, it.k1, lds, acc);
  } else {
    const HfPlanes P1{pw + mt.off_p + bufs.s1 * mt.p_stride, mt.rows_m};
    const HfPlanes P2{pw + mt.off_p + bufs.s2 * mt.p_stride, mt.rows_m};
    hf_tile_product<WN>(P1, i0, P2, j0, it.k0, it.k1, lds, acc, !idle);
  }
  if (idle) return;
  // the operands' planes hold their matrices times a power of two each
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] *= bufs.acc_scale;
  float* A32 = ws + mt.off_a;
  const int n_i = OP == kNsUpdate ? n : m;   // rows of the output; its columns are always m
  const bool partial = OP == kNsGram && it.slab >= 0;
  const bool mirror = OP != kNsUpdate && !partial && (it.tm != it.tn || wave_u == 1);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* xout = a.step_out + mt.elem_off;
  const bool vec_out = (mt.C & 3) == 0;   // rows of the tensor are 16-byte aligned
  // fp32 outputs (and Poly's transform of the accumulators) straight from the registers
  if (OP == kNsGram || OP == kNsPoly || OP == kNsProdA || (OP == kNsUpdate && last)) {
#pragma unroll
    for (int hi = 0; hi < 2; ++hi)
#pragma unroll
      for (int hj = 0; hj < WN; ++hj) {
        const int col = j0 + (wave & 1) * 32 * WN + hj * 32 + (lane & 31);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = i0 + ns_acc_row(hi, 4 * q);   // rows row .. row + 3
          if (col >= m || row >= n_i) continue;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float x = acc[hi][hj][4 * q + r];
            if (OP == kNsPoly) {
              const bool in = row + r < m;
              const float aij = in ? A32[(size_t)(row + r) * lda + col] : 0.0f;
              x = in ? c2 * x + c1 * aij + ((row + r) == col ? c0 : 0.0f) : 0.0f;
              acc[hi][hj][4 * q + r] = x;
            }
            v[r] = x;
          }
          if (OP == kNsGram || OP == kNsProdA) {
            float* out = partial ? ws + mt.off_part + (size_t)it.slab * m * lda : A32;
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (row + r < m) out[(size_t)(row + r) * lda + col] = v[r];
            if (mirror) *(gv4f*)(out + (size_t)col * lda + row) = v4f{v[0], v[1], v[2], v[3]};   // past m: zeros into the pitch's padding
          } else if (OP == kNsUpdate) {
            if (mt.tall) {   // X = Xl, n x m
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (row + r < n) xout[(size_t)(row + r) * m + col] = v[r];
            } else if (vec_out) {   // X = Xs, m x n: four consecutive columns of row `col` (n is a multiple of 4)
              *(gv4f*)(xout + (size_t)col * n + row) = v4f{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (row + r < n) xout[(size_t)col * n + row + r] = v[r];
            }
          }
        }
      }
  }
  // planes: A and B' in both halves (the tile itself through LDS, the mirrored tile from the registers), Xl'
  // (through LDS) and Xs' (registers)
  if (partial || (OP == kNsUpdate && last)) return;
  if (OP == kNsUpdate) {
    hf_store_planes<WN>(lds, acc, pw + (par ? mt.off_xl[0] : mt.off_xl[1]), mt.rows_n, i0, j0, n, m, pw + mt.off_xs, mt.rows_m,
                        bufs.out_scale);
  } else {
    hbits* D = pw + mt.off_p + (OP == kNsGram ? (int)kNsBufA : bufs.d) * mt.p_stride;
    hf_store_planes<WN>(lds, acc, D, mt.rows_m, i0, j0, m, m, mirror ? D : nullptr, mt.rows_m, bufs.out_scale);
  }
}

// A = sum over the slabs' partial matrices, in slab order, as fp32 and as planes (both halves).
__global__ __launch_bounds__(256) void k_ns_hf_gram_reduce(const NsHfMat* __restrict__ mats, const int* __restrict__ split_mats,
                                                           const PyloTensorArgs* __restrict__ dyn, float* __restrict__ ws,
                                                           hbits* __restrict__ pw, NsPick pick, float out_scale) {
  if (pick.sel == kNsShortOnly && pick.flags[split_mats[blockIdx.y]] != 0) return;
  const NsHfMat mt = mats[split_mats[blockIdx.y]];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  const int m = mt.m, lda = mt.lda;
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long long)m * m) return;
  const int i = (int)(e / m), j = (int)(e - (long long)i * m);
  if (i / 64 > j / 64) return;   // the Gram jobs compute the 64 x 64 blocks on and above the diagonal
  const size_t mm = (size_t)m * lda;
  const float* p = ws + mt.off_part + (size_t)i * lda + j;
  float s = 0.0f;
  for (int q0 = 0; q0 < mt.n_slabs; q0 += 8) {
    float v[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) v[q] = q0 + q < mt.n_slabs ? *(const gfloat*)(p + (size_t)(q0 + q) * mm) : 0.0f;
#pragma unroll
    for (int q = 0; q < 8; ++q) s += v[q];
  }
  float* A = ws + mt.off_a;
  hbits* P = pw + mt.off_p;   // buffer A
  A[(size_t)i * lda + j] = s;
  hf_store1(P, mt.rows_m, i, j, s * out_scale);
  if (i / 64 != j / 64) {
    A[(size_t)j * lda + i] = s;
    hf_store1(P, mt.rows_m, j, i, s * out_scale);
  }
}

// X0 = raw * s (s = 1 / (||raw|| + eps), scale[mat]) as planes in both layouts.  One block = one 64 x 64
// tile of the raw step (R x C): the planes in which the tensor's rows stay rows are written straight from
// the loaded values, the transposed planes through LDS.
// The length of a matrix's first chain.  With X scaled to unit Frobenius norm, ||A||_F (A = X X^T as computed) bounds
// the largest eigenvalue of A from above; what a chain of three iterations adds to the error of the result is
// proportional to it, 196 eps_A lambda_max against 16 eps_A lambda_max for a pair (head of this file), so three
// iterations are taken where ||A||_F^2 <= tau^2, with tau = 16 / 196: no worse there than a pair is on any matrix.
// Two launches, sums in a fixed order: 4096 elements of A per block, then one block per matrix.
constexpr int kNsFlagChunk = 4096;
// items[b] = {matrix, chunk of 4096 elements of its A}
__global__ __launch_bounds__(256) void k_ns_hf_chain_sumsq(const NsHfMat* __restrict__ mats, const Item* __restrict__ items,
                                                           const PyloTensorArgs* __restrict__ dyn, const float* __restrict__ ws,
                                                           float* __restrict__ part) {
  __shared__ float red[4];
  const Item it = items[blockIdx.x];
  const NsHfMat mt = mats[it.tensor];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  const long long mm = (long long)mt.m * mt.m, e0 = (long long)it.a * kNsFlagChunk;
  const float* A = ws + mt.off_a;
  float s = 0.0f;
  for (int i = 0; i < kNsFlagChunk / 256; ++i) {
    const long long e = e0 + threadIdx.x + 256 * i;
    if (e < mm) {
      const int r = (int)(e / mt.m), c = (int)(e - (long long)r * mt.m);
      const float v = *(const gfloat*)(A + (size_t)r * mt.lda + c);
      s = fmaf(v, v, s);
    }
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) part[mt.fpart0 + it.a] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(64) void k_ns_hf_chain_flag(const NsHfMat* __restrict__ mats, const int* __restrict__ list,
                                                         const PyloTensorArgs* __restrict__ dyn, const float* __restrict__ part,
                                                         float tau2, int* __restrict__ flags) {
  const int q = list[blockIdx.x];
  const NsHfMat mt = mats[q];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  float s = 0.0f;
  for (int b = threadIdx.x; b < mt.n_fpart; b += 64) s += part[mt.fpart0 + b];
  s = wave_sum(s);
  if (threadIdx.x == 0) flags[q] = s <= tau2 ? 1 : 0;
}

struct NsTileItem { int mat, tr, tc; };

__global__ __launch_bounds__(256) void k_ns_hf_split(const NsHfMat* __restrict__ mats, const NsTileItem* __restrict__ items,
                                                     const PyloTensorArgs* __restrict__ dyn, const float* __restrict__ scale,
                                                     hbits* __restrict__ pw, float plane_scale) {
  constexpr int RP = 72;   // numbers per row of the tile in LDS: 64 + 8, rows stay 16-byte aligned
  __shared__ __attribute__((aligned(16))) hbits tile[kNsPl][64][RP];
  const NsTileItem it = items[blockIdx.x];
  const NsHfMat mt = mats[it.mat];
  const PyloTensorArgs a = dyn[mt.tensor];
  if (a.grad == nullptr || !(a.flags & kArgOrthogonalize)) return;
  const float s = scale[it.mat] * plane_scale;
  const int R = mt.R, C = mt.C;
  const float* raw = a.step_out + mt.elem_off;
  const bool vec_in = (C & 3) == 0;
  // direct planes: the tensor's rows are the planes' rows; transposed planes: its columns are
  hbits* direct = pw + (mt.tall ? mt.off_xl[0] : mt.off_xs);
  hbits* transp = pw + (mt.tall ? mt.off_xs : mt.off_xl[0]);
  const int rows_d = mt.tall ? mt.rows_n : mt.rows_m, rows_t = mt.tall ? mt.rows_m : mt.rows_n;
  const int r0 = it.tr * 64, c0 = it.tc * 64;
  const int t = threadIdx.x;
  // Eight consecutive columns of one row a lane and pass: 32 bytes read, one 16-byte piece per plane written
  // to the direct planes (the two lanes of a 16-column block fill its 64 bytes) and to the tile in LDS.
  // Columns and rows past the matrix read as zero; where a piece straddles the edge the zeros land in the
  // planes' padding, which holds zeros anyway.
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int u = pass * 256 + t, lr = u >> 3, lc = 8 * (u & 7);
    const int r = r0 + lr, c = c0 + lc;
    float v[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    const bool in = r < R && c < C;
    if (in) {
      const float* src = raw + (size_t)r * C + c;
      if (vec_in) {
        const v4f x = *(const gv4f*)src;
        v[0] = x.x * s; v[1] = x.y * s; v[2] = x.z * s; v[3] = x.w * s;
        if (c + 4 < C) {
          const v4f y = *(const gv4f*)(src + 4);
          v[4] = y.x * s; v[5] = y.y * s; v[6] = y.z * s; v[7] = y.w * s;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c + e < C) v[e] = *(const gfloat*)(src + e) * s;
      }
    }
    u32x4 pl[kNsPl];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      hbits h0, l0, h1, l1;
      hf_split(v[2 * q], h0, l0);
      hf_split(v[2 * q + 1], h1, l1);
      pl[0][q] = (unsigned)h0 | (unsigned)h1 << 16;
      pl[1][q] = (unsigned)l0 | (unsigned)l1 << 16;
    }
#pragma unroll
    for (int q = 0; q < kNsPl; ++q) *(luint4*)&tile[q][lr][lc] = pl[q];
    if (in) {
      hbits* p = direct + hf_off(rows_d, r, c);
#pragma unroll
      for (int q = 0; q < kNsPl; ++q) *(u32x4*)(p + 16 * q) = pl[q];
    }
  }
  __syncthreads();
  // transposed: a lane takes one column and sixteen rows of the tile, i.e. one row and one 16-step block of
  // the transposed planes: 64 consecutive bytes, and the lanes of a wave (consecutive columns) the next 64
  {
    const int lc = t & 63, rb = t >> 6;
    const int c = c0 + lc, r = r0 + 16 * rb;
    if (c < C && r < R) {
      hbits* p = transp + hf_off(rows_t, c, r);
#pragma unroll
      for (int q = 0; q < kNsPl; ++q)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          u32x4 w;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            w[i] = (unsigned)tile[q][16 * rb + 8 * hf + 2 * i][lc] | (unsigned)tile[q][16 * rb + 8 * hf + 2 * i + 1][lc] << 16;
          *(u32x4*)(p + 16 * q + 8 * hf) = w;
        }
    }
  }
}

}  // namespace pylo
