// Gradients and parameters stored as fp16, bf16 or fp64 (PYLO_F_STORE_*).
//
// The reference instantiates its kernels per element type, widens every value to float on load and narrows
// on store (celo2_kernel.cu:70-75,280,314).  The fused passes here are written for fp32 streams (64- and
// 128-bit accesses, byte offsets of 4-byte elements), so a tagged tensor is widened once per step into fp32
// staging inside the plan's workspace (k_cast_in), every pass of the step reads and writes the staging
// through a substituted argument record (k_stage_args), and what the step wrote to the parameter is rounded
// to nearest-even back into the caller's buffer (k_cast_out).  Against 72 bytes per element of a factored
// tensor this adds 18 (16-bit types) or 36 (fp64) bytes; tensors without a tag are not touched by any of it.
#pragma once

#include "pylo_common.h"

namespace pylo {

enum : int { kStoreF32 = 0, kStoreF16 = 1, kStoreBF16 = 2, kStoreF64 = 3 };

constexpr int kCastElems = 8192;   // elements per block of the cast kernels

typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
typedef double v2d __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float widen16(unsigned short b, int store) {
  return store == kStoreBF16 ? __uint_as_float((unsigned)b << 16) : (float)__builtin_bit_cast(_Float16, b);
}
__device__ __forceinline__ unsigned short narrow16(float x, int store) {
  return store == kStoreBF16 ? __builtin_bit_cast(unsigned short, (__bf16)x)
                             : __builtin_bit_cast(unsigned short, (_Float16)x);
}

// One element of a tagged buffer (generic paths; the cast kernels below move vectors).
__device__ __forceinline__ float load_stored(const void* base, long long i, int store) {
  if (store == kStoreF64) return (float)((const double*)base)[i];
  if (store == kStoreF32) return ((const float*)base)[i];
  return widen16(((const unsigned short*)base)[i], store);
}
__device__ __forceinline__ void store_stored(void* base, long long i, int store, float x) {
  if (store == kStoreF64) ((double*)base)[i] = (double)x;
  else if (store == kStoreF32) ((float*)base)[i] = x;
  else ((unsigned short*)base)[i] = narrow16(x, store);
}

// src (storage type) -> dst (fp32), elements [0, lim) of a block's piece; both 16-byte aligned when vec.
__device__ __forceinline__ void widen_piece(const void* src, float* dst, unsigned lim, int store, bool vec) {
  if (vec && store != kStoreF64) {          // 8 elements a lane and trip: one 16-byte load, two 16-byte stores
    for (unsigned off = threadIdx.x * 8u; off < lim; off += kThreads * 8u) {
      const u16x8 w = *(const u16x8*)((const unsigned short*)src + off);
      float x[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = widen16(w[j], store);
      *(v4f*)(dst + off) = v4f{x[0], x[1], x[2], x[3]};
      *(v4f*)(dst + off + 4) = v4f{x[4], x[5], x[6], x[7]};
    }
  } else if (vec) {                         // fp64: two 16-byte loads, one 16-byte store
    for (unsigned off = threadIdx.x * 4u; off < lim; off += kThreads * 4u) {
      const v2d a = *(const v2d*)((const double*)src + off), b = *(const v2d*)((const double*)src + off + 2);
      *(v4f*)(dst + off) = v4f{(float)a.x, (float)a.y, (float)b.x, (float)b.y};
    }
  } else {
    for (unsigned off = threadIdx.x; off < lim; off += kThreads) dst[off] = load_stored(src, off, store);
  }
}

__device__ __forceinline__ void narrow_piece(const float* src, void* dst, unsigned lim, int store, bool vec) {
  if (vec && store != kStoreF64) {
    for (unsigned off = threadIdx.x * 8u; off < lim; off += kThreads * 8u) {
      const v4f a = *(const v4f*)(src + off), b = *(const v4f*)(src + off + 4);
      u16x8 w;
      w[0] = narrow16(a.x, store); w[1] = narrow16(a.y, store); w[2] = narrow16(a.z, store); w[3] = narrow16(a.w, store);
      w[4] = narrow16(b.x, store); w[5] = narrow16(b.y, store); w[6] = narrow16(b.z, store); w[7] = narrow16(b.w, store);
      *(u16x8*)((unsigned short*)dst + off) = w;
    }
  } else if (vec) {
    for (unsigned off = threadIdx.x * 4u; off < lim; off += kThreads * 4u) {
      const v4f a = *(const v4f*)(src + off);
      *(v2d*)((double*)dst + off) = v2d{(double)a.x, (double)a.y};
      *(v2d*)((double*)dst + off + 2) = v2d{(double)a.z, (double)a.w};
    }
  } else {
    for (unsigned off = threadIdx.x; off < lim; off += kThreads) store_stored(dst, off, store, src[off]);
  }
}

// Per tagged tensor: floats into the staging area of its gradient and of its parameter (-1: not tagged).
struct StageOfs { long long g, p; };

// dyn[t] = user[t], with grad / param of a tagged tensor that takes part pointing into the staging.
__global__ __launch_bounds__(256) void k_stage_args(int T, const TDesc* __restrict__ descs,
                                                    const PyloTensorArgs* __restrict__ user,
                                                    PyloTensorArgs* __restrict__ dyn, const StageOfs* __restrict__ ofs,
                                                    float* __restrict__ stage) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  PyloTensorArgs a = user[t];
  if (descs[t].store != kStoreF32 && a.grad != nullptr) {
    a.grad = stage + ofs[t].g;
    a.param = stage + ofs[t].p;
  }
  dyn[t] = a;
}

// Items: (tensor, piece of kCastElems elements).  what: 1 = gradient, 2 = parameter, 3 = both.
__global__ __launch_bounds__(kThreads) void k_cast_in(const TDesc* __restrict__ descs,
                                                      const PyloTensorArgs* __restrict__ user,
                                                      const Item* __restrict__ items, const StageOfs* __restrict__ ofs,
                                                      float* __restrict__ stage, int what) {
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = user[it.tensor];
  if (a.grad == nullptr) return;
  const long long base = (long long)it.a * kCastElems;
  const long long left = d.n - base;
  const unsigned lim = left < (long long)kCastElems ? (unsigned)left : (unsigned)kCastElems;
  const int esz = d.store == kStoreF64 ? 8 : 2;
  const bool vec = d.n % 8 == 0;   // pieces start at multiples of 8192 elements: 16-byte aligned in every type
  const StageOfs o = ofs[it.tensor];
  if (what & 1) widen_piece((const char*)a.grad + base * esz, stage + o.g + base, lim, d.store, vec);
  if (what & 2) widen_piece((const char*)a.param + base * esz, stage + o.p + base, lim, d.store, vec);
}

// The staged parameter back into the caller's buffer.  flat_only: only tensors the ELO-CELO2 step itself
// updates (its AdamW tensors; the matrices are updated by the finishing pass).
__global__ __launch_bounds__(kThreads) void k_cast_out(const TDesc* __restrict__ descs,
                                                       const PyloTensorArgs* __restrict__ user,
                                                       const Item* __restrict__ items, const StageOfs* __restrict__ ofs,
                                                       const float* __restrict__ stage, int flat_only) {
  const Item it = items[blockIdx.x];
  const TDesc d = descs[it.tensor];
  const PyloTensorArgs a = user[it.tensor];
  if (a.grad == nullptr || (flat_only && d.mode != kModeFlat)) return;
  const long long base = (long long)it.a * kCastElems;
  const long long left = d.n - base;
  const unsigned lim = left < (long long)kCastElems ? (unsigned)left : (unsigned)kCastElems;
  const int esz = d.store == kStoreF64 ? 8 : 2;
  narrow_piece(stage + ofs[it.tensor].p + base, (char*)a.param + base * esz, lim, d.store, d.n % 8 == 0);
}

}  // namespace pylo
