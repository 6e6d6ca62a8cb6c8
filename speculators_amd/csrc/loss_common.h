// Row streaming helpers shared by the vocabulary-loss kernels (gfx950): 8-element chunk
// loads / stores of bf16 or fp32 rows with 16-byte non-temporal accesses.
#pragma once

#include "spx_common.h"

namespace spx {

constexpr int kLossThreads = 256;
constexpr int kLossWaves = kLossThreads / 64;

// ---- 8-element chunk loads -------------------------------------------------
// VEC: the row base is 16-byte aligned and the chunk is complete.
template <typename T>
__device__ __forceinline__ void load8_vec(const T* p, float v[8]);

// streaming accesses bypass the cache hierarchy's allocate-on-access policy: every row is
// read (and every gradient row written) exactly once per launch
#define SPX_LOSS_NT 1
__device__ __forceinline__ u32x4 ld16(const void* p) {
#if SPX_LOSS_NT
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
#else
  return *reinterpret_cast<const u32x4*>(p);
#endif
}
__device__ __forceinline__ void st16(void* p, u32x4 v) {
#if SPX_LOSS_NT
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
#else
  *reinterpret_cast<u32x4*>(p) = v;
#endif
}
template <>
__device__ __forceinline__ void load8_vec<uint16_t>(const uint16_t* p, float v[8]) {
  u32x4 raw = ld16(p);
  v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x);
  v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
  v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z);
  v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
}
template <>
__device__ __forceinline__ void load8_vec<float>(const float* p, float v[8]) {
  f32x4 a = *reinterpret_cast<const f32x4*>(p);
  f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

__device__ __forceinline__ float load1(const uint16_t* p) { return bf16_bits_to_f32(*p); }
__device__ __forceinline__ float load1(const float* p) { return *p; }

template <typename T>
__device__ __forceinline__ void load8_guard(const T* p, int64_t base, int64_t n, float v[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (base + i < n) ? load1(p + base + i) : kNegBig;
}

template <typename T, bool VEC>
__device__ __forceinline__ void load8(const T* row, int64_t base, int64_t n, float v[8]) {
  if (VEC && base + 8 <= n) load8_vec<T>(row + base, v);
  else load8_guard<T>(row, base, n, v);
}

template <typename T>
__device__ __forceinline__ void store8_vec(T* p, const float v[8]);
template <>
__device__ __forceinline__ void store8_vec<uint16_t>(uint16_t* p, const float v[8]) {
  u32x4 raw;
  raw.x = pack_bf16x2(v[0], v[1]); raw.y = pack_bf16x2(v[2], v[3]);
  raw.z = pack_bf16x2(v[4], v[5]); raw.w = pack_bf16x2(v[6], v[7]);
  st16(p, raw);
}
template <>
__device__ __forceinline__ void store8_vec<float>(float* p, const float v[8]) {
  f32x4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
  *reinterpret_cast<f32x4*>(p) = a;
  *reinterpret_cast<f32x4*>(p + 4) = b;
}
__device__ __forceinline__ void store1(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
__device__ __forceinline__ void store1(float* p, float v) { *p = v; }

template <typename T, bool VEC>
__device__ __forceinline__ void store8(T* row, int64_t base, int64_t n, const float v[8]) {
  if (VEC && base + 8 <= n) store8_vec<T>(row + base, v);
  else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (base + i < n) store1(row + base + i, v[i]);
  }
}

__host__ __device__ __forceinline__ bool ptr_aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

}  // namespace spx
