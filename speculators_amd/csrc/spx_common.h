// Shared device / host helpers of the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <string>

#define SPX_OK 0
#define SPX_ERR_ARG 1
#define SPX_ERR_HIP 2

namespace spx {

// thread-local message returned by spx_last_error()
std::string& last_error();
int fail_arg(const char* fn, const char* what);
int check_launch(const char* fn);
// Raises a kernel's dynamic-LDS limit to `bytes`, once per device: `done` (one object per kernel
// instantiation) holds one bit per device ordinal on which the limit has been raised.  The
// attribute is idempotent, so two threads that race here at worst both set it; devices with an
// ordinal of 64 or more set it on every call.
int ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* fn);

#define SPX_REQUIRE(cond, what) \
  do {                          \
    if (!(cond)) return spx::fail_arg(__func__, what); \
  } while (0)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;  // finite stand-in for -inf in running maxima

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
// two fp32 -> packed bf16 pair with the gfx950 conversion instruction
// (v_cvt_pk_bf16_f32, round-to-nearest-even)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  union { bf16x2_t b; uint32_t u; } c;
  f32x2_t v = {lo, hi};
  c.b = __builtin_convertvector(v, bf16x2_t);
  return c.u;
}

// 16-byte LDS read at a 32-bit LDS address; a constant added to the address goes into the offset
// field of the instruction
__device__ __forceinline__ u32x4 lds_read128(uint32_t addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>((uintptr_t)addr);
}

// acc += a * b with v_mfma_f32_16x16x32_bf16, the accumulator pinned to the accumulation registers
// and written in place.  (With 64 accumulator tuples that fill that register file, the compiler's own
// choice of destination leaves them permuted at the end of a loop body and moves them back through
// vector registers on every trip.)  The compiler does not know what the statement is: whoever reads
// an accumulator with a vector instruction afterwards waits for the matrix pipe first
// (`mfma_results_ready`).
//
// Cross-check build: compiled with -DSPX_MFMA_BUILTIN=1 the same statement is the compiler's own
// builtin, whose result hazards the compiler places itself (slower: the accumulators are copied
// around, see above).  The GEMM tests must pass on both builds; running them once on that build
// after an edit of a kernel that uses mfma16 shows whether a hand-placed wait has gone missing.
#ifndef SPX_MFMA_BUILTIN
#define SPX_MFMA_BUILTIN 0
#endif
__device__ __forceinline__ void mfma16(f32x4& acc, bf16x8 a, bf16x8 b) {
#if SPX_MFMA_BUILTIN
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
#else
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
#endif
}
// more wait states than the longest matrix instruction needs before its result may be read
__device__ __forceinline__ void mfma_results_ready() {
#if !SPX_MFMA_BUILTIN
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#endif
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

template <typename T>
__device__ __forceinline__ T wave_xor(T v, int lane_mask) {
  return __shfl_xor(v, lane_mask, 64);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}

// 64 lanes x 16 bytes, global -> LDS at M0 + IMM + 16 * lane; the global address is
// base + voff + soff + IMM.  Lanes whose voff + IMM lies outside the resource write
// zeros.  M0 is an input operand: the compiler writes it only when the value changes.
// The s_nop covers the M0-write -> LDS-DMA wait state for the first load of a group.
template <int IMM>
__device__ __forceinline__ void load_to_lds16(u32x4 rsrc, uint32_t lds_addr, int voff, int soff) {
  // wave-uniform by contract; the reads cost nothing where the compiler already knows it
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  soff = __builtin_amdgcn_readfirstlane(soff);
  if (IMM == 0)
    asm volatile("s_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "{m0}"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
  else
    asm volatile("buffer_load_dwordx4 %1, %2, %3 offen offset:%4 lds"
                 :
                 : "{m0}"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM)
                 : "memory");
}

// 64 lanes x 4 bytes, global -> LDS at M0 + 4 * lane (same addressing as load_to_lds16)
__device__ __forceinline__ void load_to_lds4(u32x4 rsrc, uint32_t lds_addr, int voff, int soff) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  soff = __builtin_amdgcn_readfirstlane(soff);
  asm volatile("s_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "{m0}"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}

// buffer resource over `bytes` bytes at p (raw, no stride): offsets past the end read as zero
__device__ __forceinline__ u32x4 make_rsrc(const void* p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  u32x4 r;
  r.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r.z = __builtin_amdgcn_readfirstlane(bytes);
  r.w = 0x00020000u;
  return r;
}

}  // namespace spx
