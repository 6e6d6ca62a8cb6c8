// Hardware probes for gfx950 (measurement only; built into libspx_probes.so, which nothing but
// `bench.py --probes` loads).  Each probe answers one question the kernels of this library were
// designed around, with a kernel small enough to read:
//   0  matrix pipe: v_mfma_f32_32x32x16_bf16 from registers only, random or zero operands
//      -> TFLOP/s and the shader clock the chip holds under that load
//   1  LDS read bandwidth per CU (ds_read_b128, conflict free, 8 waves)
//   2  what a wave's vector arithmetic costs while the other wave of its SIMD keeps the matrix
//      pipe busy (two waves per SIMD, one role each)
//   3  what a wave pays for issuing global -> LDS loads (buffer_load_dwordx4 ... lds) while the
//      other waves of the CU read LDS and run MFMAs
//   4  matrix pipe as in 0 with v_mfma_f32_16x16x32_bf16 (the same multiply-adds per cycle; the
//      accumulator is read and written half as often per multiply-add)
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

#define PROBE_CHECK(x) do { if ((x) != hipSuccess) return -1; } while (0)

// ---- 0: matrix pipe ---------------------------------------------------------------------------
__global__ __launch_bounds__(256, 1) void mfma_kernel(const float* seed, float* out, unsigned long long* clk,
                                                      int iters, int zero) {
  const int lane = threadIdx.x & 63;
  bf16x8 x, y;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] = (__bf16)(zero ? 0.f : seed[(threadIdx.x * 8 + i) & 4095]);
    y[i] = (__bf16)(zero ? 0.f : seed[(threadIdx.x * 8 + i + 2048) & 4095]);
  }
  f32x16 a0 = {}, a1 = {}, a2 = {}, a3 = {};
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      a0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a1, 0, 0, 0);
      a2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a2, 0, 0, 0);
      a3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a3, 0, 0, 0);
    }
  }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0 && blockIdx.x == 0) { clk[0] = c1 - c0; clk[1] = r1 - r0; }
  out[blockIdx.x * 256 + threadIdx.x] = a0[lane & 15] + a1[1] + a2[2] + a3[3];
}

// ---- 4: matrix pipe, 16 x 16 x 32 --------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) float f32x4;
__global__ __launch_bounds__(256, 1) void mfma16_kernel(const float* seed, float* out, unsigned long long* clk,
                                                        int iters, int zero) {
  bf16x8 x[4], y[4];
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x[f][i] = (__bf16)(zero ? 0.f : seed[(threadIdx.x * 8 + i + 97 * f) & 4095]);
      y[f][i] = (__bf16)(zero ? 0.f : seed[(threadIdx.x * 8 + i + 2048 + 131 * f) & 4095]);
    }
  f32x4 a[64];
#pragma unroll
  for (int q = 0; q < 64; ++q) a[q] = {};
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int q = 0; q < 64; ++q)
      a[q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[q & 3], y[(q >> 2) & 3], a[q], 0, 0, 0);
  }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0 && blockIdx.x == 0) { clk[0] = c1 - c0; clk[1] = r1 - r0; }
  float r = 0.f;
#pragma unroll
  for (int q = 0; q < 64; ++q) r += a[q][1];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

// ---- 1: LDS reads -----------------------------------------------------------------------------
__global__ __launch_bounds__(512, 1) void lds_kernel(uint32_t* out, unsigned long long* clk, int iters) {
  extern __shared__ __attribute__((aligned(16))) uint8_t sm[];
  for (int i = threadIdx.x; i < 8192; i += 512) reinterpret_cast<uint32_t*>(sm)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  u32x4 acc = {0, 0, 0, 0};
  const unsigned long long c0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
    const __attribute__((address_space(3))) uint8_t* p =
        (const __attribute__((address_space(3))) uint8_t*)sm + lane * 16 + ((it & 1) << 14);
    u32x4 v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      v[u] = *reinterpret_cast<const volatile __attribute__((address_space(3))) u32x4*>(p + u * 1024);
#pragma unroll
    for (int u = 0; u < 16; ++u) acc ^= v[u];
  }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime();
  if (threadIdx.x == 0 && blockIdx.x == 0) clk[0] = c1 - c0;
  out[blockIdx.x * 512 + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

// ---- 2: vector arithmetic beside a busy matrix pipe ---------------------------------------------
template <int MODE>  // 0: v_exp_f32, 1: v_fma_f32, 2: v_max_f32 + v_add_f32
__global__ __launch_bounds__(512, 1) void coexec_kernel(float* out, unsigned long long* clk, int iters, int run_mfma,
                                                        int run_valu) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  float r = 0.f;
  if (wave < 4) {  // waves w and w + 4 share a SIMD
    if (run_mfma) {
      f32x16 a0 = {}, a1 = {}, a2 = {}, a3 = {};
      bf16x8 x, y;
      for (int i = 0; i < 8; ++i) { x[i] = (__bf16)(lane * 0.001f + i); y[i] = (__bf16)(lane * 0.002f - i); }
      for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          a0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a0, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a1, 0, 0, 0);
          a2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a2, 0, 0, 0);
          a3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a3, 0, 0, 0);
        }
      }
      r = a0[0] + a1[1] + a2[2] + a3[3];
    }
  } else if (run_valu) {
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = lane * 0.01f + i;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (MODE == 0) v[i] = __builtin_amdgcn_exp2f(v[i]);
          else if (MODE == 1) v[i] = v[i] * 1.0001f + 0.5f;
          else v[i] = fmaxf(v[i], v[(i + 1) & 15]) + 1.f;
          asm volatile("" : "+v"(v[i]));
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) r += v[i];
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  if (lane == 0 && blockIdx.x == 0) clk[wave] = t1 - t0;
  out[blockIdx.x * 512 + threadIdx.x] = r;
}

// ---- 3: issuing global -> LDS loads ---------------------------------------------------------------
__device__ __forceinline__ u32x4 make_rsrc(const void* p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  u32x4 r;
  r.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r.z = __builtin_amdgcn_readfirstlane(bytes);
  r.w = 0x00020000u;
  return r;
}
template <int BG>  // waves 4-7: 0 idle, 1 read LDS and run MFMAs
__global__ __launch_bounds__(512, 1) void dma_kernel(const uint32_t* src, uint32_t* out, unsigned long long* clk,
                                                     int iters) {
  extern __shared__ __attribute__((aligned(16))) uint8_t sm[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const u32x4 rs = make_rsrc(src, 1u << 24);  // range-checked: an offset past the end reads zeros
  u32x4 acc = {0, 0, 0, 0};
  unsigned long long issue = 0;
  constexpr int NB = 4;
  if (wave < 4) {
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)sm + 65536 + wave * NB * 1024;
    for (int it = 0; it < iters; ++it) {
      const int base = ((it * 4 + wave) * NB * 1024) & ((1 << 20) - 1);
      const unsigned long long t0 = __builtin_amdgcn_s_memtime();
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds0 + j * 1024);
        asm volatile("s_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "{m0}"(m0), "v"(lane * 16 + base + j * 1024), "s"(rs), "s"(0)
                     : "memory");
      }
      issue += __builtin_amdgcn_s_memtime() - t0;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_sleep(8);
    }
  } else if (BG) {
    const __attribute__((address_space(3))) uint8_t* lp =
        (const __attribute__((address_space(3))) uint8_t*)sm + (wave - 4) * 16384 + lane * 16;
    f32x16 a0 = {}, a1 = {};
    bf16x8 x, y;
    for (int i = 0; i < 8; ++i) { x[i] = (__bf16)(lane * 0.001f + i); y[i] = (__bf16)(lane * 0.002f - i); }
    for (int it = 0; it < iters * 6; ++it) {
      u32x4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        v[u] = *reinterpret_cast<const volatile __attribute__((address_space(3))) u32x4*>(lp + u * 1024);
        if (u & 1) a1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a1, 0, 0, 0);
        else a0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, a0, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    acc.x ^= __float_as_uint(a0[0] + a1[1]);
  }
  if (lane == 0 && blockIdx.x == 0 && wave == 0) clk[0] = issue;
  out[blockIdx.x * 512 + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

struct Buffers {
  float* seed = nullptr;
  float* out = nullptr;
  unsigned long long* clk = nullptr;
  uint32_t* src = nullptr;
  ~Buffers() { (void)hipFree(seed); (void)hipFree(out); (void)hipFree(clk); (void)hipFree(src); }
};

template <typename F>
int timed(F&& launch, float* ms) {
  hipEvent_t a, b;
  PROBE_CHECK(hipEventCreate(&a));
  PROBE_CHECK(hipEventCreate(&b));
  launch();  // warm-up
  PROBE_CHECK(hipEventRecord(a, 0));
  launch();
  PROBE_CHECK(hipEventRecord(b, 0));
  PROBE_CHECK(hipEventSynchronize(b));
  PROBE_CHECK(hipEventElapsedTime(ms, a, b));
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

// out[0 .. n): results of probe `which` (see the head of the file); returns the number of values written, < 0 on error.
//   0: {TFLOP/s random operands, shader GHz under that load, TFLOP/s zero operands, shader GHz}
//   1: {bytes per shader clock per CU, bytes per ns per CU}
//   2: for each of the three vector mixes {cycles per 32 MFMAs alone, cycles of the vector loop body alone,
//      cycles per 32 MFMAs together, cycles of the vector loop body together}  (12 values)
//   3: {cycles per 1 KB load with the other waves idle, with the other waves reading LDS and running MFMAs}
//   4: as 0, with v_mfma_f32_16x16x32_bf16
extern "C" int spx_probe(int which, double* out, int n) {
  Buffers b;
  hipDeviceProp_t prop;
  PROBE_CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  PROBE_CHECK(hipMalloc(&b.seed, 4096 * 4));
  PROBE_CHECK(hipMalloc(&b.out, (size_t)cus * 8 * 512 * 4));
  PROBE_CHECK(hipMalloc(&b.clk, 64 * 8));
  PROBE_CHECK(hipMalloc(&b.src, 1 << 24));
  PROBE_CHECK(hipMemset(b.src, 1, 1 << 24));
  std::vector<float> h(4096);
  uint32_t s = 12345u;
  for (auto& v : h) { s = s * 1664525u + 1013904223u; v = ((s >> 8) & 0xffff) / 32768.f - 1.f; }
  PROBE_CHECK(hipMemcpy(b.seed, h.data(), 4096 * 4, hipMemcpyHostToDevice));
  unsigned long long clk[8];
  if (which == 0) {
    if (n < 4) return -2;
    const int iters = 4000, wgs = cus * 4;  // four workgroups of four waves per CU: occupancy is one wave per SIMD
    for (int zero = 0; zero < 2; ++zero) {
      float ms;
      if (timed([&] { hipLaunchKernelGGL(mfma_kernel, dim3(wgs), dim3(256), 0, 0, b.seed, b.out, b.clk, iters, zero); }, &ms))
        return -1;
      PROBE_CHECK(hipMemcpy(clk, b.clk, 16, hipMemcpyDeviceToHost));
      const double flop = (double)wgs * 4 * iters * 32 * 2.0 * 32 * 32 * 16;
      out[2 * zero] = flop / (ms * 1e-3) / 1e12;
      out[2 * zero + 1] = (double)clk[0] / ((double)clk[1] * 10.0);  // s_memrealtime counts at 100 MHz
    }
    return 4;
  }
  if (which == 4) {
    if (n < 4) return -2;
    const int iters = 2000, wgs = cus * 4;  // 64 MFMAs of 16 x 16 x 32 per iteration = 32 of 32 x 32 x 16
    for (int zero = 0; zero < 2; ++zero) {
      float ms;
      if (timed([&] { hipLaunchKernelGGL(mfma16_kernel, dim3(wgs), dim3(256), 0, 0, b.seed, b.out, b.clk, iters, zero); }, &ms))
        return -1;
      PROBE_CHECK(hipMemcpy(clk, b.clk, 16, hipMemcpyDeviceToHost));
      const double flop = (double)wgs * 4 * iters * 64 * 2.0 * 16 * 16 * 32;
      out[2 * zero] = flop / (ms * 1e-3) / 1e12;
      out[2 * zero + 1] = (double)clk[0] / ((double)clk[1] * 10.0);
    }
    return 4;
  }
  if (which == 1) {
    if (n < 2) return -2;
    const int iters = 4000;
    float ms;
    if (timed([&] { hipLaunchKernelGGL(lds_kernel, dim3(cus), dim3(512), 32768, 0, (uint32_t*)b.out, b.clk, iters); }, &ms))
      return -1;
    PROBE_CHECK(hipMemcpy(clk, b.clk, 8, hipMemcpyDeviceToHost));
    const double bytes = 8.0 * 16 * 1024 * iters;
    out[0] = bytes / (double)clk[0];
    out[1] = bytes / (ms * 1e6);
    return 2;
  }
  if (which == 2) {
    if (n < 12) return -2;
    const int iters = 2000;
    for (int mode = 0; mode < 3; ++mode)
      for (int cfg = 0; cfg < 3; ++cfg) {
        const int rm = cfg != 1, rv = cfg != 0;
        for (int rep = 0; rep < 2; ++rep) {
          if (mode == 0) hipLaunchKernelGGL(coexec_kernel<0>, dim3(cus), dim3(512), 0, 0, b.out, b.clk, iters, rm, rv);
          else if (mode == 1) hipLaunchKernelGGL(coexec_kernel<1>, dim3(cus), dim3(512), 0, 0, b.out, b.clk, iters, rm, rv);
          else hipLaunchKernelGGL(coexec_kernel<2>, dim3(cus), dim3(512), 0, 0, b.out, b.clk, iters, rm, rv);
        }
        PROBE_CHECK(hipDeviceSynchronize());
        PROBE_CHECK(hipMemcpy(clk, b.clk, 64, hipMemcpyDeviceToHost));
        if (cfg == 0) out[4 * mode + 0] = (double)clk[0] / iters;
        if (cfg == 1) out[4 * mode + 1] = (double)clk[4] / iters;
        if (cfg == 2) { out[4 * mode + 2] = (double)clk[0] / iters; out[4 * mode + 3] = (double)clk[4] / iters; }
      }
    return 12;
  }
  if (which == 3) {
    if (n < 2) return -2;
    const int iters = 300;
    PROBE_CHECK(hipFuncSetAttribute((const void*)dma_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, 81920));
    PROBE_CHECK(hipFuncSetAttribute((const void*)dma_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 81920));
    for (int bg = 0; bg < 2; ++bg) {
      for (int rep = 0; rep < 2; ++rep) {
        if (bg == 0) hipLaunchKernelGGL(dma_kernel<0>, dim3(cus), dim3(512), 81920, 0, b.src, (uint32_t*)b.out, b.clk, iters);
        else hipLaunchKernelGGL(dma_kernel<1>, dim3(cus), dim3(512), 81920, 0, b.src, (uint32_t*)b.out, b.clk, iters);
      }
      PROBE_CHECK(hipDeviceSynchronize());
      PROBE_CHECK(hipMemcpy(clk, b.clk, 8, hipMemcpyDeviceToHost));
      out[bg] = (double)clk[0] / iters / 4;
    }
    return 2;
  }
  return -3;
}
