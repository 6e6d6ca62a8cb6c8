// Row movement around the expert products of a sparse MoE block for gfx950 (HBM-bound, bf16 rows,
// 16-byte accesses).  The (token, slot) pairs of the router's top-k choice are sorted by expert on
// the host side of the library (a permutation, no arithmetic); these kernels move rows between the
// token order [T, H] and the sorted order [T * k, H]:
//   gather   sorted[p]  = scale[p] * x[src_row[p]]                      (scale optional)
//   combine  out[t]     = sum_j weight[t, j] * sorted[pos[t, j]]        (weight optional)
//   dot      d[t, j]    = <a[t], sorted[pos[t, j]]>                     (gradient of the router scores)
// Sums run in fp32 in the order j = 0 .. k-1 and are rounded once.

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {
namespace moe {

__device__ __forceinline__ void unpack8(u32x4 raw, float v[8]) {
  v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x);
  v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
  v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z);
  v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
}
__device__ __forceinline__ u32x4 pack8(const float v[8]) {
  u32x4 r;
  r.x = pack_bf16x2(v[0], v[1]); r.y = pack_bf16x2(v[2], v[3]);
  r.z = pack_bf16x2(v[4], v[5]); r.w = pack_bf16x2(v[6], v[7]);
  return r;
}

// one thread: 8 consecutive columns of one sorted row
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint16_t* __restrict__ x, int64_t ld_x,
                                                          const int32_t* __restrict__ src_row,
                                                          const float* __restrict__ scale,
                                                          uint16_t* __restrict__ out, int64_t ld_out,
                                                          int64_t rows, int64_t src_rows, int h8) {
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= rows * h8) return;
  const int64_t p = item / h8;
  const int c = (int)(item % h8) * 8;
  const int64_t r = src_row[p];
  u32x4 raw = {0u, 0u, 0u, 0u};
  if (r >= 0 && r < src_rows) raw = *reinterpret_cast<const u32x4*>(x + r * ld_x + c);
  if (scale) {
    float v[8];
    unpack8(raw, v);
    const float s = scale[p];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= s;
    raw = pack8(v);
  }
  *reinterpret_cast<u32x4*>(out + p * ld_out + c) = raw;
}

// one thread: 8 consecutive columns of one token row, the k sorted rows added in slot order
__global__ __launch_bounds__(256) void combine_rows_kernel(const uint16_t* __restrict__ sorted, int64_t ld_s,
                                                           const int32_t* __restrict__ pos,
                                                           const float* __restrict__ weight,
                                                           uint16_t* __restrict__ out, int64_t ld_out,
                                                           int64_t tokens, int k, int64_t sorted_rows, int h8) {
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= tokens * h8) return;
  const int64_t t = item / h8;
  const int c = (int)(item % h8) * 8;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < k; ++j) {
    const int64_t p = pos[t * k + j];
    if (p < 0 || p >= sorted_rows) continue;
    float v[8];
    unpack8(*reinterpret_cast<const u32x4*>(sorted + p * ld_s + c), v);
    const float w = weight ? weight[t * k + j] : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += w * v[e];
  }
  *reinterpret_cast<u32x4*>(out + t * ld_out + c) = pack8(acc);
}

// one wave per (token, slot)
__global__ __launch_bounds__(256) void pair_dot_kernel(const uint16_t* __restrict__ a, int64_t ld_a,
                                                       const uint16_t* __restrict__ sorted, int64_t ld_s,
                                                       const int32_t* __restrict__ pos, float* __restrict__ out,
                                                       int64_t pairs, int k, int64_t sorted_rows, int h8) {
  const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = pair / k;
  const int64_t p = pos[pair];
  float sum = 0.f;
  if (p >= 0 && p < sorted_rows) {
    for (int ch = lane; ch < h8; ch += 64) {
      float u[8], v[8];
      unpack8(*reinterpret_cast<const u32x4*>(a + t * ld_a + ch * 8), u);
      unpack8(*reinterpret_cast<const u32x4*>(sorted + p * ld_s + ch * 8), v);
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += u[e] * v[e];
    }
  }
  sum = wave_sum(sum);
  if (lane == 0) out[pair] = sum;
}

}  // namespace moe
}  // namespace spx

using namespace spx;

static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" int spx_moe_gather_rows(const void* x, int64_t ld_x, int64_t src_rows, const int32_t* src_row,
                                   const float* scale, void* out, int64_t ld_out, int64_t rows, int64_t H,
                                   void* stream) {
  SPX_REQUIRE(rows > 0 && src_rows > 0 && H > 0 && H % 8 == 0, "rows > 0 and H a positive multiple of 8");
  SPX_REQUIRE(x && src_row && out && al16(x) && al16(out), "null or unaligned buffer");
  SPX_REQUIRE(ld_x % 8 == 0 && ld_out % 8 == 0 && ld_x >= H && ld_out >= H, "row strides must be multiples of 8 and at least H");
  const int64_t items = rows * (H / 8);
  hipLaunchKernelGGL(moe::gather_rows_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(x), ld_x, src_row,
                     scale, reinterpret_cast<uint16_t*>(out), ld_out, rows, src_rows, (int)(H / 8));
  return check_launch(__func__);
}

extern "C" int spx_moe_combine_rows(const void* sorted, int64_t ld_sorted, int64_t sorted_rows,
                                    const int32_t* pos, const float* weight, void* out, int64_t ld_out,
                                    int64_t tokens, int32_t k, int64_t H, void* stream) {
  SPX_REQUIRE(tokens > 0 && k > 0 && sorted_rows > 0 && H > 0 && H % 8 == 0, "tokens, k > 0 and H a positive multiple of 8");
  SPX_REQUIRE(sorted && pos && out && al16(sorted) && al16(out), "null or unaligned buffer");
  SPX_REQUIRE(ld_sorted % 8 == 0 && ld_out % 8 == 0 && ld_sorted >= H && ld_out >= H,
              "row strides must be multiples of 8 and at least H");
  const int64_t items = tokens * (H / 8);
  hipLaunchKernelGGL(moe::combine_rows_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(sorted), ld_sorted,
                     pos, weight, reinterpret_cast<uint16_t*>(out), ld_out, tokens, (int)k, sorted_rows,
                     (int)(H / 8));
  return check_launch(__func__);
}

extern "C" int spx_moe_pair_dot(const void* a, int64_t ld_a, const void* sorted, int64_t ld_sorted,
                                int64_t sorted_rows, const int32_t* pos, float* out, int64_t tokens,
                                int32_t k, int64_t H, void* stream) {
  SPX_REQUIRE(tokens > 0 && k > 0 && sorted_rows > 0 && H > 0 && H % 8 == 0, "tokens, k > 0 and H a positive multiple of 8");
  SPX_REQUIRE(a && sorted && pos && out && al16(a) && al16(sorted), "null or unaligned buffer");
  SPX_REQUIRE(ld_a % 8 == 0 && ld_sorted % 8 == 0 && ld_a >= H && ld_sorted >= H,
              "row strides must be multiples of 8 and at least H");
  const int64_t pairs = tokens * k;
  hipLaunchKernelGGL(moe::pair_dot_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(a), ld_a,
                     reinterpret_cast<const uint16_t*>(sorted), ld_sorted, pos, out, pairs, (int)k, sorted_rows,
                     (int)(H / 8));
  return check_launch(__func__);
}
