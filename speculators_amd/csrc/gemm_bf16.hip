// C[M, N] = A[M, K] * B[N, K]^T  (the nn.Linear product), bf16 in, fp32
// accumulate, bf16 out, for gfx950.
//
// One workgroup of 4 waves owns a 256 x 256 tile of C and walks K in steps of
// 64; each wave owns a 128 x 128 quadrant as 4 x 4 accumulators of
// v_mfma_f32_32x32x16_bf16 (256 accumulator registers per lane).  A and B
// tiles are staged global -> registers -> LDS with the next tile's global
// loads in flight during the current tile's MFMAs.  LDS rows are padded by 16
// bytes so the 16-byte operand reads of 16 consecutive lanes hit 16 distinct
// bank groups.  Workgroup ids are remapped so that each XCD (ids are dealt
// round-robin over the 8 XCDs) works on a compact band of tiles and shares
// its A / B panels in that XCD's L2.

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

constexpr int kGemmThreads = 256;
constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kLdsStride = kTK + 8;  // elements
constexpr int kGemmSmem = (kTM + kTN) * kLdsStride * 2;

__device__ __forceinline__ bf16x8 lds_frag(const uint16_t* p) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = *reinterpret_cast<const u32x4*>(p);
  return c.b;
}

__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_nt_kernel(
    const uint16_t* __restrict__ A, int64_t lda, const uint16_t* __restrict__ B, int64_t ldb,
    uint16_t* __restrict__ C, int64_t ldc, int M, int N, int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* As = smem;
  uint16_t* Bs = smem + kTM * kLdsStride;

  // workgroup id -> tile: XCD-contiguous bands, then groups of 8 tile rows
  const int n_wg = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per_xcd = (n_wg + 7) / 8;
    const int xcd = pid % 8, local = pid / 8;
    const int cand = xcd * per_xcd + local;
    // only remap when the grid divides evenly, otherwise keep the identity
    if (n_wg % 8 == 0) pid = cand;
  }
  constexpr int GROUP_M = 8;
  const int in_group = GROUP_M * tiles_n;
  const int group_id = pid / in_group;
  const int first_m = group_id * GROUP_M;
  const int group_sz = min(tiles_m - first_m, GROUP_M);
  const int tile_m = first_m + (pid % in_group) % group_sz;
  const int tile_n = (pid % in_group) / group_sz;
  const int m0 = tile_m * kTM, n0 = tile_n * kTN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, col = lane & 31;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;

  // global -> register staging: 8 chunks of 16 bytes per operand per thread
  const int lrow = tid >> 3, lcol = (tid & 7) * 8;
  u32x4 areg[8], breg[8];
  auto fetch = [&](int k0) {
    const bool kin = k0 + lcol < K;
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      const int r = lrow + 32 * n;
      const int am = min(m0 + r, M - 1), bn = min(n0 + r, N - 1);
      const u32x4 z = {0, 0, 0, 0};
      areg[n] = kin ? *reinterpret_cast<const u32x4*>(A + (int64_t)am * lda + k0 + lcol) : z;
      breg[n] = kin ? *reinterpret_cast<const u32x4*>(B + (int64_t)bn * ldb + k0 + lcol) : z;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      const int r = lrow + 32 * n;
      *reinterpret_cast<u32x4*>(&As[r * kLdsStride + lcol]) = areg[n];
      *reinterpret_cast<u32x4*>(&Bs[r * kLdsStride + lcol]) = breg[n];
    }
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += kTK) {
    __syncthreads();
    stash();
    __syncthreads();
    if (k0 + kTK < K) fetch(k0 + kTK);
#pragma unroll
    for (int kk = 0; kk < kTK / 16; ++kk) {
      bf16x8 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = lds_frag(&As[(wm + i * 32 + col) * kLdsStride + kk * 16 + g * 8]);
        bf[i] = lds_frag(&Bs[(wn + i * 32 + col) * kLdsStride + kk * 16 + g * 8]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  }

  // accumulator (i, j): lane column = n, register r = row 8*(r/4) + 4*g + r%4
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + wn + j * 32 + col;
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (m < M) C[(int64_t)m * ldc + n] = (uint16_t)f32_to_bf16_bits(acc[i][j][r]);
      }
    }
}

}  // namespace spx

using namespace spx;

extern "C" int spx_gemm_bf16_nt(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                int64_t ldc, int64_t M, int64_t N, int64_t K, void* stream) {
  SPX_REQUIRE(M > 0 && N > 0 && K > 0, "M, N, K must be positive");
  SPX_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "dimension too large");
  SPX_REQUIRE(a && b && c, "null buffer");
  SPX_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0, "K, lda, ldb must be multiples of 8");
  SPX_REQUIRE(lda >= K && ldb >= K && ldc >= N, "leading dimension too small");
  SPX_REQUIRE(((uintptr_t)a | (uintptr_t)b) % 16 == 0, "a and b must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_bf16_nt_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kGemmSmem);
    if (e != hipSuccess) {
      last_error() = std::string("spx_gemm_bf16_nt: hipFuncSetAttribute: ") + hipGetErrorString(e);
      return SPX_ERR_HIP;
    }
    attr_set = true;
  }
  const int tiles_m = (int)((M + kTM - 1) / kTM), tiles_n = (int)((N + kTN - 1) / kTN);
  SPX_REQUIRE((int64_t)tiles_m * tiles_n < (1ll << 31), "too many tiles");
  hipLaunchKernelGGL(gemm_bf16_nt_kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(kGemmThreads),
                     kGemmSmem, st, reinterpret_cast<const uint16_t*>(a), lda,
                     reinterpret_cast<const uint16_t*>(b), ldb, reinterpret_cast<uint16_t*>(c), ldc,
                     (int)M, (int)N, (int)K, tiles_m, tiles_n);
  return check_launch(__func__);
}
