// C[M, N] = A[M, K] * B[N, K]^T  (the nn.Linear product), bf16 in, fp32
// accumulate, bf16 out, for gfx950.
//
// One workgroup of 8 waves (4 along M x 2 along N) owns a 256 x 256 tile of C
// and walks K in steps of 64; each wave owns a 64 x 128 patch as 2 x 4
// accumulators of v_mfma_f32_32x32x16_bf16, two waves per SIMD so one wave's
// LDS reads overlap the other's MFMAs.  A and B tiles are staged global ->
// registers -> LDS (buffer loads: rows past the edge read as zero, no per-lane
// predicates) through two LDS stages (the next tile is written while the
// current one is read: one barrier per K step) with the next tile's global
// loads in flight during the current tile's MFMAs.  LDS rows are padded by 16
// bytes so the 16-byte operand reads of consecutive lanes hit distinct bank
// groups (measured: zero bank conflicts).  Workgroup ids are remapped so that
// each XCD (ids are dealt round-robin over the 8 XCDs) works on a compact
// band of tiles and shares its A / B panels in that XCD's L2.

#include <type_traits>

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

#ifndef SPX_GEMM_WM
#define SPX_GEMM_WM 4
#endif
#ifndef SPX_GEMM_WN
#define SPX_GEMM_WN 2
#endif
#ifndef SPX_GEMM_PGR
#define SPX_GEMM_PGR 1
#endif
constexpr int kWM = SPX_GEMM_WM, kWN = SPX_GEMM_WN;  // waves along M / N of the tile
constexpr int kPGR = SPX_GEMM_PGR;  // K tiles whose global loads are in flight ahead of the MFMAs
constexpr int kGemmThreads = 64 * kWM * kWN;
constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kMI = kTM / kWM / 32, kNI = kTN / kWN / 32;  // 32x32 accumulators per wave
constexpr int kLdsStride = kTK + 8;  // elements
constexpr int kStageElems = (kTM + kTN) * kLdsStride;
constexpr int kGemmSmem = 2 * kStageElems * 2;  // two stages

__device__ __forceinline__ bf16x8 lds_frag(const uint16_t* p) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = *reinterpret_cast<const u32x4*>(p);
  return c.b;
}

__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_nt_kernel(
    const uint16_t* __restrict__ A, int64_t lda, const uint16_t* __restrict__ B, int64_t ldb,
    uint16_t* __restrict__ C, int64_t ldc, int M, int N, int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

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
  const int wm = (wave / kWN) * (kTM / kWM), wn = (wave % kWN) * (kTN / kWN);

  // global -> register staging: 16-byte chunks, 8 per row of the 64-wide K tile
  constexpr int kRowsPerPass = kGemmThreads / 8;
  constexpr int kPasses = kTM / kRowsPerPass;
  const int lrow = tid >> 3, lcol = (tid & 7) * 8;
  u32x4 areg[kPGR][kPasses], breg[kPGR][kPasses];
  f32x16 acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // buffer loads: one resource per operand, a fixed 32-bit byte offset per staged row and
  // the K position in the scalar offset.  Rows past the matrix edge fall outside the
  // resource and read as zero, so no clamping or per-lane predicate is needed.
  const __amdgpu_buffer_rsrc_t ares = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(A), 0, (int)((((int64_t)M - 1) * lda + K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(B), 0, (int)((((int64_t)N - 1) * ldb + K) * 2), 0x00020000);
  int aoff[kPasses], boff[kPasses];
#pragma unroll
  for (int n = 0; n < kPasses; ++n) {
    const int r = lrow + kRowsPerPass * n;
    // a row index past the edge is moved far outside the resource (the plain product
    // row * ld could wrap around 2^32 for huge strides)
    aoff[n] = (m0 + r < M) ? (int)((((int64_t)(m0 + r)) * lda + lcol) * 2) : 0x7ffffff0;
    boff[n] = (n0 + r < N) ? (int)((((int64_t)(n0 + r)) * ldb + lcol) * 2) : 0x7ffffff0;
  }
  const bool ktail = (K % kTK) != 0;
#define SPX_FETCH(k0v, S)                                                              \
  do {                                                                                 \
    const int k0_ = (k0v);                                                             \
    _Pragma("unroll") for (int n = 0; n < kPasses; ++n) {                              \
      areg[S][n] = __builtin_amdgcn_raw_buffer_load_b128(ares, aoff[n], k0_ * 2, 0);   \
      breg[S][n] = __builtin_amdgcn_raw_buffer_load_b128(bres, boff[n], k0_ * 2, 0);   \
    }                                                                                  \
    if (ktail && k0_ + lcol >= K) {                                                    \
      const u32x4 z = {0, 0, 0, 0};                                                    \
      _Pragma("unroll") for (int n = 0; n < kPasses; ++n) { areg[S][n] = z; breg[S][n] = z; } \
    }                                                                                  \
  } while (0)
#define SPX_STASH(stagev, S)                                                           \
  do {                                                                                 \
    uint16_t* As_ = smem + (stagev) * kStageElems;                                     \
    uint16_t* Bs_ = As_ + kTM * kLdsStride;                                            \
    _Pragma("unroll") for (int n = 0; n < kPasses; ++n) {                              \
      const int r = lrow + kRowsPerPass * n;                                           \
      *reinterpret_cast<u32x4*>(&As_[r * kLdsStride + lcol]) = areg[S][n];             \
      *reinterpret_cast<u32x4*>(&Bs_[r * kLdsStride + lcol]) = breg[S][n];             \
    }                                                                                  \
  } while (0)
  auto compute = [&](int stage) {
    const uint16_t* As = smem + stage * kStageElems;
    const uint16_t* Bs = As + kTM * kLdsStride;
#ifndef SPX_GEMM_KKUNROLL
#define SPX_GEMM_KKUNROLL 4
#endif
#pragma unroll SPX_GEMM_KKUNROLL
    for (int kk = 0; kk < kTK / 16; ++kk) {
      bf16x8 af[kMI], bf[kNI];
#pragma unroll
      for (int i = 0; i < kMI; ++i) af[i] = lds_frag(&As[(wm + i * 32 + col) * kLdsStride + kk * 16 + g * 8]);
#pragma unroll
      for (int j = 0; j < kNI; ++j) bf[j] = lds_frag(&Bs[(wn + j * 32 + col) * kLdsStride + kk * 16 + g * 8]);
#pragma unroll
      for (int i = 0; i < kMI; ++i)
#pragma unroll
        for (int j = 0; j < kNI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  };
  constexpr int S1 = kPGR - 1;
  // two LDS stages: the next tile is written while the current one is read, one
  // barrier per K step.  kPGR = 2 keeps the global loads of TWO tiles in flight (in two
  // register sets) so that a tile's load latency is covered by two K steps of MFMAs.
  if (kPGR == 1) {
    SPX_FETCH(0, 0);
    SPX_STASH(0, 0);
    __syncthreads();
    int stage = 0;
    for (int k0 = 0; k0 < K; k0 += kTK) {
      const bool more = k0 + kTK < K;
      if (more) SPX_FETCH(k0 + kTK, 0);
      compute(stage);
      if (more) SPX_STASH(stage ^ 1, 0);
      __syncthreads();
      stage ^= 1;
    }
  } else {
    SPX_FETCH(0, 0);
    if (kTK < K) SPX_FETCH(kTK, S1);
    SPX_STASH(0, 0);
    __syncthreads();
    int stage = 0;
    for (int k0 = 0; k0 < K; k0 += kTK) {
      // tile k0 sits in LDS stage `stage`; the register set of the other parity holds
      // tile k0 + 1, this parity's set is free for tile k0 + 2
      const bool more1 = k0 + kTK < K, more2 = k0 + 2 * kTK < K;
      if (more2) {
        if (stage == 0) SPX_FETCH(k0 + 2 * kTK, 0);
        else SPX_FETCH(k0 + 2 * kTK, S1);
      }
      compute(stage);
      if (more1) {
        if (stage == 0) SPX_STASH(1, S1);
        else SPX_STASH(0, 0);
      }
      __syncthreads();
      stage ^= 1;
    }
  }
#undef SPX_FETCH
#undef SPX_STASH

  // accumulator (i, j): lane column = n, register r = row 8*(r/4) + 4*g + r%4
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
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
  SPX_REQUIRE(((M - 1) * lda + K) * 2 < 0x7ffffff0ll && ((N - 1) * ldb + K) * 2 < 0x7ffffff0ll,
              "each operand must span less than 2 GiB (32-bit buffer offsets)");
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
