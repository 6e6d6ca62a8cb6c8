// Weight-gradient GEMM for gfx950: C[M, N] (+)= A[T, M]^T * B[T, N], bf16 operands, fp32
// accumulation, bf16 result (optionally added to what C holds: the gradient of a weight that
// is applied once per TTT step accumulates in place).  Both operands are stored with the
// contraction index T as the SLOW dimension (A = the output gradient dY [T, M], B = the layer
// input X [T, N]), so an MFMA fragment -- 8 consecutive t for one m -- is a column of 8
// rows in memory.  The tile is turned on its way into LDS:
//   * every thread loads an 8 (t) x 8 (m) block with eight 16-byte row loads (a wave reads whole
//     128-byte lines), transposes it in registers with sixteen-bit byte permutes (v_perm_b32, 32 per
//     block) and writes eight 16-byte LDS rows [m][t0..t0+7];
//   * LDS rows are 64 t-values + 16 bytes of padding (pitch 144): with it both the transposed
//     writes (lanes = 8 t-chunks x 8 m-chunks) and the fragment reads (lanes = 32 rows) touch
//     every bank the same number of times;
// from there on it is the NT kernel: 256 x 256 tile, 4 waves x 128 x 128, slabs of 64 along
// T in two LDS buffers, v_mfma_f32_32x32x16_bf16 with one LDS read issued per MFMA,
// transposed accumulators and v_permlane32_swap for 16-byte stores.  The register transposes
// ride between the MFMAs of the second half of a slab (the vector pipe is idle there).
// Two sets of staging registers keep two slabs of loads in flight.
//
// What bounds it: the LDS pipe.  A 16-byte LDS write from registers occupies the pipe twice as
// long as a 16-byte read (counters: 8 against 4 index cycles), so the 16 writes per lane and
// slab cost as much as the 32 fragment reads and the pipe is busy about 80 % of the kernel's
// time, against 55 % in the NT kernel, whose tiles reach LDS without passing through registers.
// Measured 0.95 - 1.05 PFLOP/s on the draft layers' weight-gradient shapes (T = 4096), the
// vendor library's TN kernels 1.08 - 1.18: the host side of this package keeps the library
// for the weight gradients and this kernel serves callers of the C interface.

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

namespace tn {

constexpr int kNW = 4, kThreads = 256;
constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kWM = 2, kWN = 2;
constexpr int kMI = kTM / kWM / 32, kNI = kTN / kWN / 32;  // 4 x 4 accumulators of 32 x 32 per wave
constexpr int kPitch = kTK * 2 + 16;                        // 144 bytes per LDS row
constexpr int kOpBytes = kTM * kPitch;                      // one operand of one slab: 36864
constexpr int kBufBytes = 2 * kOpBytes;                     // A + B
constexpr int kSmem = 2 * kBufBytes;                        // 147456
constexpr int kOob = 0x7ffffff0;
#ifndef SPX_GEMM_TN_GROUP_M
#define SPX_GEMM_TN_GROUP_M 8
#endif

__device__ __forceinline__ bf16x8 as_frag(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

// output row i (0..7) of the transposed 8 x 8 block: element e of the result = in[e] element i
__device__ __forceinline__ u32x4 transposed_row(const u32x4 (&in)[8], int i) {
  const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
  const int w = i >> 1;
  u32x4 o;
  o.x = __builtin_amdgcn_perm(in[1][w], in[0][w], sel);
  o.y = __builtin_amdgcn_perm(in[3][w], in[2][w], sel);
  o.z = __builtin_amdgcn_perm(in[5][w], in[4][w], sel);
  o.w = __builtin_amdgcn_perm(in[7][w], in[6][w], sel);
  return o;
}

template <bool ACC>
__global__ __launch_bounds__(kThreads, 1) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_bf16_tn_kernel(
    const uint16_t* __restrict__ A, int64_t lda, const uint16_t* __restrict__ B, int64_t ldb,
    uint16_t* __restrict__ C, int64_t ldc, int M, int N, int T, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  // workgroup id -> tile: XCD-contiguous bands, then groups of GROUP_M tile rows
  const int n_wg = tiles_m * tiles_n;
  int pid = blockIdx.x;
  if (n_wg % 8 == 0) pid = (pid % 8) * (n_wg / 8) + pid / 8;
  constexpr int GROUP_M = SPX_GEMM_TN_GROUP_M;
  const int in_group = GROUP_M * tiles_n;
  const int first_m = (pid / in_group) * GROUP_M;
  const int group_sz = min(tiles_m - first_m, GROUP_M);
  const int tile_m = first_m + (pid % in_group) % group_sz;
  const int tile_n = (pid % in_group) / group_sz;
  const int m0 = tile_m * kTM, n0 = tile_n * kTN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, col = lane & 31;
  const int wm = (wave / kWN) * (kTM / kWM), wn = (wave % kWN) * (kTN / kWN);

  f32x16 acc[kNI][kMI];
#pragma unroll
  for (int j = 0; j < kNI; ++j)
#pragma unroll
    for (int i = 0; i < kMI; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][i][r] = 0.f;

  // ---- global side: this thread's 8 x 8 block of each operand: t rows tb*8 .. tb*8+7 of the slab,
  // columns mc*8 .. mc*8+7 of the tile.  Rows past T (every row of a slab past the end) lie outside
  // the buffer resource and read as zero: the whole offset is in the VGPR, which the range check sees.
  const int tb = lane & 7, mc = (lane >> 3) + 8 * wave;
  const __amdgpu_buffer_rsrc_t ares = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(A), 0, (int)((((int64_t)T - 1) * lda + M) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(B), 0, (int)((((int64_t)T - 1) * ldb + N) * 2), 0x00020000);
  // A column chunk past the matrix edge may read the next row's valid memory instead of zeros: it
  // only feeds rows / columns of C that are never stored.
  const int a_row = (int)(lda * 2), b_row = (int)(ldb * 2);
  const int a_v0 = tb * 8 * a_row + (m0 + mc * 8) * 2, b_v0 = tb * 8 * b_row + (n0 + mc * 8) * 2;

  // two register sets: set p holds the slabs of parity p between their loads and their staging
  u32x4 ra[2][8], rb[2][8];
  auto fetch_a = [&](int s, int p) __attribute__((always_inline)) {
    const int base = a_v0 + s * (kTK * a_row);
#pragma unroll
    for (int j = 0; j < 8; ++j) ra[p][j] = __builtin_amdgcn_raw_buffer_load_b128(ares, base + j * a_row, 0, 0);
  };
  auto fetch_b = [&](int s, int p) __attribute__((always_inline)) {
    const int base = b_v0 + s * (kTK * b_row);
#pragma unroll
    for (int j = 0; j < 8; ++j) rb[p][j] = __builtin_amdgcn_raw_buffer_load_b128(bres, base + j * b_row, 0, 0);
  };
  // LDS side of the same block: rows mc*8 + i, 16-byte chunk tb
  const int wr_off = (mc * 8) * kPitch + tb * 16;
  // unit u (0..15): transposed row u % 8 of operand u / 8 (register set p), written to slab buffer `buf`
  auto stage_unit = [&](int u, int buf, int p) __attribute__((always_inline)) {
    const int i = u & 7;
    const u32x4 o = (u < 8) ? transposed_row(ra[p], i) : transposed_row(rb[p], i);
    *reinterpret_cast<u32x4*>(smem + buf * kBufBytes + (u < 8 ? 0 : kOpBytes) + wr_off + i * kPitch) = o;
  };

  // ---- read side: row = lane % 32 of a 32-row block, t chunk 2 kk + g
  const int rd0 = col * kPitch + g * 16;
  const int a_rd = (wm)*kPitch + rd0, b_rd = kOpBytes + wn * kPitch + rd0;
  bf16x8 fa[2][kMI], fb[2][kNI];
  auto read_one = [&](int set, int buf, int kk, int f) __attribute__((always_inline)) {
    if (f < kMI)
      fa[set][f] = as_frag(*reinterpret_cast<const u32x4*>(smem + buf * kBufBytes + a_rd + kk * 32 + f * 32 * kPitch));
    else
      fb[set][f - kMI] = as_frag(
          *reinterpret_cast<const u32x4*>(smem + buf * kBufBytes + b_rd + kk * 32 + (f - kMI) * 32 * kPitch));
  };
  // One step of 16 along T: the 16 MFMAs on register set `set`; between them, one at a time, the
  // LDS reads that fill the other set with step rk of buffer rbuf.  `plan` says what else rides
  // along: 1 = the staging units of A of the next slab (buffer wbuf), then the loads of A of
  // slab nxt into the registers just freed; 2 = the same for B
  auto step = [&](int set, int rbuf, int rk, int plan, int wbuf, int nxt) __attribute__((always_inline)) {
    constexpr int kF = kMI + kNI;
    int reads = 0;
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int i = 0; i < kMI; ++i) {
        acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[set][j], fa[set][i], acc[j][i], 0, 0, 0);
        const int idx = j * kMI + i;
        __builtin_amdgcn_sched_barrier(0);
        if (reads < kF) {
          read_one(set ^ 1, rbuf, rk, reads++);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (plan == 1 || plan == 2) {
          if (idx & 1) stage_unit((plan == 2 ? 8 : 0) + (idx >> 1), wbuf, wbuf);
          if (idx == 15) {
            if (plan == 1) fetch_a(nxt, wbuf); else fetch_b(nxt, wbuf);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
  };

  const int nslab = (T + kTK - 1) / kTK;
  // prologue: slab 0 through the registers into buffer 0, slabs 1 and 2 on their way
  fetch_a(0, 0);
  fetch_b(0, 0);
#pragma unroll
  for (int u = 0; u < 16; ++u) stage_unit(u, 0, 0);
  __syncthreads();
  fetch_a(1, 1);  // past the end: zeros
  fetch_b(1, 1);
  fetch_a(2, 0);
  fetch_b(2, 0);
#pragma unroll
  for (int f = 0; f < kMI + kNI; ++f) read_one(0, 0, 0, f);

  // one slab: on entry register set 0 holds (or is receiving) step 0 of slab s (buffer cur) and the
  // staging registers of parity cur ^ 1 hold (or are receiving) slab s + 1, those of parity cur slab
  // s + 2.  A register set is reloaded, with the slab two further on, as soon as it has been written to
  // LDS: a load has more than a slab's worth of MFMAs to arrive.
  auto slab = [&](int s, int cur) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    step(0, cur, 1, 0, 0, 0);
    step(1, cur, 2, 1, cur ^ 1, s + 3);
    step(0, cur, 3, 2, cur ^ 1, s + 3);
    // every read of this slab's buffer has returned once set 1 is complete; the barrier says: slab
    // s + 1 is in LDS for everybody, this buffer is free
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    // step 3 of slab s, under it the reads of step 0 of slab s + 1
    step(1, cur ^ 1, 0, 0, 0, 0);
  };
  int s = 0;
  for (; s + 1 < nslab; s += 2) {
    slab(s, 0);
    slab(s + 1, 1);
  }
  if (s < nslab) slab(s, 0);

  // epilogue: a lane holds row m of C and, per accumulator, columns 8 q + 4 g + {0..3}
  // (q = 0..3).  Swapping the q-odd words of the lower half-wave with the q-even words of
  // the upper half-wave leaves every lane with 8 consecutive columns: 16-byte stores.
  const bool fast = (ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0) && (n0 + kTN <= N);
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    const int m = m0 + wm + i * 32 + col;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
      f32x16 a = acc[j][i];
      if (ACC && fast) {
        // swap the fp32 words, add what C holds (one 16-byte load per lane, the store's own layout)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float v[8];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(a[8 * h + e]),
                                                            __float_as_uint(a[8 * h + 4 + e]), false, false);
            v[e] = __uint_as_float(sw[0]);
            v[4 + e] = __uint_as_float(sw[1]);
          }
          const int n = n0 + wn + j * 32 + 16 * h + 8 * g;
          if (m < M) {
            u32x4* cp = reinterpret_cast<u32x4*>(&C[(int64_t)m * ldc + n]);
            const u32x4 old = *cp;
            u32x4 o;
            o.x = pack_bf16x2(v[0] + bf16_lo(old.x), v[1] + bf16_hi(old.x));
            o.y = pack_bf16x2(v[2] + bf16_lo(old.y), v[3] + bf16_hi(old.y));
            o.z = pack_bf16x2(v[4] + bf16_lo(old.z), v[5] + bf16_hi(old.z));
            o.w = pack_bf16x2(v[6] + bf16_lo(old.w), v[7] + bf16_hi(old.w));
            *cp = o;
          }
        }
        continue;
      }
      if (ACC && m < M) {
        // ragged edge: what C holds, read in the accumulator's own layout (4 consecutive columns per q)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn + j * 32 + 8 * q + 4 * g;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) a[4 * q + e] += bf16_bits_to_f32(C[(int64_t)m * ldc + n + e]);
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {  // q pair (2h, 2h+1)
        const uint32_t e0 = pack_bf16x2(a[8 * h + 0], a[8 * h + 1]), e1 = pack_bf16x2(a[8 * h + 2], a[8 * h + 3]);
        const uint32_t o0 = pack_bf16x2(a[8 * h + 4], a[8 * h + 5]), o1 = pack_bf16x2(a[8 * h + 6], a[8 * h + 7]);
        const auto s0 = __builtin_amdgcn_permlane32_swap(e0, o0, false, false);
        const auto s1 = __builtin_amdgcn_permlane32_swap(e1, o1, false, false);
        u32x4 v;
        v.x = s0[0]; v.y = s1[0]; v.z = s0[1]; v.w = s1[1];
        const int n = n0 + wn + j * 32 + 16 * h + 8 * g;
        if (fast) {
          if (m < M) *reinterpret_cast<u32x4*>(&C[(int64_t)m * ldc + n]) = v;
        } else if (m < M) {
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < N) C[(int64_t)m * ldc + n + e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
  }
}

}  // namespace tn
}  // namespace spx

using namespace spx;

extern "C" int spx_gemm_bf16_tn(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                int64_t ldc, int64_t M, int64_t N, int64_t T, int accumulate,
                                void* stream) {
  SPX_REQUIRE(M > 0 && N > 0 && T > 0, "M, N, T must be positive");
  SPX_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && T < (1ll << 31), "dimension too large");
  SPX_REQUIRE(a && b && c, "null buffer");
  SPX_REQUIRE(M % 8 == 0 && N % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0, "M, N, lda, ldb must be multiples of 8");
  SPX_REQUIRE(lda >= M && ldb >= N && ldc >= N, "leading dimension too small");
  SPX_REQUIRE(((uintptr_t)a | (uintptr_t)b) % 16 == 0, "a and b must be 16-byte aligned");
  SPX_REQUIRE(((T + 4 * tn::kTK) * lda) * 2 < 0x7ffffff0ll && ((T + 4 * tn::kTK) * ldb) * 2 < 0x7ffffff0ll,
              "each operand must span less than 2 GiB (32-bit buffer offsets)");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  static std::atomic<uint64_t> lds_set[2];  // per kernel instantiation, one bit per device
  const void* fn = accumulate ? reinterpret_cast<const void*>(&tn::gemm_bf16_tn_kernel<true>)
                              : reinterpret_cast<const void*>(&tn::gemm_bf16_tn_kernel<false>);
  if (int rc = ensure_dynamic_lds(fn, tn::kSmem, lds_set[accumulate ? 1 : 0], __func__)) return rc;
  const int tiles_m = (int)((M + tn::kTM - 1) / tn::kTM), tiles_n = (int)((N + tn::kTN - 1) / tn::kTN);
  const dim3 grid((unsigned)(tiles_m * tiles_n)), block(tn::kThreads);
  auto ap = reinterpret_cast<const uint16_t*>(a);
  auto bp = reinterpret_cast<const uint16_t*>(b);
  auto cp = reinterpret_cast<uint16_t*>(c);
  if (accumulate)
    hipLaunchKernelGGL(tn::gemm_bf16_tn_kernel<true>, grid, block, tn::kSmem, st, ap, lda, bp, ldb, cp, ldc,
                       (int)M, (int)N, (int)T, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL(tn::gemm_bf16_tn_kernel<false>, grid, block, tn::kSmem, st, ap, lda, bp, ldb, cp, ldc,
                       (int)M, (int)N, (int)T, tiles_m, tiles_n);
  return check_launch(__func__);
}
