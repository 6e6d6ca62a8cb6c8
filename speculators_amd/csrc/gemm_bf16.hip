// C[M, N] = A[M, K] * B[N, K]^T  (the nn.Linear product), bf16 in, fp32
// accumulate, bf16 out, for gfx950.
//
// One workgroup of 4 waves owns a 256 x 256 tile of C (each wave a 128 x 128
// patch = 8 x 8 accumulators of v_mfma_f32_16x16x32_bf16, one wave per SIMD)
// and walks K in slabs of 64.  (The 16 x 16 x 32 form of the instruction reads and
// writes its accumulator half as often per multiply-add as the 32 x 32 x 16 form:
// a register-only loop of it holds 2.09 PFLOP/s at the power limit of the chip, the
// 32 x 32 x 16 form 1.83.)
//
// Global -> LDS directly (buffer_load ... lds): no staging registers and no
// LDS store instructions.  A wave-load fills 8 rows x 128 B of LDS linearly
// (lane i -> byte 16 i), so every fetch is a whole 128-byte line; the
// bank-conflict-free layout comes from WHICH 16-byte K chunk a lane fetches:
// chunk c of row r sits in slot c ^ f(r), f(r) = (r & 7) ^ ((r >> 3) & 1).
// Two slab buffers: the loads of slab s+1 are in flight while slab s is
// multiplied.  They are issued one at a time between the MFMAs (a burst would
// stall the wave at issue until the memory pipeline has room), and so are the
// LDS reads: operand fragments are double buffered in registers, the reads of
// K step kk+1 (32 columns) run under the MFMAs of step kk, and the last step of a
// slab is multiplied after the barrier that opens the next slab, so no LDS latency
// is exposed and there is one barrier per slab.
//
// The accumulators are kept transposed (lane = row of C, registers = 4
// consecutive columns); v_permlane16_swap pairs them into 8 consecutive
// columns for 16-byte stores.  Workgroup ids are remapped so that each XCD
// (ids are dealt round-robin over the 8 XCDs) works on a compact band of
// tiles and shares its A / B panels in that XCD's L2.

#include <type_traits>

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

#define SPX_GEMM_WM 2
#define SPX_GEMM_WN 2
#define SPX_GEMM_MINW 1
#define SPX_GEMM_READ_EVERY 2  // MFMAs per LDS fragment read
constexpr int kWM = SPX_GEMM_WM, kWN = SPX_GEMM_WN;  // waves along M / N of the tile
constexpr int kNW = kWM * kWN;
constexpr int kGemmThreads = 64 * kNW;
constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kMI = kTM / kWM / 16, kNI = kTN / kWN / 16;  // 16x16 accumulators per wave
constexpr int kKSteps = kTK / 32;                          // MFMA K steps per slab
constexpr int kRowBytes = kTK * 2;                          // 128
constexpr int kABytes = kTM * kRowBytes;                    // one slab of A: 32 KB
constexpr int kBBytes = kTN * kRowBytes;
constexpr int kBBase = 2 * kABytes;
constexpr int kGemmSmem = 2 * (kABytes + kBBytes);  // 128 KB
constexpr int kLA = kTM / 8 / kNW;                  // wave-loads of A per wave per slab
constexpr int kLB = kTN / 8 / kNW;
constexpr int kL = kLA + kLB;
constexpr int kOob = 0x7ffffff0;
static_assert(kABytes == 32768 && kBBytes == 32768, "the buffer toggle flips bit 15");
static_assert(kLA % 4 == 0 && kLB % 4 == 0, "loads are grouped in fours (immediate offsets)");

__device__ __forceinline__ bf16x8 as_frag(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}


// kImm: consecutive loads of a group of four share one M0 value and differ in the
// instruction's immediate offset (which moves the LDS and the global address alike, so
// the per-lane global offset is stored minus that immediate).  Needs every row offset to
// be at least the immediate: lda, ldb >= 64.  Without it every load sets M0 itself.
// Into how many parts the contraction of a product of n_tiles tiles is cut (each part a workgroup of
// its own with an fp32 partial result): the number s <= max_parts for which the rounds the chip needs,
// ceil(n_tiles s / cus) / s, are fewest -- if that saves a tenth or more and leaves every part at least
// 16 slabs.  192 tiles on 256 compute units: 4 parts (3 rounds of a quarter instead of 1 round of a
// whole); 128: 2; 256: 1.  Evaluated on the device by the product and by the kernel that adds the parts.
__device__ __forceinline__ int choose_k_parts(int n_tiles, int max_parts, int cus, int nslab) {
  if (n_tiles <= 0) return 1;
  const int64_t r1 = (n_tiles + cus - 1) / cus;
  int best = 1;
  int64_t best_r = r1;
  for (int s2 = 2; s2 <= max_parts; ++s2) {
    if (nslab / s2 < 16) break;
    const int64_t r = ((int64_t)n_tiles * s2 + cus - 1) / cus;
    if (r * 10 <= 9 * r1 * s2 && r * best < best_r * s2) { best = s2; best_r = r; }
  }
  return best;
}

// kStats != 0: the epilogue also reduces every row of the tile to the soft-max statistics of its 256
// bf16-rounded results -- the row maximum, with bit 0 of kStats sum_n 2^((c[m, n] - max) log2 e) and
// with bit 1 the first column that holds the maximum -- and leaves them in stat_ws, laid out [3][tiles_n][M] (maxima as
// float, sums as float, columns as int32); gemm_row_stats_reduce_kernel folds the tiles_n entries
// of a row into log-sum-exp and arg-max.  C may then be null: the product itself is not stored
// (a cross-entropy against arg-max targets needs nothing else of the target logits).
// The tiles of the last, partly filled round of a product (n_tiles % cus of them, when they are at most
// half a round): each is cut along the contraction into as many parts as fill the idle compute units
// (at most max_parts, every part at least 16 slabs), so that the round takes a part's time instead of a
// tile's.  384 tiles on 256 compute units: 256 whole tiles, then 128 tiles x 2 halves -- 1.5 rounds of
// work in 1.5 rounds of time instead of 2.  first = index of the first tile that is cut (n_tiles: none).
__host__ __device__ __forceinline__ void tail_plan(int n_tiles, int cus, int nslab, int max_parts, int& first,
                                                   int& parts) {
  first = n_tiles;
  parts = 1;
  if (n_tiles <= 0 || cus <= 0) return;
  const int rem = n_tiles % cus;
  if (rem == 0 || rem * 2 > cus) return;
  int tp = cus / rem;
  if (tp > max_parts) tp = max_parts;
  while (tp > 1 && nslab / tp < 16) --tp;
  if (tp > 1) { first = n_tiles - rem; parts = tp; }
}

// tile index -> (tile row, tile column).  256 consecutive indices (what the chip runs at a time) are a block of
// 16 x 16 tiles, so that a 256-row band of either operand is used by 16 of the tiles in flight, and the blocks walk
// along the longer side of the tile grid; 32 consecutive indices (what one XCD runs: see the kernel) are 8 tiles
// along the longer side x 4 along the shorter, 12 operand bands through that XCD's L2.  In detail: panels of 16
// along the shorter side; inside a panel groups of 8 along the longer side; inside a group the longer side first.
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  constexpr int kPanel = 16, kGroup = 8;
  const bool m_long = tiles_m >= tiles_n;
  const int tl = m_long ? tiles_m : tiles_n, ts = m_long ? tiles_n : tiles_m;
  const int panel = pid / (tl * kPanel);
  const int ps = min(ts - panel * kPanel, kPanel);
  const int p = pid - panel * tl * kPanel;
  const int g = p / (kGroup * ps);
  const int gsz = min(tl - g * kGroup, kGroup);
  const int r = p - g * kGroup * ps;
  const int l = g * kGroup + r % gsz, sh = panel * kPanel + r / gsz;
  tile_m = m_long ? l : sh;
  tile_n = m_long ? sh : l;
}

template <bool kImm, int kStats = 0>
__global__ __launch_bounds__(kGemmThreads, SPX_GEMM_MINW)
__attribute__((amdgpu_waves_per_eu(SPX_GEMM_MINW, SPX_GEMM_MINW))) void gemm_bf16_nt_kernel(
    const uint16_t* __restrict__ A, int64_t lda, const uint16_t* __restrict__ B, int64_t ldb,
    uint16_t* __restrict__ C, int64_t ldc, int M, int N, int K, int tiles_m, int tiles_n,
    const int32_t* __restrict__ m_live, const int32_t* __restrict__ tile_tab,
    const int32_t* __restrict__ group_off, int64_t b_group_stride, float* __restrict__ part_ws,
    int max_parts, int cus, float* __restrict__ stat_ws = nullptr, int tail_mode = 0) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int M_host = M;
  // the row count may live on the device (rows packed to the front by the producer of A): the tile
  // grid shrinks to the rows that count and the workgroups beyond it leave at once
  if (m_live) {
    M = min(M, max(*m_live, 0));
    tiles_m = (M + kTM - 1) / kTM;
  }
  // grouped product: the rows of A are sorted by group, group e = rows [group_off[e], group_off[e+1])
  // is multiplied by its own B (b_group_stride elements apart).  The tile rows come from a table on
  // the device (tile_tab[0] = their number, then (group, first row) per tile row): no tile spans
  // two groups, and the host never learns the group sizes
  if (tile_tab) tiles_m = min(tile_tab[0], tiles_m);

  // workgroup id -> tile index (tile_coords turns that into a tile).  Workgroups go to the eight XCDs round
  // robin, XCD x gets the ids x, x + 8, ...: they are renumbered so that in every round of 256 workgroups each
  // XCD has 32 consecutive tile indices, and in what is left after the last whole round one contiguous piece
  // (the first n % 8 XCDs one more).
  // contraction in parts (part_ws): the workgroups of part p multiply columns [p, p + 1) * part length of
  // K and leave an fp32 partial in part_ws[p]; gemm_splitk_reduce_kernel adds the parts in order
  const int n_tiles = tiles_m * tiles_n;
  // tail_mode: only the tiles of the last, partly filled round are cut (tail_plan); their partials go to
  // part_ws as whole tiles, [part][tail tile][256][256] fp32, and gemm_tail_reduce_kernel adds them
  int parts = 1, tail_first = n_tiles, tail_parts = 1;
  if (tail_mode) tail_plan(n_tiles, cus, (K + kTK - 1) / kTK, max_parts, tail_first, tail_parts);
  else if (part_ws) parts = choose_k_parts(n_tiles, max_parts, cus, (K + kTK - 1) / kTK);
  const int n_tail = n_tiles - tail_first;
  const int n_wg = tail_mode ? n_tiles + n_tail * (tail_parts - 1) : n_tiles * parts;
  if ((int)blockIdx.x >= n_wg) return;
  int pid;
  {
    constexpr int kRound = 256, kPer = kRound / 8;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    // tail_mode with a cut last round: the whole tiles are whole rounds, the parts of the cut tiles are "what
    // is left" -- dispatched after them (workgroups start in the order of their ids) and everywhere at once
    const int whole = (tail_mode && tail_parts > 1) ? tail_first : n_wg;
    const int full = whole / kRound * kRound;
    if ((int)blockIdx.x < full) {
      pid = (local / kPer) * kRound + xcd * kPer + local % kPer;
    } else {
      const int nr = n_wg - full;
      pid = full + xcd * (nr >> 3) + min(xcd, nr & 7) + (local - full / 8);
    }
  }
  int part;
  if (tail_mode) {
    part = 0;
    if (pid >= tail_first) {
      const int qq = pid - tail_first;
      part = qq / n_tail;
      pid = tail_first + qq % n_tail;
      parts = tail_parts;
    }
  } else {
    part = pid / n_tiles;
    pid -= part * n_tiles;
  }
  if (parts > 1) {
    const int slabs = ((K + kTK - 1) / kTK + parts - 1) / parts;
    const int k_begin = part * slabs * kTK;
    A += k_begin;
    B += k_begin;
    K = max(min(K - k_begin, slabs * kTK), 0);
  }
  int tile_m, tile_n;
  tile_coords(pid, tiles_m, tiles_n, tile_m, tile_n);
  int m0 = tile_m * kTM;
  const int n0 = tile_n * kTN;
  if (tile_tab) {
    const int grp = tile_tab[1 + 2 * tile_m];
    m0 = tile_tab[2 + 2 * tile_m];
    M = min(M, max(group_off[grp + 1], 0));  // rows from here on belong to the next group
    B += (int64_t)grp * b_group_stride;
  }

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r16 = lane & 15;
  const int wm = (wave / kWN) * (kTM / kWM), wn = (wave % kWN) * (kTN / kWN);

  // acc[j][i]: lane = row wm + 16 i + lane % 16 of C, registers = columns wn + 16 j + 4 (lane / 16) + {0..3}
  f32x4 acc[kNI][kMI];
#pragma unroll
  for (int j = 0; j < kNI; ++j)
#pragma unroll
    for (int i = 0; i < kMI; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[j][i][r] = 0.f;

  // One buffer resource per operand; the K position goes into the scalar offset.  Rows
  // past the matrix edge get an offset outside the resource and read as zero, so no
  // clamping or per-lane predicate is needed.
  // (the resources start at the tile's first row: offsets stay below 256 rows whatever the operand's size)
  const u32x4 ares = make_rsrc(A + (int64_t)m0 * lda, (uint32_t)((((int64_t)min(M - m0, kTM) - 1) * lda + K) * 2));
  const u32x4 bres = make_rsrc(B + (int64_t)n0 * ldb, (uint32_t)((((int64_t)min(N - n0, kTN) - 1) * ldb + K) * 2));

  // global side: wave-load j of this wave covers tile rows wave*8*kLA + 8 j + lane/8; the
  // lane's LDS slot is lane % 8, so it fetches chunk slot ^ f(row)
  const int lrow = lane >> 3;
  int gchunk[2];
  gchunk[0] = (lane & 7) ^ (lrow & 7);      // rows 0..7 of a 16-row group
  gchunk[1] = (lane & 7) ^ (lrow & 7) ^ 1;  // rows 8..15
  int aoff[kLA], boff[kLB];
#pragma unroll
  for (int j = 0; j < kLA; ++j) {
    const int r = wave * (8 * kLA) + j * 8 + lrow;
    const int imm = kImm ? (j & 3) * 8 * kRowBytes : 0;
    aoff[j] = (m0 + r < M) ? (int)(((int64_t)r * lda + gchunk[j & 1] * 8) * 2) - imm : kOob;
  }
#pragma unroll
  for (int j = 0; j < kLB; ++j) {
    const int r = wave * (8 * kLB) + j * 8 + lrow;
    const int imm = kImm ? (j & 3) * 8 * kRowBytes : 0;
    boff[j] = (n0 + r < N) ? (int)(((int64_t)r * ldb + gchunk[j & 1] * 8) * 2) - imm : kOob;
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
  const uint32_t lds_a = lds0 + wave * (8 * kLA) * kRowBytes;
  const uint32_t lds_b = lds0 + kBBase + wave * (8 * kLB) * kRowBytes;

  uint32_t bufoff = 0;  // slab buffer the next loads go to
  int ld_k0 = 0;        // first K column of the slab being loaded
  // load l (A loads first, then B) of the slab at ld_k0; full: the slab lies inside K
  auto issue_one = [&](int l, bool full) __attribute__((always_inline)) {
    const bool isa = l < kLA;
    const int j = isa ? l : l - kLA;
    int voff = isa ? aoff[j] : boff[j];
    if (!full) voff = (ld_k0 + gchunk[j & 1] * 8 < K) ? voff : kOob;
    const u32x4 res = isa ? ares : bres;
    const uint32_t base = (isa ? lds_a : lds_b) + bufoff;
    if (kImm) {
      const uint32_t grp = base + (j & ~3) * 8 * kRowBytes;
      switch (j & 3) {
        case 0: load_to_lds16<0>(res, grp, voff, ld_k0 * 2); break;
        case 1: load_to_lds16<8 * kRowBytes>(res, grp, voff, ld_k0 * 2); break;
        case 2: load_to_lds16<16 * kRowBytes>(res, grp, voff, ld_k0 * 2); break;
        default: load_to_lds16<24 * kRowBytes>(res, grp, voff, ld_k0 * 2); break;
      }
    } else {
      load_to_lds16<0>(res, base + j * 8 * kRowBytes, voff, ld_k0 * 2);
    }
  };
  auto next_slab = [&]() __attribute__((always_inline)) { bufoff ^= kABytes; ld_k0 += kTK; };

  // read side: row = lane % 16 of a 16-row block, K chunk 4 kk + lane / 16 in slot chunk ^ f(row)
  const int fr = (r16 & 7) ^ (r16 >> 3);
  const int off0 = r16 * kRowBytes + ((q ^ fr) * 16);
  uint32_t a_rd[kKSteps], b_rd[kKSteps];  // per K step of 32; bit 15 selects the slab buffer
#pragma unroll
  for (int kk = 0; kk < kKSteps; ++kk) {
    a_rd[kk] = wm * kRowBytes + (off0 ^ (kk * 64));
    b_rd[kk] = kBBase + wn * kRowBytes + (off0 ^ (kk * 64));
  }

  bf16x8 fa[2][kMI], fb[2][kNI];
  // operand fragment f (A fragments first, then B) of K step kk into register set `set`
  auto read_one = [&](int set, int kk, int f) __attribute__((always_inline)) {
    if (f < kMI)
      fa[set][f] = as_frag(*reinterpret_cast<const u32x4*>(smem + a_rd[kk] + f * 16 * kRowBytes));
    else
      fb[set][f - kMI] = as_frag(*reinterpret_cast<const u32x4*>(smem + b_rd[kk] + (f - kMI) * 16 * kRowBytes));
  };
  // One K step: the kNI x kMI MFMAs on register set `set`; between them, one at a time,
  // the LDS reads that fill the other set with K step rk and the global loads
  // [l0, l0 + nl).  A read after every second MFMA (a 16 x 16 x 32 MFMA occupies the pipe for 16
  // cycles: a read and its address arithmetic behind each one leave the pipe waiting), in the first
  // half of the step: their data is needed at the next step.
  auto step = [&](int set, int rk, int l0, int nl, bool full) __attribute__((always_inline)) {
    constexpr int kN = kNI * kMI, kF = kMI + kNI;
    int reads = 0, loads = 0;
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int i = 0; i < kMI; ++i) {
        mfma16(acc[j][i], fb[set][j], fa[set][i]);
        const int idx = j * kMI + i;
        __builtin_amdgcn_sched_barrier(0);
        if (reads < kF && idx % SPX_GEMM_READ_EVERY == SPX_GEMM_READ_EVERY - 1) {
          read_one(set ^ 1, rk, reads++);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (nl > 0 && (nl >= kN || idx % (kN / nl) == kN / nl - 1) && loads < nl) {
          issue_one(l0 + loads++, full);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
  };

  // the loads of a slab are issued in the step after the barrier that frees its buffer, one per
  // four MFMAs; the step after that gives them time to land
  static_assert(kKSteps == 2, "a slab is two K steps: one before, one after the barrier");
  constexpr int kLdT = kL;
  // one slab: on entry set 0 holds (or is receiving) K step 0 of slab s and the loads of slab s+1
  // are issued
  auto slab = [&](bool full) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    step(0, 1, 0, 0, full);
    next_slab();
    // every read of this slab's buffer has returned once set 1 is complete; then the
    // barrier says: slab s+1 has landed for everybody, this buffer is free
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) { a_rd[kk] ^= kABytes; b_rd[kk] ^= kBBytes; }
    // K step 1 of slab s, under it the reads of step 0 of slab s+1 and the loads of slab s+2
    step(1, 0, 0, kLdT, full);
  };

  const int nslab = (K + kTK - 1) / kTK;
#pragma unroll
  for (int l = 0; l < kL; ++l) issue_one(l, false);
  next_slab();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  // past the last slab every lane is out of range: zeros go into the free buffer
#pragma unroll
  for (int l = 0; l < kLdT; ++l) issue_one(l, false);
#pragma unroll
  for (int f = 0; f < kMI + kNI; ++f) read_one(0, 0, f);
  // slab s issues loads of slabs s+1 and s+2: no K-edge predicate while (s+3)*64 <= K
  const int nfull = max(K / kTK - 2, 0);
  int s = 0;
  for (; s < nfull; ++s) slab(true);
  for (; s < nslab; ++s) slab(false);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  mfma_results_ready();
  if (parts > 1 && tail_mode) {
    // this part's fp32 partial of a tile of the last round: a 256 x 256 tile of its own
    float* const P = part_ws + ((int64_t)(part * n_tail + (pid - tail_first)) << 16);
#pragma unroll
    for (int i = 0; i < kMI; ++i) {
      const int rr = wm + i * 16 + r16;
#pragma unroll
      for (int j = 0; j < kNI; ++j) *reinterpret_cast<f32x4*>(P + rr * kTN + wn + j * 16 + 4 * q) = acc[j][i];
    }
    return;
  }
  if (parts > 1) {
    // this part's fp32 partial, in the accumulators' own layout: 16 bytes per lane and accumulator
    float* const P = part_ws + (int64_t)part * M_host * N;
#pragma unroll
    for (int i = 0; i < kMI; ++i) {
      const int m = m0 + wm + i * 16 + r16;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < kNI; ++j) {
        const int n = n0 + wn + j * 16 + 4 * q;
        if (n < N) *reinterpret_cast<f32x4*>(P + (int64_t)m * N + n) = acc[j][i];  // (N is a multiple of 8 here)
      }
    }
    return;
  }
  // epilogue: a lane holds row m of C and, per accumulator, columns 4 q + {0..3} of a 16-column
  // block (q = lane / 16).  Swapping the words of the q-odd lanes for block j with those of the
  // q-even lanes for block j + 1 leaves every lane with 8 consecutive columns: 16-byte stores.
  const bool fast = (ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0) && (n0 + kTN <= N);
  // kStats: (maximum, sum, first column) of this wave's 128 columns per row, lanes q == 0 -> LDS.
  // The slab buffers are dead, but another wave's last (all-zero) global -> LDS loads may still be
  // landing in them: everybody has waited for their own above, the barrier makes that mutual
  float* const st_lds = reinterpret_cast<float*>(smem);  // [wave][3][128]
  if constexpr (kStats != 0) __syncthreads();
  const bool edge_n = n0 + kTN > N;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    const int m = m0 + wm + i * 16 + r16;
    uint32_t pk[kNI][2];
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
      pk[j][0] = pack_bf16x2(acc[j][i][0], acc[j][i][1]);
      pk[j][1] = pack_bf16x2(acc[j][i][2], acc[j][i][3]);
    }
    if constexpr (kStats != 0) {
      // the 32 values of this lane, as the consumer of C reads them (rounded to bf16).  Every
      // comparison below is a floating-point one: -0 and +0 are one value, as for torch.argmax
      float v[kNI][4];
#pragma unroll
      for (int j = 0; j < kNI; ++j) {
        v[j][0] = bf16_lo(pk[j][0]); v[j][1] = bf16_hi(pk[j][0]);
        v[j][2] = bf16_lo(pk[j][1]); v[j][3] = bf16_hi(pk[j][1]);
      }
      const int nb = n0 + wn + 4 * q;  // column of v[j][r] = nb + 16 j + r
      if (edge_n) {
#pragma unroll
        for (int j = 0; j < kNI; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) v[j][r] = (nb + 16 * j + r < N) ? v[j][r] : -INFINITY;
      }
      float mx = v[0][0];
#pragma unroll
      for (int j = 0; j < kNI; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, v[j][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m2 = (mx == -INFINITY) ? 0.f : mx * kLog2e;  // (a half tile past the last column)
      float z = 0.f;
      int first = 0x7fffffff;
      if constexpr ((kStats & 1) != 0) {
#pragma unroll
        for (int j = 0; j < kNI; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) z += fast_exp2(fmaf(v[j][r], kLog2e, -m2));
        z += __shfl_xor(z, 16, 64);
        z += __shfl_xor(z, 32, 64);
      }
      if constexpr ((kStats & 2) != 0) {
        int loc = 128;  // column inside the lane's 128-column stripe (a constant per element); 128 = none
#pragma unroll
        for (int j = kNI - 1; j >= 0; --j)
#pragma unroll
          for (int r = 3; r >= 0; --r) loc = (v[j][r] == mx) ? 16 * j + r : loc;  // descending: the lowest stays
        first = (loc < 128) ? nb + loc : 0x7fffffff;
        first = min(first, __shfl_xor(first, 16, 64));
        first = min(first, __shfl_xor(first, 32, 64));
      }
      if (q == 0) {
        float* const d = st_lds + wave * 384 + i * 16 + r16;
        d[0] = mx; d[128] = z; d[256] = __int_as_float(first);
      }
    }
    if (kStats != 0 && C == nullptr) continue;
#pragma unroll
    for (int j = 0; j < kNI; j += 2) {
      const uint32_t e0 = pk[j][0], e1 = pk[j][1], o0 = pk[j + 1][0], o1 = pk[j + 1][1];
      // odd rows of 16 lanes of the first operand <-> even rows of the second
      const auto s0 = __builtin_amdgcn_permlane16_swap(e0, o0, false, false);
      const auto s1 = __builtin_amdgcn_permlane16_swap(e1, o1, false, false);
      // q even: (own, neighbour's) words of block j = its columns 4 q + 0..7;
      // q odd: (neighbour's, own) words of block j + 1 = its columns 4 (q - 1) + 0..7
      u32x4 v;
      v.x = s0[0]; v.y = s1[0]; v.z = s0[1]; v.w = s1[1];
      const int n = n0 + wn + (j + (q & 1)) * 16 + 4 * (q & 2);
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
  if constexpr (kStats != 0) {
    // the two waves that share a band of rows: the left one (lower columns) folds both halves
    static_assert(kWN == 2 && kTM / kWM == 128, "two column halves per row band");
    __syncthreads();
    if (wn == 0) {
      const float* const a = st_lds + wave * 384;
      const float* const b = a + 384;  // wave + 1: the same rows, columns 128 .. 255
#pragma unroll
      for (int rr = lane; rr < 128; rr += 64) {
        const int m = m0 + wm + rr;
        if (m >= M) continue;
        const float ma = a[rr], mb = b[rr];
        const float mm = fmaxf(ma, mb);  // (ma is finite: the left half always has a column inside N)
        const float z = a[128 + rr] * fast_exp2((ma - mm) * kLog2e) +
                        ((mb == -INFINITY) ? 0.f : b[128 + rr] * fast_exp2((mb - mm) * kLog2e));
        const int first = (mb > ma) ? __float_as_int(b[256 + rr]) : __float_as_int(a[256 + rr]);
        const int64_t at = (int64_t)tile_n * M_host + m, plane = (int64_t)tiles_n * M_host;
        stat_ws[at] = mm;
        stat_ws[plane + at] = z;
        reinterpret_cast<int32_t*>(stat_ws)[2 * plane + at] = first;
      }
    }
  }
}

// Folds the per-tile statistics of gemm_bf16_nt_kernel<.., kStats> into one log-sum-exp (natural
// logarithm) and one first-index arg-max per row: the tiles in ascending column order, a later
// tile wins only with a strictly greater maximum.  A workgroup takes 32 rows; eight threads share a row,
// each folds a contiguous eighth of the tiles (reads of one tile's entries are contiguous over the rows),
// and the eight partial results are folded in their order through LDS.
__global__ __launch_bounds__(256) void gemm_row_stats_reduce_kernel(const float* __restrict__ stat_ws, int M,
                                                                    int tiles_n, float* __restrict__ lse,
                                                                    int32_t* __restrict__ argmax) {
  __shared__ float sm[8][32], sz[8][32];
  __shared__ int si[8][32];
  const int row = threadIdx.x & 31, part = threadIdx.x >> 5;
  const int m = blockIdx.x * 32 + row;
  const int64_t plane = (int64_t)tiles_n * M;
  const int per = (tiles_n + 7) / 8;
  const int t0 = part * per, t1 = min(t0 + per, tiles_n);
  float mm = -INFINITY, z = 0.f;
  int first = 0x7fffffff;
  if (m < M) {
    for (int t = t0; t < t1; ++t) {
      const int64_t at = (int64_t)t * M + m;
      const float pm = stat_ws[at], pz = stat_ws[plane + at];
      if (pm > mm) {
        z = z * fast_exp2((mm - pm) * kLog2e) + pz;  // (the first tile: 0 * 2^-inf)
        mm = pm;
        first = reinterpret_cast<const int32_t*>(stat_ws)[2 * plane + at];
      } else {
        z += pz * fast_exp2((pm - mm) * kLog2e);
      }
    }
  }
  sm[part][row] = mm; sz[part][row] = z; si[part][row] = first;
  __syncthreads();
  if (part != 0 || m >= M) return;
  for (int p = 1; p < 8; ++p) {
    const float pm = sm[p][row], pz = sz[p][row];
    if (pm > mm) {
      z = z * fast_exp2((mm - pm) * kLog2e) + pz;
      mm = pm;
      first = si[p][row];
    } else if (pm != -INFINITY) {  // (a part with no tiles)
      z += pz * fast_exp2((pm - mm) * kLog2e);
    }
  }
  if (lse) lse[m] = (mm * kLog2e + fast_log2(z)) * kLn2;
  if (argmax) argmax[m] = first;
}

// The tiles of the last round of a product cut by tail_plan: C[tile] = the sum of its parts, in their
// order, fp32, one rounding.  blockIdx.x = (tail tile, one of kTailSlices bands of 32 rows): 256 threads x 4
// passes of 8 columns, enough workgroups to fill the chip for the 128 tiles of half a round.
constexpr int kTailSlices = 8;
__global__ __launch_bounds__(256) void gemm_tail_reduce_kernel(const float* __restrict__ part_ws,
                                                               uint16_t* __restrict__ C, int64_t ldc, int M, int N,
                                                               int K, int tiles_m, int tiles_n, int max_parts,
                                                               int cus) {
  int tail_first, tail_parts;
  tail_plan(tiles_m * tiles_n, cus, (K + kTK - 1) / kTK, max_parts, tail_first, tail_parts);
  const int n_tail = tiles_m * tiles_n - tail_first;
  const int tail_idx = (int)blockIdx.x / kTailSlices, slice = (int)blockIdx.x % kTailSlices;
  if (tail_parts <= 1 || tail_idx >= n_tail) return;
  int tile_m, tile_n;
  tile_coords(tail_first + tail_idx, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * kTM, n0 = tile_n * kTN;
  const bool fast = (ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0);
  constexpr int kItems = kTM * (kTN / 8) / kTailSlices;
  for (int it = slice * kItems + threadIdx.x; it < (slice + 1) * kItems; it += 256) {
    const int rr = it / (kTN / 8), cc = (it % (kTN / 8)) * 8;
    const int m = m0 + rr, n = n0 + cc;
    if (m >= M || n >= N) continue;
    f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < tail_parts; ++p) {
      const float* src = part_ws + ((int64_t)(p * n_tail + tail_idx) << 16) + rr * kTN + cc;
      const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
      lo[0] += a[0]; lo[1] += a[1]; lo[2] += a[2]; lo[3] += a[3];
      hi[0] += b[0]; hi[1] += b[1]; hi[2] += b[2]; hi[3] += b[3];
    }
    u32x4 v;
    v.x = pack_bf16x2(lo[0], lo[1]); v.y = pack_bf16x2(lo[2], lo[3]);
    v.z = pack_bf16x2(hi[0], hi[1]); v.w = pack_bf16x2(hi[2], hi[3]);
    if (fast && n + 8 <= N) {
      *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
    } else {
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int e = 0; e < 8; ++e)
        if (n + e < N) C[(int64_t)m * ldc + n + e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
    }
  }
}

// C[m, n .. n + 7] = the sum of the parts of a product whose contraction was cut (in the order of the
// parts, fp32, one rounding).  Re-derives the number of parts like the product did; nothing to do for one.
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part_ws,
                                                                 uint16_t* __restrict__ C, int64_t ldc, int M_host,
                                                                 int N, int K, int tiles_n,
                                                                 const int32_t* __restrict__ m_live, int max_parts,
                                                                 int cus) {
  const int M = m_live ? min(M_host, max(*m_live, 0)) : M_host;
  const int parts = choose_k_parts(((M + kTM - 1) / kTM) * tiles_n, max_parts, cus, (K + kTK - 1) / kTK);
  if (parts <= 1) return;
  const int n8 = N / 8;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= (int64_t)M * n8) return;
  const int m = (int)(item / n8), n = (int)(item % n8) * 8;
  f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
  for (int p = 0; p < parts; ++p) {
    const float* src = part_ws + ((int64_t)p * M_host + m) * N + n;
    const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
    lo[0] += a[0]; lo[1] += a[1]; lo[2] += a[2]; lo[3] += a[3];
    hi[0] += b[0]; hi[1] += b[1]; hi[2] += b[2]; hi[3] += b[3];
  }
  u32x4 v;
  v.x = pack_bf16x2(lo[0], lo[1]); v.y = pack_bf16x2(lo[2], lo[3]);
  v.z = pack_bf16x2(hi[0], hi[1]); v.w = pack_bf16x2(hi[2], hi[3]);
  *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
}

}  // namespace spx

using namespace spx;

// compute units of the current device (looked up once per device)
static int compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n <= 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// an upper bound of compute_units() over the devices this library runs on (MI355X: 256)
static int compute_units_max() { return 512; }

#define SPX_REQ_FN(cond, what) do { if (!(cond)) return spx::fail_arg(fname, what); } while (0)
static int gemm_nt_impl(const char* fname, const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                        int64_t ldc, int64_t M, int64_t N, int64_t K, const int32_t* m_live, void* stream,
                        const int32_t* tile_tab = nullptr, const int32_t* group_off = nullptr,
                        int64_t b_group_stride = 0, int64_t groups = 0, float* part_ws = nullptr,
                        int max_parts = 1, float* stat_ws = nullptr, int stats_mode = 0, int tail_mode = 0) {
  SPX_REQ_FN(M > 0 && N > 0 && K > 0, "M, N, K must be positive");
  SPX_REQ_FN(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "dimension too large");
  SPX_REQ_FN(a && b && (c || stat_ws), "null buffer");
  SPX_REQ_FN(K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0, "K, lda, ldb must be multiples of 8");
  SPX_REQ_FN(lda >= K && ldb >= K && ldc >= N, "leading dimension too small");
  SPX_REQ_FN(((uintptr_t)a | (uintptr_t)b) % 16 == 0, "a and b must be 16-byte aligned");
  SPX_REQ_FN((kTM * lda + K) * 2 < 0x7ffffff0ll && (kTN * ldb + K) * 2 < 0x7ffffff0ll,
             "256 rows of an operand must span less than 2 GiB (32-bit offsets inside a tile)");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool imm = lda >= kTK && ldb >= kTK;
  static std::atomic<uint64_t> lds_set[8];  // per kernel instantiation, one bit per device
  const int which = (imm ? 1 : 0) + 2 * (stat_ws ? stats_mode : 0);
  const void* const fns[8] = {reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<false, 0>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<true, 0>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<false, 1>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<true, 1>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<false, 2>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<true, 2>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<false, 3>),
                              reinterpret_cast<const void*>(&gemm_bf16_nt_kernel<true, 3>)};
  if (int rc = ensure_dynamic_lds(fns[which], kGemmSmem, lds_set[which], fname)) return rc;
  // grouped: every group may end in a partly filled tile row
  const int64_t tiles_m64 = (M + kTM - 1) / kTM + (tile_tab ? groups : 0);
  const int tiles_n = (int)((N + kTN - 1) / kTN);
  SPX_REQ_FN(tiles_m64 * tiles_n < (1ll << 31), "too many tiles");
  const int tiles_m = (int)tiles_m64;
  // (a contraction in parts: room for every part of every tile; the kernel decides how many it uses)
  SPX_REQ_FN((int64_t)tiles_m * tiles_n * max_parts < (1ll << 31), "too many tiles");
  const int cus = compute_units();
  int64_t n_grid = (int64_t)tiles_m * tiles_n * (part_ws ? max_parts : 1);
  int tail_first = tiles_m * tiles_n, tail_parts = 1;
  if (tail_mode) {
    tail_plan(tiles_m * tiles_n, cus, (int)((K + kTK - 1) / kTK), max_parts, tail_first, tail_parts);
    n_grid = (int64_t)tiles_m * tiles_n + (int64_t)(tiles_m * tiles_n - tail_first) * (tail_parts - 1);
  }
  const dim3 grid((unsigned)n_grid), block(kGemmThreads);
#define SPX_GEMM_LAUNCH(IMM, STATS)                                                                              \
  hipLaunchKernelGGL((gemm_bf16_nt_kernel<IMM, STATS>), grid, block, kGemmSmem, st,                              \
                     reinterpret_cast<const uint16_t*>(a), lda, reinterpret_cast<const uint16_t*>(b), ldb,       \
                     reinterpret_cast<uint16_t*>(c), ldc, (int)M, (int)N, (int)K, tiles_m, tiles_n, m_live,      \
                     tile_tab, group_off, b_group_stride, part_ws, max_parts, cus, stat_ws, tail_mode)
  switch (which) {
    case 0: SPX_GEMM_LAUNCH(false, 0); break;
    case 1: SPX_GEMM_LAUNCH(true, 0); break;
    case 2: SPX_GEMM_LAUNCH(false, 1); break;
    case 3: SPX_GEMM_LAUNCH(true, 1); break;
    case 4: SPX_GEMM_LAUNCH(false, 2); break;
    case 5: SPX_GEMM_LAUNCH(true, 2); break;
    case 6: SPX_GEMM_LAUNCH(false, 3); break;
    default: SPX_GEMM_LAUNCH(true, 3); break;
  }
#undef SPX_GEMM_LAUNCH
  if (int rc = check_launch(fname)) return rc;
  if (tail_mode) {
    if (tail_parts > 1) {
      hipLaunchKernelGGL(gemm_tail_reduce_kernel,
                         dim3((unsigned)((tiles_m * tiles_n - tail_first) * kTailSlices)), dim3(256), 0, st,
                         part_ws, reinterpret_cast<uint16_t*>(c), ldc, (int)M, (int)N, (int)K, tiles_m, tiles_n,
                         max_parts, cus);
      return check_launch(fname);
    }
    return 0;
  }
  if (part_ws) {
    const int64_t items = M * (N / 8);
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, part_ws,
                       reinterpret_cast<uint16_t*>(c), ldc, (int)M, (int)N, (int)K, tiles_n, m_live, max_parts, cus);
    return check_launch(fname);
  }
  return 0;
}

namespace spx {
// tab[0] = number of tile rows, then (group, first row) of every tile row: group e contributes
// ceil(rows_e / kTM) of them.  One workgroup; thread t owns a contiguous run of groups.
__global__ __launch_bounds__(256) void gemm_group_tiles_kernel(const int32_t* __restrict__ group_off, int groups,
                                                               int rows, int max_tiles,
                                                               int32_t* __restrict__ tab) {
  __shared__ int sums[256];
  const int t = threadIdx.x;
  const int per = (groups + 255) / 256;
  const int e0 = min(t * per, groups), e1 = min(e0 + per, groups);
  int mine = 0;
  // (offsets are clamped to [0, rows]: the table is sized for that many rows whatever they hold)
  auto clamped = [&](int e) { return min(max(group_off[e], 0), rows); };
  for (int e = e0; e < e1; ++e) mine += (max(clamped(e + 1) - clamped(e), 0) + kTM - 1) / kTM;
  sums[t] = mine;
  __syncthreads();
  if (t == 0) {
    int run = 0;
    for (int i = 0; i < 256; ++i) {
      const int v = sums[i];
      sums[i] = run;
      run += v;
    }
    tab[0] = min(run, max_tiles);  // (offsets that do not ascend could ask for more than the table holds)
  }
  __syncthreads();
  int at = sums[t];
  for (int e = e0; e < e1; ++e) {
    const int r0 = clamped(e), r1 = clamped(e + 1);
    for (int r = r0; r < r1; r += kTM, ++at) {
      if (at >= max_tiles) break;
      tab[1 + 2 * at] = e;
      tab[2 + 2 * at] = r;
    }
  }
}
}  // namespace spx

extern "C" int64_t spx_gemm_grouped_workspace_bytes(int64_t rows, int64_t groups) {
  if (rows < 0 || groups < 0) return 0;
  return (int64_t)sizeof(int32_t) * (1 + 2 * ((rows + kTM - 1) / kTM + groups));
}

extern "C" int spx_gemm_bf16_nt_grouped(const void* a, int64_t lda, const void* b, int64_t ldb,
                                        int64_t b_group_stride, void* c, int64_t ldc, int64_t rows,
                                        int64_t N, int64_t K, const int32_t* group_offsets,
                                        int64_t groups, void* workspace, int64_t workspace_bytes,
                                        void* stream) {
  const char* fname = __func__;
  SPX_REQ_FN(groups > 0 && groups < (1 << 24), "groups must be positive");
  SPX_REQ_FN(group_offsets && workspace, "null group offsets or workspace");
  SPX_REQ_FN(workspace_bytes >= spx_gemm_grouped_workspace_bytes(rows, groups), "workspace too small");
  SPX_REQ_FN(((uintptr_t)workspace) % 4 == 0 && b_group_stride % 8 == 0 && b_group_stride >= 0,
             "unaligned workspace or group stride");
  int32_t* tab = reinterpret_cast<int32_t*>(workspace);
  hipLaunchKernelGGL(gemm_group_tiles_kernel, dim3(1), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     group_offsets, (int)groups, (int)rows, (int)((rows + kTM - 1) / kTM + groups), tab);
  if (int rc = check_launch(fname)) return rc;
  return gemm_nt_impl(fname, a, lda, b, ldb, c, ldc, rows, N, K, nullptr, stream, tab, group_offsets,
                      b_group_stride, groups);
}

extern "C" int spx_gemm_bf16_nt(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                int64_t ldc, int64_t M, int64_t N, int64_t K, void* stream) {
  return gemm_nt_impl(__func__, a, lda, b, ldb, c, ldc, M, N, K, nullptr, stream);
}

extern "C" int64_t spx_gemm_tail_workspace_bytes(void) {
  // (tiles of the last round) x (parts) never exceeds the compute units; one fp32 tile each
  return (int64_t)compute_units_max() * kTM * kTN * (int64_t)sizeof(float);
}

extern "C" int spx_gemm_bf16_nt_tail(const void* a, int64_t lda, const void* b, int64_t ldb, void* c, int64_t ldc,
                                     int64_t M, int64_t N, int64_t K, int32_t max_parts, void* workspace,
                                     int64_t workspace_bytes, void* stream) {
  const char* fname = __func__;
  SPX_REQ_FN(max_parts >= 1 && max_parts <= 8, "max_parts must be 1 .. 8");
  SPX_REQ_FN(workspace && ((uintptr_t)workspace) % 16 == 0, "null or unaligned workspace");
  SPX_REQ_FN(workspace_bytes >= spx_gemm_tail_workspace_bytes(), "workspace too small");
  return gemm_nt_impl(fname, a, lda, b, ldb, c, ldc, M, N, K, nullptr, stream, nullptr, nullptr, 0, 0,
                      reinterpret_cast<float*>(workspace), max_parts, nullptr, 0, 1);
}

extern "C" int64_t spx_gemm_stats_workspace_bytes(int64_t M, int64_t N) {
  if (M <= 0 || N <= 0) return 0;
  return 3 * ((N + kTN - 1) / kTN) * M * (int64_t)sizeof(float);
}

extern "C" int spx_gemm_bf16_nt_stats(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                      int64_t ldc, int64_t M, int64_t N, int64_t K, float* lse,
                                      int32_t* argmax, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
  const char* fname = __func__;
  SPX_REQ_FN(lse || argmax, "null lse and null argmax: nothing to compute");
  SPX_REQ_FN(workspace && ((uintptr_t)workspace) % 4 == 0, "null or unaligned workspace");
  SPX_REQ_FN(M > 0 && N > 0 && workspace_bytes >= spx_gemm_stats_workspace_bytes(M, N), "workspace too small");
  if (int rc = gemm_nt_impl(fname, a, lda, b, ldb, c, c ? ldc : N, M, N, K, nullptr, stream, nullptr, nullptr, 0,
                            0, nullptr, 1, reinterpret_cast<float*>(workspace), (lse ? 1 : 0) + (argmax ? 2 : 0)))
    return rc;
  hipLaunchKernelGGL(gemm_row_stats_reduce_kernel, dim3((unsigned)((M + 31) / 32)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const float*>(workspace), (int)M,
                     (int)((N + kTN - 1) / kTN), lse, argmax);
  return check_launch(fname);
}

extern "C" int64_t spx_gemm_split_workspace_bytes(int64_t M, int64_t N, int32_t max_parts) {
  if (M <= 0 || N <= 0 || max_parts < 1) return 0;
  return (int64_t)max_parts * M * N * (int64_t)sizeof(float);
}

extern "C" int spx_gemm_bf16_nt_rows_split(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                           int64_t ldc, int64_t M, int64_t N, int64_t K, const int32_t* m_live,
                                           int32_t max_parts, void* workspace, int64_t workspace_bytes,
                                           void* stream) {
  const char* fname = __func__;
  SPX_REQ_FN(max_parts >= 1 && max_parts <= 8, "max_parts must be 1 .. 8");
  SPX_REQ_FN(N % 8 == 0 && ldc % 8 == 0 && c && ((uintptr_t)c) % 16 == 0,
             "N and ldc must be multiples of 8 and c 16-byte aligned");
  SPX_REQ_FN(workspace && ((uintptr_t)workspace) % 16 == 0, "null or unaligned workspace");
  SPX_REQ_FN(M > 0 && workspace_bytes >= spx_gemm_split_workspace_bytes(M, N, max_parts), "workspace too small");
  return gemm_nt_impl(fname, a, lda, b, ldb, c, ldc, M, N, K, m_live, stream, nullptr, nullptr, 0, 0,
                      reinterpret_cast<float*>(workspace), max_parts);
}

extern "C" int spx_gemm_bf16_nt_rows(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                     int64_t ldc, int64_t M, int64_t N, int64_t K,
                                     const int32_t* m_live, void* stream) {
  if (!m_live) {
    last_error() = std::string(__func__) + ": null row count";
    return SPX_ERR_ARG;
  }
  return gemm_nt_impl(__func__, a, lda, b, ldb, c, ldc, M, N, K, m_live, stream);
}
#undef SPX_REQ_FN
