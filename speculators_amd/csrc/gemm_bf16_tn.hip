// Weight-gradient GEMM for gfx950: C[M, N] (+)= A[T, M]^T * B[T, N], bf16 operands, fp32
// accumulation; the result is bf16 or fp32 and may be added to what C holds (the gradient of a
// weight that is applied once per TTT step accumulates in place, in fp32 without any rounding
// between the steps).  Both operands are stored with the contraction index T as the SLOW
// dimension (A = the output gradient dY [T, M], B = the layer input X [T, N]), so an MFMA
// fragment -- 8 consecutive t for one m -- is a column of 8 rows in memory.
//
// The tiles are NOT transposed on their way in.  A slab of 64 t-rows x 256 columns of each
// operand goes global -> LDS directly (buffer_load ... lds, whole 512-byte rows), exactly as it
// lies in memory, and the fragments are taken with the transposing LDS read of gfx950
// (ds_read_b64_tr_b16: inside every group of 16 lanes, lane 4u + w receives as element j element
// w of the 8 bytes lane 4j + u points at).  Two such reads make one 16 x 32 operand fragment of
// v_mfma_f32_16x16x32_bf16: lane (G = lane / 16, s = lane % 16) points at row 8 G + s / 4 (+ 4 for
// the second read) of the 32-row K step and at bytes 8 (s % 4) of the fragment's 32-byte column
// block, and ends up with rows 8 G .. 8 G + 7 of column s.
// Bank conflicts: the rows of a slab are 512 bytes apart, so the 32-byte piece p of row t sits at
// piece position p ^ h(t), h(t) = t % 4 + 4 (t / 8 % 2): the 8 rows that one half of the lanes of a
// read touches then cover all 64 banks once.
//
// From there on it is the NT kernel: 256 x 256 tile, 4 waves x 128 x 128 (one per SIMD), two
// slab buffers, 8 x 8 accumulators of 16 x 16 per wave pinned to the accumulation registers, the LDS
// reads of K step kk+1 and the global loads of the next slab issued one at a time between the MFMAs
// of step kk, one barrier per slab, accumulators kept transposed (lane = row of C).  The slab loop is
// written out for two slabs, so that the buffer a read goes to is a constant: a fragment read is an
// address register per fragment plus an immediate, with no vector arithmetic between the MFMAs
// (with 16-cycle MFMAs the kernel is bound by what a wave can issue, and every instruction counts).

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

namespace tn {

constexpr int kNW = 4, kThreads = 256;
constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kWM = 2, kWN = 2;
constexpr int kMI = kTM / kWM / 16, kNI = kTN / kWN / 16;  // 8 x 8 accumulators of 16 x 16 per wave
constexpr int kKSteps = kTK / 32;                          // MFMA K steps per slab
#define SPX_GEMM_TN_READ_EVERY 2  // MFMAs per LDS fragment (two transposing reads) in the K step before the barrier
#define SPX_GEMM_TN_READ_EVERY_B 4  // the same in the K step after it, which also issues the global loads
constexpr int kRowBytes = kTM * 2;                          // 512: one t-row of a slab
constexpr int kABytes = kTK * kRowBytes;                    // one slab of A: 32 KB
constexpr int kBBytes = kABytes;
constexpr int kBBase = 2 * kABytes;
constexpr int kSmem = 2 * (kABytes + kBBytes);              // 128 KB
constexpr int kLA = kTK / 2 / kNW;                          // wave-loads (2 rows each) of A per wave per slab
constexpr int kLB = kLA;
constexpr int kL = kLA + kLB;
constexpr int kOob = 0x7ffffff0;
static_assert(kTM == kTN, "both operands use one slab layout");
static_assert(kABytes + (kKSteps - 1) * 32 * kRowBytes + 4 * kRowBytes < 65536,
              "slab buffer, K step and row pair of a fragment read go into the 16-bit offset field");

typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
// transposing read at a 32-bit LDS address (base included): a constant added to it goes into the
// offset field of the instruction
__device__ __forceinline__ i16x4 lds_read_tr16_at(uint32_t addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(uintptr_t)addr);
}

// OUT: 0 = bf16 result, 1 = bf16 result added to C, 2 = fp32 result, 3 = fp32 result added to C
// MULTI: the operands are n_seg segments of T rows each, one below the other; group e owns the rows
// [group_off[s][e], group_off[s][e+1]) of every segment s and its contraction runs over all of them
// (the expert-sorted rows of several uses of one expert stack: one product, one write of C)
template <int OUT, bool MULTI = false>
__global__ __launch_bounds__(kThreads, 1) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_bf16_tn_kernel(
    const uint16_t* __restrict__ A, int64_t lda, const uint16_t* __restrict__ B, int64_t ldb,
    void* __restrict__ Cv, int64_t ldc, int M, int N, int T, int tiles_m, int tiles_n,
    const int32_t* __restrict__ group_off, int64_t c_group_stride, int n_seg = 1, int n_groups = 0) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // grouped product (blockIdx.y = group): the contraction runs over the group's rows
  // [group_off[e], group_off[e+1]) of both operands, and every group has a C of its own.  An empty
  // group multiplies nothing: zeros are written (or C is left as it is when the result is added)
  const uint16_t* const A0 = A;
  const uint16_t* const B0 = B;
  const int seg_rows = T;
  int seg = 0;
  // rows [first, last) of segment s that belong to this workgroup's group
  auto seg_range = [&](int s, int& first, int& last) __attribute__((always_inline)) {
    const int e = blockIdx.y;
    const int32_t* o = group_off + (MULTI ? (int64_t)s * (n_groups + 1) : 0);
    first = min(max(o[e], 0), seg_rows);
    last = min(max(o[e + 1], first), seg_rows);
  };
  int total_slabs = 0;
  if (group_off) {
    int t0, t1;
    if (MULTI) {
      for (int s2 = 0; s2 < n_seg; ++s2) {
        seg_range(s2, t0, t1);
        total_slabs += (t1 - t0 + kTK - 1) / kTK;
      }
      // the first segment that has rows (n_seg if none has)
      for (seg = 0; seg < n_seg; ++seg) {
        seg_range(seg, t0, t1);
        if (t1 > t0) break;
      }
      if (seg == n_seg) t0 = t1 = 0;
    } else {
      seg_range(0, t0, t1);
    }
    A += ((int64_t)seg * seg_rows + t0) * lda;
    B += ((int64_t)seg * seg_rows + t0) * ldb;
    T = t1 - t0;
    Cv = reinterpret_cast<uint8_t*>(Cv) + blockIdx.y * c_group_stride * (OUT >= 2 ? 4 : 2);
    if ((OUT & 1) && (MULTI ? total_slabs == 0 : T == 0)) return;
  }

  // workgroup id -> tile.  The operands of a weight gradient are GBs (the contraction runs over the rows of
  // several steps): what a tile order can save is memory traffic behind the L2s.  The 256 tiles that run at a
  // time (a round) form a block of 16 x 16 tiles, so every 256-column band of either operand that the round
  // touches is used by 16 of its tiles, and the rounds walk along the longer side of the tile grid: a band of
  // the operand on that side is read in one round only, the other operand again every round.  Inside a round
  // each XCD (workgroups go to them round robin) has 32 neighbouring tiles, 8 along the longer side x 4: 12
  // bands through its L2, and a band of the longer side's operand is shared by four XCDs at the same time.
  const int n_wg = tiles_m * tiles_n;
  int pid;
  {
    constexpr int kRound = 256, kPer = kRound / 8;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int full = n_wg / kRound * kRound;
    if ((int)blockIdx.x < full) {
      pid = (local / kPer) * kRound + xcd * kPer + local % kPer;
    } else {  // the last, partial round: one contiguous piece per XCD (the first n % 8 get one tile more)
      const int nr = n_wg - full, base = nr >> 3, rem = nr & 7;
      pid = full + xcd * base + min(xcd, rem) + (local - full / 8);
    }
  }
  int tile_m, tile_n;
  {
    // tiles in the order of pid: panels of kPanel along the shorter side; inside a panel groups of kGroup along
    // the longer side; inside a group the longer side first (the NT kernel's tile_coords: same order)
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
  const int m0 = tile_m * kTM, n0 = tile_n * kTN;

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

  // One buffer resource per operand, starting at the tile's first column.  The whole offset of a load,
  // the slab's first row included, is in the vector register, which is what the range check sees: rows
  // past T lie outside the resource and read as zero.  A 16-byte chunk past the last column would read
  // the next row instead, so those lanes get an offset outside the resource.
  u32x4 ares = make_rsrc(A + m0, T > 0 ? (uint32_t)((((int64_t)T - 1) * lda + min(M - m0, kTM)) * 2) : 0u);
  u32x4 bres = make_rsrc(B + n0, T > 0 ? (uint32_t)((((int64_t)T - 1) * ldb + min(N - n0, kTN)) * 2) : 0u);

  // global side: wave-load j of this wave covers slab rows 2 (wave * kLA + j) + lane / 32; the lane's LDS
  // position is 16-byte chunk lane % 32 of the row, which holds a chunk of the 32-byte piece
  // (position / 2) ^ h(row)
  const int lrow = lane >> 5, lpos = lane & 31;
  int aoff[kLA], boff[kLB];
#pragma unroll
  for (int j = 0; j < kLA; ++j) {
    const int r = 2 * (wave * kLA + j) + lrow;
    const int hr = (r & 3) | (((r >> 3) & 1) << 2);
    const int c8 = ((((lpos >> 1) ^ hr) << 1) | (lpos & 1)) * 8;  // first column of the chunk
    aoff[j] = (m0 + c8 < M) ? (int)(((int64_t)r * lda + c8) * 2) : kOob;
    boff[j] = (n0 + c8 < N) ? (int)(((int64_t)r * ldb + c8) * 2) : kOob;
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
  const uint32_t lds_a = lds0 + wave * kLA * 1024;
  const uint32_t lds_b = lds0 + kBBase + wave * kLB * 1024;

  uint32_t bufoff = 0;  // slab buffer the next loads go to
  int ld_t0 = 0;        // first row of the slab being loaded
  const int a_row = (int)(lda * 2), b_row = (int)(ldb * 2);
  // load l (A loads first, then B) of the slab at ld_t0
  auto issue_one = [&](int l) __attribute__((always_inline)) {
    const bool isa = l < kLA;
    const int j = isa ? l : l - kLA;
    const uint32_t voff = (uint32_t)(isa ? aoff[j] : boff[j]) + (uint32_t)ld_t0 * (uint32_t)(isa ? a_row : b_row);
    // (a lane that is out of range stays so: kOob plus the row offset lies past any resource size)
    load_to_lds16<0>(isa ? ares : bres, (isa ? lds_a : lds_b) + bufoff + j * 1024, (int)voff, 0);
  };
  auto next_slab = [&]() __attribute__((always_inline)) {
    bufoff ^= kABytes;
    ld_t0 += kTK;
    if (MULTI && ld_t0 >= T && seg < n_seg) {
      // this segment's rows are all requested: go on with the next segment that has rows (the
      // resources are rebuilt around it, so rows past its end read as zero like before); when
      // there is none left the resources are empty and every further load brings zeros
      int t0 = 0, t1 = 0;
      for (++seg; seg < n_seg; ++seg) {
        seg_range(seg, t0, t1);
        if (t1 > t0) break;
      }
      if (seg >= n_seg) t0 = t1 = 0;
      T = t1 - t0;
      ld_t0 = 0;
      const int64_t row0 = (int64_t)min(seg, n_seg - 1) * seg_rows + t0;
      ares = make_rsrc(A0 + row0 * lda + m0, T > 0 ? (uint32_t)((((int64_t)T - 1) * lda + min(M - m0, kTM)) * 2) : 0u);
      bres = make_rsrc(B0 + row0 * ldb + n0, T > 0 ? (uint32_t)((((int64_t)T - 1) * ldb + min(N - n0, kTN)) * 2) : 0u);
    }
  };

  // read side (see the head of the file)
  const int trow = 8 * q + (r16 >> 2);
  const int lane_off = trow * kRowBytes + (((r16 >> 2) | ((q & 1) << 2)) * 32) + 8 * (r16 & 3);
  uint32_t a_rd[kMI], b_rd[kNI];  // per fragment: LDS address in slab buffer 0
#pragma unroll
  for (int f = 0; f < kMI; ++f) {
    a_rd[f] = lds0 + (lane_off ^ ((wm / 16 + f) * 32));
    b_rd[f] = lds0 + kBBase + (lane_off ^ ((wn / 16 + f) * 32));
    // (kept opaque: otherwise the B operand's 64 KB base is folded out of the register into the
    // constant and no longer fits the offset field)
    asm volatile("" : "+v"(a_rd[f]), "+v"(b_rd[f]));
  }

  i16x4 fa[2][kMI][2], fb[2][kNI][2];
  // operand fragment f (A fragments first, then B) of K step kk of slab buffer buf into register
  // set `set`; buf and kk are constants where this is called, so they end up in the offset field
  auto read_one = [&](int set, int buf, int kk, int f) __attribute__((always_inline)) {
    const uint32_t o = buf * kABytes + kk * 32 * kRowBytes;
    if (f < kMI) {
      fa[set][f][0] = lds_read_tr16_at(a_rd[f] + o);
      fa[set][f][1] = lds_read_tr16_at(a_rd[f] + o + 4 * kRowBytes);
    } else {
      fb[set][f - kMI][0] = lds_read_tr16_at(b_rd[f - kMI] + o);
      fb[set][f - kMI][1] = lds_read_tr16_at(b_rd[f - kMI] + o + 4 * kRowBytes);
    }
  };
  auto frag = [&](const i16x4 (&h)[2]) __attribute__((always_inline)) {
    const i16x8 v = __builtin_shufflevector(h[0], h[1], 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
  };
  // One K step: the kNI x kMI MFMAs on register set `set`; between them, one at a time, the LDS
  // reads that fill the other set with K step rk and the global loads [l0, l0 + nl).
  auto step = [&](int set, int rbuf, int rk, int l0, int nl, int every) __attribute__((always_inline)) {
    constexpr int kN = kNI * kMI, kF = kMI + kNI;
    int reads = 0, loads = 0;
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int i = 0; i < kMI; ++i) {
        mfma16(acc[j][i], frag(fb[set][j]), frag(fa[set][i]));
        const int idx = j * kMI + i;
        __builtin_amdgcn_sched_barrier(0);
        if (reads < kF && idx % every == every - 1) {
          read_one(set ^ 1, rbuf, rk, reads++);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (nl > 0 && (nl >= kN || idx % (kN / nl) == kN / nl - 1) && loads < nl) {
          issue_one(l0 + loads++);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
  };

  // the loads of a slab are issued in the step after the barrier that frees its buffer, one per four
  // MFMAs; the step after that gives them time to land
  static_assert(kKSteps == 2, "a slab is two K steps: one before, one after the barrier");
  constexpr int kLdT = kL;
  // buf: the buffer slab s lies in, a constant in each of the two copies of the loop body
  auto slab = [&](int buf) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    step(0, buf, 1, 0, 0, SPX_GEMM_TN_READ_EVERY);
    next_slab();
    // every read of this slab's buffer has returned once set 1 is complete; then the barrier says:
    // slab s+1 has landed for everybody, this buffer is free
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    // K step 1 of slab s, under it the reads of step 0 of slab s+1 and the loads of slab s+2
    step(1, buf ^ 1, 0, 0, kLdT, SPX_GEMM_TN_READ_EVERY_B);
  };

  const int nslab = MULTI ? total_slabs : (T + kTK - 1) / kTK;
#pragma unroll
  for (int l = 0; l < kL; ++l) issue_one(l);
  next_slab();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  // (past the last slab every row is out of range: zeros go into the free buffer)
#pragma unroll
  for (int l = 0; l < kLdT; ++l) issue_one(l);
#pragma unroll
  for (int f = 0; f < kMI + kNI; ++f) read_one(0, 0, 0, f);
  int s = 0;
  for (; s + 1 < nslab; s += 2) {
    slab(0);
    slab(1);
  }
  if (s < nslab) slab(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  mfma_results_ready();
  // epilogue: a lane holds row m of C and, per accumulator, columns 4 q + {0..3} of a 16-column block
  if constexpr (OUT >= 2) {
    float* const C = reinterpret_cast<float*>(Cv);
    const bool fast = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0) && (n0 + kTN <= N);
#pragma unroll
    for (int i = 0; i < kMI; ++i) {
      const int m = m0 + wm + i * 16 + r16;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < kNI; ++j) {
        const f32x4& a = acc[j][i];
        const int n = n0 + wn + j * 16 + 4 * q;
        float* cp = C + (int64_t)m * ldc + n;
        if (fast) {
          f32x4 v = a;
          if (OUT == 3) {
            const f32x4 old = *reinterpret_cast<const f32x4*>(cp);
            v[0] += old[0]; v[1] += old[1]; v[2] += old[2]; v[3] += old[3];
          }
          *reinterpret_cast<f32x4*>(cp) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) cp[e] = (OUT == 3 ? cp[e] : 0.f) + a[e];
        }
      }
    }
    return;
  } else {
    // Swapping the words of the q-odd lanes for block j with those of the q-even lanes for block j + 1
    // (v_permlane16_swap) leaves every lane with 8 consecutive columns: 16-byte stores.
    uint16_t* const C = reinterpret_cast<uint16_t*>(Cv);
    constexpr bool ACC = OUT == 1;
    const bool fast = (ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0) && (n0 + kTN <= N);
#pragma unroll
    for (int i = 0; i < kMI; ++i) {
      const int m = m0 + wm + i * 16 + r16;
#pragma unroll
      for (int j = 0; j < kNI; j += 2) {
        f32x4 a = acc[j][i], b = acc[j + 1][i];
        // q even: columns 4 q + 0..7 of block j; q odd: columns 4 (q - 1) + 0..7 of block j + 1
        const int n = n0 + wn + (j + (q & 1)) * 16 + 4 * (q & 2);
        if (ACC && fast) {
          // swap the fp32 words, add what C holds (one 16-byte load per lane, the store's own layout)
          float v[8];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(a[e]), __float_as_uint(b[e]), false, false);
            v[e] = __uint_as_float(sw[0]);
            v[4 + e] = __uint_as_float(sw[1]);
          }
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
          continue;
        }
        if (ACC && m < M) {
          // ragged edge: what C holds, read in the accumulators' own layout (4 consecutive columns each)
          const int na = n0 + wn + j * 16 + 4 * q;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (na + e < N) a[e] += bf16_bits_to_f32(C[(int64_t)m * ldc + na + e]);
            if (na + 16 + e < N) b[e] += bf16_bits_to_f32(C[(int64_t)m * ldc + na + 16 + e]);
          }
        }
        const uint32_t e0 = pack_bf16x2(a[0], a[1]), e1 = pack_bf16x2(a[2], a[3]);
        const uint32_t o0 = pack_bf16x2(b[0], b[1]), o1 = pack_bf16x2(b[2], b[3]);
        const auto s0 = __builtin_amdgcn_permlane16_swap(e0, o0, false, false);
        const auto s1 = __builtin_amdgcn_permlane16_swap(e1, o1, false, false);
        u32x4 v;
        v.x = s0[0]; v.y = s1[0]; v.z = s0[1]; v.w = s1[1];
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

#define SPX_REQ_FN(cond, what) do { if (!(cond)) return spx::fail_arg(fname, what); } while (0)
template <int OUT, bool MULTI = false>
static int launch_tn(const char* fname, const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                     int64_t ldc, int64_t M, int64_t N, int64_t T, void* stream,
                     const int32_t* group_off = nullptr, int64_t c_group_stride = 0, int64_t groups = 1,
                     int64_t segments = 1) {
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  static std::atomic<uint64_t> lds_set;  // per kernel instantiation, one bit per device
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&tn::gemm_bf16_tn_kernel<OUT, MULTI>), tn::kSmem,
                                  lds_set, fname))
    return rc;
  const int tiles_m = (int)((M + tn::kTM - 1) / tn::kTM), tiles_n = (int)((N + tn::kTN - 1) / tn::kTN);
  const dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)groups), block(tn::kThreads);
  hipLaunchKernelGGL((tn::gemm_bf16_tn_kernel<OUT, MULTI>), grid, block, tn::kSmem, st,
                     reinterpret_cast<const uint16_t*>(a), lda, reinterpret_cast<const uint16_t*>(b), ldb, c,
                     ldc, (int)M, (int)N, (int)T, tiles_m, tiles_n, group_off, c_group_stride, (int)segments,
                     (int)groups);
  return check_launch(fname);
}

static int gemm_tn_check(const char* fname, const void* a, int64_t lda, const void* b, int64_t ldb,
                         const void* c, int64_t ldc, int64_t M, int64_t N, int64_t T) {
  SPX_REQ_FN(M > 0 && N > 0 && T > 0, "M, N, T must be positive");
  SPX_REQ_FN(M < (1ll << 31) && N < (1ll << 31) && T < (1ll << 31), "dimension too large");
  SPX_REQ_FN(a && b && c, "null buffer");
  SPX_REQ_FN(M % 8 == 0 && N % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0, "M, N, lda, ldb must be multiples of 8");
  SPX_REQ_FN(lda >= M && ldb >= N && ldc >= N, "leading dimension too small");
  SPX_REQ_FN(((uintptr_t)a | (uintptr_t)b) % 16 == 0, "a and b must be 16-byte aligned");
  SPX_REQ_FN(((T + 4 * tn::kTK) * lda) * 2 < 0x7ffffff0ll && ((T + 4 * tn::kTK) * ldb) * 2 < 0x7ffffff0ll,
             "each operand must span less than 2 GiB (32-bit buffer offsets)");
  SPX_REQ_FN((int64_t)((M + tn::kTM - 1) / tn::kTM) * ((N + tn::kTN - 1) / tn::kTN) < (1ll << 31), "too many tiles");
  return SPX_OK;
}

extern "C" int spx_gemm_bf16_tn(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                int64_t ldc, int64_t M, int64_t N, int64_t T, int accumulate,
                                void* stream) {
  if (int rc = gemm_tn_check(__func__, a, lda, b, ldb, c, ldc, M, N, T)) return rc;
  return accumulate ? launch_tn<1>(__func__, a, lda, b, ldb, c, ldc, M, N, T, stream)
                    : launch_tn<0>(__func__, a, lda, b, ldb, c, ldc, M, N, T, stream);
}

extern "C" int spx_gemm_bf16_tn_f32(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                    int64_t ldc, int64_t M, int64_t N, int64_t T, int accumulate,
                                    void* stream) {
  if (int rc = gemm_tn_check(__func__, a, lda, b, ldb, c, ldc, M, N, T)) return rc;
  return accumulate ? launch_tn<3>(__func__, a, lda, b, ldb, c, ldc, M, N, T, stream)
                    : launch_tn<2>(__func__, a, lda, b, ldb, c, ldc, M, N, T, stream);
}

extern "C" int spx_gemm_bf16_tn_grouped(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                        int64_t ldc, int64_t c_group_stride, int64_t M, int64_t N,
                                        int64_t rows, const int32_t* group_offsets, int64_t groups,
                                        int out_f32, int accumulate, void* stream) {
  const char* fname = __func__;
  if (int rc = gemm_tn_check(fname, a, lda, b, ldb, c, ldc, M, N, rows)) return rc;
  SPX_REQ_FN(group_offsets && groups > 0 && groups < 65536, "null group offsets or a group count outside 1 .. 65535");
  SPX_REQ_FN(c_group_stride >= (M - 1) * ldc + N, "groups of c overlap");
  SPX_REQ_FN(c_group_stride % (out_f32 ? 4 : 8) == 0, "the groups of c must be 16-byte aligned among each other");
  if (out_f32)
    return accumulate ? launch_tn<3>(fname, a, lda, b, ldb, c, ldc, M, N, rows, stream, group_offsets, c_group_stride, groups)
                      : launch_tn<2>(fname, a, lda, b, ldb, c, ldc, M, N, rows, stream, group_offsets, c_group_stride, groups);
  return accumulate ? launch_tn<1>(fname, a, lda, b, ldb, c, ldc, M, N, rows, stream, group_offsets, c_group_stride, groups)
                    : launch_tn<0>(fname, a, lda, b, ldb, c, ldc, M, N, rows, stream, group_offsets, c_group_stride, groups);
}

extern "C" int spx_gemm_bf16_tn_grouped_multi(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                              int64_t ldc, int64_t c_group_stride, int64_t M, int64_t N,
                                              int64_t segment_rows, int64_t segments,
                                              const int32_t* group_offsets, int64_t groups, int out_f32,
                                              int accumulate, void* stream) {
  const char* fname = __func__;
  if (int rc = gemm_tn_check(fname, a, lda, b, ldb, c, ldc, M, N, segment_rows)) return rc;
  SPX_REQ_FN(group_offsets && groups > 0 && groups < 65536, "null group offsets or a group count outside 1 .. 65535");
  SPX_REQ_FN(segments > 0 && segments <= 64, "1 .. 64 segments");
  SPX_REQ_FN(c_group_stride >= (M - 1) * ldc + N, "groups of c overlap");
  SPX_REQ_FN(c_group_stride % (out_f32 ? 4 : 8) == 0, "the groups of c must be 16-byte aligned among each other");
  if (out_f32)
    return accumulate ? launch_tn<3, true>(fname, a, lda, b, ldb, c, ldc, M, N, segment_rows, stream, group_offsets,
                                           c_group_stride, groups, segments)
                      : launch_tn<2, true>(fname, a, lda, b, ldb, c, ldc, M, N, segment_rows, stream, group_offsets,
                                           c_group_stride, groups, segments);
  return accumulate ? launch_tn<1, true>(fname, a, lda, b, ldb, c, ldc, M, N, segment_rows, stream, group_offsets,
                                         c_group_stride, groups, segments)
                    : launch_tn<0, true>(fname, a, lda, b, ldb, c, ldc, M, N, segment_rows, stream, group_offsets,
                                         c_group_stride, groups, segments);
}
#undef SPX_REQ_FN
