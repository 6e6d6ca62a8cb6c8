// Draft-model attention for gfx950: EAGLE3 test-time-training (TTT) attention
// and DFlash anchored-block attention, forward and backward, from one family
// of interval-masked flash-attention kernels.
//
// Every query row r sees up to two key INTERVALS of the K/V rows, plus (TTT
// only) a few single keys:
//   * context keys      a1[r] <= c < b1[r]          (rows [0, T) of K/V)
//   * block keys    T + a2[r] <= c < T + b2[r]      (rows [T, T+NQ): DFlash's own
//                                                    mask-token block)
//   * TTT diagonal keys: rows j*T + r, j = 1..n_extra -- ONE key per earlier
//     step, handled as n_extra dot products per row instead of 128x128 tiles.
// TTT:    a1 = row_lo (document start / window / the row itself for padding),
//         b1 = r + 1, no block interval.
// DFlash: a1 = max(doc start, anchor - W), b1 = anchor, a2/b2 = the query's own
//         block (all of it, or up to the query under a causal window layer).
// Key tiles that no row of a workgroup can see are skipped analytically; no
// dense mask or BlockMask exists anywhere.

#include <type_traits>

#include "attn_common.h"
#include "../../include/spx.h"

namespace spx {

struct AttnParams {
  const uint16_t* Q; int64_t q_hs;   // [Hq][NQ][D]
  const uint16_t* K; int64_t k_hs;   // [Hkv][>= NKV (+ n_extra*T)][D]
  const uint16_t* V; int64_t v_hs;
  const int32_t* a1; const int32_t* b1;  // b1 == nullptr: b1[r] = r + 1
  const int32_t* a2; const int32_t* b2;  // nullptr: no block interval
  int NQ, T, NKV, NKVp;  // NKVp: row length of the transposed operands (multiple of 128)
  int n_extra, Hq, Hkv;
  float scale_log2e, scaling;
};

// ---------------------------------------------------------------- mask descriptors
template <typename I>
__global__ __launch_bounds__(1024) void ttt_row_lo_kernel(const I* __restrict__ doc, int64_t T,
                                                          int64_t window, int32_t* __restrict__ lo) {
  __shared__ int seg_max[1024];
  const int t = threadIdx.x;
  const int64_t len = (T + 1023) / 1024;
  const int64_t b = t * len, e = (b + len < T) ? b + len : T;
  int run = -1;
  for (int64_t i = b; i < e; ++i)
    if (i == 0 || doc[i] != doc[i - 1]) run = (int)i;
  seg_max[t] = run;
  __syncthreads();
  int carry = -1;
  for (int s = 0; s < t; ++s) carry = max(carry, seg_max[s]);
  run = carry;
  for (int64_t i = b; i < e; ++i) {
    if (i == 0 || doc[i] != doc[i - 1]) run = (int)i;
    int v = run;
    if (doc[i] == (I)-1) v = (int)i;
    else if (window > 0 && i - window + 1 > v) v = (int)(i - window + 1);
    lo[i] = v;
  }
}

// start of the run of equal document ids that contains position i
template <typename I>
__global__ __launch_bounds__(1024) void doc_run_start_kernel(const I* __restrict__ doc, int64_t T,
                                                             int32_t* __restrict__ start) {
  __shared__ int seg_max[1024];
  const int t = threadIdx.x;
  const int64_t len = (T + 1023) / 1024;
  const int64_t b = t * len, e = (b + len < T) ? b + len : T;
  int run = -1;
  for (int64_t i = b; i < e; ++i)
    if (i == 0 || doc[i] != doc[i - 1]) run = (int)i;
  seg_max[t] = run;
  __syncthreads();
  int carry = -1;
  for (int s = 0; s < t; ++s) carry = max(carry, seg_max[s]);
  run = carry;
  for (int64_t i = b; i < e; ++i) {
    if (i == 0 || doc[i] != doc[i - 1]) run = (int)i;
    start[i] = run;
  }
}

template <typename I, typename J>
__global__ __launch_bounds__(256) void dflash_ranges_kernel(
    const I* __restrict__ doc, const int32_t* __restrict__ run_start, const J* __restrict__ anchors,
    int64_t n_anchors, int block_size, int64_t window, int causal_block, int64_t T,
    int32_t* __restrict__ a1, int32_t* __restrict__ b1, int32_t* __restrict__ a2,
    int32_t* __restrict__ b2) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= n_anchors * block_size) return;
  const int64_t j = r / block_size;
  int64_t a = (int64_t)anchors[j];
  a = a < 0 ? 0 : (a >= T ? T - 1 : a);
  int lo = 0, hi = 0;
  if (doc[a] != (I)-1) {
    lo = run_start[a];
    if (window > 0 && a - window > lo) lo = (int)(a - window);
    hi = (int)a;
    if (hi < lo) hi = lo;
  }
  a1[r] = lo;
  b1[r] = hi;
  a2[r] = (int)(j * block_size);
  b2[r] = causal_block ? (int)(r + 1) : (int)((j + 1) * block_size);
}

// Eight bf16 values times a scalar, rounded back to bf16 (round to nearest even).  The queries
// enter every score product as bf16(q * scale * log2 e): the forward, the dQ kernel (both scale
// their register fragments with this function) and the dK/dV and diagonal-key kernels (which
// read the copy the backward's prologue writes with it) must see the SAME rounded values, or the
// probabilities the backward recomputes would not match the forward's log-sum-exp.
__device__ __forceinline__ u32x4 scale_bf16x8(u32x4 raw, float c) {
  u32x4 w;
  w.x = pack_bf16x2(bf16_lo(raw.x) * c, bf16_hi(raw.x) * c);
  w.y = pack_bf16x2(bf16_lo(raw.y) * c, bf16_hi(raw.y) * c);
  w.z = pack_bf16x2(bf16_lo(raw.z) * c, bf16_hi(raw.z) * c);
  w.w = pack_bf16x2(bf16_lo(raw.w) * c, bf16_hi(raw.w) * c);
  return w;
}

// ---------------------------------------------------------------- transpose
// dst[h][c][perm(r)] = src[h][r][c] for r < rows, c < cols; dst row stride ld_dst >= rows
// (a multiple of 16), the columns of r in rows..ld_dst-1 are zero filled.  perm swaps bits
// 2 and 3 of r: inside every group of 16 the order is 0-3, 8-11, 4-7, 12-15, which puts
// the 8 rows a lane half needs as MFMA k-slots (4 g + 0..3 and 8 + 4 g + 0..3) side by
// side, so that operand is ONE 16-byte LDS read.
// One wave per 64 x 64 tile, no LDS: a lane loads an 8 (r) x 8 (c) block with eight 16-byte row loads
// (eight lanes read a whole 128-byte line), transposes it in registers (v_perm_b32) and writes, for each
// of its 8 columns, the two 4-row halves of the block to their permuted places (8 bytes each; the eight
// lanes that share a column fill its 128-byte line in two store instructions).  cols a multiple of 8.
// SCALED: the elements are multiplied by `scale` first (scale_bf16x8) and the scaled rows are also
// written row-major to `scaled` ([h][rows][cols], head stride rows * cols).
template <bool SCALED>
__global__ __launch_bounds__(64) void transpose_bf16_kernel(
    const uint16_t* __restrict__ src, int64_t src_hs, int64_t src_ld, int rows, int cols,
    uint16_t* __restrict__ dst, int64_t dst_hs, int64_t ld_dst, float scale,
    uint16_t* __restrict__ scaled) {
  const int h = blockIdx.z;
  const int lane = threadIdx.x;
  const int rb = lane >> 3, cb = lane & 7;
  const int r0 = blockIdx.x * 64 + rb * 8, c0 = blockIdx.y * 64 + cb * 8;
  if (c0 >= cols) return;
  const uint16_t* s = src + (int64_t)h * src_hs + c0;
  u32x4 in[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const u32x4 z = {0, 0, 0, 0};
    in[j] = (r0 + j < rows) ? *reinterpret_cast<const u32x4*>(s + (int64_t)(r0 + j) * src_ld) : z;
    if (SCALED) {
      in[j] = scale_bf16x8(in[j], scale);
      if (r0 + j < rows)
        *reinterpret_cast<u32x4*>(scaled + ((int64_t)h * rows + r0 + j) * cols + c0) = in[j];
    }
  }
  if (SCALED && dst == nullptr) return;  // only the scaled row-major copy is wanted
  // where the block's two halves go: r0 % 16 == 0 -> r0 and r0 + 8, r0 % 16 == 8 -> r0 - 4 and r0 + 4
  const int p_lo = (r0 & 8) ? r0 - 4 : r0, p_hi = (r0 & 8) ? r0 + 4 : r0 + 8;
  uint16_t* d = dst + (int64_t)h * dst_hs + (int64_t)c0 * ld_dst;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // column c0 + i of the block: element e = in[e] element i
    const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
    const int w = i >> 1;
    u32x2 lo, hi;
    lo.x = __builtin_amdgcn_perm(in[1][w], in[0][w], sel);
    lo.y = __builtin_amdgcn_perm(in[3][w], in[2][w], sel);
    hi.x = __builtin_amdgcn_perm(in[5][w], in[4][w], sel);
    hi.y = __builtin_amdgcn_perm(in[7][w], in[6][w], sel);
    *reinterpret_cast<u32x2*>(d + (int64_t)i * ld_dst + p_lo) = lo;
    *reinterpret_cast<u32x2*>(d + (int64_t)i * ld_dst + p_hi) = hi;
  }
}

// per-lane intervals of the NSB query rows a lane owns, and their wave / block extents
template <int NSB>
struct RowBounds {
  int a1[NSB], b1[NSB], a2[NSB], b2[NSB];
  int w_a1min, w_a1max, w_b1min, w_b1max;
  int w_a2min, w_a2max, w_b2min, w_b2max;
  int blk_a1, blk_b1, blk_a2, blk_b2;
};

// value of the partner lane (lane ^ 32) combined with the own one, through v_permlane32_swap
// (a VALU move) instead of an LDS permute: swapping (x, x) leaves the lower half of the wave's
// values in every lane of the first result and the upper half in the second
__device__ __forceinline__ float half_swap_max(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto s = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(s[0]), __uint_as_float(s[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto s = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}

__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = min(v, __shfl_xor(v, m, 64));
  return v;
}
__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = max(v, __shfl_xor(v, m, 64));
  return v;
}

template <int NSB, int NW>
__device__ __forceinline__ void load_bounds(const AttnParams& p, const int (&ic)[NSB], int wave,
                                            int lane, int* red /* [4 * NW] LDS */, RowBounds<NSB>& rb) {
  int a1mn = 0x7fffffff, a1mx = 0, b1mn = 0x7fffffff, b1mx = 0;
  int a2mn = 0x7fffffff, a2mx = 0, b2mn = 0x7fffffff, b2mx = 0;
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    rb.a1[sb] = p.a1[ic[sb]];
    rb.b1[sb] = p.b1 ? p.b1[ic[sb]] : ic[sb] + 1;
    if (p.a2) {
      rb.a2[sb] = p.T + p.a2[ic[sb]];
      rb.b2[sb] = p.T + p.b2[ic[sb]];
    } else {
      rb.a2[sb] = 0; rb.b2[sb] = 0;
    }
    a1mn = min(a1mn, rb.a1[sb]); a1mx = max(a1mx, rb.a1[sb]);
    b1mn = min(b1mn, rb.b1[sb]); b1mx = max(b1mx, rb.b1[sb]);
    a2mn = min(a2mn, rb.a2[sb]); a2mx = max(a2mx, rb.a2[sb]);
    b2mn = min(b2mn, rb.b2[sb]); b2mx = max(b2mx, rb.b2[sb]);
  }
  // wave-uniform values are moved to scalar registers: the tests on them then compile to
  // scalar branches (a masked and an unmasked tile path) instead of per-lane selects
  auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  rb.w_a1min = uni(wave_min_i(a1mn)); rb.w_a1max = uni(wave_max_i(a1mx));
  rb.w_b1min = uni(wave_min_i(b1mn)); rb.w_b1max = uni(wave_max_i(b1mx));
  rb.w_a2min = uni(wave_min_i(a2mn)); rb.w_a2max = uni(wave_max_i(a2mx));
  rb.w_b2min = uni(wave_min_i(b2mn)); rb.w_b2max = uni(wave_max_i(b2mx));
  if (lane == 0) {
    red[wave * 4 + 0] = rb.w_a1min; red[wave * 4 + 1] = rb.w_b1max;
    red[wave * 4 + 2] = rb.w_a2min; red[wave * 4 + 3] = rb.w_b2max;
  }
  __syncthreads();
  rb.blk_a1 = red[0]; rb.blk_b1 = red[1]; rb.blk_a2 = red[2]; rb.blk_b2 = red[3];
#pragma unroll
  for (int w = 1; w < NW; ++w) {
    rb.blk_a1 = min(rb.blk_a1, red[w * 4 + 0]); rb.blk_b1 = max(rb.blk_b1, red[w * 4 + 1]);
    rb.blk_a2 = min(rb.blk_a2, red[w * 4 + 2]); rb.blk_b2 = max(rb.blk_b2, red[w * 4 + 3]);
  }
  rb.blk_a1 = uni(rb.blk_a1); rb.blk_b1 = uni(rb.blk_b1);
  rb.blk_a2 = uni(rb.blk_a2); rb.blk_b2 = uni(rb.blk_b2);
}

// Passes a score block through an empty volatile asm statement.  Placed inside the branch that
// masks a tile it keeps the compiler from turning that branch into selects which every tile, masked
// or not, would then execute (96 vector instructions per tile): volatile asm is never speculated.
__device__ __forceinline__ void pin_block(f32x16& a) {
  asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
  asm volatile("" : "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
}

// ---------------------------------------------------------------- forward
// One workgroup = 4 waves = 4 * 32 * NSB query rows of one head (NSB = 2: a wave owns two 32-row
// sub-blocks and every K / V^T fragment read from LDS feeds two MFMAs; the kernels run NSB = 1).
// Wave priorities (s_setprio) per phase, (matrix phase, vector phase) per kernel; equal values = no changes.
// Forward: the wave that is in its soft-max gets the higher priority.  Its vector instructions are short and
// slot in between the MFMAs of the other wave, which needs one issue slot per 32 cycles; the other way
// round (matrix phase first) the vector wave waits behind MFMAs that are themselves waiting for the pipe
// (measured at the Llama-3.1-8B shape: 825 TFLOP/s with the matrix phase first, 826 without priorities, 880
// with the vector phase first).  The dQ and dK/dV kernels measure best with the matrix phase first.
#define SPX_FWD_PRIO 0, 3
#define SPX_DQ_PRIO 3, 0
#define SPX_DKV_PRIO 3, 0
constexpr int prio_first(int a, int) { return a; }
constexpr int prio_second(int, int b) { return b; }
template <int M, int V>
struct PrioPair {
  static __device__ __forceinline__ void matrix() { if constexpr (M != V) __builtin_amdgcn_s_setprio(M); }
  static __device__ __forceinline__ void vector() { if constexpr (M != V) __builtin_amdgcn_s_setprio(V); }
};
#define SPX_FWD_PRIO_MFMA() PrioPair<prio_first(SPX_FWD_PRIO), prio_second(SPX_FWD_PRIO)>::matrix()
#define SPX_FWD_PRIO_VALU() PrioPair<prio_first(SPX_FWD_PRIO), prio_second(SPX_FWD_PRIO)>::vector()
#define SPX_DQ_PRIO_MFMA() PrioPair<prio_first(SPX_DQ_PRIO), prio_second(SPX_DQ_PRIO)>::matrix()
#define SPX_DQ_PRIO_VALU() PrioPair<prio_first(SPX_DQ_PRIO), prio_second(SPX_DQ_PRIO)>::vector()
#define SPX_DKV_PRIO_MFMA() PrioPair<prio_first(SPX_DKV_PRIO), prio_second(SPX_DKV_PRIO)>::matrix()
#define SPX_DKV_PRIO_VALU() PrioPair<prio_first(SPX_DKV_PRIO), prio_second(SPX_DKV_PRIO)>::vector()
#define SPX_DKV_REMAT 1
#define SPX_FWD_MINB 2
#define SPX_DQ_MINB 2
#define SPX_DKV_MINB 1
// How the forward kernel brings a key tile into LDS: through registers at the point of use (0),
// through registers one tile ahead (1), or with global -> LDS loads into the other of two tile
// buffers (2).  A 16-byte LDS write from registers holds the LDS pipe twice as long as a 16-byte
// read, and these kernels keep that pipe busy all the time: mode 2 takes the writes off it.
template <int D, int NW, int PF>
struct FwdSmem {
  static constexpr int KS = D + kKPad, VS = kBN + kVPad;
  static constexpr int kTileK = kBN * D * 2, kTileV = D * kBN * 2;  // mode 2: unpadded, swizzled
  static constexpr int kBuf = kTileK + kTileV;
  static constexpr int kTiles = PF == 2 ? 2 * kBuf : (kBN * KS + D * VS) * 2;
  static constexpr int kBytes = kTiles + 4 * NW * (int)sizeof(int);
};

// operand fragments in flight per product (registers: 4 per fragment): the LDS pipe delivers
// well over 150 B/clk per CU, what a wave waits for is the latency of its own reads
#define SPX_FWD_RING 8
template <int D, int NSB, int NW, int PF>
__global__ __launch_bounds__(64 * NW, D > 128 ? 1 : SPX_FWD_MINB) void attn_fwd_kernel(AttnParams p,
                                                                const uint16_t* __restrict__ Vt,
                                                                uint16_t* __restrict__ O,
                                                                float* __restrict__ LSE) {
  using SM = FwdSmem<D, NW, PF>;
  constexpr int KS = SM::KS;
  constexpr int VS = SM::VS;
  constexpr int NKK = D / 16;
  constexpr int NDB = D / 32;
  constexpr int NT = 64 * NW;
  constexpr int CPT = (kBN * D / 8) / NT;
  constexpr int BMW = 32 * NSB;
  constexpr int BM = NW * BMW;

  extern __shared__ __attribute__((aligned(16))) uint8_t fwd_smem[];
  uint16_t* const Ks = reinterpret_cast<uint16_t*>(fwd_smem);
  uint16_t* const Vs = Ks + kBN * KS;
  int* const red = reinterpret_cast<int*>(fwd_smem + SM::kTiles);

  const int group = p.Hq / p.Hkv;
  const int L = blockIdx.x;
  const int kvh = L % p.Hkv;
  const int rest = L / p.Hkv;
  const int h = kvh * group + rest % group;
  const int n_qb = (p.NQ + BM - 1) / BM;
  const int qb = n_qb - 1 - rest / group;  // late (heavy, under a causal mask) blocks first
  const int m0 = qb * BM;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: what derives from it is scalar too
  const int g = lane >> 5, col = lane & 31;
  int i[NSB], ic[NSB];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    i[sb] = m0 + wave * BMW + sb * 32 + col;
    ic[sb] = i[sb] < p.NQ ? i[sb] : p.NQ - 1;
  }
  RowBounds<NSB> rb;
  load_bounds<NSB, NW>(p, ic, wave, lane, red, rb);

  // The query fragments carry the soft-max scale and log2(e): the scores then come out of the
  // MFMA in the base-2 exponent domain and need no multiply of their own.
  bf16x8 qf[NSB][NKK];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    const uint16_t* qrow = p.Q + (int64_t)h * p.q_hs + (int64_t)ic[sb] * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk)
      qf[sb][kk] = as_bf16x8(scale_bf16x8(*reinterpret_cast<const u32x4*>(qrow + kk * 16), p.scale_log2e));
  }
  // Soft-max bookkeeping per query (a lane owns one query; its partner lane ^ 32 the same one):
  //   m_ref  the value subtracted from the scores before the exp2.  It is NOT the running maximum:
  //          it only moves when a tile's largest score exceeds it by more than kRefSlack (or when
  //          the row sees its first key), so most tiles skip the rescaling pass altogether.  A
  //          common factor 2^k on a row's probabilities is exact in binary floating point and
  //          cancels in O / l; the slack only has to keep 2^(s - m_ref) far from overflow.
  //   nref   -m_ref in all sixteen accumulator slots: the C operand of the first score MFMA, so
  //          the subtraction costs no instruction.
  //   l_run  this LANE's part of the row sum (its 32 of a tile's 64 keys); the halves are added
  //          once, after the last tile.
  constexpr float kRefSlack = 12.f;
  f32x16 acc[NSB][NDB], nref[NSB];
  float m_ref[NSB], l_run[NSB];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    m_ref[sb] = -INFINITY; l_run[sb] = 0.f;  // -inf: the row has not seen a key yet
#pragma unroll
    for (int r = 0; r < 16; ++r) nref[sb][r] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[sb][db][r] = 0.f;
  }

  const uint16_t* Kh = p.K + (int64_t)kvh * p.k_hs;
  const uint16_t* Vth = Vt + (int64_t)kvh * D * p.NKVp;
  const int last_row = p.NKV - 1;

  u32x4 kreg[CPT], vreg[CPT];
  auto fetch = [&](int n0) {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + NT * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      const int kr = min(n0 + krow, last_row);
      kreg[n] = *reinterpret_cast<const u32x4*>(Kh + (int64_t)kr * D + kcol);
      const int vd = c >> 3, vcol = (c & 7) * 8;
      vreg[n] = *reinterpret_cast<const u32x4*>(Vth + (int64_t)vd * p.NKVp + n0 + vcol);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + NT * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      *reinterpret_cast<u32x4*>(&Ks[krow * KS + kcol]) = kreg[n];
      const int vd = c >> 3, vcol = (c & 7) * 8;
      *reinterpret_cast<u32x4*>(&Vs[vd * VS + vcol]) = vreg[n];
    }
  };

  auto direct = [&](int n0) {  // global -> LDS without holding the tile in registers
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + NT * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      const int kr = min(n0 + krow, last_row);
      *reinterpret_cast<u32x4*>(&Ks[krow * KS + kcol]) =
          *reinterpret_cast<const u32x4*>(Kh + (int64_t)kr * D + kcol);
      const int vd = c >> 3, vcol = (c & 7) * 8;
      const u32x4 t = *reinterpret_cast<const u32x4*>(Vth + (int64_t)vd * p.NKVp + n0 + vcol);
      *reinterpret_cast<u32x4*>(&Vs[vd * VS + vcol]) = t;
    }
  };

  // ---- mode 2: tiles as 1 KB wave loads global -> LDS.  K tile: rows of D * 2 bytes, V^T tile: rows
  // of 128 bytes; the 16-byte chunk c of row r lives in slot c ^ swz(r), which makes the fragment
  // reads (32 lanes = 32 rows, one logical chunk) conflict free without padding.
  constexpr int RBK = D * 2, CKK = RBK / 16;             // bytes and chunks per K row
  constexpr int LPK = (kBN * RBK / 1024) / NW;           // wave loads per wave: K tile
  constexpr int LPV = (D * 128 / 1024) / NW;             // V^T tile
  auto swz_k = [](int r) { return CKK == 8 ? (r >> 1) & 7 : r & 15; };
  auto swz_v = [](int r) { return (r >> 1) & 7; };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)fwd_smem;
  u32x4 kres, vres;
  int k_row[PF == 2 ? LPK : 1], k_col[PF == 2 ? LPK : 1], v_off[PF == 2 ? LPV : 1];
  if constexpr (PF == 2) {
    kres = make_rsrc(Kh, (uint32_t)((int64_t)p.NKV * RBK));
    vres = make_rsrc(Vth, (uint32_t)((int64_t)D * p.NKVp * 2));
#pragma unroll
    for (int j = 0; j < LPK; ++j) {
      const int r = (wave * LPK + j) * (1024 / RBK) + lane / CKK;
      k_row[j] = r;
      k_col[j] = ((lane % CKK) ^ swz_k(r)) * 16;
    }
#pragma unroll
    for (int j = 0; j < LPV; ++j) {
      const int r = (wave * LPV + j) * 8 + lane / 8;
      v_off[j] = r * p.NKVp * 2 + ((lane & 7) ^ swz_v(r)) * 16;
    }
  }
  auto issue = [&](int n0, int buf) __attribute__((always_inline)) {
    if constexpr (PF == 2) {
      const uint32_t kb = lds0 + buf * SM::kBuf + wave * LPK * 1024;
      if (n0 + kBN <= p.NKV) {
        // every row of the tile exists: the lane's offset inside a tile is loop invariant, the tile's
        // first row goes into the scalar offset (no vector arithmetic per load)
#pragma unroll
        for (int j = 0; j < LPK; ++j) load_to_lds16<0>(kres, kb + j * 1024, k_row[j] * RBK + k_col[j], n0 * RBK);
      } else {
        // the last, ragged tile: rows past the end repeat the last one (they are masked out)
#pragma unroll
        for (int j = 0; j < LPK; ++j)
          load_to_lds16<0>(kres, kb + j * 1024, min(n0 + k_row[j], last_row) * RBK + k_col[j], 0);
      }
      const uint32_t vb = lds0 + buf * SM::kBuf + SM::kTileK + wave * LPV * 1024;
#pragma unroll
      for (int j = 0; j < LPV; ++j) load_to_lds16<0>(vres, vb + j * 1024, v_off[j], n0 * 2);
    }
  };
  // fragment reads of mode 2: byte offsets of this lane's row and chunk (step 0) inside a tile
  const int rdk = col * RBK + ((g ^ swz_k(col)) * 16);
  const int rdv = col * 128 + ((g ^ swz_v(col)) * 16);
  // The fragment reads as LDS addresses, one register per swizzle term, kept opaque to the
  // compiler: what is added to them per read (buffer, key half, D block) is a constant and goes
  // into the offset field.  Formed on the symbol of the dynamic array instead, every read costs a
  // vector add of that link-time constant.
  // Only where both tile buffers lie inside the 64 KB an offset field reaches (head_dim <= 128); past
  // that the constants need an add again and the registers are better left to the accumulators.
  constexpr bool kAbsRd = PF == 2 && 2 * SM::kBuf <= 65536;
  uint32_t krd[kAbsRd ? NKK : 1], vrd[kAbsRd ? 4 : 1];
  if constexpr (kAbsRd) {
#pragma unroll
    for (int j = 0; j < NKK; ++j) {
      krd[j] = lds0 + (uint32_t)(rdk ^ (j * 32));
      asm volatile("" : "+v"(krd[j]));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      vrd[j] = lds0 + (uint32_t)(SM::kTileK + (rdv ^ (j * 32)));
      asm volatile("" : "+v"(vrd[j]));
    }
  }

  // one pass over the key tiles of one interval class.  The tile loop is unrolled over the two tile
  // buffers: the buffer is then a compile-time constant and the fragment reads address it through
  // the immediate offset of ds_read (no vector add per read).
  auto run_pass = [&](const int (&aa)[NSB], const int (&bb)[NSB], int w_amin, int w_amax,
                      int w_bmin, int w_bmax, int blk_a, int blk_b) {
    if (blk_b <= blk_a) return;
    const int n_begin = (blk_a / kBN) * kBN;
    if (PF == 1) fetch(n_begin);
    if constexpr (PF == 2) {
      __syncthreads();  // a previous pass may still be reading either buffer
      issue(n_begin, 0);
    }
    auto tile = [&](int n0, auto buf_c) __attribute__((always_inline)) {
      constexpr int buf = decltype(buf_c)::value;
      if constexpr (PF == 2) {
        // this wave's loads of tile n0 have landed; after the barrier everybody's have, and nobody
        // reads the other buffer any more: the next tile goes there
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (n0 + kBN < blk_b) issue(n0 + kBN, buf ^ 1);
      } else {
        __syncthreads();
        if (PF) stash(); else direct(n0);
        __syncthreads();
        if (PF && n0 + kBN < blk_b) fetch(n0 + kBN);
      }
      const uint8_t* const tk = fwd_smem + buf * SM::kBuf;
      const uint8_t* const tv = tk + SM::kTileK;
      if (n0 >= w_bmax || n0 + kBN <= w_amin) return;  // nothing visible for this wave

      f32x16 st[NSB][2];
      SPX_FWD_PRIO_MFMA();
      // K fragments go through a ring of four registers: the read of fragment f + 4 is
      // issued right after the MFMA of fragment f, so no MFMA waits for LDS; the two
      // 32-key halves alternate so that consecutive MFMAs use different accumulators
      {
        constexpr int NF = 2 * NKK;
        constexpr int RG = SPX_FWD_RING;
        bf16x8 kfr[RG];
        auto kread = [&](int f) {
          if constexpr (kAbsRd)
            kfr[f % RG] = as_bf16x8(lds_read128(krd[f >> 1] + buf * SM::kBuf + (f & 1) * 32 * RBK));
          else if constexpr (PF == 2)
            kfr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                tk + (f & 1) * 32 * RBK + (rdk ^ ((f >> 1) * 32))));
          else
            kfr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                &Ks[((f & 1) * 32 + col) * KS + g * 8 + (f >> 1) * 16]));
        };
#pragma unroll
        for (int f = 0; f < RG; ++f) kread(f);
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
            st[sb][f & 1] = mfma32(kfr[f % RG], qf[sb][f >> 1], f < 2 ? nref[sb] : st[sb][f & 1]);
          __builtin_amdgcn_sched_barrier(0);
          if (f + RG < NF) kread(f + RG);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      SPX_FWD_PRIO_VALU();
      const bool need_mask = (n0 < w_amax) || (n0 + kBN > w_bmin);
      int m_lo[NSB], m_hi[NSB];
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) { m_lo[sb] = aa[sb] - n0 - 4 * g; m_hi[sb] = bb[sb] - n0 - 4 * g; }
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        // running max on the raw scores; the soft-max scale is folded into the exp2 argument
        if (need_mask) {
          // a real (scalar) branch: the asm statement keeps the compiler from turning the
          // masking into selects that every tile would pay for
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) {
            pin_block(st[sb][kb]);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              // key index = n0 + 4 g + (compile-time part): compare the constant part
              const int cr = kb * 32 + 8 * (r >> 2) + (r & 3);
              if (cr < m_lo[sb] || cr >= m_hi[sb]) st[sb][kb][r] = -INFINITY;
            }
            pin_block(st[sb][kb]);
          }
        }
        // st holds s - m_ref.  Largest of the 32 scores of this lane (three-operand maxima)
        float mx = fmaxf(st[sb][0][0], st[sb][1][0]);
#pragma unroll
        for (int r = 1; r < 16; r += 2) {
          mx = fmaxf(fmaxf(mx, st[sb][0][r]), st[sb][0][r + 1 < 16 ? r + 1 : r]);
          mx = fmaxf(fmaxf(mx, st[sb][1][r]), st[sb][1][r + 1 < 16 ? r + 1 : r]);
        }
        mx = half_swap_max(mx);
        const bool unset = m_ref[sb] == -INFINITY;
        const bool move = mx > -INFINITY && (unset || mx > kRefSlack);
        if (__any(move)) {
          // some row's reference moves: shift its scores, rescale its sum and its accumulator
          asm volatile("; reference moves");
          const float delta = move ? mx : 0.f;
          const float alpha = (move && !unset) ? fast_exp2(-delta) : 1.f;  // unset rows hold zeros
          m_ref[sb] = move ? (unset ? mx : m_ref[sb] + mx) : m_ref[sb];
          const float nr = unset && !move ? 0.f : -m_ref[sb];
#pragma unroll
          for (int r = 0; r < 16; ++r) nref[sb][r] = nr;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) st[sb][kb][r] -= delta;
          l_run[sb] *= alpha;
#pragma unroll
          for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[sb][db][r] *= alpha;
        }
        float rs0 = 0.f, rs1 = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p0 = fast_exp2(st[sb][0][r]), p1 = fast_exp2(st[sb][1][r]);
          st[sb][0][r] = p0; st[sb][1][r] = p1;
          rs0 += p0; rs1 += p1;
        }
        l_run[sb] += rs0 + rs1;
      }
      SPX_FWD_PRIO_MFMA();
      {
        // V^T fragments through the same kind of ring; fragment f = (16-key step s, D block db)
        constexpr int NF = 4 * NDB;
        constexpr int RG = SPX_FWD_RING;
        bf16x8 vfr[RG];
        auto vread = [&](int f) {
          if constexpr (kAbsRd)
            vfr[f % RG] = as_bf16x8(lds_read128(vrd[f / NDB] + buf * SM::kBuf + (f % NDB) * 32 * 128));
          else if constexpr (PF == 2)
            vfr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                tv + (f % NDB) * 32 * 128 + (rdv ^ ((f / NDB) * 32))));
          else
            vfr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                &Vs[((f % NDB) * 32 + col) * VS + (f / NDB) * 16 + 8 * g]));
        };
#pragma unroll
        for (int f = 0; f < RG; ++f) vread(f);
        bf16x8 pb[NSB];
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          const int s = f / NDB, db = f % NDB;
          if (db == 0) {
#pragma unroll
            for (int sb = 0; sb < NSB; ++sb) pb[sb] = pack8(st[sb][s >> 1], (s & 1) * 8);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb) acc[sb][db] = mfma32(vfr[f % RG], pb[sb], acc[sb][db]);
          __builtin_amdgcn_sched_barrier(0);
          if (f + RG < NF) vread(f + RG);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      SPX_FWD_PRIO_VALU();
    };
    for (int n0 = n_begin; n0 < blk_b; n0 += 2 * kBN) {
      tile(n0, std::integral_constant<int, 0>{});
      if (n0 + kBN < blk_b) tile(n0 + kBN, std::integral_constant<int, 1>{});
    }
  };

  run_pass(rb.a1, rb.b1, rb.w_a1min, rb.w_a1max, rb.w_b1min, rb.w_b1max, rb.blk_a1, rb.blk_b1);
  if (p.a2)
    run_pass(rb.a2, rb.b2, rb.w_a2min, rb.w_a2max, rb.w_b2min, rb.w_b2max, rb.blk_a2, rb.blk_b2);

  // from here on l_run is the whole row's sum in both lanes of a query
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) l_run[sb] = half_swap_sum(l_run[sb]);
  float (&m_run)[NSB] = m_ref;

  // TTT diagonal keys (j, r), j = 1..n_extra: one dot product each.  The key / value rows of a
  // wave's 32 queries are 32 CONSECUTIVE rows of step j: they come in as whole 1 KB wave loads
  // global -> LDS (a lane reading its own row from global memory touches 32 lines per instruction)
  // into this wave's quarter of the tile buffers, chunk c of row r in slot c ^ (r mod chunks), and
  // each lane then picks its row's pieces from LDS.  The loads of step j + 1 are issued as soon
  // as step j's rows have been read.
  if (p.n_extra > 0) {
    static_assert(NSB == 1, "one 32-row block per wave");
    constexpr int XCK = RBK / 16;                  // 16-byte chunks per row
    constexpr int XRL = 1024 / RBK;                // rows per 1 KB wave load
    constexpr int XNL = 32 / XRL;                  // wave loads per 32 rows
    static_assert(SM::kTiles / NW >= 2 * 32 * RBK, "a wave's share of the tile buffers holds K and V rows");
    __syncthreads();  // every wave is done with the tile buffers
    const uint32_t xk = lds0 + wave * (2 * 32 * RBK), xv = xk + 32 * RBK;
    const int64_t kv_bytes = (int64_t)(p.n_extra + 1) * p.T * RBK;
    const u32x4 xkres = make_rsrc(p.K + (int64_t)kvh * p.k_hs, (uint32_t)kv_bytes);
    const u32x4 xvres = make_rsrc(p.V + (int64_t)kvh * p.v_hs, (uint32_t)kv_bytes);
    int goff[XNL];
#pragma unroll
    for (int n = 0; n < XNL; ++n) {
      const int r = n * XRL + lane / XCK;
      goff[n] = r * RBK + (((lane % XCK) ^ (r & (XCK - 1))) * 16);
    }
    const int row0 = __builtin_amdgcn_readfirstlane(m0 + wave * BMW);
    auto issue_x = [&](const u32x4& res, uint32_t dst, int j) __attribute__((always_inline)) {
      const int soff = __builtin_amdgcn_readfirstlane((j * p.T + row0) * RBK);
#pragma unroll
      for (int n = 0; n < XNL; ++n) load_to_lds16<0>(res, dst + n * 1024, goff[n], soff);
    };
    const uint8_t* const xkp = fwd_smem + wave * (2 * 32 * RBK);
    const uint8_t* const xvp = xkp + 32 * RBK;
    const int xrow = col * RBK, xsw = col & (XCK - 1);
    issue_x(xkres, xk, 1);
    issue_x(xvres, xv, 1);
    for (int j = 1; j <= p.n_extra; ++j) {
      // K rows of step j have landed (the V rows, issued after them, may still be in flight)
      if constexpr (XNL == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else if constexpr (XNL == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
      float dot = 0.f;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk)
        dot = dot8_bf16(qf[0][kk], *reinterpret_cast<const u32x4*>(xkp + xrow + (((2 * kk + g) ^ xsw) * 16)), dot);
      const float sj = half_swap_sum(dot);  // the query fragments carry the scale
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // V rows landed, K rows read
      if (j < p.n_extra) issue_x(xkres, xk, j + 1);
      const float m_new = fmaxf(m_run[0], sj);
      const float alpha = fast_exp2(m_run[0] - m_new);  // a row without context keys: exp2(-inf) = 0
      const float pv = fast_exp2(sj - m_new);
      l_run[0] = l_run[0] * alpha + pv;
      m_run[0] = m_new;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          float vv[4];
          unpack4(*reinterpret_cast<const u32x2*>(xvp + xrow + (((db * 4 + r4) ^ xsw) * 16) + 8 * g), vv);
#pragma unroll
          for (int t = 0; t < 4; ++t)
            acc[0][db][r4 * 4 + t] = fmaf(pv, vv[t], acc[0][db][r4 * 4 + t] * alpha);
        }
      if (j < p.n_extra) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // V rows read
        issue_x(xvres, xv, j + 1);
      }
    }
  }

#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    if (i[sb] >= p.NQ) continue;
    const float inv = l_run[sb] > 0.f ? 1.f / l_run[sb] : 0.f;
    uint16_t* orow = O + ((int64_t)i[sb] * p.Hq + h) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2 w;
        w.x = pack_bf16x2(acc[sb][db][r4 * 4 + 0] * inv, acc[sb][db][r4 * 4 + 1] * inv);
        w.y = pack_bf16x2(acc[sb][db][r4 * 4 + 2] * inv, acc[sb][db][r4 * 4 + 3] * inv);
        *reinterpret_cast<u32x2*>(orow + db * 32 + 8 * r4) = w;
      }
    // a row that sees no key at all (cannot happen for the two masks built here) gets lse = 0
    if (g == 0) LSE[(int64_t)h * p.NQ + i[sb]] = l_run[sb] > 0.f ? m_run[sb] + fast_log2(l_run[sb]) : 0.f;
  }
}

// ---------------------------------------------------------------- backward
// delta[h, i] = sum_d dO[i, h, d] * O[i, h, d]
// sum over each row of sixteen lanes, left in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
  // quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror: afterwards every lane
  // of a 16-lane row holds the sum over the row
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));
  return v;
}

// EPL (4, 8 or 16) consecutive bf16 of one lane in 8- or 16-byte accesses
template <int EPL>
__device__ __forceinline__ void ld_bf16s(const uint16_t* p, float (&v)[EPL]) {
  if constexpr (EPL == 4) {
    const u32x2 u = *reinterpret_cast<const u32x2*>(p);
    v[0] = bf16_lo(u.x); v[1] = bf16_hi(u.x); v[2] = bf16_lo(u.y); v[3] = bf16_hi(u.y);
  } else {
    static_assert(EPL % 8 == 0, "4, 8 or 16 elements per lane");
#pragma unroll
    for (int c = 0; c < EPL / 8; ++c) {
      const u32x4 u = *reinterpret_cast<const u32x4*>(p + 8 * c);
      v[8 * c + 0] = bf16_lo(u.x); v[8 * c + 1] = bf16_hi(u.x);
      v[8 * c + 2] = bf16_lo(u.y); v[8 * c + 3] = bf16_hi(u.y);
      v[8 * c + 4] = bf16_lo(u.z); v[8 * c + 5] = bf16_hi(u.z);
      v[8 * c + 6] = bf16_lo(u.w); v[8 * c + 7] = bf16_hi(u.w);
    }
  }
}
template <int EPL>
__device__ __forceinline__ void st_bf16s(uint16_t* p, const float (&v)[EPL]) {
  if constexpr (EPL == 4) {
    u32x2 u;
    u.x = pack_bf16x2(v[0], v[1]); u.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<u32x2*>(p) = u;
  } else {
#pragma unroll
    for (int c = 0; c < EPL / 8; ++c) {
      u32x4 u;
      u.x = pack_bf16x2(v[8 * c + 0], v[8 * c + 1]); u.y = pack_bf16x2(v[8 * c + 2], v[8 * c + 3]);
      u.z = pack_bf16x2(v[8 * c + 4], v[8 * c + 5]); u.w = pack_bf16x2(v[8 * c + 6], v[8 * c + 7]);
      *reinterpret_cast<u32x4*>(p + 8 * c) = u;
    }
  }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float* __restrict__ x, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = 0.f;
}

template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const uint16_t* __restrict__ O,
                                                         const uint16_t* __restrict__ dO, int NQ,
                                                         int Hq, float* __restrict__ delta,
                                                         const float* __restrict__ lse, int NQp,
                                                         float* __restrict__ neg) {
  // sixteen lanes per (row, head): D / 16 consecutive elements each, summed with DPP moves
  constexpr int EPL = D / 16;
  const int64_t n_rows = (int64_t)NQ * Hq;
  const int64_t raw = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + ((threadIdx.x & 63) >> 4);
  const int64_t row = raw < n_rows ? raw : n_rows - 1;  // = i * Hq + h
  const int d0 = (threadIdx.x & 15) * EPL;
  float a[EPL], b[EPL];
  ld_bf16s<EPL>(O + row * D + d0, a);
  ld_bf16s<EPL>(dO + row * D + d0, b);
  float acc = 0.f;
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc = fmaf(a[e], b[e], acc);
  acc = row16_sum(acc);
  if ((threadIdx.x & 15) == 0 && raw < n_rows) {
    const int64_t hh = row % Hq, i = row / Hq;
    delta[hh * NQ + i] = acc;
    // -lse and -delta in rows of NQp (the padding stays zero: see the launcher), the C operands of the
    // wave-specialised dK/dV kernel's score products
    neg[hh * NQp + i] = -lse[hh * NQ + i];
    neg[((int64_t)Hq + hh) * NQp + i] = -acc;
  }
}

// dQ: same tiling as the forward.
//   P^T = exp2(S'^T - lse), dP^T = V dO^T, dS^T = P^T (dP^T - delta), dQ^T += K^T dS^T
// PF: how a key tile reaches LDS: 0 through registers at the point of use, 1 through registers one tile
// ahead, 3 global -> LDS directly into the other of two buffers, with tiles of 32 instead of 64 keys so
// that two buffers of the three tiles (K, V, K^T) fit beside a second workgroup (see FwdSmem).
// Four 16-bit values per lane from LDS, transposed inside every group of 16 lanes: lane 4u + w of
// a group receives, as element j, element w of the 8 bytes that lane 4j + u of the group points at.
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ i16x4 lds_read_tr16(const uint8_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) i16x4*)(uintptr_t)(uint32_t)(uintptr_t)(
          (__attribute__((address_space(3))) const uint8_t*)p));
}

template <int D, int NW, int PF>
struct DqSmem {
  // mode 4: only the row-major K and V tiles, 64 keys each; the K^T fragments of the dQ product come
  // out of the K tile through transposing LDS reads
  static constexpr int TB = PF == 3 ? 32 : (PF == 4 ? 64 : kBN);     // keys per tile
  static constexpr int KS = D + kKPad, VS = kBN + kVPad;
  static constexpr int kTileK = TB * D * 2, kTileT = PF == 4 ? 0 : D * TB * 2;  // modes 3, 4: unpadded, swizzled
  static constexpr int kBuf = 2 * kTileK + kTileT;
  static constexpr int kDiag = NW * 2 * 32 * D * 2;  // K and V rows of 32 queries per wave (TTT diagonal keys)
  static constexpr int kTiles0 = PF >= 3 ? 2 * kBuf : (2 * kBN * KS + D * VS) * 2;
  static constexpr int kTiles = kTiles0 > kDiag ? kTiles0 : kDiag;
  static constexpr int kBytes = kTiles + 4 * NW * (int)sizeof(int);
};

template <int D, int NSB, int NW, int PF>
__global__ __launch_bounds__(64 * NW, D > 128 ? 1 : SPX_DQ_MINB) void attn_bwd_dq_kernel(
    AttnParams p, const uint16_t* __restrict__ dO, const uint16_t* __restrict__ Kt,
    const float* __restrict__ LSE, const float* __restrict__ Delta, uint16_t* __restrict__ dQ,
    int64_t dq_hs) {
  using SM = DqSmem<D, NW, PF>;
  constexpr bool kDma = PF >= 3;
  constexpr bool kTR = PF == 4;
  constexpr int TB = SM::TB;
  constexpr int KS = SM::KS;
  constexpr int VS = SM::VS;
  constexpr int NKK = D / 16;
  constexpr int NDB = D / 32;
  constexpr int NT = 64 * NW;
  constexpr int CPT = (kBN * D / 8) / NT;
  constexpr int BMW = 32 * NSB;
  constexpr int BM = NW * BMW;

  extern __shared__ __attribute__((aligned(16))) uint8_t dq_smem[];
  uint16_t* const Ks = reinterpret_cast<uint16_t*>(dq_smem);
  uint16_t* const Vn = Ks + kBN * KS;
  uint16_t* const Kts = Vn + kBN * KS;
  int* const red = reinterpret_cast<int*>(dq_smem + SM::kTiles);

  const int group = p.Hq / p.Hkv;
  const int L = blockIdx.x;
  const int kvh = L % p.Hkv;
  const int rest = L / p.Hkv;
  const int h = kvh * group + rest % group;
  const int n_qb = (p.NQ + BM - 1) / BM;
  const int qb = n_qb - 1 - rest / group;
  const int m0 = qb * BM;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, col = lane & 31;
  int i[NSB], ic[NSB];
  float lse_i[NSB], delta_i[NSB];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    i[sb] = m0 + wave * BMW + sb * 32 + col;
    ic[sb] = i[sb] < p.NQ ? i[sb] : p.NQ - 1;
    lse_i[sb] = LSE[(int64_t)h * p.NQ + ic[sb]];
    delta_i[sb] = Delta[(int64_t)h * p.NQ + ic[sb]];
  }
  RowBounds<NSB> rb;
  load_bounds<NSB, NW>(p, ic, wave, lane, red, rb);

  // the query fragments carry scale * log2(e) (see scale_bf16x8); -lse and -delta of the lane's
  // query sit in all sixteen slots of two blocks that the first MFMA of each product takes as its
  // C operand, so s - lse and dP - delta come out of the matrix pipe
  bf16x8 qf[NSB][NKK], dof[NSB][NKK];
  f32x16 nlse[NSB], ndel[NSB];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    const uint16_t* qrow = p.Q + (int64_t)h * p.q_hs + (int64_t)ic[sb] * D + g * 8;
    const uint16_t* drow = dO + ((int64_t)ic[sb] * p.Hq + h) * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      qf[sb][kk] = as_bf16x8(scale_bf16x8(*reinterpret_cast<const u32x4*>(qrow + kk * 16), p.scale_log2e));
      dof[sb][kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(drow + kk * 16));
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) { nlse[sb][r] = -lse_i[sb]; ndel[sb][r] = -delta_i[sb]; }
  }
  f32x16 acc[NSB][NDB];
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[sb][db][r] = 0.f;

  const uint16_t* Kh = p.K + (int64_t)kvh * p.k_hs;
  const uint16_t* Vh = p.V + (int64_t)kvh * p.v_hs;
  const uint16_t* Kth = Kt + (int64_t)kvh * D * p.NKVp;
  const int last_row = p.NKV - 1;

  u32x4 kreg[CPT], vreg[CPT], treg[CPT];
  auto fetch = [&](int n0) {
    // offsets recomputed per tile on purpose (see the dK/dV kernel): kept live through the loop they spill
    // at head_dim 256, and a spill reload waits for the prefetch issued here
    int tid_v = tid;
    if (SPX_DKV_REMAT) asm volatile("" : "+v"(tid_v));
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid_v + NT * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      const int kr = min(n0 + krow, last_row);
      kreg[n] = *reinterpret_cast<const u32x4*>(Kh + (int64_t)kr * D + kcol);
      vreg[n] = *reinterpret_cast<const u32x4*>(Vh + (int64_t)kr * D + kcol);
      const int vd = c >> 3, vcol = (c & 7) * 8;
      treg[n] = *reinterpret_cast<const u32x4*>(Kth + (int64_t)vd * p.NKVp + n0 + vcol);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + NT * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      *reinterpret_cast<u32x4*>(&Ks[krow * KS + kcol]) = kreg[n];
      *reinterpret_cast<u32x4*>(&Vn[krow * KS + kcol]) = vreg[n];
      const int vd = c >> 3, vcol = (c & 7) * 8;
      *reinterpret_cast<u32x4*>(&Kts[vd * VS + vcol]) = treg[n];
    }
  };

  auto direct = [&](int n0) {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + NT * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      const int kr = min(n0 + krow, last_row);
      *reinterpret_cast<u32x4*>(&Ks[krow * KS + kcol]) =
          *reinterpret_cast<const u32x4*>(Kh + (int64_t)kr * D + kcol);
      *reinterpret_cast<u32x4*>(&Vn[krow * KS + kcol]) =
          *reinterpret_cast<const u32x4*>(Vh + (int64_t)kr * D + kcol);
      const int vd = c >> 3, vcol = (c & 7) * 8;
      const u32x4 t = *reinterpret_cast<const u32x4*>(Kth + (int64_t)vd * p.NKVp + n0 + vcol);
      *reinterpret_cast<u32x4*>(&Kts[vd * VS + vcol]) = t;
    }
  };

  // ---- mode 3: the three tiles as 1 KB wave loads global -> LDS (chunk c of row r in slot c ^ swz(r))
  constexpr int RBK = D * 2, CKK = RBK / 16;   // bytes / 16-byte chunks per row of K and V
  constexpr int RBT = TB * 2, CKT = RBT / 16;  // ... of K^T
  constexpr int LPK = (TB * RBK / 1024) / NW, LPT = (D * RBT / 1024) / NW;
  auto swz_k = [](int r) {
    // (transposing reads touch 4 + 4 rows x 64 bytes: those rows must fall into different 64-byte bank groups)
    if (kTR) return CKK == 8 ? ((r & 4) | ((r >> 2) & 2) | ((r >> 1) & 1)) : ((r & 3) << 2) | ((r >> 2) & 3);
    return CKK == 8 ? (r >> 1) & 7 : r & 15;
  };
  auto swz_t = [](int r) { return CKT == 8 ? (r >> 1) & 7 : (r >> 2) & 3; };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)dq_smem;
  u32x4 kres, vres, tres;
  if constexpr (kDma) {
    static_assert(!kDma || (LPK >= 1 && LPT >= 1), "a tile is at least one 1 KB load per wave");
    kres = make_rsrc(Kh, (uint32_t)((int64_t)p.NKV * RBK));
    vres = make_rsrc(Vh, (uint32_t)((int64_t)p.NKV * RBK));
    tres = make_rsrc(Kth, (uint32_t)((int64_t)D * p.NKVp * 2));
  }
  auto issue = [&](int n0, int b) __attribute__((always_inline)) {
    if constexpr (kDma) {
      int lane_v = lane;
      if (SPX_DKV_REMAT) asm volatile("" : "+v"(lane_v));  // offsets recomputed per tile, not kept live
      const uint32_t kb0 = lds0 + b * SM::kBuf + wave * LPK * 1024;
#pragma unroll
      for (int j = 0; j < LPK; ++j) {
        const int r = (wave * LPK + j) * (1024 / RBK) + lane_v / CKK;
        const int off = min(n0 + r, last_row) * RBK + ((lane_v % CKK) ^ swz_k(r)) * 16;
        load_to_lds16<0>(kres, kb0 + j * 1024, off, 0);
        load_to_lds16<0>(vres, kb0 + SM::kTileK + j * 1024, off, 0);
      }
      const uint32_t tb0 = lds0 + b * SM::kBuf + 2 * SM::kTileK + wave * LPT * 1024;
#pragma unroll
      for (int j = 0; j < (kTR ? 0 : LPT); ++j) {
        const int r = (wave * LPT + j) * (1024 / RBT) + lane_v / CKT;
        load_to_lds16<0>(tres, tb0 + j * 1024, r * p.NKVp * 2 + ((lane_v % CKT) ^ swz_t(r)) * 16, n0 * 2);
      }
    }
  };
  const int rdk = col * RBK + ((g ^ swz_k(col)) * 16);
  const int rdt = col * RBT + ((g ^ swz_t(col)) * 16);
  // transposing reads (see the dK/dV kernel): rows 4 (G >> 1) + (s >> 2) (+ 8) of a 16-key step
  const int tG = lane >> 4, ts = lane & 15;
  const int trow = 4 * (tG >> 1) + (ts >> 2);
  const int tcl = 2 * (tG & 1) + ((ts & 3) >> 1);
  const int rt0 = trow * RBK + ((tcl ^ swz_k(trow)) * 16) + (ts & 1) * 8;
  const int rt1 = (trow + 8) * RBK + ((tcl ^ swz_k(trow + 8)) * 16) + (ts & 1) * 8;

  auto run_pass = [&](const int (&aa)[NSB], const int (&bb)[NSB], int w_amin, int w_amax,
                      int w_bmin, int w_bmax, int blk_a, int blk_b) {
    if (blk_b <= blk_a) return;
    const int n_begin = (blk_a / TB) * TB;
    if (PF == 1) fetch(n_begin);
    int buf = 0;
    if constexpr (kDma) {
      __syncthreads();  // a previous pass may still be reading either buffer
      issue(n_begin, 0);
    }
    for (int n0 = n_begin; n0 < blk_b; n0 += TB) {
      if constexpr (kDma) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (n0 + TB < blk_b) issue(n0 + TB, buf ^ 1);
      } else {
        __syncthreads();
        if (PF) stash(); else direct(n0);
        __syncthreads();
        if (PF && n0 + kBN < blk_b) fetch(n0 + kBN);
      }
      const uint8_t* const tile = dq_smem + buf * SM::kBuf;
      buf ^= 1;
      if (n0 >= w_bmax || n0 + TB <= w_amin) continue;

      const bool need_mask = (n0 < w_amax) || (n0 + TB > w_bmin);
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb) {
        // the 32-key halves of the tile one after the other: 32 score registers live
#pragma unroll(kTR && D > 128 ? 1 : TB / 32)
        for (int kb = 0; kb < TB / 32; ++kb) {
          f32x16 st, dp;
          // K and V fragments alternate through a ring of four registers (fragment 2 kk is
          // K, 2 kk + 1 is V): the read of fragment f + 4 follows the MFMA of fragment f
          SPX_DQ_PRIO_MFMA();
          {
            constexpr int NF = 2 * NKK;
            bf16x8 fr[4];
            auto fread = [&](int f) {
              if constexpr (kDma) {
                fr[f & 3] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                    tile + ((f & 1) ? SM::kTileK : 0) + kb * 32 * RBK + (rdk ^ ((f >> 1) * 32))));
              } else {
                const uint16_t* base = (f & 1) ? Vn : Ks;
                fr[f & 3] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                    &base[(kb * 32 + col) * KS + g * 8 + (f >> 1) * 16]));
              }
            };
#pragma unroll
            for (int f = 0; f < 4; ++f) fread(f);
#pragma unroll
            for (int f = 0; f < NF; ++f) {
              __builtin_amdgcn_sched_barrier(0);
              if (f & 1) dp = mfma32(fr[f & 3], dof[sb][f >> 1], f == 1 ? ndel[sb] : dp);
              else st = mfma32(fr[f & 3], qf[sb][f >> 1], f == 0 ? nlse[sb] : st);
              __builtin_amdgcn_sched_barrier(0);
              if (f + 4 < NF) fread(f + 4);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          SPX_DQ_PRIO_VALU();
#pragma unroll
          for (int r = 0; r < 16; ++r) st[r] = fast_exp2(st[r]);
          if (need_mask) {
            // a real (scalar) branch, see the forward kernel
            const int lo = aa[sb] - n0 - 4 * g, hi = bb[sb] - n0 - 4 * g;
            pin_block(st);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int cr = kb * 32 + 8 * (r >> 2) + (r & 3);
              if (cr < lo || cr >= hi) st[r] = 0.f;
            }
            pin_block(st);
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) dp[r] *= st[r];
          SPX_DQ_PRIO_MFMA();
          {
            // K^T fragments through the same kind of ring; fragment f = (16-key step s2, D block db)
            constexpr int NF = 2 * NDB;
            bf16x8 fr[4];
            auto fread = [&](int f) {
              if constexpr (kTR) {
                const uint8_t* base = tile + (kb * 32 + (f / NDB) * 16) * RBK;
                const i16x4 lo = lds_read_tr16(base + (rt0 ^ ((f % NDB) * 64)));
                const i16x4 hi = lds_read_tr16(base + (rt1 ^ ((f % NDB) * 64)));
                fr[f & 3] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
              } else if constexpr (kDma)
                fr[f & 3] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                    tile + 2 * SM::kTileK + (f % NDB) * 32 * RBT + (rdt ^ ((kb * 2 + f / NDB) * 32))));
              else
                fr[f & 3] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                    &Kts[((f % NDB) * 32 + col) * VS + (kb * 2 + f / NDB) * 16 + 8 * g]));
            };
#pragma unroll
            for (int f = 0; f < 4 && f < NF; ++f) fread(f);
            bf16x8 db8 = pack8(dp, 0);
#pragma unroll
            for (int f = 0; f < NF; ++f) {
              if (f == NDB) db8 = pack8(dp, 8);
              __builtin_amdgcn_sched_barrier(0);
              acc[sb][f % NDB] = mfma32(fr[f & 3], db8, acc[sb][f % NDB]);
              __builtin_amdgcn_sched_barrier(0);
              if (f + 4 < NF) fread(f + 4);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          SPX_DQ_PRIO_VALU();
        }
      }
    }
  };

  run_pass(rb.a1, rb.b1, rb.w_a1min, rb.w_a1max, rb.w_b1min, rb.w_b1max, rb.blk_a1, rb.blk_b1);
  if (p.a2)
    run_pass(rb.a2, rb.b2, rb.w_a2min, rb.w_a2max, rb.w_b2min, rb.w_b2max, rb.blk_a2, rb.blk_b2);

  // TTT diagonal keys: the key / value rows of a wave's 32 queries come in as coalesced 1 KB wave
  // loads global -> LDS into the wave's share of the tile buffers (see the forward kernel)
  if (p.n_extra > 0) {
    static_assert(NSB == 1, "one 32-row block per wave");
    constexpr int XCK = RBK / 16, XRL = 1024 / RBK, XNL = 32 / XRL;
    __syncthreads();  // every wave is done with the tile buffers
    const uint32_t xk = lds0 + wave * (2 * 32 * RBK), xv = xk + 32 * RBK;
    const int64_t kv_bytes = (int64_t)(p.n_extra + 1) * p.T * RBK;
    const u32x4 xkres = make_rsrc(Kh, (uint32_t)kv_bytes);
    const u32x4 xvres = make_rsrc(Vh, (uint32_t)kv_bytes);
    int goff[XNL];
#pragma unroll
    for (int n = 0; n < XNL; ++n) {
      const int r = n * XRL + lane / XCK;
      goff[n] = r * RBK + (((lane % XCK) ^ (r & (XCK - 1))) * 16);
    }
    const int row0 = __builtin_amdgcn_readfirstlane(m0 + wave * BMW);
    auto issue_x = [&](const u32x4& res, uint32_t dst, int j) __attribute__((always_inline)) {
      const int soff = __builtin_amdgcn_readfirstlane((j * p.T + row0) * RBK);
#pragma unroll
      for (int n = 0; n < XNL; ++n) load_to_lds16<0>(res, dst + n * 1024, goff[n], soff);
    };
    const uint8_t* const xkp = dq_smem + wave * (2 * 32 * RBK);
    const uint8_t* const xvp = xkp + 32 * RBK;
    const int xrow = col * RBK, xsw = col & (XCK - 1);
    for (int j = 1; j <= p.n_extra; ++j) {
      issue_x(xkres, xk, j);
      issue_x(xvres, xv, j);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      float dot = 0.f, dpv = 0.f;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        const int o = xrow + (((2 * kk + g) ^ xsw) * 16);
        dot = dot8_bf16(qf[0][kk], *reinterpret_cast<const u32x4*>(xkp + o), dot);
        dpv = dot8_bf16(dof[0][kk], *reinterpret_cast<const u32x4*>(xvp + o), dpv);
      }
      dot = half_swap_sum(dot);
      dpv = half_swap_sum(dpv);
      const float pv = fast_exp2(dot - lse_i[0]);  // the query fragments carry the scale
      const float ds = pv * (dpv - delta_i[0]);
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          float kk4[4];
          unpack4(*reinterpret_cast<const u32x2*>(xkp + xrow + (((db * 4 + r4) ^ xsw) * 16) + 8 * g), kk4);
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[0][db][r4 * 4 + t] = fmaf(ds, kk4[t], acc[0][db][r4 * 4 + t]);
        }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // rows read before the next step overwrites them
    }
  }

#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    if (i[sb] >= p.NQ) continue;
    uint16_t* orow = dQ + (int64_t)h * dq_hs + (int64_t)i[sb] * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2 w;
        w.x = pack_bf16x2(acc[sb][db][r4 * 4 + 0] * p.scaling, acc[sb][db][r4 * 4 + 1] * p.scaling);
        w.y = pack_bf16x2(acc[sb][db][r4 * 4 + 2] * p.scaling, acc[sb][db][r4 * 4 + 3] * p.scaling);
        *reinterpret_cast<u32x2*>(orow + db * 32 + 8 * r4) = w;
      }
  }
}

// per 64-row query tile: min / max of the interval ends of both classes (for the dK/dV
// tile loop): [a1min, a1max, b1min, b1max, a2min, a2max, b2min, b2max]
// rows[4][NQp] (NQp a multiple of 64): the interval ends of every row as the kernels compare them
// (a1, b1, T + a2, T + b2; an empty interval where a class is absent or the row is padding)
__global__ __launch_bounds__(64) void attn_tile_bounds_kernel(AttnParams p, int32_t* __restrict__ tb,
                                                              int NQp, int32_t* __restrict__ rows) {
  const int tile = blockIdx.x;
  const int r = tile * 64 + threadIdx.x;
  const bool ok = r < p.NQ;
  const int a1 = ok ? p.a1[r] : 0x7fffffff;
  const int b1 = ok ? (p.b1 ? p.b1[r] : r + 1) : 0;
  const int a2 = (ok && p.a2) ? p.T + p.a2[r] : 0x7fffffff;
  const int b2 = (ok && p.a2) ? p.T + p.b2[r] : 0;
  if (r < NQp) {
    rows[r] = a1; rows[NQp + r] = b1; rows[2 * (int64_t)NQp + r] = a2; rows[3 * (int64_t)NQp + r] = b2;
  }
  const int v[8] = {wave_min_i(a1), wave_max_i(a1), wave_min_i(b1), wave_max_i(b1),
                    wave_min_i(a2), wave_max_i(a2), wave_min_i(b2), wave_max_i(b2)};
  if (threadIdx.x == 0 && tile * 64 < p.NQ) {
#pragma unroll
    for (int k = 0; k < 8; ++k) tb[tile * 8 + k] = v[k];
  }
}

// dK / dV of the tiled keys: one workgroup = 128 keys x ONE query head (a wave owns 32
// keys: lane column = key), looping over the 64-row query tiles that can see the block.
// Scores are produced in the S = Q K^T orientation so that a lane holds one KEY:
//   dV^T += dO^T P,   dK^T += Q^T dS,   dS = P (dO V^T - delta)
// The per-head results go to fp32 partial buffers that attn_dkv_reduce_kernel sums over
// the heads of a group (fixed order: deterministic, no atomics).
// PASS 0 computes dK and dV together; PASS 1 only dV, PASS 2 only dK (head_dim 256: the two
// accumulator sets and both operand fragments do not fit the register file together, so
// the kernel is launched once per pass and the scores are recomputed).
#define SPX_DKV_XCD 1
// PF: how the query tiles reach LDS (see FwdSmem): 0 at the point of use, 1 through registers one
// tile ahead, 2 global -> LDS into the other of two buffers, 3 the same with tiles of 32 instead of 64
// query rows.  A buffer holds the tiles the pass multiplies with: Q always, dO and Q^T for dK, dO^T for
// dV.  At head_dim 256 two buffers of 64-row tiles fit the 160 KB of LDS only for the dV pass; with
// 32-row tiles all four fit, the register staging is gone and dK and dV come out of ONE pass.
// 4: like 2, but only the row-major Q and dO tiles are loaded: the A operands of the accumulating
// products (Q^T, dO^T fragments) come out of them through the transposing LDS read of gfx950
// (ds_read_b64_tr_b16), so two buffers of 64-row tiles fit at head_dim 256 as well, a step is 64
// rows long and half as many loads are issued per row.
template <int D, int PASS, int QT = 64, bool TR = false>
struct DkvSmem {
  static constexpr bool kDoV = PASS != 2, kDoK = PASS != 1;
  static constexpr int kTileR = QT * D * 2, kTileT = TR ? 0 : D * QT * 2;  // Q / dO and Q^T / dO^T tiles, unpadded
  static constexpr int kOffdO = kTileR;
  static constexpr int kOffQt = ((kDoK || TR) ? 2 : 1) * kTileR;
  static constexpr int kOffdOt = kOffQt + (kDoK ? kTileT : 0);
  static constexpr int kBuf = kOffdOt + (kDoV ? kTileT : 0);
  static constexpr int kSmall = 6 * 64 * 4;                     // lse, delta, a1, b1, a2, b2 of 64 rows
  static constexpr int kBytesDma = 2 * kBuf + 2 * kSmall;
  static constexpr int kBytes = (2 * 64 * (D + kKPad) + 2 * D * (64 + kVPad)) * 2 + kSmall;
};

// operand fragments in flight per product in the dK/dV kernel (one wave per SIMD: nothing else
// hides the latency of its LDS reads)
#define SPX_DKV_RING 8
template <int D, int NW, int PF, int PASS>
__global__ __launch_bounds__(64 * NW, SPX_DKV_MINB) void attn_bwd_dkv_kernel(
    AttnParams p, const uint16_t* __restrict__ dO, const uint16_t* __restrict__ Qt,
    const uint16_t* __restrict__ dOt, int NQp, const float* __restrict__ LSE,
    const float* __restrict__ Delta, const int32_t* __restrict__ tile_bounds,
    float* __restrict__ dKp, float* __restrict__ dVp) {
  constexpr int QS = D + kKPad;
  constexpr int TS = 64 + kVPad;
  constexpr int NKK = D / 16;
  constexpr int NDB = D / 32;
  constexpr int NT = 64 * NW;
  constexpr int KB = 32 * NW;  // keys per workgroup
  constexpr int CPT = (64 * D / 8) / NT;

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* Qs = smem;                 // [64][QS]
  uint16_t* dOs = Qs + 64 * QS;        // [64][QS]
  uint16_t* Qts = dOs + 64 * QS;       // [D][TS]
  uint16_t* dOts = Qts + D * TS;       // [D][TS]
  constexpr bool kDma = PF >= 2;
  constexpr bool kTR = PF == 4;                  // transposed operands by transposing LDS reads
  constexpr int QT = PF == 3 ? 32 : 64;          // query rows per LDS tile
  constexpr int NQB = QT / 32, NSUB = 64 / QT;   // 32-row halves per tile, tiles per 64-row step
  using SM = DkvSmem<D, PASS, QT, kTR>;
  static_assert(!kTR || PASS == 0, "the transposing-read mode computes both gradients");
  static_assert(!kDma || SM::kBytesDma <= 160 * 1024, "two buffers of this pass's tiles do not fit in LDS");
  uint8_t* const sm8 = reinterpret_cast<uint8_t*>(smem);
  float* lse_s = reinterpret_cast<float*>(kDma ? sm8 + 2 * SM::kBuf : sm8 + (2 * 64 * QS + 2 * D * TS) * 2);  // [64]
  float* delta_s = lse_s + 64;                               // [64]
  int* a1_s = reinterpret_cast<int*>(delta_s + 64);          // [64] each
  int* b1_s = a1_s + 64;
  int* a2_s = b1_s + 64;
  int* b2_s = a2_s + 64;

  // Workgroups go to the eight XCDs round robin.  The query-side tiles a workgroup streams belong to
  // its query head, so the workgroups that share an XCD (and its L2) at a time get the SAME head and
  // consecutive key blocks: neighbours in that order read the same tile two steps apart.
  // Heavy key blocks first: under a causal mask the EARLY key blocks are seen by most rows.
  int h, kb_idx;
  if (SPX_DKV_XCD && p.Hq % 8 == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, n_kb = gridDim.x / p.Hq;
    h = xcd + 8 * (slot / n_kb);
    kb_idx = slot % n_kb;
  } else {
    h = blockIdx.x % p.Hq;
    kb_idx = blockIdx.x / p.Hq;
  }
  const int kvh = h / (p.Hq / p.Hkv);
  const int n0 = kb_idx * KB;
  const int key_last = min(n0 + KB - 1, p.NKV - 1);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, col = lane & 31;
  const int cw = n0 + wave * 32;
  const int c = cw + col;
  const int cc = c < p.NKV ? c : p.NKV - 1;

  constexpr bool kDoV = PASS != 2, kDoK = PASS != 1;
  constexpr int NVF = kDoK ? NKK : 1;                    // V fragments feed dP, a dK-only term
  constexpr int NAK = kDoK ? NDB : 1, NAV = kDoV ? NDB : 1;
  bf16x8 kf[NKK], vf[NVF];
  {
    const uint16_t* krow = p.K + (int64_t)kvh * p.k_hs + (int64_t)cc * D + g * 8;
    const uint16_t* vrow = p.V + (int64_t)kvh * p.v_hs + (int64_t)cc * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      kf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(krow + kk * 16));
      if (kDoK) vf[kk % NVF] = as_bf16x8(*reinterpret_cast<const u32x4*>(vrow + kk * 16));
    }
  }
  f32x16 acc_dk[NAK], acc_dv[NAV];
#pragma unroll
  for (int db = 0; db < NAK; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_dk[db][r] = 0.f;
#pragma unroll
  for (int db = 0; db < NAV; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_dv[db][r] = 0.f;

  const uint16_t* Qh = p.Q + (int64_t)h * p.q_hs;
  const uint16_t* Qth = Qt + (int64_t)h * D * NQp;
  const uint16_t* dOth = dOt + (int64_t)h * D * NQp;
  const int n_qt = (p.NQ + 63) / 64;

  u32x4 qreg[CPT], dreg[CPT], qtreg[CPT], dtreg[CPT];
  float lse_r = 0.f, delta_r = 0.f;
  int a1_r = 0, b1_r = 0, a2_r = 0, b2_r = 0;
  auto visible = [&](int qt) {
    const int ta1 = tile_bounds[qt * 8 + 0], tb1 = tile_bounds[qt * 8 + 3];
    const int ta2 = tile_bounds[qt * 8 + 4], tb2 = tile_bounds[qt * 8 + 7];
    return (ta1 <= key_last && tb1 > n0) || (ta2 <= key_last && tb2 > n0);
  };
  // every row of the tile sees every key of this block: no per-element interval test
  auto fully_visible = [&](int qt) {
    return (tile_bounds[qt * 8 + 1] <= n0 && tile_bounds[qt * 8 + 2] >= n0 + KB) ||
           (tile_bounds[qt * 8 + 5] <= n0 && tile_bounds[qt * 8 + 6] >= n0 + KB);
  };
  // the per-row scalars of a query tile: wave 0 loads them into registers ...
  auto small_fetch = [&](int mq) {
    if (tid < 64) {
      const int ir = mq + tid;
      const bool ok = ir < p.NQ;
      lse_r = ok ? -LSE[(int64_t)h * p.NQ + ir] : 0.f;    // negated: they are MFMA C operands
      delta_r = ok ? -Delta[(int64_t)h * p.NQ + ir] : 0.f;
      a1_r = ok ? p.a1[ir] : 0x7fffffff;
      b1_r = ok ? (p.b1 ? p.b1[ir] : ir + 1) : 0;
      a2_r = (ok && p.a2) ? p.T + p.a2[ir] : 0x7fffffff;
      b2_r = (ok && p.a2) ? p.T + p.b2[ir] : 0;
    }
  };
  // ... and writes them to LDS (set `b` of the six arrays: only the two-buffer mode has a second one)
  auto small_stash = [&](int b) {
    if (tid < 64) {
      const int o = b * (SM::kSmall / 4);
      lse_s[o + tid] = lse_r; delta_s[o + tid] = delta_r;
      a1_s[o + tid] = a1_r; b1_s[o + tid] = b1_r; a2_s[o + tid] = a2_r; b2_s[o + tid] = b2_r;
    }
  };
  auto fetch = [&](int mq) {
    // The per-load row / column offsets are recomputed here on purpose.  Hoisted out of the tile loop they
    // stay live through it, and at head_dim 256 that is what spills; a spill reload inside the loop waits
    // for every older vector-memory operation, i.e. for the prefetch this function has just issued.
    int tid_v = tid;
    if (SPX_DKV_REMAT) asm volatile("" : "+v"(tid_v));
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int ch = tid_v + NT * n;
      const int qr = ch / (D / 8), qc = (ch % (D / 8)) * 8;
      const int ir = min(mq + qr, p.NQ - 1);
      qreg[n] = *reinterpret_cast<const u32x4*>(Qh + (int64_t)ir * D + qc);
      if (kDoK) dreg[n] = *reinterpret_cast<const u32x4*>(dO + ((int64_t)ir * p.Hq + h) * D + qc);
      const int td = ch >> 3, tc = (ch & 7) * 8;
      if (kDoK) qtreg[n] = *reinterpret_cast<const u32x4*>(Qth + (int64_t)td * NQp + mq + tc);
      if (kDoV) dtreg[n] = *reinterpret_cast<const u32x4*>(dOth + (int64_t)td * NQp + mq + tc);
    }
    small_fetch(mq);
  };
  auto stash = [&]() {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int ch = tid + NT * n;
      const int qr = ch / (D / 8), qc = (ch % (D / 8)) * 8;
      *reinterpret_cast<u32x4*>(&Qs[qr * QS + qc]) = qreg[n];
      if (kDoK) *reinterpret_cast<u32x4*>(&dOs[qr * QS + qc]) = dreg[n];
      const int td = ch >> 3, tc = (ch & 7) * 8;
      if (kDoK) *reinterpret_cast<u32x4*>(&Qts[td * TS + tc]) = qtreg[n];
      if (kDoV) *reinterpret_cast<u32x4*>(&dOts[td * TS + tc]) = dtreg[n];
    }
    small_stash(0);
  };

  auto direct = [&](int mq) {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int ch = tid + NT * n;
      const int qr = ch / (D / 8), qc = (ch % (D / 8)) * 8;
      const int ir = min(mq + qr, p.NQ - 1);
      // only the tiles this pass multiplies with: Q always (scores), dO and Q^T for dK,
      // dO^T for dV
      *reinterpret_cast<u32x4*>(&Qs[qr * QS + qc]) =
          *reinterpret_cast<const u32x4*>(Qh + (int64_t)ir * D + qc);
      if (kDoK)
        *reinterpret_cast<u32x4*>(&dOs[qr * QS + qc]) =
            *reinterpret_cast<const u32x4*>(dO + ((int64_t)ir * p.Hq + h) * D + qc);
      const int td = ch >> 3, tc = (ch & 7) * 8;
      if (kDoK)
        *reinterpret_cast<u32x4*>(&Qts[td * TS + tc]) =
            *reinterpret_cast<const u32x4*>(Qth + (int64_t)td * NQp + mq + tc);
      if (kDoV)
        *reinterpret_cast<u32x4*>(&dOts[td * TS + tc]) =
            *reinterpret_cast<const u32x4*>(dOth + (int64_t)td * NQp + mq + tc);
    }
    if (tid < 64) {
      const int ir = mq + tid;
      const bool ok = ir < p.NQ;
      lse_s[tid] = ok ? -LSE[(int64_t)h * p.NQ + ir] : 0.f;
      delta_s[tid] = ok ? -Delta[(int64_t)h * p.NQ + ir] : 0.f;
      a1_s[tid] = ok ? p.a1[ir] : 0x7fffffff;
      b1_s[tid] = ok ? (p.b1 ? p.b1[ir] : ir + 1) : 0;
      a2_s[tid] = (ok && p.a2) ? p.T + p.a2[ir] : 0x7fffffff;
      b2_s[tid] = (ok && p.a2) ? p.T + p.b2[ir] : 0;
    }
  };

  // ---- two-buffer modes: the tiles as 1 KB wave loads global -> LDS; chunk c of row r lives in
  // slot c ^ swz(r) (conflict-free fragment reads without padding)
  constexpr int RBQ = D * 2, CKQ = RBQ / 16;   // bytes / 16-byte chunks per row of Q and dO
  constexpr int RBT = QT * 2, CKT = RBT / 16;  // ... of Q^T and dO^T
  constexpr int LPR = (QT * RBQ / 1024) / NW, LPT = (D * RBT / 1024) / NW;  // wave loads per wave and tile
  // (with transposing reads the rows of a 4 + 4 row group must also fall into different 64-byte bank
  // groups: the row's two low bits go to the chunk index's bits 2 - 3)
  auto swz_r = [](int r) {
    if (kTR) return CKQ == 8 ? ((r & 4) | ((r >> 2) & 2) | ((r >> 1) & 1)) : ((r & 3) << 2) | ((r >> 2) & 3);
    return CKQ == 8 ? (r >> 1) & 7 : r & 15;
  };
  auto swz_t = [](int r) { return CKT == 8 ? (r >> 1) & 7 : (r >> 2) & 3; };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)sm8;
  u32x4 qres, dres, qtres, dtres;
  if constexpr (kDma) {
    qres = make_rsrc(Qh, (uint32_t)((int64_t)p.NQ * RBQ));
    dres = make_rsrc(dO + (int64_t)h * D, (uint32_t)((((int64_t)p.NQ - 1) * p.Hq * D + D) * 2));
    qtres = make_rsrc(Qth, (uint32_t)((int64_t)D * NQp * 2));
    dtres = make_rsrc(dOth, (uint32_t)((int64_t)D * NQp * 2));
  }
  auto issue = [&](int mq, int b) __attribute__((always_inline)) {
    if constexpr (kDma) {
      // per-load offsets recomputed here on purpose: hoisted out of the tile loop they cost registers that
      // the two-workgroups-per-CU build does not have
      int lane_v = lane;
      if (SPX_DKV_REMAT) asm volatile("" : "+v"(lane_v));
      const uint32_t rb = lds0 + b * SM::kBuf + wave * LPR * 1024;
#pragma unroll
      for (int j = 0; j < LPR; ++j) {
        const int r = (wave * LPR + j) * (1024 / RBQ) + lane_v / CKQ;
        const int cofs = ((lane_v % CKQ) ^ swz_r(r)) * 16;
        const int ir = min(mq + r, p.NQ - 1);
        load_to_lds16<0>(qres, rb + j * 1024, ir * RBQ + cofs, 0);
        if (kDoK || kTR) load_to_lds16<0>(dres, rb + SM::kOffdO + j * 1024, ir * (p.Hq * RBQ) + cofs, 0);
      }
      const uint32_t tb2 = lds0 + b * SM::kBuf + wave * LPT * 1024;
#pragma unroll
      for (int j = 0; j < (kTR ? 0 : LPT); ++j) {
        const int r = (wave * LPT + j) * (1024 / RBT) + lane_v / CKT;
        const int tofs = r * NQp * 2 + ((lane_v % CKT) ^ swz_t(r)) * 16;
        if (kDoK) load_to_lds16<0>(qtres, tb2 + SM::kOffQt + j * 1024, tofs, mq * 2);
        if (kDoV) load_to_lds16<0>(dtres, tb2 + SM::kOffdOt + j * 1024, tofs, mq * 2);
      }
    }
  };
  const int rdr = col * RBQ + ((g ^ swz_r(col)) * 16);
  const int rdt = col * RBT + ((g ^ swz_t(col)) * 16);
  // transposing reads: lane s of 16-lane group G points at row 4 (G >> 1) + (s >> 2) (+ 8 for the
  // second read) of a 16-row k step, bytes 8 (s & 3) of the 64-byte block 32 db + 16 (G & 1): the k
  // index order of the P / dS operands (rows 4 g .. 4 g + 3, then 8 + 4 g .. 8 + 4 g + 3)
  const int tG = lane >> 4, ts = lane & 15;
  const int trow = 4 * (tG >> 1) + (ts >> 2);
  const int tcl = 2 * (tG & 1) + ((ts & 3) >> 1);
  const int rt0 = trow * RBQ + ((tcl ^ swz_r(trow)) * 16) + (ts & 1) * 8;
  const int rt1 = (trow + 8) * RBQ + ((tcl ^ swz_r(trow + 8)) * 16) + (ts & 1) * 8;
  const float* const lse_s0 = lse_s;
  const uint8_t* tile = sm8;
  int buf = 0;

  // (walking the tiles from the last one down, so that every workgroup of a head reads the same tile at
  // the same time, was slower: 256 workgroups then hit the same few memory channels at once)
  int qi = 0, sub = 0, sbuf = 0;  // 64-row step, tile inside it, set of per-row scalars in use
  while (qi < n_qt && !visible(qi)) ++qi;
  if (PF == 1 && qi < n_qt) fetch(qi * 64);
  if (kDma && qi < n_qt) {
    issue(qi * 64, 0);
    small_fetch(qi * 64);
    small_stash(0);
  }
  while (qi < n_qt) {
    // what comes next: the other tile of this 64-row step, or the first tile of the next visible step
    int nxi = qi, nsub = sub + 1;
    if (nsub == NSUB) {
      nsub = 0;
      ++nxi;
      while (nxi < n_qt && !visible(nxi)) ++nxi;
    }
    const int qt = qi, nxt = nxi;
    const bool full = fully_visible(qt);
    const bool have_next = nxi < n_qt;
    if constexpr (kDma) {
      // this wave's loads of the tile have landed; behind the barrier everybody's have, the per-row
      // scalars written at the end of the last iteration are visible, and the other buffer is free
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (have_next) {
        issue(nxt * 64 + nsub * QT, buf ^ 1);
        if (nsub == 0) small_fetch(nxt * 64);
      }
      tile = sm8 + buf * SM::kBuf;
      const int o = sbuf * (SM::kSmall / 4);
      lse_s = const_cast<float*>(lse_s0) + o;
      delta_s = lse_s + 64;
      a1_s = reinterpret_cast<int*>(delta_s + 64);
      b1_s = a1_s + 64; a2_s = b1_s + 64; b2_s = a2_s + 64;
    } else {
      __syncthreads();
      if (PF) stash(); else direct(qt * 64);
      __syncthreads();
      if (PF && have_next) fetch(nxt * 64);
    }
    const int sub_now = sub;
    qi = nxi;
    sub = nsub;

    // the two 32-row halves of the query tile one after the other (keeps 32 score
    // registers live instead of 64)
    // (head_dim 256 has no registers to spare for two unrolled halves in flight: a real loop there)
#pragma unroll(kTR ? 1 : NQB)
    for (int qbl = 0; qbl < NQB; ++qbl) {
      const int qb = sub_now * NQB + qbl;  // 32-row half inside the 64-row step (per-row scalars); qbl: inside the LDS tile
      // the scores start from -lse of their query row and dO V^T from -delta (LDS holds both
      // negated): s - lse and dP - delta come out of the matrix pipe.  The Q tile is the scaled
      // copy (bf16(q * scale * log2 e)), so the scores are base-2 exponents already
      f32x16 st, dp;
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int q0 = qb * 32 + 8 * r4 + 4 * g;  // 4 consecutive query rows: one 16-byte LDS read each
        const f32x4 ls = *reinterpret_cast<const f32x4*>(&lse_s[q0]);
#pragma unroll
        for (int t = 0; t < 4; ++t) st[r4 * 4 + t] = ls[t];
        if (kDoK) {
          const f32x4 dl = *reinterpret_cast<const f32x4*>(&delta_s[q0]);
#pragma unroll
          for (int t = 0; t < 4; ++t) dp[r4 * 4 + t] = dl[t];
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) dp[r4 * 4 + t] = 0.f;
        }
      }
      {
        // Q (and, for dK, dO) row fragments through a ring of four registers: the read of
        // fragment f + 4 follows the MFMA of fragment f, so no MFMA waits for LDS
        constexpr int PER = kDoK ? 2 : 1;  // fragments per K step: Q [, dO]
        constexpr int NF = PER * NKK;
        constexpr int RG = SPX_DKV_RING;
        bf16x8 fr[RG];
        auto fread = [&](int f) {
          if constexpr (kDma) {
            const uint8_t* base = tile + ((PER == 2 && (f & 1)) ? SM::kOffdO : 0);
            fr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                base + qbl * 32 * RBQ + (rdr ^ ((f / PER) * 32))));
          } else {
            const uint16_t* base = (PER == 2 && (f & 1)) ? dOs : Qs;
            fr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                &base[(qb * 32 + col) * QS + g * 8 + (f / PER) * 16]));
          }
        };
#pragma unroll
        for (int f = 0; f < RG && f < NF; ++f) fread(f);
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          __builtin_amdgcn_sched_barrier(0);
          if (PER == 2 && (f & 1)) dp = mfma32(fr[f % RG], vf[(f / PER) % NVF], dp);
          else st = mfma32(fr[f % RG], kf[f / PER], st);
          __builtin_amdgcn_sched_barrier(0);
          if (f + RG < NF) fread(f + RG);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] = fast_exp2(st[r]);
      if (!full) {
        // a real (scalar) branch: only tiles that straddle an interval edge pay for the mask
        typedef __attribute__((ext_vector_type(4))) int i32x4;
        pin_block(st);
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int q0 = qb * 32 + 8 * r4 + 4 * g;
          const i32x4 a1v = *reinterpret_cast<const i32x4*>(&a1_s[q0]);
          const i32x4 b1v = *reinterpret_cast<const i32x4*>(&b1_s[q0]);
          const i32x4 a2v = *reinterpret_cast<const i32x4*>(&a2_s[q0]);
          const i32x4 b2v = *reinterpret_cast<const i32x4*>(&b2_s[q0]);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const bool ok = ((c >= a1v[t] && c < b1v[t]) || (c >= a2v[t] && c < b2v[t])) && (c < p.NKV);
            if (!ok) st[r4 * 4 + t] = 0.f;
          }
        }
        pin_block(st);
      }
      if (kDoK) {
#pragma unroll
        for (int r = 0; r < 16; ++r) dp[r] *= st[r];
      }
      {
        // dO^T / Q^T fragments through the same kind of ring; per (16-row step s2, D block db):
        // dO^T [, Q^T]
        constexpr int PER = (kDoV ? 1 : 0) + (kDoK ? 1 : 0);
        constexpr int NF = PER * 2 * NDB;
        constexpr int RG = SPX_DKV_RING;
        bf16x8 fr[RG];
        auto fread = [&](int f) {
          const int e = f / PER, s2 = e / NDB, db = e % NDB;
          const bool is_q = kDoK && (!kDoV || (f % PER) == 1);
          if constexpr (kTR) {
            const uint8_t* base = tile + (is_q ? 0 : SM::kOffdO) + (qbl * 32 + s2 * 16) * RBQ;
            const i16x4 lo = lds_read_tr16(base + (rt0 ^ (db * 64)));
            const i16x4 hi = lds_read_tr16(base + (rt1 ^ (db * 64)));
            fr[f % RG] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          } else if constexpr (kDma) {
            const uint8_t* base = tile + (is_q ? SM::kOffQt : SM::kOffdOt);
            fr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                base + db * 32 * RBT + (rdt ^ ((qbl * 2 + s2) * 32))));
          } else {
            const uint16_t* base = is_q ? Qts : dOts;
            fr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
                &base[(db * 32 + col) * TS + (qb * 2 + s2) * 16 + 8 * g]));
          }
        };
#pragma unroll
        for (int f = 0; f < RG && f < NF; ++f) fread(f);
        bf16x8 pb = pack8(st, 0), sb8 = pack8(dp, 0);
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          const int e = f / PER, s2 = e / NDB, db = e % NDB;
          const bool is_q = kDoK && (!kDoV || (f % PER) == 1);
          if (f == PER * NDB) { pb = pack8(st, 8); sb8 = pack8(dp, 8); }
          __builtin_amdgcn_sched_barrier(0);
          if (is_q) acc_dk[db % NAK] = mfma32(fr[f % RG], sb8, acc_dk[db % NAK]);
          else acc_dv[db % NAV] = mfma32(fr[f % RG], pb, acc_dv[db % NAV]);
          __builtin_amdgcn_sched_barrier(0);
          if (f + RG < NF) fread(f + RG);
          (void)s2;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (kDma) {
      // the per-row scalars of the next 64-row step go into the other set: nobody reads it before the
      // barrier
      if (nsub == 0) {
        if (have_next) {
          lse_s = const_cast<float*>(lse_s0); delta_s = lse_s + 64;
          a1_s = reinterpret_cast<int*>(delta_s + 64); b1_s = a1_s + 64; a2_s = b1_s + 64; b2_s = a2_s + 64;
          small_stash(sbuf ^ 1);
        }
        sbuf ^= 1;
      }
      buf ^= 1;
    }
  }

  if (c < p.NKV) {
    float* krow = dKp + ((int64_t)h * p.NKV + c) * D + 4 * g;
    float* vrow = dVp + ((int64_t)h * p.NKV + c) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        if (kDoK) {
          const f32x16& a = acc_dk[db % NAK];
          f32x4 wk = {a[r4 * 4 + 0], a[r4 * 4 + 1], a[r4 * 4 + 2], a[r4 * 4 + 3]};
          *reinterpret_cast<f32x4*>(krow + db * 32 + 8 * r4) = wk;
        }
        if (kDoV) {
          const f32x16& a = acc_dv[db % NAV];
          f32x4 wv = {a[r4 * 4 + 0], a[r4 * 4 + 1], a[r4 * 4 + 2], a[r4 * 4 + 3]};
          *reinterpret_cast<f32x4*>(vrow + db * 32 + 8 * r4) = wv;
        }
      }
  }
}

// ---------------------------------------------------------------- dK / dV, wave-specialised
// The work of attn_bwd_dkv_kernel for head_dim <= 128 (both gradients in one pass), split over
// TWO waves per SIMD that run different halves of it, so that each SIMD has a wave for the matrix
// pipe while the other is in its vector phase, and every MFMA works on plain vector registers:
//   producer wave i (waves 0-3): keeps K / V fragments of its 32 keys; per 32-row query tile
//     S = Q' K^T - lse and dP = dO V^T - delta (16 MFMAs at head_dim 128), P = exp2(S), dS = P dP,
//     both rounded to bf16 in the B-operand layout and handed over through a 4 KB LDS slot;
//   consumer wave i (waves 4-7, same SIMD): keeps the dK / dV accumulators of those 32 keys
//     (128 registers); per tile dV^T += dO^T P and dK^T += Q'^T dS (16 MFMAs) from the slot.
// Both roles read the SAME row-major query tile (32 rows of Q' and of dO): the consumers take
// their A operands (dO^T, Q'^T fragments) with transposing LDS reads (ds_read_b64_tr_b16), so no
// transposed copy of the queries exists in memory.  Everything a step needs comes global -> LDS
// directly, kAhead tiles ahead, into a ring of kStages buffers: the tile, and the per-row scalars
// (-lse, -delta: the C operands of the score products; the mask interval ends).  In step b the
// producers turn the scores of tile b (computed one step earlier) into P and dS first, while the
// consumers' MFMAs of tile b - 1 run, and compute the scores of tile b + 1 after that.  One
// workgroup barrier per step; slots are double buffered.
template <int D>
struct DkvWsSmem {
  static constexpr int kStages = 6;
  static constexpr int kAhead = 4;                     // tile b + kAhead is issued in step b
  static constexpr int kTile = 2 * 32 * D * 2;         // Q', dO: 32 rows of D each
  static constexpr int kSlot = 16 * 64 * 4;            // 16 registers of 64 lanes
  static constexpr int kOffSlot = kStages * kTile;
  static constexpr int kOffSmall = kOffSlot + 4 * 2 * kSlot;
  static constexpr int kSmall = 6 * 32 * 4;            // -lse, -delta, a1, b1, a2, b2 of 32 rows
  static constexpr int kSets = 8;                      // sets of per-row scalars (tile k: set k % 8)
  static constexpr int kOffList = kOffSmall + kSets * kSmall + 256;  // (+ a spare area)
  static constexpr int kListCap = 2048;                // visible 64-row tiles per key block, at most
  static constexpr int kList = (kListCap + 1) * 4;     // ... their list, closed by an end mark
  static constexpr int kBytes = kOffList + 2 * kList + 64;  // two key blocks; scratch of the list builder
  static constexpr uint32_t kListEnd = 0x7fffffffu;
  static_assert(kStages >= kAhead + 2, "a buffer is free two steps after its tile's scores");
};

// Values a non-inlined device function receives arrive in vector registers; these make them
// wave-uniform (scalar registers) again, which addresses of the global -> LDS loads must be.
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename T>
__device__ __forceinline__ T* uni(T* q) {
  const uint64_t a = reinterpret_cast<uint64_t>(q);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int64_t uni(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}



// One role of the kernel as a function of its own (not inlined): the register allocation of the
// producers (K / V fragments, scores) and of the consumers (128 accumulator registers) then do not
// add up.  Both roles walk the same sequence of steps and meet at the same barriers.
template <int D, bool PRODUCER>
__device__ __attribute__((noinline)) void dkv_ws_role(
    const AttnParams& p_in, const uint16_t* dO_in, int NQp_in, const float* neg_in,
    const int32_t* mrows_in, float* dKp_in, float* dVp_in) {
  using SM = DkvWsSmem<D>;
  extern __shared__ __attribute__((aligned(16))) uint8_t ws_smem[];
  AttnParams p;
  p.Q = uni(p_in.Q); p.q_hs = uni(p_in.q_hs);
  p.K = uni(p_in.K); p.k_hs = uni(p_in.k_hs);
  p.V = uni(p_in.V); p.v_hs = uni(p_in.v_hs);
  p.a1 = nullptr; p.b1 = nullptr; p.a2 = nullptr; p.b2 = nullptr;
  p.NQ = uni(p_in.NQ); p.T = uni(p_in.T); p.NKV = uni(p_in.NKV); p.NKVp = uni(p_in.NKVp);
  p.n_extra = uni(p_in.n_extra); p.Hq = uni(p_in.Hq); p.Hkv = uni(p_in.Hkv);
  p.scale_log2e = p_in.scale_log2e; p.scaling = p_in.scaling;
  const uint16_t* __restrict__ dO = uni(dO_in);
  const int NQp = uni(NQp_in);
  const float* __restrict__ neg = uni(neg_in);        // -lse [Hq][NQp], -delta [Hq][NQp]
  const int32_t* __restrict__ mrows = uni(mrows_in);  // interval ends of every row, [4][NQp]
  float* __restrict__ dKp = uni(dKp_in);
  float* __restrict__ dVp = uni(dVp_in);

  constexpr bool producer = PRODUCER;
  constexpr int NKK = D / 16, NDB = D / 32;
  constexpr int KB = 128;                                 // keys per workgroup
  constexpr int RBQ = D * 2, CKQ = RBQ / 16;              // bytes / 16-byte chunks per row of Q' and dO
  constexpr int NLQ = 32 * RBQ / 1024;                    // 1 KB wave loads per 32-row operand
  constexpr int LPW = 2 * NLQ / 4;                        // tile loads per consumer wave (they issue them all)
  constexpr int kLoads = LPW + 1;                         // ... plus one of per-row scalars
  constexpr int RG = 4;
  constexpr int NS = SM::kStages, AH = SM::kAhead;
  static_assert(LPW >= 1 && 2 * NLQ % 4 == 0, "every consumer wave issues the same number of loads per tile");
  // A workgroup takes key blocks i and n_kb - 1 - i of one head, one after the other: under a causal
  // mask block i is seen by all later query tiles and its partner by correspondingly few, so every
  // workgroup walks about the same number of tiles.
  const int n_kb = (p.NKV + KB - 1) / KB, n_pair = (n_kb + 1) / 2;
  int h, pair;
  if (SPX_DKV_XCD && p.Hq % 8 == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    h = xcd + 8 * (slot / n_pair);
    pair = slot % n_pair;
  } else {
    h = blockIdx.x % p.Hq;
    pair = blockIdx.x / p.Hq;
  }
  const int kvh = h / (p.Hq / p.Hkv);
  for (int part = 0; part < 2; ++part) {
  const int kb_idx = part == 0 ? pair : n_kb - 1 - pair;
  if (part == 1) {
    if (kb_idx == pair) break;   // the middle block of an odd count has no partner
    __syncthreads();             // everybody is done with the ring, the slots and the sets
  }
  const int n0 = kb_idx * KB;
  const int key_last = min(n0 + KB - 1, p.NKV - 1);

  const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6);
  const int pw = wave & 3;                 // pair index: the 32 keys of this wave
  const int g = lane >> 5, col = lane & 31;
  const int c = n0 + pw * 32 + col;
  const int cc = c < p.NKV ? c : p.NKV - 1;
  const int n_qt = (p.NQ + 63) / 64;

  // the steps: the two 32-row halves of every 64-row query tile that sees the block, in order.  The
  // kernel has listed those tiles in LDS (bit 31: every key of the block is visible to all rows of the
  // tile); step k is half k & 1 of list entry k / 2.
  const uint32_t* const lst = reinterpret_cast<const uint32_t*>(ws_smem + SM::kOffList + part * SM::kList);
  const int s_end = n_qt * 2;
  auto step_of = [&](uint32_t e, int k_) { return (e & 0x7fffffffu) == SM::kListEnd ? s_end : (int)(e & 0x7fffffffu) * 2 + (k_ & 1); };
  const int n_vis = uni(reinterpret_cast<const int*>(ws_smem + SM::kOffList + 2 * SM::kList)[8 + part]);
  auto entry = [&](int k_) { return lst[min(k_ >> 1, n_vis)]; };

  // position of 16-byte chunk c of row r inside its LDS row: c ^ swz_r(r).  Row-wise 16-byte reads of 32
  // rows (the producers) and the transposing reads of 4 + 4 rows x 64 bytes (the consumers) both
  // spread evenly over the banks.
  auto swz_r = [](int r) {
    return CKQ == 8 ? ((r & 4) | ((r >> 2) & 2) | ((r >> 1) & 1)) : ((r & 3) << 2) | ((r >> 2) & 3);
  };
  const uint32_t lds0 = (uint32_t)uni((int)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)ws_smem);
  const u32x4 qres = make_rsrc(p.Q + (int64_t)h * p.q_hs, (uint32_t)((int64_t)p.NQ * RBQ));
  const u32x4 dres = make_rsrc(dO + (int64_t)h * D, (uint32_t)((((int64_t)p.NQ - 1) * p.Hq * D + D) * 2));
  // per-row scalars of a tile: -lse | -delta, a1 | b1, a2 | b2 (32 values each), one 256-byte load
  // by each of consumer waves 0-2 (the fourth repeats the first into a spare area so that all count
  // alike).  The consumers issue every load: they have time to spare, the producers do not.
  const u32x4 nres = make_rsrc(neg + (int64_t)h * NQp, (uint32_t)((((int64_t)p.Hq + 1) * NQp) * 4));
  const u32x4 mres = make_rsrc(mrows, (uint32_t)(4 * (int64_t)NQp * 4));
  const bool sm_mask = pw == 1 || pw == 2;
  const int sm_off = (lane & 31) * 4 + (lane >> 5) * (sm_mask ? NQp * 4 : p.Hq * NQp * 4) +
                     (pw == 2 ? 2 * NQp * 4 : 0);
  // this wave's loads of a tile: load li = pw + 4 j of the 2 * NLQ that make it (Q' first, then dO);
  // rows past the last query read as zeros (and contribute nothing)
  int ld_off[LPW], ld_mul[LPW], ld_dst[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int li = pw + 4 * j;
    const bool is_do = li >= NLQ;
    const int l = is_do ? li - NLQ : li;
    const int r = l * (1024 / RBQ) + lane / CKQ;
    const int cofs = ((lane % CKQ) ^ swz_r(r)) * 16;
    ld_mul[j] = is_do ? p.Hq * RBQ : RBQ;          // bytes per query row in global memory
    ld_off[j] = r * ld_mul[j] + cofs;
    ld_dst[j] = (is_do ? 32 * RBQ : 0) + l * 1024;
  }
  auto issue = [&](int s_, int buf, int set) __attribute__((always_inline)) {
    const int mq = s_ * 32;
    const uint32_t rb = lds0 + buf * SM::kTile;
#pragma unroll
    for (int j = 0; j < LPW; ++j)
      load_to_lds16<0>(pw + 4 * j >= NLQ ? dres : qres, rb + ld_dst[j], ld_off[j] + mq * ld_mul[j], 0);
    const uint32_t sb = lds0 + SM::kOffSmall + (pw == 3 ? SM::kSets * SM::kSmall : set * SM::kSmall + pw * 256);
    load_to_lds4(sm_mask ? mres : nres, sb, sm_off + mq * 4, 0);
  };
  float* const small0 = reinterpret_cast<float*>(ws_smem + SM::kOffSmall);

  // ---- role state
  bf16x8 kf[producer ? NKK : 1], vf[producer ? NKK : 1];
  f32x16 acc_dk[producer ? 1 : NDB], acc_dv[producer ? 1 : NDB];
  if constexpr (producer) {
    const uint16_t* krow = p.K + (int64_t)kvh * p.k_hs + (int64_t)cc * D + g * 8;
    const uint16_t* vrow = p.V + (int64_t)kvh * p.v_hs + (int64_t)cc * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      kf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(krow + kk * 16));
      vf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(vrow + kk * 16));
    }
  } else {
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc_dk[db][r] = 0.f; acc_dv[db][r] = 0.f; }
  }
  // producers: row `col`, 16-byte chunk 2 kk + g of Q' / dO
  const int rdr = col * RBQ + ((g ^ swz_r(col)) * 16);
  // consumers: lane s of 16-lane group G points at row 4 (G >> 1) + (s >> 2) (+ 8 for the second read) of
  // a 16-row k step, bytes 8 (s & 3) of the 64-byte block 32 db + 16 (G & 1).  (The k index of the
  // P / dS operand: element j of the lanes with g = lane / 32 is query row 4 g + j for j < 4 and
  // 8 + 4 g + j - 4 after that, the accumulator layout of the score product.)
  const int tG = lane >> 4, ts = lane & 15;
  const int trow = 4 * (tG >> 1) + (ts >> 2);
  const int tcl = 2 * (tG & 1) + ((ts & 3) >> 1);
  const int rt0 = trow * RBQ + ((tcl ^ swz_r(trow)) * 16) + (ts & 1) * 8;
  const int rt1 = (trow + 8) * RBQ + ((tcl ^ swz_r(trow + 8)) * 16) + (ts & 1) * 8;
  uint8_t* const slot0 = ws_smem + SM::kOffSlot + pw * 2 * SM::kSlot;

  // ---- the producers' two halves of a tile (kIdx: its index in the sequence of steps)
  f32x16 st, dp;      // scores / dP of the tile in work
  f32x16 stn, dpn;    // -lse, -delta of the next tile (the C operands of its first products)
  constexpr int NFP = 2 * NKK;
  bf16x8 pfr[RG];
  const uint8_t* ptile = ws_smem;
  auto pfread = [&](int f) __attribute__((always_inline)) {
    pfr[f % RG] = as_bf16x8(*reinterpret_cast<const u32x4*>(
        ptile + ((f & 1) ? 32 * RBQ : 0) + (rdr ^ ((f / 2) * 32))));
  };
  // first half: the LDS reads whose results the products start from (issued before the soft-max half
  // of the previous tile, so that they are back when it ends)
  auto score_begin = [&](int buf, int set) __attribute__((always_inline)) {
    ptile = ws_smem + buf * SM::kTile;
    const float* const lse_s = small0 + set * (SM::kSmall / 4);
    const float* const delta_s = lse_s + 32;
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int q0 = 8 * r4 + 4 * g;  // 4 consecutive query rows: one 16-byte LDS read each
      const f32x4 ls = *reinterpret_cast<const f32x4*>(&lse_s[q0]);
      const f32x4 dl = *reinterpret_cast<const f32x4*>(&delta_s[q0]);
#pragma unroll
      for (int t = 0; t < 4; ++t) { stn[r4 * 4 + t] = ls[t]; dpn[r4 * 4 + t] = dl[t]; }
    }
#pragma unroll
    for (int f = 0; f < RG; ++f) pfread(f);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto score_finish = [&]() __attribute__((always_inline)) {
    SPX_DKV_PRIO_MFMA();
#pragma unroll
    for (int f = 0; f < NFP; ++f) {
      __builtin_amdgcn_sched_barrier(0);
      if (f & 1) dp = mfma32(pfr[f % RG], vf[producer ? f / 2 : 0], f == 1 ? dpn : dp);
      else st = mfma32(pfr[f % RG], kf[producer ? f / 2 : 0], f == 0 ? stn : st);
      __builtin_amdgcn_sched_barrier(0);
      if (f + RG < NFP) pfread(f + RG);
    }
    __builtin_amdgcn_sched_barrier(0);
    SPX_DKV_PRIO_VALU();
  };
  auto soft_valu = [&](int set, int par, bool full) __attribute__((always_inline)) {
    const int* const a1_s = reinterpret_cast<const int*>(small0 + set * (SM::kSmall / 4) + 64);
    const int* const b1_s = a1_s + 32; const int* const a2_s = b1_s + 32; const int* const b2_s = a2_s + 32;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = fast_exp2(st[r]);
    if (!full) {
      typedef __attribute__((ext_vector_type(4))) int i32x4;
      pin_block(st);
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int q0 = 8 * r4 + 4 * g;
        const i32x4 a1v = *reinterpret_cast<const i32x4*>(&a1_s[q0]);
        const i32x4 b1v = *reinterpret_cast<const i32x4*>(&b1_s[q0]);
        const i32x4 a2v = *reinterpret_cast<const i32x4*>(&a2_s[q0]);
        const i32x4 b2v = *reinterpret_cast<const i32x4*>(&b2_s[q0]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bool ok = ((c >= a1v[t] && c < b1v[t]) || (c >= a2v[t] && c < b2v[t])) && (c < p.NKV);
          if (!ok) st[r4 * 4 + t] = 0.f;
        }
      }
      pin_block(st);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) dp[r] *= st[r];
    // hand P and dS over: four 16-byte stores per lane, slot row = register quad, column = lane
    uint8_t* const slot = slot0 + par * SM::kSlot + lane * 16;
    *reinterpret_cast<bf16x8*>(slot + 0 * 1024) = pack8(st, 0);
    *reinterpret_cast<bf16x8*>(slot + 1 * 1024) = pack8(st, 8);
    *reinterpret_cast<bf16x8*>(slot + 2 * 1024) = pack8(dp, 0);
    *reinterpret_cast<bf16x8*>(slot + 3 * 1024) = pack8(dp, 8);
  };
  // ---- the consumers' half: dV^T += dO^T P, dK^T += Q'^T dS
  auto consume = [&](int buf, int par) __attribute__((always_inline)) {
    const uint8_t* const tile = ws_smem + buf * SM::kTile;
    const uint8_t* const slot = slot0 + par * SM::kSlot + lane * 16;
    bf16x8 pb[2], sb[2];
    pb[0] = *reinterpret_cast<const bf16x8*>(slot + 0 * 1024);
    pb[1] = *reinterpret_cast<const bf16x8*>(slot + 1 * 1024);
    sb[0] = *reinterpret_cast<const bf16x8*>(slot + 2 * 1024);
    sb[1] = *reinterpret_cast<const bf16x8*>(slot + 3 * 1024);
    SPX_DKV_PRIO_MFMA();
    constexpr int NF = 2 * 2 * NDB;
    i16x4 lo[RG], hi[RG];
    // fragment f: even = dO^T (for dV), odd = Q'^T (for dK); e = f / 2: k step s2 = e / NDB, row block db
    auto fread = [&](int f) {
      const int e = f / 2, s2 = e / NDB, db = e % NDB;
      const uint8_t* const base = tile + ((f & 1) ? 0 : 32 * RBQ) + s2 * 16 * RBQ;
      lo[f % RG] = lds_read_tr16(base + (rt0 ^ (db * 64)));
      hi[f % RG] = lds_read_tr16(base + (rt1 ^ (db * 64)));
    };
    auto frag = [&](int f) {
      const i16x8 v = __builtin_shufflevector(lo[f % RG], hi[f % RG], 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    };
#pragma unroll
    for (int f = 0; f < RG; ++f) fread(f);
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const int e = f / 2, s2 = e / NDB, db = e % NDB;
      __builtin_amdgcn_sched_barrier(0);
      if (f & 1) acc_dk[producer ? 0 : db] = mfma32(frag(f), sb[s2], acc_dk[producer ? 0 : db]);   // Q'^T dS
      else acc_dv[producer ? 0 : db] = mfma32(frag(f), pb[s2], acc_dv[producer ? 0 : db]);         // dO^T P
      __builtin_amdgcn_sched_barrier(0);
      if (f + RG < NF) fread(f + RG);
    }
    __builtin_amdgcn_sched_barrier(0);
    SPX_DKV_PRIO_VALU();
  };

  // ---- prologue.  Tile k of the sequence of steps lives in ring buffer k % kStages, its per-row
  // scalars in set k % kSets, its P / dS in slot k % 2.
  int sq[AH + 1];               // sq[i]: the step (tile) of sequence index b + i
  bool fq[AH + 1];              // ... whether every key of the block is visible to all of its rows
#pragma unroll
  for (int i = 0; i <= AH; ++i) {
    const uint32_t e = (uint32_t)uni((int)entry(i));
    sq[i] = step_of(e, i);
    fq[i] = (e >> 31) != 0;
  }
  uint32_t pref = entry(AH + 1);   // fetched one step before it joins the queue
  int sC = s_end;               // the consumers' tile: b - 1
  if constexpr (!producer) {
#pragma unroll
    for (int i = 0; i < AH; ++i)
      if (sq[i] < s_end) issue(sq[i], i, i);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  if constexpr (producer) {
    if (sq[0] < s_end) { score_begin(0, 0); score_finish(); }
  }
  int rb = 0, kP = 0;           // ring buffer of tile b; b itself
  auto wrap = [](int x) { return x >= NS ? x - NS : x; };
  for (;; ++kP) {
    const bool p_active = sq[0] < s_end, c_active = sC < s_end;
    if (!p_active && !c_active) break;
    // tile b + 1 has landed when at most the loads of tiles b + 2 .. b + kAhead - 1 are in flight
    static_assert(AH == 4, "the wait below counts two tiles");
    if constexpr (!producer) {
      const int later = (sq[2] < s_end ? 1 : 0) + (sq[3] < s_end ? 1 : 0);
      if (later == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoads) : "memory");
      else if (later == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    if constexpr (producer) {
      if (p_active) {
        if (sq[1] < s_end) score_begin(wrap(rb + 1), (kP + 1) & (SM::kSets - 1));
        soft_valu(kP & (SM::kSets - 1), kP & 1, fq[0]);
        if (sq[1] < s_end) score_finish();
      }
    } else {
      if (c_active) {
        consume(wrap(rb + NS - 1), (kP - 1) & 1);
      }
      // tile b + kAhead into the buffer tile b - 2 left behind
      if (sq[AH] < s_end) issue(sq[AH], wrap(rb + AH), (kP + AH) & (SM::kSets - 1));
    }
    // next step
    sC = sq[0];
#pragma unroll
    for (int i = 0; i < AH; ++i) { sq[i] = sq[i + 1]; fq[i] = fq[i + 1]; }
    {
      const uint32_t e = (uint32_t)uni((int)pref);
      sq[AH] = step_of(e, kP + 1 + AH);
      fq[AH] = (e >> 31) != 0;
      pref = entry(kP + 2 + AH);
    }
    rb = wrap(rb + 1);
  }

  if constexpr (!producer) if (c < p.NKV) {
    float* krow = dKp + ((int64_t)h * p.NKV + c) * D + 4 * g;
    float* vrow = dVp + ((int64_t)h * p.NKV + c) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const f32x4 wk = {acc_dk[db][r4 * 4 + 0], acc_dk[db][r4 * 4 + 1], acc_dk[db][r4 * 4 + 2], acc_dk[db][r4 * 4 + 3]};
        const f32x4 wv = {acc_dv[db][r4 * 4 + 0], acc_dv[db][r4 * 4 + 1], acc_dv[db][r4 * 4 + 2], acc_dv[db][r4 * 4 + 3]};
        *reinterpret_cast<f32x4*>(krow + db * 32 + 8 * r4) = wk;
        *reinterpret_cast<f32x4*>(vrow + db * 32 + 8 * r4) = wv;
      }
  }
  }  // part
}

template <int D>
__global__ __launch_bounds__(512, 1) void attn_bwd_dkv_ws_kernel(
    AttnParams p, const uint16_t* __restrict__ dO, int NQp, const float* __restrict__ neg,
    const int32_t* __restrict__ mrows, const int32_t* __restrict__ tile_bounds,
    float* __restrict__ dKp, float* __restrict__ dVp) {
  using SM = DkvWsSmem<D>;
  extern __shared__ __attribute__((aligned(16))) uint8_t ws_smem[];
  // ---- the visible query tiles of both key blocks, in order, into LDS (all 512 threads)
  {
    constexpr int KB = 128;
    const int n_kb = (p.NKV + KB - 1) / KB, n_pair = (n_kb + 1) / 2;
    const int pair = (SPX_DKV_XCD && p.Hq % 8 == 0) ? (int)(blockIdx.x >> 3) % n_pair : (int)blockIdx.x / p.Hq;
    const int n_qt = (p.NQ + 63) / 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int* const wtot = reinterpret_cast<int*>(ws_smem + SM::kOffList + 2 * SM::kList);
    for (int part = 0; part < 2; ++part) {
      const int kb_idx = part == 0 ? pair : n_kb - 1 - pair;
      const int n0 = kb_idx * KB, key_last = min(n0 + KB - 1, p.NKV - 1);
      uint32_t* const lst = reinterpret_cast<uint32_t*>(ws_smem + SM::kOffList + part * SM::kList);
      int base = 0;
      for (int q0 = 0; q0 < n_qt; q0 += 512) {
        const int qt = q0 + tid;
        bool vis = false, full = false;
        if (qt < n_qt) {
          const int32_t* tb = tile_bounds + qt * 8;
          vis = (tb[0] <= key_last && tb[3] > n0) || (tb[4] <= key_last && tb[7] > n0);
          full = (tb[1] <= n0 && tb[2] >= n0 + KB) || (tb[5] <= n0 && tb[6] >= n0 + KB);
        }
        const unsigned long long m = __ballot(vis);
        const int before = __popcll(m & ((1ull << lane) - 1));
        if (lane == 0) wtot[wave] = __popcll(m);
        __syncthreads();
        int off = base, all = 0;
        for (int w = 0; w < 8; ++w) {
          if (w < wave) off += wtot[w];
          all += wtot[w];
        }
        if (vis) lst[off + before] = (uint32_t)qt | (full ? 0x80000000u : 0u);
        base += all;
        __syncthreads();
      }
      if (tid == 0) {
        lst[base] = SM::kListEnd;
        wtot[8 + part] = base;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x < 256)
    dkv_ws_role<D, true>(p, dO, NQp, neg, mrows, dKp, dVp);
  else
    dkv_ws_role<D, false>(p, dO, NQp, neg, mrows, dKp, dVp);
}

// dK[kvh, c, :] = scaling * sum_{h in group} dKp[h, c, :],  dV likewise (no scaling); bf16 out.
// `accumulate`: what dK / dV hold is added (in fp32, one rounding).
__global__ __launch_bounds__(256) void attn_dkv_reduce_kernel(
    const float* __restrict__ dKp, const float* __restrict__ dVp, int NKV, int D, int Hq, int Hkv,
    float scaling, uint16_t* __restrict__ dK, int64_t dk_hs, uint16_t* __restrict__ dV, int64_t dv_hs,
    int accumulate) {
  const int64_t per_head = (int64_t)NKV * D / 4;  // float4 items
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_head * Hkv) return;
  const int kvh = (int)(idx / per_head);
  const int64_t off = (idx % per_head) * 4;
  const int group = Hq / Hkv;
  f32x4 sk = {0, 0, 0, 0}, sv = {0, 0, 0, 0};
  for (int hh = 0; hh < group; ++hh) {
    const int64_t base = ((int64_t)(kvh * group + hh) * NKV) * D + off;
    sk += *reinterpret_cast<const f32x4*>(dKp + base);
    sv += *reinterpret_cast<const f32x4*>(dVp + base);
  }
  sk *= scaling;
  u32x2 wk, wv;
  if (accumulate) {
    wk = *reinterpret_cast<const u32x2*>(dK + (int64_t)kvh * dk_hs + off);
    wv = *reinterpret_cast<const u32x2*>(dV + (int64_t)kvh * dv_hs + off);
    sk.x += bf16_lo(wk.x); sk.y += bf16_hi(wk.x); sk.z += bf16_lo(wk.y); sk.w += bf16_hi(wk.y);
    sv.x += bf16_lo(wv.x); sv.y += bf16_hi(wv.x); sv.z += bf16_lo(wv.y); sv.w += bf16_hi(wv.y);
  }
  wk.x = pack_bf16x2(sk.x, sk.y); wk.y = pack_bf16x2(sk.z, sk.w);
  wv.x = pack_bf16x2(sv.x, sv.y); wv.y = pack_bf16x2(sv.z, sv.w);
  *reinterpret_cast<u32x2*>(dK + (int64_t)kvh * dk_hs + off) = wk;
  *reinterpret_cast<u32x2*>(dV + (int64_t)kvh * dv_hs + off) = wv;
}

// dK / dV of the TTT diagonal keys (j, i), j >= 1: sixteen lanes per (position, K/V head)
// item, four items per wave; each such key is seen by exactly the `group` query heads at its
// own position.  A lane holds D / 16 consecutive elements (one or two 16-byte accesses); the dot
// products are summed over the sixteen lanes with DPP moves (no LDS traffic).  The sums over the
// heads of a group stay in fp32 registers until the one store (one rounding to bf16).
// MAXG = query heads per K/V head whose rows are kept in registers: a group of at most MAXG heads
// reads its query / output-gradient rows once for all diagonals; a wider group walks its heads in
// passes of MAXG inside every diagonal (rows re-read per diagonal, from L2).
template <int D, int MAXG>
__global__ __launch_bounds__(256) void ttt_attn_bwd_diag_kernel(
    const uint16_t* __restrict__ Q, int64_t q_hs, const uint16_t* __restrict__ K, int64_t k_hs,
    const uint16_t* __restrict__ V, int64_t v_hs, const uint16_t* __restrict__ dO,
    const float* __restrict__ LSE, const float* __restrict__ Delta, int T, int n_extra, int Hq,
    int Hkv, float scale_log2e, float scaling, uint16_t* dK, int64_t dk_hs, uint16_t* dV,
    int64_t dv_hs, int accumulate) {
  constexpr int EPL = D / 16;
  // item = kvh * T + i: neighbouring 16-lane rows take neighbouring positions of one K/V head, so
  // their key / value / gradient rows are contiguous in memory.  The tail clamps (no early
  // return: the DPP sums need whole rows of lanes)
  const int64_t n_items = (int64_t)T * Hkv;
  const int64_t raw = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + ((threadIdx.x & 63) >> 4);
  const bool live = raw < n_items;
  const int64_t item = live ? raw : n_items - 1;
  const int kvh = (int)(item / T), i = (int)(item % T);
  const int group = Hq / Hkv;
  const int d0 = (threadIdx.x & 15) * EPL;
  const bool one_pass = group <= MAXG;

  float qv[MAXG][EPL], dv[MAXG][EPL], lse_h[MAXG], delta_h[MAXG];
  auto load_heads = [&](int h0, int ng) {
#pragma unroll
    for (int hh = 0; hh < MAXG; ++hh) {
      const int h = kvh * group + h0 + (hh < ng ? hh : 0);
      ld_bf16s<EPL>(Q + (int64_t)h * q_hs + (int64_t)i * D + d0, qv[hh]);
      ld_bf16s<EPL>(dO + ((int64_t)i * Hq + h) * D + d0, dv[hh]);
      lse_h[hh] = LSE[(int64_t)h * T + i];
      delta_h[hh] = Delta[(int64_t)h * T + i];
    }
  };
  if (one_pass) load_heads(0, group);
  // the key / value rows of diagonal j + 1 are requested before diagonal j is worked on: the
  // loop is a chain of dependent global loads otherwise
  float kn[EPL], vn[EPL];
  {
    const int64_t r1 = ((int64_t)T + i) * D + d0;
    ld_bf16s<EPL>(K + (int64_t)kvh * k_hs + r1, kn);
    ld_bf16s<EPL>(V + (int64_t)kvh * v_hs + r1, vn);
  }
  for (int j = 1; j <= n_extra; ++j) {
    const int64_t gko = (int64_t)kvh * dk_hs + ((int64_t)j * T + i) * D + d0;
    const int64_t gvo = (int64_t)kvh * dv_hs + ((int64_t)j * T + i) * D + d0;
    float kv[EPL], vv[EPL], gk[EPL], gv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      kv[e] = kn[e];
      vv[e] = vn[e];
      gk[e] = 0.f;
      gv[e] = 0.f;
    }
    if (accumulate) {  // what the gradient rows hold is the starting value
      ld_bf16s<EPL>(dK + gko, gk);
      ld_bf16s<EPL>(dV + gvo, gv);
    }
    if (j < n_extra) {
      const int64_t rn = ((int64_t)(j + 1) * T + i) * D + d0;
      ld_bf16s<EPL>(K + (int64_t)kvh * k_hs + rn, kn);
      ld_bf16s<EPL>(V + (int64_t)kvh * v_hs + rn, vn);
    }
    for (int h0 = 0; h0 < group; h0 += MAXG) {
      const int ng = min(group - h0, MAXG);
      if (!one_pass) load_heads(h0, ng);
#pragma unroll
      for (int hh = 0; hh < MAXG; ++hh) {
        if (hh < ng) {
          float dot = 0.f, dpv = 0.f;
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            dot = fmaf(qv[hh][e], kv[e], dot);
            dpv = fmaf(dv[hh][e], vv[e], dpv);
          }
          dot = row16_sum(dot);
          dpv = row16_sum(dpv);
          const float pv = fast_exp2(fmaf(dot, scale_log2e, -lse_h[hh]));
          const float ds = pv * (dpv - delta_h[hh]) * scaling;
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            gv[e] = fmaf(pv, dv[hh][e], gv[e]);
            gk[e] = fmaf(ds, qv[hh][e], gk[e]);
          }
        }
      }
    }
    if (live) {
      st_bf16s<EPL>(dK + gko, gk);
      st_bf16s<EPL>(dV + gvo, gv);
    }
  }
}

// ---------------------------------------------------------------- launchers
static int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

#define SPX_FWD_CFG 1, 4, 2
#define SPX_DQ_CFG 1, 4, 4
// head_dim 256: the next tile is prefetched into registers as well; the few registers that
// spill cost far less than exposing the global-load latency with one workgroup per CU
#define SPX_FWD256_PF 2
#define SPX_DQ256_PF 4
#define SPX_DKV_CFG 4, 2
// (sub-blocks per wave, waves per workgroup, register prefetch) of the forward / dQ kernels,
// (waves per workgroup, register prefetch) of the dK/dV kernel
constexpr int cfg_nsb(int nsb, int, int) { return nsb; }
constexpr int cfg_nw(int, int nw, int) { return nw; }
constexpr int cfg_pf(int, int, int pf) { return pf; }
constexpr int cfg_nw(int nw, int) { return nw; }
constexpr int cfg_pf(int, int pf) { return pf; }
constexpr int kFwdNSB = cfg_nsb(SPX_FWD_CFG), kFwdNW = cfg_nw(SPX_FWD_CFG), kFwdPF = cfg_pf(SPX_FWD_CFG);
constexpr int kDqNSB = cfg_nsb(SPX_DQ_CFG), kDqNW = cfg_nw(SPX_DQ_CFG), kDqPF = cfg_pf(SPX_DQ_CFG);
constexpr int kDkvNW = cfg_nw(SPX_DKV_CFG), kDkvPF = cfg_pf(SPX_DKV_CFG);

static int64_t fwd_workspace_bytes(int64_t NKV, int Hkv, int D) {
  return round_up((int64_t)Hkv * D * round_up(NKV, 128) * 2, 256);
}
static int64_t bwd_workspace_bytes(int64_t NQ, int64_t NKV, int Hq, int Hkv, int D) {
  const int64_t NKVp = round_up(NKV, 128), NQp = round_up(NQ, 128);
  int64_t b = (int64_t)Hkv * D * NKVp * 2;          // K^T
  b += 2 * (int64_t)Hq * D * NQp * 2;                // Q^T (scaled), dO^T
  b = round_up(b, 256) + round_up((int64_t)Hq * NQ * 4, 256);       // delta
  b += round_up(((NQ + 63) / 64) * 32, 256);                        // tile bounds
  b += 2 * round_up((int64_t)Hq * NKV * D * 4, 256);                // fp32 per-head dK, dV
  b += round_up((int64_t)Hq * NQ * D * 2, 256);                     // Q scaled, row-major
  b += round_up(2 * (int64_t)Hq * NQp * 4, 256);                    // -lse, -delta in padded rows
  b += round_up(4 * NQp * 4, 256);                                  // interval ends of every row
  return b;
}

template <int D>
static int launch_fwd(AttnParams p, void* workspace, uint16_t* O, float* lse, hipStream_t st,
                      const char* fn) {
  uint16_t* vt = reinterpret_cast<uint16_t*>(workspace);
  dim3 tgrid((unsigned)(p.NKVp / 64), (unsigned)((D + 63) / 64), (unsigned)p.Hkv);
  hipLaunchKernelGGL(transpose_bf16_kernel<false>, tgrid, dim3(64), 0, st, p.V, p.v_hs, (int64_t)D, p.NKV, D,
                     vt, (int64_t)D * p.NKVp, (int64_t)p.NKVp, 1.f, nullptr);
  constexpr int BM = 32 * kFwdNSB * kFwdNW;
  const int n_qb = (p.NQ + BM - 1) / BM;
  constexpr int PF = D > 128 ? (int)SPX_FWD256_PF : kFwdPF;
  constexpr int smem = FwdSmem<D, kFwdNW, PF>::kBytes;
  if (PF == 2 && ((int64_t)p.NKV * D * 2 >= (1ll << 31) || (int64_t)D * p.NKVp * 2 >= (1ll << 31))) {
    last_error() = std::string(fn) + ": keys of one head must span less than 2 GiB";
    return SPX_ERR_ARG;
  }
  static std::atomic<uint64_t> lds_set;  // per head_dim instantiation, one bit per device
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&attn_fwd_kernel<D, kFwdNSB, kFwdNW, PF>),
                                  smem, lds_set, fn))
    return rc;
  hipLaunchKernelGGL((attn_fwd_kernel<D, kFwdNSB, kFwdNW, PF>), dim3((unsigned)(n_qb * p.Hq)),
                     dim3(64 * kFwdNW), smem, st, p, vt, O, lse);
  return check_launch(fn);
}

template <int D>
static int launch_bwd(AttnParams p, const uint16_t* Op, const uint16_t* dOp, const float* lse,
                      uint16_t* dQp, int64_t dq_hs, uint16_t* dKp, int64_t dk_hs, uint16_t* dVp,
                      int64_t dv_hs, void* workspace, hipStream_t st, const char* fn, int accumulate = 0) {
  const int NQp = (int)round_up(p.NQ, 128);
  char* w = reinterpret_cast<char*>(workspace);
  uint16_t* kt = reinterpret_cast<uint16_t*>(w);
  // (the room behind K^T once held Q^T and dO^T; the layout of the workspace has not moved)
  w += round_up(((int64_t)p.Hkv * D * p.NKVp + 2 * (int64_t)p.Hq * D * NQp) * 2, 256);
  float* delta = reinterpret_cast<float*>(w);
  w += round_up((int64_t)p.Hq * p.NQ * 4, 256);
  int32_t* tb = reinterpret_cast<int32_t*>(w);
  w += round_up(((p.NQ + 63) / 64) * 32, 256);
  float* dkp = reinterpret_cast<float*>(w);
  w += round_up((int64_t)p.Hq * p.NKV * D * 4, 256);
  float* dvp = reinterpret_cast<float*>(w);
  w += round_up((int64_t)p.Hq * p.NKV * D * 4, 256);
  uint16_t* qs = reinterpret_cast<uint16_t*>(w);  // bf16(q * scale * log2 e), [Hq][NQ][D]
  w += round_up((int64_t)p.Hq * p.NQ * D * 2, 256);
  float* neg = reinterpret_cast<float*>(w);       // -lse [Hq][NQp], -delta [Hq][NQp]
  w += round_up(2 * (int64_t)p.Hq * NQp * 4, 256);
  int32_t* mrows = reinterpret_cast<int32_t*>(w); // [4][NQp]

  // (the dQ kernel's transposing-read mode takes its K^T fragments from the row-major K tile)
  constexpr bool kNeedKt = (D > 128 ? (int)SPX_DQ256_PF : kDqPF) != 4;
  dim3 tgrid((unsigned)(p.NKVp / 64), (unsigned)((D + 63) / 64), (unsigned)p.Hkv);
  if (kNeedKt)
    hipLaunchKernelGGL(transpose_bf16_kernel<false>, tgrid, dim3(64), 0, st, p.K, p.k_hs, (int64_t)D, p.NKV, D,
                       kt, (int64_t)D * p.NKVp, (int64_t)p.NKVp, 1.f, nullptr);
  dim3 qgrid((unsigned)(NQp / 64), (unsigned)((D + 63) / 64), (unsigned)p.Hq);
  // (neither dK/dV kernel needs Q^T / dO^T: both transpose inside LDS.  The wave-specialised one lists the
  // query tiles that see a key block in LDS, which bounds their number)
  if (D <= 128 && (p.NQ + 63) / 64 > DkvWsSmem<(D <= 128 ? D : 128)>::kListCap) {
    last_error() = std::string(fn) + ": more than " +
                   std::to_string(64 * DkvWsSmem<(D <= 128 ? D : 128)>::kListCap) +
                   " query rows in one call at head_dim <= 128";
    return SPX_ERR_ARG;
  }
  hipLaunchKernelGGL(transpose_bf16_kernel<true>, qgrid, dim3(64), 0, st, p.Q, p.q_hs, (int64_t)D, p.NQ, D,
                     (uint16_t*)nullptr, (int64_t)D * NQp, (int64_t)NQp, p.scale_log2e, qs);
  // the dK/dV and diagonal-key kernels read the scaled queries: their scores are q' . k with no
  // factor of their own, and what they accumulate against q' carries scale * log2(e) once too
  // often: dK = ln 2 * sum dS q'
  AttnParams ps = p;
  ps.Q = qs;
  ps.q_hs = (int64_t)p.NQ * D;
  if (NQp != p.NQ)  // the padding of the negated rows reads as zero
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((2 * (int64_t)p.Hq * NQp + 255) / 256)), dim3(256), 0,
                       st, neg, 2 * (int64_t)p.Hq * NQp);
  hipLaunchKernelGGL(attn_delta_kernel<D>, dim3((unsigned)(((int64_t)p.NQ * p.Hq + 15) / 16)), dim3(256),
                     0, st, Op, dOp, p.NQ, p.Hq, delta, lse, NQp, neg);
  hipLaunchKernelGGL(attn_tile_bounds_kernel, dim3((unsigned)(NQp / 64)), dim3(64), 0, st, p, tb, NQp, mrows);

  constexpr int BM = 32 * kDqNSB * kDqNW;
  const int n_qb = (p.NQ + BM - 1) / BM;
  {
    constexpr int kDqPFd = D > 128 ? (int)SPX_DQ256_PF : kDqPF;
    constexpr int dq_smem = DqSmem<D, kDqNW, kDqPFd>::kBytes;
    if (kDqPFd >= 3 && ((int64_t)p.NKV * D * 2 >= (1ll << 31) || (int64_t)D * p.NKVp * 2 >= (1ll << 31))) {
      last_error() = std::string(fn) + ": keys of one head must span less than 2 GiB";
      return SPX_ERR_ARG;
    }
    static std::atomic<uint64_t> dq_lds_set;  // per head_dim instantiation, one bit per device
    if (int rc = ensure_dynamic_lds(
            reinterpret_cast<const void*>(&attn_bwd_dq_kernel<D, kDqNSB, kDqNW, kDqPFd>), dq_smem,
            dq_lds_set, fn))
      return rc;
    hipLaunchKernelGGL((attn_bwd_dq_kernel<D, kDqNSB, kDqNW, kDqPFd>), dim3((unsigned)(n_qb * p.Hq)),
                       dim3(64 * kDqNW), dq_smem, st, p, dOp, kt, lse, delta, dQp, dq_hs);
  }

  if (D > 128 && (int64_t)p.NQ * p.Hq * D * 2 >= (1ll << 31)) {
    last_error() = std::string(fn) + ": queries must span less than 2 GiB";
    return SPX_ERR_ARG;
  }
  static std::atomic<uint64_t> dkv_lds_set;  // per head_dim instantiation, one bit per device
  if constexpr (D <= 128) {
    // producer / consumer waves, two per SIMD (see attn_bwd_dkv_ws_kernel)
    constexpr int smem = DkvWsSmem<D>::kBytes;
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&attn_bwd_dkv_ws_kernel<D>), smem,
                                    dkv_lds_set, fn))
      return rc;
    const int n_pair_ws = ((p.NKV + 127) / 128 + 1) / 2;  // a workgroup takes two key blocks
    hipLaunchKernelGGL((attn_bwd_dkv_ws_kernel<D>), dim3((unsigned)(n_pair_ws * p.Hq)), dim3(512), smem, st, ps,
                       dOp, NQp, neg, mrows, tb, dkp, dvp);
  } else {
    // dK and dV in one pass over 64-row tiles of Q and dO alone (two buffers of two 32 KB tiles); the
    // transposed operands come out of them through transposing LDS reads
    const int n_kb = (p.NKV + 32 * kDkvNW - 1) / (32 * kDkvNW);
    const dim3 kgrid((unsigned)(n_kb * p.Hq)), kblock(64 * kDkvNW);
    constexpr size_t smem = DkvSmem<D, 0, 64, true>::kBytesDma;
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&attn_bwd_dkv_kernel<D, kDkvNW, 4, 0>),
                                    (int)smem, dkv_lds_set, fn))
      return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<D, kDkvNW, 4, 0>), kgrid, kblock, smem, st, ps, dOp,
                       (const uint16_t*)nullptr, (const uint16_t*)nullptr, NQp, lse, delta, tb, dkp, dvp);
  }
  const int64_t items = (int64_t)p.NKV * D / 4 * p.Hkv;
  hipLaunchKernelGGL(attn_dkv_reduce_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, dkp,
                     dvp, p.NKV, D, p.Hq, p.Hkv, kLn2, dKp, dk_hs, dVp, dv_hs, accumulate);
  if (p.n_extra > 0) {
    const dim3 dgrid((unsigned)(((int64_t)p.T * p.Hkv + 15) / 16));
    // eight heads per K/V head in registers where they fit (head_dim <= 128), else four
    if (D <= 128 && p.Hq / p.Hkv > 4)
      hipLaunchKernelGGL((ttt_attn_bwd_diag_kernel<D, (D <= 128 ? 8 : 4)>), dgrid, dim3(256), 0, st, ps.Q,
                         ps.q_hs, p.K, p.k_hs, p.V, p.v_hs, dOp, lse, delta, p.T, p.n_extra, p.Hq, p.Hkv,
                         1.f, kLn2, dKp, dk_hs, dVp, dv_hs, accumulate);
    else
      hipLaunchKernelGGL((ttt_attn_bwd_diag_kernel<D, 4>), dgrid, dim3(256), 0, st, ps.Q, ps.q_hs, p.K,
                         p.k_hs, p.V, p.v_hs, dOp, lse, delta, p.T, p.n_extra, p.Hq, p.Hkv,
                         1.f, kLn2, dKp, dk_hs, dVp, dv_hs, accumulate);
  }
  return check_launch(fn);
}

static int shape_checks(const char* fn, int64_t NQ, int64_t NKV, int32_t Hq, int32_t Hkv, int32_t D) {
  if (!(NQ > 0 && NQ < (1ll << 24) && NKV > 0 && NKV < (1ll << 26))) return fail_arg(fn, "sequence length out of range");
  if (!(Hkv > 0 && Hq > 0 && Hq % Hkv == 0)) return fail_arg(fn, "Hq must be a multiple of Hkv");
  if (!(D == 64 || D == 128 || D == 256)) return fail_arg(fn, "head_dim must be 64, 128 or 256");
  return SPX_OK;
}

static bool all_aligned16(std::initializer_list<const void*> ps) {
  for (const void* q : ps)
    if (reinterpret_cast<uintptr_t>(q) & 15) return false;
  return true;
}

}  // namespace spx

using namespace spx;

// ================================================================ TTT entry points
extern "C" int spx_ttt_row_lo(const void* document_ids, int doc_kind, int64_t T,
                              int64_t sliding_window, int32_t* row_lo, void* stream) {
  SPX_REQUIRE(doc_kind == SPX_KIND_I32 || doc_kind == SPX_KIND_I64, "document_ids must be int32 or int64");
  SPX_REQUIRE(T > 0 && T < (1ll << 30), "0 < T < 2^30");
  SPX_REQUIRE(document_ids && row_lo, "null buffer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (doc_kind == SPX_KIND_I32)
    hipLaunchKernelGGL(ttt_row_lo_kernel<int32_t>, dim3(1), dim3(1024), 0, st,
                       reinterpret_cast<const int32_t*>(document_ids), T, sliding_window, row_lo);
  else
    hipLaunchKernelGGL(ttt_row_lo_kernel<int64_t>, dim3(1), dim3(1024), 0, st,
                       reinterpret_cast<const int64_t*>(document_ids), T, sliding_window, row_lo);
  return check_launch(__func__);
}

extern "C" int64_t spx_ttt_attn_workspace_bytes(int64_t T, int32_t Hq, int32_t Hkv, int32_t D,
                                                int32_t backward) {
  return backward ? bwd_workspace_bytes(T, T, Hq, Hkv, D) : fwd_workspace_bytes(T, Hkv, D);
}

static AttnParams ttt_params(const void* q, int64_t q_hs, const void* k, int64_t k_hs, const void* v,
                             int64_t v_hs, const int32_t* row_lo, int64_t T, int32_t ttt_step,
                             int32_t Hq, int32_t Hkv, float scaling) {
  AttnParams p;
  p.Q = reinterpret_cast<const uint16_t*>(q); p.q_hs = q_hs;
  p.K = reinterpret_cast<const uint16_t*>(k); p.k_hs = k_hs;
  p.V = reinterpret_cast<const uint16_t*>(v); p.v_hs = v_hs;
  p.a1 = row_lo; p.b1 = nullptr; p.a2 = nullptr; p.b2 = nullptr;
  p.NQ = (int)T; p.T = (int)T; p.NKV = (int)T; p.NKVp = (int)round_up(T, 128);
  p.n_extra = ttt_step; p.Hq = Hq; p.Hkv = Hkv;
  p.scaling = scaling; p.scale_log2e = scaling * kLog2e;
  return p;
}

extern "C" int spx_ttt_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                                int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                const int32_t* row_lo, int64_t T, int32_t ttt_step, int32_t Hq,
                                int32_t Hkv, int32_t D, float scaling, void* out, float* lse,
                                void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = shape_checks(__func__, T, T, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(ttt_step >= 0 && ttt_step < 64, "0 <= ttt_step < 64");
  SPX_REQUIRE(q && k && v && row_lo && out && lse && workspace, "null buffer");
  SPX_REQUIRE(q_head_stride >= T * D, "q head stride smaller than T*D");
  SPX_REQUIRE(k_head_stride >= (int64_t)(ttt_step + 1) * T * D &&
              v_head_stride >= (int64_t)(ttt_step + 1) * T * D,
              "k/v head stride smaller than (ttt_step+1)*T*D");
  SPX_REQUIRE(q_head_stride % 8 == 0 && k_head_stride % 8 == 0 && v_head_stride % 8 == 0,
              "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= fwd_workspace_bytes(T, Hkv, D), "workspace too small");
  SPX_REQUIRE(all_aligned16({q, k, v, out, workspace}), "buffers must be 16-byte aligned");
  AttnParams p = ttt_params(q, q_head_stride, k, k_head_stride, v, v_head_stride, row_lo, T, ttt_step,
                            Hq, Hkv, scaling);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (D == 256) return launch_fwd<256>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
  if (D == 128) return launch_fwd<128>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
  return launch_fwd<64>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
}

#define SPX_REQ_FN(cond, what) do { if (!(cond)) return spx::fail_arg(fname, what); } while (0)
static int ttt_attn_bwd_impl(const char* fname, int accumulate, const void* q, int64_t q_head_stride,
                             const void* k, int64_t k_head_stride, const void* v, int64_t v_head_stride,
                             const void* out, const void* dout, const float* lse, const int32_t* row_lo,
                             int64_t T, int32_t ttt_step, int32_t Hq, int32_t Hkv, int32_t D, float scaling,
                             void* dq, int64_t dq_head_stride, void* dk, int64_t dk_head_stride, void* dv,
                             int64_t dv_head_stride, void* workspace, int64_t workspace_bytes,
                             void* stream) {
  if (int rc = shape_checks(fname, T, T, Hq, Hkv, D)) return rc;
  SPX_REQ_FN(ttt_step >= 0 && ttt_step < 64, "0 <= ttt_step < 64");
  SPX_REQ_FN(q && k && v && out && dout && lse && row_lo && dq && dk && dv && workspace, "null buffer");
  const int64_t kv_rows = (int64_t)(ttt_step + 1) * T * D;
  SPX_REQ_FN(q_head_stride >= T * D && dq_head_stride >= T * D, "q / dq head stride smaller than T*D");
  SPX_REQ_FN(k_head_stride >= kv_rows && v_head_stride >= kv_rows && dk_head_stride >= kv_rows &&
              dv_head_stride >= kv_rows, "k/v/dk/dv head stride smaller than (ttt_step+1)*T*D");
  SPX_REQ_FN((q_head_stride | k_head_stride | v_head_stride | dq_head_stride | dk_head_stride |
               dv_head_stride) % 8 == 0, "head strides must be multiples of 8 elements");
  SPX_REQ_FN(workspace_bytes >= bwd_workspace_bytes(T, T, Hq, Hkv, D), "workspace too small");
  SPX_REQ_FN(all_aligned16({q, k, v, out, dout, dq, dk, dv, workspace}), "buffers must be 16-byte aligned");
  AttnParams p = ttt_params(q, q_head_stride, k, k_head_stride, v, v_head_stride, row_lo, T, ttt_step,
                            Hq, Hkv, scaling);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  auto Op = reinterpret_cast<const uint16_t*>(out);
  auto dOp = reinterpret_cast<const uint16_t*>(dout);
  auto dQp = reinterpret_cast<uint16_t*>(dq);
  auto dKp = reinterpret_cast<uint16_t*>(dk);
  auto dVp = reinterpret_cast<uint16_t*>(dv);
  if (D == 256)
    return launch_bwd<256>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride,
                           workspace, st, fname, accumulate);
  if (D == 128)
    return launch_bwd<128>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp,
                           dv_head_stride, workspace, st, fname, accumulate);
  return launch_bwd<64>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride,
                        workspace, st, fname, accumulate);
}

extern "C" int spx_ttt_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                                int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                const void* out, const void* dout, const float* lse,
                                const int32_t* row_lo, int64_t T, int32_t ttt_step, int32_t Hq,
                                int32_t Hkv, int32_t D, float scaling, void* dq,
                                int64_t dq_head_stride, void* dk, int64_t dk_head_stride, void* dv,
                                int64_t dv_head_stride, void* workspace, int64_t workspace_bytes,
                                void* stream) {
  return ttt_attn_bwd_impl(__func__, 0, q, q_head_stride, k, k_head_stride, v, v_head_stride, out, dout, lse,
                           row_lo, T, ttt_step, Hq, Hkv, D, scaling, dq, dq_head_stride, dk, dk_head_stride,
                           dv, dv_head_stride, workspace, workspace_bytes, stream);
}

extern "C" int spx_ttt_attn_bwd_accumulate(const void* q, int64_t q_head_stride, const void* k,
                                           int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                           const void* out, const void* dout, const float* lse,
                                           const int32_t* row_lo, int64_t T, int32_t ttt_step, int32_t Hq,
                                           int32_t Hkv, int32_t D, float scaling, void* dq,
                                           int64_t dq_head_stride, void* dk, int64_t dk_head_stride,
                                           void* dv, int64_t dv_head_stride, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  return ttt_attn_bwd_impl(__func__, 1, q, q_head_stride, k, k_head_stride, v, v_head_stride, out, dout, lse,
                           row_lo, T, ttt_step, Hq, Hkv, D, scaling, dq, dq_head_stride, dk, dk_head_stride,
                           dv, dv_head_stride, workspace, workspace_bytes, stream);
}

// ================================================================ span attention
// Per query an interval [row_lo, row_hi) of visible keys out of T (no diagonal keys): the mask of a
// padded batch row, where a query sees the non-padding keys up to itself.
static AttnParams span_params(const void* q, int64_t q_hs, const void* k, int64_t k_hs, const void* v,
                              int64_t v_hs, const int32_t* row_lo, const int32_t* row_hi, int64_t T,
                              int32_t Hq, int32_t Hkv, float scaling) {
  AttnParams p = ttt_params(q, q_hs, k, k_hs, v, v_hs, row_lo, T, 0, Hq, Hkv, scaling);
  p.b1 = row_hi;
  return p;
}

extern "C" int spx_span_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                                 int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                 const int32_t* row_lo, const int32_t* row_hi, int64_t T, int32_t Hq,
                                 int32_t Hkv, int32_t D, float scaling, void* out, float* lse,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = shape_checks(__func__, T, T, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(q && k && v && row_lo && row_hi && out && lse && workspace, "null buffer");
  SPX_REQUIRE(q_head_stride >= T * D && k_head_stride >= T * D && v_head_stride >= T * D,
              "head stride smaller than T*D");
  SPX_REQUIRE(q_head_stride % 8 == 0 && k_head_stride % 8 == 0 && v_head_stride % 8 == 0,
              "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= fwd_workspace_bytes(T, Hkv, D), "workspace too small");
  SPX_REQUIRE(all_aligned16({q, k, v, out, workspace}), "buffers must be 16-byte aligned");
  AttnParams p = span_params(q, q_head_stride, k, k_head_stride, v, v_head_stride, row_lo, row_hi, T, Hq,
                             Hkv, scaling);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (D == 256) return launch_fwd<256>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
  if (D == 128) return launch_fwd<128>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
  return launch_fwd<64>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
}

extern "C" int spx_span_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                                 int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                 const void* out, const void* dout, const float* lse,
                                 const int32_t* row_lo, const int32_t* row_hi, int64_t T, int32_t Hq,
                                 int32_t Hkv, int32_t D, float scaling, void* dq,
                                 int64_t dq_head_stride, void* dk, int64_t dk_head_stride, void* dv,
                                 int64_t dv_head_stride, void* workspace, int64_t workspace_bytes,
                                 void* stream) {
  if (int rc = shape_checks(__func__, T, T, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(q && k && v && out && dout && lse && row_lo && row_hi && dq && dk && dv && workspace,
              "null buffer");
  SPX_REQUIRE(q_head_stride >= T * D && dq_head_stride >= T * D && k_head_stride >= T * D &&
              v_head_stride >= T * D && dk_head_stride >= T * D && dv_head_stride >= T * D,
              "head stride smaller than T*D");
  SPX_REQUIRE((q_head_stride | k_head_stride | v_head_stride | dq_head_stride | dk_head_stride |
               dv_head_stride) % 8 == 0, "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= bwd_workspace_bytes(T, T, Hq, Hkv, D), "workspace too small");
  SPX_REQUIRE(all_aligned16({q, k, v, out, dout, dq, dk, dv, workspace}), "buffers must be 16-byte aligned");
  AttnParams p = span_params(q, q_head_stride, k, k_head_stride, v, v_head_stride, row_lo, row_hi, T, Hq,
                             Hkv, scaling);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  auto Op = reinterpret_cast<const uint16_t*>(out);
  auto dOp = reinterpret_cast<const uint16_t*>(dout);
  auto dQp = reinterpret_cast<uint16_t*>(dq);
  auto dKp = reinterpret_cast<uint16_t*>(dk);
  auto dVp = reinterpret_cast<uint16_t*>(dv);
  if (D == 256)
    return launch_bwd<256>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride,
                           workspace, st, __func__);
  if (D == 128)
    return launch_bwd<128>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp,
                           dv_head_stride, workspace, st, __func__);
  return launch_bwd<64>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride,
                        workspace, st, __func__);
}

// ---------------------------------------------------------------- allocation-free variant
// The forward's only scratch is the key-contiguous copy V^T [Hkv, D, round_up(T, 128)].  Here it
// lives in a file-scope device array instead of a caller-owned workspace.  Every GPU holds its
// own copy of the array at its own address: the address is looked up once per device with that
// device current and kept; host code never uses the array's name as a pointer.
constexpr int64_t kStaticScratchBytes = 16ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static int static_scratch(void** out, const char* fn) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    last_error() = std::string(fn) + ": hipGetDevice: " + hipGetErrorString(e);
    return SPX_ERR_HIP;
  }
  if (dev < 0 || dev >= kMaxDevices) return fail_arg(fn, "device ordinal out of range");
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      last_error() = std::string(fn) + ": hipGetSymbolAddress: " + hipGetErrorString(e);
      return SPX_ERR_HIP;
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // same value from every thread
  }
  *out = ptr;
  return SPX_OK;
}

extern "C" int64_t spx_ttt_attn_fwd_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int spx_ttt_attn_fwd_static(const void* q, int64_t q_head_stride, const void* k,
                                       int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                       const int32_t* row_lo, int64_t T, int32_t ttt_step,
                                       int32_t Hq, int32_t Hkv, int32_t D, float scaling, void* out,
                                       float* lse, void* stream) {
  if (int rc = shape_checks(__func__, T, T, Hq, Hkv, D)) return rc;
  if (fwd_workspace_bytes(T, Hkv, D) > kStaticScratchBytes)
    return fail_arg(__func__, "Hkv * D * round_up(T, 128) * 2 bytes exceed the 16 MiB static scratch; "
                              "use spx_ttt_attn_fwd with a caller-owned workspace");
  void* ws = nullptr;
  if (int rc = static_scratch(&ws, __func__)) return rc;
  // every byte of V^T the kernel reads is rewritten by this call's transpose (padding columns
  // included), so nothing of an earlier call has to be cleared
  return spx_ttt_attn_fwd(q, q_head_stride, k, k_head_stride, v, v_head_stride, row_lo, T, ttt_step, Hq,
                          Hkv, D, scaling, out, lse, ws, kStaticScratchBytes, stream);
}

// ================================================================ DFlash entry points
extern "C" int spx_dflash_row_ranges(const void* document_ids, int doc_kind, int64_t T,
                                     const void* anchors, int anchor_kind, int64_t n_anchors,
                                     int32_t block_size, int64_t sliding_window, int32_t causal_block,
                                     int32_t* ctx_lo, int32_t* ctx_hi, int32_t* blk_lo, int32_t* blk_hi,
                                     int32_t* run_start_scratch, void* stream) {
  SPX_REQUIRE(doc_kind == SPX_KIND_I32 || doc_kind == SPX_KIND_I64, "document_ids must be int32 or int64");
  SPX_REQUIRE(anchor_kind == SPX_KIND_I32 || anchor_kind == SPX_KIND_I64, "anchors must be int32 or int64");
  SPX_REQUIRE(T > 0 && T < (1ll << 30) && n_anchors > 0 && block_size > 0, "bad sizes");
  SPX_REQUIRE(n_anchors * block_size < (1ll << 24), "too many block rows");
  SPX_REQUIRE(document_ids && anchors && ctx_lo && ctx_hi && blk_lo && blk_hi && run_start_scratch, "null buffer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const unsigned grid = (unsigned)((n_anchors * block_size + 255) / 256);
#define SPX_RANGES(I, J)                                                                          \
  do {                                                                                            \
    hipLaunchKernelGGL(doc_run_start_kernel<I>, dim3(1), dim3(1024), 0, st,                       \
                       reinterpret_cast<const I*>(document_ids), T, run_start_scratch);           \
    hipLaunchKernelGGL((dflash_ranges_kernel<I, J>), dim3(grid), dim3(256), 0, st,                \
                       reinterpret_cast<const I*>(document_ids), run_start_scratch,               \
                       reinterpret_cast<const J*>(anchors), n_anchors, (int)block_size,           \
                       sliding_window, (int)causal_block, T, ctx_lo, ctx_hi, blk_lo, blk_hi);     \
  } while (0)
  if (doc_kind == SPX_KIND_I32 && anchor_kind == SPX_KIND_I32) SPX_RANGES(int32_t, int32_t);
  else if (doc_kind == SPX_KIND_I32) SPX_RANGES(int32_t, int64_t);
  else if (anchor_kind == SPX_KIND_I32) SPX_RANGES(int64_t, int32_t);
  else SPX_RANGES(int64_t, int64_t);
#undef SPX_RANGES
  return check_launch(__func__);
}

extern "C" int64_t spx_dflash_attn_workspace_bytes(int64_t T, int64_t NQ, int32_t Hq, int32_t Hkv,
                                                   int32_t D, int32_t backward) {
  return backward ? bwd_workspace_bytes(NQ, T + NQ, Hq, Hkv, D) : fwd_workspace_bytes(T + NQ, Hkv, D);
}

static AttnParams dflash_params(const void* q, int64_t q_hs, const void* k, int64_t k_hs, const void* v,
                                int64_t v_hs, const int32_t* a1, const int32_t* b1, const int32_t* a2,
                                const int32_t* b2, int64_t T, int64_t NQ, int32_t Hq, int32_t Hkv,
                                float scaling) {
  AttnParams p;
  p.Q = reinterpret_cast<const uint16_t*>(q); p.q_hs = q_hs;
  p.K = reinterpret_cast<const uint16_t*>(k); p.k_hs = k_hs;
  p.V = reinterpret_cast<const uint16_t*>(v); p.v_hs = v_hs;
  p.a1 = a1; p.b1 = b1; p.a2 = a2; p.b2 = b2;
  p.NQ = (int)NQ; p.T = (int)T; p.NKV = (int)(T + NQ); p.NKVp = (int)round_up(T + NQ, 128);
  p.n_extra = 0; p.Hq = Hq; p.Hkv = Hkv;
  p.scaling = scaling; p.scale_log2e = scaling * kLog2e;
  return p;
}

extern "C" int spx_dflash_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                                   int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                   const int32_t* ctx_lo, const int32_t* ctx_hi, const int32_t* blk_lo,
                                   const int32_t* blk_hi, int64_t T, int64_t NQ, int32_t Hq, int32_t Hkv,
                                   int32_t D, float scaling, void* out, float* lse, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  if (int rc = shape_checks(__func__, NQ, T + NQ, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(T > 0, "T must be positive");
  SPX_REQUIRE(q && k && v && ctx_lo && ctx_hi && blk_lo && blk_hi && out && lse && workspace, "null buffer");
  SPX_REQUIRE(q_head_stride >= NQ * D, "q head stride smaller than NQ*D");
  SPX_REQUIRE(k_head_stride >= (T + NQ) * D && v_head_stride >= (T + NQ) * D,
              "k/v head stride smaller than (T+NQ)*D");
  SPX_REQUIRE(q_head_stride % 8 == 0 && k_head_stride % 8 == 0 && v_head_stride % 8 == 0,
              "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= fwd_workspace_bytes(T + NQ, Hkv, D), "workspace too small");
  SPX_REQUIRE(all_aligned16({q, k, v, out, workspace}), "buffers must be 16-byte aligned");
  AttnParams p = dflash_params(q, q_head_stride, k, k_head_stride, v, v_head_stride, ctx_lo, ctx_hi,
                               blk_lo, blk_hi, T, NQ, Hq, Hkv, scaling);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (D == 256) return launch_fwd<256>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
  if (D == 128) return launch_fwd<128>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
  return launch_fwd<64>(p, workspace, reinterpret_cast<uint16_t*>(out), lse, st, __func__);
}

extern "C" int spx_dflash_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                                   int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                   const void* out, const void* dout, const float* lse,
                                   const int32_t* ctx_lo, const int32_t* ctx_hi, const int32_t* blk_lo,
                                   const int32_t* blk_hi, int64_t T, int64_t NQ, int32_t Hq, int32_t Hkv,
                                   int32_t D, float scaling, void* dq, int64_t dq_head_stride, void* dk,
                                   int64_t dk_head_stride, void* dv, int64_t dv_head_stride,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = shape_checks(__func__, NQ, T + NQ, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(T > 0, "T must be positive");
  SPX_REQUIRE(q && k && v && out && dout && lse && ctx_lo && ctx_hi && blk_lo && blk_hi && dq && dk &&
              dv && workspace, "null buffer");
  SPX_REQUIRE(q_head_stride >= NQ * D && dq_head_stride >= NQ * D, "q / dq head stride smaller than NQ*D");
  const int64_t kv_rows = (T + NQ) * D;
  SPX_REQUIRE(k_head_stride >= kv_rows && v_head_stride >= kv_rows && dk_head_stride >= kv_rows &&
              dv_head_stride >= kv_rows, "k/v/dk/dv head stride smaller than (T+NQ)*D");
  SPX_REQUIRE((q_head_stride | k_head_stride | v_head_stride | dq_head_stride | dk_head_stride |
               dv_head_stride) % 8 == 0, "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= bwd_workspace_bytes(NQ, T + NQ, Hq, Hkv, D), "workspace too small");
  SPX_REQUIRE(all_aligned16({q, k, v, out, dout, dq, dk, dv, workspace}), "buffers must be 16-byte aligned");
  AttnParams p = dflash_params(q, q_head_stride, k, k_head_stride, v, v_head_stride, ctx_lo, ctx_hi,
                               blk_lo, blk_hi, T, NQ, Hq, Hkv, scaling);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  auto Op = reinterpret_cast<const uint16_t*>(out);
  auto dOp = reinterpret_cast<const uint16_t*>(dout);
  auto dQp = reinterpret_cast<uint16_t*>(dq);
  auto dKp = reinterpret_cast<uint16_t*>(dk);
  auto dVp = reinterpret_cast<uint16_t*>(dv);
  if (D == 256)
    return launch_bwd<256>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride,
                           workspace, st, __func__);
  if (D == 128)
    return launch_bwd<128>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp,
                           dv_head_stride, workspace, st, __func__);
  return launch_bwd<64>(p, Op, dOp, lse, dQp, dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride,
                        workspace, st, __func__);
}
