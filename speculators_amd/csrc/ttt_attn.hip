// EAGLE3 test-time-training attention for gfx950.
//
// At TTT step k a query at position i attends to
//   * context keys c of the step-0 K/V with row_lo[i] <= c <= i (causal, same
//     document, optional sliding window; a padding row sees only c == i), and
//   * ONE key per later step j = 1..k: the key at its own position, (j, i).
// The context part is a flash-attention loop over 64-key tiles with the tiles
// outside [min row_lo, last row] of the 128-row block skipped analytically; the
// k diagonal keys are folded into the same online soft-max as k extra
// length-D dot products per row, instead of k more 128x128 mask blocks.

#include "attn_common.h"
#include "../../include/spx.h"

namespace spx {

// ---------------------------------------------------------------- row_lo
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

// ---------------------------------------------------------------- transpose
// dst[h][c][r] = src[h][r][c] for r < rows, c < cols; dst row stride ld_dst >= rows,
// columns rows..ld_dst-1 of dst are zero filled.  64x64 tiles through LDS.
__global__ __launch_bounds__(256) void transpose_bf16_kernel(
    const uint16_t* __restrict__ src, int64_t src_hs, int64_t src_ld, int rows, int cols,
    uint16_t* __restrict__ dst, int64_t dst_hs, int64_t ld_dst) {
  __shared__ uint16_t tile[64][66];
  const int h = blockIdx.z;
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const uint16_t* s = src + (int64_t)h * src_hs;
  uint16_t* d = dst + (int64_t)h * dst_hs;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int rr = ty; rr < 64; rr += 4) {
    int r = r0 + rr, c = c0 + tx;
    tile[rr][tx] = (r < rows && c < cols) ? s[(int64_t)r * src_ld + c] : (uint16_t)0;
  }
  __syncthreads();
  for (int cc = ty; cc < 64; cc += 4) {
    int c = c0 + cc, r = r0 + tx;
    if (c < cols && r < ld_dst) d[(int64_t)c * ld_dst + r] = tile[tx][cc];
  }
}

// ---------------------------------------------------------------- forward
template <int D>
__global__ __launch_bounds__(kAttnThreads) void ttt_attn_fwd_kernel(
    const uint16_t* __restrict__ Q, int64_t q_hs, const uint16_t* __restrict__ K, int64_t k_hs,
    const uint16_t* __restrict__ V, int64_t v_hs, const uint16_t* __restrict__ Vt,
    const int32_t* __restrict__ row_lo, int T, int Tp, int n_extra, int Hq, int Hkv,
    float scale_log2e, uint16_t* __restrict__ O, float* __restrict__ LSE) {
  constexpr int KS = D + kKPad;    // K tile row stride (elements)
  constexpr int VS = kBN + kVPad;  // V^T tile row stride
  constexpr int NKK = D / 16;      // k-steps of the score product
  constexpr int NDB = D / 32;      // 32-row blocks of O^T
  constexpr int CPT = D / 32;      // 16-byte chunks per thread per tile

  __shared__ __attribute__((aligned(16))) uint16_t Ks[kBN * KS];
  __shared__ __attribute__((aligned(16))) uint16_t Vs[D * VS];
  __shared__ int lo_red[4];

  // tile -> (kv head, query head, query block); heavy (late) blocks first, and
  // consecutive workgroup ids walk the kv heads so that the heads sharing a
  // K/V head meet on one XCD's L2
  const int group = Hq / Hkv;
  const int L = blockIdx.x;
  const int kvh = L % Hkv;
  const int rest = L / Hkv;
  const int h = kvh * group + rest % group;
  const int n_qb = (T + kBM - 1) / kBM;
  const int qb = n_qb - 1 - rest / group;
  const int m0 = qb * kBM;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, col = lane & 31;
  const int mw = m0 + wave * 32;  // first row of this wave
  const int i = mw + col;         // this lane's query row
  const int ic = i < T ? i : T - 1;
  const int my_lo = row_lo[ic];

  // block / wave extents of the visible context
  int wlo_min = my_lo, wlo_max = my_lo;
#pragma unroll
  for (int m = 16; m >= 1; m >>= 1) {
    wlo_min = min(wlo_min, __shfl_xor(wlo_min, m, 64));
    wlo_max = max(wlo_max, __shfl_xor(wlo_max, m, 64));
  }
  if (lane == 0) lo_red[wave] = wlo_min;
  __syncthreads();
  const int blk_lo = min(min(lo_red[0], lo_red[1]), min(lo_red[2], lo_red[3]));
  const int n_begin = (blk_lo / kBN) * kBN;
  const int n_last = min(m0 + kBM - 1, T - 1);

  // Q fragment: B operand, lane = (query col, k half g)
  bf16x8 qf[NKK];
  {
    const uint16_t* qrow = Q + (int64_t)h * q_hs + (int64_t)ic * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) qf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(qrow + kk * 16));
  }

  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
  float m_run = kNegBig, l_run = 0.f;

  const uint16_t* Kh = K + (int64_t)kvh * k_hs;
  const uint16_t* Vth = Vt + (int64_t)kvh * D * Tp;

  u32x4 kreg[CPT], vreg[CPT];
  auto fetch = [&](int n0) {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + kAttnThreads * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      const int kr = min(n0 + krow, T - 1);
      kreg[n] = *reinterpret_cast<const u32x4*>(Kh + (int64_t)kr * D + kcol);
      const int vd = c >> 3, vcol = (c & 7) * 8;
      vreg[n] = *reinterpret_cast<const u32x4*>(Vth + (int64_t)vd * Tp + n0 + vcol);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + kAttnThreads * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      *reinterpret_cast<u32x4*>(&Ks[krow * KS + kcol]) = kreg[n];
      const int vd = c >> 3, vcol = (c & 7) * 8;
      u32x2 a = {vreg[n].x, vreg[n].y}, b = {vreg[n].z, vreg[n].w};
      *reinterpret_cast<u32x2*>(&Vs[vd * VS + vcol]) = a;
      *reinterpret_cast<u32x2*>(&Vs[vd * VS + vcol + 4]) = b;
    }
  };

  if (n_begin <= n_last) fetch(n_begin);
  for (int n0 = n_begin; n0 <= n_last; n0 += kBN) {
    __syncthreads();
    stash();
    __syncthreads();
    if (n0 + kBN <= n_last) fetch(n0 + kBN);
    if (n0 > mw + 31 || n0 + kBN <= wlo_min) continue;  // nothing visible for this wave

    f32x16 st[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[kb][r] = 0.f;
      const uint16_t* krow = &Ks[(kb * 32 + col) * KS + g * 8];
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk)
        st[kb] = mfma32(as_bf16x8(*reinterpret_cast<const u32x4*>(krow + kk * 16)), qf[kk], st[kb]);
    }
    const bool need_mask = (n0 + kBN - 1 > mw) || (n0 < wlo_max);
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float s = st[kb][r] * scale_log2e;
        if (need_mask) {
          const int c = n0 + kb * 32 + acc_row(r, g);
          if (c < my_lo || c > i) s = -INFINITY;
        }
        st[kb][r] = s;
        mx = fmaxf(mx, s);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = fast_exp2(m_run - m_new);
    float rs = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = fast_exp2(st[kb][r] - m_new);
        st[kb][r] = p;
        rs += p;
      }
    rs += __shfl_xor(rs, 32, 64);
    l_run = l_run * alpha + rs;
    m_run = m_new;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[db][r] *= alpha;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bf16x8 pb = pack8(st[s >> 1], (s & 1) * 8);
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        const uint16_t* vrow = &Vs[(db * 32 + col) * VS + s * 16 + 4 * g];
        const bf16x8 va = join_bf16x4(*reinterpret_cast<const u32x2*>(vrow),
                                      *reinterpret_cast<const u32x2*>(vrow + 8));
        acc[db] = mfma32(va, pb, acc[db]);
      }
    }
  }

  // the k diagonal keys (j, i), j = 1..k: one dot product each
  for (int j = 1; j <= n_extra; ++j) {
    const uint16_t* kj = K + (int64_t)kvh * k_hs + ((int64_t)j * T + ic) * D + g * 8;
    float dot = 0.f;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      float kv[8];
      unpack8(*reinterpret_cast<const u32x4*>(kj + kk * 16), kv);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = fmaf((float)qf[kk][e], kv[e], dot);
    }
    dot += __shfl_xor(dot, 32, 64);
    const float s = dot * scale_log2e;
    const float m_new = fmaxf(m_run, s);
    const float alpha = fast_exp2(m_run - m_new);
    const float p = fast_exp2(s - m_new);
    l_run = l_run * alpha + p;
    m_run = m_new;
    const uint16_t* vj = V + (int64_t)kvh * v_hs + ((int64_t)j * T + ic) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        float vv[4];
        unpack4(*reinterpret_cast<const u32x2*>(vj + db * 32 + 8 * r4), vv);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[db][r4 * 4 + t] = fmaf(p, vv[t], acc[db][r4 * 4 + t] * alpha);
      }
  }

  if (i < T) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    uint16_t* orow = O + ((int64_t)i * Hq + h) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2 w;
        w.x = pack_bf16x2(acc[db][r4 * 4 + 0] * inv, acc[db][r4 * 4 + 1] * inv);
        w.y = pack_bf16x2(acc[db][r4 * 4 + 2] * inv, acc[db][r4 * 4 + 3] * inv);
        *reinterpret_cast<u32x2*>(orow + db * 32 + 8 * r4) = w;
      }
    if (g == 0) LSE[(int64_t)h * T + i] = m_run + fast_log2(l_run);
  }
}

static int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

// ---------------------------------------------------------------- backward
// delta[h, i] = sum_d dO[i, h, d] * O[i, h, d]
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const uint16_t* __restrict__ O,
                                                         const uint16_t* __restrict__ dO, int T,
                                                         int Hq, float* __restrict__ delta) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // = i * Hq + h
  if (row >= (int64_t)T * Hq) return;
  const int lane = threadIdx.x & 63;
  float acc = 0.f;
  for (int d = lane * 2; d < D; d += 128) {
    uint32_t a = *reinterpret_cast<const uint32_t*>(O + row * D + d);
    uint32_t b = *reinterpret_cast<const uint32_t*>(dO + row * D + d);
    acc = fmaf(bf16_lo(a), bf16_lo(b), acc);
    acc = fmaf(bf16_hi(a), bf16_hi(b), acc);
  }
  acc = wave_sum(acc);
  if (lane == 0) delta[(row % Hq) * (int64_t)T + row / Hq] = acc;
}

// dQ: one workgroup = 128 query rows of one head, loop over the visible key tiles.
//   P^T = exp2(S'^T - lse), dP^T = V dO^T, dS^T = P^T (dP^T - delta), dQ^T += K^T dS^T
template <int D>
__global__ __launch_bounds__(kAttnThreads) void ttt_attn_bwd_dq_kernel(
    const uint16_t* __restrict__ Q, int64_t q_hs, const uint16_t* __restrict__ K, int64_t k_hs,
    const uint16_t* __restrict__ V, int64_t v_hs, const uint16_t* __restrict__ dO,
    const uint16_t* __restrict__ Kt, const float* __restrict__ LSE, const float* __restrict__ Delta,
    const int32_t* __restrict__ row_lo, int T, int Tp, int n_extra, int Hq, int Hkv,
    float scale_log2e, float scaling, uint16_t* __restrict__ dQ, int64_t dq_hs) {
  constexpr int KS = D + kKPad;
  constexpr int VS = kBN + kVPad;
  constexpr int NKK = D / 16;
  constexpr int NDB = D / 32;
  constexpr int CPT = D / 32;

  __shared__ __attribute__((aligned(16))) uint16_t Ks[kBN * KS];
  __shared__ __attribute__((aligned(16))) uint16_t Vn[kBN * KS];
  __shared__ __attribute__((aligned(16))) uint16_t Kts[D * VS];
  __shared__ int lo_red[4];

  const int group = Hq / Hkv;
  const int L = blockIdx.x;
  const int kvh = L % Hkv;
  const int rest = L / Hkv;
  const int h = kvh * group + rest % group;
  const int n_qb = (T + kBM - 1) / kBM;
  const int qb = n_qb - 1 - rest / group;
  const int m0 = qb * kBM;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, col = lane & 31;
  const int mw = m0 + wave * 32;
  const int i = mw + col;
  const int ic = i < T ? i : T - 1;
  const int my_lo = row_lo[ic];
  const float lse_i = LSE[(int64_t)h * T + ic];
  const float delta_i = Delta[(int64_t)h * T + ic];

  int wlo_min = my_lo, wlo_max = my_lo;
#pragma unroll
  for (int m = 16; m >= 1; m >>= 1) {
    wlo_min = min(wlo_min, __shfl_xor(wlo_min, m, 64));
    wlo_max = max(wlo_max, __shfl_xor(wlo_max, m, 64));
  }
  if (lane == 0) lo_red[wave] = wlo_min;
  __syncthreads();
  const int blk_lo = min(min(lo_red[0], lo_red[1]), min(lo_red[2], lo_red[3]));
  const int n_begin = (blk_lo / kBN) * kBN;
  const int n_last = min(m0 + kBM - 1, T - 1);

  bf16x8 qf[NKK], dof[NKK];
  {
    const uint16_t* qrow = Q + (int64_t)h * q_hs + (int64_t)ic * D + g * 8;
    const uint16_t* drow = dO + ((int64_t)ic * Hq + h) * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      qf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(qrow + kk * 16));
      dof[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(drow + kk * 16));
    }
  }

  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  const uint16_t* Kh = K + (int64_t)kvh * k_hs;
  const uint16_t* Vh = V + (int64_t)kvh * v_hs;
  const uint16_t* Kth = Kt + (int64_t)kvh * D * Tp;

  for (int n0 = n_begin; n0 <= n_last; n0 += kBN) {
    __syncthreads();
#pragma unroll
    for (int n = 0; n < CPT; ++n) {
      const int c = tid + kAttnThreads * n;
      const int krow = c / (D / 8), kcol = (c % (D / 8)) * 8;
      const int kr = min(n0 + krow, T - 1);
      *reinterpret_cast<u32x4*>(&Ks[krow * KS + kcol]) =
          *reinterpret_cast<const u32x4*>(Kh + (int64_t)kr * D + kcol);
      *reinterpret_cast<u32x4*>(&Vn[krow * KS + kcol]) =
          *reinterpret_cast<const u32x4*>(Vh + (int64_t)kr * D + kcol);
      const int vd = c >> 3, vcol = (c & 7) * 8;
      u32x4 t = *reinterpret_cast<const u32x4*>(Kth + (int64_t)vd * Tp + n0 + vcol);
      u32x2 a = {t.x, t.y}, b = {t.z, t.w};
      *reinterpret_cast<u32x2*>(&Kts[vd * VS + vcol]) = a;
      *reinterpret_cast<u32x2*>(&Kts[vd * VS + vcol + 4]) = b;
    }
    __syncthreads();
    if (n0 > mw + 31 || n0 + kBN <= wlo_min) continue;

    f32x16 st[2], dp[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) { st[kb][r] = 0.f; dp[kb][r] = 0.f; }
      const uint16_t* krow = &Ks[(kb * 32 + col) * KS + g * 8];
      const uint16_t* vrow = &Vn[(kb * 32 + col) * KS + g * 8];
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        st[kb] = mfma32(as_bf16x8(*reinterpret_cast<const u32x4*>(krow + kk * 16)), qf[kk], st[kb]);
        dp[kb] = mfma32(as_bf16x8(*reinterpret_cast<const u32x4*>(vrow + kk * 16)), dof[kk], dp[kb]);
      }
    }
    const bool need_mask = (n0 + kBN - 1 > mw) || (n0 < wlo_max);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = fast_exp2(fmaf(st[kb][r], scale_log2e, -lse_i));
        if (need_mask) {
          const int c = n0 + kb * 32 + acc_row(r, g);
          if (c < my_lo || c > i) p = 0.f;
        }
        dp[kb][r] = p * (dp[kb][r] - delta_i);
      }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bf16x8 db8 = pack8(dp[s >> 1], (s & 1) * 8);
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        const uint16_t* trow = &Kts[(db * 32 + col) * VS + s * 16 + 4 * g];
        const bf16x8 ka = join_bf16x4(*reinterpret_cast<const u32x2*>(trow),
                                      *reinterpret_cast<const u32x2*>(trow + 8));
        acc[db] = mfma32(ka, db8, acc[db]);
      }
    }
  }

  for (int j = 1; j <= n_extra; ++j) {
    const uint16_t* kj = K + (int64_t)kvh * k_hs + ((int64_t)j * T + ic) * D;
    const uint16_t* vj = V + (int64_t)kvh * v_hs + ((int64_t)j * T + ic) * D;
    float dot = 0.f, dpv = 0.f;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      float kv[8], vv[8];
      unpack8(*reinterpret_cast<const u32x4*>(kj + g * 8 + kk * 16), kv);
      unpack8(*reinterpret_cast<const u32x4*>(vj + g * 8 + kk * 16), vv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        dot = fmaf((float)qf[kk][e], kv[e], dot);
        dpv = fmaf((float)dof[kk][e], vv[e], dpv);
      }
    }
    dot += __shfl_xor(dot, 32, 64);
    dpv += __shfl_xor(dpv, 32, 64);
    const float p = fast_exp2(fmaf(dot, scale_log2e, -lse_i));
    const float ds = p * (dpv - delta_i);
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        float kk4[4];
        unpack4(*reinterpret_cast<const u32x2*>(kj + 4 * g + db * 32 + 8 * r4), kk4);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[db][r4 * 4 + t] = fmaf(ds, kk4[t], acc[db][r4 * 4 + t]);
      }
  }

  if (i < T) {
    uint16_t* orow = dQ + (int64_t)h * dq_hs + (int64_t)i * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2 w;
        w.x = pack_bf16x2(acc[db][r4 * 4 + 0] * scaling, acc[db][r4 * 4 + 1] * scaling);
        w.y = pack_bf16x2(acc[db][r4 * 4 + 2] * scaling, acc[db][r4 * 4 + 3] * scaling);
        *reinterpret_cast<u32x2*>(orow + db * 32 + 8 * r4) = w;
      }
  }
}

// dK / dV of the context keys: one workgroup = 128 keys of one K/V head (a wave
// owns 32 keys: lane column = key), loop over the query heads of the group and
// over the 64-row query tiles that can see the block.  Scores are produced in
// the S = Q K^T orientation here so that a lane holds one KEY:
//   dV^T += dO^T P,   dK^T += Q^T dS,   dS = P (dO V^T - delta)
template <int D>
__global__ __launch_bounds__(kAttnThreads) void ttt_attn_bwd_dkv_kernel(
    const uint16_t* __restrict__ Q, int64_t q_hs, const uint16_t* __restrict__ K, int64_t k_hs,
    const uint16_t* __restrict__ V, int64_t v_hs, const uint16_t* __restrict__ dO,
    const uint16_t* __restrict__ Qt, const uint16_t* __restrict__ dOt,
    const float* __restrict__ LSE, const float* __restrict__ Delta,
    const int32_t* __restrict__ row_lo, int T, int Tp, int Hq, int Hkv, float scale_log2e,
    float scaling, uint16_t* __restrict__ dK, int64_t dk_hs, uint16_t* __restrict__ dV,
    int64_t dv_hs) {
  constexpr int QS = D + kKPad;
  constexpr int TS = 64 + kVPad;
  constexpr int NKK = D / 16;
  constexpr int NDB = D / 32;
  constexpr int CPT = D / 32;  // 16-byte chunks per thread per 64 x D tile

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* Qs = smem;                 // [64][QS]
  uint16_t* dOs = Qs + 64 * QS;        // [64][QS]
  uint16_t* Qts = dOs + 64 * QS;       // [D][TS]
  uint16_t* dOts = Qts + D * TS;       // [D][TS]
  float* lse_s = reinterpret_cast<float*>(dOts + D * TS);  // [64]
  float* delta_s = lse_s + 64;                               // [64]
  int* lo_s = reinterpret_cast<int*>(delta_s + 64);          // [64]

  const int group = Hq / Hkv;
  const int kvh = blockIdx.x % Hkv;
  const int kb_idx = blockIdx.x / Hkv;
  const int n0 = kb_idx * 128;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, col = lane & 31;
  const int cw = n0 + wave * 32;  // first key of this wave
  const int c = cw + col;         // this lane's key
  const int cc = c < T ? c : T - 1;

  bf16x8 kf[NKK], vf[NKK];
  {
    const uint16_t* krow = K + (int64_t)kvh * k_hs + (int64_t)cc * D + g * 8;
    const uint16_t* vrow = V + (int64_t)kvh * v_hs + (int64_t)cc * D + g * 8;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      kf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(krow + kk * 16));
      vf[kk] = as_bf16x8(*reinterpret_cast<const u32x4*>(vrow + kk * 16));
    }
  }
  f32x16 acc_dk[NDB], acc_dv[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc_dk[db][r] = 0.f; acc_dv[db][r] = 0.f; }

  const int key_last = min(n0 + 127, T - 1);
  for (int hh = 0; hh < group; ++hh) {
    const int h = kvh * group + hh;
    const uint16_t* Qh = Q + (int64_t)h * q_hs;
    const uint16_t* Qth = Qt + (int64_t)h * D * Tp;
    const uint16_t* dOth = dOt + (int64_t)h * D * Tp;
    for (int mq = (n0 / 64) * 64; mq < T; mq += 64) {
      // row_lo is non-decreasing: once the first row of a tile starts after this
      // key block, no later row sees it
      if (row_lo[mq] > key_last) break;
      __syncthreads();
#pragma unroll
      for (int n = 0; n < CPT; ++n) {
        const int ch = tid + kAttnThreads * n;
        const int qr = ch / (D / 8), qc = (ch % (D / 8)) * 8;
        const int ir = min(mq + qr, T - 1);
        *reinterpret_cast<u32x4*>(&Qs[qr * QS + qc]) =
            *reinterpret_cast<const u32x4*>(Qh + (int64_t)ir * D + qc);
        *reinterpret_cast<u32x4*>(&dOs[qr * QS + qc]) =
            *reinterpret_cast<const u32x4*>(dO + ((int64_t)ir * Hq + h) * D + qc);
        const int td = ch >> 3, tc = (ch & 7) * 8;
        u32x4 a = *reinterpret_cast<const u32x4*>(Qth + (int64_t)td * Tp + mq + tc);
        u32x4 b = *reinterpret_cast<const u32x4*>(dOth + (int64_t)td * Tp + mq + tc);
        u32x2 a0 = {a.x, a.y}, a1 = {a.z, a.w}, b0 = {b.x, b.y}, b1 = {b.z, b.w};
        *reinterpret_cast<u32x2*>(&Qts[td * TS + tc]) = a0;
        *reinterpret_cast<u32x2*>(&Qts[td * TS + tc + 4]) = a1;
        *reinterpret_cast<u32x2*>(&dOts[td * TS + tc]) = b0;
        *reinterpret_cast<u32x2*>(&dOts[td * TS + tc + 4]) = b1;
      }
      if (tid < 64) {
        const int ir = mq + tid;
        const bool ok = ir < T;
        lse_s[tid] = ok ? LSE[(int64_t)h * T + ir] : 0.f;
        delta_s[tid] = ok ? Delta[(int64_t)h * T + ir] : 0.f;
        lo_s[tid] = ok ? row_lo[ir] : 0x7fffffff;
      }
      __syncthreads();
      if (mq + 63 < cw) continue;  // every row of the tile precedes this wave's keys

      f32x16 st[2], dp[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) { st[qb][r] = 0.f; dp[qb][r] = 0.f; }
        const uint16_t* qrow = &Qs[(qb * 32 + col) * QS + g * 8];
        const uint16_t* drow = &dOs[(qb * 32 + col) * QS + g * 8];
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
          st[qb] = mfma32(as_bf16x8(*reinterpret_cast<const u32x4*>(qrow + kk * 16)), kf[kk], st[qb]);
          dp[qb] = mfma32(as_bf16x8(*reinterpret_cast<const u32x4*>(drow + kk * 16)), vf[kk], dp[qb]);
        }
      }
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int qi = qb * 32 + acc_row(r, g);
          const int irow = mq + qi;
          const bool ok = (c >= lo_s[qi]) && (c <= irow) && (c < T);
          const float p = ok ? fast_exp2(fmaf(st[qb][r], scale_log2e, -lse_s[qi])) : 0.f;
          st[qb][r] = p;
          dp[qb][r] = p * (dp[qb][r] - delta_s[qi]);
        }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const bf16x8 pb = pack8(st[s >> 1], (s & 1) * 8);
        const bf16x8 sb = pack8(dp[s >> 1], (s & 1) * 8);
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const uint16_t* arow = &dOts[(db * 32 + col) * TS + s * 16 + 4 * g];
          const uint16_t* brow = &Qts[(db * 32 + col) * TS + s * 16 + 4 * g];
          acc_dv[db] = mfma32(join_bf16x4(*reinterpret_cast<const u32x2*>(arow),
                                          *reinterpret_cast<const u32x2*>(arow + 8)), pb, acc_dv[db]);
          acc_dk[db] = mfma32(join_bf16x4(*reinterpret_cast<const u32x2*>(brow),
                                          *reinterpret_cast<const u32x2*>(brow + 8)), sb, acc_dk[db]);
        }
      }
    }
  }

  if (c < T) {
    uint16_t* krow = dK + (int64_t)kvh * dk_hs + (int64_t)c * D + 4 * g;
    uint16_t* vrow = dV + (int64_t)kvh * dv_hs + (int64_t)c * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2 w;
        w.x = pack_bf16x2(acc_dk[db][r4 * 4 + 0] * scaling, acc_dk[db][r4 * 4 + 1] * scaling);
        w.y = pack_bf16x2(acc_dk[db][r4 * 4 + 2] * scaling, acc_dk[db][r4 * 4 + 3] * scaling);
        *reinterpret_cast<u32x2*>(krow + db * 32 + 8 * r4) = w;
        w.x = pack_bf16x2(acc_dv[db][r4 * 4 + 0], acc_dv[db][r4 * 4 + 1]);
        w.y = pack_bf16x2(acc_dv[db][r4 * 4 + 2], acc_dv[db][r4 * 4 + 3]);
        *reinterpret_cast<u32x2*>(vrow + db * 32 + 8 * r4) = w;
      }
  }
}

// dK / dV of the diagonal keys (j, i), j >= 1: one wave per (position, K/V head);
// each such key is seen by exactly the `group` query heads at its own position.
template <int D>
__global__ __launch_bounds__(256) void ttt_attn_bwd_diag_kernel(
    const uint16_t* __restrict__ Q, int64_t q_hs, const uint16_t* __restrict__ K, int64_t k_hs,
    const uint16_t* __restrict__ V, int64_t v_hs, const uint16_t* __restrict__ dO,
    const float* __restrict__ LSE, const float* __restrict__ Delta, int T, int n_extra, int Hq,
    int Hkv, float scale_log2e, float scaling, uint16_t* __restrict__ dK, int64_t dk_hs,
    uint16_t* __restrict__ dV, int64_t dv_hs) {
  constexpr int EPL = D / 64;  // elements per lane
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // = i * Hkv + kvh
  if (item >= (int64_t)T * Hkv) return;
  const int lane = threadIdx.x & 63;
  const int i = (int)(item / Hkv), kvh = (int)(item % Hkv);
  const int group = Hq / Hkv;
  const int d0 = lane * EPL;
  for (int j = 1; j <= n_extra; ++j) {
    const int64_t krow = (int64_t)kvh * k_hs + ((int64_t)j * T + i) * D + d0;
    const int64_t vrow = (int64_t)kvh * v_hs + ((int64_t)j * T + i) * D + d0;
    float kv[EPL], vv[EPL], gk[EPL], gv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      kv[e] = bf16_bits_to_f32(K[krow + e]);
      vv[e] = bf16_bits_to_f32(V[vrow + e]);
      gk[e] = 0.f; gv[e] = 0.f;
    }
    for (int hh = 0; hh < group; ++hh) {
      const int h = kvh * group + hh;
      float qv[EPL], dv[EPL];
      float dot = 0.f, dpv = 0.f;
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        qv[e] = bf16_bits_to_f32(Q[(int64_t)h * q_hs + (int64_t)i * D + d0 + e]);
        dv[e] = bf16_bits_to_f32(dO[((int64_t)i * Hq + h) * D + d0 + e]);
        dot = fmaf(qv[e], kv[e], dot);
        dpv = fmaf(dv[e], vv[e], dpv);
      }
      dot = wave_sum(dot);
      dpv = wave_sum(dpv);
      const float p = fast_exp2(fmaf(dot, scale_log2e, -LSE[(int64_t)h * T + i]));
      const float ds = p * (dpv - Delta[(int64_t)h * T + i]) * scaling;
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        gv[e] = fmaf(p, dv[e], gv[e]);
        gk[e] = fmaf(ds, qv[e], gk[e]);
      }
    }
    const int64_t gko = (int64_t)kvh * dk_hs + ((int64_t)j * T + i) * D + d0;
    const int64_t gvo = (int64_t)kvh * dv_hs + ((int64_t)j * T + i) * D + d0;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      dK[gko + e] = (uint16_t)f32_to_bf16_bits(gk[e]);
      dV[gvo + e] = (uint16_t)f32_to_bf16_bits(gv[e]);
    }
  }
}

template <int D>
static int launch_bwd_all(const uint16_t* Qp, int64_t q_hs, const uint16_t* Kp, int64_t k_hs,
                          const uint16_t* Vp, int64_t v_hs, const uint16_t* Op, const uint16_t* dOp,
                          const float* lse, const int32_t* row_lo, int T, int n_extra, int Hq, int Hkv,
                          float scaling, uint16_t* dQp, int64_t dq_hs, uint16_t* dKp, int64_t dk_hs,
                          uint16_t* dVp, int64_t dv_hs, void* workspace, hipStream_t st) {
  const int Tp = (int)((T + kBM - 1) / kBM * kBM);
  uint16_t* kt = reinterpret_cast<uint16_t*>(workspace);
  uint16_t* qt = kt + (int64_t)Hkv * D * Tp;
  uint16_t* dot = qt + (int64_t)Hq * D * Tp;
  float* delta = reinterpret_cast<float*>(dot + (int64_t)Hq * D * Tp);
  const float sl2 = scaling * kLog2e;
  dim3 tgrid((unsigned)(Tp / 64), (unsigned)((D + 63) / 64), (unsigned)Hkv);
  hipLaunchKernelGGL(transpose_bf16_kernel, tgrid, dim3(256), 0, st, Kp, k_hs, (int64_t)D, T, D, kt,
                     (int64_t)D * Tp, (int64_t)Tp);
  tgrid.z = Hq;
  hipLaunchKernelGGL(transpose_bf16_kernel, tgrid, dim3(256), 0, st, Qp, q_hs, (int64_t)D, T, D, qt,
                     (int64_t)D * Tp, (int64_t)Tp);
  hipLaunchKernelGGL(transpose_bf16_kernel, tgrid, dim3(256), 0, st, dOp, (int64_t)D, (int64_t)Hq * D,
                     T, D, dot, (int64_t)D * Tp, (int64_t)Tp);
  hipLaunchKernelGGL(attn_delta_kernel<D>, dim3((unsigned)(((int64_t)T * Hq + 3) / 4)), dim3(256), 0, st,
                     Op, dOp, T, Hq, delta);
  const int n_qb = (T + kBM - 1) / kBM;
  hipLaunchKernelGGL(ttt_attn_bwd_dq_kernel<D>, dim3((unsigned)(n_qb * Hq)), dim3(kAttnThreads), 0, st,
                     Qp, q_hs, Kp, k_hs, Vp, v_hs, dOp, kt, lse, delta, row_lo, T, Tp, n_extra, Hq, Hkv,
                     sl2, scaling, dQp, dq_hs);
  const size_t smem = (size_t)(2 * 64 * (D + kKPad) + 2 * D * (64 + kVPad)) * 2 + 64 * 12;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&ttt_attn_bwd_dkv_kernel<D>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      last_error() = std::string("spx_ttt_attn_bwd: hipFuncSetAttribute: ") + hipGetErrorString(e);
      return SPX_ERR_HIP;
    }
    attr_set = true;
  }
  const int n_kb = (T + 127) / 128;
  hipLaunchKernelGGL(ttt_attn_bwd_dkv_kernel<D>, dim3((unsigned)(n_kb * Hkv)), dim3(kAttnThreads), smem,
                     st, Qp, q_hs, Kp, k_hs, Vp, v_hs, dOp, qt, dot, lse, delta, row_lo, T, Tp, Hq, Hkv,
                     sl2, scaling, dKp, dk_hs, dVp, dv_hs);
  if (n_extra > 0)
    hipLaunchKernelGGL(ttt_attn_bwd_diag_kernel<D>, dim3((unsigned)(((int64_t)T * Hkv + 3) / 4)),
                       dim3(256), 0, st, Qp, q_hs, Kp, k_hs, Vp, v_hs, dOp, lse, delta, T, n_extra, Hq,
                       Hkv, sl2, scaling, dKp, dk_hs, dVp, dv_hs);
  return check_launch("spx_ttt_attn_bwd");
}

}  // namespace spx

using namespace spx;

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
  if (!backward) return round_up((int64_t)Hkv * D * round_up(T, kBN) * 2, 256);  // V^T
  const int64_t Tp = round_up(T, kBM);
  // K^T, Q^T, dO^T (bf16) and delta = rowsum(dO * O) (f32)
  return round_up(((int64_t)Hkv + 2 * (int64_t)Hq) * D * Tp * 2 + (int64_t)Hq * T * 4, 256);
}

static int attn_common_checks(const char* fn, int64_t T, int32_t ttt_step, int32_t Hq, int32_t Hkv,
                              int32_t D) {
  if (!(T > 0 && T < (1ll << 24))) return fail_arg(fn, "0 < T < 2^24");
  if (!(ttt_step >= 0 && ttt_step < 64)) return fail_arg(fn, "0 <= ttt_step < 64");
  if (!(Hkv > 0 && Hq > 0 && Hq % Hkv == 0)) return fail_arg(fn, "Hq must be a multiple of Hkv");
  if (!(D == 64 || D == 128)) return fail_arg(fn, "head_dim must be 64 or 128");
  return SPX_OK;
}

extern "C" int spx_ttt_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                                int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                const int32_t* row_lo, int64_t T, int32_t ttt_step, int32_t Hq,
                                int32_t Hkv, int32_t D, float scaling, void* out, float* lse,
                                void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = attn_common_checks(__func__, T, ttt_step, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(q && k && v && row_lo && out && lse && workspace, "null buffer");
  SPX_REQUIRE(q_head_stride >= T * D, "q head stride smaller than T*D");
  SPX_REQUIRE(k_head_stride >= (int64_t)(ttt_step + 1) * T * D &&
              v_head_stride >= (int64_t)(ttt_step + 1) * T * D,
              "k/v head stride smaller than (ttt_step+1)*T*D");
  SPX_REQUIRE(q_head_stride % 8 == 0 && k_head_stride % 8 == 0 && v_head_stride % 8 == 0,
              "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= spx_ttt_attn_workspace_bytes(T, Hq, Hkv, D, 0), "workspace too small");
  SPX_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)workspace) % 16 == 0,
              "buffers must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int Tp = (int)round_up(T, kBN);
  uint16_t* vt = reinterpret_cast<uint16_t*>(workspace);
  {
    dim3 grid((unsigned)((Tp + 63) / 64), (unsigned)((D + 63) / 64), (unsigned)Hkv);
    hipLaunchKernelGGL(transpose_bf16_kernel, grid, dim3(256), 0, st,
                       reinterpret_cast<const uint16_t*>(v), v_head_stride, (int64_t)D, (int)T, (int)D,
                       vt, (int64_t)D * Tp, (int64_t)Tp);
  }
  const int n_qb = (int)((T + kBM - 1) / kBM);
  dim3 grid((unsigned)(n_qb * Hq));
  const float sl2 = scaling * kLog2e;
  auto Qp = reinterpret_cast<const uint16_t*>(q);
  auto Kp = reinterpret_cast<const uint16_t*>(k);
  auto Vp = reinterpret_cast<const uint16_t*>(v);
  auto Op = reinterpret_cast<uint16_t*>(out);
  if (D == 128)
    hipLaunchKernelGGL(ttt_attn_fwd_kernel<128>, grid, dim3(kAttnThreads), 0, st, Qp, q_head_stride, Kp,
                       k_head_stride, Vp, v_head_stride, vt, row_lo, (int)T, Tp, (int)ttt_step, (int)Hq,
                       (int)Hkv, sl2, Op, lse);
  else
    hipLaunchKernelGGL(ttt_attn_fwd_kernel<64>, grid, dim3(kAttnThreads), 0, st, Qp, q_head_stride, Kp,
                       k_head_stride, Vp, v_head_stride, vt, row_lo, (int)T, Tp, (int)ttt_step, (int)Hq,
                       (int)Hkv, sl2, Op, lse);
  return check_launch(__func__);
}

extern "C" int spx_ttt_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                                int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                const void* out, const void* dout, const float* lse,
                                const int32_t* row_lo, int64_t T, int32_t ttt_step, int32_t Hq,
                                int32_t Hkv, int32_t D, float scaling, void* dq,
                                int64_t dq_head_stride, void* dk, int64_t dk_head_stride, void* dv,
                                int64_t dv_head_stride, void* workspace, int64_t workspace_bytes,
                                void* stream) {
  if (int rc = attn_common_checks(__func__, T, ttt_step, Hq, Hkv, D)) return rc;
  SPX_REQUIRE(q && k && v && out && dout && lse && row_lo && dq && dk && dv && workspace, "null buffer");
  const int64_t kv_rows = (int64_t)(ttt_step + 1) * T * D;
  SPX_REQUIRE(q_head_stride >= T * D && dq_head_stride >= T * D, "q / dq head stride smaller than T*D");
  SPX_REQUIRE(k_head_stride >= kv_rows && v_head_stride >= kv_rows && dk_head_stride >= kv_rows &&
              dv_head_stride >= kv_rows, "k/v/dk/dv head stride smaller than (ttt_step+1)*T*D");
  SPX_REQUIRE((q_head_stride | k_head_stride | v_head_stride | dq_head_stride | dk_head_stride |
               dv_head_stride) % 8 == 0, "head strides must be multiples of 8 elements");
  SPX_REQUIRE(workspace_bytes >= spx_ttt_attn_workspace_bytes(T, Hq, Hkv, D, 1), "workspace too small");
  SPX_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)dout |
               (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv | (uintptr_t)workspace) % 16 == 0,
              "buffers must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  auto Qp = reinterpret_cast<const uint16_t*>(q);
  auto Kp = reinterpret_cast<const uint16_t*>(k);
  auto Vp = reinterpret_cast<const uint16_t*>(v);
  auto Op = reinterpret_cast<const uint16_t*>(out);
  auto dOp = reinterpret_cast<const uint16_t*>(dout);
  auto dQp = reinterpret_cast<uint16_t*>(dq);
  auto dKp = reinterpret_cast<uint16_t*>(dk);
  auto dVp = reinterpret_cast<uint16_t*>(dv);
  if (D == 128)
    return launch_bwd_all<128>(Qp, q_head_stride, Kp, k_head_stride, Vp, v_head_stride, Op, dOp, lse,
                               row_lo, (int)T, (int)ttt_step, (int)Hq, (int)Hkv, scaling, dQp,
                               dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride, workspace, st);
  return launch_bwd_all<64>(Qp, q_head_stride, Kp, k_head_stride, Vp, v_head_stride, Op, dOp, lse,
                            row_lo, (int)T, (int)ttt_step, (int)Hq, (int)Hkv, scaling, dQp,
                            dq_head_stride, dKp, dk_head_stride, dVp, dv_head_stride, workspace, st);
}
