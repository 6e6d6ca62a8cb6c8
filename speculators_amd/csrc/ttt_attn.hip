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
  const int64_t Tp = round_up(T, kBN);
  int64_t elems = (int64_t)Hkv * D * Tp;               // V^T of the context keys
  if (backward) elems += (int64_t)Hkv * D * Tp          // K^T
                         + 2 * (int64_t)Hq * D * round_up(T, kBM);  // Q^T, dO^T
  int64_t bytes = elems * 2;
  if (backward) bytes += (int64_t)Hq * T * 4;           // delta = rowsum(dO * O)
  return round_up(bytes, 256);
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
