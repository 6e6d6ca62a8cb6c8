// Fused vocabulary loss for gfx950: one workgroup streams one (draft row,
// target row) pair with 16-byte loads, keeps online soft-max statistics of
// both rows, the first-index arg-max of both rows and the loss reduction in
// registers, and never materialises probabilities.  HBM-bound: algorithmic
// traffic is 2 rows read (forward) and 2 rows read + 1 row written (backward).
//
// All exponentials run in the base-2 domain (v_exp_f32 is 2^x): logits are
// pre-scaled by log2(e), statistics are converted back at the end.

#include "loss_common.h"
#include "../../include/spx.h"

namespace spx {

// ---- running statistics ----------------------------------------------------
struct RowStats {
  float md, zd;        // draft: running max (base-2 scaled) and sum of 2^(x' - md)
  float mt, zt, at;    // target: same, and sum of 2^(y' - mt) * (y - x)
  float bd; int id;    // draft arg-max value / first index
  float bt; int it; float xt;  // target arg-max value / first index / draft logit there
};

__device__ __forceinline__ void merge(RowStats& a, const RowStats& b) {
  float m = fmaxf(a.md, b.md);
  a.zd = a.zd * fast_exp2(a.md - m) + b.zd * fast_exp2(b.md - m);
  a.md = m;
  m = fmaxf(a.mt, b.mt);
  float ra = fast_exp2(a.mt - m), rb = fast_exp2(b.mt - m);
  a.zt = a.zt * ra + b.zt * rb;
  a.at = a.at * ra + b.at * rb;
  a.mt = m;
  if (b.bd > a.bd || (b.bd == a.bd && b.id < a.id)) { a.bd = b.bd; a.id = b.id; }
  if (b.bt > a.bt || (b.bt == a.bt && b.it < a.it)) { a.bt = b.bt; a.it = b.it; a.xt = b.xt; }
}

__device__ __forceinline__ RowStats shuffle_xor(const RowStats& s, int m) {
  RowStats o;
  o.md = __shfl_xor(s.md, m, 64); o.zd = __shfl_xor(s.zd, m, 64);
  o.mt = __shfl_xor(s.mt, m, 64); o.zt = __shfl_xor(s.zt, m, 64);
  o.at = __shfl_xor(s.at, m, 64);
  o.bd = __shfl_xor(s.bd, m, 64); o.id = __shfl_xor(s.id, m, 64);
  o.bt = __shfl_xor(s.bt, m, 64); o.it = __shfl_xor(s.it, m, 64);
  o.xt = __shfl_xor(s.xt, m, 64);
  return o;
}

__device__ __forceinline__ float block_sum(float v, float* lds) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < kLossWaves; ++w) t += lds[w];
  return t;
}

// log((2^a' + 2^b')/2) in natural units from natural-log inputs
__device__ __forceinline__ float log_mix(float la, float lb) {
  float mx = fmaxf(la, lb);
  float s = fast_exp2((la - mx) * kLog2e) + fast_exp2((lb - mx) * kLog2e);
  return mx + fast_log2(s) * kLn2 - kLn2;
}

// ---- mask element access ---------------------------------------------------
__device__ __forceinline__ float mask_value(const void* p, int kind, int64_t i) {
  switch (kind) {
    case SPX_KIND_U8: return (float)reinterpret_cast<const uint8_t*>(p)[i];
    case SPX_KIND_I32: return (float)reinterpret_cast<const int32_t*>(p)[i];
    case SPX_KIND_I64: return (float)reinterpret_cast<const int64_t*>(p)[i];
    case SPX_KIND_F32: return reinterpret_cast<const float*>(p)[i];
    default: return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  }
}
__device__ __forceinline__ void store_flag(void* p, int kind, int64_t i, bool v) {
  switch (kind) {
    case SPX_KIND_U8: reinterpret_cast<uint8_t*>(p)[i] = v ? 1 : 0; break;
    case SPX_KIND_I32: reinterpret_cast<int32_t*>(p)[i] = v ? 1 : 0; break;
    case SPX_KIND_I64: reinterpret_cast<int64_t*>(p)[i] = v ? 1 : 0; break;
    case SPX_KIND_F32: reinterpret_cast<float*>(p)[i] = v ? 1.f : 0.f; break;
    default: reinterpret_cast<uint16_t*>(p)[i] = v ? 0x3f80 : 0; break;
  }
}

// ---- what one TTT step adds to the row pass --------------------------------------
// d2t != nullptr: `targets` are full-vocabulary rows (vt wide) and target element i is read at
// i + d2t[i] (model.py:161-169, train/vocab_mapping.py:86-96); `gathered` (may be nullptr) then
// receives the draft-vocabulary row, for the later steps and the backward.
// counts != nullptr: the row's part of the acceptance chain (models/metrics.py:6-36): with
// m = mask[r] != 0, was = prev[r] != 0, hit = argmax_draft == argmax_target, now = was && hit:
//   counts[0] += m && now,  counts[1] += m,  counts[2] += was,  prev[r] = now.
// Integer atomics: the sums do not depend on the order of the rows.
struct StepArgs {
  const int64_t* d2t; int64_t vt;
  void* gathered; int64_t ld_gathered;
  const void* mask; int mask_kind;
  void* prev; int prev_kind;
  int32_t* counts;
};

// eight target elements through the offset table (ascending indices: neighbouring lanes read
// neighbouring sectors of the full row)
template <typename T>
__device__ __forceinline__ void load8_gather(const T* full, const int64_t* __restrict__ d2t, int64_t base,
                                             int64_t n, int64_t vt, float v[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float val = kNegBig;  // tail padding, like load8_guard
    if (base + i < n) {
      const int64_t j = base + i + d2t[base + i];
      val = (j >= 0 && j < vt) ? load1(full + j) : -INFINITY;
    }
    v[i] = val;
  }
}

// ---- forward ---------------------------------------------------------------
// KNOWN: lse_target / argmax_target are INPUTS (the target row's statistics from an
// earlier pass over the same row); the target max / sum / arg-max tracking is skipped and
// the cross-entropy reduction does not read the target row at all.
// GATHER: the target row is read through the d2t offset table (see StepArgs).
template <typename T, int OP, bool VEC, bool KNOWN, bool GATHER>
__global__ __launch_bounds__(kLossThreads) void loss_fwd_kernel(
    const T* __restrict__ logits, int64_t ld_logits, const T* __restrict__ targets,
    int64_t ld_targets, int64_t vocab, float* __restrict__ loss, float* __restrict__ lse_draft,
    float* __restrict__ lse_target, float* __restrict__ extra, int32_t* __restrict__ argmax_draft,
    int32_t* __restrict__ argmax_target, StepArgs sa) {
  const int64_t r = blockIdx.x;
  const T* xrow = logits + r * ld_logits;
  const T* yrow = targets + r * ld_targets;
  T* grow = (GATHER && sa.gathered) ? reinterpret_cast<T*>(sa.gathered) + r * sa.ld_gathered : nullptr;
  const int tid = threadIdx.x;
  const int64_t nchunks = (vocab + 7) >> 3;

  const float lt2_known = KNOWN ? lse_target[r] * kLog2e : 0.f;  // base-2 target lse
  const bool read_y = !(KNOWN && OP == SPX_LOSS_CE);
  RowStats s;
  s.md = kNegBig; s.zd = 0.f; s.mt = kNegBig; s.zt = 0.f; s.at = 0.f;
  s.bd = -INFINITY; s.id = 0x7fffffff; s.bt = -INFINITY; s.it = 0x7fffffff; s.xt = 0.f;

  // GATHER: the draft ids of one tile (256 chunks) map to an ascending span of the full row.
  // The span is brought into LDS with coalesced 16-byte loads and the eight elements of a lane
  // are picked from there; a span that does not fit (or rows without 16-byte alignment) and any
  // id that falls outside the span (a table that is not ascending) read the row directly.
  constexpr int kStageElems = GATHER ? 32768 / (int)sizeof(T) : 1;
  __shared__ __attribute__((aligned(16))) T stage[kStageElems];
  for (int64_t c0 = 0; c0 < nchunks; c0 += kLossThreads) {
    const int64_t c = c0 + tid;
    const bool active = c < nchunks;
    const int64_t base = c << 3;
    float x[8], y[8];
    if (GATHER) {
      // this lane's draft row chunk and its eight target columns first: their latency runs
      // under the staging of the span
      int64_t jj[8];
      if (active) {
        load8<T, VEC>(xrow, base, vocab, x);
        if (base + 8 <= vocab && ptr_aligned16(sa.d2t)) {
          const u32x4* dp = reinterpret_cast<const u32x4*>(sa.d2t + base);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const u32x4 w = dp[q];
            jj[2 * q] = base + 2 * q + (int64_t)(((uint64_t)w.y << 32) | w.x);
            jj[2 * q + 1] = base + 2 * q + 1 + (int64_t)(((uint64_t)w.w << 32) | w.z);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) jj[i] = base + i < vocab ? base + i + sa.d2t[base + i] : -1;
        }
      }
      const int64_t i0 = c0 << 3, i1 = min(vocab, (c0 + kLossThreads) << 3) - 1;
      int64_t lo = i0 + sa.d2t[i0], hi = i1 + sa.d2t[i1] + 1;
      lo = max((int64_t)0, min(lo, sa.vt)) & ~(int64_t)7;
      hi = max(lo, min(hi, sa.vt));
      constexpr int EPV = 16 / (int)sizeof(T);  // elements per 16-byte access
      const bool staged = VEC && (hi - lo) <= kStageElems && ((ld_targets & 7) == 0) &&
                          ptr_aligned16(targets);
      if (staged) {
        __syncthreads();  // the previous tile's picks are done
        for (int64_t e = (int64_t)tid * EPV; lo + e < hi; e += kLossThreads * EPV) {
          if (lo + e + EPV <= sa.vt)
            *reinterpret_cast<u32x4*>(&stage[e]) = ld16(yrow + lo + e);
          else
            for (int q = 0; q < EPV; ++q)
              if (lo + e + q < sa.vt) stage[e + q] = yrow[lo + e + q];
        }
        __syncthreads();
      }
      if (active) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float val = kNegBig;  // tail padding, like load8_guard
          if (base + i < vocab) {
            const int64_t j = jj[i];
            if (staged && j >= lo && j < hi) val = load1(&stage[j - lo]);
            else val = (j >= 0 && j < sa.vt) ? load1(yrow + j) : -INFINITY;
          }
          y[i] = val;
        }
        if (grow) store8<T, VEC>(grow, base, vocab, y);
      }
    } else if (active) {
      load8<T, VEC>(xrow, base, vocab, x);
      if (read_y) load8<T, VEC>(yrow, base, vocab, y);
    }
    if (!active) continue;
    float cx = x[0], cy = y[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) cx = fmaxf(cx, x[i]);
    if (!KNOWN) {
#pragma unroll
      for (int i = 1; i < 8; ++i) cy = fmaxf(cy, y[i]);
    }
    if (cx > s.bd) {  // strict: an earlier chunk of this thread keeps a tie
      int k = 7;
#pragma unroll
      for (int i = 6; i >= 0; --i) k = (x[i] == cx) ? i : k;
      s.bd = cx; s.id = (int)base + k;
    }
    if (!KNOWN && cy > s.bt) {
      int k = 7;
      float xv = x[7];
#pragma unroll
      for (int i = 6; i >= 0; --i) {
        const bool hit = y[i] == cy;
        k = hit ? i : k;
        xv = hit ? x[i] : xv;
      }
      s.bt = cy; s.it = (int)base + k; s.xt = xv;
    }
    {
      const float cxs = cx * kLog2e;
      float mn = s.md, z = s.zd;
      if (cxs > mn) {  // the running max moves rarely once a few chunks have been seen
        z *= fast_exp2(mn - cxs);
        mn = cxs;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) z += fast_exp2(fmaf(x[i], kLog2e, -mn));
      s.zd = z; s.md = mn;
    }
    if (KNOWN && OP != SPX_LOSS_CE) {
      float a = s.at;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float pr = fast_exp2(fmaf(y[i], kLog2e, -lt2_known));  // the target probability
        a = fmaf(pr, y[i] - x[i], a);
      }
      s.at = a;
    } else if (OP != SPX_LOSS_CE) {
      float mn = fmaxf(s.mt, cy * kLog2e);
      float rs = fast_exp2(s.mt - mn);
      float z = s.zt * rs, a = s.at * rs;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float e = fast_exp2(fmaf(y[i], kLog2e, -mn));
        z += e;
        a = fmaf(e, y[i] - x[i], a);
      }
      s.zt = z; s.at = a; s.mt = mn;
    }
  }

  // tail padding must never win an arg-max: padded values are kNegBig, and
  // a padded index only enters when cx == kNegBig > -inf on an all-padding
  // chunk, which cannot exist (every chunk holds at least one real element).
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) merge(s, shuffle_xor(s, m));

  __shared__ RowStats part[kLossWaves];
  __shared__ float red[kLossWaves];
  if ((tid & 63) == 0) part[tid >> 6] = s;
  __syncthreads();
  s = part[0];
#pragma unroll
  for (int w = 1; w < kLossWaves; ++w) merge(s, part[w]);

  const float lse_d = (s.md + fast_log2(s.zd)) * kLn2;
  const float lse_t = KNOWN ? lse_target[r]
                            : ((OP != SPX_LOSS_CE) ? (s.mt + fast_log2(s.zt)) * kLn2 : 0.f);
  if (KNOWN) {
    s.it = argmax_target ? argmax_target[r] : 0;
    if (OP == SPX_LOSS_CE) s.xt = load1(xrow + s.it);
  }

  float row_loss = 0.f, row_extra = 0.f;
  if (OP == SPX_LOSS_KL) {
    row_loss = (KNOWN ? s.at : s.at / s.zt) - lse_t + lse_d;
    row_extra = row_loss;
  } else if (OP == SPX_LOSS_CE) {
    row_loss = lse_d - s.xt;
  } else {
    // second streaming pass (the row pair is L2 resident by now)
    float acc = 0.f, ext = 0.f;
    for (int64_t c = tid; c < nchunks; c += kLossThreads) {
      const int64_t base = c << 3;
      float x[8], y[8];
      load8<T, VEC>(xrow, base, vocab, x);
      if (GATHER) load8_gather<T>(yrow, sa.d2t, base, vocab, sa.vt, y);
      else load8<T, VEC>(yrow, base, vocab, y);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float ldp = x[i] - lse_d, ltp = y[i] - lse_t;
        float dp = fast_exp2(ldp * kLog2e), tp = fast_exp2(ltp * kLog2e);
        if (OP == SPX_LOSS_RKL) {
          acc = fmaf(dp, ldp - ltp, acc);
        } else if (OP == SPX_LOSS_JSD) {
          float lm = log_mix(ldp, ltp);
          acc = fmaf(dp, ldp - lm, acc);
          ext = fmaf(tp, ltp - lm, ext);
        } else {  // TV
          acc += fminf(dp, tp);
          ext += (dp <= tp) ? dp : 0.f;
        }
      }
    }
    acc = block_sum(acc, red);
    if (OP != SPX_LOSS_RKL) ext = block_sum(ext, red);
    if (OP == SPX_LOSS_RKL) { row_loss = acc; row_extra = acc; }
    else if (OP == SPX_LOSS_JSD) { row_loss = 0.5f * (acc + ext); row_extra = acc; }
    else { row_loss = 1.f - acc; row_extra = ext; }
  }
  if (tid == 0) {
    loss[r] = row_loss;
    lse_draft[r] = lse_d;
    extra[r] = row_extra;
    if (argmax_draft) argmax_draft[r] = s.id;
    if (!KNOWN) {
      lse_target[r] = lse_t;
      if (argmax_target) argmax_target[r] = s.it;
    }
    if (sa.counts) {
      const bool m = sa.mask ? mask_value(sa.mask, sa.mask_kind, r) != 0.f : true;
      const bool was = sa.prev ? mask_value(sa.prev, sa.prev_kind, r) != 0.f : true;
      const bool now = was && (s.id == s.it);
      if (m && now) atomicAdd(&sa.counts[0], 1);
      if (m) atomicAdd(&sa.counts[1], 1);
      if (was) atomicAdd(&sa.counts[2], 1);
      if (sa.prev) store_flag(sa.prev, sa.prev_kind, r, now);
    }
  }
}

// ---- forward and logits gradient in one pass -------------------------------------------------------
// The head of a TTT step is frozen while the draft layers train, and which rows carry a gradient is
// known before the loss is (the loss mask): the row pass can then leave the gradient of the logits
// behind as well, and the row pair is read ONCE instead of once by the forward and once more by the
// backward.  One workgroup of 512 threads holds a whole row pair in registers (eight 16-byte chunks of
// each row per thread as they come from memory, requested before anything is computed: vocab <= 32768,
// bf16), reduces it to the row statistics exactly like loss_fwd_kernel, and, for a row that row_map
// sends to a slot >= 0, goes over its registers a second time and writes
//   grad[slot, :] = softmax(x) - softmax(y)   (kl)      softmax(x) - onehot(argmax y)   (ce)
// -- the gradient for a row weight of ONE; the caller applies the weight the reduction behind the loss
// gives the row to the input-gradient product's result (which is linear in it).  Rows mapped to -1 get
// no gradient row, and with the target statistics handed in (KNOWN) their target row is not read at
// all, no soft-max of their draft row is formed and their loss is written as zero: a masked row's loss enters
// no sum.  (Their arg-max outputs and their part of the acceptance chain are those of any row.)
constexpr int kFgThreads = 512, kFgWaves = kFgThreads / 64, kFgChunks = 8;
template <int OP, bool KNOWN>
__global__ __launch_bounds__(kFgThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void loss_fwd_grad_kernel(
    const uint16_t* __restrict__ logits, int64_t ld_logits, const uint16_t* __restrict__ targets,
    int64_t ld_targets, int64_t vocab, float* __restrict__ loss, float* __restrict__ lse_draft,
    float* __restrict__ lse_target, float* __restrict__ extra, int32_t* __restrict__ argmax_draft,
    int32_t* __restrict__ argmax_target, StepArgs sa, const int32_t* __restrict__ row_map,
    uint16_t* __restrict__ grad, int64_t ld_grad) {
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int nchunks = (int)(vocab >> 3);  // vocab is a multiple of 8 here
  const int slot = row_map[r];
  const bool live = slot >= 0;
  const uint16_t* xrow = logits + r * ld_logits;
  const uint16_t* yrow = targets ? targets + r * ld_targets : nullptr;
  const bool read_y = !(KNOWN && (OP == SPX_LOSS_CE || !live));
  u32x4 xr[kFgChunks], yr[kFgChunks];
#pragma unroll
  for (int k = 0; k < kFgChunks; ++k) {
    const int c = tid + k * kFgThreads;
    if (c < nchunks) {
      xr[k] = ld16(xrow + ((int64_t)c << 3));
      if (read_y) yr[k] = ld16(yrow + ((int64_t)c << 3));
    }
  }
  const float lt2_known = KNOWN ? lse_target[r] * kLog2e : 0.f;  // base-2 target lse
  // a masked row whose target statistics are known needs nothing but the draft row's arg-max
  const bool soft_x = live || !KNOWN;
  RowStats s;
  s.md = kNegBig; s.zd = 0.f; s.mt = kNegBig; s.zt = 0.f; s.at = 0.f;
  s.bd = -INFINITY; s.id = 0x7fffffff; s.bt = -INFINITY; s.it = 0x7fffffff; s.xt = 0.f;
  auto unpack = [](u32x4 raw, float v[8]) {
    v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x); v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
    v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z); v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
  };
#pragma unroll
  for (int k = 0; k < kFgChunks; ++k) {
    const int c = tid + k * kFgThreads;
    if (c >= nchunks) continue;
    const int base = c << 3;
    float x[8], y[8];
    unpack(xr[k], x);
    if (read_y) unpack(yr[k], y);
    float cx = x[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) cx = fmaxf(cx, x[i]);
    if (cx > s.bd) {  // strict: an earlier chunk of this thread keeps a tie
      int kk = 7;
#pragma unroll
      for (int i = 6; i >= 0; --i) kk = (x[i] == cx) ? i : kk;
      s.bd = cx; s.id = base + kk;
    }
    if (soft_x) {
      const float cxs = cx * kLog2e;
      float mn = s.md, z = s.zd;
      if (cxs > mn) {
        z *= fast_exp2(mn - cxs);
        mn = cxs;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) z += fast_exp2(fmaf(x[i], kLog2e, -mn));
      s.zd = z; s.md = mn;
    }
    if (!KNOWN) {
      float cy = y[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) cy = fmaxf(cy, y[i]);
      if (cy > s.bt) {
        int kk = 7;
        float xv = x[7];
#pragma unroll
        for (int i = 6; i >= 0; --i) {
          const bool hit = y[i] == cy;
          kk = hit ? i : kk;
          xv = hit ? x[i] : xv;
        }
        s.bt = cy; s.it = base + kk; s.xt = xv;
      }
      if (OP != SPX_LOSS_CE) {
        float mn = fmaxf(s.mt, cy * kLog2e);
        float rs = fast_exp2(s.mt - mn);
        float z = s.zt * rs, a = s.at * rs;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float e = fast_exp2(fmaf(y[i], kLog2e, -mn));
          z += e;
          a = fmaf(e, y[i] - x[i], a);
        }
        s.zt = z; s.at = a; s.mt = mn;
      }
    } else if (OP != SPX_LOSS_CE && live) {
      float a = s.at;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float pr = fast_exp2(fmaf(y[i], kLog2e, -lt2_known));  // the target probability
        a = fmaf(pr, y[i] - x[i], a);
      }
      s.at = a;
    }
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) merge(s, shuffle_xor(s, m));
  __shared__ RowStats part[kFgWaves];
  if ((tid & 63) == 0) part[tid >> 6] = s;
  __syncthreads();
  s = part[0];
#pragma unroll
  for (int w = 1; w < kFgWaves; ++w) merge(s, part[w]);

  const float lse_d = soft_x ? (s.md + fast_log2(s.zd)) * kLn2 : 0.f;
  const float lse_t = KNOWN ? lse_target[r]
                            : ((OP != SPX_LOSS_CE) ? (s.mt + fast_log2(s.zt)) * kLn2 : 0.f);
  if (KNOWN) {
    s.it = argmax_target[r];
    if (OP == SPX_LOSS_CE) s.xt = (s.it >= 0 && s.it < vocab) ? load1(xrow + s.it) : 0.f;
  }
  if (tid == 0) {
    float row_loss;
    if (!soft_x) row_loss = 0.f;
    else if (OP == SPX_LOSS_KL) row_loss = (KNOWN ? s.at : s.at / s.zt) - lse_t + lse_d;
    else row_loss = lse_d - s.xt;
    loss[r] = row_loss;
    lse_draft[r] = lse_d;
    extra[r] = OP == SPX_LOSS_KL ? row_loss : 0.f;
    if (argmax_draft) argmax_draft[r] = s.id;
    if (!KNOWN) {
      lse_target[r] = lse_t;
      if (argmax_target) argmax_target[r] = s.it;
    }
    if (sa.counts) {
      const bool m = sa.mask ? mask_value(sa.mask, sa.mask_kind, r) != 0.f : true;
      const bool was = sa.prev ? mask_value(sa.prev, sa.prev_kind, r) != 0.f : true;
      const bool now = was && (s.id == s.it);
      if (m && now) atomicAdd(&sa.counts[0], 1);
      if (m) atomicAdd(&sa.counts[1], 1);
      if (was) atomicAdd(&sa.counts[2], 1);
      if (sa.prev) store_flag(sa.prev, sa.prev_kind, r, now);
    }
  }
  if (!live) return;
  uint16_t* grow = grad + (int64_t)slot * ld_grad;
  const float cd = -lse_d * kLog2e, ct = -lse_t * kLog2e;
  const int label = s.it;
  // (the packed chunks are what stays in registers between the passes, not their 64 + 64 unpacked values)
#pragma unroll
  for (int k = 0; k < kFgChunks; ++k) {
    asm volatile("" : "+v"(xr[k].x), "+v"(xr[k].y), "+v"(xr[k].z), "+v"(xr[k].w));
    if (OP != SPX_LOSS_CE) asm volatile("" : "+v"(yr[k].x), "+v"(yr[k].y), "+v"(yr[k].z), "+v"(yr[k].w));
  }
#pragma unroll
  for (int k = 0; k < kFgChunks; ++k) {
    const int c = tid + k * kFgThreads;
    if (c >= nchunks) continue;
    const int base = c << 3;
    float x[8], y[8], o[8];
    unpack(xr[k], x);
    if (OP != SPX_LOSS_CE) unpack(yr[k], y);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float dp = fast_exp2(fmaf(x[i], kLog2e, cd));
      if (OP == SPX_LOSS_CE) o[i] = dp - ((base + i) == label ? 1.f : 0.f);
      else o[i] = dp - fast_exp2(fmaf(y[i], kLog2e, ct));
    }
    store8_vec<uint16_t>(grow + ((int64_t)c << 3), o);
  }
}

// ---- forward with the d2t gather, pipelined ------------------------------------------------------
// The first step of a TTT loop whose targets arrive as full-vocabulary verifier logits: the same row pass
// as loss_fwd_kernel<.., GATHER> (gather through d2t, both online soft-maxes, KL or CE, both arg-maxes,
// the gathered row written out, the acceptance chain), arranged so that nothing waits for memory:
//   * the draft ids are walked in tiles of 2048; the ascending span [lo, hi) of the full row that a tile
//     maps to is known for every tile before the loop starts (a table in LDS, built from 2 table reads
//     per tile), so the span of tile t + 2 and that tile's piece of the draft row are requested -- global
//     -> LDS directly, no registers -- while tile t is reduced: a ring of three slots, one workgroup
//     barrier per tile, a fixed number of loads per wave and tile so that one s_waitcnt constant tells
//     when a slot has landed;
//   * picking element i + d2t[i] out of the staged span is done with lane = id (consecutive lanes read
//     LDS addresses a few bytes apart: about two lanes per bank) instead of lane = chunk of 8 ids (lanes
//     64 bytes apart: 16 lanes per bank); each wave then turns its 512 picks into 8-id chunks through a
//     1 KB LDS strip of its own, so the gathered row is written 16 bytes per lane;
//   * a tile whose span does not fit a slot (a table that is not spread evenly) reads its elements
//     from global memory directly, as the general kernel does.
// bf16 rows, 16-byte aligned, KL or CE; everything else stays with loss_fwd_kernel<.., GATHER>.
constexpr int kPipeTileIds = kLossThreads * 8;        // 2048 draft ids per tile
constexpr int kPipeSpanLoads = 5;                     // 1 KB wave-loads per wave and span
constexpr int kPipeCap = kPipeSpanLoads * kLossWaves * 512;  // 10240 elements of the full row per slot
constexpr int kPipeSlotBytes = kPipeCap * 2 + kPipeTileIds * 2;  // span + the tile's draft-row piece
constexpr int kPipeSlots = 3;
constexpr int kPipeMaxTiles = 128;                    // draft vocabulary <= 262144
constexpr int kPipeOffY = kPipeSlots * kPipeSlotBytes;  // byte offsets inside the dynamic LDS block
constexpr int kPipeOffSpan = kPipeOffY + kPipeTileIds * 2;
constexpr int kPipeSmem = kPipeOffSpan + kPipeMaxTiles * 2 * 4;
static_assert(2 * kPipeSmem + 1024 <= 160 * 1024, "two workgroups per compute unit");

template <int OP>
__global__ __launch_bounds__(kLossThreads) void loss_fwd_gather_pipe_kernel(
    const uint16_t* __restrict__ logits, int64_t ld_logits, const uint16_t* __restrict__ targets,
    int64_t ld_targets, int64_t vocab, float* __restrict__ loss, float* __restrict__ lse_draft,
    float* __restrict__ lse_target, float* __restrict__ extra, int32_t* __restrict__ argmax_draft,
    int32_t* __restrict__ argmax_target, StepArgs sa) {
  extern __shared__ __attribute__((aligned(16))) uint8_t psm[];
  uint16_t* const ybuf = reinterpret_cast<uint16_t*>(psm + kPipeOffY);  // [4 waves][512]
  int* const span = reinterpret_cast<int*>(psm + kPipeOffSpan);         // [tiles][2]: lo, length (-1: direct)
  const int64_t r = blockIdx.x;
  const uint16_t* xrow = logits + r * ld_logits;
  const uint16_t* yrow = targets + r * ld_targets;
  uint16_t* grow = sa.gathered ? reinterpret_cast<uint16_t*>(sa.gathered) + r * sa.ld_gathered : nullptr;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ntiles = (int)((vocab + kPipeTileIds - 1) / kPipeTileIds);

  for (int t = tid; t < ntiles; t += kLossThreads) {
    const int64_t i0 = (int64_t)t * kPipeTileIds, i1 = min(vocab, i0 + kPipeTileIds) - 1;
    int64_t lo = i0 + sa.d2t[i0], hi = i1 + sa.d2t[i1] + 1;
    lo = max((int64_t)0, min(lo, sa.vt)) & ~(int64_t)7;
    hi = max(lo, min(hi, sa.vt));
    span[2 * t] = (int)lo;
    span[2 * t + 1] = (hi - lo <= kPipeCap) ? (int)(hi - lo) : -1;
  }
  __syncthreads();

  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)psm;
  // Per-lane byte offsets that never change: every tile moves the BASE of its buffer resources (scalar
  // arithmetic) and sets their size to what the tile may touch, so lanes past a span's end, past the
  // draft vocabulary or past the table fetch nothing and deliver zeros, without a vector instruction
  int span_voff[kPipeSpanLoads];
#pragma unroll
  for (int k = 0; k < kPipeSpanLoads; ++k) span_voff[k] = ((k * kLossWaves + wave) * 512 + lane * 8) * 2;
  const int x_voff = (wave * 512 + lane * 8) * 2;
  const int off_voff = lane * 8;
  // tile u into slot u % 3: kPipeSpanLoads wave-loads of the span (the four waves interleaved) and one of
  // this wave's 512 ids of the draft row -- always six loads, also for a tile past the last one (resources
  // of size zero)
  auto request = [&](int u) __attribute__((always_inline)) {
    const bool live = u < ntiles;
    const int lo = live ? span[2 * u] : 0, len = live ? span[2 * u + 1] : -1;
    // (sizes in whole 16-byte pieces: a load that straddles the end of a resource delivers nothing at
    // all, and the rows' pitch, a multiple of 8 elements, covers the rounding)
    const u32x4 yres = make_rsrc(yrow + lo, len > 0 ? (uint32_t)((len + 7) & ~7) * 2u : 0u);
    const int64_t x0 = (int64_t)u * kPipeTileIds;
    const u32x4 xres = make_rsrc(xrow + x0,
                                 live ? (uint32_t)((min((int64_t)kPipeTileIds, vocab - x0) + 7) & ~(int64_t)7) * 2u : 0u);
    const uint32_t dst = lds0 + (u % kPipeSlots) * kPipeSlotBytes;
#pragma unroll
    for (int k = 0; k < kPipeSpanLoads; ++k)
      load_to_lds16<0>(yres, dst + (k * kLossWaves + wave) * 1024, span_voff[k], 0);
    load_to_lds16<0>(xres, dst + kPipeCap * 2 + wave * 1024, x_voff, 0);
  };
  // The table entries of this lane's 8 picks of tile u (lane = id inside the wave's 512 ids; the low
  // words of the int64 offsets: |d2t| < 2^31; 0 past the vocabulary).  The loads are statements the
  // compiler does not look into, like the span requests: it would otherwise guard their first use with a
  // wait that also covers every span request issued since (it does not count those), and the ring would
  // run one tile deep.  Their registers must not be read before `landed` has named them.
  auto load_offsets = [&](int u, int (&d)[8]) __attribute__((always_inline)) {
    const int64_t w0 = (int64_t)u * kPipeTileIds + wave * 512;
    const u32x4 dres = make_rsrc(sa.d2t + min(w0, vocab), (uint32_t)max((int64_t)0, min((int64_t)512, vocab - w0)) * 8u);
#define SPX_LOAD_OFF(K) \
    asm volatile("buffer_load_dword %0, %1, %2, 0 offen offset:%3" : "=v"(d[K]) : "v"(off_voff), "s"(dres), "n"(K * 512) : "memory")
    SPX_LOAD_OFF(0); SPX_LOAD_OFF(1); SPX_LOAD_OFF(2); SPX_LOAD_OFF(3);
    SPX_LOAD_OFF(4); SPX_LOAD_OFF(5); SPX_LOAD_OFF(6); SPX_LOAD_OFF(7);
#undef SPX_LOAD_OFF
  };
  // all vector-memory operations but the newest six have completed; d is what the wait releases.
  // (No branch may stand between a load_offsets and the `landed` that names its registers: a merge of
  // two paths lets the compiler copy the registers, and a copy made before the wait copies stale data.)
  auto landed = [&](int (&d)[8]) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(6)"
                 : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]), "+v"(d[4]), "+v"(d[5]), "+v"(d[6]), "+v"(d[7])
                 :: "memory");
  };

  RowStats s;
  s.md = kNegBig; s.zd = 0.f; s.mt = kNegBig; s.zt = 0.f; s.at = 0.f;
  s.bd = -INFINITY; s.id = 0x7fffffff; s.bt = -INFINITY; s.it = 0x7fffffff; s.xt = 0.f;

  // One tile.  Order of the vector-memory operations (they complete in order): offsets(0), slot(0),
  // slot(1), and per tile t: offsets(t + 1), the gathered row's store of t, slot(t + 2) -- every tile,
  // also those past the last one, whose loads fetch nothing.  At the top of tile t the six newest are
  // slot(t + 1): waiting for all but six says offsets(t) and slot(t) are in
  auto tile = [&](int t, int (&cur)[8], int (&nxt)[8]) __attribute__((always_inline)) {
    landed(cur);
    __syncthreads();  // every wave's part of slot(t) has landed, every wave is done with slot(t - 1)
    load_offsets(t + 1, nxt);
    const bool live = t < ntiles;
    const int lo = live ? span[2 * t] : 0, len = live ? span[2 * t + 1] : -1;
    const uint8_t* const slot = psm + (t % kPipeSlots) * kPipeSlotBytes;
    const uint16_t* const buf = reinterpret_cast<const uint16_t*>(slot);
    const int64_t wbase = (int64_t)t * kPipeTileIds + wave * 512;
    uint16_t* const ystrip = ybuf + wave * 512;
    // (32-bit arithmetic: ids and columns are below 2^30 here)
    const int id0 = (int)wbase + lane, nvocab = (int)vocab, nvt = (int)sa.vt;
    const unsigned ulen = len > 0 ? (unsigned)len : 0u;
    const int delta = id0 - lo;
    bool need = false;  // some pick of this lane is not in the staged span
    int rel[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      rel[k] = cur[k] + delta + 64 * k;  // column - lo
      const bool staged = (unsigned)rel[k] < ulen;
      need |= !staged;
      ystrip[lane + 64 * k] = buf[staged ? rel[k] : 0];
    }
    if (__any(need)) {  // (wave-uniform: the common case issues no global load here)
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int j = rel[k] + lo;
        if ((id0 + 64 * k < nvocab) && !((unsigned)rel[k] < ulen))  // -inf: a column outside the full row
          ystrip[lane + 64 * k] = ((unsigned)j < (unsigned)nvt) ? yrow[j] : (uint16_t)0xff80;
      }
    }
    // the strip is private to the wave: its own writes, in order, then its own reads
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int64_t base = wbase + lane * 8;
    const u32x4 yraw = *reinterpret_cast<const u32x4*>(ystrip + lane * 8);
    const u32x4 xraw = *reinterpret_cast<const u32x4*>(slot + kPipeCap * 2 + wave * 1024 + lane * 16);
    if (grow && base + 8 <= vocab) st16(grow + base, yraw);
    request(t + 2);
    if (base < vocab) {
      float x[8], y[8];
      x[0] = bf16_lo(xraw.x); x[1] = bf16_hi(xraw.x); x[2] = bf16_lo(xraw.y); x[3] = bf16_hi(xraw.y);
      x[4] = bf16_lo(xraw.z); x[5] = bf16_hi(xraw.z); x[6] = bf16_lo(xraw.w); x[7] = bf16_hi(xraw.w);
      y[0] = bf16_lo(yraw.x); y[1] = bf16_hi(yraw.x); y[2] = bf16_lo(yraw.y); y[3] = bf16_hi(yraw.y);
      y[4] = bf16_lo(yraw.z); y[5] = bf16_hi(yraw.z); y[6] = bf16_lo(yraw.w); y[7] = bf16_hi(yraw.w);
      if (base + 8 > vocab) {  // the draft vocabulary ends inside this chunk (the last tile only)
        const uint32_t yw[4] = {yraw.x, yraw.y, yraw.z, yraw.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (base + i < vocab) {
            if (grow) grow[base + i] = (uint16_t)(yw[i >> 1] >> (16 * (i & 1)));
          } else {
            x[i] = kNegBig; y[i] = kNegBig;  // tail padding, like load8_guard
          }
        }
      }
      float cx = x[0], cy = y[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) { cx = fmaxf(cx, x[i]); cy = fmaxf(cy, y[i]); }
      if (cx > s.bd) {  // strict: an earlier chunk of this thread keeps a tie
        int k = 7;
#pragma unroll
        for (int i = 6; i >= 0; --i) k = (x[i] == cx) ? i : k;
        s.bd = cx; s.id = (int)base + k;
      }
      if (cy > s.bt) {
        int k = 7;
        float xv = x[7];
#pragma unroll
        for (int i = 6; i >= 0; --i) {
          const bool hit = y[i] == cy;
          k = hit ? i : k;
          xv = hit ? x[i] : xv;
        }
        s.bt = cy; s.it = (int)base + k; s.xt = xv;
      }
      {
        const float cxs = cx * kLog2e;
        float mn = s.md, z = s.zd;
        if (cxs > mn) {
          z *= fast_exp2(mn - cxs);
          mn = cxs;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) z += fast_exp2(fmaf(x[i], kLog2e, -mn));
        s.zd = z; s.md = mn;
      }
      if (OP != SPX_LOSS_CE) {
        float mn = fmaxf(s.mt, cy * kLog2e);
        float rs = fast_exp2(s.mt - mn);
        float z = s.zt * rs, a = s.at * rs;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float e = fast_exp2(fmaf(y[i], kLog2e, -mn));
          z += e;
          a = fmaf(e, y[i] - x[i], a);
        }
        s.zt = z; s.at = a; s.mt = mn;
      }
    }
  };

  int off_a[8], off_b[8];
  load_offsets(0, off_a);
  request(0);
  request(1);
  // two tiles per trip: the two register sets swap roles, nothing is copied; an odd tile count runs one
  // tile past the end (all of its work is switched off by its ids)
  for (int t = 0; t < ntiles; t += 2) {
    tile(t, off_a, off_b);
    tile(t + 1, off_b, off_a);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the requests past the end still write LDS
  __syncthreads();

#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) merge(s, shuffle_xor(s, m));
  __shared__ RowStats part[kLossWaves];
  if (lane == 0) part[wave] = s;
  __syncthreads();
  s = part[0];
#pragma unroll
  for (int w = 1; w < kLossWaves; ++w) merge(s, part[w]);
  const float lse_d = (s.md + fast_log2(s.zd)) * kLn2;
  const float lse_t = (OP != SPX_LOSS_CE) ? (s.mt + fast_log2(s.zt)) * kLn2 : 0.f;
  float row_loss;
  if (OP == SPX_LOSS_KL) row_loss = s.at / s.zt - lse_t + lse_d;
  else row_loss = lse_d - s.xt;
  if (tid == 0) {
    loss[r] = row_loss;
    lse_draft[r] = lse_d;
    extra[r] = (OP == SPX_LOSS_KL) ? row_loss : 0.f;
    if (argmax_draft) argmax_draft[r] = s.id;
    lse_target[r] = lse_t;
    if (argmax_target) argmax_target[r] = s.it;
    if (sa.counts) {
      const bool m = sa.mask ? mask_value(sa.mask, sa.mask_kind, r) != 0.f : true;
      const bool was = sa.prev ? mask_value(sa.prev, sa.prev_kind, r) != 0.f : true;
      const bool now = was && (s.id == s.it);
      if (m && now) atomicAdd(&sa.counts[0], 1);
      if (m) atomicAdd(&sa.counts[1], 1);
      if (was) atomicAdd(&sa.counts[2], 1);
      if (sa.prev) store_flag(sa.prev, sa.prev_kind, r, now);
    }
  }
}

// ---- backward --------------------------------------------------------------
template <typename T, int OP, bool VEC>
__global__ __launch_bounds__(kLossThreads) void loss_bwd_kernel(
    const T* __restrict__ logits, int64_t ld_logits, const T* __restrict__ targets,
    int64_t ld_targets, int64_t vocab, const float* __restrict__ lse_draft,
    const float* __restrict__ lse_target, const float* __restrict__ extra,
    const int32_t* __restrict__ argmax_target, const float* __restrict__ row_grad,
    const float* __restrict__ scale, T* __restrict__ grad, int64_t ld_grad,
    const int32_t* __restrict__ row_map) {
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t nchunks = (vocab + 7) >> 3;
  // with a row map the gradient of row r goes to row row_map[r] and rows mapped to -1 (zero gradient)
  // are not written: the live rows packed to the front
  int64_t dst = r;
  if (row_map) {
    dst = row_map[r];
    if (dst < 0) return;
  }
  T* grow = grad + dst * ld_grad;
  float g = row_grad[r];
  if (scale) g *= *scale;
  if (g == 0.f) {
    const float z[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t c = tid; c < nchunks; c += kLossThreads) store8<T, VEC>(grow, c << 3, vocab, z);
    return;
  }
  const T* xrow = logits + r * ld_logits;
  const T* yrow = (OP != SPX_LOSS_CE) ? targets + r * ld_targets : nullptr;
  const float lse_d = lse_draft[r];
  const float lse_t = (OP != SPX_LOSS_CE) ? lse_target[r] : 0.f;
  const float ex = (OP == SPX_LOSS_RKL || OP == SPX_LOSS_JSD || OP == SPX_LOSS_TV) ? extra[r] : 0.f;
  const int label = (OP == SPX_LOSS_CE) ? argmax_target[r] : -1;
  const float cd = -lse_d * kLog2e, ct = -lse_t * kLog2e;

#define SPX_LOSS_BWD_UNROLL 1
  constexpr int UNR = SPX_LOSS_BWD_UNROLL;
  for (int64_t c0 = tid; c0 < nchunks; c0 += kLossThreads * UNR) {
    float xs[UNR][8], ys[UNR][8];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int64_t c = c0 + (int64_t)u * kLossThreads;
      if (c < nchunks) {
        load8<T, VEC>(xrow, c << 3, vocab, xs[u]);
        if (OP != SPX_LOSS_CE) load8<T, VEC>(yrow, c << 3, vocab, ys[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
    const int64_t c = c0 + (int64_t)u * kLossThreads;
    if (c >= nchunks) break;
    const int64_t base = c << 3;
    float o[8];
    float* x = xs[u];
    float* y = ys[u];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (OP == SPX_LOSS_CE) {
        float dp = fast_exp2(fmaf(x[i], kLog2e, cd));
        o[i] = g * (dp - (((int)base + i) == label ? 1.f : 0.f));
      } else if (OP == SPX_LOSS_KL) {
        float dp = fast_exp2(fmaf(x[i], kLog2e, cd));
        float tp = fast_exp2(fmaf(y[i], kLog2e, ct));
        o[i] = g * (dp - tp);
      } else {
        // same expressions as the forward's second pass, so that the
        // q <= p comparison of tv resolves identically in both directions
        float ldp = x[i] - lse_d, ltp = y[i] - lse_t;
        float dp = fast_exp2(ldp * kLog2e), tp = fast_exp2(ltp * kLog2e);
        if (OP == SPX_LOSS_RKL) o[i] = g * dp * (ldp - ltp - ex);
        else if (OP == SPX_LOSS_JSD) o[i] = g * 0.5f * dp * (ldp - log_mix(ldp, ltp) - ex);
        else o[i] = -g * dp * ((dp <= tp ? 1.f : 0.f) - ex);
      }
    }
    store8<T, VEC>(grow, base, vocab, o);
    }
  }
}

// ---- gather through the d2t offset table -------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void vocab_gather_kernel(
    const T* __restrict__ full, int64_t ld_full, const int64_t* __restrict__ d2t,
    T* __restrict__ out, int64_t ld_out, int64_t vd, int64_t vt, T neg_inf_bits) {
  const int64_t r = blockIdx.y;
  const T* src = full + r * ld_full;
  T* dst = out + r * ld_out;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < vd; i += (int64_t)gridDim.x * 256) {
    int64_t j = i + d2t[i];
    dst[i] = (j >= 0 && j < vt) ? src[j] : neg_inf_bits;
  }
}

constexpr int kReduceThreads = 1024;

__device__ __forceinline__ float block_sum_f(float v, float* lds) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < kReduceThreads / 64; ++w) t += lds[w];
  return t;
}
__device__ __forceinline__ int block_sum_i(int v, int* lds) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  int t = 0;
  for (int w = 0; w < kReduceThreads / 64; ++w) t += lds[w];
  return t;
}

__global__ __launch_bounds__(kReduceThreads) void ttt_step_reduce_kernel(
    const float* __restrict__ loss, const int32_t* __restrict__ pred,
    const int32_t* __restrict__ tgt, const void* __restrict__ mask, int mask_kind,
    void* prev, int prev_kind, int64_t rows, float weight, float* __restrict__ out,
    float* __restrict__ row_weight, const int32_t* __restrict__ counts) {
  __shared__ float fl[kReduceThreads / 64];
  __shared__ int il[kReduceThreads / 64];
  float lsum = 0.f, msum = 0.f;
  int full_total = 0, correct = 0, cond_total = 0;
  // counts != nullptr: the acceptance chain was done row by row in the loss pass (StepArgs);
  // only the masked mean is left here and the counts are copied out
  for (int64_t r = threadIdx.x; r < rows; r += kReduceThreads) {
    float m = mask ? mask_value(mask, mask_kind, r) : 1.f;
    if (!counts) {
      bool was = prev ? (mask_value(prev, prev_kind, r) != 0.f) : true;
      bool hit = pred[r] == tgt[r];
      bool now = was && hit;
      cond_total += was ? 1 : 0;
      if (prev) store_flag(prev, prev_kind, r, now);
      if (m != 0.f) { full_total += 1; correct += now ? 1 : 0; }
    }
    lsum = fmaf(loss[r], m, lsum);
    msum += m;
  }
  lsum = block_sum_f(lsum, fl);
  msum = block_sum_f(msum, fl);
  if (!counts) {
    full_total = block_sum_i(full_total, il);
    correct = block_sum_i(correct, il);
    cond_total = block_sum_i(cond_total, il);
  } else {
    correct = counts[0]; full_total = counts[1]; cond_total = counts[2];
  }
  const float inv = weight / (msum + 1e-5f);
  if (threadIdx.x == 0) {
    out[0] = lsum * inv;
    out[1] = (float)correct;
    out[2] = (float)full_total;
    out[3] = (float)correct;
    out[4] = (prev || counts) ? (float)cond_total : (float)rows;
    out[5] = msum;
  }
  if (row_weight) {
    for (int64_t r = threadIdx.x; r < rows; r += kReduceThreads) {
      float m = mask ? mask_value(mask, mask_kind, r) : 1.f;
      row_weight[r] = m * inv;
    }
  }
}

__global__ __launch_bounds__(kReduceThreads) void block_reduce_kernel(
    const float* __restrict__ loss, const int32_t* __restrict__ pred,
    const int32_t* __restrict__ tgt, const void* __restrict__ mask, int mask_kind,
    const float* __restrict__ pos_weight, int64_t rows, int block_size, float* __restrict__ out,
    float* __restrict__ correct, float* __restrict__ total, float* __restrict__ row_weight) {
  __shared__ float fl[kReduceThreads / 64];
  extern __shared__ int slots[];  // [2 * block_size]
  for (int i = threadIdx.x; i < 2 * block_size; i += kReduceThreads) slots[i] = 0;
  __syncthreads();
  float lsum = 0.f, msum = 0.f;
  for (int64_t r = threadIdx.x; r < rows; r += kReduceThreads) {
    float m = mask ? mask_value(mask, mask_kind, r) : 1.f;
    float w = pos_weight ? pos_weight[r] : 1.f;
    if (m != 0.f) {
      int s = (int)(r % block_size);
      atomicAdd(&slots[block_size + s], 1);
      if (pred[r] == tgt[r]) atomicAdd(&slots[s], 1);
    }
    lsum = fmaf(loss[r] * m, w, lsum);
    msum += m;
  }
  lsum = block_sum_f(lsum, fl);
  msum = block_sum_f(msum, fl);
  const float inv = 1.f / (msum + 1e-5f);
  if (threadIdx.x == 0) { out[0] = lsum * inv; out[1] = msum; }
  __syncthreads();
  for (int i = threadIdx.x; i < block_size; i += kReduceThreads) {
    correct[i] = (float)slots[i];
    total[i] = (float)slots[block_size + i];
  }
  if (row_weight) {
    for (int64_t r = threadIdx.x; r < rows; r += kReduceThreads) {
      float m = mask ? mask_value(mask, mask_kind, r) : 1.f;
      float w = pos_weight ? pos_weight[r] : 1.f;
      row_weight[r] = m * w * inv;
    }
  }
}

// ---- dispatch ----------------------------------------------------------------
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T, bool VEC, bool KNOWN, bool GATHER>
static void launch_fwd(int op, const T* lg, int64_t ldl, const T* tg, int64_t ldt, int64_t rows,
                       int64_t vocab, float* loss, float* lsd, float* lst, float* ex, int32_t* ad,
                       int32_t* at, const StepArgs& sa, hipStream_t st) {
  dim3 grid((unsigned)rows), block(kLossThreads);
#define SPX_FWD(OPV)                                                                                 \
  case OPV:                                                                                          \
    hipLaunchKernelGGL((loss_fwd_kernel<T, OPV, VEC, KNOWN, GATHER>), grid, block, 0, st, lg, ldl,   \
                       tg, ldt, vocab, loss, lsd, lst, ex, ad, at, sa);                              \
    break;
  switch (op) {
    SPX_FWD(SPX_LOSS_KL) SPX_FWD(SPX_LOSS_RKL) SPX_FWD(SPX_LOSS_JSD) SPX_FWD(SPX_LOSS_CE)
    SPX_FWD(SPX_LOSS_TV)
  }
#undef SPX_FWD
}

template <typename T, bool VEC>
static void launch_bwd(int op, const T* lg, int64_t ldl, const T* tg, int64_t ldt, int64_t rows,
                       int64_t vocab, const float* lsd, const float* lst, const float* ex,
                       const int32_t* at, const float* rg, const float* sc, T* grad, int64_t ldg,
                       const int32_t* row_map, hipStream_t st) {
  dim3 grid((unsigned)rows), block(kLossThreads);
#define SPX_BWD(OPV)                                                                         \
  case OPV:                                                                                  \
    hipLaunchKernelGGL((loss_bwd_kernel<T, OPV, VEC>), grid, block, 0, st, lg, ldl, tg, ldt, \
                       vocab, lsd, lst, ex, at, rg, sc, grad, ldg, row_map);                 \
    break;
  switch (op) {
    SPX_BWD(SPX_LOSS_KL) SPX_BWD(SPX_LOSS_RKL) SPX_BWD(SPX_LOSS_JSD) SPX_BWD(SPX_LOSS_CE)
    SPX_BWD(SPX_LOSS_TV)
  }
#undef SPX_BWD
}

}  // namespace spx

using namespace spx;

static bool kind_ok(int k) { return k >= SPX_KIND_U8 && k <= SPX_KIND_BF16; }

#define SPX_REQ_FN(cond, what) do { if (!(cond)) return spx::fail_arg(fname, what); } while (0)
static int loss_fwd_impl(const char* fname, int op, const void* logits, int64_t ld_logits,
                         const void* targets, int64_t ld_targets, int64_t rows, int64_t vocab,
                         int dtype, float* loss, float* lse_draft, float* lse_target, float* extra,
                         int32_t* argmax_draft, int32_t* argmax_target, int reuse_target_stats,
                         const StepArgs& sa, void* stream) {
  SPX_REQ_FN(op >= SPX_LOSS_KL && op <= SPX_LOSS_TV, "unknown loss op");
  SPX_REQ_FN(dtype == SPX_DTYPE_BF16 || dtype == SPX_DTYPE_F32, "dtype must be bf16 or f32");
  SPX_REQ_FN(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "rows >= 0 and 0 < vocab < 2^31");
  const bool gather = sa.d2t != nullptr;
  // cross-entropy with the target rows' arg-max handed in reads no target element: the rows may be absent
  const bool no_targets = !targets && reuse_target_stats && op == SPX_LOSS_CE && !gather;
  SPX_REQ_FN(ld_logits >= vocab && (no_targets || ld_targets >= (gather ? sa.vt : vocab)),
             "row stride smaller than vocab");
  SPX_REQ_FN(rows < (1ll << 31), "too many rows");
  if (gather) {
    SPX_REQ_FN(sa.vt > 0 && sa.vt < (1ll << 31), "0 < vt < 2^31");
    SPX_REQ_FN(!reuse_target_stats, "the gather form computes the target statistics itself");
    SPX_REQ_FN(!sa.gathered || sa.ld_gathered >= vocab, "gathered row stride smaller than vocab");
  }
  if (sa.counts) {
    SPX_REQ_FN(argmax_draft && argmax_target, "the acceptance chain needs both arg-max outputs");
    SPX_REQ_FN(!sa.mask || kind_ok(sa.mask_kind), "unknown mask element kind");
    SPX_REQ_FN(!sa.prev || kind_ok(sa.prev_kind), "unknown prev_correct element kind");
  }
  if (rows == 0) return SPX_OK;
  SPX_REQ_FN(logits && (targets || no_targets) && loss && lse_draft && lse_target && extra, "null buffer");
  // the second-pass reductions (rkl, jsd, tv) recompute from both rows anyway
  const bool known = reuse_target_stats && (op == SPX_LOSS_KL || op == SPX_LOSS_CE);
  if (known && op == SPX_LOSS_CE) SPX_REQ_FN(argmax_target, "ce with reused statistics needs argmax_target");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t per16 = dtype == SPX_DTYPE_BF16 ? 8 : 4;
  const bool vec = aligned16(logits) && ld_logits % per16 == 0 &&
                   (gather ? (!sa.gathered || (aligned16(sa.gathered) && sa.ld_gathered % per16 == 0))
                           : (no_targets || (aligned16(targets) && ld_targets % per16 == 0)));
  // the first step of the verifier-logits entry in its common form: the pipelined kernel
  if (gather && vec && dtype == SPX_DTYPE_BF16 && (op == SPX_LOSS_KL || op == SPX_LOSS_CE) &&
      aligned16(targets) && ld_targets % 8 == 0 && vocab <= (int64_t)kPipeMaxTiles * kPipeTileIds &&
      sa.vt < (1ll << 30)) {
    static std::atomic<uint64_t> lds_set[2];  // per instantiation, one bit per device
    const bool kl = op == SPX_LOSS_KL;
    const void* fn = kl ? reinterpret_cast<const void*>(&loss_fwd_gather_pipe_kernel<SPX_LOSS_KL>)
                        : reinterpret_cast<const void*>(&loss_fwd_gather_pipe_kernel<SPX_LOSS_CE>);
    if (int rc = ensure_dynamic_lds(fn, kPipeSmem, lds_set[kl], fname)) return rc;
    const dim3 grid((unsigned)rows), block(kLossThreads);
    auto lg = reinterpret_cast<const uint16_t*>(logits);
    auto tg = reinterpret_cast<const uint16_t*>(targets);
    if (kl)
      hipLaunchKernelGGL(loss_fwd_gather_pipe_kernel<SPX_LOSS_KL>, grid, block, kPipeSmem, st, lg, ld_logits, tg,
                         ld_targets, vocab, loss, lse_draft, lse_target, extra, argmax_draft, argmax_target, sa);
    else
      hipLaunchKernelGGL(loss_fwd_gather_pipe_kernel<SPX_LOSS_CE>, grid, block, kPipeSmem, st, lg, ld_logits, tg,
                         ld_targets, vocab, loss, lse_draft, lse_target, extra, argmax_draft, argmax_target, sa);
    return check_launch(fname);
  }
#define SPX_GO(TT, VV, KK, GG)                                                                    \
  launch_fwd<TT, VV, KK, GG>(op, reinterpret_cast<const TT*>(logits), ld_logits,                  \
                             reinterpret_cast<const TT*>(targets), ld_targets, rows, vocab, loss, \
                             lse_draft, lse_target, extra, argmax_draft, argmax_target, sa, st)
#define SPX_GO_T(TT)                                                                   \
  do {                                                                                 \
    if (gather) { if (vec) SPX_GO(TT, true, false, true); else SPX_GO(TT, false, false, true); } \
    else if (vec) { if (known) SPX_GO(TT, true, true, false); else SPX_GO(TT, true, false, false); } \
    else { if (known) SPX_GO(TT, false, true, false); else SPX_GO(TT, false, false, false); } \
  } while (0)
  if (dtype == SPX_DTYPE_BF16) SPX_GO_T(uint16_t);
  else SPX_GO_T(float);
#undef SPX_GO_T
#undef SPX_GO
  return check_launch(fname);
}

extern "C" int spx_fused_vocab_loss_fwd(int op, const void* logits, int64_t ld_logits,
                                        const void* targets, int64_t ld_targets, int64_t rows,
                                        int64_t vocab, int dtype, float* loss, float* lse_draft,
                                        float* lse_target, float* extra, int32_t* argmax_draft,
                                        int32_t* argmax_target, int reuse_target_stats,
                                        void* stream) {
  const StepArgs none = {nullptr, 0, nullptr, 0, nullptr, 0, nullptr, 0, nullptr};
  return loss_fwd_impl(__func__, op, logits, ld_logits, targets, ld_targets, rows, vocab, dtype, loss,
                       lse_draft, lse_target, extra, argmax_draft, argmax_target, reuse_target_stats,
                       none, stream);
}

extern "C" int spx_vocab_loss_step_fwd(int op, const void* logits, int64_t ld_logits,
                                       const void* targets, int64_t ld_targets, const int64_t* d2t,
                                       int64_t vt, void* gathered, int64_t ld_gathered, int64_t rows,
                                       int64_t vocab, int dtype, float* loss, float* lse_draft,
                                       float* lse_target, float* extra, int32_t* argmax_draft,
                                       int32_t* argmax_target, int reuse_target_stats,
                                       const void* mask, int mask_kind, void* prev_correct,
                                       int prev_kind, int32_t* counts, void* stream) {
  const StepArgs sa = {d2t, vt, gathered, ld_gathered, mask, mask_kind, prev_correct, prev_kind, counts};
  return loss_fwd_impl(__func__, op, logits, ld_logits, targets, ld_targets, rows, vocab, dtype, loss,
                       lse_draft, lse_target, extra, argmax_draft, argmax_target, reuse_target_stats,
                       sa, stream);
}

extern "C" int spx_vocab_loss_step_fwd_grad(int op, const void* logits, int64_t ld_logits,
                                            const void* targets, int64_t ld_targets, int64_t rows,
                                            int64_t vocab, float* loss, float* lse_draft,
                                            float* lse_target, float* extra, int32_t* argmax_draft,
                                            int32_t* argmax_target, int reuse_target_stats,
                                            const void* mask, int mask_kind, void* prev_correct,
                                            int prev_kind, int32_t* counts, const int32_t* row_map,
                                            void* grad_logits, int64_t ld_grad, void* stream) {
  const char* fname = __func__;
  SPX_REQ_FN(op == SPX_LOSS_KL || op == SPX_LOSS_CE, "the one-pass form is built for kl and ce");
  SPX_REQ_FN(rows >= 0 && rows < (1ll << 31), "bad row count");
  SPX_REQ_FN(vocab > 0 && vocab % 8 == 0 && vocab <= (int64_t)kFgThreads * kFgChunks * 8,
             "vocab must be a multiple of 8, at most 32768");
  const bool known = reuse_target_stats != 0;
  const bool no_targets = known && op == SPX_LOSS_CE;
  SPX_REQ_FN(ld_logits >= vocab && ld_grad >= vocab && (no_targets || ld_targets >= vocab),
             "row stride smaller than vocab");
  SPX_REQ_FN(ld_logits % 8 == 0 && ld_grad % 8 == 0 && (no_targets || ld_targets % 8 == 0),
             "row strides must be multiples of 8 elements");
  if (counts) {
    SPX_REQ_FN(!mask || kind_ok(mask_kind), "unknown mask element kind");
    SPX_REQ_FN(!prev_correct || kind_ok(prev_kind), "unknown prev_correct element kind");
  }
  if (rows == 0) return SPX_OK;
  SPX_REQ_FN(logits && (targets || no_targets) && loss && lse_draft && lse_target && extra && argmax_target &&
                 row_map && grad_logits, "null buffer");
  SPX_REQ_FN(!counts || argmax_draft, "the acceptance chain needs both arg-max outputs");
  SPX_REQ_FN(aligned16(logits) && aligned16(grad_logits) && (no_targets || aligned16(targets)),
             "rows must be 16-byte aligned");
  const StepArgs sa = {nullptr, 0, nullptr, 0, mask, mask_kind, prev_correct, prev_kind, counts};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)rows), block(kFgThreads);
  auto lg = reinterpret_cast<const uint16_t*>(logits);
  auto tg = reinterpret_cast<const uint16_t*>(targets);
  auto gr = reinterpret_cast<uint16_t*>(grad_logits);
#define SPX_FG(OPV, KN)                                                                                     \
  hipLaunchKernelGGL((loss_fwd_grad_kernel<OPV, KN>), grid, block, 0, st, lg, ld_logits, tg, ld_targets, vocab, \
                     loss, lse_draft, lse_target, extra, argmax_draft, argmax_target, sa, row_map, gr, ld_grad)
  if (op == SPX_LOSS_KL) { if (known) SPX_FG(SPX_LOSS_KL, true); else SPX_FG(SPX_LOSS_KL, false); }
  else { if (known) SPX_FG(SPX_LOSS_CE, true); else SPX_FG(SPX_LOSS_CE, false); }
#undef SPX_FG
  return check_launch(fname);
}

static int loss_bwd_impl(const char* fname, int op, const void* logits, int64_t ld_logits,
                         const void* targets, int64_t ld_targets, int64_t rows,
                         int64_t vocab, int dtype, const float* lse_draft,
                         const float* lse_target, const float* extra,
                         const int32_t* argmax_target, const float* row_grad,
                         const float* scale, void* grad_logits, int64_t ld_grad,
                         const int32_t* row_map, void* stream) {
  SPX_REQ_FN(op >= SPX_LOSS_KL && op <= SPX_LOSS_TV, "unknown loss op");
  SPX_REQ_FN(dtype == SPX_DTYPE_BF16 || dtype == SPX_DTYPE_F32, "dtype must be bf16 or f32");
  SPX_REQ_FN(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "rows >= 0 and 0 < vocab < 2^31");
  SPX_REQ_FN(ld_logits >= vocab && ld_grad >= vocab, "row stride smaller than vocab");
  SPX_REQ_FN(rows < (1ll << 31), "too many rows");
  if (rows == 0) return SPX_OK;
  SPX_REQ_FN(logits && grad_logits && lse_draft && row_grad, "null buffer");
  if (op == SPX_LOSS_CE) SPX_REQ_FN(argmax_target, "ce needs argmax_target");
  else SPX_REQ_FN(targets && lse_target && ld_targets >= vocab, "targets / lse_target missing");
  if (op == SPX_LOSS_RKL || op == SPX_LOSS_JSD || op == SPX_LOSS_TV) SPX_REQ_FN(extra, "extra missing");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t per16 = dtype == SPX_DTYPE_BF16 ? 8 : 4;
  const bool vec = aligned16(logits) && (op == SPX_LOSS_CE || (aligned16(targets) && ld_targets % per16 == 0)) &&
                   aligned16(grad_logits) && ld_logits % per16 == 0 && ld_grad % per16 == 0;
  if (dtype == SPX_DTYPE_BF16) {
    auto lg = reinterpret_cast<const uint16_t*>(logits);
    auto tg = reinterpret_cast<const uint16_t*>(targets);
    auto gr = reinterpret_cast<uint16_t*>(grad_logits);
    if (vec) launch_bwd<uint16_t, true>(op, lg, ld_logits, tg, ld_targets, rows, vocab, lse_draft, lse_target, extra, argmax_target, row_grad, scale, gr, ld_grad, row_map, st);
    else launch_bwd<uint16_t, false>(op, lg, ld_logits, tg, ld_targets, rows, vocab, lse_draft, lse_target, extra, argmax_target, row_grad, scale, gr, ld_grad, row_map, st);
  } else {
    auto lg = reinterpret_cast<const float*>(logits);
    auto tg = reinterpret_cast<const float*>(targets);
    auto gr = reinterpret_cast<float*>(grad_logits);
    if (vec) launch_bwd<float, true>(op, lg, ld_logits, tg, ld_targets, rows, vocab, lse_draft, lse_target, extra, argmax_target, row_grad, scale, gr, ld_grad, row_map, st);
    else launch_bwd<float, false>(op, lg, ld_logits, tg, ld_targets, rows, vocab, lse_draft, lse_target, extra, argmax_target, row_grad, scale, gr, ld_grad, row_map, st);
  }
  return check_launch(fname);
}
#undef SPX_REQ_FN

extern "C" int spx_fused_vocab_loss_bwd(int op, const void* logits, int64_t ld_logits,
                                        const void* targets, int64_t ld_targets, int64_t rows,
                                        int64_t vocab, int dtype, const float* lse_draft,
                                        const float* lse_target, const float* extra,
                                        const int32_t* argmax_target, const float* row_grad,
                                        const float* scale, void* grad_logits, int64_t ld_grad,
                                        void* stream) {
  return loss_bwd_impl(__func__, op, logits, ld_logits, targets, ld_targets, rows, vocab, dtype, lse_draft,
                       lse_target, extra, argmax_target, row_grad, scale, grad_logits, ld_grad, nullptr, stream);
}

extern "C" int spx_fused_vocab_loss_bwd_packed(int op, const void* logits, int64_t ld_logits,
                                               const void* targets, int64_t ld_targets, int64_t rows,
                                               int64_t vocab, int dtype, const float* lse_draft,
                                               const float* lse_target, const float* extra,
                                               const int32_t* argmax_target, const float* row_grad,
                                               const float* scale, const int32_t* row_map,
                                               void* grad_logits, int64_t ld_grad, void* stream) {
  if (!row_map) return spx::fail_arg(__func__, "null row map");
  return loss_bwd_impl(__func__, op, logits, ld_logits, targets, ld_targets, rows, vocab, dtype, lse_draft,
                       lse_target, extra, argmax_target, row_grad, scale, grad_logits, ld_grad, row_map, stream);
}

extern "C" int spx_vocab_gather(const void* full, int64_t ld_full, const int64_t* d2t, void* out,
                                int64_t ld_out, int64_t rows, int64_t vd, int64_t vt, int dtype,
                                void* stream) {
  SPX_REQUIRE(dtype == SPX_DTYPE_BF16 || dtype == SPX_DTYPE_F32, "dtype must be bf16 or f32");
  SPX_REQUIRE(rows >= 0 && vd > 0 && vt > 0, "rows >= 0, vd > 0, vt > 0");
  SPX_REQUIRE(ld_full >= vt && ld_out >= vd, "row stride smaller than the row");
  SPX_REQUIRE(rows < 65536, "at most 65535 rows per call");
  if (rows == 0) return SPX_OK;
  SPX_REQUIRE(full && d2t && out, "null buffer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  unsigned gx = (unsigned)((vd + 256 * 4 - 1) / (256 * 4));
  dim3 grid(gx, (unsigned)rows), block(256);
  if (dtype == SPX_DTYPE_BF16)
    hipLaunchKernelGGL(vocab_gather_kernel<uint16_t>, grid, block, 0, st,
                       reinterpret_cast<const uint16_t*>(full), ld_full, d2t,
                       reinterpret_cast<uint16_t*>(out), ld_out, vd, vt, (uint16_t)0xff80);
  else
    hipLaunchKernelGGL(vocab_gather_kernel<float>, grid, block, 0, st,
                       reinterpret_cast<const float*>(full), ld_full, d2t,
                       reinterpret_cast<float*>(out), ld_out, vd, vt, -INFINITY);
  return check_launch(__func__);
}

extern "C" int spx_ttt_step_reduce(const float* loss, const int32_t* argmax_draft,
                                   const int32_t* argmax_target, const void* mask, int mask_kind,
                                   void* prev_correct, int prev_kind, int64_t rows, float weight,
                                   float* out, float* row_weight, void* stream) {
  SPX_REQUIRE(rows >= 0 && rows < (1ll << 24), "0 <= rows < 2^24");
  SPX_REQUIRE(loss && argmax_draft && argmax_target && out, "null buffer");
  SPX_REQUIRE(!mask || kind_ok(mask_kind), "unknown mask element kind");
  SPX_REQUIRE(!prev_correct || kind_ok(prev_kind), "unknown prev_correct element kind");
  hipLaunchKernelGGL(ttt_step_reduce_kernel, dim3(1), dim3(kReduceThreads), 0,
                     reinterpret_cast<hipStream_t>(stream), loss, argmax_draft, argmax_target, mask,
                     mask_kind, prev_correct, prev_kind, rows, weight, out, row_weight, nullptr);
  return check_launch(__func__);
}

extern "C" int spx_ttt_step_mean(const float* loss, const void* mask, int mask_kind, int64_t rows,
                                 float weight, const int32_t* counts, float* out, float* row_weight,
                                 void* stream) {
  SPX_REQUIRE(rows >= 0 && rows < (1ll << 24), "0 <= rows < 2^24");
  SPX_REQUIRE(loss && counts && out, "null buffer");
  SPX_REQUIRE(!mask || kind_ok(mask_kind), "unknown mask element kind");
  hipLaunchKernelGGL(ttt_step_reduce_kernel, dim3(1), dim3(kReduceThreads), 0,
                     reinterpret_cast<hipStream_t>(stream), loss, nullptr, nullptr, mask, mask_kind,
                     nullptr, 0, rows, weight, out, row_weight, counts);
  return check_launch(__func__);
}

extern "C" int spx_block_reduce(const float* loss, const int32_t* argmax_draft,
                                const int32_t* argmax_target, const void* mask, int mask_kind,
                                const float* pos_weight, int64_t rows, int32_t block_size,
                                float* out, float* correct, float* total, float* row_weight,
                                void* stream) {
  SPX_REQUIRE(rows >= 0 && rows < (1ll << 24), "0 <= rows < 2^24");
  SPX_REQUIRE(block_size > 0 && block_size <= 4096, "0 < block_size <= 4096");
  SPX_REQUIRE(loss && argmax_draft && argmax_target && out && correct && total, "null buffer");
  SPX_REQUIRE(!mask || kind_ok(mask_kind), "unknown mask element kind");
  hipLaunchKernelGGL(block_reduce_kernel, dim3(1), dim3(kReduceThreads),
                     2 * block_size * sizeof(int), reinterpret_cast<hipStream_t>(stream), loss,
                     argmax_draft, argmax_target, mask, mask_kind, pos_weight, rows, block_size, out,
                     correct, total, row_weight);
  return check_launch(__func__);
}
