// Cross-entropy of full-vocabulary logits against integer labels with an
// ignore index (the multi-token-prediction loss), for gfx950.  One workgroup
// streams one logits row once with 16-byte non-temporal loads and keeps the
// online soft-max statistics in registers: loss = logsumexp(x) - x[label].
// Ignored rows are not read at all.  HBM-bound: algorithmic traffic is one row
// read (forward), one row read + one row written (backward).
//
// Exponentials run in the base-2 domain (v_exp_f32 is 2^x).

#include "loss_common.h"
#include "../../include/spx.h"

namespace spx {

struct CeStats {
  float m, z;       // running max of x * log2(e), sum of 2^(x' - m)
  float best; int idx;  // arg-max value (unscaled) / first index
};

__device__ __forceinline__ void ce_merge(CeStats& a, float bm, float bz, float bb, int bi) {
  const float m = fmaxf(a.m, bm);
  a.z = a.z * fast_exp2(a.m - m) + bz * fast_exp2(bm - m);
  a.m = m;
  if (bb > a.best || (bb == a.best && bi < a.idx)) { a.best = bb; a.idx = bi; }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kLossThreads) void label_ce_fwd_kernel(
    const T* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels, int64_t vocab,
    int64_t ignore_index, float* __restrict__ loss, float* __restrict__ lse_out,
    int32_t* __restrict__ argmax_out) {
  __shared__ float sm[kLossWaves], sz[kLossWaves], sb[kLossWaves];
  __shared__ int si[kLossWaves];
  const int64_t r = blockIdx.x;
  const int64_t label = labels[r];
  const bool ignored = label == ignore_index;
  if (ignored && argmax_out == nullptr) {  // uniform over the workgroup
    if (threadIdx.x == 0) { loss[r] = 0.f; lse_out[r] = 0.f; }
    return;
  }
  const T* row = logits + r * ld;
  const int tid = threadIdx.x;
  const int64_t nchunks = (vocab + 7) >> 3;

  CeStats s;
  s.m = kNegBig; s.z = 0.f; s.best = -INFINITY; s.idx = 0x7fffffff;
  for (int64_t c = tid; c < nchunks; c += kLossThreads) {
    const int64_t base = c << 3;
    float x[8];
    load8<T, VEC>(row, base, vocab, x);
    float cm = x[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) cm = fmaxf(cm, x[i]);
    if (cm > s.best) {
      // first index inside the chunk that attains the chunk maximum
      int k = 7;
#pragma unroll
      for (int i = 6; i >= 0; --i) k = (x[i] == cm) ? i : k;
      s.best = cm; s.idx = (int)base + k;
    }
    const float cm2 = cm * kLog2e;
    if (cm2 > s.m) {  // the running maximum moved: rescale the sum
      s.z *= fast_exp2(s.m - cm2);
      s.m = cm2;
    }
    float zz = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) zz += fast_exp2(fmaf(x[i], kLog2e, -s.m));
    s.z += zz;
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1)
    ce_merge(s, __shfl_xor(s.m, m, 64), __shfl_xor(s.z, m, 64), __shfl_xor(s.best, m, 64),
             __shfl_xor(s.idx, m, 64));
  if ((tid & 63) == 0) { sm[tid >> 6] = s.m; sz[tid >> 6] = s.z; sb[tid >> 6] = s.best; si[tid >> 6] = s.idx; }
  __syncthreads();
  if (tid == 0) {
#pragma unroll
    for (int w = 1; w < kLossWaves; ++w) ce_merge(s, sm[w], sz[w], sb[w], si[w]);
    const float lse = (s.m + fast_log2(s.z)) * kLn2;
    float l = 0.f;
    if (!ignored) {
      // a label outside [0, vocab) that is not the ignore index has no defined loss
      l = (label >= 0 && label < vocab) ? lse - load1(row + label) : __builtin_nanf("");
    }
    loss[r] = l;
    lse_out[r] = lse;
    if (argmax_out) argmax_out[r] = s.idx;
  }
}

// dlogits[r, j] = g[r] * (softmax(x[r])[j] - [j == label[r]]); rows with g == 0 or an ignored
// label are written as zeros without reading the logits.  With a row map the gradient of row r
// goes to row row_map[r] of the output and rows mapped to -1 are not written at all (the live
// rows packed to the front: the product that consumes them skips the dead ones).
template <typename T, bool VEC>
__global__ __launch_bounds__(kLossThreads) void label_ce_bwd_kernel(
    const T* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels,
    const float* __restrict__ lse, const float* __restrict__ grad_rows, int64_t vocab,
    int64_t ignore_index, T* __restrict__ dlogits, int64_t ld_out, const int32_t* __restrict__ row_map) {
  const int64_t r = blockIdx.x;
  const int64_t label = labels[r];
  const float g = grad_rows[r];
  const T* row = logits + r * ld;
  int64_t dst = r;
  if (row_map) {
    dst = row_map[r];
    if (dst < 0) return;
  }
  T* out = dlogits + dst * ld_out;
  const int tid = threadIdx.x;
  const int64_t nchunks = (vocab + 7) >> 3;
  if (g == 0.f || label == ignore_index) {
    const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int64_t c = tid; c < nchunks; c += kLossThreads) store8<T, VEC>(out, c << 3, vocab, z);
    return;
  }
  const float l2 = lse[r] * kLog2e;
  for (int64_t c = tid; c < nchunks; c += kLossThreads) {
    const int64_t base = c << 3;
    float x[8], d[8];
    load8<T, VEC>(row, base, vocab, x);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = fast_exp2(fmaf(x[i], kLog2e, -l2));
      d[i] = g * (p - ((base + i == label) ? 1.f : 0.f));
    }
    store8<T, VEC>(out, base, vocab, d);
  }
}

// loss[r] = lse[r] - x[r, label[r]] for rows whose log-sum-exp is already known (the statistics
// epilogue of the head product, spx_gemm_bf16_nt_stats): one element of the row is read instead of
// the row.  Ignored rows: loss 0; a label outside [0, vocab) that is not the ignore index: NaN,
// as in label_ce_fwd_kernel.
template <typename T>
__global__ __launch_bounds__(256) void label_ce_pick_kernel(const T* __restrict__ logits, int64_t ld,
                                                            const int64_t* __restrict__ labels, int64_t rows,
                                                            int64_t vocab, int64_t ignore_index,
                                                            const float* __restrict__ lse,
                                                            float* __restrict__ loss) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  const int64_t label = labels[r];
  float l = 0.f;
  if (label != ignore_index)
    l = (label >= 0 && label < vocab) ? lse[r] - load1(logits + r * ld + label) : __builtin_nanf("");
  loss[r] = l;
}

}  // namespace spx

using namespace spx;

static int label_ce_checks(const char* fn, const void* logits, int64_t ld, const void* labels,
                           int64_t rows, int64_t vocab, int dtype) {
  if (!(rows > 0 && rows < (1ll << 31))) return fail_arg(fn, "rows out of range");
  if (!(vocab > 0 && vocab < (1ll << 31))) return fail_arg(fn, "vocab out of range");
  if (!(logits && labels)) return fail_arg(fn, "null buffer");
  if (ld < vocab) return fail_arg(fn, "leading dimension smaller than vocab");
  if (!(dtype == SPX_DTYPE_BF16 || dtype == SPX_DTYPE_F32)) return fail_arg(fn, "dtype must be bf16 or fp32");
  return SPX_OK;
}

extern "C" int spx_label_ce_fwd(const void* logits, int64_t ld_logits, const int64_t* labels,
                                int64_t rows, int64_t vocab, int dtype, int64_t ignore_index,
                                float* loss, float* lse, int32_t* argmax, void* stream) {
  if (int rc = label_ce_checks(__func__, logits, ld_logits, labels, rows, vocab, dtype)) return rc;
  SPX_REQUIRE(loss && lse, "null output");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int esz = dtype == SPX_DTYPE_BF16 ? 2 : 4;
  const bool vec = ptr_aligned16(logits) && (ld_logits * esz) % 16 == 0;
  const dim3 grid((unsigned)rows), block(kLossThreads);
#define SPX_LAUNCH(T, V)                                                                       \
  hipLaunchKernelGGL((label_ce_fwd_kernel<T, V>), grid, block, 0, st,                          \
                     reinterpret_cast<const T*>(logits), ld_logits, labels, vocab, ignore_index, \
                     loss, lse, argmax)
  if (dtype == SPX_DTYPE_BF16) { if (vec) SPX_LAUNCH(uint16_t, true); else SPX_LAUNCH(uint16_t, false); }
  else { if (vec) SPX_LAUNCH(float, true); else SPX_LAUNCH(float, false); }
#undef SPX_LAUNCH
  return check_launch(__func__);
}

extern "C" int spx_label_ce_from_lse(const void* logits, int64_t ld_logits, const int64_t* labels,
                                     int64_t rows, int64_t vocab, int dtype, int64_t ignore_index,
                                     const float* lse, float* loss, void* stream) {
  if (int rc = label_ce_checks(__func__, logits, ld_logits, labels, rows, vocab, dtype)) return rc;
  SPX_REQUIRE(loss && lse, "null buffer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((rows + 255) / 256)), block(256);
  if (dtype == SPX_DTYPE_BF16)
    hipLaunchKernelGGL(label_ce_pick_kernel<uint16_t>, grid, block, 0, st,
                       reinterpret_cast<const uint16_t*>(logits), ld_logits, labels, rows, vocab, ignore_index,
                       lse, loss);
  else
    hipLaunchKernelGGL(label_ce_pick_kernel<float>, grid, block, 0, st, reinterpret_cast<const float*>(logits),
                       ld_logits, labels, rows, vocab, ignore_index, lse, loss);
  return check_launch(__func__);
}

static int label_ce_bwd_impl(const char* fn, const void* logits, int64_t ld_logits, const int64_t* labels,
                             const float* lse, const float* grad_rows, int64_t rows, int64_t vocab,
                             int dtype, int64_t ignore_index, void* dlogits, int64_t ld_out,
                             const int32_t* row_map, void* stream) {
  if (int rc = label_ce_checks(fn, logits, ld_logits, labels, rows, vocab, dtype)) return rc;
  if (!(lse && grad_rows && dlogits)) return fail_arg(fn, "null buffer");
  if (ld_out < vocab) return fail_arg(fn, "leading dimension of the gradient smaller than vocab");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int esz = dtype == SPX_DTYPE_BF16 ? 2 : 4;
  const bool vec = ptr_aligned16(logits) && ptr_aligned16(dlogits) && (ld_logits * esz) % 16 == 0 &&
                   (ld_out * esz) % 16 == 0;
  const dim3 grid((unsigned)rows), block(kLossThreads);
#define SPX_LAUNCH(T, V)                                                                       \
  hipLaunchKernelGGL((label_ce_bwd_kernel<T, V>), grid, block, 0, st,                          \
                     reinterpret_cast<const T*>(logits), ld_logits, labels, lse, grad_rows, vocab, \
                     ignore_index, reinterpret_cast<T*>(dlogits), ld_out, row_map)
  if (dtype == SPX_DTYPE_BF16) { if (vec) SPX_LAUNCH(uint16_t, true); else SPX_LAUNCH(uint16_t, false); }
  else { if (vec) SPX_LAUNCH(float, true); else SPX_LAUNCH(float, false); }
#undef SPX_LAUNCH
  return check_launch(fn);
}

extern "C" int spx_label_ce_bwd(const void* logits, int64_t ld_logits, const int64_t* labels,
                                const float* lse, const float* grad_rows, int64_t rows,
                                int64_t vocab, int dtype, int64_t ignore_index, void* dlogits,
                                int64_t ld_out, void* stream) {
  return label_ce_bwd_impl(__func__, logits, ld_logits, labels, lse, grad_rows, rows, vocab, dtype,
                           ignore_index, dlogits, ld_out, nullptr, stream);
}

extern "C" int spx_label_ce_bwd_packed(const void* logits, int64_t ld_logits, const int64_t* labels,
                                       const float* lse, const float* grad_rows, int64_t rows,
                                       int64_t vocab, int dtype, int64_t ignore_index,
                                       const int32_t* row_map, void* dlogits, int64_t ld_out,
                                       void* stream) {
  if (!row_map) return fail_arg(__func__, "null row map");
  return label_ce_bwd_impl(__func__, logits, ld_logits, labels, lse, grad_rows, rows, vocab, dtype,
                           ignore_index, dlogits, ld_out, row_map, stream);
}
