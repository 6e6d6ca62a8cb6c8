// Packs per-sample verifier hidden states into the one-row training batch of the
// draft models, on the device (gfx950).  The samples arrive back to back exactly as the
// hidden-state files hold them, `[rows, layers + 1, hidden]` plus token ids and loss mask;
// one launch writes the whole batch: the auxiliary layers flattened to
// `[max_len, layers * hidden]`, the last layer `[max_len, hidden]`, token ids, loss
// mask, position ids and document ids, cast to bf16, truncated at `max_len`, zero
// padded, with the one-token alignment shift of the EAGLE3 layout folded into the row
// indices.  Pure HBM-bound copy work: every source element is read once with 16-byte
// loads and every output element written once.
//
// One workgroup per output row.  Row r belongs to document d = the last d with
// out_start[d] <= r; its offset o = r - out_start[d] picks source row
// src_start[d] + o for the auxiliary layers and src_start[d] + o + shift for everything
// else.

#include "loss_common.h"
#include "../../include/spx.h"

namespace spx {

struct PackArgs {
  const void* src_hs;
  const int64_t* src_ids;
  const unsigned char* src_mask;
  const int64_t* src_pos;
  const int64_t* src_start;
  const int64_t* out_start;
  void* out_aux;
  void* out_last;
  int64_t* out_ids;
  unsigned char* out_mask;
  int64_t* out_pos;
  int64_t* out_doc;
  int64_t n_src_rows, layers, hidden, n_docs, shift;
  int mask_elem;
};

// fp32 -> bf16 as PyTorch casts: round to nearest even; a NaN becomes the quiet NaN 0x7fc0
__device__ __forceinline__ uint32_t cast_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

template <typename S>
__device__ __forceinline__ void copy8(const S* src, uint16_t* dst);
template <>
__device__ __forceinline__ void copy8<uint16_t>(const uint16_t* src, uint16_t* dst) {
  st16(dst, ld16(src));
}
template <>
__device__ __forceinline__ void copy8<float>(const float* src, uint16_t* dst) {
  float v[8];
  load8_vec<float>(src, v);
  u32x4 raw;
  raw.x = cast_bf16(v[0]) | (cast_bf16(v[1]) << 16);
  raw.y = cast_bf16(v[2]) | (cast_bf16(v[3]) << 16);
  raw.z = cast_bf16(v[4]) | (cast_bf16(v[5]) << 16);
  raw.w = cast_bf16(v[6]) | (cast_bf16(v[7]) << 16);
  st16(dst, raw);
}

__device__ __forceinline__ uint16_t cast1(uint16_t v) { return v; }
__device__ __forceinline__ uint16_t cast1(float v) { return (uint16_t)cast_bf16(v); }

// dst[0:n] = bf16(src[0:n]) (src == nullptr: zeros)
template <typename S, bool VEC>
__device__ __forceinline__ void copy_span(const S* src, uint16_t* dst, int64_t n, int tid) {
  if (src == nullptr) {
    if (VEC) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int64_t c = tid; c < (n >> 3); c += kLossThreads) st16(dst + (c << 3), z);
    } else {
      for (int64_t i = tid; i < n; i += kLossThreads) dst[i] = 0;
    }
    return;
  }
  if (VEC) {
    for (int64_t c = tid; c < (n >> 3); c += kLossThreads) copy8<S>(src + (c << 3), dst + (c << 3));
  } else {
    for (int64_t i = tid; i < n; i += kLossThreads) dst[i] = cast1(src[i]);
  }
}

template <typename S, bool VEC>
__global__ __launch_bounds__(kLossThreads) void pack_batch_kernel(PackArgs a) {
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  // number of documents that start at or before row r (out_start is non-decreasing and
  // out_start[0] == 0): uniform over the workgroup
  int64_t lo = 0, hi = a.n_docs;  // invariant: out_start[lo] <= r, answer in [lo, hi)
  const bool pad = r >= a.out_start[a.n_docs];
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (a.out_start[mid] <= r) lo = mid; else hi = mid;
  }
  const int64_t d = lo;
  const int64_t o = r - a.out_start[d];
  const int64_t s_aux = a.src_start[d] + o;
  const int64_t s_tok = s_aux + a.shift;
  // a row outside the staged samples is never dereferenced: it is written as padding
  const bool live = !pad && s_aux >= 0 && s_tok < a.n_src_rows;
  const int64_t h = a.hidden, lh = a.layers * a.hidden, ld = lh + h;
  const S* src = reinterpret_cast<const S*>(a.src_hs);
  if (a.out_aux)
    copy_span<S, VEC>(live ? src + s_aux * ld : nullptr,
                      reinterpret_cast<uint16_t*>(a.out_aux) + r * lh, lh, tid);
  if (a.out_last)
    copy_span<S, VEC>(live ? src + s_tok * ld + lh : nullptr,
                      reinterpret_cast<uint16_t*>(a.out_last) + r * h, h, tid);
  if (tid == 0) {
    a.out_ids[r] = live ? a.src_ids[s_tok] : 0;
    a.out_pos[r] = live ? (a.src_pos ? a.src_pos[s_tok] : o + a.shift) : 0;
    a.out_doc[r] = live ? d : -1;
  }
  if (tid < a.mask_elem)
    a.out_mask[r * a.mask_elem + tid] = live ? a.src_mask[s_tok * a.mask_elem + tid] : 0;
}

}  // namespace spx

using namespace spx;

extern "C" int spx_pack_batch(const void* src_hs, int src_dtype, int64_t n_src_rows, int64_t layers,
                              int64_t hidden, const int64_t* src_ids, const void* src_mask,
                              int mask_elem, const int64_t* src_pos, const int64_t* src_start,
                              const int64_t* out_start, int64_t n_docs, int64_t max_len,
                              int shift, void* out_aux, void* out_last, int64_t* out_ids,
                              void* out_mask, int64_t* out_pos, int64_t* out_doc, void* stream) {
  SPX_REQUIRE(max_len > 0 && max_len < (1ll << 31), "max_len out of range");
  SPX_REQUIRE(n_docs >= 1, "at least one document (it may be empty)");
  SPX_REQUIRE(n_src_rows >= 0 && layers >= 0 && hidden > 0, "bad source shape");
  SPX_REQUIRE(shift == 0 || shift == 1, "shift must be 0 or 1");
  SPX_REQUIRE(mask_elem == 1 || mask_elem == 2 || mask_elem == 4 || mask_elem == 8,
              "loss mask element size must be 1, 2, 4 or 8 bytes");
  SPX_REQUIRE(src_dtype == SPX_DTYPE_BF16 || src_dtype == SPX_DTYPE_F32, "source dtype must be bf16 or fp32");
  SPX_REQUIRE(src_start && out_start && out_ids && out_mask && out_pos && out_doc, "null buffer");
  SPX_REQUIRE(n_src_rows == 0 || (src_hs && src_ids && src_mask), "null source");
  SPX_REQUIRE(out_aux || out_last, "no hidden-state output requested");
  SPX_REQUIRE(!(out_aux && layers == 0), "auxiliary output requested from a source without auxiliary layers");
  PackArgs a;
  a.src_hs = src_hs; a.src_ids = src_ids; a.src_mask = static_cast<const unsigned char*>(src_mask);
  a.src_pos = src_pos; a.src_start = src_start; a.out_start = out_start;
  a.out_aux = out_aux; a.out_last = out_last; a.out_ids = out_ids;
  a.out_mask = static_cast<unsigned char*>(out_mask); a.out_pos = out_pos; a.out_doc = out_doc;
  a.n_src_rows = n_src_rows; a.layers = layers; a.hidden = hidden; a.n_docs = n_docs; a.shift = shift;
  a.mask_elem = mask_elem;
  const bool vec = hidden % 8 == 0 && ptr_aligned16(src_hs) && (!out_aux || ptr_aligned16(out_aux)) &&
                   (!out_last || ptr_aligned16(out_last));
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)max_len), block(kLossThreads);
#define SPX_LAUNCH(S, V) hipLaunchKernelGGL((pack_batch_kernel<S, V>), grid, block, 0, st, a)
  if (src_dtype == SPX_DTYPE_BF16) { if (vec) SPX_LAUNCH(uint16_t, true); else SPX_LAUNCH(uint16_t, false); }
  else { if (vec) SPX_LAUNCH(float, true); else SPX_LAUNCH(float, false); }
#undef SPX_LAUNCH
  return check_launch(__func__);
}
