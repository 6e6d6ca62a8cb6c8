// HBM-bound glue of the draft decoder layer for gfx950: RMSNorm, rotary
// embedding fused with the [T, heads*D] -> [heads, T, D] relayout, and the
// SwiGLU gate.  bf16 in / out, fp32 inside, 16-byte accesses.  Rounding points
// follow the HF blocks the reference is built from (LlamaRMSNorm,
// apply_rotary_pos_emb, LlamaMLP): every bf16 tensor op of the eager path is
// one rounding here.

#include "spx_common.h"
#include "../../include/spx.h"

namespace spx {

__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

__device__ __forceinline__ void unpack8f(u32x4 raw, float v[8]) {
  v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x);
  v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
  v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z);
  v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
}
__device__ __forceinline__ u32x4 pack8f(const float v[8]) {
  u32x4 r;
  r.x = pack_bf16x2(v[0], v[1]); r.y = pack_bf16x2(v[2], v[3]);
  r.z = pack_bf16x2(v[4], v[5]); r.w = pack_bf16x2(v[6], v[7]);
  return r;
}

__device__ __forceinline__ float block_sum_256(float v, float* lds) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  return lds[0] + lds[1] + lds[2] + lds[3];
}

// ---------------------------------------------------------------- RMSNorm
// y = w * bf16(x * rsqrt(mean(x^2) + eps));  one workgroup per row (H >= 512) or one
// wave per row (small H, e.g. per-head q/k norm).  MAXC = 16-byte chunks a lane keeps.
// RES: x is the sum of two tensors, x = bf16(x + res) (one rounding, as a bf16 tensor add),
// which is also written to `sum` for the residual stream.
template <int MAXC, bool WAVE_ROWS, bool RES = false>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(
    const uint16_t* __restrict__ x, int64_t ld_x, const uint16_t* __restrict__ w,
    uint16_t* __restrict__ y, int64_t ld_y, float* __restrict__ rstd, int64_t rows, int H,
    float eps, const uint16_t* __restrict__ res = nullptr, int64_t ld_res = 0,
    uint16_t* __restrict__ sum = nullptr, int64_t ld_sum = 0) {
  __shared__ float red[4];
  const int nthr = WAVE_ROWS ? 64 : 256;
  const int t = WAVE_ROWS ? (threadIdx.x & 63) : threadIdx.x;
  const int64_t row = WAVE_ROWS ? (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  if (WAVE_ROWS && row >= rows) return;
  const int nch = H / 8;
  float v[MAXC][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = t + c * nthr;
    if (ch < nch) {
      unpack8f(*reinterpret_cast<const u32x4*>(x + row * ld_x + ch * 8), v[c]);
      if (RES) {
        float b[8];
        unpack8f(*reinterpret_cast<const u32x4*>(res + row * ld_res + ch * 8), b);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] += b[e];
        const u32x4 packed = pack8f(v[c]);
        *reinterpret_cast<u32x4*>(sum + row * ld_sum + ch * 8) = packed;
        unpack8f(packed, v[c]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(v[c][e], v[c][e], ss);
    }
  }
  ss = WAVE_ROWS ? wave_sum(ss) : block_sum_256(ss, red);
  const float r = rsqrtf(ss / (float)H + eps);
  if (t == 0 && rstd) rstd[row] = r;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = t + c * nthr;
    if (ch < nch) {
      float wv[8], o[8];
      unpack8f(*reinterpret_cast<const u32x4*>(w + ch * 8), wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = wv[e] * round_bf16(v[c][e] * r);
      *reinterpret_cast<u32x4*>(y + row * ld_y + ch * 8) = pack8f(o);
    }
  }
}

// dx = rstd * (g - xhat * mean(g * xhat)), g = dy * w, xhat = x * rstd;
// dw partial sums: block b accumulates the rows b, b + gridDim.x, ... per column.
// dres (may be null): gradient that reaches x along the residual stream, added before the
// one rounding of dx.  dx may be null (only dw wanted).  accumulate: the partial sums start from
// what dw_part holds (a gain that is applied several times per forward: one buffer, one final sum).
template <int MAXC, bool WAVE_ROWS>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(
    const uint16_t* __restrict__ x, int64_t ld_x, const uint16_t* __restrict__ w,
    const uint16_t* __restrict__ dy, int64_t ld_dy, const float* __restrict__ rstd,
    uint16_t* __restrict__ dx, int64_t ld_dx, float* __restrict__ dw_part, int64_t rows, int H,
    const uint16_t* __restrict__ dres = nullptr, int64_t ld_dres = 0, int accumulate = 0) {
  __shared__ float red[4];
  const int nthr = WAVE_ROWS ? 64 : 256;
  const int t = WAVE_ROWS ? (threadIdx.x & 63) : threadIdx.x;
  const int wave = threadIdx.x >> 6;
  const int nch = H / 8;
  float wv[MAXC][8], dwacc[MAXC][8];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = t + c * nthr;
    if (ch < nch) unpack8f(*reinterpret_cast<const u32x4*>(w + ch * 8), wv[c]);
#pragma unroll
    for (int e = 0; e < 8; ++e) dwacc[c][e] = 0.f;
    if (accumulate && dw_part && ch < nch) {
      const int64_t slot0 = WAVE_ROWS ? (int64_t)blockIdx.x * 4 + wave : blockIdx.x;
      const float* o = dw_part + slot0 * H + ch * 8;
      const f32x4 a = *reinterpret_cast<const f32x4*>(o), b = *reinterpret_cast<const f32x4*>(o + 4);
      dwacc[c][0] = a.x; dwacc[c][1] = a.y; dwacc[c][2] = a.z; dwacc[c][3] = a.w;
      dwacc[c][4] = b.x; dwacc[c][5] = b.y; dwacc[c][6] = b.z; dwacc[c][7] = b.w;
    }
  }
  const int64_t first = WAVE_ROWS ? (int64_t)blockIdx.x * 4 + wave : blockIdx.x;
  const int64_t stride = WAVE_ROWS ? (int64_t)gridDim.x * 4 : gridDim.x;
  for (int64_t row = first; row < rows; row += stride) {
    const float r = rstd[row];
    float xh[MAXC][8], g[MAXC][8];
    float dot = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int ch = t + c * nthr;
      if (ch < nch) {
        float xv[8], dv[8];
        unpack8f(*reinterpret_cast<const u32x4*>(x + row * ld_x + ch * 8), xv);
        unpack8f(*reinterpret_cast<const u32x4*>(dy + row * ld_dy + ch * 8), dv);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xh[c][e] = xv[e] * r;
          g[c][e] = dv[e] * wv[c][e];
          dot = fmaf(g[c][e], xh[c][e], dot);
          dwacc[c][e] = fmaf(dv[e], xh[c][e], dwacc[c][e]);
        }
      }
    }
    if (dx == nullptr) continue;  // uniform: only the weight gradient is wanted
    dot = WAVE_ROWS ? wave_sum(dot) : block_sum_256(dot, red);
    const float mean = dot / (float)H;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int ch = t + c * nthr;
      if (ch < nch) {
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = r * (g[c][e] - xh[c][e] * mean);
        if (dres) {
          float dr[8];
          unpack8f(*reinterpret_cast<const u32x4*>(dres + row * ld_dres + ch * 8), dr);
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] += dr[e];
        }
        *reinterpret_cast<u32x4*>(dx + row * ld_dx + ch * 8) = pack8f(o);
      }
    }
  }
  if (dw_part) {
    const int64_t slot = WAVE_ROWS ? (int64_t)blockIdx.x * 4 + wave : blockIdx.x;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int ch = t + c * nthr;
      if (ch < nch) {
        float* o = dw_part + slot * H + ch * 8;
        f32x4 a = {dwacc[c][0], dwacc[c][1], dwacc[c][2], dwacc[c][3]};
        f32x4 b = {dwacc[c][4], dwacc[c][5], dwacc[c][6], dwacc[c][7]};
        *reinterpret_cast<f32x4*>(o) = a;
        *reinterpret_cast<f32x4*>(o + 4) = b;
      }
    }
  }
}

// dw[c] = sum_s dw_part[s, c]  (fixed order: deterministic), bf16 out.  One workgroup
// sums 32 columns (one 128-byte line per slot row): lane = (slot row j of 32, 4 columns),
// thread j adds the slots j, j + 32, ..., then the 32 partial sums are combined through LDS
// in a fixed order.
__global__ __launch_bounds__(256) void colsum_kernel(const float* __restrict__ part, int64_t slots,
                                                     int H, uint16_t* __restrict__ out) {
  __shared__ float red[32][33];
  const int q = threadIdx.x & 7, j = threadIdx.x >> 3;
  const int c = blockIdx.x * 32 + q * 4;
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  if (c < H)
    for (int64_t i = j; i < slots; i += 32) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(part + i * H + c);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
  red[j][q * 4 + 0] = s.x; red[j][q * 4 + 1] = s.y; red[j][q * 4 + 2] = s.z; red[j][q * 4 + 3] = s.w;
  __syncthreads();
  if (threadIdx.x < 32 && blockIdx.x * 32 + threadIdx.x < H) {
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 32; ++k) t += red[k][threadIdx.x];
    out[blockIdx.x * 32 + threadIdx.x] = (uint16_t)f32_to_bf16_bits(t);
  }
}

// ---------------------------------------------------------------- RoPE + relayout
// forward:  out[h, t, :] = rope(x[t, h, :], pos[t])      x: [T, heads*D] (row stride ld_x)
// inverse:  out[t, h, :] = rope^T(x[h, t, :], pos[t])    (the backward of the above)
// rotate == 0: relayout only (used for V).  cos / sin are evaluated in fp32 from
// pos * inv_freq and rounded to bf16, as the HF rotary module does.
template <bool INVERSE>
__global__ __launch_bounds__(256) void rope_kernel(const uint16_t* __restrict__ x, int64_t ld_x,
                                                   const int64_t* __restrict__ pos,
                                                   const float* __restrict__ inv_freq,
                                                   uint16_t* __restrict__ out, int64_t ld_out, int T,
                                                   int heads, int D, int rotate, int64_t pos_offset,
                                                   int tok_head_stride, int rot, float table_scale) {
  // one thread: 8 consecutive d of the first half of the rotated part and the matching 8 of its
  // second half, or 16 consecutive d of the part that passes unrotated (rot < D: partial rotary)
  const int per_row = D / 16;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)T * heads * per_row;
  if (item >= total) return;
  const int d0 = (int)(item % per_row) * 8;
  const int h = (int)((item / per_row) % heads);
  const int t = (int)(item / ((int64_t)per_row * heads));
  const bool pass = d0 * 2 >= rot;  // items past the rotated part copy 16 contiguous elements
  const int half = pass ? 8 : rot / 2;
  const int dA = pass ? d0 * 2 : d0;
  // the head-major side is [heads][T][D] with a head stride of its own (0 = T * D, contiguous):
  // it may be a window of a longer key / value cache
  const int64_t hs = INVERSE ? (ld_x ? ld_x : (int64_t)T * D) : (ld_out ? ld_out : (int64_t)T * D);
  const uint16_t* src = INVERSE ? x + (int64_t)h * hs + (int64_t)t * D : x + (int64_t)t * ld_x + h * tok_head_stride;
  uint16_t* dst = INVERSE ? out + (int64_t)t * ld_out + h * tok_head_stride : out + (int64_t)h * hs + (int64_t)t * D;
  float a[8], b[8], oa[8], ob[8];
  unpack8f(*reinterpret_cast<const u32x4*>(src + dA), a);
  unpack8f(*reinterpret_cast<const u32x4*>(src + half + dA), b);
  if (rotate && !pass) {
    const float p = (float)(pos[t] + pos_offset);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float ang = p * inv_freq[d0 + e];
      // (table_scale: the attention factor some frequency scalings put on both tables, 1 otherwise)
      const float c = round_bf16(cosf(ang) * table_scale);
      float s = round_bf16(sinf(ang) * table_scale);
      if (INVERSE) s = -s;
      // x*cos + rotate_half(x)*sin with each bf16 op rounded
      oa[e] = round_bf16(a[e] * c) + round_bf16(-b[e] * s);
      ob[e] = round_bf16(b[e] * c) + round_bf16(a[e] * s);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) { oa[e] = a[e]; ob[e] = b[e]; }
  }
  *reinterpret_cast<u32x4*>(dst + dA) = pack8f(oa);
  *reinterpret_cast<u32x4*>(dst + half + dA) = pack8f(ob);
}

// out[b][c][r] = in[b][r][c] for a stack of bf16 matrices (the per-expert transposes the input
// gradient products of a stack of expert weights need).  One wave = one 64 x 64 tile, one lane =
// one 8 x 8 block transposed in registers: every load and store instruction moves whole 128-byte
// row segments (8 lanes x 16 bytes) and no LDS is involved.
__global__ __launch_bounds__(256) void transpose_stack_kernel(const uint16_t* __restrict__ in, int64_t ld_in,
                                                              int64_t bs_in, uint16_t* __restrict__ out,
                                                              int64_t ld_out, int64_t bs_out, int R, int C,
                                                              int tiles_r, int tiles_c, int64_t n_tiles) {
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= n_tiles) return;
  const int lane = threadIdx.x & 63;
  const int tc = (int)(tile % tiles_c);
  const int tr = (int)((tile / tiles_c) % tiles_r);
  const int64_t b = tile / ((int64_t)tiles_c * tiles_r);
  const int r0 = tr * 64 + (lane >> 3) * 8, c0 = tc * 64 + (lane & 7) * 8;
  if (r0 >= R || c0 >= C) return;  // R and C are multiples of 8: a block is inside or outside
  const uint16_t* src = in + b * bs_in + (int64_t)r0 * ld_in + c0;
  uint16_t* dst = out + b * bs_out + (int64_t)c0 * ld_out + r0;
  u32x4 v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)i * ld_in);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t o[4];
#pragma unroll
    for (int ip = 0; ip < 4; ++ip) {
      const uint32_t a = v[2 * ip][j >> 1], c = v[2 * ip + 1][j >> 1];
      o[ip] = (j & 1) ? ((a >> 16) | (c & 0xffff0000u)) : ((a & 0xffffu) | (c << 16));
    }
    u32x4 w;
    w.x = o[0]; w.y = o[1]; w.z = o[2]; w.w = o[3];
    *reinterpret_cast<u32x4*>(dst + (int64_t)j * ld_out) = w;
  }
}

// Output gate of the gated attention (Qwen3-Next): y = bf16(o * bf16(sigmoid(gate))), every tensor
// [rows, heads, D] with a row stride and a head stride of its own (the gate is the second half of
// every head's 2 D columns of the widened q projection).  One thread: 8 consecutive elements.
__global__ __launch_bounds__(256) void sigmoid_gate_fwd_kernel(
    const uint16_t* __restrict__ o, int64_t ld_o, const uint16_t* __restrict__ gate, int64_t ld_g, int hs_g,
    uint16_t* __restrict__ y, int64_t ld_y, int64_t rows, int heads, int D) {
  const int per_head = D / 8;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= rows * heads * per_head) return;
  const int d0 = (int)(item % per_head) * 8;
  const int h = (int)((item / per_head) % heads);
  const int64_t r = item / ((int64_t)per_head * heads);
  float a[8], g[8], out[8];
  unpack8f(*reinterpret_cast<const u32x4*>(o + r * ld_o + h * D + d0), a);
  unpack8f(*reinterpret_cast<const u32x4*>(gate + r * ld_g + (int64_t)h * hs_g + d0), g);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = a[e] * round_bf16(1.f / (1.f + __expf(-g[e])));
  *reinterpret_cast<u32x4*>(y + r * ld_y + h * D + d0) = pack8f(out);
}

// do = bf16(dy * sig), dgate = bf16(dy * o * sig * (1 - sig)), sig = sigmoid(gate) in fp32
__global__ __launch_bounds__(256) void sigmoid_gate_bwd_kernel(
    const uint16_t* __restrict__ o, int64_t ld_o, const uint16_t* __restrict__ gate, int64_t ld_g, int hs_g,
    const uint16_t* __restrict__ dy, int64_t ld_dy, uint16_t* __restrict__ d_o, int64_t ld_do,
    uint16_t* __restrict__ dgate, int64_t ld_dg, int hs_dg, int64_t rows, int heads, int D) {
  const int per_head = D / 8;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= rows * heads * per_head) return;
  const int d0 = (int)(item % per_head) * 8;
  const int h = (int)((item / per_head) % heads);
  const int64_t r = item / ((int64_t)per_head * heads);
  float a[8], g[8], d[8], oa[8], og[8];
  unpack8f(*reinterpret_cast<const u32x4*>(o + r * ld_o + h * D + d0), a);
  unpack8f(*reinterpret_cast<const u32x4*>(gate + r * ld_g + (int64_t)h * hs_g + d0), g);
  unpack8f(*reinterpret_cast<const u32x4*>(dy + r * ld_dy + h * D + d0), d);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float sg = 1.f / (1.f + __expf(-g[e]));
    oa[e] = d[e] * sg;
    og[e] = d[e] * a[e] * sg * (1.f - sg);
  }
  *reinterpret_cast<u32x4*>(d_o + r * ld_do + h * D + d0) = pack8f(oa);
  *reinterpret_cast<u32x4*>(dgate + r * ld_dg + (int64_t)h * hs_dg + d0) = pack8f(og);
}

// ---------------------------------------------------------------- SwiGLU
// rows x F elements per tensor, every tensor with its own row stride (so gate and up may be the
// two column halves of one merged projection output); chunk = 8 consecutive elements of a row
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const uint16_t* __restrict__ g, int64_t ld_g,
                                                         const uint16_t* __restrict__ u, int64_t ld_u,
                                                         uint16_t* __restrict__ out, int64_t ld_o,
                                                         int64_t rows, int64_t f8) {
  const int64_t n8 = rows * f8;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / f8, c = (i - r * f8) * 8;
    float gv[8], uv[8], o[8];
    unpack8f(*reinterpret_cast<const u32x4*>(g + r * ld_g + c), gv);
    unpack8f(*reinterpret_cast<const u32x4*>(u + r * ld_u + c), uv);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sg = 1.f / (1.f + __expf(-gv[e]));
      o[e] = round_bf16(gv[e] * sg) * uv[e];
    }
    *reinterpret_cast<u32x4*>(out + r * ld_o + c) = pack8f(o);
  }
}

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t* __restrict__ g, int64_t ld_g,
                                                         const uint16_t* __restrict__ u, int64_t ld_u,
                                                         const uint16_t* __restrict__ dout, int64_t ld_d,
                                                         uint16_t* __restrict__ dg, int64_t ld_dg,
                                                         uint16_t* __restrict__ du, int64_t ld_du,
                                                         int64_t rows, int64_t f8) {
  const int64_t n8 = rows * f8;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / f8, c = (i - r * f8) * 8;
    float gv[8], uv[8], dv[8], og[8], ou[8];
    unpack8f(*reinterpret_cast<const u32x4*>(g + r * ld_g + c), gv);
    unpack8f(*reinterpret_cast<const u32x4*>(u + r * ld_u + c), uv);
    unpack8f(*reinterpret_cast<const u32x4*>(dout + r * ld_d + c), dv);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sg = 1.f / (1.f + __expf(-gv[e]));
      const float act = gv[e] * sg;
      ou[e] = dv[e] * act;
      og[e] = dv[e] * uv[e] * (sg * (1.f + gv[e] * (1.f - sg)));
    }
    *reinterpret_cast<u32x4*>(dg + r * ld_dg + c) = pack8f(og);
    *reinterpret_cast<u32x4*>(du + r * ld_du + c) = pack8f(ou);
  }
}

static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- packed rows: map of the live rows, and back to one row per position
// row_map[r] = number of live rows before r if row r is live (row_grad[r] != 0 and, with labels,
// labels[r] != ignore_index), else -1; *count = number of live rows.  One workgroup, rows in order.
__global__ __launch_bounds__(1024) void pack_row_map_kernel(const float* __restrict__ row_grad,
                                                            const int64_t* __restrict__ labels,
                                                            int64_t ignore_index, int rows,
                                                            int32_t* __restrict__ row_map,
                                                            int32_t* __restrict__ count) {
  __shared__ int wave_tot[16];
  __shared__ int base_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) base_s = 0;
  __syncthreads();
  for (int r0 = 0; r0 < rows; r0 += 1024) {
    const int r = r0 + tid;
    const bool live = r < rows && row_grad[r] != 0.f && (!labels || labels[r] != ignore_index);
    const unsigned long long m = __ballot(live);
    const int before = __popcll(m & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[wave] = __popcll(m);
    __syncthreads();
    int off = base_s;
    for (int w = 0; w < wave; ++w) off += wave_tot[w];
    if (r < rows) row_map[r] = live ? off + before : -1;
    __syncthreads();
    if (tid == 0) {
      int t = 0;
      for (int w = 0; w < 16; ++w) t += wave_tot[w];
      base_s += t;
    }
    __syncthreads();
  }
  if (tid == 0) *count = base_s;
}

// out[r, :] = row_map[r] >= 0 ? packed[row_map[r], :] : 0 for r < rows, 0 for rows <= r < total_rows;
// with row_scale every live row is multiplied by row_scale[r] on its way (fp32, one rounding)
__global__ __launch_bounds__(256) void unpack_rows_kernel(const uint16_t* __restrict__ packed, int64_t ld,
                                                          const int32_t* __restrict__ row_map, int rows,
                                                          int cols8, uint16_t* __restrict__ out,
                                                          int64_t ld_out,
                                                          const float* __restrict__ row_scale = nullptr) {
  const int r = blockIdx.x;
  const int src = r < rows ? row_map[r] : -1;
  u32x4* o = reinterpret_cast<u32x4*>(out + (int64_t)r * ld_out);
  if (src < 0) {
    const u32x4 z = {0, 0, 0, 0};
    for (int c = threadIdx.x; c < cols8; c += 256) o[c] = z;
    return;
  }
  const u32x4* in = reinterpret_cast<const u32x4*>(packed + (int64_t)src * ld);
  if (!row_scale) {
    for (int c = threadIdx.x; c < cols8; c += 256) o[c] = in[c];
    return;
  }
  const float f = row_scale[r];
  for (int c = threadIdx.x; c < cols8; c += 256) {
    const u32x4 v = in[c];
    u32x4 w;
    w.x = pack_bf16x2(bf16_lo(v.x) * f, bf16_hi(v.x) * f);
    w.y = pack_bf16x2(bf16_lo(v.y) * f, bf16_hi(v.y) * f);
    w.z = pack_bf16x2(bf16_lo(v.z) * f, bf16_hi(v.z) * f);
    w.w = pack_bf16x2(bf16_lo(v.w) * f, bf16_hi(v.w) * f);
    o[c] = w;
  }
}

}  // namespace spx

using namespace spx;

extern "C" int spx_pack_row_map(const float* row_grad, const int64_t* labels, int64_t ignore_index,
                                int64_t rows, int32_t* row_map, int32_t* count, void* stream) {
  SPX_REQUIRE(rows > 0 && rows < (1ll << 31), "rows out of range");
  SPX_REQUIRE(row_grad && row_map && count, "null buffer");
  hipLaunchKernelGGL(pack_row_map_kernel, dim3(1), dim3(1024), 0, reinterpret_cast<hipStream_t>(stream), row_grad,
                     labels, ignore_index, (int)rows, row_map, count);
  return check_launch(__func__);
}

extern "C" int spx_unpack_rows(const void* packed, int64_t ld_packed, const int32_t* row_map, int64_t rows,
                               int64_t total_rows, int64_t cols, void* out, int64_t ld_out, void* stream) {
  SPX_REQUIRE(rows > 0 && total_rows >= rows && total_rows < (1ll << 31), "rows out of range");
  SPX_REQUIRE(cols > 0 && cols % 8 == 0 && ld_packed % 8 == 0 && ld_out % 8 == 0 && ld_packed >= cols && ld_out >= cols,
              "cols and the row strides must be multiples of 8 (bf16), strides at least cols");
  SPX_REQUIRE(packed && row_map && out, "null buffer");
  SPX_REQUIRE(al16(packed) && al16(out), "buffers must be 16-byte aligned");
  hipLaunchKernelGGL(unpack_rows_kernel, dim3((unsigned)total_rows), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(packed), ld_packed,
                     row_map, (int)rows, (int)(cols / 8), reinterpret_cast<uint16_t*>(out), ld_out);
  return check_launch(__func__);
}

extern "C" int spx_unpack_rows_scaled(const void* packed, int64_t ld_packed, const int32_t* row_map,
                                      const float* row_scale, int64_t rows, int64_t total_rows, int64_t cols,
                                      void* out, int64_t ld_out, void* stream) {
  SPX_REQUIRE(rows > 0 && total_rows >= rows && total_rows < (1ll << 31), "rows out of range");
  SPX_REQUIRE(cols > 0 && cols % 8 == 0 && ld_packed % 8 == 0 && ld_out % 8 == 0 && ld_packed >= cols && ld_out >= cols,
              "cols and the row strides must be multiples of 8 (bf16), strides at least cols");
  SPX_REQUIRE(packed && row_map && row_scale && out, "null buffer");
  SPX_REQUIRE(al16(packed) && al16(out), "buffers must be 16-byte aligned");
  hipLaunchKernelGGL(unpack_rows_kernel, dim3((unsigned)total_rows), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(packed), ld_packed,
                     row_map, (int)rows, (int)(cols / 8), reinterpret_cast<uint16_t*>(out), ld_out, row_scale);
  return check_launch(__func__);
}

extern "C" int64_t spx_rmsnorm_bwd_slots(int64_t rows, int64_t H) {
  if (H <= 512) return 4 * (rows < 8192 ? (rows + 3) / 4 : 2048);  // one wave per slot, 8 workgroups per CU
  return rows < 1024 ? rows : 1024;  // four workgroups per compute unit
}

static int rmsnorm_fwd_launch(const char* fn, const void* x, int64_t ld_x, const void* res, int64_t ld_res,
                              void* sum, int64_t ld_sum, const void* weight, void* y, int64_t ld_y,
                              float* rstd, int64_t rows, int64_t H, float eps, void* stream) {
  if (!(rows >= 0 && H > 0)) return fail_arg(fn, "bad sizes");
  if (!(H % 8 == 0 && ld_x % 8 == 0 && ld_y % 8 == 0 && ld_res % 8 == 0 && ld_sum % 8 == 0))
    return fail_arg(fn, "H and the row strides must be multiples of 8");
  if (H > 16384) return fail_arg(fn, "H must be at most 16384");
  if (rows >= (1ll << 31)) return fail_arg(fn, "too many rows");
  if (rows == 0) return SPX_OK;
  if (!(x && weight && y)) return fail_arg(fn, "null buffer");
  if (!(al16(x) && al16(weight) && al16(y) && al16(res) && al16(sum)))
    return fail_arg(fn, "buffers must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  auto xp = reinterpret_cast<const uint16_t*>(x);
  auto rp = reinterpret_cast<const uint16_t*>(res);
  auto sp = reinterpret_cast<uint16_t*>(sum);
  auto wp = reinterpret_cast<const uint16_t*>(weight);
  auto yp = reinterpret_cast<uint16_t*>(y);
#define SPX_LAUNCH(MAXC, WR, GRID)                                                                  \
  do {                                                                                              \
    if (res)                                                                                        \
      hipLaunchKernelGGL((rmsnorm_fwd_kernel<MAXC, WR, true>), dim3((unsigned)(GRID)), dim3(256), 0, st, \
                         xp, ld_x, wp, yp, ld_y, rstd, rows, (int)H, eps, rp, ld_res, sp, ld_sum);  \
    else                                                                                            \
      hipLaunchKernelGGL((rmsnorm_fwd_kernel<MAXC, WR, false>), dim3((unsigned)(GRID)), dim3(256), 0, st, \
                         xp, ld_x, wp, yp, ld_y, rstd, rows, (int)H, eps, nullptr, 0, nullptr, 0);  \
  } while (0)
  if (H <= 512) SPX_LAUNCH(1, true, (rows + 3) / 4);
  else if (H <= 4096) SPX_LAUNCH(2, false, rows);
  else SPX_LAUNCH(8, false, rows);
#undef SPX_LAUNCH
  return check_launch(fn);
}

extern "C" int spx_rmsnorm_fwd(const void* x, int64_t ld_x, const void* weight, void* y, int64_t ld_y,
                               float* rstd, int64_t rows, int64_t H, float eps, void* stream) {
  return rmsnorm_fwd_launch(__func__, x, ld_x, nullptr, 0, nullptr, 0, weight, y, ld_y, rstd, rows, H, eps,
                            stream);
}

extern "C" int spx_add_rmsnorm_fwd(const void* a, int64_t ld_a, const void* b, int64_t ld_b, void* sum,
                                   int64_t ld_sum, const void* weight, void* y, int64_t ld_y, float* rstd,
                                   int64_t rows, int64_t H, float eps, void* stream) {
  SPX_REQUIRE(rows == 0 || (b && sum), "null buffer");
  return rmsnorm_fwd_launch(__func__, a, ld_a, b, ld_b, sum, ld_sum, weight, y, ld_y, rstd, rows, H, eps,
                            stream);
}

static int rmsnorm_bwd_launch(const char* fn, const void* x, int64_t ld_x, const void* weight, const void* dy,
                              int64_t ld_dy, const void* dres, int64_t ld_dres, const float* rstd, void* dx,
                              int64_t ld_dx, void* dweight, float* dw_scratch, int64_t rows, int64_t H,
                              void* stream, bool partial_only = false, int accumulate = 0) {
  if (!(rows > 0 && H > 0)) return fail_arg(fn, "bad sizes");
  if (!(H % 8 == 0 && ld_x % 8 == 0 && ld_dy % 8 == 0 && ld_dx % 8 == 0 && ld_dres % 8 == 0))
    return fail_arg(fn, "H and the row strides must be multiples of 8");
  if (H > 16384) return fail_arg(fn, "H must be at most 16384");
  if (!(x && weight && dy && rstd)) return fail_arg(fn, "null buffer");
  if (!(dx || dweight || partial_only)) return fail_arg(fn, "neither dx nor dweight requested");
  if (partial_only && !dw_scratch) return fail_arg(fn, "null dw_scratch");
  if (dres && !dx) return fail_arg(fn, "a residual gradient needs dx");
  if (dweight && !dw_scratch)
    return fail_arg(fn, "dweight needs dw_scratch (spx_rmsnorm_bwd_slots(rows, H) * H floats)");
  if (!(al16(x) && al16(weight) && al16(dy) && al16(dx) && al16(dw_scratch) && al16(dres)))
    return fail_arg(fn, "buffers must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  auto xp = reinterpret_cast<const uint16_t*>(x);
  auto wp = reinterpret_cast<const uint16_t*>(weight);
  auto dyp = reinterpret_cast<const uint16_t*>(dy);
  auto drp = reinterpret_cast<const uint16_t*>(dres);
  auto dxp = reinterpret_cast<uint16_t*>(dx);
  float* part = (dweight || partial_only) ? dw_scratch : nullptr;
  const int64_t slots = spx_rmsnorm_bwd_slots(rows, H);
  if (H <= 512)
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<1, true>), dim3((unsigned)(slots / 4)), dim3(256), 0, st, xp, ld_x,
                       wp, dyp, ld_dy, rstd, dxp, ld_dx, part, rows, (int)H, drp, ld_dres, accumulate);
  else if (H <= 4096)
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<2, false>), dim3((unsigned)slots), dim3(256), 0, st, xp, ld_x, wp,
                       dyp, ld_dy, rstd, dxp, ld_dx, part, rows, (int)H, drp, ld_dres, accumulate);
  else
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<8, false>), dim3((unsigned)slots), dim3(256), 0, st, xp, ld_x, wp,
                       dyp, ld_dy, rstd, dxp, ld_dx, part, rows, (int)H, drp, ld_dres, accumulate);
  if (dweight)
    hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((H + 31) / 32)), dim3(256), 0, st, part, slots, (int)H,
                       reinterpret_cast<uint16_t*>(dweight));
  return check_launch(fn);
}

extern "C" int spx_rmsnorm_bwd(const void* x, int64_t ld_x, const void* weight, const void* dy,
                               int64_t ld_dy, const float* rstd, void* dx, int64_t ld_dx, void* dweight,
                               float* dw_scratch, int64_t rows, int64_t H, void* stream) {
  return rmsnorm_bwd_launch(__func__, x, ld_x, weight, dy, ld_dy, nullptr, 0, rstd, dx, ld_dx, dweight,
                            dw_scratch, rows, H, stream);
}

extern "C" int spx_add_rmsnorm_bwd(const void* x, int64_t ld_x, const void* weight, const void* dy,
                                   int64_t ld_dy, const void* dres, int64_t ld_dres, const float* rstd,
                                   void* dx, int64_t ld_dx, void* dweight, float* dw_scratch, int64_t rows,
                                   int64_t H, void* stream) {
  return rmsnorm_bwd_launch(__func__, x, ld_x, weight, dy, ld_dy, dres, ld_dres, rstd, dx, ld_dx, dweight,
                            dw_scratch, rows, H, stream);
}

extern "C" int spx_rmsnorm_bwd_partial(const void* x, int64_t ld_x, const void* weight, const void* dy,
                                       int64_t ld_dy, const void* dres, int64_t ld_dres, const float* rstd,
                                       void* dx, int64_t ld_dx, float* dw_scratch, int32_t accumulate,
                                       int64_t rows, int64_t H, void* stream) {
  return rmsnorm_bwd_launch(__func__, x, ld_x, weight, dy, ld_dy, dres, ld_dres, rstd, dx, ld_dx, nullptr,
                            dw_scratch, rows, H, stream, true, accumulate != 0);
}

extern "C" int spx_rmsnorm_dweight(const float* dw_scratch, int64_t slots, int64_t H, void* dweight,
                                   void* stream) {
  const char* fn = __func__;
  if (!(slots > 0 && H > 0 && H % 8 == 0 && H <= 16384)) return fail_arg(fn, "bad sizes");
  if (!(dw_scratch && dweight && al16(dw_scratch))) return fail_arg(fn, "null or unaligned buffer");
  hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((H + 31) / 32)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), dw_scratch, slots, (int)H,
                     reinterpret_cast<uint16_t*>(dweight));
  return check_launch(fn);
}

static int rope_relayout_impl(const char* fn, const void* x, int64_t ld_x, const int64_t* position_ids,
                              const float* inv_freq, void* out, int64_t ld_out, int64_t T, int32_t heads,
                              int32_t D, int32_t rotate, int32_t inverse, int64_t position_offset,
                              int32_t tok_head_stride, int32_t rot, float table_scale, void* stream);

extern "C" int spx_rope_relayout(const void* x, int64_t ld_x, const int64_t* position_ids,
                                 const float* inv_freq, void* out, int64_t ld_out, int64_t T,
                                 int32_t heads, int32_t D, int32_t rotate, int32_t inverse,
                                 int64_t position_offset, void* stream) {
  return rope_relayout_impl(__func__, x, ld_x, position_ids, inv_freq, out, ld_out, T, heads, D, rotate,
                            inverse, position_offset, D, D, 1.f, stream);
}

extern "C" int spx_rope_relayout_partial(const void* x, int64_t ld_x, int32_t x_head_stride,
                                         const int64_t* position_ids, const float* inv_freq, void* out,
                                         int64_t ld_out, int64_t T, int32_t heads, int32_t D,
                                         int32_t rotary_dim, int32_t rotate, int32_t inverse,
                                         int64_t position_offset, float table_scale, void* stream) {
  return rope_relayout_impl(__func__, x, ld_x, position_ids, inv_freq, out, ld_out, T, heads, D, rotate,
                            inverse, position_offset, x_head_stride, rotary_dim, table_scale, stream);
}

#define SPX_REQ_FN(cond, what) do { if (!(cond)) return spx::fail_arg(fn, what); } while (0)
extern "C" int spx_transpose_bf16(const void* in, int64_t ld_in, int64_t batch_stride_in, void* out,
                                  int64_t ld_out, int64_t batch_stride_out, int64_t R, int64_t C,
                                  int64_t batches, void* stream) {
  const char* fn = __func__;
  SPX_REQ_FN(R > 0 && C > 0 && batches > 0 && R % 8 == 0 && C % 8 == 0 && R < (1ll << 31) && C < (1ll << 31),
             "R and C must be positive multiples of 8");
  SPX_REQ_FN(in && out && in != out && al16(in) && al16(out), "null, aliased or unaligned buffer");
  SPX_REQ_FN(ld_in % 8 == 0 && ld_out % 8 == 0 && ld_in >= C && ld_out >= R, "row strides must be multiples of 8, ld_in >= C, ld_out >= R");
  SPX_REQ_FN(batch_stride_in % 8 == 0 && batch_stride_out % 8 == 0 && batch_stride_in >= 0 && batch_stride_out >= 0,
             "batch strides must be multiples of 8");
  const int tiles_r = (int)((R + 63) / 64), tiles_c = (int)((C + 63) / 64);
  const int64_t n_tiles = (int64_t)tiles_r * tiles_c * batches;
  SPX_REQ_FN((n_tiles + 3) / 4 < (1ll << 31), "too many tiles");
  hipLaunchKernelGGL(transpose_stack_kernel, dim3((unsigned)((n_tiles + 3) / 4)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(in), ld_in,
                     batch_stride_in, reinterpret_cast<uint16_t*>(out), ld_out, batch_stride_out, (int)R, (int)C,
                     tiles_r, tiles_c, n_tiles);
  return check_launch(fn);
}

extern "C" int spx_sigmoid_gate_fwd(const void* o, int64_t ld_o, const void* gate, int64_t ld_gate,
                                    int32_t gate_head_stride, void* y, int64_t ld_y, int64_t rows,
                                    int32_t heads, int32_t D, void* stream) {
  const char* fn = __func__;
  SPX_REQ_FN(rows > 0 && heads > 0 && D > 0 && D % 8 == 0, "rows, heads > 0 and D a positive multiple of 8");
  SPX_REQ_FN(o && gate && y && al16(o) && al16(gate) && al16(y), "null or unaligned buffer");
  const int64_t hd = (int64_t)heads * D;
  SPX_REQ_FN(ld_o % 8 == 0 && ld_y % 8 == 0 && ld_gate % 8 == 0 && gate_head_stride % 8 == 0, "strides must be multiples of 8");
  SPX_REQ_FN(ld_o >= hd && ld_y >= hd && gate_head_stride >= D && ld_gate >= (int64_t)(heads - 1) * gate_head_stride + D,
             "stride too small");
  const int64_t items = rows * heads * (D / 8);
  hipLaunchKernelGGL(sigmoid_gate_fwd_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(o), ld_o,
                     reinterpret_cast<const uint16_t*>(gate), ld_gate, (int)gate_head_stride,
                     reinterpret_cast<uint16_t*>(y), ld_y, rows, (int)heads, (int)D);
  return check_launch(fn);
}

extern "C" int spx_sigmoid_gate_bwd(const void* o, int64_t ld_o, const void* gate, int64_t ld_gate,
                                    int32_t gate_head_stride, const void* dy, int64_t ld_dy, void* d_o,
                                    int64_t ld_do, void* dgate, int64_t ld_dgate,
                                    int32_t dgate_head_stride, int64_t rows, int32_t heads, int32_t D,
                                    void* stream) {
  const char* fn = __func__;
  SPX_REQ_FN(rows > 0 && heads > 0 && D > 0 && D % 8 == 0, "rows, heads > 0 and D a positive multiple of 8");
  SPX_REQ_FN(o && gate && dy && d_o && dgate, "null buffer");
  SPX_REQ_FN(al16(o) && al16(gate) && al16(dy) && al16(d_o) && al16(dgate), "buffers must be 16-byte aligned");
  const int64_t hd = (int64_t)heads * D;
  SPX_REQ_FN(ld_o % 8 == 0 && ld_dy % 8 == 0 && ld_do % 8 == 0 && ld_gate % 8 == 0 && ld_dgate % 8 == 0 &&
                 gate_head_stride % 8 == 0 && dgate_head_stride % 8 == 0, "strides must be multiples of 8");
  SPX_REQ_FN(ld_o >= hd && ld_dy >= hd && ld_do >= hd && gate_head_stride >= D && dgate_head_stride >= D &&
                 ld_gate >= (int64_t)(heads - 1) * gate_head_stride + D &&
                 ld_dgate >= (int64_t)(heads - 1) * dgate_head_stride + D, "stride too small");
  const int64_t items = rows * heads * (D / 8);
  hipLaunchKernelGGL(sigmoid_gate_bwd_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(o), ld_o,
                     reinterpret_cast<const uint16_t*>(gate), ld_gate, (int)gate_head_stride,
                     reinterpret_cast<const uint16_t*>(dy), ld_dy, reinterpret_cast<uint16_t*>(d_o), ld_do,
                     reinterpret_cast<uint16_t*>(dgate), ld_dgate, (int)dgate_head_stride, rows, (int)heads, (int)D);
  return check_launch(fn);
}

static int rope_relayout_impl(const char* fn, const void* x, int64_t ld_x, const int64_t* position_ids,
                              const float* inv_freq, void* out, int64_t ld_out, int64_t T, int32_t heads,
                              int32_t D, int32_t rotate, int32_t inverse, int64_t position_offset,
                              int32_t tok_head_stride, int32_t rot, float table_scale, void* stream) {
  SPX_REQ_FN(table_scale > 0.f && table_scale < 1e4f, "the table scale must be positive and finite");
  SPX_REQ_FN(T > 0 && heads > 0 && D > 0 && D % 16 == 0, "T, heads > 0 and D a multiple of 16");
  SPX_REQ_FN(rot > 0 && rot <= D && rot % 16 == 0, "the rotary dimension must be a multiple of 16 in 16 .. D");
  SPX_REQ_FN(tok_head_stride >= D && tok_head_stride % 8 == 0, "bad head stride of the token-major side");
  SPX_REQ_FN(x && out && (!rotate || (position_ids && inv_freq)), "null buffer");
  SPX_REQ_FN(al16(x) && al16(out), "buffers must be 16-byte aligned");
  const int64_t tok_row = (int64_t)(heads - 1) * tok_head_stride + D;
  if (inverse) {
    SPX_REQ_FN(ld_out % 8 == 0 && ld_out >= tok_row, "bad output row stride");
    SPX_REQ_FN(ld_x == 0 || (ld_x % 8 == 0 && ld_x >= T * D), "bad head stride of the head-major input");
  } else {
    SPX_REQ_FN(ld_x % 8 == 0 && ld_x >= tok_row, "bad input row stride");
    SPX_REQ_FN(ld_out == 0 || (ld_out % 8 == 0 && ld_out >= T * D), "bad head stride of the head-major output");
  }
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t total = T * heads * (D / 16);
  const unsigned grid = (unsigned)((total + 255) / 256);
  auto xp = reinterpret_cast<const uint16_t*>(x);
  auto op = reinterpret_cast<uint16_t*>(out);
  if (inverse)
    hipLaunchKernelGGL(rope_kernel<true>, dim3(grid), dim3(256), 0, st, xp, ld_x, position_ids, inv_freq, op,
                       ld_out, (int)T, (int)heads, (int)D, (int)rotate, position_offset, (int)tok_head_stride, (int)rot,
                       table_scale);
  else
    hipLaunchKernelGGL(rope_kernel<false>, dim3(grid), dim3(256), 0, st, xp, ld_x, position_ids, inv_freq, op,
                       ld_out, (int)T, (int)heads, (int)D, (int)rotate, position_offset, (int)tok_head_stride, (int)rot,
                       table_scale);
  return check_launch(fn);
}
#undef SPX_REQ_FN

static unsigned swiglu_grid(int64_t n8) {
  return (unsigned)((n8 + 255) / 256 < 65536 ? (n8 + 255) / 256 : 65536);
}

extern "C" int spx_swiglu_rows_fwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                   void* out, int64_t ld_out, int64_t rows, int64_t F, void* stream) {
  SPX_REQUIRE(rows > 0 && F > 0 && F % 8 == 0, "rows > 0 and F a positive multiple of 8");
  SPX_REQUIRE(ld_gate >= F && ld_up >= F && ld_out >= F && ld_gate % 8 == 0 && ld_up % 8 == 0 && ld_out % 8 == 0,
              "row strides must be multiples of 8 and at least F");
  SPX_REQUIRE(gate && up && out && al16(gate) && al16(up) && al16(out), "null or unaligned buffer");
  const int64_t f8 = F / 8;
  hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(swiglu_grid(rows * f8)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(gate), ld_gate,
                     reinterpret_cast<const uint16_t*>(up), ld_up, reinterpret_cast<uint16_t*>(out), ld_out,
                     rows, f8);
  return check_launch(__func__);
}

extern "C" int spx_swiglu_rows_bwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                   const void* dout, int64_t ld_dout, void* dgate, int64_t ld_dgate,
                                   void* dup, int64_t ld_dup, int64_t rows, int64_t F, void* stream) {
  SPX_REQUIRE(rows > 0 && F > 0 && F % 8 == 0, "rows > 0 and F a positive multiple of 8");
  SPX_REQUIRE(ld_gate >= F && ld_up >= F && ld_dout >= F && ld_dgate >= F && ld_dup >= F &&
                  ld_gate % 8 == 0 && ld_up % 8 == 0 && ld_dout % 8 == 0 && ld_dgate % 8 == 0 && ld_dup % 8 == 0,
              "row strides must be multiples of 8 and at least F");
  SPX_REQUIRE(gate && up && dout && dgate && dup, "null buffer");
  SPX_REQUIRE(al16(gate) && al16(up) && al16(dout) && al16(dgate) && al16(dup), "buffers must be 16-byte aligned");
  const int64_t f8 = F / 8;
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(swiglu_grid(rows * f8)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t*>(gate), ld_gate,
                     reinterpret_cast<const uint16_t*>(up), ld_up, reinterpret_cast<const uint16_t*>(dout), ld_dout,
                     reinterpret_cast<uint16_t*>(dgate), ld_dgate, reinterpret_cast<uint16_t*>(dup), ld_dup, rows,
                     f8);
  return check_launch(__func__);
}

extern "C" int spx_swiglu_fwd(const void* gate, const void* up, void* out, int64_t n, void* stream) {
  return spx_swiglu_rows_fwd(gate, n, up, n, out, n, 1, n, stream);
}

extern "C" int spx_swiglu_bwd(const void* gate, const void* up, const void* dout, void* dgate, void* dup,
                              int64_t n, void* stream) {
  return spx_swiglu_rows_bwd(gate, n, up, n, dout, n, dgate, n, dup, n, 1, n, stream);
}
