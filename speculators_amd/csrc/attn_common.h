// Pieces shared by the TTT and anchored-block attention kernels (gfx950).
//
// Tiling: one workgroup = 4 waves = 128 query rows of one query head; each
// wave owns 32 query rows.  Scores are produced TRANSPOSED, S^T = K Q^T, with
// v_mfma_f32_32x32x16_bf16: in the 32x32 accumulator a lane then holds ONE
// query (column = lane % 32) and 16 keys (row = 8*(r/4) + 4*(lane/32) + r%4
// for register r), so soft-max row statistics are per-lane scalars plus one
// cross-half shuffle, and the probabilities feed the second product
// O^T = V^T P^T directly as the B operand (a lane's registers 8s..8s+7 are the
// eight k-slots of the 16-key step s).  The A operand of that product needs V
// with keys contiguous, so V is transposed once per call into a workspace.
#pragma once

#include "spx_common.h"

namespace spx {

constexpr int kAttnThreads = 256;
constexpr int kBM = 128;  // query rows per workgroup
constexpr int kBN = 64;   // keys per tile
constexpr int kKPad = 8;  // K tile row stride = D + 8 elements  (272 B at D=128)
constexpr int kVPad = 8;  // V^T tile row stride = 64 + 8 elements (144 B: 16-byte aligned rows)

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// key (row) index of accumulator register r for lane half g, inside a 32-row block
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}
__device__ __forceinline__ bf16x8 join_bf16x4(u32x2 lo, u32x2 hi) {
  union { u32x4 u; bf16x8 b; } c;
  c.u.x = lo.x; c.u.y = lo.y; c.u.z = hi.x; c.u.w = hi.y;
  return c.b;
}
// eight consecutive accumulator registers -> bf16x8 (B operand of the next product)
__device__ __forceinline__ bf16x8 pack8(const f32x16& a, int base) {
  union { u32x4 u; bf16x8 b; } c;
  c.u.x = pack_bf16x2(a[base + 0], a[base + 1]);
  c.u.y = pack_bf16x2(a[base + 2], a[base + 3]);
  c.u.z = pack_bf16x2(a[base + 4], a[base + 5]);
  c.u.w = pack_bf16x2(a[base + 6], a[base + 7]);
  return c.b;
}

// dot product of two 8-element bf16 fragments, accumulated in fp32 with the packed
// bf16 dot instruction (v_dot2c_f32_bf16): no conversion of the operands to fp32
__device__ __forceinline__ float dot8_bf16(bf16x8 a, u32x4 b, float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  union { bf16x8 v; bf16x2_t p[4]; } ua;
  union { u32x4 v; bf16x2_t p[4]; } ub;
  ua.v = a;
  ub.v = b;
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(ua.p[i], ub.p[i], acc, false);
  return acc;
}

__device__ __forceinline__ void unpack8(u32x4 raw, float v[8]) {
  v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x);
  v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
  v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z);
  v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
}
__device__ __forceinline__ void unpack4(u32x2 raw, float v[4]) {
  v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x);
  v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
}

}  // namespace spx
