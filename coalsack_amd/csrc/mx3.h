// Activations as three block-scaled FP6 terms, the A operand of the scaled
// matrix instructions (v_mfma_scale_f32_32x32x64_f8f6f4, A = E2M3, B = E2M1).
//
// A block of 32 consecutive values x is written as
//     x = 2^(s0-127) q0 + 2^(s1-127) q1 + 2^(s2-127) q2 + r,
// q_t = 32 E2M3 codes (sign, 2 exponent bits, 3 mantissa bits; |q| <= 7.5), each
// term the round-to-nearest of what the terms before it left over, its scale
// chosen so that the largest leftover lands in [4, 8).  Every term removes at
// least 4.9 bits of the block maximum, so |r| <= 2^-14.7 max|x| and, measured on
// N(0,1) rows, a 2880-long contraction differs from fp32 by 2.3e-5 relative rms.
// The MXFP4 weights are the instruction's B operand as they are stored (codes and
// E8M0 scale bytes are the hardware's own), products are exact, sums are fp32.
//
// Storage: [row][K/32][3 terms] x 32 bytes:
//     bytes 0..23  32 codes x 6 bits, code j at bits [6j, 6j+6) (little endian)
//     byte  24     E8M0 scale byte of the term
//     bytes 25..31 zero
// so a lane's operand for one matrix instruction is two aligned 16-byte chunks
// and carries its own scale.
#pragma once
#include "common.h"

namespace csk {

constexpr int kMx3Terms = 3;
constexpr int kMx3ChunksPerBlock = 2 * kMx3Terms;  // 16-byte chunks per 32-value block

// Rows are padded with all-zero blocks (codes 0, scale byte 127) to a whole number of the
// GEMM's four-block K steps, so that the GEMM never has to clamp or mask at the end of K.
__host__ __device__ inline int mx3_row_blocks(int nblk) { return (nblk + 3) & ~3; }

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef uint32_t u32x6 __attribute__((ext_vector_type(6)));

// Quantises one block held in registers; out[2t], out[2t+1] are the chunks of term t.
// v_cvt_scalef32_2xpk16_fp6_f32 divides by the scale, rounds to nearest even, saturates
// at +-7.5 and packs value i of its first operand at position 2i, of its second at
// 2i+1; v_cvt_scalef32_pk32_f32_fp6 is its inverse in position order (both probed).
__device__ __forceinline__ void mx3_quantize_block(float (&r)[32], u32x4 (&out)[kMx3ChunksPerBlock]) {
#pragma unroll
  for (int t = 0; t < kMx3Terms; ++t) {
    uint32_t eb;
    if (t == 0) {
      // the maximum of the magnitudes as integers: unlike a floating-point maximum it keeps a
      // NaN (and an infinity), which then shows as exponent byte 255
      uint32_t mb = 0u;
#pragma unroll
      for (int j = 0; j < 32; ++j) mb = max(mb, __float_as_uint(r[j]) & 0x7fffffffu);
      eb = mb >> 23;
    } else {
      float m = 0.0f;
#pragma unroll
      for (int j = 0; j < 32; ++j) m = fmaxf(m, fabsf(r[j]));
      eb = (__float_as_uint(m) >> 23) & 0xffu;
    }
    // block maximum / scale in [4, 8); blocks below 2^-124 are stored as zeros.  A block
    // that holds a NaN or an infinity gets scale byte 255 on its first term -- the E8M0 NaN,
    // which the matrix instruction turns into NaN products: every output of that row is then
    // NaN, as in fp32 arithmetic, instead of a saturated finite value.
    const bool nonfinite = t == 0 && eb == 255u;
    const uint32_t s = nonfinite ? 255u : eb < 3u ? 127u : min(eb - 2u, 252u);
    const float sc = __uint_as_float(min(s, 252u) << 23);  // 2^(s-127)
    f32x16 ev, od;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      ev[j] = r[2 * j];
      od[j] = r[2 * j + 1];
    }
    const u32x6 q = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(ev, od, sc);
    if (t + 1 < kMx3Terms) {
      const f32x32 d = __builtin_amdgcn_cvt_scalef32_pk32_f32_fp6(q, sc);
#pragma unroll
      for (int j = 0; j < 32; ++j) r[j] = r[j] - d[j];  // exact: d is r rounded to 4 bits
    }
    out[2 * t] = u32x4{q[0], q[1], q[2], q[3]};
    out[2 * t + 1] = u32x4{q[4], q[5], s, 0u};
  }
}

// rows of fp32 -> three-term FP6 blocks, one thread per block (padding blocks included):
//   x3[(row * mx3_row_blocks(nblk) + kb) * 6 + c] <- quantise(x[src(row)][32 kb .. 32 kb + 31] * w(row))
// src(row) = gather_tok[row] and w(row) = gather_w[row] when given (rows gathered and
// pre-scaled per dispatch position, expert_mlp_node.h:515-522), else row and 1.
__device__ __forceinline__ void mx3_rows_block(long b, const float* __restrict__ x, u32x4* __restrict__ x3,
                                               long rows, int nblk, const int* __restrict__ gather_tok,
                                               const float* __restrict__ gather_w) {
  const int rowblk = mx3_row_blocks(nblk);
  if (b >= rows * rowblk) return;
  const long row = b / rowblk;
  const int kb = (int)(b - row * rowblk);
  u32x4 out[kMx3ChunksPerBlock];
  if (kb >= nblk) {
#pragma unroll
    for (int t = 0; t < kMx3Terms; ++t) {
      out[2 * t] = u32x4{0u, 0u, 0u, 0u};
      out[2 * t + 1] = u32x4{0u, 0u, 127u, 0u};
    }
  } else {
    const long srow = gather_tok ? gather_tok[row] : row;
    const float gw = gather_w ? gather_w[row] : 1.0f;
    float r[32];
    const float4* src = reinterpret_cast<const float4*>(x + (srow * nblk + kb) * 32);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float4 v = src[i];
      r[4 * i] = v.x, r[4 * i + 1] = v.y, r[4 * i + 2] = v.z, r[4 * i + 3] = v.w;
    }
    if (gather_w) {
#pragma unroll
      for (int i = 0; i < 32; ++i) r[i] = r[i] * gw;
    }
    mx3_quantize_block(r, out);
  }
#pragma unroll
  for (int c = 0; c < kMx3ChunksPerBlock; ++c) x3[b * kMx3ChunksPerBlock + c] = out[c];
}
__global__ __launch_bounds__(256) void mx3_rows_kernel(const float* __restrict__ x,
                                                       u32x4* __restrict__ x3, long rows, int nblk,
                                                       const int* __restrict__ gather_tok,
                                                       const float* __restrict__ gather_w) {
  mx3_rows_block((long)blockIdx.x * 256 + threadIdx.x, x, x3, rows, nblk, gather_tok, gather_w);
}

// The same work as a rider of another kernel's launch: workgroups first_wg, first_wg + 1, ...
// of that kernel's grid write the rows (x3 == nullptr: no such workgroups were launched).
struct Mx3Rider {
  const float* x;
  u32x4* x3;
  long rows;
  int nblk;
  int first_wg;
};

}  // namespace csk
