// MXFP4 storage kernels: repack the reference's 17-byte blocks into the tiled
// device layout, the inverse, device-side dequantisation, and the synthetic
// weight generator.  All are one thread per (tile, block, row-in-tile) entry of
// the packed layout, so packed-side accesses are fully coalesced.
#pragma once
#include "common.h"

namespace csk {

// Reference block (include/coalsack/gguf/gguf_dequant.h:437-455): byte 0 scale,
// byte 1+j = element j (low nibble) | element j+16 (high nibble).
// Packed entry: byte b = element 2b (low) | element 2b+1 (high).
__device__ __forceinline__ uint4 ref_block_to_entry(const uint8_t* blk) {
  uint32_t w[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    uint32_t v = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int b = d * 4 + c;  // packed byte index, elements 2b and 2b+1
      uint32_t lo, hi;
      if (b < 8) {
        lo = blk[1 + 2 * b] & 15u;
        hi = blk[2 + 2 * b] & 15u;
      } else {
        lo = blk[1 + 2 * b - 16] >> 4;
        hi = blk[2 + 2 * b - 16] >> 4;
      }
      v |= (lo | (hi << 4)) << (8 * c);
    }
    w[d] = v;
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

__device__ __forceinline__ void entry_to_ref_block(uint4 q, uint8_t scale, uint8_t* blk) {
  const uint32_t w[4] = {q.x, q.y, q.z, q.w};
  uint8_t code[32];
#pragma unroll
  for (int b = 0; b < 16; ++b) {
    const uint32_t byte = (w[b >> 2] >> (8 * (b & 3))) & 0xFFu;
    code[2 * b] = byte & 15u;
    code[2 * b + 1] = byte >> 4;
  }
  blk[0] = scale;
#pragma unroll
  for (int j = 0; j < 16; ++j) blk[1 + j] = (uint8_t)(code[j] | (code[j + 16] << 4));
}

// Every code of the entry is 0 or 0.5 in magnitude (E2M1 codes 0, 1, 8, 9).
__device__ __forceinline__ bool entry_below_one(const uint4& e) {
  return ((e.x | e.y | e.z | e.w) & 0x66666666u) == 0u;
}
// Such an entry with every magnitude doubled: code 1 (0.5) becomes code 2 (1.0), signs stay.
__device__ __forceinline__ uint32_t double_small_codes(uint32_t w) {
  return (w & 0x88888888u) | ((w & 0x11111111u) << 1);
}

// entries = ntile * nblk * 16
// Scale bytes: every byte the reference decodes to a finite value is kept as it is
// (gguf_dequant.h:419-433: 0 and 1 are 2^-128 and 2^-127 on the doubled code table; ggml
// writes 0 for an all-zero block).  Byte 255 is 2^127 on the doubled code table in the
// reference and "not a number" to the matrix instruction.  Its finite values -- codes 0 and
// +-0.5, i.e. 0 and +-2^127 -- are stored exactly as byte 254 with the codes doubled (+-0.5
// becomes +-1); a block that holds any larger code decodes to an infinity in the reference
// (2 x 2^127 and up overflow fp32) and `bad` receives the lowest such block index (it must
// hold ~0 on entry).
__global__ void pack_mxfp4_kernel(const uint8_t* __restrict__ src, uint4* __restrict__ q,
                                  uint8_t* __restrict__ s, int rows, int nblk, long entries,
                                  unsigned long long* __restrict__ bad) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= entries) return;
  const int n = (int)(i & 15);
  const long tk = i >> 4;
  const int kb = (int)(tk % nblk);
  const long tile = tk / nblk;
  const long row = tile * 16 + n;
  const size_t si = scale_index(tile, kb, n, scale_slots(nblk));
  if (row >= rows) {
    q[i] = make_uint4(0, 0, 0, 0);
    s[si] = 127;
    return;
  }
  const uint8_t* blk = src + (row * nblk + kb) * 17;
  uint4 e = ref_block_to_entry(blk);
  uint8_t sb = blk[0];
  if (sb == 255) {
    if (entry_below_one(e)) {
      e = make_uint4(double_small_codes(e.x), double_small_codes(e.y), double_small_codes(e.z), double_small_codes(e.w));
      sb = 254;
    } else if (bad) {
      atomicMin(bad, (unsigned long long)(row * nblk + kb));
    }
  }
  q[i] = e;
  s[si] = sb;
}

__global__ void export_mxfp4_kernel(const uint4* __restrict__ q, const uint8_t* __restrict__ s,
                                    uint8_t* __restrict__ dst, int rows, int nblk, long entries) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= entries) return;
  const int n = (int)(i & 15);
  const long tk = i >> 4;
  const int kb = (int)(tk % nblk);
  const long tile = tk / nblk;
  const long row = tile * 16 + n;
  const size_t si = scale_index(tile, kb, n, scale_slots(nblk));
  if (row >= rows) return;
  entry_to_ref_block(q[i], s[si], dst + (row * nblk + kb) * 17);
}

// Dequantise through the same conversion instruction the expert kernels use
// (v_cvt_scalef32_pk_bf16_fp4), then widen bf16 -> f32, which is exact.
// Code 8 (sign set, magnitude 0) converts to -0.0 in hardware where the
// reference's integer table gives +0.0 (gguf_dequant.h:413-415); adding +0.0
// canonicalises it.  Inside a contraction the two zeros are interchangeable.
__global__ void dequant_mxfp4_kernel(const uint4* __restrict__ q, const uint8_t* __restrict__ s,
                                     float* __restrict__ dst, int rows, int nblk, long entries) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= entries) return;
  const int n = (int)(i & 15);
  const long tk = i >> 4;
  const int kb = (int)(tk % nblk);
  const long tile = tk / nblk;
  const long row = tile * 16 + n;
  const size_t si = scale_index(tile, kb, n, scale_slots(nblk));
  if (row >= rows) return;
  const uint4 e = q[i];
  const uint32_t w[4] = {e.x, e.y, e.z, e.w};
  float* o = dst + (row * nblk + kb) * 32;
  if (s[si] < 2) {
    // scale bytes 0 and 1: the products are fp32 denormals, which the conversion instruction
    // does not produce; the reference's own arithmetic instead (doubled code table times
    // 2^-128 or 2^-127, gguf_dequant.h:413-455).  The expert kernels treat these blocks as
    // what they are to any contraction: zero to within 1e-37.
    const float half_scale = __uint_as_float(0x00200000u << s[si]);
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const uint32_t code = (w[j >> 3] >> (4 * (j & 7))) & 15u;
      const int mag = (code & 7u) < 5u ? (int)(code & 7u) : ((code & 7u) == 5u ? 6 : ((code & 7u) == 6u ? 8 : 12));
      o[j] = (float)((code & 8u) ? -mag : mag) * half_scale;
    }
    return;
  }
  const float sc = e8m0_scale(s[si]);
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    bf16x2 r0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], sc, 0);
    bf16x2 r1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], sc, 1);
    bf16x2 r2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], sc, 2);
    bf16x2 r3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], sc, 3);
    o[d * 8 + 0] = (float)r0[0] + 0.0f;
    o[d * 8 + 1] = (float)r0[1] + 0.0f;
    o[d * 8 + 2] = (float)r1[0] + 0.0f;
    o[d * 8 + 3] = (float)r1[1] + 0.0f;
    o[d * 8 + 4] = (float)r2[0] + 0.0f;
    o[d * 8 + 5] = (float)r2[1] + 0.0f;
    o[d * 8 + 6] = (float)r3[0] + 0.0f;
    o[d * 8 + 7] = (float)r3[1] + 0.0f;
  }
}

// Synthetic weights, generated straight into the packed layout.  Block b =
// row * nblk + kb of the stream with key `key` is, in the reference's format,
//   scale byte = scale_lo + (h0 >> 33) % scale_span,
//   quant bytes 1..8 = little-endian bytes of h1, 9..16 = those of h2,
// with h_i = mix64(key + 3 b + i).
__global__ void synth_mxfp4_kernel(uint4* __restrict__ q, uint8_t* __restrict__ s, int rows,
                                   int nblk, long entries, uint64_t key, int scale_lo,
                                   int scale_span) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= entries) return;
  const int n = (int)(i & 15);
  const long tk = i >> 4;
  const int kb = (int)(tk % nblk);
  const long tile = tk / nblk;
  const long row = tile * 16 + n;
  const size_t si = scale_index(tile, kb, n, scale_slots(nblk));
  if (row >= rows) {
    q[i] = make_uint4(0, 0, 0, 0);
    s[si] = 127;
    return;
  }
  const uint64_t b = (uint64_t)(row * nblk + kb);
  const uint64_t h0 = mix64(key + 3 * b), h1 = mix64(key + 3 * b + 1), h2 = mix64(key + 3 * b + 2);
  uint8_t blk[17];
  blk[0] = (uint8_t)(scale_lo + (int)((h0 >> 33) % (uint64_t)scale_span));
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    blk[1 + j] = (uint8_t)(h1 >> (8 * j));
    blk[9 + j] = (uint8_t)(h2 >> (8 * j));
  }
  q[i] = ref_block_to_entry(blk);
  s[si] = blk[0];
}

}  // namespace csk
