// Expert MLP with fp16 weights (include/coalsack/nn/nn_ops/expert_mlp_node.h:269-389,
// compute_token :533-647): the branch the reference takes when the expert tensors arrive
// as float16 (dense checkpoints, or Q4_K / Q6_K experts widened at load,
// src/llm/moe_weight_provider.cpp:134-159).
//
// Weights [rows, K] are kept as tiles of 16 rows x 32 columns in matrix-instruction
// order,
//     w : [ceil(rows/16)][ceil(K/32)][64 lanes] x 16 B,
//     lane (n = lane % 16, g = lane / 16) = row 16*tile + n, columns 32*kb + 8*g .. + 7,
// zero beyond rows and K, so that a wave fetches one operand of v_mfma_f32_16x16x32_f16
// as 1 KiB of contiguous memory and no dimension needs to be a multiple of anything.
// The values are the checkpoint's own halves; nothing is rounded.
//
// Activations are fp32 in the reference.  Here a row is written as two fp16 terms of the
// row divided by a power of two chosen so that the row maximum lands in [2^14, 2^15):
//     x = 2^s * (hi + lo),  hi = fp16(x / 2^s),  lo = fp16(x / 2^s - hi),
// 22 significant bits for every element within 2^-14 of the row maximum (smaller ones keep
// an absolute error below 2^-25 of it).  Products of halves are exact in fp32, sums are
// fp32.  Storage [row][ceil(K/32)][hi: 32 halves | lo: 32 halves] (128 B per block) plus
// one fp32 scale per row.
#pragma once
#include "common.h"
#include "expert_stream_kernel.h"  // moe_activation

namespace csk {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

__host__ __device__ inline long f16_tile_count(long rows) { return (rows + 15) / 16; }
__host__ __device__ inline long f16_block_count(long K) { return (K + 31) / 32; }
// 16-byte entries of one packed matrix
__host__ __device__ inline long f16_entries(long rows, long K) {
  return f16_tile_count(rows) * f16_block_count(K) * 64;
}

// row-major halves [rows, K] -> tiles; one thread per 16-byte entry
__global__ __launch_bounds__(256) void f16_pack_kernel(const uint16_t* __restrict__ src,
                                                       u32x4* __restrict__ dst, long rows, long K,
                                                       long entries) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= entries) return;
  const long nkb = f16_block_count(K);
  const int lane = (int)(idx & 63);
  const long kb = (idx >> 6) % nkb, tile = (idx >> 6) / nkb;
  const long row = tile * 16 + (lane & 15), k0 = kb * 32 + 8 * (lane >> 4);
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (row < rows) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const long k = k0 + j;
      const uint32_t h = k < K ? src[row * K + k] : 0u;
      w[j >> 1] |= h << (16 * (j & 1));
    }
  }
  dst[idx] = u32x4{w[0], w[1], w[2], w[3]};
}

// Largest magnitude of an fp32 array, as the bit pattern of |w| (a NaN or an infinity
// compares above every finite value); *out must hold 0 on entry.
__global__ __launch_bounds__(256) void f32_absmax_bits_kernel(const float* __restrict__ src, long n,
                                                              unsigned int* __restrict__ out) {
  unsigned int m = 0u;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
    m = max(m, __float_as_uint(src[i]) & 0x7fffffffu);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = max(m, (unsigned int)__shfl_xor((int)m, o, 64));
  if ((threadIdx.x & 63) == 0 && m != 0u) atomicMax(out, m);
}

// Row-major fp32 [rows, K] -> tiles of the fp16 matrix [rows, 2 K] = [hi | lo] of w' = w * inv,
// hi = fp16(w'), lo = fp16(w' - hi): the two-term form of an fp32 weight, contracted against
// activation rows that repeat themselves ([x | x], see f16_split_rows_kernel), so that
// x . w' = x . hi + x . lo  comes out of the fp16 kernels unchanged.  inv is the power of two
// that brings the matrix's largest magnitude into [2^14, 2^15) -- the kernels multiply their
// sums by its reciprocal (wscale) -- so that hi and lo are normal fp16 numbers for every
// weight down to 2^-18 of the largest (22 significant bits; below that the absolute error
// is 2^-39 of the largest weight), whatever the matrix's overall magnitude.
__global__ __launch_bounds__(256) void f32_split_pack_kernel(const float* __restrict__ src,
                                                             u32x4* __restrict__ dst, long rows, long K,
                                                             long entries, float inv) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= entries) return;
  const long nkb = f16_block_count(2 * K);
  const int lane = (int)(idx & 63);
  const long kb = (idx >> 6) % nkb, tile = (idx >> 6) / nkb;
  const long row = tile * 16 + (lane & 15), k0 = kb * 32 + 8 * (lane >> 4);
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (row < rows) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const long k = k0 + j;
      if (k >= 2 * K) continue;
      const float v = src[row * K + (k < K ? k : k - K)] * inv;
      const _Float16 h = (_Float16)v;
      const _Float16 r = k < K ? h : (_Float16)(v - (float)h);
      w[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, r) << (16 * (j & 1));
    }
  }
  dst[idx] = u32x4{w[0], w[1], w[2], w[3]};
}

// tiles -> row-major halves (the export used to check that packing changed no bit)
__global__ __launch_bounds__(256) void f16_unpack_kernel(const u32x4* __restrict__ src,
                                                         uint16_t* __restrict__ dst, long rows,
                                                         long K, long entries) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= entries) return;
  const long nkb = f16_block_count(K);
  const int lane = (int)(idx & 63);
  const long kb = (idx >> 6) % nkb, tile = (idx >> 6) / nkb;
  const long row = tile * 16 + (lane & 15), k0 = kb * 32 + 8 * (lane >> 4);
  if (row >= rows) return;
  const u32x4 v = src[idx];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const long k = k0 + j;
    if (k < K) dst[row * K + k] = (uint16_t)(v[j >> 1] >> (16 * (j & 1)));
  }
}

// ---- K-quant expert tensors widened to fp16 at load
// (src/llm/moe_weight_provider.cpp:17-33, 134-159: dequantize_block_q4_K / q6_K to fp32,
// then fp32_to_fp16; include/coalsack/gguf/gguf_dequant.h:149-258, 458-487).  The
// arithmetic is the reference's operation by operation -- every product and difference
// rounded separately, and the conversion of a build without F16C, which truncates the
// mantissa -- so the resident halves equal the ones its provider would hand to the node.
constexpr int kGgmlQ4K = 12, kGgmlQ6K = 14;

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// gguf_dequant.h:463-487
__device__ __forceinline__ uint32_t f32_to_f16_truncating(float f) {
  const uint32_t bits = __float_as_uint(f);
  const uint32_t sign = (bits >> 16) & 0x8000u;
  const int e = (int)((bits >> 23) & 0xffu) - 127 + 15;
  uint32_t m = (bits >> 13) & 0x3ffu;
  if (e <= 0) {
    if (e < -10) return sign;
    m |= 0x400u;
    m >>= (1 - e);
    return sign | m;
  }
  if (e >= 31) return sign | 0x7c00u;
  return sign | ((uint32_t)e << 10) | m;
}

// value idx of a Q4_K stream (144-byte super-blocks of 256; gguf_dequant.h:149-204)
__device__ __forceinline__ float q4k_value(const uint8_t* __restrict__ src, long idx) {
#pragma clang fp contract(off)
  const uint8_t* blk = src + (idx >> 8) * 144;
  const int w = (int)(idx & 255), j = w >> 5, l = w & 31;
  const float d = half_bits_to_float(blk[0] | (blk[1] << 8));
  const float dmin = half_bits_to_float(blk[2] | (blk[3] << 8));
  const uint8_t* sc = blk + 4;
  uint32_t s6, m6;
  if (j < 4) {
    s6 = sc[j] & 0x3F;
    m6 = sc[j + 4] & 0x3F;
  } else {
    s6 = (sc[j + 4] & 0x0F) | ((sc[j - 4] >> 6) << 4);
    m6 = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4);
  }
  const float dj = d * (float)s6;
  const float mj = dmin * (float)m6;
  const uint32_t qb = blk[16 + 32 * (j >> 1) + l];
  const float prod = dj * (float)((j & 1) ? (qb >> 4) : (qb & 0x0F));
  return prod - mj;
}

// value idx of a Q6_K stream (210-byte super-blocks of 256; gguf_dequant.h:220-258)
__device__ __forceinline__ float q6k_value(const uint8_t* __restrict__ src, long idx) {
#pragma clang fp contract(off)
  const uint8_t* blk = src + (idx >> 8) * 210;
  const int w = (int)(idx & 255), n = w >> 7, r = w & 127, g = r >> 5, l = r & 31;
  const uint8_t* ql = blk + 64 * n;
  const uint8_t* qh = blk + 128 + 32 * n;
  const int8_t* sc = reinterpret_cast<const int8_t*>(blk + 192) + 8 * n;
  const uint32_t lb = ql[l + 32 * (g & 1)];
  const uint32_t low = g >= 2 ? (lb >> 4) : (lb & 0xF);
  const uint32_t high = (qh[l] >> (2 * g)) & 3;
  const int q = (int)(int8_t)(low | (high << 4)) - 32;
  const float d = half_bits_to_float(blk[208] | (blk[209] << 8));
  const float ds = d * (float)sc[(l >> 4) + 2 * g];
  return ds * (float)q;
}

// K-quant stream of a row-major [rows, K] matrix -> fp16 tiles; one thread per 16-byte entry
template <int TYPE>
__global__ __launch_bounds__(256) void kquant_pack_kernel(const uint8_t* __restrict__ src,
                                                          u32x4* __restrict__ dst, long rows, long K,
                                                          long entries) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= entries) return;
  const long nkb = f16_block_count(K);
  const int lane = (int)(idx & 63);
  const long kb = (idx >> 6) % nkb, tile = (idx >> 6) / nkb;
  const long row = tile * 16 + (lane & 15), k0 = kb * 32 + 8 * (lane >> 4);
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (row < rows) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const long k = k0 + j;
      if (k < K) {
        const float v = TYPE == kGgmlQ4K ? q4k_value(src, row * K + k) : q6k_value(src, row * K + k);
        w[j >> 1] |= f32_to_f16_truncating(v) << (16 * (j & 1));
      }
    }
  }
  dst[idx] = u32x4{w[0], w[1], w[2], w[3]};
}

// synthetic weights straight into the tiles: halves j / 2^14, j uniform in [-2048, 2047]
// (every value exact in fp16), a function of (key, row, column) only; zero in the padding
__global__ __launch_bounds__(256) void synth_f16_kernel(u32x4* __restrict__ dst, long rows, long K,
                                                        long entries, uint64_t key) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= entries) return;
  const long nkb = f16_block_count(K);
  const int lane = (int)(idx & 63);
  const long kb = (idx >> 6) % nkb, tile = (idx >> 6) / nkb;
  const long row = tile * 16 + (lane & 15), k0 = kb * 32 + 8 * (lane >> 4);
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (row < rows) {
    const uint64_t r = mix64(key ^ (uint64_t)(row * nkb * 4 + kb * 4 + (lane >> 4)));
    const uint64_t r2 = mix64(r);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int v = (int)(((j < 4 ? r : r2) >> (16 * (j & 3))) & 0xfff) - 2048;
      const _Float16 h = (_Float16)((float)v * (1.0f / 16384.0f));
      if (k0 + j < K) w[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, h) << (16 * (j & 1));
    }
  }
  dst[idx] = u32x4{w[0], w[1], w[2], w[3]};
}

// fp32 rows -> scaled two-term fp16 rows.  One workgroup per output row; the source row is
// gather_tok[row] scaled by gather_w[row] when given (weight_before_ffn: the reference
// multiplies the token by its routing weight in fp32 first, expert_mlp_node.h:766-772).
// The logical row has K elements read from a source row of Ksrc: element k is source element
// k mod Ksrc (K = Ksrc, or 2 Ksrc for the repeated rows that two-term fp32 weights need).
__global__ __launch_bounds__(256) void f16_split_rows_kernel(const float* __restrict__ x, long K, long Ksrc,
                                                             const int* __restrict__ gather_tok,
                                                             const float* __restrict__ gather_w,
                                                             u32x4* __restrict__ out,
                                                             float* __restrict__ rscale) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const long srow = gather_tok ? gather_tok[row] : row;
  const float gw = gather_w ? gather_w[row] : 1.0f;
  const float* xr = x + srow * Ksrc;
  float m = 0.0f;
  for (long i = threadIdx.x; i < Ksrc; i += 256) m = fmaxf(m, fabsf(xr[i] * gw));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  // 2^s with the row maximum / 2^s in [2^14, 2^15); rows of zeros (or of non-finite
  // values, which then propagate as they would in fp32) keep s = 0
  const int eb = (int)((__float_as_uint(m) >> 23) & 0xffu);
  int s = (eb == 0 || eb == 255) ? 0 : eb - 127 - 14;
  s = max(-100, min(100, s));
  const float inv = __uint_as_float((uint32_t)(127 - s) << 23);
  if (threadIdx.x == 0) rscale[row] = __uint_as_float((uint32_t)(127 + s) << 23);
  const long nkb = f16_block_count(K);
  // one thread per 8 consecutive elements: chunk c of block kb
  for (long i = threadIdx.x; i < nkb * 4; i += 256) {
    const long kb = i >> 2;
    const int c = (int)(i & 3);
    uint32_t hi[4] = {0u, 0u, 0u, 0u}, lo[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const long k = kb * 32 + c * 8 + j;
      const float v = k < K ? (xr[k < Ksrc ? k : k - Ksrc] * gw) * inv : 0.0f;
      const _Float16 h = (_Float16)v;
      const _Float16 l = (_Float16)(v - (float)h);
      hi[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, h) << (16 * (j & 1));
      lo[j >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, l) << (16 * (j & 1));
    }
    u32x4* dst = out + (row * nkb + kb) * 8;
    dst[c] = u32x4{hi[0], hi[1], hi[2], hi[3]};
    dst[4 + c] = u32x4{lo[0], lo[1], lo[2], lo[3]};
  }
}

struct ExpertF16Args {
  const WorkDesc* desc;  // [n_slots]: active experts first, the rest with Te = 0
  int n_slots;
  const int* list_row;   // activation row of a packed position, or null: the position itself
  const u32x4* B;        // two-term fp16 activation rows
  const float* rscale;   // their scales
  float wscale[2];       // power-of-two scale of the weights: gate and up (MODE 0), down (MODE 1, [0]); 1 for fp16 weights
  int nkb;               // ceil(K / 32)
  int N;                 // output features: F (gate/up) or H (down)
  int ntile;             // ceil(N / 16)
  int act_type;
  float* out;            // MODE 0: activations [P, N] fp32; MODE 1: y [P, N]
};

constexpr int kF16Depth = 4;  // K blocks in flight per wave

// MODE 0: act = activation(W_gate x + b_gate, W_up x + b_up); MODE 1: y = W_down act + b_down.
// A workgroup of four waves takes one work unit at a time: (expert, pair of 16-row weight
// tiles -- gate and up tile p, or down tiles 2p and 2p+1 --, group of up to 16 dispatched
// tokens).  Units are numbered expert-major, then pair, then group, so the groups of one
// expert meet their weight tiles in cache at the same time.  The four waves split K; each
// keeps kF16Depth blocks of loads in flight in a rotating register set; the partial sums
// meet in LDS and are added in a fixed order.  The weights are the A operand (rows 4g..4g+3
// of the tile end up in one lane), the tokens the B operand (lane % 16).
constexpr int kF16GroupTokens = 16;

template <int MODE>
__global__ __launch_bounds__(256) void expert_f16_kernel(ExpertF16Args a) {
  __shared__ int prefix[kMaxExperts + 1];
  __shared__ floatx4 red[4][2][64];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int npair = MODE == 0 ? a.ntile : (a.ntile + 1) / 2;
  constexpr int GT = kF16GroupTokens;
  // units per slot, exclusive prefix over slots (wave 0; four consecutive slots per lane)
  if (wv == 0) {
    int c[4], tot = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = lane * 4 + j;
      const int te = s < a.n_slots ? a.desc[s].Te : 0;
      c[j] = ((te + GT - 1) / GT) * npair;
      tot += c[j];
    }
    int inc = tot;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(inc, o, 64);
      if (lane >= o) inc += t;
    }
    int run = inc - tot;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      prefix[lane * 4 + j] = run;
      run += c[j];
    }
    if (lane == 63) prefix[kMaxExperts] = inc;
  }
  __syncthreads();
  const int n_units = prefix[kMaxExperts];
  const int kq = (a.nkb + 3) / 4;
  const int kb_lo = min(wv * kq, a.nkb), kb_hi = min(kb_lo + kq, a.nkb);

  for (int u = blockIdx.x; u < n_units; u += gridDim.x) {
    // slot of unit u: last slot whose prefix is <= u (binary search over 256 entries)
    int s = 0;
#pragma unroll
    for (int step = kMaxExperts / 2; step > 0; step >>= 1)
      if (prefix[s + step] <= u) s += step;
    const WorkDesc* wd = a.desc + s;
    const int te = wd->Te, base = wd->base;
    const int ngrp = (te + GT - 1) / GT;
    const int r = u - prefix[s];
    const int p = r / ngrp, m0 = (r - p * ngrp) * GT;
    const int cnt = min(GT, te - m0);
    // weight tiles of the pair
    const int t0 = MODE == 0 ? p : 2 * p;
    const int t1 = MODE == 0 ? p : min(2 * p + 1, a.ntile - 1);
    const CSK_GLOBAL u32x4* A0 = as_global(reinterpret_cast<const u32x4*>(MODE == 0 ? wd->w.q_gate : wd->w.q_down)) + (long)t0 * a.nkb * 64 + lane;
    const CSK_GLOBAL u32x4* A1 = as_global(reinterpret_cast<const u32x4*>(MODE == 0 ? wd->w.q_up : wd->w.q_down)) + (long)t1 * a.nkb * 64 + lane;
    // activation row of the lane's token slot (slots past the group re-read its last row)
    const int pos_l = base + m0 + min(n16, cnt - 1);
    const long row = a.list_row ? a.list_row[pos_l] : pos_l;
    const CSK_GLOBAL u32x4* Brow = as_global(a.B) + row * a.nkb * 8 + g;
    const float scale = a.rscale[row] * a.wscale[0];                          // row scale x weight scale: powers of two
    const float scale1 = a.rscale[row] * a.wscale[MODE == 0 ? 1 : 0];
    floatx4 acc[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};

    u32x4 qa[kF16Depth][2], qh[kF16Depth], ql[kF16Depth];
    auto fetch = [&](int slot, int kb) {
      const int kc = min(kb, kb_hi - 1);  // past the wave's range: re-read its last block
      qa[slot][0] = A0[(long)kc * 64];
      qa[slot][1] = A1[(long)kc * 64];
      qh[slot] = Brow[(long)kc * 8];
      ql[slot] = Brow[(long)kc * 8 + 4];
    };
    auto fma_block = [&](int slot) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const half8 wa = __builtin_bit_cast(half8, qa[slot][t]);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, __builtin_bit_cast(half8, qh[slot]), acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, __builtin_bit_cast(half8, ql[slot]), acc[t], 0, 0, 0);
      }
    };
    if (kb_lo < kb_hi) {
#pragma unroll
      for (int j = 0; j < kF16Depth; ++j) fetch(j, kb_lo + j);
      for (int kb = kb_lo; kb < kb_hi; kb += kF16Depth) {
#pragma unroll
        for (int j = 0; j < kF16Depth; ++j) {
          if (kb + j < kb_hi) fma_block(j);
          fetch(j, kb + j + kF16Depth);
        }
      }
    }
    red[wv][0][lane] = acc[0];
    red[wv][1][lane] = acc[1];
    __syncthreads();
    // wave 0 finishes the unit: partial sums in wave order, row scale, bias, activation
    if (wv == 0 && n16 < cnt) {
      floatx4 v[2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
        v[t] = ((red[0][t][lane] + red[1][t][lane]) + red[2][t][lane]) + red[3][t][lane];
      const long pos = base + m0 + n16;
      const CSK_GLOBAL float* b0 = as_global(MODE == 0 ? wd->w.b_gate : wd->w.b_down);
      const CSK_GLOBAL float* b1 = as_global(MODE == 0 ? wd->w.b_up : wd->w.b_down);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (MODE == 0) {
          const int f = 16 * p + 4 * g + i;
          if (f < a.N)
            a.out[pos * a.N + f] = moe_activation(v[0][i] * scale + b0[f], v[1][i] * scale1 + b1[f], a.act_type);
        } else {
          const int h0 = 16 * (2 * p) + 4 * g + i, h1 = h0 + 16;
          if (h0 < a.N) a.out[pos * a.N + h0] = v[0][i] * scale + b0[h0];
          if (h1 < a.N) a.out[pos * a.N + h1] = v[1][i] * scale1 + b1[h1];
        }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- many tokens
// Grouped GEMM for batches in which an expert sees tens to hundreds of tokens.  A
// workgroup (4 waves) owns 64 dispatched tokens x 256 weight rows (128 features of gate
// and up, or 256 rows of down) on v_mfma_f32_32x32x16_f16: tokens are the A operand
// (accumulator register <-> token), weight rows the B operand (lane % 32 <-> row), so a
// wave's stores are 128 contiguous bytes per token.  Per K step of 64 the token panel
// (64 tokens x [hi | lo] = 16 KB) goes through LDS, double buffered, 16-byte chunks
// XOR-swizzled by token so that the 32 lanes of a fragment read hit distinct banks; the
// weights go from memory straight to registers, one step ahead, each slice reloaded into
// the registers it has just been consumed from.  Work units (M tile, N
// tile) are numbered expert by expert and dealt to the eight dies in contiguous eighths.
struct ExpertF16GemmArgs {
  const WorkDesc* desc;
  const int* mtiles;    // (slot, first token) per 64-token M tile
  const int* n_mtiles;
  const int* list_row;  // activation row of a packed position, or null: the position itself
  const u32x4* B;       // two-term fp16 activation rows
  const float* rscale;
  float wscale[2];      // as in ExpertF16Args
  int nkb, N, ntile, n_ntiles, act_type;
  float* out;
};

constexpr int kF16Dies = 8;

template <int MODE>
__global__ __launch_bounds__(256, 3) void expert_f16_gemm_kernel(ExpertF16GemmArgs a) {
  __shared__ u32x4 panel[2][64 * 16];  // [buffer][token][16 chunks: block 0 hi 0-3, lo 0-3, block 1 ...]
  __shared__ float rs_sh[64];
  const int n_units = *a.n_mtiles * a.n_ntiles;
  const int per_die = (n_units + kF16Dies - 1) / kF16Dies;
  const int slot_i = blockIdx.x / kF16Dies;
  const int unit = (blockIdx.x % kF16Dies) * per_die + slot_i;
  if (slot_i >= per_die || unit >= n_units) return;
  const int mt_seq = unit / a.n_ntiles;
  const WorkDesc* wd = a.desc + a.mtiles[2 * mt_seq];
  int nt = unit - mt_seq * a.n_ntiles, m0 = a.mtiles[2 * mt_seq + 1];
  if (MODE == 0) {
    // Gate/up has more N tiles than a die holds workgroups per M tile, and fp16 weight rows are
    // the larger operand: within an expert's block of the sequence the units run N tile by N
    // tile, the expert's M tiles side by side, so that the workgroups resident together read
    // the same weight rows at about the same time and those come from memory once (measured:
    // 698 -> 610 us at 2048 tokens; the down projection, whose twelve N tiles are all in
    // flight at once either way, is faster in M-tile order).
    const int tiles_e = (wd->Te + 63) / 64;
    const int r = unit - (mt_seq - m0 / 64) * a.n_ntiles;  // position within the expert's block
    nt = r / tiles_e;
    m0 = (r - nt * tiles_e) * 64;
  }
  const int base = wd->base + m0;
  const int mcount = min(64, wd->Te - m0);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n32 = lane & 31, kg = lane >> 5;
  const int n16 = n32 & 15, th = n32 >> 4;
  const int nkb = a.nkb, nsteps = (nkb + 1) >> 1;

  // this lane's weight entries: row n32 of the wave's two 32-row groups
  int rows[2];
  const CSK_GLOBAL u32x4* W[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int t = MODE == 0 ? nt * 8 + wv * 2 + th : nt * 16 + wv * 4 + 2 * s + th;
    rows[s] = t * 16 + n16;
    const uint4* q = MODE == 0 ? (s == 0 ? wd->w.q_gate : wd->w.q_up) : wd->w.q_down;
    W[s] = as_global(reinterpret_cast<const u32x4*>(q)) + (long)min(t, a.ntile - 1) * nkb * 64 + n16 + 16 * kg;
  }
  // staging: thread copies chunk sc of tokens st + 16 i
  const int sc = threadIdx.x & 15, st = threadIdx.x >> 4;
  const CSK_GLOBAL u32x4* Arow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int pos = base + min(st + 16 * i, mcount - 1);  // tokens past the tile re-read its last
    const long row = a.list_row ? a.list_row[pos] : pos;
    Arow[i] = as_global(a.B) + row * nkb * 8 + (sc & 7);
    if (sc == 0) rs_sh[st + 16 * i] = a.rscale[row];
  }
  const int sblk = sc >> 3;  // block of the step this thread's chunk belongs to

  floatx16 acc[2][2];  // [32-token half][row group]
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ms][s][r] = 0.0f;

  u32x4 wq[2][4];  // [row group][16-wide K slice of the step]
  u32x4 aq[4];
  // Every load of the loop is unconditional (addresses are clamped, never branched around):
  // with a branch around a load the compiler's wait-count pass gives up at the join and
  // drains the whole queue at the head of every step.  A block past K (odd block count: the
  // second half of the last step) re-reads the last block of the weights and meets a panel
  // chunk of zeros.
  auto load_w = [&](int s, int sl, int j) {
    const int kb = min(2 * j + (sl >> 1), nkb - 1);
    wq[s][sl] = W[s][(long)kb * 64 + 32 * (sl & 1)];
  };
  auto load_a = [&](int j) {
    const int kbs = min(2 * j + sblk, nkb - 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) aq[i] = Arow[i][(long)kbs * 8];
  };
  auto stash = [&](int buf, int j) {
    const bool past = 2 * j + sblk >= nkb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = st + 16 * i;
      panel[buf][tok * 16 + (sc ^ (tok & 15))] = past ? u32x4{0u, 0u, 0u, 0u} : aq[i];
    }
  };
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) load_w(s, sl, 0);
  load_a(0);
  stash(0, 0);
  __syncthreads();
  // One step = 64 of K: four 16-wide slices, each 2 row groups x 2 token halves x 2 terms of
  // matrix instructions.  The panel fragments of a token half are read from LDS while the
  // matrix instructions of the other half issue (the same four fragment registers in
  // rotation); a slice's weight registers are reloaded for the next step as soon as its
  // matrix instructions have issued; the next step's panel rows are requested at the head
  // of the step and stored to the other LDS buffer at its end, behind a wait that leaves the
  // weight loads in flight.
  auto step = [&](int j, auto more_t) {
    constexpr bool more = decltype(more_t)::value;
    const int buf = j & 1;
    if (more) load_a(j + 1);
    half8 hi[2], lo[2];
    auto read_half = [&](int sl, int ms) {
      // logical chunk of this lane's 8 halves: block sl / 2, [hi | lo], quarter 2 (sl % 2) + kg
      const int c_hi = (sl >> 1) * 8 + 2 * (sl & 1) + kg, c_lo = c_hi + 4;
      const int tok = ms * 32 + n32;
      hi[ms] = __builtin_bit_cast(half8, panel[buf][tok * 16 + (c_hi ^ n16)]);
      lo[ms] = __builtin_bit_cast(half8, panel[buf][tok * 16 + (c_lo ^ n16)]);
    };
    read_half(0, 0);
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      read_half(sl, 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const half8 w = __builtin_bit_cast(half8, wq[s][sl]);
        acc[0][s] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hi[0], w, acc[0][s], 0, 0, 0);
        acc[0][s] = __builtin_amdgcn_mfma_f32_32x32x16_f16(lo[0], w, acc[0][s], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (sl + 1 < 4) read_half(sl + 1, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const half8 w = __builtin_bit_cast(half8, wq[s][sl]);
        acc[1][s] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hi[1], w, acc[1][s], 0, 0, 0);
        acc[1][s] = __builtin_amdgcn_mfma_f32_32x32x16_f16(lo[1], w, acc[1][s], 0, 0, 0);
      }
      // the slice's registers are free as soon as its matrix instructions have issued:
      // the next step's weights go straight back into them (one register set in rotation)
      if (more) {
        load_w(0, sl, j + 1);
        load_w(1, sl, j + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) stash(buf ^ 1, j + 1);
    __syncthreads();
  };
  for (int j = 0; j + 1 < nsteps; ++j) step(j, std::true_type{});
  step(nsteps - 1, std::false_type{});

  // accumulator register r is token (r % 4) + 8 (r / 4) + 4 kg of its 32-token half
  const CSK_GLOBAL float* b0 = as_global(MODE == 0 ? wd->w.b_gate : wd->w.b_down);
  const CSK_GLOBAL float* b1 = as_global(MODE == 0 ? wd->w.b_up : wd->w.b_down);
  float bias[2];
  bool rv[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    rv[s] = rows[s] < a.N;
    bias[s] = rv[s] ? (s == 0 ? b0 : b1)[rows[s]] : 0.0f;
  }
#pragma unroll
  for (int ms = 0; ms < 2; ++ms) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
      if (tl >= mcount) continue;
      const float sc_t = rs_sh[tl] * a.wscale[0];
      float* o = a.out + (long)(base + tl) * a.N;
      if (MODE == 0) {
        const float sc_u = rs_sh[tl] * a.wscale[1];
        if (rv[0])
          o[rows[0]] = moe_activation(acc[ms][0][r] * sc_t + bias[0], acc[ms][1][r] * sc_u + bias[1], a.act_type);
      } else {
#pragma unroll
        for (int s = 0; s < 2; ++s)
          if (rv[s]) o[rows[s]] = acc[ms][s][r] * sc_t + bias[s];
      }
    }
  }
}

}  // namespace csk
