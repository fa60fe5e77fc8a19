// Prologue (optional RMSNorm of the activations), router
// (gate GEMV, wavefront top-k, softmax over the selected k), dispatch
// (histogram -> prefix scan -> ordered scatter) and the weighted combine.
#pragma once
#include "common.h"
#include "mx3.h"
#include "route_select.h"

namespace csk {

// ---------------------------------------------------------------- prologue
// One workgroup per row: RMSNorm (include/coalsack/nn/nn_ops/rmsnorm_node.h:62-83:
// rms = sqrt(sum x^2 / H + eps), out = (x / rms) * w), written as f32.
__global__ __launch_bounds__(256) void prep_kernel(const float* __restrict__ src,
                                                   const float* __restrict__ norm_w, float eps,
                                                   float* __restrict__ xn, int H) {
  const int row = blockIdx.x;
  const float* x = src + (size_t)row * H;
  float ss = 0.0f;
  for (int d = threadIdx.x; d < H; d += 256) ss += x[d] * x[d];
  ss = wave_sum(ss);
  __shared__ float part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const float den = sqrtf(ss / (float)H + eps);
  for (int d = threadIdx.x; d < H; d += 256) xn[(size_t)row * H + d] = (x[d] / den) * norm_w[d];
}

// ------------------------------------------------------------ router logits
// logits[t][e] = sum_d x[t][d] * g[e][d] + b[e]
// (include/coalsack/nn/nn_ops/moe_router_node.h:161-167).  One wave per
// (TT tokens, one expert): the gate row is read once per wave with 128-bit
// loads and reused for TT tokens; lanes own strided float4 chunks and the
// partial sums meet in a butterfly reduction.
template <int TT>
__global__ __launch_bounds__(256) void router_logits_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ g,
                                                            const float* __restrict__ b,
                                                            float* __restrict__ logits, int T,
                                                            int E, int H) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int t0 = blockIdx.y * TT;
  if (e >= E) return;
  const int H4 = H >> 2;
  const float4* g4 = reinterpret_cast<const float4*>(g + (size_t)e * H);
  float acc[TT];
#pragma unroll
  for (int i = 0; i < TT; ++i) acc[i] = 0.0f;
  for (int c = lane; c < H4; c += 64) {
    const float4 gv = g4[c];
#pragma unroll
    for (int i = 0; i < TT; ++i) {
      if (t0 + i < T) {
        const float4 xv = reinterpret_cast<const float4*>(x + (size_t)(t0 + i) * H)[c];
        acc[i] += xv.x * gv.x + xv.y * gv.y + xv.z * gv.z + xv.w * gv.w;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < TT; ++i) {
    const float s = wave_sum(acc[i]);
    if (lane == 0 && t0 + i < T) logits[(size_t)(t0 + i) * E + e] = s + (b ? b[e] : 0.0f);
  }
}

// ------------------------------------------------- router logits, many tokens
// The same logits as an fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32: fp32
// operands, fp32 accumulation, so nothing is rounded to a narrower type).  Workgroup
// (x, y) owns 32 tokens and split y of H (up to kRouterChunks chunks of 64): it loads its
// part of the 32 token rows into registers once and walks all the experts, 32 at a time,
// so the hidden states are read once however many experts there are, and the splits give
// a batch of a few thousand tokens enough workgroups to fill the chip.  Within a chunk the
// four waves take 16-wide slices; their partial tiles are added in LDS in a fixed order
// and written as partial logits [split][T][E], which the top-k kernel sums in split order
// and completes with the bias.  Operand ownership: lane l holds row l%32 (token, or
// expert) and k index l/32 of the two; each lane loads eight consecutive values of its
// row per chunk and feeds them to eight instructions -- any assignment of k to
// (instruction, lane half) is valid as long as both operands use the same one.
// H must be a multiple of 16.
constexpr int kRouterChunks = 12;     // chunks of 64 per split: the token rows of a split stay in registers
constexpr int kRouterMaxSplits = 8;

__global__ __launch_bounds__(256) void router_logits_mfma_kernel(const float* __restrict__ x,
                                                                 const float* __restrict__ g,
                                                                 float* __restrict__ partial, int T,
                                                                 int E, int H, int chunks_per_split) {
  __shared__ float part[4][32][33];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r32 = lane & 31, half = lane >> 5;
  const int t0 = blockIdx.x * 32;
  const int c0 = blockIdx.y * chunks_per_split;
  const int k_lane = 16 * wv + 8 * half;  // this lane's eight columns within a chunk
  const float* xr = x + (size_t)min(t0 + r32, T - 1) * H + k_lane;
  // the split's part of the token rows; columns past H are zeros (they then add nothing)
  floatx4 xa[kRouterChunks], xb[kRouterChunks];
#pragma unroll
  for (int i = 0; i < kRouterChunks; ++i) {
    const int k0 = 64 * (c0 + i);
    const bool in = i < chunks_per_split && k0 + k_lane + 8 <= H;
    xa[i] = in ? *reinterpret_cast<const floatx4*>(xr + k0) : floatx4{0.f, 0.f, 0.f, 0.f};
    xb[i] = in ? *reinterpret_cast<const floatx4*>(xr + k0 + 4) : floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // the last chunk this lane may load from the expert rows (clamped loads meet zeros above)
  const int c_last = max(0, (H - k_lane - 8) / 64);
  float* out = partial + (size_t)blockIdx.y * T * E;
  for (int e0 = 0; e0 < E; e0 += 32) {
    const float* gr = g + (size_t)min(e0 + r32, E - 1) * H + k_lane;
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    // expert rows: loads run two chunks ahead of the arithmetic (three rolling register sets)
    floatx4 ga[3], gb[3];
    auto load = [&](int u, int i) {
      const int k0 = 64 * min(c0 + i, c_last);
      ga[u] = *reinterpret_cast<const floatx4*>(gr + k0);
      gb[u] = *reinterpret_cast<const floatx4*>(gr + k0 + 4);
    };
    load(0, 0);
    load(1, 1);
#pragma unroll
    for (int i = 0; i < kRouterChunks; ++i) {
      if (i < chunks_per_split) {
        const int u = i % 3;
        load((u + 2) % 3, i + 2);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i][0], ga[u][0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i][1], ga[u][1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i][2], ga[u][2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i][3], ga[u][3], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xb[i][0], gb[u][0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xb[i][1], gb[u][1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xb[i][2], gb[u][2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xb[i][3], gb[u][3], acc, 0, 0, 0);
      }
    }
    // accumulator register r of lane (expert column r32, half) is token (r%4) + 8 (r/4) + 4 half
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wv][(r & 3) + 8 * (r >> 2) + 4 * half][r32] = acc[r];
    __syncthreads();
    for (int i = threadIdx.x; i < 32 * 32; i += 256) {
      const int tl = i >> 5, el = i & 31;
      if (t0 + tl < T && e0 + el < E)
        out[(size_t)(t0 + tl) * E + e0 + el] =
            (part[0][tl][el] + part[1][tl][el]) + (part[2][tl][el] + part[3][tl][el]);
    }
    __syncthreads();
  }
}

// --------------------------------------------- small batches: prologue + logits
// One launch for small T: workgroups x in [0, ceil(E / EPW)) compute the logits of EPW experts
// for the four tokens of tile y (the four waves split H, so all loads of a row are in flight
// at once; the token rows stay in registers across the experts); the next four workgroups
// run the prologue of one token of tile y each (RMSNorm, written as f32).  With
// RMSNorm the expert workgroups recompute each token's normalisation themselves -- 2 H flops
// per token -- instead of waiting for the prologue.  EPW = 1 spreads a handful of tokens
// over as many workgroups as there are experts (latency); EPW = 4 is for batches whose
// one-expert workgroups would not all be resident at once (64 tokens, 128 experts: 2112 of
// them, 18.6 us; a quarter as many read the token rows a quarter as often).
// Restates moe_router_node.h:161-167 and rmsnorm_node.h:62-83.
template <int EPW>
__global__ __launch_bounds__(256) void router_prep_logits_kernel(
    const float* __restrict__ hidden, const float* __restrict__ norm_w, float eps,
    float* __restrict__ xn, const float* __restrict__ g,
    const float* __restrict__ b, float* __restrict__ logits, int T, int E, int H,
    u32x4* __restrict__ x3) {
  __shared__ float part[4][4];
  __shared__ float dots[EPW][4][4];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n_ewg = (E + EPW - 1) / EPW;  // workgroups that compute logits
  if ((int)blockIdx.x >= n_ewg) {  // ---- prologue of token t (one of four per token tile)
    const int t = (blockIdx.x - n_ewg) + 4 * blockIdx.y;
    if (blockIdx.x - n_ewg >= 4 || t >= T || (!norm_w && !x3)) return;  // without a norm the rows are used as they are
    // four columns per thread, the row's loads all in flight at once and kept in registers
    // between the two passes (rows longer than 4096 take further rounds of the same)
    const float4* x4 = reinterpret_cast<const float4*>(hidden + (size_t)t * H);
    const float4* nw4 = reinterpret_cast<const float4*>(norm_w);
    const int H4p = H >> 2;
    constexpr int kIter = 4;
    const bool one_round = H4p <= 256 * kIter;  // the row and the norm weights are then read once, up front
    float4 x0[kIter], w0[kIter];
    if (one_round) {
#pragma unroll
      for (int j = 0; j < kIter; ++j) {
        const int c = threadIdx.x + 256 * j;
        x0[j] = c < H4p ? x4[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        w0[j] = (norm_w && c < H4p) ? nw4[c] : make_float4(1.f, 1.f, 1.f, 1.f);
      }
    }
    float den = 1.0f;
    if (norm_w) {
      float ss = 0.0f;
      for (int c0 = 0; c0 < H4p; c0 += 256 * kIter) {
        float4 xv[kIter];
#pragma unroll
        for (int j = 0; j < kIter; ++j) {
          const int c = c0 + threadIdx.x + 256 * j;
          xv[j] = one_round ? x0[j] : (c < H4p ? x4[c] : make_float4(0.f, 0.f, 0.f, 0.f));
        }
#pragma unroll
        for (int j = 0; j < kIter; ++j) ss += xv[j].x * xv[j].x + xv[j].y * xv[j].y + xv[j].z * xv[j].z + xv[j].w * xv[j].w;
      }
      ss = wave_sum(ss);
      if (lane == 0) part[wv][0] = ss;
      __syncthreads();
      ss = (part[0][0] + part[1][0]) + (part[2][0] + part[3][0]);
      den = sqrtf(ss / (float)H + eps);
    }
    for (int c0 = 0; c0 < H4p; c0 += 256 * kIter) {
      float4 xv[kIter], wv4[kIter];
#pragma unroll
      for (int j = 0; j < kIter; ++j) {
        const int c = c0 + threadIdx.x + 256 * j;
        if (one_round) {
          xv[j] = x0[j], wv4[j] = w0[j];
        } else if (c < H4p) {
          xv[j] = x4[c];
          if (norm_w) wv4[j] = nw4[c];
        }
      }
#pragma unroll
      for (int j = 0; j < kIter; ++j) {
        const int c = c0 + threadIdx.x + 256 * j;
        if (c < H4p) {
          float4 v = xv[j];
          if (norm_w) {
            v.x = (v.x / den) * wv4[j].x, v.y = (v.y / den) * wv4[j].y;
            v.z = (v.z / den) * wv4[j].z, v.w = (v.w / den) * wv4[j].w;
            reinterpret_cast<float4*>(xn + (size_t)t * H)[c] = v;
          }
        }
      }
    }
    if (x3) {
      // The row the experts will contract, as three FP6 terms (mx3.h), one thread per 32-value
      // block: the weight-streaming kernels copy it into LDS instead of each of their
      // workgroups quantising the rows of its token group again (a team of fifteen workgroups
      // used to do the same 1.4 us of vector arithmetic per block and thread fifteen times).
      // The values are formed from the inputs with the operations of the loop above, so they
      // are the bits of xn.  H is a multiple of 32 here.
      const int nblk = H >> 5, rowblk = mx3_row_blocks(nblk);
      for (int kb = threadIdx.x; kb < rowblk; kb += 256) {
        u32x4 out[kMx3ChunksPerBlock];
        if (kb >= nblk) {
#pragma unroll
          for (int tt = 0; tt < kMx3Terms; ++tt) {
            out[2 * tt] = u32x4{0u, 0u, 0u, 0u};
            out[2 * tt + 1] = u32x4{0u, 0u, 127u, 0u};
          }
        } else {
          float r[32];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            float4 v = x4[kb * 8 + i];
            if (norm_w) {
              const float4 w = nw4[kb * 8 + i];
              v.x = (v.x / den) * w.x, v.y = (v.y / den) * w.y, v.z = (v.z / den) * w.z, v.w = (v.w / den) * w.w;
            }
            r[4 * i] = v.x, r[4 * i + 1] = v.y, r[4 * i + 2] = v.z, r[4 * i + 3] = v.w;
          }
          mx3_quantize_block(r, out);
        }
        u32x4* dst = x3 + ((size_t)t * rowblk + kb) * kMx3ChunksPerBlock;
#pragma unroll
        for (int c = 0; c < kMx3ChunksPerBlock; ++c) dst[c] = out[c];
      }
    }
    return;
  }
  // ---- logits of experts e0 .. e0 + EPW - 1 for four tokens (token tile blockIdx.y)
  const int e0 = blockIdx.x * EPW;
  const int H4 = H >> 2;
  const float4* w4 = reinterpret_cast<const float4*>(norm_w);
  const int t0 = blockIdx.y * 4;
  const int nt = min(4, T - t0);  // tokens of this tile (the same in every thread)
  // this thread's part of the token rows stays in registers between the passes
  constexpr int kMaxIter = 4;     // 256 threads x 4 float4 x 4 = H up to 4096; longer rows are read again
  float4 xr[4][kMaxIter];
  const bool held = H4 <= 256 * kMaxIter;
  if (held) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < nt) {
#pragma unroll
        for (int j = 0; j < kMaxIter; ++j) {
          const int c = threadIdx.x + 256 * j;
          xr[i][j] = c < H4 ? reinterpret_cast<const float4*>(hidden + (size_t)(t0 + i) * H)[c]
                            : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
  }
  auto row = [&](int i, int c) -> float4 {
    return reinterpret_cast<const float4*>(hidden + (size_t)(t0 + i) * H)[c];
  };
  // the norm weights and the first expert's gate row are requested now, beside the token
  // rows, not after the reductions that need only the rows
  float4 wq[kMaxIter], gq[2][kMaxIter];
  auto load_gate = [&](float4(&q)[kMaxIter], int ee) {
    const float4* g4 = reinterpret_cast<const float4*>(g + (size_t)min(e0 + ee, E - 1) * H);
#pragma unroll
    for (int j = 0; j < kMaxIter; ++j) {
      const int c = threadIdx.x + 256 * j;
      q[j] = c < H4 ? g4[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  if (held) {
    load_gate(gq[0], 0);
    if (norm_w) {
#pragma unroll
      for (int j = 0; j < kMaxIter; ++j) {
        const int c = threadIdx.x + 256 * j;
        wq[j] = c < H4 ? w4[c] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  }
  // 1 / rms per token: the logits only have to be within the close-call tolerance of the
  // reference's (a token inside it is recomputed from the exactly normalised row the
  // prologue workgroups write), so the rows are scaled by a reciprocal here, one
  // multiplication per element where the exact form is a correctly rounded division; the
  // difference, 1 ulp per element, moves a logit by about a hundredth of the tolerance's unit
  float inv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
  if (norm_w) {
    float ss[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < nt) {
        if (held) {
#pragma unroll
          for (int j = 0; j < kMaxIter; ++j) {
            const float4 xv = xr[i][j];  // chunks past H are zeros
            ss[i] += xv.x * xv.x + xv.y * xv.y + xv.z * xv.z + xv.w * xv.w;
          }
        } else {
          for (int c = threadIdx.x; c < H4; c += 256) {
            const float4 xv = row(i, c);
            ss[i] += xv.x * xv.x + xv.y * xv.y + xv.z * xv.z + xv.w * xv.w;
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float sum = wave_sum(ss[i]);
      if (lane == 0) part[wv][i] = sum;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i)
      inv[i] = 1.0f / sqrtf(((part[0][i] + part[1][i]) + (part[2][i] + part[3][i])) / (float)H + eps);
    if (held) {  // normalise the held rows once, for all the experts of this workgroup
#pragma unroll
      for (int j = 0; j < kMaxIter; ++j) {
        const int c = threadIdx.x + 256 * j;
        if (c < H4) {
          const float4 wv4 = wq[j];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (i < nt) {
              xr[i][j].x = (xr[i][j].x * inv[i]) * wv4.x;
              xr[i][j].y = (xr[i][j].y * inv[i]) * wv4.y;
              xr[i][j].z = (xr[i][j].z * inv[i]) * wv4.z;
              xr[i][j].w = (xr[i][j].w * inv[i]) * wv4.w;
            }
          }
        }
      }
    }
  }
  // the gate row of the next expert is requested before the current one is used
#pragma unroll
  for (int ee = 0; ee < EPW; ++ee) {
    const int e = min(e0 + ee, E - 1);  // a workgroup past the last expert repeats it; nothing is stored
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (held) {
      if (ee + 1 < EPW) load_gate(gq[(ee + 1) & 1], ee + 1);
#pragma unroll
      for (int j = 0; j < kMaxIter; ++j) {
        const float4 gv = gq[ee & 1][j];  // chunks past H are zeros on both sides
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (i < nt) {
            const float4 xv = xr[i][j];
            acc[i] += xv.x * gv.x + xv.y * gv.y + xv.z * gv.z + xv.w * gv.w;
          }
        }
      }
    } else {
      const float4* g4 = reinterpret_cast<const float4*>(g + (size_t)e * H);
      for (int c = threadIdx.x; c < H4; c += 256) {
        const float4 gv = g4[c];
        float4 wv4 = make_float4(1.f, 1.f, 1.f, 1.f);
        if (norm_w) wv4 = w4[c];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (i < nt) {
            float4 xv = row(i, c);
            if (norm_w) {
              xv.x = (xv.x * inv[i]) * wv4.x;
              xv.y = (xv.y * inv[i]) * wv4.y;
              xv.z = (xv.z * inv[i]) * wv4.z;
              xv.w = (xv.w * inv[i]) * wv4.w;
            }
            acc[i] += xv.x * gv.x + xv.y * gv.y + xv.z * gv.z + xv.w * gv.w;
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float sum = wave_sum(acc[i]);
      if (lane == 0) dots[ee][wv][i] = sum;
    }
  }
  __syncthreads();
  if (threadIdx.x < 4 * EPW) {
    const int ee = threadIdx.x >> 2, i = threadIdx.x & 3, e = e0 + ee;
    if (e < E && i < nt)
      logits[(size_t)(t0 + i) * E + e] =
          ((dots[ee][0][i] + dots[ee][1][i]) + (dots[ee][2][i] + dots[ee][3][i])) + (b ? b[e] : 0.0f);
  }
}

// ------------------------------------------------------------------- top-k
// One wave per token (select_topk).  Weights
// follow moe_router_node.h:180-202: sigmoid of the raw logit, or softmax over
// the selected k with max subtraction, sum in slot order, multiply by 1/sum.
__global__ __launch_bounds__(256) void router_topk_kernel(float* __restrict__ logits,
                                                          float* __restrict__ pairs,
                                                          int* __restrict__ ids, int T, int E,
                                                          int k, int sigmoid,
                                                          const float* __restrict__ x,
                                                          const float* __restrict__ g,
                                                          const float* __restrict__ b, int H,
                                                          const float* __restrict__ partial,
                                                          int nsplit, Mx3Rider rider) {
  __shared__ CloseCallLds cc;
  __shared__ float cc_thr[4];
  __shared__ int cc_flag[4];
  // Riders: workgroups past the tokens' rewrite the activation rows as FP6 terms for the
  // grouped GEMM.  The two jobs share only their input; a token with a close call keeps
  // one workgroup of this kernel busy for a chain of H dependent additions, during which
  // the rest of the chip would have nothing to do.
  if (rider.x3 && (int)blockIdx.x >= rider.first_wg) {
    mx3_rows_block((long)(blockIdx.x - rider.first_wg) * 256 + threadIdx.x, rider.x, rider.x3, rider.rows, rider.nblk,
                   nullptr, nullptr);
    return;
  }
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wv;
  const bool live = t < T;  // waves past the end stay for the barriers below
  const float NEG = -__builtin_inff();
  float v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e = lane + 64 * j;
    v[j] = NEG;
    if (live && e < E) {
      if (nsplit > 0) {
        // partial logits of the splits of H, in split order, then the bias; the sum is kept
        // for the recomputation below and for callers that ask for the logits
        float sum = partial[(size_t)t * E + e];
        for (int sp = 1; sp < nsplit; ++sp) sum += partial[((size_t)sp * T + t) * E + e];
        v[j] = sum + (b ? b[e] : 0.0f);
        logits[(size_t)t * E + e] = v[j];
      } else {
        v[j] = logits[(size_t)t * E + e];
      }
    }
  }
  float my_val, vmax, runner_up;  // lane s keeps slot s
  int my_idx;
  bool close_call;
  const float tol = close_call_tolerance(H);
  select_topk(v, lane, E, k, my_val, my_idx, vmax, close_call, tol, runner_up);
  close_call = close_call && live;
  if (lane == 0) {
    cc_flag[wv] = close_call;
    cc_thr[wv] = runner_up - 2.0f * tol * fmaxf(1.0f, fabsf(runner_up));
  }
  if (__syncthreads_or(close_call)) {
    // rare: some token of this workgroup has a close call among its k+1 largest logits;
    // the four waves recompute it together, its own wave selects again
    for (int w = 0; w < 4; ++w) {
      if (!cc_flag[w]) continue;
      const int tw = blockIdx.x * 4 + w;
      logits_reference_order_wg<256>(x + (size_t)tw * H, g, b, logits + (size_t)tw * E, E, H,
                                     cc_thr[w], cc);
      if (wv == w) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = lane + 64 * j;
          v[j] = e < E ? cc.fixed[e] : NEG;
        }
        select_topk(v, lane, E, k, my_val, my_idx, vmax, close_call, 0.0f, runner_up);
      }
      __syncthreads();
    }
  }
  if (!live) return;
  const float w = routing_weight(my_val, vmax, lane, k, sigmoid);
  if (lane < k) {
    float2* o = reinterpret_cast<float2*>(pairs) + (size_t)t * k + lane;
    *o = make_float2((float)my_idx, w);
    ids[(size_t)t * k + lane] = my_idx;
  }
}

// Expert ids from an existing router output (node-level expert / merge calls):
// static_cast<int>(float) as expert_mlp_node.h:788 does.
__global__ void pairs_to_ids_kernel(const float* __restrict__ pairs, int* __restrict__ ids, int P) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p < P) ids[p] = (int)pairs[2 * (size_t)p];
}

// ----------------------------------------------------------------- dispatch
// Workgroup c places the 1024 assignments [1024 c, 1024 c + 1024).  It counts, with LDS
// atomics over all P expert ids (they are L2-resident; every workgroup does this, which
// saves a launch and any global atomics), how many assignments name each expert in total
// and how many of them lie before its own chunk; inside the chunk the lanes of a wave
// that name the same expert find one another by ballots, and a prefix over the sixteen
// waves completes the rank.  An assignment's place is offset(expert) + before + rank: each
// expert's list is ascending in token index -- the order the reference's per-expert token
// loop visits them (expert_mlp_node.h:503-529).  Ids below zero (assignments that do not
// name the one expert of a node-level call) are skipped.  Workgroup 0 also publishes
// counts, offsets[0..E], the work descriptors of the experts with at least one token
// (moe_weight_fetch_node.h:31-60), the streaming kernel's token groups and the GEMM's M
// tiles.
constexpr int kDispatchThreads = 1024;
__global__ __launch_bounds__(kDispatchThreads) void dispatch_scatter_kernel(
    const int* __restrict__ ids, const float* __restrict__ pairs, int P, int k, int E,
    int* __restrict__ counts, const ExpertW* __restrict__ ew, int* __restrict__ offsets,
    WorkDesc* __restrict__ desc, StreamGroup* __restrict__ groups, int* __restrict__ nv,
    int* __restrict__ mtiles, int* __restrict__ n_mtiles, int* __restrict__ list_tok,
    float* __restrict__ list_w, int* __restrict__ pos_of_slot, int group_tokens) {
  constexpr int NW = kDispatchThreads / 64;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const bool pub = blockIdx.x == 0;
  const int chunk0 = blockIdx.x * kDispatchThreads;
  __shared__ int cnt[kMaxExperts], before[kMaxExperts], off_sh[kMaxExperts], act_e[kMaxExperts];
  __shared__ int wcnt[NW][kMaxExperts];
  __shared__ int na_sh;
  if (tid < kMaxExperts) cnt[tid] = 0, before[tid] = 0;
  for (int i = tid; i < NW * kMaxExperts; i += kDispatchThreads) (&wcnt[0][0])[i] = 0;
  __syncthreads();
  for (int p0 = 0; p0 < P; p0 += kDispatchThreads * 4) {  // four loads in flight per thread
    int id[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p = p0 + kDispatchThreads * j + tid;
      id[j] = p < P ? ids[p] : -1;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (id[j] >= 0) {
        atomicAdd(&cnt[id[j]], 1);
        if (p0 + kDispatchThreads * j + tid < chunk0) atomicAdd(&before[id[j]], 1);
      }
    }
  }
  __syncthreads();
  // exclusive scan over the experts, active experts, token groups, M tiles: wave 0, four
  // consecutive experts per lane, wave-wide prefix sums; every workgroup needs the offsets,
  // workgroup 0 writes the results out
  if (wv == 0) {
    int cc[4], tot = 0, nact = 0, ngrp = 0, nmt = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ee = lane * 4 + j;
      cc[j] = ee < E ? cnt[ee] : 0;
      tot += cc[j];
      nact += cc[j] > 0;
      ngrp += group_count(cc[j], group_tokens);
      nmt += (cc[j] + 63) / 64;
    }
    int s_tot = tot, s_act = nact, s_grp = ngrp, s_mt = nmt;  // inclusive scans over lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t0 = __shfl_up(s_tot, o, 64), t1 = __shfl_up(s_act, o, 64);
      const int t2 = __shfl_up(s_grp, o, 64), t3 = __shfl_up(s_mt, o, 64);
      if (lane >= o) {
        s_tot += t0;
        s_act += t1;
        s_grp += t2;
        s_mt += t3;
      }
    }
    int run = s_tot - tot, slot = s_act - nact, gi = s_grp - ngrp, mi = s_mt - nmt;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ee = lane * 4 + j;
      if (ee < E) {
        off_sh[ee] = run;
        if (pub) offsets[ee] = run;
        if (cc[j] > 0) {
          if (pub) {
            if (groups) {
              for (int gb = 0; gb < cc[j]; gb += group_tokens) {
                write_stream_group(groups + gi, ew + ee, ee, cc[j] - gb, run + gb);
                ++gi;
              }
            }
            for (int m0 = 0; m0 < cc[j]; m0 += 64) {
              mtiles[2 * mi] = slot;
              mtiles[2 * mi + 1] = m0;
              ++mi;
            }
          }
          act_e[slot++] = ee;
        }
        run += cc[j];
      }
    }
    if (lane == 63) {
      na_sh = s_act;
      if (pub) {
        offsets[E] = s_tot;
        *nv = groups ? s_grp : 0;
        *n_mtiles = s_mt;
      }
    }
  }
  // this chunk: lanes of a wave that name the same expert, their rank among themselves
  const int my_p = chunk0 + tid;
  const int my_id = my_p < P ? ids[my_p] : -1;
  unsigned long long same = 0ull, todo = __ballot(my_id >= 0);
  while (todo != 0ull) {  // the same in every lane
    const int id0 = __builtin_amdgcn_readlane(my_id, (int)__builtin_ctzll(todo));
    const unsigned long long m = __ballot(my_id == id0);
    if (my_id == id0) same = m;
    todo &= ~m;
  }
  const int rank_in_wave = __popcll(same & ((1ull << lane) - 1ull));
  if (my_id >= 0 && rank_in_wave == 0) wcnt[wv][my_id] = __popcll(same);
  __syncthreads();
  if (pub && tid < E) {
    counts[tid] = cnt[tid];
    const bool on = tid < na_sh;
    const int e = on ? act_e[tid] : 0;
    write_work_desc(desc + tid, on, e, cnt[e], off_sh[e], ew);
  }
  if (tid < E) {  // per expert: how many of the chunk's assignments sit in the waves before
    int run = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const int v = wcnt[w][tid];
      wcnt[w][tid] = run;
      run += v;
    }
  }
  __syncthreads();
  if (my_id >= 0) {
    const int pos = off_sh[my_id] + before[my_id] + wcnt[wv][my_id] + rank_in_wave;
    list_tok[pos] = my_p / k;
    list_w[pos] = pairs[2 * (size_t)my_p + 1];
    pos_of_slot[my_p] = pos;
  }
}

// ------------------------------------- small batches: top-k + dispatch, one launch
// A single workgroup of sixteen waves routes the batch (route_workgroup) and writes every
// output.
constexpr int kRouteSmallThreads = 1024;
constexpr int kRouteSmallMaxP = 1024;
__global__ __launch_bounds__(kRouteSmallThreads) void route_small_kernel(RouteIn in, RouteOut out) {
  __shared__ RouteLds<kCcBatch, kRouteSmallMaxP> lds;
  route_workgroup<kRouteSmallThreads, kCcBatch, kRouteSmallMaxP>(in, out, lds);
}

// ------------------------- up to four tokens: top-k + dispatch, one wave per token
// Four tokens name at most 4 k <= 64 assignments.  Wave t selects the experts of token t
// (select_topk, close calls recomputed by the four waves together, as router_topk_kernel
// does); then lane p of wave 0 places assignment p by counting, across the wave, the
// assignments that come before it: those of experts with a lower index, and those of its own
// expert from earlier tokens -- an expert's list stays ascending in token index, the order of
// the reference's per-expert token loop (expert_mlp_node.h:503-529).  No histogram and no
// scan, two barriers.  No expert has more than four tokens, so each active expert is one
// token group of the weight-streaming kernels.  Writes what those kernels, the combine and
// csk_layer_last_dispatch read: pairs, ids, positions, the lists, counts, the token groups
// and their number; the grouped GEMM's descriptors and tiles are not written.
constexpr int kRouteTinyTokens = 4;
constexpr int kRouteTinyMaxP = 64;
__global__ __launch_bounds__(256) void route_tiny_kernel(RouteIn r, RouteOut o) {
  __shared__ CloseCallLds cc;
  __shared__ float cc_thr[4];
  __shared__ int cc_flag[4];
  __shared__ int s_ids[kRouteTinyMaxP];
  __shared__ float s_w[kRouteTinyMaxP];
  constexpr int kEwWords = kMaxExperts * (int)(sizeof(ExpertW) / 8), kEwPerThread = (kEwWords + 255) / 256;
  __shared__ unsigned long long s_ew[kEwWords];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int T = r.T, E = r.E, k = r.k, P = T * k;
  const int t = wv;
  const bool live = t < T;  // waves past the last token stay for the barriers
  const float NEG = -__builtin_inff();
  // the table of weight pointers is needed last (token groups); its load runs beside that of the logits
  unsigned long long ew_reg[kEwPerThread];
#pragma unroll
  for (int i = 0; i < kEwPerThread; ++i) {
    const int w = threadIdx.x + i * 256;
    ew_reg[i] = w < E * (int)(sizeof(ExpertW) / 8) ? reinterpret_cast<const unsigned long long*>(r.ew)[w] : 0ull;
  }
  float v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e = lane + 64 * j;
    v[j] = (live && e < E) ? r.logits[(size_t)t * E + e] : NEG;
  }
  float my_val, vmax, runner_up;  // lane s keeps slot s
  int my_idx;
  bool close_call;
  const float tol = close_call_tolerance(r.H);
  select_topk(v, lane, E, k, my_val, my_idx, vmax, close_call, tol, runner_up);
  close_call = close_call && live;
  if (lane == 0) {
    cc_flag[wv] = close_call;
    cc_thr[wv] = runner_up - 2.0f * tol * fmaxf(1.0f, fabsf(runner_up));
  }
#pragma unroll
  for (int i = 0; i < kEwPerThread; ++i) {
    const int w = threadIdx.x + i * 256;
    if (w < kEwWords) s_ew[w] = ew_reg[i];
  }
  if (__syncthreads_or(close_call)) {
    for (int w = 0; w < 4; ++w) {
      if (!cc_flag[w]) continue;
      logits_reference_order_wg<256>(r.x + (size_t)w * r.H, r.g, r.b, r.logits + (size_t)w * E, E, r.H,
                                     cc_thr[w], cc);
      if (wv == w) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = lane + 64 * j;
          v[j] = e < E ? cc.fixed[e] : NEG;
        }
        select_topk(v, lane, E, k, my_val, my_idx, vmax, close_call, 0.0f, runner_up);
      }
      __syncthreads();
    }
  }
  if (live) {
    const float w = routing_weight(my_val, vmax, lane, k, r.sigmoid);
    if (lane < k) {
      reinterpret_cast<float2*>(o.pairs)[(size_t)t * k + lane] = make_float2((float)my_idx, w);
      o.ids[t * k + lane] = my_idx;
      s_ids[t * k + lane] = my_idx;
      s_w[t * k + lane] = w;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) {
    int c = 0;
    for (int q = 0; q < P; ++q) c += s_ids[q] == e;
    o.counts[e] = c;
  }
  if (wv != 0) return;
  const bool lp = lane < P;
  const int my = lp ? s_ids[lane] : 0x7fffffff;
  int lower = 0, same_before = 0, same = 0;
  for (int q = 0; q < P; ++q) {  // q is the same in every lane
    const int idq = __builtin_amdgcn_readlane(my, q);
    lower += idq < my;
    same += idq == my;
    same_before += (idq == my) && q < lane;
  }
  const bool first = lp && same_before == 0;  // the expert's first assignment stands for its token group
  const unsigned long long firsts = __ballot(first);
  int groups_before = 0;
  for (unsigned long long m = firsts; m != 0ull; m &= m - 1ull) {
    const int idq = __builtin_amdgcn_readlane(my, (int)__builtin_ctzll(m));
    groups_before += idq < my;
  }
  if (lp) {
    const int pos = lower + same_before;
    const unsigned inv_k = (65536u + (unsigned)k - 1u) / (unsigned)k;  // p / k == p * inv_k >> 16 for p < 64, k <= 16
    o.list_tok[pos] = (int)(((unsigned)lane * inv_k) >> 16);
    o.list_w[pos] = s_w[lane];
    o.pos_of_slot[lane] = pos;
    if (first) write_stream_group(o.groups + groups_before, reinterpret_cast<const ExpertW*>(s_ew) + my, my, same, pos);
  }
  if (lane == 0) *o.nv = __popcll(firsts);
}

// ------------------------------------------------------------------ combine
// out[t] = sum over slots in router order of w * y[pos(t, slot)]
// (include/coalsack/nn/nn_ops/expert_merge_node.h:97-128), multiply and add
// rounded separately as the reference's scalar loop does; no atomics, one
// thread owns one output element.  residual != null adds the layer input
// (add_node.h:8-55).
__global__ __launch_bounds__(256) void combine_kernel(const float* __restrict__ y,
                                                      const float* __restrict__ pairs,
                                                      const int* __restrict__ pos_of_slot,
                                                      const float* __restrict__ residual,
                                                      float* __restrict__ out, int T, int k, int H,
                                                      int pre_weighted) {
#pragma clang fp contract(off)  // w * y and the add round separately, as in the reference
  const int t = blockIdx.y;
  const int d = (blockIdx.x * 256 + threadIdx.x) * 4;  // four adjacent columns per thread (H % 32 == 0)
  if (d >= H) return;
  float4 res = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (residual) res = *reinterpret_cast<const float4*>(residual + (size_t)t * H + d);  // requested first, used last
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  // four slots at a time: their positions and weights are requested together, then their
  // rows, so that a token's k rows cost two memory latencies, not 2 k; the sums stay in
  // slot order
  for (int s0 = 0; s0 < k; s0 += 4) {
    int pos[4];
    float w[4];
    float4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = min(s0 + j, k - 1);
      pos[j] = s0 + j < k ? pos_of_slot[(size_t)t * k + s] : -1;
      w[j] = pre_weighted ? 1.0f : pairs[2 * ((size_t)t * k + s) + 1];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      v[j] = pos[j] >= 0 ? *reinterpret_cast<const float4*>(y + (size_t)pos[j] * H + d) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (pos[j] < 0) continue;  // empty expert tensor: skipped (expert_merge_node.h:111-113)
      if (pre_weighted) {
        acc.x = acc.x + v[j].x, acc.y = acc.y + v[j].y, acc.z = acc.z + v[j].z, acc.w = acc.w + v[j].w;
      } else {
        const float4 wv = make_float4(w[j] * v[j].x, w[j] * v[j].y, w[j] * v[j].z, w[j] * v[j].w);
        acc.x = acc.x + wv.x, acc.y = acc.y + wv.y, acc.z = acc.z + wv.z, acc.w = acc.w + wv.w;
      }
    }
  }
  if (residual) acc.x = res.x + acc.x, acc.y = res.y + acc.y, acc.z = res.z + acc.z, acc.w = res.w + acc.w;
  *reinterpret_cast<float4*>(out + (size_t)t * H + d) = acc;
}

// Dense per-expert output of the node-level call (expert_mlp_node.h:503-529):
// row t = y[pos] if token t selected the expert, else zeros.
__global__ __launch_bounds__(256) void expand_expert_rows_kernel(const float* __restrict__ y,
                                                                 const int* __restrict__ ids,
                                                                 const int* __restrict__ pos_of_slot,
                                                                 float* __restrict__ out, int k,
                                                                 int H, int expert_id) {
  const int t = blockIdx.y;
  const int d = blockIdx.x * 256 + threadIdx.x;
  if (d >= H) return;
  int pos = -1;
  for (int s = 0; s < k; ++s) {
    if (ids[(size_t)t * k + s] == expert_id) {
      pos = pos_of_slot[(size_t)t * k + s];
      break;  // first matching slot, as is_token_selecting_expert / get_router_weight
    }
  }
  out[(size_t)t * H + d] = (pos >= 0) ? y[(size_t)pos * H + d] : 0.0f;
}

}  // namespace csk
