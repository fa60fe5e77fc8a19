// Expert MLP for the weight-streaming (decode) regime.
//
// Each workgroup owns one 16-row tile of one active expert's matrix (gate and
// up together, or down) and streams it from HBM exactly once: 64 lanes x 16
// bytes = 1 KiB of contiguous nibbles per matrix per step, the four waves
// taking interleaved K steps.  MXFP4 is expanded in registers by
// v_cvt_scalef32_pk_bf16_fp4 (exact: an E2M1 value times a power of two always
// fits bf16) and contracted on the matrix cores against up to 16*MT tokens of
// that expert.  Activations arrive as two bf16 terms (hi + lo, 16 mantissa
// bits) so the products are those of the reference's fp32 x exactly-dequantised
// weight to within 2^-17; accumulation is fp32.
//
// Restates include/coalsack/nn/nn_ops/expert_mlp_node.h:651-732
// (compute_token_mxfp4): gate/up projections + bias, activation (:699-706),
// down projection + bias; the token loop of :503-529 becomes the M dimension.
#pragma once
#include "common.h"

namespace csk {

struct ExpertStreamArgs {
  const ExpertW* ew;
  const int* active;     // compact list of experts with tokens
  const int* n_active;
  const int* counts;     // [E]
  const int* offsets;    // [E+1] packed position of each expert's first token
  const int* list_row;   // packed position -> row of A; null: row = packed position
  const uint4* A;        // [rows][nblk][8] x 16 B: 32 bf16 hi then 32 bf16 lo per block
  int nblk;              // K / 32
  int N;                 // output features (F for gate/up, H for down)
  int act_type;
  uint16_t* act_out;     // gate/up: [P][N/32][64] bf16 hi|lo
  float* y_out;          // down: [P][N] f32
};

__device__ __forceinline__ float moe_activation(float gate_v, float up_v, int act_type) {
  if (act_type == 0) {  // expert_mlp_node.h:699-703
    const float x = fminf(gate_v, 7.0f);
    const float y = fminf(fmaxf(up_v, -7.0f), 7.0f);
    const float glu = x / (1.0f + expf(1.702f * (-x)));
    return glu * (y + 1.0f);
  }
  const float silu = gate_v / (1.0f + expf(-gate_v));  // :705-706
  return silu * up_v;
}

__device__ __forceinline__ bf16x8 cvt_fp4x8(uint32_t w, float sc) {
  const bf16x2 r0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 0);
  const bf16x2 r1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 1);
  const bf16x2 r2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 2);
  const bf16x2 r3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 3);
  bf16x8 b;
  b[0] = r0[0];
  b[1] = r0[1];
  b[2] = r1[0];
  b[3] = r1[1];
  b[4] = r2[0];
  b[5] = r2[1];
  b[6] = r3[0];
  b[7] = r3[1];
  return b;
}

union U4B8 {
  uint4 u;
  bf16x8 b;
};

// NMAT = 2: gate and up tiles together, SwiGLU epilogue.  NMAT = 1: down.
// MT = number of 16-token M tiles kept live per pass over the weights.
template <int NMAT, int MT>
__global__ __launch_bounds__(256) void expert_stream_kernel(ExpertStreamArgs a) {
  const int u = blockIdx.y;
  if (u >= *a.n_active) return;
  const int e = a.active[u];
  const int Te = a.counts[e];
  const int base = a.offsets[e];
  const ExpertW w = a.ew[e];
  const int R = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int nblk = a.nblk;
  const size_t tile0 = (size_t)R * nblk * 16;
  const uint4* q0 = (NMAT == 2 ? w.q_gate : w.q_down) + tile0;
  const uint8_t* s0 = (NMAT == 2 ? w.s_gate : w.s_down) + tile0;
  const uint4* q1 = w.q_up + tile0;
  const uint8_t* s1 = w.s_up + tile0;
  const int nsteps = (nblk + 3) >> 2;

  __shared__ float red[3][MT * NMAT * 4][64];

  for (int mbase = 0; mbase < Te; mbase += 16 * MT) {
    floatx4 acc[MT][NMAT];
    size_t arow[MT];
    bool av[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int m = 0; m < NMAT; ++m) acc[mt][m] = floatx4{0.f, 0.f, 0.f, 0.f};
      const int idx = mbase + mt * 16 + n;
      av[mt] = idx < Te;
      const int row = av[mt] ? (a.list_row ? a.list_row[base + idx] : base + idx) : 0;
      arow[mt] = (size_t)row * nblk * 8;
    }
    const int mlive = min(MT, (Te - mbase + 15) >> 4);  // wave-uniform

    for (int j = wv; j < nsteps; j += 4) {
      const int kb = 4 * j + g;
      const bool kv = kb < nblk;
      uint4 qa = make_uint4(0, 0, 0, 0), qb = make_uint4(0, 0, 0, 0);
      float sa = 0.0f, sb = 0.0f;
      if (kv) {
        qa = q0[kb * 16 + n];
        sa = e8m0_scale(s0[kb * 16 + n]);
        if (NMAT == 2) {
          qb = q1[kb * 16 + n];
          sb = e8m0_scale(s1[kb * 16 + n]);
        }
      }
      U4B8 ah[MT][4], al[MT][4];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < mlive) {
          if (kv && av[mt]) {
            const uint4* ap = a.A + arow[mt] + (size_t)kb * 8;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              ah[mt][i].u = ap[i];
              al[mt][i].u = ap[4 + i];
            }
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              ah[mt][i].u = make_uint4(0, 0, 0, 0);
              al[mt][i].u = make_uint4(0, 0, 0, 0);
            }
          }
        }
      }
      const uint32_t qaw[4] = {qa.x, qa.y, qa.z, qa.w};
      const uint32_t qbw[4] = {qb.x, qb.y, qb.z, qb.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bf16x8 b0 = cvt_fp4x8(qaw[i], sa);
        bf16x8 b1;
        if (NMAT == 2) b1 = cvt_fp4x8(qbw[i], sb);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          if (mt < mlive) {
            acc[mt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[mt][i].b, b0, acc[mt][0], 0, 0, 0);
            acc[mt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[mt][i].b, b0, acc[mt][0], 0, 0, 0);
            if (NMAT == 2) {
              acc[mt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[mt][i].b, b1, acc[mt][1], 0, 0, 0);
              acc[mt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[mt][i].b, b1, acc[mt][1], 0, 0, 0);
            }
          }
        }
      }
    }

    // Sum the four waves' K slices (fixed order: wave 0 + 1 + 2 + 3).
    if (wv > 0) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
          for (int i = 0; i < 4; ++i) red[wv - 1][(mt * NMAT + m) * 4 + i][lane] = acc[mt][m][i];
    }
    __syncthreads();
    if (wv == 0) {
      const int r = R * 16 + n;  // output feature
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < mlive) {
#pragma unroll
          for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int o = (mt * NMAT + m) * 4 + i;
              acc[mt][m][i] = ((acc[mt][m][i] + red[0][o][lane]) + red[1][o][lane]) + red[2][o][lane];
            }
          if (r < a.N) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int idx = mbase + mt * 16 + g * 4 + i;  // token within this expert
              if (idx < Te) {
                const size_t p = (size_t)(base + idx);
                if (NMAT == 2) {
                  const float gate_v = acc[mt][0][i] + (w.b_gate ? w.b_gate[r] : 0.0f);
                  const float up_v = acc[mt][1][i] + (w.b_up ? w.b_up[r] : 0.0f);
                  uint16_t hi, lo;
                  split_bf16(moe_activation(gate_v, up_v, a.act_type), hi, lo);
                  uint16_t* o = a.act_out + (p * (size_t)(a.N >> 5) + (r >> 5)) * 64 + (r & 31);
                  o[0] = hi;
                  o[32] = lo;
                } else {
                  a.y_out[p * (size_t)a.N + r] = acc[mt][0][i] + (w.b_down ? w.b_down[r] : 0.0f);
                }
              }
            }
          }
        }
      }
    }
    __syncthreads();
  }
}

}  // namespace csk
