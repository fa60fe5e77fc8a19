// Expert MLP for the weight-streaming (decode) regime.
//
// Every active expert's matrices are streamed from HBM once per group of up to
// four of its tokens: 64 lanes x 16 bytes = 1 KiB of contiguous nibbles per
// 16-row tile per K step, the four waves of a workgroup taking interleaved K
// steps (128 elements each).  MXFP4 is expanded in registers by
// v_cvt_scalef32_pk_bf16_fp4 (exact: an E2M1 value times a power of two always
// fits bf16) and contracted on the matrix cores.  Activations arrive as two
// bf16 terms (hi + lo, 16 mantissa bits), so each product is that of the
// reference's fp32 activation and exactly dequantised weight to within 2^-17;
// accumulation is fp32.  The K slices of the four waves meet in LDS in a fixed
// order.
//
// Restates include/coalsack/nn/nn_ops/expert_mlp_node.h:651-732
// (compute_token_mxfp4): gate/up projections + bias, activation (:699-706),
// down projection + bias; the token loop of :503-529 becomes the M dimension.
#pragma once
#include "common.h"

namespace csk {

// Bias pointers inside desc[].w must not be null for expert_stream_kernel: the
// host substitutes a zero vector for an absent bias, so that the loads are
// unconditional.
struct ExpertStreamArgs {
  const WorkDesc* desc;
  const StreamGroup* groups;  // [nv]: the groups of up to G tokens
  const int* nv;         // number of such groups
  const int* list_row;   // packed position -> row of A; null: row = packed position
  const uint4* A;        // [rows][nblk][8] x 16 B: 32 bf16 hi then 32 bf16 lo per block
  int nblk;              // K / 32
  int ntile;             // ceil(N / 16)
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

__device__ __forceinline__ uint32_t u4_word(const uint4& v, int i) {
  return i == 0 ? v.x : (i == 1 ? v.y : (i == 2 ? v.z : v.w));
}

// ---------------------------------------------------------------------------
// Persistent, software-pipelined kernel (K <= 3072).
//
// MODE 0: a work unit is the pair (gate tile R, up tile R), SwiGLU epilogue.
// MODE 1: a work unit is the pair of down tiles (2R, 2R+1).
// G = tokens contracted per pass (rows 0..G-1 of the 16-row MFMA tile).
//
// The work is (token group of an expert) x (tile pair): every group costs the
// same, so teams of gridDim.x / groups workgroups take one group each and
// interleave its units, and the load is balanced whatever the routing was.
// Memory-level parallelism bounds this kernel, so it never lets the memory
// queue drain: a group's activation rows are copied once into LDS
// (global_load_lds, no registers), and the weight registers are refilled step
// by step as the matrix cores consume them: the loads of unit t+1 -- issued
// unconditionally from clamped addresses so that no full wait separates them
// -- are in flight while unit t is contracted.  The four waves split K;
// their partial sums meet in double-buffered LDS (one barrier per unit) in the
// fixed order w0 + w1 + w2 + w3, and wave t mod 4 finishes unit t.
template <int MODE, int G>
__global__ __launch_bounds__(256) void expert_stream_kernel(ExpertStreamArgs a) {
  constexpr int NS = 6;  // K steps per wave: 4 waves x 6 x 128 = 3072 elements
  constexpr int NV = 8;  // accumulator floats per lane per unit
  extern __shared__ __align__(16) unsigned char smem[];
  const int nblk = a.nblk;
  const int row_u4 = nblk * 8;                   // uint4 per activation row
  uint4* As = reinterpret_cast<uint4*>(smem);    // [G][row_u4]
  constexpr int LG = (G + 3) / 4;  // lane groups g whose accumulator rows 4g..4g+3 hold tokens
  float* red = reinterpret_cast<float*>(smem + (size_t)G * row_u4 * 16);  // [2][4][LG][NV][16]: live lanes only

  const int npair = MODE == 0 ? a.ntile : (a.ntile + 1) >> 1;
  // Teams of W workgroups share one token group and interleave its units
  // (workgroup j takes units j, j + W, ...), so that at any moment a team reads one
  // contiguous window of the expert's planes.
  const int nvv = *a.nv;
  const int W = max(1, (int)gridDim.x / max(nvv, 1));
  const int teams = gridDim.x / W;
  const int team = blockIdx.x / W, tj = blockIdx.x % W;
  if (team >= teams || tj >= npair) return;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int arow = min(n, G - 1) * row_u4;  // lanes past G re-read a live row; their outputs are unused

  struct WSet {
    u32x4 q[NS][2];
    u32x2 sc[2];  // this wave's scale bytes of the two tiles, one byte per K step
    float b0, b1;
  };

  int par = 0;
  for (int v = team; v < nvv; v += teams) {
    const int p_begin = tj, p_end = npair;
    const StreamGroup* gr = a.groups + v;
    const int gcount = min(G, gr->left);
    const int base = gr->base;
    const CSK_GLOBAL u32x4* q0 = as_global(reinterpret_cast<const u32x4*>(MODE == 0 ? gr->w.q_gate : gr->w.q_down)) + n;
    const CSK_GLOBAL u32x2* s0 = as_global(reinterpret_cast<const u32x2*>(MODE == 0 ? gr->w.s_gate : gr->w.s_down)) + wv * 64 + lane;
    const CSK_GLOBAL u32x4* q1 = as_global(reinterpret_cast<const u32x4*>(MODE == 0 ? gr->w.q_up : gr->w.q_down)) + n;
    const CSK_GLOBAL u32x2* s1 = as_global(reinterpret_cast<const u32x2*>(MODE == 0 ? gr->w.s_up : gr->w.s_down)) + wv * 64 + lane;
    const CSK_GLOBAL float* bp0 = as_global(MODE == 0 ? gr->w.b_gate : gr->w.b_down);
    const CSK_GLOBAL float* bp1 = as_global(MODE == 0 ? gr->w.b_up : gr->w.b_down);

    // activation rows of this token group -> LDS (every wave is past its last
    // read of the previous group: it has crossed that unit's barrier)
#pragma unroll
    for (int rr = 0; rr < G; ++rr) {
      if (rr < gcount) {
        const int row = a.list_row ? a.list_row[base + rr] : base + rr;
        const uint4* src = a.A + (size_t)row * row_u4;
        for (int c0 = wv * 64; c0 < row_u4; c0 += 256) {
          if (c0 + lane < row_u4)
            __builtin_amdgcn_global_load_lds(
                src + c0 + lane,
                reinterpret_cast<__attribute__((address_space(3))) uint4*>(
                    reinterpret_cast<uintptr_t>(As + rr * row_u4 + c0)),
                16, 0, 0);
        }
      }
    }

    // tiles of a unit: (R, R) for gate/up, (2R, 2R+1) for down
    // `idle`: a refill whose data nobody will use (past the workgroup's last unit).  It is
    // still issued, so that the count of loads in flight is the same on every path, but
    // every step aims at the same 1 KiB of the unit, which the caches hold: the tail of a
    // workgroup must not cost HBM traffic.
    auto load_step = [&](WSet& ws, int unit, int s, bool idle) {
      const int ta = MODE == 0 ? unit : 2 * unit;
      const int tb = MODE == 0 ? unit : min(2 * unit + 1, a.ntile - 1);
      const size_t ea = (size_t)ta * nblk * 16, eb = (size_t)tb * nblk * 16;
      const int kb = idle ? g : min(4 * (wv + 4 * s) + g, nblk - 1);
      ws.q[s][0] = q0[ea + kb * 16];
      ws.q[s][1] = q1[eb + kb * 16];
    };
    // per-unit scalars: the wave's scale bytes (scale plane: [tile][wave][lane][8]) and biases
    auto load_unit_scalars = [&](u32x2& sc0, u32x2& sc1, float& b0, float& b1, int unit) {
      const int ta = MODE == 0 ? unit : 2 * unit;
      const int tb = MODE == 0 ? unit : min(2 * unit + 1, a.ntile - 1);
      sc0 = s0[(size_t)ta * 256];
      sc1 = s1[(size_t)tb * 256];
      b0 = bp0[min(ta * 16 + n, a.N - 1)];  // bias pointers are never null (absent bias = zero vector)
      b1 = bp1[min(tb * 16 + n, a.N - 1)];
    };
    static_assert(G <= 8, "the reduction buffer holds two lane groups");
    const bool live = g < LG;  // token t is accumulator row t % 4 of lanes 16 (t / 4) .. 16 (t / 4) + 15

    // Contracts unit `unit` out of ws and, step by step, refills ws with unit `next`.
    auto compute_unit = [&](WSet& ws, int unit, int next) {
      const bool idle = next == unit;
      const float bias0 = ws.b0, bias1 = ws.b1;
      const u32x2 scb0 = ws.sc[0], scb1 = ws.sc[1];
      floatx4 acc[2][2];  // [tile of the pair][hi, lo term]: independent accumulation chains
#pragma unroll
      for (int m = 0; m < 2; ++m) acc[m][0] = acc[m][1] = floatx4{0.f, 0.f, 0.f, 0.f};
      U4B8 ahi[2], alo[2];  // activation fragments run one quarter-step ahead of the matrix cores
      {
        const int kb0 = min(4 * wv + g, nblk - 1);
        ahi[0].u = As[arow + kb0 * 8];
        alo[0].u = As[arow + kb0 * 8 + 4];
      }
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int kb = 4 * (wv + 4 * s) + g;
        const bool kvs = kb < nblk;
        const uint32_t byte0 = ((s < 4 ? scb0.x : scb0.y) >> (8 * (s & 3))) & 0xFFu;
        const uint32_t byte1 = ((s < 4 ? scb1.x : scb1.y) >> (8 * (s & 3))) & 0xFFu;
        const float sc0 = kvs ? e8m0_scale(byte0) : 0.0f;
        const float sc1 = kvs ? e8m0_scale(byte1) : 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int cur = (s * 4 + i) & 1, nxt = cur ^ 1;
          if (s * 4 + i + 1 < NS * 4) {
            const int s2 = (s * 4 + i + 1) >> 2, i2 = (s * 4 + i + 1) & 3;
            const int kb2 = min(4 * (wv + 4 * s2) + g, nblk - 1);
            ahi[nxt].u = As[arow + kb2 * 8 + i2];
            alo[nxt].u = As[arow + kb2 * 8 + 4 + i2];
          }
          const bf16x8 b0 = cvt_fp4x8(ws.q[s][0][i], sc0);
          acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ahi[cur].b, b0, acc[0][0], 0, 0, 0);
          acc[0][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(alo[cur].b, b0, acc[0][1], 0, 0, 0);
          const bf16x8 b1 = cvt_fp4x8(ws.q[s][1][i], sc1);
          acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ahi[cur].b, b1, acc[1][0], 0, 0, 0);
          acc[1][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(alo[cur].b, b1, acc[1][1], 0, 0, 0);
        }
        load_step(ws, next, s, idle);  // this step's registers are free: start the next unit's loads
      }
      load_unit_scalars(ws.sc[0], ws.sc[1], ws.b0, ws.b1, next);
      float* rbuf = red + (size_t)par * 4 * LG * NV * 16;
      par ^= 1;
      if (live) {
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int i = 0; i < 4; ++i) rbuf[((wv * LG + g) * NV + m * 4 + i) * 16 + n] = acc[m][0][i] + acc[m][1][i];
      }
      __syncthreads();
      if (wv == (unit & 3) && live) {
        float v2[2][4];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int o = m * 4 + i;
            v2[m][i] = ((rbuf[((0 * LG + g) * NV + o) * 16 + n] + rbuf[((1 * LG + g) * NV + o) * 16 + n]) +
                        rbuf[((2 * LG + g) * NV + o) * 16 + n]) + rbuf[((3 * LG + g) * NV + o) * 16 + n];
          }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = g * 4 + i;  // token slot within the group
          if (t < gcount) {
            const size_t p = (size_t)(base + t);
            if (MODE == 0) {
              const int r = unit * 16 + n;  // output feature
              if (r < a.N) {
                uint16_t hi, lo;
                split_bf16(moe_activation(v2[0][i] + bias0, v2[1][i] + bias1, a.act_type), hi, lo);
                uint16_t* o = a.act_out + (p * (size_t)(a.N >> 5) + (r >> 5)) * 64 + (r & 31);
                o[0] = hi;
                o[32] = lo;
              }
            } else {
              const int ra = 2 * unit * 16 + n, rb = ra + 16;
              if (ra < a.N) a.y_out[p * (size_t)a.N + ra] = v2[0][i] + bias0;
              if (rb < a.N) a.y_out[p * (size_t)a.N + rb] = v2[1][i] + bias1;
            }
          }
        }
      }
    };

    // One register set, refilled step by step as it is consumed: the loads of unit
    // t+1 are issued during unit t and stay one unit ahead of their use.  Refills
    // are unconditional (past the last unit they re-read one cached KiB of it), so
    // that the number of loads in flight is the same on every path and the waits in
    // front of the matrix cores stay partial.
    const int t_last = p_begin + ((p_end - 1 - p_begin) / W) * W;  // last unit of this workgroup
    WSet ws;
#pragma unroll
    for (int s = 0; s < NS; ++s) load_step(ws, p_begin, s, false);
    load_unit_scalars(ws.sc[0], ws.sc[1], ws.b0, ws.b1, p_begin);
    __syncthreads();  // the LDS copies have landed (the compiler waits for them before the barrier)
    for (int t = p_begin; t < p_end; t += W) compute_unit(ws, t, min(t + W, t_last));
  }
}

}  // namespace csk
