// Expert MLP for the compute-bound (prefill) regime: grouped GEMM over the
// dispatched tokens on the matrix cores.
//
// A workgroup owns one M tile (64 tokens of one expert) x one N tile (128
// output features: gate and up rows together, or 256 down rows) and walks K in
// steps of 128 elements.  Per step
//   * the activation tile (64 tokens x 128 elements, two bf16 terms = 32 KiB)
//     is copied into LDS by global_load_lds, gathered by token, with a 16-byte
//     XOR swizzle chosen at the *source* side (each lane picks which chunk it
//     fetches) so that the 16 lanes of a fragment read hit 16 different bank
//     groups;
//   * each wave loads its four weight entries (16 rows x 4 blocks x 16 B, the
//     resident packed layout is already fragment order) straight into
//     registers, one step ahead, and expands them with
//     v_cvt_scalef32_pk_bf16_fp4;
//   * 128 MFMAs (16x16x32 bf16) per wave contract hi and lo terms into fp32.
// Two LDS stages, one barrier per step.  The epilogue fuses bias + SwiGLU (and
// the bf16 split the next GEMM reads) or bias + store.
//
// Restates include/coalsack/nn/nn_ops/expert_mlp_node.h:651-732 with the token
// loop of :503-529 as the M dimension.
#pragma once
#include "common.h"
#include "expert_stream_kernel.h"

namespace csk {

constexpr int kGemmBM = 64;  // tokens per M tile
constexpr int kDies = 8;     // accelerator dies (XCDs) of the part, each with a private L2

struct ExpertGemmArgs {
  const WorkDesc* desc;
  const int* mtiles;     // [2 * n]: (expert slot, first token) of each M tile
  const int* n_mtiles;
  const int* list_row;   // packed position -> row of A; null: row = packed position
  const uint4* A;        // [rows][nblk][8] x 16 B: 32 bf16 hi then 32 bf16 lo per block
  int nblk;              // K / 32
  int ntile;             // ceil(N / 16) weight row tiles
  int n_ntiles;          // N tiles per M tile: ceil(ntile / 8) (MODE 0) or ceil(ntile / 16)
  int N;
  int act_type;
  uint16_t* act_out;     // MODE 0
  float* y_out;          // MODE 1
};

// MODE 0: N tile = 128 features; wave w owns gate tiles {8x+2w, 8x+2w+1} and the
//         same up tiles.  MODE 1: N tile = 256 rows; wave w owns down tiles 16x+4w..+3.
template <int MODE>
__global__ __launch_bounds__(256) void expert_gemm_kernel(ExpertGemmArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint4* As = reinterpret_cast<uint4*>(smem);  // [2 stages][64 tokens][32 chunks]
  // Work unit = (M tile, N tile), numbered M-tile major.  Workgroups are handed to
  // the eight accelerator dies round-robin by linear id, and each die has its own L2:
  // die x takes the x-th contiguous eighth of the unit sequence, so that the
  // workgroups resident on one die at one time share a few activation panels and a few
  // experts' weights, which then come from that L2 instead of from memory.
  const int n_units = *a.n_mtiles * a.n_ntiles;
  const int per_die = (n_units + kDies - 1) / kDies;
  const int slot = blockIdx.x / kDies;
  const int unit = (blockIdx.x % kDies) * per_die + slot;
  if (slot >= per_die || unit >= n_units) return;
  const int mt = unit / a.n_ntiles, nt = unit - mt * a.n_ntiles;
  const WorkDesc* wd = a.desc + a.mtiles[2 * mt];
  const int m0 = a.mtiles[2 * mt + 1];
  const int Te = wd->Te;
  const int base = wd->base + m0;
  const int mcount = min(kGemmBM, Te - m0);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int nblk = a.nblk;
  const int nsteps = (nblk + 3) >> 2;
  const int slots = scale_slots(nblk);

  // this wave's four weight row tiles
  int tiles[4];
  const CSK_GLOBAL u32x4* qp[4];
  const CSK_GLOBAL uint8_t* sp[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    int t;
    if (MODE == 0) t = nt * 8 + wv * 2 + (e & 1);
    else t = nt * 16 + wv * 4 + e;
    tiles[e] = t;
    const int tc = min(t, a.ntile - 1);
    const uint4* qb = MODE == 0 ? (e < 2 ? wd->w.q_gate : wd->w.q_up) : wd->w.q_down;
    const uint8_t* sb = MODE == 0 ? (e < 2 ? wd->w.s_gate : wd->w.s_up) : wd->w.s_down;
    qp[e] = as_global(reinterpret_cast<const u32x4*>(qb)) + (size_t)tc * nblk * 16 + n;
    sp[e] = as_global(sb) + scale_index(tc, 0, n, slots);
  }
  if (tiles[0] >= a.ntile) {
    // the whole wave is past N; it still takes part in the copies and barriers below
  }

  // rows this lane copies: instruction c (0..7) of wave wv moves tokens 2*(8*wv+c), +1
  const uint4* arow[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int tl = min(2 * (8 * wv + c) + (lane >> 5), mcount - 1);  // tokens past the tile re-read its last one
    const int row = a.list_row ? a.list_row[base + tl] : base + tl;
    arow[c] = a.A + (size_t)row * nblk * 8;
  }
  auto copy_a = [&](int stage, int j) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int q = 8 * wv + c;                    // copy instruction index within the stage
      const int tl = 2 * q + (lane >> 5);          // token slot this lane serves
      const int ci = (lane & 31) ^ (tl & 15);      // logical chunk stored at this lane's position
      const int kb = min(4 * j + (ci >> 3), nblk - 1);
      __builtin_amdgcn_global_load_lds(
          arow[c] + (size_t)kb * 8 + (ci & 7),
          reinterpret_cast<__attribute__((address_space(3))) uint4*>(
              reinterpret_cast<uintptr_t>(As + stage * 2048 + q * 64)),
          16, 0, 0);
    }
  };
  struct BSet {
    u32x4 q[4];
    uint32_t s[4];
  };
  auto load_b = [&](BSet& b, int j) {
    const int kb = min(4 * j + g, nblk - 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      b.q[e] = qp[e][kb * 16];
      b.s[e] = sp[e][scale_index(0, kb, 0, slots)];
    }
  };

  floatx4 acc[4][4];  // [m sub-tile][weight tile]
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[mt][e] = floatx4{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](const BSet& b, int stage, int j) {
    const bool kv = 4 * j + g < nblk;
    float sc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) sc[e] = kv ? e8m0_scale(b.s[e]) : 0.0f;
    const uint4* at = As + stage * 2048;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      U4B8 ah[4], al[4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        const int tok = mt * 16 + n;
        ah[mt].u = at[tok * 32 + ((g * 8 + i) ^ n)];
        al[mt].u = at[tok * 32 + ((g * 8 + 4 + i) ^ n)];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bf16x8 bw = cvt_fp4x8(b.q[e][i], sc[e]);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
          acc[mt][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[mt].b, bw, acc[mt][e], 0, 0, 0);
          acc[mt][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[mt].b, bw, acc[mt][e], 0, 0, 0);
        }
      }
    }
  };

  BSet ba, bb;
  copy_a(0, 0);
  load_b(ba, 0);
  for (int j = 0; j < nsteps; j += 2) {
    __syncthreads();  // stage 0 has landed; every wave is done with stage 1
    copy_a(1, min(j + 1, nsteps - 1));
    load_b(bb, min(j + 1, nsteps - 1));
    compute(ba, 0, j);
    __syncthreads();  // stage 1 has landed; every wave is done with stage 0
    copy_a(0, min(j + 2, nsteps - 1));
    load_b(ba, min(j + 2, nsteps - 1));
    if (j + 1 < nsteps) compute(bb, 1, j + 1);
  }

  // epilogue: lane (n, g) holds tokens mt*16 + 4g + i of weight row n of each tile
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tl = mt * 16 + g * 4 + i;
      if (tl >= mcount) continue;
      const size_t p = (size_t)(base + tl);
      if (MODE == 0) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int r = tiles[e] * 16 + n;
          if (tiles[e] < a.ntile && r < a.N) {
            const float gate_v = acc[mt][e][i] + wd->w.b_gate[r];
            const float up_v = acc[mt][e + 2][i] + wd->w.b_up[r];
            uint16_t hi, lo;
            split_bf16(moe_activation(gate_v, up_v, a.act_type), hi, lo);
            uint16_t* o = a.act_out + (p * (size_t)(a.N >> 5) + (r >> 5)) * 64 + (r & 31);
            o[0] = hi;
            o[32] = lo;
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = tiles[e] * 16 + n;
          if (tiles[e] < a.ntile && r < a.N) a.y_out[p * (size_t)a.N + r] = acc[mt][e][i] + wd->w.b_down[r];
        }
      }
    }
  }
}

}  // namespace csk
