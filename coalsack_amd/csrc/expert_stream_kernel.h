// Expert MLP for the weight-streaming (decode) regime.
//
// Every active expert's matrices are streamed from HBM once per group of up to
// four (or six) of its tokens: 64 lanes x 16 bytes = 1 KiB of contiguous nibbles per
// 16-row tile per K step, the four waves of a workgroup taking interleaved K
// steps (128 elements each).  The MXFP4 entries are the B operand of the block-scaled
// matrix instruction as they are stored, their E8M0 bytes its scale operand; the group's
// activation rows are its A operand as three FP6 terms (mx3.h), so each product is that of
// the reference's fp32 activation (to 2^-14.7 of its block's maximum) and the exactly
// dequantised weight; accumulation is fp32.  The K slices of the four waves meet in LDS in
// a fixed order.
//
// Restates include/coalsack/nn/nn_ops/expert_mlp_node.h:651-732
// (compute_token_mxfp4): gate/up projections + bias, activation (:699-706),
// down projection + bias; the token loop of :503-529 becomes the M dimension.
#pragma once
#include "common.h"
#include "mx3.h"
#include "route_select.h"

namespace csk {

// Bias pointers inside desc[].w must not be null for expert_stream_kernel: the
// host substitutes a zero vector for an absent bias, so that the loads are
// unconditional.
struct ExpertStreamArgs {
  const WorkDesc* desc;
  const StreamGroup* groups;  // [nv]: the groups of up to G tokens
  const int* nv;         // number of such groups
  int nv_known;          // > 0: the number of groups is known at launch (one token: its k experts), *nv is not read
  const int* list_row;   // packed position -> row of X; null: row = packed position
  const float* gather_w; // packed position -> factor applied to its row (weight_before_ffn); null: 1
  const float* X;        // [rows][32 nblk] fp32 activation rows
  const u32x4* X3;       // the same rows already as three FP6 terms, [rows][mx3_row_blocks(nblk)][6] (mx3.h), or null
  const float* zeros;    // at least 16 bytes of zeros (with X3)
  int nblk;              // K / 32
  int ntile;             // ceil(N / 16)
  int N;                 // output features (F for gate/up, H for down)
  int act_type;
  float* act_out;        // gate/up: [P][N] fp32
  float* y_out;          // down: [P][N] fp32
  RouteIn rin;           // ROUTE1 form only: what the token is routed from ...
  RouteOut rout;         // ... and where workgroup 0 leaves the router's output and the lists
};

// exp and the reciprocal are the hardware's own approximations (v_exp_f32 on x log2 e,
// v_rcp_f32: one ulp each, a relative error near 1e-6 after the argument's rounding at
// |x| <= 12), not libm's expf and an IEEE division: the epilogue of the grouped GEMM
// evaluates 64 of these per lane and was spending more vector instructions on them than
// on anything else.  Both regimes use this one function, so they agree with each other.
__device__ __forceinline__ float fast_sigmoid_mul(float x, float slope) {  // x * sigmoid(slope x)
  const float e = __builtin_amdgcn_exp2f(x * (-slope * 1.4426950408889634f));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float moe_activation(float gate_v, float up_v, int act_type) {
  if (act_type == 0) {  // expert_mlp_node.h:699-703
    const float x = fminf(gate_v, 7.0f);
    const float y = fminf(fmaxf(up_v, -7.0f), 7.0f);
    return fast_sigmoid_mul(x, 1.702f) * (y + 1.0f);
  }
  return fast_sigmoid_mul(gate_v, 1.0f) * up_v;  // :705-706
}

// ---------------------------------------------------------------------------
// Persistent, software-pipelined kernel (K <= 3072) on the block-scaled matrix
// instruction v_mfma_scale_f32_16x16x128_f8f6f4: A = the group's activation rows as
// three FP6 terms (mx3.h), B = the MXFP4 weights exactly as they are stored -- lane
// (g = lane / 16, n = lane % 16) holds K block g of the step of weight row n, which is the
// 16-byte entry the repacked plane keeps for it, and passes that block's E8M0 byte as the
// instruction's scale operand.  No conversion instruction touches a weight.
//
// MODE 0: a work unit is the pair (gate tile R, up tile R), SwiGLU epilogue.
// MODE 1: a work unit is the pair of down tiles (2R, 2R+1).
// G = tokens contracted per pass (rows 0..G-1 of the instruction's 16 token rows).
//
// The work is (token group of an expert) x (tile pair): every group costs the
// same, so teams of gridDim.x / groups workgroups take one group each and
// interleave its units, and the load is balanced whatever the routing was.
// Memory-level parallelism bounds this kernel, so it never lets the memory
// queue drain: the weight registers are refilled step by step as the matrix cores
// consume them: the loads of unit t+1 -- issued unconditionally from clamped addresses so
// that no full wait separates them -- are in flight while unit t is contracted.  A
// group's activation rows arrive as fp32 and are quantised to the three-term form by the
// workgroup itself, into LDS, while its first weight loads are under way.  The four waves
// split K; their partial sums meet in double-buffered LDS (one barrier per unit) in the
// fixed order w0 + w1 + w2 + w3, and wave t mod 4 finishes unit t.
typedef int i32x8 __attribute__((ext_vector_type(8)));

// Descriptor of a whole weight plane as a raw buffer (the pointer is the same in every lane).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stream_plane_rsrc(const void* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(((uint64_t)hi << 32) | lo), 0, 0x7fffffff, 0x00020000);
}

//
// ROUTE1 (gate/up of a one-token batch): there is no routing kernel in front.  Every
// workgroup selects the token's k experts itself from the logits -- select_topk in each of
// its four waves, so that nothing passes from wave to wave; a close call recomputed by the
// whole workgroup, exactly as route_tiny_kernel does; all workgroups compute the same thing
// from the same inputs -- and takes the expert whose rank among the selected ones is its
// team's number: that rank is the expert's packed position, as the dispatch would have
// numbered it.  The experts' pointer table is staged in LDS while the logits are on their
// way.  Workgroup 0 also writes what the routing kernel would have written (pairs, ids,
// positions, lists, counts, token groups) for the down kernel, the combine and
// csk_layer_last_dispatch.  A 5.4 us launch with its dependent reads is replaced by 3 us in
// front of this kernel's first weight loads (120b shape: 32.6 -> 30.0 us per layer).
template <int MODE, int G, bool ROUTE1 = false>
__global__ __launch_bounds__(256, 2) void expert_stream_kernel(ExpertStreamArgs a) {
  static_assert(!ROUTE1 || MODE == 0, "the gate/up kernel is the one that routes");
  constexpr int NS = 6;  // K steps per wave: 4 waves x 6 x 128 = 3072 elements
  constexpr int NV = 8;  // accumulator floats per lane per unit
  extern __shared__ __align__(16) unsigned char smem[];
  const int nblk = a.nblk;
  // blocks per activation row in LDS: all the blocks the steps touch, those past K zero, so
  // that nothing in the main loop is clamped or masked (weight blocks past K are then the
  // next tile's, or the slack behind the plane, times exact zeros)
  constexpr int lrb = NS * 16;
  u32x4* As = reinterpret_cast<u32x4*>(smem);  // [G][lrb][3 terms][2] x 16 B
  constexpr int LG = (G + 3) / 4;  // lane groups g whose accumulator rows 4g..4g+3 hold tokens
  float* red = reinterpret_cast<float*>(smem + (size_t)G * lrb * (kMx3ChunksPerBlock * 16));  // [2][4][LG][NV][16]: live lanes only

  const int npair = MODE == 0 ? a.ntile : (a.ntile + 1) >> 1;
  // Teams of W workgroups share one token group and interleave its units
  // (workgroup j takes units j, j + W, ...), so that at any moment a team reads one
  // contiguous window of the expert's planes.
  const int nvv = a.nv_known > 0 ? a.nv_known : *a.nv;  // one dependent read fewer in front of the first weights
  const int W = max(1, (int)gridDim.x / max(nvv, 1));
  const int teams = gridDim.x / W;
  const int team = blockIdx.x / W, tj = blockIdx.x % W;
  if (team >= teams || tj >= npair) return;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;

  // ROUTE1: slot s of the token in lane s of every wave (all four waves select, from the same
  // logits, so that nothing has to be handed from wave to wave)
  int r_idx = 0;
  float r_wt = 0.0f;
  constexpr int kEwWords = kMaxExperts * (int)(sizeof(ExpertW) / 8), kEwPerThread = (kEwWords + 255) / 256;
  __shared__ unsigned long long s_ew[ROUTE1 ? kEwWords : 1];  // the experts' weight pointers, staged beside the logits
  if constexpr (ROUTE1) {
    const RouteIn& r = a.rin;
    const RouteOut& o = a.rout;
    const int E = r.E, k = r.k;
    // the recomputation's staging area lies where the activation rows go afterwards
    CloseCallLds& cc = *reinterpret_cast<CloseCallLds*>(smem);
    const float NEG = -__builtin_inff();
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = lane + 64 * j;
      v[j] = e < E ? r.logits[e] : NEG;
    }
    unsigned long long ew_reg[kEwPerThread];
#pragma unroll
    for (int i = 0; i < kEwPerThread; ++i) {
      const int w = threadIdx.x + i * 256;
      ew_reg[i] = w < E * (int)(sizeof(ExpertW) / 8) ? reinterpret_cast<const unsigned long long*>(r.ew)[w] : 0ull;
    }
    float my_val, vmax, runner_up;  // lane s keeps slot s
    bool close_call;
    const float tol = close_call_tolerance(r.H);
    select_topk(v, lane, E, k, my_val, r_idx, vmax, close_call, tol, runner_up);
#pragma unroll
    for (int i = 0; i < kEwPerThread; ++i) {
      const int w = threadIdx.x + i * 256;
      if (w < kEwWords) s_ew[w] = ew_reg[i];
    }
    if (close_call) {  // the same in every wave, and in every workgroup
      const float thr = runner_up - 2.0f * tol * fmaxf(1.0f, fabsf(runner_up));
      logits_reference_order_wg<256>(r.x, r.g, r.b, r.logits, E, r.H, thr, cc);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        v[j] = e < E ? cc.fixed[e] : NEG;
      }
      select_topk(v, lane, E, k, my_val, r_idx, vmax, close_call, 0.0f, runner_up);
    }
    r_wt = routing_weight(my_val, vmax, lane, k, r.sigmoid);
    __syncthreads();  // the pointer table is in LDS; every thread is done with cc before the activation rows overwrite it
    if (blockIdx.x == 0) {
      // what the routing kernel would have written
      __shared__ int w_ids[kMaxTopK];
      if (wv == 0 && lane < k) w_ids[lane] = r_idx;
      __syncthreads();
      for (int e = threadIdx.x; e < E; e += 256) {
        int c = 0;
        for (int q = 0; q < k; ++q) c += w_ids[q] == e;
        o.counts[e] = c;
      }
      if (wv == 0 && lane < k) {
        int pos = 0;
        for (int q = 0; q < k; ++q) pos += w_ids[q] < r_idx;  // the k experts are distinct
        reinterpret_cast<float2*>(o.pairs)[lane] = make_float2((float)r_idx, r_wt);
        o.ids[lane] = r_idx;
        o.list_tok[pos] = 0;
        o.list_w[pos] = r_wt;
        o.pos_of_slot[lane] = pos;
        write_stream_group(o.groups + pos, reinterpret_cast<const ExpertW*>(s_ew) + r_idx, r_idx, 1, pos);
      }
      if (threadIdx.x == 0) *o.nv = k;
    }
  }

  struct WSet {
    u32x4 q[NS][2];
    u32x2 sc[2];  // this wave's scale bytes of the two tiles, one byte per K step
    float b0, b1;
  };

  int par = 0;
  for (int v = team; v < nvv; v += teams) {
    const int p_begin = tj, p_end = npair;
    const StreamGroup* gr = a.groups + v;
    int r_e = 0;
    float r_gw = 1.0f;
    if constexpr (ROUTE1) {  // the selected expert with v selected experts below it: packed position v
      const int k = a.rin.k;
      int lower = 0;
      for (int q = 0; q < k; ++q) lower += __builtin_amdgcn_readlane(r_idx, q) < r_idx;
      const unsigned long long mine = __ballot(lane < k && lower == v);
      const int sl = (int)__builtin_ctzll(mine | (1ull << 63));
      r_e = __builtin_amdgcn_readlane(r_idx, sl);
      r_gw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r_wt), sl));
    }
    const ExpertW* gw_ptr = ROUTE1 ? reinterpret_cast<const ExpertW*>(s_ew) + r_e : &gr->w;
    const int gcount = ROUTE1 ? 1 : min(G, gr->left);
    const int base = ROUTE1 ? v : gr->base;
    // One buffer descriptor per weight plane: the unit's tile and the K step go into the
    // scalar offset of a load, the lane's place within the step (block g, row n) into its
    // vector offset, which never changes.
    const auto q_rsrc0 = stream_plane_rsrc(MODE == 0 ? gw_ptr->q_gate : gw_ptr->q_down);
    const auto q_rsrc1 = stream_plane_rsrc(MODE == 0 ? gw_ptr->q_up : gw_ptr->q_down);
    const uint32_t qoff = (uint32_t)((g * 16 + n) * 16);
    const CSK_GLOBAL u32x2* s0 = as_global(reinterpret_cast<const u32x2*>(MODE == 0 ? gw_ptr->s_gate : gw_ptr->s_down)) + wv * 64 + lane;
    const CSK_GLOBAL u32x2* s1 = as_global(reinterpret_cast<const u32x2*>(MODE == 0 ? gw_ptr->s_up : gw_ptr->s_down)) + wv * 64 + lane;
    const CSK_GLOBAL float* bp0 = as_global(MODE == 0 ? gw_ptr->b_gate : gw_ptr->b_down);
    const CSK_GLOBAL float* bp1 = as_global(MODE == 0 ? gw_ptr->b_up : gw_ptr->b_down);

    // tiles of a unit: (R, R) for gate/up, (2R, 2R+1) for down.
    // `idle`: a refill whose data nobody will use (past the workgroup's last unit).  It is
    // still issued, so that the count of loads in flight is the same on every path, but
    // every step aims at the same 1 KiB of the unit, which the caches hold: the tail of a
    // workgroup must not cost HBM traffic.
    auto load_step = [&](WSet& ws, int unit, int s, bool idle) {
      const int ta = MODE == 0 ? unit : 2 * unit;
      const int tb = MODE == 0 ? unit : min(2 * unit + 1, a.ntile - 1);
      // four blocks of 16 rows x 16 B per step; a step that lies wholly past K (its activations
      // are zeros) re-reads the cached start of the tile instead of fetching the next tile's blocks
      const uint32_t step = (idle || 4 * (wv + 4 * s) >= nblk) ? 0u : (uint32_t)(wv + 4 * s) * 1024u;
      ws.q[s][0] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc0, qoff, (uint32_t)ta * (uint32_t)nblk * 256u + step, 0);
      ws.q[s][1] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc1, qoff, (uint32_t)tb * (uint32_t)nblk * 256u + step, 0);
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

    // A thread's first block of activations is requested first (loads return in order: asked
    // for after the weights it would arrive behind them), then the first unit's weights ...
    const int nfill = gcount * lrb;
    // Rows that arrive as FP6 terms already (written once per token by the routing prologue)
    // are only copied into LDS, behind the first unit's weights (below).
    const bool copy_rows = MODE == 0 && a.X3 != nullptr && a.gather_w == nullptr;
    int copy_row[G];  // the rows' numbers, read before the weights are requested
    if (copy_rows) {
#pragma unroll
      for (int rr = 0; rr < G; ++rr) {
        const int p = base + min(rr, gcount - 1);
        copy_row[rr] = ROUTE1 ? 0 : a.list_row ? a.list_row[p] : p;
      }
    }
    float4 pre[8];
    if (!copy_rows) {
      const int rr = threadIdx.x / lrb, kb = threadIdx.x - rr * lrb;
      if ((int)threadIdx.x < nfill && kb < nblk) {
        const int row = ROUTE1 ? 0 : a.list_row ? a.list_row[base + rr] : base + rr;
        const float4* src = reinterpret_cast<const float4*>(a.X + ((size_t)row * nblk + kb) * 32);
#pragma unroll
        for (int i = 0; i < 8; ++i) pre[i] = src[i];
      }
    }
    WSet ws;
#pragma unroll
    for (int s = 0; s < NS; ++s) load_step(ws, p_begin, s, false);
    load_unit_scalars(ws.sc[0], ws.sc[1], ws.b0, ws.b1, p_begin);

    // ... and while those are under way the group's activation rows are
    // quantised into LDS, one thread per 32-value block (every wave is past its last read
    // of the previous group: it has crossed that unit's barrier).  Rows may be gathered
    // through list_row and scaled by the routing weight (weight_before_ffn).
    if (MODE == 0 && copy_rows) {
      // The LDS image of a row is its blocks in order, [lrb][6 chunks of 16 bytes]; the row in
      // memory has mx3_row_blocks(nblk) of them, the rest are zeros (any scale byte will do
      // for a block of zero codes: they come from the library's page of zeros).  Copied by
      // global_load_lds -- nothing of it lives in a register; instruction i of wave wv fills
      // the 64 chunks from (4 i + wv) * 64 on -- and waited for explicitly: the compiler does
      // not count these loads, so none of them may be in flight past the wait below.
      const int rowblk = mx3_row_blocks(nblk);
      constexpr int kRowChunks = lrb * kMx3ChunksPerBlock;
      constexpr int kCopyInstr = (G * kRowChunks + 255) / 256;
      const int total = gcount * kRowChunks;
      const uint32_t lds_as = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
#pragma unroll 1
      for (int i = 0; i < kCopyInstr; ++i) {
        const int ch0 = (4 * i + wv) * 64;
        const int ch = ch0 + lane;
        if (ch < total) {
          const int rr = ch / kRowChunks, q = ch - rr * kRowChunks;
          int row = copy_row[0];
#pragma unroll
          for (int x = 1; x < G; ++x) row = rr == x ? copy_row[x] : row;
          const u32x4* src = q < rowblk * kMx3ChunksPerBlock ? a.X3 + (size_t)row * rowblk * kMx3ChunksPerBlock + q
                                                            : reinterpret_cast<const u32x4*>(a.zeros);
          asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                       :
                       : "v"(src), "s"(__builtin_amdgcn_readfirstlane((int)(lds_as + (uint32_t)ch0 * 16u)))
                       : "memory");
        }
      }
      __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0): the copies (and the first weights) have landed
    }
#pragma unroll 1
    for (int idx = threadIdx.x; idx < (copy_rows ? 0 : nfill); idx += 256) {
      const int rr = idx / lrb, kb = idx - rr * lrb;
      u32x4 out[kMx3ChunksPerBlock];
      if (kb >= nblk) {
#pragma unroll
        for (int t = 0; t < kMx3Terms; ++t) {
          out[2 * t] = u32x4{0u, 0u, 0u, 0u};
          out[2 * t + 1] = u32x4{0u, 0u, 127u, 0u};
        }
      } else {
        float r[32];
        if (idx != (int)threadIdx.x) {  // later blocks of this thread: fetched here
          const int row = ROUTE1 ? 0 : a.list_row ? a.list_row[base + rr] : base + rr;
          const float4* src = reinterpret_cast<const float4*>(a.X + ((size_t)row * nblk + kb) * 32);
#pragma unroll
          for (int i = 0; i < 8; ++i) pre[i] = src[i];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) r[4 * i] = pre[i].x, r[4 * i + 1] = pre[i].y, r[4 * i + 2] = pre[i].z, r[4 * i + 3] = pre[i].w;
        if (a.gather_w) {
          const float gw = ROUTE1 ? r_gw : a.gather_w[base + rr];  // (the list of weights is being written by workgroup 0)
#pragma unroll
          for (int i = 0; i < 32; ++i) r[i] = r[i] * gw;
        }
        mx3_quantize_block(r, out);
      }
      u32x4* dst = As + (size_t)idx * kMx3ChunksPerBlock;
#pragma unroll
      for (int c = 0; c < kMx3ChunksPerBlock; ++c) dst[c] = out[c];
    }
    // lanes past the group's tokens re-read its last row; their outputs are unused
    const u32x4* afrag = As + ((size_t)(min(n, gcount - 1) * lrb + 4 * wv + g) * kMx3Terms) * 2;

    // Contracts unit `unit` out of ws and, step by step, refills ws with unit `next`.
    auto compute_unit = [&](WSet& ws, int unit, int next) {
      const bool idle = next == unit;
      const float bias0 = ws.b0, bias1 = ws.b1;
      const u32x2 scb0 = ws.sc[0], scb1 = ws.sc[1];
      floatx4 acc[2];  // one 16 x 16 tile each
#pragma unroll
      for (int m = 0; m < 2; ++m) acc[m] = floatx4{0.f, 0.f, 0.f, 0.f};
      u32x4 flo[2], fhi[2];  // activation fragments run one term ahead of the matrix cores
      auto read_frag = [&](int i) {  // fragment i = (step, term)
        const int s = i / kMx3Terms, t = i - s * kMx3Terms;
        const u32x4* f = afrag + (16 * s * kMx3Terms + t) * 2;  // a constant offset from the lane's base
        flo[i & 1] = f[0];
        fhi[i & 1] = f[1];
      };
      read_frag(0);
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int byte0 = (int)(((s < 4 ? scb0.x : scb0.y) >> (8 * (s & 3))) & 0xFFu);
        const int byte1 = (int)(((s < 4 ? scb1.x : scb1.y) >> (8 * (s & 3))) & 0xFFu);
        const i32x8 bw0 = (i32x8)__builtin_shufflevector(ws.q[s][0], ws.q[s][0], 0, 1, 2, 3, -1, -1, -1, -1);
        const i32x8 bw1 = (i32x8)__builtin_shufflevector(ws.q[s][1], ws.q[s][1], 0, 1, 2, 3, -1, -1, -1, -1);
#pragma unroll
        for (int t = 0; t < kMx3Terms; ++t) {
          const int i = s * kMx3Terms + t;
          if (i + 1 < NS * kMx3Terms) read_frag(i + 1);
          // FP6 reads the first six registers; register 6 holds the term's scale byte
          const i32x8 aw = (i32x8)__builtin_shufflevector(flo[i & 1], fhi[i & 1], 0, 1, 2, 3, 4, 5, 6, 7);
          acc[0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aw, bw0, acc[0], 2, 4, 0, aw[6], 0, byte0);
          acc[1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aw, bw1, acc[1], 2, 4, 0, aw[6], 0, byte1);
          // fragments are read one ahead, not all at once: the scheduler may not hoist the LDS reads over this point
          __builtin_amdgcn_sched_barrier(0);
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
          for (int i = 0; i < 4; ++i) rbuf[((wv * LG + g) * NV + m * 4 + i) * 16 + n] = acc[m][i];
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
              if (r < a.N) a.act_out[p * (size_t)a.N + r] = moe_activation(v2[0][i] + bias0, v2[1][i] + bias1, a.act_type);
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
    __syncthreads();  // the quantised rows are in LDS
    for (int t = p_begin; t < p_end; t += W) compute_unit(ws, t, min(t + W, t_last));
  }
}

}  // namespace csk
