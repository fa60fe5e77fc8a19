// Expert MLP for the compute-bound (prefill) regime on the block-scaled matrix
// instruction: v_mfma_scale_f32_32x32x64_f8f6f4 with A = activations as three
// FP6 (E2M3) terms (mx3.h) and B = the MXFP4 weights exactly as they are stored.
//
// Measured on this part with random operands: 5.6-6.2 PFLOP/s for FP6 x FP4 in
// the 32x32x64 form, against 1.9 PFLOP/s for bf16 32x32x16 (1.3 for 16x16x32);
// three FP6 terms instead of two bf16 terms therefore cost about half the matrix
// time, need no weight expansion (no conversion instruction at all), and the
// activation tile is 24 KiB per stage instead of 32.
//
// Operand ownership of the instruction (found by one-hot probing): lane l holds
// row l%32 of A (a token) or column l%32 of B (a weight row) and the 32 K values
// of block l/32 of the 64; position p of A pairs with position p of B; each lane
// passes the E8M0 scale of its own block.  A weight "column" l%32 is row l%16 of
// tile (l%32)/16 of a pair of packed 16-row tiles, and its 16-byte packed entry
// (32 nibbles in element order) is the operand.
//
// A workgroup of four waves owns 64 tokens of one expert x (128 NG) weight rows -- gate and
// up rows of the same 64 NG features together, or 128 NG down rows -- and walks K in steps
// of 128 (4 blocks).  A wave owns NG groups of 32 weight rows (NG/2 gate groups and the NG/2
// up groups of the same features) for all 64 tokens: NG x 2 accumulator tiles of 32 x 32.
// The activations are the expensive operand (three terms of 32 bytes per 32 values against
// 17 bytes of weights), so the tile is tall in weight rows: every activation fragment read
// from LDS feeds NG matrix instructions, and NG = 4 is what still leaves two workgroups per
// compute unit (128 accumulator + 80 weight registers per lane).  Measured with cycle
// stamps per step: a wave spends 80-85 % of the K loop issuing matrix instructions at one
// per ~40 cycles (the scaled form is a pair: scale load + product), 10-17 % waiting for the
// next step's loads and 3-5 % at the barrier; a quarter of a workgroup's time lies outside
// the loop (first loads, epilogue, the ragged last round of units).
// The activation tile (64 tokens x 4 blocks x 3 terms x 32 B) goes to LDS by
// global_load_lds with a 16-byte XOR swizzle applied on the source side; weights go
// straight to registers; both are requested one step ahead (two LDS stages and register
// sets, one barrier per step).
// The gate/up epilogue applies bias + SwiGLU, stages each wave's 64 x 16 NG tile in LDS as
// fp32 and re-quantises it to the three-term format the down GEMM reads.
//
// Restates include/coalsack/nn/nn_ops/expert_mlp_node.h:651-732 with the token
// loop of :503-529 as the M dimension.
#pragma once
#include "common.h"
#include "expert_stream_kernel.h"
#include "mx3.h"

namespace csk {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32_unaligned __attribute__((aligned(1)));

struct ExpertGemmMxArgs {
  const WorkDesc* desc;
  const int* mtiles;     // [2 * n]: (expert slot, first token) of each M tile
  const int* n_mtiles;
  const int* list_row;   // packed position -> row of A; null: row = packed position
  const uint4* A;        // [rows][mx3_row_blocks(nblk)][6] x 16 B (mx3.h); blocks past nblk are zeros
  int nblk;              // K / 32
  int ntile;             // N / 16 weight row tiles (even: N is a multiple of 32)
  int n_ntiles;          // N tiles per M tile: ceil(ntile / (4 NG)) (MODE 0) or ceil(ntile / (8 NG))
  int N;
  int act_type;
  u32x4* act_out;        // MODE 0: [P][mx3_row_blocks(N / 32)][6] x 16 B
  float* y_out;          // MODE 1: [P][N]
};

constexpr int kGemmBM = 64;  // tokens per M tile
constexpr int kDies = 8;     // accelerator dies (XCDs) of the part, each with a private L2

constexpr int kMxStageChunks = kGemmBM * 4 * kMx3ChunksPerBlock;  // 1536 x 16 B = 24 KiB
constexpr int kMxRowChunks = 4 * kMx3ChunksPerBlock;              // 24 chunks per token per step
constexpr int kMxWaves = 4;                                       // waves per workgroup
constexpr int kMxCopies = kMxStageChunks / 64 / kMxWaves;         // copy instructions per wave per step
constexpr int kMxNG = 4;                                          // groups of 32 weight rows per wave

// Geometry that follows from NG.
template <int NG>
struct MxGeom {
  static_assert(NG >= 2 && NG % 2 == 0, "a wave pairs NG/2 gate groups with NG/2 up groups");
  static constexpr int kStepLoads = kMxCopies + 4 * NG;  // load instructions per wave per step
  // the wave's memory counter holds 63 loads: two steps of them in flight where they fit
  // One step: the weight registers of a step are loaded while the step before it is
  // contracted.  (Two steps ahead needs a third register set, which at NG = 4 no longer fits
  // two workgroups per compute unit, and the second resident workgroup hides more latency
  // than the deeper queue does.)
  static constexpr int kAhead = 1;
  static constexpr int kStages = kAhead + 1;
  static constexpr int kEpiRow = 16 * NG + 1;  // floats per token in a wave's epilogue tile (+1: bank spread)
  static constexpr size_t kLdsBytes =
      (size_t)kStages * kMxStageChunks * 16 > (size_t)kMxWaves * kGemmBM * kEpiRow * 4
          ? (size_t)kStages * kMxStageChunks * 16
          : (size_t)kMxWaves * kGemmBM * kEpiRow * 4;
  static constexpr int tiles_per_wg(int mode) { return mode == 0 ? 4 * NG : 8 * NG; }
};

__device__ __forceinline__ const char* uniform_ptr(const char* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
}

// Descriptor of a whole weight plane as a raw buffer (no stride, no range to speak of: the
// offsets are tile arithmetic checked on the host).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t plane_rsrc(const void* p) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(uniform_ptr(reinterpret_cast<const char*>(p))), 0,
                                           0x7fffffff, 0x00020000);
}

template <int MODE, int NG>
__global__ __launch_bounds__(64 * kMxWaves, 2) void expert_gemm_mx_kernel(ExpertGemmMxArgs a) {
  using G = MxGeom<NG>;
  constexpr int kStepLoads = G::kStepLoads, kAhead = G::kAhead, kStages = G::kStages;
  extern __shared__ __align__(16) unsigned char smem[];
  uint4* As = reinterpret_cast<uint4*>(smem);  // [kStages][64 tokens][24 chunks]
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
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, and known to be
  const int n32 = lane & 31, kg = lane >> 5;
  const int n16 = n32 & 15, th = n32 >> 4;  // row within a packed tile, tile of the pair
  const int nblk = a.nblk;
  const int nsteps = (nblk + 3) >> 2;
  const int slots = scale_slots(nblk);

  // Group g of this wave is the pair of packed tiles (t0(g), t0(g) + 1).  Every address of
  // the main loop is a wave-uniform base (the group's plane and tile pair, advanced per step
  // on the scalar unit) plus a 32-bit per-lane byte offset that never changes and is the
  // same for every group, so the loads cost no vector instructions.  Nothing is clamped
  // along K: activation rows are padded with zero blocks to a whole number of steps, so
  // the weight blocks read past K (the next tile's, or the slack behind the last plane)
  // and the scale bytes read past K (slot padding, 127) are multiplied by exact zeros.
  // Groups past the last tile (ragged last N tile) re-read the last pair; their results
  // are dropped.
  auto group_tile = [&](int g) {
    if (MODE == 0) return nt * (4 * NG) + wv * NG + 2 * (g % (NG / 2));
    return nt * (8 * NG) + wv * (2 * NG) + 2 * g;
  };
  // One buffer descriptor per weight plane; a group's tile pair and the K step go into the
  // scalar offset of the load, the lane's place within the pair into the vector offset.
  const ExpertW& w = wd->w;
  const auto q_rsrc0 = plane_rsrc(MODE == 0 ? w.q_gate : w.q_down);
  const auto q_rsrc1 = plane_rsrc(MODE == 0 ? w.q_up : w.q_down);
  const auto s_rsrc0 = plane_rsrc(MODE == 0 ? w.s_gate : w.s_down);
  const auto s_rsrc1 = plane_rsrc(MODE == 0 ? w.s_up : w.s_down);
  uint32_t goff_q[NG], goff_s[NG];  // byte offset of the group's tile pair in its planes
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int tc = min(group_tile(g), a.ntile - 2);
    goff_q[g] = (uint32_t)__builtin_amdgcn_readfirstlane(tc * nblk * 256);
    goff_s[g] = (uint32_t)__builtin_amdgcn_readfirstlane(tc * 256 * slots);
  }
  const uint32_t qoff = (uint32_t)(((th * nblk + kg) * 16 + n16) * 16);  // entry (tile th, block kg, row)
  const uint32_t soff = (uint32_t)scale_index(th, kg, n16, slots);
  const int rowblk = mx3_row_blocks(nblk);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  // Copy instruction c of wave wv fills chunks [(kMxCopies wv + c) * 64, +64) of the
  // stage, in token-major order; the lane's chunk is physical position pc of token tl
  // and holds logical chunk lc (XOR swizzle on the low three bits).
  uint32_t aoff[kMxCopies];  // byte offset of this lane's chunk at step 0 from a.A
#pragma unroll
  for (int c = 0; c < kMxCopies; ++c) {
    const int lin = (kMxCopies * wv + c) * 64 + lane;
    const int tl = lin / kMxRowChunks, pc = lin - tl * kMxRowChunks;
    const int lc = (pc & ~7) | ((pc & 7) ^ ((tl >> 1) & 7));
    const int tlc = min(tl, mcount - 1);  // tokens past the tile re-read its last one
    const int row = a.list_row ? a.list_row[base + tlc] : base + tlc;
    aoff[c] = (uint32_t)(((size_t)row * rowblk * kMx3ChunksPerBlock + lc) * 16);
  }
  // LDS destination of copy c of this wave within a stage (wave-uniform)
  const uint32_t lds_wave = lds0 + (uint32_t)(kMxCopies * wv * 64 * 16);
  struct BSet {
    u32x4 q[2][NG];     // [64-wide K chunk of the step][row group]
    uint32_t s[2][NG];  // byte 0 = the block's scale byte (the matrix instruction reads only that byte)
  };
  // The kStepLoads load instructions of step j, one at a time: n < kMxCopies copies a part
  // of the activation tile into LDS, the next 2 NG fetch the weight entries, the last 2 NG
  // the scale bytes.  The LDS copies are inline assembly (nothing of theirs lives in a
  // register; the explicit wait at the step boundary guarantees their arrival).
  auto issue_load = [&](int n, int stage, BSet& b, int j) {
    if (n < kMxCopies) {
      const char* abase = reinterpret_cast<const char*>(a.A) + (size_t)j * (4 * kMx3ChunksPerBlock * 16);
      const uint32_t lds = lds_wave + (uint32_t)((stage * kMxStageChunks + n * 64) * 16);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(aoff[n]), "s"(abase), "s"(lds)
                   : "memory");
    } else {
      // Weights: buffer loads the compiler can see.  Loads hidden in inline assembly would
      // save its wait bookkeeping, but the register allocator moves values between register
      // files around the matrix instructions, and a register it moves while an untracked load
      // is still in flight takes stale data along (seen as rare wrong rows in ragged tiles).
      const int m = (n - kMxCopies) % (2 * NG), kc = m / NG, g = m % NG;
      const bool second = MODE == 0 && g >= NG / 2;  // up rows
      if (n < kMxCopies + 2 * NG) {
        const uint32_t so = goff_q[g] + (uint32_t)j * 1024u + (uint32_t)kc * 512u;
        b.q[kc][g] = __builtin_amdgcn_raw_buffer_load_b128(second ? q_rsrc1 : q_rsrc0, qoff, so, 0);
      } else {
        // the block's scale byte (the matrix instruction reads only byte 0 of its scale operand)
        const uint32_t so = goff_s[g] + (uint32_t)(((j & 3) * 64 + 32 * kc) * slots + (j >> 2));
        b.s[kc][g] = __builtin_amdgcn_raw_buffer_load_b8(second ? s_rsrc1 : s_rsrc0, soff, so, 0);
      }
    }
  };
  auto load_all = [&](int stage, BSet& b, int j) {
#pragma unroll
    for (int n = 0; n < kStepLoads; ++n) issue_load(n, stage, b, j);
  };

  floatx16 acc[2][NG];  // [32-token sub-tile][row group]
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ms][g][r] = 0.0f;

  const int sw = (n32 >> 1) & 7;
  // Fragment i = (kc, term, 32-token sub-tile) of a step feeds NG matrix instructions (the
  // wave's row groups).  Fragments are requested from LDS two ahead of their use.  The loads
  // of the step being prefetched are issued a few per fragment between the matrix
  // instructions rather than in a burst at the step boundary: the texture address unit
  // takes 16 cycles per 64-lane 128-bit load, and a burst per wave would hold every wave at
  // the start of the step.
  auto compute = [&](const BSet& b, int stage, BSet& bn, int stage_n, int jn) {
    const u32x4* at = reinterpret_cast<const u32x4*>(As) + stage * kMxStageChunks;
    u32x4 flo[3], fhi[3];
    auto read_frag = [&](int i) {
      const int kc = i / 6, t = (i % 6) >> 1, ms = i & 1;
      const int c0 = ((2 * kc + kg) * kMx3Terms + t) * 2;
      const int tok = ms * 32 + n32;
      flo[i % 3] = at[tok * kMxRowChunks + ((c0 & ~7) | ((c0 & 7) ^ sw))];
      fhi[i % 3] = at[tok * kMxRowChunks + (((c0 + 1) & ~7) | (((c0 + 1) & 7) ^ sw))];
    };
    read_frag(0);
    read_frag(1);
#pragma unroll
    for (int i = 0; i < 12; ++i) {
      const int kc = i / 6, ms = i & 1;
      if (i + 2 < 12) read_frag(i + 2);
#pragma unroll
      for (int n = i; n < kStepLoads; n += 12) issue_load(n, stage_n, bn, jn);
      __builtin_amdgcn_sched_barrier(0);
      // FP6 reads the first six registers; fhi[2] (register 6) is the term's scale byte
      i32x8 aw = (i32x8)__builtin_shufflevector(flo[i % 3], fhi[i % 3], 0, 1, 2, 3, 4, 5, 6, 7);
      // the fragment stays in ordinary vector registers: left to itself the register allocator
      // parks fragments in accumulation registers that it frees by moving parts of an
      // accumulator tile out and back around the matrix instructions
      asm volatile("" : "+v"(aw));
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        // FP4 reads four registers
        const i32x8 bw = (i32x8)__builtin_shufflevector(b.q[kc][g], b.q[kc][g], 0, 1, 2, 3, -1, -1, -1, -1);
        acc[ms][g] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aw, bw, acc[ms][g], 2, 4, 0,
                                                                     aw[6], 0, (int)b.s[kc][g]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // kStages LDS stages and register sets, loads kAhead steps ahead.  The step boundary is
  // an explicit wait + bare barrier: everything this wave requested for step j (during step
  // j - kAhead) has landed once at most (kAhead - 1) steps' worth of its loads are still in
  // flight (loads retire in order), and the barrier extends that to the other waves' parts
  // of the activation tile and tells that every wave is done reading the stage about to
  // be overwritten.
  constexpr int kInFlight = (kAhead - 1) * kStepLoads;
  constexpr int kWaitStep = (kInFlight & 15) | (7 << 4) | (15 << 8) | ((kInFlight >> 4) << 14);
  BSet bs[kStages];
#pragma unroll
  for (int u = 0; u < kAhead; ++u) load_all(u, bs[u], min(u, nsteps - 1));
  // the loop is entered with nothing in flight, so that its body is the steady state from the first iteration on
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0)
#pragma unroll
  for (int u = 0; u < kAhead; ++u)
#pragma unroll
    for (int kc = 0; kc < 2; ++kc)
#pragma unroll
      for (int g = 0; g < NG; ++g) asm volatile("" : "+v"(bs[u].q[kc][g]), "+v"(bs[u].s[kc][g]));
  __builtin_amdgcn_sched_barrier(0);
  auto step = [&](int u, int jj) {
    __builtin_amdgcn_s_waitcnt(kWaitStep);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    compute(bs[u], u, bs[(u + kAhead) % kStages], (u + kAhead) % kStages, min(jj + kAhead, nsteps - 1));
    __builtin_amdgcn_sched_barrier(0);
  };
  static_assert(kStages == 2, "the K loop below alternates two stages");
  for (int j = 0;; j += 2) {  // (exits in the middle rather than a conditional second step: no join inside the loop)
    step(0, j);
    if (j + 1 >= nsteps) break;
    step(1, j + 1);
    if (j + 2 >= nsteps) break;
  }
  // the copies requested past the last step are still in flight: nothing may reuse their LDS before they land
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0)
  __builtin_amdgcn_sched_barrier(0);

  // epilogue: lane holds weight row n32 of each group; accumulator register r is token
  // (r % 4) + 8 * (r / 4) + 4 * kg of the 32-token sub-tile
  if (MODE == 0) {
    // bias + activation into this wave's LDS tile as fp32 [token][16 NG features + 1], then
    // one lane per token re-quantises 32 features at a time to the three-term format
    __syncthreads();  // the copies issued for the steps after the last have landed; all waves are past their reads
    float* tile = reinterpret_cast<float*>(smem) + (size_t)wv * kGemmBM * G::kEpiRow;
#pragma unroll
    for (int gi = 0; gi < NG / 2; ++gi) {
      const int row = group_tile(gi) * 16 + n32;  // feature
      const bool rv = row < a.N;
      const float bg = rv ? wd->w.b_gate[row] : 0.0f;
      const float bu = rv ? wd->w.b_up[row] : 0.0f;
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
          // features past N belong to the zero padding of the output rows
          tile[tl * G::kEpiRow + 32 * gi + n32] =
              rv ? moe_activation(acc[ms][gi][r] + bg, acc[ms][NG / 2 + gi][r] + bu, a.act_type) : 0.0f;
        }
      }
    }
    __syncthreads();
    const int tl = lane;
    const int out_rowblk = mx3_row_blocks(a.N >> 5);  // the down GEMM reads rows padded to whole steps
#pragma unroll 1
    for (int bi = 0; bi < NG / 2; ++bi) {
      const int kb = (nt * (4 * NG) + wv * NG) / 2 + bi;
      if (tl < mcount && kb < out_rowblk) {
        float v[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = tile[tl * G::kEpiRow + 32 * bi + i];
        u32x4 out[kMx3ChunksPerBlock];
        mx3_quantize_block(v, out);
        u32x4* o = a.act_out + ((size_t)(base + tl) * out_rowblk + kb) * kMx3ChunksPerBlock;
#pragma unroll
        for (int c = 0; c < kMx3ChunksPerBlock; ++c) o[c] = out[c];
      }
    }
  } else {
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const int row = group_tile(g) * 16 + n32;
      if (row >= a.N) continue;
      const float bd = wd->w.b_down[row];
#pragma unroll
      for (int ms = 0; ms < 2; ++ms) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
          if (tl >= mcount) continue;
          a.y_out[(size_t)(base + tl) * (size_t)a.N + row] = acc[ms][g][r] + bd;
        }
      }
    }
  }
}

}  // namespace csk
