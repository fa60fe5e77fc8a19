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
// A workgroup of four waves owns 64 tokens of one expert (32 for the tail of an expert's
// token list) x (128 NG) weight rows -- gate and up rows of the same 64 NG features
// together, or 128 NG down rows -- and walks K in steps of 128 (4 blocks).  A wave owns NG
// groups of 32 weight rows (NG/2 gate groups and the NG/2 up groups of the same features)
// for all the tokens: NG x 2 accumulator tiles of 32 x 32, kept in the accumulation half
// of the register file, which they fill.  The activations are the expensive operand
// (three terms of 32 bytes per 32 values against 17 bytes of weights), so the tile is tall
// in weight rows: every activation fragment read from LDS feeds NG matrix instructions,
// and NG = 4 is what still leaves two workgroups per compute unit.
// The activation tile (64 tokens x 4 blocks x 3 terms x 32 B) goes to LDS by
// global_load_lds with a 16-byte XOR swizzle applied on the source side; weights go
// straight to registers; both are requested one step ahead (two LDS stages and register
// sets, one barrier per step), the weights of the step's second K half half a step later
// than the rest, so that no request is waited for sooner than half a step after it was
// made.
// Where a work unit's time goes (cycle counter per unit, 120b shape, 4096 tokens, two
// workgroups per compute unit at a shader clock of about 1.6 GHz): 67 us in all -- 10 us
// until the first step's operands have landed (descriptor chain, token rows, then the
// loads themselves, which take twice as long as on an idle memory system), 49 us in the K
// loop (2.1 us per step of 48 matrix instructions per wave: with the instruction at 32
// cycles the matrix pipe is 46 % busy when one workgroup of the compute unit is in its
// loop and the other is not, which is the case 56 % of the time), 8 us of epilogue.  One
// workgroup per compute unit reaches the same throughput as two (the clock rises to
// 1.9 GHz): the kernel is not short of occupancy.  With every weight request answered by
// the L2 (all units reading one tile pair: wrong results, timing only) gate/up takes 461
// instead of 558 us, so about a sixth of the time is the memory system behind the L2.
// The accumulators start from the bias.  The gate/up epilogue applies SwiGLU (hardware exp
// and reciprocal), stages each wave's 64 x 16 NG tile in LDS as fp32 and re-quantises it
// to the three-term format the down GEMM reads.
//
// Restates include/coalsack/nn/nn_ops/expert_mlp_node.h:651-732 with the token
// loop of :503-529 as the M dimension.
#pragma once
#include "common.h"
#include "expert_stream_kernel.h"
#include "mx3.h"

namespace csk {

typedef int i32x8 __attribute__((ext_vector_type(8)));

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

constexpr int kGemmBM = 64;  // tokens per M tile of the dispatch kernels' tile list
constexpr int kDies = 8;     // accelerator dies (XCDs) of the part, each with a private L2

constexpr int kMxRowChunks = 4 * kMx3ChunksPerBlock;  // 24 chunks per token per step
constexpr int kMxWaves = 4;                           // waves per workgroup
constexpr int kMxNG = 4;                              // groups of 32 weight rows per wave

// Geometry that follows from NG (32-row weight groups per wave) and MS (32-token sub-tiles
// per work unit: 2 for an M tile of more than 32 tokens, 1 for the tail of an expert's list).
template <int NG, int MS>
struct MxGeom {
  static_assert(NG >= 2 && NG % 2 == 0, "a wave pairs NG/2 gate groups with NG/2 up groups");
  static_assert(MS == 1 || MS == 2, "one or two 32-token sub-tiles");
  static constexpr int kBM = 32 * MS;                                // tokens per workgroup
  static constexpr int kStageChunks = kBM * kMxRowChunks;            // 16-byte chunks per LDS stage
  static constexpr int kCopies = kStageChunks / 64 / kMxWaves;       // copy instructions per wave per step
  static constexpr int kFrags = 6 * MS;                              // activation fragments per step
  static constexpr int kStages = 2;
  static constexpr int kEpiRow = 16 * NG + 1;  // floats per token in a wave's epilogue tile (+1: bank spread)
  static constexpr size_t kLdsBytes =
      (size_t)kStages * kStageChunks * 16 > (size_t)kMxWaves * kBM * kEpiRow * 4
          ? (size_t)kStages * kStageChunks * 16
          : (size_t)kMxWaves * kBM * kEpiRow * 4;
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

typedef __attribute__((address_space(3))) const u32x4 lds_u32x4;

// One work unit: M tile (expert `wd`, tokens [m0, m0 + mcount) of its list) x N tile nt.
// MS = 2 for M tiles that hold more than 32 tokens, MS = 1 for those that hold at most 32
// (the ragged end of an expert's token list), so that a tail of a few tokens costs one
// 32-token sub-tile of matrix work instead of two.
template <int MODE, int NG, int MS>
__device__ __forceinline__ void expert_gemm_mx_unit(const ExpertGemmMxArgs& a, const WorkDesc* wd, int m0, int mcount,
                                                    int nt, unsigned char* smem) {
  using G = MxGeom<NG, MS>;
  constexpr int kCopies = G::kCopies, kStages = G::kStages;
  constexpr int kStageChunks = G::kStageChunks, kFrags = G::kFrags, kBM = G::kBM;
  const int base = wd->base + m0;
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
  // are dropped.  A wave none of whose groups exists (the ragged last N tile again: with
  // 2880 features three of its four waves) issues no matrix instructions at all and only
  // takes its part in copying the activation tile, which leaves its share of the matrix
  // pipe to the other workgroup on the compute unit.
  auto group_tile = [&](int g) {
    if (MODE == 0) return nt * (4 * NG) + wv * NG + 2 * (g % (NG / 2));
    return nt * (8 * NG) + wv * (2 * NG) + 2 * g;
  };
  const bool idle_wave = __builtin_amdgcn_readfirstlane((int)(group_tile(0) >= a.ntile)) != 0;
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

  // LDS image of a stage: [token][24 chunks].  A token's chunks of one step are ordered by
  // the index 4 f + 2 kg + h -- f = 3 kc + term (kc: 64-wide half of the step), kg: which
  // 32-value block of that half, h: low / high 16 bytes of the term -- and chunk index c of
  // token tl sits at physical position (c & ~7) | ((c & 7) ^ ((tl >> 1) & 7)): the sixteen
  // lanes that read one chunk index of sixteen consecutive tokens then hit sixteen
  // different 16-byte bank groups.  Because kg and h occupy bits of their own in the index,
  // the swizzled position of every fragment is one of four per-lane addresses
  // (frag_addr[f & 1][h]) plus a constant.
  // Copy instruction c of wave wv fills chunks [(kCopies wv + c) * 64, +64) of the stage
  // (the LDS destinations of the instruction are fixed: lane order), so the swizzle and the
  // chunk order are applied on the source side: each lane fetches the chunk that belongs
  // at its position.
  uint32_t aoff[kCopies];  // byte offset of this lane's chunk at step 0 from a.A
#pragma unroll
  for (int c = 0; c < kCopies; ++c) {
    const int lin = (kCopies * wv + c) * 64 + lane;
    const int tl = lin / kMxRowChunks, pc = lin - tl * kMxRowChunks;
    const int ci = (pc & ~7) | ((pc & 7) ^ ((tl >> 1) & 7));        // chunk index 4 f + 2 kg + h
    const int f = ci >> 2, ckg = (ci >> 1) & 1, h = ci & 1;
    const int gch = ((2 * (f / 3) + ckg) * kMx3Terms + f % 3) * 2 + h;  // chunk of the row's step in memory
    const int tlc = min(tl, mcount - 1);  // tokens past the tile re-read its last one
    const int row = a.list_row ? a.list_row[base + tlc] : base + tlc;
    aoff[c] = (uint32_t)(((size_t)row * rowblk * kMx3ChunksPerBlock + gch) * 16);
  }
  uint32_t frag_addr[2][2];
#pragma unroll
  for (int fb = 0; fb < 2; ++fb)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      frag_addr[fb][h] = lds0 + (uint32_t)((n32 * kMxRowChunks + (((fb << 2) | h) ^ (kg << 1) ^ ((n32 >> 1) & 7))) * 16);
  // LDS destination of copy c of this wave within a stage (wave-uniform)
  const uint32_t lds_wave = lds0 + (uint32_t)(kCopies * wv * 64 * 16);
  struct BSet {
    u32x4 q[2][NG];     // [64-wide K chunk of the step][row group]
    uint8_t s[2][NG];   // the block's scale byte (widened where it is used: widening it where it is loaded would wait for the load there)
  };
  // copy c of the activation tile of step j into LDS stage `stage` (inline assembly: nothing
  // of it lives in a register; the explicit wait at the step boundary guarantees its arrival)
  auto issue_copy = [&](int c, int stage, int j) {
    const char* abase = reinterpret_cast<const char*>(a.A) + (size_t)j * (4 * kMx3ChunksPerBlock * 16);
    const uint32_t lds = lds_wave + (uint32_t)((stage * kStageChunks + c * 64) * 16);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(aoff[c]), "s"(abase), "s"(lds)
                 : "memory");
  };
  // Weights: buffer loads the compiler can see.  Loads hidden in inline assembly would
  // save its wait bookkeeping, but the register allocator moves values between register
  // files around the matrix instructions, and a register it moves while an untracked load
  // is still in flight takes stale data along (seen as rare wrong rows in ragged tiles).
  auto issue_q = [&](int kc, int g, BSet& b, int j) {
    const bool second = MODE == 0 && g >= NG / 2;  // up rows
    const uint32_t so = goff_q[g] + (uint32_t)j * 1024u + (uint32_t)kc * 512u;
    b.q[kc][g] = __builtin_amdgcn_raw_buffer_load_b128(second ? q_rsrc1 : q_rsrc0, qoff, so, 0);
  };
  auto issue_s = [&](int kc, int g, BSet& b, int j) {
    const bool second = MODE == 0 && g >= NG / 2;
    // the block's scale byte (the matrix instruction reads only byte 0 of its scale operand)
    const uint32_t so = goff_s[g] + (uint32_t)(((j & 3) * 64 + 32 * kc) * slots + (j >> 2));
    b.s[kc][g] = __builtin_amdgcn_raw_buffer_load_b8(second ? s_rsrc1 : s_rsrc0, soff, so, 0);
  };
  // The loads of step j are issued in two parts, each spread over the fragments of half a
  // step: first the activation tile and the weights of the step's first K half, then the
  // weights of its second K half.  Loads retire in order, so at the step boundary only the
  // first part has to have landed -- the 2 NG loads of the second part stay in flight and are
  // waited for in the middle of the next step, which gives every load at least half a step
  // of lead (with one wait for everything at the boundary the last loads issued had none).
  constexpr int kHalf = kFrags / 2;
  constexpr int kFragBufs = 3;  // fragments are requested from LDS kFragBufs - 1 ahead of their use
  auto issue_part = [&](int part, int x, int stage, BSet& b, int j) {  // item x of a part
    if (part == 0) {
      if (x < kCopies) issue_copy(x, stage, j);
      if (x < NG) {
        issue_q(0, x, b, j);
        issue_s(0, x, b, j);
      }
    } else if (x < NG) {
      issue_q(1, x, b, j);
      issue_s(1, x, b, j);
    }
  };
  constexpr int kPart0Items = kCopies > NG ? kCopies : NG;

  constexpr int kWaitAll = (7 << 4) | (15 << 8);  // vmcnt(0)
  if (idle_wave) {
    // the same sequence of copies, waits and barriers as below without the weights and the
    // arithmetic; what this wave owes the output is the zero padding of the rows
#pragma unroll
    for (int c = 0; c < kCopies; ++c) issue_copy(c, 0, 0);
    for (int j = 0; j < nsteps; ++j) {
      __builtin_amdgcn_s_waitcnt(kWaitAll);
      __builtin_amdgcn_s_barrier();
#pragma unroll
      for (int c = 0; c < kCopies; ++c) issue_copy(c, (j + 1) & 1, min(j + 1, nsteps - 1));
    }
    __builtin_amdgcn_s_waitcnt(kWaitAll);
    if (MODE == 0) {
      __syncthreads();
      __syncthreads();
      const int out_rowblk = mx3_row_blocks(a.N >> 5);
      for (int bi = 0; bi < NG / 2; ++bi) {
        const int kb = (nt * (4 * NG) + wv * NG) / 2 + bi;
        if (lane < mcount && kb < out_rowblk) {
          u32x4* o = a.act_out + ((size_t)(base + lane) * out_rowblk + kb) * kMx3ChunksPerBlock;
#pragma unroll
          for (int t = 0; t < kMx3Terms; ++t) {
            o[2 * t] = u32x4{0u, 0u, 0u, 0u};
            o[2 * t + 1] = u32x4{0u, 0u, 127u, 0u};
          }
        }
      }
    }
    return;
  }

  floatx16 acc[MS][NG];  // [32-token sub-tile][row group]

  // Fragment i = (kc, term, 32-token sub-tile) of a step feeds NG matrix instructions (the
  // wave's row groups).  Fragments are requested from LDS two ahead of their use.  The loads
  // of the step being prefetched are issued a few per fragment between the matrix
  // instructions rather than in a burst at the step boundary: the texture address unit
  // takes 16 cycles per 64-lane 128-bit load, and a burst per wave would hold every wave at
  // the start of the step.
  auto compute = [&](const BSet& b, int stage, BSet& bn, int stage_n, int jn, auto prefetch) {
    u32x4 flo[kFragBufs], fhi[kFragBufs];
    auto read_frag = [&](int i) {
      const int kc = i / (3 * MS), t = (i % (3 * MS)) / MS, ms = i % MS;
      const int f = 3 * kc + t;
      const uint32_t off = (uint32_t)((stage * kStageChunks + ms * 32 * kMxRowChunks + (f >> 1) * 8) * 16);
      flo[i % kFragBufs] = *reinterpret_cast<lds_u32x4*>(frag_addr[f & 1][0] + off);
      fhi[i % kFragBufs] = *reinterpret_cast<lds_u32x4*>(frag_addr[f & 1][1] + off);
    };
#pragma unroll
    for (int i = 0; i < kFragBufs - 1; ++i) read_frag(i);
#pragma unroll
    for (int i = 0; i < kFrags; ++i) {
      const int kc = i / (3 * MS), ms = i % MS;
      if (i + kFragBufs - 1 < kFrags) read_frag(i + kFragBufs - 1);
      if constexpr (!decltype(prefetch)::value) {
        // the last step of an odd count: nothing left to request
      } else
#pragma unroll
      for (int x = i % kHalf; x < (i < kHalf ? kPart0Items : NG); x += kHalf) issue_part(i / kHalf, x, stage_n, bn, jn);
      __builtin_amdgcn_sched_barrier(0);
      // FP6 reads the first six registers; fhi[2] (register 6) is the term's scale byte
      i32x8 aw = (i32x8)__builtin_shufflevector(flo[i % kFragBufs], fhi[i % kFragBufs], 0, 1, 2, 3, 4, 5, 6, 7);
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

  // Two LDS stages and register sets, loads one step ahead.  The step boundary is an explicit
  // wait + bare barrier: the first part of what this wave requested for step j (during step
  // j - 1) has landed once at most the 2 NG loads of the second part are still in flight,
  // and the barrier extends that to the other waves' parts of the activation tile and tells
  // that every wave is done reading the stage about to be overwritten.
  constexpr int kInFlight = 2 * NG;
  constexpr int kWaitStep = (kInFlight & 15) | (7 << 4) | (15 << 8) | ((kInFlight >> 4) << 14);
  // First step: the activation tile and the weights in the order of the steady state, then
  // the biases.
  BSet bs[kStages];
#pragma unroll
  for (int x = 0; x < kPart0Items; ++x) issue_part(0, x, 0, bs[0], 0);
#pragma unroll
  for (int x = 0; x < NG; ++x) issue_part(1, x, 0, bs[0], 0);
  float bias0[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int row = group_tile(g) * 16 + n32;
    const float* bias = MODE == 1 ? wd->w.b_down : (g < NG / 2 ? wd->w.b_gate : wd->w.b_up);
    bias0[g] = row < a.N ? bias[row] : 0.0f;
  }
  // The accumulators start from the bias of the lane's weight row (features past N: zero),
  // so that the epilogue has neither a load nor an addition left to do for it.
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int ms = 0; ms < MS; ++ms)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ms][g][r] = bias0[g];
  // The accumulators live in the accumulation half of the register file (one use of that
  // register class is enough to make the compiler select the matrix instructions' form that
  // accumulates there and to split the wave's 256 registers 128 / 128): they fill it
  // exactly, and the 16-register tiles no longer compete with the weights and fragments for
  // aligned runs of ordinary registers, which made the allocator spill whole tiles.
#pragma unroll
  for (int ms = 0; ms < MS; ++ms)
#pragma unroll
    for (int g = 0; g < NG; ++g) asm volatile("" : "+a"(acc[ms][g]));

  {
    auto step = [&](int u, int jj, auto prefetch) {
      __builtin_amdgcn_s_waitcnt(kWaitStep);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      compute(bs[u], u, bs[u ^ 1], u ^ 1, min(jj + 1, nsteps - 1), prefetch);
      __builtin_amdgcn_sched_barrier(0);
    };
    // Steps in pairs (the two register sets and LDS stages alternate), the last step of an
    // odd count on its own and without requests for a step after it.  One loop body and one
    // back edge: with an exit in the middle of the body the compiler's wait-count pass
    // loses track across the two exits and drains the load queue before the first fragment
    // reads of every step.
    int j = 0;
    for (; j + 1 < nsteps; j += 2) {
      step(0, j, std::true_type{});
      step(1, j + 1, std::true_type{});
    }
    if (j < nsteps) step(0, j, std::false_type{});
  }
  // the copies requested past the last step are still in flight: nothing may reuse their LDS before they land
  __builtin_amdgcn_s_waitcnt(kWaitAll);
  __builtin_amdgcn_sched_barrier(0);

  // epilogue: lane holds weight row n32 of each group; accumulator register r is token
  // (r % 4) + 8 * (r / 4) + 4 * kg of the 32-token sub-tile
  if (MODE == 0) {
    // bias + activation into this wave's LDS tile as fp32 [token][16 NG features + 1], then
    // one lane per token re-quantises 32 features at a time to the three-term format
    __syncthreads();  // the copies issued for the steps after the last have landed; all waves are past their reads
    float* tile = reinterpret_cast<float*>(smem) + (size_t)wv * kBM * G::kEpiRow;
    auto activate = [&](auto act_const) {
      constexpr int kAct = decltype(act_const)::value;
#pragma unroll
      for (int gi = 0; gi < NG / 2; ++gi) {
        const bool rv = group_tile(gi) * 16 + n32 < a.N;  // features past N belong to the zero padding of the output rows
#pragma unroll
        for (int ms = 0; ms < MS; ++ms) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
            const float v = moe_activation(acc[ms][gi][r], acc[ms][NG / 2 + gi][r], kAct);
            tile[tl * G::kEpiRow + 32 * gi + n32] = rv ? v : 0.0f;
          }
          // one pair of accumulator tiles at a time: left to itself the scheduler copies several
          // tiles out of the accumulation registers ahead of their use and spills one of them
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    if (a.act_type == 0) activate(std::integral_constant<int, 0>{});
    else activate(std::integral_constant<int, 1>{});
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
#pragma unroll
      for (int ms = 0; ms < MS; ++ms) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
          if (tl >= mcount) continue;
          a.y_out[(size_t)(base + tl) * (size_t)a.N + row] = acc[ms][g][r];
        }
      }
    }
  }
}

// Work unit = (M tile, N tile), numbered expert by expert (M-tile major for the down
// projection).  Workgroups are handed to the eight accelerator dies round-robin by linear id,
// and each die has its own L2: die x takes the x-th contiguous eighth of the unit sequence,
// so that the workgroups resident on one die at one time share a few activation panels and
// a few experts' weights, which then come from that L2 instead of from memory.
template <int MODE, int NG>
__global__ __launch_bounds__(64 * kMxWaves, 2) void expert_gemm_mx_kernel(ExpertGemmMxArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int n_units = *a.n_mtiles * a.n_ntiles;
  const int per_die = (n_units + kDies - 1) / kDies;
  const int slot = blockIdx.x / kDies;
  const int unit = (blockIdx.x % kDies) * per_die + slot;
  if (slot >= per_die || unit >= n_units) return;
  const int mt = unit / a.n_ntiles;
  int nt = unit - mt * a.n_ntiles;
  const WorkDesc* wd = a.desc + a.mtiles[2 * mt];
  int m0 = a.mtiles[2 * mt + 1];
  if (MODE == 0) {
    // Within an expert's block of the sequence the gate/up units run N tile by N tile, the
    // expert's M tiles side by side: the workgroups resident together then read the same
    // weight rows at about the same time (20b shape, 2048 tokens: 525 -> 506 us per layer;
    // the down projection is no faster that way and keeps the M-tile-major order).
    const int tiles_e = (wd->Te + kGemmBM - 1) / kGemmBM;
    const int r = unit - (mt - m0 / kGemmBM) * a.n_ntiles;  // position within the expert's block
    nt = r / tiles_e;
    m0 = (r - nt * tiles_e) * kGemmBM;
  }
  const int mcount = min(kGemmBM, wd->Te - m0);
  if (mcount <= 32)
    expert_gemm_mx_unit<MODE, NG, 1>(a, wd, m0, mcount, nt, smem);
  else
    expert_gemm_mx_unit<MODE, NG, 2>(a, wd, m0, mcount, nt, smem);
}

}  // namespace csk
