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
// A workgroup of eight waves owns 64 tokens of one expert x 256 features (gate and
// up rows together) or 512 down rows, and walks K in steps of 128 (4 blocks); the
// kernel is bound by what the compute units can pull from L2, and the activation
// tile is fetched once per workgroup, so the wide tile is what sets its speed.  The
// activation tile (64 tokens x 4 blocks x 3 terms x 32 B) goes to LDS by
// global_load_lds with a 16-byte XOR swizzle applied on the source side; weights
// go straight to registers; both are requested two steps ahead (three LDS stages, one
// barrier per step).
// The gate/up epilogue applies bias + SwiGLU, stages the 64 x 128 tile in LDS as
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
  int ntile;             // ceil(N / 16) weight row tiles
  int n_ntiles;          // N tiles per M tile: ceil(ntile / 16) (MODE 0) or ceil(ntile / 32)
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
constexpr int kStepLoads = kMxCopies + 2 * 2 * 2;                 // load instructions per wave per step

template <int MODE>
__global__ __launch_bounds__(64 * kMxWaves, 8 / kMxWaves) void expert_gemm_mx_kernel(ExpertGemmMxArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint4* As = reinterpret_cast<uint4*>(smem);  // [3 stages][64 tokens][24 chunks]
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
  const int n32 = lane & 31, kg = lane >> 5;
  const int n16 = n32 & 15, th = n32 >> 4;  // row within a packed tile, tile of the pair
  const int nblk = a.nblk;
  const int nsteps = (nblk + 3) >> 2;
  const int slots = scale_slots(nblk);

  // this wave's two 32-row groups (each a pair of packed tiles).  Every address of the main
  // loop is a wave-uniform base (advanced per step on the scalar unit) plus a 32-bit per-lane
  // byte offset that never changes, so the loads cost no vector instructions.  Nothing is
  // clamped: activation rows are padded with zero blocks to a whole number of steps, so the
  // weight blocks read past K (the next tile's, or the slack behind the last plane) and the
  // scale bytes read past K (slot padding, 127) are multiplied by exact zeros.
  int tiles[2];  // this lane's packed tile in each group
  const char* qbase[2];
  const char* sbase[2];
  uint32_t qoff[2], soff[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    int t;
    if (MODE == 0) t = nt * (2 * kMxWaves) + wv * 2 + th;
    else t = nt * (4 * kMxWaves) + wv * 4 + 2 * s + th;
    tiles[s] = t;
    const int tc = min(t, a.ntile - 1);
    const uint4* qb = MODE == 0 ? (s == 0 ? wd->w.q_gate : wd->w.q_up) : wd->w.q_down;
    const uint8_t* sb = MODE == 0 ? (s == 0 ? wd->w.s_gate : wd->w.s_up) : wd->w.s_down;
    qbase[s] = reinterpret_cast<const char*>(qb);
    sbase[s] = reinterpret_cast<const char*>(sb);
    qoff[s] = (uint32_t)((((size_t)tc * nblk + kg) * 16 + n16) * 16);  // entry (tile, block kg, row)
    soff[s] = (uint32_t)scale_index(tc, kg, n16, slots);
  }
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
  const uint32_t lds_wave = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(kMxCopies * wv * 64 * 16);
  struct BSet {
    u32x4 q[2][2];     // [64-wide K chunk of the step][row group]
    uint32_t s[2][2];  // byte 0 = the block's scale byte (the matrix instruction reads only that byte)
  };
  // The kStepLoads load instructions of step j, one at a time: n < kMxCopies copies a part
  // of the activation tile into LDS, the next four fetch the weight entries, the last four
  // the scale bytes.
  // All loads are inline assembly in the scalar-base form.  Besides saving the address
  // arithmetic this keeps them out of the compiler's wait tracking, which otherwise drains
  // the whole queue once per loop iteration over a register it reuses; the explicit count at
  // the step boundary is what guarantees their arrival.
  auto issue_load = [&](int n, int stage, BSet& b, int j) {
    if (n < kMxCopies) {
      const char* abase = reinterpret_cast<const char*>(a.A) + (size_t)j * (4 * kMx3ChunksPerBlock * 16);
      const uint32_t lds = lds_wave + (uint32_t)((stage * kMxStageChunks + n * 64) * 16);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(aoff[n]), "s"(abase), "s"(lds)
                   : "memory");
    } else {
      const int m = (n - kMxCopies) & 3, kc = m >> 1, s = m & 1;
      if (n < kMxCopies + 4) {
        const char* base_q = qbase[s] + (size_t)j * 1024 + kc * 512;
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(b.q[kc][s]) : "v"(qoff[s]), "s"(base_q) : "memory");
      } else {
        // a dword load at the byte's own (unaligned) address: the matrix instruction reads
        // only byte 0 of its scale operand, so no widening instruction is needed
        const char* base_s = sbase[s] + (size_t)((j & 3) * 64 + 32 * kc) * slots + (j >> 2);
        asm volatile("global_load_dword %0, %1, %2" : "=v"(b.s[kc][s]) : "v"(soff[s]), "s"(base_s) : "memory");
      }
    }
  };
  auto copy_a = [&](int stage, int j) {
    BSet unused;
#pragma unroll
    for (int c = 0; c < kMxCopies; ++c) issue_load(c, stage, unused, j);
  };
  auto load_b = [&](BSet& b, int j) {
#pragma unroll
    for (int n = kMxCopies; n < kMxCopies + 8; ++n) issue_load(n, 0, b, j);
  };

  floatx16 acc[2][2];  // [32-token sub-tile][row group]
#pragma unroll
  for (int ms = 0; ms < 2; ++ms)
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ms][s][r] = 0.0f;

  const int sw = (n32 >> 1) & 7;
  // Fragment i = (kc, term, 32-token sub-tile) of a step feeds two matrix instructions
  // (the two row groups).  Fragments are requested from LDS two ahead of their use, so
  // the LDS latency is covered by the four matrix instructions in between.
  // The loads of the step after next are issued one per fragment between the matrix
  // instructions rather than in a burst at the step boundary: the texture address unit
  // takes 16 cycles per 64-lane 128-bit load, and a burst of 14 per wave, 8 waves per
  // compute unit, held every wave at the start of the step for longer than the step's
  // matrix work.
  auto compute = [&](const BSet& b, int stage, int j, BSet& bn, int stage_n, int jn) {
    const u32x4* at = reinterpret_cast<const u32x4*>(As) + stage * kMxStageChunks;
    i32x8 bw[2][2];
#pragma unroll
    for (int kc = 0; kc < 2; ++kc)
#pragma unroll
      for (int s = 0; s < 2; ++s)  // FP4 reads four registers
        bw[kc][s] = (i32x8)__builtin_shufflevector(b.q[kc][s], b.q[kc][s], 0, 1, 2, 3, -1, -1, -1, -1);
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
      issue_load(i, stage_n, bn, jn);
      if (i + 12 < kStepLoads) issue_load(i + 12, stage_n, bn, jn);
      __builtin_amdgcn_sched_barrier(0);
      // FP6 reads the first six registers; fhi[2] (register 6) is the term's scale byte
      const i32x8 aw = (i32x8)__builtin_shufflevector(flo[i % 3], fhi[i % 3], 0, 1, 2, 3, 4, 5, 6, 7);
      acc[ms][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aw, bw[kc][0], acc[ms][0], 2, 4, 0,
                                                                   (int)fhi[i % 3][2], 0, (int)b.s[kc][0]);
      acc[ms][1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aw, bw[kc][1], acc[ms][1], 2, 4, 0,
                                                                   (int)fhi[i % 3][2], 0, (int)b.s[kc][1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Three LDS stages, loads two steps ahead.  A __syncthreads() would drain every
  // outstanding load (its fence waits for vmcnt(0)), so the step boundary is an explicit
  // count + bare barrier: a wave's loads of step j are older than the kStepLoads loads of
  // step j+1, memory counters retire in order, so vmcnt(kStepLoads) means "my part of
  // step j has landed", and the barrier extends that to the other waves' parts and
  // tells that every wave is done reading the stage about to be overwritten.
  constexpr int kWaitStep = (kStepLoads & 15) | (7 << 4) | (15 << 8) | ((kStepLoads >> 4) << 14);
  // The first two steps are requested and awaited in full before the loop, so that the
  // loop is entered with nothing in flight and its body is the steady state from the
  // first iteration on (loads still pending at the loop entry would make the compiler's
  // own wait insertion fall back to vmcnt(0) inside the loop).
  BSet bs[3];
  copy_a(0, 0);
  load_b(bs[0], 0);
  copy_a(1, min(1, nsteps - 1));
  load_b(bs[1], min(1, nsteps - 1));
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0)
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int kc = 0; kc < 2; ++kc)
#pragma unroll
      for (int g = 0; g < 2; ++g)  // "use" the loaded registers so the compiler, too, knows they have arrived
        asm volatile("" : "+v"(bs[i].q[kc][g]), "+v"(bs[i].s[kc][g]));
  __builtin_amdgcn_sched_barrier(0);
  auto step = [&](int u, int jj) {
    __builtin_amdgcn_s_waitcnt(kWaitStep);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    compute(bs[u], u, jj, bs[(u + 2) % 3], (u + 2) % 3, min(jj + 2, nsteps - 1));
    __builtin_amdgcn_sched_barrier(0);
  };
  // no control-flow joins between the steps of the steady state
  for (int j = 0;; j += 3) {
    step(0, j);
    if (j + 1 >= nsteps) break;
    step(1, j + 1);
    if (j + 2 >= nsteps) break;
    step(2, j + 2);
    if (j + 3 >= nsteps) break;
  }
  // The re-reads requested past the last step are still in flight and the compiler does
  // not know it (those loads are inline assembly): nothing may follow the loop before
  // they have landed, or a register they are about to overwrite could be given a new role.
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0)
  __builtin_amdgcn_sched_barrier(0);

  // epilogue: lane holds weight row n32 of each group; accumulator register r is token
  // (r % 4) + 8 * (r / 4) + 4 * kg of the 32-token sub-tile
  if (MODE == 0) {
    // bias + activation into LDS as fp32 [token][block = wave][32 + 1], then one thread per
    // (token, block) re-quantises 32 features to the three-term format
    __syncthreads();  // the copies issued for the step after the last have landed; all waves are past their reads
    float* stage = reinterpret_cast<float*>(smem);
    const int row = tiles[0] * 16 + n16;  // feature
    const bool rv = tiles[0] < a.ntile && row < a.N;
    const float bg = rv ? wd->w.b_gate[row] : 0.0f;
    const float bu = rv ? wd->w.b_up[row] : 0.0f;
#pragma unroll
    for (int ms = 0; ms < 2; ++ms) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
        // features past N belong to the zero padding of the output rows
        stage[(tl * kMxWaves + wv) * 33 + n32] =
            rv ? moe_activation(acc[ms][0][r] + bg, acc[ms][1][r] + bu, a.act_type) : 0.0f;
      }
    }
    __syncthreads();
    const int tl = threadIdx.x / kMxWaves, blk = threadIdx.x % kMxWaves;
    const int kb = nt * kMxWaves + blk;
    const int out_rowblk = mx3_row_blocks(a.N >> 5);  // the down GEMM reads rows padded to whole steps
    if (tl < mcount && kb < out_rowblk) {
      float v[32];
#pragma unroll
      for (int i = 0; i < 32; ++i) v[i] = stage[(tl * kMxWaves + blk) * 33 + i];
      u32x4 out[kMx3ChunksPerBlock];
      mx3_quantize_block(v, out);
      u32x4* o = a.act_out + ((size_t)(base + tl) * out_rowblk + kb) * kMx3ChunksPerBlock;
#pragma unroll
      for (int c = 0; c < kMx3ChunksPerBlock; ++c) o[c] = out[c];
    }
  } else {
#pragma unroll
    for (int ms = 0; ms < 2; ++ms) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int tl = ms * 32 + (r & 3) + 8 * (r >> 2) + 4 * kg;
        if (tl >= mcount) continue;
        const size_t p = (size_t)(base + tl);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int row = tiles[s] * 16 + n16;
          if (tiles[s] < a.ntile && row < a.N) a.y_out[p * (size_t)a.N + row] = acc[ms][s][r] + wd->w.b_down[row];
        }
      }
    }
  }
}

}  // namespace csk
