// Shared device/host declarations for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace csk {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes, address-space friendly

constexpr int kWave = 64;
constexpr int kTileRows = 16;   // weight rows per packed tile (= MFMA N)
constexpr int kBlk = 32;        // MXFP4 block length along K
constexpr int kMaxTopK = 16;
constexpr int kMaxExperts = 256;
constexpr int kStreamG = 4;      // tokens per pass of the weight-streaming expert kernel: batches of up to four tokens
constexpr int kStreamGWide = 7;  // ... and larger ones (rows of 9 KiB as three FP6 terms: seven per workgroup leave room for two workgroups per compute unit)

// Resident weights of one expert.  Each matrix [rows, K] is stored as
//   q: [rows/16][K/32][16] x 16 bytes -- byte b of an entry holds elements
//      2b (low nibble) and 2b+1 (high nibble) of one 32-element block, which
//      is the order v_cvt_scalef32_pk_*_fp4 consumes;
//   s: scale bytes (E8M0), per tile [4 waves][64 lanes][slots]: the scale of block kb
//      of row n sits with wave (kb/4)%4, lane (kb%4)*16+n, slot kb/16, so that the
//      wave that owns K steps w, w+4, ... fetches all its scales of a tile with one
//      8-byte load per lane (slots = K steps per wave, rounded up to 8).
// A wave reading entries [kb..kb+3][0..15] of one tile fetches 1 KiB of
// contiguous nibbles; lane (g = lane/16, n = lane%16) owns block kb+g of row n.
struct ExpertW {
  const uint4* q_gate;
  const uint8_t* s_gate;
  const uint4* q_up;
  const uint8_t* s_up;
  const uint4* q_down;
  const uint8_t* s_down;
  const float* b_gate;  // may be null
  const float* b_up;
  const float* b_down;
};

// One entry per active expert, written by the dispatch kernels; entries past
// the active count have Te == 0.
struct WorkDesc {
  int e, Te, base, pad;
  ExpertW w;
};

// One entry per group of tokens of an expert that the streaming kernel contracts in one
// pass over the expert's weights: everything a workgroup needs to start, in one record,
// so that its first weight loads wait for two dependent reads (group count, record), not
// for a chain through the group list and the expert's descriptor.
struct StreamGroup {
  ExpertW w;
  int e;      // expert
  int left;   // tokens of the expert from this group's first on (the group holds min(G, left))
  int base;   // packed position of the group's first token
  int pad;
};

__device__ __forceinline__ void write_stream_group(StreamGroup* g, const ExpertW* w, int e, int left, int base) {
  g->w.q_gate = w->q_gate, g->w.s_gate = w->s_gate, g->w.q_up = w->q_up, g->w.s_up = w->s_up;
  g->w.q_down = w->q_down, g->w.s_down = w->s_down;
  g->w.b_gate = w->b_gate, g->w.b_up = w->b_up, g->w.b_down = w->b_down;
  g->e = e, g->left = left, g->base = base, g->pad = 0;
}

// Pointers read out of device structures are generic to the compiler, which
// would then use FLAT loads (tracked by both memory counters and therefore
// always waited for in full).  These casts pin them to global memory.
#define CSK_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ const CSK_GLOBAL T* as_global(const T* p) {
  return (const CSK_GLOBAL T*)p;
}

// Scale-plane geometry (see ExpertW).
__host__ __device__ inline int scale_slots(int nblk) {
  const int per_wave = (((nblk + 3) >> 2) + 3) >> 2;
  return (per_wave + 7) & ~7;
}
__host__ __device__ inline size_t scale_index(long tile, int kb, int n, int slots) {
  const int j = kb >> 2;
  return ((size_t)tile * 256 + (size_t)(j & 3) * 64 + (kb & 3) * 16 + n) * slots + (j >> 2);
}

// E8M0 byte -> scale of true E2M1 values, 2^(b-127); exact for b in 1..254.
__device__ __forceinline__ float e8m0_scale(uint32_t b) { return __uint_as_float(b << 23); }

__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) { return __uint_as_float(h << 16); }

// Round-to-nearest-even fp32 -> bf16 bit pattern (finite inputs).
__device__ __forceinline__ uint32_t float_to_bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}

// Sum over the 64 lanes, the same value returned in every lane: four cross-lane steps
// inside each row of 16 (quad swaps, half-row and row mirrors -- ordinary vector-ALU
// latency, where a shuffle through the LDS crossbar takes ten times as long), then the four
// row sums through scalar registers.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float a) {
  const int x = __float_as_int(a);
  return a + __int_as_float(__builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror
  const int x = __float_as_int(v);
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(x, 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(x, 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(x, 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(x, 48));
  return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

}  // namespace csk
