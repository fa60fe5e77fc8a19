// Kernels of the node-level operations that sit beside the MoE path in the reference's graph
// and are kept bit-exact rather than fast: the float64 router and the broadcasting add.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace csk {

// ------------------------------------------------------------ router, float64
// logits[t][e] = (sum over d, in order, of x[t][d] * g[e][d]) + (double)b[e]
// (include/coalsack/nn/nn_ops/moe_router_node.h:161-167 with T = double).  The sum is the
// reference's: one product and one addition per element, each rounded, in index order, so a
// thread owns one (token, expert) pair and walks the hidden dimension alone.  A workgroup
// takes 64 experts x 4 tokens; the operands of a chunk of 32 columns are staged through LDS
// so that the global reads are coalesced although every thread reads its own row.
constexpr int kR64Chunk = 32;

__global__ __launch_bounds__(256) void router_f64_logits_kernel(const double* __restrict__ x,
                                                                const double* __restrict__ g,
                                                                const float* __restrict__ b,
                                                                double* __restrict__ logits, int T, int E,
                                                                int H) {
#pragma clang fp contract(off)  // a product and a sum, each rounded: no fused multiply-add
  __shared__ double gs[64][kR64Chunk + 1];
  __shared__ double xs[4][kR64Chunk];
  const int el = threadIdx.x & 63, tl = threadIdx.x >> 6;
  const int e0 = blockIdx.x * 64, t0 = blockIdx.y * 4;
  double sum = 0.0;
  for (int d0 = 0; d0 < H; d0 += kR64Chunk) {
    const int n = min(kR64Chunk, H - d0);
    for (int i = threadIdx.x; i < 64 * kR64Chunk; i += 256) {
      const int r = i / kR64Chunk, c = i % kR64Chunk;
      gs[r][c] = (e0 + r < E && c < n) ? g[(size_t)(e0 + r) * H + d0 + c] : 0.0;
    }
    if (threadIdx.x < 4 * kR64Chunk) {
      const int r = threadIdx.x / kR64Chunk, c = threadIdx.x % kR64Chunk;
      xs[r][c] = (t0 + r < T && c < n) ? x[(size_t)(t0 + r) * H + d0 + c] : 0.0;
    }
    __syncthreads();
    for (int c = 0; c < n; ++c) {
      const double prod = xs[tl][c] * gs[el][c];
      sum = sum + prod;
    }
    __syncthreads();
  }
  if (e0 + el < E && t0 + tl < T)
    logits[(size_t)(t0 + tl) * E + e0 + el] = sum + (b ? (double)b[e0 + el] : 0.0);
}

// The k largest logits of a token in the order std::partial_sort leaves them with the
// comparator a.first > b.first (moe_router_node.h:175-177): libstdc++'s heap selection
// (a heap of the first k entries, every later entry that beats the heap's root replaces it,
// then the heap is taken apart), so that ties come out where the reference puts them.  One
// thread per token; its E (value, index) entries live in global memory with the token as
// the fastest index, element i of token t at [i * stride + t].
struct Scored64 {
  double* v;
  int* ix;
  int64_t stride;
  __device__ double& val(int i) const { return v[i * stride]; }
  __device__ int& idx(int i) const { return ix[i * stride]; }
  __device__ void move(int to, int from) const {
    val(to) = val(from);
    idx(to) = idx(from);
  }
};

__device__ inline void heap_place(const Scored64& h, int hole, int len, double value, int id) {
  const int top = hole;
  int child = hole;
  while (child < (len - 1) / 2) {
    child = 2 * (child + 1);
    if (h.val(child) > h.val(child - 1)) --child;
    h.move(hole, child);
    hole = child;
  }
  if ((len & 1) == 0 && child == (len - 2) / 2) {
    child = 2 * (child + 1);
    h.move(hole, child - 1);
    hole = child - 1;
  }
  int parent = (hole - 1) / 2;
  while (hole > top && h.val(parent) > value) {
    h.move(hole, parent);
    hole = parent;
    parent = (hole - 1) / 2;
  }
  h.val(hole) = value;
  h.idx(hole) = id;
}

__global__ __launch_bounds__(64) void router_f64_topk_kernel(const double* __restrict__ logits,
                                                             double* __restrict__ work_v,
                                                             int* __restrict__ work_i,
                                                             float* __restrict__ wts,
                                                             float* __restrict__ pairs, int T, int E, int k,
                                                             int sigmoid) {
  const int t = blockIdx.x * 64 + threadIdx.x;
  if (t >= T) return;
  const Scored64 h{work_v + t, work_i + t, T};
  for (int e = 0; e < E; ++e) {
    h.val(e) = logits[(size_t)t * E + e];
    h.idx(e) = e;
  }
  if (k >= 2) {
    for (int parent = (k - 2) / 2;; --parent) {
      heap_place(h, parent, k, h.val(parent), h.idx(parent));
      if (parent == 0) break;
    }
  }
  for (int i = k; i < E; ++i) {
    if (h.val(i) > h.val(0)) {
      const double value = h.val(i);
      const int id = h.idx(i);
      h.move(i, 0);
      heap_place(h, 0, k, value, id);
    }
  }
  for (int end = k; end > 1; --end) {
    const double value = h.val(end - 1);
    const int id = h.idx(end - 1);
    h.move(end - 1, 0);
    heap_place(h, 0, end - 1, value, id);
  }
  // weights in float from the double logits (moe_router_node.h:180-202)
  float* w = wts + (size_t)t * k;
  if (sigmoid) {
    for (int j = 0; j < k; ++j) w[j] = 1.0f / (1.0f + expf(-(float)h.val(j)));
  } else {
    double mx = h.val(0);
    for (int j = 1; j < k; ++j)
      if (h.val(j) > mx) mx = h.val(j);
    float sum = 0.0f;
    for (int j = 0; j < k; ++j) {
      w[j] = expf((float)(h.val(j) - mx));
      sum += w[j];
    }
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    for (int j = 0; j < k; ++j) w[j] *= inv;
  }
  for (int j = 0; j < k; ++j) {
    pairs[((size_t)t * k + j) * 2] = (float)h.idx(j);
    pairs[((size_t)t * k + j) * 2 + 1] = w[j];
  }
}

// ------------------------------------------------------------ add, broadcast
// out[i] = a[ia(i)] + b[ib(i)] with numpy-style broadcasting over trailing dimensions
// (include/coalsack/nn/nn_ops/elementwise_helpers.h:33-61): the flat output index is taken
// apart into coordinates, an operand's stride is 0 along a dimension it repeats over.
constexpr int kMaxBroadcastDims = 8;
struct BroadcastDims {
  int nd;
  int64_t out[kMaxBroadcastDims], sa[kMaxBroadcastDims], sb[kMaxBroadcastDims];
};

template <class V>
__device__ __forceinline__ V wrap_add(V x, V y) {
  return x + y;
}
template <>
__device__ __forceinline__ int32_t wrap_add<int32_t>(int32_t x, int32_t y) {
  return (int32_t)((uint32_t)x + (uint32_t)y);
}
template <>
__device__ __forceinline__ int64_t wrap_add<int64_t>(int64_t x, int64_t y) {
  return (int64_t)((uint64_t)x + (uint64_t)y);
}

template <class V>
__global__ __launch_bounds__(256) void add_broadcast_kernel(const V* __restrict__ a, const V* __restrict__ b,
                                                            V* __restrict__ out, int64_t n, BroadcastDims d) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    int64_t rest = i, ia = 0, ib = 0;
    for (int q = d.nd - 1; q >= 0; --q) {
      const int64_t c = rest % d.out[q];
      rest /= d.out[q];
      ia += c * d.sa[q];
      ib += c * d.sb[q];
    }
    out[i] = wrap_add<V>(a[ia], b[ib]);
  }
}

// ------------------------------------------------------------ rmsnorm, float64
// out[i][j] = (x[i][j] / sqrt(sum_j x[i][j]^2 / H + eps)) * w[j]   (rmsnorm_node.h:62-83 with
// T = double).  The sum of squares is the reference's: one product and one addition per
// element, each rounded, in index order -- so one lane walks the row alone (eight rows per
// workgroup, one per wave, the row staged through LDS in chunks so that the global reads are
// coalesced); division, square root, x / rms and the product with w are IEEE operations and
// are spread over the wave.  Bit-exact against the CPU path.
constexpr int kRms64Chunk = 512;

__global__ __launch_bounds__(512) void rmsnorm_f64_kernel(const double* __restrict__ x,
                                                          const double* __restrict__ w,
                                                          double* __restrict__ out, long T, long H,
                                                          float eps) {
#pragma clang fp contract(off)
  __shared__ double stage[8][kRms64Chunk];
  __shared__ double rms_sh[8];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const long row = (long)blockIdx.x * 8 + wv;
  if (row >= T) return;  // (whole waves leave: what follows synchronises within a wave only)
  const double* xr = x + row * H;
  double ss = 0.0;
  for (long c0 = 0; c0 < H; c0 += kRms64Chunk) {
    const int n = (int)min((long)kRms64Chunk, H - c0);
    for (int j = lane; j < n; j += 64) stage[wv][j] = xr[c0 + j];
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's LDS writes have landed
    if (lane == 0) {
      for (int j = 0; j < n; ++j) {
        const double v = stage[wv][j];
        ss += v * v;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) rms_sh[wv] = sqrt(ss / (double)H + (double)eps);
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0xc07f);
  const double rms = rms_sh[wv];
  for (long j = lane; j < H; j += 64) out[row * H + j] = (xr[j] / rms) * w[j];
}

}  // namespace csk
