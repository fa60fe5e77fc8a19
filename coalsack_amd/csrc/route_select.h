// Per-token expert selection (top-k, close calls recomputed in the reference's summation
// order, routing weights) and the dispatch of a small batch, as device functions of the
// router kernels.
#pragma once
#include "common.h"

namespace csk {

// --------------------------------------------------- per-token selection
// Maximum over the 64 lanes, the same value returned in every lane: four cross-lane steps
// inside each row of 16 (quad swaps, half-row and row mirrors: ordinary vector-ALU latency,
// where a shuffle through the LDS crossbar takes ten times as long) and the four row
// results combined through scalar registers.
template <int CTRL>
__device__ __forceinline__ float dpp_max(float a) {
  const int x = __float_as_int(a);
  return fmaxf(a, __int_as_float(__builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false)));
}
__device__ __forceinline__ float wave_max_all(float v) {
  v = dpp_max<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_max<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_max<0x141>(v);  // row_half_mirror
  v = dpp_max<0x140>(v);  // row_mirror
  const int x = __float_as_int(v);
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(x, 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(x, 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(x, 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(x, 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// One wave selects one token's top k.  Lane l holds the logits of experts l, l+64,
// l+128, l+192; each round finds the wave-wide maximum, locates its owner with ballots
// (ties -> lowest expert index) and retires it.  One round more than k records
// the runner-up, so that the k+1 largest logits are known: if any two adjacent ones are
// closer than the difference between this library's tree-ordered fp32 sums and the
// reference's strictly sequential ones can be (moe_router_node.h:161-167: sum += h*g,
// multiply and add rounded separately, bias added last), the caller recomputes the
// logits in question in exactly that order and selects again -- so the expert indices
// and their slot order equal the reference's whenever the inputs are the same, not only
// when no two logits are close.  Lane s < k returns slot s in (my_val, my_idx).
//
// The k experts returned are always distinct and below E, whatever the logits hold -- the
// dispatch and the one-token launch (k token groups, known before the kernel runs) rely on
// it.  Retired and out-of-range entries are -inf; the logits compete as max(logit, -FLT_MAX),
// which turns a NaN or a -inf into the lowest finite key, so that such a logit is still a
// candidate distinct from the retired ones (among equal keys the lowest index wins).  A token
// whose logits hold a NaN or +inf, or nothing but -inf, has NaN routing weights in the
// reference's softmax (moe_router_node.h:176-200: exp(inf - inf), or a NaN sum); which experts
// its partial sort then returns is unspecified.  Here such a token gets NaN in every slot's value, hence NaN
// weights, k distinct experts, and no close-call recomputation.
__device__ __forceinline__ void select_topk(float (&v)[4], int lane, int E, int k, float& my_val,
                                            int& my_idx, float& vmax, bool& close_call, float tol,
                                            float& runner_up) {
  const float NEG = -__builtin_inff();
  constexpr float kLowest = -3.402823466e+38f;
  bool bad = false, finite = false;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const bool real = lane + 64 * j < E;
    bad = bad || (real && !(v[j] <= -kLowest));           // NaN or +inf
    finite = finite || (real && fabsf(v[j]) <= -kLowest);
    if (real) v[j] = fmaxf(v[j], kLowest);
  }
  const bool poisoned = __any(bad) || !__any(finite);      // (every logit -inf: exp(-inf + inf))
  my_val = 0.0f, my_idx = 0, vmax = 0.0f;
  for (int s = 0; s <= k; ++s) {
    const float best = wave_max_all(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
    // its owner: lowest expert index among equals = lowest register j, then lowest lane
    int bi = 0;
    bool found = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned long long m = __ballot(v[j] == best);
      if (!found && m != 0ull) {
        bi = (int)__builtin_ctzll(m) + 64 * j;
        found = true;
      }
    }
    if (s == 0) vmax = best;
    if (lane == s) {
      my_val = best;
      my_idx = bi;
    }
    if (s < k && (bi & 63) == lane) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if ((bi >> 6) == j) v[j] = NEG;
    }
  }
  // lanes 0..k hold the k+1 largest in descending order (fewer when E == k)
  // the value one lane up (wave_shl:1, a vector-ALU operation) and slot min(k, E - 1) through
  // a scalar register: no trip through the LDS crossbar
  const int mv = __float_as_int(my_val);
  const float below = __int_as_float(__builtin_amdgcn_update_dpp(mv, mv, 0x130, 0xf, 0xf, false));
  const bool close = lane < k && lane + 1 < E && (my_val - below) <= tol * fmaxf(1.0f, fabsf(my_val));
  close_call = __any(close) && !poisoned;
  runner_up = __int_as_float(__builtin_amdgcn_readlane(mv, min(k, E - 1)));
  if (poisoned) {
    my_val = __builtin_nanf("");
    vmax = my_val;
  }
}

// Logits in the reference's order: a strictly sequential fp32 sum per logit, multiply and
// add rounded separately (moe_router_node.h:161-167).  The chain of H dependent additions
// cannot be shortened, everything else can be taken out of its way: the whole workgroup
// multiplies (coalesced loads, the products do not depend on the running sum) and stages
// the rounded products of up to kCcBatch logits in LDS, one chunk of K ahead; lane c of
// wave 0 then only reads row c back and adds, all rows side by side.
constexpr int kCcBatch = 8;              // logits recomputed side by side
constexpr int kCcChunk = 768;            // elements of K staged per step
constexpr int kCcStride = kCcChunk + 4;  // LDS row stride: rows start four banks apart

template <int B>
struct CloseCallLdsT {
  alignas(16) float prod[2][B][kCcStride];
  float fixed[kMaxExperts];  // the token's logits, recomputed ones replaced
  int cand[kMaxExperts];
  int ncand;
};
using CloseCallLds = CloseCallLdsT<kCcBatch>;

// Called by all NT threads of the workgroup with the same arguments.  Recomputes the
// logits that can take part in a close call -- those not below thr, which is set a safe
// margin under the (k+1)-th largest; the others keep their tree-ordered values, which the
// bound on the difference keeps on their side of thr -- and leaves all E logits of the
// token in s.fixed.  H must be a multiple of 4.
template <int NT, int B = kCcBatch>
__device__ __forceinline__ void logits_reference_order_wg(const float* __restrict__ x,
                                                          const float* __restrict__ g,
                                                          const float* __restrict__ b,
                                                          const float* __restrict__ logit_row, int E,
                                                          int H, float thr, CloseCallLdsT<B>& s) {
#pragma clang fp contract(off)
  constexpr int kC4 = kCcChunk / 4;
  constexpr int kProducers = NT - 64;  // wave 0 only adds
  constexpr int kItems = (B * kC4 + kProducers - 1) / kProducers;
  const int tid = threadIdx.x, ptid = tid - 64;
  if (tid == 0) s.ncand = 0;
  __syncthreads();
  for (int e = tid; e < E; e += NT) {
    const float v = logit_row[e];
    s.fixed[e] = v;
    if (v >= thr) s.cand[atomicAdd(&s.ncand, 1)] = e;
  }
  __syncthreads();
  const int m = s.ncand;
  const CSK_GLOBAL floatx4* x4 = as_global(reinterpret_cast<const floatx4*>(x));
  const CSK_GLOBAL floatx4* g4 = as_global(reinterpret_cast<const floatx4*>(g));
  const int H4 = H >> 2;
  const int nchunk = (H4 + kC4 - 1) / kC4;
  for (int c0 = 0; c0 < m; c0 += B) {
    const int mb = min(B, m - c0);
    // producers: rounded products of chunk ci of the batch's rows -> LDS buffer ci & 1
    auto produce = [&](int ci) {
      const int h4 = ci * kC4, len4 = min(kC4, H4 - h4);
      floatx4 xq[kItems], gq[kItems];
#pragma unroll
      for (int it = 0; it < kItems; ++it) {
        const int idx = ptid + it * kProducers, c = idx / kC4, i4 = idx - c * kC4;
        if (c < mb && i4 < len4) {
          xq[it] = x4[h4 + i4];
          gq[it] = g4[(size_t)s.cand[c0 + c] * H4 + h4 + i4];
        }
      }
#pragma unroll
      for (int it = 0; it < kItems; ++it) {
        const int idx = ptid + it * kProducers, c = idx / kC4, i4 = idx - c * kC4;
        if (c < mb && i4 < len4)
          *reinterpret_cast<floatx4*>(&s.prod[ci & 1][c][4 * i4]) = xq[it] * gq[it];
      }
    };
    if (ptid >= 0) produce(0);
    __syncthreads();
    float sum = 0.0f;
    for (int ci = 0; ci < nchunk; ++ci) {
      if (ptid >= 0) {
        if (ci + 1 < nchunk) produce(ci + 1);  // while wave 0 adds chunk ci
      } else if (tid < mb) {
        const int len4 = min(kC4, H4 - ci * kC4);
        const floatx4* row = reinterpret_cast<const floatx4*>(&s.prod[ci & 1][tid][0]);
        floatx4 qa[8], qb[8];
        // reads run up to 15 entries past the chunk (into the next row: never added)
        auto rd = [&](floatx4(&q)[8], int i0) {
#pragma unroll
          for (int i = 0; i < 8; ++i) q[i] = row[i0 + i];
        };
        auto add = [&](const floatx4(&q)[8]) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            sum = sum + q[i][0];
            sum = sum + q[i][1];
            sum = sum + q[i][2];
            sum = sum + q[i][3];
          }
        };
        auto add_tail = [&](const floatx4(&q)[8], int n) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            if (i < n) {
              sum = sum + q[i][0];
              sum = sum + q[i][1];
              sum = sum + q[i][2];
              sum = sum + q[i][3];
            }
          }
        };
        // two register sets of eight float4 in rotation: the reads of one are in flight
        // while the other is added; whole groups carry no guards
        const int full = len4 & ~7;
        int i0 = 0;
        rd(qa, 0);
        for (; i0 + 16 <= full; i0 += 16) {
          rd(qb, i0 + 8);
          add(qa);
          rd(qa, i0 + 16);
          add(qb);
        }
        if (i0 + 8 <= full) {
          rd(qb, i0 + 8);
          add(qa);
          add_tail(qb, len4 - i0 - 8);
        } else {
          add_tail(qa, len4 - i0);
        }
      }
      __syncthreads();
    }
    if (tid < mb) {
      const int e = s.cand[c0 + tid];
      s.fixed[e] = sum + (b ? b[e] : 0.0f);
    }
    __syncthreads();
  }
}

// How close is a close call.  Measured over 1.3 million logits (six shapes, H from 256 to
// 2880): |tree-ordered sum - sequential sum| / max(1, |logit|) has an rms of 0.28 and a
// maximum of 2.3 in units of 2^-24 * sqrt(H) (the random-walk size of the sequential
// sum's rounding error); the tests hold the maximum below 3.  Two logits can change rank
// only if they are closer than the sum of their two differences; the threshold is 8 units,
// twice the largest pair of differences seen.  At gpt-oss shapes about one token in 2500
// is recomputed.
__device__ __forceinline__ float close_call_tolerance(int H) { return 8.0f * 5.96e-8f * sqrtf((float)H); }

// Routing weight of slot `lane` (moe_router_node.h:180-202): sigmoid of the raw logit, or
// softmax over the selected k with max subtraction, sum in slot order, multiply by 1/sum.
__device__ __forceinline__ float routing_weight(float my_val, float vmax, int lane, int k, int sigmoid) {
  if (sigmoid) return 1.0f / (1.0f + expf(-my_val));
  float w = (lane < k) ? expf(my_val - vmax) : 0.0f;
  float sum = 0.0f;
  for (int s = 0; s < k; ++s) sum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), s));  // slot order
  const float inv = (sum > 0.0f) ? (1.0f / sum) : 0.0f;
  return w * inv;
}

// Work descriptor of one active-expert slot (all zero when the slot is unused), written
// field by field: a local copy of the structure would live in scratch memory.
__device__ __forceinline__ void write_work_desc(WorkDesc* d, bool on, int e, int Te, int base,
                                                const ExpertW* __restrict__ ew) {
  const ExpertW* src = ew + e;
  d->e = e;
  d->Te = on ? Te : 0;
  d->base = on ? base : 0;
  d->pad = 0;
  d->w.q_gate = on ? src->q_gate : nullptr;
  d->w.s_gate = on ? src->s_gate : nullptr;
  d->w.q_up = on ? src->q_up : nullptr;
  d->w.s_up = on ? src->s_up : nullptr;
  d->w.q_down = on ? src->q_down : nullptr;
  d->w.s_down = on ? src->s_down : nullptr;
  d->w.b_gate = on ? src->b_gate : nullptr;
  d->w.b_up = on ? src->b_up : nullptr;
  d->w.b_down = on ? src->b_down : nullptr;
}


// ------------------------------------- small batches: top-k + dispatch, fused
// One workgroup does, for P = T * k <= MAXP assignments, what router_topk_kernel and
// dispatch_scatter_kernel do in two launches: top-k and weights per token (one wave per
// token), per-expert counts, exclusive scan, ordered lists, work descriptors and token
// groups -- all through LDS.
struct RouteIn {
  const float* logits;  // [T, E]
  const float* x;       // [T, H] rows the logits were computed from (close calls are recomputed)
  const float* g;       // [E, H]
  const float* b;       // [E] or null
  const ExpertW* ew;    // [E]
  int T, E, k, H, sigmoid, group_tokens;
};
struct RouteOut {
  float* pairs;       // [T, k, 2]
  int* ids;           // [T * k]
  int* pos_of_slot;   // [T * k]
  int* counts;        // [E]
  int* offsets;       // [E + 1]
  WorkDesc* desc;     // [E]
  StreamGroup* groups;  // [token groups]
  int* nv;
  int* mtiles;        // [2 * M tiles]
  int* n_mtiles;
  int* list_tok;      // [T * k]
  float* list_w;      // [T * k]
};
// Inclusive prefix sum over the 64 lanes: shifts inside each row of 16 on the vector ALU
// (lanes without a source add zero), then the totals of the rows before through scalar
// registers.
template <int CTRL>
__device__ __forceinline__ int dpp_shr_add(int v) {
  return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
__device__ __forceinline__ int wave_scan_inclusive(int v, int lane) {
  v = dpp_shr_add<0x111>(v);  // row_shr:1
  v = dpp_shr_add<0x112>(v);  // row_shr:2
  v = dpp_shr_add<0x114>(v);  // row_shr:4
  v = dpp_shr_add<0x118>(v);  // row_shr:8
  const int t0 = __builtin_amdgcn_readlane(v, 15), t1 = __builtin_amdgcn_readlane(v, 31);
  const int t2 = __builtin_amdgcn_readlane(v, 47);
  const int row = lane >> 4;
  return v + (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
}

// ceil(c / g) for the group sizes in use without a run-time integer division
__device__ __forceinline__ int group_count(int c, int g) {
  return g == 4 ? (c + 3) >> 2 : g == 6 ? (c + 5) / 6 : (c + g - 1) / g;
}

template <int CCB, int MAXP>
struct RouteLds {
  int ids[MAXP];       // expert of assignment p = t * k + slot
  float wts[MAXP];     // its routing weight
  int cnt[kMaxExperts], off[kMaxExperts], act_e[kMaxExperts];
  int na;
  int cntc[MAXP / 64][kMaxExperts];  // per 64-assignment chunk: how many name the expert; then the count before the chunk
  unsigned long long ew[kMaxExperts * (sizeof(ExpertW) / 8)];  // the experts' weight pointers, staged early
  CloseCallLdsT<CCB> cc;
  int cc_tok[64], cc_n;
  float cc_thr[64];
};

template <int NT, int CCB, int MAXP>
__device__ __forceinline__ void route_workgroup(const RouteIn& r, const RouteOut& o, RouteLds<CCB, MAXP>& s) {
  constexpr int NW = NT / 64;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int T = r.T, E = r.E, k = r.k;
  const int P = T * k;
  const float NEG = -__builtin_inff();
  const float tol = close_call_tolerance(r.H);
  static_assert(MAXP <= NT && MAXP % 64 == 0, "assignment p belongs to thread p, chunk p / 64 to wave p / 64");
  const int nchunk = (P + 63) >> 6;
  for (int i = threadIdx.x; i < nchunk * kMaxExperts; i += NT) (&s.cntc[0][0])[i] = 0;
  if (threadIdx.x == 0) s.cc_n = 0;
  // the table of weight pointers is needed last (work descriptors); its load is started
  // first, so that its latency runs beside that of the logits
  static_assert(sizeof(ExpertW) % 8 == 0, "copied as 64-bit words");
  static_assert(MAXP < 32768, "counts are scanned as 16-bit halves");
  constexpr int kEwWords = kMaxExperts * (int)(sizeof(ExpertW) / 8), kEwPerThread = (kEwWords + NT - 1) / NT;
  unsigned long long ew_reg[kEwPerThread];
#pragma unroll
  for (int i = 0; i < kEwPerThread; ++i) {
    const int w = threadIdx.x + i * NT;
    ew_reg[i] = w < E * (int)(sizeof(ExpertW) / 8) ? reinterpret_cast<const unsigned long long*>(r.ew)[w] : 0ull;
  }
  __syncthreads();
  auto publish_token = [&](int t, float my_val, int my_idx, float vmax) {
    const float w = routing_weight(my_val, vmax, lane, k, r.sigmoid);
    if (lane < k) {
      reinterpret_cast<float2*>(o.pairs)[(size_t)t * k + lane] = make_float2((float)my_idx, w);
      o.ids[t * k + lane] = my_idx;
      s.ids[t * k + lane] = my_idx;
      s.wts[t * k + lane] = w;
    }
  };
  // a wave's tokens four at a time: their logits are requested together, so that a wave
  // with several tokens waits for memory once
  for (int t0 = wv; t0 < T; t0 += 4 * NW) {
    float v[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int t = t0 + q * NW;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        v[q][j] = (t < T && e < E) ? r.logits[(size_t)t * E + e] : NEG;
      }
    }
#pragma unroll 1  // one copy of the selection code: the token in turn sits in v[0], the others move up
    for (int q = 0; q < 4; ++q) {
      const int t = t0 + q * NW;
      if (t < T) {
        float my_val, vmax, runner_up;
        int my_idx;
        bool close_call;
        select_topk(v[0], lane, E, k, my_val, my_idx, vmax, close_call, tol, runner_up);
        if (close_call) {
          if (lane == 0) {
            const int n = atomicAdd(&s.cc_n, 1);
            s.cc_tok[n] = t;
            s.cc_thr[n] = runner_up - 2.0f * tol * fmaxf(1.0f, fabsf(runner_up));
          }
        } else {
          publish_token(t, my_val, my_idx, vmax);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) v[0][j] = v[1][j], v[1][j] = v[2][j], v[2][j] = v[3][j];
    }
  }
#pragma unroll
  for (int i = 0; i < kEwPerThread; ++i) {
    const int w = threadIdx.x + i * NT;
    if (w < kEwWords) s.ew[w] = ew_reg[i];
  }
  __syncthreads();
  // rare: tokens with a close call among their k+1 largest logits are recomputed in the
  // reference's order by the whole workgroup, one after the other; wave 0 selects again
  for (int n = 0; n < s.cc_n; ++n) {
    const int t = s.cc_tok[n];
    logits_reference_order_wg<NT, CCB>(r.x + (size_t)t * r.H, r.g, r.b, r.logits + (size_t)t * E, E, r.H,
                                       s.cc_thr[n], s.cc);
    if (wv == 0) {
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        v[j] = e < E ? s.cc.fixed[e] : NEG;
      }
      float my_val, vmax, runner_up;
      int my_idx;
      bool close_call;
      select_topk(v, lane, E, k, my_val, my_idx, vmax, close_call, 0.0f, runner_up);
      publish_token(t, my_val, my_idx, vmax);
    }
    __syncthreads();
  }
  __syncthreads();
  // Dispatch in O(P): thread p owns assignment p.  The lanes of a wave that name the same
  // expert find one another in a loop over the distinct experts of the wave (a ballot per
  // expert); the first of them records how many they are, the others their rank among
  // them.  Per expert, a prefix over the chunks (waves) then gives every assignment its
  // place in the expert's list: assignments stay in ascending order, as the reference's
  // per-expert token loop visits them (expert_mlp_node.h:503-529).
  const int my_p = threadIdx.x;
  const bool live_p = my_p < P;
  const int my_id = live_p ? s.ids[my_p] : -1;
  unsigned long long same = 0ull, todo = __ballot(live_p);
  while (todo != 0ull) {  // the same in every lane
    const int id0 = __builtin_amdgcn_readlane(my_id, (int)__builtin_ctzll(todo));
    const unsigned long long m = __ballot(my_id == id0);
    if (my_id == id0) same = m;
    todo &= ~m;
  }
  const int rank_in_chunk = __popcll(same & ((1ull << lane) - 1ull));
  if (live_p && rank_in_chunk == 0) s.cntc[wv][my_id] = __popcll(same);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += NT) {
    int run = 0;
    for (int c = 0; c < nchunk; ++c) {
      const int v = s.cntc[c][e];
      s.cntc[c][e] = run;
      run += v;
    }
    s.cnt[e] = run;
    o.counts[e] = run;
  }
  __syncthreads();
  // exclusive scan, active experts, token groups, M tiles: wave 0, four consecutive
  // experts per lane, wave-wide prefix sums
  if (wv == 0) {
    const int group_tokens = r.group_tokens;
    int c[4], tot = 0, nact = 0, ngrp = 0, nmt = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = lane * 4 + j;
      c[j] = e < E ? s.cnt[e] : 0;
      tot += c[j];
      nact += c[j] > 0;
      ngrp += group_count(c[j], group_tokens);
      nmt += (c[j] + 63) / 64;
    }
    // inclusive scans over the lanes, two 16-bit counts to a register (none exceeds MAXP)
    const int sa = wave_scan_inclusive(tot | (ngrp << 16), lane), sb = wave_scan_inclusive(nact | (nmt << 16), lane);
    const int s_tot = sa & 0xffff, s_grp = sa >> 16, s_act = sb & 0xffff, s_mt = sb >> 16;
    int run = s_tot - tot, slot = s_act - nact, gi = s_grp - ngrp, mi = s_mt - nmt;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = lane * 4 + j;
      if (e < E) {
        s.off[e] = run;
        o.offsets[e] = run;
        if (c[j] > 0) {
          for (int gb = 0; gb < c[j]; gb += group_tokens) {
            write_stream_group(o.groups + gi, reinterpret_cast<const ExpertW*>(s.ew) + e, e, c[j] - gb, run + gb);
            ++gi;
          }
          for (int m0 = 0; m0 < c[j]; m0 += 64) {
            o.mtiles[2 * mi] = slot;
            o.mtiles[2 * mi + 1] = m0;
            ++mi;
          }
          s.act_e[slot++] = e;
        }
        run += c[j];
      }
    }
    if (lane == 63) {
      s.na = s_act;
      o.offsets[E] = s_tot;
      *o.nv = s_grp;
      *o.n_mtiles = s_mt;
    }
  }
  __syncthreads();
  // place of assignment p: the expert's offset + its assignments in earlier chunks + its rank in this one
  if (live_p) {
    const unsigned inv_k = (65536u + (unsigned)k - 1u) / (unsigned)k;  // p / k == p * inv_k >> 16 for p <= 1024, k <= 16
    const int pos = s.off[my_id] + s.cntc[wv][my_id] + rank_in_chunk;
    o.list_tok[pos] = (int)(((unsigned)my_p * inv_k) >> 16);
    o.list_w[pos] = s.wts[my_p];
    o.pos_of_slot[my_p] = pos;
  }
  for (int i = threadIdx.x; i < E; i += NT) {
    const bool on = i < s.na;
    const int e = on ? s.act_e[i] : 0;
    write_work_desc(o.desc + i, on, e, s.cnt[e], s.off[e], reinterpret_cast<const ExpertW*>(s.ew));
  }
}
}  // namespace csk
