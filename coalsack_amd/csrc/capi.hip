// C ABI of the gfx950 MoE path: resident weight store, workspace, kernel
// launches.  Declarations and reference citations are in
// include/coalsack_moe.h.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "coalsack_moe.h"
#include "common.h"
#include "expert_stream_kernel.h"
#include "expert_prefill_kernel.h"
#include "expert_f16_kernel.h"
#include "mxfp4_kernels.h"
#include "router_kernels.h"
#include "node_extra_kernels.h"

using namespace csk;

namespace {

thread_local std::string g_err;
hipStream_t g_stream = nullptr;
bool g_ready = false;
int g_device = -1;
int g_cus = 0;
// The library owns one stream and one workspace, so calls are serialised: an entry point
// holds this lock from its first line to its return (recursive: entry points call one
// another).  Callers may therefore come from any thread, e.g. the per-layer worker threads
// of the reference's scheduler (layer_scheduler_node), without locking of their own.
std::recursive_mutex g_api;
thread_local bool t_device_bound = false;  // the current device is a per-thread setting
#define API_LOCK() std::lock_guard<std::recursive_mutex> csk_api_guard_(g_api)

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

#define HIP_TRY(expr)                                                                      \
  do {                                                                                     \
    hipError_t _e = (expr);                                                                \
    if (_e != hipSuccess)                                                                  \
      return fail(CSK_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(_e));         \
  } while (0)

#define REQUIRE_INIT()                                                          \
  API_LOCK();                                                                   \
  if (!g_ready) return fail(CSK_ERR_STATE, "csk_init has not been called");     \
  if (!t_device_bound) {                                                        \
    HIP_TRY(hipSetDevice(g_device));                                            \
    t_device_bound = true;                                                      \
  }

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(CSK_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
  return CSK_OK;
}

// Every device allocation of the library goes through here and is counted, so that a test
// can hold the allocation-free entry point to its name (csk_alloc_count).
std::atomic<uint64_t> g_alloc_count{0};
inline hipError_t counted_malloc(void** p, size_t bytes) {
  g_alloc_count.fetch_add(1, std::memory_order_relaxed);
  return hipMalloc(p, bytes);
}

template <class T>
int dev_alloc(T** p, size_t count) {
  *p = nullptr;
  if (count == 0) return CSK_OK;
  HIP_TRY(counted_malloc(reinterpret_cast<void**>(p), count * sizeof(T)));
  return CSK_OK;
}

inline long cdiv(long a, long b) { return (a + b - 1) / b; }

// Above this many token-expert assignments the token-group list of the
// weight-streaming kernel is not built.
constexpr int64_t kStreamMaxP = 2048;
constexpr size_t kWeightSlack = 32768;  // bytes of mapped memory kept behind weight planes (the streaming kernel walks 96 blocks per tile whatever K is)
constexpr int kStreamWgPerCu = 2;  // resident workgroups of the streaming kernel per compute unit

// ---- workspace shared by every layer (single stream, one call at a time) --
struct Workspace {
  int64_t T = 0, E = 0, k = 0, H = 0, F = 0;
  float* xn = nullptr;      // [T,H] normalised activations
  uint16_t* xs = nullptr;   // [T][H/32][64] bf16 hi|lo
  uint16_t* xg = nullptr;   // [P][H/32][64] gathered + pre-scaled (weight_before_ffn)
  float* logits = nullptr;  // [T,E]
  float* pairs = nullptr;   // [T,k,2]
  int* ids = nullptr;       // [P]
  int* counts = nullptr;    // [E]
  int* offsets = nullptr;   // [E+1]
  WorkDesc* desc = nullptr; // [E] work descriptors of the active experts
  StreamGroup* groups = nullptr;  // [P] token groups of the streaming kernel
  int* nv = nullptr;        // [1]
  int* list_tok = nullptr;  // [P]
  float* list_w = nullptr;  // [P]
  int* pos = nullptr;       // [P]
  uint16_t* act = nullptr;  // [P][F/32][64] bf16 hi|lo
  float* y = nullptr;       // [P,H]
  int* tiles = nullptr;     // prefill tile schedule
  int* n_tiles = nullptr;
  bool fixed = false;       // carved out of the load-time device array: never grown, never freed
  uint64_t runs = 0;        // forwards that have used this workspace

  void release() {
    void* ps[] = {xn, xs, xg, logits, pairs, ids, counts, offsets, desc, groups, nv,
                  list_tok, list_w, pos, act, y, tiles, n_tiles};
    for (void* p : ps)
      if (p) (void)hipFree(p);
    const uint64_t r = runs;
    *this = Workspace();
    runs = r + 1;  // (what a layer remembered of the old buffers no longer matches)
  }
  int ensure(int64_t T_, int64_t E_, int64_t k_, int64_t H_, int64_t F_, bool need_xg) {
    if (T_ <= T && E_ <= E && k_ <= k && H_ <= H && F_ <= F && (!need_xg || xg)) return CSK_OK;
    if (fixed) return fail(CSK_ERR_ARG, "shape exceeds the fixed workspace of the allocation-free forward");
    const int64_t nT = std::max(T, T_), nE = std::max(E, E_), nk = std::max(k, k_),
                  nH = std::max(H, H_), nF = std::max(F, F_);
    const bool had_xg = xg != nullptr;
    HIP_TRY(hipStreamSynchronize(g_stream));
    release();
    const size_t P = (size_t)nT * nk;
    int rc;
#define WS_ALLOC(ptr, cnt) \
  if ((rc = dev_alloc(&ptr, (cnt))) != CSK_OK) return rc
    WS_ALLOC(xn, (size_t)nT * nH);
    // activation rows: two bf16 terms (128 B per block) or three FP6 terms padded to whole
    // K steps (96 B per block), whichever is larger; counts are in uint16
    auto act_elems = [](size_t rows, int64_t dim) {
      const size_t bf = rows * (size_t)dim * 2;
      const size_t mx = rows * (size_t)mx3_row_blocks((int)(dim / 32)) * 48;
      return std::max(bf, mx);
    };
    WS_ALLOC(xs, act_elems((size_t)nT, nH));
    if (need_xg || had_xg) WS_ALLOC(xg, act_elems(P, nH));
    WS_ALLOC(logits, (size_t)nT * nE * (1 + kRouterMaxSplits));  // final logits, then partial ones per split of H
    WS_ALLOC(pairs, P * 2);
    WS_ALLOC(ids, P);
    WS_ALLOC(counts, (size_t)nE);
    WS_ALLOC(offsets, (size_t)nE + 1);
    WS_ALLOC(desc, (size_t)nE);
    WS_ALLOC(groups, P);
    WS_ALLOC(nv, 1);
    WS_ALLOC(list_tok, P);
    WS_ALLOC(list_w, P);
    WS_ALLOC(pos, P);
    WS_ALLOC(act, act_elems(P, nF));
    WS_ALLOC(y, P * nH);
    WS_ALLOC(tiles, (size_t)4 * (P / 16 + nE + 1));
    WS_ALLOC(n_tiles, 1);
#undef WS_ALLOC
    T = nT, E = nE, k = nk, H = nH, F = nF;
    return CSK_OK;
  }
};
Workspace g_ws;

// ---- fixed workspace of the allocation-free forward ------------------------
// Callers that cannot allocate (code under graph capture, serving loops, harnesses that
// forbid hipMalloc) get the decode-sized forward out of a workspace that exists from load
// time on: one file-scope device array per GPU, carved into the buffers of a Workspace of
// the maximum shape below.  The array's name is only a handle on the host; its device
// address is asked for once per device (csk_init, that device current) and kept.
constexpr int64_t kFixedMaxT = 64;      // tokens per call
constexpr int64_t kFixedMaxP = 512;     // token-expert assignments per call (T * top_k)
constexpr int64_t kFixedMaxDim = 3072;  // hidden_dim and expert_ffn_dim
constexpr size_t fixed_align(size_t n) { return (n + 255) & ~(size_t)255; }
constexpr size_t kFixedRowBytes = (size_t)kFixedMaxDim * 4;  // a row as f32, or as two bf16 terms
constexpr size_t kFixedScratchBytes =
    fixed_align(kFixedMaxT * kFixedRowBytes) * 2 +                                     // xn, xs
    fixed_align(kFixedMaxP * kFixedRowBytes) * 3 +                                     // xg, act, y
    fixed_align((size_t)kFixedMaxT * kMaxExperts * 4 * (1 + kRouterMaxSplits)) +       // logits
    fixed_align(kFixedMaxP * 8) + fixed_align(kFixedMaxP * 4) * 4 +                    // pairs; ids, list_tok, list_w, pos
    fixed_align(kMaxExperts * 4) + fixed_align((kMaxExperts + 1) * 4) +                // counts, offsets
    fixed_align(kMaxExperts * sizeof(WorkDesc)) + fixed_align(kFixedMaxP * sizeof(StreamGroup)) +
    fixed_align((size_t)4 * (kFixedMaxP / 16 + kMaxExperts + 1) * 4) + 2 * 256;        // tiles; nv, n_tiles
}  // namespace
static __device__ __align__(256) unsigned char scratch[kFixedScratchBytes];
namespace {
constexpr int kMaxDevices = 64;
unsigned char* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each GPU that csk_init has seen
Workspace g_ws_fixed;                             // carved out of g_scratch_ptr[g_device]

void carve_fixed_workspace(Workspace& ws, unsigned char* base) {
  size_t off = 0;
  auto take = [&](size_t bytes) {
    unsigned char* p = base + off;
    off += fixed_align(bytes);
    return p;
  };
  ws = Workspace();
  ws.xn = reinterpret_cast<float*>(take(kFixedMaxT * kFixedRowBytes));
  ws.xs = reinterpret_cast<uint16_t*>(take(kFixedMaxT * kFixedRowBytes));
  ws.xg = reinterpret_cast<uint16_t*>(take(kFixedMaxP * kFixedRowBytes));
  ws.act = reinterpret_cast<uint16_t*>(take(kFixedMaxP * kFixedRowBytes));
  ws.y = reinterpret_cast<float*>(take(kFixedMaxP * kFixedRowBytes));
  ws.logits = reinterpret_cast<float*>(take((size_t)kFixedMaxT * kMaxExperts * 4 * (1 + kRouterMaxSplits)));
  ws.pairs = reinterpret_cast<float*>(take(kFixedMaxP * 8));
  ws.ids = reinterpret_cast<int*>(take(kFixedMaxP * 4));
  ws.list_tok = reinterpret_cast<int*>(take(kFixedMaxP * 4));
  ws.list_w = reinterpret_cast<float*>(take(kFixedMaxP * 4));
  ws.pos = reinterpret_cast<int*>(take(kFixedMaxP * 4));
  ws.counts = reinterpret_cast<int*>(take(kMaxExperts * 4));
  ws.offsets = reinterpret_cast<int*>(take((kMaxExperts + 1) * 4));
  ws.desc = reinterpret_cast<WorkDesc*>(take(kMaxExperts * sizeof(WorkDesc)));
  ws.groups = reinterpret_cast<StreamGroup*>(take(kFixedMaxP * sizeof(StreamGroup)));
  ws.tiles = reinterpret_cast<int*>(take((size_t)4 * (kFixedMaxP / 16 + kMaxExperts + 1) * 4));
  ws.nv = reinterpret_cast<int*>(take(4));
  ws.n_tiles = reinterpret_cast<int*>(take(4));
  ws.T = kFixedMaxT, ws.E = kMaxExperts, ws.k = kMaxTopK, ws.H = kFixedMaxDim, ws.F = kFixedMaxDim;
  ws.fixed = true;
}

// extra buffers of the fp16 expert path
struct F16Scratch {
  size_t rows = 0, width = 0;
  float* actf = nullptr;  // [P, F] activations before they are split
  float* rs_x = nullptr;  // scale per input row
  float* rs_a = nullptr;  // scale per activation row
  int ensure(size_t rows_, size_t width_);
};
F16Scratch g_f16;
float* g_zero = nullptr;  // zero vector standing in for absent biases
constexpr size_t kZeroLen = 1 << 16;

// optional per-stage events of the last forward
bool g_timing = false;
hipEvent_t g_stage_ev[CSK_N_STAGES + 1] = {};
bool g_stage_valid = false;
inline void mark(int i) {
  if (g_timing) (void)hipEventRecord(g_stage_ev[i], g_stream);
}
// With stage timing on, the two expert kernels of the MXFP4 path are launched with a start
// and a stop event attached to the dispatch itself: their difference is the kernel's own
// begin-to-end time (the clock a kernel trace reports), free of the cost of recording events
// between launches.  [0] = gate/up, [1] = down.
hipEvent_t g_kern_ev[2][2] = {};
bool g_kern_valid = false;
template <class Kern, class Args>
inline void launch_expert_kernel(int which, Kern kernel, dim3 grid, dim3 block, size_t lds, const Args& a) {
  if (g_timing) {
    hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, g_stream, g_kern_ev[which][0], g_kern_ev[which][1], 0, a);
    g_kern_valid = true;
  } else {
    kernel<<<grid, block, lds, g_stream>>>(a);
  }
}

}  // namespace

struct csk_event {
  hipEvent_t ev;
};

struct csk_mxfp4 {
  uint4* q = nullptr;
  uint8_t* s = nullptr;
  int64_t rows = 0, K = 0;
  int64_t ntile = 0, nblk = 0;
  bool owned = true;
  long entries() const { return (long)(ntile * nblk * 16); }
  long scale_bytes() const { return (long)ntile * 256 * scale_slots((int)nblk); }
};

struct csk_layer {
  int64_t E = 0, k = 0, H = 0, F = 0;
  int sigmoid = 0, act = CSK_ACT_MODIFIED_SWIGLU, wbf = 0;
  float* gate_w = nullptr;
  float* gate_b = nullptr;
  bool has_gate = false, has_gate_b = false;
  uint4* q_all = nullptr;    // [E][gate | up | down] entries
  uint8_t* s_all = nullptr;
  bool f16 = false;          // fp16 experts: h_all holds [E][gate | up | down] tiles instead
  u32x4* h_all = nullptr;
  long ent16_gu() const { return f16_entries(F, H); }
  long ent16_d() const { return f16_entries(H, F); }
  long ent16_expert() const { return 2 * ent16_gu() + ent16_d(); }
  u32x4* view16(int64_t e, int which) const {
    return h_all + (long)e * ent16_expert() +
           (which == CSK_W_GATE ? 0 : (which == CSK_W_UP ? ent16_gu() : 2 * ent16_gu()));
  }
  float* bias_all = nullptr;  // [E][F gate | F up | H down]
  ExpertW* ew_dev = nullptr;
  std::vector<ExpertW> ew_host;
  std::vector<char> expert_set, expert_bias, matrix_set;
  float* norm_w = nullptr;
  float eps = 1e-5f;
  bool has_norm = false;
  int64_t last_T = 0;
  const void* last_ws = nullptr;  // workspace of this layer's last forward, and that workspace's forward count then
  uint64_t last_run = 0;
  // A view layer owns no expert matrices: expert e's planes are those of three csk_mxfp4
  // handles attached by the caller.  It has a workspace of its own, so that what a frame
  // leaves there (router output, per-assignment rows) stays until the next frame of this
  // layer whatever other layers do meanwhile.
  bool is_view = false;
  std::vector<char> attached;
  void* own_ws = nullptr;  // Workspace*
  struct Frame {
    bool live = false, experts_ran = false, rows_fetched = false, voided = false;
    int64_t T = 0;
    int flags = 0;
    float *d_hidden = nullptr, *d_out = nullptr;
    size_t cap = 0;  // floats in d_hidden / d_out
    std::vector<float> pairs, y;
    std::vector<int> pos;
  } frame;
  // geometry of one expert's planes
  int64_t nblkH = 0, nblkF = 0, ntF = 0, ntH = 0;
  long ent_gu() const { return (long)(ntF * nblkH * 16); }  // gate or up: [F,H]
  long ent_d() const { return (long)(ntH * nblkF * 16); }   // down: [H,F]
  long ent_expert() const { return 2 * ent_gu() + ent_d(); }
  long sc_gu() const { return (long)ntF * 256 * scale_slots((int)nblkH); }  // scale bytes of gate or up
  long sc_d() const { return (long)ntH * 256 * scale_slots((int)nblkF); }
  long sc_expert() const { return 2 * sc_gu() + sc_d(); }
  csk_mxfp4 view(int64_t e, int which) const {
    csk_mxfp4 m;
    const long base = (long)e * ent_expert();
    const long off = which == CSK_W_GATE ? 0 : (which == CSK_W_UP ? ent_gu() : 2 * ent_gu());
    m.q = q_all + base + off;
    m.s = s_all + (long)e * sc_expert() + (which == CSK_W_GATE ? 0 : (which == CSK_W_UP ? sc_gu() : 2 * sc_gu()));
    m.rows = which == CSK_W_DOWN ? H : F;
    m.K = which == CSK_W_DOWN ? F : H;
    m.ntile = which == CSK_W_DOWN ? ntH : ntF;
    m.nblk = which == CSK_W_DOWN ? nblkF : nblkH;
    m.owned = false;
    return m;
  }
};

namespace {

// Upload `rows x K` reference blocks and repack into (q, s).  The staging buffer is kept
// between calls (a checkpoint is hundreds of matrices of one size); the scale bytes are
// checked by the pack kernel as it reads them, so the host touches the blocks only to hand
// them to the copy.  After a refused block the planes of m hold partial data.
uint8_t* g_stage = nullptr;
size_t g_stage_cap = 0;
unsigned long long* g_bad = nullptr;

int pack_into(const uint8_t* host, csk_mxfp4& m) {
  const int64_t nblocks = m.rows * m.nblk;
  const size_t bytes = (size_t)nblocks * 17;
  if (bytes > g_stage_cap) {
    HIP_TRY(hipStreamSynchronize(g_stream));
    if (g_stage) (void)hipFree(g_stage);
    g_stage = nullptr, g_stage_cap = 0;
    HIP_TRY(counted_malloc((void**)&g_stage, bytes));
    g_stage_cap = bytes;
  }
  if (!g_bad) HIP_TRY(counted_malloc((void**)&g_bad, sizeof(unsigned long long)));
  HIP_TRY(hipMemsetAsync(g_bad, 0xFF, sizeof(unsigned long long), g_stream));
  HIP_TRY(hipMemcpyAsync(g_stage, host, bytes, hipMemcpyHostToDevice, g_stream));
  const long ent = m.entries();
  pack_mxfp4_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(
      g_stage, m.q, m.s, (int)m.rows, (int)m.nblk, ent, g_bad);
  int rc = check_launch("pack_mxfp4_kernel");
  if (rc != CSK_OK) return rc;
  unsigned long long bad = 0;
  HIP_TRY(hipMemcpyAsync(&bad, g_bad, sizeof bad, hipMemcpyDeviceToHost, g_stream));
  HIP_TRY(hipStreamSynchronize(g_stream));
  if (bad != ~0ull)
    return fail(CSK_ERR_SCALE, "MXFP4 scale byte 255 on block " + std::to_string(bad) +
                                   ", which holds a code of magnitude 1 or more: that value (code x 2^128) "
                                   "overflows fp32 in the reference's decoding as well");
  return CSK_OK;
}

int dequant_to_host(const csk_mxfp4& m, float* host_out) {
  float* d = nullptr;
  const size_t n = (size_t)m.rows * m.K;
  HIP_TRY(counted_malloc((void**)&d, n * sizeof(float)));
  const long ent = m.entries();
  dequant_mxfp4_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(
      m.q, m.s, d, (int)m.rows, (int)m.nblk, ent);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpyAsync(host_out, d, n * sizeof(float), hipMemcpyDeviceToHost, g_stream);
  hipError_t e2 = hipStreamSynchronize(g_stream);
  (void)hipFree(d);
  if (e != hipSuccess) return fail(CSK_ERR_HIP, std::string("dequant: ") + hipGetErrorString(e));
  if (e2 != hipSuccess) return fail(CSK_ERR_HIP, std::string("dequant sync: ") + hipGetErrorString(e2));
  return CSK_OK;
}

int export_to_host(const csk_mxfp4& m, uint8_t* host_out) {
  uint8_t* d = nullptr;
  const size_t n = (size_t)m.rows * m.nblk * 17;
  HIP_TRY(counted_malloc((void**)&d, n));
  const long ent = m.entries();
  export_mxfp4_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(
      m.q, m.s, d, (int)m.rows, (int)m.nblk, ent);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpyAsync(host_out, d, n, hipMemcpyDeviceToHost, g_stream);
  hipError_t e2 = hipStreamSynchronize(g_stream);
  (void)hipFree(d);
  if (e != hipSuccess) return fail(CSK_ERR_HIP, std::string("export: ") + hipGetErrorString(e));
  if (e2 != hipSuccess) return fail(CSK_ERR_HIP, std::string("export sync: ") + hipGetErrorString(e2));
  return CSK_OK;
}

int launch_prep(const float* src, const float* norm_w, float eps, float* xn, int64_t rows, int64_t H) {
  if (rows == 0) return CSK_OK;
  prep_kernel<<<dim3((unsigned)rows), 256, 0, g_stream>>>(src, norm_w, eps, xn, (int)H);
  return check_launch("prep_kernel");
}

// x [*, H] fp32 -> three-term FP6 rows (the grouped GEMM's activation operand).
int launch_mx3(const float* x, uint16_t* x3, int64_t rows, int64_t H, const int* gather_tok,
               const float* gather_w) {
  if (rows == 0) return CSK_OK;
  const int64_t nb = rows * mx3_row_blocks((int)(H / 32));
  mx3_rows_kernel<<<dim3((unsigned)cdiv(nb, 256)), 256, 0, g_stream>>>(
      x, reinterpret_cast<u32x4*>(x3), rows, (int)(H / 32), gather_tok, gather_w);
  return check_launch("mx3_rows_kernel");
}

// Small batches stream the weights once (HBM-bound, activations quantised in the kernel); larger
// ones run the grouped GEMM on the block-scaled matrix instruction (three-term FP6
// activations).  One decision per forward: it fixes the activation format of both GEMMs.
// What counts is tokens per expert: a 64-token M tile of the GEMM that holds a handful of
// tokens costs as much as a full one, while the streaming kernel passes over an expert once
// per seven of its tokens.  Measured crossover: about twelve assignments per expert (20b
// shape: T = 96 a tie, T = 128 the GEMM 16 % faster; 120b shape: T = 128 streaming 17 %
// faster, T = 256 8 %, T = 512 the GEMM 33 % faster).
bool stream_path(int64_t T, int64_t H, int64_t F, int64_t E, int64_t k) {
  if (H / 32 > 96 || F / 32 > 96) return false;
  return T <= 64 || (T * k <= 10 * E && T * k <= kStreamMaxP);
}

// mx3_out: also rewrite the rows x as FP6 terms (the grouped GEMM's operand), riding on the
// top-k launch.
int launch_router(const float* x, const float* gate_w, const float* gate_b, int64_t T, int64_t E,
                  int64_t H, int64_t k, int sigmoid, float* logits, float* pairs, int* ids,
                  uint16_t* mx3_out = nullptr) {
  if (T == 0) return CSK_OK;
  const unsigned gx = (unsigned)cdiv(E, 4);
  int nsplit = 0;  // > 0: the logits kernel wrote partial logits behind the [T, E] final ones
  if (T <= 2) {
    router_logits_kernel<1><<<dim3(gx, (unsigned)T), 256, 0, g_stream>>>(x, gate_w, gate_b, logits,
                                                                         (int)T, (int)E, (int)H);
  } else if (T <= 64) {
    router_logits_kernel<4><<<dim3(gx, (unsigned)cdiv(T, 4)), 256, 0, g_stream>>>(
        x, gate_w, gate_b, logits, (int)T, (int)E, (int)H);
  } else if (H % 16 == 0 && cdiv(H, 64) <= kRouterChunks * kRouterMaxSplits) {
    // splits of H: as many as it takes to keep a split's token rows in registers, and to give
    // the chip two workgroups per compute unit
    const int64_t nchunk = cdiv(H, 64);
    int64_t splits = std::max(cdiv(nchunk, kRouterChunks), cdiv(2 * std::max(g_cus, 1), cdiv(T, 32)));
    splits = std::min<int64_t>(std::min<int64_t>(splits, kRouterMaxSplits), nchunk);
    const int64_t cps = cdiv(nchunk, splits);
    nsplit = (int)cdiv(nchunk, cps);
    router_logits_mfma_kernel<<<dim3((unsigned)cdiv(T, 32), (unsigned)nsplit), 256, 0, g_stream>>>(
        x, gate_w, logits + T * E, (int)T, (int)E, (int)H, (int)cps);
  } else {
    router_logits_kernel<4><<<dim3(gx, (unsigned)cdiv(T, 4)), 256, 0, g_stream>>>(
        x, gate_w, gate_b, logits, (int)T, (int)E, (int)H);
  }
  int rc = check_launch("router_logits_kernel");
  if (rc != CSK_OK) return rc;
  Mx3Rider rider{};
  int64_t riders = 0;
  if (mx3_out) {
    rider = Mx3Rider{x, reinterpret_cast<u32x4*>(mx3_out), (long)T, (int)(H / 32), (int)cdiv(T, 4)};
    riders = cdiv(T * mx3_row_blocks((int)(H / 32)), 256);
  }
  router_topk_kernel<<<dim3((unsigned)(cdiv(T, 4) + riders)), 256, 0, g_stream>>>(
      logits, pairs, ids, (int)T, (int)E, (int)k, sigmoid, x, gate_w, gate_b, (int)H, logits + T * E, nsplit, rider);
  return check_launch("router_topk_kernel");
}

// Tokens of an expert contracted per pass over its weights by the streaming kernel.  An
// expert with more tokens than that is streamed once per group, so larger batches take
// groups of seven (what two workgroups per compute unit can hold in LDS; measured against
// six: 20b T = 64 162 -> 151 us, 120b T = 64 245 -> 239 us); up to 16 tokens few experts see
// more than four, the second pass of those that do is served by the memory-side cache, and
// the four-token form is marginally the faster one (measured at T = 8, 16, 32).
inline int stream_group_tokens(int64_t T) { return T <= 16 ? kStreamG : kStreamGWide; }

int launch_dispatch(const int* ids, const float* pairs, int64_t P, int64_t k, int64_t E,
                    const ExpertW* ew, Workspace& ws) {
  dispatch_scatter_kernel<<<dim3((unsigned)cdiv(std::max<int64_t>(P, 1), kDispatchThreads)), kDispatchThreads, 0, g_stream>>>(
      ids, pairs, (int)P, (int)k, (int)E, ws.counts, ew, ws.offsets, ws.desc,
      P <= kStreamMaxP ? ws.groups : nullptr, ws.nv, ws.tiles, ws.n_tiles, ws.list_tok, ws.list_w,
      ws.pos, stream_group_tokens(P / std::max<int64_t>(k, 1)));
  return check_launch("dispatch_scatter_kernel");
}

// Weight-streaming kernel for small batches (every expert sees few tokens, the
// layer is HBM-bound); grouped GEMM otherwise.
template <int NMAT, int G, bool ROUTE1 = false>
int launch_stream(ExpertStreamArgs a, int64_t P, Workspace& ws) {
  a.groups = ws.groups;
  a.nv = ws.nv;
  // kStreamWgPerCu workgroups per compute unit in steady state; a batch so small that
  // every work unit can have a resident workgroup of its own gets that
  const int64_t npair = NMAT == 2 ? a.ntile : (a.ntile + 1) / 2;
  const int64_t cus = std::max(g_cus, 1);
  const int64_t nwg = (G == kStreamG && P * npair <= kStreamWgPerCu * cus) ? P * npair : kStreamWgPerCu * cus;  // (small P implies G == kStreamG)
  // activation rows as three FP6 terms (96 B per block, 96 blocks per row: zeros past K) + the reduction buffers
  size_t lds = (size_t)G * 96 * (kMx3ChunksPerBlock * 16) + (size_t)2 * 4 * ((G + 3) / 4) * 8 * 16 * sizeof(float);
  if (ROUTE1) lds = std::max(lds, sizeof(CloseCallLds));  // a close call is recomputed where the rows go afterwards
  static bool lds_attr_set = false;  // per instantiation: dynamic LDS beyond the default limit is asked for once
  if (!lds_attr_set) {
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&expert_stream_kernel<NMAT == 2 ? 0 : 1, G, ROUTE1>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    lds_attr_set = true;
  }
  launch_expert_kernel(NMAT == 2 ? 0 : 1, expert_stream_kernel<NMAT == 2 ? 0 : 1, G, ROUTE1>, dim3((unsigned)nwg), dim3(256), lds, a);
  return check_launch("expert_stream_kernel");
}

template <int NMAT>
int launch_experts(ExpertStreamArgs a, const uint16_t* a_mx3, uint16_t* act_mx3, int64_t E, int64_t T, int64_t P,
                   Workspace& ws, bool stream) {
  if (stream) {
    if constexpr (NMAT == 2)
      if (a.rin.logits) return launch_stream<NMAT, kStreamG, true>(a, P, ws);  // one token, routed by the kernel itself
    return stream_group_tokens(T) == kStreamG ? launch_stream<NMAT, kStreamG>(a, P, ws)
                                              : launch_stream<NMAT, kStreamGWide>(a, P, ws);
  }
  ExpertGemmMxArgs ga{};
  ga.desc = a.desc;
  ga.mtiles = ws.tiles;
  ga.n_mtiles = ws.n_tiles;
  ga.list_row = a.list_row;
  ga.A = reinterpret_cast<const uint4*>(a_mx3);
  ga.nblk = a.nblk;
  ga.ntile = a.ntile;
  ga.N = a.N;
  ga.act_type = a.act_type;
  ga.act_out = reinterpret_cast<u32x4*>(act_mx3);
  ga.y_out = a.y_out;
  using Geom = MxGeom<kMxNG, 2>;
  constexpr int kMode = NMAT == 2 ? 0 : 1;
  if (a.ntile % 2) return fail(CSK_ERR_ARG, "grouped GEMM: the number of output features must be a multiple of 32");
  ga.n_ntiles = (int)cdiv(a.ntile, Geom::tiles_per_wg(kMode));
  // per-lane offsets into the activation rows are 32-bit (the weight offsets are tile-relative)
  const int64_t a_rows = a.list_row ? T : P;
  if (a_rows * mx3_row_blocks(a.nblk) * 96 >= ((int64_t)1 << 32))
    return fail(CSK_ERR_ARG, "batch too large for the grouped GEMM (activation rows exceed 4 GiB)");
  static bool lds_attr_set[2] = {false, false};
  if (!lds_attr_set[kMode]) {
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&expert_gemm_mx_kernel<kMode, kMxNG>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)Geom::kLdsBytes));
    lds_attr_set[kMode] = true;
  }
  const int64_t max_mtiles = P / kGemmBM + std::min<int64_t>(E, P);
  const dim3 grid((unsigned)(cdiv(max_mtiles * ga.n_ntiles, kDies) * kDies));
  launch_expert_kernel(kMode, expert_gemm_mx_kernel<kMode, kMxNG>, grid, dim3(64 * kMxWaves), Geom::kLdsBytes, ga);
  return check_launch("expert_gemm_mx_kernel");
}

// Activation rows of the expert MLPs.  The streaming path reads them as fp32 (`x`, row of a
// packed position through list_row, optionally scaled by gather_w) and quantises them
// itself; the grouped GEMM reads rows already written as three FP6 terms (`x_mx3`, indexed
// through mx3_list_row or directly by packed position).
struct ExpertInput {
  const float* x;
  const int* list_row;
  const float* gather_w;
  const uint16_t* x_mx3;
  const int* mx3_list_row;
  const uint16_t* x_mx3_tokens = nullptr;  // streaming path: the token rows already as FP6 terms (written by the routing prologue)
  const RouteIn* rin = nullptr;    // both set: a one-token batch that the gate/up kernel routes itself
  const RouteOut* rout = nullptr;
};

// Experts' MLPs over the dispatched tokens: ws.y[P,H] <- down(act(gate, up)).
int run_experts(int64_t E, int64_t T, int64_t k, int64_t H, int64_t F,
                int act_type, const ExpertInput& in, Workspace& ws, bool timed = false) {
  const int64_t P = T * k;
  const bool stream = stream_path(T, H, F, E, k);
  ExpertStreamArgs a{};
  a.desc = ws.desc;
  a.act_type = act_type;
  // a single token of a routed layer names k different experts: k token groups, known here
  a.nv_known = (stream && T == 1 && E > 1) ? (int)k : 0;
  // gate/up + activation
  a.list_row = stream ? in.list_row : in.mx3_list_row;
  a.gather_w = in.gather_w;
  a.X = in.x;
  a.X3 = stream ? reinterpret_cast<const u32x4*>(in.x_mx3_tokens) : nullptr;
  a.zeros = g_zero;
  a.nblk = (int)(H / 32);
  a.N = (int)F;
  a.ntile = (int)cdiv(F, 16);
  a.act_out = reinterpret_cast<float*>(ws.act);  // [P][F] fp32 (streaming) or three-term rows (GEMM), same bytes
  a.y_out = nullptr;
  if (timed) mark(CSK_STAGE_GATEUP);
  if (in.rin && in.rout) {
    if (!stream || T != 1) return fail(CSK_ERR_STATE, "in-kernel routing is for one token on the streaming path");
    a.rin = *in.rin, a.rout = *in.rout;
  }
  int rc = launch_experts<2>(a, in.x_mx3, ws.act, E, T, P, ws, stream);
  if (rc != CSK_OK) return rc;
  a.rin = RouteIn{}, a.rout = RouteOut{};
  if (timed) mark(CSK_STAGE_DOWN);
  // down
  a.list_row = nullptr;
  a.gather_w = nullptr;
  a.X3 = nullptr;
  a.X = reinterpret_cast<const float*>(ws.act);
  a.nblk = (int)(F / 32);
  a.N = (int)H;
  a.ntile = (int)cdiv(H, 16);
  a.act_out = nullptr;
  a.y_out = ws.y;
  return launch_experts<1>(a, ws.act, nullptr, E, T, P, ws, stream);
}

int launch_combine(const float* y, const float* pairs, const int* pos, const float* residual,
                   float* out, int64_t T, int64_t k, int64_t H, int pre_weighted) {
  if (T == 0) return CSK_OK;
  combine_kernel<<<dim3((unsigned)cdiv(H, 1024), (unsigned)T), 256, 0, g_stream>>>(
      y, pairs, pos, residual, out, (int)T, (int)k, (int)H, pre_weighted);
  return check_launch("combine_kernel");
}

int F16Scratch::ensure(size_t rows_, size_t width_) {
  if (rows_ <= rows && width_ <= width) return CSK_OK;
  HIP_TRY(hipStreamSynchronize(g_stream));
  const size_t nr = std::max(rows, rows_), nw = std::max(width, width_);
  for (void* p : {(void*)actf, (void*)rs_x, (void*)rs_a})
    if (p) (void)hipFree(p);
  actf = nullptr, rs_x = nullptr, rs_a = nullptr, rows = 0, width = 0;
  int rc = dev_alloc(&actf, nr * nw);
  if (rc == CSK_OK) rc = dev_alloc(&rs_x, nr);
  if (rc == CSK_OK) rc = dev_alloc(&rs_a, nr);
  if (rc != CSK_OK) return rc;
  rows = nr, width = nw;
  return CSK_OK;
}

// rows of K values read from source rows of Ksrc values (Ksrc = K, or K / 2: each row twice over)
int launch_f16_split(const float* x, int64_t rows, int64_t K, const int* gather_tok,
                     const float* gather_w, uint16_t* out, float* rscale, int64_t Ksrc = 0) {
  if (rows == 0) return CSK_OK;
  f16_split_rows_kernel<<<dim3((unsigned)rows), 256, 0, g_stream>>>(
      x, (long)K, (long)(Ksrc ? Ksrc : K), gather_tok, gather_w, reinterpret_cast<u32x4*>(out), rscale);
  return check_launch("f16_split_rows_kernel");
}

// y[P, N] <- W_down(expert of the position) x rows + b_down over two-term fp16 rows [P, K]:
// the down projection of the experts, and any plain linear layer (one descriptor).
int launch_f16_projection(int64_t E, int64_t T, int64_t P, int64_t K, int64_t N, const uint16_t* rows,
                          const float* rscale, float* y, Workspace& ws, float wscale = 1.0f) {
  if (T <= 64) {
    ExpertF16Args a{};
    a.desc = ws.desc;
    a.n_slots = (int)E;
    a.list_row = nullptr;
    a.B = reinterpret_cast<const u32x4*>(rows);
    a.rscale = rscale;
    a.wscale[0] = a.wscale[1] = wscale;
    a.nkb = (int)f16_block_count(K);
    a.N = (int)N;
    a.ntile = (int)f16_tile_count(N);
    a.out = y;
    expert_f16_kernel<1><<<dim3((unsigned)(4 * std::max(g_cus, 1))), 256, 0, g_stream>>>(a);
  } else {
    ExpertF16GemmArgs ga{};
    ga.desc = ws.desc;
    ga.mtiles = ws.tiles;
    ga.n_mtiles = ws.n_tiles;
    ga.list_row = nullptr;
    ga.B = reinterpret_cast<const u32x4*>(rows);
    ga.rscale = rscale;
    ga.wscale[0] = ga.wscale[1] = wscale;
    ga.nkb = (int)f16_block_count(K);
    ga.N = (int)N;
    ga.ntile = (int)f16_tile_count(N);
    ga.n_ntiles = (int)cdiv(N, 256);
    ga.out = y;
    const int64_t max_mtiles = P / 64 + std::min<int64_t>(E, P);
    expert_f16_gemm_kernel<1><<<dim3((unsigned)(cdiv(max_mtiles * ga.n_ntiles, kF16Dies) * kF16Dies)), 256, 0, g_stream>>>(ga);
  }
  return check_launch("expert_f16_kernel<1>");
}

// Experts with fp16 weights over the dispatched tokens: ws.y[P,H] <- down(act(gate, up)).
// x is [T,H] fp32.  Up to 64 tokens every expert's tokens form groups of 16 (one pass over
// the weights per group, HBM-bound); beyond that groups of 64.
// dup: the weights are fp32 matrices kept as two fp16 terms side by side ([F, 2 H] and
// [H, 2 F]), so every activation row is contracted twice over.
int run_experts_f16(int64_t E, int64_t T, int64_t k, int64_t H, int64_t F, int act_type,
                    const float* x, bool weight_before_ffn, int64_t gather_rows, Workspace& ws,
                    bool timed = false, bool identity_rows = false, bool dup = false,
                    const float* wscales = nullptr /* gate, up, down; null: all 1 */) {
  const int64_t P = T * k;
  const int64_t KH = dup ? 2 * H : H, KF = dup ? 2 * F : F;
  int rc = g_f16.ensure((size_t)P, (size_t)F);
  if (rc != CSK_OK) return rc;
  ExpertF16Args a{};
  a.desc = ws.desc;
  a.n_slots = (int)E;
  a.act_type = act_type;
  if (weight_before_ffn) {
    // rows gathered per dispatch position and scaled by the routing weight first
    rc = launch_f16_split(x, gather_rows, KH, ws.list_tok, ws.list_w, ws.xg, g_f16.rs_x, H);
    a.list_row = nullptr;
    a.B = reinterpret_cast<const u32x4*>(ws.xg);
  } else {
    rc = launch_f16_split(x, T, KH, nullptr, nullptr, ws.xs, g_f16.rs_x, H);
    a.list_row = identity_rows ? nullptr : ws.list_tok;  // identity: position p is token p
    a.B = reinterpret_cast<const u32x4*>(ws.xs);
  }
  if (rc != CSK_OK) return rc;
  const bool small = T <= 64;
  const dim3 grid((unsigned)(4 * std::max(g_cus, 1)));
  ExpertF16GemmArgs ga{};
  ga.desc = ws.desc;
  ga.mtiles = ws.tiles;
  ga.n_mtiles = ws.n_tiles;
  ga.act_type = act_type;
  const int64_t max_mtiles = P / 64 + std::min<int64_t>(E, P);
  auto gemm_grid = [&](int n_ntiles) { return dim3((unsigned)(cdiv(max_mtiles * n_ntiles, kF16Dies) * kF16Dies)); };
  a.rscale = g_f16.rs_x;
  a.wscale[0] = wscales ? wscales[0] : 1.0f;
  a.wscale[1] = wscales ? wscales[1] : 1.0f;
  a.nkb = (int)f16_block_count(KH);
  a.N = (int)F;
  a.ntile = (int)f16_tile_count(F);
  a.out = g_f16.actf;
  if (timed) mark(CSK_STAGE_GATEUP);
  if (small) {
    expert_f16_kernel<0><<<grid, 256, 0, g_stream>>>(a);
  } else {
    ga.list_row = a.list_row, ga.B = a.B, ga.rscale = a.rscale, ga.nkb = a.nkb, ga.N = a.N;
    ga.wscale[0] = a.wscale[0], ga.wscale[1] = a.wscale[1];
    ga.ntile = a.ntile, ga.out = a.out;
    ga.n_ntiles = (int)cdiv(F, 128);
    expert_f16_gemm_kernel<0><<<gemm_grid(ga.n_ntiles), 256, 0, g_stream>>>(ga);
  }
  if ((rc = check_launch("expert_f16_kernel<0>")) != CSK_OK) return rc;
  if (timed) mark(CSK_STAGE_DOWN);
  if ((rc = launch_f16_split(g_f16.actf, P, KF, nullptr, nullptr, ws.act, g_f16.rs_a, F)) != CSK_OK) return rc;
  return launch_f16_projection(E, T, P, KF, H, ws.act, g_f16.rs_a, ws.y, ws, wscales ? wscales[2] : 1.0f);
}

int check_dims(int64_t E, int64_t k, int64_t H, int64_t F) {
  if (E <= 0 || E > kMaxExperts) return fail(CSK_ERR_ARG, "num_experts must be in 1..256");
  if (k <= 0 || k > kMaxTopK || k > E) return fail(CSK_ERR_ARG, "top_k must be in 1..min(16, E)");
  if (H <= 0 || H % 32 || H > (int64_t)kZeroLen) return fail(CSK_ERR_ARG, "hidden_dim must be a positive multiple of 32, at most 65536");
  if (F <= 0 || F % 32 || F > (int64_t)kZeroLen) return fail(CSK_ERR_ARG, "expert_ffn_dim must be a positive multiple of 32, at most 65536");
  return CSK_OK;
}

}  // namespace

// ============================================================ process-wide

extern "C" int csk_init(int device) {
  API_LOCK();
  int n = 0;
  HIP_TRY(hipGetDeviceCount(&n));
  if (device < 0 || device >= n) return fail(CSK_ERR_HIP, "no such GPU device");
  HIP_TRY(hipSetDevice(device));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0)
    return fail(CSK_ERR_HIP, std::string("device is ") + prop.gcnArchName + ", this library is built for gfx950 only");
  if (!g_stream) HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
  if (!g_zero) {
    HIP_TRY(counted_malloc((void**)&g_zero, kZeroLen * sizeof(float)));
    HIP_TRY(hipMemset(g_zero, 0, kZeroLen * sizeof(float)));
  }
  if (device >= kMaxDevices) return fail(CSK_ERR_HIP, "device index beyond the library's table");
  if (!g_scratch_ptr[device]) {
    // this GPU's copy of the load-time array (the device chosen above is current)
    unsigned char* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(CSK_ERR_HIP, "hipGetSymbolAddress returned a null address for the fixed workspace");
    g_scratch_ptr[device] = ptr;
  }
  carve_fixed_workspace(g_ws_fixed, g_scratch_ptr[device]);
  g_device = device;
  g_cus = prop.multiProcessorCount;
  g_ready = true;
  t_device_bound = true;
  return CSK_OK;
}

extern "C" const char* csk_last_error(void) { return g_err.c_str(); }
// for the library's other translation units (not part of the public header)
extern "C" void csk_set_error_(const char* msg) { g_err = msg ? msg : ""; }

extern "C" int csk_device_info(char* name, size_t cap, int* compute_units, size_t* hbm_bytes) {
  REQUIRE_INIT();
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, g_device));
  if (name && cap) {
    std::snprintf(name, cap, "%s (%s)", prop.name, prop.gcnArchName);
  }
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
  return CSK_OK;
}

extern "C" int csk_device_memory(size_t* free_bytes, size_t* total_bytes) {
  REQUIRE_INIT();
  size_t f = 0, t = 0;
  HIP_TRY(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return CSK_OK;
}

extern "C" int csk_alloc_count(uint64_t* count) {
  if (!count) return fail(CSK_ERR_ARG, "csk_alloc_count: null output");
  *count = g_alloc_count.load(std::memory_order_relaxed);
  return CSK_OK;
}

extern "C" int csk_stage_timing(int enable) {
  REQUIRE_INIT();
  if (enable && !g_stage_ev[0]) {
    for (auto& e : g_stage_ev) HIP_TRY(hipEventCreate(&e));
    for (auto& pair : g_kern_ev)
      for (auto& e : pair) HIP_TRY(hipEventCreate(&e));
  }
  g_timing = enable != 0;
  g_stage_valid = false;
  g_kern_valid = false;
  return CSK_OK;
}
extern "C" int csk_kernel_times(float* ms_out) {
  REQUIRE_INIT();
  if (!ms_out) return fail(CSK_ERR_ARG, "csk_kernel_times: null output");
  if (!g_stage_valid || !g_kern_valid)
    return fail(CSK_ERR_STATE, "no forward of an MXFP4 layer has run with stage timing enabled");
  for (int i = 0; i < 2; ++i) {
    HIP_TRY(hipEventSynchronize(g_kern_ev[i][1]));
    HIP_TRY(hipEventElapsedTime(&ms_out[i], g_kern_ev[i][0], g_kern_ev[i][1]));
  }
  return CSK_OK;
}
extern "C" int csk_stage_times(float* ms_out) {
  REQUIRE_INIT();
  if (!ms_out) return fail(CSK_ERR_ARG, "csk_stage_times: null output");
  if (!g_stage_valid) return fail(CSK_ERR_STATE, "no forward has run with stage timing enabled");
  HIP_TRY(hipEventSynchronize(g_stage_ev[CSK_N_STAGES]));
  for (int i = 0; i < CSK_N_STAGES; ++i) HIP_TRY(hipEventElapsedTime(&ms_out[i], g_stage_ev[i], g_stage_ev[i + 1]));
  return CSK_OK;
}

extern "C" void* csk_dev_alloc(size_t bytes) {
  if (!g_ready) {
    g_err = "csk_init has not been called";
    return nullptr;
  }
  if (!t_device_bound && hipSetDevice(g_device) == hipSuccess) t_device_bound = true;
  void* p = nullptr;
  hipError_t e = counted_malloc(&p, bytes ? bytes : 1);
  if (e != hipSuccess) {
    g_err = std::string("hipMalloc: ") + hipGetErrorString(e);
    return nullptr;
  }
  return p;
}
extern "C" void csk_dev_free(void* p) {
  if (p) (void)hipFree(p);
}
extern "C" int csk_copy_h2d(void* dst, const void* src, size_t bytes) {
  REQUIRE_INIT();
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
  HIP_TRY(hipStreamSynchronize(g_stream));
  return CSK_OK;
}
extern "C" int csk_copy_d2h(void* dst, const void* src, size_t bytes) {
  REQUIRE_INIT();
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
  HIP_TRY(hipStreamSynchronize(g_stream));
  return CSK_OK;
}
namespace {
__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, long n) {
  const long stride = (long)gridDim.x * 256;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}
}  // namespace
extern "C" int csk_copy_d2d(void* dst, const void* src, size_t bytes) {
  REQUIRE_INIT();
  if (!dst || !src || bytes % 16) return fail(CSK_ERR_ARG, "csk_copy_d2d: null pointer or size not a multiple of 16");
  if (bytes == 0) return CSK_OK;
  const long n = (long)(bytes / 16);
  const long blocks = std::min<long>(cdiv(n, 256), 8L * std::max(g_cus, 1));
  copy_kernel<<<dim3((unsigned)blocks), 256, 0, g_stream>>>((const uint4*)src, (uint4*)dst, n);
  return check_launch("copy_kernel");
}
extern "C" int csk_synchronize(void) {
  REQUIRE_INIT();
  HIP_TRY(hipStreamSynchronize(g_stream));
  return CSK_OK;
}
extern "C" csk_event* csk_event_create(void) {
  if (!g_ready) return nullptr;
  csk_event* e = new csk_event;
  if (hipEventCreate(&e->ev) != hipSuccess) {
    delete e;
    return nullptr;
  }
  return e;
}
extern "C" void csk_event_destroy(csk_event* e) {
  if (!e) return;
  (void)hipEventDestroy(e->ev);
  delete e;
}
extern "C" int csk_event_record(csk_event* e) {
  REQUIRE_INIT();
  if (!e) return fail(CSK_ERR_ARG, "null event");
  HIP_TRY(hipEventRecord(e->ev, g_stream));
  return CSK_OK;
}
extern "C" int csk_event_elapsed_ms(csk_event* a, csk_event* b, float* ms) {
  REQUIRE_INIT();
  if (!a || !b || !ms) return fail(CSK_ERR_ARG, "null event");
  HIP_TRY(hipEventSynchronize(b->ev));
  HIP_TRY(hipEventElapsedTime(ms, a->ev, b->ev));
  return CSK_OK;
}

// ============================================================ MXFP4 matrices

extern "C" int csk_mxfp4_upload(const uint8_t* blocks, int64_t rows, int64_t K, csk_mxfp4** out) {
  REQUIRE_INIT();
  if (!blocks || !out || rows <= 0 || K <= 0 || K % 32)
    return fail(CSK_ERR_ARG, "csk_mxfp4_upload: need rows > 0 and K a positive multiple of 32");
  csk_mxfp4* m = new csk_mxfp4;
  m->rows = rows;
  m->K = K;
  m->nblk = K / 32;
  m->ntile = cdiv(rows, 16);
  int rc = dev_alloc(&m->q, (size_t)m->entries() + kWeightSlack / sizeof(uint4));
  if (rc == CSK_OK) rc = dev_alloc(&m->s, (size_t)m->scale_bytes() + kWeightSlack);
  if (rc == CSK_OK && hipMemset(m->s, 127, (size_t)m->scale_bytes()) != hipSuccess) rc = fail(CSK_ERR_HIP, "hipMemset failed");
  if (rc == CSK_OK) rc = pack_into(blocks, *m);
  if (rc != CSK_OK) {
    csk_mxfp4_free(m);
    return rc;
  }
  *out = m;
  return CSK_OK;
}
extern "C" void csk_mxfp4_free(csk_mxfp4* m) {
  if (!m) return;
  API_LOCK();
  if (m->owned) {
    if (m->q) (void)hipFree(m->q);
    if (m->s) (void)hipFree(m->s);
  }
  delete m;
}
extern "C" int csk_mxfp4_dequant(const csk_mxfp4* m, float* host_out) {
  REQUIRE_INIT();
  if (!m || !host_out) return fail(CSK_ERR_ARG, "csk_mxfp4_dequant: null argument");
  return dequant_to_host(*m, host_out);
}
extern "C" int csk_mxfp4_export(const csk_mxfp4* m, uint8_t* host_out) {
  REQUIRE_INIT();
  if (!m || !host_out) return fail(CSK_ERR_ARG, "csk_mxfp4_export: null argument");
  return export_to_host(*m, host_out);
}

// ============================================================ layer

static int layer_create(int64_t E, int64_t k, int64_t H, int64_t F, bool f16, csk_layer** out, bool view = false) {
  REQUIRE_INIT();
  if (!out) return fail(CSK_ERR_ARG, "csk_layer_create: null out");
  int rc = check_dims(E, k, H, F);
  if (rc != CSK_OK) return rc;
  csk_layer* L = new csk_layer;
  L->E = E, L->k = k, L->H = H, L->F = F;
  L->f16 = f16;
  L->is_view = view;
  if (view) {
    L->attached.assign((size_t)E, 0);
    L->own_ws = new Workspace;
  }
  L->nblkH = H / 32, L->nblkF = F / 32, L->ntF = cdiv(F, 16), L->ntH = cdiv(H, 16);
  L->expert_set.assign((size_t)E, 0);
  L->expert_bias.assign((size_t)E, 0);
  L->matrix_set.assign((size_t)E, 0);
  L->ew_host.assign((size_t)E, ExpertW{});
  rc = dev_alloc(&L->gate_w, (size_t)E * H);
  if (rc == CSK_OK) rc = dev_alloc(&L->gate_b, (size_t)E);
  // kWeightSlack: the grouped GEMM reads up to three blocks (and the scale loads three
  // bytes) past the end of a plane; behind the last plane that must still be mapped memory
  if (view) {
    // no planes of its own
  } else if (f16) {
    if (rc == CSK_OK) rc = dev_alloc(&L->h_all, (size_t)E * L->ent16_expert());
  } else {
    if (rc == CSK_OK) rc = dev_alloc(&L->q_all, (size_t)E * L->ent_expert() + kWeightSlack / sizeof(uint4));
    if (rc == CSK_OK) rc = dev_alloc(&L->s_all, (size_t)E * L->sc_expert() + kWeightSlack);
    if (rc == CSK_OK && hipMemset(L->s_all, 127, (size_t)E * L->sc_expert()) != hipSuccess) rc = fail(CSK_ERR_HIP, "hipMemset failed");
  }
  if (rc == CSK_OK) rc = dev_alloc(&L->bias_all, (size_t)E * (2 * F + H));
  if (rc == CSK_OK) rc = dev_alloc(&L->ew_dev, (size_t)E);
  if (rc == CSK_OK) rc = dev_alloc(&L->norm_w, (size_t)H);
  if (rc != CSK_OK) {
    csk_layer_destroy(L);
    return rc;
  }
  for (int64_t e = 0; e < E; ++e) {
    ExpertW& w = L->ew_host[(size_t)e];
    if (view) {
      w = ExpertW{};
    } else if (f16) {
      w.q_gate = reinterpret_cast<const uint4*>(L->view16(e, CSK_W_GATE));
      w.q_up = reinterpret_cast<const uint4*>(L->view16(e, CSK_W_UP));
      w.q_down = reinterpret_cast<const uint4*>(L->view16(e, CSK_W_DOWN));
      w.s_gate = w.s_up = w.s_down = nullptr;
    } else {
      const csk_mxfp4 g = L->view(e, CSK_W_GATE), u = L->view(e, CSK_W_UP), d = L->view(e, CSK_W_DOWN);
      w.q_gate = g.q, w.s_gate = g.s, w.q_up = u.q, w.s_up = u.s, w.q_down = d.q, w.s_down = d.s;
    }
    w.b_gate = w.b_up = w.b_down = g_zero;
  }
  hipError_t e1 = hipMemcpy(L->ew_dev, L->ew_host.data(), (size_t)E * sizeof(ExpertW), hipMemcpyHostToDevice);
  if (e1 != hipSuccess) {
    csk_layer_destroy(L);
    return fail(CSK_ERR_HIP, std::string("upload expert table: ") + hipGetErrorString(e1));
  }
  *out = L;
  return CSK_OK;
}

extern "C" int csk_layer_create(int64_t E, int64_t k, int64_t H, int64_t F, csk_layer** out) {
  return layer_create(E, k, H, F, false, out);
}
extern "C" int csk_layer_create_f16(int64_t E, int64_t k, int64_t H, int64_t F, csk_layer** out) {
  return layer_create(E, k, H, F, true, out);
}

extern "C" void csk_layer_destroy(csk_layer* L) {
  if (!L) return;
  API_LOCK();
  if (g_stream) (void)hipStreamSynchronize(g_stream);
  void* ps[] = {L->gate_w, L->gate_b, L->q_all, L->s_all, L->h_all, L->bias_all, L->ew_dev, L->norm_w,
                L->frame.d_hidden, L->frame.d_out};
  for (void* p : ps)
    if (p) (void)hipFree(p);
  if (L->own_ws) {
    static_cast<Workspace*>(L->own_ws)->release();
    delete static_cast<Workspace*>(L->own_ws);
  }
  delete L;
}

extern "C" int csk_layer_set_options(csk_layer* L, int sigmoid_gating, int activation,
                                     int weight_before_ffn) {
  if (!L) return fail(CSK_ERR_ARG, "null layer");
  if (activation != CSK_ACT_MODIFIED_SWIGLU && activation != CSK_ACT_STANDARD_SWIGLU)
    return fail(CSK_ERR_ARG, "unknown activation type");
  L->sigmoid = sigmoid_gating != 0;
  L->act = activation;
  L->wbf = weight_before_ffn != 0;
  return CSK_OK;
}

extern "C" int csk_layer_set_router(csk_layer* L, const float* gate_w, const float* gate_b) {
  REQUIRE_INIT();
  if (!L || !gate_w) return fail(CSK_ERR_ARG, "csk_layer_set_router: null argument");
  HIP_TRY(hipMemcpyAsync(L->gate_w, gate_w, (size_t)L->E * L->H * sizeof(float), hipMemcpyHostToDevice, g_stream));
  if (gate_b)
    HIP_TRY(hipMemcpyAsync(L->gate_b, gate_b, (size_t)L->E * sizeof(float), hipMemcpyHostToDevice, g_stream));
  HIP_TRY(hipStreamSynchronize(g_stream));
  L->has_gate = true;
  L->has_gate_b = gate_b != nullptr;
  return CSK_OK;
}

static int upload_biases(csk_layer* L, int64_t e, const float* b_up, const float* b_gate,
                         const float* b_down) {
  const int nb = (b_up != nullptr) + (b_gate != nullptr) + (b_down != nullptr);
  if (nb != 0 && nb != 3) return fail(CSK_ERR_ARG, "biases must be all present or all absent");
  ExpertW& w = L->ew_host[(size_t)e];
  if (nb == 3) {
    float* base = L->bias_all + (size_t)e * (2 * L->F + L->H);
    HIP_TRY(hipMemcpyAsync(base, b_gate, (size_t)L->F * sizeof(float), hipMemcpyHostToDevice, g_stream));
    HIP_TRY(hipMemcpyAsync(base + L->F, b_up, (size_t)L->F * sizeof(float), hipMemcpyHostToDevice, g_stream));
    HIP_TRY(hipMemcpyAsync(base + 2 * L->F, b_down, (size_t)L->H * sizeof(float), hipMemcpyHostToDevice, g_stream));
    w.b_gate = base, w.b_up = base + L->F, w.b_down = base + 2 * L->F;
  } else {
    w.b_gate = w.b_up = w.b_down = g_zero;
  }
  HIP_TRY(hipMemcpyAsync(L->ew_dev + e, &w, sizeof(ExpertW), hipMemcpyHostToDevice, g_stream));
  HIP_TRY(hipStreamSynchronize(g_stream));
  L->expert_bias[(size_t)e] = nb == 3;
  return CSK_OK;
}

extern "C" int csk_layer_set_expert(csk_layer* L, int64_t e, const uint8_t* w_up,
                                    const uint8_t* w_gate, const uint8_t* w_down,
                                    const float* b_up, const float* b_gate, const float* b_down) {
  REQUIRE_INIT();
  if (!L || e < 0 || e >= L->E) return fail(CSK_ERR_RANGE, "csk_layer_set_expert: expert index out of range");
  if (L->f16 && w_up) return fail(CSK_ERR_STATE, "csk_layer_set_expert: this layer holds fp16 experts (csk_layer_set_expert_f16)");
  if ((w_up == nullptr) != (w_gate == nullptr) || (w_up == nullptr) != (w_down == nullptr))
    return fail(CSK_ERR_ARG, "weights must be all present or all absent");
  if (w_up) {
    const uint8_t* src[3] = {w_up, w_gate, w_down};
    const int which[3] = {CSK_W_UP, CSK_W_GATE, CSK_W_DOWN};
    L->expert_set[(size_t)e] = 0;  // a refused matrix (scale byte out of range) leaves the expert unset
    for (int i = 0; i < 3; ++i) {
      csk_mxfp4 m = L->view(e, which[i]);
      int rc = pack_into(src[i], m);
      if (rc != CSK_OK) return rc;
    }
    L->expert_set[(size_t)e] = 1;
  }
  return upload_biases(L, e, b_up, b_gate, b_down);
}

extern "C" int csk_layer_set_norm(csk_layer* L, const float* weight, float eps) {
  REQUIRE_INIT();
  if (!L || !weight) return fail(CSK_ERR_ARG, "csk_layer_set_norm: null argument");
  HIP_TRY(hipMemcpyAsync(L->norm_w, weight, (size_t)L->H * sizeof(float), hipMemcpyHostToDevice, g_stream));
  HIP_TRY(hipStreamSynchronize(g_stream));
  L->eps = eps;
  L->has_norm = true;
  return CSK_OK;
}

extern "C" int csk_layer_fill_synthetic(csk_layer* L, uint64_t seed, int64_t layer_index,
                                        int scale_lo, int scale_span) {
  REQUIRE_INIT();
  if (!L) return fail(CSK_ERR_ARG, "null layer");
  if (scale_lo < 2 || scale_span < 1 || scale_lo + scale_span - 1 > 254)
    return fail(CSK_ERR_SCALE, "synthetic scale bytes must stay within 2..254");
  if (L->f16) {
    // halves j / 2^14 with j uniform in [-2048, 2047] (exact in fp16), zero in the padding
    for (int64_t e = 0; e < L->E; ++e) {
      for (int which = 0; which < 3; ++which) {
        const bool down = which == CSK_W_DOWN;
        const long rows = down ? L->H : L->F, K = down ? L->F : L->H, ent = f16_entries(rows, K);
        synth_f16_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(
            L->view16(e, which), rows, K, ent,
            seed ^ ((uint64_t)layer_index * 1000003ull + (uint64_t)e * 16ull + (uint64_t)which) * 0x9E3779B97F4A7C15ull);
      }
      L->expert_set[(size_t)e] = 1;
    }
    int rc = check_launch("synth_f16_kernel");
    if (rc != CSK_OK) return rc;
    HIP_TRY(hipStreamSynchronize(g_stream));
    return CSK_OK;
  }
  for (int64_t e = 0; e < L->E; ++e) {
    for (int which = 0; which < 3; ++which) {
      const csk_mxfp4 m = L->view(e, which);
      // host twin of mix64 (same constants as the device function)
      auto mix = [](uint64_t z) {
        z += 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
      };
      const uint64_t key = mix(seed ^ mix((uint64_t)layer_index * 1000003ull + (uint64_t)e * 16ull + (uint64_t)which));
      const long ent = m.entries();
      synth_mxfp4_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(
          m.q, m.s, (int)m.rows, (int)m.nblk, ent, key, scale_lo, scale_span);
    }
    L->expert_set[(size_t)e] = 1;
  }
  int rc = check_launch("synth_mxfp4_kernel");
  if (rc != CSK_OK) return rc;
  HIP_TRY(hipStreamSynchronize(g_stream));
  return CSK_OK;
}

extern "C" int csk_layer_dequant(const csk_layer* L, int64_t e, int which, float* host_out) {
  REQUIRE_INIT();
  if (!L || !host_out || e < 0 || e >= L->E || which < 0 || which > 2)
    return fail(CSK_ERR_ARG, "csk_layer_dequant: bad argument");
  if (L->f16) return fail(CSK_ERR_STATE, "csk_layer_dequant: this layer holds fp16 experts (csk_layer_export_f16)");
  return dequant_to_host(L->view(e, which), host_out);
}
extern "C" int csk_layer_export(const csk_layer* L, int64_t e, int which, uint8_t* host_out) {
  REQUIRE_INIT();
  if (!L || !host_out || e < 0 || e >= L->E || which < 0 || which > 2)
    return fail(CSK_ERR_ARG, "csk_layer_export: bad argument");
  if (L->f16) return fail(CSK_ERR_STATE, "csk_layer_export: this layer holds fp16 experts (csk_layer_export_f16)");
  return export_to_host(L->view(e, which), host_out);
}

// ------------------------------------------------------------ fp16 matrices

struct csk_f16 {
  u32x4* w = nullptr;
  int64_t rows = 0, K = 0;  // K: columns of the resident fp16 matrix
  int64_t Ksrc = 0;         // columns of the matrix the caller gave: K, or K / 2 for fp32 weights kept as [hi | lo]
  bool split() const { return K != Ksrc; }
  float wscale = 1.0f;      // the resident halves hold w / wscale (a power of two; 1 unless the matrix came in as fp32)
};

namespace {
constexpr int kGgmlF16Type = 1;
// bytes of a row-major [rows, K] matrix stored as ggml type F16, Q4_K or Q6_K; 0 = unsupported
size_t ggml_matrix_bytes(int type, int64_t rows, int64_t K) {
  const size_t n = (size_t)rows * K;
  if (type == kGgmlF16Type) return n * 2;
  if (type == kGgmlQ4K) return n % 256 ? 0 : n / 256 * 144;
  if (type == kGgmlQ6K) return n % 256 ? 0 : n / 256 * 210;
  return 0;
}
// row-major matrix on the host (halves, or a Q4_K / Q6_K stream) -> fp16 tiles at dst
int f16_pack_into(const void* data, int type, int64_t rows, int64_t K, u32x4* dst) {
  const size_t bytes = ggml_matrix_bytes(type, rows, K);
  if (!bytes)
    return fail(CSK_ERR_ARG, "fp16 experts take ggml types F16 (1), Q4_K (12) and Q6_K (14), K-quants with rows * K a multiple of 256");
  uint8_t* stage = nullptr;
  HIP_TRY(counted_malloc((void**)&stage, bytes));
  hipError_t e = hipMemcpyAsync(stage, data, bytes, hipMemcpyHostToDevice, g_stream);
  int rc = CSK_OK;
  if (e != hipSuccess) rc = fail(CSK_ERR_HIP, std::string("hipMemcpy: ") + hipGetErrorString(e));
  if (rc == CSK_OK) {
    const long ent = f16_entries(rows, K);
    const dim3 grid((unsigned)cdiv(ent, 256));
    if (type == kGgmlF16Type)
      f16_pack_kernel<<<grid, 256, 0, g_stream>>>(reinterpret_cast<const uint16_t*>(stage), dst, rows, K, ent);
    else if (type == kGgmlQ4K)
      kquant_pack_kernel<kGgmlQ4K><<<grid, 256, 0, g_stream>>>(stage, dst, rows, K, ent);
    else
      kquant_pack_kernel<kGgmlQ6K><<<grid, 256, 0, g_stream>>>(stage, dst, rows, K, ent);
    rc = check_launch("f16_pack_kernel");
  }
  (void)hipStreamSynchronize(g_stream);
  (void)hipFree(stage);
  return rc;
}
int f16_export_from(const u32x4* src, int64_t rows, int64_t K, uint16_t* halves) {
  uint16_t* stage = nullptr;
  const size_t n = (size_t)rows * K;
  HIP_TRY(counted_malloc((void**)&stage, n * sizeof(uint16_t)));
  const long ent = f16_entries(rows, K);
  f16_unpack_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(src, stage, rows, K, ent);
  int rc = check_launch("f16_unpack_kernel");
  if (rc == CSK_OK) {
    hipError_t e = hipMemcpyAsync(halves, stage, n * sizeof(uint16_t), hipMemcpyDeviceToHost, g_stream);
    if (e != hipSuccess) rc = fail(CSK_ERR_HIP, std::string("hipMemcpy: ") + hipGetErrorString(e));
  }
  (void)hipStreamSynchronize(g_stream);
  (void)hipFree(stage);
  return rc;
}
}  // namespace

namespace {
// Device staging of the host-pointer entry points.  A node-level call needs a handful of
// buffers whose sizes repeat from frame to frame (one call per expert node per frame), so
// blocks are kept in a small pool instead of going back to hipFree -- which synchronises the
// device -- and to hipMalloc on the next call.  The entry points hold the library's lock and
// end with the stream idle, so a block returned at scope exit is free for the next call.
struct StagingPool {
  struct Block {
    void* p;
    size_t cap;
  };
  std::vector<Block> idle;
  size_t idle_bytes = 0;
  static constexpr size_t kMaxIdleBytes = (size_t)1 << 30;
  static constexpr size_t kMaxIdleBlocks = 64;
  static size_t size_class(size_t bytes) {  // powers of two from 4 KiB on
    size_t c = 4096;
    while (c < bytes) c <<= 1;
    return c;
  }
  int take(size_t bytes, void** out, size_t* cap) {
    const size_t want = size_class(bytes);
    for (size_t i = 0; i < idle.size(); ++i) {
      if (idle[i].cap == want) {
        *out = idle[i].p, *cap = want;
        idle_bytes -= want;
        idle[i] = idle.back();
        idle.pop_back();
        return CSK_OK;
      }
    }
    HIP_TRY(counted_malloc(out, want));
    *cap = want;
    return CSK_OK;
  }
  void give(void* p, size_t cap) {
    if (idle.size() >= kMaxIdleBlocks || idle_bytes + cap > kMaxIdleBytes) {
      (void)hipFree(p);
      return;
    }
    idle.push_back(Block{p, cap});
    idle_bytes += cap;
  }
};
StagingPool g_staging;

// Pinned host memory between the caller's pageable buffers and the device.  A copy between
// pageable memory and the device is staged by the runtime anyway and returns only when it is
// done, one round trip per call; a node-level call makes five or six small ones.  Through
// this arena they become plain host copies plus asynchronous transfers that overlap one
// another and the kernels, and the call waits once, at its end.  Space is handed out in
// order and taken back all at once when the stream is idle (finish_fetches, or the last
// DevBuf of a call going out of scope); a transfer that does not fit takes the direct path.
struct PinnedArena {
  static constexpr size_t kBytes = (size_t)32 << 20;
  static constexpr size_t kMaxTransfer = (size_t)4 << 20;
  char* base = nullptr;
  size_t used = 0;
  bool failed = false;
  void* take(size_t bytes) {
    if (bytes == 0 || bytes > kMaxTransfer || failed) return nullptr;
    if (!base) {
      if (hipHostMalloc(reinterpret_cast<void**>(&base), kBytes, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        base = nullptr, failed = true;
        return nullptr;
      }
    }
    const size_t at = (used + 255) & ~(size_t)255;
    if (at + bytes > kBytes) return nullptr;
    used = at + bytes;
    return base + at;
  }
  void reset() { used = 0; }
};
PinnedArena g_pinned;
int g_live_devbufs = 0;

// Results on their way to the caller's memory: copied out of the arena once the stream is idle.
struct PendingFetch {
  void* host;
  const void* pinned;
  size_t bytes;
};
std::vector<PendingFetch> g_fetches;

int fetch(void* host, const void* dev, size_t bytes) {
  if (bytes == 0) return CSK_OK;
  if (void* stage = g_pinned.take(bytes)) {
    HIP_TRY(hipMemcpyAsync(stage, dev, bytes, hipMemcpyDeviceToHost, g_stream));
    g_fetches.push_back(PendingFetch{host, stage, bytes});
    return CSK_OK;
  }
  HIP_TRY(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, g_stream));
  return CSK_OK;
}

// Waits for the stream, then completes the fetches.  Every transfer staged in the arena has
// been consumed by then, so its space is free again.
int finish_fetches() {
  const hipError_t e = hipStreamSynchronize(g_stream);
  if (e == hipSuccess)
    for (const PendingFetch& f : g_fetches) std::memcpy(f.host, f.pinned, f.bytes);
  g_fetches.clear();
  g_pinned.reset();
  if (e != hipSuccess) return fail(CSK_ERR_HIP, std::string("stream synchronize: ") + hipGetErrorString(e));
  return CSK_OK;
}

#define CSK_TRY(expr)                  \
  do {                                 \
    const int _rc = (expr);            \
    if (_rc != CSK_OK) return _rc;     \
  } while (0)

// Scoped device buffer for the host-pointer entry points.
struct DevBuf {
  void* p = nullptr;
  size_t cap = 0;
  DevBuf() { ++g_live_devbufs; }
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  ~DevBuf() {
    if (p) g_staging.give(p, cap);
    if (--g_live_devbufs == 0) {  // the call is over: the stream is idle, or the call failed and its fetches are void
      g_fetches.clear();
      g_pinned.reset();
    }
  }
  int alloc(size_t bytes) {
    if (p) {
      if (bytes <= cap) return CSK_OK;
      g_staging.give(p, cap);
      p = nullptr, cap = 0;
    }
    return g_staging.take(bytes ? bytes : 1, &p, &cap);
  }
  int upload(const void* host, size_t bytes) {
    int rc = alloc(bytes);
    if (rc != CSK_OK) return rc;
    if (void* stage = g_pinned.take(bytes)) {
      std::memcpy(stage, host, bytes);
      host = stage;
    }
    HIP_TRY(hipMemcpyAsync(p, host, bytes, hipMemcpyHostToDevice, g_stream));
    return CSK_OK;
  }
  template <class T>
  T* as() {
    return reinterpret_cast<T*>(p);
  }
};

// Several host arrays in one transfer: the pieces are laid out back to back (256-byte
// aligned) in one device block and, when they fit, copied into the pinned arena and sent
// together; otherwise each piece goes up by itself.  A reserved piece is filled by the caller
// once the block's device address is known (a table of pointers into the same block).
struct PackedUpload {
  struct Piece {
    const void* host;  // null: reserved, filled through fill()
    size_t bytes, off;
    std::vector<char> own;  // a reserved piece's contents when there is no stage: alive as long as the object
  };
  DevBuf dev;
  std::vector<Piece> pieces;
  size_t total = 0;
  char* stage = nullptr;
  size_t add(const void* host, size_t bytes) {
    const size_t off = (total + 255) & ~(size_t)255;
    pieces.push_back(Piece{host, bytes, off, {}});
    total = off + bytes;
    return off;
  }
  size_t reserve(size_t bytes) { return add(nullptr, bytes); }
  int begin() {  // after the last add: the device block exists from here on
    CSK_TRY(dev.alloc(total));
    stage = static_cast<char*>(g_pinned.take(total));
    return CSK_OK;
  }
  void fill(size_t off, const void* src, size_t bytes) {
    if (stage) {
      std::memcpy(stage + off, src, bytes);
      return;
    }
    for (Piece& pc : pieces)
      if (pc.off == off) pc.own.assign(static_cast<const char*>(src), static_cast<const char*>(src) + bytes);
  }
  template <class T>
  T* at(size_t off) {
    return reinterpret_cast<T*>(static_cast<char*>(dev.p) + off);
  }
  int commit() {
    if (stage) {
      for (const Piece& pc : pieces)
        if (pc.host) std::memcpy(stage + pc.off, pc.host, pc.bytes);
      HIP_TRY(hipMemcpyAsync(dev.p, stage, total, hipMemcpyHostToDevice, g_stream));
      return CSK_OK;
    }
    for (const Piece& pc : pieces) {
      const void* src = pc.host ? pc.host : static_cast<const void*>(pc.own.data());
      if (pc.bytes && src)
        HIP_TRY(hipMemcpyAsync(static_cast<char*>(dev.p) + pc.off, src, pc.bytes, hipMemcpyHostToDevice, g_stream));
    }
    return CSK_OK;
  }
};

// What one pass of a node-level expert call sends up: the biases, the table of weight and bias
// pointers (completed here with the biases' device addresses), the router output and the
// hidden states of the pass -- one transfer.
struct ExpertCallInputs {
  PackedUpload up;
  const ExpertW* ew = nullptr;
  const float* pairs = nullptr;
  const float* x = nullptr;
  int send(ExpertW w, bool biases, const float* b_up, const float* b_gate, const float* b_down, int64_t F,
           int64_t H, const float* host_pairs, int64_t P, const float* hidden, int64_t n_hidden) {
    size_t o_bu = 0, o_bg = 0, o_bd = 0;
    if (biases) {
      o_bu = up.add(b_up, (size_t)F * 4);
      o_bg = up.add(b_gate, (size_t)F * 4);
      o_bd = up.add(b_down, (size_t)H * 4);
    }
    const size_t o_ew = up.reserve(sizeof(ExpertW));
    const size_t o_pairs = up.add(host_pairs, (size_t)P * 8);
    const size_t o_x = up.add(hidden, (size_t)n_hidden * 4);
    CSK_TRY(up.begin());
    w.b_up = biases ? up.at<float>(o_bu) : g_zero;
    w.b_gate = biases ? up.at<float>(o_bg) : g_zero;
    w.b_down = biases ? up.at<float>(o_bd) : g_zero;
    up.fill(o_ew, &w, sizeof w);
    ew = up.at<ExpertW>(o_ew);
    pairs = up.at<float>(o_pairs);
    x = up.at<float>(o_x);
    return up.commit();
  }
};

// Tokens are independent in every node-level operation, so a long batch is taken in passes:
// grids that have one row of workgroups per token stay inside the launch limits and the
// 32-bit counts of token-expert assignments cannot overflow, whatever T is.
constexpr int64_t kNodePassTokens = 16384;
template <class F>
int for_token_passes(int64_t T, F&& f) {
  for (int64_t t0 = 0; t0 < T; t0 += kNodePassTokens) {
    const int rc = f(t0, std::min(kNodePassTokens, T - t0));
    if (rc != CSK_OK) return rc;
  }
  return CSK_OK;
}
}  // namespace

extern "C" int csk_f16_upload(const uint16_t* halves, int64_t rows, int64_t K, csk_f16** out) {
  REQUIRE_INIT();
  if (!halves || !out || rows <= 0 || K <= 0)
    return fail(CSK_ERR_ARG, "csk_f16_upload: need a matrix with rows > 0 and K > 0");
  if (rows > (int64_t)kZeroLen || K > (int64_t)kZeroLen)
    return fail(CSK_ERR_ARG, "csk_f16_upload: dimensions above 65536 are not supported");
  csk_f16* m = new csk_f16;
  m->rows = rows, m->K = K, m->Ksrc = K;
  int rc = dev_alloc(&m->w, (size_t)f16_entries(rows, K));
  if (rc == CSK_OK) rc = f16_pack_into(halves, kGgmlF16Type, rows, K, m->w);
  if (rc != CSK_OK) {
    csk_f16_free(m);
    return rc;
  }
  *out = m;
  return CSK_OK;
}
extern "C" int csk_f16_upload_ggml(int ggml_type, const void* data, int64_t rows, int64_t K, csk_f16** out) {
  REQUIRE_INIT();
  if (!data || !out || rows <= 0 || K <= 0)
    return fail(CSK_ERR_ARG, "csk_f16_upload_ggml: need a matrix with rows > 0 and K > 0");
  if (rows > (int64_t)kZeroLen || K > (int64_t)kZeroLen)
    return fail(CSK_ERR_ARG, "csk_f16_upload_ggml: dimensions above 65536 are not supported");
  csk_f16* m = new csk_f16;
  m->rows = rows, m->K = K, m->Ksrc = K;
  int rc = dev_alloc(&m->w, (size_t)f16_entries(rows, K));
  if (rc == CSK_OK) rc = f16_pack_into(data, ggml_type, rows, K, m->w);
  if (rc != CSK_OK) {
    csk_f16_free(m);
    return rc;
  }
  *out = m;
  return CSK_OK;
}
extern "C" int csk_f16_upload_f32(const float* w_host, int64_t rows, int64_t K, csk_f16** out) {
  REQUIRE_INIT();
  if (!w_host || !out || rows <= 0 || K <= 0)
    return fail(CSK_ERR_ARG, "csk_f16_upload_f32: need a matrix with rows > 0 and K > 0");
  if (rows > (int64_t)kZeroLen || 2 * K > (int64_t)kZeroLen)
    return fail(CSK_ERR_ARG, "csk_f16_upload_f32: at most 65536 rows and 32768 columns");
  csk_f16* m = new csk_f16;
  m->rows = rows, m->K = 2 * K, m->Ksrc = K;
  const long ent = f16_entries(rows, 2 * K);
  DevBuf stage;
  int rc = dev_alloc(&m->w, (size_t)ent);
  if (rc == CSK_OK) rc = stage.upload(w_host, (size_t)rows * K * 4);
  if (rc == CSK_OK && !g_bad && counted_malloc((void**)&g_bad, sizeof(unsigned long long)) != hipSuccess)
    rc = fail(CSK_ERR_HIP, "hipMalloc failed");
  if (rc == CSK_OK) {
    // largest magnitude first (g_bad's eight bytes serve as the 32-bit cell), then the split of w / wscale
    const long n = (long)rows * K;
    unsigned int top = 0u;
    hipError_t e = hipMemsetAsync(g_bad, 0, sizeof(unsigned long long), g_stream);
    f32_absmax_bits_kernel<<<dim3((unsigned)std::min<long>(cdiv(n, 256), 8L * std::max(g_cus, 1))), 256, 0, g_stream>>>(
        stage.as<float>(), n, reinterpret_cast<unsigned int*>(g_bad));
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(&top, g_bad, sizeof top, hipMemcpyDeviceToHost, g_stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_stream);
    if (e != hipSuccess) {
      rc = fail(CSK_ERR_HIP, std::string("csk_f16_upload_f32: ") + hipGetErrorString(e));
    } else if (top >= 0x7f800000u) {
      rc = fail(CSK_ERR_ARG, "csk_f16_upload_f32: the matrix holds a NaN or an infinity");
    } else {
      // wscale = 2^s with max|w| / 2^s in [2^14, 2^15); s kept where 2^s and 2^-s are normal numbers
      const int eb = (int)(top >> 23);
      const int sexp = top == 0u ? 0 : std::max(-126, std::min(126, eb - 127 - 14));
      m->wscale = std::ldexp(1.0f, sexp);
      f32_split_pack_kernel<<<dim3((unsigned)cdiv(ent, 256)), 256, 0, g_stream>>>(stage.as<float>(), m->w, rows, K, ent,
                                                                                std::ldexp(1.0f, -sexp));
      rc = check_launch("f32_split_pack_kernel");
      if (rc == CSK_OK) {
        e = hipStreamSynchronize(g_stream);  // the staging buffer is released on return
        if (e != hipSuccess) rc = fail(CSK_ERR_HIP, std::string("csk_f16_upload_f32: ") + hipGetErrorString(e));
      }
    }
  }
  if (rc != CSK_OK) {
    csk_f16_free(m);
    return rc;
  }
  *out = m;
  return CSK_OK;
}
extern "C" void csk_f16_free(csk_f16* m) {
  if (!m) return;
  API_LOCK();
  if (m->w) (void)hipFree(m->w);
  delete m;
}
extern "C" int csk_f16_export(const csk_f16* m, uint16_t* halves_out) {
  REQUIRE_INIT();
  if (!m || !halves_out) return fail(CSK_ERR_ARG, "csk_f16_export: null argument");
  return f16_export_from(m->w, m->rows, m->K, halves_out);  // [rows, 2 K] = [hi | lo] for fp32 weights
}

extern "C" int csk_layer_set_expert_f16(csk_layer* L, int64_t e, const uint16_t* w_up,
                                        const uint16_t* w_gate, const uint16_t* w_down,
                                        const float* b_up, const float* b_gate,
                                        const float* b_down) {
  REQUIRE_INIT();
  if (!L || e < 0 || e >= L->E) return fail(CSK_ERR_RANGE, "csk_layer_set_expert_f16: expert index out of range");
  if (!L->f16) return fail(CSK_ERR_STATE, "csk_layer_set_expert_f16: this layer holds MXFP4 experts (csk_layer_create_f16 makes an fp16 one)");
  if ((w_up == nullptr) != (w_gate == nullptr) || (w_up == nullptr) != (w_down == nullptr))
    return fail(CSK_ERR_ARG, "weights must be all present or all absent");
  if (w_up) {
    int rc = f16_pack_into(w_up, kGgmlF16Type, L->F, L->H, L->view16(e, CSK_W_UP));
    if (rc == CSK_OK) rc = f16_pack_into(w_gate, kGgmlF16Type, L->F, L->H, L->view16(e, CSK_W_GATE));
    if (rc == CSK_OK) rc = f16_pack_into(w_down, kGgmlF16Type, L->H, L->F, L->view16(e, CSK_W_DOWN));
    if (rc != CSK_OK) return rc;
    L->matrix_set[(size_t)e] = 7;
    L->expert_set[(size_t)e] = 1;
  }
  return upload_biases(L, e, b_up, b_gate, b_down);
}
extern "C" int csk_layer_set_expert_matrix(csk_layer* L, int64_t e, int which, int ggml_type,
                                           const void* data) {
  REQUIRE_INIT();
  if (!L || !data || e < 0 || e >= L->E || which < 0 || which > 2)
    return fail(CSK_ERR_ARG, "csk_layer_set_expert_matrix: bad argument");
  if (!L->f16) return fail(CSK_ERR_STATE, "csk_layer_set_expert_matrix: this layer holds MXFP4 experts (csk_layer_create_f16 makes an fp16 one)");
  const bool down = which == CSK_W_DOWN;
  int rc = f16_pack_into(data, ggml_type, down ? L->H : L->F, down ? L->F : L->H, L->view16(e, which));
  if (rc != CSK_OK) return rc;
  L->matrix_set[(size_t)e] |= (char)(1 << which);
  if (L->matrix_set[(size_t)e] == 7) L->expert_set[(size_t)e] = 1;
  return CSK_OK;
}
extern "C" int csk_layer_export_f16(const csk_layer* L, int64_t e, int which, uint16_t* halves_out) {
  REQUIRE_INIT();
  if (!L || !halves_out || e < 0 || e >= L->E || which < 0 || which > 2)
    return fail(CSK_ERR_ARG, "csk_layer_export_f16: bad argument");
  if (!L->f16) return fail(CSK_ERR_STATE, "csk_layer_export_f16: this layer holds MXFP4 experts");
  const bool down = which == CSK_W_DOWN;
  return f16_export_from(L->view16(e, which), down ? L->H : L->F, down ? L->F : L->H, halves_out);
}

static int layer_ready(const csk_layer* L, int flags) {
  if (!L->has_gate) return fail(CSK_ERR_STATE, "router weights not set");
  for (char c : L->expert_set)
    if (!c) return fail(CSK_ERR_STATE, "not every expert has weights");
  if ((flags & CSK_FWD_RMSNORM) && !L->has_norm) return fail(CSK_ERR_STATE, "RMSNorm weight not set");
  return CSK_OK;
}

namespace {
// Tokens are independent of one another, so a long batch is processed in passes of at most
// g_pass_tokens tokens: the workspace stays bounded and the 32-bit offsets of the grouped
// GEMM always fit.  Passes are of (nearly) equal size, so that all of them take the same
// kernels.
int64_t g_pass_tokens = 32768;

// Largest batch routed by the single-workgroup kernel.  Its sixteen waves take the tokens four
// at a time one after the other; beyond 32 tokens, selection spread over T / 4 workgroups
// followed by the dispatch kernel is faster although it is a launch more (120b shape, routing
// stage: 17.6 -> 15.7 us at T = 48, 20.8 -> 15.9 at T = 64; no gain at 32, a loss at 24).
constexpr int64_t kRouteSmallTokens = 32;
// phase 0: the whole forward; 1: up to and including the dispatch (router output and lists
// are in ws); 2: the rest (experts and combine) of a pass whose phase 1 ran in the same ws.
int forward_pass(csk_layer* L, const float* hidden, int64_t T, float* out, int flags, Workspace& ws = g_ws,
                 int phase = 0) {
  int rc = CSK_OK;
  if (phase != 2) {
    rc = ws.ensure(T, L->E, L->k, L->H, L->F, L->wbf);
    if (rc != CSK_OK) return rc;
    L->last_ws = &ws;
    L->last_run = ++ws.runs;
  }
  const int64_t P = T * L->k;
  const bool norm = (flags & CSK_FWD_RMSNORM) != 0;
  const float* xr = norm ? ws.xn : hidden;
  bool route_in_kernel = false, rows_mx3_ready = false;
  RouteIn rin_kept{};
  RouteOut rout_kept{};
  if (phase == 2) {
    // routed already
  } else if (P <= 1024 && T <= 64) {
    // small batch: prologue + logits in one launch, top-k + dispatch in another
    mark(CSK_STAGE_PREP);
    mark(CSK_STAGE_ROUTER);
    // the streaming kernels copy their token rows as FP6 terms, written once per token by the
    // prologue workgroups of this launch (not when the routing weight multiplies the rows first)
    u32x4* rows_mx3 = (!L->f16 && !L->wbf && stream_path(T, L->H, L->F, L->E, L->k)) ? reinterpret_cast<u32x4*>(ws.xs) : nullptr;
    rows_mx3_ready = rows_mx3 != nullptr;
    // a workgroup takes one expert (latency) as long as all of them are resident at once, four beyond
    if (cdiv(T, 4) * (L->E + 4) <= 4 * std::max(g_cus, 1) + 64)  // four of these workgroups fit a compute unit
      router_prep_logits_kernel<1><<<dim3((unsigned)(L->E + 4), (unsigned)cdiv(T, 4)), 256, 0, g_stream>>>(
          hidden, norm ? L->norm_w : nullptr, L->eps, ws.xn, L->gate_w,
          L->has_gate_b ? L->gate_b : nullptr, ws.logits, (int)T, (int)L->E, (int)L->H, rows_mx3);
    else
      router_prep_logits_kernel<4><<<dim3((unsigned)(cdiv(L->E, 4) + 4), (unsigned)cdiv(T, 4)), 256, 0, g_stream>>>(
          hidden, norm ? L->norm_w : nullptr, L->eps, ws.xn, L->gate_w,
          L->has_gate_b ? L->gate_b : nullptr, ws.logits, (int)T, (int)L->E, (int)L->H, rows_mx3);
    if ((rc = check_launch("router_prep_logits_kernel")) != CSK_OK) return rc;
    mark(CSK_STAGE_DISPATCH);
    RouteIn rin{ws.logits, xr, L->gate_w, L->has_gate_b ? L->gate_b : nullptr, L->ew_dev,
                (int)T, (int)L->E, (int)L->k, (int)L->H, L->sigmoid, stream_group_tokens(T)};
    RouteOut rout{ws.pairs, ws.ids, ws.pos, ws.counts, ws.offsets, ws.desc, ws.groups, ws.nv,
                  ws.tiles, ws.n_tiles, ws.list_tok, ws.list_w};
    if (T == 1 && phase == 0 && L->E > 1 && !L->f16 && stream_path(T, L->H, L->F, L->E, L->k)) {
      // one token: the gate/up kernel routes it itself (no launch here); phases keep the
      // routing kernel, whose output they hand out before the experts run
      route_in_kernel = true;
      rin_kept = rin, rout_kept = rout;
    } else if (T <= kRouteTinyTokens && P <= kRouteTinyMaxP && !L->f16 && stream_path(T, L->H, L->F, L->E, L->k)) {
      // a handful of tokens on the streaming kernels: each active expert is one token group
      route_tiny_kernel<<<dim3(1), 256, 0, g_stream>>>(rin, rout);
      if ((rc = check_launch("route_tiny_kernel")) != CSK_OK) return rc;
    } else if (T > kRouteSmallTokens) {
      // more tokens than the single workgroup has waves: selection spread over T / 4
      // workgroups, then the dispatch kernel -- a launch more, each much shorter
      router_topk_kernel<<<dim3((unsigned)cdiv(T, 4)), 256, 0, g_stream>>>(
          ws.logits, ws.pairs, ws.ids, (int)T, (int)L->E, (int)L->k, L->sigmoid, xr, L->gate_w,
          L->has_gate_b ? L->gate_b : nullptr, (int)L->H, ws.logits + T * L->E, 0, Mx3Rider{});
      if ((rc = check_launch("router_topk_kernel")) != CSK_OK) return rc;
      if ((rc = launch_dispatch(ws.ids, ws.pairs, P, L->k, L->E, L->ew_dev, ws)) != CSK_OK) return rc;
    } else {
      route_small_kernel<<<dim3(1), kRouteSmallThreads, 0, g_stream>>>(rin, rout);
      if ((rc = check_launch("route_small_kernel")) != CSK_OK) return rc;
    }
    if (!L->f16 && !stream_path(T, L->H, L->F, L->E, L->k) && !L->wbf) {
      // few tokens but rows too long for the streaming kernel: the GEMM wants the FP6 form
      if ((rc = launch_mx3(xr, ws.xs, T, L->H, nullptr, nullptr)) != CSK_OK) return rc;
    }
  } else {
    mark(CSK_STAGE_PREP);
    const bool stream = !L->f16 && stream_path(T, L->H, L->F, L->E, L->k);
    if (norm) {
      rc = launch_prep(hidden, L->norm_w, L->eps, ws.xn, T, L->H);
      if (rc != CSK_OK) return rc;
    }
    // the rows' FP6 form for the grouped GEMM is written by extra workgroups of the top-k launch
    const bool ride = !L->f16 && !L->wbf;  // (the streaming kernels copy the rows in this form, too)
    rows_mx3_ready = ride && stream;
    mark(CSK_STAGE_ROUTER);
    rc = launch_router(xr, L->gate_w, L->has_gate_b ? L->gate_b : nullptr, T, L->E, L->H, L->k,
                       L->sigmoid, ws.logits, ws.pairs, ws.ids, ride ? ws.xs : nullptr);
    if (rc != CSK_OK) return rc;
    mark(CSK_STAGE_DISPATCH);
    rc = launch_dispatch(ws.ids, ws.pairs, P, L->k, L->E, L->ew_dev, ws);
    if (rc != CSK_OK) return rc;
  }
  if (phase == 1) return CSK_OK;
  if (L->f16) {
    rc = run_experts_f16(L->E, T, L->k, L->H, L->F, L->act, xr, L->wbf != 0, P, ws, true);
    if (rc != CSK_OK) return rc;
    mark(CSK_STAGE_COMBINE);
    rc = launch_combine(ws.y, ws.pairs, ws.pos, (flags & CSK_FWD_RESIDUAL) ? hidden : nullptr, out,
                        T, L->k, L->H, L->wbf);
    mark(CSK_N_STAGES);
    g_stage_valid = g_timing;
    return rc;
  }
  // streaming path: the kernel gathers, scales and quantises the fp32 rows itself;
  // grouped GEMM: rows written as three FP6 terms beforehand (per token, or gathered and
  // pre-scaled per dispatch position when the routing weight goes in front of the FFN)
  ExpertInput in{xr, ws.list_tok, L->wbf ? ws.list_w : nullptr, ws.xs, ws.list_tok};
  if (route_in_kernel) in.rin = &rin_kept, in.rout = &rout_kept;
  if (rows_mx3_ready) in.x_mx3_tokens = ws.xs;
  if (L->wbf && !stream_path(T, L->H, L->F, L->E, L->k)) {
    if ((rc = launch_mx3(xr, ws.xg, P, L->H, ws.list_tok, ws.list_w)) != CSK_OK) return rc;
    in.x_mx3 = ws.xg;
    in.mx3_list_row = nullptr;
  }
  rc = run_experts(L->E, T, L->k, L->H, L->F, L->act, in, ws, true);
  if (rc != CSK_OK) return rc;
  mark(CSK_STAGE_COMBINE);
  rc = launch_combine(ws.y, ws.pairs, ws.pos, (flags & CSK_FWD_RESIDUAL) ? hidden : nullptr, out, T,
                      L->k, L->H, L->wbf);
  mark(CSK_N_STAGES);
  g_stage_valid = g_timing;
  return rc;
}

// sizes of the passes a batch of T tokens is processed in: n passes of `each` tokens (the last one shorter)
void pass_plan(int64_t T, int64_t& n, int64_t& each) {
  n = std::max<int64_t>(1, cdiv(T, g_pass_tokens));
  each = cdiv(T, n);
}
}  // namespace

extern "C" int csk_set_pass_tokens(int64_t tokens) {
  API_LOCK();
  if (tokens < 1 || tokens > 65536) return fail(CSK_ERR_ARG, "csk_set_pass_tokens: need 1 <= tokens <= 65536");
  g_pass_tokens = tokens;
  return CSK_OK;
}

extern "C" int csk_moe_forward(csk_layer* L, const float* hidden, int64_t T, float* out, int flags) {
  REQUIRE_INIT();
  if (!L || !hidden || !out || T < 0) return fail(CSK_ERR_ARG, "csk_moe_forward: bad argument");
  int rc = layer_ready(L, flags);
  if (rc != CSK_OK) return rc;
  L->last_T = T;
  if (T == 0) return CSK_OK;
  int64_t n, each;
  pass_plan(T, n, each);
  L->last_T = n == 1 ? T : -1;  // the dispatch lists of a batch taken in several passes are those of its last pass only
  for (int64_t t0 = 0; t0 < T; t0 += each) {
    rc = forward_pass(L, hidden + t0 * L->H, std::min(each, T - t0), out + t0 * L->H, flags);
    if (rc != CSK_OK) return rc;
  }
  return CSK_OK;
}

extern "C" int csk_moe_forward_noalloc(csk_layer* L, const float* hidden, int64_t T, float* out, int flags) {
  REQUIRE_INIT();
  if (!L || !hidden || !out || T < 0) return fail(CSK_ERR_ARG, "csk_moe_forward_noalloc: bad argument");
  int rc = layer_ready(L, flags);
  if (rc != CSK_OK) return rc;
  if (L->f16) return fail(CSK_ERR_ARG, "csk_moe_forward_noalloc: MXFP4 layers only");
  if (T > kFixedMaxT || T * L->k > kFixedMaxP || L->H > kFixedMaxDim || L->F > kFixedMaxDim)
    return fail(CSK_ERR_ARG, "csk_moe_forward_noalloc: at most " + std::to_string(kFixedMaxT) + " tokens, " +
                                 std::to_string(kFixedMaxP) + " token-expert assignments (T * top_k), hidden_dim and "
                                 "expert_ffn_dim up to " + std::to_string(kFixedMaxDim) + "; got T = " +
                                 std::to_string(T) + ", top_k = " + std::to_string(L->k) + ", H = " +
                                 std::to_string(L->H) + ", F = " + std::to_string(L->F));
  L->last_T = T;
  if (T == 0) return CSK_OK;
  // same kernels as csk_moe_forward, every buffer inside this GPU's load-time array
  return forward_pass(L, hidden, T, out, flags, g_ws_fixed);
}

extern "C" int csk_moe_forward_host(csk_layer* L, const float* hidden, int64_t T, float* out,
                                    float* pairs_out, int flags) {
  REQUIRE_INIT();
  if (!L || !hidden || !out || T < 0) return fail(CSK_ERR_ARG, "csk_moe_forward_host: bad argument");
  if (T == 0) return CSK_OK;
  // device copies of the caller's rows, from the pool of staging blocks (a frame of a decoding
  // engine comes back every few milliseconds and finds its blocks idle again: no allocation
  // in steady state, nothing held that the pool's bounds do not cover); the copies in, the
  // kernels and the copies out are queued on the stream and awaited once
  const size_t n = (size_t)T * L->H;
  DevBuf dbh, dbo;
  {
    int rc0 = dbh.alloc(n * sizeof(float));
    if (rc0 == CSK_OK) rc0 = dbo.alloc(n * sizeof(float));
    if (rc0 != CSK_OK) return rc0;
  }
  float* const dh = dbh.as<float>();
  float* const dout = dbo.as<float>();
  int rc = CSK_OK;
  {
    const void* src = hidden;
    if (void* stage = g_pinned.take(n * sizeof(float))) {
      std::memcpy(stage, hidden, n * sizeof(float));
      src = stage;
    }
    const hipError_t e = hipMemcpyAsync(dh, src, n * sizeof(float), hipMemcpyHostToDevice, g_stream);
    if (e != hipSuccess) rc = fail(CSK_ERR_HIP, std::string("copy in: ") + hipGetErrorString(e));
  }
  if (rc == CSK_OK && !pairs_out) rc = csk_moe_forward(L, dh, T, dout, flags);
  if (rc == CSK_OK && pairs_out) {
    // pass by pass, as csk_moe_forward does: the router output lives in the workspace of a pass
    rc = layer_ready(L, flags);
    int64_t np, each;
    pass_plan(T, np, each);
    L->last_T = np == 1 ? T : -1;
    for (int64_t t0 = 0; t0 < T && rc == CSK_OK; t0 += each) {
      const int64_t tn = std::min(each, T - t0);
      rc = forward_pass(L, dh + t0 * L->H, tn, dout + t0 * L->H, flags);
      if (rc == CSK_OK)
        rc = csk_copy_d2h(pairs_out + t0 * L->k * 2, g_ws.pairs, (size_t)tn * L->k * 2 * sizeof(float));
    }
  }
  if (rc == CSK_OK) rc = fetch(out, dout, n * sizeof(float));
  const int rs = finish_fetches();  // also when an earlier step failed: the stream is left idle
  return rc == CSK_OK ? rs : rc;
}

extern "C" int csk_moe_stack_forward(csk_layer* const* layers, int64_t n_layers, float* hidden,
                                     int64_t T) {
  REQUIRE_INIT();
  if (!layers || n_layers < 0 || !hidden) return fail(CSK_ERR_ARG, "csk_moe_stack_forward: bad argument");
  for (int64_t i = 0; i < n_layers; ++i) {
    int rc = csk_moe_forward(layers[i], hidden, T, hidden, CSK_FWD_RMSNORM | CSK_FWD_RESIDUAL);
    if (rc != CSK_OK) return rc;
  }
  return CSK_OK;
}

// ---------------------------------------------------------------- view layers and frames
// What the drop-in node classes share per MoE block: the expert nodes own the resident
// matrices, a view layer points at them, and a frame runs router, dispatch, every selected
// expert and the merge as the fused forward does -- begun by the router node, read back by
// the expert nodes (their rows) and the merge node (the merged rows).

extern "C" int csk_layer_create_view(int64_t E, int64_t k, int64_t H, int64_t F, csk_layer** out) {
  return layer_create(E, k, H, F, false, out, true);
}

extern "C" int csk_layer_attach_expert(csk_layer* L, int64_t e, const csk_mxfp4* up, const csk_mxfp4* gate,
                                       const csk_mxfp4* down, const float* b_up, const float* b_gate,
                                       const float* b_down) {
  REQUIRE_INIT();
  if (!L || !L->is_view) return fail(CSK_ERR_ARG, "csk_layer_attach_expert: not a view layer");
  if (e < 0 || e >= L->E || !up || !gate || !down) return fail(CSK_ERR_ARG, "csk_layer_attach_expert: bad argument");
  if (up->rows != L->F || up->K != L->H || gate->rows != L->F || gate->K != L->H || down->rows != L->H ||
      down->K != L->F)
    return fail(CSK_ERR_ARG, "csk_layer_attach_expert: matrix shapes do not match the layer");
  HIP_TRY(hipStreamSynchronize(g_stream));  // nothing in flight reads the entry that is about to change
  L->frame.live = false;
  ExpertW& w = L->ew_host[(size_t)e];
  w.q_gate = gate->q, w.s_gate = gate->s, w.q_up = up->q, w.s_up = up->s, w.q_down = down->q, w.s_down = down->s;
  int rc = upload_biases(L, e, b_up, b_gate, b_down);  // also publishes the entry
  if (rc != CSK_OK) return rc;
  L->attached[(size_t)e] = 1;
  L->expert_set[(size_t)e] = 1;
  return CSK_OK;
}

extern "C" int csk_layer_detach_expert(csk_layer* L, int64_t e) {
  REQUIRE_INIT();
  if (!L || !L->is_view || e < 0 || e >= L->E) return fail(CSK_ERR_ARG, "csk_layer_detach_expert: bad argument");
  HIP_TRY(hipStreamSynchronize(g_stream));  // a frame in flight may still be reading the matrices
  L->frame.live = false;
  L->attached[(size_t)e] = 0;
  L->expert_set[(size_t)e] = 0;
  L->ew_host[(size_t)e] = ExpertW{};
  HIP_TRY(hipMemcpy(L->ew_dev + e, &L->ew_host[(size_t)e], sizeof(ExpertW), hipMemcpyHostToDevice));
  return CSK_OK;
}

extern "C" int csk_moe_frame_begin(csk_layer* L, const float* hidden, int64_t T, float* pairs_out, int flags,
                                   int* experts_running) {
  REQUIRE_INIT();
  if (!L || !L->is_view || !hidden || !pairs_out || !experts_running || T <= 0)
    return fail(CSK_ERR_ARG, "csk_moe_frame_begin: bad argument");
  if (!L->has_gate) return fail(CSK_ERR_STATE, "router weights not set");
  if ((flags & CSK_FWD_RMSNORM) && !L->has_norm) return fail(CSK_ERR_STATE, "RMSNorm weight not set");
  if (T > g_pass_tokens) return fail(CSK_ERR_ARG, "csk_moe_frame_begin: a frame is one pass (at most " + std::to_string(g_pass_tokens) + " tokens)");
  csk_layer::Frame& f = L->frame;
  *experts_running = 0;
  f.live = false;
  const size_t n = (size_t)T * L->H;
  if (n > f.cap) {
    HIP_TRY(hipStreamSynchronize(g_stream));
    if (f.d_hidden) (void)hipFree(f.d_hidden);
    if (f.d_out) (void)hipFree(f.d_out);
    f.d_hidden = f.d_out = nullptr, f.cap = 0;
    HIP_TRY(counted_malloc((void**)&f.d_hidden, n * sizeof(float)));
    HIP_TRY(counted_malloc((void**)&f.d_out, n * sizeof(float)));
    f.cap = n;
  }
  Workspace& ws = *static_cast<Workspace*>(L->own_ws);
  {
    const void* src = hidden;
    if (void* stage = g_pinned.take(n * sizeof(float))) {
      std::memcpy(stage, hidden, n * sizeof(float));
      src = stage;
    }
    HIP_TRY(hipMemcpyAsync(f.d_hidden, src, n * sizeof(float), hipMemcpyHostToDevice, g_stream));
  }
  int rc = forward_pass(L, f.d_hidden, T, f.d_out, flags, ws, 1);
  const size_t np = (size_t)T * L->k;
  f.pairs.resize(np * 2);
  if (rc == CSK_OK) rc = fetch(f.pairs.data(), ws.pairs, np * 2 * sizeof(float));
  const int rs = finish_fetches();
  if (rc == CSK_OK) rc = rs;
  if (rc != CSK_OK) return rc;
  std::memcpy(pairs_out, f.pairs.data(), np * 2 * sizeof(float));
  L->last_T = T;
  f.T = T, f.flags = flags;
  f.live = true, f.experts_ran = false, f.rows_fetched = false, f.voided = false;
  // every expert the frame selects has to be attached: the expert kernels follow the
  // descriptors of the selected experts, and only of those
  for (size_t p = 0; p < np; ++p) {
    const int e = (int)f.pairs[2 * p];
    if (e < 0 || e >= L->E || !L->attached[(size_t)e]) return CSK_OK;
  }
  rc = forward_pass(L, f.d_hidden, T, f.d_out, flags, ws, 2);
  if (rc != CSK_OK) {
    f.live = false;
    return rc;
  }
  f.experts_ran = true;
  *experts_running = 1;
  return CSK_OK;
}

extern "C" int csk_moe_frame_expert_rows(csk_layer* L, int64_t e, float* out) {
  REQUIRE_INIT();
  if (!L || !L->is_view || !out || e < 0 || e >= L->E) return fail(CSK_ERR_ARG, "csk_moe_frame_expert_rows: bad argument");
  csk_layer::Frame& f = L->frame;
  if (!f.live || !f.experts_ran) return fail(CSK_ERR_STATE, "csk_moe_frame_expert_rows: no frame with running experts");
  const size_t np = (size_t)f.T * L->k, H = (size_t)L->H;
  if (!f.rows_fetched) {
    Workspace& ws = *static_cast<Workspace*>(L->own_ws);
    f.y.resize(np * H);
    f.pos.resize(np);
    HIP_TRY(hipMemcpyAsync(f.y.data(), ws.y, np * H * sizeof(float), hipMemcpyDeviceToHost, g_stream));
    HIP_TRY(hipMemcpyAsync(f.pos.data(), ws.pos, np * sizeof(int), hipMemcpyDeviceToHost, g_stream));
    HIP_TRY(hipStreamSynchronize(g_stream));
    f.rows_fetched = true;
  }
  // row t = the expert's output for token t if t selected it (first matching slot, as
  // expert_mlp_node.h:503-529), else the zeros the caller's tensor already holds
  for (int64_t t = 0; t < f.T; ++t)
    for (int64_t s2 = 0; s2 < L->k; ++s2) {
      const size_t p = (size_t)t * L->k + s2;
      if ((int64_t)(int)f.pairs[2 * p] == e) {
        std::memcpy(out + (size_t)t * H, f.y.data() + (size_t)f.pos[p] * H, H * sizeof(float));
        break;
      }
    }
  return CSK_OK;
}

extern "C" int csk_moe_frame_void(csk_layer* L) {
  API_LOCK();
  if (!L || !L->is_view) return fail(CSK_ERR_ARG, "csk_moe_frame_void: not a view layer");
  L->frame.voided = true;
  return CSK_OK;
}

extern "C" int csk_moe_frame_merged(csk_layer* L, float* out, int* available) {
  REQUIRE_INIT();
  if (!L || !L->is_view || !out || !available) return fail(CSK_ERR_ARG, "csk_moe_frame_merged: bad argument");
  csk_layer::Frame& f = L->frame;
  *available = 0;
  if (!f.live || !f.experts_ran || f.voided) return CSK_OK;
  CSK_TRY(fetch(out, f.d_out, (size_t)f.T * L->H * sizeof(float)));
  CSK_TRY(finish_fetches());
  *available = 1;
  return CSK_OK;
}

extern "C" int csk_layer_last_dispatch(csk_layer* L, int32_t* counts_host, int32_t* tokens_host) {
  REQUIRE_INIT();
  if (!L) return fail(CSK_ERR_ARG, "null layer");
  if (L->last_T < 0)
    return fail(CSK_ERR_STATE, "the last forward took its batch in several passes: there is no single dispatch to report");
  if (L->last_T == 0 || !L->last_ws) return fail(CSK_ERR_STATE, "no forward has run on this layer");
  // the lists live in the workspace the forward ran in, which the next forward -- of any layer -- overwrites
  const Workspace* ws = static_cast<const Workspace*>(L->last_ws);
  if (ws->runs != L->last_run)
    return fail(CSK_ERR_STATE, "another forward has run since this layer's last one: its dispatch lists are gone");
  if (counts_host) {
    int rc = csk_copy_d2h(counts_host, ws->counts, (size_t)L->E * sizeof(int));
    if (rc != CSK_OK) return rc;
  }
  if (tokens_host) return csk_copy_d2h(tokens_host, ws->list_tok, (size_t)L->last_T * L->k * sizeof(int));
  return CSK_OK;
}

// ============================================================ node-level ops


namespace {
int router_host(const float* hidden, int64_t T, int64_t H, const float* gate_w, int64_t E,
                const float* gate_b, int64_t k, int sigmoid, float* out_pairs, float* out_logits,
                bool gate_on_device = false);
}

extern "C" int csk_moe_router(const float* hidden, int64_t T, int64_t H, const float* gate_w,
                              int64_t E, const float* gate_b, int64_t k, int sigmoid,
                              float* out_pairs) {
  REQUIRE_INIT();
  if (!out_pairs) return fail(CSK_ERR_ARG, "csk_moe_router: null argument");
  return router_host(hidden, T, H, gate_w, E, gate_b, k, sigmoid, out_pairs, nullptr);
}

extern "C" int csk_moe_router_resident(const float* hidden, int64_t T, int64_t H, const float* gate_w_dev,
                                       int64_t E, const float* gate_b_dev, int64_t k, int sigmoid,
                                       float* out_pairs) {
  REQUIRE_INIT();
  if (!out_pairs) return fail(CSK_ERR_ARG, "csk_moe_router: null argument");
  return router_host(hidden, T, H, gate_w_dev, E, gate_b_dev, k, sigmoid, out_pairs, nullptr, /*gate_on_device=*/true);
}

extern "C" int csk_moe_router_logits(const float* hidden, int64_t T, int64_t H, const float* gate_w,
                                     int64_t E, const float* gate_b, float* out_logits) {
  REQUIRE_INIT();
  if (!out_logits) return fail(CSK_ERR_ARG, "csk_moe_router_logits: null argument");
  return router_host(hidden, T, H, gate_w, E, gate_b, 1, 0, nullptr, out_logits);
}

namespace {
int router_host(const float* hidden, int64_t T, int64_t H, const float* gate_w, int64_t E,
                const float* gate_b, int64_t k, int sigmoid, float* out_pairs, float* out_logits,
                bool gate_on_device) {
  if (!hidden || !gate_w || T < 0) return fail(CSK_ERR_ARG, "csk_moe_router: null argument");
  if (E <= 0 || E > kMaxExperts || k <= 0 || k > kMaxTopK || k > E || H <= 0 || H % 4)
    return fail(CSK_ERR_ARG, "csk_moe_router: need 1 <= top_k <= min(16, E), E <= 256, H a multiple of 4");
  if (T == 0) return CSK_OK;
  DevBuf dx, dg, db, dl, dp, di;
  int rc;
  const float *gw = gate_w, *gb = gate_b;  // device addresses of the gate
  if (!gate_on_device) {
    if ((rc = dg.upload(gate_w, (size_t)E * H * 4)) != CSK_OK) return rc;
    if (gate_b && (rc = db.upload(gate_b, (size_t)E * 4)) != CSK_OK) return rc;
    gw = dg.as<float>(), gb = gate_b ? db.as<float>() : nullptr;
  }
  return for_token_passes(T, [&](int64_t t0, int64_t tn) -> int {
    int rc;
    if ((rc = dx.upload(hidden + t0 * H, (size_t)tn * H * 4)) != CSK_OK) return rc;
    if ((rc = dl.alloc((size_t)tn * E * 4 * (1 + kRouterMaxSplits))) != CSK_OK) return rc;
    if ((rc = dp.alloc((size_t)tn * k * 8)) != CSK_OK) return rc;
    if ((rc = di.alloc((size_t)tn * k * 4)) != CSK_OK) return rc;
    rc = launch_router(dx.as<float>(), gw, gb, tn, E, H, k, sigmoid, dl.as<float>(), dp.as<float>(), di.as<int>());
    if (rc != CSK_OK) return rc;
    if (out_pairs)
      CSK_TRY(fetch(out_pairs + t0 * k * 2, dp.p, (size_t)tn * k * 8));
    if (out_logits)
      CSK_TRY(fetch(out_logits + t0 * E, dl.p, (size_t)tn * E * 4));
    CSK_TRY(finish_fetches());
    return CSK_OK;
  });
}
}  // namespace

namespace {
__global__ void select_expert_ids_kernel(const float* __restrict__ pairs, int* __restrict__ ids,
                                         int P, int expert_id, int* __restrict__ list_tok,
                                         float* __restrict__ list_w) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  ids[p] = ((int)pairs[2 * (size_t)p] == expert_id) ? 0 : -1;
  // positions of the lists that the dispatch leaves unwritten read as token 0, weight 0
  list_tok[p] = 0;
  list_w[p] = 0.0f;
}
}  // namespace

extern "C" int csk_expert_mlp_mxfp4(int expert_id, const float* hidden, int64_t T, int64_t H,
                                    int64_t F, const csk_mxfp4* w_up, const csk_mxfp4* w_gate,
                                    const csk_mxfp4* w_down, const float* b_up,
                                    const float* b_gate, const float* b_down, const float* pairs,
                                    int64_t k, int activation, int weight_before_ffn, float* out,
                                    int* is_empty) {
  REQUIRE_INIT();
  if (!hidden || !w_up || !w_gate || !w_down || !pairs || !out || !is_empty || T < 0)
    return fail(CSK_ERR_ARG, "csk_expert_mlp_mxfp4: null argument");
  // router scan happens before the shape checks (expert_mlp_node.h:441-443)
  bool any = false;
  for (int64_t p = 0; p < T * k && !any; ++p) any = (int)pairs[2 * p] == expert_id;
  *is_empty = !any;
  if (!any) return CSK_OK;
  if (w_up->rows != F || w_up->K != H || w_gate->rows != F || w_gate->K != H || w_down->rows != H ||
      w_down->K != F)
    return fail(CSK_ERR_ARG, "expert_mlp: weight dimension mismatch");
  if (H % 32) return fail(CSK_ERR_ARG, "expert_mlp: hidden_dim must be a multiple of 32 for MXFP4, got " + std::to_string(H));
  if (F % 32) return fail(CSK_ERR_ARG, "expert_mlp: expert_ffn_dim must be a multiple of 32 for MXFP4, got " + std::to_string(F));
  if (k <= 0 || k > kMaxTopK) return fail(CSK_ERR_ARG, "expert_mlp: top_k must be in 1..16");
  if (H > (int64_t)kZeroLen || F > (int64_t)kZeroLen) return fail(CSK_ERR_ARG, "expert_mlp: dimensions above 65536 are not supported");
  const int nb = (b_up != nullptr) + (b_gate != nullptr) + (b_down != nullptr);
  if (nb != 0 && nb != 3) return fail(CSK_ERR_ARG, "expert_mlp: biases must be all present or all absent");
  Workspace& ws = g_ws;
  ExpertW w{};
  w.q_gate = w_gate->q, w.s_gate = w_gate->s, w.q_up = w_up->q, w.s_up = w_up->s;
  w.q_down = w_down->q, w.s_down = w_down->s;
  // a pass in which no token selects the expert still writes its rows (zeros, :509-512)
  return for_token_passes(T, [&](int64_t t0, int64_t tn) -> int {
    int rc = ws.ensure(tn, 1, k, H, F, weight_before_ffn != 0);
    if (rc != CSK_OK) return rc;
    const int64_t P = tn * k;
    ExpertCallInputs up;
    CSK_TRY(up.send(w, nb == 3, b_up, b_gate, b_down, F, H, pairs + t0 * k * 2, P, hidden + t0 * H, tn * H));
    DevBuf dout;
    if ((rc = dout.alloc((size_t)tn * H * 4)) != CSK_OK) return rc;
    select_expert_ids_kernel<<<dim3((unsigned)cdiv(P, 256)), 256, 0, g_stream>>>(
        up.pairs, ws.ids, (int)P, expert_id, ws.list_tok, ws.list_w);
    if ((rc = check_launch("select_expert_ids_kernel")) != CSK_OK) return rc;
    if ((rc = launch_dispatch(ws.ids, up.pairs, P, k, 1, up.ew, ws)) != CSK_OK) return rc;
    ExpertInput in{up.x, ws.list_tok, weight_before_ffn ? ws.list_w : nullptr, ws.xs, ws.list_tok};
    if (!stream_path(tn, H, F, 1, k)) {
      if (weight_before_ffn) {
        // The expert's token count is only known on the device, and at most tn
        // tokens can select it: gather tn rows.  Positions past the count read the
        // zeroed tail of the lists (token 0, weight 0) and are never consumed.
        rc = launch_mx3(up.x, ws.xg, tn, H, ws.list_tok, ws.list_w);
        in.x_mx3 = ws.xg;
        in.mx3_list_row = nullptr;
      } else {
        rc = launch_mx3(up.x, ws.xs, tn, H, nullptr, nullptr);
      }
      if (rc != CSK_OK) return rc;
    }
    rc = run_experts(1, tn, k, H, F, activation, in, ws);
    if (rc != CSK_OK) return rc;
    expand_expert_rows_kernel<<<dim3((unsigned)cdiv(H, 256), (unsigned)tn), 256, 0, g_stream>>>(
        ws.y, ws.ids, ws.pos, dout.as<float>(), (int)k, (int)H, 0);
    if ((rc = check_launch("expand_expert_rows_kernel")) != CSK_OK) return rc;
    CSK_TRY(fetch(out + t0 * H, dout.p, (size_t)tn * H * 4));
    CSK_TRY(finish_fetches());
    return CSK_OK;
  });
}

extern "C" int csk_expert_mlp_f16(int expert_id, const float* hidden, int64_t T, int64_t H, int64_t F,
                                  const csk_f16* w_up, const csk_f16* w_gate, const csk_f16* w_down,
                                  const float* b_up, const float* b_gate, const float* b_down,
                                  const float* pairs, int64_t k, int activation,
                                  int weight_before_ffn, float* out, int* is_empty) {
  REQUIRE_INIT();
  if (!hidden || !w_up || !w_gate || !w_down || !pairs || !out || !is_empty || T < 0)
    return fail(CSK_ERR_ARG, "csk_expert_mlp_f16: null argument");
  // the router scan comes before the shape checks (expert_mlp_node.h:297-306)
  bool any = false;
  for (int64_t p = 0; p < T * k && !any; ++p) any = (int)pairs[2 * p] == expert_id;
  *is_empty = !any;
  if (!any) return CSK_OK;
  if (w_up->split() || w_gate->split() || w_down->split())
    return fail(CSK_ERR_ARG, "expert_mlp: all weights must be FLOAT16");
  if (w_up->rows != F || w_up->K != H)
    return fail(CSK_ERR_ARG, "expert_mlp: w_up must be [" + std::to_string(F) + ", " + std::to_string(H) + "], got [" +
                                 std::to_string(w_up->rows) + ", " + std::to_string(w_up->K) + "]");
  if (w_gate->rows != F || w_gate->K != H)
    return fail(CSK_ERR_ARG, "expert_mlp: w_gate must be [" + std::to_string(F) + ", " + std::to_string(H) + "], got [" +
                                 std::to_string(w_gate->rows) + ", " + std::to_string(w_gate->K) + "]");
  if (w_down->rows != H || w_down->K != F)
    return fail(CSK_ERR_ARG, "expert_mlp: w_down must be [" + std::to_string(H) + ", " + std::to_string(F) + "], got [" +
                                 std::to_string(w_down->rows) + ", " + std::to_string(w_down->K) + "]");
  if (k <= 0 || k > kMaxTopK) return fail(CSK_ERR_ARG, "expert_mlp: top_k must be in 1..16");
  const int nb = (b_up != nullptr) + (b_gate != nullptr) + (b_down != nullptr);
  if (nb != 0 && nb != 3) return fail(CSK_ERR_ARG, "expert_mlp: biases must be all present or all absent");
  Workspace& ws = g_ws;
  const int64_t Hp = cdiv(H, 32) * 32, Fp = cdiv(F, 32) * 32;  // activation rows are whole blocks
  ExpertW w{};
  w.q_gate = reinterpret_cast<const uint4*>(w_gate->w);
  w.q_up = reinterpret_cast<const uint4*>(w_up->w);
  w.q_down = reinterpret_cast<const uint4*>(w_down->w);
  return for_token_passes(T, [&](int64_t t0, int64_t tn) -> int {
    int rc = ws.ensure(tn, 1, k, Hp, Fp, weight_before_ffn != 0);
    if (rc != CSK_OK) return rc;
    const int64_t P = tn * k;
    ExpertCallInputs up;
    CSK_TRY(up.send(w, nb == 3, b_up, b_gate, b_down, F, H, pairs + t0 * k * 2, P, hidden + t0 * H, tn * H));
    DevBuf dout;
    if ((rc = dout.alloc((size_t)tn * H * 4)) != CSK_OK) return rc;
    select_expert_ids_kernel<<<dim3((unsigned)cdiv(P, 256)), 256, 0, g_stream>>>(
        up.pairs, ws.ids, (int)P, expert_id, ws.list_tok, ws.list_w);
    if ((rc = check_launch("select_expert_ids_kernel")) != CSK_OK) return rc;
    if ((rc = launch_dispatch(ws.ids, up.pairs, P, k, 1, up.ew, ws)) != CSK_OK) return rc;
    // with weight_before_ffn at most tn tokens can select the expert: tn rows are gathered; the
    // ones past its count read the zeroed tail of the lists and are never consumed
    rc = run_experts_f16(1, tn, k, H, F, activation, up.x, weight_before_ffn != 0, tn, ws);
    if (rc != CSK_OK) return rc;
    expand_expert_rows_kernel<<<dim3((unsigned)cdiv(H, 256), (unsigned)tn), 256, 0, g_stream>>>(
        ws.y, ws.ids, ws.pos, dout.as<float>(), (int)k, (int)H, 0);
    if ((rc = check_launch("expand_expert_rows_kernel")) != CSK_OK) return rc;
    CSK_TRY(fetch(out + t0 * H, dout.p, (size_t)tn * H * 4));
    CSK_TRY(finish_fetches());
    return CSK_OK;
  });
}

namespace {
// One work descriptor holding every token (position p = token p) and its 64-token tiles.
__global__ void dense_desc_kernel(WorkDesc* desc, const ExpertW* ew, int T, int* mtiles, int* n_mtiles) {
  if (threadIdx.x == 0) {
    write_work_desc(desc, true, 0, T, 0, ew);
    *n_mtiles = (T + 63) / 64;
  }
  for (int i = threadIdx.x; i < (T + 63) / 64; i += blockDim.x) {
    mtiles[2 * i] = 0;
    mtiles[2 * i + 1] = 64 * i;
  }
}
}  // namespace

extern "C" int csk_dense_ffn_f16(const float* hidden, int64_t T, int64_t H, int64_t F,
                                 const csk_f16* w_gate, const csk_f16* w_up, const csk_f16* w_down,
                                 const float* b_gate, const float* b_up, const float* b_down,
                                 float* out) {
  REQUIRE_INIT();
  if (!hidden || !w_gate || !w_up || !w_down || !out || T < 0)
    return fail(CSK_ERR_ARG, "csk_dense_ffn_f16: null argument");
  if (w_gate->split() != w_up->split() || w_gate->split() != w_down->split())
    return fail(CSK_ERR_ARG, "dense_ffn: weight tensors must all be FLOAT16 or all FLOAT32");
  if (w_gate->rows != F || w_gate->Ksrc != H || w_up->rows != F || w_up->Ksrc != H)
    return fail(CSK_ERR_ARG, "dense_ffn: gate_w/up_w shape mismatch");
  if (w_down->rows != H || w_down->Ksrc != F)
    return fail(CSK_ERR_ARG, "dense_ffn: down_w shape mismatch, expected [" + std::to_string(H) + ", " +
                                 std::to_string(F) + "], got [" + std::to_string(w_down->rows) + ", " +
                                 std::to_string(w_down->Ksrc) + "]");
  if (T == 0) return CSK_OK;
  const bool dup = w_gate->split();  // fp32 weights as two fp16 terms: rows are contracted twice over
  Workspace& ws = g_ws;
  DevBuf dx, dbg, dbu, dbd, dew;
  int rc;
  // each bias is optional on its own (dense_ffn_node.h:196-197, 213)
  if (b_gate && (rc = dbg.upload(b_gate, (size_t)F * 4)) != CSK_OK) return rc;
  if (b_up && (rc = dbu.upload(b_up, (size_t)F * 4)) != CSK_OK) return rc;
  if (b_down && (rc = dbd.upload(b_down, (size_t)H * 4)) != CSK_OK) return rc;
  ExpertW w{};
  w.q_gate = reinterpret_cast<const uint4*>(w_gate->w);
  w.q_up = reinterpret_cast<const uint4*>(w_up->w);
  w.q_down = reinterpret_cast<const uint4*>(w_down->w);
  w.b_gate = b_gate ? dbg.as<float>() : g_zero;
  w.b_up = b_up ? dbu.as<float>() : g_zero;
  w.b_down = b_down ? dbd.as<float>() : g_zero;
  if ((rc = dew.upload(&w, sizeof w)) != CSK_OK) return rc;
  return for_token_passes(T, [&](int64_t t0, int64_t tn) -> int {
    int rc = ws.ensure(tn, 1, 1, cdiv(dup ? 2 * H : H, 32) * 32, cdiv(dup ? 2 * F : F, 32) * 32, false);
    if (rc != CSK_OK) return rc;
    if ((rc = dx.upload(hidden + t0 * H, (size_t)tn * H * 4)) != CSK_OK) return rc;
    dense_desc_kernel<<<1, 256, 0, g_stream>>>(ws.desc, dew.as<ExpertW>(), (int)tn, ws.tiles, ws.n_tiles);
    if ((rc = check_launch("dense_desc_kernel")) != CSK_OK) return rc;
    const float wscales[3] = {w_gate->wscale, w_up->wscale, w_down->wscale};
    rc = run_experts_f16(1, tn, 1, H, F, CSK_ACT_STANDARD_SWIGLU, dx.as<float>(), false, tn, ws, false, true, dup, wscales);
    if (rc != CSK_OK) return rc;
    CSK_TRY(fetch(out + t0 * H, ws.y, (size_t)tn * H * 4));
    CSK_TRY(finish_fetches());
    return CSK_OK;
  });
}

extern "C" int csk_matmul_transpose_f16(const float* a_host, int64_t M, int64_t K, const csk_f16* w,
                                       float* out) {
  REQUIRE_INIT();
  if (!a_host || !w || !out || M < 0 || K <= 0)
    return fail(CSK_ERR_ARG, "csk_matmul_transpose_f16: null argument");
  if (w->Ksrc != K) return fail(CSK_ERR_ARG, "matmul_transpose_mixed: incompatible dimensions");
  if (M == 0) return CSK_OK;
  const int64_t N = w->rows, K2 = w->K;  // K2 = 2 K for an fp32 weight kept as two fp16 terms
  Workspace& ws = g_ws;
  DevBuf da, dew;
  int rc;
  ExpertW ew{};
  ew.q_down = reinterpret_cast<const uint4*>(w->w);
  ew.b_gate = ew.b_up = ew.b_down = g_zero;
  if ((rc = dew.upload(&ew, sizeof ew)) != CSK_OK) return rc;
  return for_token_passes(M, [&](int64_t m0, int64_t mn) -> int {
    // rows of A take the place of the activations of a down projection: [mn, K] -> [mn, N]
    int rc = ws.ensure(mn, 1, 1, cdiv(N, 32) * 32, cdiv(K2, 32) * 32, false);
    if (rc == CSK_OK) rc = g_f16.ensure((size_t)mn, 1);
    if (rc != CSK_OK) return rc;
    if ((rc = da.upload(a_host + m0 * K, (size_t)mn * K * 4)) != CSK_OK) return rc;
    dense_desc_kernel<<<1, 256, 0, g_stream>>>(ws.desc, dew.as<ExpertW>(), (int)mn, ws.tiles, ws.n_tiles);
    if ((rc = check_launch("dense_desc_kernel")) != CSK_OK) return rc;
    if ((rc = launch_f16_split(da.as<float>(), mn, K2, nullptr, nullptr, ws.act, g_f16.rs_a, K)) != CSK_OK) return rc;
    rc = launch_f16_projection(1, mn, mn, K2, N, ws.act, g_f16.rs_a, ws.y, ws, w->wscale);
    if (rc != CSK_OK) return rc;
    CSK_TRY(fetch(out + m0 * N, ws.y, (size_t)mn * N * 4));
    CSK_TRY(finish_fetches());
    return CSK_OK;
  });
}

extern "C" int csk_expert_token_mxfp4(const float* x, const uint8_t* w_up, const uint8_t* w_gate,
                                      const uint8_t* w_down, const float* b_up,
                                      const float* b_gate, const float* b_down, float* out,
                                      int64_t H, int64_t F, int activation) {
  REQUIRE_INIT();
  if (!x || !w_up || !w_gate || !w_down || !out) return fail(CSK_ERR_ARG, "csk_expert_token_mxfp4: null argument");
  if (H <= 0 || F <= 0 || H % 32 || F % 32)
    return fail(CSK_ERR_ARG, "compute_token_mxfp4: hidden_dim and expert_ffn_dim must be multiples of 32");
  csk_mxfp4 *mu = nullptr, *mg = nullptr, *md = nullptr;
  int rc = csk_mxfp4_upload(w_up, F, H, &mu);
  if (rc == CSK_OK) rc = csk_mxfp4_upload(w_gate, F, H, &mg);
  if (rc == CSK_OK) rc = csk_mxfp4_upload(w_down, H, F, &md);
  if (rc == CSK_OK) {
    const float pairs[2] = {0.0f, 1.0f};
    int empty = 0;
    rc = csk_expert_mlp_mxfp4(0, x, 1, H, F, mu, mg, md, b_up, b_gate, b_down, pairs, 1, activation,
                              0, out, &empty);
  }
  csk_mxfp4_free(mu);
  csk_mxfp4_free(mg);
  csk_mxfp4_free(md);
  return rc;
}

extern "C" int csk_expert_merge(const float* pairs, int64_t T, int64_t k, int64_t E, int64_t H,
                                const float* const* expert_outs, int pre_weighted, float* out) {
  REQUIRE_INIT();
  if (!pairs || !expert_outs || !out || T < 0 || k <= 0 || E <= 0 || H <= 0)
    return fail(CSK_ERR_ARG, "csk_expert_merge: bad argument");
  bool any = false;
  for (int64_t e = 0; e < E; ++e) any |= expert_outs[e] != nullptr;
  if (!any) return fail(CSK_ERR_ALL_EMPTY, "expert_merge: no non-empty expert outputs found");
  if (T == 0) return CSK_OK;
  const int64_t P = T * k;
  // Gather the k rows each token needs; an empty expert contributes nothing.
  std::vector<float> rows((size_t)P * H, 0.0f);
  std::vector<int> pos((size_t)P);
  for (int64_t p = 0; p < P; ++p) {
    const int e = (int)pairs[2 * p];
    if (e < 0 || e >= E) return fail(CSK_ERR_RANGE, "expert_merge: expert_idx out of range: " + std::to_string(e));
    const float* src = expert_outs[e];
    pos[(size_t)p] = src ? (int)p : -1;
    if (src) std::memcpy(&rows[(size_t)p * H], src + (p / k) * H, (size_t)H * sizeof(float));
  }
  DevBuf dy, dpairs, dpos, dout;
  int rc;
  if ((rc = dy.upload(rows.data(), rows.size() * 4)) != CSK_OK) return rc;
  if ((rc = dpairs.upload(pairs, (size_t)P * 8)) != CSK_OK) return rc;
  if ((rc = dpos.upload(pos.data(), pos.size() * 4)) != CSK_OK) return rc;
  if ((rc = dout.alloc((size_t)T * H * 4)) != CSK_OK) return rc;
  rc = launch_combine(dy.as<float>(), dpairs.as<float>(), dpos.as<int>(), nullptr, dout.as<float>(),
                      T, k, H, pre_weighted);
  if (rc != CSK_OK) return rc;
  CSK_TRY(fetch(out, dout.p, (size_t)T * H * 4));
  CSK_TRY(finish_fetches());
  return CSK_OK;
}

namespace {
__global__ void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                           float* __restrict__ o, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) o[i] = a[i] + b[i];
}
}  // namespace

extern "C" int csk_rmsnorm(const float* x, const float* weight, float* out, int64_t T, int64_t H,
                           float eps) {
  REQUIRE_INIT();
  if (!x || !weight || !out || T < 0 || H <= 0) return fail(CSK_ERR_ARG, "csk_rmsnorm: bad argument");
  if (T == 0) return CSK_OK;
  DevBuf dx, dw, dout;
  int rc;
  if ((rc = dx.upload(x, (size_t)T * H * 4)) != CSK_OK) return rc;
  if ((rc = dw.upload(weight, (size_t)H * 4)) != CSK_OK) return rc;
  if ((rc = dout.alloc((size_t)T * H * 4)) != CSK_OK) return rc;
  rc = launch_prep(dx.as<float>(), dw.as<float>(), eps, dout.as<float>(), T, H);
  if (rc != CSK_OK) return rc;
  CSK_TRY(fetch(out, dout.p, (size_t)T * H * 4));
  CSK_TRY(finish_fetches());
  return CSK_OK;
}

extern "C" int csk_rmsnorm_f64(const double* x, const double* weight, double* out, int64_t T, int64_t H,
                               float eps) {
  REQUIRE_INIT();
  if (!x || !weight || !out || T < 0 || H <= 0) return fail(CSK_ERR_ARG, "csk_rmsnorm_f64: bad argument");
  if (T == 0) return CSK_OK;
  DevBuf dx, dw, dout;
  int rc;
  if ((rc = dx.upload(x, (size_t)T * H * 8)) != CSK_OK) return rc;
  if ((rc = dw.upload(weight, (size_t)H * 8)) != CSK_OK) return rc;
  if ((rc = dout.alloc((size_t)T * H * 8)) != CSK_OK) return rc;
  rmsnorm_f64_kernel<<<dim3((unsigned)cdiv(T, 8)), 512, 0, g_stream>>>(dx.as<double>(), dw.as<double>(),
                                                                       dout.as<double>(), (long)T, (long)H, eps);
  if ((rc = check_launch("rmsnorm_f64_kernel")) != CSK_OK) return rc;
  CSK_TRY(fetch(out, dout.p, (size_t)T * H * 8));
  CSK_TRY(finish_fetches());
  return CSK_OK;
}

extern "C" int csk_add(const float* a, const float* b, float* out, int64_t n) {
  REQUIRE_INIT();
  if (!a || !b || !out || n < 0) return fail(CSK_ERR_ARG, "csk_add: bad argument");
  if (n == 0) return CSK_OK;
  DevBuf da, db, dout;
  int rc;
  if ((rc = da.upload(a, (size_t)n * 4)) != CSK_OK) return rc;
  if ((rc = db.upload(b, (size_t)n * 4)) != CSK_OK) return rc;
  if ((rc = dout.alloc((size_t)n * 4)) != CSK_OK) return rc;
  add_kernel<<<dim3((unsigned)cdiv(n, 256)), 256, 0, g_stream>>>(da.as<float>(), db.as<float>(), dout.as<float>(), n);
  if ((rc = check_launch("add_kernel")) != CSK_OK) return rc;
  CSK_TRY(fetch(out, dout.p, (size_t)n * 4));
  CSK_TRY(finish_fetches());
  return CSK_OK;
}

extern "C" int csk_add_broadcast(const void* a, const int64_t* shape_a, int nd_a, const void* b,
                                 const int64_t* shape_b, int nd_b, int dtype, void* out) {
  REQUIRE_INIT();
  if (!a || !b || !out || nd_a < 0 || nd_b < 0 || (nd_a && !shape_a) || (nd_b && !shape_b))
    return fail(CSK_ERR_ARG, "csk_add_broadcast: bad argument");
  if (dtype < CSK_DT_FLOAT32 || dtype > CSK_DT_INT64) return fail(CSK_ERR_ARG, "add: unsupported dtype");
  const int nd = std::max(nd_a, nd_b);
  auto list = [](const int64_t* s, int n) {
    std::string r;
    for (int i = 0; i < n; ++i) r += (i ? "," : "") + std::to_string(s[i]);
    return r;
  };
  if (nd > kMaxBroadcastDims)
    return fail(CSK_ERR_ARG, "add: more than " + std::to_string(kMaxBroadcastDims) + " dimensions are not supported");
  for (int i = 0; i < nd_a; ++i)
    if (shape_a[i] < 0) return fail(CSK_ERR_ARG, "csk_add_broadcast: negative dimension");
  for (int i = 0; i < nd_b; ++i)
    if (shape_b[i] < 0) return fail(CSK_ERR_ARG, "csk_add_broadcast: negative dimension");
  // dynamic_tensor::broadcast_shape (dynamic_tensor.h:218-238), trailing dimensions aligned
  BroadcastDims d{};
  d.nd = nd;
  int64_t n = 1, na = 1, nb = 1;
  for (int i = 0; i < nd; ++i) {
    const int64_t da = i < nd_a ? shape_a[nd_a - 1 - i] : 1, db = i < nd_b ? shape_b[nd_b - 1 - i] : 1;
    if (!(da == db || da == 1 || db == 1))
      return fail(CSK_ERR_ARG, "Broadcast failed: Shape A=[" + list(shape_a, nd_a) + "], Shape B=[" +
                                   list(shape_b, nd_b) + "]");
    const int q = nd - 1 - i;
    d.out[q] = (da == 0 || db == 0) ? 0 : std::max(da, db);
    d.sa[q] = (i < nd_a && da != 1) ? na : 0;
    d.sb[q] = (i < nd_b && db != 1) ? nb : 0;
    if (__builtin_mul_overflow(n, d.out[q], &n) || __builtin_mul_overflow(na, da, &na) ||
        __builtin_mul_overflow(nb, db, &nb))
      return fail(CSK_ERR_ARG, "csk_add_broadcast: element count overflows");
  }
  if (n == 0) return CSK_OK;
  const size_t esz = (dtype == CSK_DT_FLOAT32 || dtype == CSK_DT_INT32) ? 4 : 8;
  DevBuf da_, db_, dout;
  int rc;
  if ((rc = da_.upload(a, (size_t)na * esz)) != CSK_OK) return rc;
  if ((rc = db_.upload(b, (size_t)nb * esz)) != CSK_OK) return rc;
  if ((rc = dout.alloc((size_t)n * esz)) != CSK_OK) return rc;
  const dim3 grid((unsigned)std::min<int64_t>(cdiv(n, 256), 1 << 20));
  switch (dtype) {
    case CSK_DT_FLOAT32:
      add_broadcast_kernel<float><<<grid, 256, 0, g_stream>>>(da_.as<float>(), db_.as<float>(), dout.as<float>(), n, d);
      break;
    case CSK_DT_FLOAT64:
      add_broadcast_kernel<double><<<grid, 256, 0, g_stream>>>(da_.as<double>(), db_.as<double>(), dout.as<double>(), n, d);
      break;
    case CSK_DT_INT32:
      add_broadcast_kernel<int32_t><<<grid, 256, 0, g_stream>>>(da_.as<int32_t>(), db_.as<int32_t>(), dout.as<int32_t>(), n, d);
      break;
    default:
      add_broadcast_kernel<int64_t><<<grid, 256, 0, g_stream>>>(da_.as<int64_t>(), db_.as<int64_t>(), dout.as<int64_t>(), n, d);
      break;
  }
  if ((rc = check_launch("add_broadcast_kernel")) != CSK_OK) return rc;
  CSK_TRY(fetch(out, dout.p, (size_t)n * esz));
  CSK_TRY(finish_fetches());
  return CSK_OK;
}

extern "C" int csk_moe_router_f64(const double* hidden, int64_t T, int64_t H, const double* gate_w, int64_t E,
                                  const float* gate_b, int64_t k, int sigmoid, float* out_pairs,
                                  double* out_logits) {
  REQUIRE_INIT();
  if (!hidden || !gate_w || !out_pairs || T < 0) return fail(CSK_ERR_ARG, "csk_moe_router_f64: null argument");
  if (E <= 0 || E > (int64_t)kZeroLen || k <= 0 || k > E || H <= 0 || H > (1 << 30) / E)
    return fail(CSK_ERR_ARG, "csk_moe_router_f64: need 1 <= top_k <= E <= 65536 and H * E <= 2^30");
  if (T == 0) return CSK_OK;
  DevBuf dx, dg, db, dl, dv, di, dw, dp;
  int rc;
  if ((rc = dg.upload(gate_w, (size_t)E * H * 8)) != CSK_OK) return rc;
  if (gate_b && (rc = db.upload(gate_b, (size_t)E * 4)) != CSK_OK) return rc;
  // passes small enough that tokens x experts and tokens x hidden fit 32-bit launch arithmetic
  const int64_t pass = std::max<int64_t>(1, std::min<int64_t>(kNodePassTokens, ((int64_t)1 << 28) / std::max(E, H)));
  for (int64_t t0 = 0; t0 < T; t0 += pass) {
    const int64_t tn = std::min(pass, T - t0);
    if ((rc = dx.upload(hidden + t0 * H, (size_t)tn * H * 8)) != CSK_OK) return rc;
    if ((rc = dl.alloc((size_t)tn * E * 8)) != CSK_OK) return rc;
    if ((rc = dv.alloc((size_t)tn * E * 8)) != CSK_OK) return rc;
    if ((rc = di.alloc((size_t)tn * E * 4)) != CSK_OK) return rc;
    if ((rc = dw.alloc((size_t)tn * k * 4)) != CSK_OK) return rc;
    if ((rc = dp.alloc((size_t)tn * k * 8)) != CSK_OK) return rc;
    router_f64_logits_kernel<<<dim3((unsigned)cdiv(E, 64), (unsigned)cdiv(tn, 4)), 256, 0, g_stream>>>(
        dx.as<double>(), dg.as<double>(), gate_b ? db.as<float>() : nullptr, dl.as<double>(), (int)tn, (int)E, (int)H);
    if ((rc = check_launch("router_f64_logits_kernel")) != CSK_OK) return rc;
    router_f64_topk_kernel<<<dim3((unsigned)cdiv(tn, 64)), 64, 0, g_stream>>>(
        dl.as<double>(), dv.as<double>(), di.as<int>(), dw.as<float>(), dp.as<float>(), (int)tn, (int)E, (int)k, sigmoid);
    if ((rc = check_launch("router_f64_topk_kernel")) != CSK_OK) return rc;
    CSK_TRY(fetch(out_pairs + t0 * k * 2, dp.p, (size_t)tn * k * 8));
    if (out_logits)
      CSK_TRY(fetch(out_logits + t0 * E, dl.p, (size_t)tn * E * 8));
    CSK_TRY(finish_fetches());
  }
  return CSK_OK;
}

