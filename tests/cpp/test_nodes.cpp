// Tests of the drop-in node classes (coalsack_amd/host/nodes) in the style of
// the reference's test/test_moe_router.cpp, test/test_expert_mlp.cpp and
// test/test_frame_sync.cpp, without googletest.
//   test_nodes --cpu   argument / error-path behaviour (no GPU call is reached)
//   test_nodes --gpu   numerics on the GPU against the CPU checker (oracle/)
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "coalsack/nn/nn_ops/add_node.h"
#include "coalsack/nn/nn_ops/dense_ffn_node.h"
#include "coalsack/nn/nn_ops/expert_merge_node.h"
#include "coalsack/nn/nn_ops/matmul_transpose_mixed_node.h"
#include "coalsack/nn/nn_ops/expert_mlp_node.h"
#include "coalsack/nn/nn_ops/moe_router_node.h"
#include "coalsack/nn/nn_ops/rmsnorm_node.h"

using namespace coalsack;

extern "C" {  // the CPU checker, oracle/moe_oracle.c
int orc_router(const float*, int64_t, int64_t, const float*, int64_t, const float*, int64_t, int, float*);
int orc_expert_token_mxfp4(const float*, const uint8_t*, const uint8_t*, const uint8_t*, const float*,
                           const float*, const float*, float*, int64_t, int64_t, int);
int orc_expert_mlp_mxfp4(int, const float*, int64_t, int64_t, int64_t, const uint8_t*, const uint8_t*,
                         const uint8_t*, const float*, const float*, const float*, const float*, int64_t,
                         int, int, float*, int*);
int orc_expert_merge(const float*, int64_t, int64_t, int64_t, int64_t, const float* const*, int, float*);
int orc_expert_mlp_f16(int, const float*, int64_t, int64_t, int64_t, const uint16_t*, const uint16_t*,
                       const uint16_t*, const float*, const float*, const float*, const float*, int64_t, int,
                       int, float*, int*);
int orc_dense_ffn_f16(const float*, int64_t, int64_t, int64_t, const uint16_t*, const uint16_t*, const uint16_t*,
                      const float*, const float*, const float*, float*);
void orc_matmul_transpose_f16(const float*, const uint16_t*, float*, int64_t, int64_t, int64_t);
void orc_rmsnorm(const float*, const float*, float*, int64_t, int64_t, float);
void orc_rmsnorm_f64(const double*, const double*, double*, int64_t, int64_t, float);
void orc_add(const float*, const float*, float*, int64_t);
void orc_matmul_transpose_batched(const float*, int64_t, const void*, int64_t, int, int64_t, float*, int64_t, int64_t,
                                  int64_t);
int orc_dense_ffn_f32(const float*, int64_t, int64_t, int64_t, const float*, const float*, const float*, const float*,
                      const float*, const float*, float*);
int orc_add_broadcast(const void*, const int64_t*, int, const void*, const int64_t*, int, int, void*, int64_t*);
int orc_router_f64(const double*, int64_t, int64_t, const double*, int64_t, const float*, int64_t, int, float*, double*);
}

static int g_failed = 0, g_checks = 0;
#define CHECK(cond)                                                              \
  do {                                                                           \
    ++g_checks;                                                                  \
    if (!(cond)) {                                                               \
      ++g_failed;                                                                \
      std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);            \
    }                                                                            \
  } while (0)

static bool throws_with(const std::function<void()>& fn, const std::string& text) {
  try {
    fn();
  } catch (const std::exception& e) {
    if (std::string(e.what()).find(text) != std::string::npos) return true;
    std::printf("  unexpected message: %s\n", e.what());
    return false;
  }
  return false;
}

static dynamic_tensor random_tensor(const std::vector<int64_t>& shape, std::mt19937& gen, float lo, float hi) {
  dynamic_tensor t(dtype::float32, shape);
  std::uniform_real_distribution<float> d(lo, hi);
  for (int64_t i = 0; i < t.numel(); ++i) t.data_ptr<float>()[i] = d(gen);
  return t;
}

static dynamic_mx_tensor random_mx(int64_t rows, int64_t cols, std::mt19937& gen) {
  dynamic_mx_tensor t({rows, cols});
  std::uniform_int_distribution<int> byte(0, 255), scale(117, 121);
  uint8_t* p = t.data_ptr();
  for (size_t b = 0; b < t.num_blocks(); ++b) {
    p[17 * b] = (uint8_t)scale(gen);
    for (int j = 1; j < 17; ++j) p[17 * b + j] = (uint8_t)byte(gen);
  }
  return t;
}

// captures what a node sends, like message_capture_node of test/test_frame_sync.cpp
struct capture_node : graph_node {
  std::vector<std::shared_ptr<result_message>> got;
  std::string get_proc_name() const override { return "capture"; }
  void process(std::string, graph_message_ptr m) override {
    got.push_back(std::dynamic_pointer_cast<result_message>(m));
  }
};

// ------------------------------------------------------------------ CPU mode

static void cpu_router_argument_errors() {
  std::printf("router: argument errors\n");
  moe_router_node node;
  node.set_config(8, 2);
  dynamic_tensor h3(dtype::float32, {1, 2, 4}), h2(dtype::float32, {2, 4});
  dynamic_tensor g(dtype::float32, {8, 4}), g_bad(dtype::float32, {7, 4}), g1(dtype::float32, {32});
  dynamic_tensor b(dtype::float32, {8}), b_bad(dtype::float32, {5}), b2(dtype::float32, {8, 1});
  CHECK(throws_with([&] { node.compute_test(h2, g); }, "moe_router: hidden_states must be 3D"));
  CHECK(throws_with([&] { node.compute_test(h3, g1); }, "moe_router: gate_weights must be 2D"));
  CHECK(throws_with([&] { node.compute_test(h3, g_bad); }, "moe_router: gate_weights shape mismatch, expected [8, 4], got [7, 4]"));
  CHECK(throws_with([&] { node.compute_test(h3, g, b_bad); }, "moe_router: gate_bias must have num_experts=8 elements, got 5"));
  CHECK(throws_with([&] { node.compute_test(h3, g, b2); }, "moe_router: gate_bias must be 1D"));
  CHECK(throws_with([&] { node.compute_test(dynamic_tensor(dtype::int32, {1, 2, 4}), g); },
                    "moe_router: only float32 and float64 supported"));
  CHECK(throws_with([&] { node.compute_test(dynamic_tensor(dtype::float64, {1, 2, 4}), g); },
                    "moe_router: gate_weights must have the element type of hidden_states"));
  // through process(): the exception becomes an error result with a null field (nn_op_node.h:306-314)
  capture_node cap;
  cap.set_input(node.get_output());
  node.set_input_names({"h", "g"});
  node.set_output_name("router_out");
  auto msg = result_message::ok({{"h", std::make_shared<dynamic_tensor_message>(h2)},
                                 {"g", std::make_shared<dynamic_tensor_message>(g)}});
  msg->set_frame_number(7);
  node.process("default", msg);
  CHECK(cap.got.size() == 1 && cap.got[0]->is_error() && cap.got[0]->get_frame_number() == 7);
  CHECK(cap.got[0]->get_fields().count("router_out") == 1 && cap.got[0]->get_field("router_out") == nullptr);
  CHECK(cap.got[0]->get_error_message().find("must be 3D") != std::string::npos);
}

static void cpu_expert_node_paths() {
  std::printf("expert_mlp: error propagation, missing field, unselected expert\n");
  std::mt19937 gen(42);
  expert_mlp_node node(5);
  capture_node cap;
  cap.set_input(node.get_output());
  node.set_input_names({"hidden", "w_up", "w_gate", "w_down", "router"});
  node.set_output_name("e5");
  CHECK(node.get_expert_id() == 5 && node.get_proc_name() == "expert_mlp");
  // upstream error is forwarded, compute is skipped (expert_mlp_node.h:82-91)
  node.process("default", result_message::error({{"hidden", nullptr}}, "boom"));
  CHECK(cap.got.size() == 1 && cap.got[0]->is_error() && cap.got[0]->get_error_message() == "Input error");
  // missing field (:104-106)
  auto hidden = std::make_shared<dynamic_tensor_message>(random_tensor({1, 3, 64}, gen, -1, 1));
  node.process("default", result_message::ok({{"hidden", hidden}}));
  CHECK(cap.got.size() == 2 && cap.got[1]->is_error() &&
        cap.got[1]->get_error_message() == "expert_mlp: missing field w_up");
  // no token selects expert 5: ok message with a {0}-shaped f32 tensor (:441-443), no GPU work
  auto w = std::make_shared<dynamic_mx_tensor_message>(random_mx(64, 64, gen));
  dynamic_tensor router(dtype::float32, {1, 3, 2, 2});
  for (int p = 0; p < 6; ++p) {
    router.data_ptr<float>()[2 * p] = (float)(p % 4);
    router.data_ptr<float>()[2 * p + 1] = 0.5f;
  }
  auto msg = result_message::ok({{"hidden", hidden}, {"w_up", w}, {"w_gate", w}, {"w_down", w},
                                 {"router", std::make_shared<dynamic_tensor_message>(router)}});
  msg->set_frame_number(3);
  msg->set_timestamp(1.5);
  node.process("default", msg);
  CHECK(cap.got.size() == 3 && cap.got[2]->is_ok() && cap.got[2]->get_frame_number() == 3 &&
        cap.got[2]->get_timestamp() == 1.5);
  auto out = std::dynamic_pointer_cast<dynamic_tensor_message>(cap.got[2]->get_field("e5"));
  CHECK(out && out->get_tensor().ndim() == 1 && out->get_tensor().dim(0) == 0);
  // bad router shape (:436-438) and wrong input count (:394-397)
  dynamic_tensor router3(dtype::float32, {1, 3, 4});
  node.process("default", result_message::ok({{"hidden", hidden}, {"w_up", w}, {"w_gate", w}, {"w_down", w},
                                              {"router", std::make_shared<dynamic_tensor_message>(router3)}}));
  CHECK(cap.got[3]->is_error() &&
        cap.got[3]->get_error_message() == "expert_mlp: router_output must be 4D [batch, seq_len, top_k, 2]");
  node.set_input_names({"hidden", "w_up", "w_gate", "w_down"});
  node.process("default", msg);
  CHECK(cap.got[4]->is_error() && cap.got[4]->get_error_message() == "expert_mlp: expected 5 or 8 inputs for MXFP4, got 4");
}

// float32 -> IEEE half bits, round to nearest even (test data only)
static uint16_t half_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const int32_t e = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  uint32_t m = x & 0x7fffffu;
  if (e >= 31) return (uint16_t)(sign | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    m |= 0x800000u;
    const int sh = 14 - e;
    uint32_t h = m >> sh;
    const uint32_t rem = m & ((1u << sh) - 1), half = 1u << (sh - 1);
    if (rem > half || (rem == half && (h & 1))) ++h;
    return (uint16_t)(sign | h);
  }
  uint32_t h = ((uint32_t)e << 10) | (m >> 13);
  const uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
  return (uint16_t)(sign | h);
}

static dynamic_tensor random_half_tensor(const std::vector<int64_t>& shape, std::mt19937& gen, float lo, float hi) {
  dynamic_tensor t(dtype::float16, shape);
  std::uniform_real_distribution<float> d(lo, hi);
  uint16_t* p = t.data_ptr<uint16_t>();
  for (int64_t i = 0; i < t.numel(); ++i) p[i] = half_bits(d(gen));
  return t;
}

static dynamic_tensor router_first_slot(int64_t B, int64_t S, int64_t K, int first_expert) {
  // test/test_expert_mlp.cpp:84-95: slot 0 names first_expert, slot k names expert k, weights 1 / top_k
  dynamic_tensor r(dtype::float32, {B, S, K, 2});
  float* p = r.data_ptr<float>();
  for (int64_t t = 0; t < B * S; ++t)
    for (int64_t k = 0; k < K; ++k) {
      p[(t * K + k) * 2] = k == 0 ? (float)first_expert : (float)k;
      p[(t * K + k) * 2 + 1] = 1.0f / (float)K;
    }
  return r;
}

static void cpu_expert_fp16_argument_errors() {
  std::printf("expert_mlp (float16 weights): argument errors, unselected expert\n");
  std::mt19937 gen(3);
  expert_mlp_node node(0);
  auto hidden = random_tensor({1, 2, 8}, gen, -1, 1);
  auto w_up = random_half_tensor({16, 8}, gen, -0.1f, 0.1f), w_gate = random_half_tensor({16, 8}, gen, -0.1f, 0.1f);
  auto w_down = random_half_tensor({8, 16}, gen, -0.1f, 0.1f);
  auto router = router_first_slot(1, 2, 4, 0);
  CHECK(throws_with([&] { node.compute_test({hidden, w_up, w_gate, router}); },
                    "expert_mlp: expected 5 or 8 inputs (hidden, w_up, w_gate, w_down[, b_up, b_gate, b_down], router_output), got 4"));
  CHECK(throws_with([&] { node.compute_test({hidden, w_up, w_gate, w_down, dynamic_tensor(dtype::float32, {1, 2, 8})}); },
                    "expert_mlp: router_output must be 4D [batch, seq_len, top_k, 2], got 3D"));
  CHECK(throws_with([&] { node.compute_test({dynamic_tensor(dtype::float32, {2, 8}), w_up, w_gate, w_down, router}); },
                    "expert_mlp: hidden_states must be 3D [batch, seq_len, hidden_dim], got 2D"));
  CHECK(throws_with([&] { node.compute_test({hidden, random_half_tensor({16, 7}, gen, -1, 1), w_gate, w_down, router}); },
                    "expert_mlp: w_up must be [16, 8], got [16, 7]"));
  CHECK(throws_with([&] { node.compute_test({hidden, w_up, random_half_tensor({15, 8}, gen, -1, 1), w_down, router}); },
                    "expert_mlp: w_gate must be [16, 8], got [15, 8]"));
  CHECK(throws_with([&] { node.compute_test({hidden, w_up, w_gate, random_half_tensor({8, 15}, gen, -1, 1), router}); },
                    "expert_mlp: w_down must be [8, 16], got [8, 15]"));
  CHECK(throws_with([&] { node.compute_test({hidden, w_up, w_gate, w_down, random_tensor({15}, gen, 0, 1),
                                             random_tensor({16}, gen, 0, 1), random_tensor({8}, gen, 0, 1), router}); },
                    "expert_mlp: b_up must be [expert_ffn_dim=16], got [15]"));
  CHECK(throws_with([&] { node.compute_test({hidden, random_tensor({16, 8}, gen, -1, 1), w_gate, w_down, router}); },
                    "expert_mlp: all weights must be FLOAT16"));
  // an expert no token selected returns the {0}-shaped tensor before any shape is looked at (:297-306)
  expert_mlp_node other(9);
  auto out = other.compute_test({dynamic_tensor(dtype::float32, {2, 8}), w_up, w_gate, w_down, router});
  CHECK(out.ndim() == 1 && out.dim(0) == 0);
}

static void cpu_dense_ffn_argument_errors() {
  std::printf("dense_ffn: argument errors\n");
  std::mt19937 gen(5);
  dense_ffn_node node;
  CHECK(node.get_proc_name() == "dense_ffn");
  auto hidden = random_tensor({1, 3, 8}, gen, -1, 1);
  auto gate = random_half_tensor({16, 8}, gen, -0.1f, 0.1f), up = random_half_tensor({16, 8}, gen, -0.1f, 0.1f);
  auto down = random_half_tensor({8, 16}, gen, -0.1f, 0.1f);
  CHECK(throws_with([&] { node.compute_test({hidden, gate, up}); },
                    "dense_ffn: expected 4 or 7 inputs (hidden, gate_w, up_w, down_w[, gate_b, up_b, down_b]), got 3"));
  CHECK(throws_with([&] { node.compute_test({dynamic_tensor(dtype::float32, {3, 8}), gate, up, down}); },
                    "dense_ffn: hidden_states must be 3D [B, S, D], got 2D"));
  CHECK(throws_with([&] { node.compute_test({hidden, dynamic_tensor(dtype::float16, {16}), up, down}); },
                    "dense_ffn: weight tensors must be 2D"));
  CHECK(throws_with([&] { node.compute_test({hidden, gate, random_tensor({16, 8}, gen, -1, 1), down}); },
                    "dense_ffn: weight tensors must all be FLOAT16 or all FLOAT32"));
  CHECK(throws_with([&] { node.compute_test({hidden, gate, random_half_tensor({15, 8}, gen, -1, 1), down}); },
                    "dense_ffn: gate_w/up_w shape mismatch"));
  CHECK(throws_with([&] { node.compute_test({hidden, gate, up, random_half_tensor({8, 15}, gen, -1, 1)}); },
                    "dense_ffn: down_w shape mismatch, expected [8, 16], got [8, 15]"));
  CHECK(throws_with([&] { node.compute_test({hidden, random_tensor({16, 8}, gen, -1, 1), random_tensor({16, 8}, gen, -1, 1),
                                             down}); },
                    "dense_ffn: weight tensors must all be FLOAT16 or all FLOAT32"));
}

static void cpu_matmul_argument_errors() {
  std::printf("matmul_transpose_mixed: argument errors\n");
  std::mt19937 gen(6);
  matmul_transpose_mixed_node node;
  CHECK(node.get_proc_name() == "nn_matmul_transpose_mixed");
  auto a = random_tensor({2, 3, 8}, gen, -1, 1);
  auto w = random_half_tensor({5, 8}, gen, -1, 1);
  CHECK(throws_with([&] { node.compute_test(dynamic_tensor(dtype::float64, {3, 8}), w); }, "matmul_transpose_mixed: input A must be fp32"));
  CHECK(throws_with([&] { node.compute_test(a, dynamic_tensor(dtype::int32, {5, 8})); }, "matmul_transpose_mixed: input B must be fp32 or fp16"));
  CHECK(throws_with([&] { node.compute_test(dynamic_tensor(dtype::float32, {8}), w); }, "matmul_transpose_mixed: inputs must be at least 2D"));
  CHECK(throws_with([&] { node.compute_test(a, random_half_tensor({5, 7}, gen, -1, 1)); }, "matmul_transpose_mixed: incompatible dimensions"));
  CHECK(throws_with([&] { node.compute_test(a, random_half_tensor({3, 5, 8}, gen, -1, 1)); },
                    "Incompatible shapes for broadcasting"));  // batch [2] against [3]
}

static void cpu_merge_argument_errors() {
  std::printf("expert_merge: argument errors\n");
  expert_merge_node node;
  node.set_config(4, 2);
  dynamic_tensor router(dtype::float32, {1, 2, 2, 2}), empty(dtype::float32, {0});
  CHECK(throws_with([&] { node.compute_test({router, empty}); }, "expert_merge: expected 5 inputs, got 2"));
  dynamic_tensor router_bad(dtype::float32, {1, 2, 3, 2});
  CHECK(throws_with([&] { node.compute_test({router_bad, empty, empty, empty, empty}); },
                    "expert_merge: router output must have shape [batch, seq_len, 2, 2]"));
  CHECK(throws_with([&] { node.compute_test({router, empty, empty, empty, empty}); },
                    "expert_merge: no non-empty expert outputs found"));
  dynamic_tensor a(dtype::float32, {1, 2, 8}), b(dtype::float32, {1, 3, 8});
  CHECK(throws_with([&] { node.compute_test({router, a, b, empty, empty}); },
                    "expert_merge: all non-empty expert outputs must have same shape"));
}

// ------------------------------------------------------------------ GPU mode

static void cpu_norm_add_argument_errors() {
  std::mt19937 gen(5);
  rmsnorm_node norm;
  add_node add;
  CHECK(norm.get_proc_name() == "nn_rmsnorm" && add.get_proc_name() == "nn_add");
  auto x = random_tensor({2, 3, 8}, gen, -1, 1), w = random_tensor({8}, gen, 0.5f, 1.5f);
  auto w_bad = random_tensor({7}, gen, 0.5f, 1.5f), w2 = random_tensor({1, 8}, gen, 0.5f, 1.5f);
  CHECK(throws_with([&] { norm.compute_test(dynamic_tensor(dtype::float32, {}), w); },
                    "rmsnorm: input must have at least 1 dimension"));
  CHECK(throws_with([&] { norm.compute_test(x, w_bad); }, "rmsnorm: weight shape must be [hidden_dim]"));
  CHECK(throws_with([&] { norm.compute_test(x, w2); }, "rmsnorm: weight shape must be [hidden_dim]"));
  CHECK(throws_with([&] { norm.compute_test(dynamic_tensor(dtype::float16, {2, 8}), w); },
                    "rmsnorm: only float32 and float64 supported"));  // rmsnorm_node.h:52
  CHECK(throws_with([&] { norm.compute_test(dynamic_tensor(dtype::float64, {2, 8}), w); },
                    "rmsnorm: weight must have the input's element type"));
  CHECK(throws_with([&] { add.compute_test(x, dynamic_tensor(dtype::float64, {2, 3, 8})); }, "add: input dtype mismatch"));
  CHECK(throws_with([&] { add.compute_test(x, w_bad); }, "Broadcast failed: Shape A=[2,3,8], Shape B=[7]"));
  CHECK(throws_with([&] { add.compute_test(dynamic_tensor(dtype::float16, {2}), dynamic_tensor(dtype::float16, {2})); },
                    "add: unsupported dtype"));
  // through process(): missing input names and upstream errors (nn_op_node.h:172-219)
  capture_node cap;
  cap.set_input(norm.get_output());
  norm.set_output_name("y");
  auto msg = result_message::ok({{"x", std::make_shared<dynamic_tensor_message>(x)},
                                 {"w", std::make_shared<dynamic_tensor_message>(w)}});
  msg->set_frame_number(11);
  norm.process("default", msg);
  CHECK(cap.got.size() == 1 && cap.got[0]->is_error() && cap.got[0]->get_frame_number() == 11 &&
        cap.got[0]->get_error_message() == "rmsnorm: input names not set" && cap.got[0]->get_field("y") == nullptr);
  norm.set_input_names("x", "w");
  auto err = result_message::error({{"x", nullptr}}, "upstream");
  norm.process("default", err);
  CHECK(cap.got.size() == 2 && cap.got[1]->is_error() && cap.got[1]->get_error_message() == "Input error");
  CHECK((norm.get_input_names() == std::vector<std::string>{"x", "w"}));
}

static void gpu_norm_add_tests() {
  std::mt19937 gen(77);
  const int64_t B = 2, S = 5, H = 2880;
  rmsnorm_node norm;
  add_node add;
  auto x = random_tensor({B, S, H}, gen, -2, 2), w = random_tensor({H}, gen, 0.5f, 1.5f);
  // the reference's test values (test_rmsnorm.cpp:74-115): ones with unit weight stay ones
  dynamic_tensor ones(dtype::float32, {1, 4}), w1(dtype::float32, {4});
  for (int i = 0; i < 4; ++i) ones.data_ptr<float>()[i] = 1.0f, w1.data_ptr<float>()[i] = 1.0f;
  auto o1 = norm.compute_test(ones, w1);
  for (int i = 0; i < 4; ++i) CHECK(std::fabs(o1.data_ptr<float>()[i] - 1.0f) < 1e-4f);
  norm.set_epsilon(1e-6f);
  auto y = norm.compute_test(x, w);
  std::vector<float> want((size_t)(B * S * H));
  orc_rmsnorm(x.data_ptr<float>(), w.data_ptr<float>(), want.data(), B * S, H, 1e-6f);
  CHECK(y.shape() == x.shape());
  float worst = 0;
  for (size_t i = 0; i < want.size(); ++i) worst = std::fmax(worst, std::fabs(y.data_ptr<float>()[i] - want[i]));
  CHECK(worst <= 2e-6f);
  {  // the float64 branch (rmsnorm_node.h:49-50): equal to the CPU's double arithmetic bit for bit
    dynamic_tensor xd(dtype::float64, {B, S, H}), wd(dtype::float64, {H});
    std::uniform_real_distribution<double> dx(-2.0, 2.0), dw(0.5, 1.5);
    for (int64_t i = 0; i < B * S * H; ++i) xd.data_ptr<double>()[i] = dx(gen);
    for (int64_t i = 0; i < H; ++i) wd.data_ptr<double>()[i] = dw(gen);
    auto yd = norm.compute_test(xd, wd);
    CHECK(yd.get_dtype() == dtype::float64 && yd.shape() == xd.shape());
    std::vector<double> wantd((size_t)(B * S * H));
    orc_rmsnorm_f64(xd.data_ptr<double>(), wd.data_ptr<double>(), wantd.data(), B * S, H, 1e-6f);
    CHECK(std::memcmp(yd.data_ptr<double>(), wantd.data(), wantd.size() * sizeof(double)) == 0);
    // test_rmsnorm.cpp:118-142 in double: 5 / sqrt(25) * 2 = 2
    dynamic_tensor x1(dtype::float64, {1, 1}), w1d(dtype::float64, {1});
    x1.data_ptr<double>()[0] = 5.0, w1d.data_ptr<double>()[0] = 2.0;
    norm.set_epsilon(0.0f);
    CHECK(norm.compute_test(x1, w1d).data_ptr<double>()[0] == 2.0);
    norm.set_epsilon(1e-6f);
    CHECK(norm.compute_test(dynamic_tensor(dtype::float64, {0, 8}), dynamic_tensor(dtype::float64, {8})).numel() == 0);
  }
  auto z = add.compute_test(x, y);
  orc_add(x.data_ptr<float>(), y.data_ptr<float>(), want.data(), B * S * H);
  CHECK(std::memcmp(z.data_ptr<float>(), want.data(), want.size() * sizeof(float)) == 0);
  // h <- h + f(rmsnorm(h)) wiring through messages (llm_engine.cpp:714-719, 773-777)
  capture_node cap;
  cap.set_input(add.get_output());
  add.set_input_names("h", "moe_out");
  add.set_output_name("h_next");
  auto msg = result_message::ok({{"h", std::make_shared<dynamic_tensor_message>(x)},
                                 {"moe_out", std::make_shared<dynamic_tensor_message>(y)}});
  msg->set_frame_number(4);
  add.process("default", msg);
  CHECK(cap.got.size() == 1 && cap.got[0]->is_ok() && cap.got[0]->get_frame_number() == 4);
  auto hn = std::dynamic_pointer_cast<dynamic_tensor_message>(cap.got[0]->get_field("h_next"));
  CHECK(hn && std::memcmp(hn->get_tensor().data_ptr<float>(), want.data(), want.size() * sizeof(float)) == 0);
}

static void gpu_router_tests() {
  std::printf("router: Basic / TopKSelection / GptOssScale / WeightNormalization\n");
  std::mt19937 gen(42);
  {  // test/test_moe_router.cpp:24-79
    moe_router_node node;
    node.set_config(8, 2);
    auto h = random_tensor({1, 2, 4}, gen, -1, 1), g = random_tensor({8, 4}, gen, -1, 1);
    dynamic_tensor b(dtype::float32, {8});
    std::memset(b.data_ptr<float>(), 0, b.bytes());
    auto out = node.compute_test(h, g, b);
    CHECK((out.shape() == std::vector<int64_t>{1, 2, 2, 2}));
    for (int s = 0; s < 2; ++s) {
      float sum = 0;
      for (int k = 0; k < 2; ++k) {
        const float idx = out.data_ptr<float>()[(s * 2 + k) * 2], w = out.data_ptr<float>()[(s * 2 + k) * 2 + 1];
        CHECK(idx >= 0 && idx < 8 && w > 0);
        sum += w;
      }
      CHECK(std::fabs(sum - 1.0f) < 1e-5f);
    }
  }
  {  // :82-138: hidden = 1, gate row e = e / H  =>  experts 5, 4, 3
    moe_router_node node;
    node.set_config(6, 3);
    dynamic_tensor h(dtype::float32, {1, 1, 4}), g(dtype::float32, {6, 4});
    for (int i = 0; i < 4; ++i) h.data_ptr<float>()[i] = 1.0f;
    for (int e = 0; e < 6; ++e)
      for (int d = 0; d < 4; ++d) g.data_ptr<float>()[e * 4 + d] = (float)e / 4;
    auto out = node.compute_test(h, g);
    CHECK((int)out.data_ptr<float>()[0] == 5 && (int)out.data_ptr<float>()[2] == 4 && (int)out.data_ptr<float>()[4] == 3);
  }
  {  // :141-203 gpt-oss scale, and agreement with the CPU checker
    moe_router_node node;
    node.set_config(32, 4);
    auto h = random_tensor({2, 8, 128}, gen, -1, 1), g = random_tensor({32, 128}, gen, -0.2f, 0.2f);
    auto b = random_tensor({32}, gen, -0.01f, 0.01f);
    auto out = node.compute_test(h, g, b);
    std::vector<float> want(16 * 4 * 2);
    orc_router(h.data_ptr<float>(), 16, 128, g.data_ptr<float>(), 32, b.data_ptr<float>(), 4, 0, want.data());
    for (int t = 0; t < 16; ++t) {
      float sum = 0;
      for (int k = 0; k < 4; ++k) {
        const float* o = out.data_ptr<float>() + (t * 4 + k) * 2;
        CHECK(o[0] == want[(t * 4 + k) * 2] && std::fabs(o[1] - want[(t * 4 + k) * 2 + 1]) < 1e-5f && o[1] <= 1.0f);
        sum += o[1];
      }
      CHECK(std::fabs(sum - 1.0f) < 1e-4f);
    }
  }
}

static void gpu_expert_known_answer() {
  std::printf("expert_mlp: ModifiedSwigluActivation (gate = 1.0, up = 1.5, identity down)\n");
  // test/test_expert_mlp.cpp:118-200 recast for MXFP4 storage
  const int64_t H = 32, F = 32;
  std::vector<uint8_t> wz(F * 17, 0), wd(H * 17, 0);
  for (int r = 0; r < 32; ++r) {
    wz[r * 17] = 128;
    wd[r * 17] = 128;
    if (r < 16) wd[r * 17 + 1 + r] |= 1;  // code 1 = +1.0 at element r
    else wd[r * 17 + 1 + r - 16] |= 1 << 4;
  }
  std::vector<float> x(H, 1.0f), bu(F, 1.5f), bg(F, 1.0f), bd(H, 0.0f), out(H);
  expert_mlp_node node(0);
  node.compute_test_mxfp4(x.data(), wz.data(), wz.data(), wd.data(), bu.data(), bg.data(), bd.data(), out.data(), H, F);
  const float want = 1.0f / (1.0f + std::exp(-1.702f)) * 2.5f;
  for (int i = 0; i < H; ++i) CHECK(std::fabs(out[i] - want) < 1e-3f);
  node.set_activation_type(expert_mlp_node::activation_type::STANDARD_SWIGLU);
  node.compute_test_mxfp4(x.data(), wz.data(), wz.data(), wd.data(), bu.data(), bg.data(), bd.data(), out.data(), H, F);
  const float want2 = 1.0f / (1.0f + std::exp(-1.0f)) * 1.5f;
  for (int i = 0; i < H; ++i) CHECK(std::fabs(out[i] - want2) < 1e-3f);
}

// The reference's four float16 tests (test/test_expert_mlp.cpp) on the GPU node, each
// also compared with the CPU checker.
static void gpu_expert_fp16_tests() {
  std::printf("expert_mlp (float16 weights): Basic, ModifiedSwigluActivation, MultipleExperts, GptOssScale\n");
  std::mt19937 gen(42);
  auto run_case = [&](int expert_id, int64_t B, int64_t S, int64_t H, int64_t F, int64_t K, bool through_messages) {
    auto hidden = random_tensor({B, S, H}, gen, -0.5f, 0.5f);
    auto w_up = random_half_tensor({F, H}, gen, -0.1f, 0.1f), w_gate = random_half_tensor({F, H}, gen, -0.1f, 0.1f);
    auto w_down = random_half_tensor({H, F}, gen, -0.1f, 0.1f);
    auto b_up = random_tensor({F}, gen, -0.05f, 0.05f), b_gate = random_tensor({F}, gen, -0.05f, 0.05f);
    auto b_down = random_tensor({H}, gen, -0.05f, 0.05f);
    auto router = router_first_slot(B, S, K, expert_id);
    expert_mlp_node node(expert_id);
    CHECK(node.get_expert_id() == expert_id);
    dynamic_tensor out;
    if (through_messages) {
      node.set_input_names({"hidden", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "router"});
      node.set_output_name("out");
      capture_node cap;
      cap.set_input(node.get_output());
      auto mk = [](const dynamic_tensor& t) { return std::make_shared<dynamic_tensor_message>(t); };
      node.process("default", result_message::ok({{"hidden", mk(hidden)}, {"w_up", mk(w_up)}, {"w_gate", mk(w_gate)},
                                                  {"w_down", mk(w_down)}, {"b_up", mk(b_up)}, {"b_gate", mk(b_gate)},
                                                  {"b_down", mk(b_down)}, {"router", mk(router)}}));
      CHECK(cap.got.size() == 1 && cap.got[0]->is_ok());
      out = std::dynamic_pointer_cast<dynamic_tensor_message>(cap.got[0]->get_field("out"))->get_tensor();
    } else {
      out = node.compute_test({hidden, w_up, w_gate, w_down, b_up, b_gate, b_down, router});
    }
    CHECK(out.shape() == hidden.shape());
    bool nonzero = false, nan = false;
    for (int64_t i = 0; i < out.numel(); ++i) {
      nonzero |= std::fabs(out.data_ptr<float>()[i]) > 1e-6f;
      nan |= std::isnan(out.data_ptr<float>()[i]);
    }
    CHECK(nonzero && !nan);
    std::vector<float> want(B * S * H);
    int empty = 0;
    orc_expert_mlp_f16(expert_id, hidden.data_ptr<float>(), B * S, H, F, w_up.data_ptr<uint16_t>(),
                       w_gate.data_ptr<uint16_t>(), w_down.data_ptr<uint16_t>(), b_up.data_ptr<float>(),
                       b_gate.data_ptr<float>(), b_down.data_ptr<float>(), router.data_ptr<float>(), K, 0, 0,
                       want.data(), &empty);
    float worst = 0;
    for (int64_t i = 0; i < out.numel(); ++i)
      worst = std::fmax(worst, std::fabs(out.data_ptr<float>()[i] - want[i]) / std::fmax(1.0f, std::fabs(want[i])));
    CHECK(!empty && worst <= 1e-3f);
    return worst;
  };
  run_case(0, 1, 2, 8, 16, 4, false);                                  // Basic (:49-115)
  for (int e : {0, 5, 15, 31}) run_case(e, 1, 1, 8, 16, 4, e == 5);     // MultipleExperts (:203-276)
  const float w = run_case(0, 2, 4, 128, 128, 4, true);                 // GptOssScale (:279-354)
  std::printf("  GptOssScale: max rel err against the CPU path %.3g\n", w);
  // ModifiedSwigluActivation (:118-200): hidden_dim = expert_ffn_dim = 2
  dynamic_tensor hidden(dtype::float32, {1, 1, 2});
  hidden.data_ptr<float>()[0] = 1.0f, hidden.data_ptr<float>()[1] = 0.5f;
  dynamic_tensor w_up(dtype::float16, {2, 2}), w_gate(dtype::float16, {2, 2}), w_down(dtype::float16, {2, 2});
  dynamic_tensor b_up(dtype::float32, {2}), b_gate(dtype::float32, {2}), b_down(dtype::float32, {2});
  for (auto* t : {&w_up, &w_gate, &w_down}) std::memset(t->data_ptr<uint16_t>(), 0, 8);
  for (auto* t : {&b_up, &b_gate, &b_down}) std::memset(t->data_ptr<float>(), 0, 8);
  w_up.data_ptr<uint16_t>()[0] = half_bits(1.0f);
  b_up.data_ptr<float>()[0] = 0.5f;
  w_gate.data_ptr<uint16_t>()[0] = half_bits(1.0f);
  w_down.data_ptr<uint16_t>()[0] = half_bits(1.0f);
  w_down.data_ptr<uint16_t>()[2] = half_bits(1.0f);
  dynamic_tensor router(dtype::float32, {1, 1, 4, 2});
  for (int k = 0; k < 4; ++k) router.data_ptr<float>()[2 * k] = (float)k, router.data_ptr<float>()[2 * k + 1] = k == 0;
  expert_mlp_node node(0);
  auto out = node.compute_test({hidden, w_up, w_gate, w_down, b_up, b_gate, b_down, router});
  const float want = 1.0f / (1.0f + std::exp(1.702f * -1.0f)) * (1.5f + 1.0f);
  CHECK(std::fabs(out.data_ptr<float>()[0] - want) < 1e-3f);
}

static void gpu_matmul_tests() {
  std::printf("matmul_transpose_mixed: projections against the CPU path\n");
  std::mt19937 gen(10);
  for (const auto& dims : std::vector<std::vector<int64_t>>{{1, 1, 64, 96}, {2, 40, 72, 130}, {1, 3, 30, 21}}) {
    const int64_t B = dims[0], S = dims[1], K = dims[2], N = dims[3];
    auto a = random_tensor({B, S, K}, gen, -1, 1);
    auto w = random_half_tensor({N, K}, gen, -0.2f, 0.2f);
    matmul_transpose_mixed_node node;
    auto out = node.compute_test(a, w);
    CHECK((out.shape() == std::vector<int64_t>{B, S, N}));
    std::vector<float> want(B * S * N);
    orc_matmul_transpose_f16(a.data_ptr<float>(), w.data_ptr<uint16_t>(), want.data(), B * S, K, N);
    float worst = 0;
    for (int64_t i = 0; i < out.numel(); ++i)
      worst = std::fmax(worst, std::fabs(out.data_ptr<float>()[i] - want[i]) / std::fmax(1.0f, std::fabs(want[i])));
    CHECK(worst <= 1e-3f);
  }
}

static void gpu_dense_ffn_tests() {
  std::printf("dense_ffn: shared expert through result messages, against the CPU path\n");
  std::mt19937 gen(9);
  for (const auto& dims : std::vector<std::vector<int64_t>>{{1, 5, 64, 96}, {2, 40, 72, 130}, {1, 3, 30, 20}}) {
    const int64_t B = dims[0], S = dims[1], H = dims[2], F = dims[3];
    for (bool bias : {false, true}) {
      auto hidden = random_tensor({B, S, H}, gen, -1, 1);
      auto gate = random_half_tensor({F, H}, gen, -0.2f, 0.2f), up = random_half_tensor({F, H}, gen, -0.2f, 0.2f);
      auto down = random_half_tensor({H, F}, gen, -0.2f, 0.2f);
      auto bg = random_tensor({F}, gen, -0.1f, 0.1f), bu = random_tensor({F}, gen, -0.1f, 0.1f);
      auto bd = random_tensor({H}, gen, -0.1f, 0.1f);
      dense_ffn_node node;
      capture_node cap;
      cap.set_input(node.get_output());
      node.set_output_name("out");
      auto mk = [](const dynamic_tensor& t) { return std::make_shared<dynamic_tensor_message>(t); };
      if (bias) {
        node.set_input_names({"x", "g", "u", "d", "bg", "bu", "bd"});
        node.process("default", result_message::ok({{"x", mk(hidden)}, {"g", mk(gate)}, {"u", mk(up)}, {"d", mk(down)},
                                                    {"bg", mk(bg)}, {"bu", mk(bu)}, {"bd", mk(bd)}}));
      } else {
        node.set_input_names({"x", "g", "u", "d"});
        node.process("default", result_message::ok({{"x", mk(hidden)}, {"g", mk(gate)}, {"u", mk(up)}, {"d", mk(down)}}));
      }
      CHECK(cap.got.size() == 1 && cap.got[0]->is_ok());
      auto out = std::dynamic_pointer_cast<dynamic_tensor_message>(cap.got[0]->get_field("out"))->get_tensor();
      CHECK(out.shape() == hidden.shape());
      std::vector<float> want(B * S * H);
      CHECK(orc_dense_ffn_f16(hidden.data_ptr<float>(), B * S, H, F, gate.data_ptr<uint16_t>(), up.data_ptr<uint16_t>(),
                              down.data_ptr<uint16_t>(), bias ? bg.data_ptr<float>() : nullptr,
                              bias ? bu.data_ptr<float>() : nullptr, bias ? bd.data_ptr<float>() : nullptr,
                              want.data()) == 0);
      float worst = 0;
      for (int64_t i = 0; i < out.numel(); ++i)
        worst = std::fmax(worst, std::fabs(out.data_ptr<float>()[i] - want[i]) / std::fmax(1.0f, std::fabs(want[i])));
      CHECK(worst <= 1e-3f);
    }
  }
}

// The branches beside the engine's own use of these nodes: float32 weights, batched
// weights, broadcasting / other element types in add, float64 in the router.
static void gpu_variant_branches() {
  std::printf("variants: fp32 / batched matmul, fp32 dense_ffn, broadcasting add, float64 router\n");
  std::mt19937 gen(31);
  auto rel_worst = [](const float* got, const float* want, int64_t n) {
    float worst = 0, scale = 0;
    for (int64_t i = 0; i < n; ++i) {
      worst = std::fmax(worst, std::fabs(got[i] - want[i]));
      scale = std::fmax(scale, std::fabs(want[i]));
    }
    return worst / std::fmax(scale, 1e-6f);
  };
  {  // matmul: every pairing of batch shapes the node accepts, fp16 and fp32 B
    struct shapes { std::vector<int64_t> a, b; };
    for (const shapes& sh : std::vector<shapes>{{{2, 40, 72}, {130, 72}}, {{3, 4, 16}, {3, 5, 16}}, {{4, 16}, {3, 5, 16}},
                                                {{2, 3, 4, 16}, {3, 5, 16}}, {{2, 1, 2, 8}, {1, 3, 3, 8}}, {{7, 37}, {29, 37}},
                                                {{2, 1, 4, 16}, {70, 5, 16}}}) {
      for (bool half : {true, false}) {
        auto a = random_tensor(sh.a, gen, -1, 1);
        auto b = half ? random_half_tensor(sh.b, gen, -0.2f, 0.2f) : random_tensor(sh.b, gen, -0.2f, 0.2f);
        matmul_transpose_mixed_node node;
        auto out = node.compute_test(a, b);
        const int64_t m = a.dim(-2), k = a.dim(-1), n = b.dim(-2);
        const int64_t n_a = a.numel() / (m * k), n_b = b.numel() / (n * k), n_out = out.numel() / (m * n);
        CHECK(out.dim(-2) == m && out.dim(-1) == n && n_out >= std::max(n_a, n_b));
        std::vector<float> want(out.numel());
        orc_matmul_transpose_batched(a.data_ptr<float>(), n_a, b.data_ptr<uint8_t>(), n_b, half, n_out, want.data(), m, k, n);
        CHECK(rel_worst(out.data_ptr<float>(), want.data(), out.numel()) <= (half ? 1e-3f : 2e-5f));
        const size_t uploads = node.resident_uploads();
        CHECK(uploads == (size_t)std::min<int64_t>(n_b, n_out) || n_b > matmul_transpose_mixed_node::kMaxResidentMatrices);
        if (n_b <= matmul_transpose_mixed_node::kMaxResidentMatrices) {
          node.compute_test(a, b);  // the same weight again: no new device copies
          CHECK(node.resident_uploads() == uploads);
        }
      }
    }
  }
  {  // dense_ffn with FLOAT32 weights, and a weight rewritten in place between frames
    const int64_t B = 2, S = 9, H = 72, F = 130;
    auto hidden = random_tensor({B, S, H}, gen, -1, 1);
    auto gate = random_tensor({F, H}, gen, -0.2f, 0.2f), up = random_tensor({F, H}, gen, -0.2f, 0.2f);
    auto down = random_tensor({H, F}, gen, -0.2f, 0.2f);
    auto bg = random_tensor({F}, gen, -0.1f, 0.1f), bu = random_tensor({F}, gen, -0.1f, 0.1f), bd = random_tensor({H}, gen, -0.1f, 0.1f);
    dense_ffn_node node;
    std::vector<float> want(B * S * H);
    for (int round = 0; round < 3; ++round) {
      auto out = node.compute_test({hidden, gate, up, down, bg, bu, bd});
      CHECK(orc_dense_ffn_f32(hidden.data_ptr<float>(), B * S, H, F, gate.data_ptr<float>(), up.data_ptr<float>(),
                              down.data_ptr<float>(), bg.data_ptr<float>(), bu.data_ptr<float>(), bd.data_ptr<float>(),
                              want.data()) == 0);
      CHECK(rel_worst(out.data_ptr<float>(), want.data(), out.numel()) <= 2e-5f);
      CHECK(node.resident_uploads() == (round < 2 ? 3u : 4u));
      if (round == 1) up = random_tensor({F, H}, gen, -0.2f, 0.2f);  // a reloaded weight: new storage, new bytes
    }
  }
  {  // add: broadcasting and the other element types, bit-exact
    add_node add;
    auto x = random_tensor({2, 5, 96}, gen, -2, 2), row = random_tensor({96}, gen, -2, 2), col = random_tensor({5, 1}, gen, -2, 2);
    for (const dynamic_tensor* other : {&row, &col}) {
      auto out = add.compute_test(x, *other);
      CHECK(out.shape() == x.shape());
      std::vector<float> want(x.numel());
      int64_t oshape[8];
      CHECK(orc_add_broadcast(x.data_ptr<float>(), x.shape().data(), 3, other->data_ptr<float>(), other->shape().data(),
                              (int)other->ndim(), 0, want.data(), oshape) == 0);
      CHECK(std::memcmp(out.data_ptr<float>(), want.data(), want.size() * 4) == 0);
    }
    dynamic_tensor i64a(dtype::int64, {3, 1}), i64b(dtype::int64, {1, 4}), f64a(dtype::float64, {2, 3}), f64b(dtype::float64, {3});
    dynamic_tensor i32a(dtype::int32, {4}), i32b(dtype::int32, {1});
    for (int i = 0; i < 3; ++i) i64a.data_ptr<int64_t>()[i] = (int64_t)1 << (40 + i);
    for (int i = 0; i < 4; ++i) i64b.data_ptr<int64_t>()[i] = i - 2, i32a.data_ptr<int32_t>()[i] = (int32_t)(500000000u * (uint32_t)i);
    i32b.data_ptr<int32_t>()[0] = 2000000000;  // wraps for i >= 1, like the reference's int32 sum on this target
    for (int i = 0; i < 6; ++i) f64a.data_ptr<double>()[i] = 1.0 + i * 1e-13;
    for (int i = 0; i < 3; ++i) f64b.data_ptr<double>()[i] = 1e-3 * i;
    auto o64 = add.compute_test(i64a, i64b);
    CHECK((o64.shape() == std::vector<int64_t>{3, 4}) && o64.get_dtype() == dtype::int64);
    for (int i = 0; i < 3; ++i)
      for (int j = 0; j < 4; ++j) CHECK(o64.data_ptr<int64_t>()[i * 4 + j] == ((int64_t)1 << (40 + i)) + j - 2);
    auto o32 = add.compute_test(i32a, i32b);
    for (int i = 0; i < 4; ++i)
      CHECK(o32.data_ptr<int32_t>()[i] == (int32_t)(500000000u * (uint32_t)i + 2000000000u));
    auto od = add.compute_test(f64a, f64b);
    CHECK(od.get_dtype() == dtype::float64);
    for (int i = 0; i < 6; ++i) CHECK(od.data_ptr<double>()[i] == f64a.data_ptr<double>()[i] + f64b.data_ptr<double>()[i % 3]);
    CHECK(add.compute_test(dynamic_tensor(dtype::float32, {2, 0, 3}), dynamic_tensor(dtype::float32, {1, 3})).numel() == 0);
  }
  {  // router on float64 inputs: experts exactly the CPU path's
    const int64_t B = 2, S = 8, H = 128, E = 32, K = 4;
    dynamic_tensor h(dtype::float64, {B, S, H}), g(dtype::float64, {E, H});
    std::uniform_real_distribution<double> d(-1, 1);
    for (int64_t i = 0; i < h.numel(); ++i) h.data_ptr<double>()[i] = d(gen);
    for (int64_t i = 0; i < g.numel(); ++i) g.data_ptr<double>()[i] = 0.2 * d(gen);
    auto b = random_tensor({E}, gen, -0.01f, 0.01f);
    for (bool sigmoid : {false, true}) {
      moe_router_node node;
      node.set_config(E, K);
      node.set_sigmoid_gating(sigmoid);
      auto out = node.compute_test(h, g, b);
      CHECK((out.shape() == std::vector<int64_t>{B, S, K, 2}) && out.get_dtype() == dtype::float32);
      std::vector<float> want(B * S * K * 2);
      CHECK(orc_router_f64(h.data_ptr<double>(), B * S, H, g.data_ptr<double>(), E, b.data_ptr<float>(), K, sigmoid,
                           want.data(), nullptr) == 0);
      for (int64_t p = 0; p < B * S * K; ++p)
        CHECK(out.data_ptr<float>()[2 * p] == want[2 * p] && std::fabs(out.data_ptr<float>()[2 * p + 1] - want[2 * p + 1]) < 1e-6f);
    }
  }
}

// router -> E expert nodes -> merge, wired with edges and result messages the way
// llm_engine builds the block (src/llm/llm_engine.cpp:721-753), against the CPU checker.
static void gpu_node_chain() {
  std::printf("router -> experts -> merge through result messages\n");
  std::mt19937 gen(7);
  const int64_t E = 6, K = 2, H = 64, F = 96, B = 1, S = 9, T = B * S;
  auto hidden = random_tensor({B, S, H}, gen, -1, 1);
  auto gate = random_tensor({E, H}, gen, -0.3f, 0.3f);
  auto gate_b = random_tensor({E}, gen, -0.01f, 0.01f);
  std::vector<dynamic_mx_tensor> wu, wg, wd;
  std::vector<dynamic_tensor> bu, bg, bd;
  for (int e = 0; e < E; ++e) {
    wu.push_back(random_mx(F, H, gen));
    wg.push_back(random_mx(F, H, gen));
    wd.push_back(random_mx(H, F, gen));
    bu.push_back(random_tensor({F}, gen, -0.01f, 0.01f));
    bg.push_back(random_tensor({F}, gen, -0.01f, 0.01f));
    bd.push_back(random_tensor({H}, gen, -0.01f, 0.01f));
  }
  moe_router_node router;
  router.set_config(E, K);
  router.set_input_names({"hidden", "gate_w", "gate_b"});
  router.set_output_name("router_out");
  capture_node rcap;
  rcap.set_input(router.get_output());
  auto mk = [](const dynamic_tensor& t) { return std::make_shared<dynamic_tensor_message>(t); };
  router.process("default", result_message::ok({{"hidden", mk(hidden)}, {"gate_w", mk(gate)}, {"gate_b", mk(gate_b)}}));
  CHECK(rcap.got.size() == 1 && rcap.got[0]->is_ok());
  auto router_out = std::dynamic_pointer_cast<dynamic_tensor_message>(rcap.got[0]->get_field("router_out"));
  CHECK(router_out && (router_out->get_tensor().shape() == std::vector<int64_t>{B, S, K, 2}));
  const float* pairs = router_out->get_tensor().data_ptr<float>();

  std::vector<dynamic_tensor> merge_inputs{router_out->get_tensor()};
  std::vector<std::vector<float>> want_outs(E);
  std::vector<const float*> want_ptrs(E, nullptr);
  int n_empty = 0;
  for (int e = 0; e < E; ++e) {
    expert_mlp_node node(e);
    node.set_input_names({"hidden", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "router"});
    node.set_output_name("out");
    capture_node cap;
    cap.set_input(node.get_output());
    auto msg = result_message::ok({{"hidden", mk(hidden)},
                                   {"w_up", std::make_shared<dynamic_mx_tensor_message>(wu[e])},
                                   {"w_gate", std::make_shared<dynamic_mx_tensor_message>(wg[e])},
                                   {"w_down", std::make_shared<dynamic_mx_tensor_message>(wd[e])},
                                   {"b_up", mk(bu[e])}, {"b_gate", mk(bg[e])}, {"b_down", mk(bd[e])},
                                   {"router", router_out}});
    node.process("default", msg);
    node.process("default", msg);  // second frame: weights are already resident
    CHECK(cap.got.size() == 2 && cap.got[0]->is_ok() && cap.got[1]->is_ok());
    auto out = std::dynamic_pointer_cast<dynamic_tensor_message>(cap.got[1]->get_field("out"))->get_tensor();
    want_outs[e].resize(T * H);
    int empty = 0;
    orc_expert_mlp_mxfp4(e, hidden.data_ptr<float>(), T, H, F, wu[e].data_ptr(), wg[e].data_ptr(), wd[e].data_ptr(),
                         bu[e].data_ptr<float>(), bg[e].data_ptr<float>(), bd[e].data_ptr<float>(), pairs, K, 0, 0,
                         want_outs[e].data(), &empty);
    if (empty) {
      ++n_empty;
      CHECK(out.ndim() == 1 && out.dim(0) == 0);
    } else {
      CHECK((out.shape() == std::vector<int64_t>{B, S, H}));
      want_ptrs[e] = want_outs[e].data();
      float worst = 0;
      for (int64_t i = 0; i < T * H; ++i)
        worst = std::fmax(worst, std::fabs(out.data_ptr<float>()[i] - want_outs[e][i]) / std::fmax(1.0f, std::fabs(want_outs[e][i])));
      CHECK(worst <= 1e-3f);
    }
    merge_inputs.push_back(out);
  }
  std::printf("  %d of %d experts unselected\n", n_empty, (int)E);
  expert_merge_node merge;
  merge.set_config(E, K);
  auto merged = merge.compute_test(merge_inputs);
  std::vector<float> want(T * H);
  CHECK(orc_expert_merge(pairs, T, K, E, H, want_ptrs.data(), 0, want.data()) == 0);
  float worst = 0;
  for (int64_t i = 0; i < T * H; ++i)
    worst = std::fmax(worst, std::fabs(merged.data_ptr<float>()[i] - want[i]) / std::fmax(1.0f, std::fabs(want[i])));
  std::printf("  merged layer output: max rel err %.3g\n", worst);
  CHECK(worst <= 1e-3f);
}

// The provider behind the expert nodes is an LRU (src/llm/moe_weight_provider.cpp:102-132): a
// slice that was evicted comes back in new storage, possibly at an address another matrix of
// the same shape used before.  The node's device copies must follow: same storage and bytes
// -> reused; new storage, rewritten bytes or tensors that changed roles -> uploaded again,
// never a stale copy, never more than three device matrices.
static void gpu_expert_weight_reload() {
  std::printf("expert node: device copies follow reloaded / rewritten / swapped host weights\n");
  std::mt19937 gen(99);
  const int64_t H = 64, F = 64, S = 5, K = 1;  // H == F: all three matrices have the same shape
  auto hidden = random_tensor({1, S, H}, gen, -1, 1);
  dynamic_tensor router(dtype::float32, {1, S, K, 2});
  for (int64_t t = 0; t < S; ++t) router.data_ptr<float>()[2 * t] = 0.0f, router.data_ptr<float>()[2 * t + 1] = 1.0f;
  auto mk = [](const dynamic_tensor& t) { return std::make_shared<dynamic_tensor_message>(t); };
  expert_mlp_node node(0);
  node.set_input_names({"hidden", "w_up", "w_gate", "w_down", "router"});
  node.set_output_name("out");
  capture_node cap;
  cap.set_input(node.get_output());
  auto run_and_check = [&](const dynamic_mx_tensor& up, const dynamic_mx_tensor& gate, const dynamic_mx_tensor& down) {
    node.process("default", result_message::ok({{"hidden", mk(hidden)},
                                                {"w_up", std::make_shared<dynamic_mx_tensor_message>(up)},
                                                {"w_gate", std::make_shared<dynamic_mx_tensor_message>(gate)},
                                                {"w_down", std::make_shared<dynamic_mx_tensor_message>(down)},
                                                {"router", mk(router)}}));
    CHECK(!cap.got.empty() && cap.got.back()->is_ok());
    if (cap.got.empty() || !cap.got.back()->is_ok()) return;
    auto out = std::dynamic_pointer_cast<dynamic_tensor_message>(cap.got.back()->get_field("out"))->get_tensor();
    std::vector<float> want(S * H);
    int empty = 0;
    orc_expert_mlp_mxfp4(0, hidden.data_ptr<float>(), S, H, F, up.data_ptr(), gate.data_ptr(), down.data_ptr(),
                         nullptr, nullptr, nullptr, router.data_ptr<float>(), K, 0, 0, want.data(), &empty);
    float worst = 0, scale = 0;
    for (int64_t i = 0; i < S * H; ++i) {
      worst = std::fmax(worst, std::fabs(out.data_ptr<float>()[i] - want[i]));
      scale = std::fmax(scale, std::fabs(want[i]));
    }
    CHECK(worst <= 1e-3f * std::fmax(scale, 1e-6f));
  };
  {
    auto up = random_mx(F, H, gen), gate = random_mx(F, H, gen), down = random_mx(H, F, gen);
    run_and_check(up, gate, down);
    CHECK(node.resident_uploads() == 3);
    run_and_check(up, gate, down);  // same storage, same bytes: nothing is uploaded
    CHECK(node.resident_uploads() == 3);
    run_and_check(gate, up, down);  // the same two buffers in each other's role
    CHECK(node.resident_uploads() == 5);
    std::uniform_int_distribution<int> byte(0, 255);
    for (size_t b = 0; b < up.num_blocks(); ++b)  // rewritten in place
      for (int j = 1; j < 17; ++j) up.data_ptr()[17 * b + j] = (uint8_t)byte(gen);
    run_and_check(gate, up, down);
    CHECK(node.resident_uploads() == 6);
    // one byte flipped in place, at an offset the sampled stamp does not look at: the default
    // (every byte hashed) sees it and uploads again ...
    const size_t n = down.size_bytes(), step = (n - 8) / 63;
    const size_t off = step + 9;  // between the second and the third sample
    CHECK(step > 24 && off + 1 < 2 * step);
    down.data_ptr()[off] ^= 0x10;
    run_and_check(gate, up, down);
    CHECK(node.resident_uploads() == 7);
    // ... the sampled stamp, which a host may choose when its weights are never rewritten in
    // place, does not: that is its stated contract (the result is that of the old bytes)
    csk_resident::set_content_check(csk_resident::content_check::sampled);
    run_and_check(gate, up, down);  // the policy changed, so the stamps differ: three uploads
    CHECK(node.resident_uploads() == 10);
    down.data_ptr()[off] ^= 0x10;
    const size_t before = node.resident_uploads();
    node.process("default", result_message::ok({{"hidden", mk(hidden)},
                                                {"w_up", std::make_shared<dynamic_mx_tensor_message>(gate)},
                                                {"w_gate", std::make_shared<dynamic_mx_tensor_message>(up)},
                                                {"w_down", std::make_shared<dynamic_mx_tensor_message>(down)},
                                                {"router", mk(router)}}));
    CHECK(node.resident_uploads() == before);
    down.data_ptr()[0] ^= 0x01;  // a sampled byte: noticed in either mode
    run_and_check(gate, up, down);
    CHECK(node.resident_uploads() == before + 1);
    csk_resident::set_content_check(csk_resident::content_check::full);
    run_and_check(gate, up, down);
    CHECK(node.resident_uploads() == before + 4);
  }  // the caller's references go away (an eviction); the node still holds the storage of its copies
  const size_t base_uploads = node.resident_uploads();
  for (int round = 0; round < 3; ++round) {  // reloads: fresh storage each time, wherever malloc puts it
    auto up = random_mx(F, H, gen), gate = random_mx(F, H, gen), down = random_mx(H, F, gen);
    run_and_check(up, gate, down);
    CHECK(node.resident_uploads() == base_uploads + 3 * (size_t)(round + 1));
  }
}

// One MoE block wired as the engine wires it (llm_engine.cpp:721-753): router node, one
// expert node per expert, merge node.  From the second frame on the block runs as one fused
// forward behind the nodes; the nodes' outputs stay what the reference's nodes emit, the
// merged result equals csk_moe_forward_host bit for bit, and anything that cannot be proved
// -- a weight rewritten in place, an expert not yet attached, an expert output that did not
// come from the frame -- takes the per-node path and is right all the same.
static void gpu_block_frames() {
  std::printf("block: router + experts + merge share frames; reloads and mixed paths\n");
  std::mt19937 gen(4242);
  const int64_t E = 8, K = 2, H = 96, F = 160;
  auto gate = random_tensor({E, H}, gen, -0.3f, 0.3f), gate_b = random_tensor({E}, gen, -0.05f, 0.05f);
  std::vector<dynamic_mx_tensor> wu, wg, wd;
  std::vector<dynamic_tensor> bu, bg, bd;
  for (int64_t e = 0; e < E; ++e) {
    wu.push_back(random_mx(F, H, gen)), wg.push_back(random_mx(F, H, gen)), wd.push_back(random_mx(H, F, gen));
    bu.push_back(random_tensor({F}, gen, -0.01f, 0.01f)), bg.push_back(random_tensor({F}, gen, -0.01f, 0.01f));
    bd.push_back(random_tensor({H}, gen, -0.01f, 0.01f));
  }
  auto mk = [](const dynamic_tensor& t) { return std::make_shared<dynamic_tensor_message>(t); };
  auto mx = [](const dynamic_mx_tensor& t) { return std::make_shared<dynamic_mx_tensor_message>(t); };
  moe_router_node router;
  router.set_config(E, K);
  router.set_input_names({"hidden", "gate_w", "gate_b"});
  router.set_output_name("router_out");
  capture_node rcap;
  rcap.set_input(router.get_output());
  std::vector<std::unique_ptr<expert_mlp_node>> experts;
  std::vector<std::unique_ptr<capture_node>> ecaps;
  for (int64_t e = 0; e < E; ++e) {
    experts.emplace_back(new expert_mlp_node((int)e));
    experts.back()->set_input_names({"hidden", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "router"});
    experts.back()->set_output_name("out");
    ecaps.emplace_back(new capture_node);
    ecaps.back()->set_input(experts.back()->get_output());
  }
  expert_merge_node merge;
  merge.set_config(E, K);

  struct frame_result {
    dynamic_tensor merged, router_out;
    std::vector<dynamic_tensor> outs;
    int active = 0;
  };
  // `foreign`: hand the merge node a copy of one live expert output instead of the tensor the node emitted
  auto run_frame = [&](const dynamic_tensor& hidden, bool foreign = false) {
    frame_result r;
    auto hm = mk(hidden);
    router.process("default", result_message::ok({{"hidden", hm}, {"gate_w", mk(gate)}, {"gate_b", mk(gate_b)}}));
    auto rm = std::dynamic_pointer_cast<dynamic_tensor_message>(rcap.got.back()->get_field("router_out"));
    r.router_out = rm->get_tensor();
    std::vector<dynamic_tensor> merge_in{r.router_out};
    for (int64_t e = 0; e < E; ++e) {
      experts[e]->process("default", result_message::ok({{"hidden", hm}, {"w_up", mx(wu[e])}, {"w_gate", mx(wg[e])},
                                                         {"w_down", mx(wd[e])}, {"b_up", mk(bu[e])},
                                                         {"b_gate", mk(bg[e])}, {"b_down", mk(bd[e])}, {"router", rm}}));
      CHECK(ecaps[e]->got.back()->is_ok());
      auto t = std::dynamic_pointer_cast<dynamic_tensor_message>(ecaps[e]->got.back()->get_field("out"))->get_tensor();
      r.active += t.numel() != 0;
      if (foreign && t.numel() != 0) {
        dynamic_tensor copy(dtype::float32, t.shape());
        std::memcpy(copy.data_ptr<float>(), t.data_ptr<float>(), t.bytes());
        t = copy;
        foreign = false;
      }
      merge_in.push_back(t);
      r.outs.push_back(t);
    }
    r.merged = merge.compute_test(merge_in);
    return r;
  };
  // the same block as an ordinary resident layer: what csk_moe_forward_host gives
  auto fused = [&](const dynamic_tensor& hidden) {
    csk_layer* L = nullptr;
    CHECK(csk_layer_create(E, K, H, F, &L) == CSK_OK);
    CHECK(csk_layer_set_router(L, gate.data_ptr<float>(), gate_b.data_ptr<float>()) == CSK_OK);
    for (int64_t e = 0; e < E; ++e)
      CHECK(csk_layer_set_expert(L, e, wu[e].data_ptr(), wg[e].data_ptr(), wd[e].data_ptr(), bu[e].data_ptr<float>(),
                                 bg[e].data_ptr<float>(), bd[e].data_ptr<float>()) == CSK_OK);
    dynamic_tensor out(dtype::float32, hidden.shape());
    CHECK(csk_moe_forward_host(L, hidden.data_ptr<float>(), hidden.dim(0) * hidden.dim(1), out.data_ptr<float>(),
                               nullptr, 0) == CSK_OK);
    csk_layer_destroy(L);
    return out;
  };
  auto same_bits = [](const dynamic_tensor& a, const dynamic_tensor& b) {
    return a.shape() == b.shape() && std::memcmp(a.data_ptr<float>(), b.data_ptr<float>(), a.bytes()) == 0;
  };
  auto close = [](const dynamic_tensor& a, const dynamic_tensor& b) {
    if (a.shape() != b.shape()) return false;
    float worst = 0, scale = 0;
    for (int64_t i = 0; i < a.numel(); ++i) {
      worst = std::fmax(worst, std::fabs(a.data_ptr<float>()[i] - b.data_ptr<float>()[i]));
      scale = std::fmax(scale, std::fabs(b.data_ptr<float>()[i]));
    }
    return worst <= 1e-5f * std::fmax(scale, 1e-6f);
  };
  auto rows_from_frames = [&] {
    size_t n = 0;
    for (auto& x : experts) n += x->rows_from_frames();
    return n;
  };

  // all 8 experts of a 24-token batch are selected: frame 1 is computed node by node and attaches them
  auto hidden = random_tensor({1, 24, H}, gen, -1, 1);
  auto f1 = run_frame(hidden);
  CHECK(f1.active == E);
  CHECK(router.frames_begun() == 0 && rows_from_frames() == 0 && merge.merges_from_frames() == 0);
  auto want = fused(hidden);
  CHECK(close(f1.merged, want));
  // frame 2: one fused forward behind the nodes
  auto f2 = run_frame(hidden);
  CHECK(router.frames_begun() == 1 && router.frames_with_experts() == 1);
  CHECK(rows_from_frames() == (size_t)E && merge.merges_from_frames() == 1);
  CHECK(same_bits(f2.merged, want));
  CHECK(same_bits(f2.router_out, f1.router_out) || close(f2.router_out, f1.router_out));
  for (int64_t e = 0; e < E; ++e) CHECK(close(f2.outs[e], f1.outs[e]));  // each node still emits its own dense rows
  // other tokens, fewer of them: some experts may stay unselected ({0}-shaped outputs, as ever)
  auto hidden3 = random_tensor({1, 3, H}, gen, -1, 1);
  auto f3 = run_frame(hidden3);
  CHECK(f3.active <= 6 && merge.merges_from_frames() == 2);
  CHECK(same_bits(f3.merged, fused(hidden3)));
  for (int64_t e = 0; e < E; ++e) CHECK((f3.outs[e].numel() == 0) == (f3.outs[e].ndim() == 1));
  // an expert output that did not come from the frame: the merge node computes on what it was given
  auto f4 = run_frame(hidden, true);
  CHECK(merge.merges_from_frames() == 2 && close(f4.merged, want));
  // a weight rewritten in place between two frames: that node uploads and computes itself, the
  // frame's merged rows are void, everything follows the new bytes; the next frame is fused again
  std::uniform_int_distribution<int> byte(0, 255);
  for (size_t b = 0; b < wu[3].num_blocks(); ++b)
    for (int j = 1; j < 17; ++j) wu[3].data_ptr()[17 * b + j] = (uint8_t)byte(gen);
  const size_t before_rows = rows_from_frames(), before_up = experts[3]->resident_uploads();
  auto f5 = run_frame(hidden);
  auto want5 = fused(hidden);
  CHECK(experts[3]->resident_uploads() == before_up + 1 && merge.merges_from_frames() == 2);
  CHECK(rows_from_frames() < before_rows + (size_t)E);
  CHECK(close(f5.merged, want5) && !close(f5.merged, want));
  auto f6 = run_frame(hidden);
  CHECK(merge.merges_from_frames() == 3 && same_bits(f6.merged, want5));
  // a bias replaced by another tensor: same story
  bd[5] = random_tensor({H}, gen, -0.02f, 0.02f);
  auto f7 = run_frame(hidden);
  auto want7 = fused(hidden);
  CHECK(merge.merges_from_frames() == 3 && close(f7.merged, want7));
  auto f8 = run_frame(hidden);
  CHECK(merge.merges_from_frames() == 4 && same_bits(f8.merged, want7));
  // the router's gate rewritten in place: the view layer's copy follows it
  for (int64_t i = 0; i < gate.numel(); ++i) gate.data_ptr<float>()[i] = -gate.data_ptr<float>()[i];
  auto f9 = run_frame(hidden);
  CHECK(merge.merges_from_frames() == 5 && same_bits(f9.merged, fused(hidden)));
  // an expert node goes away while attached: the block falls back to the per-node path for its experts
  experts[2].reset(new expert_mlp_node(2));
  experts[2]->set_input_names({"hidden", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "router"});
  experts[2]->set_output_name("out");
  ecaps[2]->got.clear();
  ecaps[2]->set_input(experts[2]->get_output());
  auto f10 = run_frame(hidden);
  CHECK(merge.merges_from_frames() == 5 && close(f10.merged, fused(hidden)));
  auto f11 = run_frame(hidden);
  CHECK(merge.merges_from_frames() == 6 && same_bits(f11.merged, fused(hidden)));
}

// The router node is handed the same gate tensors every frame and keeps them in device
// memory: same storage and bytes -> no upload; rewritten in place or reloaded elsewhere ->
// a new copy, and the result is that of the new gate.
static void gpu_router_gate_reload() {
  std::printf("router node: device copy of the gate follows rewritten / reloaded host tensors\n");
  std::mt19937 gen(7);
  const int64_t S = 6, H = 64, E = 16, K = 2;
  moe_router_node node;
  node.set_config(E, K);
  auto h = random_tensor({1, S, H}, gen, -1, 1);
  auto check = [&](const dynamic_tensor& g, const dynamic_tensor& b) {
    auto out = node.compute_test(h, g, b);
    std::vector<float> want(S * K * 2);
    orc_router(h.data_ptr<float>(), S, H, g.data_ptr<float>(), E, b.data_ptr<float>(), K, 0, want.data());
    for (int64_t i = 0; i < S * K; ++i) {
      CHECK(out.data_ptr<float>()[2 * i] == want[2 * i]);
      CHECK(std::fabs(out.data_ptr<float>()[2 * i + 1] - want[2 * i + 1]) <= 1e-5f);
    }
  };
  auto g = random_tensor({E, H}, gen, -0.5f, 0.5f), b = random_tensor({E}, gen, -0.1f, 0.1f);
  check(g, b);
  CHECK(node.resident_uploads() == 2);
  check(g, b);  // same storage, same bytes
  CHECK(node.resident_uploads() == 2);
  for (int64_t i = 0; i < E * H; ++i) g.data_ptr<float>()[i] = -g.data_ptr<float>()[i];  // rewritten in place
  check(g, b);
  CHECK(node.resident_uploads() == 3);
  b.data_ptr<float>()[E - 1] += 5.0f;  // the last expert now wins every token
  check(g, b);
  CHECK(node.resident_uploads() == 4);
  auto g2 = random_tensor({E, H}, gen, -0.5f, 0.5f);  // a reload: other storage
  check(g2, b);
  CHECK(node.resident_uploads() == 5);
}

// Nodes of different layers may be driven from different threads (the reference runs each
// layer's nodes on that layer's scheduler thread, layer_scheduler_node); the library
// serialises the calls, so results must equal those of the same calls made one after another.
static void gpu_concurrent_callers() {
  std::printf("concurrent callers: four threads, each with its own nodes\n");
  constexpr int kThreads = 4, kRounds = 6;
  struct Job {
    dynamic_tensor a, w, hidden, gate, up, down, want_mm, want_ffn;
    int bad = 0;
  };
  std::vector<Job> jobs(kThreads);
  std::mt19937 gen(77);
  for (int i = 0; i < kThreads; ++i) {
    Job& j = jobs[i];
    const int64_t S = 5 + 9 * i, K = 64 + 32 * i, N = 96 + 16 * i;
    j.a = random_tensor({1, S, K}, gen, -1, 1);
    j.w = random_half_tensor({N, K}, gen, -0.2f, 0.2f);
    j.hidden = random_tensor({1, S, K}, gen, -1, 1);
    j.gate = random_half_tensor({N, K}, gen, -0.2f, 0.2f);
    j.up = random_half_tensor({N, K}, gen, -0.2f, 0.2f);
    j.down = random_half_tensor({K, N}, gen, -0.2f, 0.2f);
    matmul_transpose_mixed_node mm;
    dense_ffn_node ffn;
    j.want_mm = mm.compute_test(j.a, j.w);
    j.want_ffn = ffn.compute_test({j.hidden, j.gate, j.up, j.down});
  }
  auto same = [](const dynamic_tensor& x, const dynamic_tensor& y) {
    return x.shape() == y.shape() &&
           std::memcmp(x.data_ptr<float>(), y.data_ptr<float>(), x.numel() * sizeof(float)) == 0;
  };
  std::vector<std::thread> pool;
  for (int i = 0; i < kThreads; ++i)
    pool.emplace_back([&, i] {
      Job& j = jobs[i];
      matmul_transpose_mixed_node mm;
      dense_ffn_node ffn;
      for (int r = 0; r < kRounds; ++r) {
        try {
          if (!same(mm.compute_test(j.a, j.w), j.want_mm)) ++j.bad;
          if (!same(ffn.compute_test({j.hidden, j.gate, j.up, j.down}), j.want_ffn)) ++j.bad;
        } catch (const std::exception& e) {
          std::printf("  thread %d: %s\n", i, e.what());
          ++j.bad;
        }
      }
    });
  for (auto& t : pool) t.join();
  for (int i = 0; i < kThreads; ++i) CHECK(jobs[i].bad == 0);
}

int main(int argc, char** argv) {
  const bool gpu = argc > 1 && std::string(argv[1]) == "--gpu";
  if (gpu) {
    if (csk_init(0) != CSK_OK) {
      std::printf("csk_init failed: %s\n", csk_last_error());
      return 2;
    }
    gpu_router_tests();
    gpu_expert_known_answer();
    gpu_expert_fp16_tests();
    gpu_dense_ffn_tests();
    gpu_matmul_tests();
    gpu_variant_branches();
    gpu_node_chain();
    gpu_expert_weight_reload();
    gpu_block_frames();
    gpu_router_gate_reload();
    gpu_norm_add_tests();
    gpu_concurrent_callers();
  } else {
    cpu_router_argument_errors();
    cpu_expert_node_paths();
    cpu_expert_fp16_argument_errors();
    cpu_dense_ffn_argument_errors();
    cpu_matmul_argument_errors();
    cpu_merge_argument_errors();
    cpu_norm_add_argument_errors();
  }
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  return g_failed ? 1 : 0;
}
