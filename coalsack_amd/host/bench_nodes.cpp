// Times one MoE block driven the way the engine drives it -- moe_router_node, one
// expert_mlp_node per expert, expert_merge_node, wired by result messages
// (src/llm/llm_engine.cpp:721-753) -- against the same block as one fused call
// (csk_moe_forward_host) on the same weights and inputs, and checks that both give the same
// output bit for bit.  Host wall clock per frame, weights resident, activations in host
// memory on both paths (that is what the nodes are handed).  From the second frame on the
// nodes share frames (moe_block_context.h): the router node starts the fused forward, the
// expert nodes prove their tensors unchanged and copy their rows out, the merge node takes
// the merged rows.  Both content checks of resident_weight.h are timed: `full` hashes every
// weight byte every frame (exact whatever the host does to its tensors), `sampled` is the
// contract for hosts that never rewrite a weight tensor in place.
//   bench_nodes [E] [top_k] [H] [F] [frames]      default: 32 4 2880 2880 20  (the 20b block)
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <vector>

#include "coalsack/nn/nn_ops/expert_merge_node.h"
#include "coalsack/nn/nn_ops/expert_mlp_node.h"
#include "coalsack/nn/nn_ops/moe_router_node.h"

using namespace coalsack;

struct capture_node : graph_node {
  std::shared_ptr<result_message> last;
  std::string get_proc_name() const override { return "capture"; }
  void process(std::string, graph_message_ptr m) override { last = std::dynamic_pointer_cast<result_message>(m); }
};

static dynamic_mx_tensor random_mx(int64_t rows, int64_t cols, std::mt19937_64& gen) {
  dynamic_mx_tensor t({rows, cols});
  uint8_t* p = t.data_ptr();
  const size_t n = t.num_blocks();
  for (size_t b = 0; b < n; ++b) {
    const uint64_t r0 = gen(), r1 = gen(), r2 = gen();
    p[17 * b] = (uint8_t)(118 + r0 % 4);
    std::memcpy(p + 17 * b + 1, &r1, 8);
    std::memcpy(p + 17 * b + 9, &r2, 8);
  }
  return t;
}

int main(int argc, char** argv) {
  const int64_t E = argc > 1 ? atoll(argv[1]) : 32, K = argc > 2 ? atoll(argv[2]) : 4;
  const int64_t H = argc > 3 ? atoll(argv[3]) : 2880, F = argc > 4 ? atoll(argv[4]) : 2880;
  const int frames = argc > 5 ? atoi(argv[5]) : 20;
  if (csk_init(0) != CSK_OK) {
    std::printf("csk_init failed: %s\n", csk_last_error());
    return 2;
  }
  std::mt19937_64 gen(2024);
  std::uniform_real_distribution<float> uni(-1, 1);
  dynamic_tensor gate(dtype::float32, {E, H}), gate_b(dtype::float32, {E});
  for (int64_t i = 0; i < gate.numel(); ++i) gate.data_ptr<float>()[i] = 0.05f * uni(gen);
  for (int64_t i = 0; i < E; ++i) gate_b.data_ptr<float>()[i] = 0.01f * uni(gen);
  std::vector<dynamic_mx_tensor> wu, wg, wd;
  std::vector<dynamic_tensor> bu, bg, bd;
  csk_layer* layer = nullptr;
  if (csk_layer_create(E, K, H, F, &layer) != CSK_OK || csk_layer_set_router(layer, gate.data_ptr<float>(), gate_b.data_ptr<float>()) != CSK_OK) {
    std::printf("layer: %s\n", csk_last_error());
    return 2;
  }
  for (int64_t e = 0; e < E; ++e) {
    wu.push_back(random_mx(F, H, gen));
    wg.push_back(random_mx(F, H, gen));
    wd.push_back(random_mx(H, F, gen));
    for (auto* v : {&bu, &bg}) {
      v->emplace_back(dtype::float32, std::vector<int64_t>{F});
      for (int64_t i = 0; i < F; ++i) v->back().data_ptr<float>()[i] = 0.01f * uni(gen);
    }
    bd.emplace_back(dtype::float32, std::vector<int64_t>{H});
    for (int64_t i = 0; i < H; ++i) bd.back().data_ptr<float>()[i] = 0.01f * uni(gen);
    if (csk_layer_set_expert(layer, e, wu[e].data_ptr(), wg[e].data_ptr(), wd[e].data_ptr(), bu[e].data_ptr<float>(),
                             bg[e].data_ptr<float>(), bd[e].data_ptr<float>()) != CSK_OK) {
      std::printf("set_expert: %s\n", csk_last_error());
      return 2;
    }
  }
  // the graph: one router, E experts, one merge, kept across frames like the engine's
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
  auto mk = [](const dynamic_tensor& t) { return std::make_shared<dynamic_tensor_message>(t); };
  std::vector<std::shared_ptr<dynamic_mx_tensor_message>> mu, mg, md;
  std::vector<std::shared_ptr<dynamic_tensor_message>> mbu, mbg, mbd;
  for (int64_t e = 0; e < E; ++e) {
    mu.push_back(std::make_shared<dynamic_mx_tensor_message>(wu[e]));
    mg.push_back(std::make_shared<dynamic_mx_tensor_message>(wg[e]));
    md.push_back(std::make_shared<dynamic_mx_tensor_message>(wd[e]));
    mbu.push_back(mk(bu[e])), mbg.push_back(mk(bg[e])), mbd.push_back(mk(bd[e]));
  }
  auto gate_m = mk(gate), gate_b_m = mk(gate_b);

  std::printf("E=%lld top_k=%lld H=%lld F=%lld, %d timed frames after 3 warm-up frames\n", (long long)E, (long long)K,
              (long long)H, (long long)F, frames);
  for (auto policy : {csk_resident::content_check::full, csk_resident::content_check::sampled}) {
  csk_resident::set_content_check(policy);
  std::printf("content check: %s\n", policy == csk_resident::content_check::full ? "full (every byte hashed per frame)"
                                                                                 : "sampled");
  for (int64_t T : {1, 16, 256}) {
    dynamic_tensor hidden(dtype::float32, {1, T, H});
    for (int64_t i = 0; i < hidden.numel(); ++i) hidden.data_ptr<float>()[i] = uni(gen);
    auto hidden_m = mk(hidden);
    dynamic_tensor merged;
    double t_router = 0, t_experts = 0, t_merge = 0;
    int active = 0;
    auto frame = [&](bool timed) {
      using clk = std::chrono::steady_clock;
      const auto t0 = clk::now();
      router.process("default", result_message::ok({{"hidden", hidden_m}, {"gate_w", gate_m}, {"gate_b", gate_b_m}}));
      auto router_out = std::dynamic_pointer_cast<dynamic_tensor_message>(rcap.last->get_field("router_out"));
      const auto t1 = clk::now();
      std::vector<dynamic_tensor> merge_in{router_out->get_tensor()};
      active = 0;
      for (int64_t e = 0; e < E; ++e) {
        experts[e]->process("default", result_message::ok({{"hidden", hidden_m}, {"w_up", mu[e]}, {"w_gate", mg[e]},
                                                           {"w_down", md[e]}, {"b_up", mbu[e]}, {"b_gate", mbg[e]},
                                                           {"b_down", mbd[e]}, {"router", router_out}}));
        merge_in.push_back(std::dynamic_pointer_cast<dynamic_tensor_message>(ecaps[e]->last->get_field("out"))->get_tensor());
        active += merge_in.back().numel() != 0;
      }
      const auto t2 = clk::now();
      merged = merge.compute_test(merge_in);
      const auto t3 = clk::now();
      if (timed) {
        t_router += std::chrono::duration<double, std::micro>(t1 - t0).count();
        t_experts += std::chrono::duration<double, std::micro>(t2 - t1).count();
        t_merge += std::chrono::duration<double, std::micro>(t3 - t2).count();
      }
    };
    const size_t fused_before = merge.merges_from_frames();
    for (int i = 0; i < 3; ++i) frame(false);
    for (int i = 0; i < frames; ++i) frame(true);
    const size_t from_frames = merge.merges_from_frames() - fused_before;
    std::vector<float> fused((size_t)T * H);
    double t_fused = 0;
    for (int i = 0; i < 3 + frames; ++i) {
      const auto t0 = std::chrono::steady_clock::now();
      if (csk_moe_forward_host(layer, hidden.data_ptr<float>(), T, fused.data(), nullptr, 0) != CSK_OK) {
        std::printf("forward: %s\n", csk_last_error());
        return 2;
      }
      if (i >= 3) t_fused += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    }
    const bool same = std::memcmp(fused.data(), merged.data_ptr<float>(), fused.size() * sizeof(float)) == 0;
    std::printf("T=%-4lld node chain %9.1f us/frame (router %.1f, %d of %lld experts active %.1f, merge %.1f; %zu of %d "
                "frames fused)   fused call %8.1f us   ratio %.1fx   %s\n",
                (long long)T, (t_router + t_experts + t_merge) / frames, t_router / frames, active, (long long)E,
                t_experts / frames, t_merge / frames, from_frames, 3 + frames, t_fused / frames,
                (t_router + t_experts + t_merge) / t_fused, same ? "bit-identical" : "DIFFERENT");
    if (!same) return 1;
  }
  }
  csk_layer_destroy(layer);
  return 0;
}
