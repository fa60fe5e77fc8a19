// expert_merge_node backed by the gfx950 library: same class name, setters,
// test wrapper, input order and error texts as
// include/coalsack/nn/nn_ops/expert_merge_node.h of the reference (cited by
// line below); the weighted sum runs in csk_expert_merge -- or, when the inputs are exactly
// what the expert nodes of a frame emitted (moe_block_context.h), is the frame's own merged
// rows, which are on the device already.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack/nn/nn_ops/moe_block_context.h"
#include "coalsack_moe.h"

namespace coalsack {

// inputs[0]: router output [batch, seq_len, top_k, 2]; inputs[1..E]: expert
// outputs [batch, seq_len, hidden_dim] or {0}-shaped for experts no token chose.
class expert_merge_node : public variadic_op_node {
 public:
  expert_merge_node() : variadic_op_node("expert_merge", 33) {}

  void set_config(int64_t num_experts, int64_t top_k) {  // :17-20
    num_experts_ = num_experts;
    top_k_ = top_k;
  }
  void set_weight_before_ffn(bool v) { weight_before_ffn_ = v; }  // :24
  dynamic_tensor compute_test(const std::vector<dynamic_tensor>& inputs) { return compute(inputs); }  // :27

 protected:
  dynamic_tensor compute(const std::vector<dynamic_tensor>& inputs) override {  // :30-134
    if (inputs.size() != static_cast<size_t>(num_experts_ + 1))
      throw std::runtime_error("expert_merge: expected " + std::to_string(num_experts_ + 1) +
                               " inputs, got " + std::to_string(inputs.size()));
    const dynamic_tensor& router = inputs[0];
    if (router.ndim() != 4 || router.dim(2) != top_k_ || router.dim(3) != 2)
      throw std::runtime_error("expert_merge: router output must have shape [batch, seq_len, " +
                               std::to_string(top_k_) + ", 2]");
    const int64_t batch = router.dim(0), seq_len = router.dim(1);
    auto is_live = [](const dynamic_tensor& t) { return t.ndim() == 3 && t.dim(0) > 0; };
    int64_t hidden_dim = 0;
    for (int64_t i = 1; i <= num_experts_ && hidden_dim == 0; ++i)
      if (is_live(inputs[(size_t)i])) hidden_dim = inputs[(size_t)i].dim(2);
    if (hidden_dim == 0) throw std::runtime_error("expert_merge: no non-empty expert outputs found");
    std::vector<const float*> outs((size_t)num_experts_, nullptr);
    for (int64_t i = 1; i <= num_experts_; ++i) {
      const dynamic_tensor& t = inputs[(size_t)i];
      if (!is_live(t)) continue;
      if (t.dim(0) != batch || t.dim(1) != seq_len || t.dim(2) != hidden_dim)
        throw std::runtime_error("expert_merge: all non-empty expert outputs must have same shape");
      outs[(size_t)i - 1] = t.data_ptr<float>();
    }
    if (router.get_dtype() != dtype::float32) throw std::runtime_error("expert_merge: only float32 supported");

    dynamic_tensor output(dtype::float32, {batch, seq_len, hidden_dim});
    if (from_frame(router, inputs, output)) return output;
    const int rc = csk_expert_merge(router.data_ptr<float>(), batch * seq_len, top_k_, num_experts_,
                                    hidden_dim, outs.data(), weight_before_ffn_ ? 1 : 0,
                                    output.data_ptr<float>());
    if (rc != CSK_OK) throw std::runtime_error(csk_last_error());  // texts already carry "expert_merge: "
    return output;
  }

 public:
  // merges answered by a frame's own merged rows (a test hook)
  size_t merges_from_frames() const { return merges_from_frames_; }

 private:
  // The frame's merged rows stand for this merge if the router tensor is the frame's and
  // every expert output is the very tensor the expert node of that frame emitted from it
  // (a live input), or belongs to an expert no token of the frame selected (an empty one).
  bool from_frame(const dynamic_tensor& router, const std::vector<dynamic_tensor>& inputs, dynamic_tensor& output) {
    auto ctx = csk_resident::moe_block_context::find(router.data_ptr<float>());
    if (!ctx) return false;
    std::lock_guard<std::mutex> g(ctx->m);
    const auto& f = ctx->frame;
    if (!f.valid || !f.experts_running || ctx->E != num_experts_ || ctx->k != top_k_ ||
        ctx->weight_before_ffn != (weight_before_ffn_ ? 1 : 0))
      return false;
    if ((size_t)router.numel() != f.pairs.size() ||
        std::memcmp(router.data_ptr<float>(), f.pairs.data(), f.pairs.size() * sizeof(float)) != 0)
      return false;
    if (output.dim(0) * output.dim(1) != f.T || output.dim(2) != ctx->H) return false;
    std::vector<char> selected((size_t)num_experts_, 0);
    for (size_t p = 0; p < f.pairs.size() / 2; ++p) {
      const int e = static_cast<int>(f.pairs[2 * p]);
      if (e < 0 || e >= num_experts_) return false;
      selected[(size_t)e] = 1;
    }
    for (int64_t e = 0; e < num_experts_; ++e) {
      const dynamic_tensor& t = inputs[(size_t)e + 1];
      const bool live = t.ndim() == 3 && t.dim(0) > 0;
      if (live != (selected[(size_t)e] != 0)) return false;
      if (live && t.data_ptr<float>() != f.emitted[(size_t)e]) return false;
    }
    int available = 0;
    if (csk_moe_frame_merged(ctx->layer, output.data_ptr<float>(), &available) != CSK_OK || !available) return false;
    ++merges_from_frames_;
    return true;
  }

  int64_t num_experts_ = 0;
  int64_t top_k_ = 0;
  bool weight_before_ffn_ = false;
  size_t merges_from_frames_ = 0;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::expert_merge_node, coalsack::graph_node)
