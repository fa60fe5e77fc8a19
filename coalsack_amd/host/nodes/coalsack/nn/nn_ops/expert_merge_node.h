// expert_merge_node backed by the gfx950 library: same class name, setters,
// test wrapper, input order and error texts as
// include/coalsack/nn/nn_ops/expert_merge_node.h of the reference (cited by
// line below); the weighted sum runs in csk_expert_merge.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
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
    const int rc = csk_expert_merge(router.data_ptr<float>(), batch * seq_len, top_k_, num_experts_,
                                    hidden_dim, outs.data(), weight_before_ffn_ ? 1 : 0,
                                    output.data_ptr<float>());
    if (rc != CSK_OK) throw std::runtime_error(csk_last_error());  // texts already carry "expert_merge: "
    return output;
  }

 private:
  int64_t num_experts_ = 0;
  int64_t top_k_ = 0;
  bool weight_before_ffn_ = false;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::expert_merge_node, coalsack::graph_node)
