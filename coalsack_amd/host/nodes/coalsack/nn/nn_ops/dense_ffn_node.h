// dense_ffn_node backed by the gfx950 library: same class name, input order, output
// and error texts as include/coalsack/nn/nn_ops/dense_ffn_node.h of the reference (cited
// by line below); float16 and float32 weights both run in csk_dense_ffn_f16 (float32 ones
// as two fp16 terms).  The node keeps one device copy per weight role, replaced when the
// tensor it is handed changes (the engine feeds the same weight tensors every frame,
// src/llm/llm_engine.cpp:755-771).
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack/nn/nn_ops/resident_weight.h"
#include "coalsack_moe.h"

namespace coalsack {

// output = down_proj(silu(gate_proj(x)) * up_proj(x)) for every token (:14-27).
// Inputs: hidden [B, S, D] f32, gate_w / up_w [ffn, D], down_w [D, ffn] all float16 or all float32,
// optionally gate_b, up_b [ffn], down_b [D] f32.
class dense_ffn_node : public variadic_op_node {
 public:
  dense_ffn_node() : variadic_op_node("dense_ffn", 4) {}  // :30
  ~dense_ffn_node() override = default;
  dense_ffn_node(const dense_ffn_node&) = delete;
  dense_ffn_node& operator=(const dense_ffn_node&) = delete;
  std::string get_proc_name() const override { return "dense_ffn"; }  // :32
  // not in the reference (its compute is reached through process only): for tests
  dynamic_tensor compute_test(const std::vector<dynamic_tensor>& inputs) { return compute(inputs); }
  // number of device copies made so far (tests: a changed weight must upload, a repeat must not)
  size_t resident_uploads() const { return uploads_; }

 protected:
  dynamic_tensor compute(const std::vector<dynamic_tensor>& inputs) override {  // :35-118
    if (inputs.size() != 4 && inputs.size() != 7)
      throw std::runtime_error(
          "dense_ffn: expected 4 or 7 inputs (hidden, gate_w, up_w, down_w[, gate_b, up_b, "
          "down_b]), got " +
          std::to_string(inputs.size()));
    const dynamic_tensor& hidden = inputs[0];
    const dynamic_tensor& gate_w = inputs[1];
    const dynamic_tensor& up_w = inputs[2];
    const dynamic_tensor& down_w = inputs[3];
    const bool has_bias = inputs.size() == 7;
    if (hidden.ndim() != 3)
      throw std::runtime_error("dense_ffn: hidden_states must be 3D [B, S, D], got " +
                               std::to_string(hidden.ndim()) + "D");
    if (gate_w.ndim() != 2 || up_w.ndim() != 2 || down_w.ndim() != 2)
      throw std::runtime_error("dense_ffn: weight tensors must be 2D");
    const dtype wt = gate_w.get_dtype();
    if ((wt != dtype::float16 && wt != dtype::float32) || up_w.get_dtype() != wt || down_w.get_dtype() != wt)
      throw std::runtime_error("dense_ffn: weight tensors must all be FLOAT16 or all FLOAT32");
    if (hidden.get_dtype() != dtype::float32)
      throw std::runtime_error("dense_ffn: hidden_states must be FLOAT32");
    const int64_t tokens = hidden.dim(0) * hidden.dim(1), hidden_dim = hidden.dim(2), ffn_dim = gate_w.dim(0);
    if (gate_w.dim(1) != hidden_dim || up_w.dim(0) != ffn_dim || up_w.dim(1) != hidden_dim)
      throw std::runtime_error("dense_ffn: gate_w/up_w shape mismatch");
    if (down_w.dim(0) != hidden_dim || down_w.dim(1) != ffn_dim)
      throw std::runtime_error("dense_ffn: down_w shape mismatch, expected [" + std::to_string(hidden_dim) +
                               ", " + std::to_string(ffn_dim) + "], got [" + std::to_string(down_w.dim(0)) +
                               ", " + std::to_string(down_w.dim(1)) + "]");
    dynamic_tensor output(dtype::float32, {hidden.dim(0), hidden.dim(1), hidden_dim});
    if (tokens == 0) return output;
    const int rc = csk_dense_ffn_f16(hidden.data_ptr<float>(), tokens, hidden_dim, ffn_dim, resident_copy(0, gate_w),
                                     resident_copy(1, up_w), resident_copy(2, down_w),
                                     has_bias ? inputs[4].data_ptr<float>() : nullptr,
                                     has_bias ? inputs[5].data_ptr<float>() : nullptr,
                                     has_bias ? inputs[6].data_ptr<float>() : nullptr, output.data_ptr<float>());
    if (rc != CSK_OK) throw std::runtime_error(std::string("dense_ffn: ") + csk_last_error());
    return output;
  }

 private:
  csk_f16* resident_copy(int role, const dynamic_tensor& t) {
    return resident_[role].get(t, t.dim(0), t.dim(1), 0, "dense_ffn", &uploads_);
  }
  csk_resident::weight_slot resident_[3];  // gate, up, down
  size_t uploads_ = 0;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::dense_ffn_node, coalsack::graph_node)
