// moe_router_node backed by the gfx950 library: same class name, setters, test
// wrappers, input order, output format and error texts as
// include/coalsack/nn/nn_ops/moe_router_node.h of the reference (cited by line
// below); the body calls csk_moe_router_resident (float32; the gate and its bias, the same
// tensors every frame, are kept in device memory) or csk_moe_router_f64 (float64) instead of
// the scalar CPU loops.
//
// Place this directory in front of the reference's include path to swap the
// node in; it needs only coalsack/nn/nn_op_node.h and the C ABI header.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack_moe.h"
#include "resident_weight.h"

namespace coalsack {

// Inputs: hidden_states [batch, seq_len, hidden_dim] and gate_weights
// [num_experts, hidden_dim], both f32 or both f64; optional gate_bias [num_experts] f32.
// Output: [batch, seq_len, top_k, 2] f32 = (expert index, routing weight),
// slots in descending logit order (moe_router_node.h:13-21).
class moe_router_node : public variadic_op_node {
 public:
  moe_router_node() : variadic_op_node("moe_router", 3) {}

  void set_config(int64_t num_experts, int64_t top_k) {  // :27-30
    num_experts_ = num_experts;
    top_k_ = top_k;
  }
  void set_sigmoid_gating(bool v) { use_sigmoid_gating_ = v; }  // :34

  dynamic_tensor compute_test(const dynamic_tensor& hidden_states, const dynamic_tensor& gate_weights,
                              const dynamic_tensor& gate_bias) {  // :37-42
    return compute({hidden_states, gate_weights, gate_bias});
  }
  dynamic_tensor compute_test(const dynamic_tensor& hidden_states,
                              const dynamic_tensor& gate_weights) {  // :44-48
    return compute({hidden_states, gate_weights});
  }

 protected:
  dynamic_tensor compute(const std::vector<dynamic_tensor>& inputs) override {  // :51-124
    if (inputs.size() != 2 && inputs.size() != 3)
      throw std::runtime_error(
          "moe_router: expected 2 or 3 inputs (hidden_states, gate_weights[, gate_bias]), got " +
          std::to_string(inputs.size()));
    const dynamic_tensor& hidden = inputs[0];
    const dynamic_tensor& gate = inputs[1];
    const bool has_bias = inputs.size() == 3;
    if (hidden.ndim() != 3)
      throw std::runtime_error("moe_router: hidden_states must be 3D [batch, seq_len, hidden_dim], got " +
                               std::to_string(hidden.ndim()) + "D");
    if (gate.ndim() != 2)
      throw std::runtime_error("moe_router: gate_weights must be 2D [num_experts, hidden_dim], got " +
                               std::to_string(gate.ndim()) + "D");
    if (has_bias && inputs[2].ndim() != 1)
      throw std::runtime_error("moe_router: gate_bias must be 1D [num_experts], got " +
                               std::to_string(inputs[2].ndim()) + "D");
    const int64_t batch = hidden.dim(0), seq_len = hidden.dim(1), hidden_dim = hidden.dim(2);
    if (gate.dim(0) != num_experts_ || gate.dim(1) != hidden_dim)
      throw std::runtime_error("moe_router: gate_weights shape mismatch, expected [" +
                               std::to_string(num_experts_) + ", " + std::to_string(hidden_dim) +
                               "], got [" + std::to_string(gate.dim(0)) + ", " +
                               std::to_string(gate.dim(1)) + "]");
    if (has_bias && inputs[2].dim(0) != num_experts_)
      throw std::runtime_error("moe_router: gate_bias must have num_experts=" +
                               std::to_string(num_experts_) + " elements, got " +
                               std::to_string(inputs[2].dim(0)));
    // :115-122: the element type of the hidden states picks float or double arithmetic.  The
    // reference reads the gate weights as that type whatever they hold; here a gate of
    // another type is refused instead of being reinterpreted.
    const dtype dt = hidden.get_dtype();
    if (dt != dtype::float32 && dt != dtype::float64)
      throw std::runtime_error("moe_router: only float32 and float64 supported");
    if (gate.get_dtype() != dt)
      throw std::runtime_error("moe_router: gate_weights must have the element type of hidden_states");

    dynamic_tensor output(dtype::float32, {batch, seq_len, top_k_, 2});
    int rc;
    if (dt == dtype::float32) {
      const float* gate_dev = static_cast<const float*>(gate_slot_.get(gate, "moe_router", &resident_uploads_));
      const float* bias_dev =
          has_bias ? static_cast<const float*>(bias_slot_.get(inputs[2], "moe_router", &resident_uploads_)) : nullptr;
      rc = csk_moe_router_resident(hidden.data_ptr<float>(), batch * seq_len, hidden_dim, gate_dev, num_experts_,
                                   bias_dev, top_k_, use_sigmoid_gating_ ? 1 : 0, output.data_ptr<float>());
    } else {
      const float* bias = has_bias ? inputs[2].data_ptr<float>() : nullptr;
      rc = csk_moe_router_f64(hidden.data_ptr<double>(), batch * seq_len, hidden_dim, gate.data_ptr<double>(),
                              num_experts_, bias, top_k_, use_sigmoid_gating_ ? 1 : 0, output.data_ptr<float>(),
                              nullptr);
    }
    if (rc != CSK_OK) throw std::runtime_error(std::string("moe_router: ") + csk_last_error());
    return output;
  }

 public:
  // device copies of the gate / bias made so far (a test hook: the same tensors must not go up twice)
  size_t resident_uploads() const { return resident_uploads_; }

 private:
  int64_t num_experts_ = 0;
  int64_t top_k_ = 0;
  bool use_sigmoid_gating_ = false;
  csk_resident::array_slot gate_slot_, bias_slot_;
  size_t resident_uploads_ = 0;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::moe_router_node, coalsack::graph_node)
