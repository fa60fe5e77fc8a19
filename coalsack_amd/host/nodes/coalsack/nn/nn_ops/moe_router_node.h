// moe_router_node backed by the gfx950 library: same class name, setters, test
// wrappers, input order, output format and error texts as
// include/coalsack/nn/nn_ops/moe_router_node.h of the reference (cited by line
// below); the body calls csk_moe_router_resident (float32; the gate and its bias, the same
// tensors every frame, are kept in device memory) or csk_moe_router_f64 (float64) instead of
// the scalar CPU loops.  Once the block's expert nodes have attached their resident matrices
// to this node's context (moe_block_context.h), a frame's router output comes from
// csk_moe_frame_begin, which goes on to run the selected experts and the merge on the device.
//
// Place this directory in front of the reference's include path to swap the
// node in; it needs only coalsack/nn/nn_op_node.h and the C ABI header.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack_moe.h"
#include "moe_block_context.h"
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
      if (!ctx_ || ctx_->E != num_experts_ || ctx_->k != top_k_)
        ctx_ = std::make_shared<csk_resident::moe_block_context>(num_experts_, top_k_);
      const int64_t tokens = batch * seq_len;
      int running = 0;
      bool framed = false;
      if (tokens > 0) framed = begin_frame(hidden, gate, has_bias ? &inputs[2] : nullptr, output, &running);
      if (!framed) {
        const float* gate_dev = static_cast<const float*>(gate_slot_.get(gate, "moe_router", &resident_uploads_));
        const float* bias_dev =
            has_bias ? static_cast<const float*>(bias_slot_.get(inputs[2], "moe_router", &resident_uploads_)) : nullptr;
        rc = csk_moe_router_resident(hidden.data_ptr<float>(), tokens, hidden_dim, gate_dev, num_experts_, bias_dev,
                                     top_k_, use_sigmoid_gating_ ? 1 : 0, output.data_ptr<float>());
        if (rc != CSK_OK) throw std::runtime_error(std::string("moe_router: ") + csk_last_error());
      }
      {
        // the frame the other nodes of the block will look up by this output tensor
        std::lock_guard<std::mutex> g(ctx_->m);
        auto& f = ctx_->frame;
        f.valid = tokens > 0;
        f.experts_running = framed && running != 0;
        f.hidden = hidden.data_ptr<float>();
        f.T = tokens;
        f.pairs.assign(output.data_ptr<float>(), output.data_ptr<float>() + output.numel());
        f.emitted.assign((size_t)num_experts_, nullptr);
        if (ctx_->H == 0) ctx_->H = hidden_dim;
      }
      ctx_->publish(ctx_, output.data_ptr<float>());
      return output;
    }
    const float* bias = has_bias ? inputs[2].data_ptr<float>() : nullptr;
    rc = csk_moe_router_f64(hidden.data_ptr<double>(), batch * seq_len, hidden_dim, gate.data_ptr<double>(),
                            num_experts_, bias, top_k_, use_sigmoid_gating_ ? 1 : 0, output.data_ptr<float>(),
                            nullptr);
    if (rc != CSK_OK) throw std::runtime_error(std::string("moe_router: ") + csk_last_error());
    return output;
  }

 public:
  // device copies of the gate / bias made so far (a test hook: the same tensors must not go up twice)
  size_t resident_uploads() const { return resident_uploads_; }
  // frames whose router output came from csk_moe_frame_begin / whose experts that call started
  size_t frames_begun() const { return frames_begun_; }
  size_t frames_with_experts() const { return frames_with_experts_; }

 private:
  // The context's view layer takes this frame: its router weights follow the tensors handed
  // in (same storage and stamp: nothing to do), then router, dispatch and -- if every
  // selected expert is attached -- the experts and the merge are started.  False: the view
  // is not ready (no expert attached yet, options the expert nodes disagree on, a batch
  // beyond one pass), and the router runs on its own.
  bool begin_frame(const dynamic_tensor& hidden, const dynamic_tensor& gate, const dynamic_tensor* bias,
                   dynamic_tensor& output, int* running) {
    std::lock_guard<std::mutex> g(ctx_->m);
    ctx_->frame.valid = false;
    if (!ctx_->usable() || ctx_->H != hidden.dim(2)) return false;
    const uint64_t gs = csk_resident::content_stamp(gate.data_ptr<uint8_t>(), gate.bytes());
    const uint64_t bs = bias ? csk_resident::content_stamp(bias->data_ptr<uint8_t>(), bias->bytes()) : 0;
    const bool same = ctx_->gate_set && ctx_->gate_held.data_ptr<uint8_t>() == gate.data_ptr<uint8_t>() &&
                      ctx_->gate_stamp == gs && ctx_->has_bias == (bias != nullptr) &&
                      (!bias || (ctx_->bias_held.data_ptr<uint8_t>() == bias->data_ptr<uint8_t>() && ctx_->bias_stamp == bs));
    if (!same) {
      if (csk_layer_set_router(ctx_->layer, gate.data_ptr<float>(), bias ? bias->data_ptr<float>() : nullptr) != CSK_OK)
        return false;
      ctx_->gate_held = gate, ctx_->gate_stamp = gs, ctx_->gate_set = true;
      ctx_->has_bias = bias != nullptr;
      if (bias) ctx_->bias_held = *bias, ctx_->bias_stamp = bs;
      ++resident_uploads_;
    }
    const int sg = use_sigmoid_gating_ ? 1 : 0;
    if (ctx_->sigmoid != sg) {
      if (csk_layer_set_options(ctx_->layer, sg, ctx_->activation, ctx_->weight_before_ffn) != CSK_OK) return false;
      ctx_->sigmoid = sg;
    }
    if (csk_moe_frame_begin(ctx_->layer, hidden.data_ptr<float>(), hidden.dim(0) * hidden.dim(1),
                            output.data_ptr<float>(), 0, running) != CSK_OK)
      return false;
    ++frames_begun_;
    frames_with_experts_ += *running != 0;
    return true;
  }

  std::shared_ptr<csk_resident::moe_block_context> ctx_;
  size_t frames_begun_ = 0, frames_with_experts_ = 0;
  int64_t num_experts_ = 0;
  int64_t top_k_ = 0;
  bool use_sigmoid_gating_ = false;
  csk_resident::array_slot gate_slot_, bias_slot_;
  size_t resident_uploads_ = 0;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::moe_router_node, coalsack::graph_node)
