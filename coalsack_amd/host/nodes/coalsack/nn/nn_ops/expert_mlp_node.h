// expert_mlp_node backed by the gfx950 library: same class name, constructor,
// setters, test wrapper, input order, output conventions and error texts as
// include/coalsack/nn/nn_ops/expert_mlp_node.h of the reference (cited by line
// below), for both kinds of weights process() distinguishes (:113-136): MXFP4
// messages go to csk_expert_mlp_mxfp4, float16 tensors to csk_expert_mlp_f16.
//
// Weights are uploaded (repacked into the resident device layout) and cached per
// node, one entry per role (up, gate, down).  An entry keeps a copy of the host
// tensor it was made from -- copies share the storage, so the storage cannot be
// freed and its address handed to another tensor while the entry lives -- plus a
// stamp of its bytes (resident_weight.h: a hash of all of them by default).  A role whose
// tensor arrives with the same storage, shape and stamp reuses the device copy; anything else (moe_weight_provider is an
// LRU, src/llm/moe_weight_provider.cpp:102-132: an evicted slice comes back in new
// storage) is uploaded again and the old device copy is freed, so a node never
// holds more than three device matrices and three host references.
//
// With MXFP4 weights the node also takes part in its block's frames (moe_block_context.h):
// it attaches its three resident matrices and its biases to the context the router tensor
// leads to, and when a frame's experts are already running on the device and every tensor
// it is handed is the one it attached, it copies its rows out of the frame instead of
// computing them again.  A tensor that changed is uploaded and computed here, as before,
// the frame's merged rows are declared void, and the new copy is attached for the next
// frame.
#pragma once

#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack/tensor/dynamic_mx_tensor_message.h"
#include "coalsack/nn/nn_ops/moe_block_context.h"
#include "coalsack/nn/nn_ops/resident_weight.h"
#include "coalsack_moe.h"

namespace coalsack {

class expert_mlp_node : public graph_node {
 public:
  enum class activation_type {  // :27-30
    MODIFIED_SWIGLU,
    STANDARD_SWIGLU,
  };

  explicit expert_mlp_node(int expert_id = 0)  // :32-38
      : expert_id_(expert_id), output_(std::make_shared<graph_edge>(this)) {
    set_output(output_);
  }
  ~expert_mlp_node() override {
    detach();
    for (auto& r : resident_) csk_mxfp4_free(r.handle);
    for (auto& r : resident16_) csk_f16_free(r.handle);
  }
  expert_mlp_node(const expert_mlp_node&) = delete;
  expert_mlp_node& operator=(const expert_mlp_node&) = delete;

  int get_expert_id() const { return expert_id_; }
  std::string get_proc_name() const override { return "expert_mlp"; }
  void set_input_names(const std::vector<std::string>& names) { input_names_ = names; }
  void set_output_name(const std::string& name) { output_name_ = name; }
  void set_node_name(const std::string& name) { node_name_ = name; }
  void set_activation_type(activation_type t) { activation_type_ = t; }
  activation_type get_activation_type() const { return activation_type_; }
  void set_weight_before_ffn(bool v) { weight_before_ffn_ = v; }  // :52
  std::vector<std::string> get_input_names() const { return input_names_; }
  std::string get_output_name() const { return output_name_; }

  // Public wrapper for testing (:57-60): the float16 branch on plain tensors.
  dynamic_tensor compute_test(const std::vector<dynamic_tensor>& inputs) { return compute_fp16(inputs); }

  // One token through raw 17-byte-block weights (:63-70).
  void compute_test_mxfp4(const float* hidden_vec, const uint8_t* w_up_data, const uint8_t* w_gate_data,
                          const uint8_t* w_down_data, const float* b_up_data, const float* b_gate_data,
                          const float* b_down_data, float* output_vec, int64_t hidden_dim,
                          int64_t expert_ffn_dim) {
    if (expert_ffn_dim % 2 != 0)  // :662-669
      throw std::runtime_error("compute_token_mxfp4: expert_ffn_dim must be even, got " +
                               std::to_string(expert_ffn_dim));
    if (hidden_dim % 2 != 0)
      throw std::runtime_error("compute_token_mxfp4: hidden_dim must be even, got " +
                               std::to_string(hidden_dim));
    const int rc = csk_expert_token_mxfp4(hidden_vec, w_up_data, w_gate_data, w_down_data, b_up_data,
                                          b_gate_data, b_down_data, output_vec, hidden_dim,
                                          expert_ffn_dim, act_code());
    if (rc != CSK_OK) throw std::runtime_error(std::string("expert_mlp: ") + csk_last_error());
  }

  void process(std::string /*input_name*/, graph_message_ptr message) override {  // :73-148
    auto in = std::dynamic_pointer_cast<result_message>(message);
    const uint64_t frame = in ? in->get_frame_number() : 0;
    const double stamp = in ? in->get_timestamp() : 0.0;
    std::shared_ptr<result_message> out;
    if (in && !in->is_ok()) {
      out = result_message::error({{output_name_, nullptr}}, "Input error");
    } else {
      try {
        if (!in || input_names_.empty()) throw std::runtime_error("expert_mlp: invalid input");
        std::vector<graph_message_ptr> fields;
        for (const auto& name : input_names_) {
          auto f = in->get_field(name);
          if (!f) throw std::runtime_error("expert_mlp: missing field " + name);
          fields.push_back(f);
        }
        dynamic_tensor result;
        if (fields.size() > 1 && std::dynamic_pointer_cast<dynamic_mx_tensor_message>(fields[1])) {
          result = compute_with_mxfp4(fields);
        } else {  // :120-130
          std::vector<dynamic_tensor> inputs;
          for (const auto& f : fields) {
            auto t = std::dynamic_pointer_cast<dynamic_tensor_message>(f);
            if (!t) throw std::runtime_error("expert_mlp: expected dynamic_tensor_message");
            inputs.push_back(t->get_tensor());
          }
          result = compute_fp16(inputs);
        }
        out = result_message::ok({{output_name_, std::make_shared<dynamic_tensor_message>(result)}});
      } catch (const std::exception& e) {
        out = result_message::error({{output_name_, nullptr}}, e.what());
      }
    }
    out->set_frame_number(frame);
    out->set_timestamp(stamp);
    output_->send(out);
  }

  // number of device copies made so far (tests: a reload must upload, a repeat must not)
  size_t resident_uploads() const { return uploads_; }
  // outputs taken from a frame the router node had started / computed by this node itself
  size_t rows_from_frames() const { return rows_from_frames_; }
  size_t rows_computed() const { return rows_computed_; }

 private:
  enum role { ROLE_UP = 0, ROLE_GATE = 1, ROLE_DOWN = 2 };

  int act_code() const {
    return activation_type_ == activation_type::MODIFIED_SWIGLU ? CSK_ACT_MODIFIED_SWIGLU
                                                                : CSK_ACT_STANDARD_SWIGLU;
  }

  static uint64_t content_stamp(const uint8_t* p, size_t n) { return csk_resident::content_stamp(p, n); }

  struct resident {
    csk_mxfp4* handle = nullptr;
    dynamic_mx_tensor held;  // shares the storage the copy was made from
    uint64_t stamp = 0;
  };

  csk_mxfp4* resident_copy(role r, const dynamic_mx_tensor& t) {
    resident& c = resident_[r];
    const uint64_t stamp = content_stamp(t.data_ptr(), t.size_bytes());
    if (c.handle && c.held.data_ptr() == t.data_ptr() && c.held.shape() == t.shape() && c.stamp == stamp)
      return c.handle;
    csk_mxfp4* h = nullptr;
    if (csk_mxfp4_upload(t.data_ptr(), t.dim(0), t.dim(1), &h) != CSK_OK)
      throw std::runtime_error(std::string("expert_mlp: ") + csk_last_error());
    if (c.handle) {
      detach();  // the view layer must not point at a matrix that is about to be freed
      csk_mxfp4_free(c.handle);
    }
    c.handle = h;
    c.held = t;
    c.stamp = stamp;
    ++uploads_;
    return h;
  }

  // -- the block's frames (moe_block_context.h)
  struct bias_held {
    dynamic_tensor t;
    uint64_t stamp = 0;
  };
  void detach() {
    if (auto ctx = attached_to_.lock()) {
      std::lock_guard<std::mutex> g(ctx->m);
      if (ctx->layer) (void)csk_layer_detach_expert(ctx->layer, expert_id_);
      ctx->frame.experts_running = false;  // (a frame in flight was built on the old matrices)
    }
    attached_to_.reset();
  }
  // biases as attached: same storage and stamp?
  bool biases_unchanged(bool has_bias, const dynamic_tensor* b[3]) const {
    if (has_bias != attached_bias_) return false;
    if (!has_bias) return true;
    for (int i = 0; i < 3; ++i)
      if (b[i]->data_ptr<uint8_t>() != bias_[i].t.data_ptr<uint8_t>() ||
          csk_resident::content_stamp(b[i]->data_ptr<uint8_t>(), b[i]->bytes()) != bias_[i].stamp)
        return false;
    return true;
  }
  // Points the context's view layer at this node's matrices (creating the layer when this is
  // the first expert of the block to arrive) so that the next frame can run here.
  void attach(const std::shared_ptr<csk_resident::moe_block_context>& ctx, int64_t hidden_dim, int64_t ffn,
              csk_mxfp4* up, csk_mxfp4* gate, csk_mxfp4* down, bool has_bias, const dynamic_tensor* b[3]) {
    std::lock_guard<std::mutex> g(ctx->m);
    if (expert_id_ < 0 || expert_id_ >= ctx->E) return;
    if (!ctx->layer) {
      if (csk_layer_create_view(ctx->E, ctx->k, hidden_dim, ffn, &ctx->layer) != CSK_OK) {
        ctx->layer = nullptr;
        return;
      }
      ctx->H = hidden_dim, ctx->F = ffn;
      ctx->activation = act_code(), ctx->weight_before_ffn = weight_before_ffn_ ? 1 : 0;
      ctx->sigmoid = -1;  // the router node passes the options on with its own
    }
    if (ctx->H != hidden_dim || ctx->F != ffn) return;
    // every expert node of a block has the same options; if not, the block has no frames
    if (ctx->activation != act_code() || ctx->weight_before_ffn != (weight_before_ffn_ ? 1 : 0)) {
      ctx->activation = ctx->weight_before_ffn = -2;
      return;
    }
    if (csk_layer_attach_expert(ctx->layer, expert_id_, up, gate, down, has_bias ? b[0]->data_ptr<float>() : nullptr,
                                has_bias ? b[1]->data_ptr<float>() : nullptr,
                                has_bias ? b[2]->data_ptr<float>() : nullptr) != CSK_OK)
      return;
    attached_to_ = ctx;
    attached_bias_ = has_bias;
    for (int i = 0; has_bias && i < 3; ++i) {
      bias_[i].t = *b[i];
      bias_[i].stamp = csk_resident::content_stamp(b[i]->data_ptr<uint8_t>(), b[i]->bytes());
    }
  }

  struct resident16 {
    csk_f16* handle = nullptr;
    dynamic_tensor held;
    uint64_t stamp = 0;
  };

  csk_f16* resident_copy16(role r, const dynamic_tensor& t) {
    resident16& c = resident16_[r];
    const uint8_t* bytes = reinterpret_cast<const uint8_t*>(t.data_ptr<uint16_t>());
    const uint64_t stamp = content_stamp(bytes, (size_t)t.dim(0) * (size_t)t.dim(1) * 2);
    if (c.handle && c.held.data_ptr<uint16_t>() == t.data_ptr<uint16_t>() && c.held.shape() == t.shape() &&
        c.stamp == stamp)
      return c.handle;
    csk_f16* h = nullptr;
    if (csk_f16_upload(t.data_ptr<uint16_t>(), t.dim(0), t.dim(1), &h) != CSK_OK)
      throw std::runtime_error(std::string("expert_mlp: ") + csk_last_error());
    if (c.handle) csk_f16_free(c.handle);
    c.handle = h;
    c.held = t;
    c.stamp = stamp;
    ++uploads_;
    return h;
  }

  static std::string dims2(int64_t a, int64_t b) {
    return "[" + std::to_string(a) + ", " + std::to_string(b) + "]";
  }

  dynamic_tensor compute_fp16(const std::vector<dynamic_tensor>& inputs) {  // :269-389
    if (inputs.size() != 5 && inputs.size() != 8)
      throw std::runtime_error(
          "expert_mlp: expected 5 or 8 inputs (hidden, w_up, w_gate, w_down[, b_up, b_gate, "
          "b_down], router_output), got " +
          std::to_string(inputs.size()));
    const bool has_bias = inputs.size() == 8;
    const dynamic_tensor& hidden = inputs[0];
    const dynamic_tensor& w_up = inputs[1];
    const dynamic_tensor& w_gate = inputs[2];
    const dynamic_tensor& w_down = inputs[3];
    const dynamic_tensor& router = inputs[has_bias ? 7 : 4];
    if (router.ndim() != 4 || router.dim(3) != 2)
      throw std::runtime_error("expert_mlp: router_output must be 4D [batch, seq_len, top_k, 2], got " +
                               std::to_string(router.ndim()) + "D");
    if (router.get_dtype() != dtype::float32)
      throw std::runtime_error("expert_mlp: router_output must be float32");
    // not selected by any token: a {0}-shaped tensor, before anything else is looked at (:297-306)
    const int64_t top_k = router.dim(2);
    const float* rp = router.data_ptr<float>();
    bool any = false;
    for (int64_t p = 0; p < router.dim(0) * router.dim(1) * top_k && !any; ++p)
      any = static_cast<int>(rp[2 * p]) == expert_id_;
    if (!any) return dynamic_tensor(dtype::float32, {0});
    if (hidden.ndim() != 3)
      throw std::runtime_error("expert_mlp: hidden_states must be 3D [batch, seq_len, hidden_dim], got " +
                               std::to_string(hidden.ndim()) + "D");
    const int64_t tokens = hidden.dim(0) * hidden.dim(1), hidden_dim = hidden.dim(2);
    if (w_up.ndim() != 2 || w_gate.ndim() != 2 || w_down.ndim() != 2)
      throw std::runtime_error(
          "expert_mlp: all weights must be 2D [expert_ffn_dim, hidden_dim] or [hidden_dim, "
          "expert_ffn_dim]");
    const int64_t ffn = w_up.dim(0);
    if (w_up.dim(1) != hidden_dim)
      throw std::runtime_error("expert_mlp: w_up must be " + dims2(ffn, hidden_dim) + ", got " +
                               dims2(w_up.dim(0), w_up.dim(1)));
    if (w_gate.dim(0) != ffn || w_gate.dim(1) != hidden_dim)
      throw std::runtime_error("expert_mlp: w_gate must be " + dims2(ffn, hidden_dim) + ", got " +
                               dims2(w_gate.dim(0), w_gate.dim(1)));
    if (w_down.dim(0) != hidden_dim || w_down.dim(1) != ffn)
      throw std::runtime_error("expert_mlp: w_down must be " + dims2(hidden_dim, ffn) + ", got " +
                               dims2(w_down.dim(0), w_down.dim(1)));
    if (has_bias) {
      const dynamic_tensor &b_up = inputs[4], &b_gate = inputs[5], &b_down = inputs[6];
      if (b_up.ndim() != 1 || b_up.dim(0) != ffn)
        throw std::runtime_error("expert_mlp: b_up must be [expert_ffn_dim=" + std::to_string(ffn) +
                                 "], got [" + std::to_string(b_up.dim(0)) + "]");
      if (b_gate.ndim() != 1 || b_gate.dim(0) != ffn)
        throw std::runtime_error("expert_mlp: b_gate must be [expert_ffn_dim=" + std::to_string(ffn) +
                                 "], got [" + std::to_string(b_gate.dim(0)) + "]");
      if (b_down.ndim() != 1 || b_down.dim(0) != hidden_dim)
        throw std::runtime_error("expert_mlp: b_down must be [hidden_dim=" + std::to_string(hidden_dim) +
                                 "], got [" + std::to_string(b_down.dim(0)) + "]");
    }
    if (w_up.get_dtype() != dtype::float16 || w_gate.get_dtype() != dtype::float16 ||
        w_down.get_dtype() != dtype::float16)
      throw std::runtime_error("expert_mlp: all weights must be FLOAT16");
    if (hidden.get_dtype() != dtype::float32)
      throw std::runtime_error("expert_mlp: hidden_states must be FLOAT32");

    dynamic_tensor output(dtype::float32, hidden.shape());
    int is_empty = 0;
    const int rc = csk_expert_mlp_f16(
        expert_id_, hidden.data_ptr<float>(), tokens, hidden_dim, ffn, resident_copy16(ROLE_UP, w_up),
        resident_copy16(ROLE_GATE, w_gate), resident_copy16(ROLE_DOWN, w_down),
        has_bias ? inputs[4].data_ptr<float>() : nullptr, has_bias ? inputs[5].data_ptr<float>() : nullptr,
        has_bias ? inputs[6].data_ptr<float>() : nullptr, rp, top_k, act_code(),
        weight_before_ffn_ ? 1 : 0, output.data_ptr<float>(), &is_empty);
    if (rc != CSK_OK) throw std::runtime_error(std::string("expert_mlp: ") + csk_last_error());
    if (is_empty) return dynamic_tensor(dtype::float32, {0});
    return output;
  }

  dynamic_tensor compute_with_mxfp4(const std::vector<graph_message_ptr>& msgs) {  // :392-485
    if (msgs.size() != 5 && msgs.size() != 8)
      throw std::runtime_error("expert_mlp: expected 5 or 8 inputs for MXFP4, got " +
                               std::to_string(msgs.size()));
    const bool has_bias = msgs.size() == 8;
    auto hidden_msg = std::dynamic_pointer_cast<dynamic_tensor_message>(msgs[0]);
    auto up_msg = std::dynamic_pointer_cast<dynamic_mx_tensor_message>(msgs[1]);
    auto gate_msg = std::dynamic_pointer_cast<dynamic_mx_tensor_message>(msgs[2]);
    auto down_msg = std::dynamic_pointer_cast<dynamic_mx_tensor_message>(msgs[3]);
    auto router_msg = std::dynamic_pointer_cast<dynamic_tensor_message>(msgs[has_bias ? 7 : 4]);
    std::shared_ptr<dynamic_tensor_message> b_up, b_gate, b_down;
    if (has_bias) {
      b_up = std::dynamic_pointer_cast<dynamic_tensor_message>(msgs[4]);
      b_gate = std::dynamic_pointer_cast<dynamic_tensor_message>(msgs[5]);
      b_down = std::dynamic_pointer_cast<dynamic_tensor_message>(msgs[6]);
    }
    if (!hidden_msg || !up_msg || !gate_msg || !down_msg || !router_msg)
      throw std::runtime_error("expert_mlp: invalid input message types for MXFP4");
    if (has_bias && (!b_up || !b_gate || !b_down))
      throw std::runtime_error("expert_mlp: invalid bias message types for MXFP4");

    const dynamic_tensor& hidden = hidden_msg->get_tensor();
    const dynamic_tensor& router = router_msg->get_tensor();
    const dynamic_mx_tensor& w_up = up_msg->get_mx_tensor();
    const dynamic_mx_tensor& w_gate = gate_msg->get_mx_tensor();
    const dynamic_mx_tensor& w_down = down_msg->get_mx_tensor();
    if (hidden.ndim() != 3) throw std::runtime_error("expert_mlp: hidden_states must be 3D");
    if (router.ndim() != 4 || router.dim(3) != 2)
      throw std::runtime_error("expert_mlp: router_output must be 4D [batch, seq_len, top_k, 2]");

    // not selected by any token: a {0}-shaped tensor, before any weight is looked at (:441-443)
    const int64_t tokens = hidden.dim(0) * hidden.dim(1), top_k = router.dim(2);
    const float* rp = router.data_ptr<float>();
    bool any = false;
    for (int64_t p = 0; p < router.dim(0) * router.dim(1) * top_k && !any; ++p)
      any = static_cast<int>(rp[2 * p]) == expert_id_;
    if (!any) return dynamic_tensor(dtype::float32, {0});

    const int64_t hidden_dim = hidden.dim(2);
    if (w_up.ndim() != 2 || w_gate.ndim() != 2 || w_down.ndim() != 2)
      throw std::runtime_error("expert_mlp: all weights must be 2D");
    const int64_t ffn = w_up.dim(0);
    if (w_up.dim(1) != hidden_dim || w_gate.dim(0) != ffn || w_gate.dim(1) != hidden_dim ||
        w_down.dim(0) != hidden_dim || w_down.dim(1) != ffn)
      throw std::runtime_error("expert_mlp: weight dimension mismatch");
    if (hidden_dim % 32 != 0)
      throw std::runtime_error("expert_mlp: hidden_dim must be a multiple of 32 for MXFP4, got " +
                               std::to_string(hidden_dim));
    if (ffn % 32 != 0)
      throw std::runtime_error("expert_mlp: expert_ffn_dim must be a multiple of 32 for MXFP4, got " +
                               std::to_string(ffn));

    // resident copies of the three matrices (an unchanged tensor costs its stamp)
    const size_t uploads_before = uploads_;
    csk_mxfp4* d_up = resident_copy(ROLE_UP, w_up);
    csk_mxfp4* d_gate = resident_copy(ROLE_GATE, w_gate);
    csk_mxfp4* d_down = resident_copy(ROLE_DOWN, w_down);
    const dynamic_tensor* biases[3] = {has_bias ? &b_up->get_tensor() : nullptr,
                                       has_bias ? &b_gate->get_tensor() : nullptr,
                                       has_bias ? &b_down->get_tensor() : nullptr};

    // the block's frame, if the router tensor leads to one and it is this (hidden, router) pair
    auto ctx = csk_resident::moe_block_context::find(rp);
    bool in_frame = false, frame_running = false;
    if (ctx) {
      std::lock_guard<std::mutex> g(ctx->m);
      in_frame = ctx->frame_matches(hidden, router);
      frame_running = in_frame && ctx->frame.experts_running;
    }
    const bool mine = ctx && attached_to_.lock() == ctx && uploads_ == uploads_before &&
                      biases_unchanged(has_bias, biases);
    dynamic_tensor output(dtype::float32, hidden.shape());
    if (frame_running && mine) {
      // the frame computed this expert from the very matrices and biases handed in now
      std::lock_guard<std::mutex> g(ctx->m);
      if (ctx->frame.experts_running && csk_moe_frame_expert_rows(ctx->layer, expert_id_, output.data_ptr<float>()) == CSK_OK) {
        ctx->frame.emitted[(size_t)expert_id_] = output.data_ptr<float>();
        ++rows_from_frames_;
        return output;
      }
    }
    if (frame_running) {
      // the frame ran on matrices that are not the ones handed in: its merged rows are void
      std::lock_guard<std::mutex> g(ctx->m);
      (void)csk_moe_frame_void(ctx->layer);
    }
    int is_empty = 0;
    const int rc = csk_expert_mlp_mxfp4(
        expert_id_, hidden.data_ptr<float>(), tokens, hidden_dim, ffn, d_up, d_gate, d_down,
        has_bias ? biases[0]->data_ptr<float>() : nullptr, has_bias ? biases[1]->data_ptr<float>() : nullptr,
        has_bias ? biases[2]->data_ptr<float>() : nullptr, rp, top_k, act_code(),
        weight_before_ffn_ ? 1 : 0, output.data_ptr<float>(), &is_empty);
    if (rc != CSK_OK) throw std::runtime_error(std::string("expert_mlp: ") + csk_last_error());
    ++rows_computed_;
    if (in_frame && !mine) {
      if (attached_to_.lock() != ctx) detach();
      attach(ctx, hidden_dim, ffn, d_up, d_gate, d_down, has_bias, biases);
    }
    if (is_empty) return dynamic_tensor(dtype::float32, {0});
    return output;
  }

  int expert_id_;
  graph_edge_ptr output_;
  std::vector<std::string> input_names_;
  std::string output_name_, node_name_;
  activation_type activation_type_ = activation_type::MODIFIED_SWIGLU;
  bool weight_before_ffn_ = false;
  resident resident_[3];
  resident16 resident16_[3];
  size_t uploads_ = 0;
  std::weak_ptr<csk_resident::moe_block_context> attached_to_;
  bool attached_bias_ = false;
  bias_held bias_[3];
  size_t rows_from_frames_ = 0, rows_computed_ = 0;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::expert_mlp_node, coalsack::graph_node)
