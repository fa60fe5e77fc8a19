// What the nodes of one MoE block share so that a frame runs on the device as one fused
// forward although every node still receives and emits what the reference's node does.  No
// counterpart in the reference, whose nodes each compute on their own from host memory
// (src/llm/llm_engine.cpp:721-753 wires them: router -> one expert node per expert -> merge).
//
// The router node owns a context and, after computing a frame's router output, publishes it
// under the address of that output tensor; the expert nodes and the merge node are handed
// the same tensor (messages share storage) and find the context by it.  An expert node keeps
// its resident matrices as before and attaches them to the context's view layer
// (csk_layer_create_view); once every expert a frame selects is attached, the router node's
// csk_moe_frame_begin also starts the experts and the merge on the device.  An expert node
// then only proves that the tensors it was handed are the ones it attached (same storage,
// same stamp) and copies its rows out of the frame; the merge node proves that its inputs
// are the tensors those expert nodes emitted and takes the frame's merged rows.  Whatever
// cannot be proved -- a weight that changed, an expert output that came from elsewhere, a
// router tensor that is not this frame's -- takes the per-node path, which is always correct
// on its own.
#pragma once

#include <cstring>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "coalsack/tensor/dynamic_tensor.h"
#include "coalsack_moe.h"

namespace coalsack {
namespace csk_resident {

class moe_block_context {
 public:
  moe_block_context(int64_t num_experts, int64_t top_k) : E(num_experts), k(top_k) {}
  ~moe_block_context() {
    unpublish();
    if (layer) csk_layer_destroy(layer);
  }
  moe_block_context(const moe_block_context&) = delete;
  moe_block_context& operator=(const moe_block_context&) = delete;

  const int64_t E, k;
  std::mutex m;               // frame state and layer below
  csk_layer* layer = nullptr;  // created by the first expert node that attaches (it knows F)
  int64_t H = 0, F = 0;
  int activation = -1, weight_before_ffn = -1;  // of the attached expert nodes; -2: they disagree
  int sigmoid = -1;                              // of the router node, as last given to the layer
  // the router weights the view layer holds: the tensors they were copied from and their stamps
  dynamic_tensor gate_held, bias_held;
  uint64_t gate_stamp = 0, bias_stamp = 0;
  bool gate_set = false, has_bias = false;
  // the frame the router node computed last
  struct frame_state {
    bool valid = false, experts_running = false;
    const void* hidden = nullptr;
    int64_t T = 0;
    std::vector<float> pairs;            // [T, k, 2]
    std::vector<const void*> emitted;    // per expert: storage of the tensor its node emitted from the frame
  } frame;

  bool usable() const { return layer && activation >= 0 && weight_before_ffn >= 0; }

  // Does (hidden, router) belong to the frame?  The router tensor is compared byte for byte
  // (it is small); the hidden states by storage and row count -- messages are not rewritten
  // while a frame is in flight.
  bool frame_matches(const dynamic_tensor& hidden, const dynamic_tensor& router) const {
    if (!frame.valid || hidden.data_ptr<float>() != frame.hidden) return false;
    if (hidden.ndim() != 3 || hidden.dim(0) * hidden.dim(1) != frame.T || hidden.dim(2) != H) return false;
    if ((size_t)router.numel() != frame.pairs.size()) return false;
    return std::memcmp(router.data_ptr<float>(), frame.pairs.data(), frame.pairs.size() * sizeof(float)) == 0;
  }

  // -- registry: router output storage -> context
  static std::shared_ptr<moe_block_context> find(const void* router_data) {
    std::lock_guard<std::mutex> g(registry_mutex());
    auto it = registry().find(router_data);
    return it == registry().end() ? nullptr : it->second.lock();
  }
  void publish(const std::shared_ptr<moe_block_context>& self, const void* router_data) {
    std::lock_guard<std::mutex> g(registry_mutex());
    if (published_) registry().erase(published_);
    registry()[router_data] = self;
    published_ = router_data;
  }
  void unpublish() {
    std::lock_guard<std::mutex> g(registry_mutex());
    if (published_) {
      auto it = registry().find(published_);
      if (it != registry().end() && it->second.expired()) registry().erase(it);
      published_ = nullptr;
    }
  }

 private:
  const void* published_ = nullptr;
  static std::mutex& registry_mutex() {
    static std::mutex mu;
    return mu;
  }
  static std::unordered_map<const void*, std::weak_ptr<moe_block_context>>& registry() {
    static std::unordered_map<const void*, std::weak_ptr<moe_block_context>> r;
    return r;
  }
};

}  // namespace csk_resident
}  // namespace coalsack
