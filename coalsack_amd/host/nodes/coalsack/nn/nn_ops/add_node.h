// add_node backed by the gfx950 library: same class name, element types, broadcasting and
// error texts as include/coalsack/nn/nn_ops/add_node.h of the reference (:8-55) and the
// indexer it uses (elementwise_helpers.h:9-66).  The engine's residual connections
// (llm_engine.cpp:773-777) add float32 tensors of one shape: that case runs in csk_add;
// every other shape pair and element type runs in csk_add_broadcast.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack_moe.h"

namespace coalsack {

class add_node : public binary_op_node {
 protected:
  dynamic_tensor compute(const dynamic_tensor& a, const dynamic_tensor& b) override {
    if (a.get_dtype() != b.get_dtype()) throw std::runtime_error("add: input dtype mismatch");
    const dtype dt = a.get_dtype();
    int code;
    switch (dt) {
      case dtype::float32: code = CSK_DT_FLOAT32; break;
      case dtype::float64: code = CSK_DT_FLOAT64; break;
      case dtype::int32: code = CSK_DT_INT32; break;
      case dtype::int64: code = CSK_DT_INT64; break;
      default: throw std::runtime_error("add: unsupported dtype");
    }
    std::vector<int64_t> out_shape;
    try {
      out_shape = dynamic_tensor::broadcast_shape(a.shape(), b.shape());
    } catch (const std::exception&) {  // elementwise_helpers.h:15-26
      throw std::runtime_error("Broadcast failed: Shape A=[" + list(a.shape()) + "], Shape B=[" + list(b.shape()) + "]");
    }
    dynamic_tensor out(dt, out_shape);
    if (out.numel() == 0) return out;
    int rc;
    if (dt == dtype::float32 && a.shape() == b.shape())
      rc = csk_add(a.data_ptr<float>(), b.data_ptr<float>(), out.data_ptr<float>(), out.numel());
    else
      rc = csk_add_broadcast(a.data_ptr<uint8_t>(), a.shape().data(), (int)a.ndim(), b.data_ptr<uint8_t>(),
                             b.shape().data(), (int)b.ndim(), code, out.data_ptr<uint8_t>());
    if (rc != CSK_OK) throw std::runtime_error(std::string("add: ") + csk_last_error());
    return out;
  }

 public:
  add_node() : binary_op_node("add") {}
  // not in the reference (its compute is reached through process only): for tests
  dynamic_tensor compute_test(const dynamic_tensor& a, const dynamic_tensor& b) { return compute(a, b); }

 private:
  static std::string list(const std::vector<int64_t>& s) {
    std::string r;
    for (size_t i = 0; i < s.size(); ++i) r += (i > 0 ? "," : "") + std::to_string(s[i]);
    return r;
  }
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::add_node, coalsack::graph_node)
