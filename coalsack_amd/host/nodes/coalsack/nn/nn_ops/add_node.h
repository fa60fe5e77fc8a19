// add_node backed by the gfx950 library: same class name and error texts as
// include/coalsack/nn/nn_ops/add_node.h of the reference (:8-55).  The engine uses it
// for the residual connections (llm_engine.cpp:773-777), where both operands have the
// same shape and are float32: that case runs in csk_add.  The reference's generic
// broadcasting indexer (elementwise_helpers.h:9-66) and its float64 / integer branches
// are not part of this path and are refused with a message.
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
    if (a.get_dtype() != dtype::float32) throw std::runtime_error("add: only float32 supported on this build");
    if (a.shape() != b.shape()) throw std::runtime_error("add: broadcasting is not supported on this build");
    dynamic_tensor out(dtype::float32, a.shape());
    int64_t n = 1;
    for (int64_t d : a.shape()) n *= d;
    if (n == 0) return out;
    const int rc = csk_add(a.data_ptr<float>(), b.data_ptr<float>(), out.data_ptr<float>(), n);
    if (rc != CSK_OK) throw std::runtime_error(std::string("add: ") + csk_last_error());
    return out;
  }

 public:
  add_node() : binary_op_node("add") {}
  dynamic_tensor compute_test(const dynamic_tensor& a, const dynamic_tensor& b) { return compute(a, b); }
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::add_node, coalsack::graph_node)
