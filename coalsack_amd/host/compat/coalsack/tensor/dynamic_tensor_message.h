// Stand-in for include/coalsack/tensor/dynamic_tensor_message.h.
#pragma once
#include "coalsack/core/graph_message.h"
#include "coalsack/tensor/dynamic_tensor.h"

namespace coalsack {

class dynamic_tensor_message : public graph_message {
  dynamic_tensor tensor_;

 public:
  dynamic_tensor_message() = default;
  explicit dynamic_tensor_message(const dynamic_tensor& t) : tensor_(t) {}
  const dynamic_tensor& get_tensor() const { return tensor_; }
  dynamic_tensor& get_tensor() { return tensor_; }
  void set_tensor(const dynamic_tensor& t) { tensor_ = t; }
};

}  // namespace coalsack
