// Stand-in for include/coalsack/tensor/dynamic_mx_tensor_message.h.
#pragma once
#include "coalsack/core/graph_message.h"
#include "coalsack/tensor/dynamic_mx_tensor.h"

namespace coalsack {

class dynamic_mx_tensor_message : public graph_message {
  dynamic_mx_tensor tensor_;

 public:
  dynamic_mx_tensor_message() = default;
  explicit dynamic_mx_tensor_message(const dynamic_mx_tensor& t) : tensor_(t) {}
  const dynamic_mx_tensor& get_mx_tensor() const { return tensor_; }
  dynamic_mx_tensor& get_mx_tensor() { return tensor_; }
  void set_mx_tensor(const dynamic_mx_tensor& t) { tensor_ = t; }
};

}  // namespace coalsack
