// rmsnorm_node backed by the gfx950 library: same class name, setter, test wrapper
// and error texts as include/coalsack/nn/nn_ops/rmsnorm_node.h of the reference
// (cited by line below); the normalisation runs in csk_rmsnorm / csk_rmsnorm_f64.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack_moe.h"

namespace coalsack {

// input: any shape, normalised over the last dimension; weight: [hidden_dim].
// out = (x / sqrt(mean(x^2) + epsilon)) * weight   (:62-83)
class rmsnorm_node : public binary_op_node {
 public:
  rmsnorm_node() : binary_op_node("rmsnorm"), epsilon_(1e-5f) {}  // :12
  void set_epsilon(float epsilon) { epsilon_ = epsilon; }          // :14
  dynamic_tensor compute_test(const dynamic_tensor& input, const dynamic_tensor& weight) {  // :17-19
    return compute(input, weight);
  }

 protected:
  dynamic_tensor compute(const dynamic_tensor& input, const dynamic_tensor& weight) override {  // :22-57
    const auto& shape = input.shape();
    if (shape.empty()) throw std::runtime_error("rmsnorm: input must have at least 1 dimension");
    int64_t outer_size = 1;
    for (size_t i = 0; i + 1 < shape.size(); ++i) outer_size *= shape[i];
    const int64_t hidden_dim = shape.back();
    if (weight.ndim() != 1 || weight.dim(0) != hidden_dim)
      throw std::runtime_error("rmsnorm: weight shape must be [hidden_dim]");
    // float32 or float64, as the reference (:47-53).  The reference reads the weight as the
    // input's element type whatever it holds (:65); a weight of another type is refused here
    // instead of having its bytes reinterpreted.
    const dtype dt = input.get_dtype();
    if (dt != dtype::float32 && dt != dtype::float64)
      throw std::runtime_error("rmsnorm: only float32 and float64 supported");
    if (weight.get_dtype() != dt) throw std::runtime_error("rmsnorm: weight must have the input's element type");
    dynamic_tensor output(dt, shape);
    if (outer_size == 0 || hidden_dim == 0) return output;
    const int rc = dt == dtype::float32
                       ? csk_rmsnorm(input.data_ptr<float>(), weight.data_ptr<float>(), output.data_ptr<float>(),
                                     outer_size, hidden_dim, epsilon_)
                       : csk_rmsnorm_f64(input.data_ptr<double>(), weight.data_ptr<double>(),
                                         output.data_ptr<double>(), outer_size, hidden_dim, epsilon_);
    if (rc != CSK_OK) throw std::runtime_error(std::string("rmsnorm: ") + csk_last_error());
    return output;
  }

 private:
  float epsilon_;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::rmsnorm_node, coalsack::graph_node)
