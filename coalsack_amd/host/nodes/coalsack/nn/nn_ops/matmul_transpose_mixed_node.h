// matmul_transpose_mixed_node backed by the gfx950 library: same class name, test wrapper,
// shapes and error texts as include/coalsack/nn/nn_ops/matmul_transpose_mixed_node.h of the
// reference (cited by line below): fp32 activations times a float16 or float32 weight,
// with leading batch dimensions on either side.  The products run in
// csk_matmul_transpose_f16; the node keeps one device copy per weight matrix, replaced
// when the tensor it is handed changes.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack/nn/nn_ops/resident_weight.h"
#include "coalsack_moe.h"

namespace coalsack {

// A: fp32 [*, M, K]; B: float16 or fp32 [*, N, K]; output fp32 [*, M, N] = A @ B.T   (:10-14)
class matmul_transpose_mixed_node : public binary_op_node {
 public:
  matmul_transpose_mixed_node() : binary_op_node("matmul_transpose_mixed") {}  // :17
  ~matmul_transpose_mixed_node() override = default;
  matmul_transpose_mixed_node(const matmul_transpose_mixed_node&) = delete;
  matmul_transpose_mixed_node& operator=(const matmul_transpose_mixed_node&) = delete;
  dynamic_tensor compute_test(const dynamic_tensor& a, const dynamic_tensor& b) { return compute(a, b); }  // :20-22
  // number of device copies made so far (tests: a changed weight must upload, a repeat must not)
  size_t resident_uploads() const { return uploads_; }

  // A batched weight keeps a device copy per matrix; more matrices than this are multiplied
  // through one slot that is refilled per matrix.
  static constexpr int64_t kMaxResidentMatrices = 64;

 protected:
  dynamic_tensor compute(const dynamic_tensor& a, const dynamic_tensor& b) override {  // :25-110
    if (a.get_dtype() != dtype::float32) throw std::runtime_error("matmul_transpose_mixed: input A must be fp32");
    if (b.get_dtype() != dtype::float32 && b.get_dtype() != dtype::float16)
      throw std::runtime_error("matmul_transpose_mixed: input B must be fp32 or fp16");
    if (a.ndim() < 2 || b.ndim() < 2) throw std::runtime_error("matmul_transpose_mixed: inputs must be at least 2D");
    const int64_t m = a.dim(-2), k = a.dim(-1), n = b.dim(-2);
    if (k != b.dim(-1)) throw std::runtime_error("matmul_transpose_mixed: incompatible dimensions");
    const std::vector<int64_t> a_batch(a.shape().begin(), a.shape().end() - 2);
    const std::vector<int64_t> b_batch(b.shape().begin(), b.shape().end() - 2);
    std::vector<int64_t> out_shape;
    if (!a_batch.empty() || !b_batch.empty()) out_shape = dynamic_tensor::broadcast_shape(a_batch, b_batch);  // :48-53
    int64_t batches = 1;
    for (int64_t d : out_shape) batches *= d;
    out_shape.push_back(m);
    out_shape.push_back(n);
    dynamic_tensor output(dtype::float32, out_shape);
    if (batches == 0 || m == 0 || n == 0) return output;
    if (k == 0) {  // empty sums
      std::fill_n(output.data_ptr<float>(), output.numel(), 0.0f);
      return output;
    }
    const int64_t n_a = a.numel() / (m * k), n_b = b.numel() / (n * k);
    const float* a_data = a.data_ptr<float>();
    float* out_data = output.data_ptr<float>();
    if (n_b == 1 && n_a == batches) {
      // one weight matrix for every batch entry (the engine's projections): all rows of A at once
      run(a_data, batches * m, k, weight(b, n, k, 0), out_data);
      return output;
    }
    // output matrix i pairs matrix i % n_a of A with matrix i % n_b of B (:76-78, :87-89)
    for (int64_t i = 0; i < batches; ++i)
      run(a_data + (i % n_a) * m * k, m, k, weight(b, n, k, i % n_b), out_data + i * m * n);
    return output;
  }

 private:
  void run(const float* a, int64_t rows, int64_t k, csk_f16* w, float* out) {
    if (csk_matmul_transpose_f16(a, rows, k, w, out) != CSK_OK)
      throw std::runtime_error(std::string("matmul_transpose_mixed: ") + csk_last_error());
  }
  csk_f16* weight(const dynamic_tensor& b, int64_t n, int64_t k, int64_t index) {
    const size_t slot = index < kMaxResidentMatrices ? (size_t)index : (size_t)kMaxResidentMatrices;
    if (resident_.size() <= slot) resident_.resize(slot + 1);
    return resident_[slot].get(b, n, k, index, "matmul_transpose_mixed", &uploads_);
  }
  std::vector<csk_resident::weight_slot> resident_;
  size_t uploads_ = 0;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::matmul_transpose_mixed_node, coalsack::graph_node)
