// matmul_transpose_mixed_node backed by the gfx950 library: same class name, test wrapper
// and error texts as include/coalsack/nn/nn_ops/matmul_transpose_mixed_node.h of the
// reference (cited by line below) for the case the engine uses it for -- a 2-D float16
// weight applied to fp32 activations (include/coalsack/llm/graph_builder.h:90-105); the
// product runs in csk_matmul_transpose_f16.  The weight is uploaded at the first sight of
// its storage pointer and cached per node.
#pragma once

#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "coalsack/nn/nn_op_node.h"
#include "coalsack_moe.h"

namespace coalsack {

// A: fp32 [*, M, K]; B: float16 [N, K]; output fp32 [*, M, N] = A @ B.T   (:10-14)
class matmul_transpose_mixed_node : public binary_op_node {
 public:
  matmul_transpose_mixed_node() : binary_op_node("matmul_transpose_mixed") {}  // :17
  ~matmul_transpose_mixed_node() override {
    for (auto& kv : resident_) csk_f16_free(kv.second.handle);
  }
  matmul_transpose_mixed_node(const matmul_transpose_mixed_node&) = delete;
  matmul_transpose_mixed_node& operator=(const matmul_transpose_mixed_node&) = delete;
  dynamic_tensor compute_test(const dynamic_tensor& a, const dynamic_tensor& b) { return compute(a, b); }  // :20-22

 protected:
  dynamic_tensor compute(const dynamic_tensor& a, const dynamic_tensor& b) override {  // :25-110
    if (a.get_dtype() != dtype::float32) throw std::runtime_error("matmul_transpose_mixed: input A must be fp32");
    if (b.get_dtype() != dtype::float32 && b.get_dtype() != dtype::float16)
      throw std::runtime_error("matmul_transpose_mixed: input B must be fp32 or fp16");
    if (a.ndim() < 2 || b.ndim() < 2) throw std::runtime_error("matmul_transpose_mixed: inputs must be at least 2D");
    const int64_t k = a.dim(a.ndim() - 1), n = b.dim(b.ndim() - 2);
    if (k != b.dim(b.ndim() - 1)) throw std::runtime_error("matmul_transpose_mixed: incompatible dimensions");
    // the reference also multiplies by fp32 and by batched weights (:54-57, :91-101); the
    // engine's projections have one float16 weight matrix
    if (b.get_dtype() != dtype::float16 || b.ndim() != 2)
      throw std::runtime_error("matmul_transpose_mixed: only a 2D fp16 input B is supported on this build");
    std::vector<int64_t> out_shape(a.shape().begin(), a.shape().end() - 1);
    out_shape.push_back(n);
    dynamic_tensor output(dtype::float32, out_shape);
    const int64_t rows = k ? a.numel() / k : 0;
    if (rows == 0 || n == 0) return output;
    const int rc = csk_matmul_transpose_f16(a.data_ptr<float>(), rows, k, resident_copy(b), output.data_ptr<float>());
    if (rc != CSK_OK) throw std::runtime_error(std::string("matmul_transpose_mixed: ") + csk_last_error());
    return output;
  }

 private:
  struct resident {
    csk_f16* handle;
    int64_t rows, cols;
  };
  csk_f16* resident_copy(const dynamic_tensor& t) {
    const uint16_t* key = t.data_ptr<uint16_t>();
    auto it = resident_.find(key);
    if (it != resident_.end() && it->second.rows == t.dim(0) && it->second.cols == t.dim(1))
      return it->second.handle;
    if (it != resident_.end()) {
      csk_f16_free(it->second.handle);
      resident_.erase(it);
    }
    csk_f16* h = nullptr;
    if (csk_f16_upload(key, t.dim(0), t.dim(1), &h) != CSK_OK)
      throw std::runtime_error(std::string("matmul_transpose_mixed: ") + csk_last_error());
    resident_[key] = resident{h, t.dim(0), t.dim(1)};
    return h;
  }
  std::unordered_map<const uint16_t*, resident> resident_;
};

}  // namespace coalsack

COALSACK_REGISTER_NODE(coalsack::matmul_transpose_mixed_node, coalsack::graph_node)
