// Stand-in for include/coalsack/tensor/dynamic_mx_tensor.h:19-110: MXFP4
// storage, ceil(numel / 32) blocks of 17 bytes (scale byte + 16 packed nibbles).
#pragma once
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <vector>

namespace coalsack {

class dynamic_mx_tensor {
  std::vector<int64_t> shape_;
  size_t num_elements_ = 0;
  std::shared_ptr<std::vector<uint8_t>> blocks_;

 public:
  static constexpr size_t ELEMENTS_PER_BLOCK = 32, BYTES_PER_BLOCK = 17;
  dynamic_mx_tensor() = default;
  explicit dynamic_mx_tensor(const std::vector<int64_t>& shape) : shape_(shape) {
    num_elements_ = 1;
    for (int64_t d : shape) {
      if (d < 0) throw std::invalid_argument("dynamic_mx_tensor: negative dimension");
      num_elements_ *= (size_t)d;
    }
    blocks_ = std::make_shared<std::vector<uint8_t>>(num_blocks_for(num_elements_) * BYTES_PER_BLOCK);
  }
  static size_t num_blocks_for(size_t n) { return (n + ELEMENTS_PER_BLOCK - 1) / ELEMENTS_PER_BLOCK; }
  size_t ndim() const { return shape_.size(); }
  int64_t dim(size_t i) const {
    if (i >= shape_.size()) throw std::out_of_range("dynamic_mx_tensor: dimension index out of range");
    return shape_[i];
  }
  const std::vector<int64_t>& shape() const { return shape_; }
  size_t num_elements() const { return num_elements_; }
  size_t size_bytes() const { return blocks_ ? blocks_->size() : 0; }
  size_t num_blocks() const { return size_bytes() / BYTES_PER_BLOCK; }
  uint8_t* data_ptr() {
    if (!blocks_) throw std::runtime_error("dynamic_mx_tensor: null storage");
    return blocks_->data();
  }
  const uint8_t* data_ptr() const {
    if (!blocks_) throw std::runtime_error("dynamic_mx_tensor: null storage");
    return blocks_->data();
  }
};

}  // namespace coalsack
