// Stand-in for include/coalsack/tensor/dynamic_tensor.h:114-262: runtime-typed,
// row-major, contiguous host tensor whose copies share one byte buffer.
#pragma once
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <vector>

namespace coalsack {

enum class dtype { float32, float16, int64, int32, bool_, uint8, float64 };

inline size_t dtype_size(dtype dt) {
  switch (dt) {
    case dtype::float32: case dtype::int32: return 4;
    case dtype::float16: return 2;
    case dtype::int64: case dtype::float64: return 8;
    default: return 1;
  }
}

class dynamic_tensor {
  dtype dtype_ = dtype::float32;
  std::vector<int64_t> shape_;
  std::shared_ptr<std::vector<uint8_t>> bytes_;

 public:
  dynamic_tensor() : bytes_(std::make_shared<std::vector<uint8_t>>(dtype_size(dtype::float32))) {}
  dynamic_tensor(dtype dt, const std::vector<int64_t>& shape)
      : dtype_(dt), shape_(shape), bytes_(std::make_shared<std::vector<uint8_t>>(numel(shape) * dtype_size(dt))) {}
  dynamic_tensor(dtype dt, const std::vector<int64_t>& shape, const void* data) : dynamic_tensor(dt, shape) {
    if (data) std::memcpy(bytes_->data(), data, bytes_->size());
  }
  static int64_t numel(const std::vector<int64_t>& shape) {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
  }
  dtype get_dtype() const { return dtype_; }
  const std::vector<int64_t>& shape() const { return shape_; }
  int64_t ndim() const { return (int64_t)shape_.size(); }
  int64_t dim(int64_t i) const {
    if (i < 0) i += ndim();
    if (i < 0 || i >= ndim()) throw std::out_of_range("Dimension index out of range");
    return shape_[(size_t)i];
  }
  int64_t numel() const { return numel(shape_); }
  size_t bytes() const { return (size_t)numel() * dtype_size(dtype_); }
  template <class T>
  T* data_ptr() { return reinterpret_cast<T*>(bytes_->data()); }
  template <class T>
  const T* data_ptr() const { return reinterpret_cast<const T*>(bytes_->data()); }
  bool empty() const { return numel() == 0; }
  // :218-238
  static std::vector<int64_t> broadcast_shape(const std::vector<int64_t>& a, const std::vector<int64_t>& b) {
    const size_t nd = a.size() > b.size() ? a.size() : b.size();
    std::vector<int64_t> r(nd);
    for (size_t i = 0; i < nd; ++i) {
      const int64_t da = i < a.size() ? a[a.size() - 1 - i] : 1, db = i < b.size() ? b[b.size() - 1 - i] : 1;
      if (da != db && da != 1 && db != 1) throw std::invalid_argument("Incompatible shapes for broadcasting");
      r[nd - 1 - i] = (da == 0 || db == 0) ? 0 : (da > db ? da : db);
    }
    return r;
  }
};

}  // namespace coalsack
