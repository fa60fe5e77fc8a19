// Device-resident copies of the weight tensors a node is handed every frame.  No
// counterpart in the reference, whose nodes read weights from host memory in place.
//
// A node keeps one slot per weight role (and per matrix of a batched weight).  A slot
// remembers the tensor its copy was made from -- the tensor object shares the storage, so
// that storage cannot be freed and handed out again for other bytes while the slot holds
// it -- and a stamp of its contents; a tensor with another address, shape, element type or
// stamp replaces the copy, the old device memory is released.  A node therefore holds a
// bounded number of device copies whatever the weight provider evicts and reloads.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>

#include "coalsack/tensor/dynamic_tensor.h"
#include "coalsack_moe.h"

namespace coalsack {
namespace csk_resident {

// 64 eight-byte samples spread over the buffer, its length and its ends: enough to tell a
// rewritten or reused buffer from the one a device copy was made from, at no cost that matters
inline uint64_t content_stamp(const uint8_t* p, size_t n) {
  uint64_t h = 0x9E3779B97F4A7C15ull ^ n;
  auto mix = [&h](uint64_t v) {
    h ^= v + 0x9E3779B97F4A7C15ull + (h << 6) + (h >> 2);
    h *= 0xBF58476D1CE4E5B9ull;
  };
  if (n < 8) {
    for (size_t i = 0; i < n; ++i) mix(p[i]);
    return h;
  }
  const size_t step = (n - 8) / 63 ? (n - 8) / 63 : 1;
  for (size_t off = 0; off + 8 <= n; off += step) {
    uint64_t v;
    std::memcpy(&v, p + off, 8);
    mix(v);
  }
  uint64_t v;
  std::memcpy(&v, p + n - 8, 8);
  mix(v);
  return h;
}

// One [rows, cols] float16 or float32 matrix, `index` matrices into the tensor's data.
class weight_slot {
 public:
  weight_slot() = default;
  weight_slot(const weight_slot&) = delete;
  weight_slot& operator=(const weight_slot&) = delete;
  weight_slot(weight_slot&& o) noexcept : handle_(o.handle_), held_(o.held_), index_(o.index_), stamp_(o.stamp_) {
    o.handle_ = nullptr;
  }
  ~weight_slot() {
    if (handle_) csk_f16_free(handle_);
  }

  // `who` prefixes the error text ("dense_ffn", "matmul_transpose_mixed")
  csk_f16* get(const dynamic_tensor& t, int64_t rows, int64_t cols, int64_t index, const char* who,
               size_t* uploads = nullptr) {
    const bool f32 = t.get_dtype() == dtype::float32;
    const size_t esz = f32 ? 4 : 2, bytes = (size_t)rows * (size_t)cols * esz;
    const uint8_t* base = reinterpret_cast<const uint8_t*>(t.data_ptr<uint8_t>()) + (size_t)index * bytes;
    const uint64_t stamp = content_stamp(base, bytes);
    if (handle_ && held_.data_ptr<uint8_t>() == t.data_ptr<uint8_t>() && held_.get_dtype() == t.get_dtype() &&
        held_.shape() == t.shape() && index_ == index && stamp_ == stamp)
      return handle_;
    csk_f16* h = nullptr;
    const int rc = f32 ? csk_f16_upload_f32(reinterpret_cast<const float*>(base), rows, cols, &h)
                       : csk_f16_upload(reinterpret_cast<const uint16_t*>(base), rows, cols, &h);
    if (rc != CSK_OK) throw std::runtime_error(std::string(who) + ": " + csk_last_error());
    if (handle_) csk_f16_free(handle_);
    handle_ = h;
    held_ = t;
    index_ = index;
    stamp_ = stamp;
    if (uploads) ++*uploads;
    return h;
  }

 private:
  csk_f16* handle_ = nullptr;
  dynamic_tensor held_;
  int64_t index_ = 0;
  uint64_t stamp_ = 0;
};

// A whole tensor kept as it is in device memory (the router's gate and bias): the same
// rule -- the slot holds the tensor it copied and a stamp of its contents; another address,
// shape, element type or stamp replaces the copy.
class array_slot {
 public:
  array_slot() = default;
  array_slot(const array_slot&) = delete;
  array_slot& operator=(const array_slot&) = delete;
  ~array_slot() {
    if (dev_) csk_dev_free(dev_);
  }

  // device address of t's bytes; `who` prefixes the error text
  const void* get(const dynamic_tensor& t, const char* who, size_t* uploads = nullptr) {
    const uint8_t* base = t.data_ptr<uint8_t>();
    const size_t bytes = t.bytes();
    const uint64_t stamp = content_stamp(base, bytes);
    if (dev_ && held_.data_ptr<uint8_t>() == base && held_.get_dtype() == t.get_dtype() &&
        held_.shape() == t.shape() && stamp_ == stamp)
      return dev_;
    void* d = csk_dev_alloc(bytes ? bytes : 1);
    if (!d) throw std::runtime_error(std::string(who) + ": " + csk_last_error());
    if (csk_copy_h2d(d, base, bytes) != CSK_OK) {
      csk_dev_free(d);
      throw std::runtime_error(std::string(who) + ": " + csk_last_error());
    }
    if (dev_) csk_dev_free(dev_);
    dev_ = d;
    held_ = t;
    stamp_ = stamp;
    if (uploads) ++*uploads;
    return d;
  }

 private:
  void* dev_ = nullptr;
  dynamic_tensor held_;
  uint64_t stamp_ = 0;
};

}  // namespace csk_resident
}  // namespace coalsack
