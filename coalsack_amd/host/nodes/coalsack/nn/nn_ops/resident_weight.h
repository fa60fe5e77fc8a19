// Device-resident copies of the weight tensors a node is handed every frame.  No
// counterpart in the reference, whose nodes read weights from host memory in place.
//
// A node keeps one slot per weight role (and per matrix of a batched weight).  A slot
// remembers the tensor its copy was made from -- the tensor object shares the storage, so
// that storage cannot be freed and handed out again for other bytes while the slot holds
// it -- and a stamp of its contents (a hash of every byte unless the host opts for a
// sampled one, below); a tensor with another address, shape, element type or stamp
// replaces the copy, the old device memory is released.  A node therefore holds a bounded
// number of device copies whatever the weight provider evicts and reloads.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>

#include "coalsack/tensor/dynamic_tensor.h"
#include "coalsack_moe.h"

namespace coalsack {
namespace csk_resident {

// How a slot decides that the bytes behind an unchanged address are still the bytes its
// device copy was made from.
//   full    (default) every byte is hashed, every frame: exact.  The reference reads its host
//           weights anew on every frame, so a caller may rewrite a tensor in place between
//           two frames -- a patched weight, a provider that recycles a slot for another
//           expert's slice -- and must get the new values.  Costs one pass over the weights
//           at memory speed (about 0.3 ms per 4.4 MB matrix on one core).
//   sampled 64 eight-byte samples spread over the buffer, its length and its ends: for hosts
//           whose weight tensors are never rewritten in place -- the reference's own
//           moe_weight_provider is one: every load is a fresh tensor, and the slot keeps the
//           old storage alive, so a new slice cannot appear at an old address.  A rewrite
//           that misses all the samples goes unnoticed.  Chosen per process with
//           set_content_check(content_check::sampled) or COALSACK_RESIDENT_CHECK=sampled.
enum class content_check { full, sampled };

inline content_check& content_check_policy() {
  static content_check policy = [] {
    const char* e = std::getenv("COALSACK_RESIDENT_CHECK");
    return e && std::string(e) == "sampled" ? content_check::sampled : content_check::full;
  }();
  return policy;
}
inline void set_content_check(content_check c) { content_check_policy() = c; }

inline uint64_t sampled_stamp(const uint8_t* p, size_t n) {
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

// Every byte: four independent multiply-xor lanes over 32-byte strides (the lanes keep four
// multiplications in flight, which is what lets one core run this at memory speed), folded
// together with the length and the tail.
inline uint64_t full_hash(const uint8_t* p, size_t n) {
  uint64_t a = 0x9E3779B97F4A7C15ull ^ n, b = 0xBF58476D1CE4E5B9ull, c = 0x94D049BB133111EBull, d = 0xD6E8FEB86659FD93ull;
  size_t i = 0;
  for (; i + 32 <= n; i += 32) {
    uint64_t v[4];
    std::memcpy(v, p + i, 32);
    a = (a ^ v[0]) * 0x9FB21C651E98DF25ull;
    b = (b ^ v[1]) * 0xC2B2AE3D27D4EB4Full;
    c = (c ^ v[2]) * 0x165667B19E3779F9ull;
    d = (d ^ v[3]) * 0x27D4EB2F165667C5ull;
    a ^= a >> 29, b ^= b >> 31, c ^= c >> 30, d ^= d >> 28;
  }
  uint64_t t = 0;
  for (int sh = 0; i < n; ++i, sh = (sh + 8) & 63) t ^= (uint64_t)p[i] << sh, t *= 0x9E3779B97F4A7C15ull;
  uint64_t h = a ^ (b << 1 | b >> 63) ^ (c << 2 | c >> 62) ^ (d << 3 | d >> 61) ^ t;
  h ^= h >> 33, h *= 0xFF51AFD7ED558CCDull, h ^= h >> 33;
  return h;
}

inline uint64_t content_stamp(const uint8_t* p, size_t n) {
  return content_check_policy() == content_check::full ? full_hash(p, n) : sampled_stamp(p, n);
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
