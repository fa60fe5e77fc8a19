// C entry points around the reference's own GGUF readers, compiled from the reference
// tree where they lie (src/gguf/gguf_loader.cpp and gguf_multi_loader.cpp need nothing but
// the standard library).  TEST INFRASTRUCTURE: used only to check this repository's GGUF
// parser (csk_gguf_*) against the reference's view of the same files.
// Wraps gguf_loader::load / get_tensor_names / get_tensor_info / get_uint32 / get_string
// (include/coalsack/gguf/gguf_loader.h:21-62) and gguf_multi_loader
// (include/coalsack/gguf/gguf_multi_loader.h:24-63).
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "coalsack/gguf/gguf_loader.h"
#include "coalsack/gguf/gguf_multi_loader.h"

namespace {
struct ref_gguf {
  coalsack::gguf_loader one;
  coalsack::gguf_multi_loader many;
  bool multi = false;
  std::vector<std::string> names;
};
void copy_str(const std::string& s, char* buf, size_t cap) {
  if (!cap) return;
  const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
  std::memcpy(buf, s.data(), n);
  buf[n] = 0;
}
}  // namespace

extern "C" {
void* ref_gguf_open(const char* const* paths, int64_t n) {
  auto* g = new ref_gguf;
  bool ok;
  if (n == 1) {
    ok = g->one.load(paths[0]);
    if (ok) g->names = g->one.get_tensor_names();
  } else {
    g->multi = true;
    ok = g->many.load(std::vector<std::string>(paths, paths + n));
    if (ok) g->names = g->many.get_tensor_names();
  }
  if (!ok) {
    delete g;
    return nullptr;
  }
  return g;
}
void ref_gguf_close(void* h) { delete static_cast<ref_gguf*>(h); }
int64_t ref_gguf_tensor_count(void* h) {
  auto* g = static_cast<ref_gguf*>(h);
  return (int64_t)(g->multi ? g->many.get_tensor_count() : g->one.get_tensor_count());
}
uint32_t ref_gguf_version(void* h) {
  auto* g = static_cast<ref_gguf*>(h);
  return g->multi ? g->many.get_version() : g->one.get_version();
}
// names in the order the loader's own listing returns them (an unordered map: any order)
int ref_gguf_tensor_name(void* h, int64_t i, char* buf, size_t cap) {
  auto* g = static_cast<ref_gguf*>(h);
  if (i < 0 || i >= (int64_t)g->names.size()) return 1;
  copy_str(g->names[(size_t)i], buf, cap);
  return 0;
}
int ref_gguf_tensor_info(void* h, const char* name, uint32_t* type, int32_t* n_dims, uint64_t* dims4,
                         uint64_t* offset, uint64_t* size, int32_t* shard) {
  auto* g = static_cast<ref_gguf*>(h);
  std::vector<uint64_t> shape;
  if (g->multi) {
    auto t = g->many.get_tensor_info(name);
    if (!t) return 1;
    *type = (uint32_t)t->type, *offset = t->offset, *size = t->size, *shard = (int32_t)t->shard_idx;
    shape = t->shape;
  } else {
    auto t = g->one.get_tensor_info(name);
    if (!t) return 1;
    *type = (uint32_t)t->type, *offset = t->offset, *size = t->size, *shard = 0;
    shape = t->shape;
  }
  *n_dims = (int32_t)shape.size();
  for (size_t d = 0; d < 4; ++d) dims4[d] = d < shape.size() ? shape[d] : 1;
  return 0;
}
int ref_gguf_get_u32(void* h, const char* key, uint32_t* v) {
  auto* g = static_cast<ref_gguf*>(h);
  auto r = g->multi ? g->many.get_uint32(key) : g->one.get_uint32(key);
  if (!r) return 1;
  *v = *r;
  return 0;
}
int ref_gguf_get_str(void* h, const char* key, char* buf, size_t cap) {
  auto* g = static_cast<ref_gguf*>(h);
  auto r = g->multi ? g->many.get_string(key) : g->one.get_string(key);
  if (!r) return 1;
  copy_str(*r, buf, cap);
  return 0;
}
}
