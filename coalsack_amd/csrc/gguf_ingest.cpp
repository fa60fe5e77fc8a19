// GGUF ingest for the MoE path: parses a GGUF file's metadata and tensor table and
// builds a resident MoE layer (router, MXFP4 or F16 / Q4_K / Q6_K experts, biases, FFN norm) for one
// transformer block through the public C ABI.  Host-only code.
//
// Follows the reference's reader and weight provider:
//   src/gguf/gguf_loader.cpp:383-518   header, key/value section, tensor infos, data start
//   src/gguf/gguf_loader.cpp:228-378   value encodings
//   src/llm/moe_weight_provider.cpp:75-225  expert slice = tensor offset + e * slice bytes,
//                                           shape reversal (GGUF lists the fastest dim first)
//   src/llm/llm_engine.cpp:135-225, 262-267, 714-753  architecture keys and tensor names
//   src/gguf/gguf_multi_loader.cpp:25-76  split checkpoints: shards in order, duplicate names refused
// Differences: every scalar array type is accepted (the reference rejects some), and
// general.alignment is honoured when present (the reference assumes 32, the default).
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "coalsack_moe.h"

extern "C" void csk_set_error_(const char* msg);  // capi.hip: sets the per-thread message

namespace {

constexpr uint32_t kMagic = 0x46554747u;  // "GGUF"
enum : uint32_t { T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 };
constexpr uint32_t kGgmlF32 = 0, kGgmlF16 = 1, kGgmlQ4K = 12, kGgmlQ6K = 14, kGgmlMxfp4 = 39;

int fail(int code, const std::string& msg) {
  csk_set_error_(msg.c_str());
  return code;
}

size_t scalar_size(uint32_t t) {
  switch (t) {
    case T_U8: case T_I8: case T_BOOL: return 1;
    case T_U16: case T_I16: return 2;
    case T_U32: case T_I32: case T_F32: return 4;
    case T_U64: case T_I64: case T_F64: return 8;
    default: return 0;
  }
}

struct TensorInfo {
  uint32_t type = 0;
  std::vector<uint64_t> dims;  // GGUF order: fastest-varying first
  uint64_t offset = 0;         // absolute offset in its shard's file
  uint64_t nbytes = 0;
  uint32_t shard = 0;          // which file of a split checkpoint
};

struct Value {
  uint32_t type = 0;
  uint64_t u = 0;
  int64_t i = 0;
  double f = 0;
  std::string s;
};

}  // namespace

// One file of a checkpoint.
struct GgufShard {
  FILE* fp = nullptr;
  const uint8_t* map = nullptr;  // the file mapped read-only (tensor data is handed to the GPU copies from here); null: fread
  size_t map_len = 0;
  uint32_t version = 0;
  uint64_t data_start = 0, file_size = 0;
};

// A checkpoint: one file, or the shards of a split one merged the way gguf_multi_loader
// does (src/gguf/gguf_multi_loader.cpp:25-76): tensors keep the shard they came from, a
// metadata key is answered by the first shard that has it.
struct csk_gguf {
  std::vector<GgufShard> shards;
  std::unordered_map<std::string, Value> meta;
  std::unordered_map<std::string, TensorInfo> tensors;
  std::vector<std::string> order;
};

namespace {

bool rd(FILE* fp, void* p, size_t n) { return fread(p, 1, n, fp) == n; }

bool rd_str(FILE* fp, std::string& s, uint64_t limit) {
  uint64_t len;
  if (!rd(fp, &len, 8) || len > limit) return false;
  s.resize(len);
  return len == 0 || rd(fp, &s[0], len);
}

// ggml block geometry of the types this path can meet (gguf_loader.cpp:101-200)
bool type_geometry(uint32_t t, uint64_t* block_elems, uint64_t* block_bytes) {
  switch (t) {
    case kGgmlF32: *block_elems = 1, *block_bytes = 4; return true;
    case kGgmlF16: *block_elems = 1, *block_bytes = 2; return true;
    case 2: *block_elems = 32, *block_bytes = 18; return true;    // Q4_0
    case 3: *block_elems = 32, *block_bytes = 20; return true;    // Q4_1
    case 6: *block_elems = 32, *block_bytes = 22; return true;    // Q5_0
    case 7: *block_elems = 32, *block_bytes = 24; return true;    // Q5_1
    case 8: *block_elems = 32, *block_bytes = 34; return true;    // Q8_0
    case 12: *block_elems = 256, *block_bytes = 144; return true;  // Q4_K
    case 13: *block_elems = 256, *block_bytes = 176; return true;  // Q5_K
    case 14: *block_elems = 256, *block_bytes = 210; return true;  // Q6_K
    case 24: *block_elems = 1, *block_bytes = 1; return true;     // I8
    case 25: *block_elems = 1, *block_bytes = 2; return true;     // I16
    case 26: *block_elems = 1, *block_bytes = 4; return true;     // I32
    case 27: *block_elems = 1, *block_bytes = 8; return true;     // I64
    case 28: *block_elems = 1, *block_bytes = 8; return true;     // F64
    case 30: *block_elems = 1, *block_bytes = 2; return true;     // BF16
    case kGgmlMxfp4: *block_elems = 32, *block_bytes = 17; return true;
    default: return false;
  }
}

int read_value(FILE* fp, uint32_t type, Value& v, uint64_t file_size) {
  v.type = type;
  switch (type) {
    case T_U8: { uint8_t x; if (!rd(fp, &x, 1)) return 1; v.u = x; v.i = x; return 0; }
    case T_I8: { int8_t x; if (!rd(fp, &x, 1)) return 1; v.i = x; v.u = (uint64_t)x; return 0; }
    case T_U16: { uint16_t x; if (!rd(fp, &x, 2)) return 1; v.u = x; v.i = x; return 0; }
    case T_I16: { int16_t x; if (!rd(fp, &x, 2)) return 1; v.i = x; v.u = (uint64_t)x; return 0; }
    case T_U32: { uint32_t x; if (!rd(fp, &x, 4)) return 1; v.u = x; v.i = x; return 0; }
    case T_I32: { int32_t x; if (!rd(fp, &x, 4)) return 1; v.i = x; v.u = (uint64_t)x; return 0; }
    case T_F32: { float x; if (!rd(fp, &x, 4)) return 1; v.f = x; return 0; }
    case T_BOOL: { uint8_t x; if (!rd(fp, &x, 1)) return 1; v.u = x != 0; v.i = (int64_t)v.u; return 0; }
    case T_U64: { uint64_t x; if (!rd(fp, &x, 8)) return 1; v.u = x; v.i = (int64_t)x; return 0; }
    case T_I64: { int64_t x; if (!rd(fp, &x, 8)) return 1; v.i = x; v.u = (uint64_t)x; return 0; }
    case T_F64: { double x; if (!rd(fp, &x, 8)) return 1; v.f = x; return 0; }
    case T_STR: return rd_str(fp, v.s, file_size) ? 0 : 1;
    case T_ARR: {
      // arrays (tokenizer tables, ...) are not needed on this path: skipped, length kept
      uint32_t et;
      uint64_t n;
      if (!rd(fp, &et, 4) || !rd(fp, &n, 8)) return 1;
      v.u = n;
      if (et == T_STR) {
        std::string tmp;
        for (uint64_t i = 0; i < n; ++i)
          if (!rd_str(fp, tmp, file_size)) return 1;
        return 0;
      }
      const size_t es = scalar_size(et);
      if (es == 0 || n > file_size / es) return 2;
      return fseeko(fp, (off_t)(n * es), SEEK_CUR) == 0 ? 0 : 1;
    }
    default: return 2;
  }
}

const TensorInfo* find(const csk_gguf* g, const std::string& name) {
  auto it = g->tensors.find(name);
  return it == g->tensors.end() ? nullptr : &it->second;
}

// [off, off + n) lies inside a file of `size` bytes (no sum that could wrap)
bool in_file(uint64_t off, uint64_t n, uint64_t size) { return off <= size && n <= size - off; }

bool read_at(GgufShard& sh, uint64_t off, void* dst, size_t n) {
  if (!in_file(off, n, sh.file_size)) return false;
  if (fseeko(sh.fp, (off_t)off, SEEK_SET) != 0) return false;
  return rd(sh.fp, dst, n);
}

// n bytes of the file at off without a copy: a pointer into the read-only mapping (made at
// the first call), or, where the file cannot be mapped, into `fallback` filled by fread.
const uint8_t* view_at(GgufShard& sh, uint64_t off, size_t n, std::vector<uint8_t>& fallback) {
  if (!in_file(off, n, sh.file_size)) return nullptr;
  if (!sh.map && sh.map_len == 0) {
    void* m = mmap(nullptr, (size_t)sh.file_size, PROT_READ, MAP_PRIVATE, fileno(sh.fp), 0);
    sh.map_len = (size_t)sh.file_size;  // also marks the attempt
    if (m != MAP_FAILED) sh.map = static_cast<const uint8_t*>(m);
  }
  if (sh.map) return sh.map + off;
  fallback.resize(n);
  return read_at(sh, off, fallback.data(), n) ? fallback.data() : nullptr;
}

// the slice [rel, rel + n) of tensor t, checked against the tensor's own extent
bool slice_in_tensor(const TensorInfo& t, uint64_t rel, uint64_t n) { return in_file(rel, n, t.nbytes); }

}  // namespace

namespace {
// Parses one file into shard `idx` of g (header, key/value section, tensor table).
int parse_shard(csk_gguf* g, uint32_t idx, const char* path) {
  FILE* fp = fopen(path, "rb");
  if (!fp) return fail(CSK_ERR_ARG, std::string("csk_gguf_open: cannot open ") + path);
  g->shards.emplace_back();
  GgufShard& sh = g->shards.back();
  sh.fp = fp;
  auto bad = [&](const std::string& why) { return fail(CSK_ERR_ARG, "csk_gguf_open: " + why); };
  fseeko(fp, 0, SEEK_END);
  sh.file_size = (uint64_t)ftello(fp);
  fseeko(fp, 0, SEEK_SET);
  uint32_t magic = 0;
  uint64_t n_tensors = 0, n_kv = 0;
  if (!rd(fp, &magic, 4) || magic != kMagic) return bad("not a GGUF file (bad magic)");
  if (!rd(fp, &sh.version, 4) || sh.version < 2 || sh.version > 3) return bad("unsupported GGUF version");
  if (!rd(fp, &n_tensors, 8) || !rd(fp, &n_kv, 8)) return bad("truncated header");
  if (n_tensors > sh.file_size || n_kv > sh.file_size) return bad("implausible header counts");
  std::unordered_map<std::string, Value> meta;
  for (uint64_t i = 0; i < n_kv; ++i) {
    std::string key;
    uint32_t type;
    if (!rd_str(fp, key, sh.file_size) || !rd(fp, &type, 4)) return bad("truncated metadata");
    Value v;
    const int r = read_value(fp, type, v, sh.file_size);
    if (r == 1) return bad("truncated metadata value of '" + key + "'");
    if (r == 2) return bad("unknown metadata type of '" + key + "'");
    meta[key] = std::move(v);
  }
  std::vector<std::string> names;
  for (uint64_t i = 0; i < n_tensors; ++i) {
    std::string name;
    uint32_t nd;
    TensorInfo ti;
    if (!rd_str(fp, name, sh.file_size) || !rd(fp, &nd, 4) || nd > 4) return bad("truncated tensor table");
    ti.dims.resize(nd);
    for (uint32_t d = 0; d < nd; ++d)
      if (!rd(fp, &ti.dims[d], 8)) return bad("truncated tensor table");
    if (!rd(fp, &ti.type, 4) || !rd(fp, &ti.offset, 8)) return bad("truncated tensor table");
    uint64_t ne = 1, be = 1, bb = 0;
    for (uint64_t d : ti.dims)
      if (__builtin_mul_overflow(ne, d, &ne)) return bad("tensor '" + name + "': element count overflows");
    if (type_geometry(ti.type, &be, &bb)) {
      const uint64_t blocks = ne / be + (ne % be != 0);
      if (__builtin_mul_overflow(blocks, bb, &ti.nbytes)) return bad("tensor '" + name + "': size overflows");
    }
    ti.shard = idx;
    if (g->tensors.count(name))  // gguf_multi_loader.cpp:64-67
      return bad("Duplicate tensor name '" + name + "' in shard " + std::to_string(idx));
    names.push_back(name);
    g->tensors[name] = std::move(ti);
  }
  uint64_t align = 32;
  auto it = meta.find("general.alignment");
  if (it != meta.end() && it->second.u >= 1 && it->second.u <= (1u << 20)) align = it->second.u;
  const uint64_t pos = (uint64_t)ftello(fp);
  sh.data_start = (pos + align - 1) / align * align;
  for (const std::string& name : names) {
    TensorInfo& ti = g->tensors[name];
    // relative offset -> absolute; both the sum and the tensor's end are checked without wrapping
    if (sh.data_start > sh.file_size || ti.offset > sh.file_size - sh.data_start ||
        !in_file(ti.offset + sh.data_start, ti.nbytes, sh.file_size))
      return bad("tensor '" + name + "' reaches past the end of the file");
    ti.offset += sh.data_start;
    g->order.push_back(name);
  }
  for (auto& kv : meta)  // a key is answered by the first shard that has it (gguf_multi_loader.cpp:86-92)
    if (!g->meta.count(kv.first)) g->meta[kv.first] = std::move(kv.second);
  return CSK_OK;
}
}  // namespace

extern "C" int csk_gguf_open_shards(const char* const* paths, int64_t n_paths, csk_gguf** out) {
  if (!paths || !out || n_paths < 1) return fail(CSK_ERR_ARG, "csk_gguf_open: No GGUF files specified");
  *out = nullptr;
  csk_gguf* g = new csk_gguf;
  g->shards.reserve((size_t)n_paths);
  for (int64_t i = 0; i < n_paths; ++i) {
    const int rc = paths[i] ? parse_shard(g, (uint32_t)i, paths[i]) : fail(CSK_ERR_ARG, "csk_gguf_open: null path");
    if (rc != CSK_OK) {
      csk_gguf_close(g);
      return rc;
    }
  }
  *out = g;
  return CSK_OK;
}

extern "C" int csk_gguf_open(const char* path, csk_gguf** out) {
  if (!path || !out) return fail(CSK_ERR_ARG, "csk_gguf_open: null argument");
  return csk_gguf_open_shards(&path, 1, out);
}

extern "C" void csk_gguf_close(csk_gguf* g) {
  if (!g) return;
  for (GgufShard& sh : g->shards) {
    if (sh.map) munmap(const_cast<uint8_t*>(sh.map), sh.map_len);
    if (sh.fp) fclose(sh.fp);
  }
  delete g;
}

extern "C" int csk_gguf_tensor_count(const csk_gguf* g, int64_t* n) {
  if (!g || !n) return fail(CSK_ERR_ARG, "csk_gguf_tensor_count: null argument");
  *n = (int64_t)g->order.size();
  return CSK_OK;
}

extern "C" int csk_gguf_tensor_name(const csk_gguf* g, int64_t index, char* buf, size_t cap) {
  if (!g || !buf || cap == 0) return fail(CSK_ERR_ARG, "csk_gguf_tensor_name: null argument");
  if (index < 0 || index >= (int64_t)g->order.size()) return fail(CSK_ERR_ARG, "csk_gguf_tensor_name: index out of range");
  snprintf(buf, cap, "%s", g->order[index].c_str());
  return CSK_OK;
}

extern "C" int csk_gguf_tensor_info(const csk_gguf* g, const char* name, uint32_t* ggml_type,
                                    int32_t* n_dims, uint64_t* dims4, uint64_t* file_offset,
                                    uint64_t* nbytes) {
  if (!g || !name) return fail(CSK_ERR_ARG, "csk_gguf_tensor_info: null argument");
  const TensorInfo* t = find(g, name);
  if (!t) return fail(CSK_ERR_ARG, std::string("Tensor not found: ") + name);
  if (ggml_type) *ggml_type = t->type;
  if (n_dims) *n_dims = (int32_t)t->dims.size();
  if (dims4)
    for (size_t d = 0; d < 4; ++d) dims4[d] = d < t->dims.size() ? t->dims[d] : 1;
  if (file_offset) *file_offset = t->offset;
  if (nbytes) *nbytes = t->nbytes;
  return CSK_OK;
}

extern "C" int csk_gguf_tensor_shard(const csk_gguf* g, const char* name, int32_t* shard) {
  if (!g || !name || !shard) return fail(CSK_ERR_ARG, "csk_gguf_tensor_shard: null argument");
  const TensorInfo* t = find(g, name);
  if (!t) return fail(CSK_ERR_ARG, std::string("Tensor not found: ") + name);
  *shard = (int32_t)t->shard;
  return CSK_OK;
}

extern "C" int csk_gguf_get_u32(const csk_gguf* g, const char* key, uint32_t* value) {
  if (!g || !key || !value) return fail(CSK_ERR_ARG, "csk_gguf_get_u32: null argument");
  auto it = g->meta.find(key);
  if (it == g->meta.end()) return fail(CSK_ERR_ARG, std::string("Missing required parameter: ") + key);
  const uint32_t t = it->second.type;
  if (t == T_F32 || t == T_F64 || t == T_STR || t == T_ARR)
    return fail(CSK_ERR_ARG, std::string("metadata key is not an integer: ") + key);
  *value = (uint32_t)it->second.u;
  return CSK_OK;
}

extern "C" int csk_gguf_get_str(const csk_gguf* g, const char* key, char* buf, size_t cap) {
  if (!g || !key || !buf || cap == 0) return fail(CSK_ERR_ARG, "csk_gguf_get_str: null argument");
  auto it = g->meta.find(key);
  if (it == g->meta.end() || it->second.type != T_STR)
    return fail(CSK_ERR_ARG, std::string("Missing string parameter: ") + key);
  snprintf(buf, cap, "%s", it->second.s.c_str());
  return CSK_OK;
}

extern "C" int csk_layer_from_gguf(csk_gguf* g, int64_t block, csk_layer** out) {
  if (!g || !out || block < 0) return fail(CSK_ERR_ARG, "csk_layer_from_gguf: bad argument");
  *out = nullptr;
  // architecture and its switches (llm_engine.cpp:135-161)
  std::string arch = "gpt-oss";
  auto ia = g->meta.find("general.architecture");
  if (ia != g->meta.end() && ia->second.type == T_STR) arch = ia->second.s;
  const bool llama4 = arch == "llama4";
  const std::string norm_name = llama4 ? "ffn_norm.weight" : "post_attention_norm.weight";
  uint32_t E = 32, k = 4;  // the reference's defaults (llm_engine.cpp:62-63)
  uint32_t v;
  if (csk_gguf_get_u32(g, (arch + ".expert_count").c_str(), &v) == CSK_OK) E = v;
  if (csk_gguf_get_u32(g, (arch + ".expert_used_count").c_str(), &v) == CSK_OK) k = v;
  const std::string p = "blk." + std::to_string(block);

  const TensorInfo* tg = find(g, p + ".ffn_gate_inp.weight");
  if (!tg) return fail(CSK_ERR_ARG, "Tensor not found: " + p + ".ffn_gate_inp.weight");
  if (tg->type != kGgmlF32 || tg->dims.size() != 2)
    return fail(CSK_ERR_ARG, p + ".ffn_gate_inp.weight: expected a 2-D F32 tensor");
  const uint64_t H = tg->dims[0];
  if (tg->dims[1] != E) return fail(CSK_ERR_ARG, p + ".ffn_gate_inp.weight: expert count differs from the metadata");

  const char* wn[3] = {".ffn_up_exps.weight", ".ffn_gate_exps.weight", ".ffn_down_exps.weight"};
  const char* bn[3] = {".ffn_up_exps.bias", ".ffn_gate_exps.bias", ".ffn_down_exps.bias"};
  const TensorInfo* tw[3];
  const TensorInfo* tb[3];
  uint64_t F = 0;
  for (int i = 0; i < 3; ++i) {
    tw[i] = find(g, p + wn[i]);
    if (!tw[i]) return fail(CSK_ERR_ARG, "Tensor not found: " + p + wn[i]);
    const uint32_t ty = tw[i]->type;
    if (ty != kGgmlMxfp4 && ty != kGgmlF16 && ty != kGgmlQ4K && ty != kGgmlQ6K)
      return fail(CSK_ERR_ARG, p + wn[i] + ": only MXFP4, F16, Q4_K and Q6_K expert weights are supported on this path");
    // the node decides between its two branches by the kind of w_up alone
    // (expert_mlp_node.h:113-117), so MXFP4 cannot be mixed with the fp16 kinds
    if ((ty == kGgmlMxfp4) != (tw[0]->type == kGgmlMxfp4))
      return fail(CSK_ERR_ARG, p + ": expert tensors must be all MXFP4, or each of F16 / Q4_K / Q6_K");
    if (tw[i]->dims.size() != 3 || tw[i]->dims[2] != E)
      return fail(CSK_ERR_ARG, p + wn[i] + ": expected [K, rows, experts]");
    tb[i] = find(g, p + bn[i]);
    if (tb[i] && (tb[i]->type != kGgmlF32 || tb[i]->dims.size() != 2 || tb[i]->dims[1] != E ||
                  tb[i]->dims[0] != tw[i]->dims[1]))
      return fail(CSK_ERR_ARG, p + bn[i] + ": expected F32 [rows, experts]");
  }
  F = tw[0]->dims[1];
  if (tw[0]->dims[0] != H || tw[1]->dims[0] != H || tw[1]->dims[1] != F || tw[2]->dims[0] != F ||
      tw[2]->dims[1] != H)
    return fail(CSK_ERR_ARG, p + ": expert tensor shapes are inconsistent");
  if ((tb[0] != nullptr) != (tb[1] != nullptr) || (tb[0] != nullptr) != (tb[2] != nullptr))
    return fail(CSK_ERR_ARG, p + ": expert biases must be all present or all absent");

  // F16 expert tensors take the node's float16 branch (expert_mlp_node.h:269-389)
  const bool f16 = tw[0]->type != kGgmlMxfp4;
  csk_layer* L = nullptr;
  int rc = f16 ? csk_layer_create_f16(E, k, (int64_t)H, (int64_t)F, &L)
               : csk_layer_create(E, k, (int64_t)H, (int64_t)F, &L);
  if (rc != CSK_OK) return rc;
  auto bail = [&](int code, const std::string& msg) {
    csk_layer_destroy(L);
    return msg.empty() ? code : fail(code, msg);
  };
  // gpt-oss: softmax gating, modified SwiGLU, weights applied at the merge;
  // llama4: sigmoid gating, routing weight applied before the FFN (llm_engine.cpp:145-161);
  // every architecture but gpt-oss gets the standard SwiGLU (llm_engine.cpp:738-740)
  rc = csk_layer_set_options(L, llama4 ? 1 : 0,
                             arch == "gpt-oss" ? CSK_ACT_MODIFIED_SWIGLU : CSK_ACT_STANDARD_SWIGLU,
                             llama4 ? 1 : 0);
  if (rc != CSK_OK) return bail(rc, "");

  std::vector<float> gw((size_t)E * H), gb;
  if (!slice_in_tensor(*tg, 0, gw.size() * 4) || !read_at(g->shards[tg->shard], tg->offset, gw.data(), gw.size() * 4)) return bail(CSK_ERR_ARG, "short read: " + p + ".ffn_gate_inp.weight");
  const TensorInfo* tgb = find(g, p + ".ffn_gate_inp.bias");
  if (tgb) {
    if (tgb->type != kGgmlF32 || tgb->dims.size() != 1 || tgb->dims[0] != E)
      return bail(CSK_ERR_ARG, p + ".ffn_gate_inp.bias: expected F32 [experts]");
    gb.resize(E);
    if (!read_at(g->shards[tgb->shard], tgb->offset, gb.data(), (size_t)E * 4)) return bail(CSK_ERR_ARG, "short read: " + p + ".ffn_gate_inp.bias");
  }
  rc = csk_layer_set_router(L, gw.data(), tgb ? gb.data() : nullptr);
  if (rc != CSK_OK) return bail(rc, "");

  // expert e of a stacked tensor starts at offset + e * slice bytes (moe_weight_provider.cpp:160-188)
  // (one expert's K-quant slice is a whole number of super-blocks: moe_weight_provider.cpp:136-141)
  auto slice_bytes = [&](uint32_t ty, uint64_t rows, uint64_t K) -> size_t {
    const uint64_t n = rows * K;
    switch (ty) {
      case kGgmlF16: return (size_t)(n * 2);
      case kGgmlQ4K: return (size_t)((n + 255) / 256 * 144);
      case kGgmlQ6K: return (size_t)((n + 255) / 256 * 210);
      default: return (size_t)(rows * (K / 32) * 17);
    }
  };
  const size_t sl[3] = {slice_bytes(tw[0]->type, F, H), slice_bytes(tw[1]->type, F, H),
                        slice_bytes(tw[2]->type, H, F)};
  if (f16 && (F * H) % 256 != 0)
    for (int i = 0; i < 3; ++i)
      if (tw[i]->type == kGgmlQ4K || tw[i]->type == kGgmlQ6K)
        return bail(CSK_ERR_ARG, p + wn[i] + ": a K-quant expert slice must be a multiple of 256 values");
  const size_t bl[3] = {(size_t)F, (size_t)F, (size_t)H};
  std::vector<uint8_t> w[3];  // used only where the file cannot be mapped
  std::vector<float> b[3];
  for (int i = 0; i < 3; ++i)
    if (tb[i]) b[i].resize(bl[i]);
  for (uint32_t e = 0; e < E; ++e) {
    const uint8_t* wp[3];
    for (int i = 0; i < 3; ++i) {
      // the slice must lie inside the tensor as the table describes it, not merely inside the file
      wp[i] = slice_in_tensor(*tw[i], (uint64_t)e * sl[i], sl[i])
                  ? view_at(g->shards[tw[i]->shard], tw[i]->offset + (uint64_t)e * sl[i], sl[i], w[i])
                  : nullptr;
      if (!wp[i]) return bail(CSK_ERR_ARG, "short read: " + p + wn[i]);
      if (tb[i] && (!slice_in_tensor(*tb[i], (uint64_t)e * bl[i] * 4, bl[i] * 4) ||
                    !read_at(g->shards[tb[i]->shard], tb[i]->offset + (uint64_t)e * bl[i] * 4, b[i].data(), bl[i] * 4)))
        return bail(CSK_ERR_ARG, "short read: " + p + bn[i]);
    }
    const float* bp[3] = {tb[0] ? b[0].data() : nullptr, tb[1] ? b[1].data() : nullptr,
                          tb[2] ? b[2].data() : nullptr};
    if (f16) {
      const int which[3] = {CSK_W_UP, CSK_W_GATE, CSK_W_DOWN};
      for (int i = 0; i < 3 && rc == CSK_OK; ++i)
        rc = csk_layer_set_expert_matrix(L, e, which[i], (int)tw[i]->type, wp[i]);
      if (rc == CSK_OK) rc = csk_layer_set_expert_f16(L, e, nullptr, nullptr, nullptr, bp[0], bp[1], bp[2]);
    } else {
      rc = csk_layer_set_expert(L, e, wp[0], wp[1], wp[2], bp[0], bp[1], bp[2]);
    }
    if (rc != CSK_OK) return bail(rc, "");
  }
  const TensorInfo* tn = find(g, p + "." + norm_name);
  if (tn) {
    if (tn->type != kGgmlF32 || tn->dims.size() != 1 || tn->dims[0] != H)
      return bail(CSK_ERR_ARG, p + "." + norm_name + ": expected F32 [hidden]");
    std::vector<float> nw(H);
    if (!read_at(g->shards[tn->shard], tn->offset, nw.data(), (size_t)H * 4)) return bail(CSK_ERR_ARG, "short read: " + p + "." + norm_name);
    float eps = 1e-5f;  // graph_builder.h:154
    rc = csk_layer_set_norm(L, nw.data(), eps);
    if (rc != CSK_OK) return bail(rc, "");
  }
  *out = L;
  return CSK_OK;
}
