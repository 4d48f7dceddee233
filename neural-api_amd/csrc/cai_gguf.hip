// GGUF container reader and llama/qwen2 decoder loader (host code only).
//
// The file is mapped read-only; metadata and the tensor table are parsed with the checks of the reference
// reader (TNNetGGUFReader.ParseFile, neural/neuralgguf.pas:1072-1220): magic, version 2 or 3, non-empty unique
// names, 1..8 dimensions each in 1..2^31-1, block-multiple contiguous dimension for block-quantised types,
// power-of-two general.alignment, every tensor inside the data section.  Shapes are reported row-major
// (ggml's contiguous axis last), so an HF [out, in] matrix reads [out, in] (neuralgguf.pas:1157-1162).
//
// cai_decoder_load_gguf mirrors BuildLlamaFromGGUFEx / the qwen2 branch (neural/neuralpretrained.pas:17484-17876):
// the same metadata keys and defaults, the same required tensors, a tied head when output.weight is absent.
// Blocks are uploaded in STORED order and stored type: llama.cpp's q/k row order is the interleaved-rotary
// order, which is what the decode kernels rotate (the reference de-interleaves to HF order at read time,
// neuralgguf.pas:428-438, and permutes back at placement, neuralpretrained.pas:14792-14812; the composition is
// the identity).  ffn_up and ffn_gate are fused as rows [up | gate] (neuralpretrained.pas:240-243).
#include "cai_internal.hpp"

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <map>
#include <string>

using namespace cai;

namespace {

enum { GT_U8 = 0, GT_I8, GT_U16, GT_I16, GT_U32, GT_I32, GT_F32, GT_BOOL, GT_STR, GT_ARR, GT_U64, GT_I64, GT_F64 };

struct MetaValue {
  int type = -1;          // GT_*
  uint64_t u = 0; int64_t i = 0; double f = 0.0;
  std::string s;
  int elem_type = -1; uint64_t count = 0;   // arrays: element type and length (elements are skipped)
  size_t arr_pos = 0;                       // file offset of the first array element
};

struct TensorInfo {
  std::string name;
  int ggml_type = 0, n_dims = 0;
  int64_t shape[8] = {0};   // row-major: contiguous axis last
  int64_t offset = 0, nbytes = 0, n_elems = 0;
};

// bytes per block / elements per block of the ggml types whose size is known (neuralgguf.pas:86-138)
bool ggml_block(int t, int& elems, int& bytes)
{
  switch (t) {
    case 0: elems = 1; bytes = 4; return true;        // F32
    case 1: elems = 1; bytes = 2; return true;        // F16
    case 2: elems = 32; bytes = 18; return true;      // Q4_0
    case 3: elems = 32; bytes = 20; return true;      // Q4_1
    case 6: elems = 32; bytes = 22; return true;      // Q5_0
    case 7: elems = 32; bytes = 24; return true;      // Q5_1
    case 8: elems = 32; bytes = 34; return true;      // Q8_0
    case 10: elems = 256; bytes = 84; return true;    // Q2_K
    case 11: elems = 256; bytes = 110; return true;   // Q3_K
    case 12: elems = 256; bytes = 144; return true;   // Q4_K
    case 13: elems = 256; bytes = 176; return true;   // Q5_K
    case 14: elems = 256; bytes = 210; return true;   // Q6_K
    case 30: elems = 1; bytes = 2; return true;       // BF16
    default: return false;
  }
}

}  // namespace

struct cai_gguf_s {
  std::string path;
  const uint8_t* base = nullptr; size_t size = 0;
  int version = 0, alignment = 32;
  int64_t data_start = 0;
  std::vector<std::pair<std::string, MetaValue>> meta;
  std::map<std::string, size_t> meta_index;
  std::vector<TensorInfo> tensors;
  std::map<std::string, size_t> tensor_index;
  // cai_gguf_meta_array_str: the string array last read, the index after the entry last returned and its byte position
  const MetaValue* walk_arr = nullptr; int64_t walk_next = 0; size_t walk_pos = 0;
};

namespace {

struct Cursor {
  const uint8_t* b; size_t n, p = 0; bool ok = true;
  template <typename T> T get() { T v{}; if (p + sizeof(T) > n) { ok = false; return v; } memcpy(&v, b + p, sizeof(T)); p += sizeof(T); return v; }
  std::string str() {
    const uint64_t len = get<uint64_t>();
    if (!ok || len > n - p) { ok = false; return std::string(); }
    std::string s(reinterpret_cast<const char*>(b + p), (size_t)len); p += (size_t)len; return s;
  }
};

bool read_value(Cursor& c, int type, MetaValue& v, int depth)
{
  v.type = type;
  switch (type) {
    case GT_U8: v.u = c.get<uint8_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
    case GT_I8: v.i = c.get<int8_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
    case GT_U16: v.u = c.get<uint16_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
    case GT_I16: v.i = c.get<int16_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
    case GT_U32: v.u = c.get<uint32_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
    case GT_I32: v.i = c.get<int32_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
    case GT_F32: v.f = c.get<float>(); v.i = (int64_t)v.f; break;
    case GT_BOOL: v.u = c.get<uint8_t>() ? 1 : 0; v.i = (int64_t)v.u; v.f = (double)v.u; break;
    case GT_STR: v.s = c.str(); break;
    case GT_U64: v.u = c.get<uint64_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
    case GT_I64: v.i = c.get<int64_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
    case GT_F64: v.f = c.get<double>(); v.i = (int64_t)v.f; break;
    case GT_ARR: {
      if (depth > 2) return false;
      v.elem_type = (int)c.get<uint32_t>(); v.count = c.get<uint64_t>();
      if (!c.ok) return false;
      static const int fixed[] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
      if (v.elem_type < 0 || v.elem_type > GT_F64) return false;
      v.arr_pos = c.p;
      if (fixed[v.elem_type]) {
        if (v.count > (c.n - c.p) / (uint64_t)fixed[v.elem_type]) return false;
        c.p += (size_t)(v.count * fixed[v.elem_type]);
      } else {
        for (uint64_t k = 0; k < v.count; k++) { MetaValue e; if (!read_value(c, v.elem_type, e, depth + 1) || !c.ok) return false; }
      }
      break;
    }
    default: return false;
  }
  return c.ok;
}

int parse(cai_gguf_s* g)
{
  const char* fn = g->path.c_str();
  if (g->size < 24) return set_error(CAI_ERR_INVALID, "gguf: file too small (%zu bytes; need at least the 24-byte header): %s", g->size, fn);
  Cursor c{g->base, g->size};
  const uint32_t magic = c.get<uint32_t>();
  if (magic != 0x46554747u) return set_error(CAI_ERR_INVALID, "gguf: bad magic 0x%08X (expected \"GGUF\"): %s", magic, fn);
  g->version = (int)c.get<uint32_t>();
  if (g->version != 2 && g->version != 3) return set_error(CAI_ERR_UNSUPPORTED, "gguf: unsupported version %d (supported: 2, 3): %s", g->version, fn);
  const uint64_t n_tensors = c.get<uint64_t>(), n_kv = c.get<uint64_t>();
  if (n_tensors > 0x7fffffffull || n_kv > 0x7fffffffull)
    return set_error(CAI_ERR_INVALID, "gguf: implausible header counts (%llu tensors, %llu KV pairs): %s", (unsigned long long)n_tensors, (unsigned long long)n_kv, fn);
  for (uint64_t k = 0; k < n_kv; k++) {
    std::string key = c.str();
    if (!c.ok) return set_error(CAI_ERR_INVALID, "gguf: truncated metadata (pair %llu): %s", (unsigned long long)k, fn);
    if (key.empty()) return set_error(CAI_ERR_INVALID, "gguf: empty metadata key (pair %llu): %s", (unsigned long long)k, fn);
    if (g->meta_index.count(key)) return set_error(CAI_ERR_INVALID, "gguf: duplicate metadata key \"%s\": %s", key.c_str(), fn);
    const int vt = (int)c.get<uint32_t>();
    MetaValue v;
    if (!c.ok || !read_value(c, vt, v, 0)) return set_error(CAI_ERR_INVALID, "gguf: bad or truncated value for metadata key \"%s\" (type %d): %s", key.c_str(), vt, fn);
    g->meta_index[key] = g->meta.size();
    g->meta.emplace_back(std::move(key), std::move(v));
  }
  for (uint64_t t = 0; t < n_tensors; t++) {
    TensorInfo ti;
    ti.name = c.str();
    if (!c.ok) return set_error(CAI_ERR_INVALID, "gguf: truncated tensor table (tensor %llu): %s", (unsigned long long)t, fn);
    if (ti.name.empty()) return set_error(CAI_ERR_INVALID, "gguf: empty tensor name (tensor %llu): %s", (unsigned long long)t, fn);
    if (g->tensor_index.count(ti.name)) return set_error(CAI_ERR_INVALID, "gguf: duplicate tensor name \"%s\": %s", ti.name.c_str(), fn);
    ti.n_dims = (int)c.get<uint32_t>();
    if (!c.ok || ti.n_dims < 1 || ti.n_dims > 8) return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" has implausible n_dims %d: %s", ti.name.c_str(), ti.n_dims, fn);
    int64_t dims[8]; ti.n_elems = 1;
    for (int j = 0; j < ti.n_dims; j++) {
      const uint64_t d = c.get<uint64_t>();
      if (!c.ok || d == 0 || d > 0x7fffffffull) return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" has implausible dimension %llu: %s", ti.name.c_str(), (unsigned long long)d, fn);
      dims[j] = (int64_t)d;
      if (ti.n_elems > (int64_t)(0x7fffffffffffffffll / (int64_t)d)) return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" element count overflows: %s", ti.name.c_str(), fn);
      ti.n_elems *= (int64_t)d;
    }
    for (int j = 0; j < ti.n_dims; j++) ti.shape[j] = dims[ti.n_dims - 1 - j];
    ti.ggml_type = (int)c.get<uint32_t>();
    int be = 0, bb = 0;
    const bool known = ggml_block(ti.ggml_type, be, bb);
    if (known && be > 1 && dims[0] % be)
      return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" is ggml type %d but its contiguous dimension %lld is not a multiple of the block size %d: %s",
                       ti.name.c_str(), ti.ggml_type, (long long)dims[0], be, fn);
    ti.offset = (int64_t)c.get<uint64_t>();
    if (!c.ok) return set_error(CAI_ERR_INVALID, "gguf: truncated tensor table (tensor \"%s\"): %s", ti.name.c_str(), fn);
    if (known && ti.n_elems / be > (int64_t)(0x7fffffffffffffffll / bb))   // (the product below would wrap and slip past the bounds check)
      return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" byte size overflows: %s", ti.name.c_str(), fn);
    ti.nbytes = known ? ti.n_elems / be * bb : 0;   // unknown types stay listed; loading them is refused
    g->tensor_index[ti.name] = g->tensors.size();
    g->tensors.push_back(std::move(ti));
  }
  {
    auto it = g->meta_index.find("general.alignment");
    int64_t a = 32;
    if (it != g->meta_index.end() && g->meta[it->second].second.type != GT_STR && g->meta[it->second].second.type != GT_ARR) a = g->meta[it->second].second.i;
    if (a < 1 || a > (1 << 30) || (a & (a - 1))) return set_error(CAI_ERR_INVALID, "gguf: general.alignment %lld is not a positive power of two: %s", (long long)a, fn);
    g->alignment = (int)a;
  }
  g->data_start = (int64_t)((c.p + g->alignment - 1) / g->alignment * g->alignment);
  if ((size_t)g->data_start > g->size) return set_error(CAI_ERR_INVALID, "gguf: header ends at %lld past the end of the %zu-byte file: %s", (long long)g->data_start, g->size, fn);
  const int64_t data_size = (int64_t)g->size - g->data_start;
  for (const TensorInfo& ti : g->tensors)
    if (ti.offset < 0 || ti.offset > data_size || ti.nbytes > data_size - ti.offset)
      return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" data [%lld, %lld) falls outside the data section (size %lld): %s",
                       ti.name.c_str(), (long long)ti.offset, (long long)(ti.offset + ti.nbytes), (long long)data_size, fn);
  return CAI_OK;
}

const MetaValue* find_meta(const cai_gguf_s* g, const char* key)
{
  auto it = g->meta_index.find(key);
  return it == g->meta_index.end() ? nullptr : &g->meta[it->second].second;
}
const TensorInfo* find_tensor(const cai_gguf_s* g, const std::string& name)
{
  auto it = g->tensor_index.find(name);
  return it == g->tensor_index.end() ? nullptr : &g->tensors[it->second];
}
bool is_scalar_number(const MetaValue* v) { return v && v->type != GT_STR && v->type != GT_ARR; }

// 1-D F32 / F16 tensor as floats (norm gains, biases)
int read_vector(const cai_gguf_s* g, const std::string& name, int64_t want, std::vector<float>& out)
{
  const TensorInfo* t = find_tensor(g, name);
  if (!t) return set_error(CAI_ERR_INVALID, "gguf: missing tensor \"%s\" in %s", name.c_str(), g->path.c_str());
  if (t->n_elems != want) return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" has %lld elements, expected %lld: %s", name.c_str(), (long long)t->n_elems, (long long)want, g->path.c_str());
  const uint8_t* p = g->base + g->data_start + t->offset;
  out.resize((size_t)want);
  if (t->ggml_type == 0) memcpy(out.data(), p, (size_t)want * 4);
  else if (t->ggml_type == 1) { for (int64_t i = 0; i < want; i++) { _Float16 h; memcpy(&h, p + 2 * i, 2); out[(size_t)i] = (float)h; } }
  else return set_error(CAI_ERR_UNSUPPORTED, "gguf: vector tensor \"%s\" has ggml type %d (F32 or F16 expected): %s", name.c_str(), t->ggml_type, g->path.c_str());
  return CAI_OK;
}

bool uploadable_type(int t) { return t == CAI_F32 || t == CAI_F16 || t == CAI_Q4_0 || t == CAI_Q8_0 || t == CAI_Q4_K || t == CAI_Q6_K || raw_block_type(t); }

// resident weight from one 2-D tensor (or two stacked along the rows) in stored order
int load_matrix(const cai_gguf_s* g, const std::string& name, const std::string* second, const std::string* bias_name,
                int64_t want_rows, int64_t want_cols, cai_qw_t* out)
{
  const TensorInfo* t = find_tensor(g, name);
  if (!t) return set_error(CAI_ERR_INVALID, "gguf: missing tensor \"%s\" in %s", name.c_str(), g->path.c_str());
  const TensorInfo* t2 = nullptr;
  if (second) { t2 = find_tensor(g, *second); if (!t2) return set_error(CAI_ERR_INVALID, "gguf: missing tensor \"%s\" in %s", second->c_str(), g->path.c_str()); }
  const TensorInfo* both[2] = {t, t2};
  for (const TensorInfo* q : both) {
    if (!q) continue;
    if (q->n_dims != 2) return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" has %d dimensions, expected a matrix: %s", q->name.c_str(), q->n_dims, g->path.c_str());
    if (!uploadable_type(q->ggml_type)) return set_error(CAI_ERR_UNSUPPORTED, "gguf: tensor \"%s\" has ggml type %d; resident types are F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K: %s", q->name.c_str(), q->ggml_type, g->path.c_str());
    if ((want_rows > 0 && q->shape[0] != want_rows) || (want_cols > 0 && q->shape[1] != want_cols))
      return set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" is [%lld, %lld], expected [%lld, %lld]: %s", q->name.c_str(), (long long)q->shape[0], (long long)q->shape[1], (long long)want_rows, (long long)want_cols, g->path.c_str());
  }
  if (t2 && (t2->ggml_type != t->ggml_type || t2->shape[1] != t->shape[1]))
    return set_error(CAI_ERR_UNSUPPORTED, "gguf: \"%s\" and \"%s\" differ in type or width and cannot be fused: %s", t->name.c_str(), t2->name.c_str(), g->path.c_str());
  std::vector<float> bias;
  if (bias_name && find_tensor(g, *bias_name)) { const int rc = read_vector(g, *bias_name, t->shape[0], bias); if (rc) return rc; }
  const uint8_t* p = g->base + g->data_start + t->offset;
  if (!t2) return cai_qw_create(t->ggml_type, t->shape[0], t->shape[1], p, bias.empty() ? nullptr : bias.data(), out);
  std::vector<uint8_t> cat((size_t)(t->nbytes + t2->nbytes));
  memcpy(cat.data(), p, (size_t)t->nbytes);
  memcpy(cat.data() + t->nbytes, g->base + g->data_start + t2->offset, (size_t)t2->nbytes);
  return cai_qw_create(t->ggml_type, t->shape[0] + t2->shape[0], t->shape[1], cat.data(), nullptr, out);
}

}  // namespace

// ------------------------------------------------------------------------------------------
// C ABI: container
// ------------------------------------------------------------------------------------------
extern "C" int cai_gguf_open(const char* path, cai_gguf_t* out)
{
  CAI_ENTER();
  CAI_REQUIRE(path && out, "cai_gguf_open: null argument");
  *out = nullptr;
  const int fd = open(path, O_RDONLY);
  if (fd < 0) return set_error(CAI_ERR_INVALID, "gguf: cannot open %s: %s", path, strerror(errno));
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 0) { close(fd); return set_error(CAI_ERR_INVALID, "gguf: cannot stat %s", path); }
  cai_gguf_s* g = new cai_gguf_s();
  g->path = path; g->size = (size_t)st.st_size;
  if (g->size > 0) {
    void* m = mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (m == MAP_FAILED) { close(fd); delete g; return set_error(CAI_ERR_INVALID, "gguf: cannot map %s: %s", path, strerror(errno)); }
    g->base = static_cast<const uint8_t*>(m);
  }
  close(fd);
  const int rc = parse(g);
  if (rc) { cai_gguf_close(g); return rc; }
  *out = g;
  return CAI_OK;
}

extern "C" int cai_gguf_close(cai_gguf_t g)
{
  CAI_ENTER();
  if (!g) return CAI_OK;
  if (g->base) munmap(const_cast<uint8_t*>(g->base), g->size);
  delete g;
  return CAI_OK;
}

extern "C" int cai_gguf_info(cai_gguf_t g, int* version, int* alignment, int64_t* n_tensors, int64_t* n_meta, int64_t* data_start)
{
  CAI_ENTER();
  CAI_REQUIRE(g, "cai_gguf_info: null handle");
  if (version) *version = g->version;
  if (alignment) *alignment = g->alignment;
  if (n_tensors) *n_tensors = (int64_t)g->tensors.size();
  if (n_meta) *n_meta = (int64_t)g->meta.size();
  if (data_start) *data_start = g->data_start;
  return CAI_OK;
}

extern "C" int cai_gguf_meta_int(cai_gguf_t g, const char* key, int64_t* out)
{
  CAI_ENTER();
  CAI_REQUIRE(g && key && out, "cai_gguf_meta_int: null argument");
  const MetaValue* v = find_meta(g, key);
  if (!is_scalar_number(v)) return set_error(CAI_ERR_INVALID, "gguf: metadata key \"%s\" is missing or not a number: %s", key, g->path.c_str());
  *out = v->i;
  return CAI_OK;
}

extern "C" int cai_gguf_meta_float(cai_gguf_t g, const char* key, double* out)
{
  CAI_ENTER();
  CAI_REQUIRE(g && key && out, "cai_gguf_meta_float: null argument");
  const MetaValue* v = find_meta(g, key);
  if (!is_scalar_number(v)) return set_error(CAI_ERR_INVALID, "gguf: metadata key \"%s\" is missing or not a number: %s", key, g->path.c_str());
  *out = v->f;
  return CAI_OK;
}

extern "C" int cai_gguf_meta_str(cai_gguf_t g, const char* key, char* buf, int n)
{
  CAI_ENTER();
  CAI_REQUIRE(g && key && buf && n > 0, "cai_gguf_meta_str: bad argument");
  const MetaValue* v = find_meta(g, key);
  if (!v || v->type != GT_STR) return set_error(CAI_ERR_INVALID, "gguf: metadata key \"%s\" is missing or not a string: %s", key, g->path.c_str());
  snprintf(buf, (size_t)n, "%s", v->s.c_str());
  return CAI_OK;
}

extern "C" int cai_gguf_meta_array_count(cai_gguf_t g, const char* key, int64_t* out)
{
  CAI_ENTER();
  CAI_REQUIRE(g && key && out, "cai_gguf_meta_array_count: null argument");
  const MetaValue* v = find_meta(g, key);
  if (!v || v->type != GT_ARR) return set_error(CAI_ERR_INVALID, "gguf: metadata key \"%s\" is missing or not an array: %s", key, g->path.c_str());
  *out = (int64_t)v->count;
  return CAI_OK;
}

extern "C" int cai_gguf_meta_array_str(cai_gguf_t g, const char* key, int64_t index, char* buf, int n)
{
  CAI_ENTER();
  CAI_REQUIRE(g && key && buf && n > 0, "cai_gguf_meta_array_str: bad argument");
  const MetaValue* v = find_meta(g, key);
  if (!v || v->type != GT_ARR || v->elem_type != GT_STR) return set_error(CAI_ERR_INVALID, "gguf: metadata key \"%s\" is missing or not a string array: %s", key, g->path.c_str());
  if (index < 0 || (uint64_t)index >= v->count) return set_error(CAI_ERR_INVALID, "gguf: index %lld outside the %llu entries of \"%s\": %s", (long long)index, (unsigned long long)v->count, key, g->path.c_str());
  // entries have no fixed size: remember where the last read ended so that walking a vocabulary in order costs one entry per
  // call instead of a scan from the start (GetMetaArrayString memoises likewise, neural/neuralgguf.pas)
  Cursor c{g->base, g->size}; c.p = v->arr_pos;
  int64_t k = 0;
  if (g->walk_arr == v && g->walk_next <= index) { c.p = g->walk_pos; k = g->walk_next; }
  std::string s;
  for (; k <= index; k++) s = c.str();   // entries were validated when the file was opened
  g->walk_arr = v; g->walk_next = index + 1; g->walk_pos = c.p;
  snprintf(buf, (size_t)n, "%s", s.c_str());
  return CAI_OK;
}

extern "C" int cai_gguf_find_tensor(cai_gguf_t g, const char* name, int64_t* index)
{
  CAI_ENTER();
  CAI_REQUIRE(g && name && index, "cai_gguf_find_tensor: null argument");
  auto it = g->tensor_index.find(name);
  if (it == g->tensor_index.end()) return set_error(CAI_ERR_INVALID, "gguf: missing tensor \"%s\" in %s", name, g->path.c_str());
  *index = (int64_t)it->second;
  return CAI_OK;
}

extern "C" int cai_gguf_tensor_info(cai_gguf_t g, int64_t index, char* name_buf, int name_n, int* ggml_type, int* n_dims,
                                    int64_t* shape8, int64_t* data_offset, int64_t* nbytes)
{
  CAI_ENTER();
  CAI_REQUIRE(g && index >= 0 && index < (int64_t)g->tensors.size(), "cai_gguf_tensor_info: bad index");
  const TensorInfo& t = g->tensors[(size_t)index];
  if (name_buf && name_n > 0) snprintf(name_buf, (size_t)name_n, "%s", t.name.c_str());
  if (ggml_type) *ggml_type = t.ggml_type;
  if (n_dims) *n_dims = t.n_dims;
  if (shape8) for (int j = 0; j < 8; j++) shape8[j] = j < t.n_dims ? t.shape[j] : 0;
  if (data_offset) *data_offset = t.offset;
  if (nbytes) *nbytes = t.nbytes;
  return CAI_OK;
}

extern "C" int cai_gguf_tensor_data(cai_gguf_t g, int64_t index, const void** ptr)
{
  CAI_ENTER();
  CAI_REQUIRE(g && ptr && index >= 0 && index < (int64_t)g->tensors.size(), "cai_gguf_tensor_data: bad argument");
  const TensorInfo& t = g->tensors[(size_t)index];
  if (t.nbytes == 0) return set_error(CAI_ERR_UNSUPPORTED, "gguf: tensor \"%s\" has ggml type %d of unknown size: %s", t.name.c_str(), t.ggml_type, g->path.c_str());
  *ptr = g->base + g->data_start + t.offset;
  return CAI_OK;
}

extern "C" int cai_gguf_load_qw(cai_gguf_t g, const char* name, const char* bias_name, cai_qw_t* out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(g && name && out, "cai_gguf_load_qw: null argument");
  const std::string n(name), b(bias_name ? bias_name : "");
  return load_matrix(g, n, nullptr, bias_name ? &b : nullptr, 0, 0, out);
}

// ------------------------------------------------------------------------------------------
// C ABI: llama / qwen2 decoder straight from a file
// ------------------------------------------------------------------------------------------
extern "C" int cai_decoder_load_gguf(const char* path, int max_ctx, int max_batch, int kv_dtype, cai_decoder_t* out)
{
  CAI_ENTER();
  // (the file's metadata is judged before the device is asked for: a file this path cannot run is refused with the same
  // message on a host without a GPU)
  CAI_REQUIRE(path && out, "cai_decoder_load_gguf: null argument");
  *out = nullptr;
  cai_gguf_t g = nullptr;
  int rc = cai_gguf_open(path, &g);
  if (rc) return rc;
  cai_decoder_t d = nullptr;
  auto fail = [&](int code) { if (d) cai_decoder_destroy(d); cai_gguf_close(g); return code; };

  const MetaValue* av = find_meta(g, "general.architecture");
  const std::string arch = av && av->type == GT_STR ? av->s : std::string();
  if (arch != "llama" && arch != "qwen2")
    return fail(set_error(CAI_ERR_UNSUPPORTED, "gguf decoder: general.architecture is \"%s\" - supported: llama, qwen2: %s", arch.c_str(), path));
  auto key = [&](const char* k) { return arch + "." + k; };
  auto req_int = [&](const char* k, int64_t& v) {
    const MetaValue* m = find_meta(g, key(k).c_str());
    if (!is_scalar_number(m) || m->i <= 0) return set_error(CAI_ERR_INVALID, "gguf decoder: metadata key \"%s\" is missing or not a positive integer in %s", key(k).c_str(), path);
    v = m->i; return (int)CAI_OK;
  };
  auto opt_int = [&](const char* k, int64_t dflt) { const MetaValue* m = find_meta(g, key(k).c_str()); return is_scalar_number(m) ? m->i : dflt; };
  auto opt_float = [&](const char* k, double dflt) { const MetaValue* m = find_meta(g, key(k).c_str()); return is_scalar_number(m) ? m->f : dflt; };

  int64_t dm = 0, ffn = 0, n_layers = 0, hq = 0, ctx_len = 0;
  if ((rc = req_int("embedding_length", dm)) || (rc = req_int("feed_forward_length", ffn)) || (rc = req_int("block_count", n_layers)) ||
      (rc = req_int("attention.head_count", hq)) || (rc = req_int("context_length", ctx_len))) return fail(rc);
  const int64_t hkv = opt_int("attention.head_count_kv", hq);
  int64_t hd = opt_int("attention.key_length", 0);
  if (hd <= 0) {
    if (dm % hq) return fail(set_error(CAI_ERR_INVALID, "gguf decoder: %s=%lld is not divisible by %s=%lld", key("embedding_length").c_str(), (long long)dm, key("attention.head_count").c_str(), (long long)hq));
    hd = dm / hq;
  }
  // llama files: rope.scaling.type "linear" -> Position Interpolation with rope.scaling.factor; absent / "none" = unscaled;
  // anything else is refused (neural/neuralpretrained.pas:17539-17557).  qwen2 files: the key is not read and the rotation
  // stays unscaled, as the reference's qwen2 import leaves it (neural/neuralpretrained.pas:17720).
  double rope_linear = 1.0;
  if (arch == "llama") {
    const MetaValue* st = find_meta(g, key("rope.scaling.type").c_str());
    if (st && st->type == GT_STR && st->s != "none") {
      const double f = opt_float("rope.scaling.factor", 1.0);
      if (st->s != "linear")
        return fail(set_error(CAI_ERR_UNSUPPORTED, "gguf decoder: %s \"%s\" (factor %g) is not supported (supported: none, linear): %s", key("rope.scaling.type").c_str(), st->s.c_str(), f, path));
      if (f < 1.0) return fail(set_error(CAI_ERR_INVALID, "gguf decoder: %s must be >= 1, got %g: %s", key("rope.scaling.factor").c_str(), f, path));
      rope_linear = f;
    }
  }
  // per-frequency divisors (llama.cpp's form of the Llama-3.1 rule): one F32 value per rotary pair.  The reference's import
  // never reads this tensor and rotates such a file with the plain frequencies; a caller that wants exactly that resets the
  // divisors to 1 after loading (cai_decoder_set_rope_freq_factors).
  std::vector<float> rope_factors;
  if (const TensorInfo* rf = find_tensor(g, "rope_freqs.weight")) {
    if (rf->ggml_type != CAI_F32 || rf->n_dims != 1 || rf->shape[0] != hd / 2)
      return fail(set_error(CAI_ERR_INVALID, "gguf decoder: rope_freqs.weight must be %lld F32 values (one per rotary pair): %s", (long long)(hd / 2), path));
    if (rope_linear != 1.0) return fail(set_error(CAI_ERR_UNSUPPORTED, "gguf decoder: rope_freqs.weight together with linear scaling: %s", path));
    if ((rc = read_vector(g, "rope_freqs.weight", hd / 2, rope_factors))) return fail(rc);
  }
  if (arch == "qwen2") {
    // the reference refuses sliding-window Qwen2 files rather than run them with full attention (neural/neuralpretrained.pas:17755-17760)
    const MetaValue* sw = find_meta(g, key("attention.sliding_window").c_str());
    if (sw && ((sw->type == GT_BOOL && sw->i) || (is_scalar_number(sw) && sw->i > 0)))
      return fail(set_error(CAI_ERR_UNSUPPORTED, "gguf decoder: %s is set; Qwen2 sliding-window attention is not wired into this loader: %s", key("attention.sliding_window").c_str(), path));
    for (int l = 0; l < (int)n_layers; l++)
      for (const char* b : {"attn_q.bias", "attn_k.bias", "attn_v.bias"}) {
        const std::string nm = "blk." + std::to_string(l) + "." + b;
        if (!find_tensor(g, nm)) return fail(set_error(CAI_ERR_INVALID, "gguf: missing tensor \"%s\" (qwen2 projections carry biases) in %s", nm.c_str(), path));
      }
  }
  int64_t vocab = opt_int("vocab_size", 0);
  if (vocab <= 0) {
    const TensorInfo* te = find_tensor(g, "token_embd.weight");
    if (te && te->n_dims == 2) vocab = te->shape[0];
    else { const MetaValue* tk = find_meta(g, "tokenizer.ggml.tokens"); if (tk && tk->type == GT_ARR) vocab = (int64_t)tk->count; }
  }
  if (vocab <= 0) return fail(set_error(CAI_ERR_INVALID, "gguf decoder: cannot determine the vocab size (no %s, no 2-D token_embd.weight, no tokenizer.ggml.tokens) in %s", key("vocab_size").c_str(), path));

  // The metadata is not trusted further than the tensor table bears it out: every block owns tensors, so a block count beyond
  // the table is a lie, and the first block's matrices and the embedding must have the shapes the keys promise - checked
  // before anything is sized from these numbers.
  if (n_layers > (int64_t)g->tensors.size())
    return fail(set_error(CAI_ERR_INVALID, "gguf decoder: %s=%lld but the file lists %zu tensors: %s", key("block_count").c_str(), (long long)n_layers, g->tensors.size(), path));
  if (hkv <= 0 || hq % hkv) return fail(set_error(CAI_ERR_INVALID, "gguf decoder: %lld query heads over %lld KV heads: %s", (long long)hq, (long long)hkv, path));
  const int64_t lim = (int64_t)1 << 24;
  if (dm > lim || ffn > lim || hq > lim || hd > lim || vocab > ((int64_t)1 << 28) || hq * hd > lim || (max_ctx <= 0 && ctx_len > ((int64_t)1 << 26)))
    return fail(set_error(CAI_ERR_INVALID, "gguf decoder: implausible dimensions (width %lld, feed-forward %lld, %lld heads of %lld, vocab %lld, context %lld): %s",
                          (long long)dm, (long long)ffn, (long long)hq, (long long)hd, (long long)vocab, (long long)ctx_len, path));
  {
    struct Want { const char* name; int64_t rows, cols; };
    const Want wants[] = {{"token_embd.weight", vocab, dm}, {"blk.0.attn_q.weight", hq * hd, dm}, {"blk.0.attn_k.weight", hkv * hd, dm},
                          {"blk.0.attn_output.weight", dm, hq * hd}, {"blk.0.ffn_up.weight", ffn, dm}, {"blk.0.ffn_down.weight", dm, ffn}};
    for (const Want& w : wants) {
      const TensorInfo* t = find_tensor(g, w.name);
      if (!t) continue;                        // (reported, in the order of loading, below)
      if (t->n_dims != 2 || t->shape[0] != w.rows || t->shape[1] != w.cols)
        return fail(set_error(CAI_ERR_INVALID, "gguf: tensor \"%s\" is %lld x %lld, the metadata promises %lld x %lld: %s", w.name,
                              (long long)t->shape[0], (long long)(t->n_dims > 1 ? t->shape[1] : 1), (long long)w.rows, (long long)w.cols, path));
    }
  }

  cai_decoder_config cfg{};
  cfg.n_layers = (int)n_layers; cfg.d_model = (int)dm; cfg.n_q_heads = (int)hq; cfg.n_kv_heads = (int)hkv; cfg.head_dim = (int)hd;
  cfg.ffn = (int)ffn; cfg.vocab = (int)vocab; cfg.max_ctx = max_ctx > 0 ? max_ctx : (int)ctx_len;
  // default epsilon: 1e-5 on the llama branch, 1e-6 on the qwen2 branch (neural/neuralpretrained.pas:17533, 17715)
  cfg.eps = (float)opt_float("attention.layer_norm_rms_epsilon", arch == "qwen2" ? 1e-6 : 1e-5); cfg.rope_theta = (float)opt_float("rope.freq_base", 10000.0);
  cfg.kv_dtype = kv_dtype; cfg.max_batch = max_batch > 0 ? max_batch : 1;
  { Context& cx = ctx(); if (!cx.ready) return fail(set_error(CAI_ERR_STATE, "cai_init has not been called")); }
  if ((rc = cai_decoder_create(&cfg, &d))) return fail(rc);
  if (rope_linear != 1.0 && (rc = cai_decoder_set_rope_scaling(d, CAI_ROPE_LINEAR, (float)rope_linear, 0, 0.0f, 0.0f))) return fail(rc);
  if (!rope_factors.empty() && (rc = cai_decoder_set_rope_freq_factors(d, rope_factors.data(), (int)rope_factors.size()))) return fail(rc);

  auto put_w = [&](int layer, int slot, const std::string& name, const std::string* second, const std::string* bias, int64_t rows, int64_t cols) {
    cai_qw_t w = nullptr;
    int r = load_matrix(g, name, second, bias, rows, cols, &w);
    if (r) return r;
    decoder_adopt_weight(d, w);   // the decoder frees it
    return cai_decoder_set_weight(d, layer, slot, w);
  };
  auto put_v = [&](int layer, int slot, const std::string& name, int64_t n) {
    std::vector<float> v;
    int r = read_vector(g, name, n, v);
    if (r) return r;
    return cai_decoder_set_vector(d, layer, slot, v.data(), (int)n);
  };
  const int64_t qw = hq * hd, kw = hkv * hd;
  if ((rc = put_w(-1, CAI_W_EMBED, "token_embd.weight", nullptr, nullptr, vocab, dm))) return fail(rc);
  if (find_tensor(g, "output.weight") && (rc = put_w(-1, CAI_W_HEAD, "output.weight", nullptr, nullptr, vocab, dm))) return fail(rc);   // absent = tied head
  if ((rc = put_v(-1, CAI_V_FINAL_NORM, "output_norm.weight", dm))) return fail(rc);
  for (int l = 0; l < (int)n_layers; l++) {
    const std::string p = "blk." + std::to_string(l) + ".";
    const std::string qb = p + "attn_q.bias", kb = p + "attn_k.bias", vb = p + "attn_v.bias", gate = p + "ffn_gate.weight";
    const bool with_bias = arch == "qwen2";
    if ((rc = put_w(l, CAI_W_Q, p + "attn_q.weight", nullptr, with_bias ? &qb : nullptr, qw, dm)) ||
        (rc = put_w(l, CAI_W_K, p + "attn_k.weight", nullptr, with_bias ? &kb : nullptr, kw, dm)) ||
        (rc = put_w(l, CAI_W_V, p + "attn_v.weight", nullptr, with_bias ? &vb : nullptr, kw, dm)) ||
        (rc = put_w(l, CAI_W_O, p + "attn_output.weight", nullptr, nullptr, dm, qw)) ||
        (rc = put_w(l, CAI_W_GATEUP, p + "ffn_up.weight", &gate, nullptr, ffn, dm)) ||
        (rc = put_w(l, CAI_W_DOWN, p + "ffn_down.weight", nullptr, nullptr, dm, ffn)) ||
        (rc = put_v(l, CAI_V_ATTN_NORM, p + "attn_norm.weight", dm)) ||
        (rc = put_v(l, CAI_V_MLP_NORM, p + "ffn_norm.weight", dm))) return fail(rc);
  }
  cai_gguf_close(g);
  *out = d;
  return CAI_OK;
}
