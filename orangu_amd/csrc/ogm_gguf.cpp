// GGUF reader and matrix uploader: header, metadata key/values, tensor table, alignment
// (src/gguf.rs:149-280, 300-415 of orangu) and the 2-D matrix view with its shape / size
// validation (engine/loader.rs:1552-1580), so that a .gguf file's Q8_0 / Q3_K / Q4_K / Q5_K / Q6_K matrices reach
// ogm_weight_upload without the Rust host.  The file is memory-mapped read-only; every read is
// bounds-checked, so a malformed file gives an error, never an out-of-range access.
#include <fcntl.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <new>
#include <string>
#include <vector>

#include "../../include/orangu_mi355x.h"

namespace {

const uint32_t MIN_SUPPORTED_VERSION = 2;                 // gguf.rs:38
const uint64_t DEFAULT_ALIGNMENT = 32;                    // gguf.rs:47
const uint64_t MAX_STRING_BYTES = 100ull * 1024 * 1024;   // gguf.rs:42
const uint64_t MAX_ARRAY_ELEMENTS = 200000000ull;         // gguf.rs:43

struct Value {
  uint32_t type = 0;        // GGUF value type 0..12
  uint64_t u = 0;           // unsigned / bool payload
  int64_t i = 0;            // signed payload
  double f = 0.0;           // float payload
  std::string s;            // string payload
  uint32_t elem_type = 0;   // arrays: element type, count, and where the elements start
  uint64_t count = 0, at = 0;
};

struct Tensor {
  std::string name;
  std::vector<uint64_t> dims;
  uint32_t ggml_type = 0;
  uint64_t offset = 0;  // relative to data_offset
};

// Bytes and elements per block (engine/quant.rs:132-169), for the standard types.
bool block_layout(uint32_t t, uint32_t *bytes, uint32_t *elems) {
  switch (t) {
    case 0: *bytes = 4; *elems = 1; return true;      // F32
    case 1: *bytes = 2; *elems = 1; return true;      // F16
    case 2: *bytes = 18; *elems = 32; return true;    // Q4_0
    case 3: *bytes = 20; *elems = 32; return true;    // Q4_1
    case 6: *bytes = 22; *elems = 32; return true;    // Q5_0
    case 7: *bytes = 24; *elems = 32; return true;    // Q5_1
    case 8: *bytes = 34; *elems = 32; return true;    // Q8_0
    case 10: *bytes = 84; *elems = 256; return true;  // Q2_K
    case 11: *bytes = 110; *elems = 256; return true; // Q3_K
    case 12: *bytes = 144; *elems = 256; return true; // Q4_K
    case 13: *bytes = 176; *elems = 256; return true; // Q5_K
    case 14: *bytes = 210; *elems = 256; return true; // Q6_K
    case 20: *bytes = 18; *elems = 32; return true;   // IQ4_NL
    case 26: *bytes = 4; *elems = 1; return true;     // I32
    case 30: *bytes = 2; *elems = 1; return true;     // BF16
    default: return false;
  }
}

}  // namespace

struct ogm_gguf {
  const uint8_t *base = nullptr;  // start of the GGUF segment
  size_t len = 0;                 // bytes from base to the end of the mapping / buffer
  void *map = nullptr;            // mmap address (null when parsing caller memory)
  size_t map_len = 0;
  uint32_t version = 0;
  uint64_t alignment = DEFAULT_ALIGNMENT, data_offset = 0;
  std::vector<std::pair<std::string, Value>> meta;
  std::vector<Tensor> tensors;
  std::string err;
};

namespace {

struct Cursor {
  const uint8_t *p;
  size_t len, pos = 0;
  std::string *err;
  bool take(void *dst, size_t n) {
    if (n > len - pos) {
      *err = "unexpected end of file";
      return false;
    }
    memcpy(dst, p + pos, n);
    pos += n;
    return true;
  }
  template <class T>
  bool rd(T *v) { return take(v, sizeof(T)); }
  bool str(std::string *s) {
    uint64_t n;
    if (!rd(&n)) return false;
    if (n > MAX_STRING_BYTES) {
      *err = "string metadata value of " + std::to_string(n) + " bytes exceeds the limit";
      return false;
    }
    if (n > len - pos) {
      *err = "unexpected end of file";
      return false;
    }
    s->assign((const char *)p + pos, (size_t)n);
    pos += n;
    return true;
  }
  // Reads (scalars, strings) or skips over (array elements) one value of `type`.
  bool value(uint32_t type, Value *v, int depth) {
    v->type = type;
    switch (type) {
      case 0: { uint8_t x; if (!rd(&x)) return false; v->u = x; return true; }
      case 1: { int8_t x; if (!rd(&x)) return false; v->i = x; return true; }
      case 2: { uint16_t x; if (!rd(&x)) return false; v->u = x; return true; }
      case 3: { int16_t x; if (!rd(&x)) return false; v->i = x; return true; }
      case 4: { uint32_t x; if (!rd(&x)) return false; v->u = x; return true; }
      case 5: { int32_t x; if (!rd(&x)) return false; v->i = x; return true; }
      case 6: { float x; if (!rd(&x)) return false; v->f = x; return true; }
      case 7: { uint8_t x; if (!rd(&x)) return false; v->u = x != 0; return true; }
      case 8: return str(&v->s);
      case 9: {
        if (depth > 4) { *err = "metadata arrays nested too deeply"; return false; }
        if (!rd(&v->elem_type) || !rd(&v->count)) return false;
        if (v->count > MAX_ARRAY_ELEMENTS) {
          *err = "array metadata value of " + std::to_string(v->count) + " elements exceeds the limit";
          return false;
        }
        v->at = pos;
        static const uint8_t fixed[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
        if (v->elem_type > 12) { *err = "unknown GGUF metadata value type " + std::to_string(v->elem_type); return false; }
        if (fixed[v->elem_type]) {
          const uint64_t bytes = v->count * fixed[v->elem_type];
          if (bytes > len - pos) { *err = "unexpected end of file"; return false; }
          pos += bytes;
          return true;
        }
        Value tmp;
        for (uint64_t k = 0; k < v->count; k++)
          if (!value(v->elem_type, &tmp, depth + 1)) return false;
        return true;
      }
      case 10: { uint64_t x; if (!rd(&x)) return false; v->u = x; return true; }
      case 11: { int64_t x; if (!rd(&x)) return false; v->i = x; return true; }
      case 12: { double x; if (!rd(&x)) return false; v->f = x; return true; }
      default:
        *err = "unknown GGUF metadata value type " + std::to_string(type);
        return false;
    }
  }
};

// GgufValue::as_u64 (gguf.rs:70-83)
bool as_u64(const Value &v, uint64_t *out) {
  switch (v.type) {
    case 0: case 2: case 4: case 10: case 7: *out = v.u; return true;
    case 1: case 3: case 5: case 11: if (v.i < 0) return false; *out = (uint64_t)v.i; return true;
    default: return false;
  }
}

int parse(ogm_gguf *g) {
  Cursor c{g->base, g->len, 0, &g->err};
  char magic[4];
  if (!c.take(magic, 4)) return OGM_ERR_INVALID;
  if (memcmp(magic, "GGUF", 4) != 0) {
    g->err = "not a GGUF file: bad magic";
    return OGM_ERR_INVALID;
  }
  if (!c.rd(&g->version)) return OGM_ERR_INVALID;
  if (g->version < MIN_SUPPORTED_VERSION) {
    g->err = "GGUFv" + std::to_string(g->version) + " is not supported (32-bit counts); only GGUFv2+ is";
    return OGM_ERR_UNSUPPORTED;
  }
  uint64_t n_tensors, n_kv;
  if (!c.rd(&n_tensors) || !c.rd(&n_kv)) return OGM_ERR_INVALID;
  for (uint64_t k = 0; k < n_kv; k++) {
    std::string key;
    uint32_t type;
    Value v;
    if (!c.str(&key) || !c.rd(&type) || !c.value(type, &v, 0)) return OGM_ERR_INVALID;
    g->meta.emplace_back(std::move(key), std::move(v));
  }
  for (uint64_t k = 0; k < n_tensors; k++) {
    Tensor t;
    uint32_t n_dims;
    if (!c.str(&t.name) || !c.rd(&n_dims)) return OGM_ERR_INVALID;
    if (n_dims > 8) {
      g->err = "tensor '" + t.name + "' has " + std::to_string(n_dims) + " dimensions";
      return OGM_ERR_INVALID;
    }
    t.dims.resize(n_dims);
    for (uint32_t d = 0; d < n_dims; d++)
      if (!c.rd(&t.dims[d])) return OGM_ERR_INVALID;
    if (!c.rd(&t.ggml_type) || !c.rd(&t.offset)) return OGM_ERR_INVALID;
    g->tensors.push_back(std::move(t));
  }
  // general.alignment when present and positive, else 32 (gguf.rs:258-263)
  g->alignment = DEFAULT_ALIGNMENT;
  for (auto &kv : g->meta) {
    uint64_t a;
    if (kv.first == "general.alignment") {
      if (as_u64(kv.second, &a) && a > 0) g->alignment = a;
      break;
    }
  }
  g->data_offset = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
  return OGM_OK;
}

void set_err(char *err, size_t err_len, const std::string &msg) {
  if (err && err_len) snprintf(err, err_len, "%s", msg.c_str());
}

const Value *find_meta(const ogm_gguf *g, const char *key) {
  for (auto &kv : g->meta)
    if (kv.first == key) return &kv.second;
  return nullptr;
}

}  // namespace

extern "C" int ogm_gguf_parse(const void *bytes, size_t len, ogm_gguf **out, char *err, size_t err_len) {
  if (!bytes || !out) return OGM_ERR_INVALID;
  ogm_gguf *g = new (std::nothrow) ogm_gguf();
  if (!g) return OGM_ERR_OOM;
  g->base = (const uint8_t *)bytes;
  g->len = len;
  int rc = parse(g);
  if (rc != OGM_OK) {
    set_err(err, err_len, g->err);
    delete g;
    return rc;
  }
  *out = g;
  return OGM_OK;
}

extern "C" int ogm_gguf_open(const char *path, uint64_t offset, ogm_gguf **out, char *err, size_t err_len) {
  if (!path || !out) return OGM_ERR_INVALID;
  int fd = open(path, O_RDONLY);
  if (fd < 0) {
    set_err(err, err_len, std::string("failed to open ") + path);
    return OGM_ERR_INVALID;
  }
  struct stat st;
  if (fstat(fd, &st) != 0 || (uint64_t)st.st_size <= offset) {
    close(fd);
    set_err(err, err_len, std::string("nothing to read at that offset in ") + path);
    return OGM_ERR_INVALID;
  }
  void *m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (m == MAP_FAILED) {
    set_err(err, err_len, std::string("failed to map ") + path);
    return OGM_ERR_INVALID;
  }
  ogm_gguf *g = new (std::nothrow) ogm_gguf();
  if (!g) {
    munmap(m, (size_t)st.st_size);
    return OGM_ERR_OOM;
  }
  g->map = m;
  g->map_len = (size_t)st.st_size;
  g->base = (const uint8_t *)m + offset;
  g->len = (size_t)st.st_size - (size_t)offset;
  int rc = parse(g);
  if (rc != OGM_OK) {
    set_err(err, err_len, std::string("failed to parse GGUF file ") + path + ": " + g->err);
    munmap(m, g->map_len);
    delete g;
    return rc;
  }
  *out = g;
  return OGM_OK;
}

extern "C" void ogm_gguf_close(ogm_gguf *g) {
  if (!g) return;
  if (g->map) munmap(g->map, g->map_len);
  delete g;
}

extern "C" const char *ogm_gguf_last_error(const ogm_gguf *g) { return g ? g->err.c_str() : ""; }

extern "C" int ogm_gguf_info(const ogm_gguf *g, uint32_t *version, uint64_t *alignment, uint64_t *data_offset,
                             uint64_t *n_tensors, uint64_t *n_metadata) {
  if (!g) return OGM_ERR_INVALID;
  if (version) *version = g->version;
  if (alignment) *alignment = g->alignment;
  if (data_offset) *data_offset = g->data_offset;
  if (n_tensors) *n_tensors = g->tensors.size();
  if (n_metadata) *n_metadata = g->meta.size();
  return OGM_OK;
}

extern "C" int ogm_gguf_meta_u64(const ogm_gguf *g, const char *key, uint64_t *out) {
  if (!g || !key || !out) return OGM_ERR_INVALID;
  const Value *v = find_meta(g, key);
  return v && as_u64(*v, out) ? OGM_OK : OGM_ERR_INVALID;
}

extern "C" int ogm_gguf_meta_f64(const ogm_gguf *g, const char *key, double *out) {
  if (!g || !key || !out) return OGM_ERR_INVALID;
  const Value *v = find_meta(g, key);
  if (!v) return OGM_ERR_INVALID;
  if (v->type == 6 || v->type == 12) {
    *out = v->f;
    return OGM_OK;
  }
  uint64_t u;
  if (as_u64(*v, &u)) {
    *out = (double)u;
    return OGM_OK;
  }
  if (v->type == 1 || v->type == 3 || v->type == 5 || v->type == 11) {
    *out = (double)v->i;
    return OGM_OK;
  }
  return OGM_ERR_INVALID;
}

extern "C" int ogm_gguf_meta_string(const ogm_gguf *g, const char *key, const char **out, size_t *len) {
  if (!g || !key || !out) return OGM_ERR_INVALID;
  const Value *v = find_meta(g, key);
  if (!v || v->type != 8) return OGM_ERR_INVALID;
  *out = v->s.c_str();
  if (len) *len = v->s.size();
  return OGM_OK;
}

extern "C" int ogm_gguf_meta_array(const ogm_gguf *g, const char *key, uint32_t *elem_type, uint64_t *count) {
  if (!g || !key) return OGM_ERR_INVALID;
  const Value *v = find_meta(g, key);
  if (!v || v->type != 9) return OGM_ERR_INVALID;
  if (elem_type) *elem_type = v->elem_type;
  if (count) *count = v->count;
  return OGM_OK;
}

extern "C" int64_t ogm_gguf_find_tensor(const ogm_gguf *g, const char *name) {
  if (!g || !name) return -1;
  for (size_t i = 0; i < g->tensors.size(); i++)
    if (g->tensors[i].name == name) return (int64_t)i;
  return -1;
}

extern "C" int ogm_gguf_tensor(const ogm_gguf *g, uint64_t index, const char **name, uint32_t *n_dims,
                               uint64_t dims[8], uint32_t *ggml_type, uint64_t *offset) {
  if (!g || index >= g->tensors.size()) return OGM_ERR_INVALID;
  const Tensor &t = g->tensors[index];
  if (name) *name = t.name.c_str();
  if (n_dims) *n_dims = (uint32_t)t.dims.size();
  if (dims)
    for (size_t d = 0; d < t.dims.size(); d++) dims[d] = t.dims[d];
  if (ggml_type) *ggml_type = t.ggml_type;
  if (offset) *offset = t.offset;
  return OGM_OK;
}

// Where a tensor's bytes are and how many (tensor_byte_size, quant.rs:344-357), bounds-checked.
static int tensor_bytes(ogm_gguf *g, const Tensor &t, const uint8_t **ptr, uint64_t *len) {
  uint32_t bb, be;
  if (!block_layout(t.ggml_type, &bb, &be)) {
    g->err = "tensor '" + t.name + "': ggml_type " + std::to_string(t.ggml_type) + " is not supported";
    return OGM_ERR_UNSUPPORTED;
  }
  uint64_t n = 1;
  for (uint64_t d : t.dims) {
    if (d != 0 && n > UINT64_MAX / d) {
      g->err = "tensor '" + t.name + "': element count overflows";
      return OGM_ERR_INVALID;
    }
    n *= d;
  }
  if (n % be != 0) {
    g->err = "tensor '" + t.name + "': element count " + std::to_string(n) + " is not a multiple of the " +
             std::to_string(be) + " block size";
    return OGM_ERR_INVALID;
  }
  const uint64_t bytes = n / be * bb;
  if (g->data_offset > g->len || t.offset > g->len - g->data_offset ||
      bytes > g->len - g->data_offset - t.offset) {
    g->err = "tensor '" + t.name + "' extends past the end of the file";
    return OGM_ERR_INVALID;
  }
  *ptr = g->base + g->data_offset + t.offset;
  *len = bytes;
  return OGM_OK;
}

extern "C" int ogm_gguf_tensor_data(ogm_gguf *g, uint64_t index, const void **data, uint64_t *len) {
  if (!g || index >= g->tensors.size() || !data || !len) return OGM_ERR_INVALID;
  const uint8_t *p;
  int rc = tensor_bytes(g, g->tensors[index], &p, len);
  if (rc == OGM_OK) *data = p;
  return rc;
}

// LoadedModel::matrix (loader.rs:1552-1580): 2-D, dims[0] = row length, dims[1] = rows, and
// row_bytes * rows must equal the tensor's size.
extern "C" int ogm_gguf_matrix(ogm_gguf *g, const char *name, uint32_t *ggml_type, uint32_t *in_dim,
                               uint32_t *out_dim, size_t *row_bytes, const void **raw) {
  if (!g || !name) return OGM_ERR_INVALID;
  const int64_t idx = ogm_gguf_find_tensor(g, name);
  if (idx < 0) {
    g->err = std::string("model is missing tensor '") + name + "'";
    return OGM_ERR_INVALID;
  }
  const Tensor &t = g->tensors[(size_t)idx];
  if (t.dims.size() != 2) {
    g->err = std::string("tensor '") + name + "' is not a 2D matrix";
    return OGM_ERR_INVALID;
  }
  const uint8_t *p;
  uint64_t len;
  int rc = tensor_bytes(g, t, &p, &len);
  if (rc != OGM_OK) return rc;
  uint32_t bb, be;
  block_layout(t.ggml_type, &bb, &be);
  if (t.dims[0] % be != 0 || t.dims[0] > UINT32_MAX || t.dims[1] > UINT32_MAX) {
    g->err = std::string("tensor '") + name + "': row length is not a whole number of blocks";
    return OGM_ERR_INVALID;
  }
  const uint64_t rb = t.dims[0] / be * bb;
  if (rb * t.dims[1] != len) {
    g->err = std::string("tensor '") + name + "': row size x rows doesn't match the tensor's total bytes";
    return OGM_ERR_INVALID;
  }
  if (ggml_type) *ggml_type = t.ggml_type;
  if (in_dim) *in_dim = (uint32_t)t.dims[0];
  if (out_dim) *out_dim = (uint32_t)t.dims[1];
  if (row_bytes) *row_bytes = (size_t)rb;
  if (raw) *raw = p;
  return OGM_OK;
}

extern "C" int ogm_gguf_upload_matrix(ogm_ctx *ctx, ogm_gguf *g, const char *name, ogm_weight **out) {
  if (!ctx || !g || !out) return OGM_ERR_INVALID;
  uint32_t type, in_dim, out_dim;
  size_t rb;
  const void *raw;
  int rc = ogm_gguf_matrix(g, name, &type, &in_dim, &out_dim, &rb, &raw);
  if (rc != OGM_OK) return rc;
  if (!ogm_supports(type, in_dim)) {
    g->err = std::string("tensor '") + name + "': no kernel for ggml_type " + std::to_string(type) +
             " at row length " + std::to_string(in_dim);
    return OGM_ERR_UNSUPPORTED;
  }
  // cache key as QuantMatrix::cache_key (loader.rs:674-679): address and length of the mapped bytes
  rc = ogm_weight_upload(ctx, type, raw, rb, in_dim, out_dim, (uint64_t)(uintptr_t)raw, (uint64_t)rb * out_dim, out);
  if (rc != OGM_OK) g->err = std::string("tensor '") + name + "': " + ogm_last_error(ctx);
  return rc;
}
