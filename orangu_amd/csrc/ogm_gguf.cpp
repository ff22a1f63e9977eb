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
    case 23: *bytes = 136; *elems = 256; return true; // IQ4_XS
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

// ---- a Llama-family file as a device-resident decoder ---------------------------------------

namespace {

// A small tensor (norm weights, biases, frequency factors) as f32, as LoadedModel::tensor hands
// it out (loader.rs:1512-1550): F32 as is, F16 and BF16 widened.
int small_tensor_f32(ogm_gguf *g, const std::string &name, uint64_t want, bool at_least, std::vector<float> *out) {
  const int64_t idx = ogm_gguf_find_tensor(g, name.c_str());
  if (idx < 0) {
    g->err = "model is missing tensor '" + name + "'";
    return OGM_ERR_INVALID;
  }
  const Tensor &t = g->tensors[(size_t)idx];
  const uint8_t *p;
  uint64_t len;
  int rc = tensor_bytes(g, t, &p, &len);
  if (rc != OGM_OK) return rc;
  uint64_t n = 1;
  for (uint64_t d : t.dims) n *= d;
  if (at_least ? n < want : n != want) {
    g->err = "tensor '" + name + "' has " + std::to_string(n) + " entries, need " + std::to_string(want);
    return OGM_ERR_INVALID;
  }
  out->resize((size_t)n);
  if (t.ggml_type == 0) {
    memcpy(out->data(), p, (size_t)n * 4);
  } else if (t.ggml_type == 1 || t.ggml_type == 30) {
    for (uint64_t i = 0; i < n; i++) {
      uint16_t h;
      memcpy(&h, p + 2 * i, 2);
      uint32_t bits;
      if (t.ggml_type == 30) {
        bits = (uint32_t)h << 16;
      } else {   // IEEE binary16 -> binary32, subnormals included (quant.rs:511-528)
        const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
        if (ex == 0) {
          if (man == 0) {
            bits = sign;
          } else {
            int e = -1;
            uint32_t m = man;
            do { m <<= 1; e++; } while ((m & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3FFu) << 13);
          }
        } else if (ex == 31) {
          bits = sign | 0x7F800000u | (man << 13);
        } else {
          bits = sign | ((ex + 112u) << 23) | (man << 13);
        }
      }
      memcpy(&(*out)[(size_t)i], &bits, 4);
    }
  } else {
    g->err = "tensor '" + name + "': ggml_type " + std::to_string(t.ggml_type) + " is not read as a vector here";
    return OGM_ERR_UNSUPPORTED;
  }
  return OGM_OK;
}

bool meta_u64_of(const ogm_gguf *g, const std::string &key, uint64_t *out) {
  return ogm_gguf_meta_u64(g, key.c_str(), out) == OGM_OK;
}

// metadata_f32 (loader.rs:1634-1645): only the float types count
bool meta_f32_of(const ogm_gguf *g, const std::string &key, float *out) {
  const Value *v = find_meta(g, key.c_str());
  if (!v || (v->type != 6 && v->type != 12)) return false;
  *out = (float)v->f;
  return true;
}

}  // namespace

extern "C" int ogm_llama_load_gguf(ogm_ctx *ctx, ogm_gguf *g, uint32_t max_ctx, ogm_llama **model,
                                   const ogm_weight **tok_embd, ogm_llama_config *cfg_out) {
  if (!ctx || !g || !model) return OGM_ERR_INVALID;
  const char *arch_c = nullptr;
  if (ogm_gguf_meta_string(g, "general.architecture", &arch_c, nullptr) != OGM_OK) {
    g->err = "GGUF file is missing general.architecture";
    return OGM_ERR_INVALID;
  }
  const std::string arch(arch_c);
  // LLAMA_STYLE_ARCHITECTURES (loader.rs:190): what LlamaModel runs
  static const char *const kLlamaStyle[] = {"llama", "qwen2", "qwen3", "mistral", "qwen3vl"};
  bool ours = false;
  for (const char *a : kLlamaStyle) ours = ours || arch == a;
  if (!ours) {
    g->err = "architecture '" + arch + "' is not a Llama-style one";
    return OGM_ERR_UNSUPPORTED;
  }
  // read_model_config (loader.rs:1652-1714)
  uint64_t n_embd, n_layer, n_head, n_head_kv, n_vocab, head_dim, rope_dim;
  struct { const char *suffix; uint64_t *dst; } required[] = {
      {"embedding_length", &n_embd}, {"block_count", &n_layer}, {"attention.head_count", &n_head}};
  for (auto &r : required)
    if (!meta_u64_of(g, arch + "." + r.suffix, r.dst)) {
      g->err = "GGUF file is missing " + arch + "." + r.suffix;
      return OGM_ERR_INVALID;
    }
  if (!meta_u64_of(g, arch + ".attention.head_count_kv", &n_head_kv)) n_head_kv = n_head;
  if (!meta_u64_of(g, arch + ".vocab_size", &n_vocab)) {
    uint32_t et;
    if (ogm_gguf_meta_array(g, "tokenizer.ggml.tokens", &et, &n_vocab) != OGM_OK) {
      g->err = "GGUF file has no vocab_size and no tokenizer.ggml.tokens";
      return OGM_ERR_INVALID;
    }
  }
  if (n_head == 0 || n_head_kv == 0) {
    g->err = arch + ".attention.head_count(_kv) must be nonzero";
    return OGM_ERR_INVALID;
  }
  if (!meta_u64_of(g, arch + ".attention.key_length", &head_dim)) head_dim = n_embd / n_head;
  if (head_dim == 0) {
    g->err = arch + ".attention.key_length must be nonzero";
    return OGM_ERR_INVALID;
  }
  if (!meta_u64_of(g, arch + ".rope.dimension_count", &rope_dim)) rope_dim = head_dim;
  float freq_base = 10000.0f, rms_eps = 1e-5f;
  (void)meta_f32_of(g, arch + ".rope.freq_base", &freq_base);
  (void)meta_f32_of(g, arch + ".attention.layer_norm_rms_epsilon", &rms_eps);
  // Every one of these is an untrusted u64 that ends up in a u32 field (and n_head * head_dim in a
  // u32 product inside ogm_llama_create): reject what does not fit before anything is uploaded.
  if (n_layer == 0 || n_layer > 4096 || n_embd > UINT32_MAX || n_vocab > UINT32_MAX || n_head > UINT32_MAX ||
      n_head_kv > UINT32_MAX || head_dim > UINT32_MAX || rope_dim > UINT32_MAX ||
      n_head * head_dim > UINT32_MAX || n_head_kv * head_dim > UINT32_MAX) {
    g->err = "model dimensions out of range";
    return OGM_ERR_INVALID;
  }

  // LlamaModel::load_with_backend (llama.rs:123-220)
  ogm_weight *embd = nullptr, *output = nullptr;
  int rc = ogm_gguf_upload_matrix(ctx, g, "token_embd.weight", &embd);
  if (rc != OGM_OK) return rc;
  if (ogm_gguf_find_tensor(g, "output.weight") >= 0) {
    if ((rc = ogm_gguf_upload_matrix(ctx, g, "output.weight", &output)) != OGM_OK) return rc;
  } else {
    output = embd;   // tied embeddings: the file omits output.weight
  }
  std::vector<float> output_norm;
  if ((rc = small_tensor_f32(g, "output_norm.weight", n_embd, false, &output_norm)) != OGM_OK) return rc;
  const uint64_t qd = n_head * head_dim, kvd = n_head_kv * head_dim;
  std::vector<ogm_llama_layer> layers((size_t)n_layer);
  std::vector<std::vector<float>> keep;   // the vectors the layer structs point into
  keep.reserve((size_t)n_layer * 7 + 2);
  uint32_t n_ff = 0;
  for (uint64_t i = 0; i < n_layer; i++) {
    const std::string blk = "blk." + std::to_string(i) + ".";
    ogm_llama_layer &L = layers[(size_t)i];
    memset(&L, 0, sizeof(L));
    struct { const char *name; const ogm_weight **dst; } mats[] = {
        {"attn_q.weight", &L.wq}, {"attn_k.weight", &L.wk}, {"attn_v.weight", &L.wv},
        {"attn_output.weight", &L.wo}, {"ffn_gate.weight", &L.w_gate}, {"ffn_up.weight", &L.w_up},
        {"ffn_down.weight", &L.w_down}};
    for (auto &mt : mats) {
      ogm_weight *w = nullptr;
      if ((rc = ogm_gguf_upload_matrix(ctx, g, (blk + mt.name).c_str(), &w)) != OGM_OK) return rc;
      *mt.dst = w;
    }
    if (i == 0) {
      uint32_t t, in_dim, out_dim;
      if ((rc = ogm_gguf_matrix(g, (blk + "ffn_gate.weight").c_str(), &t, &in_dim, &out_dim, nullptr, nullptr)) != OGM_OK)
        return rc;
      n_ff = out_dim;
    }
    struct { const char *name; const float **dst; uint64_t n; bool optional; } vecs[] = {
        {"attn_norm.weight", &L.attn_norm, n_embd, false}, {"ffn_norm.weight", &L.ffn_norm, n_embd, false},
        {"attn_q.bias", &L.q_bias, qd, true},              {"attn_k.bias", &L.k_bias, kvd, true},
        {"attn_v.bias", &L.v_bias, kvd, true},             {"attn_q_norm.weight", &L.q_norm, head_dim, true},
        {"attn_k_norm.weight", &L.k_norm, head_dim, true}};
    for (auto &v : vecs) {
      if (v.optional && ogm_gguf_find_tensor(g, (blk + v.name).c_str()) < 0) continue;
      keep.emplace_back();
      if ((rc = small_tensor_f32(g, blk + v.name, v.n, false, &keep.back())) != OGM_OK) return rc;
      *v.dst = keep.back().data();
    }
  }
  // rope_freqs.weight (llama.rs:186-201): at least rope_dim / 2 entries
  std::vector<float> factors;
  const bool has_factors = ogm_gguf_find_tensor(g, "rope_freqs.weight") >= 0;
  if (has_factors && (rc = small_tensor_f32(g, "rope_freqs.weight", rope_dim / 2, true, &factors)) != OGM_OK) return rc;

  ogm_llama_config cfg;
  memset(&cfg, 0, sizeof(cfg));
  cfg.n_layer = (uint32_t)n_layer;
  cfg.n_embd = (uint32_t)n_embd;
  cfg.n_head = (uint32_t)n_head;
  cfg.n_head_kv = (uint32_t)n_head_kv;
  cfg.head_dim = (uint32_t)head_dim;
  cfg.n_ff = n_ff;
  cfg.n_vocab = (uint32_t)n_vocab;
  cfg.rope_dim = (uint32_t)rope_dim;
  cfg.max_ctx = max_ctx;
  cfg.rms_eps = rms_eps;
  cfg.rope_freq_base = freq_base;
  cfg.rope_neox = (arch == "llama" || arch == "mistral") ? 0u : 1u;   // rope_layout_for, llama.rs:115-120
  cfg.rope_freq_factors = has_factors ? factors.data() : nullptr;
  rc = ogm_llama_create(ctx, &cfg, layers.data(), output_norm.data(), output, model);
  if (rc != OGM_OK) {
    g->err = std::string("ogm_llama_create: ") + ogm_last_error(ctx);
    return rc;
  }
  if (tok_embd) *tok_embd = embd;
  if (cfg_out) {
    *cfg_out = cfg;
    cfg_out->rope_freq_factors = nullptr;   // the array above does not outlive this call
  }
  return OGM_OK;
}
