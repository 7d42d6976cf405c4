// GGUF v2/v3 file reader: header, metadata key/values, tensor infos, alignment -- what Caten's
// external/gguf/{gguf-file,metadata,tensor-info}.lisp parse -- over an mmap of the file, so tensor
// bytes go from the page cache straight to the device, still packed (the reference dequantises
// every tensor on the host at load, external/gguf/tensor-info.lisp:71-77).
#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string>
#include <vector>

#include "common.h"

namespace cthip {

struct GGUFValue {
  std::string key;
  uint32_t type = 0;       // gguf metadata value type (metadata.lisp:3-17)
  uint32_t elem_type = 0;  // arrays
  uint64_t count = 1;      // arrays: element count
  const uint8_t *data = nullptr;  // first byte of the value (after array header / string length for scalars)
  uint64_t str_len = 0;    // strings
};

struct GGUFTensor {
  std::string name;
  uint32_t n_dims = 0;
  int64_t dims[4] = {1, 1, 1, 1};  // as stored: dims[0] is the innermost (contiguous) axis
  uint32_t type = 0;
  uint64_t rel_offset = 0, abs_offset = 0, nbytes = 0;
};

struct GGUF {
  int fd = -1;
  const uint8_t *base = nullptr;
  size_t size = 0;
  uint32_t version = 0;
  uint64_t alignment = 32;
  std::vector<GGUFValue> meta;
  std::vector<GGUFTensor> tensors;
};

struct Cursor {
  const uint8_t *p, *end;
  bool ok = true;
  bool need(size_t n) {
    if (!ok || (size_t)(end - p) < n) ok = false;
    return ok;
  }
  template <typename T>
  T get() {
    T v{};
    if (need(sizeof(T))) {
      memcpy(&v, p, sizeof(T));
      p += sizeof(T);
    }
    return v;
  }
  std::string str() {  // gguf-string (helpers.lisp:4-10): u64 length + utf-8 bytes
    uint64_t n = get<uint64_t>();
    std::string s;
    if (need(n)) {
      s.assign((const char *)p, n);
      p += n;
    }
    return s;
  }
};

static size_t scalar_size(uint32_t t) {
  switch (t) {
    case 0: case 1: case 7: return 1;
    case 2: case 3: return 2;
    case 4: case 5: case 6: return 4;
    case 10: case 11: case 12: return 8;
    default: return 0;
  }
}

static bool skip_value(Cursor &c, uint32_t type, GGUFValue *out) {
  if (type == 8) {
    uint64_t n = c.get<uint64_t>();
    if (out) {
      out->str_len = n;
      out->data = c.p;
    }
    if (!c.need(n)) return false;
    c.p += n;
    return true;
  }
  if (type == 9) {
    uint32_t et = c.get<uint32_t>();
    uint64_t n = c.get<uint64_t>();
    if (out) {
      out->elem_type = et;
      out->count = n;
      out->data = c.p;
    }
    if (et == 9) return false;  // nested arrays are not produced by any writer
    for (uint64_t i = 0; i < n && c.ok; i++)
      if (!skip_value(c, et, nullptr)) return false;
    return c.ok;
  }
  size_t sz = scalar_size(type);
  if (sz == 0) return false;
  if (out) out->data = c.p;
  if (!c.need(sz)) return false;
  c.p += sz;
  return true;
}

static uint64_t tensor_nbytes(uint32_t type, uint64_t n) {
  switch (type) {
    case CTHIP_F32: return n * 4;
    case CTHIP_F16: return n * 2;
    case CTHIP_Q8_0: return (n + 31) / 32 * 34;
    case CTHIP_Q4_0: return n / 32 * 18;
    default: return 0;  // other ggml types: known ids (tensor-info.lisp:3-31), no decoder here either
  }
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_gguf_open(void **out, const char *path) {
  if (!out || !path) return fail(CTHIP_E_BAD_ARG, "cthip_gguf_open: null argument");
  int fd = open(path, O_RDONLY);
  if (fd < 0) return fail(CTHIP_E_BAD_ARG, "cthip_gguf_open: cannot open '%s': %s", path, strerror(errno));
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 24) {
    close(fd);
    return fail(CTHIP_E_BAD_ARG, "cthip_gguf_open: '%s' is too short to be a GGUF file", path);
  }
  void *m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
  if (m == MAP_FAILED) {
    close(fd);
    return fail(CTHIP_E_BAD_ARG, "cthip_gguf_open: mmap of '%s' failed: %s", path, strerror(errno));
  }
  GGUF *g = new GGUF();
  g->fd = fd;
  g->base = (const uint8_t *)m;
  g->size = (size_t)st.st_size;
  auto bail = [&](const char *why) {
    munmap((void *)g->base, g->size);
    close(g->fd);
    delete g;
    return fail(CTHIP_E_BAD_ARG, "cthip_gguf_open: '%s': %s", path, why);
  };
  Cursor c{g->base, g->base + g->size};
  if (memcmp(c.p, "GGUF", 4) != 0) return bail("expecting the header to be GGUF (gguf-file.lisp:74)");
  c.p += 4;
  g->version = c.get<uint32_t>();
  if (g->version < 2 || g->version > 3) return bail("unsupported GGUF version (2 and 3 use 64-bit counts)");
  const uint64_t n_tensors = c.get<uint64_t>();
  const uint64_t n_kv = c.get<uint64_t>();
  if (n_tensors > (1u << 24) || n_kv > (1u << 24)) return bail("implausible tensor / metadata count");
  for (uint64_t i = 0; i < n_kv; i++) {
    GGUFValue v;
    v.key = c.str();
    v.type = c.get<uint32_t>();
    if (!c.ok || !skip_value(c, v.type, &v)) return bail("truncated or malformed metadata");
    if (v.key == "general.alignment" && v.type != 6 && v.type != 7 && v.type != 12 && scalar_size(v.type) >= 1) {
      uint64_t a = 0;
      memcpy(&a, v.data, scalar_size(v.type));
      if (a == 0 || (a & (a - 1))) return bail("general.alignment is not a power of two");
      g->alignment = a;
    }
    g->meta.push_back(v);
  }
  for (uint64_t i = 0; i < n_tensors; i++) {
    GGUFTensor t;
    t.name = c.str();
    t.n_dims = c.get<uint32_t>();
    if (!c.ok || t.n_dims > 4) return bail("malformed tensor info");
    uint64_t n = 1;
    for (uint32_t d = 0; d < t.n_dims; d++) {
      const uint64_t dim = c.get<uint64_t>();
      // an element count beyond what the file could hold is a malformed header, not a size to multiply on with
      if (dim > (uint64_t)INT64_MAX || __builtin_mul_overflow(n, dim, &n) || n > (uint64_t)g->size * 32)
        return bail("implausible tensor dimensions");
      t.dims[d] = (int64_t)dim;
    }
    t.type = c.get<uint32_t>();
    t.rel_offset = c.get<uint64_t>();
    if (!c.ok) return bail("truncated tensor info");
    if (t.rel_offset > g->size) return bail("tensor offset lies past the end of the file");
    t.nbytes = tensor_nbytes(t.type, n);
    g->tensors.push_back(t);
  }
  // offsets are relative to the end of the tensor infos, aligned up (tensor-info.lisp:88-98)
  const uint64_t start = (uint64_t)(c.p - g->base);
  for (GGUFTensor &t : g->tensors) {
    const uint64_t off = start + t.rel_offset;
    t.abs_offset = off + (g->alignment - off % g->alignment) % g->alignment;
    if (t.abs_offset > g->size || t.nbytes > g->size - t.abs_offset) return bail("tensor data runs past the end of the file");
  }
  *out = g;
  return 0;
}

int cthip_gguf_close(void *h) {
  if (!h) return 0;
  GGUF *g = (GGUF *)h;
  munmap((void *)g->base, g->size);
  close(g->fd);
  delete g;
  return 0;
}

int cthip_gguf_version(const void *h) { return h ? (int)((const GGUF *)h)->version : -1; }
int64_t cthip_gguf_tensor_count(const void *h) { return h ? (int64_t)((const GGUF *)h)->tensors.size() : -1; }
int64_t cthip_gguf_metadata_count(const void *h) { return h ? (int64_t)((const GGUF *)h)->meta.size() : -1; }
int64_t cthip_gguf_alignment(const void *h) { return h ? (int64_t)((const GGUF *)h)->alignment : -1; }

int cthip_gguf_tensor_info(const void *h, int64_t i, const char **name, int *ggml_type, int *n_dims, int64_t dims[4],
                           int64_t *abs_offset, int64_t *nbytes) {
  const GGUF *g = (const GGUF *)h;
  if (!g || i < 0 || i >= (int64_t)g->tensors.size()) return fail(CTHIP_E_BAD_ARG, "cthip_gguf_tensor_info: index %lld", (long long)i);
  const GGUFTensor &t = g->tensors[i];
  if (name) *name = t.name.c_str();
  if (ggml_type) *ggml_type = (int)t.type;
  if (n_dims) *n_dims = (int)t.n_dims;
  if (dims)
    for (int d = 0; d < 4; d++) dims[d] = t.dims[d];
  if (abs_offset) *abs_offset = (int64_t)t.abs_offset;
  if (nbytes) *nbytes = (int64_t)t.nbytes;
  return 0;
}

int64_t cthip_gguf_find_tensor(const void *h, const char *name) {
  const GGUF *g = (const GGUF *)h;
  if (!g || !name) return -1;
  for (size_t i = 0; i < g->tensors.size(); i++)
    if (g->tensors[i].name == name) return (int64_t)i;
  return -1;
}

const void *cthip_gguf_tensor_data(const void *h, int64_t i) {
  const GGUF *g = (const GGUF *)h;
  if (!g || i < 0 || i >= (int64_t)g->tensors.size()) return nullptr;
  return g->base + g->tensors[i].abs_offset;
}

int64_t cthip_gguf_find_metadata(const void *h, const char *key) {
  const GGUF *g = (const GGUF *)h;
  if (!g || !key) return -1;
  for (size_t i = 0; i < g->meta.size(); i++)
    if (g->meta[i].key == key) return (int64_t)i;
  return -1;
}

int cthip_gguf_metadata_info(const void *h, int64_t i, const char **key, int *type, int *elem_type, int64_t *count) {
  const GGUF *g = (const GGUF *)h;
  if (!g || i < 0 || i >= (int64_t)g->meta.size()) return fail(CTHIP_E_BAD_ARG, "cthip_gguf_metadata_info: index %lld", (long long)i);
  const GGUFValue &v = g->meta[i];
  if (key) *key = v.key.c_str();
  if (type) *type = (int)v.type;
  if (elem_type) *elem_type = (int)v.elem_type;
  if (count) *count = (int64_t)v.count;
  return 0;
}

// scalar metadata as a double (integers, floats, bool)
int cthip_gguf_metadata_number(const void *h, int64_t i, double *out) {
  const GGUF *g = (const GGUF *)h;
  if (!g || !out || i < 0 || i >= (int64_t)g->meta.size()) return fail(CTHIP_E_BAD_ARG, "cthip_gguf_metadata_number: bad argument");
  const GGUFValue &v = g->meta[i];
  switch (v.type) {
    case 0: *out = *(const uint8_t *)v.data; break;
    case 1: *out = *(const int8_t *)v.data; break;
    case 2: { uint16_t x; memcpy(&x, v.data, 2); *out = x; break; }
    case 3: { int16_t x; memcpy(&x, v.data, 2); *out = x; break; }
    case 4: { uint32_t x; memcpy(&x, v.data, 4); *out = x; break; }
    case 5: { int32_t x; memcpy(&x, v.data, 4); *out = x; break; }
    case 6: { float x; memcpy(&x, v.data, 4); *out = x; break; }
    case 7: *out = *(const uint8_t *)v.data ? 1.0 : 0.0; break;
    case 10: { uint64_t x; memcpy(&x, v.data, 8); *out = (double)x; break; }
    case 11: { int64_t x; memcpy(&x, v.data, 8); *out = (double)x; break; }
    case 12: { double x; memcpy(&x, v.data, 8); *out = x; break; }
    default: return fail(CTHIP_E_BAD_ARG, "cthip_gguf_metadata_number: '%s' is not a scalar number", v.key.c_str());
  }
  return 0;
}

// string metadata, or element `j` of an array of strings; *data is not NUL-terminated
int cthip_gguf_metadata_string(const void *h, int64_t i, int64_t j, const char **data, int64_t *len) {
  const GGUF *g = (const GGUF *)h;
  if (!g || !data || !len || i < 0 || i >= (int64_t)g->meta.size()) return fail(CTHIP_E_BAD_ARG, "cthip_gguf_metadata_string: bad argument");
  const GGUFValue &v = g->meta[i];
  if (v.type == 8) {
    *data = (const char *)v.data;
    *len = (int64_t)v.str_len;
    return 0;
  }
  if (v.type == 9 && v.elem_type == 8 && j >= 0 && (uint64_t)j < v.count) {
    const uint8_t *p = v.data;
    for (int64_t k = 0;; k++) {
      uint64_t n;
      memcpy(&n, p, 8);
      if (k == j) {
        *data = (const char *)(p + 8);
        *len = (int64_t)n;
        return 0;
      }
      p += 8 + n;
    }
  }
  return fail(CTHIP_E_BAD_ARG, "cthip_gguf_metadata_string: '%s' holds no string %lld", v.key.c_str(), (long long)j);
}

// `remap-key` of apps/gpt2/gpt2.lisp:52-75: GGUF tensor names -> the Transformer's state-dict keys
static std::string remap_gpt2(std::string k) {
  static const char *table[][2] = {
      {"blk.", "h."}, {"token_embd.weight", "wte.weight"}, {"position_embd.weight", "wpe.weight"},
      {".attn_norm.weight", ".ln_1.affine"}, {".attn_norm.bias", ".ln_1.bias"},
      {".attn_qkv.weight", ".attn.c_attn.weight"}, {".attn_qkv.bias", ".attn.c_attn.bias"},
      {".ffn_down.weight", ".mlp.c_proj.weight"}, {".ffn_down.bias", ".mlp.c_proj.bias"},
      {".ffn_norm.weight", ".ln_2.affine"}, {".ffn_norm.bias", ".ln_2.bias"},
      {".ffn_up.weight", ".mlp.c_fc.weight"}, {".ffn_up.bias", ".mlp.c_fc.bias"},
      {".attn_output.weight", ".attn.c_proj.weight"}, {".attn_output.bias", ".attn.c_proj.bias"},
      {"output.weight", "lm_head.weight"}, {"output_norm.bias", "ln_f.bias"}, {"output_norm.weight", "ln_f.affine"}};
  for (auto &r : table) {
    const std::string from = r[0], to = r[1];
    size_t pos = 0;
    while ((pos = k.find(from, pos)) != std::string::npos) {
      k.replace(pos, from.size(), to);
      pos += to.size();
    }
  }
  return k;
}

// llama.cpp tensor names -> the keys of the Llama-shaped session
static std::string remap_llama(std::string k) {
  static const char *table[][2] = {
      {"blk.", "layers."}, {"token_embd.weight", "tok_embeddings.weight"}, {".attn_norm.weight", ".attention_norm.weight"},
      {".attn_q.weight", ".attention.wq.weight"}, {".attn_k.weight", ".attention.wk.weight"},
      {".attn_v.weight", ".attention.wv.weight"}, {".attn_output.weight", ".attention.wo.weight"},
      {".ffn_gate.weight", ".feed_forward.w1.weight"}, {".ffn_down.weight", ".feed_forward.w2.weight"},
      {".ffn_up.weight", ".feed_forward.w3.weight"}, {"output_norm.weight", "norm.weight"}};
  for (auto &r : table) {
    const std::string from = r[0], to = r[1];
    size_t pos = k.find(from);
    if (pos != std::string::npos) k.replace(pos, from.size(), to);
  }
  return k;
}

// make-gpt2's load path (apps/gpt2/gpt2.lisp:82-93: gguf->state-dict, remap keys, load-state-dict) for a
// decoder session: every tensor of the file whose remapped name the model knows is uploaded from the
// mapping, packed.  Returns the number of tensors loaded in *n_loaded.
int cthip_decoder_load_gguf(void *dec, const void *h, int arch, int *n_loaded) {
  const GGUF *g = (const GGUF *)h;
  if (!dec || !g) return fail(CTHIP_E_BAD_ARG, "cthip_decoder_load_gguf: null argument");
  int n = 0;
  for (size_t i = 0; i < g->tensors.size(); i++) {
    const GGUFTensor &t = g->tensors[i];
    const std::string key = arch == CTHIP_ARCH_GPT2 ? remap_gpt2(t.name) : remap_llama(t.name);
    if (t.nbytes == 0)
      return fail(CTHIP_E_UNSUPPORTED, "cthip_decoder_load_gguf: tensor '%s' has ggml type %u (supported: F32, F16, Q4_0, Q8_0)",
                  t.name.c_str(), t.type);
    // dims are stored innermost first; (rows, cols) = (product of the outer dims, dims[0]) (tensor-info.lisp:104-120)
    int64_t rows = 1;
    for (uint32_t d = 1; d < t.n_dims; d++) rows *= t.dims[d];
    const int64_t cols = t.n_dims ? t.dims[0] : 1;
    int rc = cthip_decoder_load(dec, key.c_str(), (int)t.type, g->base + t.abs_offset, rows, cols);
    if (rc == CTHIP_E_BAD_ARG && strstr(cthip_last_error(), "is not a tensor of this model")) continue;  // e.g. tokenizer extras
    if (rc) return rc;
    n++;
  }
  if (n_loaded) *n_loaded = n;
  return 0;
}

}  // extern "C"
