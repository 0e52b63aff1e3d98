// GGUF v2/v3 container reader and the ternary-tensor loader on top of it: the data format on the
// caller's side of upload_weights. Follows read_gguf (crates/tritium-format/src/gguf.rs:550-664)
// for the container and load_ternary (crates/tritium-nn/src/model/weights.rs:143-333) for turning a
// tensor of type I2_S, TQ1_0 or TQ2_0 into packed rows plus one scale per output row.
// Host code only. Every read is length-checked; no input can make it read out of bounds.
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <new>
#include <string>
#include <string_view>
#include <vector>

#include "tk_host.h"

#define TKCHK_HOST(call)            \
  do {                              \
    const int rc_ = (call);         \
    if (rc_ != TK_OK) return rc_;   \
  } while (0)

namespace {

constexpr uint64_t kMaxStringLen = 64ull * 1024 * 1024;  // gguf.rs:38-40
constexpr uint64_t kMaxCount = 1ull << 32;               // gguf.rs:42-43
constexpr int kMaxMetadataDepth = 8;                     // gguf.rs:45-46
constexpr uint64_t kMaxMetadataArrayElements = 16000000; // gguf.rs:48-49
constexpr uint32_t kMaxDims = 8;                         // gguf.rs:51-53
constexpr uint64_t kDefaultAlignment = 32;               // gguf.rs:33
constexpr uint32_t kTypeTq1 = 34, kTypeTq2 = 35, kTypeI2s = 36, kTypeQ2 = 42;

struct Value {
  uint32_t type = 0;  // GGUF metadata value type 0..12
  uint64_t bits = 0;  // scalars: the value's little-endian bits, zero-extended
  std::string str;
  std::vector<Value> items;
};

struct Tensor {
  std::string name;
  std::vector<uint64_t> dims;
  uint32_t ggml_type = 0;
  uint64_t offset = 0, n_bytes = 0;
};

struct ParseError {
  int kind;
  uint64_t detail;
};

// Strict UTF-8 as Rust's str::from_utf8 accepts it: shortest forms only, no surrogates, <= U+10FFFF.
bool valid_utf8(const uint8_t *s, size_t n) {
  size_t i = 0;
  while (i < n) {
    const uint8_t c = s[i];
    if (c < 0x80) { ++i; continue; }
    size_t need;
    uint8_t lo = 0x80, hi = 0xBF;
    if (c >= 0xC2 && c <= 0xDF) need = 1;
    else if (c == 0xE0) { need = 2; lo = 0xA0; }
    else if (c == 0xED) { need = 2; hi = 0x9F; }
    else if (c >= 0xE1 && c <= 0xEF) need = 2;
    else if (c == 0xF0) { need = 3; lo = 0x90; }
    else if (c >= 0xF1 && c <= 0xF3) need = 3;
    else if (c == 0xF4) { need = 3; hi = 0x8F; }
    else return false;
    if (n - i <= need) return false;
    if (s[i + 1] < lo || s[i + 1] > hi) return false;
    for (size_t j = 2; j <= need; ++j)
      if ((s[i + j] & 0xC0) != 0x80) return false;
    i += need + 1;
  }
  return true;
}

struct Cursor {
  const uint8_t *buf;
  size_t len, pos = 0;
  const uint8_t *take(size_t n) {
    if (n > len - pos) throw ParseError{TK_GGUF_TRUNCATED, 0};
    const uint8_t *p = buf + pos;
    pos += n;
    return p;
  }
  uint64_t le(size_t n) {
    const uint8_t *p = take(n);
    uint64_t v = 0;
    for (size_t i = 0; i < n; ++i) v |= (uint64_t)p[i] << (8 * i);
    return v;
  }
  std::string str() {
    const uint64_t n = le(8);
    if (n > kMaxStringLen) throw ParseError{TK_GGUF_STRING_TOO_LONG, 0};
    const uint8_t *p = take((size_t)n);
    if (!valid_utf8(p, (size_t)n)) throw ParseError{TK_GGUF_INVALID_UTF8, 0};
    return std::string((const char *)p, (size_t)n);
  }
};

// gguf.rs:297-355
Value read_value(Cursor &cur, uint32_t type, int depth, uint64_t &total_array_elements) {
  static const int width[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
  Value v;
  v.type = type;
  if (type > 12) throw ParseError{TK_GGUF_UNKNOWN_VALUE_TYPE, type};
  if (type == 8) {
    v.str = cur.str();
  } else if (type == 9) {
    if (depth >= kMaxMetadataDepth) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
    const uint32_t child = (uint32_t)cur.le(4);
    if (child > 12) throw ParseError{TK_GGUF_UNKNOWN_VALUE_TYPE, child};
    const uint64_t count = cur.le(8);
    if (count > kMaxCount) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
    total_array_elements += count;  // both below 2^33: cannot wrap
    if (total_array_elements > kMaxMetadataArrayElements) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
    v.bits = child;
    v.items.reserve((size_t)(count < 1024 ? count : 1024));
    for (uint64_t i = 0; i < count; ++i) v.items.push_back(read_value(cur, child, depth + 1, total_array_elements));
  } else {
    v.bits = cur.le((size_t)width[type]);
    if (type == 7 && v.bits > 1) throw ParseError{TK_GGUF_INVALID_BOOLEAN, v.bits};
  }
  return v;
}

// (block bytes, elements per block) of the types the reader sizes (gguf.rs:407-422)
bool type_block_layout(uint32_t t, uint64_t &bytes, uint64_t &elems) {
  switch (t) {
    case 0: bytes = 4; elems = 1; return true;    // F32
    case 1: bytes = 2; elems = 1; return true;    // F16
    case 8: bytes = 34; elems = 32; return true;  // Q8_0
    case 24: bytes = 1; elems = 1; return true;   // I8
    case 25: bytes = 2; elems = 1; return true;   // I16
    case 26: bytes = 4; elems = 1; return true;   // I32
    case 30: bytes = 2; elems = 1; return true;   // BF16
    case kTypeTq1: bytes = 54; elems = 256; return true;
    case kTypeTq2: bytes = 66; elems = 256; return true;
    case kTypeQ2: bytes = 18; elems = 64; return true;
    default: return false;
  }
}

// gguf.rs:432-455: blocks never straddle rows; unknown types are sized 0
uint64_t tensor_n_bytes(uint32_t type, const std::vector<uint64_t> &dims) {
  uint64_t bb, be;
  if (!type_block_layout(type, bb, be)) return 0;
  const uint64_t row_elements = dims.empty() ? 1 : dims[0];
  if (row_elements % be != 0) throw ParseError{TK_GGUF_INVALID_TENSOR_SHAPE, 0};
  uint64_t rows = 1, out;
  for (size_t i = 1; i < dims.size(); ++i)
    if (__builtin_mul_overflow(rows, dims[i], &rows)) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
  if (__builtin_mul_overflow(row_elements / be, bb, &out) || __builtin_mul_overflow(out, rows, &out))
    throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
  return out;
}

float f32_from_bits(uint32_t b) {
  float f;
  std::memcpy(&f, &b, 4);
  return f;
}

}  // namespace

struct tk_gguf {
  uint32_t version = 0;
  uint64_t alignment = kDefaultAlignment, tensor_data_offset = 0;
  // a later duplicate key replaces the earlier one, as BTreeMap::insert does; std::less<> lets the
  // getters look a C string up without building a std::string (nothing in them can throw)
  std::map<std::string, Value, std::less<>> metadata;
  std::vector<Tensor> tensors;
};

namespace {

void parse(const uint8_t *buf, size_t len, tk_gguf &g) {
  Cursor cur{buf, len};
  if (std::memcmp(cur.take(4), "GGUF", 4) != 0) throw ParseError{TK_GGUF_BAD_MAGIC, 0};
  g.version = (uint32_t)cur.le(4);
  if (g.version != 2 && g.version != 3) throw ParseError{TK_GGUF_UNSUPPORTED_VERSION, g.version};
  const uint64_t tensor_count = cur.le(8), kv_count = cur.le(8);
  if (tensor_count > kMaxCount || kv_count > kMaxCount) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
  uint64_t total_array_elements = 0;
  for (uint64_t i = 0; i < kv_count; ++i) {
    std::string key = cur.str();
    const uint32_t type = (uint32_t)cur.le(4);
    g.metadata[std::move(key)] = read_value(cur, type, 0, total_array_elements);
  }
  // general.alignment: absent -> 32; otherwise a nonzero U32 multiple of eight (gguf.rs:509-515)
  auto al = g.metadata.find("general.alignment");
  if (al != g.metadata.end()) {
    if (al->second.type != 4 || al->second.bits == 0 || al->second.bits % 8 != 0) throw ParseError{TK_GGUF_INVALID_ALIGNMENT, 0};
    g.alignment = al->second.bits;
  }
  for (uint64_t i = 0; i < tensor_count; ++i) {
    Tensor t;
    t.name = cur.str();
    const uint32_t n_dims = (uint32_t)cur.le(4);
    if (n_dims > kMaxDims) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
    for (uint32_t d = 0; d < n_dims; ++d) t.dims.push_back(cur.le(8));
    t.ggml_type = (uint32_t)cur.le(4);
    t.offset = cur.le(8);
    g.tensors.push_back(std::move(t));
  }
  const uint64_t header_end = cur.pos, bumped = header_end + (g.alignment - 1);
  g.tensor_data_offset = bumped - bumped % g.alignment;
  const uint64_t data_len = len > g.tensor_data_offset ? len - g.tensor_data_offset : 0;
  for (Tensor &t : g.tensors) {
    uint64_t n = 1, end;
    for (uint64_t d : t.dims)
      if (__builtin_mul_overflow(n, d, &n)) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
    t.n_bytes = tensor_n_bytes(t.ggml_type, t.dims);
    if (t.n_bytes > 0) {
      if (__builtin_add_overflow(t.offset, t.n_bytes, &end)) throw ParseError{TK_GGUF_DIMS_OVERFLOW, 0};
      if (end > data_len) throw ParseError{TK_GGUF_OFFSET_OUT_OF_BOUNDS, 0};
    } else if (t.offset > data_len) {
      throw ParseError{TK_GGUF_OFFSET_OUT_OF_BOUNDS, 0};
    }
  }
}

const char *kind_text(int kind) {
  switch (kind) {  // gguf.rs:99-131
    case TK_GGUF_BAD_MAGIC: return "bad GGUF magic (expected 'GGUF')";
    case TK_GGUF_UNSUPPORTED_VERSION: return "unsupported GGUF version";
    case TK_GGUF_TRUNCATED: return "buffer truncated: read past end of input";
    case TK_GGUF_STRING_TOO_LONG: return "GGUF string length exceeds the sane bound";
    case TK_GGUF_DIMS_OVERFLOW: return "tensor dimensions or count overflowed";
    case TK_GGUF_INVALID_TENSOR_SHAPE: return "tensor shape or payload length is incompatible with its GGML type";
    case TK_GGUF_INVALID_ALIGNMENT: return "general.alignment must be a nonzero U32 multiple of eight";
    case TK_GGUF_INVALID_BOOLEAN: return "GGUF BOOL byte is not zero or one";
    case TK_GGUF_OFFSET_OUT_OF_BOUNDS: return "tensor offset/size outside the data section";
    case TK_GGUF_UNKNOWN_VALUE_TYPE: return "unknown metadata value type";
    case TK_GGUF_INVALID_UTF8: return "GGUF string was not valid UTF-8";
    default: return "ok";
  }
}

// The value a getter addresses: the key's value (index < 0) or element `index` of its array.
const Value *lookup(const tk_gguf *g, const char *key, long long index) {
  if (!g || !key) return nullptr;
  auto it = g->metadata.find(std::string_view(key));
  if (it == g->metadata.end()) return nullptr;
  const Value *v = &it->second;
  if (index < 0) return v;
  if (v->type != 9 || (uint64_t)index >= v->items.size()) return nullptr;
  return &v->items[(size_t)index];
}

void fill_info(const Tensor &t, tk_gguf_tensor *out) {
  std::memset(out, 0, sizeof *out);
  out->name = t.name.c_str();
  out->n_dims = (uint32_t)t.dims.size();
  for (size_t i = 0; i < t.dims.size(); ++i) out->dims[i] = t.dims[i];
  out->ggml_type = t.ggml_type;
  out->offset = t.offset;
  out->n_bytes = t.n_bytes;
}

const Tensor *find_tensor(const tk_gguf *g, const char *name) {
  const std::string_view want(name);
  for (const Tensor &t : g->tensors)
    if (std::string_view(t.name) == want) return &t;
  return nullptr;
}

}  // namespace

extern "C" int tk_gguf_open(const uint8_t *buf, size_t len, tk_gguf **out, int *error_kind, uint64_t *error_detail) {
  if (error_kind) *error_kind = TK_GGUF_OK;
  if (error_detail) *error_detail = 0;
  if (!out || (!buf && len)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_gguf_open: null pointer");
  *out = nullptr;
  try {
    std::unique_ptr<tk_gguf> g(new tk_gguf);
    parse(buf, len, *g);
    *out = g.release();
    return TK_OK;
  } catch (const ParseError &e) {
    if (error_kind) *error_kind = e.kind;
    if (error_detail) *error_detail = e.detail;
    if (e.kind == TK_GGUF_UNSUPPORTED_VERSION || e.kind == TK_GGUF_INVALID_BOOLEAN || e.kind == TK_GGUF_UNKNOWN_VALUE_TYPE)
      return tk_fail(TK_ERR_INVALID_INPUT, "GGUF: %s (%llu)", kind_text(e.kind), (unsigned long long)e.detail);
    return tk_fail(TK_ERR_INVALID_INPUT, "GGUF: %s", kind_text(e.kind));
  } catch (const std::bad_alloc &) {
    return tk_fail(TK_ERR_BACKEND, "tk_gguf_open: host allocation failed");
  }
}

extern "C" void tk_gguf_close(tk_gguf *g) { delete g; }
extern "C" uint32_t tk_gguf_version(const tk_gguf *g) { return g ? g->version : 0; }
extern "C" uint64_t tk_gguf_alignment(const tk_gguf *g) { return g ? g->alignment : 0; }
extern "C" uint64_t tk_gguf_tensor_data_offset(const tk_gguf *g) { return g ? g->tensor_data_offset : 0; }
extern "C" size_t tk_gguf_tensor_count(const tk_gguf *g) { return g ? g->tensors.size() : 0; }
extern "C" size_t tk_gguf_metadata_count(const tk_gguf *g) { return g ? g->metadata.size() : 0; }

extern "C" int tk_gguf_tensor_at(const tk_gguf *g, size_t index, tk_gguf_tensor *out) {
  if (!g || !out || index >= g->tensors.size()) return 0;
  fill_info(g->tensors[index], out);
  return 1;
}

extern "C" int tk_gguf_tensor_find(const tk_gguf *g, const char *name, tk_gguf_tensor *out) {
  if (!g || !name || !out) return 0;
  const Tensor *t = find_tensor(g, name);
  if (!t) return 0;
  fill_info(*t, out);
  return 1;
}

extern "C" int tk_gguf_meta_type(const tk_gguf *g, const char *key, long long index, uint32_t *value_type,
                                 uint32_t *child_type, uint64_t *array_len) {
  const Value *v = lookup(g, key, index);
  if (!v) return 0;
  if (value_type) *value_type = v->type;
  if (child_type) *child_type = v->type == 9 ? (uint32_t)v->bits : 0;
  if (array_len) *array_len = v->type == 9 ? v->items.size() : 0;
  return 1;
}

// GgufValue::as_u64 (gguf.rs:217-229): unsigned widths, and signed ones when not negative
extern "C" int tk_gguf_meta_u64(const tk_gguf *g, const char *key, long long index, uint64_t *out) {
  const Value *v = lookup(g, key, index);
  if (!v || !out) return 0;
  switch (v->type) {
    case 0: case 2: case 4: case 10: *out = v->bits; return 1;
    case 1: if ((int8_t)v->bits < 0) return 0; *out = v->bits; return 1;
    case 3: if ((int16_t)v->bits < 0) return 0; *out = v->bits; return 1;
    case 5: if ((int32_t)v->bits < 0) return 0; *out = v->bits; return 1;
    case 11: if ((int64_t)v->bits < 0) return 0; *out = v->bits; return 1;
    default: return 0;
  }
}

// GgufValue::as_i64 (gguf.rs:243-256): every integer width; U64 only when it fits
extern "C" int tk_gguf_meta_i64(const tk_gguf *g, const char *key, long long index, int64_t *out) {
  const Value *v = lookup(g, key, index);
  if (!v || !out) return 0;
  switch (v->type) {
    case 0: case 2: case 4: *out = (int64_t)v->bits; return 1;
    case 1: *out = (int8_t)v->bits; return 1;
    case 3: *out = (int16_t)v->bits; return 1;
    case 5: *out = (int32_t)v->bits; return 1;
    case 11: *out = (int64_t)v->bits; return 1;
    case 10: if (v->bits > (uint64_t)INT64_MAX) return 0; *out = (int64_t)v->bits; return 1;
    default: return 0;
  }
}

// GgufValue::as_f64 (gguf.rs:260-266): F64, or F32 widened
extern "C" int tk_gguf_meta_f64(const tk_gguf *g, const char *key, long long index, double *out) {
  const Value *v = lookup(g, key, index);
  if (!v || !out) return 0;
  if (v->type == 12) { std::memcpy(out, &v->bits, 8); return 1; }
  if (v->type == 6) { *out = (double)f32_from_bits((uint32_t)v->bits); return 1; }
  return 0;
}

// GgufValue::as_f32 (gguf.rs:270-275): F32 only
extern "C" int tk_gguf_meta_f32(const tk_gguf *g, const char *key, long long index, float *out) {
  const Value *v = lookup(g, key, index);
  if (!v || !out || v->type != 6) return 0;
  *out = f32_from_bits((uint32_t)v->bits);
  return 1;
}

extern "C" int tk_gguf_meta_bool(const tk_gguf *g, const char *key, long long index, int *out) {
  const Value *v = lookup(g, key, index);
  if (!v || !out || v->type != 7) return 0;
  *out = (int)v->bits;
  return 1;
}

extern "C" int tk_gguf_meta_str(const tk_gguf *g, const char *key, long long index, const char **out, size_t *len) {
  const Value *v = lookup(g, key, index);
  if (!v || !out || v->type != 8) return 0;
  *out = v->str.c_str();
  if (len) *len = v->str.size();
  return 1;
}

// TensorInfo::element_count (gguf.rs:392-398)
extern "C" int tk_gguf_element_count(const tk_gguf_tensor *t, uint64_t *out) {
  if (!t || !out || t->n_dims > kMaxDims) return tk_fail(TK_ERR_INVALID_INPUT, "tk_gguf_element_count: bad argument");
  uint64_t n = 1;
  for (uint32_t i = 0; i < t->n_dims; ++i)
    if (__builtin_mul_overflow(n, t->dims[i], &n)) return tk_fail(TK_ERR_INVALID_INPUT, "GGUF: %s", kind_text(TK_GGUF_DIMS_OVERFLOW));
  *out = n;
  return TK_OK;
}

// payload() of the model loader (crates/tritium-nn/src/model/weights.rs:146-166): the reader leaves
// I2_S unsized, the loader sizes it as elements/4 + 32.
extern "C" int tk_gguf_tensor_payload(const tk_gguf *g, size_t file_len, const tk_gguf_tensor *t, uint64_t *abs_offset,
                                      uint64_t *len) {
  if (!g || !t || !abs_offset || !len) return tk_fail(TK_ERR_INVALID_INPUT, "tk_gguf_tensor_payload: null pointer");
  uint64_t elems;
  TKCHK_HOST(tk_gguf_element_count(t, &elems));
  const uint64_t n = t->ggml_type == kTypeI2s ? elems / 4 + 32 : t->n_bytes;
  uint64_t start, end;
  if (__builtin_add_overflow(g->tensor_data_offset, t->offset, &start) || __builtin_add_overflow(start, n, &end) ||
      end > file_len)
    return tk_fail(TK_ERR_INVALID_INPUT, "missing tensor: %s (payload out of bounds)", t->name ? t->name : "?");
  *abs_offset = start;
  *len = n;
  return TK_OK;
}

extern "C" int tk_gguf_ternary_shape(const tk_gguf *g, const char *name, size_t *n, size_t *k, int *format) {
  if (!g || !name || !n || !k || !format) return tk_fail(TK_ERR_INVALID_INPUT, "tk_gguf_ternary_shape: null pointer");
  const Tensor *t = find_tensor(g, name);
  if (!t) return tk_fail(TK_ERR_INVALID_INPUT, "missing tensor: %s", name);
  if (t->dims.size() != 2) return tk_fail_mismatch(2, t->dims.size());  // NnError::Shape{expected: 2, got}
  if (t->ggml_type != kTypeI2s && t->ggml_type != kTypeTq1 && t->ggml_type != kTypeTq2)
    return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "unsupported tensor type %u", t->ggml_type);
  *k = (size_t)t->dims[0];  // ggml order: fastest first
  *n = (size_t)t->dims[1];
  *format = t->ggml_type == kTypeTq1 ? TK_FORMAT_TQ1_0 : TK_FORMAT_TQ2_0;
  return TK_OK;
}

extern "C" int tk_gguf_load_ternary(const tk_gguf *g, const uint8_t *file, size_t file_len, const char *name,
                                    uint8_t *packed, size_t packed_len, float *row_scales, size_t row_scales_len) {
  size_t n, k;
  int format;
  TKCHK_HOST(tk_gguf_ternary_shape(g, name, &n, &k, &format));
  if ((!file && file_len) || (!packed && packed_len) || (!row_scales && row_scales_len))
    return tk_fail(TK_ERR_INVALID_INPUT, "tk_gguf_load_ternary: null pointer");
  size_t elems;
  if (__builtin_mul_overflow(n, k, &elems)) return tk_fail(TK_ERR_INVALID_INPUT, "GGUF: %s", kind_text(TK_GGUF_DIMS_OVERFLOW));
  const size_t want = tk_packed_len(n, k, format);
  if (packed_len != want) return tk_fail_mismatch(want, packed_len);
  if (row_scales_len != n) return tk_fail_mismatch(n, row_scales_len);
  tk_gguf_tensor info;
  fill_info(*find_tensor(g, name), &info);
  uint64_t off, len;
  TKCHK_HOST(tk_gguf_tensor_payload(g, file_len, &info, &off, &len));
  const uint8_t *p = file + off;

  if (info.ggml_type == kTypeI2s) {
    float scale;
    const int rc = tk_convert_i2s_to_tq2_0(p, (size_t)len, n, k, packed, packed_len, &scale);
    if (rc == TK_ERR_INVALID_INPUT) {  // the loader reports a bad payload as a backend error (weights.rs:214-216)
      char why[256];
      std::snprintf(why, sizeof why, "%s", tk_last_error());
      return tk_fail(TK_ERR_BACKEND, "%s: %s", name, why);
    }
    if (rc != TK_OK) return rc;
    for (size_t r = 0; r < n; ++r) row_scales[r] = scale;
    return TK_OK;
  }

  // TQ1_0 / TQ2_0: one f16 scale per 256-block. A pure ternary row has one scale in all its blocks
  // that hold a nonzero trit and 0 in the others (weights.rs:219-300).
  const size_t bb = format == TK_FORMAT_TQ1_0 ? 54 : 66, nb = (k + 255) / 256, row_bytes = nb * bb;
  if (len < (uint64_t)n * row_bytes)
    return tk_fail(TK_ERR_BACKEND, "%s: payload %llu B < %zu rows x %zu B", name, (unsigned long long)len, n, row_bytes);
  int8_t zeros[256] = {0}, scratch[256];
  uint8_t zero_block[66];
  TKCHK_HOST(tk_pack_rows(zeros, 256, 1, 256, format, zero_block, bb));
  bool have_tensor_scale = false, rows_uniform = true;
  float tensor_scale = 0.0f;
  for (size_t r = 0; r < n; ++r) {
    bool have_row = false;
    float row_scale = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
      const uint8_t *src = p + r * row_bytes + b * bb;
      uint8_t *dst = packed + r * row_bytes + b * bb;
      if (tk_unpack_rows(src, bb, 1, 256, format, scratch, 256) != TK_OK)  // reserved TQ2_0 code
        return tk_fail(TK_ERR_BACKEND, "%s: row %zu block %zu: decoded value 2 outside ternary range", name, r, b);
      const uint16_t hbits = (uint16_t)(src[bb - 2] | (src[bb - 1] << 8));
      _Float16 h;
      std::memcpy(&h, &hbits, 2);
      const float dv = (float)h;
      if (dv == 0.0f) {  // an all-zero block: its values are 0 at any scale, so its trits become zero trits
        std::memcpy(dst, zero_block, bb - 2);
        dst[bb - 2] = src[bb - 2];
        dst[bb - 1] = src[bb - 1];
        continue;
      }
      std::memcpy(dst, src, bb);
      if (!have_row) {
        have_row = true;
        row_scale = dv;
      } else if (!(row_scale == dv)) {
        return tk_fail(TK_ERR_BACKEND,
                       "%s: non-uniform block scales (%g vs %g within row %zu block %zu): not a pure ternary row", name,
                       (double)row_scale, (double)dv, r, b);
      }
    }
    if (have_row) {
      if (!have_tensor_scale) {
        have_tensor_scale = true;
        tensor_scale = row_scale;
      } else if (tensor_scale != row_scale) {
        rows_uniform = false;
      }
    }
    row_scales[r] = have_row ? row_scale : 0.0f;
  }
  if (!rows_uniform) {  // rows with their own scales; all-zero rows take the first nonzero scale (weights.rs:295-305)
    for (size_t r = 0; r < n; ++r)
      if (row_scales[r] == 0.0f) row_scales[r] = tensor_scale;
    return TK_OK;
  }
  // One scale for the tensor. A repacked file keeps the source's exact f32 scale in metadata; it must
  // agree with the block scale to f16 precision (weights.rs:307-329).
  float scale = have_tensor_scale ? tensor_scale : 0.0f;
  std::string key;
  try {
    key = std::string("tritium.i2s_scale.") + name;
  } catch (const std::bad_alloc &) {
    return tk_fail(TK_ERR_BACKEND, "tk_gguf_load_ternary: host allocation failed");
  }
  float exact;
  if (tk_gguf_meta_f32(g, key.c_str(), -1, &exact)) {
    if (have_tensor_scale) {
      const float expect = (float)(_Float16)exact;
      if (!(tensor_scale == expect))
        return tk_fail(TK_ERR_BACKEND, "%s: tritium.i2s_scale metadata (%g, f16 %g) disagrees with the file's block scale (%g)",
                       name, (double)exact, (double)expect, (double)tensor_scale);
    }
    scale = exact;
  }
  for (size_t r = 0; r < n; ++r) row_scales[r] = scale;
  return TK_OK;
}
