// Weight ingest: the GGUF v3 container (header, metadata, tensor directory, bounds-checked access to the
// mapped tensor bytes) and the upload of one layer's feed-forward tensors in the formats the file holds.
// Behaviour follows crates/xabe-gguf/src/{file,reader,types,error}.rs and the upload functions of
// crates/xabe-engine/src/block/{moe,dense_ffn}.rs; host code only, nothing here launches a kernel.
//
// Layout of a file (the format comment of ggml's gguf.cpp, as file.rs:1-26 lists it): magic "GGUF", u32
// version (3), i64 tensor count, i64 key-value count, the key-value pairs (string key, i32 type tag, value;
// arrays carry an element tag and a u64 count, never nested), the tensor records (string name, u32 rank
// <= 4, i64 dimensions, i32 ggml type, u64 offset into the data section), then the data section at the
// next multiple of `general.alignment` (u32, default 32).
#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/xabe_gguf.h"
#include "host_common.h"

using xabe::set_error;

namespace {

struct TypeRow {
  int id;
  uint64_t block, bytes;
  const char* name;
};
// crates/xabe-gguf/src/types.rs:62-99
const TypeRow kTypes[] = {{XABE_GGML_F32, 1, 4, "f32"},      {XABE_GGML_F16, 1, 2, "f16"},     {XABE_GGML_Q4_0, 32, 18, "q4_0"},
                          {XABE_GGML_Q8_0, 32, 34, "q8_0"},  {XABE_GGML_Q4_K, 256, 144, "q4_K"}, {XABE_GGML_Q5_K, 256, 176, "q5_K"},
                          {XABE_GGML_Q6_K, 256, 210, "q6_K"}, {XABE_GGML_BF16, 1, 2, "bf16"}};

const TypeRow* type_row(int id) {
  for (const TypeRow& r : kTypes)
    if (r.id == id) return &r;
  return nullptr;
}

struct Value {
  int type = -1;       // gguf_type tag
  int elem_type = -1;  // arrays
  uint64_t count = 0;  // arrays
  uint64_t bits = 0;   // scalars, zero- or sign-extended little-endian bytes
  std::string str;
  std::vector<uint8_t> packed;        // numeric / bool arrays
  std::vector<std::string> strings;   // string arrays
};

struct Tensor {
  std::string name;
  uint32_t n_dims;
  uint64_t dims[4];
  int ggml_type;
  uint64_t offset, n_elements, n_bytes;
};

// Bounds-checked little-endian reader (reader.rs:13-111): a short file is a status, not a fault.
struct Cursor {
  const uint8_t* data;
  size_t len, pos = 0;
  int status = XABE_OK;

  const uint8_t* take(size_t n, const char* context) {
    if (status != XABE_OK) return nullptr;
    if (n > len - pos) {
      status = set_error(XABE_ERR_GGUF_UNEXPECTED_EOF, "unexpected end of file while reading %s at byte offset %zu",
                         context, pos);
      return nullptr;
    }
    const uint8_t* p = data + pos;
    pos += n;
    return p;
  }
  template <typename T>
  T scalar(const char* context) {
    T v{};
    if (const uint8_t* p = take(sizeof(T), context)) memcpy(&v, p, sizeof(T));  // the host is little-endian
    return v;
  }
  bool string(std::string* out);
};

bool valid_utf8(const uint8_t* s, size_t n) {
  size_t i = 0;
  while (i < n) {
    const uint8_t c = s[i];
    size_t extra;
    uint32_t cp;
    if (c < 0x80) { ++i; continue; }
    if ((c & 0xE0) == 0xC0) { extra = 1; cp = c & 0x1F; }
    else if ((c & 0xF0) == 0xE0) { extra = 2; cp = c & 0x0F; }
    else if ((c & 0xF8) == 0xF0) { extra = 3; cp = c & 0x07; }
    else return false;
    if (i + extra >= n) return false;  // truncated sequence
    for (size_t k = 1; k <= extra; ++k) {
      if ((s[i + k] & 0xC0) != 0x80) return false;
      cp = (cp << 6) | (s[i + k] & 0x3F);
    }
    // overlong forms, surrogates and values past U+10FFFF are not UTF-8
    if ((extra == 1 && cp < 0x80) || (extra == 2 && cp < 0x800) || (extra == 3 && cp < 0x10000)) return false;
    if ((cp >= 0xD800 && cp <= 0xDFFF) || cp > 0x10FFFF) return false;
    i += extra + 1;
  }
  return true;
}

bool Cursor::string(std::string* out) {
  const uint64_t n = scalar<uint64_t>("u64");
  if (status != XABE_OK) return false;
  if (n > (uint64_t)SIZE_MAX) {
    status = set_error(XABE_ERR_GGUF_UNEXPECTED_EOF, "unexpected end of file while reading string length at byte offset %zu", pos);
    return false;
  }
  const uint8_t* p = take((size_t)n, "string bytes");
  if (!p) return false;
  if (!valid_utf8(p, (size_t)n)) {
    status = set_error(XABE_ERR_GGUF_INVALID_UTF8, "metadata string is not valid UTF-8 (at byte offset %zu)", pos - (size_t)n);
    return false;
  }
  out->assign(reinterpret_cast<const char*>(p), (size_t)n);
  return true;
}

size_t scalar_bytes(int tag) {
  switch (tag) {
    case XABE_GGUF_U8: case XABE_GGUF_I8: case XABE_GGUF_BOOL: return 1;
    case XABE_GGUF_U16: case XABE_GGUF_I16: return 2;
    case XABE_GGUF_U32: case XABE_GGUF_I32: case XABE_GGUF_F32: return 4;
    case XABE_GGUF_U64: case XABE_GGUF_I64: case XABE_GGUF_F64: return 8;
  }
  return 0;
}

// file.rs:386-452
bool read_value(Cursor& cur, Value* v) {
  const int32_t tag = cur.scalar<int32_t>("i32");
  if (cur.status != XABE_OK) return false;
  v->type = tag;
  if (tag == XABE_GGUF_STRING) return cur.string(&v->str);
  if (tag == XABE_GGUF_ARRAY) {
    const int32_t et = cur.scalar<int32_t>("i32");
    const uint64_t n = cur.scalar<uint64_t>("u64");
    if (cur.status != XABE_OK) return false;
    v->elem_type = et;
    v->count = n;
    if (et == XABE_GGUF_ARRAY) {
      cur.status = set_error(XABE_ERR_GGUF_NESTED_ARRAY, "nested arrays are not supported (key had an array-of-array value)");
      return false;
    }
    if (et == XABE_GGUF_STRING) {
      v->strings.reserve((size_t)std::min<uint64_t>(n, (cur.len - cur.pos) / 8));
      for (uint64_t i = 0; i < n; ++i) {
        std::string s;
        if (!cur.string(&s)) return false;
        v->strings.push_back(std::move(s));
      }
      return true;
    }
    const size_t w = scalar_bytes(et);
    if (w == 0) {
      cur.status = set_error(XABE_ERR_GGUF_UNKNOWN_VALUE_TYPE, "unknown GGUF value type tag %d", et);
      return false;
    }
    if (n > (cur.len - cur.pos) / w) {  // also rules out n * w overflowing
      cur.status = set_error(XABE_ERR_GGUF_UNEXPECTED_EOF, "unexpected end of file while reading %s at byte offset %zu",
                             "array elements", cur.pos);
      return false;
    }
    const uint8_t* p = cur.take((size_t)n * w, "array elements");
    if (!p) return false;
    v->packed.assign(p, p + (size_t)n * w);
    if (et == XABE_GGUF_BOOL)
      for (uint8_t& b : v->packed) b = b != 0;
    return true;
  }
  const size_t w = scalar_bytes(tag);
  if (w == 0) {
    cur.status = set_error(XABE_ERR_GGUF_UNKNOWN_VALUE_TYPE, "unknown GGUF value type tag %d", tag);
    return false;
  }
  const uint8_t* p = cur.take(w, "scalar value");
  if (!p) return false;
  memcpy(&v->bits, p, w);
  if (tag == XABE_GGUF_BOOL) v->bits = (v->bits & 0xFF) != 0;
  return true;
}

}  // namespace

struct xabe_gguf_file {
  const uint8_t* data = nullptr;
  size_t len = 0;
  bool mapped = false;
  std::vector<uint8_t> owned;
  uint32_t version = 0, alignment = 0;
  uint64_t data_offset = 0;
  std::vector<std::string> keys;  // file order
  std::unordered_map<std::string, Value> metadata;
  std::vector<Tensor> tensors;
  std::unordered_map<std::string, size_t> tensor_index;

  ~xabe_gguf_file() {
    if (mapped && data) munmap(const_cast<uint8_t*>(data), len);
  }
};

namespace {

// file.rs:107-149 and :281-379
int parse(xabe_gguf_file* f) {
  Cursor cur{f->data, f->len};
  const uint8_t* magic = cur.take(4, "magic");
  if (!magic) return cur.status;
  if (memcmp(magic, "GGUF", 4) != 0)
    return set_error(XABE_ERR_GGUF_BAD_MAGIC, "bad magic bytes: expected `GGUF`, found [%02x, %02x, %02x, %02x]", magic[0],
                     magic[1], magic[2], magic[3]);
  f->version = cur.scalar<uint32_t>("u32");
  if (cur.status != XABE_OK) return cur.status;
  if (f->version != 3)
    return set_error(XABE_ERR_GGUF_UNSUPPORTED_VERSION, "unsupported GGUF version %u; only version 3 is supported", f->version);
  const int64_t n_tensors = cur.scalar<int64_t>("i64");
  if (cur.status != XABE_OK) return cur.status;
  if (n_tensors < 0) return set_error(XABE_ERR_GGUF_NEGATIVE_COUNT, "tensor count %lld is negative", (long long)n_tensors);
  const int64_t n_kv = cur.scalar<int64_t>("i64");
  if (cur.status != XABE_OK) return cur.status;
  if (n_kv < 0) return set_error(XABE_ERR_GGUF_NEGATIVE_COUNT, "kv count %lld is negative", (long long)n_kv);

  for (int64_t i = 0; i < n_kv; ++i) {
    std::string key;
    if (!cur.string(&key)) return cur.status;
    Value v;
    if (!read_value(cur, &v)) return cur.status;
    if (!f->metadata.emplace(key, std::move(v)).second)
      return set_error(XABE_ERR_GGUF_DUPLICATE_KEY, "duplicate metadata key `%s`", key.c_str());
    f->keys.push_back(std::move(key));
  }

  f->alignment = 32;  // GGUF_DEFAULT_ALIGNMENT
  auto al = f->metadata.find("general.alignment");
  if (al != f->metadata.end()) {
    if (al->second.type != XABE_GGUF_U32) return set_error(XABE_ERR_GGUF_BAD_ALIGNMENT_TYPE, "`general.alignment` must be of type u32");
    f->alignment = (uint32_t)al->second.bits;
  }
  if (f->alignment == 0 || (f->alignment & (f->alignment - 1)) != 0)
    return set_error(XABE_ERR_GGUF_BAD_ALIGNMENT, "alignment %u is not a power of two", f->alignment);

  for (int64_t i = 0; i < n_tensors; ++i) {
    Tensor t{};
    if (!cur.string(&t.name)) return cur.status;
    if (f->tensor_index.count(t.name)) return set_error(XABE_ERR_GGUF_DUPLICATE_TENSOR, "duplicate tensor name `%s`", t.name.c_str());
    t.n_dims = cur.scalar<uint32_t>("u32");
    if (cur.status != XABE_OK) return cur.status;
    if (t.n_dims > 4)
      return set_error(XABE_ERR_GGUF_TOO_MANY_DIMENSIONS, "tensor `%s` has %u dimensions, more than the maximum of 4", t.name.c_str(),
                       t.n_dims);
    t.n_elements = 1;
    bool overflow = false;
    for (uint32_t d = 0; d < t.n_dims; ++d) {
      const int64_t v = cur.scalar<int64_t>("i64");
      if (cur.status != XABE_OK) return cur.status;
      if (v <= 0) return set_error(XABE_ERR_GGUF_ZERO_DIMENSION, "tensor `%s` has a zero-sized dimension", t.name.c_str());
      t.dims[d] = (uint64_t)v;
      overflow |= __builtin_mul_overflow(t.n_elements, (uint64_t)v, &t.n_elements);
    }
    const int32_t raw_type = cur.scalar<int32_t>("i32");
    if (cur.status != XABE_OK) return cur.status;
    const TypeRow* row = type_row(raw_type);
    if (!row) return set_error(XABE_ERR_GGUF_UNSUPPORTED_GGML_TYPE, "unsupported ggml tensor type id %d", raw_type);
    t.ggml_type = raw_type;
    t.offset = cur.scalar<uint64_t>("u64");
    if (cur.status != XABE_OK) return cur.status;
    if (overflow) return set_error(XABE_ERR_GGUF_OFFSET_OVERFLOW, "tensor `%s` offset/size arithmetic overflowed", t.name.c_str());
    if (t.n_elements % row->block != 0)
      return set_error(XABE_ERR_GGUF_UNALIGNED_ELEMENT_COUNT,
                       "tensor `%s` has %llu elements of type %s, not a whole number of %llu-element blocks", t.name.c_str(),
                       (unsigned long long)t.n_elements, row->name, (unsigned long long)row->block);
    if (__builtin_mul_overflow(t.n_elements / row->block, row->bytes, &t.n_bytes))
      return set_error(XABE_ERR_GGUF_OFFSET_OVERFLOW, "tensor `%s` offset/size arithmetic overflowed", t.name.c_str());
    f->tensor_index.emplace(t.name, f->tensors.size());
    f->tensors.push_back(std::move(t));
  }

  const uint64_t a = f->alignment;
  f->data_offset = ((uint64_t)cur.pos + a - 1) & ~(a - 1);
  for (const Tensor& t : f->tensors) {
    uint64_t start, end;
    if (__builtin_add_overflow(f->data_offset, t.offset, &start) || __builtin_add_overflow(start, t.n_bytes, &end))
      return set_error(XABE_ERR_GGUF_OFFSET_OVERFLOW, "tensor `%s` offset/size arithmetic overflowed", t.name.c_str());
    if (end > (uint64_t)f->len)
      return set_error(XABE_ERR_GGUF_TENSOR_OUT_OF_BOUNDS, "tensor `%s` byte range [%llu, %llu) exceeds the file size of %zu bytes",
                       t.name.c_str(), (unsigned long long)start, (unsigned long long)end, f->len);
  }
  return XABE_OK;
}

int finish_open(xabe_gguf_file* f, xabe_gguf_file** out) {
  const int s = parse(f);
  if (s != XABE_OK) {
    delete f;
    return s;
  }
  *out = f;
  return XABE_OK;
}

const Value* find_value(const xabe_gguf_file* f, const char* key, int type) {
  if (!f || !key) return nullptr;
  auto it = f->metadata.find(key);
  if (it == f->metadata.end() || (type >= 0 && it->second.type != type)) return nullptr;
  return &it->second;
}

void fill_info(const Tensor& t, xabe_gguf_tensor_info* out) {
  out->name = t.name.c_str();
  out->n_dims = t.n_dims;
  for (int d = 0; d < 4; ++d) out->dims[d] = d < (int)t.n_dims ? t.dims[d] : 0;
  out->ggml_type = t.ggml_type;
  out->offset = t.offset;
  out->n_elements = t.n_elements;
  out->n_bytes = t.n_bytes;
}

}  // namespace

extern "C" {

uint64_t xabe_ggml_type_block_size(int t) { const TypeRow* r = type_row(t); return r ? r->block : 0; }
uint64_t xabe_ggml_type_size(int t) { const TypeRow* r = type_row(t); return r ? r->bytes : 0; }
const char* xabe_ggml_type_name(int t) { const TypeRow* r = type_row(t); return r ? r->name : nullptr; }

int xabe_ggml_type_bytes_for_elements(int t, uint64_t n, uint64_t* out) {
  const TypeRow* r = type_row(t);
  if (!r) return set_error(XABE_ERR_GGUF_UNSUPPORTED_GGML_TYPE, "unsupported ggml tensor type id %d", t);
  if (!out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null output pointer");
  if (n % r->block != 0)
    return set_error(XABE_ERR_GGUF_UNALIGNED_ELEMENT_COUNT, "%llu elements of type %s, not a whole number of %llu-element blocks",
                     (unsigned long long)n, r->name, (unsigned long long)r->block);
  if (__builtin_mul_overflow(n / r->block, r->bytes, out)) return set_error(XABE_ERR_GGUF_OFFSET_OVERFLOW, "size arithmetic overflowed");
  return XABE_OK;
}

int xabe_gguf_open(const char* path, xabe_gguf_file** out) {
  if (!path || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null path or output pointer");
  const int fd = open(path, O_RDONLY | O_CLOEXEC);
  if (fd < 0) return set_error(XABE_ERR_GGUF_IO, "I/O error: %s: %s", path, strerror(errno));
  struct stat st;
  if (fstat(fd, &st) != 0) {
    const int e = errno;
    close(fd);
    return set_error(XABE_ERR_GGUF_IO, "I/O error: %s: %s", path, strerror(e));
  }
  xabe_gguf_file* f = new xabe_gguf_file();
  f->len = (size_t)st.st_size;
  if (f->len > 0) {
    void* p = mmap(nullptr, f->len, PROT_READ, MAP_PRIVATE, fd, 0);
    if (p == MAP_FAILED) {
      const int e = errno;
      close(fd);
      delete f;
      return set_error(XABE_ERR_GGUF_IO, "I/O error: mmap of %s: %s", path, strerror(e));
    }
    f->data = static_cast<const uint8_t*>(p);
    f->mapped = true;
  }
  close(fd);  // the mapping outlives the descriptor
  return finish_open(f, out);
}

int xabe_gguf_from_bytes(const void* bytes, size_t len, xabe_gguf_file** out) {
  if ((!bytes && len) || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null bytes or output pointer");
  xabe_gguf_file* f = new xabe_gguf_file();
  f->owned.assign(static_cast<const uint8_t*>(bytes), static_cast<const uint8_t*>(bytes) + len);
  f->data = f->owned.data();
  f->len = len;
  return finish_open(f, out);
}

void xabe_gguf_close(xabe_gguf_file* f) { delete f; }

uint32_t xabe_gguf_version(const xabe_gguf_file* f) { return f ? f->version : 0; }
uint32_t xabe_gguf_alignment(const xabe_gguf_file* f) { return f ? f->alignment : 0; }
size_t xabe_gguf_n_kv(const xabe_gguf_file* f) { return f ? f->metadata.size() : 0; }
size_t xabe_gguf_n_tensors(const xabe_gguf_file* f) { return f ? f->tensors.size() : 0; }
uint64_t xabe_gguf_data_offset(const xabe_gguf_file* f) { return f ? f->data_offset : 0; }

int xabe_gguf_tensor_at(const xabe_gguf_file* f, size_t index, xabe_gguf_tensor_info* out) {
  if (!f || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null file or output pointer");
  if (index >= f->tensors.size()) return set_error(XABE_ERR_MISSING_TENSOR, "tensor index %zu of %zu", index, f->tensors.size());
  fill_info(f->tensors[index], out);
  return XABE_OK;
}

int xabe_gguf_tensor(const xabe_gguf_file* f, const char* name, xabe_gguf_tensor_info* out) {
  if (!f || !name || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null file, name or output pointer");
  auto it = f->tensor_index.find(name);
  if (it == f->tensor_index.end()) return set_error(XABE_ERR_MISSING_TENSOR, "the file has no tensor `%s`", name);
  fill_info(f->tensors[it->second], out);
  return XABE_OK;
}

const void* xabe_gguf_tensor_bytes(const xabe_gguf_file* f, const char* name, size_t* len) {
  if (!f || !name) return nullptr;
  auto it = f->tensor_index.find(name);
  if (it == f->tensor_index.end()) return nullptr;
  const Tensor& t = f->tensors[it->second];  // bounds were checked at load
  if (len) *len = (size_t)t.n_bytes;
  return f->data + f->data_offset + t.offset;
}

const char* xabe_gguf_key_at(const xabe_gguf_file* f, size_t index) {
  return f && index < f->keys.size() ? f->keys[index].c_str() : nullptr;
}

int xabe_gguf_value_type_of(const xabe_gguf_file* f, const char* key, int* type, int* elem_type, uint64_t* count) {
  const Value* v = find_value(f, key, -1);
  if (!v) return 0;
  if (type) *type = v->type;
  if (elem_type) *elem_type = v->elem_type;
  if (count) *count = v->count;
  return 1;
}

int xabe_gguf_get_u32(const xabe_gguf_file* f, const char* key, uint32_t* out) {
  const Value* v = find_value(f, key, XABE_GGUF_U32);
  if (!v || !out) return 0;
  *out = (uint32_t)v->bits;
  return 1;
}

int xabe_gguf_get_u64(const xabe_gguf_file* f, const char* key, uint64_t* out) {
  const Value* v = find_value(f, key, XABE_GGUF_U64);
  if (!v || !out) return 0;
  *out = v->bits;
  return 1;
}

int xabe_gguf_get_f32(const xabe_gguf_file* f, const char* key, float* out) {
  const Value* v = find_value(f, key, XABE_GGUF_F32);
  if (!v || !out) return 0;
  const uint32_t b = (uint32_t)v->bits;
  memcpy(out, &b, 4);
  return 1;
}

const char* xabe_gguf_get_str(const xabe_gguf_file* f, const char* key, size_t* len) {
  const Value* v = find_value(f, key, XABE_GGUF_STRING);
  if (!v) return nullptr;
  if (len) *len = v->str.size();
  return v->str.c_str();
}

const void* xabe_gguf_get_array(const xabe_gguf_file* f, const char* key, int elem_type, uint64_t* count) {
  const Value* v = find_value(f, key, XABE_GGUF_ARRAY);
  if (!v || v->elem_type != elem_type || elem_type == XABE_GGUF_STRING) return nullptr;
  if (count) *count = v->count;
  static const uint8_t kEmpty = 0;
  return v->packed.empty() ? &kEmpty : v->packed.data();
}

const char* xabe_gguf_get_string_array_item(const xabe_gguf_file* f, const char* key, uint64_t index, size_t* len) {
  const Value* v = find_value(f, key, XABE_GGUF_ARRAY);
  if (!v || v->elem_type != XABE_GGUF_STRING || index >= v->strings.size()) return nullptr;
  if (len) *len = v->strings[index].size();
  return v->strings[index].c_str();
}

}  // extern "C"

// ------------------------------------------------------------------ layer upload
namespace {

struct DeviceTensors {
  std::vector<void*> allocations;
  size_t bytes = 0;
  ~DeviceTensors() {
    for (void* p : allocations) (void)hipFree(p);
  }
  int upload(hipStream_t s, const void* host, size_t n, void** out) {
    void* d = nullptr;
    XABE_HIP_TRY(hipMalloc(&d, n ? n : 1));
    allocations.push_back(d);
    bytes += n;
    if (n) XABE_HIP_TRY(hipMemcpyAsync(d, host, n, hipMemcpyHostToDevice, s));
    *out = d;
    return XABE_OK;
  }
};

struct Raw {
  const uint8_t* bytes;
  const Tensor* info;
  std::string name;
};

// block/moe.rs:811-826
int raw_tensor(const xabe_gguf_file* f, uint32_t layer, const char* suffix, Raw* out) {
  out->name = "blk." + std::to_string(layer) + "." + suffix;
  auto it = f->tensor_index.find(out->name);
  if (it == f->tensor_index.end()) return set_error(XABE_ERR_MISSING_TENSOR, "layer %u has no `%s`", layer, suffix);
  out->info = &f->tensors[it->second];
  out->bytes = f->data + f->data_offset + out->info->offset;
  return XABE_OK;
}

int check_dims(const Raw& r, std::initializer_list<uint64_t> expected) {
  // the directory's shape check (crates/xabe-model/src/weights.rs:484-490)
  bool same = r.info->n_dims == expected.size();
  size_t d = 0;
  for (uint64_t e : expected) same = same && r.info->dims[d++] == e;
  if (same) return XABE_OK;
  std::string want, have;
  for (uint64_t e : expected) want += (want.empty() ? "" : ", ") + std::to_string(e);
  for (uint32_t i = 0; i < r.info->n_dims; ++i) have += (have.empty() ? "" : ", ") + std::to_string(r.info->dims[i]);
  return set_error(XABE_ERR_SHAPE_MISMATCH, "tensor `%s` has dimensions [%s], the geometry implies [%s]", r.name.c_str(), have.c_str(),
                   want.c_str());
}

// An unquantized tensor widened to f32 on the host (block/moe.rs:832-862): bf16 is a truncated f32, so the
// widening is a shift.
int dense_tensor(hipStream_t s, const xabe_gguf_file* f, uint32_t layer, const char* suffix,
                 std::initializer_list<uint64_t> dims, size_t expected, DeviceTensors* dev, std::vector<std::vector<float>>* keep,
                 const float** out, int* ggml_type) {
  Raw r;
  XABE_TRY(raw_tensor(f, layer, suffix, &r));
  const int ty = r.info->ggml_type;
  if (ty != XABE_GGML_F32 && ty != XABE_GGML_BF16)
    return set_error(XABE_ERR_UNSUPPORTED_DENSE_TYPE, "tensor `%s` is %s, and this block only widens f32 and bf16", r.name.c_str(),
                     xabe_ggml_type_name(ty));
  if (r.info->n_elements != expected)
    return set_error(XABE_ERR_SHAPE_MISMATCH, "tensor `%s` holds %llu elements, the geometry implies %zu", r.name.c_str(),
                     (unsigned long long)r.info->n_elements, expected);
  XABE_TRY(check_dims(r, dims));
  void* d = nullptr;
  if (ty == XABE_GGML_F32) {
    XABE_TRY(dev->upload(s, r.bytes, expected * 4, &d));
  } else {
    keep->emplace_back(expected);  // lives until the stream has been synchronised
    std::vector<float>& w = keep->back();
    for (size_t i = 0; i < expected; ++i) {
      uint16_t h;
      memcpy(&h, r.bytes + 2 * i, 2);
      const uint32_t b = (uint32_t)h << 16;
      memcpy(&w[i], &b, 4);
    }
    XABE_TRY(dev->upload(s, w.data(), expected * 4, &d));
  }
  *out = static_cast<const float*>(d);
  if (ggml_type) *ggml_type = ty;
  return XABE_OK;
}

// A quantized stack left in its serialized form (block/moe.rs:864-892): the kernels read the file's
// 210-byte / 34-byte blocks as they are.
int quantized_tensor(hipStream_t s, const xabe_gguf_file* f, uint32_t layer, const char* suffix,
                     std::initializer_list<uint64_t> dims, size_t expected, DeviceTensors* dev, xabe_quant_tensor* out) {
  Raw r;
  XABE_TRY(raw_tensor(f, layer, suffix, &r));
  int quant;
  switch (r.info->ggml_type) {
    case XABE_GGML_Q6_K: quant = XABE_QUANT_Q6K; break;
    case XABE_GGML_Q8_0: quant = XABE_QUANT_Q8_0; break;
    case XABE_GGML_Q4_0: quant = XABE_QUANT_Q4_0; break;
    case XABE_GGML_Q4_K: quant = XABE_QUANT_Q4K; break;
    case XABE_GGML_Q5_K: quant = XABE_QUANT_Q5K; break;
    default:
      return set_error(XABE_ERR_UNSUPPORTED_QUANT, "expert stack `%s` is %s, which the grouped GEMM cannot unpack", r.name.c_str(),
                       xabe_ggml_type_name(r.info->ggml_type));
  }
  if (xabe_expert_quant_is_community(quant))
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "expert stack `%s` is %s: recognised, but this library has kernels for q6_K and q8_0 only",
                     r.name.c_str(), xabe_ggml_type_name(r.info->ggml_type));
  const size_t fb = xabe_expert_quant_file_block_bytes(quant), be = xabe_expert_quant_block_elements(quant);
  const size_t n = (size_t)r.info->n_bytes;
  if (n % fb != 0 || n / fb * be != expected)
    return set_error(XABE_ERR_SHAPE_MISMATCH, "tensor `%s` holds %zu elements, the geometry implies %zu", r.name.c_str(), n / fb * be,
                     expected);
  XABE_TRY(check_dims(r, dims));
  void* d = nullptr;
  XABE_TRY(dev->upload(s, r.bytes, n, &d));
  out->bytes = static_cast<const uint8_t*>(d);
  out->len = n;
  out->quant = quant;
  return XABE_OK;
}

}  // namespace

struct xabe_moe_layer {
  uint32_t layer;
  DeviceTensors dev;
  xabe_moe_layer_weights w;
  int router_types[2];
};

struct xabe_dense_ffn_layer {
  uint32_t layer;
  DeviceTensors dev;
  xabe_dense_ffn_layer_weights w;
};

extern "C" {

int xabe_moe_layer_upload(void* stream, const xabe_gguf_file* f, uint32_t layer, const xabe_moe_geometry* g, xabe_moe_layer** out) {
  if (!f || !g || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null file, geometry or output pointer");
  hipStream_t s = xabe::as_stream(stream);
  const uint64_t H = g->hidden, I = g->intermediate, E = g->num_experts;
  const size_t one = g->intermediate * g->hidden, stack = xabe_moe_geometry_stack_elements(g);
  xabe_moe_layer* l = new xabe_moe_layer();
  l->layer = layer;
  memset(&l->w, 0, sizeof(l->w));
  std::vector<std::vector<float>> keep;
  const float* router = nullptr;
  int st = dense_tensor(s, f, layer, "post_attention_norm.weight", {H}, g->hidden, &l->dev, &keep, &l->w.post_norm, nullptr);
  if (st == XABE_OK) st = dense_tensor(s, f, layer, "ffn_gate_inp.weight", {H, E}, g->num_experts * g->hidden, &l->dev, &keep, &router, &l->router_types[0]);
  if (st == XABE_OK) st = dense_tensor(s, f, layer, "ffn_gate_inp_shexp.weight", {H}, g->hidden, &l->dev, &keep, &l->w.shared_gate_inp, &l->router_types[1]);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_gate_exps.weight", {H, I, E}, stack, &l->dev, &l->w.gate_exps);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_up_exps.weight", {H, I, E}, stack, &l->dev, &l->w.up_exps);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_down_exps.weight", {I, H, E}, stack, &l->dev, &l->w.down_exps);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_gate_shexp.weight", {H, I}, one, &l->dev, &l->w.shared_gate);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_up_shexp.weight", {H, I}, one, &l->dev, &l->w.shared_up);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_down_shexp.weight", {I, H}, one, &l->dev, &l->w.shared_down);
  // the copies read the mapping and the widened vectors: wait for them before either can go away
  const hipError_t e = hipStreamSynchronize(s);
  if (st == XABE_OK && e != hipSuccess) st = xabe::hip_error(e, "hipStreamSynchronize");
  if (st != XABE_OK) {
    delete l;
    return st;
  }
  l->w.router = router;
  l->w.router_quant = -1;  // widened to f32 whatever the file held
  *out = l;
  return XABE_OK;
}

void xabe_moe_layer_free(xabe_moe_layer* l) { delete l; }
const xabe_moe_layer_weights* xabe_moe_layer_weights_of(const xabe_moe_layer* l) { return l ? &l->w : nullptr; }
uint32_t xabe_moe_layer_index(const xabe_moe_layer* l) { return l ? l->layer : 0; }

int xabe_moe_layer_expert_quants(const xabe_moe_layer* l, int out[3]) {
  if (!l || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null layer or output pointer");
  out[0] = l->w.gate_exps.quant, out[1] = l->w.up_exps.quant, out[2] = l->w.down_exps.quant;
  return XABE_OK;
}

int xabe_moe_layer_shared_quants(const xabe_moe_layer* l, int out[3]) {
  if (!l || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null layer or output pointer");
  out[0] = l->w.shared_gate.quant, out[1] = l->w.shared_up.quant, out[2] = l->w.shared_down.quant;
  return XABE_OK;
}

int xabe_moe_layer_router_types(const xabe_moe_layer* l, int out[2]) {
  if (!l || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null layer or output pointer");
  out[0] = l->router_types[0], out[1] = l->router_types[1];
  return XABE_OK;
}

size_t xabe_moe_layer_bytes(const xabe_moe_layer* l) { return l ? l->dev.bytes : 0; }

int xabe_dense_ffn_layer_upload(void* stream, const xabe_gguf_file* f, uint32_t layer, size_t hidden, size_t intermediate,
                                xabe_dense_ffn_layer** out) {
  if (!f || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null file or output pointer");
  hipStream_t s = xabe::as_stream(stream);
  const uint64_t H = hidden, I = intermediate;
  const size_t one = hidden * intermediate;
  xabe_dense_ffn_layer* l = new xabe_dense_ffn_layer();
  l->layer = layer;
  memset(&l->w, 0, sizeof(l->w));
  std::vector<std::vector<float>> keep;
  int st = dense_tensor(s, f, layer, "post_attention_norm.weight", {H}, hidden, &l->dev, &keep, &l->w.post_norm, nullptr);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_gate.weight", {H, I}, one, &l->dev, &l->w.gate);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_up.weight", {H, I}, one, &l->dev, &l->w.up);
  if (st == XABE_OK) st = quantized_tensor(s, f, layer, "ffn_down.weight", {I, H}, one, &l->dev, &l->w.down);
  const hipError_t e = hipStreamSynchronize(s);
  if (st == XABE_OK && e != hipSuccess) st = xabe::hip_error(e, "hipStreamSynchronize");
  if (st != XABE_OK) {
    delete l;
    return st;
  }
  *out = l;
  return XABE_OK;
}

void xabe_dense_ffn_layer_free(xabe_dense_ffn_layer* l) { delete l; }
const xabe_dense_ffn_layer_weights* xabe_dense_ffn_layer_weights_of(const xabe_dense_ffn_layer* l) { return l ? &l->w : nullptr; }

int xabe_dense_ffn_layer_quants(const xabe_dense_ffn_layer* l, int out[3]) {
  if (!l || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null layer or output pointer");
  out[0] = l->w.gate.quant, out[1] = l->w.up.quant, out[2] = l->w.down.quant;
  return XABE_OK;
}

size_t xabe_dense_ffn_layer_bytes(const xabe_dense_ffn_layer* l) { return l ? l->dev.bytes : 0; }

}  // extern "C"
