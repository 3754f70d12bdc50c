// Safetensors checkpoints -> decoder parameters, by the reference's parameter names.
//
// Reference behaviour restated here:
//   - Module::update_by_safetensors (rai-core/src/nn.rs:39-55): every file is read,
//     all its tensors are collected by name (a later file wins on a duplicate name),
//     then every parameter of the model is looked up by name; a parameter that no
//     file holds is Error::ParamNotFound(name) (nn.rs:198-204); tensors that the
//     model does not have are ignored.
//   - update_by_name converts the stored tensor to the parameter's dtype
//     (`t.to_dtype(self)`, nn.rs:199-200).
//   - Tensor::from_safetensor (rai-core/src/hlops/from_safetensor.rs:51-91) accepts
//     U8, F16, BF16, U32, F32, F64 and I64 and is `todo!()` for every other dtype;
//     decoder parameters are floating point, so F16 / BF16 / F32 / F64 are converted
//     and any other source dtype is an error.
//   - ext::hf::load_safetensors (rai/src/lib.rs:17-42): the distinct file names in
//     the "weight_map" object of a model.safetensors.index.json; a missing or
//     non-object weight_map is an error.  (The hub download is not reproduced: the
//     names are resolved against the directory of the index file.)
//
// The file format: 8 bytes little-endian header length N, N bytes of JSON mapping
// tensor name -> {"dtype", "shape", "data_offsets": [begin, end)} (plus an optional
// "__metadata__" object), then the raw little-endian tensor bytes.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "common.h"

namespace rai {
namespace {

// ---------------------------------------------------------------- minimal JSON
struct JsonValue {
  enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
  bool b = false;
  double num = 0.0;
  std::string str;
  std::vector<JsonValue> arr;
  std::vector<std::pair<std::string, JsonValue>> obj;  // insertion order kept
  const JsonValue *get(const char *key) const {
    for (auto &kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

struct JsonParser {
  const char *p, *end;
  std::string err;
  bool fail(const char *what) {
    if (err.empty()) err = what;
    return false;
  }
  void ws() {
    while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p;
  }
  static void utf8(std::string &out, unsigned cp) {
    if (cp < 0x80) out.push_back((char)cp);
    else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 0x3F))); }
    else if (cp < 0x10000) {
      out.push_back((char)(0xE0 | (cp >> 12)));
      out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      out.push_back((char)(0x80 | (cp & 0x3F)));
    } else {
      out.push_back((char)(0xF0 | (cp >> 18)));
      out.push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
      out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      out.push_back((char)(0x80 | (cp & 0x3F)));
    }
  }
  bool hex4(unsigned *out) {
    if (end - p < 4) return fail("truncated \\u escape");
    unsigned v = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = *p++;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= c - '0';
      else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
      else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
      else return fail("bad \\u escape");
    }
    *out = v;
    return true;
  }
  bool string(std::string &out) {
    if (p >= end || *p != '"') return fail("expected string");
    ++p;
    while (p < end && *p != '"') {
      if (*p == '\\') {
        if (++p >= end) return fail("truncated escape");
        const char c = *p++;
        switch (c) {
          case '"': out.push_back('"'); break;
          case '\\': out.push_back('\\'); break;
          case '/': out.push_back('/'); break;
          case 'b': out.push_back('\b'); break;
          case 'f': out.push_back('\f'); break;
          case 'n': out.push_back('\n'); break;
          case 'r': out.push_back('\r'); break;
          case 't': out.push_back('\t'); break;
          case 'u': {
            unsigned cp = 0;
            if (!hex4(&cp)) return false;
            if (cp >= 0xD800 && cp < 0xDC00 && end - p >= 6 && p[0] == '\\' && p[1] == 'u') {
              p += 2;
              unsigned lo = 0;
              if (!hex4(&lo)) return false;
              cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
            }
            utf8(out, cp);
            break;
          }
          default: return fail("bad escape");
        }
      } else {
        out.push_back(*p++);
      }
    }
    if (p >= end) return fail("unterminated string");
    ++p;
    return true;
  }
  bool value(JsonValue &v, int depth) {
    if (depth > 64) return fail("nesting too deep");
    ws();
    if (p >= end) return fail("unexpected end");
    const char c = *p;
    if (c == '{') {
      v.kind = JsonValue::Object;
      ++p;
      ws();
      if (p < end && *p == '}') { ++p; return true; }
      for (;;) {
        ws();
        std::string key;
        if (!string(key)) return false;
        ws();
        if (p >= end || *p != ':') return fail("expected ':'");
        ++p;
        v.obj.emplace_back(std::move(key), JsonValue());
        if (!value(v.obj.back().second, depth + 1)) return false;
        ws();
        if (p < end && *p == ',') { ++p; continue; }
        if (p < end && *p == '}') { ++p; return true; }
        return fail("expected ',' or '}'");
      }
    }
    if (c == '[') {
      v.kind = JsonValue::Array;
      ++p;
      ws();
      if (p < end && *p == ']') { ++p; return true; }
      for (;;) {
        v.arr.emplace_back();
        if (!value(v.arr.back(), depth + 1)) return false;
        ws();
        if (p < end && *p == ',') { ++p; continue; }
        if (p < end && *p == ']') { ++p; return true; }
        return fail("expected ',' or ']'");
      }
    }
    if (c == '"') {
      v.kind = JsonValue::String;
      return string(v.str);
    }
    if (end - p >= 4 && !strncmp(p, "true", 4)) { v.kind = JsonValue::Bool; v.b = true; p += 4; return true; }
    if (end - p >= 5 && !strncmp(p, "false", 5)) { v.kind = JsonValue::Bool; v.b = false; p += 5; return true; }
    if (end - p >= 4 && !strncmp(p, "null", 4)) { v.kind = JsonValue::Null; p += 4; return true; }
    if (c == '-' || (c >= '0' && c <= '9')) {
      const char *q = p;
      while (q < end && (*q == '-' || *q == '+' || *q == '.' || *q == 'e' || *q == 'E' || (*q >= '0' && *q <= '9'))) ++q;
      std::string tok(p, q);
      char *stop = nullptr;
      v.num = strtod(tok.c_str(), &stop);
      if (stop == tok.c_str() || *stop) return fail("bad number");
      v.kind = JsonValue::Number;
      p = q;
      return true;
    }
    return fail("unexpected character");
  }
};

bool parse_json(const char *text, size_t len, JsonValue *out, std::string *err) {
  JsonParser ps{text, text + len, {}};
  if (!ps.value(*out, 0)) { *err = ps.err; return false; }
  ps.ws();
  if (ps.p != ps.end) { *err = "trailing characters after the JSON value"; return false; }
  return true;
}

// ---------------------------------------------------------------- mapped file
struct MappedFile {
  int fd = -1;
  const uint8_t *data = nullptr;
  size_t size = 0;
  ~MappedFile() {
    if (data) munmap((void *)data, size);
    if (fd >= 0) close(fd);
  }
};

int map_file(const char *path, MappedFile *f) {
  f->fd = open(path, O_RDONLY);
  RAI_REQUIRE(f->fd >= 0, RAI_ERR_IO, "safetensors: cannot open '%s': %s", path, strerror(errno));
  struct stat st;
  RAI_REQUIRE(fstat(f->fd, &st) == 0, RAI_ERR_IO, "safetensors: cannot stat '%s'", path);
  f->size = (size_t)st.st_size;
  RAI_REQUIRE(f->size >= 8, RAI_ERR_IO, "safetensors: '%s' is shorter than its 8-byte header length", path);
  void *m = mmap(nullptr, f->size, PROT_READ, MAP_PRIVATE, f->fd, 0);
  RAI_REQUIRE(m != MAP_FAILED, RAI_ERR_IO, "safetensors: cannot map '%s': %s", path, strerror(errno));
  f->data = (const uint8_t *)m;
  return RAI_OK;
}

struct StTensor {
  std::string dtype;
  std::vector<int64_t> shape;
  int64_t numel = 0;
  const uint8_t *bytes = nullptr;
  size_t nbytes = 0;
  std::string file;
};

int dtype_size(const std::string &d) {
  if (d == "F64" || d == "I64" || d == "U64") return 8;
  if (d == "F32" || d == "I32" || d == "U32") return 4;
  if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
  if (d == "U8" || d == "I8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
  return 0;
}

int index_file(const char *path, const MappedFile &f, std::map<std::string, StTensor> *out) {
  uint64_t hlen = 0;
  memcpy(&hlen, f.data, 8);  // little-endian host
  RAI_REQUIRE(hlen <= f.size - 8, RAI_ERR_IO, "safetensors: '%s' header length %llu exceeds the file", path,
              (unsigned long long)hlen);
  JsonValue root;
  std::string err;
  RAI_REQUIRE(parse_json((const char *)f.data + 8, (size_t)hlen, &root, &err), RAI_ERR_IO,
              "safetensors: '%s' header is not valid JSON: %s", path, err.c_str());
  RAI_REQUIRE(root.kind == JsonValue::Object, RAI_ERR_IO, "safetensors: '%s' header is not an object", path);
  const uint8_t *base = f.data + 8 + hlen;
  const size_t avail = f.size - 8 - (size_t)hlen;
  for (auto &kv : root.obj) {
    if (kv.first == "__metadata__") continue;
    const JsonValue &t = kv.second;
    const JsonValue *dt = t.get("dtype"), *sh = t.get("shape"), *off = t.get("data_offsets");
    RAI_REQUIRE(t.kind == JsonValue::Object && dt && sh && off && dt->kind == JsonValue::String &&
                    sh->kind == JsonValue::Array && off->kind == JsonValue::Array && off->arr.size() == 2,
                RAI_ERR_IO, "safetensors: '%s': malformed entry for tensor '%s'", path, kv.first.c_str());
    StTensor st;
    st.dtype = dt->str;
    st.numel = 1;
    for (auto &d : sh->arr) {
      // an untrusted header: every extent must be an integer a double holds exactly, and the element count must
      // stay inside the file (which also keeps the product far from overflow)
      RAI_REQUIRE(d.kind == JsonValue::Number && d.num >= 0 && d.num == std::floor(d.num) && d.num <= 9007199254740992.0,
                  RAI_ERR_IO, "safetensors: '%s': bad shape for tensor '%s'", path, kv.first.c_str());
      const int64_t ext = (int64_t)d.num;
      RAI_REQUIRE(ext == 0 || st.numel <= (int64_t)f.size / ext, RAI_ERR_IO,
                  "safetensors: '%s': shape of tensor '%s' describes more elements than the file has bytes", path,
                  kv.first.c_str());
      st.numel *= ext;
      st.shape.push_back(ext);
    }
    const double b = off->arr[0].num, e = off->arr[1].num;
    RAI_REQUIRE(off->arr[0].kind == JsonValue::Number && off->arr[1].kind == JsonValue::Number && b >= 0 && e >= b &&
                    e <= (double)avail,
                RAI_ERR_IO, "safetensors: '%s': data offsets of tensor '%s' lie outside the file", path, kv.first.c_str());
    st.bytes = base + (size_t)b;
    st.nbytes = (size_t)(e - b);
    const int es = dtype_size(st.dtype);
    RAI_REQUIRE(es > 0, RAI_ERR_BAD_DTYPE, "safetensors: '%s': tensor '%s' has unknown dtype %s", path, kv.first.c_str(),
                st.dtype.c_str());
    RAI_REQUIRE((size_t)st.numel * es == st.nbytes, RAI_ERR_IO,
                "safetensors: '%s': tensor '%s' has %lld elements of %s but %zu bytes", path, kv.first.c_str(),
                (long long)st.numel, st.dtype.c_str(), st.nbytes);
    st.file = path;
    (*out)[kv.first] = std::move(st);  // a later file replaces an earlier one (ParamMap::insert)
  }
  return RAI_OK;
}

// ---------------------------------------------------------------- dtype conversion (host)
inline float half_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
  uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {  // subnormal: normalise
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FF) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
inline float bf16_to_f32(uint16_t b) {
  const uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
inline uint16_t f32_to_bf16(float f) {  // round to nearest even, NaN kept quiet
  uint32_t bits;
  memcpy(&bits, &f, 4);
  if ((bits & 0x7F800000u) == 0x7F800000u && (bits & 0x007FFFFFu)) return (uint16_t)((bits >> 16) | 0x0040);
  bits += 0x7FFFu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

// Converts `n` elements of a floating safetensors dtype to the decoder dtype (RAI_F32 / RAI_BF16).
// F64 -> BF16 goes through f32 first, as two chained casts would.
int convert(const StTensor &t, int dst_dtype, std::vector<uint8_t> *out, const char *name) {
  const int64_t n = t.numel;
  const bool to_bf16 = dst_dtype == RAI_BF16;
  out->resize((size_t)n * (to_bf16 ? 2 : 4));
  auto put = [&](int64_t i, float v) {
    if (to_bf16) ((uint16_t *)out->data())[i] = f32_to_bf16(v);
    else ((float *)out->data())[i] = v;
  };
  if (t.dtype == "F32") {
    for (int64_t i = 0; i < n; ++i) { float v; memcpy(&v, t.bytes + 4 * i, 4); put(i, v); }
  } else if (t.dtype == "BF16") {
    for (int64_t i = 0; i < n; ++i) { uint16_t v; memcpy(&v, t.bytes + 2 * i, 2); put(i, bf16_to_f32(v)); }
  } else if (t.dtype == "F16") {
    for (int64_t i = 0; i < n; ++i) { uint16_t v; memcpy(&v, t.bytes + 2 * i, 2); put(i, half_to_f32(v)); }
  } else if (t.dtype == "F64") {
    for (int64_t i = 0; i < n; ++i) { double v; memcpy(&v, t.bytes + 8 * i, 8); put(i, (float)v); }
  } else {
    return fail(RAI_ERR_BAD_DTYPE, "safetensors: parameter '%s' is stored as %s in '%s'; a decoder parameter needs F32, F16, BF16 or F64",
                name, t.dtype.c_str(), t.file.c_str());
  }
  return RAI_OK;
}

}  // namespace
}  // namespace rai

using namespace rai;

extern "C" {

int rai_hip_decoder_load_safetensors(rai_hip_decoder *dec, const char *const *paths, int32_t n_paths) {
  RAI_REQUIRE(dec && paths && n_paths > 0, RAI_ERR_BAD_ARG, "load_safetensors: null decoder or no files");
  std::vector<std::unique_ptr<MappedFile>> files;
  std::map<std::string, StTensor> tensors;
  for (int32_t i = 0; i < n_paths; ++i) {
    RAI_REQUIRE(paths[i], RAI_ERR_BAD_ARG, "load_safetensors: path %d is null", i);
    files.emplace_back(new MappedFile());
    RAI_TRY(map_file(paths[i], files.back().get()));
    RAI_TRY(index_file(paths[i], *files.back(), &tensors));
  }
  int32_t dtype = 0, count = 0;
  RAI_TRY(rai_hip_decoder_dtype(dec, &dtype));
  RAI_TRY(rai_hip_decoder_param_count(dec, &count));
  const size_t es = dtype == RAI_BF16 ? 2 : 4;
  std::vector<uint8_t> staged;
  for (int32_t i = 0; i < count; ++i) {
    char name[256];
    int64_t numel = 0;
    RAI_TRY(rai_hip_decoder_param_name(dec, i, name, sizeof(name), &numel));
    auto it = tensors.find(name);
    RAI_REQUIRE(it != tensors.end(), RAI_ERR_PARAM_NOT_FOUND, "load_safetensors: parameter '%s' not found", name);
    const StTensor &t = it->second;
    RAI_REQUIRE(t.numel == numel, RAI_ERR_BAD_SHAPE, "load_safetensors: parameter '%s' has %lld elements, '%s' holds %lld",
                name, (long long)numel, t.file.c_str(), (long long)t.numel);
    // the same element count is not enough: a transposed or flattened matrix would load and give wrong logits
    int64_t rows = 0, cols = 0;
    RAI_TRY(rai_hip_decoder_param_shape(dec, i, &rows, &cols));
    const bool vec_ok = rows == 1 && t.shape.size() == 1 && t.shape[0] == cols;
    const bool mat_ok = t.shape.size() == 2 && t.shape[0] == rows && t.shape[1] == cols;
    RAI_REQUIRE(vec_ok || mat_ok, RAI_ERR_BAD_SHAPE, "load_safetensors: parameter '%s' is [%lld, %lld], '%s' holds rank %zu [%lld%s",
                name, (long long)rows, (long long)cols, t.file.c_str(), t.shape.size(),
                (long long)(t.shape.empty() ? 0 : t.shape[0]), t.shape.size() > 1 ? ", ..]" : "]");
    const bool same = (dtype == RAI_BF16 && t.dtype == "BF16") || (dtype == RAI_F32 && t.dtype == "F32");
    if (same) {
      RAI_TRY(rai_hip_decoder_load_param(dec, name, t.bytes, t.nbytes));
    } else {
      RAI_TRY(convert(t, dtype, &staged, name));
      RAI_TRY(rai_hip_decoder_load_param(dec, name, staged.data(), (size_t)numel * es));
    }
  }
  return RAI_OK;
}

int rai_hip_safetensors_index_files(const char *index_json_path, char *buf, size_t buflen, int32_t *n_files) {
  RAI_REQUIRE(index_json_path && buf && buflen > 0 && n_files, RAI_ERR_BAD_ARG, "safetensors index: null argument");
  MappedFile f;
  f.fd = open(index_json_path, O_RDONLY);
  RAI_REQUIRE(f.fd >= 0, RAI_ERR_IO, "safetensors index: cannot open '%s': %s", index_json_path, strerror(errno));
  struct stat st;
  RAI_REQUIRE(fstat(f.fd, &st) == 0 && st.st_size > 0, RAI_ERR_IO, "safetensors index: '%s' is empty", index_json_path);
  std::string text((size_t)st.st_size, '\0');
  size_t got = 0;
  while (got < text.size()) {
    const ssize_t r = read(f.fd, &text[got], text.size() - got);
    RAI_REQUIRE(r > 0, RAI_ERR_IO, "safetensors index: short read of '%s'", index_json_path);
    got += (size_t)r;
  }
  JsonValue root;
  std::string err;
  RAI_REQUIRE(parse_json(text.data(), text.size(), &root, &err), RAI_ERR_IO, "safetensors index: '%s' is not valid JSON: %s",
              index_json_path, err.c_str());
  const JsonValue *wm = root.kind == JsonValue::Object ? root.get("weight_map") : nullptr;
  RAI_REQUIRE(wm, RAI_ERR_IO, "safetensors index: '%s' has no weight_map", index_json_path);  // Error::MissingWeightMap
  RAI_REQUIRE(wm->kind == JsonValue::Object, RAI_ERR_IO, "safetensors index: weight_map of '%s' is not an object",
              index_json_path);                                                              // Error::InvalidWeightMap
  std::set<std::string> names;
  for (auto &kv : wm->obj)
    if (kv.second.kind == JsonValue::String) names.insert(kv.second.str);  // non-string values are skipped, as the reference does
  std::string dir(index_json_path);
  const size_t slash = dir.find_last_of('/');
  dir = slash == std::string::npos ? std::string() : dir.substr(0, slash + 1);
  std::string joined;
  for (auto &n : names) {
    if (!joined.empty()) joined.push_back('\n');
    joined += (n.empty() || n[0] == '/') ? n : dir + n;
  }
  RAI_REQUIRE(joined.size() + 1 <= buflen, RAI_ERR_BAD_ARG, "safetensors index: %zu bytes of file names do not fit the %zu-byte buffer",
              joined.size() + 1, buflen);
  memcpy(buf, joined.c_str(), joined.size() + 1);
  *n_files = (int32_t)names.size();
  return RAI_OK;
}

}  // extern "C"
