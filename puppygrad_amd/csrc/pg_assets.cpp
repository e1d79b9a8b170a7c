// Model assets for libpuppygrad_hip.so: the safetensors tensor store, the
// Hugging Face GPT-2 config file and the weight-name mapping, so that a model
// directory becomes a device-resident model without a host copy of the weights
// (tensors are handed to pg_gpt2_create straight out of the file mapping).
// Reference citations (`src/...:line`) name the puppygrad code each piece mirrors.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <mutex>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#include "pg_internal.h"

namespace {

using pgh::fail;

// ---------------------------------------------------------------------------
// A small JSON reader (RFC 8259): enough for a safetensors header and config.json.
// ---------------------------------------------------------------------------
struct Json {
  enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
  bool b = false;
  double num = 0.0;
  bool integral = false;  // written without fraction or exponent, and not negative
  uint64_t u = 0;         // its value when integral
  std::string str;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;  // file order; a later duplicate wins in find()

  const Json* find(const std::string& key) const {
    const Json* hit = nullptr;
    for (const auto& kv : obj)
      if (kv.first == key) hit = &kv.second;
    return hit;
  }
};

class JsonParser {
 public:
  JsonParser(const char* b, const char* e) : begin_(b), p_(b), e_(e) {}

  bool parse(Json& out, std::string& err) {
    bool ok = value(out, 0);
    if (ok) {
      ws();
      if (p_ != e_) ok = bad("trailing characters");
    }
    if (!ok) err = err_ + " at " + where();
    return ok;
  }

 private:
  const char* begin_;
  const char* p_;
  const char* e_;
  std::string err_;

  std::string where() const {
    size_t line = 1, col = 1;
    for (const char* q = begin_; q < p_; ++q) {
      if (*q == '\n') {
        ++line;
        col = 1;
      } else {
        ++col;
      }
    }
    return "line " + std::to_string(line) + " column " + std::to_string(col);
  }
  void ws() {
    while (p_ < e_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
  }
  bool bad(const char* what) {
    err_ = what;
    return false;
  }
  bool literal(const char* word) {
    const size_t n = std::strlen(word);
    if ((size_t)(e_ - p_) < n || std::memcmp(p_, word, n) != 0) return bad("expected value");
    p_ += n;
    return true;
  }
  static void utf8(std::string& s, uint32_t cp) {
    if (cp < 0x80) {
      s += (char)cp;
    } else if (cp < 0x800) {
      s += (char)(0xC0 | (cp >> 6));
      s += (char)(0x80 | (cp & 0x3F));
    } else if (cp < 0x10000) {
      s += (char)(0xE0 | (cp >> 12));
      s += (char)(0x80 | ((cp >> 6) & 0x3F));
      s += (char)(0x80 | (cp & 0x3F));
    } else {
      s += (char)(0xF0 | (cp >> 18));
      s += (char)(0x80 | ((cp >> 12) & 0x3F));
      s += (char)(0x80 | ((cp >> 6) & 0x3F));
      s += (char)(0x80 | (cp & 0x3F));
    }
  }
  bool hex4(uint32_t& v) {
    if (e_ - p_ < 4) return bad("EOF while parsing a string");
    v = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = *p_++;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= (uint32_t)(c - '0');
      else if (c >= 'a' && c <= 'f') v |= (uint32_t)(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') v |= (uint32_t)(c - 'A' + 10);
      else return bad("invalid escape");
    }
    return true;
  }
  bool string(std::string& out) {
    ++p_;  // opening quote
    out.clear();
    while (true) {
      if (p_ == e_) return bad("EOF while parsing a string");
      const unsigned char c = (unsigned char)*p_++;
      if (c == '"') return true;
      if (c < 0x20) return bad("control character found while parsing a string");
      if (c != '\\') {
        out += (char)c;
        continue;
      }
      if (p_ == e_) return bad("EOF while parsing a string");
      const char esc = *p_++;
      switch (esc) {
        case '"': out += '"'; break;
        case '\\': out += '\\'; break;
        case '/': out += '/'; break;
        case 'b': out += '\b'; break;
        case 'f': out += '\f'; break;
        case 'n': out += '\n'; break;
        case 'r': out += '\r'; break;
        case 't': out += '\t'; break;
        case 'u': {
          uint32_t cp;
          if (!hex4(cp)) return false;
          if (cp >= 0xD800 && cp < 0xDC00) {
            uint32_t lo;
            if (e_ - p_ < 2 || p_[0] != '\\' || p_[1] != 'u') return bad("lone leading surrogate");
            p_ += 2;
            if (!hex4(lo)) return false;
            if (lo < 0xDC00 || lo > 0xDFFF) return bad("lone leading surrogate");
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          } else if (cp >= 0xDC00 && cp <= 0xDFFF) {
            return bad("lone trailing surrogate");
          }
          utf8(out, cp);
          break;
        }
        default: return bad("invalid escape");
      }
    }
  }
  bool number(Json& out) {
    const char* s = p_;
    bool neg = false, frac = false;
    if (p_ < e_ && *p_ == '-') {
      neg = true;
      ++p_;
    }
    if (p_ == e_ || *p_ < '0' || *p_ > '9') return bad("invalid number");
    if (*p_ == '0') {
      ++p_;
    } else {
      while (p_ < e_ && *p_ >= '0' && *p_ <= '9') ++p_;
    }
    if (p_ < e_ && *p_ == '.') {
      frac = true;
      ++p_;
      if (p_ == e_ || *p_ < '0' || *p_ > '9') return bad("invalid number");
      while (p_ < e_ && *p_ >= '0' && *p_ <= '9') ++p_;
    }
    if (p_ < e_ && (*p_ == 'e' || *p_ == 'E')) {
      frac = true;
      ++p_;
      if (p_ < e_ && (*p_ == '+' || *p_ == '-')) ++p_;
      if (p_ == e_ || *p_ < '0' || *p_ > '9') return bad("invalid number");
      while (p_ < e_ && *p_ >= '0' && *p_ <= '9') ++p_;
    }
    const std::string text(s, p_);
    out.kind = Json::Num;
    out.num = std::strtod(text.c_str(), nullptr);
    out.integral = false;
    if (!neg && !frac && text.size() <= 19) {  // 19 digits always fit 64 bits
      out.integral = true;
      out.u = std::strtoull(text.c_str(), nullptr, 10);
    }
    return true;
  }
  bool value(Json& out, int depth) {
    if (depth > 128) return bad("recursion limit exceeded");
    ws();
    if (p_ == e_) return bad("EOF while parsing a value");
    switch (*p_) {
      case '{': {
        ++p_;
        out.kind = Json::Obj;
        ws();
        if (p_ < e_ && *p_ == '}') {
          ++p_;
          return true;
        }
        while (true) {
          ws();
          if (p_ == e_ || *p_ != '"') return bad("key must be a string");
          std::string key;
          if (!string(key)) return false;
          ws();
          if (p_ == e_ || *p_ != ':') return bad("expected `:`");
          ++p_;
          Json v;
          if (!value(v, depth + 1)) return false;
          out.obj.emplace_back(std::move(key), std::move(v));
          ws();
          if (p_ < e_ && *p_ == ',') {
            ++p_;
            continue;
          }
          if (p_ < e_ && *p_ == '}') {
            ++p_;
            return true;
          }
          return bad("expected `,` or `}`");
        }
      }
      case '[': {
        ++p_;
        out.kind = Json::Arr;
        ws();
        if (p_ < e_ && *p_ == ']') {
          ++p_;
          return true;
        }
        while (true) {
          Json v;
          if (!value(v, depth + 1)) return false;
          out.arr.push_back(std::move(v));
          ws();
          if (p_ < e_ && *p_ == ',') {
            ++p_;
            continue;
          }
          if (p_ < e_ && *p_ == ']') {
            ++p_;
            return true;
          }
          return bad("expected `,` or `]`");
        }
      }
      case '"':
        out.kind = Json::Str;
        return string(out.str);
      case 't':
        out.kind = Json::Bool;
        out.b = true;
        return literal("true");
      case 'f':
        out.kind = Json::Bool;
        out.b = false;
        return literal("false");
      case 'n':
        out.kind = Json::Null;
        return literal("null");
      default:
        if (*p_ == '-' || (*p_ >= '0' && *p_ <= '9')) return number(out);
        return bad("expected value");
    }
  }
};

std::string shape_text(const std::vector<uint64_t>& shape) {  // Rust's {:?} of a Vec<usize>
  std::string s = "[";
  for (size_t i = 0; i < shape.size(); ++i) s += (i ? ", " : "") + std::to_string(shape[i]);
  return s + "]";
}

// Element size of a safetensors dtype name; 0 when the name is unknown.
size_t dtype_bytes(const std::string& d) {
  static const std::map<std::string, size_t> k = {
      {"BOOL", 1}, {"U8", 1},   {"I8", 1},   {"F8_E5M2", 1}, {"F8_E4M3", 1}, {"I16", 2},
      {"U16", 2},  {"F16", 2},  {"BF16", 2}, {"I32", 4},     {"U32", 4},     {"F32", 4},
      {"F64", 8},  {"I64", 8},  {"U64", 8}};
  auto it = k.find(d);
  return it == k.end() ? 0 : it->second;
}

struct TensorInfo {
  std::string dtype;
  std::vector<uint64_t> shape;
  uint64_t begin = 0, end = 0;  // byte range inside the data section
};

}  // namespace

// TensorStore (src/models/safetensors.rs:93-138) over a read-only mapping of the file
// (the reference reads the file into a Vec first, safetensors.rs:79-84).
struct pg_tensor_store {
  std::string path;
  void* map = nullptr;
  size_t map_len = 0;
  const uint8_t* data = nullptr;  // first byte after the header
  size_t data_len = 0;
  std::map<std::string, TensorInfo> tensors;
  // A tensor whose bytes do not start on a 4-byte boundary is copied here on first use (under
  // the lock: lookups of one store may come from several threads).
  mutable std::map<std::string, std::vector<float>> realigned;
  mutable std::mutex realigned_mu;

  ~pg_tensor_store() {
    if (map && map != MAP_FAILED) munmap(map, map_len);
  }
};

namespace {

enum class Lookup { Found, Missing, Error };

pg_status parse_error(const std::string& path, const std::string& why) {
  // SafeTensorLoadError::ParseFile (src/models/safetensors.rs:46-48)
  return fail(PG_ASSET, "failed to parse safetensors file " + path + ": " + why);
}

// The container format: u64 LE header length, a JSON object
// name -> {dtype, shape, data_offsets:[begin,end]} (+ "__metadata__"), then the data.
pg_status open_store(const char* path, std::unique_ptr<pg_tensor_store>& out) {
  auto st = std::make_unique<pg_tensor_store>();
  st->path = path;
  const int fd = ::open(path, O_RDONLY | O_CLOEXEC);
  if (fd < 0)  // SafeTensorLoadError::ReadFile (src/models/safetensors.rs:43-45)
    return fail(PG_ASSET, "failed to read safetensors file " + st->path + ": " +
                              std::strerror(errno));
  struct stat sb;
  if (fstat(fd, &sb) != 0) {
    const std::string why = std::strerror(errno);
    ::close(fd);
    return fail(PG_ASSET, "failed to read safetensors file " + st->path + ": " + why);
  }
  if (!S_ISREG(sb.st_mode)) {
    ::close(fd);
    return fail(PG_ASSET, "failed to read safetensors file " + st->path + ": " +
                              (S_ISDIR(sb.st_mode) ? "Is a directory" : "not a regular file"));
  }
  st->map_len = (size_t)sb.st_size;
  if (st->map_len < 8) {
    ::close(fd);
    return parse_error(st->path, "header too small");
  }
  st->map = mmap(nullptr, st->map_len, PROT_READ, MAP_PRIVATE, fd, 0);
  const int map_errno = errno;
  ::close(fd);
  if (st->map == MAP_FAILED) {
    st->map = nullptr;
    return fail(PG_ASSET, "failed to read safetensors file " + st->path + ": " +
                              std::strerror(map_errno));
  }
  const uint8_t* bytes = (const uint8_t*)st->map;
  uint64_t n = 0;
  for (int i = 7; i >= 0; --i) n = (n << 8) | bytes[i];
  if (n > 100000000ull) return parse_error(st->path, "header too large");
  if (n > st->map_len - 8) return parse_error(st->path, "invalid header length");
  const char* hb = (const char*)bytes + 8;
  if (n == 0 || hb[0] != '{') return parse_error(st->path, "invalid header start");
  Json header;
  std::string err;
  if (!JsonParser(hb, hb + n).parse(header, err))
    return parse_error(st->path, "invalid header deserialization: " + err);
  if (header.kind != Json::Obj)
    return parse_error(st->path, "invalid header deserialization: expected an object");
  st->data = bytes + 8 + n;
  st->data_len = st->map_len - 8 - (size_t)n;

  std::vector<std::pair<std::pair<uint64_t, uint64_t>, std::string>> order;  // (begin, end), name
  for (const auto& kv : header.obj) {
    if (kv.first == "__metadata__") continue;
    const Json& t = kv.second;
    const Json* dt = t.kind == Json::Obj ? t.find("dtype") : nullptr;
    const Json* sh = t.kind == Json::Obj ? t.find("shape") : nullptr;
    const Json* of = t.kind == Json::Obj ? t.find("data_offsets") : nullptr;
    if (!dt || dt->kind != Json::Str || !sh || sh->kind != Json::Arr || !of ||
        of->kind != Json::Arr || of->arr.size() != 2 || !of->arr[0].integral ||
        !of->arr[1].integral)
      return parse_error(st->path, "invalid header deserialization: tensor `" + kv.first +
                                       "` needs dtype, shape and data_offsets");
    TensorInfo info;
    info.dtype = dt->str;
    const size_t esz = dtype_bytes(info.dtype);
    if (esz == 0)
      return parse_error(st->path, "invalid header deserialization: unknown dtype `" +
                                       info.dtype + "` of tensor `" + kv.first + "`");
    unsigned __int128 count = 1;
    for (const Json& d : sh->arr) {
      if (!d.integral)
        return parse_error(st->path, "invalid header deserialization: shape of tensor `" +
                                         kv.first + "` must hold unsigned integers");
      info.shape.push_back(d.u);
      count *= d.u;
      if (count > ((unsigned __int128)1 << 64)) return parse_error(st->path, "shape overflow");
    }
    info.begin = of->arr[0].u;
    info.end = of->arr[1].u;
    if (info.begin > info.end || info.end > st->data_len)
      return parse_error(st->path, "invalid offset for tensor `" + kv.first + "`");
    if ((unsigned __int128)(info.end - info.begin) != count * esz)
      return parse_error(st->path, "invalid tensor info for tensor `" + kv.first +
                                       "`: byte range does not match dtype and shape");
    order.emplace_back(std::make_pair(info.begin, info.end), kv.first);
    st->tensors[kv.first] = std::move(info);
  }
  // The data section is the tensors back to back, without holes or overlap, to its end.
  std::sort(order.begin(), order.end());
  uint64_t at = 0;
  for (const auto& o : order) {
    const TensorInfo& info = st->tensors[o.second];
    if (info.begin != at) return parse_error(st->path, "invalid offset for tensor `" + o.second + "`");
    at = info.end;
  }
  if (at != st->data_len) return parse_error(st->path, "metadata incomplete buffer");
  out = std::move(st);
  return PG_OK;
}

// required_f32 / optional_f32 (src/models/safetensors.rs:125-137) with validate_tensor
// (150-170) and f32_data (172-185).  `view` points into the mapping.
Lookup lookup_f32(const pg_tensor_store& st, const std::string& name,
                  const std::vector<uint64_t>& expected, pg_tensor* view, pg_status* status) {
  auto it = st.tensors.find(name);
  if (it == st.tensors.end()) return Lookup::Missing;
  const TensorInfo& t = it->second;
  if (t.dtype != "F32") {
    *status = fail(PG_ASSET, "tensor " + name + " has dtype " + t.dtype + ", expected F32");
    return Lookup::Error;
  }
  if (t.shape != expected) {
    *status = fail(PG_INVALID_WEIGHTS, "tensor " + name + " shape " + shape_text(t.shape) +
                                           " does not match expected " + shape_text(expected));
    return Lookup::Error;
  }
  const uint8_t* p = st.data + t.begin;
  const size_t n = (size_t)(t.end - t.begin) / 4;
  if (((uintptr_t)p & 3u) != 0) {
    std::lock_guard<std::mutex> lock(st.realigned_mu);
    auto& copy = st.realigned[name];
    if (copy.size() != n) {
      copy.resize(n);
      std::memcpy(copy.data(), p, n * 4);
    }
    p = (const uint8_t*)copy.data();
  }
  view->data = (const float*)p;
  view->len = n;
  return Lookup::Found;
}

pg_status not_found(const std::string& name) {
  // SafeTensorLoadError::TensorNotFound (src/models/safetensors.rs:49-51)
  return fail(PG_ASSET, "failed to read tensor " + name + ": tensor `" + name + "` not found");
}

// tensor_f32 with the `transformer.` fallback (src/models/gpt2/rust.rs:762-771).
pg_status gpt2_tensor(const pg_tensor_store& st, const std::string& name,
                      const std::vector<uint64_t>& shape, pg_tensor* out) {
  pg_status s = PG_OK;
  switch (lookup_f32(st, name, shape, out, &s)) {
    case Lookup::Found: return PG_OK;
    case Lookup::Error: return s;
    case Lookup::Missing: break;
  }
  const std::string prefixed = "transformer." + name;
  switch (lookup_f32(st, prefixed, shape, out, &s)) {
    case Lookup::Found: return PG_OK;
    case Lookup::Error: return s;
    case Lookup::Missing: break;
  }
  return not_found(prefixed);
}

// One unsigned field of HfGpt2Config (src/models/gpt2/rust.rs:684-694).
pg_status config_uint(const std::string& path, const Json& root, const char* key, bool required,
                      bool* present, uint64_t* out) {
  const Json* v = root.find(key);
  *present = false;
  if (!v || (!required && v->kind == Json::Null)) {
    if (required)
      return fail(PG_ASSET, "failed to parse config " + path + ": missing field `" + key + "`");
    return PG_OK;
  }
  if (v->kind != Json::Num || !v->integral)
    return fail(PG_ASSET, "failed to parse config " + path + ": invalid type for field `" +
                              key + "`, expected an unsigned integer");
  *present = true;
  *out = v->u;
  return PG_OK;
}

std::string join(const std::string& dir, const char* file) {
  if (dir.empty()) return file;
  return dir.back() == '/' ? dir + file : dir + "/" + file;
}

}  // namespace

extern "C" {

pg_status pg_tensor_store_open(const char* path, pg_tensor_store** out) {
  if (!path || !out) return fail(PG_INVALID_INPUT, "null argument");
  *out = nullptr;
  std::unique_ptr<pg_tensor_store> st;
  if (pg_status s = open_store(path, st)) return s;
  *out = st.release();
  return PG_OK;
}

void pg_tensor_store_close(pg_tensor_store* store) { delete store; }

uint64_t pg_tensor_store_len(const pg_tensor_store* store) {
  return store ? store->tensors.size() : 0;
}

pg_status pg_tensor_store_required_f32(const pg_tensor_store* store, const char* name,
                                       const uint64_t* shape, size_t ndim, pg_tensor* out) {
  if (!store || !name || !out || (!shape && ndim)) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s = PG_OK;
  switch (lookup_f32(*store, name, std::vector<uint64_t>(shape, shape + ndim), out, &s)) {
    case Lookup::Found: return PG_OK;
    case Lookup::Error: return s;
    case Lookup::Missing: break;
  }
  return not_found(name);
}

pg_status pg_tensor_store_optional_f32(const pg_tensor_store* store, const char* name,
                                       const uint64_t* shape, size_t ndim, int32_t* found,
                                       pg_tensor* out) {
  if (!store || !name || !out || !found || (!shape && ndim))
    return fail(PG_INVALID_INPUT, "null argument");
  pg_status s = PG_OK;
  const Lookup r = lookup_f32(*store, name, std::vector<uint64_t>(shape, shape + ndim), out, &s);
  *found = r == Lookup::Found;
  return r == Lookup::Error ? s : PG_OK;
}

pg_status pg_gpt2_load_config(const char* path, pg_gpt2_config* out) {
  if (!path || !out) return fail(PG_INVALID_INPUT, "null argument");
  std::ifstream in(path, std::ios::binary);
  if (!in)  // ConfigLoadError::Read (src/models/config.rs:22-24)
    return fail(PG_ASSET, std::string("failed to read config ") + path + ": " +
                              std::strerror(errno));
  std::stringstream buf;
  buf << in.rdbuf();
  const std::string text = buf.str();
  Json root;
  std::string err;
  if (!JsonParser(text.data(), text.data() + text.size()).parse(root, err))
    return fail(PG_ASSET, std::string("failed to parse config ") + path + ": " + err);
  if (root.kind != Json::Obj)
    return fail(PG_ASSET, std::string("failed to parse config ") + path +
                              ": invalid type, expected struct HfGpt2Config");
  pg_gpt2_config c{};
  bool have = false, have_pos = false, have_ctx = false, have_inner = false;
  uint64_t n_ctx = 0, n_inner = 0;
  pg_status s;
  if ((s = config_uint(path, root, "vocab_size", true, &have, &c.vocab_size))) return s;
  if ((s = config_uint(path, root, "n_positions", false, &have_pos, &c.n_positions))) return s;
  if ((s = config_uint(path, root, "n_ctx", false, &have_ctx, &n_ctx))) return s;
  if ((s = config_uint(path, root, "n_embd", true, &have, &c.n_embd))) return s;
  if ((s = config_uint(path, root, "n_layer", true, &have, &c.n_layer))) return s;
  if ((s = config_uint(path, root, "n_head", true, &have, &c.n_head))) return s;
  if ((s = config_uint(path, root, "n_inner", false, &have_inner, &n_inner))) return s;
  if (!have_pos) {
    if (!have_ctx)  // src/models/gpt2/rust.rs:699-701
      return fail(PG_INVALID_CONFIG, "config must contain n_positions or n_ctx");
    c.n_positions = n_ctx;
  }
  c.n_inner = have_inner ? n_inner : 4 * c.n_embd;  // Gpt2Config::new (rust.rs:41-58)
  c.layer_norm_epsilon = 1e-5f;
  if (const Json* e = root.find("layer_norm_epsilon"); e && e->kind != Json::Null) {
    if (e->kind != Json::Num)
      return fail(PG_ASSET, std::string("failed to parse config ") + path +
                                ": invalid type for field `layer_norm_epsilon`, expected f32");
    c.layer_norm_epsilon = (float)e->num;
  }
  if ((s = pgh::validate_config(c))) return s;
  *out = c;
  return PG_OK;
}

pg_status pg_hip_load_tuning(const char* path, pg_hip_options* options, int32_t* found) {
  if (!path || !options) return fail(PG_INVALID_INPUT, "null argument");
  if (found) *found = 0;
  errno = 0;  // (an earlier call's value must not decide what a failed open means)
  std::ifstream in(path, std::ios::binary);
  if (!in) {
    const int why = errno;
    if (why == ENOENT) return PG_OK;  // load_gpt2_tuning: a missing default file is no error
    return fail(PG_ASSET, std::string("failed to read tuning file ") + path + ": " +
                              std::strerror(why ? why : EIO));
  }
  std::stringstream buf;
  buf << in.rdbuf();
  const std::string text = buf.str();
  Json root;
  std::string err;
  if (!JsonParser(text.data(), text.data() + text.size()).parse(root, err))
    return fail(PG_ASSET, std::string("failed to parse tuning file ") + path + ": " + err);
  if (root.kind != Json::Obj)
    return fail(PG_ASSET, std::string("failed to parse tuning file ") + path +
                              ": expected an object of per-backend tunings");
  // The file is shared with the other backends: the reference's own `autotune gpt2` writes one
  // with only a `rust` object (SavedGpt2Tuning, src/main.rs:2564-2623).  Without a `hip`
  // object there is no tuning for this backend and the defaults stand.
  const Json* hip = root.find("hip");
  if (!hip || hip->kind == Json::Null) return PG_OK;
  if (hip->kind != Json::Obj)
    return fail(PG_ASSET, std::string("failed to parse tuning file ") + path +
                              ": invalid type for field `hip`, expected an object");
  struct Field {
    const char* key;
    uint32_t* dst;
  } fields[] = {{"attn_item_keys", &options->attn_item_keys},
                {"attn_blocks_per_cu", &options->attn_blocks_per_cu},
                {"gemm_split_items_per_cu", &options->gemm_split_items_per_cu},
                {"gemm_b9_min_rows", &options->gemm_b9_min_rows},
                {"seq_gemm_min_tokens", &options->seq_gemm_min_tokens}};
  for (const Field& f : fields) {
    const Json* v = hip->find(f.key);
    if (!v || v->kind == Json::Null) continue;
    if (v->kind != Json::Num || v->num < 0 || v->num > 4294967295.0 || v->num != std::floor(v->num))
      return fail(PG_ASSET, std::string("failed to parse tuning file ") + path +
                                ": invalid type for field `" + f.key + "`, expected u32");
    if (*f.dst == 0) *f.dst = (uint32_t)v->num;  // a value the caller set explicitly wins
  }
  if (found) *found = 1;
  return PG_OK;
}

pg_status pg_gpt2_create_from_dir(const char* model_dir, const pg_hip_options* options,
                                  pg_gpt2_model** out) {
  if (!model_dir || !out) return fail(PG_INVALID_INPUT, "null argument");
  *out = nullptr;
  // load_gpt2_tuning (src/main.rs:2564-2586): {model_dir}/puppygrad-tune.json, when it exists,
  // supplies the tunables the caller left at their defaults
  pg_hip_options tuned{};
  if (options) tuned = *options;
  {
    const std::string tune_path = join(model_dir, "puppygrad-tune.json");
    pg_status ts = pg_hip_load_tuning(tune_path.c_str(), &tuned, nullptr);
    if (ts) return ts;
    options = &tuned;
  }
  // Gpt2AssetPaths::new (src/models/gpt2/assets.rs:20-30)
  const std::string config_path = join(model_dir, "config.json");
  const std::string weights_path = join(model_dir, "model.safetensors");
  pg_gpt2_config cfg{};
  pg_status s;
  if ((s = pg_gpt2_load_config(config_path.c_str(), &cfg))) return s;
  std::unique_ptr<pg_tensor_store> st;
  if ((s = open_store(weights_path.c_str(), st))) return s;

  // load_weights (src/models/gpt2/rust.rs:713-760)
  const uint64_t C = cfg.n_embd, I = cfg.n_inner;
  std::vector<pg_gpt2_block_view> blocks(cfg.n_layer);
  for (uint64_t l = 0; l < cfg.n_layer; ++l) {
    const std::string p = "h." + std::to_string(l);
    pg_gpt2_block_view& b = blocks[l];
    if ((s = gpt2_tensor(*st, p + ".ln_1.weight", {C}, &b.ln_1_g))) return s;
    if ((s = gpt2_tensor(*st, p + ".ln_1.bias", {C}, &b.ln_1_b))) return s;
    if ((s = gpt2_tensor(*st, p + ".attn.c_attn.weight", {C, 3 * C}, &b.c_attn_w))) return s;
    if ((s = gpt2_tensor(*st, p + ".attn.c_attn.bias", {3 * C}, &b.c_attn_b))) return s;
    if ((s = gpt2_tensor(*st, p + ".attn.c_proj.weight", {C, C}, &b.c_proj_w))) return s;
    if ((s = gpt2_tensor(*st, p + ".attn.c_proj.bias", {C}, &b.c_proj_b))) return s;
    if ((s = gpt2_tensor(*st, p + ".ln_2.weight", {C}, &b.ln_2_g))) return s;
    if ((s = gpt2_tensor(*st, p + ".ln_2.bias", {C}, &b.ln_2_b))) return s;
    if ((s = gpt2_tensor(*st, p + ".mlp.c_fc.weight", {C, I}, &b.c_fc_w))) return s;
    if ((s = gpt2_tensor(*st, p + ".mlp.c_fc.bias", {I}, &b.c_fc_b))) return s;
    if ((s = gpt2_tensor(*st, p + ".mlp.c_proj.weight", {I, C}, &b.c_proj_mlp_w))) return s;
    if ((s = gpt2_tensor(*st, p + ".mlp.c_proj.bias", {C}, &b.c_proj_mlp_b))) return s;
  }
  pg_gpt2_weights_view w{};
  if ((s = gpt2_tensor(*st, "wte.weight", {cfg.vocab_size, C}, &w.wte))) return s;
  if ((s = gpt2_tensor(*st, "wpe.weight", {cfg.n_positions, C}, &w.wpe))) return s;
  if ((s = gpt2_tensor(*st, "ln_f.weight", {C}, &w.ln_f_g))) return s;
  if ((s = gpt2_tensor(*st, "ln_f.bias", {C}, &w.ln_f_b))) return s;
  w.blocks = blocks.data();
  w.n_blocks = blocks.size();
  // The upload reads each tensor once, straight from the mapping.
  return pg_gpt2_create(&cfg, &w, options, out);
}

}  // extern "C"
