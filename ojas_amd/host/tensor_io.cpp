// safetensors reader / writer and the checkpoint-v1 state file behind include/ojas_io.h.
//
// Follows ojas-io/src/safetensors.rs (header rules :1616-1800, dtype table :43-160, writer
// :1224-1260) and ojas-io/src/checkpoint.rs with docs/checkpoint-v1.md. The JSON reader below
// accepts exactly what a safetensors header may hold: objects, arrays, strings and non-negative
// integers, three levels deep, no repeated keys.
#include "ojas_io.h"

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cinttypes>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <new>
#include <set>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int32_t fail(const char* fmt, ...) {
  char buf[768];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return OIO_ERROR;
}

bool read_exact_at(int fd, void* dst, uint64_t n, uint64_t offset) {
  char* p = static_cast<char*>(dst);
  while (n > 0) {
    const ssize_t got = pread(fd, p, n, static_cast<off_t>(offset));
    if (got < 0) {
      if (errno == EINTR) continue;
      return false;
    }
    if (got == 0) {
      errno = 0;
      return false;
    }
    p += got;
    offset += static_cast<uint64_t>(got);
    n -= static_cast<uint64_t>(got);
  }
  return true;
}

// Writes `bytes` to a temporary file beside `path` and renames it over `path`.
int32_t replace_file(const char* path, const std::vector<const void*>& parts, const std::vector<uint64_t>& lens) {
  std::string tmp = std::string(path) + ".tmp." + std::to_string(static_cast<long>(getpid()));
  const int fd = open(tmp.c_str(), O_WRONLY | O_CREAT | O_EXCL | O_CLOEXEC, 0644);
  if (fd < 0) return fail("%s: %s", tmp.c_str(), strerror(errno));
  bool ok = true;
  for (size_t i = 0; ok && i < parts.size(); ++i) {
    const char* p = static_cast<const char*>(parts[i]);
    uint64_t left = lens[i];
    while (left > 0) {
      const ssize_t put = write(fd, p, left);
      if (put < 0) {
        if (errno == EINTR) continue;
        ok = false;
        break;
      }
      p += put;
      left -= static_cast<uint64_t>(put);
    }
  }
  const int werr = errno;
  if (ok && fsync(fd) != 0) ok = false;
  const int serr = ok ? 0 : (werr ? werr : errno);
  close(fd);
  if (!ok) {
    unlink(tmp.c_str());
    return fail("%s: write: %s", path, strerror(serr));
  }
  if (rename(tmp.c_str(), path) != 0) {
    const int e = errno;
    unlink(tmp.c_str());
    return fail("%s: rename: %s", path, strerror(e));
  }
  return OIO_OK;
}

// ---- dtype table (safetensors.rs:43-160): tag -> bits per element ----
struct DtypeRow {
  const char* tag;
  uint32_t bits;
};
const DtypeRow kDtypes[] = {{"F32", 32},        {"BF16", 16},       {"F16", 16},    {"I64", 64},     {"U16", 16},
                            {"BOOL", 8},        {"F4", 4},          {"F6_E2M3", 6}, {"F6_E3M2", 6},  {"U8", 8},
                            {"I8", 8},          {"F8_E5M2", 8},     {"F8_E4M3", 8}, {"F8_E8M0", 8},  {"F8_E4M3FNUZ", 8},
                            {"F8_E5M2FNUZ", 8}, {"C64", 64},        {"I16", 16},    {"I32", 32},     {"U32", 32},
                            {"F64", 64},        {"U64", 64}};
const DtypeRow* find_dtype(const std::string& tag) {
  for (const DtypeRow& row : kDtypes)
    if (tag == row.tag) return &row;
  return nullptr;
}

// byte_len (safetensors.rs:1560-1587): shape product in u64 (a zero extent makes it zero whatever
// the other extents are), times the bit width, a whole number of bytes.
int32_t byte_len(const std::string& name, const std::vector<uint64_t>& shape, const DtypeRow& dt, uint64_t* out) {
  bool zero = false;
  for (uint64_t d : shape) zero |= d == 0;
  unsigned __int128 n = 1;
  if (zero) {
    n = 0;
  } else {
    for (uint64_t d : shape) {
      n *= d;
      if (n > UINT64_MAX) return fail("\"%s\": shape product overflows", name.c_str());
    }
  }
  const unsigned __int128 bits = n * dt.bits;
  if (bits % 8 != 0)
    return fail("\"%s\": %" PRIu64 " elements of %s is not a whole number of bytes", name.c_str(),
                static_cast<uint64_t>(n), dt.tag);
  if (bits / 8 > UINT64_MAX) return fail("\"%s\": byte size overflows", name.c_str());
  *out = static_cast<uint64_t>(bits / 8);
  return OIO_OK;
}

// ---- the header's JSON ----
struct Json {
  enum Kind { Object, Array, String, Number } kind = String;
  std::vector<std::pair<std::string, Json>> fields;  // Object, in file order
  std::vector<Json> items;                           // Array
  std::string text;                                  // String
  uint64_t number = 0;                               // Number
};

struct JsonReader {
  const unsigned char* p;
  const unsigned char* end;
  std::string error;

  bool err(const char* what) {
    if (error.empty()) error = what;
    return false;
  }
  void space() {
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
  }
  bool hex4(uint32_t* out) {
    if (end - p < 4) return err("truncated \\u escape");
    uint32_t v = 0;
    for (int i = 0; i < 4; ++i) {
      const unsigned char c = p[i];
      v <<= 4;
      if (c >= '0' && c <= '9') v |= c - '0';
      else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
      else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
      else return err("bad \\u escape");
    }
    p += 4;
    *out = v;
    return true;
  }
  static void utf8(std::string& out, uint32_t c) {
    if (c < 0x80) out.push_back(static_cast<char>(c));
    else if (c < 0x800) {
      out.push_back(static_cast<char>(0xC0 | (c >> 6)));
      out.push_back(static_cast<char>(0x80 | (c & 0x3F)));
    } else if (c < 0x10000) {
      out.push_back(static_cast<char>(0xE0 | (c >> 12)));
      out.push_back(static_cast<char>(0x80 | ((c >> 6) & 0x3F)));
      out.push_back(static_cast<char>(0x80 | (c & 0x3F)));
    } else {
      out.push_back(static_cast<char>(0xF0 | (c >> 18)));
      out.push_back(static_cast<char>(0x80 | ((c >> 12) & 0x3F)));
      out.push_back(static_cast<char>(0x80 | ((c >> 6) & 0x3F)));
      out.push_back(static_cast<char>(0x80 | (c & 0x3F)));
    }
  }
  bool string(std::string* out) {
    if (p >= end || *p != '"') return err("expected a string");
    ++p;
    out->clear();
    while (true) {
      if (p >= end) return err("unterminated string");
      const unsigned char c = *p++;
      if (c == '"') return true;
      if (c < 0x20) return err("control character in a string");
      if (c != '\\') {
        out->push_back(static_cast<char>(c));
        continue;
      }
      if (p >= end) return err("unterminated escape");
      const unsigned char e = *p++;
      switch (e) {
        case '"': out->push_back('"'); break;
        case '\\': out->push_back('\\'); break;
        case '/': out->push_back('/'); break;
        case 'b': out->push_back('\b'); break;
        case 'f': out->push_back('\f'); break;
        case 'n': out->push_back('\n'); break;
        case 'r': out->push_back('\r'); break;
        case 't': out->push_back('\t'); break;
        case 'u': {
          uint32_t c1 = 0;
          if (!hex4(&c1)) return false;
          if (c1 >= 0xD800 && c1 <= 0xDBFF) {
            uint32_t c2 = 0;
            if (end - p < 2 || p[0] != '\\' || p[1] != 'u') return err("lone surrogate");
            p += 2;
            if (!hex4(&c2)) return false;
            if (c2 < 0xDC00 || c2 > 0xDFFF) return err("lone surrogate");
            c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
          } else if (c1 >= 0xDC00 && c1 <= 0xDFFF) {
            return err("lone surrogate");
          }
          utf8(*out, c1);
          break;
        }
        default: return err("unknown escape");
      }
    }
  }
  bool value(Json* out, int depth) {
    space();
    if (p >= end) return err("unexpected end of JSON");
    const unsigned char c = *p;
    if (c == '{') {
      if (depth >= 3) return err("JSON nests deeper than a safetensors header does");
      ++p;
      out->kind = Json::Object;
      std::set<std::string> seen;
      space();
      if (p < end && *p == '}') {
        ++p;
        return true;
      }
      while (true) {
        space();
        std::string key;
        if (!string(&key)) return false;
        if (!seen.insert(key).second) {
          error = "duplicate key \"" + key + "\"";
          return false;
        }
        space();
        if (p >= end || *p != ':') return err("expected ':'");
        ++p;
        Json v;
        if (!value(&v, depth + 1)) return false;
        out->fields.emplace_back(std::move(key), std::move(v));
        space();
        if (p < end && *p == ',') {
          ++p;
          continue;
        }
        if (p < end && *p == '}') {
          ++p;
          return true;
        }
        return err("expected ',' or '}'");
      }
    }
    if (c == '[') {
      if (depth >= 3) return err("JSON nests deeper than a safetensors header does");
      ++p;
      out->kind = Json::Array;
      space();
      if (p < end && *p == ']') {
        ++p;
        return true;
      }
      while (true) {
        Json v;
        if (!value(&v, depth + 1)) return false;
        out->items.push_back(std::move(v));
        space();
        if (p < end && *p == ',') {
          ++p;
          continue;
        }
        if (p < end && *p == ']') {
          ++p;
          return true;
        }
        return err("expected ',' or ']'");
      }
    }
    if (c == '"') {
      out->kind = Json::String;
      return string(&out->text);
    }
    if (c >= '0' && c <= '9') {
      out->kind = Json::Number;
      const unsigned char* start = p;
      unsigned __int128 v = 0;
      while (p < end && *p >= '0' && *p <= '9') {
        v = v * 10 + (*p - '0');
        if (v > UINT64_MAX) return err("integer exceeds u64");
        ++p;
      }
      if (p - start > 1 && *start == '0') return err("leading zero");
      if (p < end && (*p == '.' || *p == 'e' || *p == 'E')) return err("a header holds integers only");
      out->number = static_cast<uint64_t>(v);
      return true;
    }
    return err("a header holds objects, arrays, strings and non-negative integers only");
  }
};

bool valid_utf8(const unsigned char* p, size_t n) {
  size_t i = 0;
  while (i < n) {
    const unsigned char c = p[i];
    size_t extra;
    uint32_t v;
    if (c < 0x80) {
      ++i;
      continue;
    } else if ((c & 0xE0) == 0xC0) {
      extra = 1;
      v = c & 0x1F;
    } else if ((c & 0xF0) == 0xE0) {
      extra = 2;
      v = c & 0x0F;
    } else if ((c & 0xF8) == 0xF0) {
      extra = 3;
      v = c & 0x07;
    } else {
      return false;
    }
    if (i + extra >= n) return false;
    for (size_t k = 1; k <= extra; ++k) {
      if ((p[i + k] & 0xC0) != 0x80) return false;
      v = (v << 6) | (p[i + k] & 0x3F);
    }
    if ((extra == 1 && v < 0x80) || (extra == 2 && v < 0x800) || (extra == 3 && v < 0x10000)) return false;
    if (v > 0x10FFFF || (v >= 0xD800 && v <= 0xDFFF)) return false;
    i += extra + 1;
  }
  return true;
}

void push_json_str(std::string& out, const std::string& s) {  // safetensors.rs:1589-1606
  out.push_back('"');
  for (unsigned char c : s) {
    switch (c) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\r': out += "\\r"; break;
      case '\t': out += "\\t"; break;
      default:
        if (c < 0x20) {
          char buf[8];
          snprintf(buf, sizeof buf, "\\u%04x", c);
          out += buf;
        } else {
          out.push_back(static_cast<char>(c));
        }
    }
  }
  out.push_back('"');
}

struct TensorEntry {
  const DtypeRow* dtype = nullptr;
  std::vector<uint64_t> shape;
  uint64_t begin = 0, end = 0;
};

float half_to_float(uint16_t h) {  // IEEE binary16, exact
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int shift = 0;
      while (!(man & 0x400)) {
        man <<= 1;
        ++shift;
      }
      man &= 0x3FF;
      bits = sign | (static_cast<uint32_t>(127 - 15 - shift + 1) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

}  // namespace

struct oio_safetensors {
  int fd = -1;
  uint64_t data_start = 0, data_len = 0, file_len = 0;
  std::map<std::string, TensorEntry> tensors;  // ascending byte order of the names
  std::vector<const std::string*> order;
  std::map<std::string, std::string> metadata;
  std::vector<const std::string*> meta_order;
};

struct oio_ckpt {
  std::vector<uint8_t> bytes;
  std::vector<std::string> names;
  std::vector<std::vector<uint64_t>> shapes;
  std::vector<oio_blob> blobs[4];
};

namespace {

int32_t parse_header(oio_safetensors& s, const std::vector<unsigned char>& header) {
  if (!valid_utf8(header.data(), header.size())) return fail("header is not UTF-8");
  JsonReader r{header.data(), header.data() + header.size(), {}};
  Json root;
  r.space();
  if (r.p < r.end && *r.p != '{') {
    // Any other well-formed or ill-formed root is "not a JSON object" to the caller.
    return fail("header is not a JSON object");
  }
  if (!r.value(&root, 0)) return fail("header: %s", r.error.c_str());
  r.space();
  if (r.p != r.end) return fail("header: trailing bytes after the JSON object");
  for (auto& field : root.fields) {
    const std::string& name = field.first;
    Json& v = field.second;
    if (name == "__metadata__") {
      if (v.kind != Json::Object) return fail("__metadata__ is not an object");
      for (auto& kv : v.fields) {
        if (kv.second.kind != Json::String)
          return fail("__metadata__ value for \"%s\" is not a string", kv.first.c_str());
        s.metadata[kv.first] = kv.second.text;
      }
      continue;
    }
    if (name.empty()) return fail("tensor name is empty");
    if (v.kind != Json::Object) return fail("%s: entry is not an object", name.c_str());
    TensorEntry t;
    bool has_shape = false, has_offsets = false;
    for (auto& kv : v.fields) {
      const std::string& k = kv.first;
      Json& f = kv.second;
      if (k == "dtype" && f.kind == Json::String) {
        t.dtype = find_dtype(f.text);
        if (!t.dtype) return fail("%s: unknown dtype \"%s\"", name.c_str(), f.text.c_str());
      } else if (k == "shape" && f.kind == Json::Array) {
        for (Json& d : f.items) {
          if (d.kind != Json::Number) return fail("%s: shape holds a non-integer", name.c_str());
          t.shape.push_back(d.number);
        }
        has_shape = true;
      } else if (k == "data_offsets" && f.kind == Json::Array) {
        if (f.items.size() != 2 || f.items[0].kind != Json::Number || f.items[1].kind != Json::Number)
          return fail("%s: data_offsets is not [begin, end]", name.c_str());
        t.begin = f.items[0].number;
        t.end = f.items[1].number;
        has_offsets = true;
      } else {
        return fail("%s: unexpected or mistyped field \"%s\"", name.c_str(), k.c_str());
      }
    }
    if (!t.dtype || !has_shape || !has_offsets) return fail("%s: needs dtype, shape and data_offsets", name.c_str());
    s.tensors[name] = std::move(t);
  }
  // check_tiling (safetensors.rs:1762-1800).
  std::vector<std::tuple<uint64_t, uint64_t, const std::string*>> ranges;
  for (auto& kv : s.tensors) {
    const TensorEntry& t = kv.second;
    if (t.begin > t.end || t.end > s.data_len)
      return fail("%s: data_offsets [%" PRIu64 ", %" PRIu64 "] outside the %" PRIu64 "-byte data buffer",
                  kv.first.c_str(), t.begin, t.end, s.data_len);
    uint64_t want = 0;
    if (byte_len(kv.first, t.shape, *t.dtype, &want) != OIO_OK) return OIO_ERROR;
    if (t.end - t.begin != want)
      return fail("%s: %" PRIu64 " bytes in data_offsets, but its shape and dtype %s give %" PRIu64, kv.first.c_str(),
                  t.end - t.begin, t.dtype->tag, want);
    ranges.emplace_back(t.begin, t.end, &kv.first);
  }
  std::sort(ranges.begin(), ranges.end(), [](const auto& a, const auto& b) {
    if (std::get<0>(a) != std::get<0>(b)) return std::get<0>(a) < std::get<0>(b);
    if (std::get<1>(a) != std::get<1>(b)) return std::get<1>(a) < std::get<1>(b);
    return *std::get<2>(a) < *std::get<2>(b);
  });
  uint64_t at = 0;
  for (auto& rg : ranges) {
    if (std::get<0>(rg) != at)
      return fail("%s: starts at byte %" PRIu64 ", expected %" PRIu64
                  " (gap or overlap; tensors must tile the data buffer)",
                  std::get<2>(rg)->c_str(), std::get<0>(rg), at);
    at = std::get<1>(rg);
  }
  if (at != s.data_len)
    return fail("the tensors cover %" PRIu64 " of %" PRIu64 " data bytes; the rest is an unindexed gap", at, s.data_len);
  for (auto& kv : s.tensors) s.order.push_back(&kv.first);
  for (auto& kv : s.metadata) s.meta_order.push_back(&kv.first);
  return OIO_OK;
}

const TensorEntry* find_tensor(const oio_safetensors* s, const char* name) {
  if (!s || !name) {
    fail("safetensors: null argument");
    return nullptr;
  }
  auto it = s->tensors.find(name);
  if (it == s->tensors.end()) {
    fail("no tensor named \"%s\"", name);
    return nullptr;
  }
  return &it->second;
}

// ---- checkpoint helpers ----
uint32_t ckpt_dtype_size(uint32_t tag) { return tag == 0 || tag == 3 ? 4 : 2; }

int32_t blob_window_ok(const oio_blob& b) {  // window_ok, checkpoint.rs:236-270
  unsigned __int128 n = 1;
  bool zero = false;
  for (uint32_t i = 0; i < b.rank; ++i) zero |= b.shape[i] == 0;
  if (zero) n = 0;
  else
    for (uint32_t i = 0; i < b.rank; ++i) {
      n *= b.shape[i];
      if (n > UINT64_MAX) return fail("\"%s\": shape product overflows", b.name);
    }
  const unsigned __int128 nbytes = n * ckpt_dtype_size(b.dtype_tag);
  if (nbytes > UINT64_MAX) return fail("\"%s\": byte size overflows", b.name);
  const unsigned __int128 end = static_cast<unsigned __int128>(b.byte_offset) + nbytes;
  if (end > UINT64_MAX) return fail("\"%s\": byte_offset window overflows", b.name);
  if (end > b.payload_len)
    return fail("\"%s\": byte_offset %" PRIu64 " plus %" PRIu64 " bytes exceeds payload %" PRIu64, b.name,
                b.byte_offset, static_cast<uint64_t>(nbytes), b.payload_len);
  return OIO_OK;
}

const char* const kSectionNames[4] = {"weights", "muon_momentum", "adamw_first_moment", "adamw_second_moment"};

int32_t validate_checkpoint(const oio_checkpoint* c, uint64_t* len) {
  if (!c) return fail("checkpoint: null argument");
  unsigned __int128 n = 12;
  n += 8 + static_cast<unsigned __int128>(c->config_len);
  n += 32 + 20 + 8 + 8 + 8;
  n += 8 + static_cast<unsigned __int128>(c->rng_state_len);
  for (int sct = 0; sct < 4; ++sct) {
    std::set<std::string> seen;
    n += 16;
    for (uint64_t i = 0; i < c->counts[sct]; ++i) {
      const oio_blob& b = c->sections[sct][i];
      if (!b.name) return fail("%s: record %" PRIu64 " has no name", kSectionNames[sct], i);
      if (b.dtype_tag > 3) return fail("\"%s\": unknown dtype tag %u", b.name, b.dtype_tag);
      if (!seen.insert(b.name).second) return fail("%s: duplicate key \"%s\"", kSectionNames[sct], b.name);
      if (blob_window_ok(b) != OIO_OK) return OIO_ERROR;
      n += 8 + strlen(b.name) + 4 + 4 + 8ull * b.rank + 8 + 8 + static_cast<unsigned __int128>(b.payload_len);
    }
  }
  if (n > OIO_MAX_CHECKPOINT_BYTES)
    return fail("checkpoint of %" PRIu64 " bytes exceeds cap %" PRIu64, static_cast<uint64_t>(n > UINT64_MAX ? UINT64_MAX : n),
                static_cast<uint64_t>(OIO_MAX_CHECKPOINT_BYTES));
  *len = static_cast<uint64_t>(n);
  return OIO_OK;
}

void put_u64(std::vector<uint8_t>& out, uint64_t v) {
  for (int i = 0; i < 8; ++i) out.push_back(static_cast<uint8_t>(v >> (8 * i)));
}
void put_u32(std::vector<uint8_t>& out, uint32_t v) {
  for (int i = 0; i < 4; ++i) out.push_back(static_cast<uint8_t>(v >> (8 * i)));
}
void put_bytes(std::vector<uint8_t>& out, const void* p, uint64_t n) {
  const uint8_t* b = static_cast<const uint8_t*>(p);
  out.insert(out.end(), b, b + n);
}

struct Cursor {
  const uint8_t* p;
  uint64_t left;
  bool take(uint64_t n, const uint8_t** out) {
    if (n > left) return false;
    *out = p;
    p += n;
    left -= n;
    return true;
  }
  bool u64(uint64_t* v) {
    const uint8_t* b;
    if (!take(8, &b)) return false;
    *v = 0;
    for (int i = 0; i < 8; ++i) *v |= static_cast<uint64_t>(b[i]) << (8 * i);
    return true;
  }
  bool u32(uint32_t* v) {
    const uint8_t* b;
    if (!take(4, &b)) return false;
    *v = 0;
    for (int i = 0; i < 4; ++i) *v |= static_cast<uint32_t>(b[i]) << (8 * i);
    return true;
  }
};

}  // namespace

extern "C" {

size_t oio_last_error(char* buf, size_t cap) {
  if (buf && cap) {
    const size_t n = g_error.size() < cap - 1 ? g_error.size() : cap - 1;
    memcpy(buf, g_error.data(), n);
    buf[n] = 0;
  }
  return g_error.size();
}

int32_t oio_st_open(const char* path, oio_safetensors** out) {
  if (!path || !out) return fail("safetensors: null argument");
  *out = nullptr;
  const int fd = open(path, O_RDONLY | O_CLOEXEC | O_NONBLOCK);
  if (fd < 0) return fail("%s: %s", path, strerror(errno));
  struct stat st;
  if (fstat(fd, &st) != 0 || !S_ISREG(st.st_mode)) {
    close(fd);
    return fail("%s: not a regular file", path);
  }
  std::unique_ptr<oio_safetensors> s(new (std::nothrow) oio_safetensors);
  if (!s) {
    close(fd);
    return fail("%s: allocation refused", path);
  }
  s->fd = fd;
  s->file_len = static_cast<uint64_t>(st.st_size);
  auto bail = [&](int32_t) {
    const std::string inner = g_error;
    close(fd);
    s->fd = -1;
    return fail("%s: %s", path, inner.c_str());
  };
  unsigned char len8[8];
  if (s->file_len < 8 || !read_exact_at(fd, len8, 8, 0)) return bail(fail("truncated file: header length"));
  uint64_t n = 0;
  for (int i = 0; i < 8; ++i) n |= static_cast<uint64_t>(len8[i]) << (8 * i);
  if (n == 0 || n > OIO_MAX_HEADER_BYTES)
    return bail(fail("header length %" PRIu64 " outside 1..=%" PRIu64, n, static_cast<uint64_t>(OIO_MAX_HEADER_BYTES)));
  if (n > s->file_len - 8)
    return bail(fail("header length %" PRIu64 " runs past the end of a %" PRIu64 "-byte file", n, s->file_len));
  std::vector<unsigned char> header;
  try {
    header.resize(n);
  } catch (const std::bad_alloc&) {
    return bail(fail("allocation of the %" PRIu64 "-byte header refused", n));
  }
  if (!read_exact_at(fd, header.data(), n, 8)) return bail(fail("truncated file: header runs past the end"));
  s->data_start = 8 + n;
  s->data_len = s->file_len - s->data_start;
  if (parse_header(*s, header) != OIO_OK) return bail(OIO_ERROR);
  *out = s.release();
  return OIO_OK;
}

void oio_st_close(oio_safetensors* s) {
  if (!s) return;
  if (s->fd >= 0) close(s->fd);
  delete s;
}

uint64_t oio_st_count(const oio_safetensors* s) { return s ? s->order.size() : 0; }
const char* oio_st_name(const oio_safetensors* s, uint64_t index) {
  return s && index < s->order.size() ? s->order[index]->c_str() : nullptr;
}

int32_t oio_st_info(const oio_safetensors* s, const char* name, const char** dtype, uint32_t* rank, uint64_t* shape,
                    uint32_t shape_cap, uint64_t* nbytes) {
  const TensorEntry* t = find_tensor(s, name);
  if (!t) return OIO_ERROR;
  if (dtype) *dtype = t->dtype->tag;
  if (rank) *rank = static_cast<uint32_t>(t->shape.size());
  if (shape)
    for (uint32_t i = 0; i < shape_cap && i < t->shape.size(); ++i) shape[i] = t->shape[i];
  if (nbytes) *nbytes = t->end - t->begin;
  return OIO_OK;
}

int32_t oio_st_read(const oio_safetensors* s, const char* name, uint64_t offset, void* dst, uint64_t n) {
  const TensorEntry* t = find_tensor(s, name);
  if (!t) return OIO_ERROR;
  const uint64_t len = t->end - t->begin;
  if (offset > len || n > len - offset)
    return fail("%s: bytes [%" PRIu64 ", +%" PRIu64 ") outside its %" PRIu64 " bytes", name, offset, n, len);
  if (n == 0) return OIO_OK;
  if (!dst) return fail("%s: null destination", name);
  struct stat st;  // a read refuses a file that changed since it was opened (safetensors.rs:2237)
  if (fstat(s->fd, &st) != 0 || static_cast<uint64_t>(st.st_size) != s->file_len)
    return fail("%s: the file changed since it was opened", name);
  if (!read_exact_at(s->fd, dst, n, s->data_start + t->begin + offset))
    return fail("%s: read: %s", name, errno ? strerror(errno) : "short file");
  return OIO_OK;
}

int32_t oio_st_read_f32(const oio_safetensors* s, const char* name, float* dst, uint64_t numel) {
  const TensorEntry* t = find_tensor(s, name);
  if (!t) return OIO_ERROR;
  const std::string tag = t->dtype->tag;
  const uint64_t esz = tag == "F32" ? 4 : (tag == "BF16" || tag == "F16") ? 2 : 0;
  if (esz == 0) return fail("%s: dtype %s is not F32, BF16 or F16", name, tag.c_str());
  if ((t->end - t->begin) / esz != numel)
    return fail("%s: holds %" PRIu64 " elements, the caller asked for %" PRIu64, name, (t->end - t->begin) / esz, numel);
  if (numel == 0) return OIO_OK;
  if (esz == 4) return oio_st_read(s, name, 0, dst, numel * 4);
  // 16-bit values land in the upper half of the destination and are widened front to back.
  unsigned char* narrow = reinterpret_cast<unsigned char*>(dst) + 2 * numel;
  if (oio_st_read(s, name, 0, narrow, numel * 2) != OIO_OK) return OIO_ERROR;
  for (uint64_t i = 0; i < numel; ++i) {
    uint16_t h;
    memcpy(&h, narrow + 2 * i, 2);
    float f;
    if (esz == 2 && tag == "BF16") {
      const uint32_t bits = static_cast<uint32_t>(h) << 16;
      memcpy(&f, &bits, 4);
    } else {
      f = half_to_float(h);
    }
    memcpy(reinterpret_cast<unsigned char*>(dst) + 4 * i, &f, 4);
  }
  return OIO_OK;
}

uint64_t oio_st_metadata_count(const oio_safetensors* s) { return s ? s->meta_order.size() : 0; }
const char* oio_st_metadata_key(const oio_safetensors* s, uint64_t index) {
  return s && index < s->meta_order.size() ? s->meta_order[index]->c_str() : nullptr;
}
const char* oio_st_metadata(const oio_safetensors* s, const char* key) {
  if (!s || !key) return nullptr;
  auto it = s->metadata.find(key);
  return it == s->metadata.end() ? nullptr : it->second.c_str();
}

int32_t oio_st_write(const char* path, const oio_tensor_out* tensors, uint64_t count, const char* const* meta_keys,
                     const char* const* meta_values, uint64_t meta_count) {
  if (!path || (!tensors && count) || ((!meta_keys || !meta_values) && meta_count))
    return fail("safetensors: null argument");
  std::string header = "{";
  bool first = true;
  if (meta_count) {
    header += "\"__metadata__\":{";
    std::set<std::string> seen;
    for (uint64_t i = 0; i < meta_count; ++i) {
      if (!meta_keys[i] || !meta_values[i]) return fail("%s: null metadata entry", path);
      if (!seen.insert(meta_keys[i]).second) return fail("%s: duplicate metadata key \"%s\"", path, meta_keys[i]);
      if (i) header += ",";
      push_json_str(header, meta_keys[i]);
      header += ":";
      push_json_str(header, meta_values[i]);
    }
    header += "}";
    first = false;
  }
  std::set<std::string> names;
  uint64_t at = 0;
  std::vector<const void*> parts(2);
  std::vector<uint64_t> lens(2);
  for (uint64_t i = 0; i < count; ++i) {
    const oio_tensor_out& t = tensors[i];
    if (!t.name || !t.dtype) return fail("%s: tensor %" PRIu64 " has no name or dtype", path, i);
    const std::string name = t.name;
    if (name.empty()) return fail("%s: tensor name is empty", path);
    if (name == "__metadata__") return fail("%s: \"__metadata__\" is not a tensor name", path);
    if (!valid_utf8(reinterpret_cast<const unsigned char*>(name.data()), name.size()))
      return fail("%s: tensor name is not UTF-8", path);
    if (!names.insert(name).second) return fail("%s: duplicate tensor name \"%s\"", path, t.name);
    const DtypeRow* dt = find_dtype(t.dtype);
    if (!dt) return fail("%s: %s: unknown dtype \"%s\"", path, t.name, t.dtype);
    std::vector<uint64_t> shape(t.shape, t.shape + t.rank);
    uint64_t want = 0;
    if (byte_len(name, shape, *dt, &want) != OIO_OK) return OIO_ERROR;
    if (want != t.nbytes)
      return fail("%s: %s: %" PRIu64 " bytes given, its shape and dtype give %" PRIu64, path, t.name, t.nbytes, want);
    if (t.nbytes && !t.data) return fail("%s: %s: null data", path, t.name);
    if (!first) header += ",";
    first = false;
    push_json_str(header, name);
    header += ":{\"dtype\":\"";
    header += dt->tag;
    header += "\",\"shape\":[";
    for (uint32_t d = 0; d < t.rank; ++d) {
      if (d) header += ",";
      header += std::to_string(t.shape[d]);
    }
    header += "],\"data_offsets\":[" + std::to_string(at) + "," + std::to_string(at + t.nbytes) + "]}";
    at += t.nbytes;
    parts.push_back(t.data);
    lens.push_back(t.nbytes);
  }
  header += "}";
  while (header.size() % 8 != 0) header.push_back(' ');
  if (header.size() > OIO_MAX_HEADER_BYTES) return fail("%s: header of %zu bytes exceeds the cap", path, header.size());
  uint8_t len8[8];
  for (int i = 0; i < 8; ++i) len8[i] = static_cast<uint8_t>(static_cast<uint64_t>(header.size()) >> (8 * i));
  parts[0] = len8;
  lens[0] = 8;
  parts[1] = header.data();
  lens[1] = header.size();
  return replace_file(path, parts, lens);
}

int32_t oio_ckpt_file_len(const oio_checkpoint* c, uint64_t* len) {
  if (!len) return fail("checkpoint: null argument");
  return validate_checkpoint(c, len);
}

int32_t oio_ckpt_write(const char* path, const oio_checkpoint* c) {
  if (!path) return fail("checkpoint: null argument");
  uint64_t total = 0;
  if (validate_checkpoint(c, &total) != OIO_OK) return OIO_ERROR;
  if ((c->config_len && !c->config) || (c->rng_state_len && !c->rng_state)) return fail("checkpoint: null blob");
  std::vector<uint8_t> out;
  try {
    out.reserve(total);
  } catch (const std::bad_alloc&) {
    return fail("%s: allocation of %" PRIu64 " bytes refused", path, total);
  }
  put_bytes(out, "OJAS0001", 8);
  put_u32(out, 1);
  put_u64(out, c->config_len);
  put_bytes(out, c->config, c->config_len);
  put_bytes(out, c->tokenizer_hash, 32);
  put_bytes(out, c->git_sha, 20);
  put_u64(out, c->step);
  put_u64(out, c->cursor_shard);
  put_u64(out, c->cursor_token_index);
  put_u64(out, c->rng_state_len);
  put_bytes(out, c->rng_state, c->rng_state_len);
  for (int sct = 0; sct < 4; ++sct) {
    uint64_t body = 8;
    for (uint64_t i = 0; i < c->counts[sct]; ++i) {
      const oio_blob& b = c->sections[sct][i];
      body += 8 + strlen(b.name) + 4 + 4 + 8ull * b.rank + 8 + 8 + b.payload_len;
    }
    put_u64(out, body);
    put_u64(out, c->counts[sct]);
    for (uint64_t i = 0; i < c->counts[sct]; ++i) {
      const oio_blob& b = c->sections[sct][i];
      put_u64(out, strlen(b.name));
      put_bytes(out, b.name, strlen(b.name));
      put_u32(out, b.dtype_tag);
      put_u32(out, b.rank);
      for (uint32_t d = 0; d < b.rank; ++d) put_u64(out, b.shape[d]);
      put_u64(out, b.byte_offset);
      put_u64(out, b.payload_len);
      put_bytes(out, b.payload, b.payload_len);
    }
  }
  if (out.size() != total) return fail("%s: encoded %zu bytes, expected %" PRIu64, path, out.size(), total);
  return replace_file(path, {out.data()}, {static_cast<uint64_t>(out.size())});
}

int32_t oio_ckpt_read(const char* path, oio_ckpt** out, oio_checkpoint* view) {
  if (!path || !out || !view) return fail("checkpoint: null argument");
  *out = nullptr;
  const int fd = open(path, O_RDONLY | O_CLOEXEC | O_NONBLOCK);
  if (fd < 0) return fail("%s: %s", path, strerror(errno));
  struct stat st;
  if (fstat(fd, &st) != 0 || !S_ISREG(st.st_mode)) {
    close(fd);
    return fail("%s: not a regular file", path);
  }
  const uint64_t len = static_cast<uint64_t>(st.st_size);
  if (len > OIO_MAX_CHECKPOINT_BYTES) {
    close(fd);
    return fail("%s: %" PRIu64 " bytes exceeds checkpoint cap %" PRIu64, path, len,
                static_cast<uint64_t>(OIO_MAX_CHECKPOINT_BYTES));
  }
  std::unique_ptr<oio_ckpt> c(new (std::nothrow) oio_ckpt);
  bool ok = static_cast<bool>(c);
  if (ok) {
    try {
      c->bytes.resize(len);
    } catch (const std::bad_alloc&) {
      ok = false;
    }
  }
  if (ok && len) ok = read_exact_at(fd, c->bytes.data(), len, 0);
  close(fd);
  if (!ok) return fail("%s: read failed", path);
  Cursor cur{c->bytes.data(), len};
  const uint8_t* b = nullptr;
  // read_prefix (ojas-core/src/checkpoint.rs:31-50)
  if (!cur.take(12, &b)) return fail("%s: read_prefix: truncated prefix", path);
  if (memcmp(b, "OJAS0001", 8) != 0) return fail("%s: read_prefix: bad magic", path);
  uint32_t version = 0;
  for (int i = 0; i < 4; ++i) version |= static_cast<uint32_t>(b[8 + i]) << (8 * i);
  if (version != 1) return fail("%s: read_prefix: version %u, expected 1", path, version);
  auto truncated = [&]() { return fail("%s: truncated checkpoint", path); };
  memset(view, 0, sizeof *view);
  uint64_t n = 0;
  if (!cur.u64(&n) || !cur.take(n, &b)) return truncated();
  view->config = b;
  view->config_len = n;
  if (!cur.take(32, &b)) return truncated();
  memcpy(view->tokenizer_hash, b, 32);
  if (!cur.take(20, &b)) return truncated();
  memcpy(view->git_sha, b, 20);
  if (!cur.u64(&view->step) || !cur.u64(&view->cursor_shard) || !cur.u64(&view->cursor_token_index)) return truncated();
  if (!cur.u64(&n) || !cur.take(n, &b)) return truncated();
  view->rng_state = b;
  view->rng_state_len = n;
  // Records are parsed into temporaries first: names and shapes must not move once blobs point at them.
  struct Rec {
    std::string name;
    std::vector<uint64_t> shape;
    oio_blob blob;
  };
  std::vector<Rec> recs[4];
  for (int sct = 0; sct < 4; ++sct) {
    uint64_t body = 0, count = 0;
    if (!cur.u64(&body)) return truncated();
    if (body > cur.left) return truncated();
    Cursor sec{cur.p, body};
    cur.p += body;
    cur.left -= body;
    if (!sec.u64(&count)) return fail("%s: %s: section shorter than its record count", path, kSectionNames[sct]);
    if (count > sec.left / 32)  // MIN_RECORD_BYTES, checkpoint.rs:331
      return fail("%s: %s: %" PRIu64 " records cannot fit the section", path, kSectionNames[sct], count);
    std::set<std::string> seen;
    for (uint64_t i = 0; i < count; ++i) {
      Rec r;
      uint64_t name_len = 0;
      if (!sec.u64(&name_len) || !sec.take(name_len, &b)) return truncated();
      if (!valid_utf8(b, name_len)) return fail("%s: %s: record name is not UTF-8", path, kSectionNames[sct]);
      r.name.assign(reinterpret_cast<const char*>(b), name_len);
      if (r.name.find('\0') != std::string::npos) return fail("%s: %s: record name holds a NUL", path, kSectionNames[sct]);
      uint32_t tag = 0, rank = 0;
      if (!sec.u32(&tag) || !sec.u32(&rank)) return truncated();
      if (tag > 3) return fail("%s: \"%s\": unknown dtype tag %u", path, r.name.c_str(), tag);
      if (rank > sec.left / 8) return fail("%s: \"%s\": rank %u cannot fit the section", path, r.name.c_str(), rank);
      r.shape.resize(rank);
      for (uint32_t d = 0; d < rank; ++d)
        if (!sec.u64(&r.shape[d])) return truncated();
      uint64_t off = 0, plen = 0;
      if (!sec.u64(&off) || !sec.u64(&plen) || !sec.take(plen, &b)) return truncated();
      if (!seen.insert(r.name).second) return fail("%s: %s: duplicate key \"%s\"", path, kSectionNames[sct], r.name.c_str());
      r.blob = oio_blob{nullptr, tag, rank, nullptr, off, b, plen};
      recs[sct].push_back(std::move(r));
    }
    if (sec.left != 0) return fail("%s: %s: section length disagrees with its records", path, kSectionNames[sct]);
  }
  if (cur.left != 0) return fail("%s: trailing bytes after checkpoint", path);
  size_t total = 0;
  for (auto& v : recs) total += v.size();
  c->names.reserve(total);
  c->shapes.reserve(total);
  for (int sct = 0; sct < 4; ++sct) {
    for (Rec& r : recs[sct]) {
      c->names.push_back(std::move(r.name));
      c->shapes.push_back(std::move(r.shape));
      oio_blob bl = r.blob;
      bl.name = c->names.back().c_str();
      bl.shape = c->shapes.back().data();
      if (blob_window_ok(bl) != OIO_OK) {
        const std::string inner = g_error;
        return fail("%s: %s", path, inner.c_str());
      }
      c->blobs[sct].push_back(bl);
    }
    view->sections[sct] = c->blobs[sct].data();
    view->counts[sct] = c->blobs[sct].size();
  }
  *out = c.release();
  return OIO_OK;
}

void oio_ckpt_free(oio_ckpt* c) { delete c; }

}  // extern "C"
