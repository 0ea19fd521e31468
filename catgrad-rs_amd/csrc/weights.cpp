// weights.cpp — safetensors files -> Parameters, on top of the C ABI only (no backend internals),
// so the same source serves every backend that exports catgrad_hip.h.
//
// Restates the loading loop of catgrad-llm/examples/llama/main.rs:277-350 (open, mmap,
// SafeTensors::deserialize, one tensor per entry, F32 and BF16 only) and its post-processing
// concat_moe_experts (main.rs:171-262).  Differences, both on purpose: BF16 entries are handed to
// the backend as bf16 bits (cg_from_bf16) instead of being widened on the host, and the experts of
// a layer are stacked with one allocation (cg_stack) instead of a chain of concatenations.
//
// File format (safetensors): u64 little-endian header length N, N bytes of JSON
//   { "<name>": {"dtype": "F32", "shape": [..], "data_offsets": [begin, end]}, ..., "__metadata__": {..} }
// then the data; offsets are relative to the first byte after the header.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/catgrad_hip.h"

namespace {

thread_local std::string g_werr;

int werr(int code, const std::string &msg) {
  g_werr = msg;
  return code;
}

struct Entry {
  std::string name, dtype_name;
  cg_weight_dtype dtype = CG_WDT_OTHER;
  int rank = 0;
  size_t dims[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  uint64_t begin = 0, end = 0;
};

// ---- a JSON reader for exactly what a safetensors header may hold ------------------------------
struct Json {
  const char *p, *end;
  std::string err;

  bool fail(const std::string &m) {
    if (err.empty()) err = m + " at header byte " + std::to_string((size_t)(p - start));
    return false;
  }
  const char *start;
  Json(const char *b, const char *e) : p(b), end(e), start(b) {}

  void ws() {
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
  }
  bool lit(char c) {
    ws();
    if (p < end && *p == c) {
      ++p;
      return true;
    }
    return false;
  }
  bool expect(char c) { return lit(c) || fail(std::string("expected '") + c + "'"); }

  static void utf8(std::string &out, uint32_t cp) {
    if (cp < 0x80) out += (char)cp;
    else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
    else if (cp < 0x10000) {
      out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F));
    } else {
      out += (char)(0xF0 | (cp >> 18)); out += (char)(0x80 | ((cp >> 12) & 0x3F));
      out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F));
    }
  }
  bool hex4(uint32_t *v) {
    if (end - p < 4) return fail("truncated \\u escape");
    uint32_t r = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = *p++;
      r <<= 4;
      if (c >= '0' && c <= '9') r |= (uint32_t)(c - '0');
      else if (c >= 'a' && c <= 'f') r |= (uint32_t)(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') r |= (uint32_t)(c - 'A' + 10);
      else return fail("bad \\u escape");
    }
    *v = r;
    return true;
  }
  bool string(std::string *out) {
    ws();
    if (p >= end || *p != '"') return fail("expected a string");
    ++p;
    out->clear();
    while (p < end && *p != '"') {
      char c = *p++;
      if (c != '\\') {
        *out += c;
        continue;
      }
      if (p >= end) return fail("truncated escape");
      c = *p++;
      switch (c) {
        case '"': *out += '"'; break;
        case '\\': *out += '\\'; break;
        case '/': *out += '/'; break;
        case 'b': *out += '\b'; break;
        case 'f': *out += '\f'; break;
        case 'n': *out += '\n'; break;
        case 'r': *out += '\r'; break;
        case 't': *out += '\t'; break;
        case 'u': {
          uint32_t cp = 0;
          if (!hex4(&cp)) return false;
          if (cp >= 0xD800 && cp < 0xDC00 && end - p >= 6 && p[0] == '\\' && p[1] == 'u') {
            p += 2;
            uint32_t lo = 0;
            if (!hex4(&lo)) return false;
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          }
          utf8(*out, cp);
          break;
        }
        default: return fail("bad escape");
      }
    }
    if (p >= end) return fail("unterminated string");
    ++p;
    return true;
  }
  bool uint(uint64_t *v) {
    ws();
    if (p >= end || *p < '0' || *p > '9') return fail("expected a non-negative integer");
    uint64_t r = 0;
    while (p < end && *p >= '0' && *p <= '9') {
      if (r > (UINT64_MAX - 9) / 10) return fail("integer too large");
      r = r * 10 + (uint64_t)(*p++ - '0');
    }
    if (p < end && (*p == '.' || *p == 'e' || *p == 'E')) return fail("expected an integer");
    *v = r;
    return true;
  }
  // any value, skipped (the contents of "__metadata__")
  bool skip(int depth = 0) {
    if (depth > 64) return fail("nesting too deep");
    ws();
    if (p >= end) return fail("truncated value");
    if (*p == '"') {
      std::string s;
      return string(&s);
    }
    if (*p == '{' || *p == '[') {
      const char close = *p == '{' ? '}' : ']';
      const bool obj = *p == '{';
      ++p;
      if (lit(close)) return true;
      do {
        if (obj) {
          std::string k;
          if (!string(&k) || !expect(':')) return false;
        }
        if (!skip(depth + 1)) return false;
      } while (lit(','));
      return expect(close);
    }
    const char *b = p;  // number, true, false, null
    while (p < end && *p != ',' && *p != '}' && *p != ']' && *p != ' ' && *p != '\n' && *p != '\t' && *p != '\r') ++p;
    return p > b || fail("expected a value");
  }
};

size_t dtype_size(const std::string &d) {
  if (d == "F64" || d == "I64" || d == "U64") return 8;
  if (d == "F32" || d == "I32" || d == "U32") return 4;
  if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
  if (d == "I8" || d == "U8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
  return 0;
}

bool parse_entry(Json &j, Entry *e) {
  if (!j.expect('{')) return false;
  bool have_dtype = false, have_shape = false, have_off = false;
  if (!j.lit('}')) {
    do {
      std::string key;
      if (!j.string(&key) || !j.expect(':')) return false;
      if (key == "dtype") {
        if (!j.string(&e->dtype_name)) return false;
        have_dtype = true;
      } else if (key == "shape") {
        if (!j.expect('[')) return false;
        e->rank = 0;
        if (!j.lit(']')) {
          do {
            uint64_t d = 0;
            if (!j.uint(&d)) return false;
            if (e->rank >= 8) return j.fail("more than 8 dimensions");
            e->dims[e->rank++] = (size_t)d;
          } while (j.lit(','));
          if (!j.expect(']')) return false;
        }
        have_shape = true;
      } else if (key == "data_offsets") {
        if (!j.expect('[') || !j.uint(&e->begin) || !j.expect(',') || !j.uint(&e->end) || !j.expect(']')) return false;
        have_off = true;
      } else if (!j.skip()) {
        return false;
      }
    } while (j.lit(','));
    if (!j.expect('}')) return false;
  }
  if (!have_dtype || !have_shape || !have_off) return j.fail("tensor entry lacks dtype, shape or data_offsets");
  e->dtype = e->dtype_name == "F32" ? CG_WDT_F32 : e->dtype_name == "BF16" ? CG_WDT_BF16 : CG_WDT_OTHER;
  return true;
}

}  // namespace

struct cg_weights {
  int fd = -1;
  const uint8_t *map = nullptr;
  size_t map_len = 0;
  uint64_t data_start = 0;
  std::vector<Entry> entries;
  ~cg_weights() {
    if (map) munmap(const_cast<uint8_t *>(map), map_len);
    if (fd >= 0) close(fd);
  }
};

extern "C" {

const char *cg_weights_last_error(void) { return g_werr.c_str(); }

int cg_weights_open(const char *path, cg_weights **out) {
  if (!path || !out) return werr(CG_ERR_ARG, "null argument");
  *out = nullptr;
  cg_weights *w = new cg_weights();
  auto bail = [&](int code, const std::string &m) {
    delete w;
    return werr(code, std::string(path) + ": " + m);
  };
  w->fd = open(path, O_RDONLY | O_CLOEXEC);
  if (w->fd < 0) return bail(CG_ERR_IO, std::string("open: ") + std::strerror(errno));
  struct stat sb;
  if (fstat(w->fd, &sb) != 0) return bail(CG_ERR_IO, std::string("fstat: ") + std::strerror(errno));
  if (sb.st_size < 8) return bail(CG_ERR_FORMAT, "shorter than the 8-byte header length");
  w->map_len = (size_t)sb.st_size;
  void *m = mmap(nullptr, w->map_len, PROT_READ, MAP_PRIVATE, w->fd, 0);
  if (m == MAP_FAILED) {
    w->map_len = 0;
    return bail(CG_ERR_IO, std::string("mmap: ") + std::strerror(errno));
  }
  w->map = (const uint8_t *)m;
  uint64_t hlen = 0;
  for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | w->map[i];
  if (hlen > (uint64_t)100 << 20) return bail(CG_ERR_FORMAT, "header longer than 100 MiB");
  if (hlen > w->map_len - 8) return bail(CG_ERR_FORMAT, "header length exceeds the file");
  w->data_start = 8 + hlen;
  const uint64_t data_len = w->map_len - w->data_start;
  Json j((const char *)w->map + 8, (const char *)w->map + 8 + hlen);
  if (!j.expect('{')) return bail(CG_ERR_FORMAT, j.err);
  if (!j.lit('}')) {
    do {
      std::string name;
      if (!j.string(&name) || !j.expect(':')) return bail(CG_ERR_FORMAT, j.err);
      if (name == "__metadata__") {
        if (!j.skip()) return bail(CG_ERR_FORMAT, j.err);
        continue;
      }
      Entry e;
      e.name = name;
      if (!parse_entry(j, &e)) return bail(CG_ERR_FORMAT, j.err);
      if (e.begin > e.end || e.end > data_len) return bail(CG_ERR_FORMAT, "'" + name + "': data_offsets outside the file");
      const size_t es = dtype_size(e.dtype_name);
      if (!es) return bail(CG_ERR_FORMAT, "'" + name + "': unknown dtype " + e.dtype_name);
      uint64_t count = 1;
      for (int d = 0; d < e.rank; ++d) {
        if (e.dims[d] && count > UINT64_MAX / e.dims[d]) return bail(CG_ERR_FORMAT, "'" + name + "': shape overflows");
        count *= e.dims[d];
      }
      if (count > UINT64_MAX / es || count * es != e.end - e.begin)
        return bail(CG_ERR_FORMAT, "'" + name + "': data_offsets do not match shape and dtype");
      w->entries.push_back(std::move(e));
    } while (j.lit(','));
    if (!j.expect('}')) return bail(CG_ERR_FORMAT, j.err);
  }
  j.ws();
  if (j.p != j.end) return bail(CG_ERR_FORMAT, "text after the header object");
  *out = w;
  return CG_OK;
}

void cg_weights_close(cg_weights *w) { delete w; }
size_t cg_weights_count(const cg_weights *w) { return w ? w->entries.size() : 0; }
const char *cg_weights_name(const cg_weights *w, size_t i) {
  return (w && i < w->entries.size()) ? w->entries[i].name.c_str() : nullptr;
}

int cg_weights_info(const cg_weights *w, size_t i, cg_weight_dtype *dtype, const char **dtype_name, int *rank,
                    size_t *dims, uint64_t *nbytes) {
  if (!w || i >= w->entries.size()) return werr(CG_ERR_ARG, "no such tensor");
  const Entry &e = w->entries[i];
  if (dtype) *dtype = e.dtype;
  if (dtype_name) *dtype_name = e.dtype_name.c_str();
  if (rank) *rank = e.rank;
  if (dims)
    for (int d = 0; d < e.rank; ++d) dims[d] = e.dims[d];
  if (nbytes) *nbytes = e.end - e.begin;
  return CG_OK;
}

int cg_weights_tensor(cg_backend *be, const cg_weights *w, size_t i, cg_tensor **out) {
  if (!be || !w || !out || i >= w->entries.size()) return werr(CG_ERR_ARG, "null argument or no such tensor");
  const Entry &e = w->entries[i];
  const uint8_t *data = w->map + w->data_start + e.begin;
  int st;
  if (e.dtype == CG_WDT_F32) {
    // mapped data starts wherever the header ends: not necessarily 4-byte aligned
    const size_t n = (size_t)((e.end - e.begin) / 4);
    if ((uintptr_t)data % 4 == 0) {
      st = cg_from_f32(be, (const float *)data, n, e.dims, e.rank, out);
    } else {
      std::vector<float> tmp(n);
      std::memcpy(tmp.data(), data, n * 4);
      st = cg_from_f32(be, tmp.data(), n, e.dims, e.rank, out);
    }
  } else if (e.dtype == CG_WDT_BF16) {
    const size_t n = (size_t)((e.end - e.begin) / 2);
    if ((uintptr_t)data % 2 == 0) {
      st = cg_from_bf16(be, (const uint16_t *)data, n, e.dims, e.rank, out);
    } else {
      std::vector<uint16_t> tmp(n);
      std::memcpy(tmp.data(), data, n * 2);
      st = cg_from_bf16(be, tmp.data(), n, e.dims, e.rank, out);
    }
  } else {
    return werr(CG_ERR_DTYPE, "'" + e.name + "': Unsupported dtype: " + e.dtype_name);
  }
  if (st != CG_OK) return werr(st, "'" + e.name + "': " + cg_last_error(be));
  return CG_OK;
}

int cg_params_load(cg_backend *be, cg_params *params, const char *file, const char *prefix, size_t *n_loaded) {
  if (!be || !params || !file) return werr(CG_ERR_ARG, "null argument");
  if (n_loaded) *n_loaded = 0;
  cg_weights *w = nullptr;
  int st = cg_weights_open(file, &w);
  if (st != CG_OK) return st;
  const std::string pre = prefix ? prefix : "";
  for (size_t i = 0; i < w->entries.size(); ++i) {
    cg_tensor *t = nullptr;
    st = cg_weights_tensor(be, w, i, &t);
    if (st != CG_OK) break;
    st = cg_params_set(params, (pre + w->entries[i].name).c_str(), t);
    cg_tensor_release(t);
    if (st != CG_OK) {
      werr(st, "cg_params_set failed for '" + w->entries[i].name + "'");
      break;
    }
    if (n_loaded) ++*n_loaded;
  }
  cg_weights_close(w);
  return st;
}

int cg_params_stack_experts(cg_backend *be, cg_params *params, const char *prefix, size_t num_layers,
                            size_t num_experts) {
  if (!be || !params) return werr(CG_ERR_ARG, "null argument");
  if (num_experts == 0) return CG_OK;  // post_process_weights, main.rs:264-275
  const std::string pre = prefix ? prefix : "";
  static const char *const proj_names[3] = {"down_proj", "gate_proj", "up_proj"};
  for (size_t layer = 0; layer < num_layers; ++layer) {
    for (const char *proj : proj_names) {
      std::vector<cg_tensor *> parts;
      std::vector<std::string> keys;
      auto drop = [&]() {
        for (cg_tensor *t : parts) cg_tensor_release(t);
      };
      for (size_t e = 0; e < num_experts; ++e) {
        const std::string key = pre + "model.layers." + std::to_string(layer) + ".mlp.experts." + std::to_string(e) +
                                "." + proj + ".weight";
        cg_tensor *t = nullptr;
        if (cg_params_get(params, key.c_str(), &t) == CG_OK) {
          parts.push_back(t);
          keys.push_back(key);
        }
      }
      if (parts.empty()) continue;
      if (parts.size() != num_experts) {
        const size_t found = parts.size();
        drop();
        return werr(CG_ERR_LOAD, "Expected " + std::to_string(num_experts) + " experts for layer " +
                                     std::to_string(layer) + " " + proj + ", found " + std::to_string(found));
      }
      cg_tensor *stacked = nullptr;
      int st = cg_stack(be, parts.data(), parts.size(), &stacked);
      drop();
      if (st != CG_OK) return werr(st, std::string("stacking experts: ") + cg_last_error(be));
      const std::string new_key = pre + "model.layers." + std::to_string(layer) + ".mlp.experts." + proj + ".weight";
      st = cg_params_set(params, new_key.c_str(), stacked);
      cg_tensor_release(stacked);
      if (st != CG_OK) return werr(st, "cg_params_set failed for '" + new_key + "'");
      for (const std::string &k : keys) cg_params_remove(params, k.c_str());
    }
  }
  return CG_OK;
}

}  // extern "C"
