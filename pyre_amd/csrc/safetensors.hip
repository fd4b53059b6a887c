// safetensors container reader for the MTP drafter's checkpoint (host code only).
// Follows St::open / raw / row / norm / vec of the reference, src/model/mtp.rs:24-50: an 8-byte little-endian header
// length, a JSON object {name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": ...}, then the data;
// every tensor must be BF16; the prefixes "mtp." and "layers.0." are trimmed from the names.
#include "common.h"
#include <errno.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <map>
#include <string>
#include <vector>

namespace {

struct StT { std::vector<uint64_t> shape; uint64_t a = 0, b = 0; std::string dtype; };

// A small JSON reader: enough for the header (objects, arrays, strings with escapes, numbers, true / false / null).
struct Js {
  const char* p; const char* e; bool ok = true;
  void ws() { while (p < e && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
  bool eat(char c) { ws(); if (p < e && *p == c) { ++p; return true; } return false; }
  std::string str() {
    std::string s; ws(); if (p >= e || *p != '"') { ok = false; return s; } ++p;
    while (p < e && *p != '"') {
      if (*p == '\\') { if (++p >= e) break;
        switch (*p) { case 'n': s += '\n'; break; case 't': s += '\t'; break; case 'r': s += '\r'; break; case 'b': s += '\b'; break; case 'f': s += '\f'; break;
          case 'u': { unsigned v = 0; for (int i = 0; i < 4 && p + 1 < e; ++i) { ++p; const char c = *p; v = v * 16 + (c >= '0' && c <= '9' ? c - '0' : (c | 32) >= 'a' && (c | 32) <= 'f' ? (c | 32) - 'a' + 10 : 0); }
                      if (v < 0x80) s += (char)v; else if (v < 0x800) { s += (char)(0xC0 | (v >> 6)); s += (char)(0x80 | (v & 63)); } else { s += (char)(0xE0 | (v >> 12)); s += (char)(0x80 | ((v >> 6) & 63)); s += (char)(0x80 | (v & 63)); } } break;
          default: s += *p; }
        ++p;
      } else s += *p++;
    }
    if (p >= e) { ok = false; return s; } ++p; return s;
  }
  bool num(uint64_t* o) { ws(); const char* q = p; uint64_t v = 0; while (p < e && *p >= '0' && *p <= '9') { v = v * 10 + (uint64_t)(*p - '0'); ++p; } if (p == q) { ok = false; return false; } *o = v; return true; }
  void skip(int depth = 0) {            // any value
    ws(); if (p >= e || depth > 16) { ok = false; return; }
    if (*p == '"') { (void)str(); return; }
    if (*p == '{') { ++p; if (eat('}')) return; do { (void)str(); if (!eat(':')) { ok = false; return; } skip(depth + 1); } while (ok && eat(',')); if (!eat('}')) ok = false; return; }
    if (*p == '[') { ++p; if (eat(']')) return; do skip(depth + 1); while (ok && eat(',')); if (!eat(']')) ok = false; return; }
    while (p < e && *p != ',' && *p != '}' && *p != ']' && *p != ' ' && *p != '\n') ++p;            // number, true, false, null
  }
  bool arr(std::vector<uint64_t>* o) { o->clear(); if (!eat('[')) { ok = false; return false; } if (eat(']')) return true; do { uint64_t v; if (!num(&v)) return false; o->push_back(v); } while (eat(',')); if (!eat(']')) { ok = false; return false; } return true; }
};

std::string trim_prefixes(const std::string& k) {            // mtp.rs:37: trim_start_matches("mtp.") then ("layers.0."), each repeatedly
  std::string s = k;
  while (s.rfind("mtp.", 0) == 0) s.erase(0, 4);
  while (s.rfind("layers.0.", 0) == 0) s.erase(0, 9);
  return s;
}

}  // namespace

struct pyre_st { void* map = nullptr; size_t n = 0, base = 0; std::map<std::string, StT> t; std::vector<std::string> names; };

static int st_err(char* err, size_t cap, int rc, const std::string& msg) { if (err && cap) snprintf(err, cap, "%s", msg.c_str()); return rc; }

extern "C" {

void pyre_st_close(pyre_st* s) { if (!s) return; if (s->map) munmap(s->map, s->n); delete s; }

int pyre_st_open(const char* path, pyre_st** out, char* err, size_t err_cap) {
  if (!path || !out) return st_err(err, err_cap, PYRE_E_ARG, "pyre_st_open: null argument");
  *out = nullptr;
  const int fd = open(path, O_RDONLY);
  if (fd < 0) return st_err(err, err_cap, PYRE_E_ARG, std::string("open ") + path + ": " + strerror(errno));
  struct stat sb; if (fstat(fd, &sb) != 0 || sb.st_size < 8) { close(fd); return st_err(err, err_cap, PYRE_E_ARG, std::string(path) + ": shorter than a safetensors header"); }
  void* mp = mmap(nullptr, (size_t)sb.st_size, PROT_READ, MAP_PRIVATE, fd, 0); close(fd);
  if (mp == MAP_FAILED) return st_err(err, err_cap, PYRE_E_ARG, std::string("mmap ") + path + ": " + strerror(errno));
  pyre_st* s = new pyre_st(); s->map = mp; s->n = (size_t)sb.st_size;
  auto fail = [&](int rc, const std::string& m) { pyre_st_close(s); return st_err(err, err_cap, rc, std::string(path) + ": " + m); };
  uint64_t hn = 0; memcpy(&hn, mp, 8);
  if (hn > s->n - 8) return fail(PYRE_E_ARG, "header length beyond the file");
  s->base = 8 + (size_t)hn;
  Js j{(const char*)mp + 8, (const char*)mp + 8 + hn};
  if (!j.eat('{')) return fail(PYRE_E_ARG, "the header is not a JSON object");
  if (!j.eat('}')) {
    do {
      const std::string key = j.str(); if (!j.ok || !j.eat(':')) return fail(PYRE_E_ARG, "malformed header");
      if (key == "__metadata__") { j.skip(); if (!j.ok) return fail(PYRE_E_ARG, "malformed metadata"); continue; }
      StT t; bool have_off = false, have_shape = false;
      if (!j.eat('{')) return fail(PYRE_E_ARG, key + ": not an object");
      if (!j.eat('}')) {
        do {
          const std::string f = j.str(); if (!j.ok || !j.eat(':')) return fail(PYRE_E_ARG, key + ": malformed entry");
          if (f == "dtype") t.dtype = j.str();
          else if (f == "shape") have_shape = j.arr(&t.shape);
          else if (f == "data_offsets") { std::vector<uint64_t> o; if (j.arr(&o) && o.size() == 2) { t.a = o[0]; t.b = o[1]; have_off = true; } }
          else j.skip();
          if (!j.ok) return fail(PYRE_E_ARG, key + ": malformed entry");
        } while (j.eat(','));
        if (!j.eat('}')) return fail(PYRE_E_ARG, key + ": malformed entry");
      }
      if (t.dtype != "BF16") return fail(PYRE_E_TYPE, key + ": dtype " + t.dtype + " (the drafter's checkpoint is BF16)");            // mtp.rs:34
      if (!have_off || !have_shape) return fail(PYRE_E_ARG, key + ": shape or data_offsets missing");
      uint64_t cnt = 1; for (uint64_t d : t.shape) { if (d != 0 && cnt > UINT64_MAX / d) return fail(PYRE_E_ARG, key + ": shape overflows"); cnt *= d; }
      if (t.b < t.a || t.b > s->n - s->base || t.b - t.a != cnt * 2) return fail(PYRE_E_ARG, key + ": data_offsets do not match the shape or the file");
      const std::string nm = trim_prefixes(key);
      if (!s->t.emplace(nm, t).second) return fail(PYRE_E_ARG, nm + ": twice in the header");
      s->names.push_back(nm);
    } while (j.eat(','));
    if (!j.eat('}')) return fail(PYRE_E_ARG, "malformed header");
  }
  *out = s; return PYRE_OK;
}

size_t pyre_st_n_tensors(const pyre_st* s) { return s ? s->names.size() : 0; }
const char* pyre_st_tensor_name(const pyre_st* s, size_t i) { return (s && i < s->names.size()) ? s->names[i].c_str() : nullptr; }

int pyre_st_tensor(const pyre_st* s, const char* name, const void** data, uint32_t* n_dims, uint64_t* dims /*[8]*/, char* err, size_t err_cap) {
  if (!s || !name || !data) return st_err(err, err_cap, PYRE_E_ARG, "pyre_st_tensor: null argument");
  auto it = s->t.find(name);
  if (it == s->t.end()) return st_err(err, err_cap, PYRE_E_ARG, std::string("mtp tensor ") + name);            // mtp.rs:40
  if (it->second.shape.size() > 8) return st_err(err, err_cap, PYRE_E_SHAPE, std::string(name) + ": more than 8 dimensions");
  *data = (const uint8_t*)s->map + s->base + it->second.a;
  if (n_dims) *n_dims = (uint32_t)it->second.shape.size();
  if (dims) for (size_t i = 0; i < it->second.shape.size(); ++i) dims[i] = it->second.shape[i];
  return PYRE_OK;
}

}  // extern "C"
