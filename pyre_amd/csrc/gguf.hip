// GGUF container reader and the qwen4exp model loader (host code only; nothing here touches the GPU until
// pyre_model_create is called with the tensors found).
// Follows Gguf::open / shard_paths / Meta (src/model/gguf_q.rs:250-336) and Model::load's metadata keys and tensor
// names (src/model/qwen4exp_gguf.rs:462-524).
#include "formats.h"
#include <algorithm>
#include <errno.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <memory>
#include <unordered_map>

namespace {

struct Meta {            // gguf_q.rs:251: U(u64) I(i64) F(f64) B(bool) S(String) A(Vec<Meta>)
  enum Kind { U, I, F, B, S, A } kind = U;
  uint64_t u = 0; int64_t i = 0; double f = 0; std::string s; std::vector<Meta> a;
  bool as_u64(uint64_t* o) const { if (kind == U) { *o = u; return true; } if (kind == I) { *o = (uint64_t)i; return true; } if (kind == B) { *o = u; return true; } return false; }
  bool as_f64(double* o) const { if (kind == F) { *o = f; return true; } if (kind == U) { *o = (double)u; return true; } if (kind == I) { *o = (double)i; return true; } return false; }
};
struct TInfo { std::vector<uint64_t> shape; uint32_t ty = 0; size_t shard = 0, off = 0; };
struct Map { void* p = nullptr; size_t n = 0; };

struct Rd {
  const uint8_t* b; size_t n, p = 0; bool ok = true;
  const uint8_t* take(size_t k) { if (!ok || k > n - p) { ok = false; return nullptr; } const uint8_t* r = b + p; p += k; return r; }
  template <typename T> T le() { T v{}; const uint8_t* q = take(sizeof(T)); if (q) memcpy(&v, q, sizeof(T)); return v; }
  std::string str() { uint64_t k = le<uint64_t>(); if (!ok || k > n - p) { ok = false; return std::string(); } const uint8_t* q = take((size_t)k); return q ? std::string((const char*)q, (size_t)k) : std::string(); }
  Meta val(uint32_t t, int depth = 0) {
    Meta m;
    switch (t) {
      case 0: m.kind = Meta::U; m.u = le<uint8_t>(); break;
      case 1: m.kind = Meta::I; m.i = le<int8_t>(); break;
      case 2: m.kind = Meta::U; m.u = le<uint16_t>(); break;
      case 3: m.kind = Meta::I; m.i = le<int16_t>(); break;
      case 4: m.kind = Meta::U; m.u = le<uint32_t>(); break;
      case 5: m.kind = Meta::I; m.i = le<int32_t>(); break;
      case 6: { m.kind = Meta::F; float f = le<float>(); m.f = f; } break;
      case 7: m.kind = Meta::B; m.u = le<uint8_t>() != 0; break;
      case 8: m.kind = Meta::S; m.s = str(); break;
      case 9: {
        m.kind = Meta::A; uint32_t et = le<uint32_t>(); uint64_t cnt = le<uint64_t>();
        if (depth > 4 || cnt > n - p) { ok = false; break; }           // every element takes at least one byte
        m.a.reserve((size_t)cnt);
        for (uint64_t k = 0; k < cnt && ok; ++k) m.a.push_back(val(et, depth + 1));
      } break;
      case 10: m.kind = Meta::U; m.u = le<uint64_t>(); break;
      case 11: m.kind = Meta::I; m.i = le<int64_t>(); break;
      case 12: m.kind = Meta::F; m.f = le<double>(); break;
      default: ok = false;
    }
    return m;
  }
};

bool file_exists(const std::string& p) { struct stat st; return stat(p.c_str(), &st) == 0; }

// All shards of a split GGUF given any one of them (`-NNNNN-of-MMMMM.gguf`), or the single file (gguf_q.rs:282-295).
bool shard_paths(const std::string& path, std::vector<std::string>* out, std::string* err) {
  size_t slash = path.find_last_of('/'); std::string dir = slash == std::string::npos ? std::string() : path.substr(0, slash + 1);
  std::string name = slash == std::string::npos ? path : path.substr(slash + 1);
  size_t i = name.rfind("-of-");
  if (i != std::string::npos && i >= 6 && name.size() > 5 && name.compare(name.size() - 5, 5, ".gguf") == 0) {
    std::string cnt = name.substr(i + 4, name.size() - 5 - (i + 4)); char* end = nullptr; errno = 0;
    unsigned long total = strtoul(cnt.c_str(), &end, 10);
    if (cnt.empty() || *end || errno || total == 0 || total > 99999) { *err = "bad shard count in " + name; return false; }
    std::string stem = name.substr(0, i - 6);
    for (unsigned long k = 1; k <= total; ++k) {
      char buf[64]; snprintf(buf, sizeof(buf), "-%05lu-of-%05lu.gguf", k, total);
      std::string s = dir + stem + buf;
      if (!file_exists(s)) { *err = "missing shard " + s; return false; }
      out->push_back(s);
    }
    return true;
  }
  out->push_back(path); return true;
}

const char* ggml_name(uint32_t ty) {
  switch (ty) { case 0: return "F32"; case 1: return "F16"; case 2: return "Q4_0"; case 3: return "Q4_1"; case 6: return "Q5_0"; case 7: return "Q5_1"; case 8: return "Q8_0"; case 10: return "Q2_K";
    case 11: return "Q3_K"; case 12: return "Q4_K"; case 13: return "Q5_K"; case 14: return "Q6_K"; case 16: return "IQ2_XXS"; case 17: return "IQ2_XS"; case 18: return "IQ3_XXS"; case 19: return "IQ1_S";
    case 20: return "IQ4_NL"; case 21: return "IQ3_S"; case 22: return "IQ2_S"; case 23: return "IQ4_XS"; case 29: return "IQ1_M"; case 30: return "BF16"; case 42: return "Q2_0"; }
  return "unknown";
}
// block geometry of the types this library computes with (QType::geom, gguf_q.rs:33-42); false for the others
bool type_geom(uint32_t ty, size_t* el, size_t* bytes) {
  int e = 0, b = 0; if (!ggml_geom(ty, &e, &b)) return false;
  *el = (size_t)e; *bytes = (size_t)b; return true;
}

}  // namespace

struct pyre_gguf {
  std::vector<std::string> paths; std::vector<Map> maps;
  std::unordered_map<std::string, Meta> meta; std::unordered_map<std::string, TInfo> tensors; std::vector<std::string> order;
  ~pyre_gguf() { for (auto& m : maps) if (m.p) munmap(m.p, m.n); }
};

namespace {

void set_err(char* err, size_t cap, const std::string& s) { if (err && cap) { snprintf(err, cap, "%s", s.c_str()); } }

int gguf_open(const char* path, pyre_gguf** out, std::string* err) {
  std::unique_ptr<pyre_gguf> g(new pyre_gguf());
  if (!shard_paths(path, &g->paths, err)) return PYRE_E_ARG;
  for (size_t si = 0; si < g->paths.size(); ++si) {
    const std::string& p = g->paths[si];
    int fd = open(p.c_str(), O_RDONLY);
    if (fd < 0) { *err = "open " + p + ": " + strerror(errno); return PYRE_E_ARG; }
    struct stat st; if (fstat(fd, &st) != 0 || st.st_size < 24) { close(fd); *err = p + " is not GGUF (too short)"; return PYRE_E_ARG; }
    void* mp = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0); close(fd);
    if (mp == MAP_FAILED) { *err = "mmap " + p + ": " + strerror(errno); return PYRE_E_NOMEM; }
    g->maps.push_back(Map{mp, (size_t)st.st_size});
    Rd r{(const uint8_t*)mp, (size_t)st.st_size};
    const uint8_t* magic = r.take(4);
    if (!magic || memcmp(magic, "GGUF", 4) != 0) { *err = p + " is not GGUF"; return PYRE_E_ARG; }
    (void)r.le<uint32_t>(); uint64_t nt = r.le<uint64_t>(), nkv = r.le<uint64_t>();
    if (!r.ok || nt > r.n || nkv > r.n) { *err = "truncated GGUF " + p; return PYRE_E_ARG; }
    size_t align = 32;
    for (uint64_t k = 0; k < nkv; ++k) {
      std::string key = r.str(); uint32_t t = r.le<uint32_t>(); Meta v = r.val(t);
      if (!r.ok) { *err = "truncated GGUF or bad value type in " + p + " (key " + key + ")"; return PYRE_E_ARG; }
      if (key == "general.alignment") { uint64_t a = 32; if (v.as_u64(&a) && a > 0) align = (size_t)a; }
      if (si == 0 || !g->meta.count(key)) g->meta[key] = std::move(v);
    }
    struct Pending { std::string name; TInfo t; };
    std::vector<Pending> infos; infos.reserve((size_t)nt);
    for (uint64_t k = 0; k < nt; ++k) {
      Pending pe; pe.name = r.str(); uint32_t nd = r.le<uint32_t>();
      if (!r.ok || nd > 8) { *err = "truncated GGUF " + p; return PYRE_E_ARG; }
      for (uint32_t dd = 0; dd < nd; ++dd) pe.t.shape.push_back(r.le<uint64_t>());
      pe.t.ty = r.le<uint32_t>(); pe.t.off = (size_t)r.le<uint64_t>(); pe.t.shard = si;
      if (!r.ok) { *err = "truncated GGUF " + p; return PYRE_E_ARG; }
      infos.push_back(std::move(pe));
    }
    size_t data = (r.p + align - 1) / align * align;
    for (auto& pe : infos) { pe.t.off += data; if (!g->tensors.count(pe.name)) g->order.push_back(pe.name); g->tensors[pe.name] = std::move(pe.t); }
  }
  *out = g.release(); return PYRE_OK;
}

// Gguf::mat (gguf_q.rs:326-331): cols = shape[0], rows = product of the rest; the bytes must lie inside the shard
int gguf_mat(const pyre_gguf* g, const std::string& name, pyre_tensor* out, std::string* err) {
  auto it = g->tensors.find(name);
  if (it == g->tensors.end()) { *err = "missing tensor " + name; return PYRE_E_ARG; }
  const TInfo& t = it->second;
  if (t.shape.empty()) { *err = name + ": no dimensions"; return PYRE_E_SHAPE; }
  size_t el = 0, bs = 0;
  if (!type_geom(t.ty, &el, &bs)) { *err = name + ": ggml type " + std::to_string(t.ty) + " (" + ggml_name(t.ty) + ") is not supported (F32, F16, BF16, Q8_0, Q4_K, IQ2_XS, IQ3_S are)"; return PYRE_E_TYPE; }
  uint64_t cols = t.shape[0], rows = 1;
  for (size_t k = 1; k < t.shape.size(); ++k) { if (t.shape[k] != 0 && rows > (UINT64_MAX / t.shape[k])) { *err = name + ": shape overflows"; return PYRE_E_SHAPE; } rows *= t.shape[k]; }
  if (rows == 0) rows = 1;
  if (cols == 0 || cols % el) { *err = name + ": row " + std::to_string(cols) + " not a multiple of block " + std::to_string(el); return PYRE_E_SHAPE; }
  const Map& mp = g->maps[t.shard];
  unsigned __int128 need = (unsigned __int128)rows * (cols / el) * bs;
  if (t.off > mp.n || need > (unsigned __int128)(mp.n - t.off)) { *err = name + ": data runs past the end of " + g->paths[t.shard]; return PYRE_E_ARG; }
  out->ggml_type = t.ty; out->on_device = 0; out->rows = rows; out->cols = cols; out->data = (const uint8_t*)mp.p + t.off;
  return PYRE_OK;
}

}  // namespace

extern "C" {

int pyre_gguf_open(const char* path, pyre_gguf** out, char* err, size_t err_cap) {
  if (!path || !out) { set_err(err, err_cap, "pyre_gguf_open: null argument"); return PYRE_E_ARG; }
  *out = nullptr; std::string e; int rc = gguf_open(path, out, &e); if (rc) set_err(err, err_cap, e); return rc;
}
void pyre_gguf_close(pyre_gguf* g) { delete g; }
size_t pyre_gguf_n_shards(const pyre_gguf* g) { return g ? g->paths.size() : 0; }
size_t pyre_gguf_n_tensors(const pyre_gguf* g) { return g ? g->order.size() : 0; }
const char* pyre_gguf_tensor_name(const pyre_gguf* g, size_t i) { return g && i < g->order.size() ? g->order[i].c_str() : nullptr; }
int pyre_gguf_has(const pyre_gguf* g, const char* name) { return g && name && g->tensors.count(name) ? 1 : 0; }
int pyre_gguf_tensor(const pyre_gguf* g, const char* name, pyre_tensor* out, uint32_t* n_dims, uint64_t* dims /*[8]*/, char* err, size_t err_cap) {
  if (!g || !name || !out) { set_err(err, err_cap, "pyre_gguf_tensor: null argument"); return PYRE_E_ARG; }
  std::string e; int rc = gguf_mat(g, name, out, &e); if (rc) { set_err(err, err_cap, e); return rc; }
  const TInfo& t = g->tensors.at(name);
  if (n_dims) *n_dims = (uint32_t)t.shape.size();
  if (dims) for (size_t k = 0; k < t.shape.size() && k < 8; ++k) dims[k] = t.shape[k];
  return PYRE_OK;
}
// Metadata accessors with Meta::as_u64 / as_f64 / as_str / as_arr's conversions (gguf_q.rs:253-258): 0 = found.
int pyre_gguf_meta_u64(const pyre_gguf* g, const char* key, uint64_t* out) { if (!g || !key || !out) return PYRE_E_ARG; auto it = g->meta.find(key); return it != g->meta.end() && it->second.as_u64(out) ? PYRE_OK : PYRE_E_ARG; }
int pyre_gguf_meta_f64(const pyre_gguf* g, const char* key, double* out) { if (!g || !key || !out) return PYRE_E_ARG; auto it = g->meta.find(key); return it != g->meta.end() && it->second.as_f64(out) ? PYRE_OK : PYRE_E_ARG; }
int pyre_gguf_meta_str(const pyre_gguf* g, const char* key, char* out, size_t cap) {
  if (!g || !key || !out || !cap) return PYRE_E_ARG; auto it = g->meta.find(key);
  if (it == g->meta.end() || it->second.kind != Meta::S) return PYRE_E_ARG; snprintf(out, cap, "%s", it->second.s.c_str()); return PYRE_OK;
}
// Array of integers (Gguf::arr_u64): returns the element count, copies at most cap of them; -1 if the key is not an array.
long pyre_gguf_meta_arr_u64(const pyre_gguf* g, const char* key, uint64_t* out, size_t cap) {
  if (!g || !key) return -1; auto it = g->meta.find(key); if (it == g->meta.end() || it->second.kind != Meta::A) return -1;
  size_t n = 0; for (const Meta& m : it->second.a) { uint64_t v; if (m.as_u64(&v)) { if (out && n < cap) out[n] = v; ++n; } }
  return (long)n;
}

// Model::load (qwen4exp_gguf.rs:462-524): architecture check, configuration from the metadata, tensors by name.
// kv_bits / kv_recent are run-time settings of the reference (qn_ctx.rs:119, PYRE_QN_KV8_RECENT), not file contents.
int pyre_model_load_gguf(pyre_ctx* ctx, const char* path, int kv_bits, int kv_recent, int ctx_tokens, pyre_model** out) {
  if (!ctx || !path || !out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_model_load_gguf: null argument");
  *out = nullptr; pyre_gguf* gp = nullptr; std::string e;
  int rc = gguf_open(path, &gp, &e); if (rc) return pyre_fail(ctx, rc, "pyre_model_load_gguf: %s", e.c_str());
  std::unique_ptr<pyre_gguf> g(gp);
  auto arch = g->meta.find("general.architecture");
  if (arch == g->meta.end() || arch->second.kind != Meta::S || arch->second.s != "qwen4exp")
    return pyre_fail(ctx, PYRE_E_ARG, "pyre_model_load_gguf: %s: arch '%s' is not qwen4exp", path, arch != g->meta.end() && arch->second.kind == Meta::S ? arch->second.s.c_str() : "");
  bool missing = false; std::string miss;
  auto ku = [&](const char* s, long dflt = -1) -> int64_t { uint64_t v = 0; std::string k = std::string("qwen4exp.") + s; auto it = g->meta.find(k);
    if (it != g->meta.end() && it->second.as_u64(&v)) return (int64_t)v; if (dflt >= 0) return dflt; missing = true; miss = k; return 0; };
  auto kf = [&](const char* s) -> double { double v = 0; std::string k = std::string("qwen4exp.") + s; auto it = g->meta.find(k); if (it != g->meta.end() && it->second.as_f64(&v)) return v; missing = true; miss = k; return 0; };
  pyre_model_cfg c{};
  c.n_layers = (int)ku("block_count"); c.d = (int)ku("embedding_length"); c.hc = (int)ku("hyper_connection.count"); c.hc_lr = (int)ku("hyper_connection.low_rank");
  c.n_head = (int)ku("attention.head_count"); c.n_kv = (int)ku("attention.head_count_kv"); c.hd = (int)ku("attention.key_length"); c.n_rot = (int)ku("rope.dimension_count");
  c.rope_base = (float)kf("rope.freq_base"); c.eps = (float)kf("attention.layer_norm_rms_epsilon");
  c.n_exp = (int)ku("expert_count"); c.top_k = (int)ku("expert_used_count"); c.ff_exp = (int)ku("expert_feed_forward_length");
  c.lin_nk = (int)ku("ssm.group_count"); c.lin_nv = (int)ku("ssm.time_step_rank"); c.lin_dk = (int)ku("ssm.state_size"); c.lin_dv = c.lin_dk; c.conv_k = (int)ku("ssm.conv_kernel");
  c.full_every = (int)ku("full_attention_interval", 4); c.kv_bits = kv_bits; c.kv_recent = kv_recent;
  // QSA indexer and trained context, qwen4exp_gguf.rs:481-486 (same defaults); the ratio is the largest entry of compress_ratios
  c.idx_budget = (int)ku("attention.indexer.top_k", 2048); c.idx_nh = (int)ku("attention.indexer.head_count", 0); c.idx_hd = (int)ku("attention.indexer.key_length", 128);
  c.idx_ratio = 4; { auto it = g->meta.find("qwen4exp.attention.compress_ratios"); if (it != g->meta.end() && it->second.kind == Meta::A && !it->second.a.empty()) { uint64_t mx = 0; for (const Meta& e2 : it->second.a) { uint64_t v = 0; if (e2.as_u64(&v) && v > mx) mx = v; } c.idx_ratio = (int)(mx > 0 ? mx : 1); } }
  c.ctx_train = (int)ku("context_length", 262144); c.ctx = ctx_tokens > 0 ? ctx_tokens : c.ctx_train;
  const bool has_idx = c.idx_nh > 0 && g->tensors.count("blk." + std::to_string((c.full_every > 0 ? c.full_every : 1) - 1) + ".indexer.q_proj.weight") > 0;      // :489 looks at block 3
  if (!has_idx) c.idx_nh = 0;
  if (missing) return pyre_fail(ctx, PYRE_E_ARG, "pyre_model_load_gguf: gguf key %s", miss.c_str());
  // PLE, qwen4exp_gguf.rs:468-480: the listed layers carry blk.N.ple_*; the hash parameters are arrays of u64
  std::vector<int> ple_layers;
  { auto it = g->meta.find("qwen4exp.ple.layers"); if (it != g->meta.end() && it->second.kind == Meta::A) for (const Meta& e2 : it->second.a) { uint64_t v = 0; if (e2.as_u64(&v)) ple_layers.push_back((int)v); } }
  if (!ple_layers.empty()) {
    c.ple_ngram = (int)ku("ple.ngram_size", 0); c.ple_per_gram = (int)ku("ple.heads_per_ngram", 0); c.ple_conv_k = (int)ku("ple.conv_kernel", 0);
    c.ple_eos = (uint32_t)ku("ple.eos_token_id", 0); c.ple_dim = (int)ku("embedding_length_per_layer_input", 0);
    auto arr = [&](const char* key, uint64_t* dst, size_t cap) -> long { auto it = g->meta.find(std::string("qwen4exp.") + key); if (it == g->meta.end() || it->second.kind != Meta::A) return -1;
      size_t n = 0; for (const Meta& e2 : it->second.a) { uint64_t v = 0; if (!e2.as_u64(&v)) return -1; if (n < cap) dst[n] = v; ++n; } return (long)n; };
    const long nm = arr("ple.layer_multipliers", c.ple_mult, 8), no = arr("ple.head_offsets", c.ple_off, 16), nv = arr("ple.head_vocab_sizes", c.ple_vocab, 16);
    const long nh = (long)(c.ple_ngram - 1) * c.ple_per_gram;
    if (c.ple_ngram < 2 || c.ple_ngram > 8 || nh < 1 || nh > 16 || nm < c.ple_ngram || nm > 8 || no < nh || nv < nh || no > 16 || nv > 16)
      return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_model_load_gguf: PLE with n-grams of %d, %d heads per length, %ld multipliers, %ld offsets, %ld sizes is unsupported", c.ple_ngram, c.ple_per_gram, nm, no, nv);
  }
  auto emb = g->tensors.find("token_embd.weight");
  if (emb == g->tensors.end() || emb->second.shape.size() < 2) return pyre_fail(ctx, PYRE_E_ARG, "pyre_model_load_gguf: token_embd");
  c.vocab = (int)emb->second.shape[1];
  if (c.n_layers < 1 || c.n_layers > 4096) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_model_load_gguf: block_count %d", c.n_layers);
  std::vector<pyre_tensor> lt((size_t)c.n_layers * PYRE_LAYER_SLOTS, pyre_tensor{}), gl(PYRE_GLOBAL_SLOTS, pyre_tensor{});
  auto get = [&](const std::string& name, pyre_tensor* t) -> bool { int r2 = gguf_mat(g.get(), name, t, &e); if (r2) { rc = r2; return false; } return true; };
  static const char* hc_sfx[4] = {"_norm.weight", "_down.weight", "_inject.weight", "_up.weight"};
  for (int il = 0; il < c.n_layers; ++il) {
    pyre_tensor* T = lt.data() + (size_t)il * PYRE_LAYER_SLOTS; const std::string p = "blk." + std::to_string(il) + ".";
    for (int k = 0; k < 4; ++k) if (!get(p + "hc_attn" + hc_sfx[k], &T[PYRE_T_HC_ATTN_NORM + k]) || !get(p + "hc_ffn" + hc_sfx[k], &T[PYRE_T_HC_FFN_NORM + k])) return pyre_fail(ctx, rc, "pyre_model_load_gguf: %s", e.c_str());
    const bool full = (il + 1) % (c.full_every > 0 ? c.full_every : 1) == 0;
    bool ok;
    if (full) ok = get(p + "attn_q.weight", &T[PYRE_T_ATTN_Q]) && get(p + "attn_k.weight", &T[PYRE_T_ATTN_K]) && get(p + "attn_v.weight", &T[PYRE_T_ATTN_V]) && get(p + "attn_output.weight", &T[PYRE_T_ATTN_OUTPUT]) &&
                   get(p + "attn_q_norm.weight", &T[PYRE_T_ATTN_Q_NORM]) && get(p + "attn_k_norm.weight", &T[PYRE_T_ATTN_K_NORM]) &&
                   (!has_idx || (get(p + "indexer.q_proj.weight", &T[PYRE_T_INDEXER_Q_PROJ]) && get(p + "indexer.k_proj.weight", &T[PYRE_T_INDEXER_K_PROJ]) &&
                                 get(p + "indexer.q_norm.weight", &T[PYRE_T_INDEXER_Q_NORM]) && get(p + "indexer.k_norm.weight", &T[PYRE_T_INDEXER_K_NORM])));
    else ok = get(p + "attn_qkv.weight", &T[PYRE_T_ATTN_QKV]) && get(p + "attn_gate.weight", &T[PYRE_T_ATTN_GATE]) && get(p + "ssm_beta.weight", &T[PYRE_T_SSM_BETA]) && get(p + "ssm_alpha.weight", &T[PYRE_T_SSM_ALPHA]) &&
              get(p + "ssm_a", &T[PYRE_T_SSM_A]) && get(p + "ssm_dt.bias", &T[PYRE_T_SSM_DT_BIAS]) && get(p + "ssm_conv1d.weight", &T[PYRE_T_SSM_CONV1D]) && get(p + "ssm_norm.weight", &T[PYRE_T_SSM_NORM]) &&
              get(p + "ssm_out.weight", &T[PYRE_T_SSM_OUT]);
    ok = ok && get(p + "ffn_gate_inp.weight", &T[PYRE_T_FFN_GATE_INP]) && get(p + "ffn_gate_exps.weight", &T[PYRE_T_FFN_GATE_EXPS]) && get(p + "ffn_up_exps.weight", &T[PYRE_T_FFN_UP_EXPS]) &&
         get(p + "ffn_down_exps.weight", &T[PYRE_T_FFN_DOWN_EXPS]) && get(p + "ffn_gate_inp_shexp.weight", &T[PYRE_T_FFN_GATE_INP_SHEXP]) && get(p + "ffn_gate_shexp.weight", &T[PYRE_T_FFN_GATE_SHEXP]) &&
         get(p + "ffn_up_shexp.weight", &T[PYRE_T_FFN_UP_SHEXP]) && get(p + "ffn_down_shexp.weight", &T[PYRE_T_FFN_DOWN_SHEXP]);
    if (ok && std::find(ple_layers.begin(), ple_layers.end(), il) != ple_layers.end())
      ok = get(p + "ple_key.weight", &T[PYRE_T_PLE_KEY]) && get(p + "ple_value.weight", &T[PYRE_T_PLE_VALUE]) && get(p + "ple_norm_key.weight", &T[PYRE_T_PLE_NORM_KEY]) &&
           get(p + "ple_norm_query.weight", &T[PYRE_T_PLE_NORM_QUERY]) && get(p + "ple_norm_conv.weight", &T[PYRE_T_PLE_NORM_CONV]) && get(p + "ple_conv1d.weight", &T[PYRE_T_PLE_CONV1D]);
    if (!ok) return pyre_fail(ctx, rc, "pyre_model_load_gguf: %s", e.c_str());
  }
  if (!ple_layers.empty() && !get("per_layer_token_embd.weight", &gl[PYRE_G_PLE_TOKEN_EMBD])) return pyre_fail(ctx, rc, "pyre_model_load_gguf: %s", e.c_str());
  bool ok = get("token_embd.weight", &gl[PYRE_G_TOKEN_EMBD]) && get("output_hc_norm.weight", &gl[PYRE_G_OUTPUT_HC_NORM]) && get("output_hc_down.weight", &gl[PYRE_G_OUTPUT_HC_DOWN]) &&
            get("output_hc_up.weight", &gl[PYRE_G_OUTPUT_HC_UP]) && get(g->tensors.count("output.weight") ? "output.weight" : "token_embd.weight", &gl[PYRE_G_OUTPUT]);
  if (!ok) return pyre_fail(ctx, rc, "pyre_model_load_gguf: %s", e.c_str());
  return pyre_model_create(ctx, &c, lt.data(), gl.data(), out);        // copies everything to the device; the mappings go away with g
}

}  // extern "C"
