// The qwen4exp token step on the device: embed -> per layer { hc_mix -> Gated DeltaNet | gated attention -> hc_combine
// -> hc_mix -> MoE FFN -> hc_combine } -> head hc_mix -> logits, plus the multi-token verify window, rollback and the
// greedy loop.  Follows Model::forward_inner / forward_multi / spec_keep (src/model/qwen4exp_gguf.rs:2087-2157,
// 2365-2480, 2495-2515) and spec::generate's greedy branch (src/spec.rs:156-267).
#include "formats.h"
#include "digits.h"
#include <chrono>
#include <memory>
#include <stdlib.h>

namespace {

struct Layer {
  bool full = false;
  HcDev hca{}, hcf{};
  QMatDev proj{};            // attention: [q ; k ; v]   DeltaNet: [qkv ; z ; beta ; alpha]
  QMatDev outp{};            // attn_output / ssm_out
  AttnDev attn{}; GdnDev gdn{}; MoeDev moe{}; QsaDev qsa{};
  bool ple = false; PleDev pld{}; int ple_index = 0;      // per-layer n-gram embeddings in front of the layer (ring pointer lives in the state)
  int mix_index = 0;         // index among the attention or among the DeltaNet layers
  float gdn_up = 1.0f; const float* gdn_ainv = nullptr;      // DeltaNet: the power of two its output is scaled by as the f16 operand of ssm_out, and the [super-block][8] array of its inverse
};

}  // namespace

struct PromptPipe; void prompt_pipe_free(PromptPipe* P); size_t prompt_pipe_blocks(const PromptPipe* P);

struct pyre_model {
  pyre_ctx* ctx = nullptr; pyre_model_cfg c{};
  std::vector<Layer> layers; HcDev head{}; QMatDev embd{}, out{};
  std::vector<pyre_qmat*> owned; std::vector<void*> bufs;
  bool has_idx = false; int iq_off = 0; float mscale = 1.0f;       // QSA indexer on every attention layer; column of the index projections in an attention row
  float* rope_inv = nullptr; int n_attn = 0, n_lin = 0, ch = 0, pw_lin = 0, pw_attn = 0;
  size_t token_weight_bytes = 0;
  // activations for a window of up to 8 tokens
  void* work = nullptr; HcWork hw{}; MoeWork mw{};
  float *x = nullptr, *x2 = nullptr, *mixed = nullptr, *inj_a = nullptr, *inj_f = nullptr, *proj = nullptr, *core = nullptr, *o = nullptr, *y = nullptr, *hbuf = nullptr, *logits = nullptr, *co = nullptr, *emb = nullptr, *rpart = nullptr;
  uint32_t* ids = nullptr; uint32_t* toks = nullptr; int toks_cap = 0; uint32_t* best = nullptr;
  PleCfg plc{}; QMatDev ple_tab{}; PleWork pw{}; int n_ple = 0, ple_ring = 0;      // PLE: hash parameters, the token table, window workspace, ring rows per layer
  uint16_t* aop = nullptr;      // the f16 operand a producer kernel leaves for the matrix-core GEMV that follows it (one at a time: the launches are stream-ordered)
  float* gdn_sq = nullptr;      // [2][8][nv][4]: per token, head and quarter the inverse power of two of the Gated DeltaNet operand and the quarter's sum of squares (PyreAop::sq)
  float* aop_inv = nullptr;     // [super-blocks][8]: the inverse of the power of two the hyper-connection mix scaled each token of that operand by
  PromptPipe* pipe = nullptr;      // further window workspaces and streams for a long prompt (prompt_pipe), made at the first one
};

struct pyre_state {
  pyre_ctx* ctx = nullptr; const pyre_model* m = nullptr; int cap = 0, len = 0;
  void* mem = nullptr;
  std::vector<float*> conv[2], ssm[2]; std::vector<int> cur;     // DeltaNet double buffers
  std::vector<float*> proj_saved;                                // per DeltaNet layer [8][pw_lin]: inputs of the last window
  std::vector<KvDev> kv; std::vector<int> packed; AttnWork aw{};
  std::vector<QsaBuf> qsa; QsaWork qw{};                          // indexer keys per attention layer; selection workspace
  void* pipe_mem = nullptr; std::vector<AttnWork> aw_more; std::vector<QsaWork> qw_more;      // one more attention / selection workspace per further prompt stream
  int last_window = 0;                                           // tokens of the last forward_multi (0 = spec_keep unarmed)
  bool broken = false;                                           // a call failed after it had begun to advance this state: every call but reset / restore refuses it
  uint32_t* tokens_dev = nullptr; std::vector<float*> ple_ring;     // PLE models: the token history by position; per PLE layer the ring of normalised rows
  int* step_dev = nullptr; hipGraphExec_t graph_exec = nullptr; const uint32_t* graph_toks = nullptr;   // replayed decode step
  std::vector<int> graph_cur;                                    // which half of every DeltaNet double buffer the captured step works on
  // MTP drafter (attached by pyre_state_attach_mtp): the ring of final residual streams by position, of which positions
  // [r_first, r_next) are valid; the drafter's own K/V cache by cell, of which cells [m_c0, m_c0 + m_n) are valid
  const pyre_mtp* mtp = nullptr; void* mtp_mem = nullptr; float* r_ring = nullptr; int r_mask = 0, r_first = 0, r_next = 0;
  KvDev mkv{}; int* mlist = nullptr; int* mcount = nullptr; int m_c0 = 0, m_n = 0;
  // mtp_keep_r (qwen4exp_gguf.rs:2279-2285) for positions start .. start+t-1, whose rows a kernel on the stream writes
  void r_push(int start, int t, int window) {
    if (r_next > start) r_next = start;                          // newer rows are dropped (a rolled-back window)
    if (r_next <= r_first || r_next != start) r_first = start;   // a gap empties the ring
    r_next = start + t; if (r_next - r_first > window + 16) r_first = r_next - (window + 16);
  }
};

namespace {

// PYRE_PROMPT_BLOCK=0: no second layout of the expert matrices, every prompt in windows (prompt_block_ok)
static bool prompt_block_env() { static const bool on = [] { const char* e = getenv("PYRE_PROMPT_BLOCK"); return !(e && *e && atoi(e) == 0); }(); return on; }

struct Builder {
  pyre_ctx* ctx; pyre_model* m;
  int fail(int code, const char* what) { return pyre_fail(ctx, code, "pyre_model_create: %s", what); }

  // one matrix out of `n` row-concatenated tensors of one type and width
  // layout: PYRE_LAYOUT_M for the matrices that only ever meet a GEMV or a row look-up (projections, head, embedding),
  // PYRE_LAYOUT_ROWS for those the hyper-connection and MoE kernels walk themselves
  int cat(const pyre_tensor* const* ts, int n, QMatDev* out, size_t* gguf_bytes, int layout = PYRE_LAYOUT_ROWS, QMatDev* out_m = nullptr) {
    uint32_t ty = ts[0]->ggml_type; uint64_t cols = ts[0]->cols; uint32_t dev = ts[0]->on_device; uint64_t rows = 0; size_t total = 0;
    int fmt = fmt_from_ggml(ty); if (fmt < 0) return fail(PYRE_E_TYPE, "unsupported tensor type");
    struct { int el, bytes; } g{1, 4}; ggml_geom(ty, &g.el, &g.bytes);
    for (int i = 0; i < n; ++i) {
      if (!ts[i]->data) return fail(PYRE_E_ARG, "missing tensor");
      if (ts[i]->ggml_type != ty || ts[i]->cols != cols || ts[i]->on_device != dev) return fail(PYRE_E_TYPE, "tensors of one projection group differ in type, width or location");
      rows += ts[i]->rows; total += ts[i]->rows * (cols / g.el * g.bytes);
    }
    pyre_qmat* q = nullptr; int rc;
    if (cols % 256) layout = PYRE_LAYOUT_ROWS;
    if (n == 1) rc = pyre_qmat_create_layout(ctx, ty, rows, cols, ts[0]->data, dev != 0, total, layout, &q);
    else {
      void* tmp = nullptr; PYRE_HIP(ctx, hipMalloc(&tmp, total)); size_t off = 0;
      for (int i = 0; i < n; ++i) { size_t nb = ts[i]->rows * (cols / g.el * g.bytes);
        hipError_t e = hipMemcpy((uint8_t*)tmp + off, ts[i]->data, nb, dev ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice);
        if (e != hipSuccess) { (void)hipFree(tmp); return pyre_fail(ctx, PYRE_E_HIP, "pyre_model_create: copy: %s", hipGetErrorString(e)); } off += nb; }
      rc = pyre_qmat_create_layout(ctx, ty, rows, cols, tmp, true, total, layout, &q); (void)hipFree(tmp);
    }
    if (rc) return rc;
    m->owned.push_back(q); *out = q->dv; if (out_m) *out_m = q->dvm; if (gguf_bytes) *gguf_bytes += total; return PYRE_OK;
  }
  int one(const pyre_tensor& t, QMatDev* out, size_t* gguf_bytes, int layout = PYRE_LAYOUT_ROWS, QMatDev* out_m = nullptr) { const pyre_tensor* p = &t; return cat(&p, 1, out, gguf_bytes, layout, out_m); }

  // Gguf::vec: a small tensor fully dequantized to f32 on the device
  int vec(const pyre_tensor& t, size_t expect, const float** out) {
    if (!t.data) return fail(PYRE_E_ARG, "missing vector tensor");
    size_t n = t.rows * t.cols; if (n != expect) return fail(PYRE_E_SHAPE, "vector tensor has the wrong length");
    float* d = nullptr; PYRE_HIP(ctx, hipMalloc((void**)&d, n * 4)); m->bufs.push_back(d);
    if (t.ggml_type == PYRE_F32) { PYRE_HIP(ctx, hipMemcpy(d, t.data, n * 4, t.on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice)); }
    else {
      pyre_qmat* q = nullptr; int fmt = fmt_from_ggml(t.ggml_type); if (fmt < 0) return fail(PYRE_E_TYPE, "unsupported vector type"); struct { int el, bytes; } g{1, 4}; ggml_geom(t.ggml_type, &g.el, &g.bytes);
      size_t nb = n / g.el * g.bytes;
      int rc = pyre_qmat_create_layout(ctx, t.ggml_type, t.rows, t.cols, t.data, t.on_device != 0, nb, PYRE_LAYOUT_ROWS, &q); if (rc) return rc;
      rc = pyre_qmat_dequant_dev(ctx, q, d); if (!rc) rc = pyre_ctx_sync(ctx); pyre_qmat_destroy(q); if (rc) return rc;
    }
    *out = d; return PYRE_OK;
  }
  int hc(const pyre_tensor& norm, const pyre_tensor& down, const pyre_tensor* inject, const pyre_tensor& up, HcDev* h, size_t* bytes) {
    const pyre_model_cfg& c = m->c; size_t w = (size_t)c.hc * c.d;
    if (down.rows != (uint64_t)c.hc_lr || down.cols != w || up.rows != w || up.cols != (uint64_t)c.hc_lr) return fail(PYRE_E_SHAPE, "hyper-connection matrix shapes");
    if (inject && (inject->rows != (uint64_t)c.hc || inject->cols != w)) return fail(PYRE_E_SHAPE, "hyper-connection inject shape");
    // both layouts: the mixes run on the matrix cores when both matrices are IQ3_S of whole super-blocks, and the lane = row kernels stay available (PYRE_HC_ROWS)
    const pyre_tensor* grp[2] = {&down, inject}; int rc = cat(grp, inject ? 2 : 1, &h->di, bytes, PYRE_LAYOUT_BOTH, &h->di_m); if (rc) return rc;
    rc = one(up, &h->up, bytes, PYRE_LAYOUT_BOTH, &h->up_m); if (rc) return rc;
    rc = vec(norm, w, &h->norm); if (rc) return rc;
    h->d = c.d; h->hc = c.hc; h->lr = c.hc_lr; h->has_inject = inject != nullptr; return PYRE_OK;
  }
};

size_t al256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace

extern "C" {

// The activations of one window of up to 8 tokens: everything a window's launches write apart from the state.
// the window workspace of a model (activations of up to eight tokens): its size, and its pieces carved out of `base`
static size_t model_work_layout(pyre_model* m, void* base, int* kmax_out, size_t* aop_bytes) {
  const pyre_model_cfg& c = m->c;
  const size_t w = (size_t)c.hc * c.d, pmax = (size_t)(m->pw_lin > m->pw_attn ? m->pw_lin : m->pw_attn), cmax = (size_t)((c.lin_nv * c.lin_dv) > (c.n_head * c.hd) ? c.lin_nv * c.lin_dv : c.n_head * c.hd);
  HcDev hmax = m->head; hmax.lr = c.hc_lr;
  MoeDev& m0 = m->layers[0].moe; size_t moe_b = 0; for (auto& L : m->layers) { size_t b = pyre_moe_work_bytes(L.moe); if (b > moe_b) moe_b = b; }
  size_t rp_b = 4; for (auto& L : m->layers) if (pyre_hc_route_ok(L.hcf, L.moe.router)) rp_b = std::max(rp_b, (size_t)4 * 8 * (c.d / 64) * L.moe.router.tiles * 64);      // router K-slice sums
  int kmax = c.d; for (auto& L : m->layers) kmax = std::max(kmax, std::max(L.proj.cols, L.outp.cols));
  const size_t aop_b = pyre_aop_bytes((kmax + 255) / 256 * 256, 8);
  const size_t ple_b = m->n_ple > 0 ? pyre_ple_work_bytes(m->plc, c.d, c.hc) : 0;
  size_t total = al256(pyre_hc_work_bytes(hmax)) + al256(moe_b) + 2 * al256(4 * 8 * w) + 6 * al256(4 * 8 * (size_t)c.d) + al256(4 * 8 * PYRE_GEMV_PARTS * (size_t)c.d) + 2 * al256(4 * 8 * c.hc) + al256(4 * 8 * pmax) + al256(4 * 8 * cmax) +
                 al256(4 * 8 * (size_t)c.vocab) + al256(4 * 8 * (size_t)m->ch) + al256(4 * 16) + al256(8 * ((size_t)c.vocab / 32 + 4)) + al256(rp_b) + al256(aop_b) + al256(4 * 8 * (size_t)((kmax + 255) / 256)) + al256(4 * 2 * 8 * 4 * (size_t)c.lin_nv) + al256(ple_b) + 4096;
  if (kmax_out) *kmax_out = kmax;
  if (aop_bytes) *aop_bytes = aop_b;
  if (!base) return total;
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += al256(n); return r; };
  pyre_hc_work_carve(hmax, take(pyre_hc_work_bytes(hmax)), &m->hw); pyre_moe_work_carve(m0, take(moe_b), &m->mw);
  m->x = (float*)take(4 * 8 * w); m->x2 = (float*)take(4 * 8 * w); m->mixed = (float*)take(4 * 8 * (size_t)c.d); m->o = (float*)take(4 * 8 * PYRE_GEMV_PARTS * (size_t)c.d); m->y = (float*)take(4 * 8 * (size_t)c.d); m->hbuf = (float*)take(4 * 8 * (size_t)c.d);
  m->emb = (float*)take(4 * 8 * (size_t)c.d); (void)take(4 * 8 * (size_t)c.d);
  m->inj_a = (float*)take(4 * 8 * c.hc); m->inj_f = (float*)take(4 * 8 * c.hc); m->proj = (float*)take(4 * 8 * pmax); m->core = (float*)take(4 * 8 * cmax);
  m->logits = (float*)take(4 * 8 * (size_t)c.vocab); m->co = (float*)take(4 * 8 * (size_t)m->ch); m->ids = (uint32_t*)take(4 * 16); m->best = (uint32_t*)take(8 * ((size_t)c.vocab / 32 + 4));
  m->rpart = (float*)take(rp_b); m->aop = (uint16_t*)take(aop_b); m->aop_inv = (float*)take(4 * 8 * (size_t)((kmax + 255) / 256)); m->gdn_sq = (float*)take(4 * 2 * 8 * 4 * (size_t)c.lin_nv);
  if (m->n_ple > 0) pyre_ple_work_carve(m->plc, c.d, c.hc, take(ple_b), &m->pw);
  return total;
}
static int model_alloc_work(pyre_ctx* ctx, pyre_model* m, int* kmax_out) {
  size_t aop_b = 0; const size_t total = model_work_layout(m, nullptr, kmax_out, &aop_b);
  PYRE_HIP(ctx, hipMalloc(&m->work, total));
  (void)model_work_layout(m, m->work, nullptr, nullptr);
  PYRE_HIP(ctx, hipMemsetAsync(m->aop, 0, aop_b, ctx->stream));
  return PYRE_OK;
}

int pyre_model_create(pyre_ctx* ctx, const pyre_model_cfg* cfg, const pyre_tensor* lt, const pyre_tensor* gl, pyre_model** out) {
  if (!ctx || !cfg || !lt || !gl || !out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_model_create: null argument");
  *out = nullptr;
  const pyre_model_cfg& c = *cfg;
  if (c.n_layers < 1 || c.d < 64 || c.d % 64 || c.hc < 1 || c.hc > 8 || c.hc_lr < 64 || c.hc_lr % 64 || c.full_every < 1 || c.vocab < 1 || c.top_k < 1 || c.top_k > 32 || c.n_exp < c.top_k || c.n_exp > 1024)
    return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_model_create: unsupported configuration (d and hc_lr must be multiples of 64, hc <= 8)");
  PYRE_HIP(ctx, hipSetDevice(ctx->device));
  std::unique_ptr<pyre_model> M(new pyre_model()); pyre_model* m = M.get(); m->ctx = ctx; m->c = c;
  struct Guard { pyre_model* m; bool armed = true; ~Guard() { if (armed && m) { for (auto q : m->owned) pyre_qmat_destroy(q); for (auto b : m->bufs) (void)hipFree(b); if (m->work) (void)hipFree(m->work); } } } guard{m};
  Builder B{ctx, m};
  m->ch = 2 * c.lin_nk * c.lin_dk + c.lin_nv * c.lin_dv; m->pw_lin = m->ch + c.lin_nv * c.lin_dv + 2 * c.lin_nv; m->pw_attn = c.n_head * 2 * c.hd + 2 * c.n_kv * c.hd;
  m->has_idx = c.idx_nh > 0 && c.full_every <= c.n_layers && lt[(size_t)(c.full_every - 1) * PYRE_LAYER_SLOTS + PYRE_T_INDEXER_Q_PROJ].data != nullptr;
  if (m->has_idx) {
    if (c.idx_hd < 64 || c.idx_hd % 64 || c.idx_hd > 1024 || c.idx_hd < c.n_rot || c.idx_ratio < 1 || c.idx_budget < c.idx_ratio || c.idx_budget % c.idx_ratio)
      return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_model_create: indexer with %d heads of %d, block %d, budget %d is unsupported", c.idx_nh, c.idx_hd, c.idx_ratio, c.idx_budget);
    m->iq_off = m->pw_attn; m->pw_attn += c.idx_nh * c.idx_hd + c.idx_hd;
  }
  std::vector<float> inv(c.n_rot / 2); const float mscale = pyre_rope_table(c.n_rot, c.rope_base, c.ctx_train, c.ctx, inv.data());   // qn_ctx.rs:164-185
  PYRE_HIP(ctx, hipMalloc((void**)&m->rope_inv, (inv.size() + 1) * 4)); m->bufs.push_back(m->rope_inv);
  PYRE_HIP(ctx, hipMemcpy(m->rope_inv, inv.data(), inv.size() * 4, hipMemcpyHostToDevice)); m->mscale = mscale;
  size_t tok_bytes = 0; int rc;
  const int mlay = [] { const char* e = getenv("PYRE_MODEL_ROWS"); return e && *e && atoi(e) != 0; }() ? PYRE_LAYOUT_ROWS : PYRE_LAYOUT_M;      // 1: every matrix in the lane = row layout
  m->layers.resize(c.n_layers);
  for (int il = 0; il < c.n_layers; ++il) {
    const pyre_tensor* T = lt + (size_t)il * PYRE_LAYER_SLOTS; Layer& L = m->layers[il];
    L.full = (il + 1) % c.full_every == 0;
    if ((rc = B.hc(T[PYRE_T_HC_ATTN_NORM], T[PYRE_T_HC_ATTN_DOWN], &T[PYRE_T_HC_ATTN_INJECT], T[PYRE_T_HC_ATTN_UP], &L.hca, &tok_bytes))) return rc;
    if ((rc = B.hc(T[PYRE_T_HC_FFN_NORM], T[PYRE_T_HC_FFN_DOWN], &T[PYRE_T_HC_FFN_INJECT], T[PYRE_T_HC_FFN_UP], &L.hcf, &tok_bytes))) return rc;
    if (c.ple_ngram > 1 && T[PYRE_T_PLE_KEY].data) {
      const pyre_tensor* kvg[2] = {&T[PYRE_T_PLE_KEY], &T[PYRE_T_PLE_VALUE]}; const size_t wd = (size_t)c.hc * c.d; const int ein = (c.ple_ngram - 1) * c.ple_per_gram * c.ple_dim;
      if (!gl[PYRE_G_PLE_TOKEN_EMBD].data || !T[PYRE_T_PLE_VALUE].data) return B.fail(PYRE_E_ARG, "a PLE layer needs per_layer_token_embd and all six ple_* tensors");
      if (kvg[0]->rows != wd || kvg[1]->rows != (uint64_t)c.d || kvg[0]->cols != (uint64_t)ein || kvg[1]->cols != (uint64_t)ein) return B.fail(PYRE_E_SHAPE, "ple_key / ple_value shapes");
      L.ple = true; L.ple_index = m->n_ple++; size_t pb = 0;
      if ((rc = B.cat(kvg, 2, &L.pld.kv, &pb)) || (rc = B.vec(T[PYRE_T_PLE_NORM_KEY], wd, &L.pld.nk)) || (rc = B.vec(T[PYRE_T_PLE_NORM_QUERY], wd, &L.pld.nq)) ||
          (rc = B.vec(T[PYRE_T_PLE_NORM_CONV], wd, &L.pld.nc)) || (rc = B.vec(T[PYRE_T_PLE_CONV1D], wd * c.ple_conv_k, &L.pld.conv))) return rc;
      tok_bytes += pb;
    }
    if (L.full) {
      L.mix_index = m->n_attn++;
      const pyre_tensor* grp[5] = {&T[PYRE_T_ATTN_Q], &T[PYRE_T_ATTN_K], &T[PYRE_T_ATTN_V], &T[PYRE_T_INDEXER_Q_PROJ], &T[PYRE_T_INDEXER_K_PROJ]};
      if (grp[0]->rows != (uint64_t)c.n_head * 2 * c.hd || grp[1]->rows != (uint64_t)c.n_kv * c.hd || grp[2]->rows != (uint64_t)c.n_kv * c.hd || grp[0]->cols != (uint64_t)c.d)
        return B.fail(PYRE_E_SHAPE, "attention projection shapes");
      if (m->has_idx && (!grp[3]->data || !grp[4]->data || grp[3]->rows != (uint64_t)c.idx_nh * c.idx_hd || grp[4]->rows != (uint64_t)c.idx_hd)) return B.fail(PYRE_E_SHAPE, "indexer projection shapes (every attention layer needs them)");
      if ((rc = B.cat(grp, m->has_idx ? 5 : 3, &L.proj, &tok_bytes, mlay))) return rc;
      if (T[PYRE_T_ATTN_OUTPUT].rows != (uint64_t)c.d || T[PYRE_T_ATTN_OUTPUT].cols != (uint64_t)c.n_head * c.hd) return B.fail(PYRE_E_SHAPE, "attn_output shape");
      if ((rc = B.one(T[PYRE_T_ATTN_OUTPUT], &L.outp, &tok_bytes, mlay))) return rc;
      L.attn = AttnDev{nullptr, nullptr, m->rope_inv, c.n_head, c.n_kv, c.hd, c.n_rot, c.kv_bits, c.kv_recent, c.eps, mscale};
      if ((rc = B.vec(T[PYRE_T_ATTN_Q_NORM], c.hd, &L.attn.qn)) || (rc = B.vec(T[PYRE_T_ATTN_K_NORM], c.hd, &L.attn.kn))) return rc;
      if (m->has_idx) {
        L.qsa = QsaDev{nullptr, nullptr, c.idx_nh, c.idx_hd, c.idx_ratio, c.idx_budget};
        if ((rc = B.vec(T[PYRE_T_INDEXER_Q_NORM], c.idx_hd, &L.qsa.iqn)) || (rc = B.vec(T[PYRE_T_INDEXER_K_NORM], c.idx_hd, &L.qsa.ikn))) return rc;
      }
    } else {
      L.mix_index = m->n_lin++;
      const pyre_tensor* grp[4] = {&T[PYRE_T_ATTN_QKV], &T[PYRE_T_ATTN_GATE], &T[PYRE_T_SSM_BETA], &T[PYRE_T_SSM_ALPHA]};
      if (grp[0]->rows != (uint64_t)m->ch || grp[1]->rows != (uint64_t)c.lin_nv * c.lin_dv || grp[2]->rows != (uint64_t)c.lin_nv || grp[3]->rows != (uint64_t)c.lin_nv || grp[0]->cols != (uint64_t)c.d)
        return B.fail(PYRE_E_SHAPE, "DeltaNet projection shapes");
      if ((rc = B.cat(grp, 4, &L.proj, &tok_bytes, mlay))) return rc;
      if (T[PYRE_T_SSM_OUT].rows != (uint64_t)c.d || T[PYRE_T_SSM_OUT].cols != (uint64_t)c.lin_nv * c.lin_dv) return B.fail(PYRE_E_SHAPE, "ssm_out shape");
      if ((rc = B.one(T[PYRE_T_SSM_OUT], &L.outp, &tok_bytes, mlay))) return rc;
      L.gdn = GdnDev{nullptr, nullptr, nullptr, nullptr, c.lin_nk, c.lin_nv, c.lin_dk, c.lin_dv, c.conv_k, c.eps};
      if ((rc = B.vec(T[PYRE_T_SSM_A], c.lin_nv, &L.gdn.a)) || (rc = B.vec(T[PYRE_T_SSM_DT_BIAS], c.lin_nv, &L.gdn.dt)) ||
          (rc = B.vec(T[PYRE_T_SSM_CONV1D], (size_t)m->ch * c.conv_k, &L.gdn.conv_w)) || (rc = B.vec(T[PYRE_T_SSM_NORM], c.lin_dv, &L.gdn.norm_w))) return rc;
      {      // the layer's output as an f16 operand: |o_i * rms scale * w_i * sigmoid(z_i)| <= sqrt(dv) * max |w|, brought into [2^13, 2^14) by a power of two
        std::vector<float> nw(c.lin_dv); PYRE_HIP(ctx, hipMemcpy(nw.data(), L.gdn.norm_w, (size_t)c.lin_dv * 4, hipMemcpyDeviceToHost));
        float mx = 0.0f; bool fin = true; for (float v : nw) { if (!(fabsf(v) <= 3.0e38f)) fin = false; mx = fmaxf(mx, fabsf(v)); }
        const float bound = sqrtf((float)c.lin_dv) * mx; int e = 0;
        if (fin && bound > 0.0f) { uint32_t bits; memcpy(&bits, &bound, 4); e = 140 - (int)((bits >> 23) & 0xFF); e = e > 100 ? 100 : (e < -100 ? -100 : e); }
        L.gdn_up = ldexpf(1.0f, e);
        const int nsb = (c.lin_nv * c.lin_dv + 255) / 256; std::vector<float> inv((size_t)nsb * 8, ldexpf(1.0f, -e));
        float* dv = nullptr; PYRE_HIP(ctx, hipMalloc((void**)&dv, inv.size() * 4)); m->bufs.push_back(dv);
        PYRE_HIP(ctx, hipMemcpy(dv, inv.data(), inv.size() * 4, hipMemcpyHostToDevice)); L.gdn_ainv = dv;
      }
    }
    MoeDev& mo = L.moe; size_t router_b = 0, ge = 0, ue = 0, de = 0, sh = 0;
    // the expert matrices in the lane = row layout the decode and window kernels walk and, unless PYRE_PROMPT_BLOCK=0, once more in
    // the matrix-core layout a long prompt's blocks use (4.25 bit/weight on top of the first layout's bytes)
    const int elay = prompt_block_env() ? PYRE_LAYOUT_BOTH : PYRE_LAYOUT_ROWS;
    if ((rc = B.one(T[PYRE_T_FFN_GATE_INP], &mo.router, &router_b)) || (rc = B.one(T[PYRE_T_FFN_GATE_EXPS], &mo.gate_e, &ge, elay, &mo.gate_m)) || (rc = B.one(T[PYRE_T_FFN_UP_EXPS], &mo.up_e, &ue, elay, &mo.up_m)) ||
        (rc = B.one(T[PYRE_T_FFN_DOWN_EXPS], &mo.down_e, &de, elay, &mo.down_m)) || (rc = B.one(T[PYRE_T_FFN_GATE_SHEXP], &mo.sh_gate, &sh, elay, &mo.sh_gate_m)) || (rc = B.one(T[PYRE_T_FFN_UP_SHEXP], &mo.sh_up, &sh, elay, &mo.sh_up_m)) ||
        (rc = B.one(T[PYRE_T_FFN_DOWN_SHEXP], &mo.sh_down, &sh, elay, &mo.sh_down_m))) return rc;
    mo.d = c.d; mo.n_exp = c.n_exp; mo.top_k = c.top_k; mo.ff = c.ff_exp; mo.sf = mo.sh_gate.rows;
    if (mo.router.rows != c.n_exp || mo.router.cols != c.d || mo.gate_e.rows != c.n_exp * c.ff_exp || mo.up_e.rows != c.n_exp * c.ff_exp || mo.gate_e.cols != c.d || mo.up_e.cols != c.d ||
        (size_t)mo.down_e.rows != (size_t)c.n_exp * c.d || mo.down_e.cols != c.ff_exp || mo.sh_up.rows != mo.sf || mo.sh_down.rows != c.d || mo.sh_down.cols != mo.sf || c.ff_exp % 64 || mo.sf % 64)
      return B.fail(PYRE_E_SHAPE, "expert tensor shapes");
    if (mo.gate_e.fmt != mo.up_e.fmt || mo.sh_gate.fmt != mo.gate_e.fmt || mo.sh_up.fmt != mo.gate_e.fmt || mo.sh_down.fmt != mo.down_e.fmt) return B.fail(PYRE_E_TYPE, "gate/up (and shared) expert types must agree");
    if ((rc = B.vec(T[PYRE_T_FFN_GATE_INP_SHEXP], c.d, &mo.sh_gate_inp))) return rc;
    tok_bytes += router_b + sh + (ge + ue + de) / c.n_exp * c.top_k;
  }
  if (m->n_ple > 0) {
    if (c.ple_ngram > 8 || c.ple_per_gram < 1 || (c.ple_ngram - 1) * c.ple_per_gram > 16 || c.ple_conv_k < 1 || c.ple_conv_k > 64 || c.ple_dim < 64 || c.ple_dim % 64)
      return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_model_create: PLE with n-grams of %d, %d heads per length, conv kernel %d, rows of %d is unsupported", c.ple_ngram, c.ple_per_gram, c.ple_conv_k, c.ple_dim);
    if ((rc = B.one(gl[PYRE_G_PLE_TOKEN_EMBD], &m->ple_tab, nullptr))) return rc;
    m->plc.ngram = c.ple_ngram; m->plc.per_gram = c.ple_per_gram; m->plc.conv_k = c.ple_conv_k; m->plc.dim = c.ple_dim; m->plc.eos = c.ple_eos;
    for (int i = 0; i < 8; ++i) m->plc.mult[i] = c.ple_mult[i];
    for (int i = 0; i < 16; ++i) { m->plc.off[i] = c.ple_off[i]; m->plc.vocab[i] = c.ple_vocab[i]; }
    for (int h = 0; h < (c.ple_ngram - 1) * c.ple_per_gram; ++h) if (c.ple_vocab[h] == 0 || c.ple_off[h] + c.ple_vocab[h] > (uint64_t)m->ple_tab.rows) return B.fail(PYRE_E_SHAPE, "a PLE head's rows lie outside per_layer_token_embd");
    if (m->ple_tab.cols != c.ple_dim) return B.fail(PYRE_E_SHAPE, "per_layer_token_embd row width");
    int ring = 16; while (ring < (c.ple_conv_k - 1) * c.ple_ngram + 8) ring *= 2; m->ple_ring = ring;
    tok_bytes += (size_t)(c.ple_ngram - 1) * c.ple_per_gram * (c.ple_dim / m->ple_tab.gel * m->ple_tab.gbytes);
  }
  if ((rc = B.one(gl[PYRE_G_TOKEN_EMBD], &m->embd, nullptr, mlay))) return rc;
  if (m->embd.rows != c.vocab || m->embd.cols != c.d) return B.fail(PYRE_E_SHAPE, "token_embd shape");
  if ((rc = B.hc(gl[PYRE_G_OUTPUT_HC_NORM], gl[PYRE_G_OUTPUT_HC_DOWN], nullptr, gl[PYRE_G_OUTPUT_HC_UP], &m->head, &tok_bytes))) return rc;
  if ((rc = B.one(gl[PYRE_G_OUTPUT], &m->out, &tok_bytes, mlay))) return rc;
  if (m->out.rows != c.vocab || m->out.cols != c.d) return B.fail(PYRE_E_SHAPE, "output shape");
  tok_bytes += (size_t)c.d / m->embd.gel * m->embd.gbytes;
  m->token_weight_bytes = tok_bytes;
  int kmax = 0;
  if ((rc = model_alloc_work(ctx, m, &kmax))) return rc;
  { uint4* op; float* ainv;      // and the context's operand buffer for a GEMV whose producer leaves f32 only, so that no step allocates
    if ((rc = pyre_gemm_m_scratch(ctx, (kmax + 255) / 256 * 256, &op, &ainv))) return rc; }
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  guard.armed = false; *out = M.release(); return PYRE_OK;
}

void pyre_model_destroy(pyre_model* m) {
  if (!m) return; (void)hipSetDevice(m->ctx->device); (void)hipStreamSynchronize(m->ctx->stream);
  prompt_pipe_free(m->pipe);
  for (auto q : m->owned) pyre_qmat_destroy(q); for (auto b : m->bufs) (void)hipFree(b); if (m->work) (void)hipFree(m->work); if (m->toks) (void)hipFree(m->toks);
  delete m;
}
size_t pyre_model_weight_bytes_per_token(const pyre_model* m) { return m ? m->token_weight_bytes : 0; }
size_t pyre_model_prompt_blocks(const pyre_model* m) { return m && m->pipe ? prompt_pipe_blocks(m->pipe) : 0; }

int pyre_state_create(pyre_ctx* ctx, const pyre_model* m, int max_ctx, pyre_state** out) {
  if (!ctx || !m || !out || max_ctx < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_create: bad argument");
  *out = nullptr; const pyre_model_cfg& c = m->c;
  std::unique_ptr<pyre_state> S(new pyre_state()); pyre_state* s = S.get(); s->ctx = ctx; s->m = m; s->cap = (max_ctx + 8 + 255) / 256 * 256;
  size_t cs = al256((size_t)(c.conv_k - 1) * m->ch * 4), ss = al256((size_t)c.lin_nv * c.lin_dk * c.lin_dv * 4), ps = al256((size_t)8 * m->pw_lin * 4);
  AttnDev a0{nullptr, nullptr, nullptr, c.n_head, c.n_kv, c.hd, c.n_rot, c.kv_bits, c.kv_recent, c.eps};
  size_t kvb = al256(pyre_kv_bytes(a0, s->cap)), awb = al256(pyre_attn_work_bytes(a0, s->cap));
  QsaDev q0{nullptr, nullptr, m->has_idx ? c.idx_nh : 0, c.idx_hd, c.idx_ratio < 1 ? 1 : c.idx_ratio, c.idx_budget};
  size_t qbb = al256(pyre_qsa_buf_bytes(q0, s->cap)), qwb = al256(pyre_qsa_work_bytes(q0, s->cap));
  const size_t tkb = m->n_ple > 0 ? al256((size_t)s->cap * 4) : 0, prb = m->n_ple > 0 ? al256((size_t)m->ple_ring * c.hc * c.d * 4) : 0;
  size_t total = (size_t)m->n_lin * (2 * cs + 2 * ss + ps) + (size_t)m->n_attn * (kvb + qbb) + awb + qwb + tkb + (size_t)m->n_ple * prb + 4096 + 256;
  hipError_t e = hipMalloc(&s->mem, total);
  if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_state_create: hipMalloc(%zu): %s", total, hipGetErrorString(e));
  uint8_t* p = (uint8_t*)s->mem; auto take = [&](size_t n) { void* r = p; p += n; return r; };
  for (int li = 0; li < m->n_lin; ++li) { for (int b = 0; b < 2; ++b) { s->conv[b].push_back((float*)take(cs)); s->ssm[b].push_back((float*)take(ss)); } s->proj_saved.push_back((float*)take(ps)); s->cur.push_back(0); }
  for (int ai = 0; ai < m->n_attn; ++ai) { KvDev kv; pyre_kv_carve(a0, s->cap, take(kvb), &kv); s->kv.push_back(kv); s->packed.push_back(0); }
  pyre_attn_work_carve(a0, s->cap, take(awb), &s->aw);
  if (m->has_idx) { for (int ai = 0; ai < m->n_attn; ++ai) { QsaBuf qb; pyre_qsa_buf_carve(q0, s->cap, take(qbb), &qb); s->qsa.push_back(qb); } pyre_qsa_work_carve(q0, s->cap, take(qwb), &s->qw); }
  if (m->n_ple > 0) { s->tokens_dev = (uint32_t*)take(tkb); for (int pi = 0; pi < m->n_ple; ++pi) s->ple_ring.push_back((float*)take(prb)); }
  s->step_dev = (int*)take(256);
  int rc = pyre_state_reset(ctx, s); if (rc) { (void)hipFree(s->mem); return rc; }
  *out = S.release(); return PYRE_OK;
}
void pyre_state_destroy(pyre_state* s) { if (!s) return; (void)hipStreamSynchronize(s->ctx->stream); if (s->graph_exec) (void)hipGraphExecDestroy(s->graph_exec); (void)hipFree(s->mem); if (s->mtp_mem) (void)hipFree(s->mtp_mem); if (s->pipe_mem) (void)hipFree(s->pipe_mem); delete s; }
int pyre_state_reset(pyre_ctx* ctx, pyre_state* s) {
  if (!ctx || !s) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_reset: null argument");
  const pyre_model_cfg& c = s->m->c; size_t cs = (size_t)(c.conv_k - 1) * s->m->ch * 4, ss = (size_t)c.lin_nv * c.lin_dk * c.lin_dv * 4;
  for (size_t li = 0; li < s->cur.size(); ++li) { s->cur[li] = 0; PYRE_HIP(ctx, hipMemsetAsync(s->conv[0][li], 0, cs, ctx->stream)); PYRE_HIP(ctx, hipMemsetAsync(s->ssm[0][li], 0, ss, ctx->stream)); }
  for (auto& pk : s->packed) pk = 0;
  s->len = 0; s->last_window = 0; s->r_first = s->r_next = 0; s->m_c0 = s->m_n = 0; s->broken = false; PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_state_len(const pyre_state* s) { return s ? s->len : 0; }
int pyre_state_capacity(const pyre_state* s) { return s ? s->cap - 8 : 0; }
int pyre_model_max_window(const pyre_model* m) { return m ? 8 : 0; }

// ---- snapshot / restore (Model::snapshot / restore, qwen4exp_gguf.rs:3277-3298), device resident ---------------------------
// A snapshot holds the recurrent state of every DeltaNet layer and the first `len` positions of every attention
// layer's cache (f32 and 4-bit planes; the key planes are blocked by 64 positions, so a prefix of blocks is contiguous
// whatever the capacity).  It can be restored into any state of the same model with room for `len` positions.
struct pyre_snap { const pyre_model* m; int len; std::vector<int> packed; void* mem; size_t bytes; };
namespace {
struct SnapPlan { size_t cs, ss, kf, ks_kq, kq, ksc, vf, vq, vsc, ik, ib, tk, pl, total; };
SnapPlan snap_plan(const pyre_model* m, int len) {
  const pyre_model_cfg& c = m->c; SnapPlan p{};
  const size_t row = (size_t)c.n_kv * c.hd, nb = ((size_t)len + 63) / 64;
  p.cs = al256((size_t)(c.conv_k - 1) * m->ch * 4); p.ss = al256((size_t)c.lin_nv * c.lin_dk * c.lin_dv * 4);
  p.kf = al256(nb * row * 64 * 4); p.kq = al256(nb * (row / 8) * 64 * 4); p.ksc = al256(nb * (row / 32) * 64 * 4);
  p.vf = al256((size_t)len * row * 4); p.vq = al256((size_t)len * (row / 8) * 4); p.vsc = al256((size_t)len * (row / 32) * 4);
  if (m->has_idx) { p.ik = al256((size_t)len * c.idx_hd * 4); p.ib = al256(((size_t)len / c.idx_ratio + 63) / 64 * 64 * c.idx_hd * 4); }      // raw index keys; pooled block keys in whole groups of 64 blocks
  if (m->n_ple > 0) { p.tk = al256((size_t)len * 4 + 4); p.pl = al256((size_t)(c.ple_conv_k - 1) * c.ple_ngram * c.hc * c.d * 4 + 4); }      // token history; per PLE layer the conv history
  p.total = (size_t)m->n_lin * (p.cs + p.ss) + (size_t)m->n_attn * (p.kf + p.kq + p.ksc + p.vf + p.vq + p.vsc + p.ik + p.ib) + p.tk + (size_t)m->n_ple * p.pl + 256;
  return p;
}
// dir = 0: state -> snapshot buffer, 1: snapshot buffer -> state
int snap_copy(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, uint8_t* buf, int len, int dir) {
  const SnapPlan p = snap_plan(m, len); uint8_t* q = buf;
  auto cp = [&](void* st, size_t n) -> hipError_t { hipError_t e = dir == 0 ? hipMemcpyAsync(q, st, n, hipMemcpyDeviceToDevice, ctx->stream) : hipMemcpyAsync(st, q, n, hipMemcpyDeviceToDevice, ctx->stream); return e; };
  const pyre_model_cfg& c = m->c; const size_t row = (size_t)c.n_kv * c.hd, nb = ((size_t)len + 63) / 64;
  for (int li = 0; li < m->n_lin; ++li) {
    int b = s->cur[li];
    PYRE_HIP(ctx, cp(s->conv[b][li], (size_t)(c.conv_k - 1) * m->ch * 4)); q += p.cs;
    PYRE_HIP(ctx, cp(s->ssm[b][li], (size_t)c.lin_nv * c.lin_dk * c.lin_dv * 4)); q += p.ss;
  }
  for (int ai = 0; ai < m->n_attn; ++ai) {
    KvDev& kv = s->kv[ai];
    if (len > 0) {
      PYRE_HIP(ctx, cp(kv.kf, nb * row * 64 * 4)); q += p.kf; PYRE_HIP(ctx, cp(kv.kq, nb * (row / 8) * 64 * 4)); q += p.kq; PYRE_HIP(ctx, cp(kv.ks, nb * (row / 32) * 64 * 4)); q += p.ksc;
      PYRE_HIP(ctx, cp(kv.vf, (size_t)len * row * 4)); q += p.vf; PYRE_HIP(ctx, cp(kv.vq, (size_t)len * (row / 8) * 4)); q += p.vq; PYRE_HIP(ctx, cp(kv.vs, (size_t)len * (row / 32) * 4)); q += p.vsc;
    } else q += p.kf + p.kq + p.ksc + p.vf + p.vq + p.vsc;
    if (m->has_idx) {
      if (len > 0) { PYRE_HIP(ctx, cp(s->qsa[ai].ik, (size_t)len * c.idx_hd * 4)); }
      q += p.ik;
      size_t ibn = ((size_t)len / c.idx_ratio + 63) / 64 * 64 * c.idx_hd * 4;
      if (ibn) { PYRE_HIP(ctx, cp(s->qsa[ai].ib, ibn)); }
      q += p.ib;
    }
  }
  if (m->n_ple > 0) {
    if (len > 0) { PYRE_HIP(ctx, cp(s->tokens_dev, (size_t)len * 4)); }
    q += p.tk;
    const size_t wb = (size_t)c.hc * c.d * 4; const int hl = (c.ple_conv_k - 1) * c.ple_ngram;
    for (int pi = 0; pi < m->n_ple; ++pi) {      // the rows of the last hl positions, oldest first (positions before 0 have no row)
      uint8_t* q0 = q;
      for (int j = 0; j < hl; ++j) { const int pos = len - hl + j; if (pos >= 0) { q = q0 + (size_t)j * wb; PYRE_HIP(ctx, cp(s->ple_ring[pi] + (size_t)(pos & (m->ple_ring - 1)) * c.hc * c.d, wb)); } }
      q = q0 + p.pl;
    }
  }
  return PYRE_OK;
}
}  // namespace
int pyre_state_snapshot(pyre_ctx* ctx, pyre_state* s, pyre_snap** out) {
  if (!ctx || !s || !out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_snapshot: null argument");
  *out = nullptr;
  if (s->broken) return pyre_fail(ctx, PYRE_E_STATE, "%s: an earlier call failed half way through this state; pyre_state_reset or pyre_state_restore first", "pyre_state_snapshot");
  std::unique_ptr<pyre_snap> sn(new pyre_snap()); sn->m = s->m; sn->len = s->len; sn->packed = s->packed; sn->bytes = snap_plan(s->m, s->len).total; sn->mem = nullptr;
  hipError_t e = hipMalloc(&sn->mem, sn->bytes);
  if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_state_snapshot: hipMalloc(%zu): %s", sn->bytes, hipGetErrorString(e));
  int rc = snap_copy(ctx, s->m, s, (uint8_t*)sn->mem, s->len, 0);
  hipError_t e2 = hipStreamSynchronize(ctx->stream);
  if (rc || e2 != hipSuccess) { (void)hipFree(sn->mem); return rc ? rc : pyre_fail(ctx, PYRE_E_HIP, "pyre_state_snapshot: %s", hipGetErrorString(e2)); }
  *out = sn.release(); return PYRE_OK;
}
int pyre_state_restore(pyre_ctx* ctx, pyre_state* s, const pyre_snap* sn) {
  if (!ctx || !s || !sn) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_restore: null argument");
  if (s->m != sn->m) return pyre_fail(ctx, PYRE_E_STATE, "pyre_state_restore: the snapshot belongs to another model");
  if (sn->len + 8 > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "pyre_state_restore: %d positions do not fit the state's capacity %d", sn->len, s->cap - 8);
  int rc = snap_copy(ctx, s->m, s, (uint8_t*)sn->mem, sn->len, 1); if (rc) return rc;
  s->len = sn->len; s->packed = sn->packed; s->last_window = 0; s->r_first = s->r_next = 0; s->m_c0 = s->m_n = 0; s->broken = false;      // the drafter starts over
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
void pyre_snap_destroy(pyre_snap* sn) { if (!sn) return; (void)hipFree(sn->mem); delete sn; }
size_t pyre_snap_bytes(const pyre_snap* sn) { return sn ? sn->bytes : 0; }
int pyre_snap_len(const pyre_snap* sn) { return sn ? sn->len : 0; }
int pyre_state_read_gdn(pyre_ctx* ctx, pyre_state* s, int li, float* conv_host, float* ssm_host) {
  if (!ctx || !s || li < 0 || li >= (int)s->cur.size()) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_read_gdn: bad layer");
  const pyre_model_cfg& c = s->m->c; int b = s->cur[li];
  if (conv_host) PYRE_HIP(ctx, hipMemcpyAsync(conv_host, s->conv[b][li], (size_t)(c.conv_k - 1) * s->m->ch * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (ssm_host) PYRE_HIP(ctx, hipMemcpyAsync(ssm_host, s->ssm[b][li], (size_t)c.lin_nv * c.lin_dk * c.lin_dv * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_state_read_ple(pyre_ctx* ctx, pyre_state* s, int pi, float* hist_host) {
  if (!ctx || !s || !hist_host || pi < 0 || pi >= (int)s->ple_ring.size()) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_read_ple: bad argument");
  const pyre_model_cfg& c = s->m->c; const size_t w = (size_t)c.hc * c.d; const int hl = (c.ple_conv_k - 1) * c.ple_ngram;
  for (int j = 0; j < hl; ++j) {
    const int pos = s->len - hl + j;
    if (pos < 0) memset(hist_host + (size_t)j * w, 0, w * 4);
    else PYRE_HIP(ctx, hipMemcpyAsync(hist_host + (size_t)j * w, s->ple_ring[pi] + (size_t)(pos & (s->m->ple_ring - 1)) * w, w * 4, hipMemcpyDeviceToHost, ctx->stream));
  }
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_state_read_kv(pyre_ctx* ctx, pyre_state* s, int ai, float* k_host, float* v_host) {
  if (!ctx || !s || ai < 0 || ai >= (int)s->kv.size() || !k_host || !v_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_read_kv: bad argument");
  const pyre_model_cfg& c = s->m->c; size_t row = (size_t)c.n_kv * c.hd; std::vector<float> kt(row * s->cap);
  PYRE_HIP(ctx, hipMemcpyAsync(kt.data(), s->kv[ai].kf, kt.size() * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipMemcpyAsync(v_host, s->kv[ai].vf, (size_t)s->len * row * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  for (int p = 0; p < s->len; ++p) for (size_t cc = 0; cc < row; ++cc) k_host[(size_t)p * row + cc] = kt[kv_blk(cc, row, p)];
  return PYRE_OK;
}

}  // extern "C"

namespace {

}  // namespace

// A long prompt runs its windows on several streams at once: window w+1 may work on layer l as soon as window w has left
// that layer's state (an event per layer), each stream with a window workspace of its own -- a shallow copy of the model
// whose activations are separate -- and an attention workspace of its own in the state.  The launches of a window of 8
// tokens leave most of the chip idle most of the time; two or three windows in flight fill it.  Arithmetic and order per
// window are unchanged, so the state and the logits are bit for bit those of one stream.
struct PromptPipe {
  std::vector<pyre_ctx*> ctx;                  // contexts of the further streams
  std::vector<pyre_model*> mdl;                // the model's shallow copies, one per further stream
  std::vector<std::vector<hipEvent_t>> ev;     // [set][layer]; set 0 is the model's own stream
  std::vector<hipEvent_t> done;                // [set] end of the set's last window
  hipEvent_t start = nullptr;
  uint32_t* ids = nullptr; size_t ids_cap = 0; // the call's token ids on the device
  // blocks of windows taken layer by layer with the FFN of all their tokens grouped by expert (prompt_block_get)
  std::vector<pyre_model*> wmdl;               // a window workspace per window of a block
  void* blk_mem = nullptr; MoeBlk blk[2]{}; int blk_nsl = 0, blk_r64 = 0;          // two blocks in flight: one's FFN beside the other's windows
  hipEvent_t moe_done[2] = {nullptr, nullptr}; std::vector<hipEvent_t> front_done[2]; size_t blocks_done = 0;
  pyre_ctx* moe_ctx = nullptr;                 // the stream of the blocks' FFN launches
  size_t win_stride = 0;                       // bytes between the workspaces of consecutive windows of a block
  void* qmem = nullptr; size_t q_stride = 0, q_off[2] = {0, 0};      // per window of a block: the rotated queries (f32, f16 halves, scales) of an attention layer, kept from the cache write to the pass over the cache
};
size_t prompt_pipe_blocks(const PromptPipe* P) { return P->blocks_done; }
static int prompt_streams() { static const int k = [] { const char* e = getenv("PYRE_PROMPT_STREAMS"); int v = e && *e ? atoi(e) : 3; return v < 1 ? 1 : (v > 4 ? 4 : v); }(); return k; }
void prompt_pipe_free(PromptPipe* P) {
  if (!P) return;
  for (auto* mc : P->mdl) if (mc) { (void)hipStreamSynchronize(mc->ctx->stream); if (mc->work) (void)hipFree(mc->work); delete mc; }
  for (auto* cx : P->ctx) if (cx) pyre_ctx_destroy(cx);
  for (auto& v : P->ev) for (auto e : v) if (e) (void)hipEventDestroy(e);
  for (auto e : P->done) if (e) (void)hipEventDestroy(e);
  if (P->start) (void)hipEventDestroy(P->start);
  if (P->ids) (void)hipFree(P->ids);
  for (auto* mc : P->wmdl) if (mc) { if (mc->work) (void)hipFree(mc->work); delete mc; }
  if (P->blk_mem) (void)hipFree(P->blk_mem);
  for (auto e : P->moe_done) if (e) (void)hipEventDestroy(e);
  for (auto& v : P->front_done) for (auto e : v) if (e) (void)hipEventDestroy(e);
  if (P->moe_ctx) pyre_ctx_destroy(P->moe_ctx);
  if (P->qmem) (void)hipFree(P->qmem);
  delete P;
}
static int prompt_pipe_get(pyre_ctx* ctx, const pyre_model* m, PromptPipe** out) {
  pyre_model* mm = const_cast<pyre_model*>(m);          // the workspaces are the model's, like its own activations
  if (mm->pipe) { *out = mm->pipe; return PYRE_OK; }
  const int k = prompt_streams();
  std::unique_ptr<PromptPipe, void (*)(PromptPipe*)> P(new PromptPipe(), prompt_pipe_free);
  for (int i = 1; i < k; ++i) {
    pyre_ctx* cx = nullptr; int rc = pyre_ctx_create(ctx->device, &cx); if (rc) return pyre_fail(ctx, rc, "prompt streams: %s", pyre_last_error(nullptr));
    P->ctx.push_back(cx);
    pyre_model* mc = new pyre_model(*m); mc->ctx = cx; mc->owned.clear(); mc->bufs.clear(); mc->work = nullptr; mc->toks = nullptr; mc->toks_cap = 0; mc->pipe = nullptr;
    P->mdl.push_back(mc);
    int kmax = 0; rc = model_alloc_work(cx, mc, &kmax);
    if (!rc) { uint4* op; float* ainv; rc = pyre_gemm_m_scratch(cx, (kmax + 255) / 256 * 256, &op, &ainv); }
    if (rc) return pyre_fail(ctx, rc, "prompt streams: %s", cx->err.c_str());
    PYRE_HIP(ctx, hipStreamSynchronize(cx->stream));
  }
  P->ev.resize(k); P->done.resize(k, nullptr);
  for (int i = 0; i < k; ++i) {
    P->ev[i].resize(m->c.n_layers, nullptr);
    for (auto& e : P->ev[i]) PYRE_HIP(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
    PYRE_HIP(ctx, hipEventCreateWithFlags(&P->done[i], hipEventDisableTiming));
  }
  PYRE_HIP(ctx, hipEventCreateWithFlags(&P->start, hipEventDisableTiming));
  mm->pipe = P.release(); *out = mm->pipe; return PYRE_OK;
}
// the state's further attention / selection workspaces (one per further stream)
static int prompt_pipe_state(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, int k) {
  if ((int)s->aw_more.size() >= k - 1) return PYRE_OK;
  const pyre_model_cfg& c = m->c;
  AttnDev a0{nullptr, nullptr, nullptr, c.n_head, c.n_kv, c.hd, c.n_rot, c.kv_bits, c.kv_recent, c.eps};
  QsaDev q0{nullptr, nullptr, m->has_idx ? c.idx_nh : 0, c.idx_hd, c.idx_ratio < 1 ? 1 : c.idx_ratio, c.idx_budget};
  const size_t awb = al256(pyre_attn_work_bytes(a0, s->cap)), qwb = al256(pyre_qsa_work_bytes(q0, s->cap));
  if (s->pipe_mem) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); (void)hipFree(s->pipe_mem); s->pipe_mem = nullptr; s->aw_more.clear(); s->qw_more.clear(); }
  PYRE_HIP(ctx, hipMalloc(&s->pipe_mem, (size_t)(k - 1) * (awb + qwb) + 256));
  uint8_t* p = (uint8_t*)s->pipe_mem;
  for (int i = 1; i < k; ++i) {
    AttnWork aw{}; pyre_attn_work_carve(a0, s->cap, p, &aw); p += awb; s->aw_more.push_back(aw);
    QsaWork qw{}; if (m->has_idx) pyre_qsa_work_carve(q0, s->cap, p, &qw); p += qwb; s->qw_more.push_back(qw);
  }
  return PYRE_OK;
}

// ---- a long prompt in blocks of windows, layer by layer ---------------------------------------------------------------------
// Windows of eight tokens share nothing in the FFN (eight tokens pick 74 of 512 experts), which makes the expert products
// the largest part of a prompt window.  A block of up to PROMPT_BLOCK_WINDOWS windows is therefore taken layer by layer: every
// window's part of the layer up to the FFN mix (on the prompt's streams, the layer's state passing from window to window as
// before), then the FFN of all of the block's tokens in one set of launches with the tokens grouped by expert, on the
// matrix cores (pyre_moe_block_launch), whose group sums the windows' next mixes read.  Everything but the FFN is the
// windows' kernels and arithmetic; the FFN's products are those of the matrix-core GEMM (f16 halves of the activations
// instead of fixed-point digits): equal to rounding, not bit for bit.  For models whose every layer qualifies
// (prompt_block_ok); the call's last tokens (the window whose logits are read, the rows a drafter keeps) take the windows'
// path.  PYRE_PROMPT_BLOCK=0 switches it off.
static int prompt_block_windows() { static const int k = [] { const char* e = getenv("PYRE_PROMPT_BLOCK_WINDOWS"); int v = e && *e ? atoi(e) : 128; return v < 8 ? 8 : (v > 128 ? 128 : v); }(); return k; }      // the most windows a block has (read once)
#define PROMPT_BLOCK_WINDOWS prompt_block_windows()
#define PROMPT_BLOCK_MIN 8
static bool fuse_aop_on() { const char* e = getenv("PYRE_AOP_SPLIT"); return !(e && *e && atoi(e) != 0); }
static bool prompt_block_ok(const pyre_model* m) {
  if (!prompt_block_env()) return false;
  { const char* r = getenv("PYRE_ROUTER_RIDES"); if (r && *r && atoi(r) == 0) return false; }
  { const char* r = getenv("PYRE_MOE_GROUPS"); if (r && *r && atoi(r) == 0) return false; }
  const pyre_model_cfg& c = m->c;
  if (m->n_ple > 0 || c.top_k > PYRE_MOE_KMAX || c.d % 256 || !fuse_aop_on()) return false;
  for (int il = 0; il < c.n_layers; ++il) { const Layer& L = m->layers[il];
    if (!pyre_moe_block_ok(L.moe) || !pyre_hc_route_ok(L.hcf, L.moe.router) || !pyre_hc_aop_ok(L.hcf) || L.hca.di.fmt != FMT_IQ3_S || L.moe.router.tiles != m->layers[0].moe.router.tiles ||
        L.moe.ff != m->layers[0].moe.ff || L.moe.sf != m->layers[0].moe.sf || L.moe.top_k != m->layers[0].moe.top_k || L.moe.n_exp != m->layers[0].moe.n_exp) return false; }
  return true;
}
static int prompt_block_get(pyre_ctx* ctx, const pyre_model* m, PromptPipe* P) {
  if (!P->wmdl.empty()) return PYRE_OK;
  const pyre_model_cfg& c = m->c; const int NB = PROMPT_BLOCK_WINDOWS, d = c.d, K = (int)P->ctx.size() + 1;
  const MoeDev& m0 = m->layers[0].moe;
  const int nsl = d / 64, r64 = m0.router.tiles * 64;
  // the windows' workspaces of both blocks in flight in one piece, a workspace every ws bytes: what a launch does for one
  // window it can do for the next ones at the same addresses + ws; the FFN's own scratch once (its launches share a stream)
  size_t aop_b = 0; const size_t ws = model_work_layout(const_cast<pyre_model*>(m), nullptr, nullptr, &aop_b), mb = al256(pyre_moe_block_bytes(m0, NB * 8));
  PYRE_HIP(ctx, hipMalloc(&P->blk_mem, 2 * (size_t)NB * ws + mb + 256));
  PYRE_HIP(ctx, hipMemsetAsync(P->blk_mem, 0, 2 * (size_t)NB * ws, ctx->stream));
  uint8_t* p = (uint8_t*)P->blk_mem;
  for (int w = 0; w < 2; ++w) for (int j = 0; j < NB; ++j) {
    pyre_model* mc = new pyre_model(*m); mc->owned.clear(); mc->bufs.clear(); mc->work = nullptr; mc->toks = nullptr; mc->toks_cap = 0; mc->pipe = nullptr;
    P->wmdl.push_back(mc);
    (void)model_work_layout(mc, p + ((size_t)w * NB + j) * ws, nullptr, nullptr);
  }
  pyre_moe_block_carve(m0, NB * 8, p + 2 * (size_t)NB * ws, &P->blk[0]);
  P->blk[1] = P->blk[0];
  for (int w = 0; w < 2; ++w) { const pyre_model* f = P->wmdl[(size_t)w * NB]; P->blk[w].x = f->mixed; P->blk[w].rpart = f->rpart; P->blk[w].parts = f->mw.parts; P->blk[w].ws = ws / 4; }
  P->blk_nsl = nsl; P->blk_r64 = r64; P->win_stride = ws;
  { int rc = pyre_moe_block_zero_rows(ctx, m0, P->blk[0], NB * 8); if (rc) return rc; }
  if (!m->has_idx) {      // (with a sparse indexer the selection and the pass stay together in the chain)
    const size_t nq = (size_t)8 * c.n_head * c.hd;
    P->q_off[0] = al256(4 * nq); P->q_off[1] = P->q_off[0] + al256(2 * 2 * nq); P->q_stride = P->q_off[1] + al256(4 * 8 * (size_t)c.n_head);
    PYRE_HIP(ctx, hipMalloc(&P->qmem, 2 * (size_t)NB * P->q_stride));
  }
  { int rc = pyre_ctx_create(ctx->device, &P->moe_ctx); if (rc) return pyre_fail(ctx, rc, "prompt blocks: %s", pyre_last_error(nullptr)); }
  for (int w = 0; w < 2; ++w) {
    PYRE_HIP(ctx, hipEventCreateWithFlags(&P->moe_done[w], hipEventDisableTiming));
    P->front_done[w].resize(K, nullptr);
    for (auto& e : P->front_done[w]) PYRE_HIP(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
  }
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return PYRE_OK;
}

namespace {

struct WinOpt {
  int head_tokens = 1;          // 0 = no logits, 1 = last token only, t = every token (rows 0..t-1 of m->logits)
  bool greedy = false;          // t == 1: the head GEMV also leaves per-tile maxima in m->best
  bool from_best = false;       // the token is picked from the previous step's maxima inside the embedding launch
  uint32_t* toks_out = nullptr; // where the picked id is mirrored
  int* step_dev = nullptr;      // replayable form: position and output slot live in device memory (see pyre_pick_launch);
                                // recurrent state is updated in place and no host-side bookkeeping is touched
  bool inplace = false;         // update the recurrent state in its current buffer (no pre-window copy for spec_keep)
  int keep_from = 0;            // with a drafter attached: the final residual streams of tokens keep_from .. t-1 go to the state's ring
  // a prompt window that shares the GPU with its neighbours (prompt_pipe): its ids, the attention / selection workspace
  // it uses instead of the state's, and per layer the event it waits for (the previous window has left the layer) and records
  const uint32_t* ids_dev = nullptr; const AttnWork* aw = nullptr; const QsaWork* qw = nullptr; const hipEvent_t* wait_ev = nullptr; const hipEvent_t* rec_ev = nullptr;
  int start = -1;               // the window's first position when the caller keeps the count (a block of windows taken layer by layer); -1: the state's length
  bool no_len = false;          // ... and the state's length is then advanced by the caller
  size_t win_stride = 0;        // bytes between this window's workspace and the next window's of its block (0: it stands alone)
  bool router_apart = false;    // a block's window: the router's K-slice sums come from the block's FFN launch, not from this window's FFN mix
  bool proj_early = false;      // a block's window: the layer's projection is launched with the mix in front of it (front_pre_proj), a Gated DeltaNet layer's convolution once for the group (front_mid_conv): neither needs the layer's state
  bool attn_split = false; AttnWork aw_own{};      // a block's window: the attention pass over the cache leaves the chain through the layer's state (front_post_proj runs it); aw_own: the stream's attention workspace with q buffers of this window's own
};

// rows `from` .. t-1 of the window's final residual streams x [t][w] into the ring at their positions; grid (ceil(w/256), t - from)
__global__ __launch_bounds__(256) void k_ring_store(const float* __restrict__ x, float* __restrict__ ring, int mask, int start, const int* __restrict__ posp, int from, int w) {
  if (posp) start = *posp;
  const int i = blockIdx.x * 256 + threadIdx.x, ti = from + blockIdx.y; if (i >= w) return;
  ring[(size_t)((start + ti) & mask) * w + i] = x[(size_t)ti * w + i];
}
int mtp_window_of(const pyre_mtp* m);

bool outp_in_parts(const Layer& L, int d) { return pyre_gemv_parts_ok(L.outp) && (int)L.outp.rows == d && L.hcf.di.fmt == FMT_IQ3_S; }

// One window of t <= 8 tokens (ids in m->ids unless from_best).
// A Gated DeltaNet layer whose output projection is on the matrix cores runs its recurrence on nv x 4 workgroups and leaves
// the head norm to that projection (GdnQ / PyreAop::sq) -- in every call that touches the layer's state, the re-run of
// pyre_spec_keep included: the two forms of the kernel round the state differently.  PYRE_GDN_Q=0: nv workgroups.
static bool gdn_q_on(const pyre_model* m, const Layer& L) {
  const char* e = getenv("PYRE_GDN_Q");
  return !(e && *e && atoi(e) == 0) && fuse_aop_on() && !L.full && L.outp.fmt == FMT_IQ3_S_M && L.gdn.dv == 128 && L.gdn.dk == 128 && L.outp.cols == L.gdn.nv * 128 && m->gdn_sq != nullptr;
}
// One window of t <= 8 tokens as an object, so that a block of prompt windows can be taken layer by layer: begin() (embedding
// rows, history, n-gram rows), per layer front(il) (everything up to the FFN mix, whose output is the FFN's input) and
// moe(il) (the FFN; the block path runs pyre_moe_block_launch for all of its windows instead and calls moe_from_block),
// finish() (bookkeeping, head).  run_window is the four in order.
struct WinRun {
  pyre_ctx* ctx; const pyre_model* m; pyre_state* s; int t; WinOpt o;
  int start = 0; bool replay = false;
  const float* xin = nullptr; int in_ss = 0, in_ts = 0; float* xout = nullptr; float* xother = nullptr;
  MoeOut mo{}; const MoeOut* comb_moe = nullptr; const float* comb_out = nullptr; const float* comb_inj = nullptr;
  int comb_np = 1;          // vectors the pending update comes in: 1, or PYRE_GEMV_PARTS == PYRE_MOE_GROUPS to be added in order
  bool raw_moe = false, moe_groups = true, route_rides = true, fuse_aop = true, ride = false;
  WinRun(pyre_ctx* c, const pyre_model* mm, pyre_state* ss, int tt, const WinOpt& oo) : ctx(c), m(mm), s(ss), t(tt), o(oo) {}
  void advance() { xin = xout; in_ss = m->c.d; in_ts = m->c.hc * m->c.d; float* q = xout; xout = xother; xother = q; }
  bool hc_fused(const HcDev& h, const QMatDev& q) const { const int d = m->c.d; return fuse_aop && q.fmt == FMT_IQ3_S_M && q.cols == d && d % 256 == 0 && pyre_hc_aop_ok(h); }
  bool gdn_fused(const Layer& L) const { return fuse_aop && L.outp.fmt == FMT_IQ3_S_M && L.gdn_ainv != nullptr; }
  int begin() {
    const pyre_model_cfg& c = m->c; const int d = c.d;
    start = o.start >= 0 ? o.start : s->len; replay = o.step_dev != nullptr;
    if (start + t > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "forward: context %d exceeds the state's capacity %d", start + t, s->cap);
    const uint32_t* ids = o.ids_dev ? o.ids_dev : m->ids;
    int rc = o.from_best ? pyre_pick_launch(ctx, m->best, pyre_gemv_best_count(m->out), m->ids, o.toks_out, &m->embd, m->emb, o.step_dev, s->tokens_dev) : pyre_row_launch(ctx, m->embd, ids, t, m->emb, d); if (rc) return rc;
    // the residual streams alternate between two buffers: every mix reads one (first the embedding row, replicated) and
    // leaves the updated streams in the other
    xin = m->emb; in_ss = 0; in_ts = d; xout = m->x; xother = m->x2;
    raw_moe = c.top_k <= PYRE_MOE_KMAX;        // the next mix folds the unreduced FFN output itself (same arithmetic as k_moe_sum, one launch fewer per layer)
    moe_groups = [] { const char* e = getenv("PYRE_MOE_GROUPS"); return !(e && *e && atoi(e) == 0); }();      // 0: windows leave the unreduced terms as a single token does
    route_rides = [] { const char* e = getenv("PYRE_ROUTER_RIDES"); return !(e && *e && atoi(e) == 0); }();      // 0: separate router launch (what the persistent kernel mirrors)
    // the window's tokens join the history (PLE models and states with a drafter keep one)
    if (s->tokens_dev && !o.from_best && !o.ids_dev) PYRE_HIP(ctx, hipMemcpyAsync(s->tokens_dev + start, ids, (size_t)t * 4, hipMemcpyDeviceToDevice, ctx->stream));      // (a prompt on several streams has stored the whole call's ids already)
    if (m->n_ple > 0) {      // every position's n-gram rows are fetched once for all PLE layers
      if ((rc = pyre_ple_rows_launch(ctx, m->plc, m->ple_tab, m->pw, s->tokens_dev, start, o.step_dev, t))) return rc;
    }
    fuse_aop = fuse_aop_on();      // PYRE_AOP_SPLIT=1: separate split launches instead of the producers' own operand stores
    return PYRE_OK;
  }
  // whether layer il's FFN output of a window of several tokens goes to the next mix as four group sums a token: when that mix
  // can add partial vectors (an IQ3_S mix over all of the window's tokens, no PLE layer in between); otherwise, and for a
  // single token, unreduced
  bool groups_at(int il) const {
    const pyre_model_cfg& c = m->c; const Layer& L = m->layers[il];
    bool groups = raw_moe && t > 1 && moe_groups && pyre_moe_groups_ok(L.moe);
    if (groups) {
      if (il + 1 < c.n_layers) { const Layer& Ln = m->layers[il + 1]; groups = !Ln.ple && Ln.hca.di.fmt == FMT_IQ3_S; }
      else groups = (o.head_tokens >= t || (s->mtp && o.keep_from < t)) && m->head.di.fmt == FMT_IQ3_S;
    }
    return groups;
  }
  // A layer up to its FFN in three parts: the mix in front of the layer's state (pre), what reads and writes that state --
  // projection with its convolution and the recurrence, or projection and attention -- (mid), the output projection and the FFN
  // mix (post).  Only mid follows the previous window's mid; front() is the three in a row with the events around mid.
  // nz: windows this launch serves (this one and the nz - 1 after it, their workspaces o.win_stride bytes apart); 0: none -- a
  // launch of an earlier window of the group has served this one, only the bookkeeping is left
  int front_pre(int il, int nz = 1) {
    const pyre_model_cfg& c = m->c; const int d = c.d, hc = c.hc; int rc;
    const AopOut aout{m->aop, m->aop_inv, d / 256};
    auto opw = [&](const HcDev& h, const QMatDev& q) -> const AopOut* { return hc_fused(h, q) ? &aout : nullptr; };
    const Layer& L = m->layers[il];
    if (L.ple) {      // resolves the pending residual update itself and leaves plain streams
      PleDev pd = L.pld; pd.ring = s->ple_ring[L.ple_index]; pd.mask = m->ple_ring - 1;
      if ((rc = pyre_ple_launch(ctx, m->plc, pd, m->pw, d, hc, c.eps, xin, in_ss, in_ts, xout, comb_out, comb_moe, comb_inj, start, o.step_dev, t))) return rc;
      advance(); comb_out = nullptr; comb_moe = nullptr; comb_inj = nullptr;
    }
    // the mix that produces a matrix-core GEMV's input also leaves it as that GEMV's f16 operand, every token scaled by a power of
    // two (AopOut); the Gated DeltaNet step likewise with a constant of the layer; the attention output goes through the GEMV's
    // own split launch (its magnitude has no bound a single workgroup of the merge could form)
    if (nz > 0) {
      ctx->batch_n = nz; ctx->batch_stride = nz > 1 ? o.win_stride : 0;
      rc = pyre_hc_mix_launch(ctx, L.hca, m->hw, xin, in_ss, in_ts, xout, t, comb_out, comb_moe, comb_inj, c.eps, m->mixed, m->inj_a, nullptr, comb_np, opw(L.hca, L.proj));
      ctx->batch_n = 1; ctx->batch_stride = 0;
      if (rc) return rc;
    }
    advance(); comb_np = 1;
    return PYRE_OK;
  }
  // whether one launch of layer il's projection / output projection can serve several windows: the operand comes from the
  // window's own workspace (the mix's, the recurrence's per-quarter form), not through the context's split buffer
  bool proj_batchable(int il) const { const Layer& L = m->layers[il]; return hc_fused(L.hca, L.proj); }
  bool outp_batchable(int il) const { const Layer& L = m->layers[il]; return L.outp.fmt == FMT_IQ3_S_M && (L.full ? (o.attn_split && L.outp.cols % 256 == 0) : gdn_q_on(m, L)); }
  int front_pre_proj(int il, int nz = 1) {          // (proj_early) the layer's projection, without the convolution (nz as in front_pre)
    const Layer& L = m->layers[il]; if (nz <= 0) return PYRE_OK;
    const PyreAop aop_hc{(const uint4*)m->aop, m->aop_inv};
    ctx->batch_n = nz; ctx->batch_stride = nz > 1 ? o.win_stride : 0;
    const int rc = pyre_gemv_launch(ctx, L.proj, m->mixed, t, m->proj, hc_fused(L.hca, L.proj) ? &aop_hc : nullptr);
    ctx->batch_n = 1; ctx->batch_stride = 0;
    return rc;
  }
  // (proj_early) the convolution of this window and the n - 1 after it, a Gated DeltaNet layer: the history in front of this
  // window is the layer's state (first: the block's first window) or the last rows of the window before it; the last window
  // of the block leaves the state where the windows' recurrences will have turned the layer's buffers to
  int front_mid_conv(int il, int n, bool first, bool last, int flips) {          // flips: turns of the layer's state buffers between here and the end of these windows' recurrences
    const pyre_model_cfg& c = m->c; const Layer& L = m->layers[il]; if (L.full) return PYRE_OK;
    const int li = L.mix_index, b = s->cur[li], K1 = c.conv_k - 1;
    const float* prev = first ? s->conv[b][li] : m->proj - o.win_stride / 4 + (size_t)(t - K1) * m->pw_lin;
    return pyre_gdn_conv_block_launch(ctx, L.gdn, m->proj, m->pw_lin, t, n, o.win_stride / 4, prev, first ? m->ch : m->pw_lin, last ? s->conv[b ^ (flips & 1)][li] : nullptr, m->co);
  }
  // (proj_early, attn_split) the cache write of this window and the n - 1 after it, an attention layer, in one launch (and one packing step)
  int front_mid_attn(int il, int n, size_t q_stride) {
    const Layer& L = m->layers[il]; const int ai = L.mix_index;
    ctx->batch_n = n; ctx->batch_stride = n > 1 ? o.win_stride : 0; ctx->batch_stride2 = n > 1 ? q_stride : 0;
    const int rc = pyre_attn_launch_sel(ctx, L.attn, s->kv[ai], o.aw_own, m->proj, m->pw_attn, start, t, &s->packed[ai], m->core, nullptr, nullptr, 1);
    ctx->batch_n = 1; ctx->batch_stride = 0; ctx->batch_stride2 = 0;
    return rc;
  }
  // (proj_early) the recurrence of this window and the n - 1 after it in one launch: the state stays in registers from window to window
  bool gdn_group_ok(int il) const { const Layer& L = m->layers[il]; return !L.full && gdn_q_on(m, L); }
  int front_mid_gdn(int il, int n) {
    const Layer& L = m->layers[il]; const int li = L.mix_index, b = s->cur[li], nb = b ^ 1;
    const GdnQ gq{m->aop, m->gdn_sq};
    int rc = pyre_gdn_launch(ctx, L.gdn, m->proj, m->pw_lin, t, s->conv[b][li], s->conv[nb][li], s->ssm[b][li], s->ssm[nb][li], m->co, m->core, true, nullptr, L.gdn_up, &gq, n, o.win_stride / 4);
    if (rc) return rc;
    s->cur[li] = nb;
    return PYRE_OK;
  }
  int front_mid(int il) {
    const pyre_model_cfg& c = m->c; int rc;
    const AttnWork& aw = o.attn_split ? o.aw_own : (o.aw ? *o.aw : s->aw); const QsaWork& qw = o.qw ? *o.qw : s->qw;
    const PyreAop aop_hc{(const uint4*)m->aop, m->aop_inv};
    auto opnd = [&](const HcDev& h, const QMatDev& q) -> const PyreAop* { return hc_fused(h, q) ? &aop_hc : nullptr; };
    const Layer& L = m->layers[il];
    if (L.full) {
      int ai = L.mix_index;
      if (!o.proj_early && (rc = pyre_gemv_launch(ctx, L.proj, m->mixed, t, m->proj, opnd(L.hca, L.proj)))) return rc;
      if (m->has_idx && (rc = pyre_qsa_launch(ctx, L.qsa, L.attn, s->qsa[ai], qw, m->proj, m->pw_attn, m->iq_off, start, t, o.step_dev))) return rc;
      if ((rc = pyre_attn_launch_sel(ctx, L.attn, s->kv[ai], aw, m->proj, m->pw_attn, start, t, &s->packed[ai], m->core, o.step_dev, m->has_idx ? &qw : nullptr, o.attn_split ? 1 : 0))) return rc;
    } else {
      int li = L.mix_index; float* pj = o.proj_early ? m->proj : s->proj_saved[li]; int b = s->cur[li], nb = (replay || o.inplace) ? b : b ^ 1;
      GemvEpi cv{nullptr, L.gdn.conv_w, s->conv[b][li], s->conv[nb][li], m->co, m->ch, c.conv_k};      // conv1d + SiLU ride on the projection
      if (!o.proj_early && (rc = pyre_gemv_conv_launch(ctx, L.proj, m->mixed, t, pj, cv, opnd(L.hca, L.proj)))) return rc;
      const GdnQ gq{m->aop, m->gdn_sq};
      if ((rc = pyre_gdn_launch(ctx, L.gdn, pj, m->pw_lin, t, s->conv[b][li], s->conv[nb][li], s->ssm[b][li], s->ssm[nb][li], m->co, m->core, true, gdn_fused(L) ? m->aop : nullptr, L.gdn_up, gdn_q_on(m, L) ? &gq : nullptr))) return rc;
      s->cur[li] = nb;
    }
    return PYRE_OK;
  }
  int front_post_attn(int il) {          // for a block's window: the attention pass its mid left out
    const Layer& L = m->layers[il];
    if (!(L.full && o.attn_split)) return PYRE_OK;
    return pyre_attn_launch_sel(ctx, L.attn, s->kv[L.mix_index], o.aw_own, m->proj, m->pw_attn, start, t, &s->packed[L.mix_index], m->core, nullptr, nullptr, 2);
  }
  int front_post_proj(int il, int nz = 1) {          // the output projection (nz as in front_pre)
    const pyre_model_cfg& c = m->c; const int d = c.d;
    const Layer& L = m->layers[il];
    if (nz <= 0) return PYRE_OK;
    if (L.full && nz > 1) {          // an attention layer's output projection for several windows: the split into each window's own operand buffer (free since its projection), then the product
      const PyreAop own{(const uint4*)m->aop, m->aop_inv};
      ctx->batch_n = nz; ctx->batch_stride = o.win_stride;
      int rc = pyre_act_split_launch(ctx, m->core, t, L.outp.cols, (uint4*)m->aop, m->aop_inv);
      if (!rc) rc = outp_in_parts(L, d) ? pyre_gemv_parts_launch(ctx, L.outp, m->core, t, m->o, &own) : pyre_gemv_launch(ctx, L.outp, m->core, t, m->o, &own);
      ctx->batch_n = 1; ctx->batch_stride = 0;
      return rc;
    }
    const PyreAop aop_gdn{(const uint4*)m->aop, L.gdn_ainv}, aop_gdq{(const uint4*)m->aop, nullptr, m->gdn_sq, L.gdn.nv, L.gdn.eps};
    const PyreAop* oa = (!L.full && gdn_q_on(m, L)) ? &aop_gdq : ((!L.full && gdn_fused(L)) ? &aop_gdn : nullptr);
    ctx->batch_n = nz; ctx->batch_stride = nz > 1 ? o.win_stride : 0;
    // few row tiles, long rows: four workgroups per row tile leave partial sums, the mix below adds them
    const int rc = outp_in_parts(L, d) ? pyre_gemv_parts_launch(ctx, L.outp, m->core, t, m->o, oa) : pyre_gemv_launch(ctx, L.outp, m->core, t, m->o, oa);
    ctx->batch_n = 1; ctx->batch_stride = 0;
    return rc;
  }
  int front_post_mix(int il, int nz = 1) {          // the FFN mix (nz as in front_pre)
    const pyre_model_cfg& c = m->c; const int d = c.d; int rc;
    const Layer& L = m->layers[il];
    const int o_parts = outp_in_parts(L, d) ? PYRE_GEMV_PARTS : 1;
    ride = route_rides && !o.router_apart && pyre_hc_route_ok(L.hcf, L.moe.router);       // the router GEMV rides on the mix's second launch
    HcRoute hr{L.moe.router, m->rpart, m->mw.dgx};          // (the matrix-core mix leaves the digits of its output; after another mix the expert launch makes them)
    if (nz > 0) {
      ctx->batch_n = nz; ctx->batch_stride = nz > 1 ? o.win_stride : 0;
      rc = pyre_hc_mix_launch(ctx, L.hcf, m->hw, xin, in_ss, in_ts, xout, t, m->o, nullptr, m->inj_a, c.eps, m->mixed, m->inj_f, ride ? &hr : nullptr, o_parts);
      ctx->batch_n = 1; ctx->batch_stride = 0;
      if (rc) return rc;
    }
    advance();
    return PYRE_OK;
  }
  int front_post(int il) { int rc = front_post_attn(il); if (!rc) rc = front_post_proj(il); return rc ? rc : front_post_mix(il); }
  int front(int il) {
    int rc; const Layer& L = m->layers[il];
    if (o.wait_ev && L.ple) PYRE_HIP(ctx, hipStreamWaitEvent(ctx->stream, o.wait_ev[il], 0));      // the layer's ring of rows is state
    if ((rc = front_pre(il))) return rc;
    // the layer's state (cache, recurrent state, saved projection) is the previous window's until that window has left it
    if (o.wait_ev) PYRE_HIP(ctx, hipStreamWaitEvent(ctx->stream, o.wait_ev[il], 0));
    if ((rc = front_mid(il))) return rc;
    if (o.rec_ev) PYRE_HIP(ctx, hipEventRecord(o.rec_ev[il], ctx->stream));
    return front_post(il);
  }

  int moe(int il) {
    const pyre_model_cfg& c = m->c; const Layer& L = m->layers[il]; int rc;
    RouteSrc rs{m->rpart, c.d / 64, L.moe.router.tiles * 64, pyre_hc_aop_ok(L.hcf) ? m->mw.dgx : nullptr};
    const bool groups = groups_at(il);
    if ((rc = pyre_moe_launch(ctx, L.moe, m->mw, m->mixed, t, raw_moe ? nullptr : m->y, ride ? &rs : nullptr, groups))) return rc;
    if (groups) { comb_out = m->mw.parts; comb_moe = nullptr; comb_np = PYRE_MOE_GROUPS; }
    else if (raw_moe) { mo = pyre_moe_out(L.moe, m->mw, 0); comb_moe = &mo; comb_out = nullptr; } else comb_out = m->y;
    comb_inj = m->inj_f;
    return PYRE_OK;
  }
  // the block's FFN launch has left this window's group sums in m->mw.parts
  void moe_from_block() { comb_out = m->mw.parts; comb_moe = nullptr; comb_np = PYRE_MOE_GROUPS; comb_inj = m->inj_f; }
  int finish() {
    const pyre_model_cfg& c = m->c; const int d = c.d, hc = c.hc; int rc;
    const PyreAop aop_hc{(const uint4*)m->aop, m->aop_inv};
    const AopOut aout{m->aop, m->aop_inv, d / 256};
    auto opnd = [&](const HcDev& h, const QMatDev& q) -> const PyreAop* { return hc_fused(h, q) ? &aop_hc : nullptr; };
    auto opw = [&](const HcDev& h, const QMatDev& q) -> const AopOut* { return hc_fused(h, q) ? &aout : nullptr; };
    if (!replay && !o.no_len) s->len = start + t;
    const bool want_r = s->mtp && o.keep_from < t;      // the head mix resolves the pending update of every token: its x_out rows are the final residual streams
    if (o.head_tokens == 0 && !want_r) return PYRE_OK;       // prompt window whose logits nobody reads
    if (o.head_tokens >= t || want_r) {
      const bool all = o.head_tokens >= t;
      if ((rc = pyre_hc_mix_launch(ctx, m->head, m->hw, xin, in_ss, in_ts, xout, t, comb_out, comb_moe, comb_inj, c.eps, m->hbuf, m->inj_a, nullptr, comb_np, all ? opw(m->head, m->out) : nullptr))) return rc;
      if (want_r) {
        const int w = hc * d;
        hipLaunchKernelGGL(k_ring_store, dim3((w + 255) / 256, t - o.keep_from), dim3(256), 0, ctx->stream, xout, s->r_ring, s->r_mask, start, o.step_dev, o.keep_from, w); PYRE_CHECK_LAUNCH(ctx);
        if (!replay) s->r_push(start + o.keep_from, t - o.keep_from, mtp_window_of(s->mtp));
      }
      if (o.head_tokens == 0) return PYRE_OK;
      if (!all) return pyre_gemv_launch(ctx, m->out, m->hbuf + (size_t)(t - 1) * d, 1, m->logits);      // the last token's logits only
      if (o.greedy && t == 1) return pyre_gemv_argmax_launch(ctx, m->out, m->hbuf, m->logits, m->best, opnd(m->head, m->out));
      return pyre_gemv_launch(ctx, m->out, m->hbuf, t, m->logits, opnd(m->head, m->out));
    }
    // last token only: fold the pending ffn output into its streams, then the head
    const size_t last = (size_t)(t - 1) * hc * d;
    MoeOut mol{}; if (comb_moe) mol = pyre_moe_out(m->layers.back().moe, m->mw, t - 1);
    if ((rc = pyre_hc_mix_launch(ctx, m->head, m->hw, xin + last, in_ss, in_ts, xout + last, 1, comb_out ? comb_out + (size_t)(t - 1) * d : nullptr, comb_moe ? &mol : nullptr, comb_inj + (size_t)(t - 1) * hc, c.eps, m->hbuf, m->inj_a, nullptr, 1, opw(m->head, m->out)))) return rc;
    if (o.greedy) return pyre_gemv_argmax_launch(ctx, m->out, m->hbuf, m->logits, m->best, opnd(m->head, m->out));
    return pyre_gemv_launch(ctx, m->out, m->hbuf, 1, m->logits, opnd(m->head, m->out));
  }
};
int run_window(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, int t, const WinOpt& o) {
  WinRun w(ctx, m, s, t, o);
  int rc = w.begin(); if (rc) return rc;
  for (int il = 0; il < m->c.n_layers; ++il) { if ((rc = w.front(il)) || (rc = w.moe(il))) return rc; }
  return w.finish();
}

int check_ids(pyre_ctx* ctx, const pyre_model* m, const uint32_t* ids, int n) {
  for (int i = 0; i < n; ++i) if (ids[i] >= (uint32_t)m->c.vocab) return pyre_fail(ctx, PYRE_E_ARG, "forward: token id %u outside the vocabulary (%d)", ids[i], m->c.vocab);
  return PYRE_OK;
}

}  // namespace

extern "C" {

int pyre_forward(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* ids, int n, float* logits_host) {
  if (!ctx || !m || !s || !ids || n < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_forward: bad argument");
  if (s->m != m) return pyre_fail(ctx, PYRE_E_STATE, "pyre_forward: state belongs to another model");
  if (s->broken) return pyre_fail(ctx, PYRE_E_STATE, "%s: an earlier call failed half way through this state; pyre_state_reset or pyre_state_restore first", "pyre_forward");
  if (s->len + n > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "pyre_forward: %d + %d tokens exceed the state's capacity %d", s->len, n, s->cap);
  const auto t_enter = std::chrono::steady_clock::now();
  int rc = check_ids(ctx, m, ids, n); if (rc) return rc;
  s->last_window = 0;
  const int nwin = (n + 7) / 8, K = prompt_streams();
  PromptPipe* P = nullptr;
  if (K > 1 && nwin >= 2 * K && !ctx->prof_on) {      // a long prompt: K windows in flight (the per-class timing wants one stream)
    if ((rc = prompt_pipe_get(ctx, m, &P)) || (rc = prompt_pipe_state(ctx, m, s, K))) return rc;
    if (P->ids_cap < (size_t)n) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); if (P->ids) (void)hipFree(P->ids); P->ids = nullptr; P->ids_cap = 0;
      PYRE_HIP(ctx, hipMalloc((void**)&P->ids, (size_t)n * 4)); P->ids_cap = (size_t)n; }
    PYRE_HIP(ctx, hipMemcpyAsync(P->ids, ids, (size_t)n * 4, hipMemcpyHostToDevice, ctx->stream));
    if (s->tokens_dev) PYRE_HIP(ctx, hipMemcpyAsync(s->tokens_dev + s->len, P->ids, (size_t)n * 4, hipMemcpyDeviceToDevice, ctx->stream));      // the history every window's n-gram rows read
    PYRE_HIP(ctx, hipEventRecord(P->start, ctx->stream));      // the other streams begin after everything already queued here
    for (auto* cx : P->ctx) PYRE_HIP(ctx, hipStreamWaitEvent(cx->stream, P->start, 0));
  }
  int prev = -1, i_first = 0;
  const bool windows_only = [] { const char* e = getenv("PYRE_PROMPT_WINDOWS"); return e && *e && atoi(e) != 0; }();      // (read per call: 1 = this call in windows, whatever layouts the model keeps)
  if (P && !windows_only && prompt_block_ok(m)) {      // whole blocks of windows in front of the call's last tokens: layer by layer, the FFN grouped by expert
    // (a call's last block may be shorter, down to PROMPT_BLOCK_MIN windows: fewer tokens than that share too few experts to pay)
    const int NBMAX = PROMPT_BLOCK_WINDOWS, tail = 8 + (s->mtp ? mtp_window_of(s->mtp) : 0);
    int wins = n > tail ? (n - tail) / 8 : 0;
    if (wins >= PROMPT_BLOCK_MIN && (rc = prompt_block_get(ctx, m, P))) return rc;
    const int nl = m->c.n_layers;
    const int G_env = [] { const char* e = getenv("PYRE_PROMPT_GROUP"); int v = e && *e ? atoi(e) : 0; return v < 0 ? 0 : (v > PROMPT_BLOCK_WINDOWS ? PROMPT_BLOCK_WINDOWS : v); }();      // PYRE_PROMPT_GROUP: windows a group (default: a group a stream)
    const bool batch = [&] { const char* e = getenv("PYRE_PROMPT_BATCH"); if (e && *e && atoi(e) == 0) return false; for (const Layer& L : m->layers) if (!pyre_hc_aop_ok(L.hca) || !pyre_hc_aop_ok(L.hcf)) return false; return true; }();      // a group's mixes in one launch each (the matrix-core mixes; PYRE_PROMPT_BATCH=0: a launch a window)
    const bool early = batch && m->c.conv_k >= 2 && m->c.conv_k <= 9 && !(getenv("PYRE_PROMPT_PROJ_EARLY") && atoi(getenv("PYRE_PROMPT_PROJ_EARLY")) == 0);      // the projections in front of the chain through the layer's state, the convolution once a group (PYRE_PROMPT_PROJ_EARLY=0: both in the chain, a window at a time)
    const bool asplit = P->qmem && !(getenv("PYRE_PROMPT_ATTN_SPLIT") && atoi(getenv("PYRE_PROMPT_ATTN_SPLIT")) == 0);      // an attention layer's pass over the cache outside the chain (PYRE_PROMPT_ATTN_SPLIT=0: in it)
    const bool rapart = batch && !(getenv("PYRE_PROMPT_ROUTER_APART") && atoi(getenv("PYRE_PROMPT_ROUTER_APART")) == 0);      // the router's sums with the block's FFN launches (beside the other block's windows) instead of riding on every window's FFN mix (PYRE_PROMPT_ROUTER_APART=0: riding)
    const bool pairs = [] { const char* e = getenv("PYRE_PROMPT_PAIRS"); return !(e && *e && atoi(e) == 0); }();      // PYRE_PROMPT_PAIRS=0: one block at a time
    auto cxk = [&](int k) { return k ? P->ctx[k - 1] : ctx; };
    auto bail = [&](int code, pyre_ctx* cx) { s->broken = true; if (cx != ctx) pyre_fail(ctx, code, "%s", cx->err.c_str()); for (auto* c2 : P->ctx) (void)hipStreamSynchronize(c2->stream); (void)hipStreamSynchronize(P->moe_ctx->stream); (void)hipStreamSynchronize(ctx->stream); return code; };
    // Blocks are taken two at a time, layer by layer: the windows of block A, A's FFN on the FFN stream, the windows of block B
    // beside it, B's FFN beside A's windows of the next layer.  Within a block the windows go to the streams in groups of G
    // consecutive ones, a group's launches in the order pre x G, mid x G, post x G: the mids of a group follow one another in
    // their stream without an event, one event hands the layer's state to the next group's stream, and a stream that waits for
    // it has its own pres behind it, not in front.  (8192 tokens, one block at a time: groups of one 2.17 s, two 1.98, four
    // 2.05, eight 2.29, sixteen 2.58.)
    struct Blk { int which, NB, G, NG, prev_in; std::vector<WinRun> runs; };
    // the call's windows in an even number of blocks of (nearly) equal size, so that every block has a partner
    int nblk = 0, bsz = 0, brem = 0;
    if (wins >= PROMPT_BLOCK_MIN) {
      nblk = pairs ? 2 * ((wins + 2 * NBMAX - 1) / (2 * NBMAX)) : (wins + NBMAX - 1) / NBMAX;
      while (nblk > 1 && wins / nblk < PROMPT_BLOCK_MIN) --nblk;
      bsz = wins / nblk; brem = wins % nblk;
    }
    for (int bi = 0; bi < nblk; ) {
      Blk B[2]; int nb = 0; int pos = s->len, i0 = i_first, pin = prev;
      for (int w = 0; w < (pairs ? 2 : 1) && bi < nblk; ++w, ++bi) {
        Blk& b = B[nb++]; b.which = w; b.NB = bsz + (bi < brem ? 1 : 0); wins -= b.NB; b.G = G_env ? G_env : (b.NB + K - 1) / K; b.NG = (b.NB + b.G - 1) / b.G; const int G = b.G; b.prev_in = pin; b.runs.reserve(b.NB);
        for (int j = 0; j < b.NB; ++j) {
          const int set = (j / G) % K; WinOpt o; o.head_tokens = 0; o.keep_from = 8; o.start = pos + 8 * j; o.no_len = true;
          o.ids_dev = P->ids + i0 + 8 * j; if (set) { o.aw = &s->aw_more[set - 1]; o.qw = &s->qw_more[set - 1]; }
          o.win_stride = P->win_stride; o.proj_early = early; o.router_apart = rapart;
          if (asplit) {          // q buffers of the window's own; the partial sums stay the stream's
            o.attn_split = true; o.aw_own = set ? s->aw_more[set - 1] : s->aw;
            uint8_t* qb = (uint8_t*)P->qmem + (size_t)(w * NBMAX + j) * P->q_stride;
            o.aw_own.q = (float*)qb; o.aw_own.qh = (uint16_t*)(qb + P->q_off[0]); o.aw_own.qsc = (float*)(qb + P->q_off[1]);
          }
          b.runs.emplace_back(cxk(set), P->wmdl[w * NBMAX + j], s, 8, o);
          if ((rc = b.runs.back().begin())) return bail(rc, cxk(set));
        }
        pos += b.NB * 8; i0 += b.NB * 8; pin = (b.NG - 1) % K;
      }
      // a block's windows of layer il: group by group in order, so that every record is issued before the wait that names it
      auto fronts = [&](Blk& b, int il) -> int {
        const int G = b.G;
        for (int g = 0; g < b.NG; ++g) {
          const int k = g % K; pyre_ctx* cx = cxk(k); int r;
          if (il > 0 && g < K && hipStreamWaitEvent(cx->stream, P->moe_done[b.which], 0) != hipSuccess) return pyre_fail(cx, PYRE_E_HIP, "hipStreamWaitEvent failed");
          const int j0 = g * G, j1 = j0 + G < b.NB ? j0 + G : b.NB;
          for (int j = j0; j < j1; ++j) if ((r = b.runs[j].front_pre(il, batch ? (j == j0 ? j1 - j0 : 0) : 1))) return r;            // the group's mixes: one launch each
          if (early) { const bool pb = b.runs[j0].proj_batchable(il); for (int j = j0; j < j1; ++j) if ((r = b.runs[j].front_pre_proj(il, pb ? (j == j0 ? j1 - j0 : 0) : 1))) return r; }
          const int pset = g > 0 ? (g - 1) % K : b.prev_in;
          if (pset >= 0 && pset != k && hipStreamWaitEvent(cx->stream, P->ev[pset][il], 0) != hipSuccess) return pyre_fail(cx, PYRE_E_HIP, "hipStreamWaitEvent failed");
          const bool gg = early && b.runs[j0].gdn_group_ok(il);          // the group's recurrences in one launch
          if (early && (r = b.runs[j0].front_mid_conv(il, j1 - j0, j0 == 0, j1 == b.NB, gg ? 1 : j1 - j0))) return r;
          if (gg) { if ((r = b.runs[j0].front_mid_gdn(il, j1 - j0))) return r; }
          else if (early && asplit && m->layers[il].full) { if ((r = b.runs[j0].front_mid_attn(il, j1 - j0, P->q_stride))) return r; }          // the group's cache writes in one launch
          else for (int j = j0; j < j1; ++j) if ((r = b.runs[j].front_mid(il))) return r;
          if (hipEventRecord(P->ev[k][il], cx->stream) != hipSuccess) return pyre_fail(cx, PYRE_E_HIP, "hipEventRecord failed");
          for (int j = j0; j < j1; ++j) if ((r = b.runs[j].front_post_attn(il))) return r;
          { const bool ob = batch && j1 - j0 > 1 && b.runs[j0].outp_batchable(il); for (int j = j0; j < j1; ++j) if ((r = b.runs[j].front_post_proj(il, ob ? (j == j0 ? j1 - j0 : 0) : 1))) return r; }
          for (int j = j0; j < j1; ++j) if ((r = b.runs[j].front_post_mix(il, batch ? (j == j0 ? j1 - j0 : 0) : 1))) return r;
        }
        return PYRE_OK;
      };
      auto ffn = [&](Blk& b, int il) -> int {
        pyre_ctx* mx = P->moe_ctx;
        for (int k = 0; k < K && k < b.NG; ++k) { if (hipEventRecord(P->front_done[b.which][k], cxk(k)->stream) != hipSuccess || hipStreamWaitEvent(mx->stream, P->front_done[b.which][k], 0) != hipSuccess) return pyre_fail(ctx, PYRE_E_HIP, "event failed"); }
        int r = pyre_moe_block_launch(mx, m->layers[il].moe, P->blk[b.which], b.NB * 8, NBMAX * 8, P->blk_nsl, P->blk_r64, rapart);
        if (r) return pyre_fail(ctx, r, "%s", mx->err.c_str());
        if (hipEventRecord(P->moe_done[b.which], mx->stream) != hipSuccess) return pyre_fail(ctx, PYRE_E_HIP, "hipEventRecord failed");
        for (int j = 0; j < b.NB; ++j) b.runs[j].moe_from_block();
        return PYRE_OK;
      };
      for (int il = 0; il < nl; ++il) for (int w = 0; w < nb; ++w) {
        if ((rc = fronts(B[w], il))) return bail(rc, ctx);
        if (il < nl - 1 && (rc = ffn(B[w], il))) return bail(rc, ctx);            // the last layer's FFN output has no reader in these windows
      }
      for (int w = 0; w < nb; ++w) { s->len += B[w].NB * 8; i_first += B[w].NB * 8; ++P->blocks_done; }
      prev = pin;
    }
    if (i_first > 0) for (int k = 1; k < K; ++k) PYRE_HIP(ctx, hipEventRecord(P->done[k], P->ctx[k - 1]->stream));
  }
  const int nwin_tail = (n - i_first + 7) / 8;
  for (int i = i_first, w = 0; i < n; i += 8, ++w) {
    int t = n - i < 8 ? n - i : 8; bool last = i + t >= n;
    WinOpt o; o.head_tokens = last && logits_host ? 1 : 0;
    if (s->mtp) { const int k0 = n - mtp_window_of(s->mtp) - i; o.keep_from = k0 < 0 ? 0 : k0; }      // the last `window` tokens of a call (qwen4exp_gguf.rs:2148-2150)
    if (!P) {
      PYRE_HIP(ctx, hipMemcpyAsync(m->ids, ids + i, (size_t)t * 4, hipMemcpyHostToDevice, ctx->stream));
      if ((rc = run_window(ctx, m, s, t, o))) { s->broken = true; return rc; }
      continue;
    }
    const int set = (nwin_tail - 1 - w) % K;          // the last window runs on the model's own stream and workspace: its logits are the call's
    pyre_ctx* cx = set ? P->ctx[set - 1] : ctx; const pyre_model* mx = set ? P->mdl[set - 1] : m;
    o.ids_dev = P->ids + i; if (set) { o.aw = &s->aw_more[set - 1]; o.qw = &s->qw_more[set - 1]; }
    o.wait_ev = prev >= 0 ? P->ev[prev].data() : nullptr; o.rec_ev = P->ev[set].data();
    rc = run_window(cx, mx, s, t, o);
    if (!rc && hipEventRecord(P->done[set], cx->stream) != hipSuccess) rc = pyre_fail(cx, PYRE_E_HIP, "hipEventRecord failed");
    if (rc) { s->broken = true; if (cx != ctx) pyre_fail(ctx, rc, "%s", cx->err.c_str()); for (auto* c2 : P->ctx) (void)hipStreamSynchronize(c2->stream); (void)hipStreamSynchronize(ctx->stream); return rc; }      // windows already issued have advanced the bookkeeping and part of the state
    prev = set;
  }
  if (getenv("PYRE_DEBUG_ENQ")) { static auto t_prev = std::chrono::steady_clock::now(); auto t1 = std::chrono::steady_clock::now(); fprintf(stderr, "enq %d tokens (%d in blocks): %.3f ms since entry\n", n, i_first, std::chrono::duration<double>(t1 - t_enter).count() * 1e3); (void)t_prev; }
  if (P) for (int k = 1; k < K; ++k) PYRE_HIP(ctx, hipStreamWaitEvent(ctx->stream, P->done[k], 0));      // everything the other streams did precedes what follows here
  if (logits_host) PYRE_HIP(ctx, hipMemcpyAsync(logits_host, m->logits, (size_t)m->c.vocab * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

int pyre_forward_multi(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* ids, int n, float* logits_host) {
  if (!ctx || !m || !s || !ids || !logits_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_forward_multi: null argument");
  if (n < 1 || n > 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_forward_multi: window of %d tokens outside 1..8", n);
  if (s->m != m) return pyre_fail(ctx, PYRE_E_STATE, "pyre_forward_multi: state belongs to another model");
  if (s->broken) return pyre_fail(ctx, PYRE_E_STATE, "%s: an earlier call failed half way through this state; pyre_state_reset or pyre_state_restore first", "pyre_forward_multi");
  if (s->len + n > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "pyre_forward_multi: context exceeds the state's capacity %d", s->cap);
  int rc = check_ids(ctx, m, ids, n); if (rc) return rc;
  PYRE_HIP(ctx, hipMemcpyAsync(m->ids, ids, (size_t)n * 4, hipMemcpyHostToDevice, ctx->stream));
  { WinOpt o; o.head_tokens = n; if (s->mtp && n > mtp_window_of(s->mtp)) o.keep_from = n - mtp_window_of(s->mtp); if ((rc = run_window(ctx, m, s, n, o))) return rc; }
  s->last_window = n;
  PYRE_HIP(ctx, hipMemcpyAsync(logits_host, m->logits, (size_t)n * m->c.vocab * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

// First maximum of each of t logit rows (sampler::argmax, src/sampler.rs:142-148: a scan from index 0 with strict >, so the
// lowest index among equal maxima, NaNs never chosen unless at index 0): grid t, 1024 threads; a thread walks its indices in ascending order, the threads then meet by (value, index).
__global__ __launch_bounds__(1024) void k_argmax_rows(const float* __restrict__ logits, int V, uint32_t* __restrict__ best) {
  __shared__ float sv[16]; __shared__ uint32_t si[16];
  const float* l = logits + (size_t)blockIdx.x * V; const int tid = threadIdx.x;
  float bv = -INFINITY; uint32_t bi = 0xFFFFFFFFu;
  for (int i = tid; i < V; i += 1024) { const float v = l[i]; if (!(v != v) && (bi == 0xFFFFFFFFu || v > bv)) { bv = v; bi = (uint32_t)i; } }      // a NaN is never greater
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { const float ov = __shfl_xor(bv, o); const uint32_t oi = __shfl_xor(bi, o); if (oi != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; } }
  if ((tid & 63) == 0) { sv[tid >> 6] = bv; si[tid >> 6] = bi; }
  __syncthreads();
  if (tid == 0) { for (int w = 1; w < 16; ++w) if (si[w] != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || sv[w] > bv || (sv[w] == bv && si[w] < bi))) { bv = sv[w]; bi = si[w]; }
    best[blockIdx.x] = (bi == 0xFFFFFFFFu || l[0] != l[0]) ? 0u : bi; }          // the scan starts from index 0: a NaN there is never replaced, as on the host
}

// pyre_forward_multi for a caller that only wants each token's greedy pick: the picks are formed on the device and t
// integers come back instead of t x vocab logits.
static int forward_multi_picks(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* ids, int n, uint32_t* picks_host) {
  if (n < 1 || n > 8) return pyre_fail(ctx, PYRE_E_ARG, "forward_multi: window of %d tokens outside 1..8", n);
  if (s->m != m) return pyre_fail(ctx, PYRE_E_STATE, "forward_multi: state belongs to another model");
  if (s->broken) return pyre_fail(ctx, PYRE_E_STATE, "%s: an earlier call failed half way through this state; pyre_state_reset or pyre_state_restore first", "forward_multi");
  if (s->len + n > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "forward_multi: context exceeds the state's capacity %d", s->cap);
  int rc = check_ids(ctx, m, ids, n); if (rc) return rc;
  PYRE_HIP(ctx, hipMemcpyAsync(m->ids, ids, (size_t)n * 4, hipMemcpyHostToDevice, ctx->stream));
  { WinOpt o; o.head_tokens = n; if (s->mtp && n > mtp_window_of(s->mtp)) o.keep_from = n - mtp_window_of(s->mtp); if ((rc = run_window(ctx, m, s, n, o))) return rc; }
  s->last_window = n;
  hipLaunchKernelGGL(k_argmax_rows, dim3(n), dim3(1024), 0, ctx->stream, m->logits, m->c.vocab, m->best);
  PYRE_CHECK_LAUNCH(ctx);
  PYRE_HIP(ctx, hipMemcpyAsync(picks_host, m->best, (size_t)n * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

// The DeltaNet layers kept the window's inputs and their pre-window state (the other half of the double buffer): the
// first `keep` tokens are run again from there, which reproduces the checkpoint after token `keep` bit for bit.
int pyre_spec_keep(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, int t, int keep) {
  if (!ctx || !m || !s) return pyre_fail(ctx, PYRE_E_ARG, "pyre_spec_keep: null argument");
  if (keep >= t || t < 2) return PYRE_OK;
  if (keep < 1) keep = 1;
  if (s->last_window != t) return pyre_fail(ctx, PYRE_E_STATE, "pyre_spec_keep: the last forward_multi window had %d tokens, not %d", s->last_window, t);
  for (const Layer& L : m->layers) if (!L.full) {
    int li = L.mix_index, after = s->cur[li], before = after ^ 1;
    const GdnQ gq{m->aop, m->gdn_sq};          // (its operand and scales are not used: the call is for the state)
    int rc = pyre_gdn_launch(ctx, L.gdn, s->proj_saved[li], m->pw_lin, keep, s->conv[before][li], s->conv[after][li], s->ssm[before][li], s->ssm[after][li], m->co, m->core, false, nullptr, 1.0f, gdn_q_on(m, L) ? &gq : nullptr); if (rc) return rc;
  }
  s->len -= t - keep; s->last_window = 0;
  return PYRE_OK;
}

// The greedy loop on the device.  Step 0 runs eagerly from the host-supplied token; every further step is the same
// launch sequence with its position and output slot in device memory, captured once per state into a HIP graph and
// replayed (PYRE_NO_GRAPH=1, or profiling switched on, replays it eagerly instead).
int pyre_decode_greedy_dev(pyre_ctx* ctx, const pyre_model* mc, pyre_state* s, uint32_t first, int n_steps, uint32_t* tokens_host) {
  pyre_model* m = const_cast<pyre_model*>(mc);
  if (!ctx || !m || !s || n_steps < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_decode_greedy_dev: bad argument");
  if (s->m != m) return pyre_fail(ctx, PYRE_E_STATE, "pyre_decode_greedy_dev: state belongs to another model");
  if (s->broken) return pyre_fail(ctx, PYRE_E_STATE, "%s: an earlier call failed half way through this state; pyre_state_reset or pyre_state_restore first", "pyre_decode_greedy_dev");
  if (s->len + n_steps > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "pyre_decode_greedy_dev: context exceeds the state's capacity %d", s->cap);
  int rc = check_ids(ctx, m, &first, 1); if (rc) return rc;
  if (m->toks_cap < n_steps) { if (m->toks) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(m->toks)); m->toks = nullptr; } PYRE_HIP(ctx, hipMalloc((void**)&m->toks, (size_t)n_steps * 4)); m->toks_cap = n_steps; }
  s->last_window = 0;
  PYRE_HIP(ctx, hipMemcpyAsync(m->ids, &first, 4, hipMemcpyHostToDevice, ctx->stream));
  { WinOpt o; o.greedy = true; o.inplace = true; if ((rc = run_window(ctx, m, s, 1, o))) return rc; }     // in place: the captured step below keeps pointing at the current buffers
  if (n_steps > 1) {
    const bool no_graph = getenv("PYRE_NO_GRAPH") && atoi(getenv("PYRE_NO_GRAPH")) != 0;          // read per call (tests switch it)
    int step_host[2] = {s->len - 1, s->len};      // the pick increments [0] to the position it starts; slot = [0] - [1]
    PYRE_HIP(ctx, hipMemcpyAsync(s->step_dev, step_host, 8, hipMemcpyHostToDevice, ctx->stream));
    WinOpt o; o.greedy = true; o.from_best = true; o.toks_out = m->toks; o.step_dev = s->step_dev;
    if (no_graph || ctx->prof_on) {
      for (int i = 1; i < n_steps; ++i) if ((rc = run_window(ctx, m, s, 1, o))) return rc;
    } else {
      if (!s->graph_exec || s->graph_toks != m->toks || s->graph_cur != s->cur) {      // forward / forward_multi calls in between flip the double buffers
        if (s->graph_exec) { (void)hipGraphExecDestroy(s->graph_exec); s->graph_exec = nullptr; }
        hipGraph_t g = nullptr;
        PYRE_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
        rc = run_window(ctx, m, s, 1, o);
        hipError_t e = hipStreamEndCapture(ctx->stream, &g);
        if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
        if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_HIP, "pyre_decode_greedy_dev: stream capture failed: %s", hipGetErrorString(e));
        e = hipGraphInstantiate(&s->graph_exec, g, nullptr, nullptr, 0); (void)hipGraphDestroy(g);
        if (e != hipSuccess) { s->graph_exec = nullptr; return pyre_fail(ctx, PYRE_E_HIP, "pyre_decode_greedy_dev: graph instantiate failed: %s", hipGetErrorString(e)); }
        s->graph_toks = m->toks; s->graph_cur = s->cur;
      }
      for (int i = 1; i < n_steps; ++i) PYRE_HIP(ctx, hipGraphLaunch(s->graph_exec, ctx->stream));
    }
    if (s->mtp) s->r_push(s->len, n_steps - 1, mtp_window_of(s->mtp));      // the replayed steps stored their rows themselves
    s->len += n_steps - 1;
    for (size_t ai = 0; ai < s->packed.size(); ++ai) { int pb = (int)pyre_packed_boundary((size_t)s->len, m->c.kv_bits, m->c.kv_recent); if (pb > s->packed[ai]) s->packed[ai] = pb; }
  }
  if ((rc = pyre_pick_launch(ctx, m->best, pyre_gemv_best_count(m->out), m->ids, m->toks + n_steps - 1, nullptr, nullptr, nullptr))) return rc;
  if (tokens_host) { PYRE_HIP(ctx, hipMemcpyAsync(tokens_host, m->toks, (size_t)n_steps * 4, hipMemcpyDeviceToHost, ctx->stream)); PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK; }
  return PYRE_OK;
}

// Adaptive draft length of spec::generate (src/spec.rs:162-167, 186-193, 213-217, 221, 229, 258): the plain step time ts and the
// verify time tv[t] of a t-token window as running means, the running acceptance p_acc, the drafter's time per round td_avg.
// Before drafting the plan picks the draft count (0 = a plain step; now and then a probe window of at most two drafts so the
// estimates can recover); after drafting the most profitable prefix of what the drafter produced is kept.  Nothing
// happens before the first plain step has been timed.  It only chooses which drafts are verified: the output is unchanged.
struct SpecAdapt {
  bool on = false; double ts = 0, tv[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, p_acc = 0.7, td_avg = 0; int skipped = 0; bool probe = false;
  std::chrono::steady_clock::time_point t0;
  explicit SpecAdapt(const pyre_ctx* ctx) { const char* e = getenv("PYRE_SPEC_ADAPT"); on = ctx->spec_adapt >= 0 ? ctx->spec_adapt != 0 : (e && *e && strcmp(e, "0") != 0); }
  void tick() { t0 = std::chrono::steady_clock::now(); }
  double tock() const { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count(); }
  int plan(int kk) {
    probe = false;
    if (!on || kk <= 0 || ts <= 0.0) return kk;
    const int bk = pyre_adapt_plan(kk, ts, tv, p_acc, td_avg);
    bool none = true; for (int t = 2; t < 10; ++t) if (tv[t] != 0.0) none = false;
    const int every = none ? 2 : 24;            // sooner while no window has been timed yet
    if (bk > 0) { skipped = 0; return bk; }
    if (skipped >= every) { skipped = 0; probe = true; return kk < 2 ? kk : 2; }
    ++skipped; return 0;
  }
  int trim(int nd) const { return (on && !probe && nd > 0 && ts > 0.0) ? pyre_adapt_plan(nd, ts, tv, p_acc, 0.0) : nd; }
  void drafted(double dt) { td_avg = td_avg == 0.0 ? dt : 0.8 * td_avg + 0.2 * dt; }
  void plain(double dt) { ts = ts == 0.0 ? dt : 0.8 * ts + 0.2 * dt; }
  void verified(int t, double dt) { tv[t] = tv[t] == 0.0 ? dt : 0.7 * tv[t] + 0.3 * dt; }
  void accepted(int acc, int nd) { p_acc = 0.7 * p_acc + 0.3 * ((double)acc / (double)nd); }
};

static uint32_t host_argmax(const float* l, size_t n) { size_t b = 0; for (size_t i = 1; i < n; ++i) if (l[i] > l[b]) b = i; return (uint32_t)b; }

int pyre_adapt_plan(int n, double ts, const double* tv, double p, double td) {            // spec::adapt_plan, src/spec.rs:147-152
  if (!tv) return 0;
  double best = 1.0, e = 1.0, pp = 1.0; int bk = 0;
  for (int kq = 1; kq <= (n < 8 ? n : 8); ++kq) {
    pp *= p; e += pp;
    const double est = tv[kq + 1] > 0.0 ? tv[kq + 1] : ts * (1.0 + 0.75 * ((double)(kq + 1) - 1.0));
    const double g = e * ts / (est + td);
    if (g > best) { best = g; bk = kq; }
  }
  return bk;
}
void pyre_spec_set_adapt(pyre_ctx* ctx, int on) { if (ctx) ctx->spec_adapt = on < 0 ? -1 : (on != 0); }

int pyre_generate_greedy(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const float* first_logits, int n_out, uint32_t* out, int n_draft, const uint32_t* draft_stream, int* rounds_out) {
  if (!ctx || !m || !s || !first_logits || !out || n_out < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy: bad argument");
  if (n_draft < 0 || n_draft > 7) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy: n_draft %d outside 0..7", n_draft);
  const size_t V = m->c.vocab; int produced = 0, rounds = 0;
  uint32_t pending = host_argmax(first_logits, V);
  if (n_draft == 0 || !draft_stream) {
    out[produced++] = pending;
    if (produced < n_out) { int rc = pyre_decode_greedy_dev(ctx, m, s, pending, n_out - 1, out + 1); if (rc) return rc; }
    if (rounds_out) *rounds_out = 0; return PYRE_OK;
  }
  for (;;) {
    out[produced++] = pending; if (produced >= n_out) break;
    int left = n_out - produced; int kk = n_draft < left - 1 ? n_draft : left - 1;
    if (kk <= 0) { uint32_t pk; int rc = forward_multi_picks(ctx, m, s, &pending, 1, &pk); if (rc) return rc; pending = pk; continue; }
    uint32_t toks[8]; toks[0] = pending; for (int j = 0; j < kk; ++j) toks[j + 1] = draft_stream[produced + j];
    uint32_t picks[8]; int rc = forward_multi_picks(ctx, m, s, toks, kk + 1, picks); if (rc) return rc;
    int acc = 0; bool have = false; uint32_t nx = 0;
    for (int i = 0; i < kk; ++i) { uint32_t tk = picks[i]; if (tk == toks[i + 1]) { ++acc; continue; } nx = tk; have = true; break; }
    if (!have) nx = picks[kk];
    if ((rc = pyre_spec_keep(ctx, m, s, kk + 1, acc + 1))) return rc; ++rounds;
    bool stop = false; for (int i = 0; i < acc; ++i) { out[produced++] = toks[i + 1]; if (produced >= n_out) { stop = true; break; } }
    if (stop) break;
    pending = nx;
  }
  if (rounds_out) *rounds_out = rounds;
  return PYRE_OK;
}

int pyre_argmax_rows(pyre_ctx* ctx, const float* logits_host, int t, int vocab, uint32_t* picks_host) {
  if (!ctx || !logits_host || !picks_host || t < 1 || vocab < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_argmax_rows: bad argument");
  float* d = nullptr; uint32_t* b = nullptr; const size_t n = (size_t)t * vocab;
  PYRE_HIP(ctx, hipMalloc((void**)&d, n * 4 + (size_t)t * 4)); b = (uint32_t*)(d + n);
  hipError_t e = hipMemcpyAsync(d, logits_host, n * 4, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess) { hipLaunchKernelGGL(k_argmax_rows, dim3(t), dim3(1024), 0, ctx->stream, d, vocab, b); e = hipGetLastError(); }
  if (e == hipSuccess) e = hipMemcpyAsync(picks_host, b, (size_t)t * 4, hipMemcpyDeviceToHost, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  (void)hipFree(d);
  if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_HIP, "pyre_argmax_rows: %s", hipGetErrorString(e));
  return PYRE_OK;
}

int pyre_ngram_draft(const uint32_t* h, size_t len, int k, int min_n, int max_n, uint32_t* out) {
  if (!h || !out || k <= 0 || min_n < 1 || len < (size_t)min_n + 1) return 0;
  const size_t top = (size_t)max_n < len - 1 ? (size_t)max_n : len - 1;
  for (size_t n = top; n >= (size_t)min_n && n <= top; --n) {          // longest suffix first
    const uint32_t* suf = h + len - n;
    for (size_t i = len - n; i > 0;) {                                  // start positions from the most recent down, i + n < len
      --i;
      if (h[i + n - 1] == suf[n - 1] && memcmp(h + i, suf, n * sizeof(uint32_t)) == 0) {
        const size_t s0 = i + n, e = s0 + (size_t)k < len ? s0 + (size_t)k : len;
        if (e > s0) { for (size_t q = s0; q < e; ++q) out[q - s0] = h[q]; return (int)(e - s0); }
      }
    }
  }
  return 0;
}

int pyre_generate_greedy_ngram(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* history, size_t n_hist, const float* first_logits, int n_out, uint32_t* out,
                               int k, int ng_min, int ng_max, int* rounds_out, int* drafted_out, int* accepted_out) {
  if (!ctx || !m || !s || !first_logits || !out || n_out < 1 || (n_hist && !history)) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy_ngram: bad argument");
  if (k < 1 || k > 7 || ng_min < 1 || ng_max < ng_min) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy_ngram: k %d (1..7), n-gram lengths %d..%d", k, ng_min, ng_max);
  const size_t V = m->c.vocab; int produced = 0, rounds = 0, drafted = 0, accepted = 0;
  std::vector<uint32_t> hist(history, history + n_hist); hist.reserve(n_hist + (size_t)n_out + 8);
  SpecAdapt ad(ctx);
  uint32_t pending = host_argmax(first_logits, V);
  for (;;) {
    hist.push_back(pending); out[produced++] = pending; if (produced >= n_out) break;
    const int left = n_out - produced; const int kk = ad.plan(k < left - 1 ? k : left - 1);
    uint32_t toks[8]; toks[0] = pending;
    const int nd = ad.trim(kk > 0 ? pyre_ngram_draft(hist.data(), hist.size(), kk, ng_min, ng_max, toks + 1) : 0);
    if (nd == 0) { uint32_t pk; ad.tick(); int rc = forward_multi_picks(ctx, m, s, &pending, 1, &pk); if (rc) return rc; ad.plain(ad.tock()); pending = pk; continue; }
    uint32_t picks[8]; ad.tick(); int rc = forward_multi_picks(ctx, m, s, toks, nd + 1, picks); if (rc) return rc; ad.verified(nd + 1, ad.tock());
    int acc = 0; bool have = false; uint32_t nx = 0;
    for (int i = 0; i < nd; ++i) { uint32_t tk = picks[i]; if (tk == toks[i + 1]) { ++acc; continue; } nx = tk; have = true; break; }
    if (!have) nx = picks[nd];
    if ((rc = pyre_spec_keep(ctx, m, s, nd + 1, acc + 1))) return rc;
    ad.accepted(acc, nd);
    ++rounds; drafted += nd; accepted += acc;
    bool stop = false; for (int i = 0; i < acc; ++i) { hist.push_back(toks[i + 1]); out[produced++] = toks[i + 1]; if (produced >= n_out) { stop = true; break; } }
    if (stop) break;
    pending = nx;
  }
  if (rounds_out) *rounds_out = rounds; if (drafted_out) *drafted_out = drafted; if (accepted_out) *accepted_out = accepted;
  return PYRE_OK;
}

}  // extern "C"

// ---- the MTP drafter (src/model/mtp.rs; Model::mtp_draft, src/model/qwen4exp_gguf.rs:2180-2277) --------------------------------
// Launch sequence of one draft step at cell p (R = the main model's final residual streams of position p for the first
// step, the drafter's own residual afterwards; token = the token at position p + 1):
//   row look-up of the token's embedding -> k_mtp_in (the two pre-norms) -> fc_embedding GEMV, fc_hidden GEMV over the
//   hc streams -> attention mix (adds the embedding part to every stream on the way: a pending update with weight
//   2 * sigmoid(0) = 1) -> [q ; k ; v] GEMV -> attention over the cells of the window (a position list) -> output GEMV
//   -> FFN mix -> MoE FFN -> mixer -> head GEMV over the draft vocabulary -> k_mtp_best (id, probability, next token).
// The catch-up over committed cells stops after the K / V append.
struct pyre_mtp {
  pyre_ctx* ctx = nullptr; const pyre_model* main = nullptr; pyre_mtp_cfg c{};
  pyre_model shell;                 // owner of the drafter's matrices and vectors (Builder's bookkeeping)
  QMatDev fc_e{}, fc_h{}, qkv{}, outp{}, head{}; HcDev hca{}, hcf{}, mix{}; MoeDev moe{}; AttnDev attn{};
  const float *pre_e = nullptr, *pre_h = nullptr; uint32_t* ids_dev = nullptr;
  void* work = nullptr; HcWork hw{}; MoeWork mw{};
  float *emb, *en, *e2, *hn, *xh, *ra, *rb, *rc, *mixed, *inj_a, *inj_f, *inj_m, *zeros, *proj, *core, *bo, *y, *sh, *logits, *out_p;
  uint32_t *out_ids, *tok; int pw = 0;
};

namespace {
int mtp_window_of(const pyre_mtp* m) { return m->c.window; }

// grid t, 256 threads: en = rms(emb row, pre_e) [t][d]; hn = rms(R row over all hc*d values, pre_h) [t][hc*d].
// R row of cell ti: ring row (pos0 + ti) & mask, or row ti of a plain buffer when mask < 0.
__global__ __launch_bounds__(256) void k_mtp_in(const float* __restrict__ emb, const float* __restrict__ r, int mask, int pos0, const float* __restrict__ pre_e, const float* __restrict__ pre_h,
                                                int d, int w, float eps, float* __restrict__ en, float* __restrict__ hn) {
  __shared__ float red[4];
  const int ti = blockIdx.x, tid = threadIdx.x;
  const float* e = emb + (size_t)ti * d; const float* rr = r + (size_t)(mask < 0 ? ti : ((pos0 + ti) & mask)) * w;
  float se = 0.0f, sr = 0.0f;
  for (int i = tid; i < d; i += 256) se += e[i] * e[i];
  for (int i = tid; i < w; i += 256) sr += rr[i] * rr[i];
  auto bsum = [&](float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    __syncthreads(); if ((tid & 63) == 0) red[tid >> 6] = v; __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]); };
  se = bsum(se); sr = bsum(sr);
  const float ke = 1.0f / sqrtf(se / (float)d + eps), kr = 1.0f / sqrtf(sr / (float)w + eps);
  for (int i = tid; i < d; i += 256) en[(size_t)ti * d + i] = e[i] * ke * pre_e[i];
  for (int i = tid; i < w; i += 256) hn[(size_t)ti * w + i] = rr[i] * kr * pre_h[i];
}

// best (mtp.rs:424-427) of the draft head's logits: the first maximum, its probability 1 / sum exp(v - max); one block
__global__ __launch_bounds__(1024) void k_mtp_best(const float* __restrict__ l, int n, const uint32_t* __restrict__ ids, uint32_t* __restrict__ out_id, float* __restrict__ out_p, uint32_t* __restrict__ tok) {
  __shared__ float sv[16]; __shared__ uint32_t si[16]; __shared__ float bvs; __shared__ uint32_t bis;
  const int tid = threadIdx.x;
  float bv = -INFINITY; uint32_t bi = 0xFFFFFFFFu;
  for (int i = tid; i < n; i += 1024) { const float v = l[i]; if (v > bv) { bv = v; bi = (uint32_t)i; } }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { const float ov = __shfl_xor(bv, o); const uint32_t oi = __shfl_xor(bi, o); if (oi != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; } }
  if ((tid & 63) == 0) { sv[tid >> 6] = bv; si[tid >> 6] = bi; }
  __syncthreads();
  if (tid == 0) { for (int q = 1; q < 16; ++q) if (si[q] != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || sv[q] > bv || (sv[q] == bv && si[q] < bi))) { bv = sv[q]; bi = si[q]; }
    bvs = bv; bis = bi == 0xFFFFFFFFu ? 0u : bi; }
  __syncthreads();
  bv = bvs; float z = 0.0f;
  for (int i = tid; i < n; i += 1024) z += expf(l[i] - bv);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) z += __shfl_xor(z, o);
  __syncthreads();
  if ((tid & 63) == 0) sv[tid >> 6] = z;
  __syncthreads();
  if (tid == 0) { float t = 0.0f; for (int q = 0; q < 16; ++q) t += sv[q]; const uint32_t id = ids[bis]; *out_id = id; *out_p = 1.0f / t; *tok = id; }
}

struct MtpCounts { int c[8]; };
// the position list of a draft call: list[i] = lo + i; count[j] = cells step j attends to
__global__ void k_mtp_list(int* __restrict__ list, int lo, int n, int* __restrict__ count, MtpCounts cn) {
  const int i = blockIdx.x * 256 + threadIdx.x; if (i < n) list[i] = lo + i; if (i < 8) count[i] = cn.c[i];
}

// cells pos0 .. pos0+t-1 (t * hc <= 8): input, attention mix, [q ; k ; v]; leaves the streams in m->ra, the mix's inject logits in m->inj_a
int mtp_cells(pyre_ctx* ctx, const pyre_mtp* m, const float* r, int mask, int pos0, int t) {
  const pyre_model_cfg& c = m->main->c; const int d = c.d, hc = c.hc, w = hc * d; int rc;
  hipLaunchKernelGGL(k_mtp_in, dim3(t), dim3(256), 0, ctx->stream, m->emb, r, mask, pos0, m->pre_e, m->pre_h, d, w, c.eps, m->en, m->hn); PYRE_CHECK_LAUNCH(ctx);
  if ((rc = pyre_gemv_launch(ctx, m->fc_e, m->en, t, m->e2))) return rc;
  if ((rc = pyre_gemv_launch(ctx, m->fc_h, m->hn, t * hc, m->xh))) return rc;
  if ((rc = pyre_hc_mix_launch(ctx, m->hca, m->hw, m->xh, d, w, m->ra, t, m->e2, nullptr, m->zeros, c.eps, m->mixed, m->inj_a, nullptr, 1, nullptr))) return rc;
  return pyre_gemv_launch(ctx, m->qkv, m->mixed, t, m->proj);
}
}  // namespace

extern "C" {

int pyre_mtp_create(pyre_ctx* ctx, const pyre_model* main, const pyre_mtp_cfg* cfg, const pyre_tensor* T, const uint32_t* draft_ids, pyre_mtp** out) {
  if (!ctx || !main || !cfg || !T || !draft_ids || !out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_create: null argument");
  *out = nullptr; const pyre_model_cfg& c = main->c; const int d = c.d, hc = c.hc, w = hc * d;
  if (cfg->n_exp < 1 || cfg->n_exp > 1024 || cfg->top_k < 1 || cfg->top_k > 32 || cfg->top_k > cfg->n_exp || cfg->ff < 64 || cfg->ff % 64 || cfg->window < 1 || cfg->n_draft_vocab < 1 || 8 / hc < 1)
    return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_mtp_create: %d experts top %d of width %d, window %d, %d draft rows", cfg->n_exp, cfg->top_k, cfg->ff, cfg->window, cfg->n_draft_vocab);
  for (int i = 0; i < cfg->n_draft_vocab; ++i) if (draft_ids[i] >= (uint32_t)c.vocab) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_create: draft id %u outside the vocabulary (%d)", draft_ids[i], c.vocab);
  PYRE_HIP(ctx, hipSetDevice(ctx->device));
  std::unique_ptr<pyre_mtp> M(new pyre_mtp()); pyre_mtp* m = M.get(); m->ctx = ctx; m->main = main; m->c = *cfg; m->shell.ctx = ctx; m->shell.c = c;
  struct Guard { pyre_mtp* m; bool armed = true; ~Guard() { if (armed) { for (auto q : m->shell.owned) pyre_qmat_destroy(q); for (auto b : m->shell.bufs) (void)hipFree(b); if (m->work) (void)hipFree(m->work); } } } guard{m};
  Builder B{ctx, &m->shell}; int rc;
  const int mlay = [] { const char* e = getenv("PYRE_MODEL_ROWS"); return e && *e && atoi(e) != 0; }() ? PYRE_LAYOUT_ROWS : PYRE_LAYOUT_M;
  if ((rc = B.vec(T[PYRE_MTP_PRE_E], d, &m->pre_e)) || (rc = B.vec(T[PYRE_MTP_PRE_H], w, &m->pre_h))) return rc;
  if ((rc = B.one(T[PYRE_MTP_FC_E], &m->fc_e, nullptr, mlay)) || (rc = B.one(T[PYRE_MTP_FC_H], &m->fc_h, nullptr, mlay))) return rc;
  if (m->fc_e.rows != d || m->fc_e.cols != d || m->fc_h.rows != d || m->fc_h.cols != d) return B.fail(PYRE_E_SHAPE, "fc_embedding / fc_hidden must be d x d");
  auto hcb = [&](int norm, int down, int inject, int up, HcDev* h) { m->shell.c.hc_lr = (int)T[down].rows; return B.hc(T[norm], T[down], inject >= 0 ? &T[inject] : nullptr, T[up], h, nullptr); };
  if ((rc = hcb(PYRE_MTP_HCA_NORM, PYRE_MTP_HCA_DOWN, PYRE_MTP_HCA_INJECT, PYRE_MTP_HCA_UP, &m->hca)) || (rc = hcb(PYRE_MTP_HCF_NORM, PYRE_MTP_HCF_DOWN, PYRE_MTP_HCF_INJECT, PYRE_MTP_HCF_UP, &m->hcf)) ||
      (rc = hcb(PYRE_MTP_MIX_NORM, PYRE_MTP_MIX_DOWN, -1, PYRE_MTP_MIX_UP, &m->mix))) return rc;
  { const pyre_tensor* grp[3] = {&T[PYRE_MTP_Q], &T[PYRE_MTP_K], &T[PYRE_MTP_V]};
    if (grp[0]->rows != (uint64_t)c.n_head * 2 * c.hd || grp[1]->rows != (uint64_t)c.n_kv * c.hd || grp[2]->rows != (uint64_t)c.n_kv * c.hd || grp[0]->cols != (uint64_t)d) return B.fail(PYRE_E_SHAPE, "drafter attention projection shapes");
    if ((rc = B.cat(grp, 3, &m->qkv, nullptr, mlay))) return rc; m->pw = c.n_head * 2 * c.hd + 2 * c.n_kv * c.hd; }
  if (T[PYRE_MTP_O].rows != (uint64_t)d || T[PYRE_MTP_O].cols != (uint64_t)c.n_head * c.hd) return B.fail(PYRE_E_SHAPE, "drafter o_proj shape");
  if ((rc = B.one(T[PYRE_MTP_O], &m->outp, nullptr, mlay))) return rc;
  std::vector<float> inv(c.n_rot / 2 + 1); (void)pyre_rope_table(c.n_rot, c.rope_base, 0, 0, inv.data());      // mtp.rs:111: the unscaled table
  float* rinv = nullptr; PYRE_HIP(ctx, hipMalloc((void**)&rinv, inv.size() * 4)); m->shell.bufs.push_back(rinv);
  PYRE_HIP(ctx, hipMemcpy(rinv, inv.data(), inv.size() * 4, hipMemcpyHostToDevice));
  m->attn = AttnDev{nullptr, nullptr, rinv, c.n_head, c.n_kv, c.hd, c.n_rot, 0, 0, c.eps, 1.0f};
  if ((rc = B.vec(T[PYRE_MTP_QN], c.hd, &m->attn.qn)) || (rc = B.vec(T[PYRE_MTP_KN], c.hd, &m->attn.kn))) return rc;
  MoeDev& mo = m->moe;
  if ((rc = B.one(T[PYRE_MTP_ROUTER], &mo.router, nullptr)) || (rc = B.one(T[PYRE_MTP_GATE_E], &mo.gate_e, nullptr)) || (rc = B.one(T[PYRE_MTP_UP_E], &mo.up_e, nullptr)) || (rc = B.one(T[PYRE_MTP_DOWN_E], &mo.down_e, nullptr)) ||
      (rc = B.one(T[PYRE_MTP_SH_GATE], &mo.sh_gate, nullptr)) || (rc = B.one(T[PYRE_MTP_SH_UP], &mo.sh_up, nullptr)) || (rc = B.one(T[PYRE_MTP_SH_DOWN], &mo.sh_down, nullptr))) return rc;
  mo.d = d; mo.n_exp = cfg->n_exp; mo.top_k = cfg->top_k; mo.ff = cfg->ff; mo.sf = mo.sh_gate.rows;
  if (mo.router.rows != cfg->n_exp || mo.router.cols != d || mo.gate_e.rows != cfg->n_exp * cfg->ff || mo.up_e.rows != cfg->n_exp * cfg->ff || mo.gate_e.cols != d || mo.up_e.cols != d ||
      (size_t)mo.down_e.rows != (size_t)cfg->n_exp * d || mo.down_e.cols != cfg->ff || mo.sh_up.rows != mo.sf || mo.sh_down.rows != d || mo.sh_down.cols != mo.sf || mo.sf % 64)
    return B.fail(PYRE_E_SHAPE, "drafter expert tensor shapes");
  if (mo.gate_e.fmt != mo.up_e.fmt || mo.sh_gate.fmt != mo.gate_e.fmt || mo.sh_up.fmt != mo.gate_e.fmt || mo.sh_down.fmt != mo.down_e.fmt) return B.fail(PYRE_E_TYPE, "gate/up (and shared) expert types must agree");
  if ((rc = B.vec(T[PYRE_MTP_SH_GATE_INP], d, &mo.sh_gate_inp))) return rc;
  if ((rc = B.one(T[PYRE_MTP_HEAD], &m->head, nullptr, mlay))) return rc;
  if (m->head.rows != cfg->n_draft_vocab || m->head.cols != d) return B.fail(PYRE_E_SHAPE, "the draft head must hold n_draft_vocab rows of d");
  PYRE_HIP(ctx, hipMalloc((void**)&m->ids_dev, (size_t)cfg->n_draft_vocab * 4)); m->shell.bufs.push_back(m->ids_dev);
  PYRE_HIP(ctx, hipMemcpy(m->ids_dev, draft_ids, (size_t)cfg->n_draft_vocab * 4, hipMemcpyHostToDevice));
  // workspace for up to 8 rows
  HcDev hmax = m->hca; hmax.lr = std::max(m->hca.lr, std::max(m->hcf.lr, m->mix.lr));
  const size_t moe_b = pyre_moe_work_bytes(mo), f8d = 4 * 8 * (size_t)d, nhd = (size_t)c.n_head * c.hd;
  size_t total = al256(pyre_hc_work_bytes(hmax)) + al256(moe_b) + 13 * al256(f8d) + 5 * al256(4 * 64) + al256(4 * 8 * (size_t)m->pw) + al256(4 * 8 * nhd) + al256(4 * (size_t)cfg->n_draft_vocab) + 3 * 256 + 4096;
  PYRE_HIP(ctx, hipMalloc(&m->work, total)); PYRE_HIP(ctx, hipMemset(m->work, 0, total));
  uint8_t* p = (uint8_t*)m->work; auto take = [&](size_t n) { void* r = p; p += al256(n); return r; };
  pyre_hc_work_carve(hmax, take(pyre_hc_work_bytes(hmax)), &m->hw); pyre_moe_work_carve(mo, take(moe_b), &m->mw);
  m->emb = (float*)take(f8d); m->en = (float*)take(f8d); m->e2 = (float*)take(f8d); m->hn = (float*)take(f8d); m->xh = (float*)take(f8d); m->ra = (float*)take(f8d); m->rb = (float*)take(f8d); m->rc = (float*)take(f8d);
  m->mixed = (float*)take(f8d); m->bo = (float*)take(f8d); m->y = (float*)take(f8d); m->sh = (float*)take(f8d); (void)take(f8d);
  m->inj_a = (float*)take(4 * 64); m->inj_f = (float*)take(4 * 64); m->inj_m = (float*)take(4 * 64); m->zeros = (float*)take(4 * 64); (void)take(4 * 64);
  m->proj = (float*)take(4 * 8 * (size_t)m->pw); m->core = (float*)take(4 * 8 * nhd); m->logits = (float*)take(4 * (size_t)cfg->n_draft_vocab);
  m->out_p = (float*)take(4 * 8); m->out_ids = (uint32_t*)take(4 * 8); m->tok = (uint32_t*)take(4 * 8);
  { uint4* op; float* ainv; const int kmax = std::max(d, (int)nhd); if ((rc = pyre_gemm_m_scratch(ctx, (kmax + 255) / 256 * 256, &op, &ainv))) return rc; }      // no draft step allocates
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  guard.armed = false; *out = M.release(); return PYRE_OK;
}

// Mtp::load (src/model/mtp.rs:99-118) from the one-file BF16 checkpoint: tensor names as the reference reads them, norm
// vectors as 1 + w, the fused mlp.experts.gate_up_proj [experts][2 ff][d] split into its gate (rows 0 .. ff of an expert)
// and up (rows ff .. 2 ff) halves, experts and width from mlp.experts.down_proj [experts][d][ff]; the matrices stay BF16
// (the reference re-quantizes them to int8 at load, mtp.rs:11-13).  head == NULL: the draft head is the rows draft_ids
// of the main model's output matrix, dequantized exactly (f32).
int pyre_mtp_load_safetensors(pyre_ctx* ctx, const pyre_model* main, const char* path, int top_k, int window, const uint32_t* draft_ids, int n_draft_vocab, const pyre_tensor* head, pyre_mtp** out) {
  if (!ctx || !main || !path || !draft_ids || !out || n_draft_vocab < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_load_safetensors: bad argument");
  *out = nullptr; const pyre_model_cfg& c = main->c;
  char err[512] = {0}; pyre_st* st = nullptr;
  int rc = pyre_st_open(path, &st, err, sizeof err); if (rc) return pyre_fail(ctx, rc, "pyre_mtp_load_safetensors: %s", err);
  struct Closer { pyre_st* s; ~Closer() { pyre_st_close(s); } } closer{st};
  std::vector<std::vector<float>> f32s; std::vector<std::vector<uint16_t>> halves; f32s.reserve(16); halves.reserve(4);
  pyre_tensor T[PYRE_MTP_SLOTS]; memset(T, 0, sizeof T);
  auto raw = [&](const std::string& n, const uint16_t** d, std::vector<uint64_t>* sh) { const void* p; uint32_t nd; uint64_t dims[8]; int r = pyre_st_tensor(st, n.c_str(), &p, &nd, dims, err, sizeof err);
    if (r) return pyre_fail(ctx, r, "pyre_mtp_load_safetensors: %s", err); *d = (const uint16_t*)p; sh->assign(dims, dims + nd); return (int)PYRE_OK; };
  auto mat = [&](int slot, const std::string& n) { const uint16_t* d; std::vector<uint64_t> sh; int r = raw(n, &d, &sh); if (r) return r;
    if (sh.size() != 2) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_mtp_load_safetensors: %s is not a matrix", n.c_str());
    T[slot] = pyre_tensor{PYRE_BF16, 0, sh[0], sh[1], d}; return (int)PYRE_OK; };
  auto vec = [&](int slot, const std::string& n, float add) { const uint16_t* d; std::vector<uint64_t> sh; int r = raw(n, &d, &sh); if (r) return r;
    uint64_t cnt = 1; for (uint64_t v : sh) cnt *= v;
    f32s.emplace_back((size_t)cnt); std::vector<float>& y = f32s.back();
    for (size_t i = 0; i < (size_t)cnt; ++i) { const uint32_t u = (uint32_t)d[i] << 16; float f; memcpy(&f, &u, 4); y[i] = f + add; }            // St::row, St::norm
    T[slot] = pyre_tensor{PYRE_F32, 0, 1, cnt, y.data()}; return (int)PYRE_OK; };
  if ((rc = vec(PYRE_MTP_PRE_E, "pre_fc_norm_embedding.weight", 1.0f)) || (rc = vec(PYRE_MTP_PRE_H, "pre_fc_norm_hidden.weight", 1.0f)) ||
      (rc = mat(PYRE_MTP_FC_E, "fc_embedding.weight")) || (rc = mat(PYRE_MTP_FC_H, "fc_hidden.weight"))) return rc;
  const struct { const char* p; int norm, down, inject, up; } hcs[3] = {{"attn_hyper_connection", PYRE_MTP_HCA_NORM, PYRE_MTP_HCA_DOWN, PYRE_MTP_HCA_INJECT, PYRE_MTP_HCA_UP},
    {"mlp_hyper_connection", PYRE_MTP_HCF_NORM, PYRE_MTP_HCF_DOWN, PYRE_MTP_HCF_INJECT, PYRE_MTP_HCF_UP}, {"hyper_connection_mixer", PYRE_MTP_MIX_NORM, PYRE_MTP_MIX_DOWN, -1, PYRE_MTP_MIX_UP}};
  for (const auto& h : hcs) { const std::string b = h.p;
    if ((rc = vec(h.norm, b + ".hc_norm.weight", 1.0f)) || (rc = mat(h.down, b + ".input_mix_weight_down.weight")) || (rc = mat(h.up, b + ".input_mix_weight_up.weight"))) return rc;
    if (h.inject >= 0 && (rc = mat(h.inject, b + ".block_inject_weight.weight"))) return rc; }
  if ((rc = mat(PYRE_MTP_Q, "self_attn.q_proj.weight")) || (rc = mat(PYRE_MTP_K, "self_attn.k_proj.weight")) || (rc = mat(PYRE_MTP_V, "self_attn.v_proj.weight")) || (rc = mat(PYRE_MTP_O, "self_attn.o_proj.weight")) ||
      (rc = vec(PYRE_MTP_QN, "self_attn.q_norm.weight", 1.0f)) || (rc = vec(PYRE_MTP_KN, "self_attn.k_norm.weight", 1.0f)) ||
      (rc = mat(PYRE_MTP_ROUTER, "mlp.gate.weight")) || (rc = mat(PYRE_MTP_SH_GATE, "mlp.shared_expert.gate_proj.weight")) || (rc = mat(PYRE_MTP_SH_UP, "mlp.shared_expert.up_proj.weight")) ||
      (rc = mat(PYRE_MTP_SH_DOWN, "mlp.shared_expert.down_proj.weight")) || (rc = vec(PYRE_MTP_SH_GATE_INP, "mlp.shared_expert_gate.weight", 0.0f))) return rc;
  const uint16_t *gu, *dn; std::vector<uint64_t> sg, sd;
  if ((rc = raw("mlp.experts.gate_up_proj", &gu, &sg)) || (rc = raw("mlp.experts.down_proj", &dn, &sd))) return rc;
  if (sd.size() != 3 || sg.size() != 3 || sg[0] != sd[0] || sg[1] != 2 * sd[2] || sg[2] != sd[1] || sd[1] != (uint64_t)c.d)
    return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_mtp_load_safetensors: mlp.experts.gate_up_proj / down_proj are not [experts][2 ff][d] / [experts][d][ff]");
  const size_t ne = (size_t)sd[0], ff = (size_t)sd[2], d = (size_t)c.d;            // mtp.rs:104
  halves.emplace_back(ne * ff * d); halves.emplace_back(ne * ff * d);
  for (size_t e = 0; e < ne; ++e) { memcpy(halves[0].data() + e * ff * d, gu + e * 2 * ff * d, ff * d * 2); memcpy(halves[1].data() + e * ff * d, gu + (e * 2 + 1) * ff * d, ff * d * 2); }
  T[PYRE_MTP_GATE_E] = pyre_tensor{PYRE_BF16, 0, ne * ff, d, halves[0].data()}; T[PYRE_MTP_UP_E] = pyre_tensor{PYRE_BF16, 0, ne * ff, d, halves[1].data()};
  T[PYRE_MTP_DOWN_E] = pyre_tensor{PYRE_BF16, 0, ne * d, ff, dn};
  float* head_dev = nullptr; uint32_t* ids_dev = nullptr;
  struct Free { float** a; uint32_t** b; ~Free() { if (*a) (void)hipFree(*a); if (*b) (void)hipFree(*b); } } fr{&head_dev, &ids_dev};
  if (head) T[PYRE_MTP_HEAD] = *head;
  else {            // Q8Mat::from_fn(ids.len(), d, head_row(ids[r])), mtp.rs:106, without the int8 step
    for (int i = 0; i < n_draft_vocab; ++i) if (draft_ids[i] >= (uint32_t)c.vocab) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_load_safetensors: draft id %u outside the vocabulary (%d)", draft_ids[i], c.vocab);
    PYRE_HIP(ctx, hipSetDevice(ctx->device));
    PYRE_HIP(ctx, hipMalloc((void**)&head_dev, (size_t)n_draft_vocab * d * 4)); PYRE_HIP(ctx, hipMalloc((void**)&ids_dev, (size_t)n_draft_vocab * 4));
    PYRE_HIP(ctx, hipMemcpy(ids_dev, draft_ids, (size_t)n_draft_vocab * 4, hipMemcpyHostToDevice));
    for (int r0 = 0; r0 < n_draft_vocab; r0 += 32768) { const int nr = std::min(32768, n_draft_vocab - r0); if ((rc = pyre_row_launch(ctx, main->out, ids_dev + r0, nr, head_dev + (size_t)r0 * d, (int)d))) return rc; }
    PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
    T[PYRE_MTP_HEAD] = pyre_tensor{PYRE_F32, 1, (uint64_t)n_draft_vocab, (uint64_t)d, head_dev};
  }
  pyre_mtp_cfg cfg{(int32_t)ne, top_k > 0 ? std::min(top_k, c.top_k) : c.top_k, (int32_t)ff, window > 0 ? window : 128, n_draft_vocab};            // PYRE_MTP_TOPK capped by the model's, PYRE_MTP_WINDOW 128: mtp.rs:108,117
  return pyre_mtp_create(ctx, main, &cfg, T, draft_ids, out);
}

void pyre_mtp_destroy(pyre_mtp* m) {
  if (!m) return; (void)hipSetDevice(m->ctx->device); (void)hipStreamSynchronize(m->ctx->stream);
  for (auto q : m->shell.owned) pyre_qmat_destroy(q); for (auto b : m->shell.bufs) (void)hipFree(b); if (m->work) (void)hipFree(m->work);
  delete m;
}

int pyre_state_attach_mtp(pyre_ctx* ctx, pyre_state* s, const pyre_mtp* m) {
  if (!ctx || !s || !m) return pyre_fail(ctx, PYRE_E_ARG, "pyre_state_attach_mtp: null argument");
  if (s->m != m->main) return pyre_fail(ctx, PYRE_E_STATE, "pyre_state_attach_mtp: the drafter was built for another model");
  if (s->mtp) return pyre_fail(ctx, PYRE_E_STATE, "pyre_state_attach_mtp: the state already has a drafter");
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  const pyre_model_cfg& c = s->m->c; const size_t w = (size_t)c.hc * c.d;
  int rows = 32; while (rows < m->c.window + 24) rows *= 2;      // a window of 8 lands before the oldest of window + 16 kept rows is dropped
  const size_t rb = al256((size_t)rows * w * 4), kvb = al256(pyre_kv_bytes(m->attn, s->cap)), lb = al256(4 * ((size_t)m->c.window + 16)), tkb = s->tokens_dev ? 0 : al256((size_t)s->cap * 4);
  hipError_t e = hipMalloc(&s->mtp_mem, rb + kvb + lb + 256 + tkb);
  if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_state_attach_mtp: hipMalloc(%zu): %s", rb + kvb + lb + 256 + tkb, hipGetErrorString(e));
  uint8_t* p = (uint8_t*)s->mtp_mem; auto take = [&](size_t n) { void* r = p; p += n; return r; };
  s->r_ring = (float*)take(rb); s->r_mask = rows - 1; pyre_kv_carve(m->attn, s->cap, take(kvb), &s->mkv); s->mlist = (int*)take(lb); s->mcount = (int*)take(256);
  if (tkb) { s->tokens_dev = (uint32_t*)take(tkb); PYRE_HIP(ctx, hipMemset(s->tokens_dev, 0, tkb)); }
  s->r_first = s->r_next = 0; s->m_c0 = s->m_n = 0; s->mtp = m;
  if (s->graph_exec) { (void)hipGraphExecDestroy(s->graph_exec); s->graph_exec = nullptr; }      // a captured step does not store its residual yet
  return PYRE_OK;
}

int pyre_mtp_draft(pyre_ctx* ctx, const pyre_mtp* m, pyre_state* s, uint32_t pending, int k, float min_p, uint32_t* ids_host, float* probs_host, int* n_out) {
  if (!ctx || !m || !s || !ids_host || !probs_host || !n_out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_draft: null argument");
  *n_out = 0;
  if (s->mtp != m) return pyre_fail(ctx, PYRE_E_STATE, "pyre_mtp_draft: this drafter is not attached to the state");
  if (k > 7) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_draft: k = %d above 7", k);
  const pyre_model* main = m->main; const pyre_model_cfg& c = main->c; const int n = s->len, d = c.d, hc = c.hc, window = m->c.window; int rc;
  if (n == 0 || k <= 0) return PYRE_OK;
  if (pending >= (uint32_t)c.vocab) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_draft: token id %u outside the vocabulary (%d)", pending, c.vocab);
  if (n - 1 + k > s->cap) return pyre_fail(ctx, PYRE_E_STATE, "pyre_mtp_draft: cells up to %d exceed the state's capacity %d", n - 1 + k, s->cap);
  auto have_r = [&](int pos) { return pos >= s->r_first && pos < s->r_next; };
  auto grow = [&](int pos0, int t) { if (s->m_c0 + s->m_n != pos0) { s->m_c0 = pos0; s->m_n = 0; } s->m_n += t; if (s->m_n > window) { s->m_c0 += s->m_n - window; s->m_n = window; } };      // kv_append's bookkeeping, mtp.rs:163-176
  if (n - 1 < s->m_c0 + s->m_n) s->m_n = std::max(0, n - 1 - s->m_c0);                                     // kv.truncate(n - 1)
  // catch-up over the cells whose residual is known and whose token is committed (:2194-2217)
  const int first = s->r_next > s->r_first ? s->r_first : n, end = s->m_c0 + s->m_n;
  const int lo = (s->m_n > 0 && end >= first) ? end : std::max(first, std::max(0, (n - 1) - window));
  if (lo < n - 1) {
    bool ok = true; for (int i = lo; i < n - 1; ++i) ok = ok && have_r(i);
    if (ok) {
      const int per = 8 / hc;
      for (int p0 = lo; p0 < n - 1; p0 += per) {
        const int t = std::min(per, n - 1 - p0);
        if ((rc = pyre_row_launch(ctx, main->embd, s->tokens_dev + p0 + 1, t, m->emb, d))) return rc;
        if ((rc = mtp_cells(ctx, m, s->r_ring, s->r_mask, p0, t))) return rc;
        if ((rc = pyre_attn_append_launch(ctx, m->attn, s->mkv, s->aw, m->proj, m->pw, p0, t))) return rc;
        grow(p0, t);
      }
    } else { s->m_c0 = 0; s->m_n = 0; }
  }
  if (!have_r(n - 1)) return PYRE_OK;
  // the k draft steps: cell n-1+j attends to the window's cells, which the host knows in advance
  int c0 = s->m_c0, cn = s->m_n, lo0 = 0; MtpCounts cnt{}; int c0j[8];
  for (int j = 0; j < k; ++j) { const int pos = n - 1 + j; if (c0 + cn != pos) { c0 = pos; cn = 0; } ++cn; if (cn > window) { c0 += cn - window; cn = window; } c0j[j] = c0; cnt.c[j] = cn; if (j == 0) lo0 = c0; }
  const int nlist = n - 1 + k - lo0;
  hipLaunchKernelGGL(k_mtp_list, dim3((std::max(nlist, 8) + 255) / 256), dim3(256), 0, ctx->stream, s->mlist, lo0, nlist, s->mcount, cnt); PYRE_CHECK_LAUNCH(ctx);
  PYRE_HIP(ctx, hipMemcpyAsync(m->tok, &pending, 4, hipMemcpyHostToDevice, ctx->stream));
  const float* r = s->r_ring; int mask = s->r_mask, rpos = n - 1;
  for (int j = 0; j < k; ++j) {
    const int pos = n - 1 + j;
    if ((rc = pyre_row_launch(ctx, main->embd, m->tok, 1, m->emb, d))) return rc;
    if ((rc = mtp_cells(ctx, m, r, mask, rpos, 1))) return rc;
    QsaWork qw{}; qw.plist = s->mlist + (c0j[j] - lo0); qw.pcount = s->mcount + j; qw.list_stride = window;
    int packed = 0;
    if ((rc = pyre_attn_launch_sel(ctx, m->attn, s->mkv, s->aw, m->proj, m->pw, pos, 1, &packed, m->core, nullptr, &qw))) return rc;
    if ((rc = pyre_gemv_launch(ctx, m->outp, m->core, 1, m->bo))) return rc;
    if ((rc = pyre_hc_mix_launch(ctx, m->hcf, m->hw, m->ra, d, hc * d, m->rb, 1, m->bo, nullptr, m->inj_a, c.eps, m->mixed, m->inj_f, nullptr, 1, nullptr))) return rc;
    if ((rc = pyre_moe_launch(ctx, m->moe, m->mw, m->mixed, 1, m->y, nullptr))) return rc;
    if ((rc = pyre_hc_mix_launch(ctx, m->mix, m->hw, m->rb, d, hc * d, m->rc, 1, m->y, nullptr, m->inj_f, c.eps, m->sh, m->inj_m, nullptr, 1, nullptr))) return rc;
    if ((rc = pyre_gemv_launch(ctx, m->head, m->sh, 1, m->logits))) return rc;
    hipLaunchKernelGGL(k_mtp_best, dim3(1), dim3(1024), 0, ctx->stream, m->logits, m->c.n_draft_vocab, m->ids_dev, m->out_ids + j, m->out_p + j, m->tok); PYRE_CHECK_LAUNCH(ctx);
    grow(pos, 1);
    r = m->rc; mask = -1; rpos = 0;      // the drafter's own residual feeds the next step
  }
  uint32_t ids[8]; float ps[8];
  PYRE_HIP(ctx, hipMemcpyAsync(ids, m->out_ids, (size_t)k * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipMemcpyAsync(ps, m->out_p, (size_t)k * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  int got = 0; for (int j = 0; j < k; ++j) { if (j > 0 && ps[j] < min_p) break; ids_host[got] = ids[j]; probs_host[got] = ps[j]; ++got; }      // draft_gate, policy off (spec.rs:326-327)
  if (n < s->m_c0 + s->m_n) s->m_n = std::max(0, n - s->m_c0);                                            // kv.truncate(n): the drafted cells go
  *n_out = got; return PYRE_OK;
}

int pyre_mtp_read_kv(pyre_ctx* ctx, pyre_state* s, int* c0, int* n, float* k_host, float* v_host) {
  if (!ctx || !s || !s->mtp || !c0 || !n) return pyre_fail(ctx, PYRE_E_ARG, "pyre_mtp_read_kv: bad argument");
  const AttnDev& a = s->mtp->attn; const size_t row = (size_t)a.nkv * a.hd; *c0 = s->m_c0; *n = s->m_n;
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (s->m_n == 0) return PYRE_OK;
  if (v_host) PYRE_HIP(ctx, hipMemcpy(v_host, s->mkv.vf + (size_t)s->m_c0 * row, (size_t)s->m_n * row * 4, hipMemcpyDeviceToHost));
  if (k_host) {      // keys are blocked by 64 positions: fetch the blocks that hold the cells and pick the rows out on the host
    const size_t b0 = (size_t)s->m_c0 / 64, b1 = ((size_t)s->m_c0 + s->m_n + 63) / 64; std::vector<float> tmp((b1 - b0) * row * 64);
    PYRE_HIP(ctx, hipMemcpy(tmp.data(), s->mkv.kf + b0 * row * 64, tmp.size() * 4, hipMemcpyDeviceToHost));
    for (int i = 0; i < s->m_n; ++i) { const size_t p = (size_t)s->m_c0 + i; for (size_t r = 0; r < row; ++r) k_host[(size_t)i * row + r] = tmp[kv_blk(r, row, p) - b0 * row * 64]; }
  }
  return PYRE_OK;
}

// forced: the drafter runs (its cost is paid) and its ids are then replaced by forced[produced ..] -- with the plain greedy
// stream there, every draft is accepted: the accepted path timed end to end, whatever the drafter's weights would draft
static int generate_greedy_mtp(pyre_ctx* ctx, const pyre_model* m, const pyre_mtp* mtp, pyre_state* s, const float* first_logits, int n_out, uint32_t* out, int k, float min_p, int* rounds_out, int* drafted_out, int* accepted_out, const uint32_t* forced) {
  if (!ctx || !m || !mtp || !s || !first_logits || !out || n_out < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy_mtp: bad argument");
  if (k < 1 || k > 7) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy_mtp: k %d outside 1..7", k);
  if (s->mtp != mtp) return pyre_fail(ctx, PYRE_E_STATE, "pyre_generate_greedy_mtp: this drafter is not attached to the state");
  const size_t V = m->c.vocab; int produced = 0, rounds = 0, drafted = 0, accepted = 0;
  SpecAdapt ad(ctx); if (forced) ad.on = false;
  uint32_t pending = host_argmax(first_logits, V);
  for (;;) {
    out[produced++] = pending; if (produced >= n_out) break;
    const int left = n_out - produced; const int kk = ad.plan(k < left - 1 ? k : left - 1);
    uint32_t toks[8]; float ps[8]; toks[0] = pending; int nd = 0;
    if (kk > 0) { ad.tick(); int rc = pyre_mtp_draft(ctx, mtp, s, pending, kk, min_p, toks + 1, ps, &nd); if (rc) return rc; ad.drafted(ad.tock()); }
    if (forced && kk > 0) { nd = kk; for (int j = 0; j < kk; ++j) toks[j + 1] = forced[produced + j]; }
    nd = ad.trim(nd);
    uint32_t picks[8]; ad.tick(); int rc = forward_multi_picks(ctx, m, s, toks, nd + 1, picks); if (rc) return rc;
    if (nd == 0) ad.plain(ad.tock()); else ad.verified(nd + 1, ad.tock());
    int acc = 0; bool have = false; uint32_t nx = 0;
    for (int i = 0; i < nd; ++i) { uint32_t tk = picks[i]; if (tk == toks[i + 1]) { ++acc; continue; } nx = tk; have = true; break; }
    if (!have) nx = picks[nd];
    if ((rc = pyre_spec_keep(ctx, m, s, nd + 1, acc + 1))) return rc;
    if (nd > 0) ad.accepted(acc, nd);
    if (nd > 0) ++rounds; drafted += nd; accepted += acc;
    bool stop = false; for (int i = 0; i < acc; ++i) { out[produced++] = toks[i + 1]; if (produced >= n_out) { stop = true; break; } }
    if (stop) break;
    pending = nx;
  }
  if (rounds_out) *rounds_out = rounds; if (drafted_out) *drafted_out = drafted; if (accepted_out) *accepted_out = accepted;
  return PYRE_OK;
}
int pyre_generate_greedy_mtp(pyre_ctx* ctx, const pyre_model* m, const pyre_mtp* mtp, pyre_state* s, const float* first_logits, int n_out, uint32_t* out, int k, float min_p, int* rounds_out, int* drafted_out, int* accepted_out) {
  return generate_greedy_mtp(ctx, m, mtp, s, first_logits, n_out, out, k, min_p, rounds_out, drafted_out, accepted_out, nullptr);
}
int pyre_generate_greedy_mtp_forced(pyre_ctx* ctx, const pyre_model* m, const pyre_mtp* mtp, pyre_state* s, const float* first_logits, int n_out, uint32_t* out, int k, const uint32_t* forced_stream, int* rounds_out, int* drafted_out, int* accepted_out) {
  if (!forced_stream) return pyre_fail(ctx, PYRE_E_ARG, "pyre_generate_greedy_mtp_forced: null draft stream");
  return generate_greedy_mtp(ctx, m, mtp, s, first_logits, n_out, out, k, 0.0f, rounds_out, drafted_out, accepted_out, forced_stream);
}

}  // extern "C"
