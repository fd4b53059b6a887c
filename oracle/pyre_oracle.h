/* CPU oracle for the Qwen-Next (qwen4exp) decode token loop.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a from-scratch f32 restatement of the reference's host
 * path (src/model/gguf_q.rs, src/model/kv4.rs, src/model/qwen4exp_gguf.rs, src/qn_ctx.rs,
 * src/sampler.rs, src/spec.rs of the reference tree), used as the checker by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg.  Nothing in the shipped HIP
 * library links, loads or calls it.
 *
 * Pinning status (what fixes each function besides transcription):
 *   orc_dequant            known-answer blocks derived from the format definition, the
 *                          codebook digests, an independent numpy statement (tests/), sign and
 *                          scale single-bit perturbation tests
 *   orc_dot / orc_matmul   f64-accumulated dot of the dequantized rows
 *   orc_kv4_*              the reference's own test inputs and asserted properties
 *                          (kv4.rs:52-104), brute-force numpy statement
 *   orc_rope_inv           closed form base^(-2i/n_rot), qn_ctx.rs:406-411
 *   orc_argmax             sampler.rs:154-159 vector
 *   orc_top_k              brute force on distinct logits + explicit ties
 *   orc_gdn_core           closed forms (zero state, delta-rule overwrite property, pure decay,
 *                          one-hot conv = delay) + an independent numpy statement
 *   orc_attn_core          single position, uniform keys, rope at pos 0, numpy statement
 *   orc_attn_core_qsa      equals the dense branch up to budget + ratio - 1 positions; selection by brute force
 *                          (numpy sort) on distinct scores; hand-built keys that force a known block set;
 *                          block pooling closed form (identical keys -> pooled key = rope(rms(key)))
 *   orc_rope_inv_yarn      the reference's asserted properties (qn_ctx.rs:406-419) + float64 closed form
 *   orc_hc_mix             closed forms: zero up (or zero down) -> half the mean of the normalised streams;
 *                          one-hot down / inject / up rows -> silu(x_j / hc), x_m / hc and the stream-major gate
 *                          layout as explicit numbers; windows == single tokens
 *   orc_hc_combine         inject 0 -> x + out exactly; -inf -> unchanged; +inf -> x + 2 out; ln 3 -> x + 1.5 out
 *   orc_moe_ffn            closed forms: shared expert alone with a zero gate vector -> halved SwiGLU of picked
 *                          inputs; two chosen experts, one with a zero down matrix -> w1 * down_1 (silu(g) * u) with
 *                          w1 the two-way softmax; all-ones Q8_0 matrices -> sf silu(S) S sigmoid(x_0) + ff silu(S) S;
 *                          + a numpy statement built from orc_dequant'd dense weights
 *   orc_forward            all block outputs zeroed -> head(hc_mix(tiled embedding of the last token)) bit for bit;
 *                          one live FFN / one live DeltaNet layer -> the composition of the pinned block entry
 *                          points bit for bit (and not with the other mixer's inject factors); + a numpy statement
 *                          of the whole token step on a tiny model
 *   orc_ple_rows / orc_ple closed forms: multipliers that single out one context token (operand order, cut at the
 *                          sequence start and at eos, 64-bit wrap, xor); zero value -> the conv over a hand-set history
 *                          tap by tap; zero key -> the gate floor; one-hot key / stream -> the gate in closed form;
 *                          constant gated stream -> the norm weight; window == single tokens
 *   orc_mtp_draft          closed forms: a zero head -> the first draft id with probability exactly 1 / n and the min_p gate
 *                          sparing only the first draft; a zero fc_hidden -> a cell depends only on the token one position
 *                          ahead and its key is that token's key turned by the plain rope table at the cell's index (under
 *                          a YaRN-scaled main model); a zero fc_embedding -> a cell depends only on its position's residual;
 *                          catch-up start / window / both truncations as numbers worked out by hand; the draft step as the
 *                          composition of the pinned block entry points (matmul, hc_mix, hc_combine, attn_core, moe_ffn);
 *                          generation with the drafter proposing == plain greedy
 * Parity unpinned (only running the reference could pin): the last-ulp behaviour of
 * expf/log1pf/powf/sincosf on the reference's own target libm.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids, gguf_q.rs:25-28 */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_Q4_0 = 2, ORC_Q5_0 = 6, ORC_Q8_0 = 8, ORC_Q4_K = 12, ORC_Q6_K = 14, ORC_IQ2_XXS = 16, ORC_IQ2_XS = 17, ORC_IQ3_XXS = 18,
       ORC_IQ4_NL = 20, ORC_IQ3_S = 21, ORC_IQ2_S = 22, ORC_IQ4_XS = 23, ORC_BF16 = 30, ORC_Q3_K = 11, ORC_Q2_0 = 42, ORC_Q5_K = 13, ORC_IQ1_M = 29 };

typedef struct { uint32_t ty; uint64_t rows, cols; const void* data; } OrcTensor;

/* per-layer tensor slots (GGUF tensor names in comments, qwen4exp_gguf.rs:494-512) */
enum {
  ORC_HCA_NORM = 0, ORC_HCA_DOWN, ORC_HCA_INJECT, ORC_HCA_UP,       /* blk.N.hc_attn_{norm,down,inject,up} */
  ORC_HCF_NORM, ORC_HCF_DOWN, ORC_HCF_INJECT, ORC_HCF_UP,           /* blk.N.hc_ffn_* */
  ORC_ATTN_Q, ORC_ATTN_K, ORC_ATTN_V, ORC_ATTN_O, ORC_ATTN_QN, ORC_ATTN_KN,
  ORC_LIN_QKV, ORC_LIN_Z, ORC_LIN_BETA, ORC_LIN_ALPHA, ORC_LIN_A, ORC_LIN_DT, ORC_LIN_CONV, ORC_LIN_NORM, ORC_LIN_OUT,
  ORC_ROUTER, ORC_GATE_E, ORC_UP_E, ORC_DOWN_E, ORC_SH_GATE_INP, ORC_SH_GATE, ORC_SH_UP, ORC_SH_DOWN,
  ORC_IDX_Q, ORC_IDX_K, ORC_IDX_QN, ORC_IDX_KN,                     /* blk.N.indexer.{q_proj,k_proj,q_norm,k_norm}.weight (optional) */
  ORC_PLE_KEY, ORC_PLE_VALUE, ORC_PLE_NK, ORC_PLE_NQ, ORC_PLE_NC, ORC_PLE_CONV,   /* blk.N.ple_{key,value,norm_key,norm_query,norm_conv,conv1d}.weight (layers listed in ple.layers, :505) */
  ORC_LAYER_SLOTS
};
enum { ORC_G_EMBD = 0, ORC_G_HEAD_NORM, ORC_G_HEAD_DOWN, ORC_G_HEAD_UP, ORC_G_OUT, ORC_G_PLE_TAB /* per_layer_token_embd.weight (:512) */, ORC_GLOBAL_SLOTS };

typedef struct {
  int32_t n_layers, d, hc, hc_lr, n_head, n_kv, hd, n_rot;
  float rope_base, eps;
  int32_t n_exp, top_k, ff_exp;
  int32_t lin_nk, lin_nv, lin_dk, lin_dv, conv_k, full_every;
  int32_t vocab;
  int32_t kv_bits;    /* 0 = f32 cache everywhere, 4 = positions below the packed boundary are read through kv4 */
  int32_t kv_recent;  /* f32 window kept at the tail (reference default 1024) */
  /* QSA sparse indexer (qwen4exp_gguf.rs:24-25): heads (0 = none), key length, block size in tokens, token budget */
  int32_t idx_nh, idx_hd, idx_ratio, idx_budget;
  /* trained context and the context the model is built for; ctx > ctx_train > 0 switches YaRN on (qn_ctx.rs:164-185) */
  int32_t ctx_train, ctx;
  /* per-layer n-gram embeddings (qwen4exp_gguf.rs:22-23, 477-480): n-gram length (0 = none), table heads per n-gram length,
   * conv kernel length, width of a table row, the token that cuts an n-gram's context; per position of the n-gram a 64-bit
   * multiplier, per head an offset into the table and a modulus */
  int32_t ple_ngram, ple_per_gram, ple_conv_k, ple_dim;
  uint32_t ple_eos; int32_t ple_reserved;
  uint64_t ple_mult[8], ple_off[16], ple_vocab[16];
} OrcCfg;

int    orc_type_geom(uint32_t ty, int* elems, int* bytes);
int    orc_dequant(uint32_t ty, const uint8_t* x, size_t n_elems, float* y);
float  orc_dot(const float* a, const float* b, size_t n);
int    orc_matmul(uint32_t ty, const uint8_t* w, size_t rows, size_t cols, const float* x, int t, float* y, int threads);
void   orc_expand_iq3s(uint32_t* out512);
void   orc_expand_iq2xs(uint64_t* out512);
uint8_t orc_ksigns(int i);

void   orc_kv4_pack(const float* x, size_t n, uint32_t* w, float* sc);
float  orc_kv4_get(const uint32_t* w, const float* sc, size_t i);
void   orc_kvq_roundtrip(float* x, size_t n, int bits);
size_t orc_kv_packed_boundary(size_t n_visible, int kv_bits, int recent);

void   orc_rope_inv(int n_rot, float base, float* inv);
/* qn_ctx::rope_inv with the YaRN branch; returns mscale (1 when ctx <= ctx_train or ctx_train == 0). */
float  orc_rope_inv_yarn(int n_rot, float base, int ctx_train, int ctx, float* inv);
uint32_t orc_argmax(const float* logits, size_t n);
int    orc_top_k(const float* r, int n, int k, int32_t* idx, float* w);
void   orc_rms(const float* x, const float* w, float eps, float* y, size_t n);
void   orc_rms_inplace(float* x, const float* w, float eps, size_t n);
float  orc_sigm(float x);
float  orc_silu(float x);
float  orc_softplus(float x);

/* Gated DeltaNet after its projections (linear_core).  proj = qkv [t][ch], z [t][nv*dv], beta [t][nv], alpha [t][nv].
 * conv_state [(k-1)][ch] oldest first, ssm [nv][dk][dv]; both updated in place.  out [t][nv*dv]. */
void   orc_gdn_core(int nk, int nv, int dk, int dv, int conv_k, float eps,
                    const float* a, const float* dt, const float* conv_w, const float* norm_w,
                    const float* qkv, const float* z, const float* beta, const float* alpha, int t,
                    float* conv_state, float* ssm, float* out);

/* Gated attention core (attn_core, dense branch).  q [t][nh][2*hd], k,v [t][nkv*hd] (raw projections).
 * kc/vc: caller-owned caches with room for start+t rows of nkv*hd floats; rows [0,start) valid on entry. */
void   orc_attn_core(int nh, int nkv, int hd, int n_rot, float eps, const float* rope_inv,
                     const float* qn, const float* kn, const float* q, const float* k, const float* v,
                     int start, int t, int kv_bits, int kv_recent, float* kc, float* vc, float* out);

/* attn_core with the QSA indexer (qwen4exp_gguf.rs:1565-1599) and the YaRN magnitude factor.  iq [t][idx_nh*idx_hd],
 * ik [t][idx_hd] raw indexer projections; ikc [cap][idx_hd] raw index keys and ibc [cap/ratio][idx_hd] pooled block keys
 * are caller-owned like kc/vc (rows [0,start) resp. [0,start/ratio) valid on entry).  sel (optional) receives, per
 * token, the attended positions in ascending order, sel_n[ti] of them, in rows of sel_stride ints; sel_n[ti] = -1 means
 * every visible position (dense).  Among blocks of equal score the lower block index is taken first (the reference's
 * select_nth_unstable leaves that order unspecified). */
void   orc_attn_core_qsa(int nh, int nkv, int hd, int n_rot, float eps, const float* rope_inv, float mscale,
                         const float* qn, const float* kn, const float* q, const float* k, const float* v,
                         int start, int t, int kv_bits, int kv_recent, float* kc, float* vc,
                         int idx_nh, int idx_hd, int idx_ratio, int idx_budget, const float* iqn, const float* ikn,
                         const float* iq, const float* ik, float* ikc, float* ibc,
                         float* out, int32_t* sel, int32_t* sel_n, int sel_stride);

/* MoE FFN (ffn + routed f32 branch).  x [t][d] -> y [t][d]. sel_idx/sel_w (optional) receive [t][k]. */
int    orc_moe_ffn(int d, int n_exp, int top_k, int ff, const OrcTensor* router, const OrcTensor* gate_e,
                   const OrcTensor* up_e, const OrcTensor* down_e, const float* sh_gate_inp,
                   const OrcTensor* sh_gate, const OrcTensor* sh_up, const OrcTensor* sh_down,
                   const float* x, int t, float* y, int32_t* sel_idx, float* sel_w, int threads);

/* Hyper-connection mix / combine (hc_mix, hc_combine).  inject may be NULL (head mixer). */
int    orc_hc_mix(int d, int hc, float eps, const float* norm, const OrcTensor* down, const OrcTensor* inject,
                  const OrcTensor* up, const float* x, int t, float* mixed, float* inj, int threads);
void   orc_hc_combine(int d, int hc, float* x, const float* out, const float* inj, int t);

/* ---- the multi-token-prediction (MTP) drafter, src/model/mtp.rs ------------------------------------------------------
 * One extra block that pairs the main model's final residual streams R_i with the token at i + 1 (cell i, rope position
 * i) and predicts token i + 2; its own residual feeds the next draft step.  Only draft quality depends on it: every
 * emitted token comes from the verify pass.  Tensors are given in the types the caller chose (the reference builds
 * int8 copies of a BF16 checkpoint, mtp.rs:11-13); norm weights already carry their "1 + w" (mtp.rs:44-45). */
enum {
  ORC_MTP_PRE_E = 0, ORC_MTP_PRE_H,                       /* pre_fc_norm_embedding [d], pre_fc_norm_hidden [hc*d] */
  ORC_MTP_FC_E, ORC_MTP_FC_H,                             /* fc_embedding [d x d], fc_hidden [d x d] (applied per stream) */
  ORC_MTP_HCA_NORM, ORC_MTP_HCA_DOWN, ORC_MTP_HCA_INJECT, ORC_MTP_HCA_UP,      /* attn_hyper_connection.* */
  ORC_MTP_HCF_NORM, ORC_MTP_HCF_DOWN, ORC_MTP_HCF_INJECT, ORC_MTP_HCF_UP,      /* mlp_hyper_connection.* */
  ORC_MTP_MIX_NORM, ORC_MTP_MIX_DOWN, ORC_MTP_MIX_UP,                          /* hyper_connection_mixer.* (no inject) */
  ORC_MTP_Q, ORC_MTP_K, ORC_MTP_V, ORC_MTP_O, ORC_MTP_QN, ORC_MTP_KN,          /* self_attn.* */
  ORC_MTP_ROUTER, ORC_MTP_GATE_E, ORC_MTP_UP_E, ORC_MTP_DOWN_E,                /* mlp.gate, mlp.experts.{gate,up}_proj halves, down_proj */
  ORC_MTP_SH_GATE_INP, ORC_MTP_SH_GATE, ORC_MTP_SH_UP, ORC_MTP_SH_DOWN,        /* mlp.shared_expert_gate, mlp.shared_expert.* */
  ORC_MTP_HEAD,                                            /* the draft-vocabulary rows of the main model's output matrix */
  ORC_MTP_SLOTS
};
typedef struct { int32_t n_exp, top_k, ff, window, n_draft_vocab; } OrcMtpCfg;      /* geometry beyond the main model's (Geo, mtp.rs:100) */
typedef struct OrcMtp OrcMtp;
typedef struct OrcModel OrcModel;
typedef struct OrcState OrcState;
OrcMtp*   orc_mtp_create(const OrcModel* main, const OrcMtpCfg* cfg, const OrcTensor* tensors /*[ORC_MTP_SLOTS]*/, const uint32_t* draft_ids /*[n_draft_vocab]*/);
void      orc_mtp_destroy(OrcMtp*);
/* the state keeps the last window + 16 final residuals from now on (mtp_keep_r, qwen4exp_gguf.rs:2279-2285) */
void      orc_state_attach_mtp(OrcState*, const OrcMtp*);
/* mtp_draft (qwen4exp_gguf.rs:2180-2277, host path, draft policy off): catch the drafter's K/V up over the cells whose token is
 * committed, then up to k draft steps from (R_{n-1}, pending); a later draft is kept only while the drafter's probability of
 * its choice is >= min_p (spec::draft_gate, spec.rs:326-327).  Returns the number of drafts; ids / probabilities out. */
int       orc_mtp_draft(const OrcMtp*, const OrcModel* main, OrcState*, uint32_t pending, int k, float min_p, uint32_t* ids, float* probs);
/* test access: the kept final residual streams [hc*d] of position pos (NULL when not kept); cells [c0, c0 + n) of the drafter's K / V [n][nkv*hd] */
const float* orc_mtp_r(const OrcState*, int pos);
int       orc_mtp_kv(const OrcState*, int* c0, const float** k, const float** v);
/* spec::generate's greedy branch with the drafter proposing (spec.rs:156-267): n_out tokens; rounds / drafted / accepted counts out */
int       orc_generate_greedy_mtp(const OrcModel*, const OrcMtp*, OrcState*, const float* first_logits, int n_out, uint32_t* out, int k, float min_p, int* drafted, int* accepted);
OrcModel* orc_model_create(const OrcCfg* cfg, const OrcTensor* layer_tensors /*[n_layers][ORC_LAYER_SLOTS]*/,
                           const OrcTensor* globals /*[ORC_GLOBAL_SLOTS]*/, int threads);
void      orc_model_destroy(OrcModel*);
OrcState* orc_state_create(const OrcModel*);
void      orc_state_destroy(OrcState*);
int       orc_state_len(const OrcState*);
/* direct access for tests: li-th GDN layer's conv / ssm, ai-th attention layer's k / v cache */
float*    orc_state_conv(OrcState*, int li);
float*    orc_state_ssm(OrcState*, int li);
float*    orc_state_k(OrcState*, int ai);
float*    orc_state_v(OrcState*, int ai);
float*    orc_state_ik(OrcState*, int ai);
float*    orc_state_ple_hist(OrcState*, int pi);      /* pi-th PLE layer: [(conv_k-1)*ngram][hc*d], oldest first */
/* ple_rows (qwen4exp_gguf.rs:1390-1407): table rows of positions start .. start+t-1 of `tokens` -> emb [t][heads*dim] */
int       orc_ple_rows(const OrcCfg* c, const OrcTensor* tab, const uint32_t* tokens, int start, int t, float* emb);
/* ple (qwen4exp_gguf.rs:1409-1434): x [t][hc*d] += gated + silu(conv); hist [(conv_k-1)*ngram][hc*d] advanced by t rows */
int       orc_ple(const OrcCfg* c, const OrcTensor* key, const OrcTensor* value, const float* nk, const float* nq, const float* nc, const float* conv,
                  float* hist, const float* emb, float* x, int t, int threads);
float*    orc_state_ib(OrcState*, int ai);
/* Model::forward: append ids, return logits of the last token in logits[vocab]. */
int       orc_forward(const OrcModel*, OrcState*, const uint32_t* ids, int n, float* logits);
/* forward_multi semantics = n sequential steps; logits [n][vocab]; keeps per-token checkpoints. */
int       orc_forward_multi(const OrcModel*, OrcState*, const uint32_t* ids, int n, float* logits);
/* spec_keep(t, keep): roll the state back so that only the first `keep` of the last t tokens remain. */
int       orc_spec_keep(const OrcModel*, OrcState*, int t, int keep);
/* spec::generate, greedy branch, with an optional fixed draft source: drafts[i] (n_draft per round) are proposed
 * after each pending token; out receives n_out tokens.  Returns the number of verify rounds used. */
int       orc_generate_greedy(const OrcModel*, OrcState*, const float* first_logits, int n_out, uint32_t* out,
                              int n_draft, const uint32_t* draft_stream);
#ifdef __cplusplus
}
#endif
