/* pyre_hip.h - C ABI of the MI355X (gfx950) library behind pyre's Qwen-Next (qwen4exp) decode token loop.
 *
 * One context = one HIP stream = one caller thread at a time (the reference drives its GPU from a single
 * "qn-worker" thread, engine_qn.rs:13-24).  Every entry point returns 0 on success or a negative code;
 * pyre_last_error() gives the text.  Nothing throws or unwinds across this boundary.  Matrices are copied to
 * device memory at create time (the caller may drop its bytes afterwards, where the reference keeps mmap views,
 * gguf_q.rs:201); states are opaque handles owned by the caller; "host" pointers are ordinary process memory,
 * "dev" pointers are HIP device memory on the context's device and are used on the context's stream.
 *
 * Paths cited below are relative to the reference tree (Lyamc/pyre).
 */
#ifndef PYRE_HIP_H
#define PYRE_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct pyre_ctx pyre_ctx;
typedef struct pyre_qmat pyre_qmat;
typedef struct pyre_model pyre_model;
typedef struct pyre_state pyre_state;

/* ggml tensor type ids accepted by pyre_qmat_create (QType::from_id, src/model/gguf_q.rs:25-28). */
enum { PYRE_F32 = 0, PYRE_F16 = 1, PYRE_Q4_0 = 2, PYRE_Q5_0 = 6, PYRE_Q8_0 = 8, PYRE_Q3_K = 11, PYRE_Q4_K = 12, PYRE_Q5_K = 13, PYRE_Q6_K = 14, PYRE_IQ2_XXS = 16, PYRE_IQ2_XS = 17,
       PYRE_IQ3_XXS = 18, PYRE_IQ4_NL = 20, PYRE_IQ3_S = 21, PYRE_IQ2_S = 22, PYRE_IQ4_XS = 23, PYRE_IQ1_M = 29, PYRE_BF16 = 30, PYRE_Q2_0 = 42 };

enum { PYRE_OK = 0, PYRE_E_ARG = -1, PYRE_E_TYPE = -2, PYRE_E_SHAPE = -3, PYRE_E_HIP = -4, PYRE_E_STATE = -5, PYRE_E_NOMEM = -6 };

/* ---- context ------------------------------------------------------------------------------------------------- */
/* Replaces the CubeCL client + stream the reference opens in Cube::new (src/model/qn_cube.rs:6243-6250). */
int         pyre_ctx_create(int device, pyre_ctx** out);
void        pyre_ctx_destroy(pyre_ctx* ctx);
/* Text of the last failure on this context (ctx may be NULL for create-time failures). */
const char* pyre_last_error(const pyre_ctx* ctx);
/* Blocks until the context's stream is idle (the reference's blocking `read`, qn_cube.rs ComputeClient::read). */
int         pyre_ctx_sync(pyre_ctx* ctx);
/* The context's hipStream_t, for callers that time or order their own work against it. */
void*       pyre_ctx_stream(pyre_ctx* ctx);
/* Plain device buffers for harnesses that do not bring their own allocator (Cube::buf / Cube::empty, qn_cube.rs). */
int         pyre_dev_alloc(pyre_ctx* ctx, size_t nbytes, void** out_dev);
int         pyre_dev_free(pyre_ctx* ctx, void* dev);
int         pyre_dev_upload(pyre_ctx* ctx, void* dst_dev, const void* src_host, size_t nbytes);
int         pyre_dev_download(pyre_ctx* ctx, void* dst_host, const void* src_dev, size_t nbytes);

/* Per-kernel-class timing (the reference's PYRE_QN_PROFILE counters, qwen4exp_gguf.rs:2107,2155, measure phases on
 * the host; here a HIP event pair brackets every launch on the context's stream).  pyre_prof_report returns lines
 * "<kernel class> <launches> <total ms> <algorithmic bytes>" valid until the next call. */
int         pyre_prof_enable(pyre_ctx* ctx, int on);
int         pyre_prof_reset(pyre_ctx* ctx);
const char* pyre_prof_report(pyre_ctx* ctx);

/* ---- quantized matrix operator --------------------------------------------------------------------------------
 * The drop-in for pyre's quantized-matmul operator: QMat { ty, rows, cols, bytes } + QMat::matmul
 * (src/model/gguf_q.rs:201-242), which is also what the burn-gguf call sites reduce to
 * (repack_to_burn + Tensor::matmul, src/model/qn_gpu.rs:54-76; dequantize_checked, src/model/kquant.rs:118).
 * `blocks` are GGUF blocks, row-major, row r at byte r*row_bytes (Gguf::mat, gguf_q.rs:326-331); cols must be a
 * multiple of 64 (and therefore of the block size, as gguf_q.rs:329 demands). */
int    pyre_qmat_create(pyre_ctx* ctx, uint32_t ggml_type, size_t rows, size_t cols, const void* host_blocks, size_t nbytes, pyre_qmat** out);
int    pyre_qmat_create_dev(pyre_ctx* ctx, uint32_t ggml_type, size_t rows, size_t cols, const void* dev_blocks, size_t nbytes, pyre_qmat** out);
void   pyre_qmat_destroy(pyre_qmat* m);
size_t pyre_qmat_rows(const pyre_qmat* m);
size_t pyre_qmat_cols(const pyre_qmat* m);
/* GGUF bytes of the matrix (rows * row_bytes): the algorithmic weight bytes of one GEMV. */
size_t pyre_qmat_gguf_bytes(const pyre_qmat* m);
/* Bytes the matrix occupies in device memory after the load-time re-layout (what one GEMV actually streams); the
 * reference's counterpart is the size of the repacked Burn tensor (repack_to_burn, src/model/qn_gpu.rs:54). */
size_t pyre_qmat_device_bytes(const pyre_qmat* m);
/* The same per layout: 0 = the lane-per-row planes (every type; what pyre_qmatmul_f32 streams), 1 = the matrix-core layout
 * (IQ3_S only, 0 otherwise; what pyre_qmatmul streams for IQ3_S windows of 2..8 tokens), 2 = IQ3_S at the file's bits per
 * weight (112 bytes per 256 weights; what pyre_qmatmul streams for one token).  No counterpart in the reference. */
size_t pyre_qmat_layout_bytes(const pyre_qmat* m, int layout);
/* QMat::to_f32 (gguf_q.rs:212): all rows*cols values, bit-exact with gguf_q::dequant (gguf_q.rs:67-166). */
int    pyre_qmat_dequant(pyre_ctx* ctx, const pyre_qmat* m, float* out_host);
int    pyre_qmat_dequant_dev(pyre_ctx* ctx, const pyre_qmat* m, float* out_dev);
/* QMat::row (gguf_q.rs:211): one row, bit-exact. */
int    pyre_qmat_row(pyre_ctx* ctx, const pyre_qmat* m, size_t row, float* out_host);
/* QMat::matmul (gguf_q.rs:216-217): y[ti*rows + r] = sum_c W[r,c] * x[ti*cols + c], t in 1..8.
 * The result for a token does not depend on t (same operations in the same order), which is what lets a
 * multi-token verify pass equal one-token decode (qwen4exp_gguf.rs:2357-2360) -- with one exception: a single token of
 * an IQ3_S matrix takes a kernel of its own (below), so t = 1 and t >= 2 agree to rounding (both within 1e-5 of the exact
 * product), not bit for bit; PYRE_QMATMUL_NATIVE=0 in the environment sends t = 1 through the window's kernel as well. */
int    pyre_qmatmul(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host);
int    pyre_qmatmul_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev);
/* One token of an IQ3_S matrix (t = 1; the reference's GPU decode of this type, src/model/qn_cube.rs:3354-3382): the
 * matrix is streamed at the file's bits per weight -- per four weights the 9-bit codebook index and four sign bits, the
 * codebook with the signs folded in (8192 x four signed bytes) in shared memory -- and the activations are block fixed
 * point, three signed bytes per value with one power of two per 64 columns (|x - su q| <= 2^-22 of the 64 columns'
 * largest magnitude), so that four weights meet their columns in v_dot4_i32_i8; the integer sums are exact, the scales
 * d * (1 + 2 s) and the accumulation are f32.
 * Windows of 2..8 tokens of an IQ3_S matrix go through the f16 matrix cores with one kernel (the reference's verify
 * kernels, src/model/qn_cube.rs:17,6454, and lcm_dense, qwen4exp_gguf.rs:2641-2737, are this product with t > 1): each
 * 256-column stretch of a token is scaled by its own power of two and every value is written as two f16 halves (22
 * significant bits; values more than 2^14 / 6e-5 below the largest magnitude of their stretch lose resolution), the 4-bit
 * codes times their sub-block scales are exact in f16, products are exact and summed in f32.  A non-finite activation
 * makes every output of its token NaN.  An IQ3_S matrix created through pyre_qmat_create* is held in three layouts (one per
 * kernel; an IQ2_XS or Q4_K matrix in three as well: rows, the single token's native format and, for a window of a matrix of more than 128 row tiles, a matrix-core layout of its own, 4.5 bit/weight; a Q8_0 matrix in two: rows and such a matrix-core layout, 8.5 bit/weight; pyre_qmat_device_bytes counts them all, pyre_qmat_layout_bytes each).  pyre_qmatmul_f32 is the same contract on the f32 multiply-add GEMV the
 * model's expert matrices use (QMat::matmul's own arithmetic, gguf_q.rs:169-197,233-241: f32 products, f32 accumulation);
 * for every other type the two are the same code. */
int    pyre_qmatmul_f32(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host);
int    pyre_qmatmul_f32_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev);
/* pyre_qmatmul_dev for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  IQ3_S matrices (whose kernels take the
 * activations from a scratch buffer, as f16 operand rows or as fixed-point digits) and IQ2_XS and Q4_K matrices (whose
 * single-token kernel takes the digits likewise, and whose windows' matrix-core kernels take operand rows -- Q4_K also the activations'
 * sub-block sums) and Q8_0 matrices (a window's matrix-core kernel likewise); every other type's pyre_qmatmul_dev allocates nothing already.  The operand goes to a fixed device array inside the library (PYRE_QMATMUL_STATIC_MAX_COLS * 32 bytes plus
 * the scale factors and the sums, 1 MiB + 36 KiB per GPU, held until the process ends) instead of the context's grow-only buffer, and the
 * call makes no allocation, no event and no copy: two kernel launches on the context's stream.  Same kernels and launch
 * shapes as pyre_qmatmul_dev, so the result is bit-identical to it.  Matrices with more than
 * PYRE_QMATMUL_STATIC_MAX_COLS columns are rejected with PYRE_E_SHAPE.
 * All contexts on one GPU share that GPU's array: calls that overlap in time on one GPU (two contexts' streams) race. */
#define PYRE_QMATMUL_STATIC_MAX_COLS 32768
int    pyre_qmatmul_static_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev);
/* ---- synthetic tensors (no counterpart in the reference's API; its micro-benchmarks build the same kind of data
 * inline, src/model/qdot.rs:823-859, src/model/qn_cube.rs:7216-7249) ---------------------------------------------
 * Fills n_blocks raw GGUF blocks on the device: counter-based random payload bytes, every f16 scale field drawn
 * uniformly from [d_lo, d_hi].  Bit-identical to pyre_amd/synth.py:blocks(). */
int    pyre_synth_blocks(pyre_ctx* ctx, uint32_t ggml_type, size_t n_blocks, uint64_t seed, float d_lo, float d_hi, void* dev_out);


/* ---- MoE FFN block ---------------------------------------------------------------------------------------------
 * ffn + routed, f32 branch (src/model/qwen4exp_gguf.rs:1675-1684, 1721-1732, 1754-1793) with the router of
 * top_k / soft_top / nan_clean (:3121-3139): softmax over the top-k logits, ties to the lower expert id, the chosen
 * experts listed and summed in ascending id (the order the reference's device router uses, qn_cube.rs:5225-5237).
 * Expert tensors are the fused GGUF matrices: gate/up [n_exp*ff x d], down [n_exp*d x ff], expert e = rows e*ff.. /
 * e*d.. (QMat::slice_rows, gguf_q.rs:215).  The qmats are borrowed and must outlive the block. */
typedef struct pyre_moe pyre_moe;
int  pyre_moe_create(pyre_ctx* ctx, int top_k, const pyre_qmat* router, const pyre_qmat* gate_exps, const pyre_qmat* up_exps, const pyre_qmat* down_exps,
                     const float* sh_gate_inp_host /*[d]*/, const pyre_qmat* sh_gate, const pyre_qmat* sh_up, const pyre_qmat* sh_down, pyre_moe** out);
void pyre_moe_destroy(pyre_moe* m);
/* x [t][d] -> y [t][d], t in 1..8; sel_idx / sel_w (optional) receive the routing [t][top_k]. */
int  pyre_moe_ffn(pyre_ctx* ctx, pyre_moe* m, const float* x_host, int t, float* y_host, int32_t* sel_idx_host, float* sel_w_host);
int  pyre_moe_ffn_dev(pyre_ctx* ctx, pyre_moe* m, const float* x_dev, int t, float* y_dev);

/* ---- Gated DeltaNet layer core ---------------------------------------------------------------------------------
 * linear_core (qwen4exp_gguf.rs:1624-1673): causal depthwise conv (kernel conv_k, weight [ch][conv_k], newest tap
 * last) + SiLU, L2-normalised q/k, per value head h (key head h % nk) the gated delta rule on the f32 state
 * S [nv][dk][dv], gated RMSNorm.  The block owns its recurrent state (conv [(conv_k-1)][ch] oldest first, S), which
 * stays resident in HBM across calls; a, dt [nv], conv_w [ch*conv_k], norm_w [dv] are host f32. dk = dv = 128. */
typedef struct pyre_gdn pyre_gdn;
int  pyre_gdn_create(pyre_ctx* ctx, int nk, int nv, int dk, int dv, int conv_k, float eps, const float* a, const float* dt, const float* conv_w, const float* norm_w, pyre_gdn** out);
void pyre_gdn_destroy(pyre_gdn* g);
int  pyre_gdn_set_state(pyre_ctx* ctx, pyre_gdn* g, const float* conv_host /*NULL = zeros*/, const float* ssm_host /*NULL = zeros*/);
int  pyre_gdn_get_state(pyre_ctx* ctx, pyre_gdn* g, float* conv_host, float* ssm_host);
/* proj [t][ch + nv*dv + 2*nv] = per token [qkv | z | beta | alpha] -> out [t][nv*dv]; tokens run in time order. */
int  pyre_gdn_step(pyre_ctx* ctx, pyre_gdn* g, const float* proj_host, int t, float* out_host);
/* The same recurrence for a prompt of T tokens in chunked form (chunk = 64) on the fp32 matrix cores; the reference has
 * only the sequential form (linear_core above), which is therefore the oracle.  A remainder T % 64 runs through the
 * step kernels. */
int  pyre_gdn_prefill_chunked(pyre_ctx* ctx, pyre_gdn* g, const float* proj_host, int T, int chunk, float* out_host);

/* ---- gated attention layer core over a 4-bit KV cache --------------------------------------------------------------
 * attn_core, dense branch (qwen4exp_gguf.rs:1558-1615): k RMSNorm + RoPE, append; per head q RMSNorm + RoPE,
 * softmax(q.K/sqrt(hd)) V, * sigmoid(gate); q and gate interleaved per head [h][2*hd]; kv head = h / (nh/nkv);
 * partial RoPE over the first n_rot dims, pairs (i, i + n_rot/2), inv[i] = base^(-2i/n_rot) (src/qn_ctx.rs:168).
 * Cache positions below ((n - kv_recent)/64)*64 (n = positions visible to the query, only when n > kv_recent + 64)
 * are read from the 4-bit cache of src/model/kv4.rs:12-42; the rest from f32 (split of kv_push, :1519-1520).
 * kv_bits = 0 keeps everything f32.  hd = 256. */
typedef struct pyre_attn pyre_attn;
int  pyre_attn_create(pyre_ctx* ctx, int nh, int nkv, int hd, int n_rot, float rope_base, float eps, const float* qn /*[hd]*/, const float* kn /*[hd]*/,
                      int kv_bits, int kv_recent, int max_ctx, pyre_attn** out);
void pyre_attn_destroy(pyre_attn* a);
int  pyre_attn_len(const pyre_attn* a);
int  pyre_attn_truncate(pyre_ctx* ctx, pyre_attn* a, int len);
/* qkv [t][nh*2*hd + 2*nkv*hd] raw projections [q,gate per head | k | v] for the next t positions -> out [t][nh*hd]. */
int  pyre_attn_decode_kv4(pyre_ctx* ctx, pyre_attn* a, const float* qkv_host, int t, float* out_host);
/* Harness access: install n positions of (already normalised + rotated) keys and values [n][nkv*hd]; read them back. */
int  pyre_attn_load_cache(pyre_ctx* ctx, pyre_attn* a, const float* k_host, const float* v_host, int n);
int  pyre_attn_read_cache(pyre_ctx* ctx, pyre_attn* a, float* k_host, float* v_host);
/* The QSA sparse indexer of attn_core (qwen4exp_gguf.rs:1565-1599), attached before the first position: rows given to
 * pyre_attn_decode_kv4 then carry [.. | index queries idx_nh*idx_hd | index key idx_hd] after q/k/v.  A query that sees
 * more than idx_budget + idx_ratio - 1 positions attends to the idx_budget / idx_ratio blocks of idx_ratio tokens with
 * the largest sum_h relu(q_h . pooled block key) / sqrt(idx_hd) and to the incomplete tail; blocks of equal score are
 * taken lowest index first (the reference's select_nth_unstable leaves that order open). */
int  pyre_attn_set_indexer(pyre_ctx* ctx, pyre_attn* a, int idx_nh, int idx_hd, int idx_ratio, int idx_budget, const float* iqn /*[idx_hd]*/, const float* ikn /*[idx_hd]*/);
/* qn_ctx::rope_inv (src/qn_ctx.rs:164-185) for a model context of ctx_tokens: YaRN frequencies and magnitude factor when
 * ctx_tokens > ctx_train > 0. */
int  pyre_attn_set_context(pyre_ctx* ctx, pyre_attn* a, int ctx_train, int ctx_tokens);
/* Harness access: install the raw index keys [len][idx_hd] of the cached positions (complete blocks are pooled on the
 * device); read the raw keys and the pooled block keys [len/idx_ratio][idx_hd]; read the positions the last decode call
 * selected for its token ti (*count = -1: every visible position). */
int  pyre_attn_load_index(pyre_ctx* ctx, pyre_attn* a, const float* ik_host);
int  pyre_attn_read_index(pyre_ctx* ctx, pyre_attn* a, float* ik_host, float* ib_host);
int  pyre_attn_read_selection(pyre_ctx* ctx, pyre_attn* a, int ti, int32_t* pos_host, int cap, int32_t* count);

/* ---- model: the layer API engine_qn drives ------------------------------------------------------------------------
 * Model::{load, new_state, forward, forward_multi, spec_keep} (qwen4exp_gguf.rs:462, 1345, 2050, 2365, 2495) as
 * consumed through QnTarget: spec::Target (src/engine_qn.rs:245-253). */
typedef struct {
  uint32_t ggml_type;   /* PYRE_* */
  uint32_t on_device;   /* 0: data is host memory, 1: data is device memory on the context's device */
  uint64_t rows, cols;  /* Gguf::mat view: rows = prod(shape[1..]), cols = shape[0]; vectors have rows = 1 */
  const void* data;     /* raw GGUF bytes; NULL for a slot the layer does not have */
} pyre_tensor;

/* per-layer tensor slots, named after the GGUF tensors Model::load reads (qwen4exp_gguf.rs:489-512) */
enum {
  PYRE_T_HC_ATTN_NORM = 0, PYRE_T_HC_ATTN_DOWN, PYRE_T_HC_ATTN_INJECT, PYRE_T_HC_ATTN_UP,     /* blk.N.hc_attn_{norm,down,inject,up}.weight */
  PYRE_T_HC_FFN_NORM, PYRE_T_HC_FFN_DOWN, PYRE_T_HC_FFN_INJECT, PYRE_T_HC_FFN_UP,             /* blk.N.hc_ffn_* */
  PYRE_T_ATTN_Q, PYRE_T_ATTN_K, PYRE_T_ATTN_V, PYRE_T_ATTN_OUTPUT, PYRE_T_ATTN_Q_NORM, PYRE_T_ATTN_K_NORM,
  PYRE_T_ATTN_QKV, PYRE_T_ATTN_GATE, PYRE_T_SSM_BETA, PYRE_T_SSM_ALPHA, PYRE_T_SSM_A, PYRE_T_SSM_DT_BIAS, PYRE_T_SSM_CONV1D, PYRE_T_SSM_NORM, PYRE_T_SSM_OUT,
  PYRE_T_FFN_GATE_INP, PYRE_T_FFN_GATE_EXPS, PYRE_T_FFN_UP_EXPS, PYRE_T_FFN_DOWN_EXPS, PYRE_T_FFN_GATE_INP_SHEXP, PYRE_T_FFN_GATE_SHEXP, PYRE_T_FFN_UP_SHEXP, PYRE_T_FFN_DOWN_SHEXP,
  PYRE_T_INDEXER_Q_PROJ, PYRE_T_INDEXER_K_PROJ, PYRE_T_INDEXER_Q_NORM, PYRE_T_INDEXER_K_NORM,   /* blk.N.indexer.* (qwen4exp_gguf.rs:501): all attention layers or none */
  PYRE_T_PLE_KEY, PYRE_T_PLE_VALUE, PYRE_T_PLE_NORM_KEY, PYRE_T_PLE_NORM_QUERY, PYRE_T_PLE_NORM_CONV, PYRE_T_PLE_CONV1D,   /* blk.N.ple_{key,value,norm_key,norm_query,norm_conv,conv1d}.weight (:505): the layers of ple.layers; a layer has all six or none */
  PYRE_LAYER_SLOTS
};
enum { PYRE_G_TOKEN_EMBD = 0, PYRE_G_OUTPUT_HC_NORM, PYRE_G_OUTPUT_HC_DOWN, PYRE_G_OUTPUT_HC_UP, PYRE_G_OUTPUT, PYRE_G_PLE_TOKEN_EMBD /* per_layer_token_embd.weight (:512) */, PYRE_GLOBAL_SLOTS };

/* Cfg (qwen4exp_gguf.rs:18-26), the fields the decode loop uses. */
typedef struct {
  int32_t n_layers, d, hc, hc_lr, n_head, n_kv, hd, n_rot;
  float rope_base, eps;
  int32_t n_exp, top_k, ff_exp;
  int32_t lin_nk, lin_nv, lin_dk, lin_dv, conv_k, full_every;
  int32_t vocab;
  int32_t kv_bits;    /* 4 (PYRE_QN_KV_BITS default) or 0 */
  int32_t kv_recent;  /* PYRE_QN_KV8_RECENT default 1024 */
  /* QSA sparse indexer (qwen4exp_gguf.rs:24-25, 481-485): heads (0 = none), key length, tokens per block, token budget.
   * Attention is dense up to idx_budget + idx_ratio - 1 visible positions and attends to idx_budget / idx_ratio
   * selected blocks plus the incomplete tail beyond (attn_core, :1565-1599). */
  int32_t idx_nh, idx_hd, idx_ratio, idx_budget;
  /* trained context length and the context the model is built for (Cfg::ctx_train, Cfg::max_ctx): ctx > ctx_train > 0
   * switches the YaRN frequency table and magnitude factor on (qn_ctx::rope_inv, src/qn_ctx.rs:164-185). */
  int32_t ctx_train, ctx;
  /* Per-layer n-gram embeddings, PLE (qwen4exp_gguf.rs:22-23, 477-480, ple_rows :1390-1407, ple :1409-1434): n-gram length
   * (0 or 1 = none; at most 8), table heads per n-gram length ((ple_ngram - 1) * ple_per_gram <= 16 heads), conv kernel
   * length (dilation = ple_ngram), width of a table row, the token id that cuts an n-gram's context; per n-gram position a
   * 64-bit multiplier, per head an offset into the table and a modulus.  A layer has PLE when its PYRE_T_PLE_* slots are set. */
  int32_t ple_ngram, ple_per_gram, ple_conv_k, ple_dim;
  uint32_t ple_eos; int32_t ple_reserved;
  uint64_t ple_mult[8], ple_off[16], ple_vocab[16];
} pyre_model_cfg;

/* ---- GGUF container (host only, no GPU needed): Gguf::open / mat / meta accessors, src/model/gguf_q.rs:250-336 --------
 * Opens the file, or all shards of a split one given any of them (`-NNNNN-of-MMMMM.gguf`), read-only memory maps;
 * metadata value types 0..12, `general.alignment` (default 32).  Errors come back as text in err[err_cap]. */
typedef struct pyre_gguf pyre_gguf;
int    pyre_gguf_open(const char* path, pyre_gguf** out, char* err, size_t err_cap);
void   pyre_gguf_close(pyre_gguf* g);
size_t pyre_gguf_n_shards(const pyre_gguf* g);
size_t pyre_gguf_n_tensors(const pyre_gguf* g);
const char* pyre_gguf_tensor_name(const pyre_gguf* g, size_t i);            /* file order */
int    pyre_gguf_has(const pyre_gguf* g, const char* name);
/* Gguf::mat (:326-331): the tensor as a matrix view into the map (cols = shape[0], rows = product of the rest);
 * n_dims / dims[8] (optional) receive the stored shape.  Types other than the PYRE_* ones are reported as PYRE_E_TYPE. */
int    pyre_gguf_tensor(const pyre_gguf* g, const char* name, pyre_tensor* out, uint32_t* n_dims, uint64_t* dims, char* err, size_t err_cap);
/* Meta::as_u64 / as_f64 / as_str and Gguf::arr_u64 (:253-258, :323): 0 when the key exists and converts. */
int    pyre_gguf_meta_u64(const pyre_gguf* g, const char* key, uint64_t* out);
int    pyre_gguf_meta_f64(const pyre_gguf* g, const char* key, double* out);
int    pyre_gguf_meta_str(const pyre_gguf* g, const char* key, char* out, size_t cap);
long   pyre_gguf_meta_arr_u64(const pyre_gguf* g, const char* key, uint64_t* out, size_t cap);   /* element count, -1 if not an array */

/* Model::load (qwen4exp_gguf.rs:462-524): `general.architecture` must be qwen4exp; configuration from the `qwen4exp.*`
 * keys, tensors by their GGUF names (blk.N.*, token_embd, output_hc_*, output or the tied embedding).  kv_bits and
 * kv_recent are run-time settings of the reference, not file contents, and so is the context the model is built for
 * (qn_ctx::startup_tokens, PYRE_QN_CTX).  The QSA indexer is taken when `attention.indexer.head_count` > 0 and the
 * indexer tensors exist; PLE layers (`ple.layers` and the ple.* keys, :468-480) when the file lists them. */
int   pyre_model_load_gguf(pyre_ctx* ctx, const char* path, int kv_bits, int kv_recent, int ctx_tokens /* 0: the trained context */, pyre_model** out);
/* Copies (and re-lays-out) every tensor into device memory; the caller's buffers are free afterwards. */
int   pyre_model_create(pyre_ctx* ctx, const pyre_model_cfg* cfg, const pyre_tensor* layer_tensors /*[n_layers][PYRE_LAYER_SLOTS]*/,
                        const pyre_tensor* globals /*[PYRE_GLOBAL_SLOTS]*/, pyre_model** out);
void  pyre_model_destroy(pyre_model* m);
/* GGUF bytes of the weights one decode step reads (dense matrices, router, top_k + 1 experts, head, one embedding row). */
size_t pyre_model_weight_bytes_per_token(const pyre_model* m);
/* Blocks of up to 1024 prompt tokens this model's pyre_forward calls have taken layer by layer with the FFN grouped by expert on the
 * matrix cores since it was created (the prompt path at t >= 16: QMat::matmul's switch to a GEMM, src/model/gguf_q.rs:219-232, and
 * the chunk loop of src/engine_qn.rs:117-138).  A call takes that path for the whole blocks in front of its last tokens when every
 * layer's experts are IQ3_S with equal widths that are multiples of 256; PYRE_PROMPT_BLOCK=0 at model creation keeps the experts in one
 * layout only and every prompt in windows of eight, PYRE_PROMPT_WINDOWS=1 does the latter for the calls made while it is set. */
size_t pyre_model_prompt_blocks(const pyre_model* m);
/* new_state: empty token list, zero recurrent state, KV room for max_ctx positions. */
int   pyre_state_create(pyre_ctx* ctx, const pyre_model* m, int max_ctx, pyre_state** out);
void  pyre_state_destroy(pyre_state* s);
int   pyre_state_reset(pyre_ctx* ctx, pyre_state* s);
int   pyre_state_len(const pyre_state* s);
int   pyre_state_capacity(const pyre_state* s);                 /* positions the caches have room for (Model::max_ctx of this state) */
int   pyre_model_max_window(const pyre_model* m);               /* spec_max_window (qwen4exp_gguf.rs:2486-2493): 8; multi_ok is always true */
/* Model::snapshot / restore (qwen4exp_gguf.rs:3277-3298; the prefix cache of engine_qn.rs:92-138 keeps these): the
 * recurrent state and the first `len` cache positions, kept in device memory; restorable into any state of the same
 * model with enough capacity. */
typedef struct pyre_snap pyre_snap;
int   pyre_state_snapshot(pyre_ctx* ctx, pyre_state* s, pyre_snap** out);
int   pyre_state_restore(pyre_ctx* ctx, pyre_state* s, const pyre_snap* snap);
void  pyre_snap_destroy(pyre_snap* snap);
size_t pyre_snap_bytes(const pyre_snap* snap);
int   pyre_snap_len(const pyre_snap* snap);
/* Test access to the recurrent state: li-th DeltaNet layer's S [nv][dk][dv] and conv [(k-1)][ch]; ai-th attention layer's f32 K / V rows [len][nkv*hd];
 * pi-th PLE layer's history [(ple_conv_k-1)*ple_ngram][hc*d], oldest first (State::ple_hist, :196; rows before position 0 are zero). */
int   pyre_state_read_ple(pyre_ctx* ctx, pyre_state* s, int pi, float* hist_host);
int   pyre_state_read_gdn(pyre_ctx* ctx, pyre_state* s, int li, float* conv_host, float* ssm_host);
int   pyre_state_read_kv(pyre_ctx* ctx, pyre_state* s, int ai, float* k_host, float* v_host);
/* forward: append n tokens (any n >= 1; processed in windows of up to 8), logits of the last one -> logits_host[vocab]. */
int   pyre_forward(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* ids, int n, float* logits_host);
/* forward_multi: n in 1..8 tokens, logits after each -> logits_host [n][vocab]; arms spec_keep for this window. */
int   pyre_forward_multi(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* ids, int n, float* logits_host);
/* spec_keep(t, keep): keep the first `keep` of the last t tokens fed by forward_multi (recurrent state rolled back, caches truncated). */
int   pyre_spec_keep(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, int t, int keep);
/* spec::generate, greedy branch (src/spec.rs:156-267, accept loop :229-238; argmax = first maximum, src/sampler.rs:142-148).
 * first_logits_host: logits after the prompt.  n_draft = 0: plain decode, the whole loop runs on the device without
 * host round trips.  n_draft in 1..7 with draft_stream [n_out + 8]: the round that starts with `produced` tokens
 * emitted verifies draft_stream[produced .. produced + n_draft) and keeps the accepted prefix.
 * out [n_out] tokens; *rounds (optional) = verify rounds used. */
int   pyre_generate_greedy(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const float* first_logits_host, int n_out, uint32_t* out,
                           int n_draft, const uint32_t* draft_stream, int* rounds);
/* sampler::argmax (src/sampler.rs:142-148) of t rows of `vocab` logits on the device: a scan from index 0 with strict >, so
 * the first of equal maxima; a NaN is never greater, and a NaN at index 0 is never replaced.  The drafted loops below use
 * the same kernel on the window's logits; this entry point takes host rows (test and tooling use). */
int   pyre_argmax_rows(pyre_ctx* ctx, const float* logits_host, int t, int vocab, uint32_t* picks_host);
/* Prompt-lookup drafter, spec::ngram_draft (src/spec.rs:122-139): the most recent earlier occurrence of the longest suffix
 * (n = max_n .. min_n tokens) of history[0..len) and up to k tokens that followed it -> out [k]; returns how many (0: no
 * match).  Host only: no context, no GPU. */
int   pyre_ngram_draft(const uint32_t* history, size_t len, int k, int min_n, int max_n, uint32_t* out);
/* spec::generate, greedy branch, with that drafter supplying the drafts (src/spec.rs:207: drafts = ngram_draft(history, kk,
 * ng_min, ng_max), the reference's defaults are 3 and 8): history [n_hist] are the tokens the state has consumed (the
 * prompt); a round without a match is a plain single-token step.  k = drafts per round at most, 1..7.  The output equals
 * plain greedy decoding token for token.  *rounds / *drafted / *accepted (optional): verify rounds, drafts verified, drafts
 * accepted (spec::Outcome, src/spec.rs:150-154). */
int   pyre_generate_greedy_ngram(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, const uint32_t* history, size_t n_hist, const float* first_logits_host,
                                 int n_out, uint32_t* out, int k, int ng_min, int ng_max, int* rounds, int* drafted, int* accepted);
/* Adaptive draft length, spec::adapt_plan (src/spec.rs:144-152): the draft count k in 0..min(n, 8) with the best expected
 * tokens per second relative to plain decoding, from the plain step time ts, the measured verify time tv[t] of a t-token
 * window (tv[10]; an entry of 0 = unmeasured: ts * (1 + 0.75 (t - 1))), the running acceptance p and the drafter's time per
 * round td.  0 = no window is expected to beat plain steps.  Host only: no context, no GPU. */
int   pyre_adapt_plan(int n, double ts, const double* tv, double p, double td);
/* Whether pyre_generate_greedy_ngram and pyre_generate_greedy_mtp apply that plan as spec::generate does (src/spec.rs:162-167,
 * 186-193, 213-217): timings and acceptance tracked online, the decision taken before drafting (so a drafter that does not
 * pay is not run either, apart from a probe window now and then) and again on what the drafter produced.  on = 1 / 0, or
 * -1: PYRE_SPEC_ADAPT in the environment.  The reference's default is on (spec::adapt_on, src/spec.rs:34); here an unset
 * variable means off, so that the drafted / accepted counts of a run do not depend on the clock -- a binding passes
 * spec::adapt_on().  The generated tokens are the same either way. */
void  pyre_spec_set_adapt(pyre_ctx* ctx, int on);
/* ---- the multi-token-prediction (MTP) drafter: src/model/mtp.rs, Model::mtp_draft (src/model/qwen4exp_gguf.rs:2180-2277) ----
 * One extra block that pairs the main model's final residual streams R_i with the token at position i + 1 (cell i, rope
 * position i, the unscaled table) and predicts token i + 2: pre-norms and two d x d matrices form its streams, then
 * hyper-connection mix -> gated attention over its own last `window` cells -> mix -> MoE FFN -> mixer -> the draft
 * vocabulary rows of the output matrix.  Its own residual feeds the next draft step.  Only draft quality depends on it:
 * every emitted token comes from the verify window.  Tensors come in any supported type (the reference builds int8
 * copies of a BF16 checkpoint, mtp.rs:11-13); norm vectors already carry their "1 + w" (mtp.rs:44-45); the fused
 * mlp.experts.gate_up_proj is given as its gate and up halves. */
enum {
  PYRE_MTP_PRE_E = 0, PYRE_MTP_PRE_H,                       /* pre_fc_norm_embedding [d], pre_fc_norm_hidden [hc*d] */
  PYRE_MTP_FC_E, PYRE_MTP_FC_H,                             /* fc_embedding, fc_hidden [d x d] */
  PYRE_MTP_HCA_NORM, PYRE_MTP_HCA_DOWN, PYRE_MTP_HCA_INJECT, PYRE_MTP_HCA_UP,      /* attn_hyper_connection.* */
  PYRE_MTP_HCF_NORM, PYRE_MTP_HCF_DOWN, PYRE_MTP_HCF_INJECT, PYRE_MTP_HCF_UP,      /* mlp_hyper_connection.* */
  PYRE_MTP_MIX_NORM, PYRE_MTP_MIX_DOWN, PYRE_MTP_MIX_UP,                           /* hyper_connection_mixer.* (no inject) */
  PYRE_MTP_Q, PYRE_MTP_K, PYRE_MTP_V, PYRE_MTP_O, PYRE_MTP_QN, PYRE_MTP_KN,        /* self_attn.* */
  PYRE_MTP_ROUTER, PYRE_MTP_GATE_E, PYRE_MTP_UP_E, PYRE_MTP_DOWN_E,                /* mlp.gate, mlp.experts.* */
  PYRE_MTP_SH_GATE_INP, PYRE_MTP_SH_GATE, PYRE_MTP_SH_UP, PYRE_MTP_SH_DOWN,        /* mlp.shared_expert_gate, mlp.shared_expert.* */
  PYRE_MTP_HEAD,                                            /* rows draft_ids[0..n_draft_vocab) of the main model's output matrix */
  PYRE_MTP_SLOTS
};
/* geometry beyond the main model's (Geo, mtp.rs:95): routed experts, experts per token, expert width, attention window
 * in cells (PYRE_MTP_WINDOW, 128 in the reference), rows of the draft head */
typedef struct { int32_t n_exp, top_k, ff, window, n_draft_vocab; } pyre_mtp_cfg;
typedef struct pyre_mtp pyre_mtp;
int   pyre_mtp_create(pyre_ctx* ctx, const pyre_model* main, const pyre_mtp_cfg* cfg, const pyre_tensor* tensors /*[PYRE_MTP_SLOTS]*/,
                      const uint32_t* draft_ids /*[n_draft_vocab], host*/, pyre_mtp** out);
void  pyre_mtp_destroy(pyre_mtp* m);
/* The drafter's checkpoint file: the safetensors reader of src/model/mtp.rs:24-50 (St::open / raw).  An 8-byte header
 * length, a JSON header, BF16 tensors only (anything else: PYRE_E_TYPE); names have their "mtp." and "layers.0." prefixes
 * trimmed.  Host only.  pyre_st_tensor: *data points into the mapping (valid until pyre_st_close), dims[8] / *n_dims
 * (optional) receive the shape. */
typedef struct pyre_st pyre_st;
int    pyre_st_open(const char* path, pyre_st** out, char* err, size_t err_cap);
void   pyre_st_close(pyre_st* s);
size_t pyre_st_n_tensors(const pyre_st* s);
const char* pyre_st_tensor_name(const pyre_st* s, size_t i);            /* file (header) order */
int    pyre_st_tensor(const pyre_st* s, const char* name, const void** data, uint32_t* n_dims, uint64_t* dims, char* err, size_t err_cap);
/* Mtp::load (src/model/mtp.rs:99-118): the drafter from that file.  Tensor names as the reference reads them; norm vectors
 * become 1 + w; mlp.experts.gate_up_proj [experts][2 ff][d] is split into gate (rows 0 .. ff of an expert) and up; experts
 * and width come from mlp.experts.down_proj [experts][d][ff]; matrices stay BF16 (the reference re-quantizes them to int8).
 * top_k: experts per token, capped by the main model's (PYRE_MTP_TOPK; 0 = the main model's); window: 0 = 128
 * (PYRE_MTP_WINDOW); head: the draft head [n_draft_vocab][d] in any supported type, or NULL = rows draft_ids of the main
 * model's output matrix dequantized to f32. */
int   pyre_mtp_load_safetensors(pyre_ctx* ctx, const pyre_model* main, const char* path, int top_k, int window,
                                const uint32_t* draft_ids, int n_draft_vocab, const pyre_tensor* head, pyre_mtp** out);
/* From now on every forward call leaves the final residual streams of its last `window` tokens in a ring on the device
 * (mtp_keep_r, qwen4exp_gguf.rs:2279-2285: window + 16 positions are kept) and the state owns the drafter's K/V cells.
 * Snapshots do not carry either: after pyre_state_restore the drafter starts over (no drafts until a forward call has
 * left the residual of the last position again). */
int   pyre_state_attach_mtp(pyre_ctx* ctx, pyre_state* s, const pyre_mtp* m);
/* mtp_draft, host-loop form with the draft policy off: catches the drafter's cells up over the positions whose token is
 * committed, then runs up to k (1..7) draft steps from (R_{len-1}, pending) on the device and reads ids and
 * probabilities back once.  A later draft is kept only while the drafter's probability of its choice is >= min_p
 * (spec::draft_gate, src/spec.rs:326-327).  *n_out = drafts in ids_host / probs_host [k] (0 when the residual of the
 * last position is not there). */
int   pyre_mtp_draft(pyre_ctx* ctx, const pyre_mtp* m, pyre_state* s, uint32_t pending, int k, float min_p, uint32_t* ids_host, float* probs_host, int* n_out);
/* test access: cells [*c0, *c0 + *n) of the drafter's cache, k_host / v_host [*n][n_kv*hd] (either may be NULL; pass room for `window` cells) */
int   pyre_mtp_read_kv(pyre_ctx* ctx, pyre_state* s, int* c0, int* n, float* k_host, float* v_host);
/* spec::generate's greedy branch with this drafter proposing (src/spec.rs:156-267): each round verifies [pending, drafts]
 * in one window and keeps the agreeing prefix.  The output equals plain greedy decoding token for token. */
int   pyre_generate_greedy_mtp(pyre_ctx* ctx, const pyre_model* m, const pyre_mtp* mtp, pyre_state* s, const float* first_logits_host, int n_out, uint32_t* out,
                               int k, float min_p, int* rounds, int* drafted, int* accepted);
/* The same loop for measurements of the accepted path: the drafter runs every round (its cost is paid), then its ids are
 * replaced by forced_stream[produced ..] (at least n_out + 8 ids).  With the plain greedy output there (entry i = the
 * i-th token of that output, entry 0 the first pick) every draft is accepted, whatever the drafter's weights would draft.
 * No counterpart in the reference; the reference reports acceptance of trained drafters (docs/HANDOFF.md:28). */
int   pyre_generate_greedy_mtp_forced(pyre_ctx* ctx, const pyre_model* m, const pyre_mtp* mtp, pyre_state* s, const float* first_logits_host, int n_out, uint32_t* out,
                                      int k, const uint32_t* forced_stream, int* rounds, int* drafted, int* accepted);
/* The decode loop as the benchmark times it: n_steps greedy steps starting from token `first`, everything on the device;
 * tokens (optional, host) receives the n_steps generated ids after the call. */
int   pyre_decode_greedy_dev(pyre_ctx* ctx, const pyre_model* m, pyre_state* s, uint32_t first, int n_steps, uint32_t* tokens_host);

/* ---- request loop over one resident state: engine_qn::run (src/engine_qn.rs:92-170) --------------------------------
 * Prefill on the absolute chunk grid (PYRE_PREFILL_CHUNK, default 256) with a prefix cache of state snapshots
 * (PYRE_QN_PCACHE, PYRE_QN_PCACHE_MB): a prompt that strictly extends the previous request's tokens continues that
 * state, otherwise it starts from the longest snapshot it strictly extends, otherwise from an empty state; snapshots are
 * taken at grid boundaries and where the prompt leaves the previous prompt's common prefix, oldest dropped first beyond
 * cache_bytes_cap (0 = no prefix cache).  Snapshots live in device memory.  The arithmetic of a token does not depend
 * on how the prompt is split, so a resumed prompt ends in exactly the state and logits of a full prefill. */
typedef struct pyre_session pyre_session;
int   pyre_session_create(pyre_ctx* ctx, const pyre_model* m, int max_ctx, int prefill_chunk, size_t cache_bytes_cap, pyre_session** out);
void  pyre_session_destroy(pyre_session* s);
pyre_state* pyre_session_state(pyre_session* s);
/* logits_host [vocab] after the last prompt token; *cached = prompt tokens not recomputed, *from_snapshot = 1 when they
 * came from a snapshot rather than from the previous request's state.  A prompt of max_ctx tokens or more is refused
 * with the reference's message. */
int   pyre_session_prefill(pyre_ctx* ctx, pyre_session* s, const uint32_t* prompt, int n, float* logits_host, int* cached, int* from_snapshot);
/* pyre_generate_greedy on the session's state; the tokens the state consumed are recorded for the next request. */
int   pyre_session_generate_greedy(pyre_ctx* ctx, pyre_session* s, const float* first_logits_host, int n_out, uint32_t* out, int n_draft, const uint32_t* draft_stream, int* rounds);
int   pyre_session_stats(const pyre_session* s, int* n_snapshots, size_t* snapshot_bytes, int* state_len);
int   pyre_session_snapshot_len(const pyre_session* s, int i);      /* tokens of the i-th snapshot, oldest first; -1 past the end */

#ifdef __cplusplus
}
#endif
#endif
