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
enum { PYRE_F32 = 0, PYRE_F16 = 1, PYRE_Q8_0 = 8, PYRE_Q4_K = 12, PYRE_IQ2_XS = 17, PYRE_IQ3_S = 21, PYRE_BF16 = 30 };

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
/* QMat::to_f32 (gguf_q.rs:212): all rows*cols values, bit-exact with gguf_q::dequant (gguf_q.rs:67-166). */
int    pyre_qmat_dequant(pyre_ctx* ctx, const pyre_qmat* m, float* out_host);
int    pyre_qmat_dequant_dev(pyre_ctx* ctx, const pyre_qmat* m, float* out_dev);
/* QMat::row (gguf_q.rs:211): one row, bit-exact. */
int    pyre_qmat_row(pyre_ctx* ctx, const pyre_qmat* m, size_t row, float* out_host);
/* QMat::matmul (gguf_q.rs:216-217): y[ti*rows + r] = sum_c W[r,c] * x[ti*cols + c], t in 1..8.
 * The result for a token does not depend on t (same operations in the same order), which is what lets a
 * multi-token verify pass equal one-token decode (qwen4exp_gguf.rs:2357-2360). */
int    pyre_qmatmul(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host);
int    pyre_qmatmul_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev);

/* ---- synthetic tensors (no counterpart in the reference's API; its micro-benchmarks build the same kind of data
 * inline, src/model/qdot.rs:823-859, src/model/qn_cube.rs:7216-7249) ---------------------------------------------
 * Fills n_blocks raw GGUF blocks on the device: counter-based random payload bytes, every f16 scale field drawn
 * uniformly from [d_lo, d_hi].  Bit-identical to pyre_amd/synth.py:blocks(). */
int    pyre_synth_blocks(pyre_ctx* ctx, uint32_t ggml_type, size_t n_blocks, uint64_t seed, float d_lo, float d_hi, void* dev_out);

#ifdef __cplusplus
}
#endif
#endif
