// Internal definitions shared by the translation units of libpyre_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <map>
#include <string>
#include <vector>
#include "../../include/pyre_hip.h"

// Diagnostics build (-DPYRE_PHASE_TS): workgroup 0's first thread keeps 100 MHz timestamps of a kernel's phases in
// registers and leaves them in a per-file device array at the kernel's end (read back by pyre_debug_ts_*).
#ifdef PYRE_PHASE_TS
#define PYRE_TS_DECL(name) static __device__ unsigned long long name[128];
#define PYRE_TS_VARS unsigned long long ts_[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#define PYRE_TS(k) ts_[k] = wall_clock64()
#define PYRE_TS_FLUSH(name, base) do { if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0) { for (int q_ = 0; q_ < 8; ++q_) name[(base) + q_] = ts_[q_]; } } while (0)
#define PYRE_TS_EXPORT(name, fn) extern "C" int fn(unsigned long long* out) { return hipMemcpyFromSymbol(out, HIP_SYMBOL(name), sizeof(unsigned long long) * 128) == hipSuccess ? 0 : -1; }
#else
#define PYRE_TS_DECL(name)
#define PYRE_TS_VARS
#define PYRE_TS(k)
#define PYRE_TS_FLUSH(name, base)
#define PYRE_TS_EXPORT(name, fn)
#endif
#define PYRE_WAVE 64
#define PYRE_UNIT 64            // weights per decode unit (one lane decodes one unit at a time)

struct pyre_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  std::string err;
  // staging for host-pointer entry points
  void* stage = nullptr; size_t stage_bytes = 0;
  // expanded codebooks in device memory: iq3s u32[512], iq2xs u64[512]
  uint32_t* d_iq3s = nullptr; uint64_t* d_iq2xs = nullptr; uint16_t* d_cb = nullptr;
  // optional per-kernel-class timing: an event pair around every launch, resolved at pyre_prof_report
  struct ProfPending { const char* name; double bytes; hipEvent_t a, b; };
  struct ProfAcc { long count = 0; double ms = 0, bytes = 0; };
  bool prof_on = false; std::vector<ProfPending> prof_pending; std::map<std::string, ProfAcc> prof_acc; std::vector<hipEvent_t> prof_pool;
  std::string prof_text;
  void* aop_buf = nullptr; size_t aop_bytes = 0;       // split activations of the operator's matrix-core GEMM (grow-only)
  int batch_n = 1; size_t batch_stride = 0, batch_stride2 = 0;            // the matrix-core hyper-connection launches (hc.hip) for batch_n windows at once: window z's own buffers batch_stride bytes further on per window (a long prompt's blocks; 1 / 0 otherwise)
  void* aop_static = nullptr;                          // device address of this GPU's copy of the file-scope operand array (gemm_m.hip), resolved at creation
  uint32_t* d_iq2xs_sgn = nullptr;                     // IQ2_XS likewise: two tables of 8192 x four signed bytes (weights 0..3 / 4..7 of an entry)
  uint32_t* d_iq3s_sgn = nullptr;                      // IQ3_S codebook with the signs folded in: 8192 x four signed bytes (gemv_n.hip), made at first use
  void* dgn_buf = nullptr; size_t dgn_bytes = 0;       // activation digits of the native-format IQ3_S GEMV (grow-only)
  int spec_adapt = -1;                                 // adaptive draft length of the drafted greedy loops: 1 on, 0 off, -1 PYRE_SPEC_ADAPT in the environment (unset: off)
};

// Wraps one kernel launch when profiling is on (bytes = algorithmic bytes the launch moves).
struct ProfScope {
  pyre_ctx* ctx; hipEvent_t a = nullptr, b = nullptr; const char* name; double bytes;
  ProfScope(pyre_ctx* c, const char* n, double by) : ctx(c), name(n), bytes(by) {
    if (!ctx->prof_on) return;
    auto get = [&]() { hipEvent_t e = nullptr; if (!ctx->prof_pool.empty()) { e = ctx->prof_pool.back(); ctx->prof_pool.pop_back(); } else (void)hipEventCreate(&e); return e; };
    a = get(); b = get(); (void)hipEventRecord(a, ctx->stream);
  }
  ~ProfScope() { if (!a) return; (void)hipEventRecord(b, ctx->stream); ctx->prof_pending.push_back({name, bytes, a, b}); }
};

#ifdef __HIPCC__
// Workgroup barrier for exchanges that go through shared memory only: waits for the wave's own shared-memory (and
// scalar) operations, not for its outstanding global loads, so weights requested ahead of it stay in flight across it.
// (__syncthreads() carries a workgroup-scope fence, which on this part drains every outstanding vector memory
// operation first: a prefetch issued before it costs its whole latency at the barrier.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
#endif

#ifdef __HIPCC__
// Wave-wide sum / maximum on the data-parallel-primitive path: four steps inside each row of sixteen lanes (quad swaps, half
// mirror, mirror: every lane then holds its row's value), two row broadcasts, one lane read -- seven short instructions
// where six __shfl_xor steps are six trips through the shared-memory crossbar.  Every lane gets the result.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float wave_dpp(float old, float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += wave_dpp<0xB1, 0xf>(0.0f, v); v += wave_dpp<0x4E, 0xf>(0.0f, v); v += wave_dpp<0x141, 0xf>(0.0f, v); v += wave_dpp<0x140, 0xf>(0.0f, v);
  v += wave_dpp<0x142, 0xa>(0.0f, v); v += wave_dpp<0x143, 0xc>(0.0f, v);          // lane 15 of rows 0, 2 into rows 1, 3; lane 31 into rows 2, 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, wave_dpp<0xB1, 0xf>(v, v)); v = fmaxf(v, wave_dpp<0x4E, 0xf>(v, v)); v = fmaxf(v, wave_dpp<0x141, 0xf>(v, v)); v = fmaxf(v, wave_dpp<0x140, 0xf>(v, v));
  v = fmaxf(v, wave_dpp<0x142, 0xa>(v, v)); v = fmaxf(v, wave_dpp<0x143, 0xc>(v, v));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
#endif

extern thread_local std::string g_pyre_create_err;

int pyre_fail(pyre_ctx* ctx, int code, const char* fmt, ...);
#define PYRE_HIP(ctx, call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return pyre_fail((ctx), PYRE_E_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); } while (0)
#define PYRE_CHECK_LAUNCH(ctx) PYRE_HIP(ctx, hipGetLastError())

int pyre_stage(pyre_ctx* ctx, size_t nbytes, void** out);          // grow-only device staging buffer

// ---- device-side matrix view --------------------------------------------------------------------------------------
// Weights live in "lane = row" planes: rows are grouped in tiles of 64, and for every (tile, unit) the 64 rows'
// entries of a plane are contiguous, so one wave (lane l = row l of the tile) reads every plane with fully
// coalesced loads while all lanes sit on the same 64 columns (activations then come from scalar loads).
//   vector plane  p0: [tile][unit][chunk < V][lane] x 16 B
//   small planes  p1..p3: [tile][unit][lane] x e bytes
//   block plane   pb: [tile][unit/4][lane] x e bytes    (per 256-value super-block)
// FMT_IQ3_S_M (IQ3_S for the matrix cores): rows in groups of 16, columns in steps of 32 (one sub-block).  In
// v_mfma_f32_16x16x32_f16 lane l supplies, for the operand that carries the weights, row l % 16 of the group and the eight
// consecutive columns 8 * (l / 16) .. + 7 of the step, so a lane's share of a step is eight 4-bit codes = one dword:
//   mq: [row tile of 64][128-column chunk][row group of the tile][lane] x 16 B (a tile's chunk is 4 KB contiguous, a tile's
//       whole K range one contiguous run): dword s = step s of the chunk; the code of column element e of the lane's
//       eight sits at nibble e/2 + 4*(e&1), so that or-ing nibbles p and p + 4 into one register yields elements 2p, 2p + 1
//   mh: [row tile][super-block][row group][row] x 8 B: f16 d, 16 zero bits, the eight 4-bit sub-block scales (sub-block i
//       at nibble i/2 + 4*(i&1), the same order)
struct QMatDev {
  const uint8_t* p0; const uint8_t* p1; const uint8_t* p2; const uint8_t* p3; const uint8_t* pb;
  int rows, cols, U, tiles, fmt;
  uint32_t ty; int gel, gbytes;        // GGUF type the matrix was created from and its block geometry (algorithmic byte counts)
  uint32_t lut[4]; int bias;           // C4 value table (entry = value + bias)
  const uint8_t* mq; const uint8_t* mh; int SB;      // FMT_IQ3_S_M planes; SB = super-blocks (256 columns) per row
};
inline double qmat_gguf_bytes(const QMatDev& m, double rows) { return rows * (m.cols / m.gel) * m.gbytes; }

#ifdef __HIPCC__
// Kernel arguments are scalar loads from the argument block, which the compiler otherwise issues where each value is
// first needed: behind branches that is one memory round trip after another before the first vector load can go out.
// Naming the values here makes every such load leave at the kernel's first instruction, under one wait.
template <typename A> __device__ __forceinline__ void arg_now(A a) { asm volatile("" ::"s"(a)); }
template <typename... A> __device__ __forceinline__ void args_now(A... a) { (arg_now(a), ...); }
__device__ __forceinline__ void qmat_args_now(const QMatDev& m) { args_now(m.p0, m.p1, m.p2, m.p3, m.pb, m.rows, m.cols, m.U, m.tiles); }
#endif

// index of row group rg's 64 lane slots (16 B each) for chunk c in mq, and of its 16 header slots (8 B each) for super-block sb in mh
inline __host__ __device__ size_t mq_slot(size_t rg, int c, int K128) { return (((rg >> 2) * K128 + c) * 4 + (rg & 3)) * 64; }
inline __host__ __device__ size_t mh_slot(size_t rg, int sb, int SB) { return (((rg >> 2) * SB + sb) * 4 + (rg & 3)) * 16; }
// dv: the lane = row planes (every type).  dvm: the matrix-core layout, IQ3_S only (fmt == FMT_IQ3_S_M when present).
// Which of the two an IQ3_S matrix holds is decided at creation: the stand-alone operator keeps both (its entry points
// cover both kernels), the model keeps one per matrix.
enum { PYRE_LAYOUT_ROWS = 0, PYRE_LAYOUT_M = 1, PYRE_LAYOUT_BOTH = 2, PYRE_LAYOUT_ALL = 3 };      // ALL (the stand-alone operator): rows, the matrix-core layout (IQ3_S, Q4_K) and the single token's native-format layout
struct pyre_qmat {
  pyre_ctx* ctx; uint32_t ty; size_t rows, cols; size_t gguf_bytes;
  void* base; size_t dev_bytes; QMatDev dv;
  void* base_m = nullptr; size_t dev_bytes_m = 0; QMatDev dvm{};
  void* base_n = nullptr; size_t dev_bytes_n = 0;      // the same matrix at the file's bits per weight (gemv_n.hip), stand-alone operator matrices only
};
int pyre_qmat_create_layout(pyre_ctx* ctx, uint32_t ty, size_t rows, size_t cols, const void* blocks, bool on_device, size_t nbytes, int layout, pyre_qmat** out);
// IQ3_S at the file's bits per weight with the codebook in shared memory, one token (gemv_n.hip)
size_t pyre_gemv_n_bytes(size_t rows, size_t cols, int fmt = 6);          // fmt: FMT_IQ3_S (6), FMT_IQ2_XS (5) or FMT_Q4_K (4)
int pyre_gemv_n_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* nq_dev, int fmt = 6);
int pyre_gemv_n_table(pyre_ctx* ctx);                             // the codebook table, made at context creation
size_t pyre_gemv_n_digit_bytes(size_t cols);
int pyre_gemv_n_launch(pyre_ctx* ctx, const void* nq, size_t rows, size_t cols, const float* x_dev, float* y_dev, void* digits = nullptr, int fmt = 6);

// Optional work folded into the end of a GEMV launch (qmat.hip):
//   best: t = 1, per row tile (bits of the maximum, first row holding it) -> best[2*tile], best[2*tile+1]
//   co:   rows < ch are the channels of a causal depthwise conv1d (kernel kk, weights conv_w[ch][kk]); the lane that
//         owns a row runs the window's tokens in order, o = w[kk-1]*cur + sum_j w[j]*state[j], co[t][row] = silu(o),
//         and slides the row's state conv_in -> conv_out ([kk-1][ch], oldest first; in == out is fine).
struct GemvEpi { uint32_t* best; const float* conv_w; const float* conv_in; float* conv_out; float* co; int ch, kk; int four_waves; int sq_heads = 0; float sq_eps = 0.0f; };          // sq_*: PyreAop::sq travels to the kernel here
// launchers implemented in qmat.hip, used by the block / model code
// Matrices in the matrix-core layout (FMT_IQ3_S_M) take their activations as the f16 operand `a` when the caller has one (a
// producer kernel wrote it); otherwise x_dev is split into the context's operand buffer by one more launch.
struct PyreAop;
int pyre_gemv_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, const PyreAop* a = nullptr);
// waves per workgroup and units per wave the (unsplit) GEMV uses for this matrix
void pyre_gemv_plan(const QMatDev& m, int* nw, int* upw);
// K range split over `ksplit` workgroups per row tile; partial[(ks*t_count + t)*tiles*64 + row] holds the slice sums and
// the consumer adds them in slice order.
int pyre_gemv_split_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* partial_dev, int ksplit, const PyreAop* a = nullptr);
// Few row tiles, long rows (an output projection): the sixteen waves of pyre_gemv_launch's plan, same units each, as
// four workgroups of four waves per row tile (the work of a tile on four compute units instead of one).  Each
// workgroup leaves the sum of its waves, parts[(q*t_count + t)*tiles*64 + row], q < PYRE_GEMV_PARTS; the consumer adds the
// parts in order from the first.
#define PYRE_GEMV_PARTS 4
bool pyre_gemv_parts_ok(const QMatDev& m);
int pyre_gemv_parts_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* parts_dev, const PyreAop* a = nullptr);
// t = 1 GEMV that also leaves, per row tile, (bits of the maximum, first row holding it) in best[2*tile], best[2*tile+1].
// (value bits, first row) pairs the argmax form leaves in best_dev for this matrix: one per row tile
int pyre_gemv_best_count(const QMatDev& m);
int pyre_gemv_argmax_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, float* y_dev, uint32_t* best_dev, const PyreAop* a = nullptr);
// y as pyre_gemv_launch (raw projections), plus the conv epilogue described at GemvEpi (best ignored).
int pyre_gemv_conv_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, const GemvEpi& conv, const PyreAop* a = nullptr);
int pyre_row_launch(pyre_ctx* ctx, const QMatDev& m, const uint32_t* row_idx_dev, int n, float* out_dev, int out_stride);
// Greedy pick from per-tile maxima (first maximum overall) -> id_out[0] (and mirror[0] if given); when m is given the
// chosen row is dequantized into out_dev in the same launch (the next token's embedding).
// step_dev (optional, device int[2]): step_dev[0] is incremented first (the position of the token being started) and the
// id goes to mirror[step_dev[0] - step_dev[1]] instead of mirror[0].
// hist (optional, with step_dev): the token history by position; the pick is also stored at the position it starts
int pyre_pick_launch(pyre_ctx* ctx, const uint32_t* best_dev, int n_tiles, uint32_t* id_out, uint32_t* mirror, const QMatDev* m, float* out_dev, int* step_dev, uint32_t* hist = nullptr);

// ---- IQ3_S GEMM on the matrix cores (gemm_m.hip), 1 <= t <= 8, matrices in FMT_IQ3_S_M ------------------------------------
// The activations reach the kernel as its f16 operand: every value as two halves, x = h1 + h2 * 2^-11 with h1 = f16(x) and
// h2 = f16((x - h1) * 2^11) (22 significant bits), token ti's halves as operand rows 2 ti and 2 ti + 1 of R = 2, 4, 8 or 16
// rows (the power of two that holds the window, pyre_aop_rows), laid out [8-column group][row] x 16 B.  ainv (optional):
// [super-block][8] factors the super-block's sums are multiplied by per token (the inverse of the power of two the splitter
// scaled that stretch of the token by); null = 1.  Rows 2t .. R - 1 may hold anything finite or not: a row of the operand
// only ever reaches its own token's sums, so a token's result is bit-identical for every window width.
struct PyreAop { const uint4* op; const float* ainv; const float* sq = nullptr; int sq_heads = 0; float sq_eps = 0.0f; };
// sq (with op; ainv unused): the operand of a Gated DeltaNet output projection as its four workgroups per head leave it
// (GdnQ): one 128-column chunk = one head, one 32-column sub-block = one workgroup's columns, each scaled by its own power
// of two; sq[(t*heads + h)*4 + q] = that factor's inverse, sq[8*heads*4 + (t*heads + h)*4 + q] = the quarter's sum of
// squares of the un-normalised output.  The product brings a chunk's sub-blocks to a common power of two and applies
// 1 / sqrt(mean square + eps), the head's RMS norm, with the chunk's scale.
int pyre_aop_rows(int t);
size_t pyre_aop_bytes(int cols, int t);                            // operand bytes for a K range of `cols` and a window of t
// splits x [t][cols] (any magnitudes: each 256-column stretch of a token is scaled by its own power of two) into op / ainv
int pyre_act_split_launch(pyre_ctx* ctx, const float* x_dev, int t, int cols, uint4* op, float* ainv);
// y as pyre_gemv_launch / pyre_gemv_split_launch (ksplit > 1: slice sums) with the epilogues of GemvEpi
int pyre_gemm_m_best_count(const QMatDev& m);
// Q4_K on the matrix cores (gemm_q4.hip): the operator's windows
size_t pyre_gemm_q4_bytes(size_t rows, size_t cols, size_t* codes);
int pyre_gemm_q4_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* base);
size_t pyre_gemm_q4_scratch_bytes(int cols);
int pyre_gemm_q4_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, void* scratch = nullptr);
// IQ2_XS on the matrix cores (gemm_q2.hip): likewise
size_t pyre_gemm_q2_bytes(size_t rows, size_t cols, size_t* codes);
int pyre_gemm_q2_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* base);
int pyre_gemm_q2_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, void* scratch = nullptr);
// Q8_0 on the matrix cores (gemm_q8.hip): likewise
size_t pyre_gemm_q8_bytes(size_t rows, size_t cols, size_t* codes);
int pyre_gemm_q8_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* base);
int pyre_gemm_q8_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, void* scratch = nullptr);
int pyre_gemm_m_launch(pyre_ctx* ctx, const QMatDev& m, const PyreAop& a, int t, float* y_dev, int ksplit, const GemvEpi& ep, const float* xf = nullptr);
// xf: the single token's f32 activations instead of `a` (the kernel forms the operand rows itself); where that pays
bool pyre_gemm_m_x_ok(const QMatDev& m, int t, const GemvEpi& ep);
// K parts / waves per workgroup the kernel uses for this matrix (ksplit parts)
void pyre_gemm_m_plan(const QMatDev& m, int ksplit, int* nw, int* hb_per_wave);
// the operator's own scratch for the split operand (grow-only, per context), and the fixed per-GPU array of the entry point
// that allocates nothing (resolved at context creation)
int pyre_gemm_m_scratch(pyre_ctx* ctx, int cols, uint4** op, float** ainv);
int pyre_static_init(pyre_ctx* ctx);
int pyre_gemm_m_static(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev);
#ifdef __HIPCC__
// One activation into the operand a producer kernel leaves for the GEMM that follows it: element k of token ti of a window
// with R operand rows.  v is the value already multiplied by the power of two its producer scales the token by (AopOut:
// the factor brings a bound of the token's largest magnitude into [2^13, 2^14), the GEMM multiplies the sums by its inverse).
__device__ __forceinline__ void aop_store(uint16_t* __restrict__ op, int R, int k, int ti, float v) {
  const _Float16 h1 = (_Float16)v, h2 = (_Float16)((v - (float)h1) * 2048.0f);
  const size_t base = ((size_t)(k >> 3) * R + 2 * ti) * 8 + (k & 7);
  op[base] = __builtin_bit_cast(unsigned short, h1); op[base + 8] = __builtin_bit_cast(unsigned short, h2);
}
#endif

// ---- MoE FFN block (moe.hip) ----------------------------------------------------------------------------------------
struct MoeDev {
  QMatDev router, gate_e, up_e, down_e, sh_gate, sh_up, sh_down;
  const float* sh_gate_inp;
  int d, n_exp, top_k, ff, sf;
  QMatDev gate_m{}, up_m{}, down_m{}, sh_gate_m{}, sh_up_m{}, sh_down_m{};      // the expert matrices once more in the matrix-core layout (FMT_IQ3_S_M), when the model keeps it: a long prompt's blocks (pyre_moe_block_launch)
};
struct MoeWork {            // scratch for up to 8 tokens, owned by whoever launches the block
  float* logits;            // [8][n_exp]
  int32_t* sel_idx;         // [8][top_k] ascending expert id
  float* sel_w;             // [8][top_k]
  float* sg;                // [8] sigmoid(sh_gate_inp . x)
  float* h;                 // [8*(top_k+1)][max(ff, sf)]
  float* partial;           // [8*(top_k+1)][d]
  float* parts;             // [PYRE_MOE_GROUPS][t][d]: a window's output as group sums (pyre_moe_launch with in_groups)
  uint32_t* dgx;            // [8][d/64][64]: the activations' digits for the integer-dot gate/up products (IQ3_S experts)
  uint32_t* dgh;            // [8*(top_k+1)][max(ff, sf)/64][64]: the digits of h for the integer-dot down products, left by the gate/up launch of a window
};
// The FFN output of a window, left unreduced for the consumer to fold.  The k expert terms (ascending id) and the shared
// expert's form PYRE_MOE_GROUPS groups of g = (k + 4) / 4 consecutive experts, the shared expert in the last:
//   P_q = sum over the group's experts, in order, from zero, of sel_w * partial      (+ partial[shared] * sg for the last)
//   y[ti][r] = ((P_0 + P_1) + P_2) + P_3
// -- the association a window's down projection uses when it leaves the four group sums instead (k_moe_down_groups), so
// that a token's value does not depend on which of the two forms produced it.
struct MoeOut { const float* partial; const float* sel_w; const float* sg; int d, k; };
#define PYRE_MOE_KMAX 16      // moe_out_value keeps up to this many expert terms in registers
#define PYRE_MOE_GROUPS 4     // == PYRE_GEMV_PARTS: the mix reads the group sums as it reads an output projection's K parts
#define PYRE_MOE_GMAX 5       // entries of a group: (PYRE_MOE_KMAX + 4) / 4, the last group holds at most that many with the shared expert
static_assert(PYRE_MOE_GROUPS == PYRE_GEMV_PARTS, "the mix adds the group sums as it adds an output projection's K parts");
#ifdef __HIPCC__
// All loads are issued before the first add, so the value costs one memory round trip, not k + 1.
// FK > 0: the number of routed experts as a compile-time constant (the caller guarantees mo.k == FK): the loads and the
// grouping carry no predicates; the arithmetic is the same.
template <int FK = 0> __device__ __forceinline__ float moe_out_value(const MoeOut& mo, int ti, int r) {
  const int k = FK ? FK : mo.k;
  const float* p = mo.partial + (size_t)ti * (k + 1) * mo.d + r; const float* w = mo.sel_w + ti * k;
  constexpr int KM = FK ? FK : PYRE_MOE_KMAX;
  float pv[KM], wv[KM];
#pragma unroll
  for (int j = 0; j < KM; ++j) { pv[j] = j < k ? p[(size_t)j * mo.d] : 0.0f; wv[j] = j < k ? w[j] : 0.0f; }
  float sh = p[(size_t)k * mo.d], g = mo.sg[ti];
  const int gsz = (k + 4) / 4;
  float P[PYRE_MOE_GROUPS];
#pragma unroll
  for (int q = 0; q < PYRE_MOE_GROUPS; ++q) {
    float o = 0.0f;
#pragma unroll
    for (int e = 0; e < PYRE_MOE_GMAX; ++e) { const int j = q * gsz + e; if (e < gsz && j < k) o = fmaf(wv[j < KM ? j : 0], pv[j < KM ? j : 0], o); }
    P[q] = o;
  }
  P[PYRE_MOE_GROUPS - 1] = fmaf(sh, g, P[PYRE_MOE_GROUPS - 1]);
  return ((P[0] + P[1]) + P[2]) + P[3];
}
#endif
inline MoeOut pyre_moe_out(const MoeDev& m, const MoeWork& w, int first_token) {
  return MoeOut{w.partial + (size_t)first_token * (m.top_k + 1) * m.d, w.sel_w + (size_t)first_token * m.top_k, w.sg + first_token, m.d, m.top_k};
}
size_t pyre_moe_work_bytes(const MoeDev& m);
void   pyre_moe_work_carve(const MoeDev& m, void* base, MoeWork* w);
// y[t][d] = ffn(x[t][d]).  With y == nullptr (top_k <= PYRE_MOE_KMAX) the output stays unreduced in the work buffers
// (pyre_moe_out) for a consumer that evaluates moe_out_value itself.
// Router logits that arrive as K-slice sums (left by the mix that produced x, see HcRoute): logit[t][e] = the slices
// p[(s*T + t)*r64 + e], s = 0..nsl-1, added in slice order.
struct RouteSrc { const float* p; int nsl; int r64; const uint32_t* dgx = nullptr; };          // dgx: the activations' digits (digits.h), left by the same mix, or null
// in_groups (t > 1, y == nullptr, pyre_moe_groups_ok): the down projection leaves the PYRE_MOE_GROUPS group sums of every
// token in w.parts, group q of token ti at parts + (q*t + ti)*d, instead of the unreduced terms.
int pyre_moe_launch(pyre_ctx* ctx, const MoeDev& m, const MoeWork& w, const float* x_dev, int t, float* y_dev, const RouteSrc* routed = nullptr, bool in_groups = false);
inline bool pyre_moe_groups_ok(const MoeDev& m) { return m.top_k <= PYRE_MOE_KMAX; }
// The FFN of a block of prompt windows (T = 8 * windows tokens) with the tokens grouped by expert, on the matrix cores (moe.hip):
// what the windows' mixes leave in their workspaces -- window w's x [8][d] at x + w * ws, its router K-slice sums at rpart + w * ws
// (slice s of token ti at (s * 8 + ti) * r64) -- and where window w's group sums go: parts + w * ws, laid out as
// MoeWork::parts of a window of eight.  The rest is the block's own scratch (pyre_moe_block_carve): the routing, the (token, choice) pairs by
// expert, x and h as f16 operand rows a token (xh [T + 1][2][d], hh [T * (k + 1) + 1][2][ff], the last row of each zero) with
// their scale factors, the gate and up products and the unreduced down terms.
struct MoeBlk {
  const float* x; const float* rpart; float* parts; size_t ws;      // window w's x, router sums and group sums at these + w * ws floats (the windows' workspaces: one stride)
  int32_t* sel_idx; float* sel_w; float* sg; int32_t* eoff; int32_t* elist; float* g; float* u; float* partial;
  uint16_t* xh; float* xinv; uint16_t* hh; float* hinv;
};
bool   pyre_moe_block_ok(const MoeDev& m);
size_t pyre_moe_block_bytes(const MoeDev& m, int T);
void   pyre_moe_block_carve(const MoeDev& m, int T, void* base, MoeBlk* b);
int    pyre_moe_block_zero_rows(pyre_ctx* ctx, const MoeDev& m, const MoeBlk& b, int T);
int    pyre_moe_block_launch(pyre_ctx* ctx, const MoeDev& m, const MoeBlk& b, int T, int T_max, int nsl, int r64, bool router_here = false);      // router_here: the router's sums are formed by this call (k_moe_router_blk), not left by the mixes
// K parts the gate/up dot products are summed in (1 or 2; k_moe_gu)
int pyre_moe_gu_parts(const MoeDev& m);

// ---- per-layer n-gram embeddings, PLE (ple.hip; ple_rows / ple, qwen4exp_gguf.rs:1390-1434) ----------------------------------
struct PleCfg { int ngram, per_gram, conv_k, dim; uint32_t eos; unsigned long long mult[8], off[16], vocab[16]; };
// kv = [key ; value] rows (hc*d + d) x (heads * dim); ring: the normalised rows of the last positions, row of position p at
// ring[(p & mask) * hc*d] (a ring indexed by position: a rollback needs no copy, the rows are rewritten when their positions
// come again); mask + 1 >= (conv_k - 1) * ngram + 8.
struct PleDev { QMatDev kv; const float* nk; const float* nq; const float* nc; const float* conv; float* ring; int mask; };
struct PleWork { uint32_t* idx; float* emb; float* kv; float* gated; };     // [8*16] table rows, [8][heads*dim], [8][hc*d + d], [8][hc*d]
size_t pyre_ple_work_bytes(const PleCfg& c, int d, int hc);
void   pyre_ple_work_carve(const PleCfg& c, int d, int hc, void* base, PleWork* w);
// table rows of the window's positions (start or *posp .. + t - 1 of the token history) -> w.emb; once per window
int pyre_ple_rows_launch(pyre_ctx* ctx, const PleCfg& c, const QMatDev& tab, const PleWork& w, const uint32_t* tokens_dev, int start, const int* posp, int t);
// One PLE layer: the streams are read from x_in as in pyre_hc_mix_launch (pending residual update applied first), and
// x_out [t][hc][d] = updated streams + gated + silu(conv); the layer's ring advances by t positions.
int pyre_ple_launch(pyre_ctx* ctx, const PleCfg& c, const PleDev& p, const PleWork& w, int d, int hc, float eps, const float* x_in, int in_ss, int in_ts, float* x_out,
                    const float* comb_out, const MoeOut* comb_moe, const float* comb_inj, int start, const int* posp, int t);

// ---- hyper-connections (hc.hip) ---------------------------------------------------------------------------------------
struct HcDev { QMatDev di; QMatDev up; const float* norm; int d, hc, lr; bool has_inject;      // di = [down ; inject] rows
               QMatDev di_m{}, up_m{}; };      // the same two matrices in the matrix-core layout (fmt == FMT_IQ3_S_M) when they are IQ3_S of whole super-blocks
struct HcWork { float* ssq; float* o; float* smx; };    // [<=32][8] slice sums of squares of the streams, [<=32][8][tiles*64] slice sums of [down ; inject], [<=32][8] largest |x * norm weight| of each slice
size_t pyre_hc_work_bytes(const HcDev& h);
void   pyre_hc_work_carve(const HcDev& h, void* base, HcWork* w);
// Streams are read from x_in (element i of stream s of token ti at x_in[ti*in_ts + s*in_ss + i]; in_ss = 0 replicates one
// row over the streams), the pending residual update is applied first when comb_out (a [t][d] vector) or comb_moe (the
// unreduced FFN output) is given (x[ti][s][:] += out[ti][:] * 2*sigmoid(comb_inj[ti][s])), and the updated streams go to x_out [t][hc][d], which
// must not overlap x_in.  mixed [t][d] and inj [t][hc] = hc_mix(updated streams).
// The router GEMV of the FFN block that follows a mix, riding on the mix's second launch: workgroup b of that launch
// owns columns [64b, 64b+64) of the mixed vector, so it leaves the K-slice sum part[(b*T + t)*tiles*64 + row] of every
// router row; the gate/up launch adds the d/64 slices (RouteSrc).  bf16 and f32 routers, at most 64 slices.
struct HcRoute { QMatDev router; float* part; uint32_t* dgx = nullptr; };          // dgx: where the mix leaves the digits of its output for the expert products (digits.h), or null
// Where a producer kernel leaves its result as the f16 operand of the matrix-core GEMM that follows (so that GEMM needs no
// split launch of its own): op = PyreAop::op (pyre_aop_rows(t) rows), ainv = PyreAop::ainv, [nsb super-blocks][8 tokens].
// Every token is scaled by one power of two that brings a bound of its largest magnitude into [2^13, 2^14) -- a bound every
// workgroup of the producer can form without talking to the others -- and ainv holds the inverse for every super-block:
//   hyper-connection mix: |mixed_i| <= max over the streams of (RMS scale * largest |x * norm weight| of the stream), from
//     the slice maxima the mix's first launch leaves (matrix-core mixes only: pyre_hc_aop_ok)
//   Gated DeltaNet: |o_i * scale| <= sqrt(dv) after the RMS normalisation, times the largest norm weight: a constant of the
//     layer (pyre_gdn_launch takes the factor, the model keeps the matching ainv)
struct AopOut { uint16_t* op; float* ainv; int nsb; };
bool pyre_hc_aop_ok(const HcDev& h);
int pyre_hc_mix_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, const float* x_in, int in_ss, int in_ts, float* x_out, int t, const float* comb_out, const MoeOut* comb_moe, const float* comb_inj,
                       float eps, float* mixed_dev, float* inj_dev, const HcRoute* route = nullptr, int comb_parts = 1, const AopOut* aop = nullptr);
bool pyre_hc_route_ok(const HcDev& h, const QMatDev& router);
// waves per workgroup, units per wave and K slices of the norm + [down ; inject] kernel; false if the shape is unsupported
bool pyre_hc_plan(const HcDev& h, int* nw, int* upw, int* ksplit);
int pyre_hc_combine_launch(pyre_ctx* ctx, int d, int hc, float* x_dev, int t, const float* out_dev, const float* inj_dev);

// ---- Gated DeltaNet (gdn.hip) -----------------------------------------------------------------------------------------
struct GdnDev { const float* a; const float* dt; const float* conv_w; const float* norm_w; int nk, nv, dk, dv, conv_k; float eps; };
// proj [t][ch + nv*dv + 2*nv] = [qkv | z | beta | alpha] per token (row stride = proj_stride floats).
// conv_in/conv_out [(k-1)][ch], ssm_in/ssm_out [nv][dk][dv] (in != out).  co_scratch [8][ch].  out [t][nv*dv].
// conv_done: co_scratch already holds silu(conv) of the window and the conv state has been advanced (GemvEpi).
// gq: the launch runs on nv x 4 workgroups (a workgroup owns 32 columns of a head's state) and leaves, instead of out_dev,
// the un-normalised gated output as f16 operand rows with the per-quarter factors and sums of squares of PyreAop::sq.
// The state it leaves differs in rounding from the nv-workgroup form's (the column sums meet in another order): a layer
// uses one form for every call.
struct GdnQ { uint16_t* op; float* sq; };
// the convolution of n consecutive windows of t tokens in one launch (gdn.hip: k_gdn_conv_blk)
int pyre_gdn_conv_block_launch(pyre_ctx* ctx, const GdnDev& g, const float* proj, int stride, int t, int n, size_t ws, const float* prev, int prev_stride, float* conv_out, float* co);
int pyre_gdn_launch(pyre_ctx* ctx, const GdnDev& g, const float* proj, int proj_stride, int t, const float* conv_in, float* conv_out,
                    const float* ssm_in, float* ssm_out, float* co_scratch, float* out_dev, bool conv_done = false, uint16_t* aop = nullptr, float aop_up = 1.0f, const GdnQ* gq = nullptr, int nwin = 1, size_t ws = 0);      // nwin > 1: that many consecutive windows, their projections, convolution outputs and operands ws floats apart, in one launch (the per-quarter form, conv_done)

// Chunked (64-token) form of the same recurrence on the fp32 matrix cores; T must be a positive multiple of 64.
// scratch: co [T][ch], logg [T][nv], beta [T][nv], oraw [T][nv*dv].
int pyre_gdn_prefill_launch(pyre_ctx* ctx, const GdnDev& g, const float* proj, int proj_stride, int T, const float* conv_in, float* conv_out,
                            const float* ssm_in, float* ssm_out, float* co, float* logg, float* beta, float* oraw, float* out_dev);

// ---- gated attention over the KV cache (attn.hip) -----------------------------------------------------------------------
struct AttnDev { const float* qn; const float* kn; const float* rope_inv; int nh, nkv, hd, n_rot, kv_bits, kv_recent; float eps; float mscale = 1.0f; };   // mscale: YaRN magnitude factor on cos and sin
struct KvDev {
  // key planes are blocked by 64 positions: row r of R rows at position p sits at kv_blk(r, R, p), so the rows a wave
  // reads for its 64 positions are one contiguous range (lane = position reads stay coalesced)
  float* kf;        // [cap/64][nkv*hd][64]      f32 keys
  float* vf;        // [cap][nkv*hd]       f32 values, row-major
  uint32_t* kq;     // [cap/64][nkv*hd/8][64]    4-bit keys: word w of position p holds dims 8w..8w+7
  float* ks;        // [cap/64][nkv*hd/32][64]   key scales
  uint32_t* vq;     // [cap][nkv*hd/8]     4-bit values
  float* vs;        // [cap][nkv*hd/32]    value scales
  int cap;
};
__host__ __device__ inline size_t kv_blk(size_t r, size_t R, size_t p) { return ((p >> 6) * R + r) * 64 + (p & 63); }
#define PYRE_ATTN_NPW 2                       // 64-position groups per attention workgroup
#define PYRE_ATTN_CDIMS 16                    // head dims a workgroup of the chunk merge owns
#define PYRE_ATTN_CHUNK (64 * PYRE_ATTN_NPW)   // positions per chunk (one workgroup per chunk and KV head)
struct AttnWork { float* q; uint16_t* qh; float* qsc; float* part_o; float* part_ml; int max_chunks; };   // q [8][nh][hd], its f16 halves [8][nh][2][hd] and their scale [8][nh]; partials per (token, head, chunk)
size_t pyre_kv_bytes(const AttnDev& a, int cap);
void   pyre_kv_carve(const AttnDev& a, int cap, void* base, KvDev* kv);
size_t pyre_attn_work_bytes(const AttnDev& a, int cap);
void   pyre_attn_work_carve(const AttnDev& a, int cap, void* base, AttnWork* w);
// qkv [t][nh*2*hd + 2*nkv*hd] = [q (with interleaved gate) | k | v] raw projections; positions start..start+t-1 are
// appended; packed_done = number of leading positions already packed (updated by the call). out [t][nh*hd].
// posp != nullptr: the kernels take the window's first position from *posp (device memory) instead of `start`, so the
// launch sequence can be replayed from a captured graph; packed_done is then left to the caller.
int pyre_attn_launch(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, const float* qkv, int qkv_stride, int start, int t,
                     int* packed_done, float* out_dev, const int* posp);
size_t pyre_packed_boundary(size_t n_visible, int kv_bits, int recent);
// qn_ctx::rope_inv (src/qn_ctx.rs:164-185): inverse frequencies [n_rot/2]; YaRN when ctx > ctx_train > 0; returns mscale
float pyre_rope_table(int n_rot, float base, int ctx_train, int ctx, float* inv_host);

// ---- QSA sparse indexer (qsa.hip), qwen4exp_gguf.rs:1565-1599 ------------------------------------------------------------
// Blocks of `ratio` tokens; a query that sees more than budget + ratio - 1 positions attends to the budget / ratio
// blocks with the largest  sum_h relu(q_h . block key) / sqrt(hd)  and to the incomplete tail.
struct QsaDev { const float* iqn; const float* ikn; int nh, hd, ratio, budget; };      // nh == 0: the layer has no indexer
struct QsaBuf {            // per attention layer, capacity fixed with the KV cache
  float* ik;               // [cap][hd]                 raw index keys as projected
  float* ib;               // [cap/ratio/64][hd][64]    pooled block keys, blocked by 64 blocks (lane = block reads are coalesced)
};
struct QsaWork {           // per state, shared by the layers
  float* iq;               // [8][nh][hd]   normalised, rotated index queries of the window
  float* score;            // [8][cap/ratio]
  int* plist;              // [8][list_stride]  attended positions, ascending
  int* pcount;             // [8]  entries of plist in use; -1 = every visible position (dense)
  int list_stride, max_blocks;
};
__host__ __device__ inline size_t qsa_ib_at(size_t b, size_t i, size_t hd) { return ((b >> 6) * hd + i) * 64 + (b & 63); }
size_t pyre_qsa_buf_bytes(const QsaDev& q, int cap);
void   pyre_qsa_buf_carve(const QsaDev& q, int cap, void* base, QsaBuf* b);
size_t pyre_qsa_work_bytes(const QsaDev& q, int cap);
void   pyre_qsa_work_carve(const QsaDev& q, int cap, void* base, QsaWork* w);
// idx [t][..] rows hold, at column iq_off, the raw index queries [nh*hd] followed by the raw index key [hd].  Appends
// the keys, pools the blocks the window completes, and leaves the attended positions of every token in w.plist / w.pcount.
int pyre_qsa_launch(pyre_ctx* ctx, const QsaDev& q, const AttnDev& a, const QsaBuf& b, const QsaWork& w, const float* proj, int stride, int iq_off, int start, int t, const int* posp);
int pyre_qsa_pool_all(pyre_ctx* ctx, const QsaDev& q, const AttnDev& a, const QsaBuf& b, int n);
// the attention launch with an optional position list (qw == nullptr: dense)
int pyre_attn_launch_sel(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, const float* qkv, int qkv_stride, int start, int t,
                         int* packed_done, float* out_dev, const int* posp, const QsaWork* qw, int part = 0);      // part: 1 = the cache write alone, 2 = the pass over the cache and the merge alone (w.q / qh / qsc kept in between), 0 = both
int pyre_attn_append_launch(pyre_ctx* ctx, const AttnDev& a, const KvDev& kv, const AttnWork& w, const float* qkv, int stride, int start, int t);      // K / V only
