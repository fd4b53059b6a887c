// Q8_0 dequant-GEMM on the f16 matrix cores, 2..8 tokens (QMat::matmul, src/model/gguf_q.rs:217-242, for the block type of
// :79): the window path of the stand-alone operator.  The lane = row GEMV converts and multiplies a weight once per token (the
// 151936 x 2048 head: 61 us at two tokens, 105 us at eight); here, as for IQ3_S (gemm_m.hip), once whatever the window:
//   * w = d * q per 32-value block, q a signed byte;
//   * the layout keeps q + 128; one byte permute puts two of them into the mantissas of two f16 numbers 1024 + (q + 128) (the
//     permute's other source supplies the exponent bytes), one packed addition of -1152 leaves q, exactly;
//   * v_mfma_f32_16x16x32_f16 multiplies 16 weight rows x 32 columns -- one block -- with the sixteen activation rows (two f16
//     halves of up to eight tokens, gemm_m.hip); the block's d meets its f32 sums right after.
// Layout (FMT_Q8_0_M): per group of 16 rows and 128-column chunk two planes of 64 x 16 bytes (lane (g, j): row j's columns
// 32 s + 8 g .. + 7 of blocks s = 0, 1 in the first plane, 2, 3 in the second) in QMatDev::mq, and 16 x 8 bytes of the four
// blocks' f16 d a row in QMatDev::mh.  8.5 bit/weight, what the file has.
// A token's operand rows reach only its own sums: its result is bit-identical for every window width 2..8.
#include "gemm_m.h"

__host__ __device__ inline size_t q8_slot(size_t rg, int c, int K128) { return ((rg >> 2) * K128 + c) * 4 + (rg & 3); }      // the row tile's four groups side by side

// ---- the matrix: raw GGUF rows -> mq / mh; one thread per (row of the padded row groups, chunk) ------------------------------
__global__ __launch_bounds__(256) void k_repack_q8m(int rows, int rows_pad, int K128, const uint8_t* __restrict__ raw, size_t row_bytes, uint32_t* __restrict__ mq, uint2* __restrict__ mh) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * K128) return;
  const int row = (int)(idx / K128), c = (int)(idx % K128); const bool live = row < rows;      // padding rows lie past the end of the raw buffer: never read them
  const size_t slot = q8_slot((size_t)(row >> 4), c, K128); const int j = row & 15;
  const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)c * 4 * 34;
  uint32_t hd[2] = {0u, 0u};
  for (int s = 0; s < 4; ++s) {
    const uint8_t* blk = b + s * 34;
    if (live) hd[s >> 1] |= ((uint32_t)blk[0] | ((uint32_t)blk[1] << 8)) << (16 * (s & 1));
    for (int g = 0; g < 4; ++g) {
      uint32_t lo = 0x80808080u, hi = 0x80808080u;            // (a padding row: q = 0)
      if (live) { lo = 0; hi = 0; for (int e = 0; e < 4; ++e) { lo |= (uint32_t)(uint8_t)(blk[2 + 8 * g + e] + 128) << (8 * e); hi |= (uint32_t)(uint8_t)(blk[2 + 8 * g + 4 + e] + 128) << (8 * e); } }
      uint32_t* dst = mq + ((slot * 2 + (s >> 1)) * 64 + g * 16 + j) * 4 + 2 * (s & 1);
      dst[0] = lo; dst[1] = hi;
    }
  }
  mh[slot * 16 + j] = make_uint2(hd[0], hd[1]);
}

// ---- the product -----------------------------------------------------------------------------------------------------------------
struct WBuf8 { uint4 w[4][2]; uint2 h[4]; };
__device__ __forceinline__ void load_w8(const QMatDev& m, int rg0, int c, int lane, int K128, WBuf8& b) {
#pragma unroll
  for (int g = 0; g < 4; ++g) { const size_t sl = q8_slot((size_t)rg0 + g, c, K128); b.w[g][0] = ((const uint4*)m.mq)[(sl * 2) * 64 + lane]; b.w[g][1] = ((const uint4*)m.mq)[(sl * 2 + 1) * 64 + lane]; }
#pragma unroll
  for (int g = 0; g < 4; ++g) b.h[g] = ((const uint2*)m.mh)[q8_slot((size_t)rg0 + g, c, K128) * 16 + (lane & 15)];
}
// The exponent bytes of 1024 .. 2047 and the bias, in registers the compiler cannot see through (the permutes stay permutes).
struct Q8K { uint32_t ex, bias; };
__device__ __forceinline__ Q8K q8_consts() { Q8K k; asm volatile("v_mov_b32 %0, 0x64646464" : "=v"(k.ex)); asm volatile("v_mov_b32 %0, 0xE480E480" : "=v"(k.bias)); return k; }      // 0xE480: -1152 as f16
__device__ __forceinline__ void chunk_mac8(const WBuf8& wb, const ABuf& ab, const Q8K& qk, v4f (&tot)[4]) {
  const v2h bias = __builtin_bit_cast(v2h, qk.bias);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const uint32_t wd[4][2] = {{wb.w[g][0].x, wb.w[g][0].y}, {wb.w[g][0].z, wb.w[g][0].w}, {wb.w[g][1].x, wb.w[g][1].y}, {wb.w[g][1].z, wb.w[g][1].w}};
    const uint32_t a4[4][4] = {{ab.a[0].x, ab.a[0].y, ab.a[0].z, ab.a[0].w}, {ab.a[1].x, ab.a[1].y, ab.a[1].z, ab.a[1].w}, {ab.a[2].x, ab.a[2].y, ab.a[2].z, ab.a[2].w}, {ab.a[3].x, ab.a[3].y, ab.a[3].z, ab.a[3].w}};
    const uint32_t hd[2] = {wb.h[g].x, wb.h[g].y};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      uint32_t q[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {          // bytes 2 (i & 1), 2 (i & 1) + 1 of the block's word i / 2 under the exponent byte 0x64
        const uint32_t p = __builtin_amdgcn_perm(qk.ex, wd[s][i >> 1], (i & 1) ? 0x04030402u : 0x04010400u);
        q[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(v2h, p) + bias);
      }
      struct U4 { uint32_t x[4]; };
      const v8h B = __builtin_bit_cast(v8h, (U4{{q[0], q[1], q[2], q[3]}}));
      const v8h A = __builtin_bit_cast(v8h, (U4{{a4[s][0], a4[s][1], a4[s][2], a4[s][3]}}));
      const v4f acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, (v4f){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
      const float d = h2f_bits((hd[s >> 1] >> (16 * (s & 1))) & 0xFFFFu);
      const float d0 = d * ab.ai0, d1 = d * ab.ai1;
      tot[g][0] = fmaf(acc[0], d0, tot[g][0]); tot[g][1] = fmaf(acc[1], d0, tot[g][1]);
      tot[g][2] = fmaf(acc[2], d1, tot[g][2]); tot[g][3] = fmaf(acc[3], d1, tot[g][3]);
    }
  }
}
// grid = row tiles of 64, NW waves; wave w walks 128-column chunks [w * cpw, + cpw), two register buffers taking turns; the
// waves' sums meet in shared memory in wave order.  y[t * rows + row].
template <int NW> __global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void k_gemm_q8(QMatDev m, const uint4* __restrict__ aop, const float* __restrict__ ainv, float* __restrict__ y, int T, int R, int cpw) {
  __shared__ float red[NW][4][2][64];
  const int tile = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int K128 = m.cols >> 7;
  const int c0 = min(K128, wave * cpw), c1 = min(K128, c0 + cpw);
  v4f tot[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) tot[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  const Q8K qk = q8_consts();
  const AopRsrc ar = aop_rsrc(aop, m.cols, R, lane);
  WBuf8 w0, w1; ABuf a0, a1;
  if (c0 < c1) { load_a<true>(ar, ainv, R, c0, lane, a0); load_w8(m, tile * 4, c0, lane, K128, w0); }
  for (int c = c0; c < c1; c += 2) {
    if (c + 1 < c1) { load_a<true>(ar, ainv, R, c + 1, lane, a1); load_w8(m, tile * 4, c + 1, lane, K128, w1); }
    __builtin_amdgcn_sched_barrier(0);      // (keeps the compiler from sinking the loads down to their first use)
    chunk_mac8(w0, a0, qk, tot);
    __builtin_amdgcn_sched_barrier(0);
    if (c + 2 < c1) { load_a<true>(ar, ainv, R, c + 2, lane, a0); load_w8(m, tile * 4, c + 2, lane, K128, w0); }
    __builtin_amdgcn_sched_barrier(0);
    if (c + 1 < c1) chunk_mac8(w1, a1, qk, tot);
    __builtin_amdgcn_sched_barrier(0);
  }
  // lane (q, j) holds, for row group g, token 2q (rows 0, 1 of its four) and token 2q + 1 (rows 2, 3): halves h1, h2 * 2^11
#pragma unroll
  for (int g = 0; g < 4; ++g) { red[wave][g][0][lane] = tot[g][0] + tot[g][1] * (1.0f / 2048.0f); red[wave][g][1][lane] = tot[g][2] + tot[g][3] * (1.0f / 2048.0f); }
  lds_barrier();
  for (int i = threadIdx.x; i < T * 64; i += NW * 64) {
    const int t = i >> 6, rl = i & 63, l = (t >> 1) * 16 + (rl & 15), g = rl >> 4, h = t & 1;
    float s = red[0][g][h][l];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][g][h][l];
    const size_t row = (size_t)tile * 64 + rl;
    if (row < (size_t)m.rows) y[(size_t)t * m.rows + row] = s;
  }
}

size_t pyre_gemm_q8_bytes(size_t rows, size_t cols, size_t* codes) {
  const size_t rows_pad = (rows + 63) / 64 * 64, sq = (rows_pad * cols + 255) & ~(size_t)255, sh = (rows_pad * (cols / 128) * 8 + 255) & ~(size_t)255;
  if (codes) *codes = sq;
  return sq + sh;
}
int pyre_gemm_q8_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* base) {
  size_t sq; (void)pyre_gemm_q8_bytes(rows, cols, &sq);
  const int K128 = (int)(cols / 128); const size_t rows_pad = (rows + 63) / 64 * 64, total = rows_pad * K128;
  hipLaunchKernelGGL(k_repack_q8m, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, K128, raw_dev, row_bytes, (uint32_t*)base, (uint2*)((uint8_t*)base + sq));
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
// x [t][cols] f32 on the device -> y [t][rows]; the operand rows and their scale factors go to the context's grow-only scratch
// (scratch: the caller's memory of at least pyre_aop_bytes(cols, 8) rounded up to 256, plus cols / 256 * 32 bytes -- the entry
// point that allocates nothing passes the per-GPU array -- or null: the context's buffer)
int pyre_gemm_q8_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, void* scratch) {
  if (m.fmt != FMT_Q8_0_M || !m.mq || !m.mh) return pyre_fail(ctx, PYRE_E_TYPE, "gemm_q8: the matrix is not held in the Q8_0 matrix-core layout");
  if (t < 1 || t > 8 || m.cols % 256 != 0) return pyre_fail(ctx, PYRE_E_ARG, "gemm_q8: t = %d, %d columns", t, m.cols);
  uint4* op = (uint4*)scratch; float* ainv;
  if (!op) { int rc = pyre_gemm_m_scratch(ctx, m.cols, &op, &ainv); if (rc) return rc; }
  ainv = (float*)((uint8_t*)op + ((pyre_aop_bytes(m.cols, 8) + 255) & ~(size_t)255));
  int rc = pyre_act_split_launch(ctx, x_dev, t, m.cols, op, ainv); if (rc) return rc;
  const int R = pyre_aop_rows(t);
  int nw, cpw; pyre_gemm_m_plan(m, 1, &nw, &cpw);
  static const std::string names[9] = {"", "gemm_q8_0_t1", "gemm_q8_0_t2", "gemm_q8_0_t3", "gemm_q8_0_t4", "gemm_q8_0_t5", "gemm_q8_0_t6", "gemm_q8_0_t7", "gemm_q8_0_t8"};
  ProfScope ps(ctx, names[t].c_str(), qmat_gguf_bytes(m, m.rows) + 4.0 * t * ((double)m.cols + m.rows));
  if (nw == 4) hipLaunchKernelGGL((k_gemm_q8<4>), dim3(m.tiles), dim3(256), 0, ctx->stream, m, op, ainv, y_dev, t, R, cpw);
  else if (nw == 8) hipLaunchKernelGGL((k_gemm_q8<8>), dim3(m.tiles), dim3(512), 0, ctx->stream, m, op, ainv, y_dev, t, R, cpw);
  else hipLaunchKernelGGL((k_gemm_q8<16>), dim3(m.tiles), dim3(1024), 0, ctx->stream, m, op, ainv, y_dev, t, R, cpw);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
