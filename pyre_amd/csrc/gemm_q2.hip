// IQ2_XS dequant-GEMM on the f16 matrix cores, 2..8 tokens (QMat::matmul, src/model/gguf_q.rs:217-242, for the block type of
// :126-129): the window path of the stand-alone operator.  The lane = row GEMV decodes a weight once per token (the
// 151936 x 2048 head: 47 us at two tokens, 121 us at eight); here, as for IQ3_S (gemm_m.hip) and Q4_K (gemm_q4.hip), once
// whatever the window:
//   * w = d / 8 * (2 n + 1) * sign * {8, 25, 43}: n a 4-bit scale per 16 columns, the magnitude one of three;
//   * the layout keeps a weight as a 4-bit code (sign << 2 | magnitude index).  Two byte permutes look a code's f16 number up
//     in an 8-entry table held in registers (one permute per byte of the number, four codes at a time), a third pairs the
//     bytes up; one packed multiplication folds 2 n + 1 in: at most 43 * 31 = 1333, exact in f16;
//   * v_mfma_f32_16x16x32_f16 multiplies 16 weight rows x 32 columns with the sixteen activation rows (two f16 halves of up
//     to eight tokens, gemm_m.hip); a lane's eight columns lie in one half of the 32, so its scale is one number;
//     d / 8 meets the f32 sums once per 128 columns.
// Layout (FMT_IQ2_XS_M): the codes where FMT_IQ3_S_M keeps its codes (QMatDev::mq: a lane's share of a 128-column chunk is
// one 16-byte load; inside a 32-bit word the weights e = 0..3 of the lane's eight sit in the even nibbles, 4..7 in the odd
// ones); per row and super-block a 16-byte header (QMatDev::mh): d, then the block's eight scale bytes.  4.5 bit/weight.
// A token's operand rows reach only its own sums: its result is bit-identical for every window width 2..8.
#include "gemm_m.h"

// ---- the matrix: raw GGUF rows -> mq / mh; one thread per (row of the padded row groups, super-block) ----------------------
// grid: the 512 x 8 magnitudes (8, 25 or 43 a byte) of the codebook
__global__ __launch_bounds__(256) void k_repack_q2m(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, const uint64_t* __restrict__ grid, uint32_t* __restrict__ mq, uint4* __restrict__ mh) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB) return;
  const int row = (int)(idx / SB), sb = (int)(idx % SB); const bool live = row < rows;      // padding rows lie past the end of the raw buffer: never read them
  const size_t rg = (size_t)(row >> 4); const int j = row & 15; const size_t K128 = (size_t)SB * 2;
  const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 74;
  for (int ib = 0; ib < 8; ++ib) {               // sub-block ib: entries 4 ib .. + 3 of eight weights each
    for (int l = 0; l < 4; ++l) {                // entry 4 ib + l = the share of lane group l
      uint32_t wd = 0;
      if (live) {
        const uint32_t q = (uint32_t)b[2 + 2 * (4 * ib + l)] | ((uint32_t)b[3 + 2 * (4 * ib + l)] << 8);
        const uint64_t g = grid[q & 511u]; const uint32_t sg = ksigns(q >> 9);
        for (int e = 0; e < 8; ++e) {
          const uint32_t mag = (uint32_t)(g >> (8 * e)) & 0xFFu, code = (mag > 8u) + (mag > 25u) + (((sg >> e) & 1u) << 2);
          wd |= code << (4 * (e < 4 ? 2 * e : 2 * (e - 4) + 1));
        }
      }
      mq[(mq_slot(rg, 2 * sb + (ib >> 2), (int)K128) + l * 16 + j) * 4 + (ib & 3)] = wd;
    }
  }
  uint4 hd{0u, 0u, 0u, 0u};
  if (live) {
    hd.x = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
    hd.y = (uint32_t)b[66] | ((uint32_t)b[67] << 8) | ((uint32_t)b[68] << 16) | ((uint32_t)b[69] << 24);
    hd.z = (uint32_t)b[70] | ((uint32_t)b[71] << 8) | ((uint32_t)b[72] << 16) | ((uint32_t)b[73] << 24);
  }
  mh[mh_slot(rg, sb, SB) + j] = hd;
}

// ---- the product -----------------------------------------------------------------------------------------------------------------
struct WBuf2 { uint4 w[4]; uint4 h[4]; };
__device__ __forceinline__ void load_w2(const QMatDev& m, int rg0, int c, int lane, int K128, WBuf2& b) {
#pragma unroll
  for (int g = 0; g < 4; ++g) b.w[g] = ((const uint4*)m.mq)[mq_slot((size_t)rg0 + g, c, K128) + lane];
#pragma unroll
  for (int g = 0; g < 4; ++g) b.h[g] = ((const uint4*)m.mh)[mh_slot((size_t)rg0 + g, c >> 1, m.SB) + (lane & 15)];
}
// The table: entry (sign << 2 | index) -> the f16 number +-8, +-25, +-43 (0x4800, 0x4E40, 0x5160), low bytes and high bytes
// apart.  Kept in registers the compiler cannot see through, so that the permutes stay permutes.
struct LutK { uint32_t lo0, lo1, hi0, hi1, m4; };
__device__ __forceinline__ LutK lut_consts() {
  LutK k;
  asm volatile("v_mov_b32 %0, 0x00604000" : "=v"(k.lo0)); asm volatile("v_mov_b32 %0, 0x00604000" : "=v"(k.lo1));
  asm volatile("v_mov_b32 %0, 0x00514E48" : "=v"(k.hi0)); asm volatile("v_mov_b32 %0, 0x00D1CEC8" : "=v"(k.hi1));
  asm volatile("s_mov_b32 %0, 0x0F0F0F0F" : "=s"(k.m4));
  return k;
}
// eight codes of u -> four registers of two f16 numbers: weights (0, 1), (2, 3), (4, 5), (6, 7)
__device__ __forceinline__ void code_f16(uint32_t u, const LutK& k, uint32_t (&p)[4]) {
  const uint32_t ce = u & k.m4, co = (u >> 4) & k.m4;                 // the codes of weights 0..3, 4..7: a byte each
  const uint32_t le = __builtin_amdgcn_perm(k.lo1, k.lo0, ce), he = __builtin_amdgcn_perm(k.hi1, k.hi0, ce);
  const uint32_t lo = __builtin_amdgcn_perm(k.lo1, k.lo0, co), ho = __builtin_amdgcn_perm(k.hi1, k.hi0, co);
  p[0] = __builtin_amdgcn_perm(he, le, 0x05010400u); p[1] = __builtin_amdgcn_perm(he, le, 0x07030602u);
  p[2] = __builtin_amdgcn_perm(ho, lo, 0x05010400u); p[3] = __builtin_amdgcn_perm(ho, lo, 0x07030602u);
}
__device__ __forceinline__ void chunk_mac2(const WBuf2& wb, const ABuf& ab, int c, int lane, const LutK& lk, v4f (&tot)[4]) {
  const bool half = (c & 1) != 0;                // the chunk's four sub-blocks: scale bytes 0..3 or 4..7
  const uint32_t up = (uint32_t)(lane >> 5) * 4u;          // the lane's eight columns: the first sixteen of a sub-block (low nibble of its byte) or the second
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint4 hd = wb.h[g];
    const uint32_t sc = (half ? hd.z : hd.y) >> up;
    const uint32_t wd[4] = {wb.w[g].x, wb.w[g].y, wb.w[g].z, wb.w[g].w};
    const uint32_t a4[4][4] = {{ab.a[0].x, ab.a[0].y, ab.a[0].z, ab.a[0].w}, {ab.a[1].x, ab.a[1].y, ab.a[1].z, ab.a[1].w}, {ab.a[2].x, ab.a[2].y, ab.a[2].z, ab.a[2].w}, {ab.a[3].x, ab.a[3].y, ab.a[3].z, ab.a[3].w}};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      // 2 n + 1 twice over: 1024 + 2 n + 1 by its bits, less 1024
      const uint32_t n = (sc >> (8 * s)) & 15u;
      const v2h vs = __builtin_bit_cast(v2h, n * 0x00020002u + 0x64016401u) - (v2h){(_Float16)1024.0f, (_Float16)1024.0f};
      uint32_t p[4], q[4];
      code_f16(wd[s], lk, p);
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(v2h, p[i]) * vs);
      struct U4 { uint32_t x[4]; };
      const v8h B = __builtin_bit_cast(v8h, (U4{{q[0], q[1], q[2], q[3]}}));
      const v8h A = __builtin_bit_cast(v8h, (U4{{a4[s][0], a4[s][1], a4[s][2], a4[s][3]}}));
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, acc, 0, 0, 0);
    }
    const float d = h2f_bits(hd.x & 0xFFFFu) * 0.125f;
    const float d0 = d * ab.ai0, d1 = d * ab.ai1;
    tot[g][0] = fmaf(acc[0], d0, tot[g][0]); tot[g][1] = fmaf(acc[1], d0, tot[g][1]);
    tot[g][2] = fmaf(acc[2], d1, tot[g][2]); tot[g][3] = fmaf(acc[3], d1, tot[g][3]);
  }
}
// grid = row tiles of 64, NW waves; wave w walks 128-column chunks [w * cpw, + cpw), two register buffers taking turns; the
// waves' sums meet in shared memory in wave order.  y[t * rows + row].
template <int NW> __global__ __launch_bounds__(NW * 64) void k_gemm_q2(QMatDev m, const uint4* __restrict__ aop, const float* __restrict__ ainv, float* __restrict__ y, int T, int R, int cpw) {
  __shared__ float red[NW][4][2][64];
  const int tile = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int K128 = m.cols >> 7;
  const int c0 = min(K128, wave * cpw), c1 = min(K128, c0 + cpw);
  v4f tot[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) tot[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  const LutK lk = lut_consts();
  const AopRsrc ar = aop_rsrc(aop, m.cols, R, lane);
  WBuf2 w0, w1; ABuf a0, a1;
  if (c0 < c1) { load_a<true>(ar, ainv, R, c0, lane, a0); load_w2(m, tile * 4, c0, lane, K128, w0); }
  for (int c = c0; c < c1; c += 2) {
    if (c + 1 < c1) { load_a<true>(ar, ainv, R, c + 1, lane, a1); load_w2(m, tile * 4, c + 1, lane, K128, w1); }
    __builtin_amdgcn_sched_barrier(0);      // (keeps the compiler from sinking the loads down to their first use)
    chunk_mac2(w0, a0, c, lane, lk, tot);
    __builtin_amdgcn_sched_barrier(0);
    if (c + 2 < c1) { load_a<true>(ar, ainv, R, c + 2, lane, a0); load_w2(m, tile * 4, c + 2, lane, K128, w0); }
    __builtin_amdgcn_sched_barrier(0);
    if (c + 1 < c1) chunk_mac2(w1, a1, c + 1, lane, lk, tot);
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

size_t pyre_gemm_q2_bytes(size_t rows, size_t cols, size_t* codes) {
  const size_t rows_pad = (rows + 63) / 64 * 64, sq = (rows_pad * cols / 2 + 255) & ~(size_t)255, sh = (rows_pad * (cols / 256) * 16 + 255) & ~(size_t)255;
  if (codes) *codes = sq;
  return sq + sh;
}
int pyre_gemm_q2_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* base) {
  size_t sq; (void)pyre_gemm_q2_bytes(rows, cols, &sq);
  const int SB = (int)(cols / 256); const size_t rows_pad = (rows + 63) / 64 * 64, total = rows_pad * SB;
  hipLaunchKernelGGL(k_repack_q2m, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, raw_dev, row_bytes, (const uint64_t*)ctx->d_iq2xs, (uint32_t*)base, (uint4*)((uint8_t*)base + sq));
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
// x [t][cols] f32 on the device -> y [t][rows]; the operand rows and their scale factors go to the context's grow-only scratch
// (scratch: the caller's memory of at least pyre_aop_bytes(cols, 8) rounded up to 256, plus cols / 256 * 32 bytes -- the entry
// point that allocates nothing passes the per-GPU array -- or null: the context's buffer)
int pyre_gemm_q2_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, void* scratch) {
  if (m.fmt != FMT_IQ2_XS_M || !m.mq || !m.mh) return pyre_fail(ctx, PYRE_E_TYPE, "gemm_q2: the matrix is not held in the IQ2_XS matrix-core layout");
  if (t < 1 || t > 8 || m.cols % 256 != 0 || m.SB != m.cols / 256) return pyre_fail(ctx, PYRE_E_ARG, "gemm_q2: t = %d, %d columns", t, m.cols);
  uint4* op = (uint4*)scratch; float* ainv;
  if (!op) { int rc = pyre_gemm_m_scratch(ctx, m.cols, &op, &ainv); if (rc) return rc; }
  ainv = (float*)((uint8_t*)op + ((pyre_aop_bytes(m.cols, 8) + 255) & ~(size_t)255));
  int rc = pyre_act_split_launch(ctx, x_dev, t, m.cols, op, ainv); if (rc) return rc;
  const int R = pyre_aop_rows(t);
  int nw, cpw; pyre_gemm_m_plan(m, 1, &nw, &cpw);
  static const std::string names[9] = {"", "gemm_iq2xs_t1", "gemm_iq2xs_t2", "gemm_iq2xs_t3", "gemm_iq2xs_t4", "gemm_iq2xs_t5", "gemm_iq2xs_t6", "gemm_iq2xs_t7", "gemm_iq2xs_t8"};
  ProfScope ps(ctx, names[t].c_str(), qmat_gguf_bytes(m, m.rows) + 4.0 * t * ((double)m.cols + m.rows));
  if (nw == 4) hipLaunchKernelGGL((k_gemm_q2<4>), dim3(m.tiles), dim3(256), 0, ctx->stream, m, op, ainv, y_dev, t, R, cpw);
  else if (nw == 8) hipLaunchKernelGGL((k_gemm_q2<8>), dim3(m.tiles), dim3(512), 0, ctx->stream, m, op, ainv, y_dev, t, R, cpw);
  else hipLaunchKernelGGL((k_gemm_q2<16>), dim3(m.tiles), dim3(1024), 0, ctx->stream, m, op, ainv, y_dev, t, R, cpw);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
