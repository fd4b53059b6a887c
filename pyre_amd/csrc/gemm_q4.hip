// Q4_K dequant-GEMM on the f16 matrix cores, 2..8 tokens (QMat::matmul, src/model/gguf_q.rs:217-242, for the block type of
// :96-120): the window path of the stand-alone operator.  The lane = row GEMV pays byte -> float -> multiply-add per weight
// AND token (the 151936 x 2048 head: 50 us at two tokens, 117 us at eight); here, as for IQ3_S (gemm_m.hip), a weight is
// decoded once whatever the window:
//   * w = d * s * q - dmin * m per 32-value sub-block, q a 4-bit code, s and m 6-bit integers;
//   * q becomes the f16 number 16 + q by or-ing it into a mantissa, one packed fma folds the sub-block's scale in:
//     (16 + q) * s - 16 s = q s <= 945, every intermediate an integer below 2048 and exact in f16;
//   * v_mfma_f32_16x16x32_f16 multiplies 16 weight rows x 32 columns with the sixteen activation rows (two f16 halves of up
//     to eight tokens, gemm_m.hip); d meets the f32 sums once per 128 columns;
//   * the - dmin * m term needs the sub-block's sum of activations, not the activations: the launch that forms the operand
//     rows also leaves the f32 sum of every 32 columns of every token, and a lane adds m * sum for its row and its two tokens.
// Layout (FMT_Q4_K_M): the codes as FMT_IQ3_S_M keeps its codes (QMatDev::mq: a lane's share of a 128-column chunk is one
// 16-byte load); per row and super-block a 16-byte header (QMatDev::mh): d | dmin << 16, then sixteen 6-bit fields -- the
// eight scales, the eight minima -- back to back.  4.5 bit/weight, what the file has.
// A token's operand rows reach only its own sums: its result is bit-identical for every window width 2..8.
#include "gemm_m.h"

// ---- the matrix: raw GGUF rows -> mq / mh; one thread per (row of the padded row groups, super-block) ----------------------
__global__ __launch_bounds__(256) void k_repack_q4m(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, uint32_t* __restrict__ mq, uint4* __restrict__ mh) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB) return;
  const int row = (int)(idx / SB), sb = (int)(idx % SB); const bool live = row < rows;      // padding rows lie past the end of the raw buffer: never read them
  const size_t rg = (size_t)(row >> 4); const int j = row & 15; const size_t K128 = (size_t)SB * 2;
  const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 144;
  for (int ib = 0; ib < 8; ++ib) {               // sub-block ib: the low (even ib) or high nibbles of the 32 bytes of group ib / 2
    for (int l = 0; l < 4; ++l) {                // eight consecutive values = the share of lane group l
      uint32_t wd = 0;
      if (live) for (int e = 0; e < 8; ++e) { const uint32_t q = (b[16 + 32 * (ib >> 1) + 8 * l + e] >> (4 * (ib & 1))) & 0xFu; wd |= q << (4 * ((e >> 1) + 4 * (e & 1))); }
      mq[(mq_slot(rg, 2 * sb + (ib >> 2), (int)K128) + l * 16 + j) * 4 + (ib & 3)] = wd;
    }
  }
  uint4 hd{0u, 0u, 0u, 0u};
  if (live) {
    hd.x = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24);
    const uint32_t w0 = (uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24), w1 = (uint32_t)b[8] | ((uint32_t)b[9] << 8) | ((uint32_t)b[10] << 16) | ((uint32_t)b[11] << 24),
                   w2 = (uint32_t)b[12] | ((uint32_t)b[13] << 8) | ((uint32_t)b[14] << 16) | ((uint32_t)b[15] << 24);
    uint32_t f[3] = {0u, 0u, 0u};
    for (int i = 0; i < 8; ++i) {
      uint32_t s, mn; scale_min_k4(i, w0, w1, w2, s, mn);
      const int bs = 6 * i, bm = 6 * (8 + i);
      f[bs >> 5] |= s << (bs & 31); if ((bs & 31) > 26) f[(bs >> 5) + 1] |= s >> (32 - (bs & 31));
      f[bm >> 5] |= mn << (bm & 31); if ((bm & 31) > 26) f[(bm >> 5) + 1] |= mn >> (32 - (bm & 31));
    }
    hd.y = f[0]; hd.z = f[1]; hd.w = f[2];
  }
  mh[mh_slot(rg, sb, SB) + j] = hd;
}

// ---- the activation operand and the sub-block sums: grid = super-blocks (256 columns), 256 threads, thread = column ------------
// The operand rows as k_act_split leaves them (each 256-column stretch of a token on its own power of two); asum[(k / 32) * 8 + t]
// = the f32 sum of token t's columns 32 (k / 32) .. + 31, added in a fixed tree.
__global__ __launch_bounds__(256) void k_act_split_q4(const float* __restrict__ x, int T, int R, int cols, uint16_t* __restrict__ op, float* __restrict__ ainv, float* __restrict__ asum) {
  __shared__ float mx[4][8];
  const int sb = blockIdx.x, i = threadIdx.x, k = sb * 256 + i, wave = i >> 6, lane = i & 63;
  float v[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) v[t] = t < T ? x[(size_t)t * cols + k] : 0.0f;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    float a = fabsf(v[t]); a = a == a ? a : INFINITY;         // a NaN anywhere makes the stretch non-finite
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) a = fmaxf(a, __shfl_xor(a, o));
    if (lane == 0) mx[wave][t] = a;
    float s = v[t];
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if ((lane & 31) == 0) asum[(size_t)(k >> 5) * 8 + t] = s;
  }
  __syncthreads();
  uint16_t* o = op + (size_t)(k >> 3) * R * 8 + (k & 7);
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const float m = fmaxf(fmaxf(mx[0][t], mx[1][t]), fmaxf(mx[2][t], mx[3][t]));
    int e = 0;                                                // m * 2^e in [2^13, 2^14); zero and non-finite stretches stay as they are
    if (m > 0.0f && m < INFINITY) { e = 140 - (int)((__float_as_uint(m) >> 23) & 0xFF); e = e > 100 ? 100 : e; }
    const float up = __uint_as_float((uint32_t)(127 + e) << 23), dn = __uint_as_float((uint32_t)(127 - e) << 23);
    const float xs = v[t] * up;
    const _Float16 h1 = (_Float16)xs, h2 = (_Float16)((xs - (float)h1) * 2048.0f);
    if (2 * t < R) { o[(2 * t) * 8] = __builtin_bit_cast(unsigned short, h1); o[(2 * t + 1) * 8] = __builtin_bit_cast(unsigned short, h2); }
    if (i == 0) ainv[sb * 8 + t] = t < T ? dn : 0.0f;
  }
}

// ---- the product -----------------------------------------------------------------------------------------------------------------
struct WBuf4 { uint4 w[4]; uint4 h[4]; };
struct ABuf4 { ABuf a; float2 sm[4]; };
__device__ __forceinline__ void load_w4(const QMatDev& m, int rg0, int c, int lane, int K128, WBuf4& b) {
#pragma unroll
  for (int g = 0; g < 4; ++g) b.w[g] = ((const uint4*)m.mq)[mq_slot((size_t)rg0 + g, c, K128) + lane];
#pragma unroll
  for (int g = 0; g < 4; ++g) b.h[g] = ((const uint4*)m.mh)[mh_slot((size_t)rg0 + g, c >> 1, m.SB) + (lane & 15)];
}
__device__ __forceinline__ void load_a4(const AopRsrc& ar, const float* __restrict__ ainv, const float* __restrict__ asum, int R, int c, int lane, ABuf4& b) {
  load_a<true>(ar, ainv, R, c, lane, b.a);
#pragma unroll
  for (int s = 0; s < 4; ++s) b.sm[s] = *(const float2*)(asum + (size_t)(c * 4 + s) * 8 + 2 * (lane >> 4));
}
__device__ __forceinline__ void chunk_mac4(const WBuf4& wb, const ABuf4& ab, int c, const NibK& nk, v4f (&tot)[4]) {
  const bool half = (c & 1) != 0;                // the chunk's four sub-blocks: fields 0..3 or 4..7 of the scales, 8..11 or 12..15 of the minima
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint4 hd = wb.h[g];
    const uint32_t sc24 = half ? __builtin_amdgcn_alignbit(hd.z, hd.y, 24) : hd.y, mn24 = half ? (hd.w >> 8) : __builtin_amdgcn_alignbit(hd.w, hd.z, 16);
    const uint32_t wd[4] = {wb.w[g].x, wb.w[g].y, wb.w[g].z, wb.w[g].w};
    const uint32_t a4[4][4] = {{ab.a.a[0].x, ab.a.a[0].y, ab.a.a[0].z, ab.a.a[0].w}, {ab.a.a[1].x, ab.a.a[1].y, ab.a.a[1].z, ab.a.a[1].w}, {ab.a.a[2].x, ab.a.a[2].y, ab.a.a[2].z, ab.a.a[2].w}, {ab.a.a[3].x, ab.a.a[3].y, ab.a.a[3].z, ab.a.a[3].w}};
    float ms0 = 0.0f, ms1 = 0.0f;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const _Float16 hs = (_Float16)(unsigned short)((sc24 >> (6 * s)) & 63u);          // (one conversion: 16-bit integer -> f16)
      const v2h vs = {hs, hs}, vneg = vs * (v2h){(_Float16)-16.0f, (_Float16)-16.0f};
      uint32_t p[4], q[4];
      nib_f16(wd[s], nk, p);
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(v2h, p[i]), vs, vneg));
      struct U4 { uint32_t x[4]; };
      const v8h B = __builtin_bit_cast(v8h, (U4{{q[0], q[1], q[2], q[3]}}));
      const v8h A = __builtin_bit_cast(v8h, (U4{{a4[s][0], a4[s][1], a4[s][2], a4[s][3]}}));
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, acc, 0, 0, 0);
      const float mf = (float)((mn24 >> (6 * s)) & 63u);
      ms0 = fmaf(mf, ab.sm[s].x, ms0); ms1 = fmaf(mf, ab.sm[s].y, ms1);
    }
    const float d = h2f_bits(hd.x & 0xFFFFu), dmin = h2f_bits(hd.x >> 16);
    const float d0 = d * ab.a.ai0, d1 = d * ab.a.ai1;
    tot[g][0] = fmaf(acc[0], d0, tot[g][0]); tot[g][1] = fmaf(acc[1], d0, tot[g][1]);
    tot[g][2] = fmaf(acc[2], d1, tot[g][2]); tot[g][3] = fmaf(acc[3], d1, tot[g][3]);
    tot[g][0] = fmaf(-dmin, ms0, tot[g][0]); tot[g][2] = fmaf(-dmin, ms1, tot[g][2]);
  }
}
// grid = row tiles of 64, NW waves; wave w walks 128-column chunks [w * cpw, + cpw), two register buffers taking turns; the
// waves' sums meet in shared memory in wave order.  y[t * rows + row].
template <int NW> __global__ __launch_bounds__(NW * 64) void k_gemm_q4(QMatDev m, const uint4* __restrict__ aop, const float* __restrict__ ainv, const float* __restrict__ asum, float* __restrict__ y, int T, int R, int cpw) {
  __shared__ float red[NW][4][2][64];
  const int tile = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int K128 = m.cols >> 7;
  const int c0 = min(K128, wave * cpw), c1 = min(K128, c0 + cpw);
  v4f tot[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) tot[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  const NibK nk = nib_consts();
  const AopRsrc ar = aop_rsrc(aop, m.cols, R, lane);
  WBuf4 w0, w1; ABuf4 a0, a1;
  if (c0 < c1) { load_a4(ar, ainv, asum, R, c0, lane, a0); load_w4(m, tile * 4, c0, lane, K128, w0); }
  for (int c = c0; c < c1; c += 2) {
    if (c + 1 < c1) { load_a4(ar, ainv, asum, R, c + 1, lane, a1); load_w4(m, tile * 4, c + 1, lane, K128, w1); }
    __builtin_amdgcn_sched_barrier(0);      // (keeps the compiler from sinking the loads down to their first use)
    chunk_mac4(w0, a0, c, nk, tot);
    __builtin_amdgcn_sched_barrier(0);
    if (c + 2 < c1) { load_a4(ar, ainv, asum, R, c + 2, lane, a0); load_w4(m, tile * 4, c + 2, lane, K128, w0); }
    __builtin_amdgcn_sched_barrier(0);
    if (c + 1 < c1) chunk_mac4(w1, a1, c + 1, nk, tot);
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

size_t pyre_gemm_q4_bytes(size_t rows, size_t cols, size_t* codes) {
  const size_t rows_pad = (rows + 63) / 64 * 64, sq = (rows_pad * cols / 2 + 255) & ~(size_t)255, sh = (rows_pad * (cols / 256) * 16 + 255) & ~(size_t)255;
  if (codes) *codes = sq;
  return sq + sh;
}
int pyre_gemm_q4_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* base) {
  size_t sq; (void)pyre_gemm_q4_bytes(rows, cols, &sq);
  const int SB = (int)(cols / 256); const size_t rows_pad = (rows + 63) / 64 * 64, total = rows_pad * SB;
  hipLaunchKernelGGL(k_repack_q4m, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, raw_dev, row_bytes, (uint32_t*)base, (uint4*)((uint8_t*)base + sq));
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
// x [t][cols] f32 on the device -> y [t][rows]; the operand rows, their scale factors and the sub-block sums go to the context's
// grow-only scratch
// (scratch: the caller's memory of at least pyre_gemm_q4_scratch_bytes(cols) bytes -- the entry point that allocates nothing
// passes the per-GPU array -- or null: the context's buffer)
size_t pyre_gemm_q4_scratch_bytes(int cols) { return ((pyre_aop_bytes(cols, 8) + 255) & ~(size_t)255) + ((size_t)(cols / 256) * 8 + 64) * 4 + (size_t)(cols / 32) * 8 * 4; }
int pyre_gemm_q4_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev, void* scratch) {
  if (m.fmt != FMT_Q4_K_M || !m.mq || !m.mh) return pyre_fail(ctx, PYRE_E_TYPE, "gemm_q4: the matrix is not held in the Q4_K matrix-core layout");
  if (t < 1 || t > 8 || m.cols % 256 != 0 || m.SB != m.cols / 256) return pyre_fail(ctx, PYRE_E_ARG, "gemm_q4: t = %d, %d columns", t, m.cols);
  uint4* op = (uint4*)scratch; float* ainv;
  if (!op) { int rc = pyre_gemm_m_scratch(ctx, m.cols + m.cols / 16 + 256, &op, &ainv); if (rc) return rc; }      // (room for the sums behind the operand of m.cols columns)
  const size_t ob = (pyre_aop_bytes(m.cols, 8) + 255) & ~(size_t)255;
  ainv = (float*)((uint8_t*)op + ob); float* asum = ainv + (size_t)(m.cols / 256) * 8 + 64;
  const int R = pyre_aop_rows(t);
  { ProfScope ps(ctx, "act_split_f16", 4.0 * t * m.cols + (double)pyre_aop_bytes(m.cols, t));
    hipLaunchKernelGGL(k_act_split_q4, dim3(m.cols / 256), dim3(256), 0, ctx->stream, x_dev, t, R, m.cols, (uint16_t*)op, ainv, asum); } PYRE_CHECK_LAUNCH(ctx);
  int nw, cpw; pyre_gemm_m_plan(m, 1, &nw, &cpw);
  static const std::string names[9] = {"", "gemm_q4k_t1", "gemm_q4k_t2", "gemm_q4k_t3", "gemm_q4k_t4", "gemm_q4k_t5", "gemm_q4k_t6", "gemm_q4k_t7", "gemm_q4k_t8"};
  ProfScope ps(ctx, names[t].c_str(), qmat_gguf_bytes(m, m.rows) + 4.0 * t * ((double)m.cols + m.rows));
  if (nw == 4) hipLaunchKernelGGL((k_gemm_q4<4>), dim3(m.tiles), dim3(256), 0, ctx->stream, m, op, ainv, asum, y_dev, t, R, cpw);
  else if (nw == 8) hipLaunchKernelGGL((k_gemm_q4<8>), dim3(m.tiles), dim3(512), 0, ctx->stream, m, op, ainv, asum, y_dev, t, R, cpw);
  else hipLaunchKernelGGL((k_gemm_q4<16>), dim3(m.tiles), dim3(1024), 0, ctx->stream, m, op, ainv, asum, y_dev, t, R, cpw);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
