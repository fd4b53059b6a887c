// IQ3_S dequant-GEMM on the f16 matrix cores, 1..8 tokens (QMat::matmul, src/model/gguf_q.rs:217-242; the verify window of
// lcm_dense / the MTP drafter, qwen4exp_gguf.rs:2641-2737, is the same product with t > 1).
//
// The lane = row GEMV spends about 2.7 vector instructions per weight and token (nibble -> byte -> float -> fma); on the
// 151 936 x 2048 head that is as long as streaming its bytes, and every further token of a window costs the same again.
// Here a weight costs about 1.6 instructions whatever the number of tokens:
//   * the 4-bit code c of a weight w = (2c - 15) * (2n + 1) * d becomes the f16 number 16 + c by or-ing it into a
//     mantissa (0x4C00 | c << 6), two per register;
//   * one packed f16 fma per register pair folds the sub-block scale in: (16 + c) * 2s - 47s = (2c - 15) * s, s = 2n + 1,
//     every intermediate an integer below 2048 and therefore exact in f16;
//   * v_mfma_f32_16x16x32_f16 multiplies 16 weight rows x 32 columns with 16 activation rows.  An activation row is one
//     half of a token: x = h1 + h2 * 2^-11 with h1 = f16(x), h2 = f16((x - h1) * 2^11), 22 significant bits, so eight
//     tokens fill the sixteen rows and one token costs what eight do;
//   * d (per super-block and row) and the power of two the activations were scaled by meet the f32 sums once per
//     128 columns.
// Products are exact in f32 and are summed in f32, so the result differs from the exact dot product by the 2^-22
// representation of x and the usual f32 summation error.  A token's operand rows are read by nobody else's sums: its
// result is bit-identical for every window width.
//
// grid (row tiles of 64, K slices), NW waves.  Wave w of slice ks walks 128-column chunks [(ks*NW + w) * cpw, + cpw).
#include "gemm_m.h"
#include <mutex>

PYRE_TS_DECL(gemm_ts) PYRE_TS_EXPORT(gemm_ts, pyre_debug_ts_gemm)

int pyre_aop_rows(int t) { return t <= 1 ? 2 : (t == 2 ? 4 : (t <= 4 ? 8 : 16)); }
size_t pyre_aop_bytes(int cols, int t) { return (size_t)(cols / 8) * pyre_aop_rows(t) * 16; }

// ---- the activation operand from f32 rows: grid = super-blocks (256 columns), 256 threads, thread = column ---------------------
// Each 256-column stretch of a token is scaled by its own power of two so that its largest magnitude lands in [2^13, 2^14):
// the f16 halves then keep 22 bits of every value that matters to the sum, whatever the magnitudes of x.
__global__ __launch_bounds__(256) void k_act_split(const float* __restrict__ x, int T, int R, int cols, uint16_t* __restrict__ op, float* __restrict__ ainv, size_t wz) {
  __shared__ float mx[4][8];
  if (wz) { const size_t zo = (size_t)blockIdx.y * wz; x = (const float*)((const char*)x + zo); op = (uint16_t*)((char*)op + zo); ainv = (float*)((char*)ainv + zo); }      // a launch for several windows, their buffers wz bytes apart
  PYRE_TS_VARS PYRE_TS(0);
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
  PYRE_TS(1); PYRE_TS_FLUSH(gemm_ts, 24);
}

int pyre_act_split_launch(pyre_ctx* ctx, const float* x_dev, int t, int cols, uint4* op, float* ainv) {
  ProfScope ps(ctx, "act_split_f16", 4.0 * t * cols + (double)pyre_aop_bytes(cols, t));
  hipLaunchKernelGGL(k_act_split, dim3(cols / 256, ctx->batch_n), dim3(256), 0, ctx->stream, x_dev, t, pyre_aop_rows(t), cols, (uint16_t*)op, ainv, ctx->batch_stride);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

// ---- the product (the chunk loads and chunk_mac live in gemm_m.h) ---------------------------------------------------------------
//   ksplit == 1: y[t*rows + row] = sum.
//   ksplit  > 1: y is a partial buffer, y[(ks*T + t)*tiles*64 + row] = slice sum (the consumer adds the slices in order).
//   ep.best (T == 1, ksplit == 1): best[2*tile] = bits of the tile's maximum, best[2*tile+1] = its first row.
//   ep.co: conv1d + SiLU of the leading ep.ch rows (linear_core, qwen4exp_gguf.rs:1643-1647), as in the lane = row GEMV.
//   FT > 0: the window width as a compile-time constant -- T = FT, its operand rows and (CONV) four taps folded in; FT = 1 is
//   the single-token instance ("ONE" below).
//   XF (with ONE): `aop` is the token's f32 activations; every wave forms the operand rows of its chunks itself, with the
//   arithmetic of k_act_split (the 256-column stretch's power of two from a wave maximum over the stretch), so the sums
//   are bit for bit those of the split launch followed by this one -- a launch less where the producer of x cannot
//   scale (it does not know the stretch's maximum) and the matrix has few row tiles to repeat the conversion in.
__device__ __forceinline__ void load_a_x(const float* __restrict__ x, int c, int lane, ABuf& b) {
  const int row = lane & 15, kg = lane >> 4;
  const float4 sv = ((const float4*)(x + (size_t)(c >> 1) * 256))[lane];
  float4 xv[4][2];
#pragma unroll
  for (int s = 0; s < 4; ++s) { const float4* p = (const float4*)(x + (size_t)c * 128 + s * 32 + kg * 8); xv[s][0] = p[0]; xv[s][1] = p[1]; }
  auto nn = [](float v) { float a = fabsf(v); return a == a ? a : INFINITY; };          // a NaN anywhere makes the stretch non-finite
  const float m = wave_max(fmaxf(fmaxf(nn(sv.x), nn(sv.y)), fmaxf(nn(sv.z), nn(sv.w))));
  int e = 0;
  if (m > 0.0f && m < INFINITY) { e = 140 - (int)((__float_as_uint(m) >> 23) & 0xFF); e = e > 100 ? 100 : e; }
  const float up = __uint_as_float((uint32_t)(127 + e) << 23), dn = __uint_as_float((uint32_t)(127 - e) << 23);
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const float v[8] = {xv[s][0].x, xv[s][0].y, xv[s][0].z, xv[s][0].w, xv[s][1].x, xv[s][1].y, xv[s][1].z, xv[s][1].w};
    uint32_t w[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t hh[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float xs = v[2 * q + u] * up;
        const _Float16 h1 = (_Float16)xs, h2 = (_Float16)((xs - (float)h1) * 2048.0f);
        hh[u] = row == 0 ? __builtin_bit_cast(unsigned short, h1) : (row == 1 ? __builtin_bit_cast(unsigned short, h2) : 0u);
      }
      w[q] = hh[0] | (hh[1] << 16);
    }
    b.a[s] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  b.ai0 = kg == 0 ? dn : 0.0f; b.ai1 = 0.0f;
}
//   SQ: the operand of a Gated DeltaNet output projection with per-sub-block scales and the head norm (load_a_sq).
template <int NW, bool SC, bool CONV, int FT = 0, bool XF = false, bool SQ = false>
__global__ __launch_bounds__(NW * 64) void k_gemm_m(QMatDev m, const uint4* __restrict__ aop, const float* __restrict__ ainv, float* __restrict__ y, int T, int R, int cpw, GemvEpi ep, size_t wz) {
  __shared__ float red[NW][4][2][64];
  PYRE_TS_VARS PYRE_TS(0);
  qmat_args_now(m); args_now(aop, ainv, y, T, R, cpw, ep.best, ep.conv_w, ep.conv_in, ep.conv_out, ep.co, ep.ch, ep.kk);
  if (wz) {          // a launch for several windows (a long prompt's blocks): blockIdx.z's operand, scale factors and output lie wz bytes further on per window
    const size_t zo = (size_t)blockIdx.z * wz;
    aop = (const uint4*)((const char*)aop + zo); y = (float*)((char*)y + zo); if (ainv) ainv = (const float*)((const char*)ainv + zo);
  }
  constexpr bool ONE = FT == 1;
  if constexpr (FT > 0) { T = FT; R = FT <= 1 ? 2 : (FT == 2 ? 4 : (FT <= 4 ? 8 : 16)); }
  const int kk = FT > 0 ? 4 : ep.kk;
  const int tile = blockIdx.x, ks = blockIdx.y, ksplit = gridDim.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int K128 = m.cols >> 7;
  const int c0 = (ks * NW + wave) * cpw, c1 = min(K128, c0 + cpw);
  v4f tot[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) tot[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  const NibK nk = nib_consts();
  static_assert(!XF || (ONE && !CONV), "f32 activations: the single-token instance without the conv epilogue");
  const AopRsrc ar = aop_rsrc(aop, m.cols, R, lane);
  const float* xf = (const float*)aop;
  auto get_a = [&](int c, ABuf& b) { if constexpr (XF) load_a_x(xf, c, lane, b); else if constexpr (SQ) load_a_sq(ar, ainv, ep.sq_heads, ep.sq_eps, R, c, lane, b); else load_a<SC>(ar, ainv, R, c, lane, b); };
  WBuf<4> w0; ABuf a0;
  if (c0 < c1) { get_a(c0, a0); load_w<4>(m, tile * 4, c0, lane, K128, w0); }
  // conv epilogue: wave 0 fetches its rows' taps and state now, behind the weights, so the loads overlap the products
  float cw[CONV ? 8 : 1], chist[CONV ? 8 : 1]; const bool conv_row = CONV && wave == 0 && tile * 64 + lane < ep.ch;
  if constexpr (CONV) if (conv_row) {
    const size_t row = (size_t)tile * 64 + lane;
#pragma unroll
    for (int k = 0; k < 8; ++k) { cw[k] = k < kk ? ep.conv_w[row * kk + k] : 0.0f; chist[k] = k < kk - 1 ? ep.conv_in[(size_t)k * ep.ch + row] : 0.0f; }
  }
  PYRE_TS(1);
  if constexpr (NW == 16) {                   // sixteen waves: one or two chunks a wave and 128 registers a lane: one buffer, no look-ahead
    for (int c = c0; c < c1; ++c) {
      if (c > c0) { get_a(c, a0); load_w<4>(m, tile * 4, c, lane, K128, w0); }
      chunk_mac<4>(w0, a0, c, nk, tot);
    }
  } else {                                    // two buffers taking turns (a copy from one to the other would wait for the loads just issued)
    WBuf<4> w1; ABuf a1;
    for (int c = c0; c < c1; c += 2) {
      if (c + 1 < c1) { get_a(c + 1, a1); load_w<4>(m, tile * 4, c + 1, lane, K128, w1); }
      __builtin_amdgcn_sched_barrier(0);      // (keeps the compiler from sinking the loads down to their first use)
      chunk_mac<4>(w0, a0, c, nk, tot);
      __builtin_amdgcn_sched_barrier(0);
      if (c + 2 < c1) { get_a(c + 2, a0); load_w<4>(m, tile * 4, c + 2, lane, K128, w0); }
      __builtin_amdgcn_sched_barrier(0);
      if (c + 1 < c1) chunk_mac<4>(w1, a1, c + 1, nk, tot);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  PYRE_TS(2);
  // lane (q, j) holds, for row group g, token 2q (rows 0, 1 of its four) and token 2q + 1 (rows 2, 3): halves h1, h2 * 2^11
#pragma unroll
  for (int g = 0; g < 4; ++g) { red[wave][g][0][lane] = tot[g][0] + tot[g][1] * (1.0f / 2048.0f); red[wave][g][1][lane] = tot[g][2] + tot[g][3] * (1.0f / 2048.0f); }
  lds_barrier(); PYRE_TS(3);
  auto rsum = [&](int t, int rl) { const int l = (t >> 1) * 16 + (rl & 15), g = rl >> 4, h = t & 1; float s = red[0][g][h][l];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][g][h][l];
    return s; };
  const size_t r64 = (size_t)m.tiles * 64;
  for (int i = threadIdx.x; i < T * 64; i += NW * 64) {
    const int t = i >> 6, l = i & 63; const float s = rsum(t, l);
    const size_t row = (size_t)tile * 64 + l;
    if (ksplit == 1) { if (row < (size_t)m.rows) y[(size_t)t * m.rows + row] = s; }
    else y[((size_t)ks * T + t) * r64 + row] = s;
    if (T == 1 && ep.best != nullptr) {       // threads 0..63 = wave 0: first maximum of the tile (sampler::argmax order)
      float bv = row < (size_t)m.rows ? s : -INFINITY; uint32_t bi = (uint32_t)row;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) { float ov = __shfl_xor(bv, o); uint32_t oi = __shfl_xor(bi, o); if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; } }
      if (l == 0) { ep.best[2 * tile] = __float_as_uint(bv); ep.best[2 * tile + 1] = bi; }
    }
  }
  if constexpr (CONV) if (conv_row) {
    const size_t row = (size_t)tile * 64 + lane;
    for (int t = 0; t < T; ++t) {
      const float cur = rsum(t, lane);
      float o = 0.0f;
#pragma unroll
      for (int k = 0; k < 8; ++k) if (k == kk - 1) o = cw[k] * cur;
#pragma unroll
      for (int k = 0; k < 7; ++k) if (k < kk - 1) o += cw[k] * chist[k];
      ep.co[(size_t)t * ep.ch + row] = o * (1.0f / (1.0f + expf(-o)));
#pragma unroll
      for (int k = 0; k < 7; ++k) if (k + 1 < kk - 1) chist[k] = chist[k + 1];
#pragma unroll
      for (int k = 0; k < 7; ++k) if (k == kk - 2) chist[k] = cur;
    }
#pragma unroll
    for (int k = 0; k < 7; ++k) if (k < kk - 1) ep.conv_out[(size_t)k * ep.ch + row] = chist[k];
  }
  PYRE_TS(4); PYRE_TS_FLUSH(gemm_ts, (NW == 16 ? 0 : (gridDim.y > 1 ? 8 : 16)));
}

namespace {
int env_i(const char* n, int dflt) { const char* v = getenv(n); return v && *v ? atoi(v) : dflt; }
int gemm_m_nw(const QMatDev& m, int ksplit) {
  static const int force = env_i("PYRE_GEMM_M_NW", 0);
  const int per_wg = ((m.cols >> 7) + ksplit - 1) / ksplit;
  int nw = m.tiles >= 1024 ? 4 : (m.tiles >= 256 ? 8 : 16);
  while (nw > 1 && nw / 2 >= per_wg) nw /= 2;          // no idle waves
  if (nw < 4) nw = 4;
  if (force == 4 || force == 8 || force == 16) nw = force;
  return nw;
}
template <int NW> void gemm_m_go(pyre_ctx* ctx, const QMatDev& m, const PyreAop& a, int t, float* y, int ksplit, int cpw, const GemvEpi& ep, const float* xf = nullptr) {
  if (xf) { hipLaunchKernelGGL((k_gemm_m<NW, true, false, 1, true>), dim3(m.tiles, ksplit, ctx->batch_n), dim3(NW * 64), 0, ctx->stream, m, (const uint4*)xf, (const float*)nullptr, y, 1, 2, cpw, ep, ctx->batch_stride); return; }
#define GEMM_M_T(CALL) switch (t) { case 1: { constexpr int FT = 1; CALL; } break; case 2: { constexpr int FT = 2; CALL; } break; case 3: { constexpr int FT = 3; CALL; } break; case 4: { constexpr int FT = 4; CALL; } break; \
    case 5: { constexpr int FT = 5; CALL; } break; case 6: { constexpr int FT = 6; CALL; } break; case 7: { constexpr int FT = 7; CALL; } break; default: { constexpr int FT = 8; CALL; } break; }
  if (a.sq) {          // (the launcher has checked: no conv epilogue, chunks = heads)
    GemvEpi e2 = ep; e2.sq_heads = a.sq_heads; e2.sq_eps = a.sq_eps;
    GEMM_M_T(hipLaunchKernelGGL((k_gemm_m<NW, true, false, FT, false, true>), dim3(m.tiles, ksplit, ctx->batch_n), dim3(NW * 64), 0, ctx->stream, m, a.op, a.sq, y, t, pyre_aop_rows(t), cpw, e2, ctx->batch_stride));
    return;
  }
#define GEMM_M_GO(SC, CONV) hipLaunchKernelGGL((k_gemm_m<NW, SC, CONV, 0>), dim3(m.tiles, ksplit, ctx->batch_n), dim3(NW * 64), 0, ctx->stream, m, a.op, a.ainv, y, t, pyre_aop_rows(t), cpw, ep, ctx->batch_stride)
  if (a.ainv && (!ep.co || ep.kk == 4)) {          // scaled operand rows (every launch of the model and of the operator): the instance with the window width folded in
    if (ep.co) { GEMM_M_T(hipLaunchKernelGGL((k_gemm_m<NW, true, true, FT>), dim3(m.tiles, ksplit, ctx->batch_n), dim3(NW * 64), 0, ctx->stream, m, a.op, a.ainv, y, t, pyre_aop_rows(t), cpw, ep, ctx->batch_stride)); }
    else { GEMM_M_T(hipLaunchKernelGGL((k_gemm_m<NW, true, false, FT>), dim3(m.tiles, ksplit, ctx->batch_n), dim3(NW * 64), 0, ctx->stream, m, a.op, a.ainv, y, t, pyre_aop_rows(t), cpw, ep, ctx->batch_stride)); }
  }
  else if (ep.co) { if (a.ainv) GEMM_M_GO(true, true); else GEMM_M_GO(false, true); }
  else { if (a.ainv) GEMM_M_GO(true, false); else GEMM_M_GO(false, false); }
#undef GEMM_M_T
#undef GEMM_M_GO
}
}  // namespace

void pyre_gemm_m_plan(const QMatDev& m, int ksplit, int* nw, int* cpw) {
  *nw = gemm_m_nw(m, ksplit);
  const int per_wg = ((m.cols >> 7) + ksplit - 1) / ksplit; *cpw = (per_wg + *nw - 1) / *nw; if (*cpw < 1) *cpw = 1;
}

int pyre_gemm_m_best_count(const QMatDev& m) { return m.tiles; }

bool pyre_gemm_m_x_ok(const QMatDev& m, int t, const GemvEpi& ep) {
  static const bool off = env_i("PYRE_GEMM_M_X", 1) == 0;
  return !off && t == 1 && !ep.co && m.tiles <= 128;
}
int pyre_gemm_m_launch(pyre_ctx* ctx, const QMatDev& m, const PyreAop& a, int t, float* y, int ksplit, const GemvEpi& ep, const float* xf) {
  if (m.fmt != FMT_IQ3_S_M || !m.mq || !m.mh) return pyre_fail(ctx, PYRE_E_TYPE, "gemm_m: the matrix is not held in the matrix-core layout");
  if (xf && !pyre_gemm_m_x_ok(m, t, ep)) return pyre_fail(ctx, PYRE_E_ARG, "gemm_m: f32 activations are for a single token, no conv epilogue and at most 128 row tiles");
  if (t < 1 || t > 8 || ksplit < 1 || (!a.op && !xf) || !y) return pyre_fail(ctx, PYRE_E_ARG, "gemm_m: t = %d, %d K slices", t, ksplit);
  if (a.sq && (ep.co || xf || a.sq_heads * 128 != m.cols)) return pyre_fail(ctx, PYRE_E_ARG, "gemm_m: per-quarter scales need %d heads of 128 columns and no conv epilogue", a.sq_heads);
  if (m.cols % 256 != 0 || m.SB != m.cols / 256) return pyre_fail(ctx, PYRE_E_SHAPE, "gemm_m: %d columns", m.cols);
  int nw, cpw; pyre_gemm_m_plan(m, ksplit, &nw, &cpw);
  if (ep.four_waves) { nw = 4; const int per_wg = ((m.cols >> 7) + ksplit - 1) / ksplit; cpw = (per_wg + 3) / 4; }
  static const std::string names[9] = {"", "gemm_m_iq3s_t1", "gemm_m_iq3s_t2", "gemm_m_iq3s_t3", "gemm_m_iq3s_t4", "gemm_m_iq3s_t5", "gemm_m_iq3s_t6", "gemm_m_iq3s_t7", "gemm_m_iq3s_t8"};
  ProfScope ps(ctx, names[t].c_str(), qmat_gguf_bytes(m, m.rows) + 4.0 * t * ((double)m.cols + m.rows));
  if (nw == 4) gemm_m_go<4>(ctx, m, a, t, y, ksplit, cpw, ep, xf);
  else if (nw == 8) gemm_m_go<8>(ctx, m, a, t, y, ksplit, cpw, ep, xf);
  else gemm_m_go<16>(ctx, m, a, t, y, ksplit, cpw, ep, xf);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

// ---- operand scratch: the context's grow-only buffer, and the fixed per-GPU array -------------------------------------------------
int pyre_gemm_m_scratch(pyre_ctx* ctx, int cols, uint4** op, float** ainv) {
  const size_t ob = (pyre_aop_bytes(cols, 8) + 255) & ~(size_t)255, need = ob + (size_t)(cols / 256) * 8 * 4;
  if (ctx->aop_bytes < need) {
    PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (ctx->aop_buf) (void)hipFree(ctx->aop_buf);
    ctx->aop_buf = nullptr; ctx->aop_bytes = 0;
    PYRE_HIP(ctx, hipMalloc(&ctx->aop_buf, need)); ctx->aop_bytes = need;
  }
  *op = (uint4*)ctx->aop_buf; *ainv = (float*)((uint8_t*)ctx->aop_buf + ob);
  return PYRE_OK;
}

// The entry point that allocates nothing keeps its operand here: PYRE_QMATMUL_STATIC_MAX_COLS columns of operand rows
// (32 bytes a column) and their scale factors.  One copy per GPU, held until the process ends; calls on one GPU share it.
#define STATIC_MAX_COLS 32768
#define STATIC_OP_BYTES ((size_t)STATIC_MAX_COLS * 32)
static __device__ __align__(256) uint8_t scratch[STATIC_OP_BYTES + (STATIC_MAX_COLS / 256) * 8 * 4 + 256 + (STATIC_MAX_COLS / 32) * 8 * 4];      // (operand rows, scale factors; a Q4_K window's sub-block sums)
static void* g_scratch_ptr[64];
static std::mutex g_scratch_mu;          // contexts may be created from several threads

int pyre_static_init(pyre_ctx* ctx) {
  if (ctx->device < 0 || ctx->device >= 64) return pyre_fail(ctx, PYRE_E_ARG, "device %d outside 0..63", ctx->device);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[ctx->device]) {
    void* p = nullptr;
    PYRE_HIP(ctx, hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[ctx->device] = p;
  }
  ctx->aop_static = g_scratch_ptr[ctx->device];
  return PYRE_OK;
}

int pyre_gemm_m_static(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev) {
  if (m.cols > STATIC_MAX_COLS) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmatmul_static_dev: %d columns exceed the static scratch of %d columns; use pyre_qmatmul_dev", m.cols, STATIC_MAX_COLS);
  if (!ctx->aop_static) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the device array was not resolved at context creation");
  uint4* op = (uint4*)ctx->aop_static; float* ainv = (float*)((uint8_t*)ctx->aop_static + STATIC_OP_BYTES);
  int rc = pyre_act_split_launch(ctx, x_dev, t, m.cols, op, ainv); if (rc) return rc;
  return pyre_gemm_m_launch(ctx, m, PyreAop{op, ainv}, t, y_dev, 1, GemvEpi{});
}
