// IQ3_S dequant-GEMV at the file's bits per weight, single token (QMat::matmul with t = 1, src/model/gguf_q.rs:217-242;
// the GPU decode of this type in the reference: src/model/qn_cube.rs:3354-3382).
//
// The matrix-core layout (gemm_m.hip) holds an IQ3_S weight as a resolved 4-bit code: 4.25 bit/weight against the file's
// 3.4375, so a GEMV that is bound by bytes streams 1.24 x what the file holds.  Here a matrix keeps what the file keeps --
// per four weights the 9-bit codebook index and the four sign bits, per 32 the 4-bit scale, per 256 the f16 d -- and the
// codebook lives in shared memory with the signs folded in: 8192 entries (index | signs << 9) of four signed bytes,
// 32 KB per workgroup, filled once by a workgroup that then walks row tiles.
//   layout: per row and 256-column super-block 112 bytes (3.5 bit/weight: the file's 110 bytes + 2 of padding):
//           bits 13 g .. 13 g + 12 = field of group g (columns 4 g .. 4 g + 3), g < 64; bits 832 + 4 i .. = scale of
//           sub-block i; bits 864 .. 879 = d; as seven 16-byte pieces, nq[tile][super-block][piece][lane] with lane = row of
//           the tile, so a wave fetches every piece with one coalesced load.
//   activations: block fixed point as three signed bytes per value, one power of two per 64 columns
//           (x = su * q, |q| <= 2^21, q = a1 * 65536 + a2 * 256 + a3), laid out per group so that the lookups' bytes meet
//           their columns' digits in v_dot4_i32_i8; they are wave-uniform, i.e. scalar loads.
//   per four weights: two instructions for the table offset (a 32-bit window of the packed fields, a mask), one shared-memory
//           read, three dot instructions; per 32 weights the three digit sums are joined in int32 (exact), converted once and
//           scaled by d * (1 + 2 s) * su in f32.
// The only rounding beyond the f32 path's is the representation of x: |x - su q| <= 2^-22 of the 64 columns' largest
// magnitude.  t >= 2 stays on the matrix cores, where a window costs what a token does.
#include "formats.h"
#include "iq_codebooks.h"

#define DGN_STRIDE 64      // dwords per 64-column unit: 48 digit words [(sub-block*8 + group)*3 + digit], then su, pad

// ---- the matrix: raw GGUF rows -> nq; one thread per (padded row, super-block) ---------------------------------------------
__global__ __launch_bounds__(256) void k_repack_n(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, uint4* __restrict__ nq) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB) return;
  const int row = (int)(idx / SB), sb = (int)(idx % SB); const bool live = row < rows;      // padding rows lie past the end of the raw buffer: never read them
  uint32_t w[28];
  for (int i = 0; i < 28; ++i) w[i] = 0;
  if (live) {
    const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 110;
    auto put = [&](int bit, uint32_t val, int nbits) { w[bit >> 5] |= val << (bit & 31); if ((bit & 31) + nbits > 32) w[(bit >> 5) + 1] |= val >> (32 - (bit & 31)); };
    for (int ib = 0; ib < 8; ++ib) {               // gguf_q.rs:141-151: index = qs | ninth bit from qh, sign bits from the signs bytes
      const uint32_t h = b[66 + ib];
      for (int l = 0; l < 4; ++l) {
        const uint32_t sg = b[74 + 4 * ib + l];
        const uint32_t fa = (uint32_t)b[2 + 8 * ib + 2 * l] | (((h >> (2 * l)) & 1u) << 8) | ((sg & 0xFu) << 9);
        const uint32_t fb = (uint32_t)b[2 + 8 * ib + 2 * l + 1] | (((h >> (2 * l + 1)) & 1u) << 8) | ((sg >> 4) << 9);
        put(13 * (8 * ib + 2 * l), fa, 13); put(13 * (8 * ib + 2 * l + 1), fb, 13);
      }
    }
    w[26] = (uint32_t)b[106] | ((uint32_t)b[107] << 8) | ((uint32_t)b[108] << 16) | ((uint32_t)b[109] << 24);
    w[27] = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
  }
  const size_t tile = (size_t)(row >> 6); const int lane = row & 63;
  for (int p = 0; p < 7; ++p) nq[((tile * SB + sb) * 7 + p) * 64 + lane] = make_uint4(w[4 * p], w[4 * p + 1], w[4 * p + 2], w[4 * p + 3]);
}

// ---- activation digits: grid = 64-column units, one wave per unit -------------------------------------------------------------
__global__ __launch_bounds__(64) void k_act_digits_n(const float* __restrict__ x, uint32_t* __restrict__ dg) {
  __shared__ __align__(16) uint8_t sm[3][64];
  const int ku = blockIdx.x, lane = threadIdx.x;
  const float v = x[(size_t)ku * 64 + lane];
  float mx = fabsf(v);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  const bool fin = __all(isfinite(v));
  float su = 0.0f; int q = 0;
  if (!fin) su = __uint_as_float(0x7FC00000u);            // a non-finite activation makes the unit's contribution NaN
  else if (mx > 0.0f) {
    int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 126; if (e < -100) e = -100;      // mx < 2^e (subnormal maxima take the clamp)
    su = __uint_as_float((uint32_t)(e - 21 + 127) << 23); q = (int)rintf(v * __uint_as_float((uint32_t)(21 - e + 127) << 23));      // |q| <= 2^21
  }
  const int a3 = (int)(int8_t)(q & 0xFF), q1 = (q - a3) >> 8, a2 = (int)(int8_t)(q1 & 0xFF), a1 = (q1 - a2) >> 8;
  sm[0][lane] = (uint8_t)a1; sm[1][lane] = (uint8_t)a2; sm[2][lane] = (uint8_t)a3;      // byte b of group g = column 4 g + b
  __builtin_amdgcn_wave_barrier();      // one wave: its shared-memory operations execute in order
  uint32_t* o = dg + (size_t)ku * DGN_STRIDE;
  if (lane < 48) o[lane] = ((const uint32_t*)sm[lane % 3])[lane / 3];
  else if (lane == 48) o[48] = __float_as_uint(su);
}

// byte offset into the table of group G's entry: the 13-bit field at bit 13 G of the 28 words, times four
template <int G> __device__ __forceinline__ uint32_t n_off(const uint32_t (&w)[28]) {
  constexpr int bit = 13 * G - 2;                   // the window starts two bits below the field
  if constexpr (bit < 0) return (w[0] << 2) & 0x7FFCu;
  else {
    constexpr int wi = bit >> 5, sh = bit & 31;
    if constexpr (sh + 15 <= 32) return (w[wi] >> sh) & 0x7FFCu;
    else return __builtin_amdgcn_alignbit(w[wi + 1], w[wi], sh) & 0x7FFCu;
  }
}
// sub-block IB (32 weights) of the super-block held in w against its digits at p (uniform address): the three digit sums
template <int IB, int L> __device__ __forceinline__ void n_group(const uint32_t (&w)[28], const uint8_t* lt, const uint32_t* __restrict__ p, int& i1, int& i2, int& i3) {
  if constexpr (L < 8) {
#ifdef GEMV_N_NOLDS      // diagnostics: the table offset itself in place of the table's entry (no shared-memory read)
    const int e = (int)n_off<IB * 8 + L>(w);
#else
    const int e = (int)*(const uint32_t*)(lt + n_off<IB * 8 + L>(w));
#endif
    i1 = __builtin_amdgcn_sdot4(e, (int)p[L * 3 + 0], i1, false); i2 = __builtin_amdgcn_sdot4(e, (int)p[L * 3 + 1], i2, false); i3 = __builtin_amdgcn_sdot4(e, (int)p[L * 3 + 2], i3, false);
    n_group<IB, L + 1>(w, lt, p, i1, i2, i3);
  }
}
template <int IB> __device__ __forceinline__ float n_subblock(const uint32_t (&w)[28], const uint8_t* lt, const uint32_t* __restrict__ dgs, float dsu, float acc) {
  int i1 = 0, i2 = 0, i3 = 0;
  n_group<IB, 0>(w, lt, dgs + (IB & 1) * 24, i1, i2, i3);
  const int t = (int)(((uint32_t)i1 << 16) + ((uint32_t)i2 << 8) + (uint32_t)i3);          // |t| < 2^31: |i1| <= 32 * 15 * 33
  const float s = (float)(1 + 2 * (int)((w[26] >> (4 * IB)) & 0xFu));
  return fmaf(dsu * s, (float)t, acc);
}
// one super-block (256 columns) of the lane's row; dg = the digits of its four units
__device__ __forceinline__ float n_superblock(const uint4 (&r)[7], const uint8_t* lt, const uint32_t* __restrict__ dg, float acc) {
#ifdef GEMV_N_NOMATH      // diagnostics: the loads alone
  uint32_t u = 0;
#pragma unroll
  for (int p = 0; p < 7; ++p) u ^= r[p].x ^ r[p].y ^ r[p].z ^ r[p].w;
  return acc + __uint_as_float(u & 0xFFu);
#endif
  const uint32_t w[28] = {r[0].x, r[0].y, r[0].z, r[0].w, r[1].x, r[1].y, r[1].z, r[1].w, r[2].x, r[2].y, r[2].z, r[2].w, r[3].x, r[3].y, r[3].z, r[3].w,
                          r[4].x, r[4].y, r[4].z, r[4].w, r[5].x, r[5].y, r[5].z, r[5].w, r[6].x, r[6].y, r[6].z, r[6].w};
  const float d = h2f_bits(w[27] & 0xFFFFu);
  { const float dsu = d * __uint_as_float(dg[0 * DGN_STRIDE + 48]); acc = n_subblock<0>(w, lt, dg + 0 * DGN_STRIDE, dsu, acc); acc = n_subblock<1>(w, lt, dg + 0 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[1 * DGN_STRIDE + 48]); acc = n_subblock<2>(w, lt, dg + 1 * DGN_STRIDE, dsu, acc); acc = n_subblock<3>(w, lt, dg + 1 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[2 * DGN_STRIDE + 48]); acc = n_subblock<4>(w, lt, dg + 2 * DGN_STRIDE, dsu, acc); acc = n_subblock<5>(w, lt, dg + 2 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[3 * DGN_STRIDE + 48]); acc = n_subblock<6>(w, lt, dg + 3 * DGN_STRIDE, dsu, acc); acc = n_subblock<7>(w, lt, dg + 3 * DGN_STRIDE, dsu, acc); }
  return acc;
}

// grid = min(tiles, what the chip holds at once), NW waves; the workgroup fills its table, then takes row tiles
// blockIdx.x, + gridDim.x, ..; wave w walks super-blocks [w * spw, + spw) of the tile, lane l owns row tile * 64 + l; the
// waves' sums meet in shared memory in wave order.  The next super-block's seven pieces are requested before the current
// one's arithmetic starts.
template <int NW> __global__ __launch_bounds__(NW * 64) void k_gemv_n(const uint4* __restrict__ nq, int rows, int tiles, int SB, const uint4* __restrict__ tab, const uint32_t* __restrict__ dg, float* __restrict__ y, int spw) {
  __shared__ __align__(16) uint8_t lt[8192 * 4];
  __shared__ float red[NW][64];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  for (int i = tid; i < 2048; i += NW * 64) ((uint4*)lt)[i] = tab[i];
  __syncthreads();
  const int s0 = min(SB, wave * spw), s1 = min(SB, s0 + spw);
  uint4 bufa[7], bufb[7];
  const size_t tstride = (size_t)SB * 7 * 64;
  if (s0 < s1 && (int)blockIdx.x < tiles) {
#pragma unroll
    for (int p = 0; p < 7; ++p) bufa[p] = nq[(size_t)blockIdx.x * tstride + ((size_t)s0 * 7 + p) * 64 + lane];
  }
  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    float acc = 0.0f;
    if (s0 < s1) {
      const uint4* base = nq + (size_t)tile * tstride + lane;
      const int tn = tile + (int)gridDim.x < tiles ? tile + (int)gridDim.x : tile;          // the wave's first super-block of the next tile follows its last of this one
      const uint4* nbase = nq + (size_t)tn * tstride + lane;
      for (int sb = s0; sb < s1; sb += 2) {          // two buffers taking turns (a copy from one to the other would cost 28 moves a super-block)
        const bool last1 = sb + 1 >= s1, last2 = sb + 2 >= s1;
        const uint4* b1 = last1 ? nbase + (size_t)s0 * 7 * 64 : base + (size_t)(sb + 1) * 7 * 64;
#pragma unroll
        for (int p = 0; p < 7; ++p) bufb[p] = b1[(size_t)p * 64];
        acc = n_superblock(bufa, lt, dg + (size_t)sb * 4 * DGN_STRIDE, acc);
        if (last1) {
#pragma unroll
          for (int p = 0; p < 7; ++p) bufa[p] = bufb[p];          // (an odd count of super-blocks a wave: the prefetched one is the next tile's first)
        } else {
          const uint4* b2 = last2 ? nbase + (size_t)s0 * 7 * 64 : base + (size_t)(sb + 2) * 7 * 64;
#pragma unroll
          for (int p = 0; p < 7; ++p) bufa[p] = b2[(size_t)p * 64];
          acc = n_superblock(bufb, lt, dg + (size_t)(sb + 1) * 4 * DGN_STRIDE, acc);
        }
      }
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (tid < 64) {
      float s = red[0][lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) s += red[w][lane];
      const size_t row = (size_t)tile * 64 + lane;
      if (row < (size_t)rows) y[row] = s;
    }
    __syncthreads();
  }
}

namespace {
int env_i(const char* n, int dflt) { const char* s = getenv(n); return s && *s ? atoi(s) : dflt; }
}

size_t pyre_gemv_n_bytes(size_t rows, size_t cols) { return ((rows + 63) / 64) * 64 * (cols / 256) * 112; }

int pyre_gemv_n_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* nq_dev) {
  const int SB = (int)(cols / 256); const size_t rows_pad = (rows + 63) / 64 * 64, total = rows_pad * SB;
  hipLaunchKernelGGL(k_repack_n, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, raw_dev, row_bytes, (uint4*)nq_dev);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

// the table: entry (index | signs << 9) = the four codebook values of `index`, value j negated where sign bit j is set
int pyre_gemv_n_table(pyre_ctx* ctx) {
  if (ctx->d_iq3s_sgn) return PYRE_OK;
  std::vector<uint32_t> t(8192);
  for (int i = 0; i < 8192; ++i) {
    uint32_t v = 0;
    for (int j = 0; j < 4; ++j) { const int g = 2 * ((kIq3sCode[i & 511] >> (3 * j)) & 7) + 1; const int s = ((i >> (9 + j)) & 1) ? -g : g; v |= (uint32_t)(uint8_t)(int8_t)s << (8 * j); }
    t[i] = v;
  }
  PYRE_HIP(ctx, hipMalloc((void**)&ctx->d_iq3s_sgn, 8192 * 4));
  PYRE_HIP(ctx, hipMemcpyAsync(ctx->d_iq3s_sgn, t.data(), 8192 * 4, hipMemcpyHostToDevice, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return PYRE_OK;
}

size_t pyre_gemv_n_digit_bytes(size_t cols) { return cols / 64 * DGN_STRIDE * 4; }

// digits: where the activation digits go (pyre_gemv_n_digit_bytes(cols) bytes); null = the context's grow-only buffer
int pyre_gemv_n_launch(pyre_ctx* ctx, const void* nq, size_t rows, size_t cols, const float* x_dev, float* y_dev, void* digits) {
  if (cols % 256) return pyre_fail(ctx, PYRE_E_SHAPE, "gemv_n: %zu columns are not whole super-blocks", cols);
  if (!ctx->d_iq3s_sgn) return pyre_fail(ctx, PYRE_E_HIP, "gemv_n: the codebook table was not made at context creation");
  const int U = (int)(cols / 64), SB = (int)(cols / 256), tiles = (int)((rows + 63) / 64);
  const size_t need = pyre_gemv_n_digit_bytes(cols);
  if (!digits && ctx->dgn_bytes < need) {
    if (ctx->dgn_buf) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(ctx->dgn_buf)); ctx->dgn_buf = nullptr; ctx->dgn_bytes = 0; }
    PYRE_HIP(ctx, hipMalloc(&ctx->dgn_buf, need)); ctx->dgn_bytes = need;
  }
  uint32_t* dg = (uint32_t*)(digits ? digits : ctx->dgn_buf);
  { ProfScope ps(ctx, "gemv_n_digits", 4.0 * cols * 2);
    hipLaunchKernelGGL(k_act_digits_n, dim3(U), dim3(64), 0, ctx->stream, x_dev, dg); } PYRE_CHECK_LAUNCH(ctx);
  static const int fnw = env_i("PYRE_GEMV_N_NW", 0), fwg = env_i("PYRE_GEMV_N_WGS", 0);
  // eight waves a row tile when the rows are long enough (one or two super-blocks a wave), two such workgroups a compute unit:
  // measured on the 151936 x 2048 head, 31.7 us against 34.2 with four waves and four workgroups
  int nw = SB >= 8 ? 8 : (SB >= 4 ? 4 : (SB >= 2 ? 2 : 1)); if (fnw == 1 || fnw == 2 || fnw == 4 || fnw == 8) nw = fnw;
  if (nw > SB) nw = SB >= 8 ? 8 : (SB >= 4 ? 4 : (SB >= 2 ? 2 : 1));
  const int spw = (SB + nw - 1) / nw;
  const int per_cu = 16 / nw > 4 ? 4 : 16 / nw;          // 32 KB of table per workgroup: at most four on a compute unit
  int grid = fwg > 0 ? fwg : 256 * per_cu;
  static const int fgrid = env_i("PYRE_GEMV_N_GRID", 0); if (fgrid > 0) grid = fgrid;
  if (grid > tiles) grid = tiles;
  { ProfScope ps(ctx, "gemv_n_iq3_s_t1", (double)rows * (cols / 256) * 110 + 4.0 * ((double)cols + rows));
    const uint4* q = (const uint4*)nq; const uint4* tb = (const uint4*)ctx->d_iq3s_sgn;
    switch (nw) {
      case 1: hipLaunchKernelGGL((k_gemv_n<1>), dim3(grid), dim3(64), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      case 2: hipLaunchKernelGGL((k_gemv_n<2>), dim3(grid), dim3(128), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      case 8: hipLaunchKernelGGL((k_gemv_n<8>), dim3(grid), dim3(512), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      default: hipLaunchKernelGGL((k_gemv_n<4>), dim3(grid), dim3(256), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
    } }
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
