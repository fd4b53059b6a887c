// Batch 2..8 verify GEMM for IQ3_S matrices on the matrix cores (opt-in: the single-token GEMV and the default verify
// path are bit-identical per token, this one agrees with them to ~1e-7 relative, not bit for bit).
//
// The weights already sit one row per lane with 64 consecutive columns per unit (formats.h), which is exactly the
// operand layout of v_mfma_f32_4x4x4_16B_f16: sixteen independent 4x4x4 products per instruction, block b = lane / 4,
// lane 4b+i supplies row i of A (four consecutive k), lane 4b+j supplies column j of B and receives column j of D
// (rows in its four result registers).  So A = four re-coded weights of the lane's own row, B = four activations of
// token j (the same for all sixteen blocks), D = the 64 rows x 4 tokens partial products; tokens 4..7 take a second
// instruction with another B.
//
// Exactness: a 4-bit code c (w = 2c - 15) becomes the half 16 + c by or-ing c into the mantissa of 16.0 (one and-or per
// two weights); an activation is split into two halves x = h1 + h2 (22 mantissa bits, after an exact power-of-two
// scaling of the token to max |x| <= 1024), so every product is exact in f32 and
//   sum w x = 2 * (sum (16 + c)(h1 + h2)) - 47 * sum (h1 + h2)        per 32-value sub-block,
// then times the sub-block scale d * (1 + 2 s), exactly as the VALU path factors it.
#include "formats.h"

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// ---- activation prologue: one workgroup -------------------------------------------------------------------------------
// xb[((ku*16 + g)*2 + s)*8 + t] = four halves of split term s of token t for MFMA group g of unit ku, in the k order the
// weight unpacking produces: group g = 2*word + h covers columns 8*word + {0,4,1,5} (h = 0) or {2,6,3,7} (h = 1).
// sx[(ku*2 + blk)*8 + t] = sum over the sub-block of (h1 + h2);  xscale[t] = the power of two the token was scaled by.
__global__ __launch_bounds__(1024) void k_xsplit(const float* __restrict__ x, int T, int cols, uint2* __restrict__ xb, float* __restrict__ sx, float* __restrict__ xscale) {
  __shared__ float wmax[16]; __shared__ float scale[8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int t = 0; t < 8; ++t) {
    float mx = 0.0f;
    if (t < T) for (int i = tid; i < cols; i += 1024) mx = fmaxf(mx, fabsf(x[(size_t)t * cols + i]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if (lane == 0) wmax[wave] = mx;
    __syncthreads();
    if (tid == 0) {
      float m = 0.0f; for (int w = 0; w < 16; ++w) m = fmaxf(m, wmax[w]);
      int e = 0; float sc = 1.0f;
      if (m > 0.0f && isfinite(m)) { (void)frexpf(m, &e); sc = ldexpf(1.0f, 10 - e); }      // m * sc in [512, 1024)
      scale[t] = sc; xscale[t] = sc;
    }
    __syncthreads();
  }
  const int U = cols >> 6;
  // one thread per (unit, group, token)
  for (int idx = tid; idx < U * 16 * 8; idx += 1024) {
    const int t = idx & 7, g = (idx >> 3) & 15, ku = idx >> 7, word = g >> 1, h = g & 1;
    const int kk[4] = {h ? 2 : 0, h ? 6 : 4, h ? 3 : 1, h ? 7 : 5};
    uint32_t hi[2] = {0, 0}, lo[2] = {0, 0};
    if (t < T) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = x[(size_t)t * cols + (size_t)ku * 64 + 8 * word + kk[e]] * scale[t];
        _Float16 h1 = (_Float16)v; _Float16 h2 = (_Float16)(v - (float)h1);
        hi[e >> 1] |= (uint32_t)__builtin_bit_cast(unsigned short, h1) << (16 * (e & 1));
        lo[e >> 1] |= (uint32_t)__builtin_bit_cast(unsigned short, h2) << (16 * (e & 1));
      }
    }
    xb[((size_t)(ku * 16 + g) * 2 + 0) * 8 + t] = uint2{hi[0], hi[1]};
    xb[((size_t)(ku * 16 + g) * 2 + 1) * 8 + t] = uint2{lo[0], lo[1]};
  }
  // sub-block sums of the split representation, columns in ascending order
  for (int idx = tid; idx < U * 2 * 8; idx += 1024) {
    const int t = idx & 7, blk = (idx >> 3) & 1, ku = idx >> 4;
    float s = 0.0f;
    if (t < T) for (int j = 0; j < 32; ++j) {
      float v = x[(size_t)t * cols + (size_t)ku * 64 + 32 * blk + j] * scale[t];
      _Float16 h1 = (_Float16)v; _Float16 h2 = (_Float16)(v - (float)h1);
      s += (float)h1 + (float)h2;
    }
    sx[idx] = s;
  }
}

__device__ __forceinline__ half4_t as_half4(uint32_t a, uint32_t b) { uint2 u{a, b}; return __builtin_bit_cast(half4_t, u); }

// ---- the GEMM: grid ceil(tiles / TB), 8 waves.  Wave w walks units w, w + 8, ... for the workgroup's TB row tiles ------
// The activation operands of one 32-value sub-block stay in registers while the wave goes over its TB tiles, so they
// are fetched once per TB tiles.
template <int HALVES, int TB>
__global__ __launch_bounds__(512) void k_gemm_mfma_iq3s(QMatDev m, const uint2* __restrict__ xb, const float* __restrict__ sx, const float* __restrict__ xscale, float* __restrict__ y, int T) {
  __shared__ float red[8][2][HALVES][4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), tj = lane & 3;
  const int tile0 = blockIdx.x * TB;
  float4_t acc[TB][HALVES];
#pragma unroll
  for (int tl = 0; tl < TB; ++tl)
#pragma unroll
    for (int hf = 0; hf < HALVES; ++hf) acc[tl][hf] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  for (int ku = wave; ku < m.U; ku += 8) {
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      half4_t b[8][2][HALVES];
#pragma unroll
      for (int g = 0; g < 8; ++g)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int hf = 0; hf < HALVES; ++hf) { const uint2 q = xb[((size_t)(ku * 16 + 8 * blk + g) * 2 + s) * 8 + 4 * hf + tj]; b[g][s][hf] = as_half4(q.x, q.y); }
      float sxv[HALVES];
#pragma unroll
      for (int hf = 0; hf < HALVES; ++hf) sxv[hf] = sx[(size_t)(ku * 2 + blk) * 8 + 4 * hf + tj];
#pragma unroll
      for (int tl = 0; tl < TB; ++tl) {
        const int tile = min(tile0 + tl, m.tiles - 1);
        const uint4 v = ld_vec<2>(m, tile, ku, blk, lane);                      // the sub-block's four words of codes
        const float d = h2f_bits(ld_block<uint16_t>(m, tile, ku, lane)); const uint32_t sc = ld_small<uint8_t>(m.p3, m, tile, ku, lane);
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
        float4_t D[HALVES];
#pragma unroll
        for (int hf = 0; hf < HALVES; ++hf) D[hf] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            // halves 16 + c: c or-ed into the mantissa of 16.0 (0x4C00), codes {0,4 | 1,5} (h = 0) or {2,6 | 3,7} (h = 1)
            const uint32_t a0 = h == 0 ? (((u[kk] << 6) & 0x03C003C0u) | 0x4C004C00u) : (((u[kk] >> 2) & 0x03C003C0u) | 0x4C004C00u);
            const uint32_t a1 = h == 0 ? (((u[kk] << 2) & 0x03C003C0u) | 0x4C004C00u) : (((u[kk] >> 6) & 0x03C003C0u) | 0x4C004C00u);
            const half4_t A = as_half4(a0, a1);
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
              for (int hf = 0; hf < HALVES; ++hf) D[hf] = __builtin_amdgcn_mfma_f32_4x4x4f16(A, b[2 * kk + h][s][hf], D[hf], 0, 0, 0);
          }
        // sub-block scale of each of the quad's four rows, then acc += db * (2 D - 47 sum x)
        const float db = d * (float)(1 + 2 * ((sc >> (4 * blk)) & 0xF));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float dbi = __shfl(db, (lane & ~3) | i);
#pragma unroll
          for (int hf = 0; hf < HALVES; ++hf) acc[tl][hf][i] = fmaf(dbi, fmaf(-47.0f, sxv[hf], 2.0f * D[hf][i]), acc[tl][hf][i]);
        }
      }
    }
  }
#pragma unroll
  for (int tp = 0; tp < TB; tp += 2) {          // the waves' sums meet in shared memory two tiles at a time, added in wave order
#pragma unroll
    for (int tl = 0; tl < 2; ++tl)
#pragma unroll
      for (int hf = 0; hf < HALVES; ++hf)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][tl][hf][i][lane] = acc[tp + tl][hf][i];
    __syncthreads();
    for (int e = tid; e < 2 * HALVES * 4 * 64; e += 512) {
      const int l = e & 63, i = (e >> 6) & 3, hf = (e >> 8) % HALVES, tl = (e >> 8) / HALVES;
      float s = red[0][tl][hf][i][l];
#pragma unroll
      for (int w = 1; w < 8; ++w) s += red[w][tl][hf][i][l];
      const int token = 4 * hf + (l & 3); const int tile = tile0 + tp + tl; const size_t row = (size_t)tile * 64 + (l & ~3) + i;
      if (token < T && tile < m.tiles && row < (size_t)m.rows) y[(size_t)token * m.rows + row] = s / xscale[token];
    }
    __syncthreads();
  }
}

static int mfma_scratch(pyre_ctx* ctx, size_t nbytes, void** out) {
  if (nbytes > ctx->mfma_bytes) {
    if (ctx->mfma_buf) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(ctx->mfma_buf)); ctx->mfma_buf = nullptr; ctx->mfma_bytes = 0; }
    PYRE_HIP(ctx, hipMalloc(&ctx->mfma_buf, nbytes)); ctx->mfma_bytes = nbytes;
  }
  *out = ctx->mfma_buf; return PYRE_OK;
}

bool pyre_gemm_mfma_ok(const QMatDev& m, int t) { return m.fmt == FMT_IQ3_S && t >= 2 && t <= 8; }

int pyre_gemm_mfma_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y) {
  if (!pyre_gemm_mfma_ok(m, t)) return pyre_fail(ctx, PYRE_E_ARG, "verify GEMM on the matrix cores: IQ3_S and 2..8 tokens only");
  const size_t U = (size_t)m.U, nb_xb = U * 16 * 2 * 8 * sizeof(uint2), nb_sx = U * 2 * 8 * 4;
  void* buf = nullptr; int rc = mfma_scratch(ctx, nb_xb + nb_sx + 256, &buf); if (rc) return rc;
  uint2* xb = (uint2*)buf; float* sx = (float*)((uint8_t*)buf + nb_xb); float* xscale = (float*)((uint8_t*)buf + nb_xb + nb_sx);
  { ProfScope ps(ctx, "verify_xsplit", 4.0 * t * m.cols + (double)nb_xb + nb_sx);
    hipLaunchKernelGGL(k_xsplit, dim3(1), dim3(1024), 0, ctx->stream, x, t, m.cols, xb, sx, xscale); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "verify_gemm_mfma", qmat_gguf_bytes(m, m.rows) + 4.0 * t * ((double)m.cols + m.rows));
    // two tiles per workgroup: eight (activation operands fetched a quarter as often) measured slower on the 151936-row
    // head, 151 vs 117 us at t = 8 -- the kernel is bound by load latency per sub-block, not by operand fetches
    if (t <= 4) hipLaunchKernelGGL((k_gemm_mfma_iq3s<1, 2>), dim3((m.tiles + 1) / 2), dim3(512), 0, ctx->stream, m, xb, sx, xscale, y, t);
    else hipLaunchKernelGGL((k_gemm_mfma_iq3s<2, 2>), dim3((m.tiles + 1) / 2), dim3(512), 0, ctx->stream, m, xb, sx, xscale, y, t); }
  PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

extern "C" int pyre_qmatmul_mfma_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev) {
  if (!ctx || !m || !x_dev || !y_dev) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul_mfma: null argument");
  return pyre_gemm_mfma_launch(ctx, m->dv, x_dev, t, y_dev);
}
extern "C" int pyre_qmatmul_mfma(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host) {
  if (!ctx || !m || !x_host || !y_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul_mfma: null argument");
  if (!pyre_gemm_mfma_ok(m->dv, t)) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul_mfma: IQ3_S and 2..8 tokens only");
  const size_t nx = (size_t)t * m->cols * 4, ny = (size_t)t * m->rows * 4; void* st = nullptr;
  int rc = pyre_stage(ctx, nx + ny + 512, &st); if (rc) return rc;
  float* xd = (float*)st; float* yd = (float*)((uint8_t*)st + ((nx + 255) & ~(size_t)255));
  PYRE_HIP(ctx, hipMemcpyAsync(xd, x_host, nx, hipMemcpyHostToDevice, ctx->stream));
  rc = pyre_gemm_mfma_launch(ctx, m->dv, xd, t, yd); if (rc) return rc;
  PYRE_HIP(ctx, hipMemcpyAsync(y_host, yd, ny, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
