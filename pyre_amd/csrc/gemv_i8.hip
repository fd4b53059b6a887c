// IQ3_S dequant-GEMV with integer dot products (the stand-alone quantized-matmul operator, QMat::matmul,
// src/model/gguf_q.rs:217-242, t = 1..8).
//
// The f32 GEMV spends about 2.7 vector instructions per weight (nibble -> byte -> float -> fma), which on a 134 MB
// matrix is as long as streaming the bytes.  Here the activations of every 64-column unit are first written as
// block fixed point -- x = s_u * q with one power-of-two scale s_u per unit and a signed 23-bit integer q per value,
// q = a1 * 65536 + a2 * 256 + a3 in signed bytes -- and the kernel forms, per 32-value sub-block,
//     sum w q = 2 * sum c q - 15 * sum q            (w = 2c - 15, c the 4-bit code)
// with v_dot4_i32_i8 on the spread nibbles: 3 unpack + 6 dot instructions per eight weights, exact in int32, then one
// conversion per digit and the sub-block's scale d * (1 + 2 s) * s_u in f32.  The only rounding beyond the f32 path's
// is the representation of x itself: |x - s_u q| <= 2^-23 of the unit's largest magnitude.
// The per-token operation sequence does not depend on t, so a token's result is bit-identical for every window width.
#include "formats.h"

#define I8_STRIDE 64      // dwords per (token, unit): 48 digit words [(word*2 + half)*3 + digit], then s_u, -15*sum q (two sub-blocks), pad

// ---- activation digits: grid (U, t), one wave per unit --------------------------------------------------------------
__global__ __launch_bounds__(64) void k_act_digits(const float* __restrict__ x, int cols, uint32_t* __restrict__ dg) {
  __shared__ __align__(16) uint8_t sm[3][64];
  const int ku = blockIdx.x, t = blockIdx.y, U = gridDim.x, lane = threadIdx.x;
  const float v = x[(size_t)t * cols + (size_t)ku * 64 + lane];
  float mx = fabsf(v);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  const bool fin = __all(isfinite(v));
  float su = 0.0f; int q = 0;
  if (!fin) su = __uint_as_float(0x7FC00000u);            // a non-finite activation makes the unit's contribution NaN
  else if (mx > 0.0f) {
    int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 126; if (e < -100) e = -100;      // mx < 2^e (subnormal maxima take the clamp)
    su = __uint_as_float((uint32_t)(e - 22 + 127) << 23); q = (int)rintf(v * __uint_as_float((uint32_t)(22 - e + 127) << 23));      // |q| <= 2^22
  }
  const int a3 = (int)(int8_t)(q & 0xFF), q1 = (q - a3) >> 8, a2 = (int)(int8_t)(q1 & 0xFF), a1 = (q1 - a2) >> 8;
  // lane 8*word + 2*byte + half -> byte `byte` of digit word (word*2 + half): the order the spread nibbles come in
  const int pos = ((lane >> 3) * 2 + (lane & 1)) * 4 + ((lane >> 1) & 3);
  sm[0][pos] = (uint8_t)a1; sm[1][pos] = (uint8_t)a2; sm[2][pos] = (uint8_t)a3;
  int sq = q;
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
  const int sq0 = __shfl(sq, 0), sq1 = __shfl(sq, 32);
  __builtin_amdgcn_wave_barrier();      // one wave: its shared-memory operations execute in order
  uint32_t* o = dg + ((size_t)t * U + ku) * I8_STRIDE;
  if (lane < 48) o[lane] = ((const uint32_t*)sm[lane % 3])[lane / 3];
  else if (lane == 48) o[48] = __float_as_uint(su);
  else if (lane == 49) o[49] = __float_as_uint(-15.0f * (float)sq0);
  else if (lane == 50) o[50] = __float_as_uint(-15.0f * (float)sq1);
  else if (lane == 51) o[51] = 0;
}

// one unit of one token: acc += sum_j W[row, 64 ku + j] * x[64 ku + j]; p = the unit's I8_STRIDE words (uniform address)
__device__ __forceinline__ float unit_i8(const UnitRaw<FMT_IQ3_S>& r, const uint32_t* __restrict__ p, float acc) {
  const float d = h2f_bits(r.s0); const uint32_t sc = r.s1;
  const uint32_t w[8] = {r.v[0].x, r.v[0].y, r.v[0].z, r.v[0].w, r.v[1].x, r.v[1].y, r.v[1].z, r.v[1].w};
  const float su = __uint_as_float(p[48]);
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
    int i1 = 0, i2 = 0, i3 = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t u = w[4 * sb + k], lo = u & 0x0F0F0F0Fu, hi = (u >> 4) & 0x0F0F0F0Fu;
      const uint32_t* g = p + (4 * sb + k) * 6;
      i1 = __builtin_amdgcn_sdot4((int)lo, (int)g[0], i1, false); i2 = __builtin_amdgcn_sdot4((int)lo, (int)g[1], i2, false); i3 = __builtin_amdgcn_sdot4((int)lo, (int)g[2], i3, false);
      i1 = __builtin_amdgcn_sdot4((int)hi, (int)g[3], i1, false); i2 = __builtin_amdgcn_sdot4((int)hi, (int)g[4], i2, false); i3 = __builtin_amdgcn_sdot4((int)hi, (int)g[5], i3, false);
    }
    const float f = fmaf((float)i1, 65536.0f, fmaf((float)i2, 256.0f, (float)i3));
    const float db = d * (float)(1 + 2 * ((sc >> (4 * sb)) & 0xF));
    acc = fmaf(db * su, fmaf(2.0f, f, __uint_as_float(p[49 + sb])), acc);
  }
  return acc;
}

// grid (tiles), NW waves; wave w walks units [w*upw, +upw); lane l owns row tile*64 + l (the lane = row planes).
// T == 1: the digit words are wave-uniform scalar loads.  T > 1: each wave stages the T tokens' words of a unit in its
// own slice of shared memory (a wave's shared-memory operations execute in order: no workgroup barrier) and takes them
// from there; the arithmetic per token is the same.
template <int T, int NW, int UB>
__global__ __launch_bounds__(NW * 64) void k_gemv_i8(QMatDev m, const uint32_t* __restrict__ dg, float* __restrict__ y, int upw, uint32_t* __restrict__ best) {
  __shared__ float red[NW][T][64];
  __shared__ __align__(16) uint32_t xsm[T > 1 ? NW * T * I8_STRIDE : 1];
  const int tile = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int k0 = wave * upw, k1 = min(m.U, k0 + upw);
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.0f;
  // Software pipeline over batches of UB units: the next batch's weights are requested before the current batch's
  // arithmetic starts.  (A rolled loop with one batch per trip waits for its own loads first; with most workgroups
  // resident at once and in step, the chip then alternates between a memory phase and an arithmetic phase.)  The next
  // batch's first unit goes through an opaque copy so that the compiler keeps the loaded values in registers across
  // the trip instead of re-issuing the loads where they are used.
  UnitRaw<FMT_IQ3_S> cur[UB];
  if (k0 < k1) {
#pragma unroll
    for (int i = 0; i < UB; ++i) cur[i] = unit_load<FMT_IQ3_S>(m, tile, min(k0 + i, k1 - 1), lane);
  }
  for (int kb = k0; kb < k1; kb += UB) {
    int nb = kb + UB; asm volatile("" : "+s"(nb));
    UnitRaw<FMT_IQ3_S> nxt[UB];
    if (nb < k1) {
#pragma unroll
      for (int i = 0; i < UB; ++i) nxt[i] = unit_load<FMT_IQ3_S>(m, tile, min(nb + i, k1 - 1), lane);
    } else {
#pragma unroll
      for (int i = 0; i < UB; ++i) nxt[i] = cur[i];
    }
#pragma unroll
    for (int i = 0; i < UB; ++i) {
      const int ku = kb + i;
      if (ku < k1) {
        if constexpr (T == 1) {
          acc[0] = unit_i8(cur[i], dg + (size_t)ku * I8_STRIDE, acc[0]);
        } else {
          uint32_t* xw = xsm + wave * (T * I8_STRIDE);
          uint32_t xv[T];
#pragma unroll
          for (int t = 0; t < T; ++t) xv[t] = dg[((size_t)t * m.U + ku) * I8_STRIDE + lane];
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int t = 0; t < T; ++t) xw[t * I8_STRIDE + lane] = xv[t];
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int t = 0; t < T; ++t) acc[t] = unit_i8(cur[i], xw + t * I8_STRIDE, acc[t]);
          __builtin_amdgcn_wave_barrier();
        }
      }
    }
#pragma unroll
    for (int i = 0; i < UB; ++i) cur[i] = nxt[i];
  }
#pragma unroll
  for (int t = 0; t < T; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  for (int i = threadIdx.x; i < T * 64; i += NW * 64) {
    const int t = i >> 6, l = i & 63; float s = red[0][t][l];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][t][l];
    const size_t row = (size_t)tile * 64 + l;
    if (row < (size_t)m.rows) y[(size_t)t * m.rows + row] = s;
    if (T == 1 && best != nullptr) {      // threads 0..63 = wave 0: first maximum of the tile (sampler::argmax order, src/sampler.rs:142-148)
      float bv = row < (size_t)m.rows ? s : -INFINITY; uint32_t bi = (uint32_t)row;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) { float ov = __shfl_xor(bv, o); uint32_t oi = __shfl_xor(bi, o); if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; } }
      if (l == 0) { best[2 * tile] = __float_as_uint(bv); best[2 * tile + 1] = bi; }
    }
  }
}

namespace {
int i8_scratch(pyre_ctx* ctx, size_t nbytes, void** out) {
  if (nbytes > ctx->i8_bytes) {
    if (ctx->i8_buf) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(ctx->i8_buf)); ctx->i8_buf = nullptr; ctx->i8_bytes = 0; }
    PYRE_HIP(ctx, hipMalloc(&ctx->i8_buf, nbytes)); ctx->i8_bytes = nbytes;
  }
  *out = ctx->i8_buf; return PYRE_OK;
}
int env_i(const char* n) { const char* s = getenv(n); return s && *s ? atoi(s) : 0; }
template <int T, int NW, int UB> void launch_nw(pyre_ctx* ctx, const QMatDev& m, const uint32_t* dg, float* y, uint32_t* best) {
  const int upw = (m.U + NW - 1) / NW;
  hipLaunchKernelGGL((k_gemv_i8<T, NW, UB>), dim3(m.tiles), dim3(NW * 64), 0, ctx->stream, m, dg, y, upw, best);
}
template <int T> void launch_t(pyre_ctx* ctx, const QMatDev& m, const uint32_t* dg, float* y, uint32_t* best) {
  static const int fnw = env_i("PYRE_GEMV_I8_NW"), fub = env_i("PYRE_GEMV_I8_UB");
  int nw = 8;
  while (nw > 4 && nw / 2 >= m.U) nw /= 2;
  if constexpr (T == 1) {
    if (fnw) nw = fnw;
    const int ub = fub ? fub : 2;
#define I8_CASE(N, B) if (nw == N && ub == B) return launch_nw<1, N, B>(ctx, m, dg, y, best);
    I8_CASE(2, 1) I8_CASE(2, 2) I8_CASE(2, 4) I8_CASE(4, 1) I8_CASE(4, 2) I8_CASE(4, 4) I8_CASE(8, 1) I8_CASE(8, 2) I8_CASE(8, 4)
#undef I8_CASE
    return launch_nw<1, 4, 2>(ctx, m, dg, y, best);
  } else {
    if (nw == 4) launch_nw<T, 4, 1>(ctx, m, dg, y, best); else launch_nw<T, 8, 1>(ctx, m, dg, y, best);
  }
}
}  // namespace

bool pyre_gemv_i8_ok(const QMatDev& m, int t) { return m.fmt == FMT_IQ3_S && t >= 1 && t <= 8; }

// ---- the variant that allocates nothing -----------------------------------------------------------------------------
// The activation digits of pyre_qmatmul_static_dev live in this file-scope array instead of the context's grow-only
// buffer.  Every GPU the library runs on holds its own copy, at its own address, until the process ends; the name below
// is only the host-side handle of the symbol, the device address comes from hipGetSymbolAddress (once per device, at
// context creation) and is what the kernels and every other host-side use get.
#define I8_STATIC_WORDS ((size_t)PYRE_QMATMUL_STATIC_MAX_TU * I8_STRIDE)
static __device__ __align__(256) uint32_t scratch[I8_STATIC_WORDS];
#define I8_MAX_DEVICES 64
static uint32_t* g_static_ptr[I8_MAX_DEVICES];

int pyre_i8_static_init(pyre_ctx* ctx) {      // called by pyre_ctx_create with the context's device current
  if (ctx->device < 0 || ctx->device >= I8_MAX_DEVICES) return pyre_fail(ctx, PYRE_E_ARG, "device %d outside the static scratch table (%d devices)", ctx->device, I8_MAX_DEVICES);
  if (!g_static_ptr[ctx->device]) {
    void* p = nullptr;
    PYRE_HIP(ctx, hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return pyre_fail(ctx, PYRE_E_HIP, "hipGetSymbolAddress returned a null address for the static scratch");
    g_static_ptr[ctx->device] = (uint32_t*)p;
  }
  ctx->i8_static = g_static_ptr[ctx->device];
  return PYRE_OK;
}

// Same kernels, same launch shapes and therefore the same bits as pyre_gemv_i8_launch; no allocation, no event, no copy.
int pyre_gemv_i8_static_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y) {
  if (!pyre_gemv_i8_ok(m, t)) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul_static_dev: IQ3_S and 1..8 tokens only");
  if ((size_t)t * m.U > (size_t)PYRE_QMATMUL_STATIC_MAX_TU)
    return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmatmul_static_dev: t * cols / 64 = %zu exceeds the static scratch (at most %d: t = 8 up to %d columns)", (size_t)t * m.U, PYRE_QMATMUL_STATIC_MAX_TU, PYRE_QMATMUL_STATIC_MAX_TU / 8 * 64);
  uint32_t* dg = ctx->i8_static;
  if (!dg) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the static scratch of device %d was not resolved at context creation", ctx->device);
  hipLaunchKernelGGL(k_act_digits, dim3(m.U, t), dim3(64), 0, ctx->stream, x, m.cols, dg); PYRE_CHECK_LAUNCH(ctx);
  switch (t) { case 1: launch_t<1>(ctx, m, dg, y, nullptr); break; case 2: launch_t<2>(ctx, m, dg, y, nullptr); break; case 3: launch_t<3>(ctx, m, dg, y, nullptr); break; case 4: launch_t<4>(ctx, m, dg, y, nullptr); break;
    case 5: launch_t<5>(ctx, m, dg, y, nullptr); break; case 6: launch_t<6>(ctx, m, dg, y, nullptr); break; case 7: launch_t<7>(ctx, m, dg, y, nullptr); break; default: launch_t<8>(ctx, m, dg, y, nullptr); break; }
  PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

int pyre_gemv_i8_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y, uint32_t* best) {
  if (!pyre_gemv_i8_ok(m, t)) return pyre_fail(ctx, PYRE_E_ARG, "integer-dot GEMV: IQ3_S and 1..8 tokens only");
  void* buf = nullptr; int rc = i8_scratch(ctx, (size_t)t * m.U * I8_STRIDE * 4, &buf); if (rc) return rc;
  uint32_t* dg = (uint32_t*)buf;
  { ProfScope ps(ctx, "gemv_i8_digits", 4.0 * t * m.cols * 2);
    hipLaunchKernelGGL(k_act_digits, dim3(m.U, t), dim3(64), 0, ctx->stream, x, m.cols, dg); } PYRE_CHECK_LAUNCH(ctx);
  { static const char* nm[8] = {"gemv_i8_iq3_s_t1", "gemv_i8_iq3_s_t2", "gemv_i8_iq3_s_t3", "gemv_i8_iq3_s_t4", "gemv_i8_iq3_s_t5", "gemv_i8_iq3_s_t6", "gemv_i8_iq3_s_t7", "gemv_i8_iq3_s_t8"};
    ProfScope ps(ctx, nm[t - 1], qmat_gguf_bytes(m, m.rows) + 4.0 * t * ((double)m.cols + m.rows));
    switch (t) { case 1: launch_t<1>(ctx, m, dg, y, best); break; case 2: launch_t<2>(ctx, m, dg, y, best); break; case 3: launch_t<3>(ctx, m, dg, y, best); break; case 4: launch_t<4>(ctx, m, dg, y, best); break;
      case 5: launch_t<5>(ctx, m, dg, y, best); break; case 6: launch_t<6>(ctx, m, dg, y, best); break; case 7: launch_t<7>(ctx, m, dg, y, best); break; default: launch_t<8>(ctx, m, dg, y, best); break; } }
  PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
