// Hyper-connection mix / combine around every block: grouped RMSNorm over the hc residual streams, low-rank sigmoid
// gate, stream mean; residual update.  Follows hc_mix / hc_combine, src/model/qwen4exp_gguf.rs:1357-1388 (f32 branch).
//
// One mix is two launches.  k_hc_norm_down folds the pending residual update, the norm weights and the [down ; inject]
// GEMV (K cut into slices, one slice per workgroup) and leaves each slice's sum of squares; k_hc_up_mix turns those
// into the streams' RMS scales, adds the scaled slice sums, applies silu, runs the up GEMV from shared memory and
// reduces the gated, normalized streams to their mean.
#include "gemm_m.h"
#include "digits.h"
#include <stdlib.h>
#include <algorithm>

PYRE_TS_DECL(hc_ts) PYRE_TS_EXPORT(hc_ts, pyre_debug_ts_hc)
__device__ __forceinline__ float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }

// Stream element i of token ti with the pending residual update applied: x + out * w  (:1384-1387), w = 2*sigm(inj).
// `out` is a plain [t][d] vector (comb_out) or the unreduced FFN output (mo.partial != nullptr).
// NP > 1: `out` comes as NP partial vectors, part q of token ti at comb_out + (q*T + ti)*d, added in order from the first
// (pyre_gemv_parts_launch); all parts are fetched before the first add.
template <int T, int NP, int FK = 0> __device__ __forceinline__ float hc_x_new(const float* __restrict__ x_in, int in_ss, int in_ts, const float* __restrict__ comb_out, const MoeOut& mo, float w, int d, int ti, int s, int i) {
  float v = x_in[(size_t)ti * in_ts + (size_t)s * in_ss + i];
  if constexpr (NP > 1) {
    float sv[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) sv[q] = (comb_out + ((size_t)q * T + ti) * d)[i];
    float o = sv[0];
#pragma unroll
    for (int q = 1; q < NP; ++q) o += sv[q];
    v = v + o * w;
  } else {
    if (mo.partial) v = v + moe_out_value<FK>(mo, ti, i) * w;
    else if (comb_out) v = v + comb_out[(size_t)ti * d + i] * w;
  }
  return v;
}

// The slices of one output row, all loads in flight together: groups of eight behind a branch the whole launch agrees on
// (ksplit is a kernel argument), so that unused groups cost neither loads nor instruction fetch; inside a group slices
// past ksplit repeat the last one and are never added.  `want` is the thread's own condition (one execution mask).
__device__ __forceinline__ void hc_load_run(float (&sv)[32], const float* __restrict__ p, int n, int stride) {      // n (<= 32) values at p, p + stride, ..
#pragma unroll
  for (int k = 0; k < 32; ++k) sv[k] = 0.0f;
#pragma unroll
  for (int g = 0; g < 8; ++g) if (g * 4 < n) {
#pragma unroll
    for (int j = 0; j < 4; ++j) sv[g * 4 + j] = p[(size_t)min(g * 4 + j, n - 1) * stride];
  }
}
template <int T> __device__ __forceinline__ void hc_load_slices(float (&pv)[32], const float* __restrict__ part, bool want, int ksplit, int t, int r64, int i) {
#pragma unroll
  for (int ks = 0; ks < 32; ++ks) pv[ks] = 0.0f;
  const unsigned off = (unsigned)(t * r64 + i);
  if (want) {
#pragma unroll
    for (int g = 0; g < 4; ++g) if (g * 8 < ksplit) {
#pragma unroll
      for (int j = 0; j < 8; ++j) pv[g * 8 + j] = (part + (size_t)min(g * 8 + j, ksplit - 1) * T * r64)[off];      // launch-uniform base + the thread's 32-bit offset
    }
  }
}

// grid (row tiles of [down ; inject], K slices), nw waves.  A workgroup owns L = nw*upw*64 columns of one stream s.
// The RMS scale of a stream multiplies every term of a row's dot product, so it is applied after the dot (by
// k_hc_up_mix, which also sums the slices): a workgroup never needs the sum of squares of the whole stream.
//   1. its L columns of x_new (the pending residual update applied) times the norm weight go to shared memory; the
//      squares of x_new are summed over the slice -> ssq[ks*T + t]; the tile-0 workgroup of the slice also publishes the
//      updated stream (x_out, never the buffer x_in points into)
//   2. each wave takes upw units of the slice; partial sums -> part[(ks*T + t)*tiles*64 + row]
template <int FMT, int T, int NP> __global__ __launch_bounds__(512) void k_hc_norm_down(QMatDev m, const float* __restrict__ x_in, int in_ss, int in_ts, float* __restrict__ x_out,
    const float* __restrict__ comb_out, MoeOut mo, const float* __restrict__ comb_inj, const float* __restrict__ norm, int d, int hc, float* __restrict__ ssq,
    float* __restrict__ part, int upw, const uint2* __restrict__ g2) {
  const uint2* lds2 = nullptr;          // no format needs a codebook in shared memory any more
  PYRE_TS_VARS PYRE_TS(0);
  qmat_args_now(m); args_now(x_in, in_ss, in_ts, x_out, comb_out, mo.partial, mo.sel_w, mo.sg, mo.d, mo.k, comb_inj, norm, d, hc, ssq, part, upw);
  extern __shared__ __align__(16) float sm[];
  const int nthr = blockDim.x, nw = nthr >> 6, tid = threadIdx.x, L = nw * upw * 64;
  float* xs = sm;                         // [T][L]
  float* red = sm + (size_t)T * L;        // [nw][T][64]
  float* wsum = red + (size_t)nw * T * 64;   // [nw][T]
  const int tile = blockIdx.x, ks = blockIdx.y;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int c0 = ks * L, s = c0 / d, i0 = c0 - s * d;
  // Loads return in the order they were issued: the streams (and the pending update's terms) first, since the copy into
  // shared memory waits for them, then the first unit's weights, which stay in flight across the barrier.
  float w[T], ss[T];
#pragma unroll
  for (int t = 0; t < T; ++t) { w[t] = (comb_out || mo.partial) ? 2.0f * sigm(comb_inj[t * hc + s]) : 0.0f; ss[t] = 0.0f; }
  float v0[T]; float nv0 = 0.0f;
  if (tid < L) {
    nv0 = norm[(size_t)s * d + i0 + tid];
#pragma unroll
    for (int t = 0; t < T; ++t) v0[t] = hc_x_new<T, NP>(x_in, in_ss, in_ts, comb_out, mo, w[t], d, t, s, i0 + tid);
  }
  UnitRaw<FMT> raw = unit_load<FMT>(m, tile, ks * nw * upw + wave * upw, lane);
  if (tid < L) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const float v = v0[t];
      ss[t] += v * v;
      xs[(size_t)t * L + tid] = v * nv0;
      if (tile == 0) x_out[((size_t)t * hc + s) * d + i0 + tid] = v;
    }
  }
  for (int j = tid + nthr; j < L; j += nthr) {
    const float nv = norm[(size_t)s * d + i0 + j];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float v = hc_x_new<T, NP>(x_in, in_ss, in_ts, comb_out, mo, w[t], d, t, s, i0 + j);
      ss[t] += v * v;
      xs[(size_t)t * L + j] = v * nv;
      if (tile == 0) x_out[((size_t)t * hc + s) * d + i0 + j] = v;
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss[t] += __shfl_xor(ss[t], o);
    if (lane == 0) wsum[wave * T + t] = ss[t];
  }
  lds_barrier(); PYRE_TS(1);
  if (tile == 0 && tid < T) { float tot = wsum[tid]; for (int q = 1; q < nw; ++q) tot += wsum[q * T + tid]; ssq[ks * T + tid] = tot; }
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.0f;
  for (int u = 0; u < upw; ++u) { int lu = wave * upw + u; if (u > 0) raw = unit_load<FMT>(m, tile, ks * nw * upw + lu, lane); unit_fma<FMT, T>(m, raw, ks * nw * upw + lu, lds2, lane, xs + lu * 64, L, acc); }
#pragma unroll
  for (int t = 0; t < T; ++t) red[((size_t)wave * T + t) * 64 + lane] = acc[t];
  PYRE_TS(2);
  lds_barrier(); PYRE_TS(3);
  const size_t r64 = (size_t)m.tiles * 64;
  for (int i = tid; i < T * 64; i += nthr) {
    int t = i >> 6, l = i & 63; float a = red[(size_t)t * 64 + l];
    for (int q = 1; q < nw; ++q) a += red[((size_t)q * T + t) * 64 + l];
    part[((size_t)ks * T + t) * r64 + (size_t)tile * 64 + l] = a;
  }
  PYRE_TS(4); PYRE_TS_FLUSH(hc_ts, NP > 1 ? 0 : 8);
}

// grid (d / 64), hc*U waves (U = lr / 64 units of the up matrix).  Prologue: the streams' RMS scales from the slice
// sums of squares, scale_s = 1 / sqrt(sum / d + eps) (rms, :209); o = the slice sums of [down ; inject], each times
// its stream's scale, added in slice order;
// lo = silu(o / hc) for the first lr rows -> shared memory, inj = o[lr + s] / hc (zeros without inject) (:1376-1378).
// Wave (s, ku) takes unit ku of row tile s*(d/64) + blockIdx.x of `up`; the gate logit of stream s is the sum of its
// waves in unit order; mixed[i] = (sum_s xn[s][i] * sigm(gate_s[i])) / hc with xn = (x * scale_s) * norm, s ascending
// from zero (:1380).
// RF >= 0: the launch also leaves its K slice of the router GEMV over the mixed vector (format RF; HcRoute): wave w
// takes router tile w, w + nw, .. at unit blockIdx.x, the first tile's weights fetched ahead of the up GEMV.
template <int FMT, int T, int RF> __global__ __launch_bounds__(1024) void k_hc_up_mix(QMatDev up, const float* __restrict__ part, const float* __restrict__ ssq, int ksplit, int r64, int lr, int hc, int has_inject,
    const float* __restrict__ xnew, const float* __restrict__ norm, float eps, int d, float* __restrict__ mixed, float* __restrict__ inj, const uint2* __restrict__ g2,
    QMatDev router, float* __restrict__ rpart) {
  constexpr bool ROUTE = RF >= 0; constexpr int RFX = ROUTE ? RF : FMT_F32;
  const uint2* lds2 = nullptr;          // no format needs a codebook in shared memory any more
  PYRE_TS_VARS PYRE_TS(0);
  qmat_args_now(up); args_now(part, ssq, ksplit, r64, lr, hc, has_inject, xnew, norm, eps, d, mixed, inj);

  extern __shared__ __align__(16) float sm[];
  const int nthr = blockDim.x, tid = threadIdx.x, U = lr >> 6, kps = ksplit / hc, nw = nthr >> 6;
  float* lo = sm;                         // [T][lr]
  float* red = sm + (size_t)T * lr;       // [nw][T][64]
  float* sls = red + (size_t)nw * T * 64;   // [T][32]: the RMS scale of the stream each slice belongs to
  float* term = sls + (size_t)T * 32;     // [T*hc][64]: the streams' gated, normalized values before they are added
  const int n_o = lr + hc;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int s = wave / U, ku = wave - s * U;
  // Loads return in the order they were issued, so they are issued in the order they are needed: the slice sums of
  // squares and of [down ; inject] first (the prologue waits for nothing else), then the up weights, the epilogue's
  // operands and the router tile, all of which stay in flight across the barriers below (which exchange through shared
  // memory only).
  float ssv[32];
#pragma unroll
  for (int k = 0; k < 32; ++k) ssv[k] = 0.0f;
  const int stt = tid / hc, sq = tid - stt * hc;
  if (tid < T * hc) hc_load_run(ssv, ssq + (size_t)(sq * kps) * T + stt, kps, T);          // all of the stream's slices before the first add: one round trip
  float pv[32]; int idx = tid; int t = idx / n_o, i = idx - t * n_o;
  bool have = idx < T * n_o;
  hc_load_slices<T>(pv, part, have && (i < lr || has_inject), ksplit, t, r64, i);
  UnitRaw<FMT> raw = unit_load<FMT>(up, s * (d >> 6) + blockIdx.x, ku, lane);
  // the epilogue's stream value and norm weight of this wave's first (token, stream) item
  float xpre = 0.0f, npre = 0.0f;
  if (wave < T * hc) { const int t0 = wave / hc, q0 = wave - t0 * hc; xpre = (xnew + ((size_t)t0 * hc + q0) * d + blockIdx.x * 64)[lane]; npre = (norm + (size_t)q0 * d + blockIdx.x * 64)[lane]; }
  UnitRaw<RFX> rraw;
  constexpr bool R_EARLY = RFX != FMT_F32;      // an f32 tile is 64 registers: fetched once the up GEMV has freed them
  if (ROUTE && R_EARLY && wave < router.tiles) rraw = unit_load<RFX>(router, wave, blockIdx.x, lane);
  if (tid < T * hc) {
    float tot = ssv[0];
#pragma unroll
    for (int k = 1; k < 32; ++k) if (k < kps) tot += ssv[k];
    const float sc = 1.0f / sqrtf(tot / (float)d + eps);
    for (int k = 0; k < kps; ++k) sls[stt * 32 + sq * kps + k] = sc;
  }
  lds_barrier(); PYRE_TS(1);
  while (have) {
    float o = 0.0f;                 // slices in order, each times its stream's scale
    if (i < lr || has_inject) {
#pragma unroll
      for (int ks = 0; ks < 32; ++ks) if (ks < ksplit) { const float tm = pv[ks] * sls[t * 32 + ks]; o = ks == 0 ? tm : o + tm; }
    }
    const float v = o / (float)hc;
    if (i < lr) lo[t * lr + i] = v * sigm(v);
    else if (blockIdx.x == 0) inj[t * hc + (i - lr)] = has_inject ? v : 0.0f;
    idx += nthr; have = idx < T * n_o;
    if (have) { t = idx / n_o; i = idx - t * n_o; hc_load_slices<T>(pv, part, i < lr || has_inject, ksplit, t, r64, i); }
  }
  lds_barrier(); PYRE_TS(2);
  float acc[T];
#pragma unroll
  for (int t2 = 0; t2 < T; ++t2) acc[t2] = 0.0f;
  unit_fma<FMT, T>(up, raw, ku, lds2, lane, lo + ku * 64, lr, acc);
#pragma unroll
  for (int t2 = 0; t2 < T; ++t2) red[((size_t)wave * T + t2) * 64 + lane] = acc[t2];
  if (ROUTE && !R_EARLY && wave < router.tiles) rraw = unit_load<RFX>(router, wave, blockIdx.x, lane);
  PYRE_TS(3);
  lds_barrier(); PYRE_TS(4);
  // one wave per (token, stream): the gate logit is the sum of the stream's waves in unit order; xn * sigm(gate) -> term
  for (int w = wave; w < T * hc; w += nw) {
    const int t2 = w / hc, q = w - t2 * hc, col = blockIdx.x * 64 + lane;
    float g = red[((size_t)(q * U) * T + t2) * 64 + lane];
    for (int k = 1; k < U; ++k) g += red[((size_t)(q * U + k) * T + t2) * 64 + lane];
    const float xv = w == wave ? xpre : xnew[((size_t)t2 * hc + q) * d + col];
    const float nv = w == wave ? npre : norm[(size_t)q * d + col];
    term[(size_t)w * 64 + lane] = xv * sls[t2 * 32 + q * kps] * nv * sigm(g);            // rms, :209: (x * s) * w
  }
  lds_barrier();
  for (int i2 = tid; i2 < T * 64; i2 += nthr) {
    const int t2 = i2 >> 6, l = i2 & 63, col = blockIdx.x * 64 + l; float mx = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; ++q) if (q < hc) mx += term[(size_t)(t2 * hc + q) * 64 + l];          // streams ascending from zero (:1380)
    const float mv = mx / (float)hc;
    mixed[(size_t)t2 * d + col] = mv;
    if (ROUTE) lo[t2 * 64 + l] = mv;          // lo is free after the barrier above
  }
  PYRE_TS(5);
  if (ROUTE) {
    lds_barrier(); PYRE_TS(6);
    const size_t rr64 = (size_t)router.tiles * 64;
    for (int tile = wave; tile < router.tiles; tile += nw) {
      if (tile != wave) rraw = unit_load<RFX>(router, tile, blockIdx.x, lane);
#pragma unroll 1
      for (int t2 = 0; t2 < T; ++t2) {          // one token at a time (same operations per token): T tokens at once would keep 64*T activations in registers
        float ra[1] = {0.0f};
        unit_fma<RFX, 1>(router, rraw, blockIdx.x, lds2, lane, lo + t2 * 64, 0, ra);
        rpart[((size_t)blockIdx.x * T + t2) * rr64 + (size_t)tile * 64 + lane] = ra[0];
      }
    }
  }
  PYRE_TS(7); PYRE_TS_FLUSH(hc_ts, ROUTE ? 16 : 24);
}

// ---- the same two launches with both GEMVs on the f16 matrix cores -------------------------------------------------------
// For [down ; inject] and up held in the IQ3_S matrix-core layout (QMatDev::mq / mh).  The lane = row kernels above pay
// one multiply-add per weight and token on top of the decode; here a weight costs the same whatever the window width,
// and a token's sums do not depend on the width either (its two operand rows are its own), so a window still equals
// single steps bit for bit.  The operand rows are formed inside the kernels, in shared memory: x = h1 + h2 * 2^-11 after
// a power-of-two scaling per token and slice (k_act_split's rule).
__device__ __forceinline__ void hc_scale_of(float m, float* up, float* dn) {      // m * 2^e in [2^13, 2^14); zero and non-finite maxima leave e = 0
  int e = 0;
  if (m > 0.0f && m < INFINITY) { e = 140 - (int)((__float_as_uint(m) >> 23) & 0xFF); e = e > 100 ? 100 : e; }
  *up = __uint_as_float((uint32_t)(127 + e) << 23); *dn = __uint_as_float((uint32_t)(127 - e) << 23);
}
__device__ __forceinline__ void hc_split_store(uint16_t* ah, int k, int t, float xs) {      // operand rows 2t, 2t+1 of column k: [8-column group][16 rows][8]
  const _Float16 h1 = (_Float16)xs, h2 = (_Float16)((xs - (float)h1) * 2048.0f);
  uint16_t* o = ah + ((size_t)(k >> 3) * 16 + 2 * t) * 8 + (k & 7);
  o[0] = __builtin_bit_cast(unsigned short, h1); o[8] = __builtin_bit_cast(unsigned short, h2);
}
__device__ __forceinline__ void hc_lds_a(const uint16_t* ah, int c, int lane, ABuf& b) {      // chunk c (128 columns) of the operand in shared memory
#pragma unroll
  for (int s = 0; s < 4; ++s) b.a[s] = ((const uint4*)ah)[((c * 4 + s) * 4 + (lane >> 4)) * 16 + (lane & 15)];
}

// grid (row tiles of [down ; inject], slices of 256*CS columns), 4*CS waves, a thread prepares one column of the slice.
// Wave (p, g) takes row group g of the tile over chunk pair p of the slice; with CS = 2 the two pairs' sums meet in
// shared memory (pair 0 + pair 1).  Outputs as k_hc_norm_down: ssq[ks*T + t], part[(ks*T + t)*tiles*64 + row], x_out.
// FD, FK > 0: the model width d and the routed experts per token as compile-time constants (the launcher checks them): the
// stream index of a slice is a shift, the gather of the unreduced FFN output carries no predicates -- same arithmetic.
template <int T, int NP, int CS, int FD = 0, int FK = 0> __global__ __launch_bounds__(256 * CS) void k_hc_norm_down_m(QMatDev m, const float* __restrict__ x_in, int in_ss, int in_ts, float* __restrict__ x_out,
    const float* __restrict__ comb_out, MoeOut mo, const float* __restrict__ comb_inj, const float* __restrict__ norm, int d, int hc, float* __restrict__ ssq, float* __restrict__ part, float* __restrict__ smx, size_t wz) {
  constexpr int NW = 4 * CS;
  __shared__ __align__(16) uint16_t ah[CS * 32 * 16 * 8];
  __shared__ float wsum[NW][8], wmax[NW][8], hsum[4][2][64];
  PYRE_TS_VARS PYRE_TS(0);
  qmat_args_now(m); args_now(x_in, in_ss, in_ts, x_out, comb_out, mo.partial, mo.sel_w, mo.sg, mo.d, mo.k, comb_inj, norm, d, hc, ssq, part);
  if (wz) {          // a launch for several windows: blockIdx.z's window has everything that is its own wz bytes further on per window
    const size_t zo = (size_t)blockIdx.z * wz;
    x_in = (const float*)((const char*)x_in + zo); x_out = (float*)((char*)x_out + zo); ssq = (float*)((char*)ssq + zo); part = (float*)((char*)part + zo); smx = (float*)((char*)smx + zo);
    if (comb_out) comb_out = (const float*)((const char*)comb_out + zo);
    if (comb_inj) comb_inj = (const float*)((const char*)comb_inj + zo);
  }
  const int tile = blockIdx.x, ks = blockIdx.y, tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = wave & 3, p = wave >> 2;
  if constexpr (FD > 0) d = FD;
  const int c0 = ks * 256 * CS, s = c0 / d, i0 = c0 - s * d, K128 = m.cols >> 7;
  float w[T], v[T];
#pragma unroll
  for (int t = 0; t < T; ++t) w[t] = (comb_out || mo.partial) ? 2.0f * sigm(comb_inj[t * hc + s]) : 0.0f;
  const float nv = norm[(size_t)s * d + i0 + tid];
#pragma unroll
  for (int t = 0; t < T; ++t) v[t] = hc_x_new<T, NP, FK>(x_in, in_ss, in_ts, comb_out, mo, w[t], d, t, s, i0 + tid);
  const int ch0 = ks * 2 * CS + 2 * p;
  WBuf<1> w0, w1; load_w<1>(m, tile * 4 + g, ch0, lane, K128, w0); load_w<1>(m, tile * 4 + g, ch0 + 1, lane, K128, w1);
  const NibK nk = nib_consts();
  float xs[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    float ss = v[t] * v[t]; xs[t] = v[t] * nv;
    if (tile == 0) x_out[((size_t)t * hc + s) * d + i0 + tid] = v[t];
    float a = fabsf(xs[t]); a = a == a ? a : INFINITY;
    ss = wave_sum(ss); a = wave_max(a);
    if (lane == 0) { wsum[wave][t] = ss; wmax[wave][t] = a; }
  }
#pragma unroll
  for (int r = 2 * T; r < 16; ++r) ah[((size_t)(tid >> 3) * 16 + r) * 8 + (tid & 7)] = 0;      // rows no token of the window owns
  PYRE_TS(1);
  lds_barrier(); PYRE_TS(2);
  auto slice_max = [&](int t) { float mx = wmax[0][t];
#pragma unroll
    for (int k = 1; k < NW; ++k) mx = fmaxf(mx, wmax[k][t]);
    return mx; };
  if (tile == 0 && tid < T) { float tot = wsum[0][tid];
#pragma unroll
    for (int k = 1; k < NW; ++k) tot += wsum[k][tid];
    ssq[ks * T + tid] = tot; smx[ks * T + tid] = slice_max(tid); }          // (the largest |x * norm weight| of the slice: the second launch bounds the mixed vector with it)
#pragma unroll
  for (int t = 0; t < T; ++t) { float up, dn; hc_scale_of(slice_max(t), &up, &dn); hc_split_store(ah, tid, t, xs[t] * up); }
  lds_barrier(); PYRE_TS(3);
  const int q = lane >> 4;
  float upf, dn0 = 0.0f, dn1 = 0.0f;
  if (2 * q < T) hc_scale_of(slice_max(2 * q), &upf, &dn0);
  if (2 * q + 1 < T) hc_scale_of(slice_max(2 * q + 1), &upf, &dn1);
  v4f tot[1] = {v4f{0.0f, 0.0f, 0.0f, 0.0f}};
  { ABuf a0, a1; hc_lds_a(ah, 2 * p, lane, a0); hc_lds_a(ah, 2 * p + 1, lane, a1); a0.ai0 = dn0; a0.ai1 = dn1; a1.ai0 = dn0; a1.ai1 = dn1;
    chunk_mac<1>(w0, a0, ch0, nk, tot); chunk_mac<1>(w1, a1, ch0 + 1, nk, tot); }
  PYRE_TS(4);
  float r0 = tot[0][0] + tot[0][1] * (1.0f / 2048.0f), r1 = tot[0][2] + tot[0][3] * (1.0f / 2048.0f);
  if constexpr (CS == 2) {
    if (p == 1) { hsum[g][0][lane] = r0; hsum[g][1][lane] = r1; }
    lds_barrier();
    if (p == 1) return;
    r0 += hsum[g][0][lane]; r1 += hsum[g][1][lane];
  }
  const size_t r64 = (size_t)m.tiles * 64, row = (size_t)tile * 64 + g * 16 + (lane & 15);
  if (2 * q < T) part[((size_t)ks * T + 2 * q) * r64 + row] = r0;
  if (2 * q + 1 < T) part[((size_t)ks * T + 2 * q + 1) * r64 + row] = r1;
  PYRE_TS(5); PYRE_TS(6); PYRE_TS(7); PYRE_TS_FLUSH(hc_ts, NP > 1 ? 48 : 56);
}

__device__ __forceinline__ void hc_load_run16(float (&sv)[16], const float* __restrict__ p, int n, int stride) {      // n (<= 16) values at p, p + stride, ..
#pragma unroll
  for (int k = 0; k < 16; ++k) sv[k] = 0.0f;
#pragma unroll
  for (int g = 0; g < 4; ++g) if (g * 4 < n) {
#pragma unroll
    for (int j = 0; j < 4; ++j) sv[g * 4 + j] = p[(size_t)min(g * 4 + j, n - 1) * stride];
  }
}
// up to sixteen slice sums of one output row, all loads in flight together (as hc_load_slices)
template <int T> __device__ __forceinline__ void hc_load_slices16(float (&pv)[16], const float* __restrict__ part, bool want, int ksplit, int t, int r64, int i) {
#pragma unroll
  for (int ks = 0; ks < 16; ++ks) pv[ks] = 0.0f;
  const unsigned off = (unsigned)(t * r64 + i);
  if (want) {
#pragma unroll
    for (int g = 0; g < 2; ++g) if (g * 8 < ksplit) {
#pragma unroll
      for (int j = 0; j < 8; ++j) pv[g * 8 + j] = (part + (size_t)min(g * 8 + j, ksplit - 1) * T * r64)[off];
    }
  }
}
__device__ __forceinline__ float hc_slice_sum16(const float (&pv)[16], const float* sls_t, int ksplit) {      // slices in order, each times its stream's scale
  float o = 0.0f;
#pragma unroll
  for (int ks = 0; ks < 16; ++ks) if (ks < ksplit) { const float tm = pv[ks] * sls_t[ks]; o = ks == 0 ? tm : o + tm; }
  return o;
}

// grid (d / CW), hc * (CW / 16) waves, CW = 1 << lcw = 16, 32 or 64 columns of the mixed vector per workgroup: wave (s, g)
// takes row group g of the workgroup's CW rows of stream s of `up` over all lr columns (at most sixteen slices).  A single
// token without a riding router runs on d / 16 workgroups of hc waves: the launch is bound by the vector instructions a
// compute unit issues, not by bytes, so 128 compute units with one wave per SIMD finish the same arithmetic four times
// sooner than 32 with four.  Prologue, epilogue and the riding router GEMV (CW = 64 only: a workgroup owns one 64-column
// unit of the router) as k_hc_up_mix, except that every load the prologue and the epilogue need is issued at the start
// (two rows of lo and one inject row a thread, the streams of one column a thread), and lo goes through shared memory
// twice: f32, then as operand rows scaled per token by the power of two of its largest magnitude.  Operand rows no token
// of the window owns are left as they are: a row only ever reaches its own sums.  A value's arithmetic does not depend on CW.
// FHC, FLR, FKS > 0: the stream count, the low rank and the slice count as compile-time constants (the launcher checks
// them): divisions become shifts, the slice loops lose their predicates -- same arithmetic.
template <int T, int RF, int FHC = 0, int FLR = 0, int FKS = 0> __global__ __launch_bounds__(1024) void k_hc_up_mix_m(QMatDev up, const float* __restrict__ part, const float* __restrict__ ssq, int ksplit, int r64, int lr, int hc, int has_inject,
    const float* __restrict__ xnew, const float* __restrict__ norm, float eps, int d, float* __restrict__ mixed, float* __restrict__ inj,
    QMatDev router, float* __restrict__ rpart, uint16_t* __restrict__ aop, int aop_rows, int lcw, const float* __restrict__ smx, float* __restrict__ aop_inv, int aop_nsb, uint32_t* __restrict__ dgx, size_t wz) {
  constexpr bool ROUTE = RF >= 0; constexpr int RFX = ROUTE ? RF : FMT_F32;
  __shared__ uint8_t dsm[ROUTE ? T : 1][3][64];          // the digit waves' staging
  const uint2* lds2 = nullptr;
  PYRE_TS_VARS PYRE_TS(0);
  qmat_args_now(up); args_now(part, ssq, ksplit, r64, lr, hc, has_inject, xnew, norm, eps, d, mixed, inj, lcw);
  if (wz) {          // a launch for several windows, as k_hc_norm_down_m
    const size_t zo = (size_t)blockIdx.z * wz;
    part = (const float*)((const char*)part + zo); ssq = (const float*)((const char*)ssq + zo); xnew = (const float*)((const char*)xnew + zo); smx = (const float*)((const char*)smx + zo);
    mixed = (float*)((char*)mixed + zo); inj = (float*)((char*)inj + zo);
    if (rpart) rpart = (float*)((char*)rpart + zo);
    if (aop) aop = (uint16_t*)((char*)aop + zo);
    if (aop_inv) aop_inv = (float*)((char*)aop_inv + zo);
    if (dgx) dgx = (uint32_t*)((char*)dgx + zo);
  }
  if constexpr (FHC > 0) { hc = FHC; lr = FLR; ksplit = FKS; }
  extern __shared__ __align__(16) float sm[];
  const int nthr = blockDim.x, tid = threadIdx.x, kps = ksplit / hc, nw = nthr >> 6, CW = 1 << lcw, lg = lcw - 4;
  float* lo = sm;                                 // [T][lr]
  float* red = lo + (size_t)T * lr;               // [hc][T][CW]: the gate logits
  float* sls = red + (size_t)hc * T * 64;         // [T][16]
  uint32_t* lmax = (uint32_t*)(sls + (size_t)T * 16);      // [8]: bits of the largest |lo| of each token
  float* bnd = (float*)(lmax + 8);                // [T][4]: RMS scale * largest |x * norm weight| of each stream
  uint16_t* ah = (uint16_t*)(bnd + 32);           // [lr/8][16][8]
  const int K128 = lr >> 7, n_lo = T * lr;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int s = wave >> lg, g = wave & ((1 << lg) - 1), q = lane >> 4;
  const int col0 = blockIdx.x << lcw;
  float ssv[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) ssv[k] = 0.0f;
  const int stt = tid / hc, sq = tid - stt * hc;
  const bool own_stream = tid < T * hc;                      // thread (token stt, stream sq): the stream's scale, and the stream's inject row
  float smv[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) smv[k] = 0.0f;
  if (own_stream) { hc_load_run16(ssv, ssq + (size_t)(sq * kps) * T + stt, kps, T); if (aop) hc_load_run16(smv, smx + (size_t)(sq * kps) * T + stt, kps, T); }
  float pva[16], pvb[16], pvi[16];
  const int ia = tid, ib = tid + nthr;
  const int ta = ia / lr, ra = ia - ta * lr, tb = ib / lr, rb = ib - tb * lr;
  hc_load_slices16<T>(pva, part, ia < n_lo, ksplit, ta, r64, ra);
  hc_load_slices16<T>(pvb, part, ib < n_lo, ksplit, tb, r64, rb);
  hc_load_slices16<T>(pvi, part, own_stream && has_inject, ksplit, stt, r64, lr + sq);
  const int rg = ((s * d + col0) >> 4) + g;
  WBuf<1> w0, w1; load_w<1>(up, rg, 0, lane, K128, w0); load_w<1>(up, rg, 1, lane, K128, w1);
  const NibK nk = nib_consts();
  // the epilogue's operands: thread (token tid / CW, column tid % CW) adds the streams of its column itself
  float xpre[4] = {0.0f, 0.0f, 0.0f, 0.0f}, npre[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  const int et = tid >> lcw, el = tid & (CW - 1);
  if (tid < (T << lcw)) {
#pragma unroll
    for (int qs = 0; qs < 4; ++qs) if (qs < hc) { xpre[qs] = xnew[((size_t)et * hc + qs) * d + col0 + el]; npre[qs] = norm[(size_t)qs * d + col0 + el]; }
  }
  UnitRaw<RFX> rraw;
  constexpr bool R_EARLY = RFX != FMT_F32;      // an f32 tile is 64 registers: fetched once the up GEMV has freed them; others once the slice sums are used up
  if (tid < 8) lmax[tid] = 0u;
  if (own_stream) {
    float tot = ssv[0];
#pragma unroll
    for (int k = 1; k < 16; ++k) if (k < kps) tot += ssv[k];
    const float sc = 1.0f / sqrtf(tot / (float)d + eps);
    for (int k = 0; k < kps; ++k) sls[stt * 16 + sq * kps + k] = sc;
    float mxs = smv[0];
#pragma unroll
    for (int k = 1; k < 16; ++k) if (k < kps) mxs = fmaxf(mxs, smv[k]);
    bnd[stt * 4 + (sq & 3)] = sc * mxs;          // |x_i * scale * norm_i| <= this for every column i of the stream
  }
  PYRE_TS(1);
  lds_barrier(); PYRE_TS(2);
  const bool hc_p2 = (hc & (hc - 1)) == 0; const float rhc = 1.0f / (float)hc;          // a power-of-two stream count: the division is a multiplication, bit for bit
  auto put_lo = [&](int t, int i, const float (&pv)[16]) {
    const float sv = hc_slice_sum16(pv, sls + t * 16, ksplit); float v;
    if (hc_p2) v = sv * rhc; else v = sv / (float)hc;
    const float lv = v * sigm(v);
    lo[t * lr + i] = lv; float a = fabsf(lv); a = a == a ? a : INFINITY; atomicMax(&lmax[t], __float_as_uint(a)); };
  if (ia < n_lo) put_lo(ta, ra, pva);
  if (ib < n_lo) put_lo(tb, rb, pvb);
  for (int idx = tid + 2 * nthr; idx < n_lo; idx += nthr) { const int t = idx / lr, i = idx - t * lr; hc_load_slices16<T>(pva, part, true, ksplit, t, r64, i); put_lo(t, i, pva); }
  if (own_stream && blockIdx.x == 0) inj[stt * hc + sq] = has_inject ? hc_slice_sum16(pvi, sls + stt * 16, ksplit) / (float)hc : 0.0f;
  // the router's tiles go round the waves; with waves to spare (16 waves, 8 tiles) wave w and wave w + tiles share tile w and split the tokens
  const int rnt = ROUTE ? max(1, (int)router.tiles) : 1, rsets = T == 1 ? 1 : max(1, nw / rnt), rtile = T == 1 ? wave : wave % rnt, rset = T == 1 ? 0 : wave / rnt;
  const bool rwave = ROUTE && (T == 1 ? wave < rnt : (rset < rsets && rset < T));          // (a set without a token fetches nothing; a single token: one set, no division)
  if (rwave && R_EARLY) rraw = unit_load<RFX>(router, rtile, blockIdx.x, lane);
  lds_barrier(); PYRE_TS(3);
  for (int j = tid; j < n_lo; j += nthr) {
    const int t2 = j / lr, k = j - t2 * lr; float upf, dn; hc_scale_of(__uint_as_float(lmax[t2]), &upf, &dn);
    hc_split_store(ah, k, t2, lo[j] * upf);
  }
  lds_barrier(); PYRE_TS(4);
  v4f tot[1] = {v4f{0.0f, 0.0f, 0.0f, 0.0f}};
  { float upf, dn0 = 0.0f, dn1 = 0.0f;
    if (2 * q < T) hc_scale_of(__uint_as_float(lmax[2 * q]), &upf, &dn0);
    if (2 * q + 1 < T) hc_scale_of(__uint_as_float(lmax[2 * q + 1]), &upf, &dn1);
    for (int c = 0; c < K128; c += 2) {
      if (c > 0) { load_w<1>(up, rg, c, lane, K128, w0); load_w<1>(up, rg, c + 1, lane, K128, w1); }
      ABuf a0, a1; hc_lds_a(ah, c, lane, a0); hc_lds_a(ah, c + 1, lane, a1);
      a0.ai0 = dn0; a0.ai1 = dn1; a1.ai0 = dn0; a1.ai1 = dn1;
      chunk_mac<1>(w0, a0, c, nk, tot); chunk_mac<1>(w1, a1, c + 1, nk, tot);
    } }
  if (2 * q < T) red[(((size_t)s * T + 2 * q) << lcw) + g * 16 + (lane & 15)] = tot[0][0] + tot[0][1] * (1.0f / 2048.0f);
  if (2 * q + 1 < T) red[(((size_t)s * T + 2 * q + 1) << lcw) + g * 16 + (lane & 15)] = tot[0][2] + tot[0][3] * (1.0f / 2048.0f);
  if (rwave && !R_EARLY) rraw = unit_load<RFX>(router, rtile, blockIdx.x, lane);
  PYRE_TS(5);
  lds_barrier(); PYRE_TS(6);
  if (tid < (T << lcw)) {          // the gated, normalised streams of the column, streams ascending from zero (:1380)
    const int t2 = et, l = el, col = col0 + l; float mx = 0.0f;
#pragma unroll
    for (int qs = 0; qs < 4; ++qs) if (qs < hc) mx += xpre[qs] * sls[t2 * 16 + qs * kps] * npre[qs] * sigm(red[(((size_t)qs * T + t2) << lcw) + l]);            // rms: (x * s) * w
    const float mv = mx / (float)hc;
    mixed[(size_t)t2 * d + col] = mv;
    if (aop) {          // the f16 operand of the GEMM that follows: the token scaled by the power of two of a bound of its largest magnitude
      float b = bnd[t2 * 4];
#pragma unroll
      for (int qs = 1; qs < 4; ++qs) if (qs < hc) b = fmaxf(b, bnd[t2 * 4 + qs]);
      b = b == b ? b : INFINITY;
      float upf, dn; hc_scale_of(b, &upf, &dn);
      aop_store(aop, aop_rows, col, t2, mv * upf);
      if (blockIdx.x == 0 && l == 0) for (int sb = 0; sb < aop_nsb; ++sb) aop_inv[sb * 8 + t2] = dn;
    }
    if (ROUTE) lo[t2 * 64 + l] = mv;
  }
  if (ROUTE) {
    lds_barrier();
    // the digits of the workgroup's 64 columns for the expert products that follow: token t2 by wave nw - 1 - t2 (the waves the router's tiles leave idle)
    if (dgx && lcw == 6) for (int t2 = nw - 1 - wave; t2 < T; t2 += nw) digits_eo_wave(lo[t2 * 64 + lane], lane, dsm[ROUTE ? t2 : 0], dgx + ((size_t)t2 * (d >> 6) + blockIdx.x) * DGX_STRIDE);
    const size_t rr64 = (size_t)router.tiles * 64;
    for (int tile = rtile; rwave && tile < rnt; tile += nw) {          // (more tiles than waves: one set, the tiles in turns)
      if (tile != rtile) rraw = unit_load<RFX>(router, tile, blockIdx.x, lane);
#pragma unroll 1
      for (int t2 = rset; t2 < T; t2 += rsets) {
        float ra[1] = {0.0f};
        unit_fma<RFX, 1>(router, rraw, blockIdx.x, lds2, lane, lo + t2 * 64, 0, ra);
        rpart[((size_t)blockIdx.x * T + t2) * rr64 + (size_t)tile * 64 + lane] = ra[0];
      }
    }
  }
  PYRE_TS(7); PYRE_TS_FLUSH(hc_ts, ROUTE ? 32 : 40);
}

__global__ void k_hc_combine(float* __restrict__ x, const float* __restrict__ out, const float* __restrict__ inj, int d, int hc) {
  int i = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.y, ti = blockIdx.z; if (i >= d) return;
  float w = 2.0f * sigm(inj[ti * hc + s]);
  x[((size_t)ti * hc + s) * d + i] += out[(size_t)ti * d + i] * w;
}

namespace {
// Waves per workgroup and units per wave of k_hc_norm_down: a workgroup's columns must lie inside one stream, and at
// most 32 K slices fit the slice-sum buffer.
struct DownPlan { int nw, upw, ksplit; };
DownPlan down_plan(const HcDev& h) {
  int ud = h.d / 64, nw = 8; while (nw > 1 && ud % nw) nw >>= 1;
  int upw = 1; while ((h.di.U / (nw * upw)) > 32 && (ud / nw) % (2 * upw) == 0) upw *= 2;
  return DownPlan{nw, upw, h.di.U / (nw * upw)};
}

template <int FMT, int T> int norm_down_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, const DownPlan& p, const float* x_in, int in_ss, int in_ts, float* x_out,
                                               const float* comb_out, int comb_parts, const MoeOut& mo, const float* comb_inj, float eps) {
  const int L = p.nw * p.upw * 64; size_t lds = 4 * ((size_t)T * L + (size_t)p.nw * T * 64 + (size_t)p.nw * T);
  ProfScope ps(ctx, "hc_norm_down", qmat_gguf_bytes(h.di, h.di.rows) + 4.0 * T * h.hc * h.d * 4);
#define NORM_DOWN_GO(NP) hipLaunchKernelGGL((k_hc_norm_down<FMT, T, NP>), dim3(h.di.tiles, p.ksplit), dim3(p.nw * 64), lds, ctx->stream, h.di, x_in, in_ss, in_ts, x_out, comb_out, mo, comb_inj, h.norm, h.d, h.hc, \
                     w.ssq, w.o, p.upw, (const uint2*)ctx->d_iq2xs)
  if constexpr (FMT == FMT_IQ3_S) { if (comb_parts > 1) NORM_DOWN_GO(PYRE_GEMV_PARTS); else NORM_DOWN_GO(1); } else NORM_DOWN_GO(1);
#undef NORM_DOWN_GO
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
template <int FMT, int T> int up_mix_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, int ksplit, const float* xnew, float eps, float* mixed, float* inj, const HcRoute* rt) {
  const int nw = h.hc * h.up.U; size_t lds = 4 * ((size_t)T * h.lr + (size_t)nw * T * 64 + (size_t)T * 32 + (size_t)T * h.hc * 64);
  const QMatDev rq = rt ? rt->router : QMatDev{}; float* rp = rt ? rt->part : nullptr;
  ProfScope ps(ctx, rt ? "hc_up_mix_router" : "hc_up_mix", qmat_gguf_bytes(h.up, h.up.rows) + 4.0 * T * (h.hc * h.d + h.d + (double)ksplit * (h.lr + h.hc)) +
               (rt ? qmat_gguf_bytes(rq, rq.rows) + 4.0 * T * (h.d / 64) * rq.tiles * 64 : 0.0));
#define UP_MIX_GO(RF) hipLaunchKernelGGL((k_hc_up_mix<FMT, T, RF>), dim3(h.d / 64), dim3(nw * 64), lds, ctx->stream, h.up, w.o, w.ssq, ksplit, h.di.tiles * 64, h.lr, h.hc, h.has_inject ? 1 : 0, xnew, h.norm, eps, \
                     h.d, mixed, inj, (const uint2*)ctx->d_iq2xs, rq, rp)
  if constexpr (FMT == FMT_IQ3_S || FMT == FMT_BF16 || FMT == FMT_F16 || FMT == FMT_F32) {
    if (rt && rq.fmt == FMT_BF16) UP_MIX_GO(FMT_BF16); else if (rt && rq.fmt == FMT_F32) UP_MIX_GO(FMT_F32); else UP_MIX_GO(-1);
  } else UP_MIX_GO(-1);
#undef UP_MIX_GO
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
int hc_m_cs(const HcDev& h) { return h.d % 512 == 0 ? 2 : 1; }      // columns a thread of k_hc_norm_down_m prepares
int hc_m_slices(const HcDev& h) { return h.hc * h.d / (256 * hc_m_cs(h)); }
bool hc_on_matrix_cores(const HcDev& h) {
  static const bool off = [] { const char* e = getenv("PYRE_HC_ROWS"); return e && *e && atoi(e) != 0; }();      // 1: the lane = row kernels for every window width
  return !off && h.di_m.fmt == FMT_IQ3_S_M && h.up_m.fmt == FMT_IQ3_S_M && h.d % 256 == 0 && hc_m_slices(h) <= 16 && h.lr % 256 == 0 && h.hc * 4 <= 16 && h.di_m.tiles == h.di.tiles;
}
template <int T> int norm_down_m_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, const float* x_in, int in_ss, int in_ts, float* x_out, const float* comb_out, int comb_parts, const MoeOut& mo, const float* comb_inj) {
  ProfScope ps(ctx, "hc_norm_down", qmat_gguf_bytes(h.di, h.di.rows) + 4.0 * T * h.hc * h.d * 4);
#define NORM_DOWN_M_GO(NP, CS) hipLaunchKernelGGL((k_hc_norm_down_m<T, NP, CS>), dim3(h.di_m.tiles, hc_m_slices(h), ctx->batch_n), dim3(256 * CS), 0, ctx->stream, h.di_m, x_in, in_ss, in_ts, x_out, comb_out, mo, comb_inj, h.norm, h.d, h.hc, w.ssq, w.o, w.smx, ctx->batch_stride)
#define NORM_DOWN_M_FIX(NP) hipLaunchKernelGGL((k_hc_norm_down_m<T, NP, 2, 2048, 10>), dim3(h.di_m.tiles, hc_m_slices(h), ctx->batch_n), dim3(512), 0, ctx->stream, h.di_m, x_in, in_ss, in_ts, x_out, comb_out, mo, comb_inj, h.norm, h.d, h.hc, w.ssq, w.o, w.smx, ctx->batch_stride)
  bool done = false;
  {          // the width of the A3B configuration: the instances with its constants folded in
    if (h.d == 2048 && (!mo.partial || mo.k == 10)) { if (comb_parts > 1) NORM_DOWN_M_FIX(PYRE_GEMV_PARTS); else NORM_DOWN_M_FIX(1); done = true; }
  }
  if (done) {}
  else if (hc_m_cs(h) == 2) { if (comb_parts > 1) NORM_DOWN_M_GO(PYRE_GEMV_PARTS, 2); else NORM_DOWN_M_GO(1, 2); }
  else { if (comb_parts > 1) NORM_DOWN_M_GO(PYRE_GEMV_PARTS, 1); else NORM_DOWN_M_GO(1, 1); }
#undef NORM_DOWN_M_GO
#undef NORM_DOWN_M_FIX
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
// columns of the mixed vector a workgroup of the matrix-core up / mix launch owns (log2): a single token without a riding
// router spreads over d / 16 workgroups, everything else keeps 64 (the router rides in units of 64 columns; a window's
// prologue grows with its width and would be redone by four times as many workgroups)
int hc_m_lcw(const HcDev& h, int t, bool route) {
  static const int force = [] { const char* e = getenv("PYRE_HC_CW"); return e && *e ? atoi(e) : 0; }();      // 16 / 32 / 64: one width for every launch without a router
  if (route) return 6;
  if (force == 16) return 4; if (force == 32) return 5; if (force == 64) return 6;
  return t == 1 ? 4 : 6;
}
template <int T> int up_mix_m_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, int ksplit, const float* xnew, float eps, float* mixed, float* inj, const HcRoute* rt, const AopOut* aop) {
  const int lcw = hc_m_lcw(h, T, rt != nullptr), nw = h.hc << (lcw - 4); const size_t lds = 4 * ((size_t)T * h.lr + (size_t)h.hc * T * 64 + (size_t)T * 16 + 8 + 32) + (size_t)h.lr * 32;
  const QMatDev rq = rt ? rt->router : QMatDev{}; float* rp = rt ? rt->part : nullptr;
  ProfScope ps(ctx, rt ? "hc_up_mix_router" : "hc_up_mix", qmat_gguf_bytes(h.up, h.up.rows) + 4.0 * T * (h.hc * h.d + h.d + (double)ksplit * (h.lr + h.hc)) +
               (rt ? qmat_gguf_bytes(rq, rq.rows) + 4.0 * T * (h.d / 64) * rq.tiles * 64 : 0.0));
#define UP_MIX_M_ARGS dim3(h.d >> lcw, 1, ctx->batch_n), dim3(nw * 64), lds, ctx->stream, h.up_m, w.o, w.ssq, ksplit, h.di.tiles * 64, h.lr, h.hc, h.has_inject ? 1 : 0, xnew, h.norm, eps, \
                     h.d, mixed, inj, rq, rp, aop ? aop->op : nullptr, pyre_aop_rows(T), lcw, w.smx, aop ? aop->ainv : nullptr, aop ? aop->nsb : 0, rt ? rt->dgx : nullptr, ctx->batch_stride
#define UP_MIX_M_GO(RF) hipLaunchKernelGGL((k_hc_up_mix_m<T, RF>), UP_MIX_M_ARGS)
#define UP_MIX_M_FIX(RF) hipLaunchKernelGGL((k_hc_up_mix_m<T, RF, 4, 256, 16>), UP_MIX_M_ARGS)
  bool done = false;
  {          // four streams, a low rank of 256 and sixteen slices (the A3B configuration): constants folded in
    if (h.hc == 4 && h.lr == 256 && ksplit == 16) { if (rt && rq.fmt == FMT_BF16) UP_MIX_M_FIX(FMT_BF16); else if (rt && rq.fmt == FMT_F32) UP_MIX_M_FIX(FMT_F32); else UP_MIX_M_FIX(-1); done = true; }
  }
  if (done) {}
  else if (rt && rq.fmt == FMT_BF16) UP_MIX_M_GO(FMT_BF16); else if (rt && rq.fmt == FMT_F32) UP_MIX_M_GO(FMT_F32); else UP_MIX_M_GO(-1);
#undef UP_MIX_M_FIX
#undef UP_MIX_M_ARGS
#undef UP_MIX_M_GO
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
#define HC_M_T_SWITCH(FN, ...) \
  switch (t) { case 1: return FN<1>(__VA_ARGS__); case 2: return FN<2>(__VA_ARGS__); case 3: return FN<3>(__VA_ARGS__); case 4: return FN<4>(__VA_ARGS__); \
    case 5: return FN<5>(__VA_ARGS__); case 6: return FN<6>(__VA_ARGS__); case 7: return FN<7>(__VA_ARGS__); default: return FN<8>(__VA_ARGS__); }
int norm_down_m(pyre_ctx* ctx, const HcDev& h, const HcWork& w, const float* x_in, int in_ss, int in_ts, float* x_out, int t, const float* comb_out, int comb_parts, const MoeOut& mo, const float* comb_inj) {
  HC_M_T_SWITCH(norm_down_m_launch, ctx, h, w, x_in, in_ss, in_ts, x_out, comb_out, comb_parts, mo, comb_inj)
}
int up_mix_m(pyre_ctx* ctx, const HcDev& h, const HcWork& w, int ksplit, int t, const float* xnew, float eps, float* mixed, float* inj, const HcRoute* rt, const AopOut* aop) {
  HC_M_T_SWITCH(up_mix_m_launch, ctx, h, w, ksplit, xnew, eps, mixed, inj, rt, aop)
}
#define HC_T_SWITCH(F, FN, ...) \
  switch (t) { case 1: return FN<F, 1>(__VA_ARGS__); case 2: return FN<F, 2>(__VA_ARGS__); case 3: return FN<F, 3>(__VA_ARGS__); case 4: return FN<F, 4>(__VA_ARGS__); \
    case 5: return FN<F, 5>(__VA_ARGS__); case 6: return FN<F, 6>(__VA_ARGS__); case 7: return FN<F, 7>(__VA_ARGS__); default: return FN<F, 8>(__VA_ARGS__); }
#define HC_FMT_SWITCH(fmt, BODY) \
  switch (fmt) { case FMT_F32: { constexpr int F = FMT_F32; BODY } case FMT_F16: { constexpr int F = FMT_F16; BODY } case FMT_BF16: { constexpr int F = FMT_BF16; BODY } \
    case FMT_Q8_0: { constexpr int F = FMT_Q8_0; BODY } case FMT_Q4_K: { constexpr int F = FMT_Q4_K; BODY } case FMT_IQ2_XS: { constexpr int F = FMT_IQ2_XS; BODY } \
    case FMT_C4: { constexpr int F = FMT_C4; BODY } case FMT_C8: { constexpr int F = FMT_C8; BODY } \
    default: { constexpr int F = FMT_IQ3_S; BODY } }
int norm_down(pyre_ctx* ctx, const HcDev& h, const HcWork& w, const DownPlan& p, const float* x_in, int in_ss, int in_ts, float* x_out, int t, const float* comb_out, int comb_parts, const MoeOut& mo, const float* comb_inj, float eps) {
  HC_FMT_SWITCH(h.di.fmt, HC_T_SWITCH(F, norm_down_launch, ctx, h, w, p, x_in, in_ss, in_ts, x_out, comb_out, comb_parts, mo, comb_inj, eps))
}
int up_mix(pyre_ctx* ctx, const HcDev& h, const HcWork& w, int ksplit, int t, const float* xnew, float eps, float* mixed, float* inj, const HcRoute* rt) {
  HC_FMT_SWITCH(h.up.fmt, HC_T_SWITCH(F, up_mix_launch, ctx, h, w, ksplit, xnew, eps, mixed, inj, rt))
}
}  // namespace

bool pyre_hc_aop_ok(const HcDev& h) { return hc_on_matrix_cores(h) && h.hc <= 4; }
bool pyre_hc_route_ok(const HcDev& h, const QMatDev& router) {
  const int f = h.up.fmt;
  return (f == FMT_IQ3_S || f == FMT_BF16 || f == FMT_F16 || f == FMT_F32) && (router.fmt == FMT_BF16 || router.fmt == FMT_F32) && router.cols == h.d && h.d / 64 <= 64 && router.U == h.d / 64;
}
bool pyre_hc_plan(const HcDev& h, int* nw, int* upw, int* ksplit) {
  if (h.d % 64 || h.lr % 64 || h.hc * h.up.U > 16 || h.up.tiles != h.hc * (h.d / 64) || h.di.U != h.hc * (h.d / 64)) return false;
  DownPlan p = down_plan(h); *nw = p.nw; *upw = p.upw; *ksplit = p.ksplit;
  return p.ksplit >= 1 && p.ksplit <= 32 && p.ksplit * p.nw * p.upw == h.di.U;
}
size_t pyre_hc_work_bytes(const HcDev& h) { return 256 * 4 + 2 * 4 * 8 * 32 + 4 * 8 * 32 * ((size_t)h.lr + h.hc + 64); }
void pyre_hc_work_carve(const HcDev& h, void* base, HcWork* w) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  w->ssq = (float*)take(4 * 8 * 32); w->smx = (float*)take(4 * 8 * 32); w->o = (float*)take(4 * 8 * 32 * ((size_t)h.lr + h.hc + 64));
}

int pyre_hc_mix_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, const float* x_in, int in_ss, int in_ts, float* x_out, int t, const float* comb_out, const MoeOut* comb_moe, const float* comb_inj,
                       float eps, float* mixed, float* inj, const HcRoute* route, int comb_parts, const AopOut* aop) {
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: t = %d outside 1..8", t);
  if (comb_parts != 1 && !(comb_parts == PYRE_GEMV_PARTS && h.di.fmt == FMT_IQ3_S && comb_out && !comb_moe)) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: %d partial vectors (1, or %d with an IQ3_S mix)", comb_parts, PYRE_GEMV_PARTS);
  if (route && !pyre_hc_route_ok(h, route->router)) return pyre_fail(ctx, PYRE_E_SHAPE, "hc_mix: this router cannot ride on the mix");
  if (x_in == x_out) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: the updated streams must go to another buffer");
  if (h.d % 64 || h.lr % 64 || h.hc * h.up.U > 16 || h.up.tiles != h.hc * (h.d / 64) || h.di.U != h.hc * (h.d / 64))
    return pyre_fail(ctx, PYRE_E_SHAPE, "hc_mix: needs d and the low rank in multiples of 64 and hc * (low rank / 64) <= 16 (d %d, low rank %d, hc %d)", h.d, h.lr, h.hc);
  DownPlan p = down_plan(h);
  if (p.ksplit < 1 || p.ksplit > 32 || p.ksplit * p.nw * p.upw != h.di.U) return pyre_fail(ctx, PYRE_E_SHAPE, "hc_mix: d = %d cannot be cut into at most 32 slices of whole waves", h.d);
  const bool on_m = hc_on_matrix_cores(h);
  if (ctx->batch_n > 1 && !on_m) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: only the matrix-core mix serves several windows a launch");
  if (aop && !(on_m && aop->op && aop->ainv && aop->nsb >= 1 && h.hc <= 4)) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: only the matrix-core mix leaves an operand (pyre_hc_aop_ok)");
  MoeOut mo = comb_moe ? *comb_moe : MoeOut{nullptr, nullptr, nullptr, 0, 0};
  if (mo.partial && (mo.k > PYRE_MOE_KMAX || mo.d != h.d)) return pyre_fail(ctx, PYRE_E_SHAPE, "hc_mix: unreduced FFN output with top_k %d / width %d", mo.k, mo.d);
  if (on_m) {
    int rc = norm_down_m(ctx, h, w, x_in, in_ss, in_ts, x_out, t, comb_out, comb_parts, mo, comb_inj); if (rc) return rc;
    return up_mix_m(ctx, h, w, hc_m_slices(h), t, x_out, eps, mixed, inj, route, aop);
  }
  int rc = norm_down(ctx, h, w, p, x_in, in_ss, in_ts, x_out, t, comb_out, comb_parts, mo, comb_inj, eps); if (rc) return rc;
  return up_mix(ctx, h, w, p.ksplit, t, x_out, eps, mixed, inj, route);
}

int pyre_hc_combine_launch(pyre_ctx* ctx, int d, int hc, float* x, int t, const float* out, const float* inj) {
  { ProfScope ps(ctx, "hc_combine", 4.0 * t * d * (2 * hc + 1)); hipLaunchKernelGGL(k_hc_combine, dim3((d + 255) / 256, hc, t), dim3(256), 0, ctx->stream, x, out, inj, d, hc); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
