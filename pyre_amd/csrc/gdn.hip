// Gated DeltaNet recurrent step: causal depthwise conv1d + SiLU, L2-normalised q/k, gated delta rule on the fp32
// state kept resident in HBM, gated RMSNorm.  Follows linear_core, src/model/qwen4exp_gguf.rs:1624-1673.
#include "formats.h"
PYRE_TS_DECL(gdn_ts) PYRE_TS_EXPORT(gdn_ts, pyre_debug_ts_gdn)

__device__ __forceinline__ float g_sigm(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float g_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// grid ceil(ch/256): channel c runs its t tokens in order (:1643-1647): o = w[k-1]*cur + sum_j w[j]*state[j], co = silu(o),
// then the window slides.  State rows are oldest first.
__global__ __launch_bounds__(256) void k_gdn_conv(const float* __restrict__ proj, int stride, int t, int ch, int kk, const float* __restrict__ conv_w,
                                                  const float* __restrict__ conv_in, float* __restrict__ conv_out, float* __restrict__ co) {
  int c = blockIdx.x * 256 + threadIdx.x; if (c >= ch) return;
  float w[8], hist[8];
  for (int k = 0; k < kk; ++k) w[k] = conv_w[(size_t)c * kk + k];
  for (int k = 0; k < kk - 1; ++k) hist[k] = conv_in[(size_t)k * ch + c];
  for (int ti = 0; ti < t; ++ti) {
    float cur = proj[(size_t)ti * stride + c];
    float o = w[kk - 1] * cur;
    for (int k = 0; k < kk - 1; ++k) o += w[k] * hist[k];
    co[(size_t)ti * ch + c] = o * g_sigm(o);
    for (int k = 0; k + 1 < kk - 1; ++k) hist[k] = hist[k + 1];
    hist[kk - 2] = cur;
  }
  for (int k = 0; k < kk - 1; ++k) conv_out[(size_t)k * ch + c] = hist[k];
}

// The same for n consecutive windows of t tokens in one launch (a long prompt's blocks): grid (ceil(ch/256), n).  Window z's
// projection rows lie at proj + z * ws, its output at co + z * ws (the windows' workspaces, ws floats apart); its history is
// the last kk - 1 rows of window z - 1's projection -- for window 0 the kk - 1 rows at prev (row stride prev_stride: the
// layer's convolution state, or the projection rows of the window in front of the group).  The last window leaves the state
// in conv_out if that is given.  A channel's arithmetic is k_gdn_conv's, so are its bits.  Needs t >= kk - 1.
__global__ __launch_bounds__(256) void k_gdn_conv_blk(const float* __restrict__ proj, int stride, int t, int ch, int kk, const float* __restrict__ conv_w, size_t ws,
                                                      const float* __restrict__ prev, int prev_stride, float* __restrict__ conv_out, float* __restrict__ co) {
  const int c = blockIdx.x * 256 + threadIdx.x, z = blockIdx.y; if (c >= ch) return;
  const float* pz = proj + (size_t)z * ws;
  float w[8], hist[8];
  for (int k = 0; k < kk; ++k) w[k] = conv_w[(size_t)c * kk + k];
  if (z == 0) { for (int k = 0; k < kk - 1; ++k) hist[k] = prev[(size_t)k * prev_stride + c]; }
  else { const float* pp = pz - ws + (size_t)(t - (kk - 1)) * stride; for (int k = 0; k < kk - 1; ++k) hist[k] = pp[(size_t)k * stride + c]; }
  float* cz = co + (size_t)z * ws;
  for (int ti = 0; ti < t; ++ti) {
    float cur = pz[(size_t)ti * stride + c];
    float o = w[kk - 1] * cur;
    for (int k = 0; k < kk - 1; ++k) o += w[k] * hist[k];
    cz[(size_t)ti * ch + c] = o * g_sigm(o);
    for (int k = 0; k + 1 < kk - 1; ++k) hist[k] = hist[k + 1];
    hist[kk - 2] = cur;
  }
  if (conv_out && z == (int)gridDim.y - 1) for (int k = 0; k < kk - 1; ++k) conv_out[(size_t)k * ch + c] = hist[k];
}

// grid nv, 512 threads (8 waves), at most 8 tokens.  Thread (grp = tid/128, j = tid%128) keeps rows 32*grp..32*grp+31 of
// column j of the head's 128x128 state in registers across the whole window, so the state is read once and written once
// per launch.  Whatever does not depend on the state is done per token by one wave each, before the recurrence (wave ti
// fetches token ti's q, k, v, z and gate inputs -- eight requests a lane, all tokens in flight together -- and leaves
// the L2-normalised q and k, v, z, the decay and beta in shared memory) and after it (wave ti: RMSNorm and gate of token
// ti's output).  A token of the recurrence itself costs one barrier:
//   S *= g; mem = S^T k -> barrier -> delta = (v - mem) beta; S += k (x) delta; o = S^T q      (linear_core, :1655-1668)
// FT, FNK, FNV > 0: the window width and the head counts as compile-time constants (the launcher checks them) -- same arithmetic.
template <int DK, int DV, int FT = 0, int FNK = 0, int FNV = 0>
__global__ __launch_bounds__(512) void k_gdn_delta(GdnDev p, const float* __restrict__ proj, int stride, int t, const float* __restrict__ co_all,
                                                   const float* __restrict__ ssm_in, float* __restrict__ ssm_out, float* __restrict__ out, uint16_t* __restrict__ aop, int aop_rows, float aop_up) {
  static_assert(DK == 128 && DV == 128, "tiling assumes 128x128 heads");
  constexpr int G = 4, R = DK / G, MT = 8;
  PYRE_TS_VARS PYRE_TS(0);
  args_now(p.a, p.dt, p.norm_w, p.nk, p.nv, p.eps, proj, stride, t, co_all, ssm_in, ssm_out, out);
  if constexpr (FT > 0) { t = FT; p.nk = FNK; p.nv = FNV; }
  __shared__ float qs[MT][DK], ks[MT][DK], vs[MT][DV], zs[MT][DV], pm[2][G][DV], po[MT][G][DV], gs[MT], bs[MT];
  const int h = blockIdx.x, kh = h % p.nk, tid = threadIdx.x, j = tid & (DV - 1), grp = tid >> 7, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ch = 2 * p.nk * DK + p.nv * DV, w = p.nv * DV;
  const float* sin_ = ssm_in + (size_t)h * DK * DV; float* sout = ssm_out + (size_t)h * DK * DV;
  float q0 = 0.0f, q1 = 0.0f, k0 = 0.0f, k1 = 0.0f, v0 = 0.0f, v1 = 0.0f, z0 = 0.0f, z1 = 0.0f, alpha_raw = 0.0f, beta_raw = 0.0f;
  if (wave < t) {
    const float* co = co_all + (size_t)wave * ch; const float* pr = proj + (size_t)wave * stride;
    q0 = co[kh * DK + lane]; q1 = co[kh * DK + lane + 64]; k0 = co[p.nk * DK + kh * DK + lane]; k1 = co[p.nk * DK + kh * DK + lane + 64];
    v0 = co[2 * p.nk * DK + h * DV + lane]; v1 = co[2 * p.nk * DK + h * DV + lane + 64];
    z0 = pr[ch + h * DV + lane]; z1 = pr[ch + h * DV + lane + 64];                      // z at [ch + h*dv + j]
    alpha_raw = pr[ch + w + p.nv + h]; beta_raw = pr[ch + w + h];                        // alpha at [ch + nv*dv + nv + h], beta at [ch + nv*dv + h]
  }
  const float a = p.a[h], dtb = p.dt[h], nw0 = p.norm_w[lane], nw1 = p.norm_w[lane + 64];
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = sin_[(size_t)(grp * R + r) * DV + j];
  auto wsum = [](float x) { return wave_sum(x); };
  if (wave < t) {          // L2 norms of q and k (:1649-1651): the sum of each half of the vector, then the two halves
    const float sq = wsum(q0 * q0) + wsum(q1 * q1), sk = wsum(k0 * k0) + wsum(k1 * k1);
    const float fq = (1.0f / sqrtf(sq + 1e-6f)) * (1.0f / sqrtf((float)DK)), fk = (1.0f / sqrtf(sk + 1e-6f)) * 1.0f;
    qs[wave][lane] = q0 * fq; qs[wave][lane + 64] = q1 * fq; ks[wave][lane] = k0 * fk; ks[wave][lane + 64] = k1 * fk;
    vs[wave][lane] = v0; vs[wave][lane + 64] = v1; zs[wave][lane] = z0; zs[wave][lane + 64] = z1;
    if (lane == 0) { gs[wave] = expf(g_softplus(alpha_raw + dtb) * a); bs[wave] = g_sigm(beta_raw); }
  }
  lds_barrier(); PYRE_TS(1);
  for (int ti = 0; ti < t; ++ti) {
    const float g = gs[ti], b = bs[ti];
    float pmv = 0.0f;
#pragma unroll
    for (int r = 0; r < R; ++r) { S[r] *= g; pmv += S[r] * ks[ti][grp * R + r]; }
    pm[ti & 1][grp][j] = pmv;
    lds_barrier();
    const float mem = ((pm[ti & 1][0][j] + pm[ti & 1][1][j]) + pm[ti & 1][2][j]) + pm[ti & 1][3][j];
    const float delta = (vs[ti][j] - mem) * b;
    float pov = 0.0f;
#pragma unroll
    for (int r = 0; r < R; ++r) { S[r] += ks[ti][grp * R + r] * delta; pov += S[r] * qs[ti][grp * R + r]; }
    po[ti][grp][j] = pov;
  }
  PYRE_TS(2);
#pragma unroll
  for (int r = 0; r < R; ++r) sout[(size_t)(grp * R + r) * DV + j] = S[r];
  lds_barrier(); PYRE_TS(3);
  if (wave < t) {
    const float o0 = ((po[wave][0][lane] + po[wave][1][lane]) + po[wave][2][lane]) + po[wave][3][lane];
    const float o1 = ((po[wave][0][lane + 64] + po[wave][1][lane + 64]) + po[wave][2][lane + 64]) + po[wave][3][lane + 64];
    const float sc = 1.0f / sqrtf((wsum(o0 * o0) + wsum(o1 * o1)) / (float)DV + p.eps);
    const float r0 = (o0 * (sc * nw0)) * g_sigm(zs[wave][lane]), r1 = (o1 * (sc * nw1)) * g_sigm(zs[wave][lane + 64]);      // rms_inplace: x *= s * w  (:210)
    out[(size_t)wave * w + h * DV + lane] = r0; out[(size_t)wave * w + h * DV + lane + 64] = r1;
    if (aop) { aop_store(aop, aop_rows, h * DV + lane, wave, r0 * aop_up); aop_store(aop, aop_rows, h * DV + lane + 64, wave, r1 * aop_up); }      // the f16 operand of the output projection (matrix-core layout), scaled by the layer's power of two
  }
  PYRE_TS(4); PYRE_TS(5); PYRE_TS(6); PYRE_TS(7); PYRE_TS_FLUSH(gdn_ts, 0);
}

// The same recurrence on nv x 4 workgroups: workgroup (h, q) owns the 32 columns 32*q .. of head h's state (the columns of
// the delta rule are independent), 16 KB instead of 64 KB to fetch and to store.  Thread (rg = tid/32, j = tid%32) keeps rows
// 8*rg .. 8*rg+7 of column 32*q + j; the sixteen row groups' sums meet in shared memory in order.  The head's RMS norm needs
// all 128 columns, so it is left to the consumer (the output projection, PyreAop::sq): wave ti leaves token ti's
// un-normalised gated output u = (o * norm_w) * sigmoid(z) of its 32 columns as f16 operand rows scaled by the quarter's own
// power of two (its largest magnitude into [2^13, 2^14)), that factor's inverse, and the quarter's sum of o^2.
// nwin > 1 (a long prompt's blocks): nwin consecutive windows of t tokens in one launch -- window wi's projection, convolution
// output, operand rows and sums lie ws floats further on per window (the windows' workspaces); the state stays in registers
// from window to window, is fetched once and stored once.  A token's arithmetic is the same whatever nwin.
template <int DK, int DV, int FT = 0, int FNK = 0, int FNV = 0>
__global__ __launch_bounds__(512) void k_gdn_delta_q(GdnDev p, const float* __restrict__ proj, int stride, int t, const float* __restrict__ co_all,
                                                     const float* __restrict__ ssm_in, float* __restrict__ ssm_out, uint16_t* __restrict__ aop, int aop_rows, float* __restrict__ sq, int nwin, size_t ws) {
  static_assert(DK == 128 && DV == 128, "tiling assumes 128x128 heads");
  constexpr int QC = 32, G = 16, R = DK / G, MT = 8;
  args_now(p.a, p.dt, p.norm_w, p.nk, p.nv, p.eps, proj, stride, t, co_all, ssm_in, ssm_out, aop, sq);
  if constexpr (FT > 0) { t = FT; p.nk = FNK; p.nv = FNV; }
  __shared__ float qs[MT][DK], ks[MT][DK], vs[MT][QC], zs[MT][QC], pm[2][G][QC], po[MT][G][QC], gs[MT], bs[MT];
  const int h = blockIdx.x, qd = blockIdx.y, kh = h % p.nk, tid = threadIdx.x, j = tid & (QC - 1), rg = tid >> 5, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ch = 2 * p.nk * DK + p.nv * DV, w = p.nv * DV, jc = qd * QC + j;
  const float* sin_ = ssm_in + (size_t)h * DK * DV; float* sout = ssm_out + (size_t)h * DK * DV;
  float q0 = 0.0f, q1 = 0.0f, k0 = 0.0f, k1 = 0.0f, v0 = 0.0f, z0 = 0.0f, alpha_raw = 0.0f, beta_raw = 0.0f;
  auto fetch = [&](int wi) {          // wave ti: token ti's inputs of window wi
    if (wave < t) {
      const float* co = co_all + (size_t)wi * ws + (size_t)wave * ch; const float* pr = proj + (size_t)wi * ws + (size_t)wave * stride;
      q0 = co[kh * DK + lane]; q1 = co[kh * DK + lane + 64]; k0 = co[p.nk * DK + kh * DK + lane]; k1 = co[p.nk * DK + kh * DK + lane + 64];
      v0 = co[2 * p.nk * DK + h * DV + qd * QC + (lane & 31)]; z0 = pr[ch + h * DV + qd * QC + (lane & 31)];
      alpha_raw = pr[ch + w + p.nv + h]; beta_raw = pr[ch + w + h];
    }
  };
  fetch(0);
  const float a = p.a[h], dtb = p.dt[h], nw = p.norm_w[qd * QC + (lane & 31)];
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = sin_[(size_t)(rg * R + r) * DV + jc];
  for (int wi = 0; wi < nwin; ++wi) {
    if (wave < t) {          // L2 norms of q and k (:1649-1651): the sum of each half of the vector, then the two halves -- as in k_gdn_delta
      const float sq_ = wave_sum(q0 * q0) + wave_sum(q1 * q1), sk = wave_sum(k0 * k0) + wave_sum(k1 * k1);
      const float fq = (1.0f / sqrtf(sq_ + 1e-6f)) * (1.0f / sqrtf((float)DK)), fk = (1.0f / sqrtf(sk + 1e-6f)) * 1.0f;
      qs[wave][lane] = q0 * fq; qs[wave][lane + 64] = q1 * fq; ks[wave][lane] = k0 * fk; ks[wave][lane + 64] = k1 * fk;
      if (lane < QC) { vs[wave][lane] = v0; zs[wave][lane] = z0; }
      if (lane == 0) { gs[wave] = expf(g_softplus(alpha_raw + dtb) * a); bs[wave] = g_sigm(beta_raw); }
    }
    if (wi + 1 < nwin) fetch(wi + 1);          // the next window's inputs travel behind this window's recurrence
    lds_barrier();
    for (int ti = 0; ti < t; ++ti) {
      const float g = gs[ti], b = bs[ti];
      float pmv = 0.0f;
#pragma unroll
      for (int r = 0; r < R; ++r) { S[r] *= g; pmv += S[r] * ks[ti][rg * R + r]; }
      pm[ti & 1][rg][j] = pmv;
      lds_barrier();
      float mem = pm[ti & 1][0][j];
#pragma unroll
      for (int k = 1; k < G; ++k) mem += pm[ti & 1][k][j];
      const float delta = (vs[ti][j] - mem) * b;
      float pov = 0.0f;
#pragma unroll
      for (int r = 0; r < R; ++r) { S[r] += ks[ti][rg * R + r] * delta; pov += S[r] * qs[ti][rg * R + r]; }
      po[ti][rg][j] = pov;
    }
    if (wi + 1 == nwin) {
#pragma unroll
      for (int r = 0; r < R; ++r) sout[(size_t)(rg * R + r) * DV + jc] = S[r];
    }
    lds_barrier();
    if (wave < t) {
      const int jl = lane & 31; const bool on = lane < QC;
      float o = po[wave][0][jl];
#pragma unroll
      for (int k = 1; k < G; ++k) o += po[wave][k][jl];
      const float ss = wave_sum(on ? o * o : 0.0f);
      const float u = (o * nw) * g_sigm(zs[wave][jl]);
      float am = on ? fabsf(u) : 0.0f; am = am == am ? am : INFINITY;
      am = wave_max(am);
      int e = 0;
      if (am > 0.0f && am < INFINITY) { e = 140 - (int)((__float_as_uint(am) >> 23) & 0xFF); e = e > 100 ? 100 : e; }
      uint16_t* aw = aop + (size_t)wi * ws * 2; float* sw = sq + (size_t)wi * ws;
      if (on) aop_store(aw, aop_rows, h * DV + qd * QC + jl, wave, u * __uint_as_float((uint32_t)(127 + e) << 23));
      if (lane == 0) { sw[((size_t)wave * p.nv + h) * 4 + qd] = __uint_as_float((uint32_t)(127 - e) << 23); sw[(size_t)8 * p.nv * 4 + ((size_t)wave * p.nv + h) * 4 + qd] = ss; }
    }
    if (wi + 1 < nwin) lds_barrier();          // the next window's inputs overwrite what this window's outputs were read from
  }
}

int pyre_gdn_launch(pyre_ctx* ctx, const GdnDev& g, const float* proj, int stride, int t, const float* conv_in, float* conv_out,
                    const float* ssm_in, float* ssm_out, float* co, float* out, bool conv_done, uint16_t* aop, float aop_up, const GdnQ* gq, int nwin, size_t ws) {
  if (nwin < 1 || (nwin > 1 && !(gq && conv_done))) return pyre_fail(ctx, PYRE_E_ARG, "gdn: several windows a launch need the per-quarter form behind a finished convolution");
  if (aop && t > 8) return pyre_fail(ctx, PYRE_E_ARG, "gdn: an f16 operand holds at most 8 tokens, not %d", t);
  if (gq && (!gq->op || !gq->sq)) return pyre_fail(ctx, PYRE_E_ARG, "gdn: the per-quarter form needs its operand and scale arrays");
  if (g.dk != 128 || g.dv != 128) return pyre_fail(ctx, PYRE_E_SHAPE, "gdn: head dims %dx%d unsupported (128x128 only)", g.dk, g.dv);
  if (g.conv_k < 2 || g.conv_k > 8) return pyre_fail(ctx, PYRE_E_SHAPE, "gdn: conv kernel %d outside 2..8", g.conv_k);
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "gdn: t = %d outside 1..8", t);
  int ch = 2 * g.nk * g.dk + g.nv * g.dv;
  if (!conv_done) { ProfScope ps(ctx, "gdn_conv", 4.0 * ch * (2.0 * (g.conv_k - 1) + g.conv_k + 2.0 * t)); hipLaunchKernelGGL(k_gdn_conv, dim3((ch + 255) / 256), dim3(256), 0, ctx->stream, proj, stride, t, ch, g.conv_k, g.conv_w, conv_in, conv_out, co); } PYRE_CHECK_LAUNCH(ctx);
  if (gq) {
    ProfScope ps(ctx, "gdn_delta", 8.0 * g.nv * g.dk * g.dv + 4.0 * t * (ch + 2.0 * g.nv * g.dv));
#define GDN_Q_FIX(FT) hipLaunchKernelGGL((k_gdn_delta_q<128, 128, FT, 16, 32>), dim3(g.nv, 4), dim3(512), 0, ctx->stream, g, proj, stride, t, co, ssm_in, ssm_out, gq->op, pyre_aop_rows(t), gq->sq, nwin, ws)
    if (g.nk == 16 && g.nv == 32) {          // the A3B geometry: the window width and the head counts folded in
      switch (t) { case 1: GDN_Q_FIX(1); break; case 2: GDN_Q_FIX(2); break; case 3: GDN_Q_FIX(3); break; case 4: GDN_Q_FIX(4); break; case 5: GDN_Q_FIX(5); break; case 6: GDN_Q_FIX(6); break; case 7: GDN_Q_FIX(7); break; default: GDN_Q_FIX(8); break; }
    }
#undef GDN_Q_FIX
    else hipLaunchKernelGGL((k_gdn_delta_q<128, 128>), dim3(g.nv, 4), dim3(512), 0, ctx->stream, g, proj, stride, t, co, ssm_in, ssm_out, gq->op, pyre_aop_rows(t), gq->sq, nwin, ws);
    PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
  }
  { ProfScope ps(ctx, "gdn_delta", 8.0 * g.nv * g.dk * g.dv + 4.0 * t * (ch + 2.0 * g.nv * g.dv)); if (t == 1 && g.nk == 16 && g.nv == 32) hipLaunchKernelGGL((k_gdn_delta<128, 128, 1, 16, 32>), dim3(g.nv), dim3(512), 0, ctx->stream, g, proj, stride, t, co, ssm_in, ssm_out, out, aop, aop ? pyre_aop_rows(t) : 0, aop_up);          // a single token of the A3B geometry: constants folded in
    else hipLaunchKernelGGL((k_gdn_delta<128, 128>), dim3(g.nv), dim3(512), 0, ctx->stream, g, proj, stride, t, co, ssm_in, ssm_out, out, aop, aop ? pyre_aop_rows(t) : 0, aop_up); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

int pyre_gdn_conv_block_launch(pyre_ctx* ctx, const GdnDev& g, const float* proj, int stride, int t, int n, size_t ws, const float* prev, int prev_stride, float* conv_out, float* co) {
  if (g.conv_k < 2 || g.conv_k > 8 || t < g.conv_k - 1 || t > 8 || n < 1) return pyre_fail(ctx, PYRE_E_ARG, "gdn block conv: kernel %d, %d windows of %d tokens", g.conv_k, n, t);
  const int ch = 2 * g.nk * g.dk + g.nv * g.dv;
  ProfScope ps(ctx, "gdn_conv", 4.0 * ch * n * (g.conv_k + 2.0 * t));
  hipLaunchKernelGGL(k_gdn_conv_blk, dim3((ch + 255) / 256, n), dim3(256), 0, ctx->stream, proj, stride, t, ch, g.conv_k, g.conv_w, ws, prev, prev_stride, conv_out, co);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

// ---- C ABI: standalone layer core for the block harness ---------------------------------------------------------------
struct pyre_gdn {
  pyre_ctx* ctx; GdnDev dv; float* params; int ch, pw;      // pw = projection width per token
  float* conv[2]; float* ssm[2]; int cur; float* co; float* io; size_t io_tokens;
};

extern "C" {

int pyre_gdn_create(pyre_ctx* ctx, int nk, int nv, int dk, int dv, int conv_k, float eps, const float* a, const float* dt, const float* conv_w, const float* norm_w, pyre_gdn** out) {
  if (!ctx || !out || !a || !dt || !conv_w || !norm_w) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_create: null argument");
  *out = nullptr;
  if (dk != 128 || dv != 128 || nk < 1 || nv < 1 || nv % nk || conv_k < 2 || conv_k > 8) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_gdn_create: unsupported geometry nk %d nv %d dk %d dv %d conv %d", nk, nv, dk, dv, conv_k);
  pyre_gdn* g = new pyre_gdn(); g->ctx = ctx; g->ch = 2 * nk * dk + nv * dv; g->pw = g->ch + nv * dv + 2 * nv; g->cur = 0; g->io = nullptr; g->io_tokens = 0;
  size_t np = (size_t)2 * nv + (size_t)g->ch * conv_k + dv;
  std::vector<float> hp(np); memcpy(hp.data(), a, 4 * nv); memcpy(hp.data() + nv, dt, 4 * nv); memcpy(hp.data() + 2 * nv, conv_w, 4 * (size_t)g->ch * conv_k); memcpy(hp.data() + 2 * nv + (size_t)g->ch * conv_k, norm_w, 4 * dv);
  size_t cs = (size_t)(conv_k - 1) * g->ch, ss = (size_t)nv * dk * dv;
  hipError_t e = hipMalloc((void**)&g->params, np * 4);
  if (e == hipSuccess) e = hipMemcpy(g->params, hp.data(), np * 4, hipMemcpyHostToDevice);
  for (int i = 0; i < 2 && e == hipSuccess; ++i) { e = hipMalloc((void**)&g->conv[i], cs * 4); if (e == hipSuccess) e = hipMalloc((void**)&g->ssm[i], ss * 4);
    if (e == hipSuccess) e = hipMemset(g->conv[i], 0, cs * 4); if (e == hipSuccess) e = hipMemset(g->ssm[i], 0, ss * 4); }
  if (e == hipSuccess) e = hipMalloc((void**)&g->co, (size_t)8 * g->ch * 4);
  if (e != hipSuccess) { int rc = pyre_fail(ctx, PYRE_E_HIP, "pyre_gdn_create: %s", hipGetErrorString(e)); delete g; return rc; }
  g->dv = GdnDev{g->params, g->params + nv, g->params + 2 * nv, g->params + 2 * nv + (size_t)g->ch * conv_k, nk, nv, dk, dv, conv_k, eps};
  *out = g; return PYRE_OK;
}
void pyre_gdn_destroy(pyre_gdn* g) { if (!g) return; (void)hipStreamSynchronize(g->ctx->stream); (void)hipFree(g->params); for (int i = 0; i < 2; ++i) { (void)hipFree(g->conv[i]); (void)hipFree(g->ssm[i]); } (void)hipFree(g->co); if (g->io) (void)hipFree(g->io); delete g; }

int pyre_gdn_set_state(pyre_ctx* ctx, pyre_gdn* g, const float* conv_host, const float* ssm_host) {
  if (!ctx || !g) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_set_state: null argument");
  size_t cs = (size_t)(g->dv.conv_k - 1) * g->ch * 4, ss = (size_t)g->dv.nv * g->dv.dk * g->dv.dv * 4;
  if (conv_host) PYRE_HIP(ctx, hipMemcpyAsync(g->conv[g->cur], conv_host, cs, hipMemcpyHostToDevice, ctx->stream)); else PYRE_HIP(ctx, hipMemsetAsync(g->conv[g->cur], 0, cs, ctx->stream));
  if (ssm_host) PYRE_HIP(ctx, hipMemcpyAsync(g->ssm[g->cur], ssm_host, ss, hipMemcpyHostToDevice, ctx->stream)); else PYRE_HIP(ctx, hipMemsetAsync(g->ssm[g->cur], 0, ss, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_gdn_get_state(pyre_ctx* ctx, pyre_gdn* g, float* conv_host, float* ssm_host) {
  if (!ctx || !g) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_get_state: null argument");
  size_t cs = (size_t)(g->dv.conv_k - 1) * g->ch * 4, ss = (size_t)g->dv.nv * g->dv.dk * g->dv.dv * 4;
  if (conv_host) PYRE_HIP(ctx, hipMemcpyAsync(conv_host, g->conv[g->cur], cs, hipMemcpyDeviceToHost, ctx->stream));
  if (ssm_host) PYRE_HIP(ctx, hipMemcpyAsync(ssm_host, g->ssm[g->cur], ss, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

static int gdn_io(pyre_ctx* ctx, pyre_gdn* g, size_t tokens) {
  if (tokens <= g->io_tokens) return PYRE_OK;
  if (g->io) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(g->io)); g->io = nullptr; g->io_tokens = 0; }
  PYRE_HIP(ctx, hipMalloc((void**)&g->io, tokens * ((size_t)g->pw + (size_t)g->dv.nv * g->dv.dv) * 4)); g->io_tokens = tokens; return PYRE_OK;
}

// The recurrent decode / verify step over t tokens (sequential in time): proj [t][ch + nv*dv + 2*nv] -> out [t][nv*dv].
int pyre_gdn_step(pyre_ctx* ctx, pyre_gdn* g, const float* proj_host, int t, float* out_host) {
  if (!ctx || !g || !proj_host || !out_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_step: null argument");
  if (t < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_step: t = %d", t);
  int rc = gdn_io(ctx, g, t); if (rc) return rc;
  float* pd = g->io; float* od = g->io + (size_t)t * g->pw; size_t ow = (size_t)g->dv.nv * g->dv.dv;
  PYRE_HIP(ctx, hipMemcpyAsync(pd, proj_host, (size_t)t * g->pw * 4, hipMemcpyHostToDevice, ctx->stream));
  for (int t0 = 0; t0 < t; t0 += 8) {          // the conv scratch holds 8 tokens
    int n = t - t0 < 8 ? t - t0 : 8; int nx = g->cur ^ 1;
    rc = pyre_gdn_launch(ctx, g->dv, pd + (size_t)t0 * g->pw, g->pw, n, g->conv[g->cur], g->conv[nx], g->ssm[g->cur], g->ssm[nx], g->co, od + (size_t)t0 * ow); if (rc) return rc;
    g->cur = nx;
  }
  PYRE_HIP(ctx, hipMemcpyAsync(out_host, od, (size_t)t * ow * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

// Prefill of T tokens: whole chunks of 64 go through the matrix-core chunked form, the remainder through the step kernels.
int pyre_gdn_prefill_chunked(pyre_ctx* ctx, pyre_gdn* g, const float* proj_host, int T, int chunk, float* out_host) {
  if (!ctx || !g || !proj_host || !out_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_prefill_chunked: null argument");
  if (T < 1) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_prefill_chunked: T = %d", T);
  if (chunk != 64) return pyre_fail(ctx, PYRE_E_ARG, "pyre_gdn_prefill_chunked: chunk size %d unsupported (64 only)", chunk);
  int rc = gdn_io(ctx, g, T); if (rc) return rc;
  float* pd = g->io; float* od = g->io + (size_t)T * g->pw; size_t ow = (size_t)g->dv.nv * g->dv.dv;
  PYRE_HIP(ctx, hipMemcpyAsync(pd, proj_host, (size_t)T * g->pw * 4, hipMemcpyHostToDevice, ctx->stream));
  int Tc = T / 64 * 64;
  if (Tc) {
    float* scr = nullptr; size_t n = (size_t)Tc * ((size_t)g->ch + 2 * g->dv.nv + ow);
    PYRE_HIP(ctx, hipMalloc((void**)&scr, n * 4));
    float* co = scr; float* lg = co + (size_t)Tc * g->ch; float* be = lg + (size_t)Tc * g->dv.nv; float* oraw = be + (size_t)Tc * g->dv.nv; int nx = g->cur ^ 1;
    rc = pyre_gdn_prefill_launch(ctx, g->dv, pd, g->pw, Tc, g->conv[g->cur], g->conv[nx], g->ssm[g->cur], g->ssm[nx], co, lg, be, oraw, od);
    hipError_t e = hipStreamSynchronize(ctx->stream); (void)hipFree(scr);
    if (rc) return rc; if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_HIP, "pyre_gdn_prefill_chunked: %s", hipGetErrorString(e));
    g->cur = nx;
  }
  for (int t0 = Tc; t0 < T; t0 += 8) {
    int n = T - t0 < 8 ? T - t0 : 8; int nx = g->cur ^ 1;
    rc = pyre_gdn_launch(ctx, g->dv, pd + (size_t)t0 * g->pw, g->pw, n, g->conv[g->cur], g->conv[nx], g->ssm[g->cur], g->ssm[nx], g->co, od + (size_t)t0 * ow); if (rc) return rc;
    g->cur = nx;
  }
  PYRE_HIP(ctx, hipMemcpyAsync(out_host, od, (size_t)T * ow * 4, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

}  // extern "C"
