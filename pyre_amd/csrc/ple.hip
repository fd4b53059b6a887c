// Per-layer n-gram embeddings (PLE) of the qwen4exp token step: ple_rows and ple, src/model/qwen4exp_gguf.rs:1390-1434.
//
// Once per window: every position hashes its n-grams (the token and up to ngram - 1 predecessors, cut at the start of
// the sequence and at the eos token) into rows of the per-layer token table, (ngram - 1) * per_gram heads of `dim`
// values each.  Per PLE layer, before the layer's first hyper-connection mix:
//   key [hc*d], value [d] = [key ; value] x emb                      (one GEMV, lane = row)
//   per stream s: g_s = sigmoid(sign(c) * sqrt(max(|c|, 1e-6))), c = rms(key_s, nk_s) . rms(x_s, nq_s) / sqrt(d)
//   gated_s = value * g_s,  nrm_s = rms(gated_s, nc_s)
//   x += gated + silu(depthwise causal conv of nrm over the last conv_k positions, dilation ngram)
// The conv's history is a ring of nrm rows indexed by position, so a rolled-back window leaves nothing to restore.
#include "formats.h"

namespace {
__device__ __forceinline__ float p_sigm(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float p_silu(float x) { return x * p_sigm(x); }

// one thread per (token of the window, head): the table row of that head's n-gram
__global__ __launch_bounds__(128) void k_ple_idx(PleCfg c, const uint32_t* __restrict__ tokens, int start, const int* __restrict__ posp, int t, uint32_t* __restrict__ idx) {
  if (posp) start = *posp;
  const int nh = (c.ngram - 1) * c.per_gram, i = threadIdx.x; if (i >= t * nh) return;
  const int ti = i / nh, h = i - ti * nh, n = 2 + h / c.per_gram, p = start + ti;
  unsigned long long mixed = (unsigned long long)tokens[p] * c.mult[0];
  bool cut = false;
  for (int s = 1; s < n; ++s) {                      // context position s: the token s places back, eos from the first cut on
    const bool none = cut || p < s; const uint32_t tk = none ? 0u : tokens[p - s];
    cut = cut || none || tk == c.eos;
    mixed ^= (unsigned long long)(cut ? c.eos : tk) * c.mult[s];
  }
  idx[i] = (uint32_t)(mixed % c.vocab[h] + c.off[h]);
}

// block sum of one float per thread (256 threads), result to everybody
__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// grid (hc, t), 256 threads: stream s of token ti.  Writes the resolved stream (pending residual update applied) to x_out,
// the gated value to `gated` and the normalised row into the ring at the token's position.
__global__ __launch_bounds__(256) void k_ple_gate(PleDev p, int d, int hc, float eps, const float* __restrict__ x_in, int in_ss, int in_ts, float* __restrict__ x_out,
                                                  const float* __restrict__ comb_out, MoeOut mo, const float* __restrict__ comb_inj, const float* __restrict__ kv,
                                                  float* __restrict__ gated, int start, const int* __restrict__ posp) {
  __shared__ float red[4];
  if (posp) start = *posp;
  const int s = blockIdx.x, ti = blockIdx.y, tid = threadIdx.x, w = hc * d;
  const float cw = (comb_out || mo.partial) ? 2.0f * p_sigm(comb_inj[ti * hc + s]) : 0.0f;
  const float* key = kv + (size_t)ti * (w + d) + (size_t)s * d; const float* val = kv + (size_t)ti * (w + d) + w;
  float* xo = x_out + ((size_t)ti * hc + s) * d;
  float ssk = 0.0f, ssx = 0.0f;
  for (int i = tid; i < d; i += 256) {
    float xv = x_in[(size_t)ti * in_ts + (size_t)s * in_ss + i];
    if (mo.partial) xv = xv + moe_out_value(mo, ti, i) * cw; else if (comb_out) xv = xv + comb_out[(size_t)ti * d + i] * cw;
    xo[i] = xv;
    const float kk = key[i]; ssk += kk * kk; ssx += xv * xv;
  }
  ssk = block_sum(ssk, red); ssx = block_sum(ssx, red);
  const float sk = 1.0f / sqrtf(ssk / (float)d + eps), sx = 1.0f / sqrtf(ssx / (float)d + eps);
  float dp = 0.0f;
  for (int i = tid; i < d; i += 256) dp += (key[i] * (sk * p.nk[(size_t)s * d + i])) * ((xo[i] * sx) * p.nq[(size_t)s * d + i]);      // rms_inplace: x * (s * w); rms: (x * s) * w
  dp = block_sum(dp, red);
  const float sc = dp / sqrtf((float)d);
  const float g = sc != sc ? sc : p_sigm(copysignf(1.0f, sc) * sqrtf(fmaxf(fabsf(sc), 1e-6f)));
  float ssg = 0.0f;
  for (int i = tid; i < d; i += 256) { const float gv = val[i] * g; gated[(size_t)ti * w + (size_t)s * d + i] = gv; ssg += gv * gv; }
  ssg = block_sum(ssg, red);
  const float sg = 1.0f / sqrtf(ssg / (float)d + eps);
  float* ring = p.ring + (size_t)((start + ti) & p.mask) * w + (size_t)s * d;
  for (int i = tid; i < d; i += 256) ring[i] = (val[i] * g) * (sg * p.nc[(size_t)s * d + i]);
}

// grid (hc*d / 256, t), 256 threads: one channel of one token; taps k = 0 .. K-2 lie (K-1-k) * dil positions back
__global__ __launch_bounds__(256) void k_ple_conv(PleDev p, int w, int K, int dil, float* __restrict__ x_out, const float* __restrict__ gated, int start, const int* __restrict__ posp) {
  if (posp) start = *posp;
  const int ch = blockIdx.x * 256 + threadIdx.x, ti = blockIdx.y; if (ch >= w) return;
  const int pos = start + ti;
  float o = p.conv[(size_t)ch * K + K - 1] * p.ring[(size_t)(pos & p.mask) * w + ch];
  for (int k = 0; k < K - 1; ++k) {
    const int q = pos - (K - 1 - k) * dil;
    const float hv = q >= 0 ? p.ring[(size_t)(q & p.mask) * w + ch] : 0.0f;       // the history starts as zeros
    o += p.conv[(size_t)ch * K + k] * hv;
  }
  x_out[(size_t)ti * w + ch] += gated[(size_t)ti * w + ch] + p_silu(o);
}
}  // namespace

size_t pyre_ple_work_bytes(const PleCfg& c, int d, int hc) {
  const size_t nh = (size_t)(c.ngram - 1) * c.per_gram, w = (size_t)hc * d;
  return 4 * 256 + 4 * 8 * 16 + 4 * 8 * nh * c.dim + 4 * 8 * (w + d) + 4 * 8 * w;
}
void pyre_ple_work_carve(const PleCfg& c, int d, int hc, void* base, PleWork* wk) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  const size_t nh = (size_t)(c.ngram - 1) * c.per_gram, w = (size_t)hc * d;
  wk->idx = (uint32_t*)take(4 * 8 * 16); wk->emb = (float*)take(4 * 8 * nh * c.dim); wk->kv = (float*)take(4 * 8 * (w + d)); wk->gated = (float*)take(4 * 8 * w);
}

int pyre_ple_rows_launch(pyre_ctx* ctx, const PleCfg& c, const QMatDev& tab, const PleWork& w, const uint32_t* tokens_dev, int start, const int* posp, int t) {
  const int nh = (c.ngram - 1) * c.per_gram;
  if (t < 1 || t > 8 || nh < 1 || nh > 16 || c.ngram > 8 || tab.cols != c.dim) return pyre_fail(ctx, PYRE_E_SHAPE, "ple: window %d, %d heads, n-grams of %d, table rows of %d for dim %d", t, nh, c.ngram, tab.cols, c.dim);
  { ProfScope ps(ctx, "ple_idx", 4.0 * t * c.ngram); hipLaunchKernelGGL(k_ple_idx, dim3(1), dim3(128), 0, ctx->stream, c, tokens_dev, start, posp, t, w.idx); } PYRE_CHECK_LAUNCH(ctx);
  return pyre_row_launch(ctx, tab, w.idx, t * nh, w.emb, c.dim);
}

int pyre_ple_launch(pyre_ctx* ctx, const PleCfg& c, const PleDev& p, const PleWork& w, int d, int hc, float eps, const float* x_in, int in_ss, int in_ts, float* x_out,
                    const float* comb_out, const MoeOut* comb_moe, const float* comb_inj, int start, const int* posp, int t) {
  const int wd = hc * d, hl = (c.conv_k - 1) * c.ngram;
  if (t < 1 || t > 8 || p.kv.rows != wd + d || p.kv.cols != (c.ngram - 1) * c.per_gram * c.dim || p.mask + 1 < hl + 8 || ((p.mask + 1) & p.mask))
    return pyre_fail(ctx, PYRE_E_SHAPE, "ple: [key ; value] is %d x %d for %d streams of %d, ring of %d rows for a history of %d", p.kv.rows, p.kv.cols, hc, d, p.mask + 1, hl);
  if (x_in == x_out) return pyre_fail(ctx, PYRE_E_ARG, "ple: the updated streams must go to another buffer");
  int rc = pyre_gemv_launch(ctx, p.kv, w.emb, t, w.kv); if (rc) return rc;
  MoeOut mo = comb_moe ? *comb_moe : MoeOut{nullptr, nullptr, nullptr, 0, 0};
  { ProfScope ps(ctx, "ple_gate", 4.0 * t * (3.0 * wd + d)); hipLaunchKernelGGL(k_ple_gate, dim3(hc, t), dim3(256), 0, ctx->stream, p, d, hc, eps, x_in, in_ss, in_ts, x_out, comb_out, mo, comb_inj, w.kv, w.gated, start, posp); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "ple_conv", 4.0 * t * wd * (2.0 + c.conv_k)); hipLaunchKernelGGL(k_ple_conv, dim3((wd + 255) / 256, t), dim3(256), 0, ctx->stream, p, wd, c.conv_k, c.ngram, x_out, w.gated, start, posp); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
