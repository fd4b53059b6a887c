// QSA sparse indexer: raw index keys, pooled block keys, block scores, exact top-k block selection into a sorted
// position list.  Follows attn_core's indexer branch, src/model/qwen4exp_gguf.rs:1565-1599, and the YaRN frequency
// table of src/qn_ctx.rs:164-185.
#include "formats.h"
#include <math.h>

float pyre_rope_table(int n_rot, float base, int ctx_train, int ctx, float* inv) {
  const int half = n_rot / 2;
  const float scale = (ctx_train > 0 && ctx > ctx_train) ? (float)ctx / (float)ctx_train : 1.0f;
  if (scale <= 1.0f) { for (int i = 0; i < half; ++i) inv[i] = powf(base, -(2.0f * (float)i) / (float)n_rot); return 1.0f; }     // qn_ctx.rs:168
  const float dim = (float)n_rot;
  auto corr = [&](float rot) { return (dim * logf((float)ctx_train / (rot * 2.0f * 3.14159265358979323846f))) / (2.0f * logf(base)); };
  const float low = fmaxf(floorf(corr(32.0f)), 0.0f), high = fminf(ceilf(corr(1.0f)), (float)(half > 0 ? half - 1 : 0));
  for (int i = 0; i < half; ++i) {
    float extrap = powf(base, -(2.0f * (float)i) / dim), interp = extrap / scale;
    float ramp = fabsf(high - low) < 1e-6f ? 1.0f : fminf(fmaxf(((float)i - low) / (high - low), 0.0f), 1.0f);
    inv[i] = interp * (1.0f - ramp) + extrap * ramp;       // low indices (high frequency) interpolated, high indices keep the trained frequency
  }
  return 1.0f + 0.1f * logf(scale);
}

namespace {

// grid (1 + nh + npool, t), hd threads.
// pool_from < 0 (the decode path):
//   block 0:            the token's raw index key -> ik[pos]
//   blocks 1..nh:       index query head -> rms_inplace(iqn) -> rope(pos) -> iq[ti][h]
//   blocks nh+1.. (row ti == 0 of the grid only): j-th block of `ratio` tokens the window may complete: mean of its raw
//                       keys (earlier positions from ik, the window's own from the projections, added in position order,
//                       then divided) -> rms_inplace(ikn) -> rope(first position of the block) -> ib[block]
__global__ void k_qsa_prep(QsaDev q, AttnDev a, QsaBuf b, const float* __restrict__ proj, int stride, int iq_off, int start, int t, const int* __restrict__ posp, float* __restrict__ iq_out, int pool_from) {
  __shared__ float buf[1024]; __shared__ float red[16];
  if (posp) start = *posp;
  const int bx = blockIdx.x, ti = blockIdx.y, tid = threadIdx.x, hd = q.hd, pos = start + ti;
  const float* row = proj + (size_t)ti * stride + iq_off;
  const bool is_q = bx <= q.nh;
  if (pool_from >= 0 && is_q) return;                            // pool-only launch (keys installed from outside): no projections to read
  if (bx == 0) { b.ik[(size_t)pos * hd + tid] = row[(size_t)q.nh * hd + tid]; return; }
  float v; const float* nw; int rpos, blk = 0;
  if (is_q) { v = row[(size_t)(bx - 1) * hd + tid]; nw = q.iqn; rpos = pos; }
  else {
    if (ti != 0) return;
    blk = (pool_from >= 0 ? pool_from : start / q.ratio) + (bx - 1 - q.nh);
    if ((blk + 1) * q.ratio > start + t) return;                 // this window does not complete the block
    float sacc = 0.0f;
    for (int p = blk * q.ratio; p < (blk + 1) * q.ratio; ++p) sacc += p >= start ? proj[(size_t)(p - start) * stride + iq_off + (size_t)q.nh * hd + tid] : b.ik[(size_t)p * hd + tid];
    v = sacc / (float)q.ratio; nw = q.ikn; rpos = blk * q.ratio;
  }
  const int half = a.n_rot / 2, ri = tid < half ? tid : tid - half;
  const float nwt = nw[tid], rinv = tid < a.n_rot ? a.rope_inv[ri] : 0.0f;
  float ss = v * v;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.0f;
  for (int i = 0; i < hd / 64; ++i) tot += red[i];
  const float sc = 1.0f / sqrtf(tot / (float)hd + a.eps);
  v = v * (sc * nwt);            // rms_inplace: x *= s * w
  buf[tid] = v;
  __syncthreads();
  if (tid < a.n_rot) {
    float ang = (float)rpos * rinv;
    float sn = sinf(ang), cs = cosf(ang);
    if (a.mscale != 1.0f) { cs = cs * a.mscale; sn = sn * a.mscale; }
    float x0 = buf[ri], x1 = buf[ri + half];
    v = tid < half ? x0 * cs - x1 * sn : x1 * cs + x0 * sn;
  }
  if (is_q) iq_out[((size_t)ti * q.nh + (bx - 1)) * hd + tid] = v;
  else b.ib[qsa_ib_at((size_t)blk, (size_t)tid, (size_t)hd)] = v;
}

// grid (ceil(max_blocks / 64), t), 256 threads: lane = block, the four waves split the key length.
// score[ti][b] = sum_h relu(q_h . key_b) / sqrt(hd) for the n / ratio complete blocks a query with n visible positions
// can choose from; nothing while the query is dense.
constexpr int QSA_HB = 4;
__global__ __launch_bounds__(256) void k_qsa_score(QsaDev q, QsaBuf b, const float* __restrict__ iq, int start, const int* __restrict__ posp, float* __restrict__ score, int max_blocks) {
  extern __shared__ float qs[];             // [round_up(nh, QSA_HB)][hd] queries (rows past nh are zero), then [4][nhp][64] partial dots
  if (posp) start = *posp;
  const int ti = blockIdx.y, n = start + ti + 1, hd = q.hd, tid = threadIdx.x;
  if (n <= q.budget + q.ratio - 1) return;
  const int nb = n / q.ratio, nhp = (q.nh + QSA_HB - 1) / QSA_HB * QSA_HB;
  if ((int)blockIdx.x * 64 >= nb) return;
  float* part = qs + (size_t)nhp * hd;
  for (int i = tid; i < nhp * hd; i += 256) qs[i] = i < q.nh * hd ? iq[(size_t)ti * q.nh * hd + i] : 0.0f;
  __syncthreads();
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), blk = blockIdx.x * 64 + lane;
  const int seg = hd / 4, i0 = wave * seg;                      // this wave's slice of the key
  const float* kb = b.ib + (size_t)blockIdx.x * hd * 64 + lane;
  for (int h0 = 0; h0 < nhp; h0 += QSA_HB) {
    float acc[QSA_HB];
#pragma unroll
    for (int j = 0; j < QSA_HB; ++j) acc[j] = 0.0f;
#pragma unroll 8
    for (int i = i0; i < i0 + seg; ++i) {
      const float kv = kb[(size_t)i * 64];
#pragma unroll
      for (int j = 0; j < QSA_HB; ++j) acc[j] = fmaf(qs[(h0 + j) * hd + i], kv, acc[j]);
    }
#pragma unroll
    for (int j = 0; j < QSA_HB; ++j) part[((size_t)wave * nhp + h0 + j) * 64 + lane] = acc[j];
  }
  __syncthreads();
  if (wave == 0 && blk < nb) {
    float total = 0.0f;
    for (int h = 0; h < q.nh; ++h) { float d = ((part[((size_t)0 * nhp + h) * 64 + lane] + part[((size_t)1 * nhp + h) * 64 + lane]) + part[((size_t)2 * nhp + h) * 64 + lane]) + part[((size_t)3 * nhp + h) * 64 + lane]; total += fmaxf(d, 0.0f); }
    score[(size_t)ti * max_blocks + blk] = total * (1.0f / sqrtf((float)hd));
  }
}

// exclusive prefix sum of one int per thread over a 1024-thread workgroup; *total receives the sum
__device__ __forceinline__ int block_excl_scan(int v, int* wtot, int* total) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) { int u = __shfl_up(inc, o); if (lane >= o) inc += u; }
  __syncthreads();                           // wtot may still be read from the previous call
  if (lane == 63) wtot[wave] = inc;
  __syncthreads();
  int base = 0, all = 0;
  for (int w = 0; w < 16; ++w) { int x = wtot[w]; if (w < wave) base += x; all += x; }
  *total = all;
  return base + inc - v;
}

// grid (t), 1024 threads.  Exact selection of the budget / ratio best blocks: the k-th largest score by four radix passes
// over the (non-negative) float bits, then every block above it plus, among the blocks equal to it, the lowest indices;
// the chosen blocks are compacted in index order into positions, followed by the incomplete tail.
__global__ __launch_bounds__(1024) void k_qsa_select(QsaDev q, const float* __restrict__ score, int start, const int* __restrict__ posp, int* __restrict__ plist, int* __restrict__ pcount, int list_stride, int max_blocks) {
  __shared__ unsigned hist[256]; __shared__ unsigned wsuf[4]; __shared__ unsigned s_prefix, s_need; __shared__ int wtot[16];
  if (posp) start = *posp;
  const int ti = blockIdx.x, tid = threadIdx.x, n = start + ti + 1;
  if (n <= q.budget + q.ratio - 1) { if (tid == 0) pcount[ti] = -1; return; }
  const int nb = n / q.ratio, kk = q.budget / q.ratio;
  const float* sc = score + (size_t)ti * max_blocks;
  int* out = plist + (size_t)ti * list_stride;
  unsigned prefix = 0, need = (unsigned)kk;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass; const unsigned mask_hi = pass ? (0xFFFFFFFFu << (shift + 8)) : 0u;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int bk = tid; bk < nb; bk += 1024) { unsigned u = __float_as_uint(sc[bk]) & 0x7FFFFFFFu; if ((u & mask_hi) == prefix) atomicAdd(&hist[(u >> shift) & 255u], 1u); }
    __syncthreads();
    // bucket d of the current digit is the one that holds the need-th largest key when the count of keys in buckets
    // >= d reaches need and the count in buckets > d does not: a suffix sum over the 256 buckets by threads 0..255
    if (tid < 256) {
      unsigned suf = hist[tid];                                // inclusive suffix sum inside the wave (this lane and the lanes above)
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) { unsigned u = __shfl_down(suf, o); if ((tid & 63) + o < 64) suf += u; }
      if ((tid & 63) == 0) wsuf[tid >> 6] = suf;               // the wave's total
      hist[tid] = suf;
    }
    __syncthreads();
    if (tid < 256) {
      unsigned above = 0; for (int w = (tid >> 6) + 1; w < 4; ++w) above += wsuf[w];
      const unsigned incl = hist[tid] + above;                 // keys in buckets >= tid
      const unsigned up = __shfl_down(incl, 1);
      const unsigned excl = (tid & 63) == 63 ? above : up;     // keys in buckets > tid
      if (incl >= need && excl < need) { s_prefix = prefix | ((unsigned)tid << shift); s_need = need - excl; }
    }
    __syncthreads();
    prefix = s_prefix; need = s_need;
  }
  const unsigned T = prefix;                 // the k-th largest key; `need` blocks equal to it are taken, lowest index first
  const int per = (nb + 1023) / 1024, lo = min(nb, tid * per), hi = min(nb, lo + per);
  int eq = 0;
  for (int bk = lo; bk < hi; ++bk) eq += ((__float_as_uint(sc[bk]) & 0x7FFFFFFFu) == T) ? 1 : 0;
  int tot; int eq_rank = block_excl_scan(eq, wtot, &tot);
  int nsel = 0; { int er = eq_rank; for (int bk = lo; bk < hi; ++bk) { unsigned u = __float_as_uint(sc[bk]) & 0x7FFFFFFFu; bool s = u > T || (u == T && er++ < (int)need); nsel += s ? 1 : 0; } }
  int j = block_excl_scan(nsel, wtot, &tot);
  { int er = eq_rank; for (int bk = lo; bk < hi; ++bk) { unsigned u = __float_as_uint(sc[bk]) & 0x7FFFFFFFu; bool s = u > T || (u == T && er++ < (int)need);
      if (s) { if (j < kk) for (int r = 0; r < q.ratio; ++r) out[j * q.ratio + r] = bk * q.ratio + r; ++j; } } }
  const int tail = n - nb * q.ratio;
  if (tid < tail) out[kk * q.ratio + tid] = nb * q.ratio + tid;
  if (tid == 0) pcount[ti] = kk * q.ratio + tail;
}

}  // namespace

size_t pyre_qsa_buf_bytes(const QsaDev& q, int cap) {
  if (q.nh <= 0) return 0;
  size_t nblk = ((size_t)cap / q.ratio + 63) / 64 * 64;
  return 2 * 256 + (size_t)cap * q.hd * 4 + nblk * q.hd * 4;
}
void pyre_qsa_buf_carve(const QsaDev& q, int cap, void* base, QsaBuf* b) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t nblk = ((size_t)cap / q.ratio + 63) / 64 * 64;
  b->ik = (float*)take((size_t)cap * q.hd * 4); b->ib = (float*)take(nblk * q.hd * 4);
}
size_t pyre_qsa_work_bytes(const QsaDev& q, int cap) {
  if (q.nh <= 0) return 0;
  size_t nblk = ((size_t)cap / q.ratio + 63) / 64 * 64, ls = ((size_t)q.budget + 2 * q.ratio + 3) & ~(size_t)3;
  return 4 * 256 + 8 * (size_t)q.nh * q.hd * 4 + 8 * nblk * 4 + 8 * ls * 4 + 8 * 4;
}
void pyre_qsa_work_carve(const QsaDev& q, int cap, void* base, QsaWork* w) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t nblk = ((size_t)cap / q.ratio + 63) / 64 * 64, ls = ((size_t)q.budget + 2 * q.ratio + 3) & ~(size_t)3;
  w->iq = (float*)take(8 * (size_t)q.nh * q.hd * 4); w->score = (float*)take(8 * nblk * 4); w->plist = (int*)take(8 * ls * 4); w->pcount = (int*)take(8 * 4);
  w->list_stride = (int)ls; w->max_blocks = (int)nblk;
}

// pools every complete block of the first n positions from the raw keys already in b.ik
int pyre_qsa_pool_all(pyre_ctx* ctx, const QsaDev& q, const AttnDev& a, const QsaBuf& b, int n) {
  const int nblk = n / q.ratio; if (nblk < 1) return PYRE_OK;
  hipLaunchKernelGGL(k_qsa_prep, dim3(1 + q.nh + nblk, 1), dim3(q.hd), 0, ctx->stream, q, a, b, (const float*)nullptr, 0, 0, n, 0, (const int*)nullptr, (float*)nullptr, 0);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

int pyre_qsa_launch(pyre_ctx* ctx, const QsaDev& q, const AttnDev& a, const QsaBuf& b, const QsaWork& w, const float* proj, int stride, int iq_off, int start, int t, const int* posp) {
  if (q.nh < 1 || q.hd < 64 || q.hd > 1024 || q.hd % 64 || q.ratio < 1 || q.budget < q.ratio || q.budget % q.ratio) return pyre_fail(ctx, PYRE_E_SHAPE, "indexer: %d heads of %d, block %d, budget %d unsupported", q.nh, q.hd, q.ratio, q.budget);
  if (a.n_rot > q.hd) return pyre_fail(ctx, PYRE_E_SHAPE, "indexer: key length %d below the rotated width %d", q.hd, a.n_rot);
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "indexer: t = %d outside 1..8", t);
  const int npool = t / q.ratio + 1;
  { ProfScope ps(ctx, "qsa_prep", 4.0 * t * (q.nh + 2.0) * q.hd); hipLaunchKernelGGL(k_qsa_prep, dim3(1 + q.nh + npool, t), dim3(q.hd), 0, ctx->stream, q, a, b, proj, stride, iq_off, start, t, posp, w.iq, -1); } PYRE_CHECK_LAUNCH(ctx);
  // with the position on the host, a window that stays dense needs no scores; with it on the device the kernels decide
  const bool maybe_sparse = posp != nullptr || start + t > q.budget + q.ratio - 1;
  const int nbmax = posp ? w.max_blocks : (start + t) / q.ratio;
  if (maybe_sparse && nbmax > 0) {
    const int nhp = (q.nh + QSA_HB - 1) / QSA_HB * QSA_HB;
    if (((size_t)nhp * q.hd + 4 * (size_t)nhp * 64) * 4 > 65536) return pyre_fail(ctx, PYRE_E_SHAPE, "indexer: %d heads of %d do not fit the score kernel's shared memory", q.nh, q.hd);
    ProfScope ps(ctx, "qsa_score", 4.0 * t * ((double)nbmax * q.hd + (double)q.nh * q.hd + nbmax));
    hipLaunchKernelGGL(k_qsa_score, dim3((nbmax + 63) / 64, t), dim3(256), ((size_t)nhp * q.hd + 4 * (size_t)nhp * 64) * 4, ctx->stream, q, b, w.iq, start, posp, w.score, w.max_blocks); PYRE_CHECK_LAUNCH(ctx);
  }
  { ProfScope ps(ctx, "qsa_select", 4.0 * t * (5.0 * nbmax + q.budget)); hipLaunchKernelGGL(k_qsa_select, dim3(t), dim3(1024), 0, ctx->stream, q, w.score, start, posp, w.plist, w.pcount, w.list_stride, w.max_blocks); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
