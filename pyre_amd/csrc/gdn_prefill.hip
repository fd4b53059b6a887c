// Gated DeltaNet prefill in chunked form on the fp32 matrix cores (v_mfma_f32_32x32x2_f32).
//
// The reference has no chunked form (linear_core runs the recurrence token by token, src/model/qwen4exp_gguf.rs:
// 1654-1670); this is the same recurrence regrouped per chunk of C = 64 tokens.  With L_i = sum_{j<=i} log g_j inside
// the chunk and S_0 the state at its start,
//     delta_i = beta_i ( v_i - e^{L_i} S_0^T k_i - sum_{j<i} e^{L_i-L_j} (k_i.k_j) delta_j )        (I + A) Delta = B
//     o_i     = e^{L_i} S_0^T q_i + sum_{j<=i} e^{L_i-L_j} (q_i.k_j) delta_j                        O = O1 + P Delta
//     S_C     = e^{L_C} S_0 + sum_j e^{L_C-L_j} k_j (x) delta_j
// Every decay factor is the exponential of a non-positive difference of log-decays, so nothing overflows however
// strong the gate is.  State columns are independent, so each value head is split into column blocks of 32.
#include "formats.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float p_sigm(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float p_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// conv + SiLU for every (token, channel); the window of the first conv_k-1 tokens reaches into conv_in (oldest first).
__global__ void k_gdnp_conv(const float* __restrict__ proj, int stride, int T, int ch, int kk, const float* __restrict__ conv_w, const float* __restrict__ conv_in,
                            float* __restrict__ co, float* __restrict__ conv_out) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, ti = blockIdx.y; if (c >= ch) return;
  float o = conv_w[(size_t)c * kk + kk - 1] * proj[(size_t)ti * stride + c];
  for (int k = 0; k < kk - 1; ++k) { int src = ti - (kk - 1) + k; float v = src >= 0 ? proj[(size_t)src * stride + c] : conv_in[(size_t)(kk - 1 + src) * ch + c]; o += conv_w[(size_t)c * kk + k] * v; }
  co[(size_t)ti * ch + c] = o * p_sigm(o);
  if (ti == T - 1) for (int k = 0; k < kk - 1; ++k) { int src = T - (kk - 1) + k; conv_out[(size_t)k * ch + c] = src >= 0 ? proj[(size_t)src * stride + c] : conv_in[(size_t)(kk - 1 + src) * ch + c]; }
}

// grid (T, nk + 1), 128 threads.  y < nk: L2-normalise q (x 1/sqrt(dk)) and k of key head y in place;
// y == nk: per value head log-decay softplus(alpha + dt) * a and beta = sigmoid(beta).
__global__ __launch_bounds__(128) void k_gdnp_prep(GdnDev p, const float* __restrict__ proj, int stride, float* __restrict__ co, float* __restrict__ logg, float* __restrict__ beta) {
  __shared__ float red[4];
  const int ti = blockIdx.x, y = blockIdx.y, tid = threadIdx.x; const int ch = 2 * p.nk * p.dk + p.nv * p.dv, w = p.nv * p.dv;
  if (y == p.nk) { for (int h = tid; h < p.nv; h += 128) { const float* pr = proj + (size_t)ti * stride; logg[(size_t)ti * p.nv + h] = p_softplus(pr[ch + w + p.nv + h] + p.dt[h]) * p.a[h]; beta[(size_t)ti * p.nv + h] = p_sigm(pr[ch + w + h]); } return; }
  float* q = co + (size_t)ti * ch + (size_t)y * p.dk; float* k = q + (size_t)p.nk * p.dk;
  float qv = q[tid], kv = k[tid], sq = qv * qv, sk = kv * kv;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { sq += __shfl_xor(sq, o); sk += __shfl_xor(sk, o); }
  if ((tid & 63) == 0) { red[tid >> 6] = sq; red[2 + (tid >> 6)] = sk; }
  __syncthreads();
  q[tid] = qv * ((1.0f / sqrtf(red[0] + red[1] + 1e-6f)) * (1.0f / sqrtf((float)p.dk)));
  k[tid] = kv * ((1.0f / sqrtf(red[2] + red[3] + 1e-6f)) * 1.0f);
}

// grid (nv, dv/32), 256 threads (4 waves).  One workgroup carries 32 columns of one head's state through all chunks.
template <int DK, int C>
__global__ __launch_bounds__(256) void k_gdnp_chunk(GdnDev p, const float* __restrict__ co, const float* __restrict__ logg, const float* __restrict__ beta, int nchunks,
                                                    const float* __restrict__ ssm_in, float* __restrict__ ssm_out, float* __restrict__ oraw) {
  static_assert(DK == 128 && C == 64, "tiling assumes dk = 128 and chunks of 64");
  __shared__ float S[DK][33];        // state block [i][c]
  __shared__ float A[C][C + 1];      // beta_i e^{L_i-L_j} k_i.k_j, j < i
  __shared__ float P[C][C + 1];      // e^{L_i-L_j} q_i.k_j, j <= i
  __shared__ float D[C][33];         // B, then Delta
  __shared__ float L[C], Bt[C];
  __shared__ __align__(16) float Qs[C][DK + 4], Ks[C][DK + 4];      // the chunk's q and k rows, staged once (rows padded against bank conflicts)
  const int h = blockIdx.x, cb = blockIdx.y, kh = h % p.nk, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ch = 2 * p.nk * DK + p.nv * p.dv, w = p.nv * p.dv, r = lane & 31, kk = lane >> 5;
  const float* sin_ = ssm_in + (size_t)h * DK * p.dv + cb * 32; float* sout = ssm_out + (size_t)h * DK * p.dv + cb * 32;
  for (int i = tid; i < DK * 32; i += 256) S[i >> 5][i & 31] = sin_[(size_t)(i >> 5) * p.dv + (i & 31)];
  for (int c = 0; c < nchunks; ++c) {
    const int t0 = c * C;
    const float* qc = co + (size_t)t0 * ch + (size_t)kh * DK;                 // q_i at qc + i*ch
    const float* kc = qc + (size_t)p.nk * DK;
    const float* vc = co + (size_t)t0 * ch + 2 * (size_t)p.nk * DK + (size_t)h * p.dv + cb * 32;
    __syncthreads();                                                           // previous chunk done with L, A, P, D, Qs, Ks; S final
    for (int i = tid; i < C * (DK / 4); i += 256) {                            // coalesced: a row is 512 contiguous bytes
      const int row = i / (DK / 4), c4 = i % (DK / 4);
      *(float4*)&Qs[row][4 * c4] = *(const float4*)(qc + (size_t)row * ch + 4 * c4); *(float4*)&Ks[row][4 * c4] = *(const float4*)(kc + (size_t)row * ch + 4 * c4);
    }
    // the chunk's log-decays are fetched by 64 threads at once (one thread walking them would pay a memory round trip per
    // token), then summed in token order by one
    if (tid < C) { Bt[tid] = beta[(size_t)(t0 + tid) * p.nv + h]; L[tid] = logg[(size_t)(t0 + tid) * p.nv + h]; }
    __syncthreads();
    if (tid == 0) { float acc = 0.0f; for (int i = 0; i < C; ++i) { acc += L[i]; L[i] = acc; } }
    __syncthreads();
    // ---- A and P: 64x64x128 each, tile (ti, tj) with tj <= ti; waves 0..2 take A tiles (0,0),(1,0),(1,1), then P likewise
    for (int job = wave; job < 6; job += 4) {
      const int which = job / 3, tsel = job % 3, ti = tsel == 0 ? 0 : 1, tj = tsel == 2 ? 1 : 0;
      const float* arow = which == 0 ? Ks[32 * ti + r] : Qs[32 * ti + r]; const float* brow = Ks[32 * tj + r];
      floatx16 acc = {0};
      for (int k0 = 0; k0 < DK; k0 += 8) {
        float4 a4 = *(const float4*)(arow + k0 + 4 * kk), b4 = *(const float4*)(brow + k0 + 4 * kk);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.x, b4.x, acc, 0, 0, 0); acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.y, b4.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.z, b4.z, acc, 0, 0, 0); acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.w, b4.w, acc, 0, 0, 0);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        int i = 32 * ti + 8 * (e >> 2) + 4 * kk + (e & 3), j = 32 * tj + r;
        float dec = j <= i ? expf(L[i] - L[j]) : 0.0f;
        if (which == 0) A[i][j] = j < i ? Bt[i] * dec * acc[e] : 0.0f; else P[i][j] = dec * acc[e];
      }
    }
    if (wave == 3) { for (int i = lane; i < 32 * 32; i += 64) { A[i >> 5][32 + (i & 31)] = 0.0f; P[i >> 5][32 + (i & 31)] = 0.0f; } }     // upper-right tiles
    // ---- K S_0 (waves 0,1) and Q S_0 (waves 2,3): 64x32x128, row tile = wave & 1
    floatx16 acc1 = {0};
    {
      const int ti = wave & 1; const float* arow = wave < 2 ? Ks[32 * ti + r] : Qs[32 * ti + r];
      for (int k0 = 0; k0 < DK; k0 += 8) {
        float4 a4 = *(const float4*)(arow + k0 + 4 * kk); const int kb = k0 + 4 * kk;
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.x, S[kb][r], acc1, 0, 0, 0); acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.y, S[kb + 1][r], acc1, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.z, S[kb + 2][r], acc1, 0, 0, 0); acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.w, S[kb + 3][r], acc1, 0, 0, 0);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        int i = 32 * ti + 8 * (e >> 2) + 4 * kk + (e & 3); float eL = expf(L[i]);
        if (wave < 2) D[i][r] = Bt[i] * (vc[(size_t)i * ch + r] - eL * acc1[e]);      // B = beta (v - e^{L} K S_0)
        else acc1[e] = eL * acc1[e];                                                 // O1 = e^{L} Q S_0, stays in registers
      }
    }
    __syncthreads();
    // ---- forward substitution (I + A) Delta = B, column by column of A: once Delta_j is final every later row takes its
    // term, all 256 threads at work; an element still receives its terms in ascending j, as a row-by-row solve would give it
    // The 32 columns of Delta are independent: wave w solves columns 8w .. 8w+7 with eight lanes per column (lane t of a column
    // takes the rows j+1+t, j+1+t+8, ..), and a wave's shared-memory operations execute in order, so the 63 steps need no
    // workgroup barrier.
    {
      const int c = 8 * wave + (lane & 7), tr = lane >> 3;
      for (int j = 0; j < C - 1; ++j) {
        const float dj = D[j][c];
        for (int i = j + 1 + tr; i < C; i += 8) D[i][c] -= A[i][j] * dj;
        __builtin_amdgcn_wave_barrier();
      }
    }
    __syncthreads();
    // ---- O = O1 + P Delta (waves 2,3): 64x32x64
    if (wave >= 2) {
      const int ti = wave & 1;
      for (int k0 = 0; k0 < C; k0 += 2) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(P[32 * ti + r][k0 + kk], D[k0 + kk][r], acc1, 0, 0, 0);
#pragma unroll
      for (int e = 0; e < 16; ++e) { int i = 32 * ti + 8 * (e >> 2) + 4 * kk + (e & 3); oraw[(size_t)(t0 + i) * w + (size_t)h * p.dv + cb * 32 + r] = acc1[e]; }
    }
    // ---- S_C = e^{L_C} S_0 + (e^{L_C-L_j} k_j)^T Delta: 128x32x64, row tile = wave
    {
      floatx16 acc2; const float eLC = expf(L[C - 1]);
#pragma unroll
      for (int e = 0; e < 16; ++e) acc2[e] = eLC * S[32 * wave + 8 * (e >> 2) + 4 * kk + (e & 3)][r];
      for (int k0 = 0; k0 < C; k0 += 2) { int j = k0 + kk; float a = Ks[j][32 * wave + r] * expf(L[C - 1] - L[j]); acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, D[j][r], acc2, 0, 0, 0); }
      __syncthreads();                                                        // every wave has read the old S
#pragma unroll
      for (int e = 0; e < 16; ++e) S[32 * wave + 8 * (e >> 2) + 4 * kk + (e & 3)][r] = acc2[e];
    }
  }
  __syncthreads();
  for (int i = tid; i < DK * 32; i += 256) sout[(size_t)(i >> 5) * p.dv + (i & 31)] = S[i >> 5][i & 31];
}

// grid (T, nv), dv threads: out = rms_inplace(o, norm) * sigmoid(z)
__global__ __launch_bounds__(128) void k_gdnp_norm(GdnDev p, const float* __restrict__ proj, int stride, const float* __restrict__ oraw, float* __restrict__ out) {
  __shared__ float red[2];
  const int ti = blockIdx.x, h = blockIdx.y, j = threadIdx.x; const int ch = 2 * p.nk * p.dk + p.nv * p.dv, w = p.nv * p.dv;
  float o = oraw[(size_t)ti * w + (size_t)h * p.dv + j], ss = o * o;
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) ss += __shfl_xor(ss, d);
  if ((j & 63) == 0) red[j >> 6] = ss;
  __syncthreads();
  float sc = 1.0f / sqrtf((red[0] + red[1]) / (float)p.dv + p.eps);
  out[(size_t)ti * w + (size_t)h * p.dv + j] = (o * (sc * p.norm_w[j])) * p_sigm(proj[(size_t)ti * stride + ch + (size_t)h * p.dv + j]);
}

// T must be a multiple of 64.  scratch: co [T][ch], logg [T][nv], beta [T][nv], oraw [T][nv*dv].
int pyre_gdn_prefill_launch(pyre_ctx* ctx, const GdnDev& g, const float* proj, int stride, int T, const float* conv_in, float* conv_out,
                            const float* ssm_in, float* ssm_out, float* co, float* logg, float* beta, float* oraw, float* out) {
  if (g.dk != 128 || g.dv != 128) return pyre_fail(ctx, PYRE_E_SHAPE, "gdn prefill: head dims %dx%d unsupported (128x128 only)", g.dk, g.dv);
  if (T < 64 || T % 64) return pyre_fail(ctx, PYRE_E_ARG, "gdn prefill: %d tokens is not a positive multiple of the chunk size 64", T);
  const int ch = 2 * g.nk * g.dk + g.nv * g.dv;
  { ProfScope ps(ctx, "gdn_prefill_conv", 8.0 * T * ch); hipLaunchKernelGGL(k_gdnp_conv, dim3((ch + 255) / 256, T), dim3(256), 0, ctx->stream, proj, stride, T, ch, g.conv_k, g.conv_w, conv_in, co, conv_out); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "gdn_prefill_prep", 16.0 * T * g.nk * g.dk); hipLaunchKernelGGL(k_gdnp_prep, dim3(T, g.nk + 1), dim3(128), 0, ctx->stream, g, proj, stride, co, logg, beta); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "gdn_prefill_chunk", 8.0 * g.nv * g.dk * g.dv + 4.0 * T * (ch + g.nv * g.dv));
    hipLaunchKernelGGL((k_gdnp_chunk<128, 64>), dim3(g.nv, g.dv / 32), dim3(256), 0, ctx->stream, g, co, logg, beta, T / 64, ssm_in, ssm_out, oraw); } PYRE_CHECK_LAUNCH(ctx);
  { ProfScope ps(ctx, "gdn_prefill_norm", 12.0 * T * g.nv * g.dv); hipLaunchKernelGGL(k_gdnp_norm, dim3(T, g.nv), dim3(128), 0, ctx->stream, g, proj, stride, oraw, out); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
