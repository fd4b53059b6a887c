// Hyper-connection mix / combine around every block: grouped RMSNorm over the hc residual streams, low-rank sigmoid
// gate, stream mean; residual update.  Follows hc_mix / hc_combine, src/model/qwen4exp_gguf.rs:1357-1388 (f32 branch).
#include "formats.h"

__device__ __forceinline__ float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  int tid = threadIdx.x; red[tid] = v; __syncthreads();
  for (int s = 128; s > 0; s >>= 1) { if (tid < s) red[tid] += red[tid + s]; __syncthreads(); }
  float r = red[0]; __syncthreads(); return r;
}

// grid (hc, t), 256 threads: optional residual update x[ti][s][:] += out[ti][:] * 2*sigm(inj[ti][s]), then
// xn[ti][s][:] = x * rsqrt(mean(x^2) + eps) * norm[s][:]     (rms, :209: (x * s) * w)
__global__ __launch_bounds__(256) void k_hc_rms(float* __restrict__ x, const float* __restrict__ comb_out, const float* __restrict__ comb_inj, const float* __restrict__ norm,
                                                int d, int hc, float eps, float* __restrict__ xn) {
  __shared__ float red[256];
  const int s = blockIdx.x, ti = blockIdx.y, tid = threadIdx.x;
  float* xs = x + ((size_t)ti * hc + s) * d;
  float ss = 0.0f;
  if (comb_out) {
    float w = 2.0f * sigm(comb_inj[ti * hc + s]);
    for (int i = tid; i < d; i += 256) { float v = xs[i] + comb_out[(size_t)ti * d + i] * w; xs[i] = v; ss += v * v; }
  } else for (int i = tid; i < d; i += 256) { float v = xs[i]; ss += v * v; }
  float tot = block_sum_256(ss, red);
  float sc = 1.0f / sqrtf(tot / (float)d + eps);
  for (int i = tid; i < d; i += 256) xn[((size_t)ti * hc + s) * d + i] = xs[i] * sc * norm[(size_t)s * d + i];
}

// lo[ti][i] = silu(o[ti][i] / hc) for i < lr ; inj[ti][s] = o[ti][lr + s] / hc (zeros without inject)   (:1376-1378)
__global__ void k_hc_lo(const float* __restrict__ o, int orow, int lr, int hc, int has_inject, float* __restrict__ lo, float* __restrict__ inj) {
  int i = blockIdx.x * blockDim.x + threadIdx.x, ti = blockIdx.y;
  if (i < lr) { float v = o[(size_t)ti * orow + i] / (float)hc; lo[(size_t)ti * lr + i] = v * sigm(v); }
  else if (i < lr + hc) inj[ti * hc + (i - lr)] = has_inject ? o[(size_t)ti * orow + i] / (float)hc : 0.0f;
}

// mixed[ti][i] = (sum_s xn[ti][s][i] * sigm(gate[ti][s][i])) / hc, s ascending from zero   (:1380)
__global__ void k_hc_mixed(const float* __restrict__ xn, const float* __restrict__ gate, int d, int hc, float* __restrict__ mixed) {
  int i = blockIdx.x * blockDim.x + threadIdx.x, ti = blockIdx.y; if (i >= d) return;
  float m = 0.0f;
  for (int s = 0; s < hc; ++s) { size_t k = ((size_t)ti * hc + s) * d + i; m += xn[k] * sigm(gate[k]); }
  mixed[(size_t)ti * d + i] = m / (float)hc;
}

__global__ void k_hc_combine(float* __restrict__ x, const float* __restrict__ out, const float* __restrict__ inj, int d, int hc) {
  int i = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.y, ti = blockIdx.z; if (i >= d) return;
  float w = 2.0f * sigm(inj[ti * hc + s]);
  x[((size_t)ti * hc + s) * d + i] += out[(size_t)ti * d + i] * w;
}

size_t pyre_hc_work_bytes(const HcDev& h) { size_t w = (size_t)h.hc * h.d; return 256 * 4 + 4 * 8 * (2 * w + (size_t)h.lr + h.hc + h.lr); }
void pyre_hc_work_carve(const HcDev& h, void* base, HcWork* w) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t wd = (size_t)h.hc * h.d;
  w->xn = (float*)take(4 * 8 * wd); w->o = (float*)take(4 * 8 * ((size_t)h.lr + h.hc)); w->lo = (float*)take(4 * 8 * (size_t)h.lr); w->gate = (float*)take(4 * 8 * wd);
}

int pyre_hc_mix_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, float* x, int t, const float* comb_out, const float* comb_inj, float eps, float* mixed, float* inj) {
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: t = %d outside 1..8", t);
  hipLaunchKernelGGL(k_hc_rms, dim3(h.hc, t), dim3(256), 0, ctx->stream, x, comb_out, comb_inj, h.norm, h.d, h.hc, eps, w.xn); PYRE_CHECK_LAUNCH(ctx);
  int rc = pyre_gemv_launch(ctx, h.di, w.xn, t, w.o); if (rc) return rc;
  int orow = h.di.rows;
  hipLaunchKernelGGL(k_hc_lo, dim3((h.lr + h.hc + 255) / 256, t), dim3(256), 0, ctx->stream, w.o, orow, h.lr, h.hc, h.has_inject ? 1 : 0, w.lo, inj); PYRE_CHECK_LAUNCH(ctx);
  rc = pyre_gemv_launch(ctx, h.up, w.lo, t, w.gate); if (rc) return rc;
  hipLaunchKernelGGL(k_hc_mixed, dim3((h.d + 255) / 256, t), dim3(256), 0, ctx->stream, w.xn, w.gate, h.d, h.hc, mixed); PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

int pyre_hc_combine_launch(pyre_ctx* ctx, int d, int hc, float* x, int t, const float* out, const float* inj) {
  hipLaunchKernelGGL(k_hc_combine, dim3((d + 255) / 256, hc, t), dim3(256), 0, ctx->stream, x, out, inj, d, hc); PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
