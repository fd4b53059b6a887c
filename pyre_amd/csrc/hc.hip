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

// o = slice sums of the [down ; inject] GEMV, part[(ks*t + ti)*r64 + i], added in slice order;
// lo[ti][i] = silu(o[i] / hc) for i < lr ; inj[ti][s] = o[lr + s] / hc (zeros without inject)   (:1376-1378)
__global__ void k_hc_lo(const float* __restrict__ part, int ksplit, int r64, int lr, int hc, int has_inject, float* __restrict__ lo, float* __restrict__ inj) {
  int i = blockIdx.x * blockDim.x + threadIdx.x, ti = blockIdx.y, t = gridDim.y;
  if (i >= lr + hc) return;
  float o = 0.0f;
  if (i < lr || has_inject) { o = part[(size_t)ti * r64 + i]; for (int ks = 1; ks < ksplit; ++ks) o += part[((size_t)ks * t + ti) * r64 + i]; }
  float v = o / (float)hc;
  if (i < lr) lo[(size_t)ti * lr + i] = v * sigm(v); else inj[ti * hc + (i - lr)] = has_inject ? v : 0.0f;
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

// the [down ; inject] matrix has few rows and a long K: its K range is cut into slices so that about 96 workgroups run
static int hc_ksplit(const HcDev& h) { int ks = 96 / h.di.tiles; if (ks < 1) ks = 1; if (ks > h.di.U / 4) ks = h.di.U / 4; if (ks < 1) ks = 1; if (ks > 32) ks = 32; return ks; }
size_t pyre_hc_work_bytes(const HcDev& h) { size_t w = (size_t)h.hc * h.d; return 256 * 4 + 4 * 8 * (2 * w + (size_t)h.lr) + 4 * 8 * 32 * ((size_t)h.lr + h.hc + 64); }
void pyre_hc_work_carve(const HcDev& h, void* base, HcWork* w) {
  uint8_t* p = (uint8_t*)base; auto take = [&](size_t n) { void* r = p; p += (n + 255) & ~(size_t)255; return r; };
  size_t wd = (size_t)h.hc * h.d;
  w->xn = (float*)take(4 * 8 * wd); w->o = (float*)take(4 * 8 * 32 * ((size_t)h.lr + h.hc + 64)); w->lo = (float*)take(4 * 8 * (size_t)h.lr); w->gate = (float*)take(4 * 8 * wd); w->ksplit = 0;
}

int pyre_hc_mix_launch(pyre_ctx* ctx, const HcDev& h, const HcWork& w, float* x, int t, const float* comb_out, const float* comb_inj, float eps, float* mixed, float* inj) {
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "hc_mix: t = %d outside 1..8", t);
  { ProfScope ps(ctx, "hc_rms", 4.0 * t * h.hc * h.d * 3); hipLaunchKernelGGL(k_hc_rms, dim3(h.hc, t), dim3(256), 0, ctx->stream, x, comb_out, comb_inj, h.norm, h.d, h.hc, eps, w.xn); } PYRE_CHECK_LAUNCH(ctx);
  const int ks = hc_ksplit(h), r64 = ks == 1 ? h.di.rows : h.di.tiles * 64;
  int rc = pyre_gemv_split_launch(ctx, h.di, w.xn, t, w.o, ks); if (rc) return rc;
  { ProfScope ps(ctx, "hc_lo", 4.0 * t * (h.lr + h.hc) * (ks + 1)); hipLaunchKernelGGL(k_hc_lo, dim3((h.lr + h.hc + 255) / 256, t), dim3(256), 0, ctx->stream, w.o, ks, r64, h.lr, h.hc, h.has_inject ? 1 : 0, w.lo, inj); } PYRE_CHECK_LAUNCH(ctx);
  rc = pyre_gemv_launch(ctx, h.up, w.lo, t, w.gate); if (rc) return rc;
  { ProfScope ps(ctx, "hc_mixed", 4.0 * t * h.d * (2 * h.hc + 1)); hipLaunchKernelGGL(k_hc_mixed, dim3((h.d + 255) / 256, t), dim3(256), 0, ctx->stream, w.xn, w.gate, h.d, h.hc, mixed); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}

int pyre_hc_combine_launch(pyre_ctx* ctx, int d, int hc, float* x, int t, const float* out, const float* inj) {
  { ProfScope ps(ctx, "hc_combine", 4.0 * t * d * (2 * hc + 1)); hipLaunchKernelGGL(k_hc_combine, dim3((d + 255) / 256, hc, t), dim3(256), 0, ctx->stream, x, out, inj, d, hc); } PYRE_CHECK_LAUNCH(ctx);
  return PYRE_OK;
}
