// Context, device memory helpers, and the synthetic-tensor generator.
#include "common.h"
#include "formats.h"
#include "iq_codebooks.h"
#include <stdarg.h>

thread_local std::string g_pyre_create_err;

int pyre_fail(pyre_ctx* ctx, int code, const char* fmt, ...) {
  char buf[512]; va_list ap; va_start(ap, fmt); vsnprintf(buf, sizeof buf, fmt, ap); va_end(ap);
  if (ctx) ctx->err = buf; else g_pyre_create_err = buf;
  return code;
}

int pyre_stage(pyre_ctx* ctx, size_t nbytes, void** out) {
  if (nbytes > ctx->stage_bytes) {
    if (ctx->stage) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(ctx->stage)); ctx->stage = nullptr; ctx->stage_bytes = 0; }
    size_t n = (nbytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
    PYRE_HIP(ctx, hipMalloc(&ctx->stage, n)); ctx->stage_bytes = n;
  }
  *out = ctx->stage; return PYRE_OK;
}

// ---- synthetic blocks: pyre_amd/synth.py:blocks() on the device -----------------------------------------------------
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull; z ^= z >> 27; z *= 0x94D049BB133111EBull; z ^= z >> 31; return z;
}
__global__ void k_synth_payload(uint64_t seed, size_t nbytes, uint8_t* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; size_t nw = (nbytes + 7) / 8;
  if (i >= nw) return;
  uint64_t w = mix64(seed + (i + 1) * 0x9E3779B97F4A7C15ull);
  size_t o = i * 8;
  if (o + 8 <= nbytes && (((uintptr_t)(out + o)) & 7) == 0) *(uint64_t*)(out + o) = w;
  else for (int k = 0; k < 8 && o + k < nbytes; ++k) out[o + k] = (uint8_t)(w >> (8 * k));
}
__global__ void k_synth_scales(uint64_t seed, size_t n_blocks, int bs, int nfields, int off0, int off1, float lo, float hi, uint8_t* out) {
  size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= n_blocks) return;
  uint64_t w = mix64((seed ^ 0xD1B54A32D192ED03ull) + (b + 1) * 0x9E3779B97F4A7C15ull);
  for (int f = 0; f < nfields; ++f) {
    uint32_t bits = f == 0 ? (uint32_t)(w >> 40) : (uint32_t)((w >> 16) & 0xFFFFFF);
    float u = (float)bits * 5.9604644775390625e-08f;    // 2^-24
    float v = lo + (hi - lo) * u;
    unsigned short h = __half_as_ushort(__float2half_rn(v));
    if (off0 < 0) { uint8_t* q = out + b * bs + 48; for (int k = 0; k < 4; ++k) q[2 * k + 1] = (uint8_t)((q[2 * k + 1] & 0x0F) | (((h >> (4 * k)) & 0xF) << 4)); continue; }      // IQ1_M: nibble k of d in the top nibble of scale word k
    uint8_t* p = out + b * bs + (f == 0 ? off0 : off1); p[0] = (uint8_t)(h & 0xFF); p[1] = (uint8_t)(h >> 8);
  }
}

extern "C" {

int pyre_ctx_create(int device, pyre_ctx** out) {
  if (!out) return pyre_fail(nullptr, PYRE_E_ARG, "pyre_ctx_create: out is NULL");
  *out = nullptr;
  int n = 0; hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) return pyre_fail(nullptr, PYRE_E_HIP, "pyre_ctx_create: no HIP device (%s)", hipGetErrorString(e));
  if (device < 0 || device >= n) return pyre_fail(nullptr, PYRE_E_ARG, "pyre_ctx_create: device %d out of range (%d devices)", device, n);
  pyre_ctx* ctx = new pyre_ctx(); ctx->device = device;
  if ((e = hipSetDevice(device)) != hipSuccess || (e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess) {
    int rc = pyre_fail(nullptr, PYRE_E_HIP, "pyre_ctx_create: %s", hipGetErrorString(e)); delete ctx; return rc; }
  // expand the compact codebooks (see iq_codebooks.h) and keep them in device memory
  std::vector<uint32_t> g3(512); std::vector<uint64_t> g2(512); static const uint8_t tri[3] = {8, 25, 43};
  for (int i = 0; i < 512; ++i) {
    uint32_t v = 0; for (int j = 0; j < 4; ++j) v |= (uint32_t)(2 * ((kIq3sCode[i] >> (3 * j)) & 7) + 1) << (8 * j); g3[i] = v;
    uint64_t w = 0; for (int j = 0; j < 8; ++j) w |= (uint64_t)tri[(kIq2xsCode[i] >> (2 * j)) & 3] << (8 * j); g2[i] = w;
  }
  std::vector<uint16_t> cb(4096);          // compact codes as they are: [iq2xxs 256 | iq2s 1024 | iq3xxs 256 | iq2xs 512 | iq1s 2048], used once per matrix by the load-time re-coding
  for (int i = 0; i < 2048; ++i) cb[2048 + i] = kIq1sCode[i];
  for (int i = 0; i < 256; ++i) { cb[i] = kIq2xxsCode[i]; cb[1280 + i] = kIq3xxsCode[i]; }
  for (int i = 0; i < 1024; ++i) cb[256 + i] = kIq2sCode[i];
  for (int i = 0; i < 512; ++i) cb[1536 + i] = kIq2xsCode[i];
  if ((e = hipMalloc((void**)&ctx->d_cb, 4096 * 2)) != hipSuccess || (e = hipMemcpy(ctx->d_cb, cb.data(), 4096 * 2, hipMemcpyHostToDevice)) != hipSuccess ||
      (e = hipMalloc((void**)&ctx->d_iq3s, 512 * 4)) != hipSuccess || (e = hipMalloc((void**)&ctx->d_iq2xs, 512 * 8)) != hipSuccess ||
      (e = hipMemcpy(ctx->d_iq3s, g3.data(), 512 * 4, hipMemcpyHostToDevice)) != hipSuccess || (e = hipMemcpy(ctx->d_iq2xs, g2.data(), 512 * 8, hipMemcpyHostToDevice)) != hipSuccess) {
    int rc = pyre_fail(nullptr, PYRE_E_HIP, "pyre_ctx_create: codebook upload: %s", hipGetErrorString(e)); pyre_ctx_destroy(ctx); return rc; }
  if (pyre_gemv_n_table(ctx) != PYRE_OK || pyre_static_init(ctx) != PYRE_OK) { int rc = pyre_fail(nullptr, PYRE_E_HIP, "pyre_ctx_create: %s", ctx->err.c_str()); pyre_ctx_destroy(ctx); return rc; }
  *out = ctx; return PYRE_OK;
}

}  // extern "C"

extern "C" {

void pyre_ctx_destroy(pyre_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  if (ctx->stage) (void)hipFree(ctx->stage);
  if (ctx->d_iq3s) (void)hipFree(ctx->d_iq3s);
  if (ctx->d_cb) (void)hipFree(ctx->d_cb);
  if (ctx->aop_buf) (void)hipFree(ctx->aop_buf);
  if (ctx->d_iq2xs) (void)hipFree(ctx->d_iq2xs);
  if (ctx->d_iq3s_sgn) (void)hipFree(ctx->d_iq3s_sgn);
  if (ctx->d_iq2xs_sgn) (void)hipFree(ctx->d_iq2xs_sgn);
  if (ctx->dgn_buf) (void)hipFree(ctx->dgn_buf);
  for (auto& p : ctx->prof_pending) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
  for (auto e : ctx->prof_pool) (void)hipEventDestroy(e);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

const char* pyre_last_error(const pyre_ctx* ctx) { return ctx ? ctx->err.c_str() : g_pyre_create_err.c_str(); }
int pyre_ctx_sync(pyre_ctx* ctx) { if (!ctx) return PYRE_E_ARG; PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK; }
void* pyre_ctx_stream(pyre_ctx* ctx) { return ctx ? (void*)ctx->stream : nullptr; }

int pyre_dev_alloc(pyre_ctx* ctx, size_t nbytes, void** out) {
  if (!ctx || !out) return PYRE_E_ARG;
  PYRE_HIP(ctx, hipMalloc(out, nbytes ? nbytes : 1)); return PYRE_OK;
}
int pyre_dev_free(pyre_ctx* ctx, void* p) { if (!ctx) return PYRE_E_ARG; if (p) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(p)); } return PYRE_OK; }
int pyre_dev_upload(pyre_ctx* ctx, void* dst, const void* src, size_t n) {
  if (!ctx || (!dst && n) || (!src && n)) return pyre_fail(ctx, PYRE_E_ARG, "pyre_dev_upload: null pointer");
  PYRE_HIP(ctx, hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, ctx->stream)); PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_dev_download(pyre_ctx* ctx, void* dst, const void* src, size_t n) {
  if (!ctx || (!dst && n) || (!src && n)) return pyre_fail(ctx, PYRE_E_ARG, "pyre_dev_download: null pointer");
  PYRE_HIP(ctx, hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, ctx->stream)); PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

int pyre_prof_enable(pyre_ctx* ctx, int on) { if (!ctx) return PYRE_E_ARG; ctx->prof_on = on != 0; return PYRE_OK; }
int pyre_prof_reset(pyre_ctx* ctx) {
  if (!ctx) return PYRE_E_ARG; PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  for (auto& p : ctx->prof_pending) { ctx->prof_pool.push_back(p.a); ctx->prof_pool.push_back(p.b); }
  ctx->prof_pending.clear(); ctx->prof_acc.clear(); return PYRE_OK;
}
const char* pyre_prof_report(pyre_ctx* ctx) {
  if (!ctx) return "";
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& p : ctx->prof_pending) { float ms = 0; if (hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) { auto& a = ctx->prof_acc[p.name]; a.count++; a.ms += ms; a.bytes += p.bytes; } ctx->prof_pool.push_back(p.a); ctx->prof_pool.push_back(p.b); }
  ctx->prof_pending.clear();
  ctx->prof_text.clear(); char line[256];
  for (auto& kv : ctx->prof_acc) { snprintf(line, sizeof line, "%s %ld %.6f %.0f\n", kv.first.c_str(), kv.second.count, kv.second.ms, kv.second.bytes); ctx->prof_text += line; }
  return ctx->prof_text.c_str();
}

int pyre_synth_blocks(pyre_ctx* ctx, uint32_t ty, size_t n_blocks, uint64_t seed, float d_lo, float d_hi, void* dev_out) {
  if (!ctx || !dev_out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_synth_blocks: null argument");
  int fmt = fmt_from_ggml(ty); if (fmt < 0) return pyre_fail(ctx, PYRE_E_TYPE, "pyre_synth_blocks: unsupported ggml type %u", ty);
  struct { int el, bytes; } g{1, 4}; ggml_geom(ty, &g.el, &g.bytes); size_t nbytes = n_blocks * (size_t)g.bytes; if (!nbytes) return PYRE_OK;
  size_t nw = (nbytes + 7) / 8;
  hipLaunchKernelGGL(k_synth_payload, dim3((unsigned)((nw + 255) / 256)), dim3(256), 0, ctx->stream, seed, nbytes, (uint8_t*)dev_out);
  PYRE_CHECK_LAUNCH(ctx);
  int nf = (fmt == FMT_Q4_K || ty == PYRE_Q5_K) ? 2 : (fmt >= FMT_Q8_0 ? 1 : 0);      // Q4_K, Q5_K: d and dmin
  if (nf) {      // the f16 super-block scale sits at byte 0 of every block format except Q6_K (byte 208) and Q3_K (byte 108)
    hipLaunchKernelGGL(k_synth_scales, dim3((unsigned)((n_blocks + 255) / 256)), dim3(256), 0, ctx->stream, seed, n_blocks, g.bytes, nf, ty == PYRE_Q6_K ? 208 : (ty == PYRE_Q3_K ? 108 : (ty == PYRE_IQ1_M ? -1 : 0)), 2, d_lo, d_hi, (uint8_t*)dev_out);
    PYRE_CHECK_LAUNCH(ctx);
  }
  return PYRE_OK;
}

}  // extern "C"
