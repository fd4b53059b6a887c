// The single-token decode step as ONE persistent kernel: 256 workgroups of 1024 threads stay resident for a run of
// tokens and walk the step's stages together, separated by a grid-wide barrier instead of a kernel boundary (a
// dependent launch costs about 4.6 us on this part, the barrier about 2 us including the data hand-off).
//
// Every stage repeats, operation for operation, the arithmetic of the stand-alone kernel it replaces (qmat.hip, hc.hip,
// gdn.hip, attn.hip, moe.hip at t = 1), so the token stream and the state are bit-identical to the launch-per-stage
// path and to the verify window.  A stage is cut into the same "virtual blocks" the kernel's grid had; a virtual block
// of VT threads occupies the first VT threads of a workgroup (or one of 1024/VT slots of it), the other waves idle
// through the same barriers.
//
// Memory rule: the L2 caches of the eight XCDs are not coherent with each other inside a kernel.  Anything one
// workgroup writes and another reads later in the same launch (activations, the KV cache, routing results) goes through
// agent-scope relaxed atomics (ldc / stc: write-through stores, cache-bypassing loads); weights and other read-only
// data use ordinary loads; recurrent state that only its owner workgroup touches uses ordinary accesses too.
// Activations feeding a dot product are first staged in shared memory (scalar loads would read a non-coherent cache).
#pragma once
#include "formats.h"

namespace mega {

constexpr int WGT = 1024;            // threads per workgroup
constexpr int LDS_BYTES = 61440;     // dynamic shared memory per workgroup

__device__ __forceinline__ float ldc(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ldc(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int32_t ldc(const int32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void stc(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void stc(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void stc(int32_t* p, int32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float nib_val(uint32_t w, int i) { return (float)(((int)(w << (28 - 4 * i))) >> 28); }

// ---- grid barrier ---------------------------------------------------------------------------------------------------
// ctl (u32, zeroed before the launch): [0] round flag, [16] abort flag, [48] top counter, [64 + 16*g] group counters.
// Workgroups count in groups of 16 on their own cache line, the last of a group counts on the top line, the last overall
// publishes the round.  Every wait is bounded: past `limit` polls the waiter raises the abort flag and the whole grid
// leaves (the host reports it as an error).
struct Bar { unsigned* ctl; unsigned round; int nwg; unsigned limit; };
__device__ __forceinline__ bool grid_sync(Bar& b, unsigned* ok_lds) {
  __syncthreads();
  b.round += 1;
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");      // this wave's stores are out; no L2 write-back
    const int gs = 16, grp = blockIdx.x / gs, ngrp = (b.nwg + gs - 1) / gs, gsz = min(gs, b.nwg - grp * gs);
    unsigned* gcnt = b.ctl + 64 + grp * 16; unsigned* top = b.ctl + 48; unsigned* flag = b.ctl; unsigned* abort_flag = b.ctl + 16;
    unsigned prev = __hip_atomic_fetch_add(gcnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (prev + 1 == b.round * (unsigned)gsz) {
      unsigned pt = __hip_atomic_fetch_add(top, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (pt + 1 == b.round * (unsigned)ngrp) __hip_atomic_store(flag, b.round, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    unsigned spins = 0, good = 1;
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < b.round) {
      if (++spins > b.limit || __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); good = 0; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    *ok_lds = good;
  }
  __syncthreads();
  return *ok_lds != 0;
}

// A barrier over the nwg workgroups of ONE launch that leaves its control words ready for the next launch (no host
// reset, so it can sit in a replayed graph): arrivals count up, the last arriver zeroes the count and bumps the
// generation word everybody else polls.  ctl: [0] generation, [16] abort flag, [32] arrival count.  Bounded like grid_sync.
__device__ __forceinline__ bool launch_sync(unsigned* ctl, int nwg, unsigned limit, unsigned* ok_lds) {
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    unsigned* gen = ctl; unsigned* abort_flag = ctl + 16; unsigned* cnt = ctl + 32;
    const unsigned g0 = __hip_atomic_load(gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);      // read before arriving: it cannot move until this workgroup has arrived
    unsigned good = 1;
    if (__hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == (unsigned)nwg) {
      __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(gen, g0 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      unsigned spins = 0;
      while (__hip_atomic_load(gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == g0) {
        if (++spins > limit) { __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); good = 0; break; }
        __builtin_amdgcn_s_sleep(1);
      }
    }
    *ok_lds = good;
  }
  __syncthreads();
  return *ok_lds != 0;
}

// ---- device-side description of the model and of one run --------------------------------------------------------------
struct HcPlan { int nw, upw, ksplit; };
struct GemvPlan { int nw, upw; int grp = 0; };      // grp > 1: the waves' sums are added in groups of grp, then the groups (the stage path's K slices)
struct Layer {
  HcDev hca, hcf; HcPlan pa, pf;
  QMatDev proj, outp; GemvPlan gp, go, gr;      // gr: router
  MoeDev moe; AttnDev attn; GdnDev gdn; KvDev kv;
  float* conv; float* ssm; float* proj_saved;    // DeltaNet: current state buffers (updated in place), raw projections [pw_lin]
  int full;
  int gu_parts;         // K parts of the gate/up dot products (pyre_moe_gu_parts)
};
struct Args {
  const Layer* layers; int n_layers;
  HcDev head; HcPlan ph; QMatDev embd, out; GemvPlan gh;
  int d, hc, ch, pw_lin, pw_attn, conv_k; float eps;
  // activations (one token)
  float *emb, *xa, *xb, *ssq, *part, *mixed, *inj_a, *inj_f, *proj, *co, *core, *o, *hbuf, *vlogits;
  uint32_t* best; MoeWork mw; AttnWork aw;
  uint32_t* toks; uint32_t first; int start_pos, n_steps;
  unsigned* ctl; unsigned limit;
  unsigned long long* stage_ticks;     // optional [16]: 100 MHz ticks per stage class, accumulated by workgroup 0 (diagnostics)
};

struct MoeOutC { const float* partial; const float* sel_w; const float* sg; int d, k; };
__device__ __forceinline__ float moe_out_value_c(const MoeOutC& mo, int r) {          // moe_out_value (common.h) with coherent loads
  const float* p = mo.partial + r;
  float pv[PYRE_MOE_KMAX], wv[PYRE_MOE_KMAX];
#pragma unroll
  for (int j = 0; j < PYRE_MOE_KMAX; ++j) { pv[j] = j < mo.k ? ldc(p + (size_t)j * mo.d) : 0.0f; wv[j] = j < mo.k ? ldc(mo.sel_w + j) : 0.0f; }
  float sh = ldc(p + (size_t)mo.k * mo.d), g = ldc(mo.sg);
  float o = 0.0f;
#pragma unroll
  for (int j = 0; j < PYRE_MOE_KMAX; ++j) if (j < mo.k) o += wv[j] * pv[j];
  return sh * g + o;
}

// ---- stage: hyper-connection norm + [down ; inject] slices (k_hc_norm_down at T = 1) -----------------------------------
struct Comb { const float* out; MoeOutC mo; const float* inj; };       // pending residual update: plain vector, or unreduced FFN output
__device__ __forceinline__ float hc_x_new(const float* x_in, int in_ss, const Comb& cb, float w, int d, int s, int i) {
  float v = ldc(x_in + (size_t)s * in_ss + i);
  if (cb.mo.partial) v = v + moe_out_value_c(cb.mo, i) * w;
  else if (cb.out) v = v + ldc(cb.out + i) * w;
  return v;
}
template <int FMT> __device__ __forceinline__ void st_norm_down(const HcDev& h, const HcPlan& pl, const float* x_in, int in_ss, float* x_out, const Comb& cb,
                                                float* ssq, float* part, const uint2* g2, char* lds) {
  const QMatDev& m = h.di; const int d = h.d, hc = h.hc, nvb = m.tiles * pl.ksplit, VT = pl.nw * 64, upw = pl.upw, nw = pl.nw, L = nw * upw * 64;
  float* xs = (float*)lds; float* red = xs + L; float* wsum = red + nw * 64;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  for (int vb = blockIdx.x; vb < nvb; vb += gridDim.x) {
    const int tile = vb % m.tiles, ks = vb / m.tiles; const bool act = tid < VT;
    const int c0 = ks * L, s = c0 / d, i0 = c0 - s * d;
    UnitRaw<FMT> raw; float w = 0.0f, ss = 0.0f;
    if (act) {
      raw = unit_load<FMT>(m, tile, ks * nw * upw + wave * upw, lane);
      w = (cb.out || cb.mo.partial) ? 2.0f * sigm(ldc(cb.inj + s)) : 0.0f;
      for (int j = tid; j < L; j += VT) {
        const float nv = h.norm[(size_t)s * d + i0 + j];
        float v = hc_x_new(x_in, in_ss, cb, w, d, s, i0 + j);
        ss += v * v;
        xs[j] = v * nv;
        if (tile == 0) stc(x_out + (size_t)s * d + i0 + j, v);
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
      if (lane == 0) wsum[wave] = ss;
    }
    __syncthreads();
    if (tile == 0 && tid == 0) { float tot = wsum[0]; for (int q = 1; q < nw; ++q) tot += wsum[q]; stc(ssq + ks, tot); }
    if (act) {
      float acc[1] = {0.0f};
      for (int u = 0; u < upw; ++u) { int lu = wave * upw + u; if (u > 0) raw = unit_load<FMT>(m, tile, ks * nw * upw + lu, lane); unit_fma<FMT, 1>(m, raw, ks * nw * upw + lu, (const uint2*)nullptr, lane, xs + lu * 64, L, acc); }
      red[wave * 64 + lane] = acc[0];
    }
    __syncthreads();
    if (tid < 64) {
      float a = red[lane]; for (int q = 1; q < nw; ++q) a += red[q * 64 + lane];
      stc(part + (size_t)ks * m.tiles * 64 + (size_t)tile * 64 + lane, a);
    }
    __syncthreads();
  }
  (void)g2; (void)hc;
}

// n (<= 32) values at p, p + stride, ...: groups of four behind launch-uniform branches, all loads of a group in flight
__device__ __forceinline__ void hc_load_run(float (&sv)[32], const float* p, int n, int stride) {
#pragma unroll
  for (int k = 0; k < 32; ++k) sv[k] = 0.0f;
#pragma unroll
  for (int g = 0; g < 8; ++g) if (g * 4 < n) {
#pragma unroll
    for (int j = 0; j < 4; ++j) sv[g * 4 + j] = ldc(p + (size_t)min(g * 4 + j, n - 1) * stride);
  }
}

// ---- stage: stream scales + scaled slice sums + silu + up GEMV + gated stream mean (k_hc_up_mix at T = 1) ----------------
template <int FMT> __device__ __forceinline__ void st_up_mix(const HcDev& h, int ksplit, const float* part, const float* ssq, const float* xnew, float eps, float* mixed, float* inj, char* lds) {
  const QMatDev& up = h.up; const int lr = h.lr, hc = h.hc, d = h.d, U = lr >> 6, r64 = h.di.tiles * 64, nvb = d / 64, VT = hc * U * 64, n_o = lr + hc, kps = ksplit / hc;
  float* lo = (float*)lds; float* red = lo + lr; float* sls = red + (size_t)hc * U * 64;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  auto load_slices = [&](float (&pv)[32], bool want, int i) {
#pragma unroll
    for (int ks = 0; ks < 32; ++ks) pv[ks] = 0.0f;
    if (want) {
#pragma unroll
      for (int g = 0; g < 4; ++g) if (g * 8 < ksplit) {
#pragma unroll
        for (int j = 0; j < 8; ++j) pv[g * 8 + j] = ldc(part + (size_t)min(g * 8 + j, ksplit - 1) * r64 + i);
      }
    }
  };
  for (int vb = blockIdx.x; vb < nvb; vb += gridDim.x) {
    const bool act = tid < VT; const int s = wave / U, ku = wave - s * U;
    UnitRaw<FMT> raw; float pv[32]; int i = tid; bool have = act && i < n_o;
    if (act) raw = unit_load<FMT>(up, s * (d >> 6) + vb, ku, lane);
    load_slices(pv, have && (i < lr || h.has_inject), i);
    if (tid < hc) {
      float sv[32];
      hc_load_run(sv, ssq + tid * kps, kps, 1);
      float tot = sv[0];
#pragma unroll
      for (int k = 1; k < 32; ++k) if (k < kps) tot += sv[k];
      const float sc = 1.0f / sqrtf(tot / (float)d + eps);
      for (int k = 0; k < kps; ++k) sls[tid * kps + k] = sc;
    }
    __syncthreads();
    while (have) {
      float o = 0.0f;
      if (i < lr || h.has_inject) {
#pragma unroll
        for (int ks = 0; ks < 32; ++ks) if (ks < ksplit) { const float term = pv[ks] * sls[ks]; o = ks == 0 ? term : o + term; }
      }
      const float v = o / (float)hc;
      if (i < lr) lo[i] = v * sigm(v);
      else if (vb == 0) stc(inj + (i - lr), h.has_inject ? v : 0.0f);
      i += VT; have = i < n_o;
      if (have) load_slices(pv, i < lr || h.has_inject, i);
    }
    __syncthreads();
    if (act) {
      float acc[1] = {0.0f};
      unit_fma<FMT, 1>(up, raw, ku, (const uint2*)nullptr, lane, lo + ku * 64, lr, acc);
      red[wave * 64 + lane] = acc[0];
    }
    __syncthreads();
    if (tid < 64) {
      const int col = vb * 64 + lane; float mx = 0.0f;
      for (int q = 0; q < hc; ++q) {
        float g = red[(q * U) * 64 + lane];
        for (int k = 1; k < U; ++k) g += red[(q * U + k) * 64 + lane];
        mx += ldc(xnew + (size_t)q * d + col) * sls[q * kps] * h.norm[(size_t)q * d + col] * sigm(g);
      }
      stc(mixed + col, mx / (float)hc);
    }
    __syncthreads();
  }
}

// ---- stage: GEMV with the conv / per-tile-maximum epilogues (k_gemv at T = 1, ksplit = 1) ---------------------------------
// x (cols floats) is staged into shared memory once per workgroup; a virtual block is one row tile handled by nw waves,
// 16 / nw of them side by side in a workgroup.
struct Epi { uint32_t* best; const float* conv_w; float* conv; float* co; int ch, kk; };
template <int FMT> __device__ __forceinline__ void st_gemv(const QMatDev& m, const GemvPlan& gp, const float* x, float* y, const Epi& ep, char* lds) {
  const int tid = threadIdx.x, VT = gp.nw * 64, slots = WGT / VT, slot = tid / VT, vt = tid - slot * VT;
  const int wave = __builtin_amdgcn_readfirstlane(vt >> 6), lane = tid & 63, nw = gp.nw, upw = gp.upw;
  float* xs = (float*)lds; float* red = xs + m.cols + (size_t)slot * nw * 64;
  if ((int)blockIdx.x * slots >= m.tiles) return;                       // no virtual block for this workgroup (uniform)
  for (int i = tid; i < m.cols; i += WGT) xs[i] = ldc(x + i);
  __syncthreads();
  for (int vb0 = blockIdx.x * slots; vb0 < m.tiles; vb0 += gridDim.x * slots) {
    const int tile = vb0 + slot; const bool act = tile < m.tiles;
    float cw[8], chist[8]; const bool conv_row = act && ep.co != nullptr && wave == 0 && tile * 64 + lane < ep.ch;
    if (conv_row) {
      const size_t row = (size_t)tile * 64 + lane;
#pragma unroll
      for (int k = 0; k < 8; ++k) { cw[k] = k < ep.kk ? ep.conv_w[row * ep.kk + k] : 0.0f; chist[k] = k < ep.kk - 1 ? ep.conv[(size_t)k * ep.ch + row] : 0.0f; }
    }
    float acc[1] = {0.0f};
    if (act) {
      const int k0 = wave * upw, k1 = min(m.U, k0 + upw);
      for (int ku = k0; ku < k1; ++ku) unit_dot<FMT, 1>(m, (const uint2*)nullptr, tile, ku, lane, xs + (size_t)ku * 64, m.cols, acc);
    }
    red[wave * 64 + lane] = acc[0];
    __syncthreads();
    if (act && vt < 64) {
      float s = red[lane];
      if (gp.grp > 1) {
        for (int w = 1; w < gp.grp; ++w) s += red[w * 64 + lane];
        for (int g = gp.grp; g < nw; g += gp.grp) { float gs = red[g * 64 + lane]; for (int w = 1; w < gp.grp; ++w) gs += red[(g + w) * 64 + lane]; s += gs; }
      } else for (int w = 1; w < nw; ++w) s += red[w * 64 + lane];
      const size_t row = (size_t)tile * 64 + lane;
      if (row < (size_t)m.rows) stc(y + row, s);
      if (ep.best != nullptr) {
        float bv = row < (size_t)m.rows ? s : -INFINITY; uint32_t bi = (uint32_t)row;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { float ov = __shfl_xor(bv, o); uint32_t oi = __shfl_xor(bi, o); if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; } }
        if (lane == 0) { stc(ep.best + 2 * tile, __float_as_uint(bv)); stc(ep.best + 2 * tile + 1, bi); }
      }
      if (conv_row) {
        float cur = s;
        float o = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) if (k == ep.kk - 1) o = cw[k] * cur;
#pragma unroll
        for (int k = 0; k < 7; ++k) if (k < ep.kk - 1) o += cw[k] * chist[k];
        stc(ep.co + row, o * (1.0f / (1.0f + expf(-o))));
#pragma unroll
        for (int k = 0; k < 7; ++k) if (k + 1 < ep.kk - 1) chist[k] = chist[k + 1];
#pragma unroll
        for (int k = 0; k < 7; ++k) if (k == ep.kk - 2) chist[k] = cur;
#pragma unroll
        for (int k = 0; k < 7; ++k) if (k < ep.kk - 1) ep.conv[(size_t)k * ep.ch + row] = chist[k];
      }
    }
    __syncthreads();
  }
}

// ---- stage: Gated DeltaNet recurrence for one token (k_gdn_delta at t = 1) ----------------------------------------------------
__device__ __forceinline__ void st_delta(const GdnDev& p, const float* pr, const float* co, float* ssm, float* out, char* lds) {
  constexpr int DK = 128, DV = 128, G = 4, R = DK / G, VT = 512;
  float* qs = (float*)lds; float* ks = qs + DK; float* pm = ks + DK; float* po = pm + G * DV; float* red = po + G * DV;
  const int tid = threadIdx.x, j = tid & (DV - 1), grp = tid >> 7;
  const int ch = 2 * p.nk * DK + p.nv * DV, w = p.nv * DV;
  for (int h = blockIdx.x; h < p.nv; h += gridDim.x) {
    const bool act = tid < VT; const int kh = h % p.nk;
    float* st = ssm + (size_t)h * DK * DV;
    float S[R]; float v = 0.0f, g = 0.0f, b = 0.0f;
    if (act) {
#pragma unroll
      for (int r = 0; r < R; ++r) S[r] = st[(size_t)(grp * R + r) * DV + j];
      if (tid < DK) v = ldc(co + kh * DK + tid); else if (tid < 2 * DK) v = ldc(co + p.nk * DK + kh * DK + (tid - DK));
      float sq = v * v;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
      if ((tid & 63) == 0) red[tid >> 6] = sq;
    }
    __syncthreads();
    if (act) {
      if (tid < DK) qs[tid] = v * ((1.0f / sqrtf(red[0] + red[1] + 1e-6f)) * (1.0f / sqrtf((float)DK)));
      else if (tid < 2 * DK) ks[tid - DK] = v * ((1.0f / sqrtf(red[2] + red[3] + 1e-6f)) * 1.0f);
      g = expf(softplus(ldc(pr + ch + w + p.nv + h) + p.dt[h]) * p.a[h]);
      b = sigm(ldc(pr + ch + w + h));
    }
    __syncthreads();
    if (act) {
      float pmv = 0.0f;
#pragma unroll
      for (int r = 0; r < R; ++r) { S[r] *= g; pmv += S[r] * ks[grp * R + r]; }
      pm[grp * DV + j] = pmv;
    }
    __syncthreads();
    if (act) {
      const float mem = ((pm[0 * DV + j] + pm[1 * DV + j]) + pm[2 * DV + j]) + pm[3 * DV + j];
      const float delta = (ldc(co + 2 * p.nk * DK + h * DV + j) - mem) * b;
      float pov = 0.0f;
#pragma unroll
      for (int r = 0; r < R; ++r) { S[r] += ks[grp * R + r] * delta; pov += S[r] * qs[grp * R + r]; }
      po[grp * DV + j] = pov;
    }
    __syncthreads();
    if (tid < DV) {
      float o = ((po[0 * DV + j] + po[1 * DV + j]) + po[2 * DV + j]) + po[3 * DV + j];
      float ss = o * o;
#pragma unroll
      for (int dd = 32; dd > 0; dd >>= 1) ss += __shfl_xor(ss, dd);
      if ((tid & 63) == 0) red[4 + (tid >> 6)] = ss;
      pm[j] = o;
    }
    __syncthreads();
    if (tid < DV) {
      float sc = 1.0f / sqrtf((red[4] + red[5]) / (float)DV + p.eps);
      float o = pm[j] * (sc * p.norm_w[j]);
      stc(out + h * DV + j, o * sigm(ldc(pr + ch + h * DV + j)));
    }
    if (act) {
#pragma unroll
      for (int r = 0; r < R; ++r) st[(size_t)(grp * R + r) * DV + j] = S[r];
    }
    __syncthreads();
  }
}

// ---- stage: attention prep (q/k RMSNorm + RoPE + cache append) and 4-bit packing (k_attn_prep, k_kv_pack) -----------------
__device__ __forceinline__ void st_attn_prep(const AttnDev& a, const KvDev& kv, const float* qkv, int pos, float* qout, char* lds) {
  constexpr int HD = 256;
  float* buf = (float*)lds; float* red = buf + HD;
  const int tid = threadIdx.x, nprep = a.nkv + a.nh;
  for (int b = blockIdx.x; b < nprep; b += gridDim.x) {
    const bool act = tid < HD; const bool is_k = b < a.nkv; const int h = is_k ? b : b - a.nkv;
    const float* src = is_k ? qkv + (size_t)a.nh * 2 * HD + (size_t)h * HD : qkv + (size_t)h * 2 * HD;
    float v = 0.0f;
    if (act) {
      v = ldc(src + tid);
      float ss = v * v;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
      if ((tid & 63) == 0) red[tid >> 6] = ss;
    }
    __syncthreads();
    if (act) {
      float tot = 0.0f;
#pragma unroll
      for (int i = 0; i < HD / 64; ++i) tot += red[i];
      const float sc = 1.0f / sqrtf(tot / (float)HD + a.eps);
      v = v * (sc * (is_k ? a.kn[tid] : a.qn[tid]));
      buf[tid] = v;
    }
    __syncthreads();
    if (act) {
      const int half = a.n_rot / 2;
      if (tid < a.n_rot) {
        int i = tid < half ? tid : tid - half;
        float ang = (float)pos * a.rope_inv[i];
        float sn = sinf(ang), cs = cosf(ang);
        float x0 = buf[i], x1 = buf[i + half];
        v = tid < half ? x0 * cs - x1 * sn : x1 * cs + x0 * sn;
      }
      if (is_k) {
        stc(kv.kf + kv_blk((size_t)h * HD + tid, (size_t)a.nkv * HD, pos), v);
        stc(kv.vf + (size_t)pos * a.nkv * HD + (size_t)h * HD + tid, ldc(qkv + (size_t)a.nh * 2 * HD + (size_t)a.nkv * HD + (size_t)h * HD + tid));
      } else stc(qout + (size_t)h * HD + tid, v);
    }
    __syncthreads();
  }
  // kv4::pack for the positions that fall below the packed boundary when the context grows to pos + 1 (older rows only)
  const int n = pos + 1;
  const int p1 = (a.kv_bits == 4 && n > a.kv_recent + 64) ? ((n - a.kv_recent) / 64) * 64 : 0;
  const int p0 = (a.kv_bits == 4 && n - 1 > a.kv_recent + 64) ? ((n - 1 - a.kv_recent) / 64) * 64 : 0;
  if (p1 > p0 && (int)blockIdx.x >= nprep) {
    const int bpr = a.nkv * HD / 32; const size_t per = (size_t)(p1 - p0) * bpr;
    for (size_t gid0 = (size_t)(blockIdx.x - nprep) * WGT + tid; gid0 < 2 * per; gid0 += (size_t)(gridDim.x - nprep) * WGT) {
      size_t gid = gid0; const bool is_v = gid >= per; if (is_v) gid -= per;
      const int pp = p0 + (int)(gid / bpr), blk = (int)(gid % bpr), kvh = blk / (HD / 32), bb = blk % (HD / 32);
      float x[32];
      for (int i = 0; i < 32; ++i) x[i] = is_v ? ldc(kv.vf + (size_t)pp * a.nkv * HD + (size_t)blk * 32 + i) : ldc(kv.kf + kv_blk((size_t)kvh * HD + bb * 32 + i, (size_t)a.nkv * HD, pp));
      float mm = 0.0f; for (int i = 0; i < 32; ++i) mm = fmaxf(mm, fabsf(x[i]));
      const float s = (mm > 0.0f && isfinite(mm)) ? mm / 7.0f : 0.0f;
      for (int w = 0; w < 4; ++w) {
        uint32_t u = 0;
        for (int jn = 0; jn < 8; ++jn) { int q = s > 0.0f ? (int)fminf(fmaxf(roundf(x[8 * w + jn] / s), -7.0f), 7.0f) : 0; u |= ((uint32_t)q & 0xFu) << (4 * jn); }
        if (is_v) stc(kv.vq + (size_t)pp * (a.nkv * HD / 8) + (size_t)blk * 4 + w, u);
        else stc(kv.kq + kv_blk((size_t)kvh * (HD / 8) + bb * 4 + w, (size_t)a.nkv * (HD / 8), pp), u);
      }
      if (is_v) stc(kv.vs + (size_t)pp * bpr + blk, s); else stc(kv.ks + kv_blk((size_t)kvh * (HD / 32) + bb, (size_t)a.nkv * (HD / 32), pp), s);
    }
  }
}

// ---- stage: attention over the cache, one 256-position chunk x kv head per virtual block (k_attn_decode<256, G>) ---------
typedef float f4m __attribute__((ext_vector_type(4)));
template <int G> __device__ __forceinline__ void st_attn_decode(const AttnDev& a, const KvDev& kv, const float* qbuf, int n, float* part_o, float* part_ml, int max_chunks, char* lds) {
  constexpr int HD = 256, NPW = PYRE_ATTN_NPW, CH = PYRE_ATTN_CHUNK, NT = 256 * NPW;      // the stand-alone kernel's workgroup: NT threads
  float* red = (float*)lds; float* scb = red + 4 * CH * G; float* wmax = scb + CH * G; float* wsum = wmax + NPW * G; float* cm = wsum + NPW * G;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), pw = wave % NPW, dq = (wave / NPW) & 3;
  const bool act = tid < NT;                                // the other waves only keep the barriers company
  const int nchunks = (n + CH - 1) / CH, nvb = nchunks * a.nkv;
  const int pb = (int)((a.kv_bits == 4 && n > a.kv_recent + 64) ? ((n - a.kv_recent) / 64) * 64 : 0);
  const float scale = 1.0f / sqrtf((float)HD);
  const int li = lane & 15, lg = lane >> 4, row = a.nkv * HD;
  for (int vb = blockIdx.x; vb < nvb; vb += gridDim.x) {
    const int chunk = vb % nchunks, kvh = vb / nchunks;
    const int wbase = chunk * CH + pw * 64, p = wbase + lane;
    const bool valid = act && p < n, packed = wbase < pb, active = act && wbase < n;
    {
      f4m D[4];
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) D[pt] = f4m{0.0f, 0.0f, 0.0f, 0.0f};
      if (active) {
        float B[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) B[s] = li < G ? ldc(qbuf + ((size_t)kvh * G + (li < G ? li : 0)) * HD + dq * 64 + 16 * lg + s) : 0.0f;
        float A[4][16];
        if (packed) {
          uint32_t kw[4][2]; float ksc[4];
#pragma unroll
          for (int pt = 0; pt < 4; ++pt) {
            const size_t pp = (size_t)wbase + 16 * pt + li;
            kw[pt][0] = ldc(kv.kq + kv_blk((size_t)kvh * (HD / 8) + dq * 8 + 2 * lg, (size_t)a.nkv * (HD / 8), pp)); kw[pt][1] = ldc(kv.kq + kv_blk((size_t)kvh * (HD / 8) + dq * 8 + 2 * lg + 1, (size_t)a.nkv * (HD / 8), pp));
            ksc[pt] = ldc(kv.ks + kv_blk((size_t)kvh * (HD / 32) + dq * 2 + (lg >> 1), (size_t)a.nkv * (HD / 32), pp));
          }
#pragma unroll
          for (int pt = 0; pt < 4; ++pt)
#pragma unroll
            for (int s = 0; s < 16; ++s) A[pt][s] = nib_val(kw[pt][s >> 3], s & 7) * ksc[pt];
        } else {
#pragma unroll
          for (int pt = 0; pt < 4; ++pt) {
            const size_t pp = (size_t)min(wbase + 16 * pt + li, n - 1);
#pragma unroll
            for (int s = 0; s < 16; ++s) A[pt][s] = ldc(kv.kf + kv_blk((size_t)kvh * HD + dq * 64 + 16 * lg + s, (size_t)a.nkv * HD, pp));
          }
        }
#pragma unroll
        for (int s = 0; s < 16; ++s)
#pragma unroll
          for (int pt = 0; pt < 4; ++pt) D[pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[pt][s], B[s], D[pt], 0, 0, 0);
      }
      if (act && li < G) {
#pragma unroll
        for (int pt = 0; pt < 4; ++pt)
#pragma unroll
          for (int r = 0; r < 4; ++r) red[((size_t)dq * CH + pw * 64 + 16 * pt + 4 * lg + r) * G + li] = D[pt][r];
      }
    }
    __syncthreads();
    constexpr int GH = (G + 3) / 4;
    const int pos = pw * 64 + lane;
    float sv[GH];
#pragma unroll
    for (int gi = 0; gi < GH; ++gi) {
      const int g = dq + 4 * gi; sv[gi] = -INFINITY;
      if (act && g < G) {
        float v = ((red[((size_t)0 * CH + pos) * G + g] + red[((size_t)1 * CH + pos) * G + g]) + red[((size_t)2 * CH + pos) * G + g]) + red[((size_t)3 * CH + pos) * G + g];
        sv[gi] = valid ? v * scale : -INFINITY;
        float mx = sv[gi];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        if (lane == 0) wmax[pw * G + g] = mx;
      }
    }
    __syncthreads();
    if (tid < G) { float mm = wmax[tid]; for (int q = 1; q < NPW; ++q) mm = fmaxf(mm, wmax[q * G + tid]); cm[tid] = mm; }
    __syncthreads();
#pragma unroll
    for (int gi = 0; gi < GH; ++gi) {
      const int g = dq + 4 * gi;
      if (act && g < G) {
        float e = valid ? expf(sv[gi] - cm[g]) : 0.0f; scb[pos * G + g] = e;
        float l = e;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o);
        if (lane == 0) wsum[pw * G + g] = l;
      }
    }
    __syncthreads();
    {
      f4m D[4];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) D[dt] = f4m{0.0f, 0.0f, 0.0f, 0.0f};
      if (active) {
        float A[4][16];
        if (packed) {
          uint32_t vw[16]; float vsc[16];
#pragma unroll
          for (int s = 0; s < 16; ++s) {
            const size_t pg = (size_t)wbase + 4 * s + lg;
            vw[s] = ldc(kv.vq + pg * (row / 8) + (size_t)kvh * (HD / 8) + dq * 8 + (li >> 1));
            vsc[s] = ldc(kv.vs + pg * (row / 32) + (size_t)kvh * (HD / 32) + dq * 2 + (li >> 3));
          }
#pragma unroll
          for (int s = 0; s < 16; ++s) {
            const uint32_t hw = vw[s] >> (16 * (li & 1));
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) A[dt][s] = nib_val(hw, dt) * vsc[s];
          }
        } else {
#pragma unroll
          for (int s = 0; s < 16; ++s) {
            const size_t pg = (size_t)min(wbase + 4 * s + lg, n - 1);
            const float* vp = kv.vf + pg * row + (size_t)kvh * HD + dq * 64 + 4 * li;
            A[0][s] = ldc(vp); A[1][s] = ldc(vp + 1); A[2][s] = ldc(vp + 2); A[3][s] = ldc(vp + 3);
          }
        }
        float B[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) B[s] = li < G ? scb[(pw * 64 + 4 * s + lg) * G + (li < G ? li : 0)] : 0.0f;
#pragma unroll
        for (int s = 0; s < 16; ++s)
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) D[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[dt][s], B[s], D[dt], 0, 0, 0);
      }
      if (act && li < G) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) red[((size_t)pw * G + li) * HD + dq * 64 + 4 * (4 * lg + r) + dt] = D[dt][r];
      }
    }
    __syncthreads();
    for (int i = tid; i < G * HD; i += WGT) {
      int g = i / HD, dd = i % HD;
      float o = red[((size_t)0 * G + g) * HD + dd];
#pragma unroll
      for (int q = 1; q < NPW; ++q) o += red[((size_t)q * G + g) * HD + dd];
      stc(part_o + (((size_t)kvh * G + g) * max_chunks + chunk) * HD + dd, o);
    }
    if (tid < G) {
      float l = wsum[tid]; for (int q = 1; q < NPW; ++q) l += wsum[q * G + tid];
      float* ml = part_ml + (((size_t)kvh * G + tid) * max_chunks + chunk) * 2;
      stc(ml, cm[tid]); stc(ml + 1, l);
    }
    __syncthreads();
  }
}

// ---- stage: merge the chunk partials, normalise, gate (k_attn_combine) ------------------------------------------------------
__device__ __forceinline__ void st_attn_combine(const AttnDev& a, const float* qkv, int n, const float* part_o, const float* part_ml, int max_chunks, float* out, char* lds) {
  constexpr int HD = 256;
  float* wmax = (float*)lds; float* so = wmax + 16; float* sl = so + 4 * HD;
  const int tid = threadIdx.x, grp = tid / HD, dd = tid % HD, nc = (n + PYRE_ATTN_CHUNK - 1) / PYRE_ATTN_CHUNK;
  for (int h = blockIdx.x; h < a.nh; h += gridDim.x) {
    const float* ml = part_ml + (size_t)h * max_chunks * 2;
    const float* po = part_o + (size_t)h * max_chunks * HD;
    float M = -INFINITY; for (int c = tid; c < nc; c += 4 * HD) M = fmaxf(M, ldc(ml + 2 * c));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
    if ((tid & 63) == 0) wmax[tid >> 6] = M;
    __syncthreads();
    M = wmax[0];
#pragma unroll
    for (int i = 1; i < 4 * HD / 64; ++i) M = fmaxf(M, wmax[i]);
    float L = 0.0f, o = 0.0f;
#pragma unroll 4
    for (int c = grp; c < nc; c += 4) { float f = expf(ldc(ml + 2 * c) - M); L = fmaf(ldc(ml + 2 * c + 1), f, L); o = fmaf(ldc(po + (size_t)c * HD + dd), f, o); }
    so[grp * HD + dd] = o; if (dd == 0) sl[grp] = L;
    __syncthreads();
    if (grp == 0) {
      o = ((so[0 * HD + dd] + so[1 * HD + dd]) + so[2 * HD + dd]) + so[3 * HD + dd]; L = ((sl[0] + sl[1]) + sl[2]) + sl[3];
      float gate = ldc(qkv + (size_t)h * 2 * HD + HD + dd);
      stc(out + (size_t)h * HD + dd, (o / L) * sigm(gate));
    }
    __syncthreads();
  }
}

// ---- stage: routing + expert gate/up (route_topk + k_moe_gu<FMT, 16>) -------------------------------------------------------
struct RouteLds { float c_val[16 * 32]; int c_idx[16 * 32]; float r_val[32]; int r_idx[32]; float s_val[32]; int s_idx[32]; float s_w[32]; };
__device__ __forceinline__ void route_topk(const float* logits, int n_exp, int k, RouteLds& L) {
  const int e = threadIdx.x, lane = e & 63, wave = e >> 6, nwa = (n_exp + 63) >> 6;
  if (wave < nwa) {
    float v = -INFINITY;
    if (e < n_exp) { v = ldc(logits + e); if (isnan(v)) v = -INFINITY; }
    int lr = 0;
#pragma unroll
    for (int j = 0; j < 64; ++j) { float u = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), j)); lr += (u > v || (u == v && j < lane)) ? 1 : 0; }
    if (lr < k) { L.c_val[wave * k + lr] = v; L.c_idx[wave * k + lr] = e; }
  }
  __syncthreads();
  const int nc = nwa * k; int SP = 8; while (SP > 1 && nc * SP > WGT) SP >>= 1;
  {
    const int c = e / SP, part = e % SP, per = (nc + SP - 1) / SP; int rank = 0;
    float cv = 0.0f; int ci = 0;
    if (c < nc) {
      cv = L.c_val[c]; ci = L.c_idx[c];
      const int j1 = min(nc, (part + 1) * per);
      for (int j = part * per; j < j1; ++j) { float u = L.c_val[j]; int ui = L.c_idx[j]; rank += (u > cv || (u == cv && ui < ci)) ? 1 : 0; }
    }
    for (int o = 1; o < SP; o <<= 1) rank += __shfl_xor(rank, o);
    if (c < nc && part == 0 && rank < k) { L.r_val[rank] = cv; L.r_idx[rank] = ci; }
  }
  __syncthreads();
  if (e < k) { int me = L.r_idx[e], pos = 0; for (int j = 0; j < k; ++j) pos += L.r_idx[j] < me ? 1 : 0; L.s_idx[pos] = me; L.s_val[pos] = L.r_val[e]; }
  __syncthreads();
}
__device__ __forceinline__ void route_weights(int k, RouteLds& L) {
  const int e = threadIdx.x;
  float mx = -INFINITY, ex = 1.0f;
  if (e < k) { for (int i = 0; i < k; ++i) mx = fmaxf(mx, L.s_val[i]); ex = isfinite(mx) ? expf(L.s_val[e] - mx) : 1.0f; L.r_val[e] = ex; }
  __syncthreads();
  if (e < k) {
    float w;
    if (!isfinite(mx)) w = 1.0f / (float)k;
    else { float sum = 0.0f; for (int i = 0; i < k; ++i) sum += L.r_val[i]; w = ex / sum; }
    L.s_w[e] = w;
  }
}
template <int FMT> __device__ __forceinline__ void st_route_gu(const MoeDev& m, const float* logits, int32_t* sel_idx, float* sel_w, float* sg, const float* x, float* h, int hstride, int parts, char* lds) {
  constexpr int NW = 16, PMAX = 2;       // red: [gate, up][part][wave][64]
  float* xs = (float*)lds; float* red = xs + m.d; RouteLds& rl = *(RouteLds*)(red + 2 * PMAX * NW * 64);
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int tiles = hstride / 64, k1 = m.top_k + 1, nvb = tiles * k1;
  if ((int)blockIdx.x >= nvb) return;
  for (int i = tid; i < m.d; i += WGT) xs[i] = ldc(x + i);
  __syncthreads();
  for (int vb = blockIdx.x; vb < nvb; vb += gridDim.x) {
    const int bx = vb % tiles, j = vb / tiles; const bool shared = j == m.top_k;
    const int nrows = shared ? m.sf : m.ff;
    if (bx * 64 >= nrows) continue;                     // uniform over the workgroup
    int expert = 0;
    if (!shared) {
      route_topk(logits, m.n_exp, m.top_k, rl);
      expert = __builtin_amdgcn_readfirstlane(rl.s_idx[j]);
    } else if (bx == 0) {
      float p = 0.0f; for (int i = tid; i < m.d; i += NW * 64) p = fmaf(m.sh_gate_inp[i], xs[i], p);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) p += __shfl_xor(p, o);
      if (lane == 0) red[wave * 64] = p;
      __syncthreads();
      if (tid == 0) { float tot = 0.0f; for (int w = 0; w < NW; ++w) tot += red[w * 64]; rl.s_w[0] = 1.0f / (1.0f + expf(-tot)); }
      __syncthreads();
    }
    const QMatDev& Gm = shared ? m.sh_gate : m.gate_e; const QMatDev& Up = shared ? m.sh_up : m.up_e;
    const int tile = (shared ? 0 : expert * (m.ff >> 6)) + bx;
    // a dot product is the sum of its K parts in order, a part the sum of its wave shares in wave order (k_moe_gu)
    const int upw = (Gm.U + NW * parts - 1) / (NW * parts);
    for (int p = 0; p < parts; ++p) {
      const int k0 = min(Gm.U, (wave * parts + p) * upw), kend = min(Gm.U, k0 + upw);
      float ag[1] = {0.0f}, au[1] = {0.0f};
      for (int ku = k0; ku < kend; ++ku) { unit_dot<FMT, 1>(Gm, (const uint2*)nullptr, tile, ku, lane, xs + ku * 64, 0, ag); unit_dot<FMT, 1>(Up, (const uint2*)nullptr, tile, ku, lane, xs + ku * 64, 0, au); }
      red[(p * NW + wave) * 64 + lane] = ag[0]; red[((PMAX + p) * NW + wave) * 64 + lane] = au[0];
    }
    __syncthreads();
    if (tid < 64) {
      float g = 0.0f, u = 0.0f;
      for (int p = 0; p < parts; ++p) {
        float gp = red[(p * NW) * 64 + lane], up = red[((PMAX + p) * NW) * 64 + lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) { gp += red[(p * NW + w) * 64 + lane]; up += red[((PMAX + p) * NW + w) * 64 + lane]; }
        if (p == 0) { g = gp; u = up; } else { g += gp; u += up; }
      }
      float s = 1.0f / (1.0f + expf(-g));
      stc(h + (size_t)j * hstride + bx * 64 + lane, (g * s) * u);
    }
    if (bx == 0) {
      if (shared) { if (tid == 0) stc(sg, rl.s_w[0]); }
      else if (j == 0) {
        route_weights(m.top_k, rl);
        if (tid < m.top_k) { stc(sel_idx + tid, rl.s_idx[tid]); stc(sel_w + tid, rl.s_w[tid]); }
      }
    }
    __syncthreads();
  }
}

// ---- stage: expert down projections (k_moe_down<FMT, 8>), two virtual blocks per workgroup -------------------------------------
template <int FMT> __device__ __forceinline__ void st_moe_down(const MoeDev& m, const int32_t* sel_idx, const float* h, int hstride, float* partial, char* lds) {
  constexpr int NW = 8, VT = NW * 64, SLOTS = WGT / VT;
  const int tid = threadIdx.x, slot = tid / VT, vt = tid - slot * VT, wave = __builtin_amdgcn_readfirstlane(vt >> 6), lane = tid & 63;
  const int tiles = m.d / 64, k1 = m.top_k + 1, nvb = tiles * k1;
  float* xs = (float*)lds + (size_t)slot * (hstride + NW * 64); float* red = xs + hstride;
  for (int vb0 = blockIdx.x * SLOTS; vb0 < nvb; vb0 += gridDim.x * SLOTS) {
    const int vb = vb0 + slot; const bool act = vb < nvb;
    const int bx = act ? vb % tiles : 0, j = act ? vb / tiles : 0; const bool shared = j == m.top_k;
    const QMatDev& D = shared ? m.sh_down : m.down_e;
    if (act) for (int i = vt; i < D.cols; i += VT) xs[i] = ldc(h + (size_t)j * hstride + i);
    int tile = bx;
    if (act && !shared) tile = ldc(sel_idx + j) * (m.d >> 6) + bx;
    __syncthreads();
    float acc[1] = {0.0f};
    if (act) {
      const int upw = (D.U + NW - 1) / NW, k0 = wave * upw, kend = min(D.U, k0 + upw);
      for (int ku = k0; ku < kend; ++ku) unit_dot<FMT, 1>(D, (const uint2*)nullptr, tile, ku, lane, xs + ku * 64, 0, acc);
    }
    red[wave * 64 + lane] = acc[0];
    __syncthreads();
    if (act && vt < 64) {
      float s = red[lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) s += red[w * 64 + lane];
      stc(partial + (size_t)j * m.d + bx * 64 + lane, s);
    }
    __syncthreads();
  }
}

// ---- stage: greedy pick from the head's per-tile maxima + embedding row of the chosen token (k_pick) -------------------------
template <int FMT> __device__ __forceinline__ void st_pick_embed(const uint32_t* best, int n_tiles, bool have_best, uint32_t given, const QMatDev& embd, float* emb, uint32_t* tok_out, char* lds) {
  float* sv = (float*)lds; uint32_t* si = (uint32_t*)(sv + 16); uint32_t* chosen = si + 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nvb = emb ? (embd.U + WGT - 1) / WGT : 1;  // embedding units are spread over workgroups; every one redoes the scan
  if ((int)blockIdx.x >= nvb) return;
  uint32_t id = given;
  if (have_best) {
    float bv = -INFINITY; uint32_t bi = 0xFFFFFFFFu;
    for (int i = tid; i < n_tiles; i += WGT) { float v = __uint_as_float(ldc(best + 2 * i)); uint32_t r = ldc(best + 2 * i + 1); if (bi == 0xFFFFFFFFu || v > bv || (v == bv && r < bi)) { bv = v; bi = r; } }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { float ov = __shfl_xor(bv, o); uint32_t oi = __shfl_xor(bi, o); if (oi != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; } }
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
      float fv = sv[0]; uint32_t fi = si[0];
      for (int w = 1; w < WGT / 64; ++w) { float ov = sv[w]; uint32_t oi = si[w]; if (oi != 0xFFFFFFFFu && (fi == 0xFFFFFFFFu || ov > fv || (ov == fv && oi < fi))) { fv = ov; fi = oi; } }
      if (fi == 0xFFFFFFFFu) fi = 0;
      *chosen = fi;
    }
    __syncthreads();
    id = *chosen;
  }
  if (blockIdx.x == 0 && tid == 0 && tok_out) stc(tok_out, id);
  const int ku = blockIdx.x * WGT + tid;
  if (emb && ku < embd.U && id < (uint32_t)embd.rows) {
    float y[64];
    decode_exact<FMT>(embd, (const uint64_t*)nullptr, (int)(id >> 6), ku, (int)(id & 63), y);
    for (int i = 0; i < 64; ++i) stc(emb + (size_t)ku * 64 + i, y[i]);
  }
}

// ---- one hyper-connection mix in one launch (single-token steps): norm + [down ; inject] slices, a barrier over the
// launch's own workgroups instead of a kernel boundary, then slice sums + up GEMV + gated stream mean --------------------
template <int FMT> __global__ __launch_bounds__(WGT) void k_hc_mix_fused(HcDev h, HcPlan pl, const float* x_in, int in_ss, float* x_out, Comb cb, float eps,
                                                                       float* ssq, float* part, float* mixed, float* inj, unsigned* ctl, unsigned limit) {
  extern __shared__ __align__(16) char lds[];
  __shared__ unsigned bar_ok;
  st_norm_down<FMT>(h, pl, x_in, in_ss, x_out, cb, ssq, part, nullptr, lds);
  if (!launch_sync(ctl, (int)gridDim.x, limit, &bar_ok)) return;
  st_up_mix<FMT>(h, pl.ksplit, part, ssq, x_out, eps, mixed, inj, lds);
}

// ---- the kernel --------------------------------------------------------------------------------------------------------
// FW: format of every matrix except the router (FR).  One launch runs a.n_steps tokens.
template <int FW, int FR> __global__ __launch_bounds__(WGT) void k_decode(Args a) {
  extern __shared__ __align__(16) char lds[];
  __shared__ unsigned bar_ok;
  Bar bar{a.ctl, 0u, (int)gridDim.x, a.limit};
  unsigned long long t_last = a.stage_ticks ? wall_clock64() : 0ull, t_acc[13] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};     // kept in registers
#define MEGA_SYNC(cls) do { if (!grid_sync(bar, &bar_ok)) return; \
    if (a.stage_ticks) { unsigned long long t_now = wall_clock64(); t_acc[cls] += t_now - t_last; t_last = t_now; } } while (0)
  const int d = a.d, hc = a.hc;
  for (int step = 0; step < a.n_steps; ++step) {
    const int pos = a.start_pos + step;
    // token: given for the first step, afterwards the greedy pick of the previous head; its embedding row
    st_pick_embed<FW>(a.best, a.out.tiles, step > 0, a.first, a.embd, a.emb, step > 0 ? a.toks + (step - 1) : nullptr, lds);
    MEGA_SYNC(0);
    const float* xin = a.emb; int in_ss = 0; float* xout = a.xa; float* xother = a.xb;
    Comb cb{nullptr, MoeOutC{nullptr, nullptr, nullptr, 0, 0}, nullptr};
    for (int il = 0; il < a.n_layers; ++il) {
      const Layer& L = a.layers[il];
      st_norm_down<FW>(L.hca, L.pa, xin, in_ss, xout, cb, a.ssq, a.part, nullptr, lds);
      MEGA_SYNC(1);
      xin = xout; in_ss = d; { float* q = xout; xout = xother; xother = q; }
      st_up_mix<FW>(L.hca, L.pa.ksplit, a.part, a.ssq, xin, a.eps, a.mixed, a.inj_a, lds);
      MEGA_SYNC(2);
      if (L.full) {
        st_gemv<FW>(L.proj, L.gp, a.mixed, a.proj, Epi{nullptr, nullptr, nullptr, nullptr, 0, 0}, lds);
        MEGA_SYNC(3);
        st_attn_prep(L.attn, L.kv, a.proj, pos, a.aw.q, lds);
        MEGA_SYNC(4);
        const int G = L.attn.nh / L.attn.nkv;
        if (G == 8) st_attn_decode<8>(L.attn, L.kv, a.aw.q, pos + 1, a.aw.part_o, a.aw.part_ml, a.aw.max_chunks, lds);
        else if (G == 4) st_attn_decode<4>(L.attn, L.kv, a.aw.q, pos + 1, a.aw.part_o, a.aw.part_ml, a.aw.max_chunks, lds);
        else if (G == 2) st_attn_decode<2>(L.attn, L.kv, a.aw.q, pos + 1, a.aw.part_o, a.aw.part_ml, a.aw.max_chunks, lds);
        else st_attn_decode<1>(L.attn, L.kv, a.aw.q, pos + 1, a.aw.part_o, a.aw.part_ml, a.aw.max_chunks, lds);
        MEGA_SYNC(5);
        st_attn_combine(L.attn, a.proj, pos + 1, a.aw.part_o, a.aw.part_ml, a.aw.max_chunks, a.core, lds);
        MEGA_SYNC(6);
      } else {
        st_gemv<FW>(L.proj, L.gp, a.mixed, L.proj_saved, Epi{nullptr, L.gdn.conv_w, L.conv, a.co, a.ch, a.conv_k}, lds);
        MEGA_SYNC(3);
        st_delta(L.gdn, L.proj_saved, a.co, L.ssm, a.core, lds);
        MEGA_SYNC(7);
      }
      st_gemv<FW>(L.outp, L.go, a.core, a.o, Epi{nullptr, nullptr, nullptr, nullptr, 0, 0}, lds);
      MEGA_SYNC(8);
      Comb ca{a.o, MoeOutC{nullptr, nullptr, nullptr, 0, 0}, a.inj_a};
      st_norm_down<FW>(L.hcf, L.pf, xin, in_ss, xout, ca, a.ssq, a.part, nullptr, lds);
      MEGA_SYNC(1);
      xin = xout; { float* q = xout; xout = xother; xother = q; }
      st_up_mix<FW>(L.hcf, L.pf.ksplit, a.part, a.ssq, xin, a.eps, a.mixed, a.inj_f, lds);
      MEGA_SYNC(2);
      st_gemv<FR>(L.moe.router, L.gr, a.mixed, a.mw.logits, Epi{nullptr, nullptr, nullptr, nullptr, 0, 0}, lds);
      MEGA_SYNC(9);
      const int hs = L.moe.ff > L.moe.sf ? L.moe.ff : L.moe.sf;
      st_route_gu<FW>(L.moe, a.mw.logits, a.mw.sel_idx, a.mw.sel_w, a.mw.sg, a.mixed, a.mw.h, hs, L.gu_parts, lds);
      MEGA_SYNC(10);
      st_moe_down<FW>(L.moe, a.mw.sel_idx, a.mw.h, hs, a.mw.partial, lds);
      MEGA_SYNC(11);
      cb = Comb{nullptr, MoeOutC{a.mw.partial, a.mw.sel_w, a.mw.sg, d, L.moe.top_k}, a.inj_f};
    }
    st_norm_down<FW>(a.head, a.ph, xin, in_ss, xout, cb, a.ssq, a.part, nullptr, lds);
    MEGA_SYNC(1);
    st_up_mix<FW>(a.head, a.ph.ksplit, a.part, a.ssq, xout, a.eps, a.hbuf, a.inj_a, lds);
    MEGA_SYNC(2);
    st_gemv<FW>(a.out, a.gh, a.hbuf, a.vlogits, Epi{a.best, nullptr, nullptr, nullptr, 0, 0}, lds);
    MEGA_SYNC(12);
  }
  // the last token's pick (no embedding needed)
  st_pick_embed<FW>(a.best, a.out.tiles, true, 0u, a.embd, nullptr, a.toks + (a.n_steps - 1), lds);
  if (a.stage_ticks && blockIdx.x == 0 && threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < 13; ++i) a.stage_ticks[i] += t_acc[i];
  }
#undef MEGA_SYNC
  (void)hc;
}

}  // namespace mega
