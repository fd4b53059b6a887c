// The pieces of the IQ3_S matrix-core product that more than one kernel uses: what a wave fetches for a 128-column chunk
// of the matrix-core layout (QMatDev::mq / mh) and chunk_mac, the product of that chunk with sixteen activation rows
// (two f16 halves of up to eight tokens).  See gemm_m.hip for the arithmetic.
#pragma once
#include "formats.h"

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

// What a wave fetches for one chunk: from the matrix (memory) its row groups' codes and super-block headers, from the
// operand (second-level cache) the sixteen activation rows and their scale factors.
template <int G> struct WBuf { uint4 w[G]; uint2 h[G]; };
struct ABuf { uint4 a[4]; float ai0, ai1; };

template <int G> __device__ __forceinline__ void load_w(const QMatDev& m, int rg0, int c, int lane, int K128, WBuf<G>& b) {
#pragma unroll
  for (int g = 0; g < G; ++g) b.w[g] = ((const uint4*)m.mq)[mq_slot((size_t)rg0 + g, c, K128) + lane];
#pragma unroll
  for (int g = 0; g < G; ++g) b.h[g] = ((const uint2*)m.mh)[mh_slot((size_t)rg0 + g, c >> 1, m.SB) + (lane & 15)];
}
// Every load is unconditional, so that the compiler's count of outstanding loads is exact and a wait for one chunk never
// drains the chunks requested after it: operand rows the window does not have are read through a buffer descriptor at an
// offset past its end, which returns zeros without touching memory.
struct AopRsrc { __amdgpu_buffer_rsrc_t r; int lane_off; };       // lane_off: byte offset of the lane's row inside an (8-column group) x R block, or -1
__device__ __forceinline__ AopRsrc aop_rsrc(const uint4* aop, int cols, int R, int lane) {
  AopRsrc a; a.r = __builtin_amdgcn_make_buffer_rsrc((void*)aop, 0, (cols >> 3) * R * 16, 0x00020000);
  a.lane_off = (lane & 15) < R ? ((lane >> 4) * R + (lane & 15)) * 16 : -1; return a;
}
template <bool SC> __device__ __forceinline__ void load_a(const AopRsrc& ar, const float* __restrict__ ainv, int R, int c, int lane, ABuf& b) {
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int off = ar.lane_off < 0 ? -1 : ar.lane_off + (c * 4 + s) * 4 * R * 16;
    const auto v = __builtin_amdgcn_raw_buffer_load_b128(ar.r, off, 0, 0);
    b.a[s] = make_uint4(v[0], v[1], v[2], v[3]);
  }
  b.ai0 = 1.0f; b.ai1 = 1.0f;
  if constexpr (SC) { const float2 p = ((const float2*)ainv)[(c >> 1) * 4 + (lane >> 4)]; b.ai0 = p.x; b.ai1 = p.y; }
}

// The operand of PyreAop::sq: chunk c is head c, sub-block s the columns of the head's workgroup s.  A lane rescales its
// row's four sub-blocks from their own powers of two to the largest factor's inverse (exact: a multiplication of an f16
// number by a power of two not above one; what falls below the subnormals is 2^-24 of the chunk's largest value) and takes,
// for the two tokens whose sums it holds, that factor times 1 / sqrt(mean square + eps) as the chunk's scale.
__device__ __forceinline__ void load_a_sq(const AopRsrc& ar, const float* __restrict__ sq, int heads, float eps, int R, int c, int lane, ABuf& b) {
  typedef _Float16 h2v_ __attribute__((ext_vector_type(2)));
  const int trow = (lane & 15) >> 1, q = lane >> 4;
  const float4 dr = *(const float4*)(sq + ((size_t)trow * heads + c) * 4);
  const float4 d0 = *(const float4*)(sq + ((size_t)(2 * q) * heads + c) * 4), d1 = *(const float4*)(sq + ((size_t)(2 * q + 1) * heads + c) * 4);
  const float* ssq = sq + (size_t)8 * heads * 4;
  const float4 s0 = *(const float4*)(ssq + ((size_t)(2 * q) * heads + c) * 4), s1 = *(const float4*)(ssq + ((size_t)(2 * q + 1) * heads + c) * 4);
  const float mr = fmaxf(fmaxf(dr.x, dr.y), fmaxf(dr.z, dr.w));
  // the quotients of two powers of two, by their exponents (no division on this path)
  const uint32_t mb = __float_as_uint(mr) - 0x3F800000u;
  const float fr[4] = {__uint_as_float(__float_as_uint(dr.x) - mb), __uint_as_float(__float_as_uint(dr.y) - mb), __uint_as_float(__float_as_uint(dr.z) - mb), __uint_as_float(__float_as_uint(dr.w) - mb)};
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int off = ar.lane_off < 0 ? -1 : ar.lane_off + (c * 4 + s) * 4 * R * 16;
    const auto v = __builtin_amdgcn_raw_buffer_load_b128(ar.r, off, 0, 0);
    const h2v_ f = {(_Float16)fr[s], (_Float16)fr[s]};
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2v_, (uint32_t)v[k]) * f);
    b.a[s] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  const float m0 = fmaxf(fmaxf(d0.x, d0.y), fmaxf(d0.z, d0.w)), m1 = fmaxf(fmaxf(d1.x, d1.y), fmaxf(d1.z, d1.w));
  b.ai0 = m0 * __builtin_amdgcn_rsqf((((s0.x + s0.y) + s0.z) + s0.w) * (1.0f / 128.0f) + eps);          // (the hardware reciprocal square root: one unit in the last place)
  b.ai1 = m1 * __builtin_amdgcn_rsqf((((s1.x + s1.y) + s1.z) + s1.w) * (1.0f / 128.0f) + eps);
}

// The two constants of the nibble -> f16 step.  They are kept in registers the compiler cannot see through, so that
// (x & K) | E stays one instruction (a second literal would split it).
struct NibK { uint32_t K, E; };
__device__ __forceinline__ NibK nib_consts() { NibK k; asm volatile("s_mov_b32 %0, 0x03C003C0" : "=s"(k.K)); asm volatile("v_mov_b32 %0, 0x4C004C00" : "=v"(k.E)); return k; }
// eight 4-bit fields of u -> four registers of two f16 numbers 16 + field: fields 0 and 4, 1 and 5, 2 and 6, 3 and 7
__device__ __forceinline__ void nib_f16(uint32_t u, const NibK& k, uint32_t (&p)[4]) {
  p[0] = ((u << 6) & k.K) | k.E; p[1] = ((u << 2) & k.K) | k.E; p[2] = ((u >> 2) & k.K) | k.E; p[3] = ((u >> 6) & k.K) | k.E;
}

// tot[g] += (this chunk's 128 columns of row group g) x (the sixteen activation rows), scaled
template <int G> __device__ __forceinline__ void chunk_mac(const WBuf<G>& wb, const ABuf& ab, int c, const NibK& nk, v4f (&tot)[G]) {
  const int sh = 8 * (c & 1);                // the chunk's four sub-block scales: header fields (0, 4, 1, 5) of the scale word shifted by this
  const v2h four = {(_Float16)4.0f, (_Float16)4.0f}, m62 = {(_Float16)-62.0f, (_Float16)-62.0f}, m235 = {(_Float16)-23.5f, (_Float16)-23.5f};
#pragma unroll
  for (int g = 0; g < G; ++g) {
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t wd[4] = {wb.w[g].x, wb.w[g].y, wb.w[g].z, wb.w[g].w};
    const uint32_t a4[4][4] = {{ab.a[0].x, ab.a[0].y, ab.a[0].z, ab.a[0].w}, {ab.a[1].x, ab.a[1].y, ab.a[1].z, ab.a[1].w}, {ab.a[2].x, ab.a[2].y, ab.a[2].z, ab.a[2].w}, {ab.a[3].x, ab.a[3].y, ab.a[3].z, ab.a[3].w}};
    // the sub-block scales as f16 pairs: 16 + n -> 2s = 4 (16 + n) - 62 and -47s = -23.5 * 2s, s = 2n + 1, all exact
    const uint32_t hs = wb.h[g].y >> sh;
    const uint32_t np0 = ((hs << 6) & nk.K) | nk.E, np1 = ((hs << 2) & nk.K) | nk.E;
    v2h s2[2], s47[2];
    s2[0] = __builtin_elementwise_fma(__builtin_bit_cast(v2h, np0), four, m62); s2[1] = __builtin_elementwise_fma(__builtin_bit_cast(v2h, np1), four, m62);
    s47[0] = s2[0] * m235; s47[1] = s2[1] * m235;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const v2h vs2 = {s2[s >> 1][s & 1], s2[s >> 1][s & 1]}, vs47 = {s47[s >> 1][s & 1], s47[s >> 1][s & 1]};
      uint32_t p[4], q[4];
      nib_f16(wd[s], nk, p);
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(v2h, p[i]), vs2, vs47));
      struct U4 { uint32_t x[4]; };
      const v8h B = __builtin_bit_cast(v8h, (U4{{q[0], q[1], q[2], q[3]}}));
      const v8h A = __builtin_bit_cast(v8h, (U4{{a4[s][0], a4[s][1], a4[s][2], a4[s][3]}}));
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, acc, 0, 0, 0);
    }
    const float d = h2f_bits(wb.h[g].x & 0xFFFFu);
    const float d0 = d * ab.ai0, d1 = d * ab.ai1;
    tot[g][0] = fmaf(acc[0], d0, tot[g][0]); tot[g][1] = fmaf(acc[1], d0, tot[g][1]);
    tot[g][2] = fmaf(acc[2], d1, tot[g][2]); tot[g][3] = fmaf(acc[3], d1, tot[g][3]);
  }
}

