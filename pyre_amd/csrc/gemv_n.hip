// IQ3_S dequant-GEMV at the file's bits per weight, single token (QMat::matmul with t = 1, src/model/gguf_q.rs:217-242;
// the GPU decode of this type in the reference: src/model/qn_cube.rs:3354-3382).
//
// The matrix-core layout (gemm_m.hip) holds an IQ3_S weight as a resolved 4-bit code: 4.25 bit/weight against the file's
// 3.4375, so a GEMV that is bound by bytes streams 1.24 x what the file holds.  Here a matrix keeps what the file keeps --
// per four weights the 9-bit codebook index and the four sign bits, per 32 the 4-bit scale, per 256 the f16 d -- and the
// codebook lives in shared memory with the signs folded in: 8192 entries (index | signs << 9) of four signed bytes,
// 32 KB per workgroup, filled once by a workgroup that then walks row tiles.
//   layout: per row and 256-column super-block 112 bytes (3.5 bit/weight: the file's 110 bytes + 2 of padding):
//           bits 13 g .. 13 g + 12 = field of group g (columns 4 g .. 4 g + 3), g < 64; bits 832 + 4 i .. = scale of
//           sub-block i; bits 864 .. 879 = d; as seven 16-byte pieces, nq[tile][super-block][piece][lane] with lane = row of
//           the tile, so a wave fetches every piece with one coalesced load.
//   activations: block fixed point as three signed bytes per value, one power of two per 64 columns
//           (x = su * q, |q| <= 2^21, q = a1 * 65536 + a2 * 256 + a3), laid out per group so that the lookups' bytes meet
//           their columns' digits in v_dot4_i32_i8; they are wave-uniform, i.e. scalar loads.
//   per four weights: two instructions for the table offset (a 32-bit window of the packed fields, a mask), one shared-memory
//           read, three dot instructions; per 32 weights the three digit sums are joined in int32 (exact), converted once and
//           scaled by d * (1 + 2 s) * su in f32.
// The only rounding beyond the f32 path's is the representation of x: |x - su q| <= 2^-22 of the 64 columns' largest
// magnitude.  t >= 2 stays on the matrix cores, where a window costs what a token does.
//
// IQ2_XS (F = 1 below; gguf_q.rs:126-129) goes the same way.  The file keeps per eight weights a 16-bit word (9-bit codebook
// index, 7-bit index into the sign table, whose eighth sign is the parity of the seven); here the parity is resolved at load
// and a field is 17 bits: index | signs of weights 0..3 << 9 | signs of weights 4..7 << 13.  32 fields + 8 scale bytes + d =
// 78 bytes, kept as five 16-byte pieces: 80 bytes per 256 weights (2.5 bit/weight against the file's 2.3125).  The signed
// codebook is two tables of 8192 entries (weights 0..3 and 4..7 of an entry: index | four signs << 9), 64 KB of shared
// memory; a 16-weight half of a sub-block has its own 4-bit scale, (2 n + 1) / 8, so the digit sums are joined per half.
//
// Q4_K (P = 9; gguf_q.rs:96-120) needs no table: a block's 144 bytes are kept as they are, nine lane = row pieces (the header
// with d, dmin and the twelve scale bytes, then the 128 bytes of nibbles).  A dword of nibbles is four weights of one
// sub-block (low nibbles) and four of the next (high nibbles): two masks give the two byte vectors for v_dot4_i32_i8, and
// the dmin * min term leaves through the sub-block's sum of activation digits, which the digits launch provides.
#include "formats.h"
#include "iq_codebooks.h"

#define DGN_STRIDE 64      // dwords per 64-column unit: 48 digit words [(sub-block*8 + group)*3 + digit], then su, the two sub-blocks' integer sums, pad

// ---- the matrix: raw GGUF rows -> nq; one thread per (padded row, super-block) ---------------------------------------------
__global__ __launch_bounds__(256) void k_repack_n(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, uint4* __restrict__ nq) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB) return;
  const int row = (int)(idx / SB), sb = (int)(idx % SB); const bool live = row < rows;      // padding rows lie past the end of the raw buffer: never read them
  uint32_t w[28];
  for (int i = 0; i < 28; ++i) w[i] = 0;
  if (live) {
    const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 110;
    auto put = [&](int bit, uint32_t val, int nbits) { w[bit >> 5] |= val << (bit & 31); if ((bit & 31) + nbits > 32) w[(bit >> 5) + 1] |= val >> (32 - (bit & 31)); };
    for (int ib = 0; ib < 8; ++ib) {               // gguf_q.rs:141-151: index = qs | ninth bit from qh, sign bits from the signs bytes
      const uint32_t h = b[66 + ib];
      for (int l = 0; l < 4; ++l) {
        const uint32_t sg = b[74 + 4 * ib + l];
        const uint32_t fa = (uint32_t)b[2 + 8 * ib + 2 * l] | (((h >> (2 * l)) & 1u) << 8) | ((sg & 0xFu) << 9);
        const uint32_t fb = (uint32_t)b[2 + 8 * ib + 2 * l + 1] | (((h >> (2 * l + 1)) & 1u) << 8) | ((sg >> 4) << 9);
        put(13 * (8 * ib + 2 * l), fa, 13); put(13 * (8 * ib + 2 * l + 1), fb, 13);
      }
    }
    w[26] = (uint32_t)b[106] | ((uint32_t)b[107] << 8) | ((uint32_t)b[108] << 16) | ((uint32_t)b[109] << 24);
    w[27] = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
  }
  const size_t tile = (size_t)(row >> 6); const int lane = row & 63;
  for (int p = 0; p < 7; ++p) nq[((tile * SB + sb) * 7 + p) * 64 + lane] = make_uint4(w[4 * p], w[4 * p + 1], w[4 * p + 2], w[4 * p + 3]);
}

// IQ2_XS: raw GGUF rows -> five pieces per (row, super-block); one thread per (padded row, super-block)
__global__ __launch_bounds__(256) void k_repack_n2(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, uint4* __restrict__ nq) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB) return;
  const int row = (int)(idx / SB), sb = (int)(idx % SB); const bool live = row < rows;
  uint32_t w[20];
  for (int i = 0; i < 20; ++i) w[i] = 0;
  if (live) {
    const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 74;
    auto put = [&](int bit, uint32_t val, int nbits) { w[bit >> 5] |= val << (bit & 31); if ((bit & 31) + nbits > 32) w[(bit >> 5) + 1] |= val >> (32 - (bit & 31)); };
    for (int e = 0; e < 32; ++e) {
      const uint32_t q = (uint32_t)b[2 + 2 * e] | ((uint32_t)b[3 + 2 * e] << 8);
      const uint32_t s7 = q >> 9, s8 = s7 | ((uint32_t)(__popc(s7) & 1) << 7);          // ksigns(i) = i | parity(i) << 7
      put(17 * e, (q & 511u) | (s8 << 9), 17);
    }
    w[17] = (uint32_t)b[66] | ((uint32_t)b[67] << 8) | ((uint32_t)b[68] << 16) | ((uint32_t)b[69] << 24);
    w[18] = (uint32_t)b[70] | ((uint32_t)b[71] << 8) | ((uint32_t)b[72] << 16) | ((uint32_t)b[73] << 24);
    w[19] = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
  }
  const size_t tile = (size_t)(row >> 6); const int lane = row & 63;
  for (int p = 0; p < 5; ++p) nq[((tile * SB + sb) * 5 + p) * 64 + lane] = make_uint4(w[4 * p], w[4 * p + 1], w[4 * p + 2], w[4 * p + 3]);
}

// Q4_K: the block's nine 16-byte pieces as they are, transposed to lane = row planes; one thread per (padded row, super-block, piece)
__global__ __launch_bounds__(256) void k_repack_n4(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, uint4* __restrict__ nq) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB * 9) return;
  const int p = (int)(idx % 9); const size_t rs = idx / 9; const int row = (int)(rs / SB), sb = (int)(rs % SB);
  uint32_t w[4] = {0, 0, 0, 0};
  if (row < rows) {
    const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 144 + p * 16;          // (rows of 144-byte blocks are 16-byte aligned only if the buffer is: bytes)
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = (uint32_t)b[4 * k] | ((uint32_t)b[4 * k + 1] << 8) | ((uint32_t)b[4 * k + 2] << 16) | ((uint32_t)b[4 * k + 3] << 24);
  }
  const size_t tile = (size_t)(row >> 6); const int lane = row & 63;
  nq[((tile * SB + sb) * 9 + p) * 64 + lane] = make_uint4(w[0], w[1], w[2], w[3]);
}

// ---- activation digits: grid = 64-column units, one wave per unit -------------------------------------------------------------
__global__ __launch_bounds__(64) void k_act_digits_n(const float* __restrict__ x, uint32_t* __restrict__ dg) {
  __shared__ __align__(16) uint8_t sm[3][64];
  const int ku = blockIdx.x, lane = threadIdx.x;
  const float v = x[(size_t)ku * 64 + lane];
  float mx = fabsf(v);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  const bool fin = __all(isfinite(v));
  float su = 0.0f; int q = 0;
  if (!fin) su = __uint_as_float(0x7FC00000u);            // a non-finite activation makes the unit's contribution NaN
  else if (mx > 0.0f) {
    int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 126; if (e < -100) e = -100;      // mx < 2^e (subnormal maxima take the clamp)
    su = __uint_as_float((uint32_t)(e - 21 + 127) << 23); q = (int)rintf(v * __uint_as_float((uint32_t)(21 - e + 127) << 23));      // |q| <= 2^21
  }
  const int a3 = (int)(int8_t)(q & 0xFF), q1 = (q - a3) >> 8, a2 = (int)(int8_t)(q1 & 0xFF), a1 = (q1 - a2) >> 8;
  sm[0][lane] = (uint8_t)a1; sm[1][lane] = (uint8_t)a2; sm[2][lane] = (uint8_t)a3;      // byte b of group g = column 4 g + b
  __builtin_amdgcn_wave_barrier();      // one wave: its shared-memory operations execute in order
  uint32_t* o = dg + (size_t)ku * DGN_STRIDE;
  int qs = q;                                            // the sum of each half's integers (|sum| <= 2^26), for the formats with an offset per sub-block
#pragma unroll
  for (int o2 = 16; o2 > 0; o2 >>= 1) qs += __shfl_xor(qs, o2);
  if (lane < 48) o[lane] = ((const uint32_t*)sm[lane % 3])[lane / 3];
  else if (lane == 48) o[48] = __float_as_uint(su);
  if (lane == 0) o[49] = (uint32_t)qs;
  if (lane == 32) o[50] = (uint32_t)qs;
}

// byte offset into the table of group G's entry: the 13-bit field at bit 13 G of the 28 words, times four
template <int G> __device__ __forceinline__ uint32_t n_off(const uint32_t (&w)[28]) {
  constexpr int bit = 13 * G - 2;                   // the window starts two bits below the field
  if constexpr (bit < 0) return (w[0] << 2) & 0x7FFCu;
  else {
    constexpr int wi = bit >> 5, sh = bit & 31;
    if constexpr (sh + 15 <= 32) return (w[wi] >> sh) & 0x7FFCu;
    else return __builtin_amdgcn_alignbit(w[wi + 1], w[wi], sh) & 0x7FFCu;
  }
}
// sub-block IB (32 weights) of the super-block held in w against its digits at p (uniform address): the three digit sums
template <int IB, int L> __device__ __forceinline__ void n_group(const uint32_t (&w)[28], const uint8_t* lt, const uint32_t* __restrict__ p, int& i1, int& i2, int& i3) {
  if constexpr (L < 8) {
#ifdef GEMV_N_NOLDS      // diagnostics: the table offset itself in place of the table's entry (no shared-memory read)
    const int e = (int)n_off<IB * 8 + L>(w);
#else
    const int e = (int)*(const uint32_t*)(lt + n_off<IB * 8 + L>(w));
#endif
    i1 = __builtin_amdgcn_sdot4(e, (int)p[L * 3 + 0], i1, false); i2 = __builtin_amdgcn_sdot4(e, (int)p[L * 3 + 1], i2, false); i3 = __builtin_amdgcn_sdot4(e, (int)p[L * 3 + 2], i3, false);
    n_group<IB, L + 1>(w, lt, p, i1, i2, i3);
  }
}
template <int IB> __device__ __forceinline__ float n_subblock(const uint32_t (&w)[28], const uint8_t* lt, const uint32_t* __restrict__ dgs, float dsu, float acc) {
  int i1 = 0, i2 = 0, i3 = 0;
  n_group<IB, 0>(w, lt, dgs + (IB & 1) * 24, i1, i2, i3);
  const int t = (int)(((uint32_t)i1 << 16) + ((uint32_t)i2 << 8) + (uint32_t)i3);          // |t| < 2^31: |i1| <= 32 * 15 * 33
  const float s = (float)(1 + 2 * (int)((w[26] >> (4 * IB)) & 0xFu));
  return fmaf(dsu * s, (float)t, acc);
}
// one super-block (256 columns) of the lane's row; dg = the digits of its four units
__device__ __forceinline__ float n_superblock(const uint4 (&r)[7], const uint8_t* lt, const uint32_t* __restrict__ dg, float acc) {
#ifdef GEMV_N_NOMATH      // diagnostics: the loads alone
  uint32_t u = 0;
#pragma unroll
  for (int p = 0; p < 7; ++p) u ^= r[p].x ^ r[p].y ^ r[p].z ^ r[p].w;
  return acc + __uint_as_float(u & 0xFFu);
#endif
  const uint32_t w[28] = {r[0].x, r[0].y, r[0].z, r[0].w, r[1].x, r[1].y, r[1].z, r[1].w, r[2].x, r[2].y, r[2].z, r[2].w, r[3].x, r[3].y, r[3].z, r[3].w,
                          r[4].x, r[4].y, r[4].z, r[4].w, r[5].x, r[5].y, r[5].z, r[5].w, r[6].x, r[6].y, r[6].z, r[6].w};
  const float d = h2f_bits(w[27] & 0xFFFFu);
  { const float dsu = d * __uint_as_float(dg[0 * DGN_STRIDE + 48]); acc = n_subblock<0>(w, lt, dg + 0 * DGN_STRIDE, dsu, acc); acc = n_subblock<1>(w, lt, dg + 0 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[1 * DGN_STRIDE + 48]); acc = n_subblock<2>(w, lt, dg + 1 * DGN_STRIDE, dsu, acc); acc = n_subblock<3>(w, lt, dg + 1 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[2 * DGN_STRIDE + 48]); acc = n_subblock<4>(w, lt, dg + 2 * DGN_STRIDE, dsu, acc); acc = n_subblock<5>(w, lt, dg + 2 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[3 * DGN_STRIDE + 48]); acc = n_subblock<6>(w, lt, dg + 3 * DGN_STRIDE, dsu, acc); acc = n_subblock<7>(w, lt, dg + 3 * DGN_STRIDE, dsu, acc); }
  return acc;
}

// ---- IQ2_XS: entry E (eight weights) of the 20 words: the two table offsets (weights 0..3: first table; 4..7: second, 32 KB on)
template <int E> __device__ __forceinline__ void n2_offs(const uint32_t (&w)[20], uint32_t& o0, uint32_t& o1) {
  constexpr int bit = 17 * E - 2;                   // the window starts two bits below the field: index at bits 2..10, signs at 11..14 and 15..18
  uint32_t f;
  if constexpr (bit < 0) f = w[0] << 2;
  else { constexpr int wi = bit >> 5, sh = bit & 31; if constexpr (sh + 19 <= 32) f = w[wi] >> sh; else f = __builtin_amdgcn_alignbit(w[wi + 1], w[wi], sh); }
  o0 = f & 0x7FFCu;
  o1 = ((f & 0x07FCu) | ((f >> 4) & 0x7800u)) + 32768u;
}
template <int IB, int L> __device__ __forceinline__ void n2_group(const uint32_t (&w)[20], const uint8_t* lt, const uint32_t* __restrict__ p, int (&ia)[3], int (&ib)[3]) {
  if constexpr (L < 4) {
    uint32_t o0, o1; n2_offs<IB * 4 + L>(w, o0, o1);
    const int e0 = (int)*(const uint32_t*)(lt + o0), e1 = (int)*(const uint32_t*)(lt + o1);
    int (&acc)[3] = L < 2 ? ia : ib;                 // entries 0, 1: the sub-block's first sixteen weights; 2, 3: its second
#pragma unroll
    for (int k = 0; k < 3; ++k) { acc[k] = __builtin_amdgcn_sdot4(e0, (int)p[(2 * L) * 3 + k], acc[k], false); acc[k] = __builtin_amdgcn_sdot4(e1, (int)p[(2 * L + 1) * 3 + k], acc[k], false); }
    n2_group<IB, L + 1>(w, lt, p, ia, ib);
  }
}
template <int IB> __device__ __forceinline__ float n2_subblock(const uint32_t (&w)[20], const uint8_t* lt, const uint32_t* __restrict__ dgs, float dsu, float acc) {
  int ia[3] = {0, 0, 0}, ib[3] = {0, 0, 0};
  n2_group<IB, 0>(w, lt, dgs + (IB & 1) * 24, ia, ib);
  const int ta = (int)(((uint32_t)ia[0] << 16) + ((uint32_t)ia[1] << 8) + (uint32_t)ia[2]), tb = (int)(((uint32_t)ib[0] << 16) + ((uint32_t)ib[1] << 8) + (uint32_t)ib[2]);      // |t| < 2^31: |i1| <= 16 * 43 * 33
  const uint32_t sc = (w[17 + (IB >> 2)] >> (8 * (IB & 3))) & 0xFFu;
  const float sa = (float)(1 + 2 * (int)(sc & 0xFu)) * 0.125f, sbf = (float)(1 + 2 * (int)(sc >> 4)) * 0.125f;          // (0.5 + n) * 0.25
  return fmaf(dsu * sbf, (float)tb, fmaf(dsu * sa, (float)ta, acc));
}
__device__ __forceinline__ float n_superblock(const uint4 (&r)[5], const uint8_t* lt, const uint32_t* __restrict__ dg, float acc) {
  const uint32_t w[20] = {r[0].x, r[0].y, r[0].z, r[0].w, r[1].x, r[1].y, r[1].z, r[1].w, r[2].x, r[2].y, r[2].z, r[2].w, r[3].x, r[3].y, r[3].z, r[3].w, r[4].x, r[4].y, r[4].z, r[4].w};
  const float d = h2f_bits(w[19] & 0xFFFFu);
  { const float dsu = d * __uint_as_float(dg[0 * DGN_STRIDE + 48]); acc = n2_subblock<0>(w, lt, dg + 0 * DGN_STRIDE, dsu, acc); acc = n2_subblock<1>(w, lt, dg + 0 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[1 * DGN_STRIDE + 48]); acc = n2_subblock<2>(w, lt, dg + 1 * DGN_STRIDE, dsu, acc); acc = n2_subblock<3>(w, lt, dg + 1 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[2 * DGN_STRIDE + 48]); acc = n2_subblock<4>(w, lt, dg + 2 * DGN_STRIDE, dsu, acc); acc = n2_subblock<5>(w, lt, dg + 2 * DGN_STRIDE, dsu, acc); }
  { const float dsu = d * __uint_as_float(dg[3 * DGN_STRIDE + 48]); acc = n2_subblock<6>(w, lt, dg + 3 * DGN_STRIDE, dsu, acc); acc = n2_subblock<7>(w, lt, dg + 3 * DGN_STRIDE, dsu, acc); }
  return acc;
}

// ---- Q4_K: unit C (64 weights: sub-blocks 2C and 2C + 1) of the block's 36 words
template <int C> __device__ __forceinline__ float n4_unit(const uint32_t (&w)[36], const uint32_t* __restrict__ dgu, float d, float dmin, float acc) {
  int ia[3] = {0, 0, 0}, ib[3] = {0, 0, 0};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t u = w[4 + 8 * C + j]; const int lo = (int)(u & 0x0F0F0F0Fu), hi = (int)((u >> 4) & 0x0F0F0F0Fu);
#pragma unroll
    for (int k = 0; k < 3; ++k) { ia[k] = __builtin_amdgcn_sdot4(lo, (int)dgu[j * 3 + k], ia[k], false); ib[k] = __builtin_amdgcn_sdot4(hi, (int)dgu[(8 + j) * 3 + k], ib[k], false); }
  }
  const int ta = (int)(((uint32_t)ia[0] << 16) + ((uint32_t)ia[1] << 8) + (uint32_t)ia[2]), tb = (int)(((uint32_t)ib[0] << 16) + ((uint32_t)ib[1] << 8) + (uint32_t)ib[2]);      // |t| < 2^31: |i1| <= 32 * 15 * 33
  uint32_t s1, m1, s2, m2; scale_min_k4(2 * C, w[1], w[2], w[3], s1, m1); scale_min_k4(2 * C + 1, w[1], w[2], w[3], s2, m2);
  const float su = __uint_as_float(dgu[48]), dsu = d * su, msu = dmin * su;
  acc = fmaf(dsu * (float)s1, (float)ta, acc); acc = fmaf(-(msu * (float)m1), (float)(int)dgu[49], acc);
  acc = fmaf(dsu * (float)s2, (float)tb, acc); acc = fmaf(-(msu * (float)m2), (float)(int)dgu[50], acc);
  return acc;
}
__device__ __forceinline__ float n_superblock(const uint4 (&r)[9], const uint8_t* lt, const uint32_t* __restrict__ dg, float acc) {
  uint32_t w[36];
#pragma unroll
  for (int p = 0; p < 9; ++p) { w[4 * p] = r[p].x; w[4 * p + 1] = r[p].y; w[4 * p + 2] = r[p].z; w[4 * p + 3] = r[p].w; }
  const float d = h2f_bits(w[0] & 0xFFFFu), dmin = h2f_bits(w[0] >> 16);
  acc = n4_unit<0>(w, dg + 0 * DGN_STRIDE, d, dmin, acc); acc = n4_unit<1>(w, dg + 1 * DGN_STRIDE, d, dmin, acc);
  acc = n4_unit<2>(w, dg + 2 * DGN_STRIDE, d, dmin, acc); acc = n4_unit<3>(w, dg + 3 * DGN_STRIDE, d, dmin, acc);
  return acc;
}

// grid = min(tiles, what the chip holds at once), NW waves; the workgroup fills its table, then takes row tiles
// blockIdx.x, + gridDim.x, ..; wave w walks super-blocks [w * spw, + spw) of the tile, lane l owns row tile * 64 + l; the
// waves' sums meet in shared memory in wave order.  The next super-block's seven pieces are requested before the current
// one's arithmetic starts.
// P: 16-byte pieces a super-block has (7: IQ3_S, one 32 KB table; 5: IQ2_XS, two; 9: Q4_K, none)
template <int NW, int P = 7> __global__ __launch_bounds__(NW * 64) void k_gemv_n(const uint4* __restrict__ nq, int rows, int tiles, int SB, const uint4* __restrict__ tab, const uint32_t* __restrict__ dg, float* __restrict__ y, int spw) {
  constexpr int TW = P == 7 ? 2048 : (P == 5 ? 4096 : 0);          // 16-byte words of the table(s)
  __shared__ __align__(16) uint8_t lt[TW ? TW * 16 : 16];
  __shared__ float red[NW][64];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  if constexpr (TW > 0) {
    for (int i = tid; i < TW; i += NW * 64) ((uint4*)lt)[i] = tab[i];
    __syncthreads();
  }
  const int s0 = min(SB, wave * spw), s1 = min(SB, s0 + spw);
  uint4 bufa[P], bufb[P];
  const size_t tstride = (size_t)SB * P * 64;
  if (s0 < s1 && (int)blockIdx.x < tiles) {
#pragma unroll
    for (int p = 0; p < P; ++p) bufa[p] = nq[(size_t)blockIdx.x * tstride + ((size_t)s0 * P + p) * 64 + lane];
  }
  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    float acc = 0.0f;
    if (s0 < s1) {
      const uint4* base = nq + (size_t)tile * tstride + lane;
      const int tn = tile + (int)gridDim.x < tiles ? tile + (int)gridDim.x : tile;          // the wave's first super-block of the next tile follows its last of this one
      const uint4* nbase = nq + (size_t)tn * tstride + lane;
      for (int sb = s0; sb < s1; sb += 2) {          // two buffers taking turns (a copy from one to the other would cost 28 moves a super-block)
        const bool last1 = sb + 1 >= s1, last2 = sb + 2 >= s1;
        const uint4* b1 = last1 ? nbase + (size_t)s0 * P * 64 : base + (size_t)(sb + 1) * P * 64;
#pragma unroll
        for (int p = 0; p < P; ++p) bufb[p] = b1[(size_t)p * 64];
        acc = n_superblock(bufa, lt, dg + (size_t)sb * 4 * DGN_STRIDE, acc);
        if (last1) {
#pragma unroll
          for (int p = 0; p < P; ++p) bufa[p] = bufb[p];          // (an odd count of super-blocks a wave: the prefetched one is the next tile's first)
        } else {
          const uint4* b2 = last2 ? nbase + (size_t)s0 * P * 64 : base + (size_t)(sb + 2) * P * 64;
#pragma unroll
          for (int p = 0; p < P; ++p) bufa[p] = b2[(size_t)p * 64];
          acc = n_superblock(bufb, lt, dg + (size_t)(sb + 1) * 4 * DGN_STRIDE, acc);
        }
      }
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (tid < 64) {
      float s = red[0][lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) s += red[w][lane];
      const size_t row = (size_t)tile * 64 + lane;
      if (row < (size_t)rows) y[row] = s;
    }
    __syncthreads();
  }
}

namespace {
int env_i(const char* n, int dflt) { const char* s = getenv(n); return s && *s ? atoi(s) : dflt; }
}

size_t pyre_gemv_n_bytes(size_t rows, size_t cols, int fmt) { return ((rows + 63) / 64) * 64 * (cols / 256) * (fmt == FMT_IQ2_XS ? 80 : (fmt == FMT_Q4_K ? 144 : 112)); }

int pyre_gemv_n_repack(pyre_ctx* ctx, size_t rows, size_t cols, const uint8_t* raw_dev, size_t row_bytes, void* nq_dev, int fmt) {
  const int SB = (int)(cols / 256); const size_t rows_pad = (rows + 63) / 64 * 64, total = rows_pad * SB;
  if (fmt == FMT_Q4_K) { hipLaunchKernelGGL(k_repack_n4, dim3((unsigned)((total * 9 + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, raw_dev, row_bytes, (uint4*)nq_dev); PYRE_CHECK_LAUNCH(ctx); return PYRE_OK; }
  if (fmt == FMT_IQ2_XS) { hipLaunchKernelGGL(k_repack_n2, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, raw_dev, row_bytes, (uint4*)nq_dev); PYRE_CHECK_LAUNCH(ctx); return PYRE_OK; }
  hipLaunchKernelGGL(k_repack_n, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, raw_dev, row_bytes, (uint4*)nq_dev);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

// the table: entry (index | signs << 9) = the four codebook values of `index`, value j negated where sign bit j is set
int pyre_gemv_n_table(pyre_ctx* ctx) {
  if (ctx->d_iq3s_sgn) return PYRE_OK;
  {      // IQ2_XS: table h (h = 0: weights 0..3 of an entry, 1: weights 4..7), entry (index | four signs << 9)
    std::vector<uint32_t> t2(16384);
    static const int tri[3] = {8, 25, 43};
    for (int h = 0; h < 2; ++h) for (int i = 0; i < 8192; ++i) {
      uint32_t v = 0;
      for (int j = 0; j < 4; ++j) { const int g = tri[(kIq2xsCode[i & 511] >> (2 * (4 * h + j))) & 3]; const int sgn = ((i >> (9 + j)) & 1) ? -g : g; v |= (uint32_t)(uint8_t)(int8_t)sgn << (8 * j); }
      t2[(size_t)h * 8192 + i] = v;
    }
    PYRE_HIP(ctx, hipMalloc((void**)&ctx->d_iq2xs_sgn, 16384 * 4));
    PYRE_HIP(ctx, hipMemcpyAsync(ctx->d_iq2xs_sgn, t2.data(), 16384 * 4, hipMemcpyHostToDevice, ctx->stream));
    PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  }
  std::vector<uint32_t> t(8192);
  for (int i = 0; i < 8192; ++i) {
    uint32_t v = 0;
    for (int j = 0; j < 4; ++j) { const int g = 2 * ((kIq3sCode[i & 511] >> (3 * j)) & 7) + 1; const int s = ((i >> (9 + j)) & 1) ? -g : g; v |= (uint32_t)(uint8_t)(int8_t)s << (8 * j); }
    t[i] = v;
  }
  PYRE_HIP(ctx, hipMalloc((void**)&ctx->d_iq3s_sgn, 8192 * 4));
  PYRE_HIP(ctx, hipMemcpyAsync(ctx->d_iq3s_sgn, t.data(), 8192 * 4, hipMemcpyHostToDevice, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return PYRE_OK;
}

size_t pyre_gemv_n_digit_bytes(size_t cols) { return cols / 64 * DGN_STRIDE * 4; }

// digits: where the activation digits go (pyre_gemv_n_digit_bytes(cols) bytes); null = the context's grow-only buffer
int pyre_gemv_n_launch(pyre_ctx* ctx, const void* nq, size_t rows, size_t cols, const float* x_dev, float* y_dev, void* digits, int fmt) {
  if (cols % 256) return pyre_fail(ctx, PYRE_E_SHAPE, "gemv_n: %zu columns are not whole super-blocks", cols);
  if (!ctx->d_iq3s_sgn || !ctx->d_iq2xs_sgn) return pyre_fail(ctx, PYRE_E_HIP, "gemv_n: the codebook tables were not made at context creation");
  const int U = (int)(cols / 64), SB = (int)(cols / 256), tiles = (int)((rows + 63) / 64);
  const size_t need = pyre_gemv_n_digit_bytes(cols);
  if (!digits && ctx->dgn_bytes < need) {
    if (ctx->dgn_buf) { PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); PYRE_HIP(ctx, hipFree(ctx->dgn_buf)); ctx->dgn_buf = nullptr; ctx->dgn_bytes = 0; }
    PYRE_HIP(ctx, hipMalloc(&ctx->dgn_buf, need)); ctx->dgn_bytes = need;
  }
  uint32_t* dg = (uint32_t*)(digits ? digits : ctx->dgn_buf);
  { ProfScope ps(ctx, "gemv_n_digits", 4.0 * cols * 2);
    hipLaunchKernelGGL(k_act_digits_n, dim3(U), dim3(64), 0, ctx->stream, x_dev, dg); } PYRE_CHECK_LAUNCH(ctx);
  static const int fnw = env_i("PYRE_GEMV_N_NW", 0), fwg = env_i("PYRE_GEMV_N_WGS", 0);
  // eight waves a row tile when the rows are long enough (one or two super-blocks a wave), two such workgroups a compute unit:
  // measured on the 151936 x 2048 head, 31.7 us against 34.2 with four waves and four workgroups
  int nw = SB >= 8 ? 8 : (SB >= 4 ? 4 : (SB >= 2 ? 2 : 1)); if (fnw == 1 || fnw == 2 || fnw == 4 || fnw == 8) nw = fnw;
  if (nw > SB) nw = SB >= 8 ? 8 : (SB >= 4 ? 4 : (SB >= 2 ? 2 : 1));
  const int spw = (SB + nw - 1) / nw;
  const int per_cu = 16 / nw > 4 ? 4 : 16 / nw;          // 32 KB of table per workgroup: at most four on a compute unit
  int grid = fwg > 0 ? fwg : 256 * per_cu;
  static const int fgrid = env_i("PYRE_GEMV_N_GRID", 0); if (fgrid > 0) grid = fgrid;
  if (grid > tiles) grid = tiles;
  if (fmt == FMT_Q4_K) {
    ProfScope ps(ctx, "gemv_n_q4_k_t1", (double)rows * (cols / 256) * 144 + 4.0 * ((double)cols + rows));
    const uint4* q = (const uint4*)nq;
    switch (nw) {
      case 1: hipLaunchKernelGGL((k_gemv_n<1, 9>), dim3(grid), dim3(64), 0, ctx->stream, q, (int)rows, tiles, SB, nullptr, dg, y_dev, spw); break;
      case 2: hipLaunchKernelGGL((k_gemv_n<2, 9>), dim3(grid), dim3(128), 0, ctx->stream, q, (int)rows, tiles, SB, nullptr, dg, y_dev, spw); break;
      case 8: hipLaunchKernelGGL((k_gemv_n<8, 9>), dim3(grid), dim3(512), 0, ctx->stream, q, (int)rows, tiles, SB, nullptr, dg, y_dev, spw); break;
      default: hipLaunchKernelGGL((k_gemv_n<4, 9>), dim3(grid), dim3(256), 0, ctx->stream, q, (int)rows, tiles, SB, nullptr, dg, y_dev, spw); break;
    }
    PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
  }
  if (fmt == FMT_IQ2_XS) {          // two 32 KB tables a workgroup: eight waves, two workgroups a compute unit
    ProfScope ps(ctx, "gemv_n_iq2_xs_t1", (double)rows * (cols / 256) * 74 + 4.0 * ((double)cols + rows));
    const uint4* q = (const uint4*)nq; const uint4* tb = (const uint4*)ctx->d_iq2xs_sgn;
    if (grid > 512 && fgrid <= 0) grid = 512 < tiles ? 512 : tiles;
    switch (nw) {
      case 1: hipLaunchKernelGGL((k_gemv_n<1, 5>), dim3(grid), dim3(64), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      case 2: hipLaunchKernelGGL((k_gemv_n<2, 5>), dim3(grid), dim3(128), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      case 8: hipLaunchKernelGGL((k_gemv_n<8, 5>), dim3(grid), dim3(512), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      default: hipLaunchKernelGGL((k_gemv_n<4, 5>), dim3(grid), dim3(256), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
    }
    PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
  }
  { ProfScope ps(ctx, "gemv_n_iq3_s_t1", (double)rows * (cols / 256) * 110 + 4.0 * ((double)cols + rows));
    const uint4* q = (const uint4*)nq; const uint4* tb = (const uint4*)ctx->d_iq3s_sgn;
    switch (nw) {
      case 1: hipLaunchKernelGGL((k_gemv_n<1>), dim3(grid), dim3(64), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      case 2: hipLaunchKernelGGL((k_gemv_n<2>), dim3(grid), dim3(128), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      case 8: hipLaunchKernelGGL((k_gemv_n<8>), dim3(grid), dim3(512), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
      default: hipLaunchKernelGGL((k_gemv_n<4>), dim3(grid), dim3(256), 0, ctx->stream, q, (int)rows, tiles, SB, tb, dg, y_dev, spw); break;
    } }
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
