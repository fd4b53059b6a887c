// GGUF block formats on the device: plane geometry, bit-exact element decode, and the factored per-unit
// dot products the GEMV kernels use.  Format definitions: src/model/gguf_q.rs:67-166 of the reference.
#pragma once
#include "common.h"
#include "iq_codebooks.h"

// Device formats.  The first seven keep the GGUF block's own fields; C4 and C8 are what every other supported GGUF
// type is re-coded into at load: one f32 scale per 16 values (the exact f32 product the reference forms before its
// last multiply) and, per value, a 4-bit code into a 16-entry table of small integers (C4) or an int8 (C8), so that
// value = scale * integer is the reference's own last multiply.
// FMT_IQ3_S_M is the second home of an IQ3_S matrix: the same 4-bit codes laid out for the matrix cores (see QMatDev), used by
// the matrices that only ever meet a GEMV (projections, the vocabulary head, the stand-alone operator).
enum { FMT_F32 = 0, FMT_F16 = 1, FMT_BF16 = 2, FMT_Q8_0 = 3, FMT_Q4_K = 4, FMT_IQ2_XS = 5, FMT_IQ3_S = 6, FMT_C4 = 7, FMT_C8 = 8, FMT_IQ3_S_M = 9, FMT_Q4_K_M = 10, FMT_IQ2_XS_M = 11, FMT_Q8_0_M = 12, FMT_COUNT = 13 };      // FMT_Q4_K_M, FMT_IQ2_XS_M, FMT_Q8_0_M: Q4_K / IQ2_XS / Q8_0 codes and headers laid out for the matrix cores (gemm_q4.hip, gemm_q2.hip, gemm_q8.hip; the operator's windows only)

struct FmtGeom { int V; int e1, e2, e3, eb; };   // plane entry sizes: 16-byte chunks per unit in p0; bytes per unit in p1..p3; bytes per super-block in pb
__host__ __device__ inline FmtGeom fmt_geom(int fmt) {
  switch (fmt) {
    case FMT_F32:    return {16, 0, 0, 0, 0};
    case FMT_F16:    return {8, 0, 0, 0, 0};
    case FMT_BF16:   return {8, 0, 0, 0, 0};
    case FMT_Q8_0:   return {4, 4, 0, 0, 0};     // p1: the two f16 scales of the unit's two blocks
    case FMT_Q4_K:   return {2, 0, 0, 0, 16};    // pb: d, dmin, scales[12]
    case FMT_IQ2_XS: return {1, 2, 8, 0, 2};     // IQ2_XS / IQ2_XXS / IQ2_S, re-coded at load: p0: 64 two-bit magnitude codes; p1: four scale nibbles; p2: 64 sign bits; pb: d
    case FMT_C4:     return {2, 16, 0, 0, 0};    // p0: 64 four-bit codes; p1: four f32 scales
    case FMT_C8:     return {4, 16, 0, 0, 0};    // p0: 64 int8 values; p1: four f32 scales
    default:         return {2, 0, 0, 1, 2};     // IQ3_S, re-coded at load: p0: 64 four-bit codes, p3: scale byte; pb: d
  }
}
// Planes of a matrix of GGUF type ty in device format fmt: Q5_K (value = d*s*q - dmin*m, gguf_q.rs:108-113) rides on C8 with
// a second f32 per 16 values in p2, the offset dmin*m subtracted after the scale multiply.
__host__ __device__ inline FmtGeom qmat_geom(int fmt, uint32_t ty) { FmtGeom g = fmt_geom(fmt); if (fmt == FMT_C8 && ty == PYRE_Q5_K) g.e2 = 16; return g; }
// GGUF block geometry (elements, bytes) of the types the library loads (QType::geom, gguf_q.rs:33-42); false for the rest
__host__ __device__ inline bool ggml_geom(uint32_t ty, int* el, int* bytes) {
  switch (ty) {
    case PYRE_F32: *el = 1; *bytes = 4; return true;  case PYRE_F16: case PYRE_BF16: *el = 1; *bytes = 2; return true;
    case PYRE_Q4_0: *el = 32; *bytes = 18; return true;  case PYRE_Q5_0: *el = 32; *bytes = 22; return true;  case PYRE_Q8_0: *el = 32; *bytes = 34; return true;
    case PYRE_Q4_K: *el = 256; *bytes = 144; return true;  case PYRE_Q6_K: *el = 256; *bytes = 210; return true;
    case PYRE_Q3_K: *el = 256; *bytes = 110; return true;  case PYRE_Q2_0: *el = 64; *bytes = 18; return true;  case PYRE_Q5_K: *el = 256; *bytes = 176; return true;
    case PYRE_IQ1_M: *el = 256; *bytes = 56; return true;
    case PYRE_IQ2_XXS: *el = 256; *bytes = 66; return true;  case PYRE_IQ2_XS: *el = 256; *bytes = 74; return true;  case PYRE_IQ2_S: *el = 256; *bytes = 82; return true;
    case PYRE_IQ3_XXS: *el = 256; *bytes = 98; return true;  case PYRE_IQ3_S: *el = 256; *bytes = 110; return true;
    case PYRE_IQ4_NL: *el = 32; *bytes = 18; return true;  case PYRE_IQ4_XS: *el = 256; *bytes = 136; return true;
  }
  return false;
}
inline int fmt_from_ggml(uint32_t ty) {
  switch (ty) { case PYRE_F32: return FMT_F32; case PYRE_F16: return FMT_F16; case PYRE_BF16: return FMT_BF16; case PYRE_Q8_0: return FMT_Q8_0;
    case PYRE_Q4_K: return FMT_Q4_K; case PYRE_IQ2_XS: return FMT_IQ2_XS; case PYRE_IQ3_S: return FMT_IQ3_S;
    case PYRE_IQ2_XXS: case PYRE_IQ2_S: return FMT_IQ2_XS;
    case PYRE_Q4_0: case PYRE_IQ4_NL: case PYRE_IQ4_XS: case PYRE_IQ3_XXS: case PYRE_Q3_K: case PYRE_Q2_0: case PYRE_IQ1_M: return FMT_C4;
    case PYRE_Q5_0: case PYRE_Q6_K: case PYRE_Q5_K: return FMT_C8; }
  return -1;
}
// The C4 value table of a GGUF type: entry c (byte c%4 of word c/4) holds value + bias, 0..255.
//   Q4_0: c - 8.  IQ4_NL, IQ4_XS: the sixteen non-linear levels (kIq4nlValues).  IQ3_XXS codes a value as
//   (negative << 3) | magnitude index, magnitudes {4, 12, .., 52, 62}.  Q3_K: code = two low bits | high-mask bit << 2, value
//   code - 4 (gguf_q.rs:99: low - (mask set ? 0 : 4)).  Q2_0: the two-bit code - 1 (gguf_q.rs:50).  IQ1_M (gguf_q.rs:152-165): a value is
//   s * (g + delta), g in {-1, 0, 1}, delta = +-0.125; code = (g + 1) | (delta negative) << 2 stands for the integer 8 g +- 1 and the
//   group's scale is s / 8 (a power-of-two scaling: the product rounds exactly as the reference's).
inline void c4_table(uint32_t ty, uint32_t lut[4], int* bias) {
  int v[16] = {0}; int b = 0;
  static const int lv3[8] = {4, 12, 20, 28, 36, 44, 52, 62};
  switch (ty) {
    case PYRE_Q4_0: for (int c = 0; c < 16; ++c) v[c] = c - 8; b = 8; break;
    case PYRE_IQ4_NL: case PYRE_IQ4_XS: for (int c = 0; c < 16; ++c) v[c] = kIq4nlValues[c]; b = 127; break;
    case PYRE_IQ3_XXS: for (int c = 0; c < 8; ++c) { v[c] = lv3[c]; v[8 + c] = -lv3[c]; } b = 62; break;
    case PYRE_Q3_K: for (int c = 0; c < 8; ++c) v[c] = c - 4; b = 8; break;
    case PYRE_Q2_0: for (int c = 0; c < 4; ++c) v[c] = c - 1; b = 8; break;
    case PYRE_IQ1_M: for (int c = 0; c < 8; ++c) v[c] = 8 * ((c & 3) - 1) + ((c & 4) ? -1 : 1); b = 17; break;
    default: break;
  }
  for (int w = 0; w < 4; ++w) { lut[w] = 0; for (int k = 0; k < 4; ++k) lut[w] |= (uint32_t)(v[4 * w + k] + b) << (8 * k); }
  *bias = b;
}

// ---- plane accessors ------------------------------------------------------------------------------------------------
template <int V> __device__ __forceinline__ uint4 ld_vec(const QMatDev& m, int tile, int ku, int chunk, int lane) {
  return ((const uint4*)m.p0)[(((size_t)tile * m.U + ku) * V + chunk) * 64 + lane];
}
template <typename E> __device__ __forceinline__ E ld_small(const uint8_t* p, const QMatDev& m, int tile, int ku, int lane) {
  return ((const E*)p)[((size_t)tile * m.U + ku) * 64 + lane];
}
template <typename E> __device__ __forceinline__ E ld_block(const QMatDev& m, int tile, int ku, int lane) {
  return ((const E*)m.pb)[((size_t)tile * (m.U >> 2) + (ku >> 2)) * 64 + lane];
}

__device__ __forceinline__ float h2f_bits(uint32_t h) { return __half2float(__ushort_as_half((unsigned short)(h & 0xFFFF))); }
__device__ __forceinline__ float flip(float v, uint32_t neg) { return __uint_as_float(__float_as_uint(v) ^ (neg << 31)); }
__device__ __forceinline__ uint32_t ksigns(uint32_t i) { return i | ((__popc(i) & 1u) << 7); }   // KSIGNS_IQ2XS closed form
// byte i (0..11) of the Q4_K scales field held in three dwords (selects, so the words stay in registers)
__device__ __forceinline__ uint32_t k4_byte(uint32_t a, uint32_t b, uint32_t c, int i) { uint32_t w = i < 4 ? a : (i < 8 ? b : c); return (w >> (8 * (i & 3))) & 0xFF; }
__device__ __forceinline__ void scale_min_k4(int j, uint32_t a, uint32_t b, uint32_t c, uint32_t& s, uint32_t& m) {    // gguf_q.rs:62-64
  if (j < 4) { s = k4_byte(a, b, c, j) & 63; m = k4_byte(a, b, c, j + 4) & 63; }
  else { s = (k4_byte(a, b, c, j + 4) & 0xF) | ((k4_byte(a, b, c, j - 4) >> 6) << 4); m = (k4_byte(a, b, c, j + 4) >> 4) | ((k4_byte(a, b, c, j) >> 6) << 4); }
}

// IQ3_S values are sign * grid with grid in {1, 3, .., 15}: sixteen odd integers -15..15.  At load each value w is
// re-coded as the 4-bit number (w + 15) / 2 (code c of value j of a unit sits in bits 4*(j%8).. of word j/8), which
// decodes without the codebook: w = 2c - 15.
__host__ __device__ inline uint32_t iq3s_code(uint32_t grid_byte, uint32_t neg) { int w = neg ? -(int)grid_byte : (int)grid_byte; return (uint32_t)((w + 15) >> 1); }

// The 2-bit i-quants (IQ2_XS, IQ2_XXS, IQ2_S) hold sign * magnitude with magnitude in {8, 25, 43} and one scale nibble
// per 16 values (IQ2_XXS: per 32, stored twice).  At load the codebook and sign-table lookups are resolved once; per
// unit the device keeps, for value e = 4r + b (round r, byte b) of 16-value group g:
//   magnitude index (0, 1, 2) at bits 8b + 2r of dword g of the unit's 16-byte chunk,
//   sign at bit 8b + r + 4*(g & 1) of dword g / 2 of the unit's 8 sign bytes,
// so that `round r` of a group yields four 3-bit codes (sign << 2 | index), one per byte, with two shifts and two
// masks, and one v_perm_b32 turns them into the four biased values magnitude * sign + 43.
__device__ __forceinline__ uint32_t iq2_mag(uint32_t idx) { return idx == 0 ? 8u : (idx == 1 ? 25u : 43u); }
#define PYRE_IQ2_TLO 0x00564433u      // codes 0..3: 43 + {8, 25, 43}, unused
#define PYRE_IQ2_THI 0x00001223u      // codes 4..7: 43 - {8, 25, 43}, unused

// ---- bit-exact decode of one unit (64 consecutive values of one row) -----------------------------------------------
// Same operations in the same order as gguf_q::dequant; compiled with -ffp-contract=off so nothing is fused.
template <int FMT> __device__ inline void decode_exact(const QMatDev& m, const uint64_t* g2, int tile, int ku, int lane, float* y) {
  if constexpr (FMT == FMT_F32) {
    for (int c = 0; c < 16; ++c) { uint4 v = ld_vec<16>(m, tile, ku, c, lane); y[4 * c] = __uint_as_float(v.x); y[4 * c + 1] = __uint_as_float(v.y); y[4 * c + 2] = __uint_as_float(v.z); y[4 * c + 3] = __uint_as_float(v.w); }
  } else if constexpr (FMT == FMT_F16 || FMT == FMT_BF16) {
    for (int c = 0; c < 8; ++c) {
      uint4 v = ld_vec<8>(m, tile, ku, c, lane); uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int k = 0; k < 4; ++k) for (int hh = 0; hh < 2; ++hh) { uint32_t u = (w[k] >> (16 * hh)) & 0xFFFF; y[8 * c + 2 * k + hh] = FMT == FMT_F16 ? h2f_bits(u) : __uint_as_float(u << 16); }
    }
  } else if constexpr (FMT == FMT_Q8_0) {          // gguf_q.rs:79
    uint32_t dd = ld_small<uint32_t>(m.p1, m, tile, ku, lane);
    for (int c = 0; c < 4; ++c) {
      float d = h2f_bits(dd >> (16 * (c >> 1)));
      uint4 v = ld_vec<4>(m, tile, ku, c, lane); uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int k = 0; k < 16; ++k) y[16 * c + k] = (float)(int)(int8_t)(w[k >> 2] >> (8 * (k & 3))) * d;
    }
  } else if constexpr (FMT == FMT_Q4_K) {          // gguf_q.rs:103-107
    uint4 hb = ld_block<uint4>(m, tile, ku, lane);
    float d = h2f_bits(hb.x), mn = h2f_bits(hb.x >> 16);
    int j = ku & 3; uint32_t s1, m1, s2, m2; scale_min_k4(2 * j, hb.y, hb.z, hb.w, s1, m1); scale_min_k4(2 * j + 1, hb.y, hb.z, hb.w, s2, m2);
    float d1 = d * (float)s1, M1 = mn * (float)m1, d2 = d * (float)s2, M2 = mn * (float)m2;
    for (int c = 0; c < 2; ++c) {
      uint4 v = ld_vec<2>(m, tile, ku, c, lane); uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int k = 0; k < 16; ++k) { uint32_t b = (w[k >> 2] >> (8 * (k & 3))) & 0xFF; y[16 * c + k] = d1 * (float)(b & 0xF) - M1; y[32 + 16 * c + k] = d2 * (float)(b >> 4) - M2; }
    }
  } else if constexpr (FMT == FMT_IQ2_XS) {        // gguf_q.rs:122-135 from the re-coded planes: (db * magnitude) * sign
    float d = h2f_bits(ld_block<uint16_t>(m, tile, ku, lane));
    uint32_t sc = ld_small<uint16_t>(m.p1, m, tile, ku, lane);
    uint2 sg = ld_small<uint2>(m.p2, m, tile, ku, lane); uint32_t S[2] = {sg.x, sg.y};
    uint4 v = ld_vec<1>(m, tile, ku, 0, lane); uint32_t M[4] = {v.x, v.y, v.z, v.w};
    for (int g = 0; g < 4; ++g) {
      float db = d * (0.5f + (float)((sc >> (4 * g)) & 0xF)) * 0.25f;
      for (int e = 0; e < 16; ++e) { int r = e >> 2, b = e & 3; uint32_t idx = (M[g] >> (8 * b + 2 * r)) & 3, neg = (S[g >> 1] >> (8 * b + r + 4 * (g & 1))) & 1;
        y[16 * g + e] = flip(db * (float)iq2_mag(idx), neg); }
    }
  } else if constexpr (FMT == FMT_C4) {            // scale * table[code]: the last multiply of gguf_q.rs:75,83,88,125,135,140
    uint4 sq = ld_small<uint4>(m.p1, m, tile, ku, lane); float sc[4] = {__uint_as_float(sq.x), __uint_as_float(sq.y), __uint_as_float(sq.z), __uint_as_float(sq.w)};
    for (int c = 0; c < 2; ++c) {
      uint4 v = ld_vec<2>(m, tile, ku, c, lane); uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int j = 0; j < 32; ++j) { uint32_t code = (w[j >> 3] >> (4 * (j & 7))) & 0xF; int val = (int)((m.lut[code >> 2] >> (8 * (code & 3))) & 0xFF) - m.bias; y[32 * c + j] = sc[2 * c + (j >> 4)] * (float)val; }
    }
  } else if constexpr (FMT == FMT_C8) {            // scale * int8: the last multiply of gguf_q.rs:78,120-121
    uint4 sq = ld_small<uint4>(m.p1, m, tile, ku, lane); float sc[4] = {__uint_as_float(sq.x), __uint_as_float(sq.y), __uint_as_float(sq.z), __uint_as_float(sq.w)};
    for (int c = 0; c < 4; ++c) {
      uint4 v = ld_vec<4>(m, tile, ku, c, lane); uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int k = 0; k < 16; ++k) y[16 * c + k] = sc[c] * (float)(int)(int8_t)(w[k >> 2] >> (8 * (k & 3)));
    }
    if (m.ty == PYRE_Q5_K) {                       // gguf_q.rs:112: d1 * q - m1, the subtraction after the rounded product
      uint4 oq = ld_small<uint4>(m.p2, m, tile, ku, lane); float off[4] = {__uint_as_float(oq.x), __uint_as_float(oq.y), __uint_as_float(oq.z), __uint_as_float(oq.w)};
      for (int k = 0; k < 64; ++k) y[k] = y[k] - off[k >> 4];
    }
  } else if constexpr (FMT == FMT_IQ3_S_M) {       // the same codes in the matrix-core layout (QMatDev::mq / mh)
    const size_t row = (size_t)tile * 64 + lane, rgi = row >> 4; const int j = (int)(row & 15);
    const int sb = ku >> 2, k128 = ku >> 1;
    const uint2 hdr = ((const uint2*)m.mh)[mh_slot(rgi, sb, m.SB) + j];
    const float d = h2f_bits(hdr.x);
    for (int c = 0; c < 2; ++c) {                  // sub-block 2*(ku&3) + c of the super-block = step 2*(ku&1) + c of its 128-column half
      const int sbi = 2 * (ku & 3) + c, st = 2 * (ku & 1) + c;
      const float db = d * (float)(1 + 2 * ((hdr.y >> (4 * ((sbi >> 1) + 4 * (sbi & 1)))) & 0xF));
      for (int kg = 0; kg < 4; ++kg) {
        const uint32_t w = ((const uint32_t*)m.mq)[(mq_slot(rgi, k128, m.cols >> 7) + kg * 16 + j) * 4 + st];
        for (int e = 0; e < 8; ++e) { const int sv = 2 * (int)((w >> (4 * ((e >> 1) + 4 * (e & 1)))) & 0xF) - 15; y[32 * c + 8 * kg + e] = flip(db * (float)(sv < 0 ? -sv : sv), sv < 0 ? 1u : 0u); }
      }
    }
  } else {                                         // IQ3_S, gguf_q.rs:141-151, from the 4-bit codes (see iq3s_code)
    float d = h2f_bits(ld_block<uint16_t>(m, tile, ku, lane));
    uint32_t sc = ld_small<uint8_t>(m.p3, m, tile, ku, lane);
    for (int c = 0; c < 2; ++c) {
      float db = d * (float)(1 + 2 * ((sc >> (4 * c)) & 0xF));
      uint4 v = ld_vec<2>(m, tile, ku, c, lane); uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int j = 0; j < 32; ++j) { int sv = 2 * (int)((w[j >> 3] >> (4 * (j & 7))) & 0xF) - 15; y[32 * c + j] = flip(db * (float)(sv < 0 ? -sv : sv), sv < 0 ? 1u : 0u); }
    }
  }
}

// ---- factored per-unit dot products for the GEMV ------------------------------------------------------------------
// A unit's packed data is fetched first (unit_load) and consumed later (unit_fma), so a kernel can issue the weight
// loads ahead of a barrier or of the previous unit's arithmetic; unit_dot does both at once.
template <int FMT> struct UnitRaw { uint4 v[FMT == FMT_F32 ? 16 : (FMT == FMT_F16 || FMT == FMT_BF16) ? 8 : (FMT == FMT_Q8_0 || FMT == FMT_C8) ? 4 : (FMT == FMT_Q4_K || FMT == FMT_IQ3_S || FMT == FMT_C4) ? 2 : 1]; uint4 hb; uint4 hb2; uint32_t s0, s1; };
template <int FMT> __device__ __forceinline__ UnitRaw<FMT> unit_load(const QMatDev& m, int tile, int ku, int lane) {
  UnitRaw<FMT> r; r.hb = uint4{0, 0, 0, 0}; r.hb2 = uint4{0, 0, 0, 0}; r.s0 = 0; r.s1 = 0;
  constexpr int V = sizeof(r.v) / sizeof(uint4);
#pragma unroll
  for (int c = 0; c < V; ++c) r.v[c] = ld_vec<V>(m, tile, ku, c, lane);
  if constexpr (FMT == FMT_Q8_0) r.s0 = ld_small<uint32_t>(m.p1, m, tile, ku, lane);
  if constexpr (FMT == FMT_Q4_K) r.hb = ld_block<uint4>(m, tile, ku, lane);
  if constexpr (FMT == FMT_C4 || FMT == FMT_C8) r.hb = ld_small<uint4>(m.p1, m, tile, ku, lane);
  if constexpr (FMT == FMT_C8) { if (m.ty == PYRE_Q5_K) r.hb2 = ld_small<uint4>(m.p2, m, tile, ku, lane); }
  if constexpr (FMT == FMT_IQ2_XS) { r.s0 = ld_block<uint16_t>(m, tile, ku, lane); r.s1 = ld_small<uint16_t>(m.p1, m, tile, ku, lane); uint2 sg = ld_small<uint2>(m.p2, m, tile, ku, lane); r.hb.x = sg.x; r.hb.y = sg.y; }
  if constexpr (FMT == FMT_IQ3_S) { r.s0 = ld_block<uint16_t>(m, tile, ku, lane); r.s1 = ld_small<uint8_t>(m.p3, m, tile, ku, lane); }
  return r;
}
// xs points at the unit's 64 activations of token 0 (wave-uniform address -> scalar loads); token t is xs + t*xstride.
// acc[t] += sum_j W[row, 64*ku + j] * x[t][64*ku + j].  The operation sequence per token does not depend on T.
// Four table look-ups at once: byte k of `codes` (0..15) -> byte k of the result.  v_perm_b32 picks bytes of the
// low / high half of the table by the codes' low three bits; bit 3 then chooses between the halves.
__device__ __forceinline__ uint32_t c4_lookup(const QMatDev& m, uint32_t codes) {
  uint32_t i7 = codes & 0x07070707u, b3 = codes & 0x08080808u, pick = (b3 << 5) - (b3 >> 3);     // 0xFF in every byte whose code has bit 3
  uint32_t lo = __builtin_amdgcn_perm(m.lut[1], m.lut[0], i7), hi = __builtin_amdgcn_perm(m.lut[3], m.lut[2], i7);
  return (lo & ~pick) | (hi & pick);
}
template <int FMT, int T> __device__ __forceinline__ void unit_fma(const QMatDev& m, const UnitRaw<FMT>& r, int ku, const uint2* lds2, int lane,
                                                                   const float* __restrict__ xs, int xstride, float (&acc)[T]) {
  if constexpr (FMT == FMT_F32) {
#pragma unroll
    for (int c = 0; c < 16; ++c) { uint4 v = r.v[c]; float w[4] = {__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int t = 0; t < T; ++t) acc[t] = fmaf(w[k], xs[t * xstride + 4 * c + k], acc[t]); }
  } else if constexpr (FMT == FMT_F16 || FMT == FMT_BF16) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      uint4 v = r.v[c]; uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float lo = FMT == FMT_F16 ? h2f_bits(w[k]) : __uint_as_float(w[k] << 16), hi = FMT == FMT_F16 ? h2f_bits(w[k] >> 16) : __uint_as_float(w[k] & 0xFFFF0000u);
#pragma unroll
        for (int t = 0; t < T; ++t) { acc[t] = fmaf(lo, xs[t * xstride + 8 * c + 2 * k], acc[t]); acc[t] = fmaf(hi, xs[t * xstride + 8 * c + 2 * k + 1], acc[t]); }
      }
    }
  } else if constexpr (FMT == FMT_Q8_0) {
    uint32_t dd = r.s0;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      float part[T];
_Pragma("unroll")
      for (int t = 0; t < T; ++t) part[t] = 0.0f;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        uint4 v = r.v[2 * b + c]; uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 16; ++k) { float f = (float)(int)(int8_t)(w[k >> 2] >> (8 * (k & 3)));
#pragma unroll
          for (int t = 0; t < T; ++t) part[t] = fmaf(f, xs[t * xstride + 32 * b + 16 * c + k], part[t]); }
      }
      float d = h2f_bits(dd >> (16 * b));
#pragma unroll
      for (int t = 0; t < T; ++t) acc[t] = fmaf(d, part[t], acc[t]);
    }
  } else if constexpr (FMT == FMT_Q4_K) {
    uint4 hb = r.hb;
    float d = h2f_bits(hb.x), mn = h2f_bits(hb.x >> 16);
    int j = ku & 3; uint32_t s1, m1, s2, m2; scale_min_k4(2 * j, hb.y, hb.z, hb.w, s1, m1); scale_min_k4(2 * j + 1, hb.y, hb.z, hb.w, s2, m2);
    float d1 = d * (float)s1, M1 = mn * (float)m1, d2 = d * (float)s2, M2 = mn * (float)m2;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      uint4 v = r.v[c]; uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        uint32_t b = (w[k >> 2] >> (8 * (k & 3))) & 0xFF;
        float lo = fmaf(d1, (float)(b & 0xF), -M1), hi = fmaf(d2, (float)(b >> 4), -M2);
#pragma unroll
        for (int t = 0; t < T; ++t) { acc[t] = fmaf(lo, xs[t * xstride + 16 * c + k], acc[t]); acc[t] = fmaf(hi, xs[t * xstride + 32 + 16 * c + k], acc[t]); }
      }
    }
  } else if constexpr (FMT == FMT_IQ2_XS) {   // biased value = sign * magnitude + 43 by one byte permute per four values; per group  db * (sum biased x - 43 sum x)
    float d = h2f_bits(r.s0);
    uint32_t sc = r.s1;
    uint4 v = r.v[0]; uint32_t M[4] = {v.x, v.y, v.z, v.w}; uint32_t S[2] = {r.hb.x, r.hb.y};
    float sx[T][4];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float xv = xs[t * xstride + lane];
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) xv += __shfl_xor(xv, o);
#pragma unroll
      for (int g = 0; g < 4; ++g) sx[t][g] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv), 16 * g));
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float part[T];
_Pragma("unroll")
      for (int t = 0; t < T; ++t) part[t] = 0.0f;
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int k = rr + 4 * (g & 1);
        uint32_t idx4 = (M[g] >> (2 * rr)) & 0x03030303u, sgn = k >= 2 ? (S[g >> 1] >> (k - 2)) : (S[g >> 1] << (2 - k));
        uint32_t bv = __builtin_amdgcn_perm(PYRE_IQ2_THI, PYRE_IQ2_TLO, (sgn & 0x04040404u) | idx4);
#pragma unroll
        for (int b = 0; b < 4; ++b) { float f = (float)((bv >> (8 * b)) & 0xFF);
#pragma unroll
          for (int t = 0; t < T; ++t) part[t] = fmaf(f, xs[t * xstride + 16 * g + 4 * rr + b], part[t]); }
      }
      float db = d * (0.5f + (float)((sc >> (4 * g)) & 0xF)) * 0.25f;
#pragma unroll
      for (int t = 0; t < T; ++t) acc[t] = fmaf(db, fmaf(-43.0f, sx[t][g], part[t]), acc[t]);
    }
  } else if constexpr (FMT == FMT_C4) {   // value = table[c] - bias: per 16-value group  scale * (sum table[c] x - bias sum x)
    uint4 v0 = r.v[0], v1 = r.v[1];
    uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
    float sc[4] = {__uint_as_float(r.hb.x), __uint_as_float(r.hb.y), __uint_as_float(r.hb.z), __uint_as_float(r.hb.w)};
    float sx[T][4];            // group sums of the activations: lane j holds x[j], folded inside each quarter of the wave
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float xv = xs[t * xstride + lane];
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) xv += __shfl_xor(xv, o);
#pragma unroll
      for (int g = 0; g < 4; ++g) sx[t][g] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv), 16 * g));
    }
    const float nbias = -(float)m.bias;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float part[T];
_Pragma("unroll")
      for (int t = 0; t < T; ++t) part[t] = 0.0f;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        uint32_t u = w[2 * g + k], lo = c4_lookup(m, u & 0x0F0F0F0Fu), hi = c4_lookup(m, (u >> 4) & 0x0F0F0F0Fu);
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          float fl = (float)((lo >> (8 * b)) & 0xFF), fh = (float)((hi >> (8 * b)) & 0xFF);
#pragma unroll
          for (int t = 0; t < T; ++t) { part[t] = fmaf(fl, xs[t * xstride + 16 * g + 8 * k + 2 * b], part[t]); part[t] = fmaf(fh, xs[t * xstride + 16 * g + 8 * k + 2 * b + 1], part[t]); }
        }
      }
#pragma unroll
      for (int t = 0; t < T; ++t) acc[t] = fmaf(sc[g], fmaf(nbias, sx[t][g], part[t]), acc[t]);
    }
  } else if constexpr (FMT == FMT_C8) {
    float sc[4] = {__uint_as_float(r.hb.x), __uint_as_float(r.hb.y), __uint_as_float(r.hb.z), __uint_as_float(r.hb.w)};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float part[T];
_Pragma("unroll")
      for (int t = 0; t < T; ++t) part[t] = 0.0f;
      uint4 v = r.v[c]; uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 16; ++k) { float f = (float)(int)(int8_t)(w[k >> 2] >> (8 * (k & 3)));
#pragma unroll
        for (int t = 0; t < T; ++t) part[t] = fmaf(f, xs[t * xstride + 16 * c + k], part[t]); }
#pragma unroll
      for (int t = 0; t < T; ++t) acc[t] = fmaf(sc[c], part[t], acc[t]);
    }
    if (m.ty == PYRE_Q5_K) {             // value = scale * q - offset: the offsets leave through the groups' activation sums
      const float off[4] = {__uint_as_float(r.hb2.x), __uint_as_float(r.hb2.y), __uint_as_float(r.hb2.z), __uint_as_float(r.hb2.w)};
#pragma unroll
      for (int t = 0; t < T; ++t) {
        float xv = xs[t * xstride + lane];
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) xv += __shfl_xor(xv, o);
#pragma unroll
        for (int g = 0; g < 4; ++g) acc[t] = fmaf(-off[g], __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv), 16 * g)), acc[t]);
      }
    }
  } else {   // IQ3_S from 4-bit codes c = (w + 15) / 2: sum w x = 2 sum c x - 15 sum x per 32-value sub-block
    float d = h2f_bits(r.s0);
    uint32_t sc = r.s1;
    uint4 v0 = r.v[0], v1 = r.v[1];
    uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
    float sx[T][2];            // sub-block sums of the activations: lane j holds x[j], folded inside each half of the wave
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float xv = xs[t * xstride + lane];
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) xv += __shfl_xor(xv, o);
      sx[t][0] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv), 0)); sx[t][1] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv), 32));
    }
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      float part[T];
_Pragma("unroll")
      for (int t = 0; t < T; ++t) part[t] = 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        uint32_t u = w[4 * sb + k], lo = u & 0x0F0F0F0Fu, hi = (u >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          float fl = (float)((lo >> (8 * b)) & 0xFF), fh = (float)((hi >> (8 * b)) & 0xFF);
#pragma unroll
          for (int t = 0; t < T; ++t) { part[t] = fmaf(fl, xs[t * xstride + 32 * sb + 8 * k + 2 * b], part[t]); part[t] = fmaf(fh, xs[t * xstride + 32 * sb + 8 * k + 2 * b + 1], part[t]); }
        }
      }
      float db = d * (float)(1 + 2 * ((sc >> (4 * sb)) & 0xF));
#pragma unroll
      for (int t = 0; t < T; ++t) acc[t] = fmaf(db, fmaf(-15.0f, sx[t][sb], 2.0f * part[t]), acc[t]);
    }
  }
}
template <int FMT, int T> __device__ __forceinline__ void unit_dot(const QMatDev& m, const uint2* lds2, int tile, int ku, int lane,
                                                                   const float* __restrict__ xs, int xstride, float (&acc)[T]) {
  UnitRaw<FMT> r = unit_load<FMT>(m, tile, ku, lane);
  unit_fma<FMT, T>(m, r, ku, lds2, lane, xs, xstride, acc);
}
