// Activations as block fixed point for the integer-dot form of a GEMV over 4-bit codes: per 64 columns one power of two
// and, per value, three signed-byte digits in base 256 (|q| <= 2^22: with codes of at most 15 a 32-value sub-block's
// sum stays below 2^31), so that sum(code * x) is three v_dot4_i32_i8 sums joined in integers.  The digit bytes are arranged for the lane = row layout of the 4-bit codes (QMatDev::p0 of an IQ3_S
// matrix: nibble i of word k is value 8k + i): word 2k of a digit plane holds columns 8k, 8k+2, 8k+4, 8k+6 -- what the
// mask 0x0F0F0F0F leaves of code word k -- and word 2k+1 columns 8k+1, .., 8k+7 -- what it leaves after a shift by four.
//   unit u of a token: dg[u * 64 + w * 3 + j], w = 0..15 the word, j = 0..2 the digit (most significant first);
//   dg[u * 64 + 48] the unit's power of two (f32 bits), [49] / [50] the integer sums of the values of columns 0..31 / 32..63.
#pragma once
#include "formats.h"
#include "common.h"

#define DGX_STRIDE 64

// one wave, lane = column: v is the lane's activation; sm is [3][64] bytes of the wave's own shared memory
__device__ __forceinline__ void digits_eo_wave(float v, int lane, uint8_t (*sm)[64], uint32_t* __restrict__ o) {
  const float mx = wave_max(fabsf(v));
  const bool fin = __all(isfinite(v));
  float su = 0.0f; int q = 0;
  if (!fin) su = __uint_as_float(0x7FC00000u);            // a non-finite activation makes the unit's contribution NaN
  else if (mx > 0.0f) {
    int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 126; if (e < -100) e = -100;      // mx < 2^e (subnormal maxima take the clamp)
    su = __uint_as_float((uint32_t)(e - 22 + 127) << 23); q = (int)rintf(v * __uint_as_float((uint32_t)(22 - e + 127) << 23));      // |q| <= 2^22
  }
  const int a3 = (int)(int8_t)(q & 0xFF), q1 = (q - a3) >> 8, a2 = (int)(int8_t)(q1 & 0xFF), a1 = (q1 - a2) >> 8;
  const int pos = (((lane >> 3) * 2 + (lane & 1)) << 2) + ((lane & 7) >> 1);
  sm[0][pos] = (uint8_t)a1; sm[1][pos] = (uint8_t)a2; sm[2][pos] = (uint8_t)a3;
  // the integer sums of the two halves (|sum of 32| <= 2^27): four steps inside each row of sixteen lanes, then lane 15 of rows 0 and 2
  // into rows 1 and 3 -- lanes 16..31 hold the first half's sum, lanes 48..63 the second's
  int qs = q;
  qs += __builtin_amdgcn_update_dpp(0, qs, 0xB1, 0xf, 0xf, false); qs += __builtin_amdgcn_update_dpp(0, qs, 0x4E, 0xf, 0xf, false);
  qs += __builtin_amdgcn_update_dpp(0, qs, 0x141, 0xf, 0xf, false); qs += __builtin_amdgcn_update_dpp(0, qs, 0x140, 0xf, 0xf, false);
  qs += __builtin_amdgcn_update_dpp(0, qs, 0x142, 0xa, 0xf, false);
  __builtin_amdgcn_wave_barrier();      // one wave: its shared-memory operations execute in order
  if (lane < 48) o[lane] = ((const uint32_t*)sm[lane % 3])[lane / 3];
  else if (lane == 48) o[48] = __float_as_uint(su);
  if (lane == 16) o[49] = (uint32_t)qs;
  if (lane == 48) o[50] = (uint32_t)qs;
}

// acc += sum_j W[row, unit's 64 columns] * x[j] for the lane's row of an IQ3_S unit in the lane = row layout, the
// activations given as the unit's digits (dgu, wave-uniform -> scalar loads).  w = 2c - 15 per value: per sub-block
// d * (2n + 1) * 2^e * (2 * sum(c q) - 15 * sum(q)), the sums exact integers.
__device__ __forceinline__ void unit_idot_iq3s(const UnitRaw<FMT_IQ3_S>& r, const uint32_t* __restrict__ dgu, float& acc) {
  const float d = h2f_bits(r.s0) * __uint_as_float(dgu[48]);
  const uint32_t sc = r.s1;
  const uint32_t w[8] = {r.v[0].x, r.v[0].y, r.v[0].z, r.v[0].w, r.v[1].x, r.v[1].y, r.v[1].z, r.v[1].w};
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
    int i1 = 0, i2 = 0, i3 = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t u = w[4 * sb + k]; const int lo = (int)(u & 0x0F0F0F0Fu), hi = (int)((u >> 4) & 0x0F0F0F0Fu);
      const uint32_t* p = dgu + (4 * sb + k) * 6;
      i1 = __builtin_amdgcn_sdot4(lo, (int)p[0], i1, false); i2 = __builtin_amdgcn_sdot4(lo, (int)p[1], i2, false); i3 = __builtin_amdgcn_sdot4(lo, (int)p[2], i3, false);
      i1 = __builtin_amdgcn_sdot4(hi, (int)p[3], i1, false); i2 = __builtin_amdgcn_sdot4(hi, (int)p[4], i2, false); i3 = __builtin_amdgcn_sdot4(hi, (int)p[5], i3, false);
    }
    const int t = (int)(((uint32_t)i1 << 16) + ((uint32_t)i2 << 8) + (uint32_t)i3);          // |t| <= 32 * 15 * 2^22 < 2^31
    const float db = d * (float)(1 + 2 * ((sc >> (4 * sb)) & 0xF));
    acc = fmaf(db, fmaf(-15.0f, (float)(int)dgu[49 + sb], 2.0f * (float)t), acc);
  }
}
