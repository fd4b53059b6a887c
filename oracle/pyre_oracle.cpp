// CPU oracle: f32 restatement of the reference's host path.  TEST INFRASTRUCTURE ONLY - see pyre_oracle.h.
// Every function cites the reference lines it follows (paths relative to the reference tree).
// Build: g++ -O2 -std=c++17 -mavx2 -mfma -ffp-contract=off -fPIC -shared -pthread (see oracle/Makefile).
#include "pyre_oracle.h"
#include <deque>
#include "iq_codebooks.h"
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <functional>
#include <thread>
#include <vector>

namespace {

// ---------- small scalar helpers -------------------------------------------------------------
// IEEE binary16 -> binary32 (the `half` crate's f16::to_f32, used by h2f at gguf_q.rs:60).
inline float h2f(const uint8_t* b) {
  uint32_t h = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
  uint32_t s = (h & 0x8000u) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF, u;
  if (e == 0) {
    if (m == 0) u = s;
    else { int sh = 0; while (!(m & 0x400)) { m <<= 1; ++sh; } m &= 0x3FF; u = s | ((uint32_t)(113 - sh) << 23) | (m << 13); }
  } else if (e == 31) u = s | 0x7F800000u | (m << 13);
  else u = s | ((e + 112) << 23) | (m << 13);
  float f; memcpy(&f, &u, 4); return f;
}

struct Tables { uint32_t iq3s[512]; uint64_t iq2xs[512]; uint8_t ksigns[128]; uint64_t iq2xxs[256]; uint64_t iq2s[1024]; uint32_t iq3xxs[256]; };
const Tables& tables() {
  static Tables t = [] {
    Tables t{};
    static const uint8_t tri[3] = {8, 25, 43};
    for (int e = 0; e < 512; ++e) {
      uint32_t v = 0; for (int j = 0; j < 4; ++j) v |= (uint32_t)(2 * ((kIq3sCode[e] >> (3 * j)) & 7) + 1) << (8 * j);
      t.iq3s[e] = v;
      uint64_t w = 0; for (int j = 0; j < 8; ++j) w |= (uint64_t)tri[(kIq2xsCode[e] >> (2 * j)) & 3] << (8 * j);
      t.iq2xs[e] = w;
    }
    auto tri8 = [](uint16_t code) { uint64_t w = 0; for (int j = 0; j < 8; ++j) w |= (uint64_t)tri[(code >> (2 * j)) & 3] << (8 * j); return w; };
    static const uint8_t lv3[8] = {4, 12, 20, 28, 36, 44, 52, 62};
    for (int e = 0; e < 256; ++e) {
      t.iq2xxs[e] = tri8(kIq2xxsCode[e]);
      uint32_t v = 0; for (int j = 0; j < 4; ++j) v |= (uint32_t)lv3[(kIq3xxsCode[e] >> (3 * j)) & 7] << (8 * j);
      t.iq3xxs[e] = v;
    }
    for (int e = 0; e < 1024; ++e) t.iq2s[e] = tri8(kIq2sCode[e]);
    for (int i = 0; i < 128; ++i) t.ksigns[i] = (uint8_t)(i | ((__builtin_popcount(i) & 1) << 7));
    return t;
  }();
  return t;
}

// put8, gguf_q.rs:58: y[j] = d * g[j] * s[j], evaluated left to right.
inline void put8(float* y, float d, const float* g, uint8_t signs) {
  for (int j = 0; j < 8; ++j) { float s = (signs >> j) & 1 ? -1.0f : 1.0f; y[j] = d * g[j] * s; }
}

// scale_min_k4, gguf_q.rs:62-64
inline void scale_min_k4(int j, const uint8_t* q, uint8_t* s, uint8_t* m) {
  if (j < 4) { *s = q[j] & 63; *m = q[j + 4] & 63; }
  else { *s = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4)); *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4)); }
}

bool geom(uint32_t ty, int* el, int* by) {
  switch (ty) {  // QType::geom, gguf_q.rs:33-41
    case ORC_F32: *el = 1; *by = 4; return true;
    case ORC_F16: case ORC_BF16: *el = 1; *by = 2; return true;
    case ORC_Q8_0: *el = 32; *by = 34; return true;
    case ORC_Q4_K: *el = 256; *by = 144; return true;
    case ORC_IQ2_XS: *el = 256; *by = 74; return true;
    case ORC_IQ3_S: *el = 256; *by = 110; return true;
    case ORC_Q4_0: *el = 32; *by = 18; return true;
    case ORC_Q5_0: *el = 32; *by = 22; return true;
    case ORC_Q6_K: *el = 256; *by = 210; return true;
    case ORC_IQ4_NL: *el = 32; *by = 18; return true;
    case ORC_IQ4_XS: *el = 256; *by = 136; return true;
    case ORC_IQ2_XXS: *el = 256; *by = 66; return true;
    case ORC_IQ2_S: *el = 256; *by = 82; return true;
    case ORC_IQ3_XXS: *el = 256; *by = 98; return true;
    case ORC_Q3_K: *el = 256; *by = 110; return true;
    case ORC_Q2_0: *el = 64; *by = 18; return true;
    case ORC_Q5_K: *el = 256; *by = 176; return true;
    case ORC_IQ1_M: *el = 256; *by = 56; return true;
  }
  return false;
}

// dequant, gguf_q.rs:67-166 (arms F32 :71, F16 :72, BF16 :73, Q4_0 :74-75, Q5_0 :76-78, Q8_0 :79, IQ4NL :82-83, IQ4XS :84-89,
// Q2_0 :80-81, Q3K :90-102, Q4K :103-107, Q5K :108-113, Q6K :114-121, IQ1M :152-165, IQ2XXS :122-125, IQ2XS :126-129, IQ2S :130-135, IQ3XXS :136-140, IQ3S :141-151)
bool dequant(uint32_t ty, const uint8_t* x, size_t n, float* y) {
  int qk, bs; if (!geom(ty, &qk, &bs)) return false;
  size_t nb = n / qk;
  const Tables& T = tables();
  switch (ty) {
    case ORC_F32: memcpy(y, x, 4 * n); break;
    case ORC_F16: for (size_t i = 0; i < n; ++i) y[i] = h2f(x + 2 * i); break;
    case ORC_BF16: for (size_t i = 0; i < n; ++i) { uint32_t u = ((uint32_t)x[2 * i] | ((uint32_t)x[2 * i + 1] << 8)) << 16; memcpy(&y[i], &u, 4); } break;
    case ORC_Q8_0:
      for (size_t i = 0; i < nb; ++i) { const uint8_t* b = x + i * bs; float d = h2f(b); for (int j = 0; j < 32; ++j) y[i * 32 + j] = (float)(int8_t)b[2 + j] * d; }
      break;
    case ORC_Q4_K:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b), mn = h2f(b + 2); const uint8_t* sc = b + 4; const uint8_t* q = b + 16; float* yy = y + i * 256;
        for (int j = 0; j < 4; ++j) {
          uint8_t s1, m1, s2, m2; scale_min_k4(2 * j, sc, &s1, &m1); scale_min_k4(2 * j + 1, sc, &s2, &m2);
          float d1 = d * (float)s1, M1 = mn * (float)m1, d2 = d * (float)s2, M2 = mn * (float)m2;
          for (int l = 0; l < 32; ++l) { yy[l] = d1 * (float)(q[l] & 0xF) - M1; yy[l + 32] = d2 * (float)(q[l] >> 4) - M2; }
          yy += 64; q += 32;
        }
      }
      break;
    case ORC_IQ1_M:         // gguf_q.rs:152-165; grid entry e, byte j as int8 = ((kIq1sCode[e] >> 2j) & 3) - 1
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; const uint8_t* qs = b; const uint8_t* qh = b + 32; const uint8_t* scb = b + 48;
        const uint16_t sc[4] = {(uint16_t)(scb[0] | (scb[1] << 8)), (uint16_t)(scb[2] | (scb[3] << 8)), (uint16_t)(scb[4] | (scb[5] << 8)), (uint16_t)(scb[6] | (scb[7] << 8))};
        const uint16_t su = (uint16_t)((sc[0] >> 12) | ((sc[1] >> 8) & 0x00f0) | ((sc[2] >> 4) & 0x0f00) | (sc[3] & 0xf000));
        const uint8_t sub[2] = {(uint8_t)(su & 0xFF), (uint8_t)(su >> 8)}; const float d = h2f(sub); float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ++ib) {
          const float dl1 = d * (float)(2 * ((sc[ib / 2] >> (6 * (ib % 2))) & 7) + 1), dl2 = d * (float)(2 * ((sc[ib / 2] >> (6 * (ib % 2) + 3)) & 7) + 1);
          const size_t idx[4] = {(size_t)qs[0] | (((size_t)qh[0] << 8) & 0x700), (size_t)qs[1] | (((size_t)qh[0] << 4) & 0x700), (size_t)qs[2] | (((size_t)qh[1] << 8) & 0x700), (size_t)qs[3] | (((size_t)qh[1] << 4) & 0x700)};
          const float dl[4] = {(qh[0] & 0x08) ? -0.125f : 0.125f, (qh[0] & 0x80) ? -0.125f : 0.125f, (qh[1] & 0x08) ? -0.125f : 0.125f, (qh[1] & 0x80) ? -0.125f : 0.125f};
          for (int l = 0; l < 4; ++l) { const uint16_t gc = kIq1sCode[idx[l]]; const float s = l < 2 ? dl1 : dl2;
            for (int j = 0; j < 8; ++j) yy[j] = s * ((float)((int)((gc >> (2 * j)) & 3) - 1) + dl[l]);
            yy += 8; }
          qs += 4; qh += 2;
        }
      }
      break;
    case ORC_Q5_K:          // gguf_q.rs:108-113: as Q4_K with a fifth bit per value from qh (bit 2j for the low nibbles, 2j+1 for the high)
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b), mn = h2f(b + 2); const uint8_t* sc = b + 4; const uint8_t* qh = b + 16; const uint8_t* ql = b + 48; float* yy = y + i * 256;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 4; ++j) {
          uint8_t s1, m1, s2, m2; scale_min_k4(2 * j, sc, &s1, &m1); scale_min_k4(2 * j + 1, sc, &s2, &m2);
          float d1 = d * (float)s1, M1 = mn * (float)m1, d2 = d * (float)s2, M2 = mn * (float)m2;
          for (int l = 0; l < 32; ++l) { yy[l] = d1 * (float)((ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0)) - M1; yy[l + 32] = d2 * (float)((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - M2; }
          yy += 64; ql += 32; u1 = (uint8_t)(u1 << 2); u2 = (uint8_t)(u2 << 2);
        }
      }
      break;
    case ORC_IQ2_XS:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b); const uint8_t* qs = b + 2; const uint8_t* sc = b + 66; float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ++ib) {
          float db[2] = { d * (0.5f + (float)(sc[ib] & 0xF)) * 0.25f, d * (0.5f + (float)(sc[ib] >> 4)) * 0.25f };
          for (int l = 0; l < 4; ++l) {
            uint32_t q = (uint32_t)qs[2 * (4 * ib + l)] | ((uint32_t)qs[2 * (4 * ib + l) + 1] << 8);
            uint64_t gv = T.iq2xs[q & 511]; float g[8]; for (int j = 0; j < 8; ++j) g[j] = (float)((gv >> (8 * j)) & 0xFF);
            put8(yy, db[l / 2], g, T.ksigns[q >> 9]); yy += 8;
          }
        }
      }
      break;
    case ORC_IQ3_S:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b); const uint8_t* qs = b + 2; const uint8_t* qh = b + 66; const uint8_t* signs = b + 74; const uint8_t* sc = b + 106;
        float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ib += 2) {
          for (int half = 0; half < 2; ++half) {
            uint8_t s = sc[ib / 2]; float db = d * (float)(1 + 2 * (half == 0 ? (s & 0xF) : (s >> 4)));
            for (int l = 0; l < 4; ++l) {
              uint32_t g1 = T.iq3s[qs[2 * l] | (((uint32_t)qh[half] << (8 - 2 * l)) & 256)];
              uint32_t g2 = T.iq3s[qs[2 * l + 1] | (((uint32_t)qh[half] << (7 - 2 * l)) & 256)];
              float g[8]; for (int j = 0; j < 4; ++j) { g[j] = (float)((g1 >> (8 * j)) & 0xFF); g[4 + j] = (float)((g2 >> (8 * j)) & 0xFF); }
              put8(yy, db, g, signs[l]); yy += 8;
            }
            qs += 8; signs += 4;
          }
          qh += 2;
        }
      }
      break;
    case ORC_Q2_0:          // gguf_q.rs:80-81 with lut q2 (:50): value j of byte k = ((byte >> 2j) & 3) - 1, times d
      for (size_t i = 0; i < nb; ++i) { const uint8_t* b = x + i * bs; float d = h2f(b); float* yy = y + i * 64;
        for (int k = 0; k < 16; ++k) for (int j = 0; j < 4; ++j) yy[4 * k + j] = (float)((int)((b[2 + k] >> (2 * j)) & 3) - 1) * d; }
      break;
    case ORC_Q3_K:          // gguf_q.rs:90-102
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; const uint8_t* hm = b; const uint8_t* q = b + 32; const uint8_t* sc = b + 96; const float d_all = h2f(b + 108);
        auto a = [&](int k) { return (uint32_t)sc[4 * k] | ((uint32_t)sc[4 * k + 1] << 8) | ((uint32_t)sc[4 * k + 2] << 16) | ((uint32_t)sc[4 * k + 3] << 24); };
        const uint32_t a0 = a(0), a1 = a(1), tmp = a(2), k1 = 0x03030303u, k2 = 0x0f0f0f0fu;
        const uint32_t aux[4] = {(a0 & k2) | ((tmp & k1) << 4), (a1 & k2) | (((tmp >> 2) & k1) << 4), ((a0 >> 4) & k2) | (((tmp >> 4) & k1) << 4), ((a1 >> 4) & k2) | (((tmp >> 6) & k1) << 4)};
        int8_t scales[16]; for (int k = 0; k < 16; ++k) scales[k] = (int8_t)((aux[k >> 2] >> (8 * (k & 3))) & 0xFF);
        float* yy = y + i * 256; int is = 0; uint8_t m = 1;
        for (int n = 0; n < 2; ++n) { int shift = 0;
          for (int j = 0; j < 4; ++j) {
            for (int half = 0; half < 2; ++half) { const float dl = d_all * (float)((int)scales[is] - 32); ++is;
              for (int l = 0; l < 16; ++l) { const int o = l + 16 * half; yy[l] = dl * (float)((int)((q[o] >> shift) & 3) - ((hm[o] & m) ? 0 : 4)); }
              yy += 16; }
            shift += 2; m = (uint8_t)(m << 1); }
          q += 32; }
      }
      break;
    case ORC_Q4_0:
      for (size_t i = 0; i < nb; ++i) { const uint8_t* b = x + i * bs; float d = h2f(b); float* yy = y + i * 32;
        for (int j = 0; j < 16; ++j) { yy[j] = (float)((int)(b[2 + j] & 0xF) - 8) * d; yy[j + 16] = (float)((int)(b[2 + j] >> 4) - 8) * d; } }
      break;
    case ORC_Q5_0:
      for (size_t i = 0; i < nb; ++i) { const uint8_t* b = x + i * bs; float d = h2f(b); uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
        const uint8_t* qs = b + 6; float* yy = y + i * 32;
        for (int j = 0; j < 16; ++j) { uint8_t h0 = (uint8_t)(((qh >> j) << 4) & 0x10), h1 = (uint8_t)((qh >> (j + 12)) & 0x10);
          yy[j] = (float)((int)((qs[j] & 0xF) | h0) - 16) * d; yy[j + 16] = (float)((int)((qs[j] >> 4) | h1) - 16) * d; } }
      break;
    case ORC_IQ4_NL:
      for (size_t i = 0; i < nb; ++i) { const uint8_t* b = x + i * bs; float d = h2f(b); float* lo = y + i * 32; float* hi = lo + 16;
        for (int j = 0; j < 16; ++j) { lo[j] = d * (float)kIq4nlValues[b[2 + j] & 0xF]; hi[j] = d * (float)kIq4nlValues[b[2 + j] >> 4]; } }
      break;
    case ORC_IQ4_XS:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b); uint32_t sh = (uint32_t)b[2] | ((uint32_t)b[3] << 8); const uint8_t* sl = b + 4; const uint8_t* qs = b + 8; float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ++ib) {
          int ls = (int)((sl[ib / 2] >> (4 * (ib % 2))) & 0xF) | (int)(((sh >> (2 * ib)) & 3) << 4); float dl = d * (float)(ls - 32);
          for (int j = 0; j < 16; ++j) { yy[j] = (float)kIq4nlValues[qs[j] & 0xF] * dl; yy[j + 16] = (float)kIq4nlValues[qs[j] >> 4] * dl; }
          yy += 32; qs += 16;
        }
      }
      break;
    case ORC_Q6_K:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; const uint8_t* ql = b; const uint8_t* qh = b + 128; const int8_t* sc = (const int8_t*)(b + 192); float d = h2f(b + 208); float* yy = y + i * 256;
        for (int n = 0; n < 2; ++n) {
          for (int l = 0; l < 32; ++l) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32, q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32, q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            yy[l] = d * (float)sc[is] * (float)q1; yy[l + 32] = d * (float)sc[is + 2] * (float)q2;
            yy[l + 64] = d * (float)sc[is + 4] * (float)q3; yy[l + 96] = d * (float)sc[is + 6] * (float)q4;
          }
          yy += 128; ql += 64; qh += 32; sc += 8;
        }
      }
      break;
    case ORC_IQ2_XXS:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b); const uint8_t* qs = b + 2; float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ++ib) {
          const uint8_t* a0 = qs + 8 * ib; uint32_t a1 = (uint32_t)a0[4] | ((uint32_t)a0[5] << 8) | ((uint32_t)a0[6] << 16) | ((uint32_t)a0[7] << 24);
          float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
          for (int l = 0; l < 4; ++l) {
            uint64_t gv = T.iq2xxs[a0[l]]; float g[8]; for (int j = 0; j < 8; ++j) g[j] = (float)((gv >> (8 * j)) & 0xFF);
            put8(yy, db, g, T.ksigns[(a1 >> (7 * l)) & 127]); yy += 8;
          }
        }
      }
      break;
    case ORC_IQ2_S:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b); const uint8_t* qs = b + 2; const uint8_t* signs = b + 34; const uint8_t* qh = b + 66; const uint8_t* sc = b + 74; float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ++ib) {
          float db[2] = { d * (0.5f + (float)(sc[ib] & 0xF)) * 0.25f, d * (0.5f + (float)(sc[ib] >> 4)) * 0.25f };
          for (int l = 0; l < 4; ++l) {
            uint32_t idx = (uint32_t)qs[l] | (((uint32_t)qh[ib] << (8 - 2 * l)) & 0x300);
            uint64_t gv = T.iq2s[idx]; float g[8]; for (int j = 0; j < 8; ++j) g[j] = (float)((gv >> (8 * j)) & 0xFF);
            put8(yy, db[l / 2], g, signs[l]); yy += 8;
          }
          qs += 4; signs += 4;
        }
      }
      break;
    case ORC_IQ3_XXS:
      for (size_t i = 0; i < nb; ++i) {
        const uint8_t* b = x + i * bs; float d = h2f(b); const uint8_t* qs = b + 2; const uint8_t* ss = b + 66; float* yy = y + i * 256;
        for (int ib = 0; ib < 8; ++ib) {
          uint32_t a = (uint32_t)ss[4 * ib] | ((uint32_t)ss[4 * ib + 1] << 8) | ((uint32_t)ss[4 * ib + 2] << 16) | ((uint32_t)ss[4 * ib + 3] << 24);
          float db = d * (0.5f + (float)(a >> 28)) * 0.5f;
          for (int l = 0; l < 4; ++l) {
            uint32_t g1 = T.iq3xxs[qs[8 * ib + 2 * l]], g2 = T.iq3xxs[qs[8 * ib + 2 * l + 1]];
            float g[8]; for (int j = 0; j < 4; ++j) { g[j] = (float)((g1 >> (8 * j)) & 0xFF); g[4 + j] = (float)((g2 >> (8 * j)) & 0xFF); }
            put8(yy, db, g, T.ksigns[(a >> (7 * l)) & 127]); yy += 8;
          }
        }
      }
      break;
    default: return false;
  }
  return true;
}

// dot_avx2, gguf_q.rs:175-197: four 8-lane FMA accumulators over strides of 32, an 8-wide tail into the first,
// (s0+s1)+(s2+s3), the 8 lanes summed in order, then a scalar tail (mul then add, not fused: `r += a[i] * b[i]`).
float dot(const float* a, const float* b, size_t n) {
  float s[4][8] = {};
  size_t i = 0;
  for (; i + 32 <= n; i += 32)
    for (int k = 0; k < 4; ++k)
      for (int j = 0; j < 8; ++j) s[k][j] = __builtin_fmaf(a[i + 8 * k + j], b[i + 8 * k + j], s[k][j]);
  for (; i + 8 <= n; i += 8) for (int j = 0; j < 8; ++j) s[0][j] = __builtin_fmaf(a[i + j], b[i + j], s[0][j]);
  float t[8]; for (int j = 0; j < 8; ++j) t[j] = (s[0][j] + s[1][j]) + (s[2][j] + s[3][j]);
  float r = 0.0f; for (int j = 0; j < 8; ++j) r += t[j];
  for (; i < n; ++i) r += a[i] * b[i];
  return r;
}

void parallel_for(size_t n, int threads, const std::function<void(size_t, size_t)>& f) {
  if (threads <= 1 || n < 2) { f(0, n); return; }
  size_t nt = std::min<size_t>(threads, n);
  std::vector<std::thread> th; th.reserve(nt);
  std::atomic<size_t> next{0};
  size_t chunk = std::max<size_t>(1, n / (nt * 8));
  for (size_t k = 0; k < nt; ++k) th.emplace_back([&] { for (;;) { size_t a = next.fetch_add(chunk); if (a >= n) break; f(a, std::min(n, a + chunk)); } });
  for (auto& t : th) t.join();
}

// QMat::matmul for t < 16, gguf_q.rs:233-241: each row dequantized once, dotted against every token.
// y[ti*rows + r] = sum_c W[r,c] * x[ti*cols + c]   (gguf_q.rs:216)
bool matmul(uint32_t ty, const uint8_t* w, size_t rows, size_t cols, const float* x, int t, float* y, int threads) {
  int qk, bs; if (!geom(ty, &qk, &bs) || cols % qk) return false;
  size_t rb = cols / qk * bs;
  int th = (rows * cols < (1u << 18)) ? 1 : threads;
  parallel_for(rows, th, [&](size_t r0, size_t r1) {
    std::vector<float> buf(cols);
    for (size_t r = r0; r < r1; ++r) { dequant(ty, w + r * rb, cols, buf.data()); for (int ti = 0; ti < t; ++ti) y[(size_t)ti * rows + r] = dot(buf.data(), x + (size_t)ti * cols, cols); }
  });
  return true;
}
inline bool mm(const OrcTensor* m, const float* x, int t, float* y, int threads) { return matmul(m->ty, (const uint8_t*)m->data, m->rows, m->cols, x, t, y, threads); }

inline float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }               // qwen4exp_gguf.rs:457
inline float silu(float x) { return x * sigm(x); }                             // :458
inline float softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }     // :459

// rms, qwen4exp_gguf.rs:209: y = x * s * w ;  rms_inplace, :210: x *= s * w  (different association)
inline float rms_scale(const float* x, size_t n, float eps) { float ss = 0.0f; for (size_t i = 0; i < n; ++i) ss += x[i] * x[i]; return 1.0f / sqrtf(ss / (float)n + eps); }
void rms(const float* x, const float* w, float eps, float* y, size_t n) { float s = rms_scale(x, n, eps); for (size_t i = 0; i < n; ++i) y[i] = x[i] * s * w[i]; }
void rms_inplace(float* x, const float* w, float eps, size_t n) { float s = rms_scale(x, n, eps); for (size_t i = 0; i < n; ++i) x[i] *= s * w[i]; }

// kv4::pack, kv4.rs:12-31 (Rust f32::round = half away from zero = roundf)
void kv4_pack(const float* x, size_t n, uint32_t* w, float* sc) {
  for (size_t b = 0; b < n / 32; ++b) {
    const float* p = x + 32 * b; float m = 0.0f; for (int i = 0; i < 32; ++i) m = fmaxf(m, fabsf(p[i]));
    float s = (m > 0.0f && std::isfinite(m)) ? m / 7.0f : 0.0f; sc[b] = s;
    for (int c = 0; c < 4; ++c) {
      uint32_t u = 0;
      for (int j = 0; j < 8; ++j) { int q = s > 0.0f ? (int)fminf(fmaxf(roundf(p[8 * c + j] / s), -7.0f), 7.0f) : 0; u |= ((uint32_t)(uint8_t)(int8_t)q & 0xF) << (4 * j); }
      w[4 * b + c] = u;
    }
  }
}
inline float kv4_get(const uint32_t* w, const float* sc, size_t i) {  // kv4.rs:35-39
  uint32_t nib = (w[i / 8] >> (4 * (i % 8))) & 0xF; int q = (int)nib - (nib >= 8 ? 16 : 0); return (float)q * sc[i / 32];
}
// kvq_roundtrip, qwen4exp_gguf.rs:3313-3317
void kvq_roundtrip(float* x, size_t n, int bits) {
  float q = (float)((1 << (bits - 1)) - 1);
  for (size_t b = 0; b < n / 32; ++b) { float* p = x + 32 * b; float m = 0.0f; for (int i = 0; i < 32; ++i) m = fmaxf(m, fabsf(p[i]));
    if (m == 0.0f || !std::isfinite(m)) continue; float s = m / q; for (int i = 0; i < 32; ++i) p[i] = fminf(fmaxf(roundf(p[i] / s), -q), q) * s; }
}
// Packed region of the cache for a query that sees n positions: [0, ((n - recent)/64)*64), the split of
// kv_push's packed branch (qwen4exp_gguf.rs:1519-1520: `cl > dense + recent + 64`, `q8n = ((cl - recent)/64)*64`),
// applied at every step instead of only when the device buffer is reallocated.
size_t packed_boundary(size_t n, int kv_bits, int recent) { if (kv_bits != 4 || n <= (size_t)recent + 64) return 0; return ((n - recent) / 64) * 64; }

// top_k + soft_top, qwen4exp_gguf.rs:3121-3139.  The reference's host selection leaves the order among the k chosen
// unspecified (select_nth_unstable); its device router ranks with lower-index-wins ties and lists the chosen experts
// in ascending id (qn_cube.rs:5225-5237).  This statement fixes: ties -> lower index, order -> ascending id,
// max / exp / sum / divide over that order.  NaN logits -> -inf, all non-finite max -> uniform (:3121-3129).
bool top_k(const float* r0, int n, int k, int32_t* idx, float* w) {
  if (k > n || k <= 0) return false;
  std::vector<float> r(r0, r0 + n);
  for (auto& v : r) if (std::isnan(v)) v = -INFINITY;
  int c = 0;
  for (int e = 0; e < n; ++e) { int rank = 0; for (int j = 0; j < n; ++j) if (r[j] > r[e] || (r[j] == r[e] && j < e)) ++rank; if (rank < k) idx[c++] = e; }
  float mx = -INFINITY; for (int i = 0; i < k; ++i) mx = fmaxf(mx, r[idx[i]]);
  if (!std::isfinite(mx)) { for (int i = 0; i < k; ++i) w[i] = 1.0f / (float)k; return true; }
  float sum = 0.0f; for (int i = 0; i < k; ++i) { w[i] = expf(r[idx[i]] - mx); sum += w[i]; }
  for (int i = 0; i < k; ++i) w[i] = w[i] / sum;
  return true;
}

// linear_core, qwen4exp_gguf.rs:1624-1673 (the t == 1 loop form, :1642-1647, applied per token)
void gdn_core(int nk, int nv, int dk, int dv, int kk, float eps, const float* a, const float* dt, const float* conv, const float* norm,
              const float* m, const float* zz, const float* bb, const float* aa, int t, float* cs, float* s, float* o_all) {
  int ch = 2 * nk * dk + nv * dv; int w = nv * dv;
  std::vector<float> co(ch), mem(dv), delta(dv);
  for (int ti = 0; ti < t; ++ti) {
    const float* cur = m + (size_t)ti * ch;
    for (int cc = 0; cc < ch; ++cc) { float o = conv[cc * kk + kk - 1] * cur[cc]; for (int k = 0; k < kk - 1; ++k) o += conv[cc * kk + k] * cs[(size_t)k * ch + cc]; co[cc] = silu(o); }
    memmove(cs, cs + ch, sizeof(float) * (size_t)(kk - 2) * ch); memcpy(cs + (size_t)(kk - 2) * ch, cur, sizeof(float) * ch);
    for (int h = 0; h < nk; ++h) {  // :1649-1651
      float* qp = co.data() + h * dk; float* kp = co.data() + nk * dk + h * dk;
      float sq = 0.0f; for (int i = 0; i < dk; ++i) sq += qp[i] * qp[i]; float nq = (1.0f / sqrtf(sq + 1e-6f)) * (1.0f / sqrtf((float)dk)); for (int i = 0; i < dk; ++i) qp[i] *= nq;
      float sk = 0.0f; for (int i = 0; i < dk; ++i) sk += kp[i] * kp[i]; float nkk = (1.0f / sqrtf(sk + 1e-6f)) * 1.0f; for (int i = 0; i < dk; ++i) kp[i] *= nkk;
    }
    for (int h = 0; h < nv; ++h) {  // :1654-1670
      int kh = h % nk; float* sh = s + (size_t)h * dk * dv;
      const float* qv = co.data() + kh * dk; const float* kv = co.data() + nk * dk + kh * dk; const float* vv = co.data() + 2 * nk * dk + h * dv;
      float g = expf(softplus(aa[ti * nv + h] + dt[h]) * a[h]); float b = sigm(bb[ti * nv + h]);
      for (int i = 0; i < dk * dv; ++i) sh[i] *= g;
      for (int j = 0; j < dv; ++j) mem[j] = 0.0f;
      for (int i = 0; i < dk; ++i) { float ki = kv[i]; const float* row = sh + (size_t)i * dv; for (int j = 0; j < dv; ++j) mem[j] += row[j] * ki; }
      for (int j = 0; j < dv; ++j) delta[j] = (vv[j] - mem[j]) * b;
      float* oh = o_all + (size_t)ti * w + h * dv; for (int j = 0; j < dv; ++j) oh[j] = 0.0f;
      for (int i = 0; i < dk; ++i) { float ki = kv[i], qi = qv[i]; float* row = sh + (size_t)i * dv; for (int j = 0; j < dv; ++j) { row[j] += ki * delta[j]; oh[j] += row[j] * qi; } }
      rms_inplace(oh, norm, eps, dv); const float* zh = zz + (size_t)ti * w + h * dv; for (int j = 0; j < dv; ++j) oh[j] *= sigm(zh[j]);
    }
  }
}

// rope, qwen4exp_gguf.rs:1436-1439 with rope_cs :529-533: angle = pos as f32 * inv[i]; cos and sin are multiplied by
// the YaRN magnitude factor only when it is not 1
void rope(float* v, int pos, int n_rot, const float* inv, float mscale = 1.0f) {
  int half = n_rot / 2;
  for (int i = 0; i < half; ++i) { float a = (float)pos * inv[i]; float s = sinf(a), c = cosf(a); if (mscale != 1.0f) { c = c * mscale; s = s * mscale; }
    float x0 = v[i], x1 = v[i + half]; v[i] = x0 * c - x1 * s; v[i + half] = x1 * c + x0 * s; }
}

// attn_core, qwen4exp_gguf.rs:1558-1615.  Cache rows below the packed boundary are read through the 4-bit round trip
// (kvq_roundtrip semantics, :1535), the cache itself keeps f32.  With an indexer (idx_nh > 0): raw index keys are
// appended, every completed block of `ratio` tokens is pooled (mean, RMSNorm, RoPE at the block's first position,
// :1571-1578), and a query that sees more than budget + ratio - 1 positions attends only to the budget/ratio blocks
// with the largest  sum_h relu(q_h . block key) / sqrt(idx_hd)  plus the incomplete tail (:1589-1599).
struct Qsa { int nh = 0, hd = 0, ratio = 1, budget = 0; const float* iqn = nullptr; const float* ikn = nullptr; const float* iq = nullptr; const float* ik = nullptr;
             float* ikc = nullptr; float* ibc = nullptr; int32_t* sel = nullptr; int32_t* sel_n = nullptr; int sel_stride = 0; };
void attn_core(int nh, int nkv, int hd, int n_rot, float eps, const float* inv, float mscale, const float* qn, const float* kn,
               const float* qf, const float* kf_in, const float* vf, int start, int t, int kv_bits, int recent, float* kc, float* vc, float* att, const Qsa& qs = Qsa()) {
  size_t row = (size_t)nkv * hd;
  std::vector<float> kf(kf_in, kf_in + (size_t)t * row);
  for (int ti = 0; ti < t; ++ti) for (int h = 0; h < nkv; ++h) { float* kh = kf.data() + ti * row + (size_t)h * hd; rms_inplace(kh, kn, eps, hd); rope(kh, start + ti, n_rot, inv, mscale); }
  memcpy(kc + start * row, kf.data(), sizeof(float) * t * row); memcpy(vc + start * row, vf, sizeof(float) * t * row);
  const int ihd = qs.hd, ir = qs.ratio, inh = qs.nh; const int dense_n = inh > 0 ? qs.budget + ir - 1 : INT32_MAX;
  std::vector<float> iqs;
  if (inh > 0) {
    memcpy(qs.ikc + (size_t)start * ihd, qs.ik, sizeof(float) * (size_t)t * ihd);
    int nt = start + t;
    for (int b = start / ir; b < nt / ir; ++b) {          // blocks [0, start / ir) were pooled by earlier calls
      float* pk = qs.ibc + (size_t)b * ihd; for (int i = 0; i < ihd; ++i) pk[i] = 0.0f;
      for (int p = b * ir; p < (b + 1) * ir; ++p) for (int i = 0; i < ihd; ++i) pk[i] += qs.ikc[(size_t)p * ihd + i];
      for (int i = 0; i < ihd; ++i) pk[i] /= (float)ir;
      rms_inplace(pk, qs.ikn, eps, ihd); rope(pk, b * ir, n_rot, inv, mscale);
    }
    if (start + t > dense_n) {
      iqs.assign(qs.iq, qs.iq + (size_t)t * inh * ihd);
      for (int ti = 0; ti < t; ++ti) for (int h = 0; h < inh; ++h) { float* qh = iqs.data() + ((size_t)ti * inh + h) * ihd; rms_inplace(qh, qs.iqn, eps, ihd); rope(qh, start + ti, n_rot, inv, mscale); }
    }
  }
  float scale = 1.0f / sqrtf((float)hd); int grp = nh / nkv;
  std::vector<float> qh(hd), krt(row), vrt(row);
  for (int ti = 0; ti < t; ++ti) {
    int n = start + ti + 1; size_t pb = packed_boundary(n, kv_bits, recent);
    std::vector<int> ps;                      // attended positions, ascending
    bool sparse = !iqs.empty() && n > dense_n;
    if (sparse) {
      int nb = n / ir, kk = qs.budget / ir; float iscale = 1.0f / sqrtf((float)ihd);
      const float* q = iqs.data() + (size_t)ti * inh * ihd;
      std::vector<std::pair<float, int>> sc(nb);
      for (int b = 0; b < nb; ++b) { const float* kb = qs.ibc + (size_t)b * ihd; float sm = 0.0f; for (int h = 0; h < inh; ++h) sm += fmaxf(dot(q + (size_t)h * ihd, kb, ihd), 0.0f); sc[b] = {sm * iscale, b}; }
      std::stable_sort(sc.begin(), sc.end(), [](const std::pair<float, int>& a, const std::pair<float, int>& b) { return a.first > b.first; });   // ties: lower block first
      std::vector<int> blocks; for (int i = 0; i < kk && i < nb; ++i) blocks.push_back(sc[i].second);
      std::sort(blocks.begin(), blocks.end());
      for (int b : blocks) for (int p = b * ir; p < (b + 1) * ir; ++p) ps.push_back(p);
      for (int p = nb * ir; p < n; ++p) ps.push_back(p);
    } else { ps.resize(n); for (int p = 0; p < n; ++p) ps[p] = p; }
    if (qs.sel_n) { qs.sel_n[ti] = sparse ? (int32_t)ps.size() : -1; if (sparse && qs.sel) for (size_t i = 0; i < ps.size() && (int)i < qs.sel_stride; ++i) qs.sel[(size_t)ti * qs.sel_stride + i] = ps[i]; }
    const int np = (int)ps.size();
    for (int h = 0; h < nh; ++h) {
      size_t base = (size_t)ti * nh * 2 * hd + (size_t)h * 2 * hd;
      memcpy(qh.data(), qf + base, sizeof(float) * hd); rms_inplace(qh.data(), qn, eps, hd); rope(qh.data(), start + ti, n_rot, inv, mscale);
      int kvh = h / grp; float* out = att + ((size_t)ti * nh + h) * hd; for (int i = 0; i < hd; ++i) out[i] = 0.0f;
      std::vector<float> sc(np);
      for (int j = 0; j < np; ++j) {
        int p = ps[j]; const float* kr = kc + p * row + (size_t)kvh * hd;
        if ((size_t)p < pb) { memcpy(krt.data(), kr, sizeof(float) * hd); kvq_roundtrip(krt.data(), hd, 4); kr = krt.data(); }
        sc[j] = dot(qh.data(), kr, hd) * scale;
      }
      float mx = -INFINITY; for (int j = 0; j < np; ++j) mx = fmaxf(mx, sc[j]);
      float sum = 0.0f; for (int j = 0; j < np; ++j) { sc[j] = expf(sc[j] - mx); sum += sc[j]; }
      float iv = 1.0f / sum;
      for (int j = 0; j < np; ++j) {
        int p = ps[j]; float wgt = sc[j] * iv; const float* vr = vc + p * row + (size_t)kvh * hd;
        if ((size_t)p < pb) { memcpy(vrt.data(), vr, sizeof(float) * hd); kvq_roundtrip(vrt.data(), hd, 4); vr = vrt.data(); }
        for (int i = 0; i < hd; ++i) out[i] += wgt * vr[i];
      }
      const float* gate = qf + base + hd; for (int i = 0; i < hd; ++i) out[i] *= sigm(gate[i]);
    }
  }
}

// ffn + routed (f32 branch), qwen4exp_gguf.rs:1675-1684, 1721-1732, 1754-1793.
bool moe_ffn(int d, int n_exp, int k, int ff, const OrcTensor* router, const OrcTensor* gate_e, const OrcTensor* up_e, const OrcTensor* down_e,
             const float* sh_gate_inp, const OrcTensor* sh_gate, const OrcTensor* sh_up, const OrcTensor* sh_down,
             const float* x, int t, float* y, int32_t* sel_idx, float* sel_w, int threads) {
  size_t sf = sh_gate->rows;
  std::vector<float> lg((size_t)t * n_exp), g((size_t)t * sf), u((size_t)t * sf);
  if (!mm(router, x, t, lg.data(), threads) || !mm(sh_gate, x, t, g.data(), threads) || !mm(sh_up, x, t, u.data(), threads)) return false;
  for (size_t i = 0; i < g.size(); ++i) g[i] = silu(g[i]) * u[i];
  if (!mm(sh_down, g.data(), t, y, threads)) return false;
  for (int ti = 0; ti < t; ++ti) { float sg = sigm(dot(sh_gate_inp, x + (size_t)ti * d, d)); for (int i = 0; i < d; ++i) y[(size_t)ti * d + i] *= sg; }
  std::vector<std::vector<std::pair<int, float>>> by_exp(n_exp);
  std::vector<int32_t> idx(k); std::vector<float> w(k);
  for (int ti = 0; ti < t; ++ti) {
    if (!top_k(lg.data() + (size_t)ti * n_exp, n_exp, k, idx.data(), w.data())) return false;
    for (int i = 0; i < k; ++i) { by_exp[idx[i]].push_back({ti, w[i]}); if (sel_idx) sel_idx[ti * k + i] = idx[i]; if (sel_w) sel_w[ti * k + i] = w[i]; }
  }
  int qk, bs; geom(gate_e->ty, &qk, &bs); size_t rb_g = (size_t)d / qk * bs; geom(up_e->ty, &qk, &bs); size_t rb_u = (size_t)d / qk * bs; geom(down_e->ty, &qk, &bs); size_t rb_d = (size_t)ff / qk * bs;
  std::vector<int> work; for (int e = 0; e < n_exp; ++e) if (!by_exp[e].empty()) work.push_back(e);
  // hidden rows per expert: h[r] = silu(gate_e[r].x) * (up_e[r].x)   (:1773-1776)
  std::vector<std::vector<float>> hid(n_exp);
  for (int e : work) hid[e].assign(by_exp[e].size() * (size_t)ff, 0.0f);
  parallel_for(work.size() * (size_t)ff, threads, [&](size_t a, size_t b) {
    std::vector<float> buf(d);
    for (size_t q = a; q < b; ++q) {
      int e = work[q / ff]; size_t r = q % ff;
      dequant(gate_e->ty, (const uint8_t*)gate_e->data + ((size_t)e * ff + r) * rb_g, d, buf.data());
      std::vector<float> gv(by_exp[e].size()); for (size_t j = 0; j < by_exp[e].size(); ++j) gv[j] = dot(buf.data(), x + (size_t)by_exp[e][j].first * d, d);
      dequant(up_e->ty, (const uint8_t*)up_e->data + ((size_t)e * ff + r) * rb_u, d, buf.data());
      for (size_t j = 0; j < by_exp[e].size(); ++j) hid[e][j * ff + r] = silu(gv[j]) * dot(buf.data(), x + (size_t)by_exp[e][j].first * d, d);
    }
  });
  // o[ti][r] += w * (down_e[e*d + r] . hid), experts in ascending id from 0, then y += o   (:1786-1793)
  std::vector<float> o((size_t)t * d, 0.0f);
  parallel_for(d, threads, [&](size_t r0, size_t r1) {
    std::vector<float> buf(ff);
    for (size_t r = r0; r < r1; ++r) for (int e : work) {
      dequant(down_e->ty, (const uint8_t*)down_e->data + ((size_t)e * d + r) * rb_d, ff, buf.data());
      for (size_t j = 0; j < by_exp[e].size(); ++j) { int ti = by_exp[e][j].first; o[(size_t)ti * d + r] += by_exp[e][j].second * dot(buf.data(), hid[e].data() + j * ff, ff); }
    }
  });
  for (size_t i = 0; i < o.size(); ++i) y[i] += o[i];
  return true;
}

// hc_mix, qwen4exp_gguf.rs:1357-1382 (f32 branch :1373-1381); hc_combine :1384-1388
bool hc_mix(int d, int hc, float eps, const float* norm, const OrcTensor* down, const OrcTensor* inject, const OrcTensor* up,
            const float* x, int t, float* mixed, float* inj, int threads) {
  size_t w = (size_t)hc * d; size_t lr = down->rows;
  std::vector<float> xn(t * w), lo((size_t)t * lr), gate(t * w);
  for (size_t i = 0; i < (size_t)t * hc; ++i) { size_t s = i % hc; rms(x + i * d, norm + s * d, eps, xn.data() + i * d, d); }
  if (!mm(down, xn.data(), t, lo.data(), threads)) return false;
  for (auto& v : lo) v = silu(v / (float)hc);
  if (inject) { if (!mm(inject, xn.data(), t, inj, threads)) return false; for (int i = 0; i < t * hc; ++i) inj[i] /= (float)hc; }
  else for (int i = 0; i < t * hc; ++i) inj[i] = 0.0f;
  if (!mm(up, lo.data(), t, gate.data(), threads)) return false;
  for (int ti = 0; ti < t; ++ti) {
    float* mr = mixed + (size_t)ti * d; for (int i = 0; i < d; ++i) mr[i] = 0.0f;
    for (int s = 0; s < hc; ++s) for (int i = 0; i < d; ++i) { size_t k = ti * w + (size_t)s * d + i; mr[i] += xn[k] * sigm(gate[k]); }
    for (int i = 0; i < d; ++i) mr[i] /= (float)hc;
  }
  return true;
}
void hc_combine(int d, int hc, float* x, const float* out, const float* inj, int t) {
  for (int ti = 0; ti < t; ++ti) for (int s = 0; s < hc; ++s) { float w = 2.0f * sigm(inj[ti * hc + s]); float* r = x + ((size_t)ti * hc + s) * d; for (int i = 0; i < d; ++i) r[i] += out[(size_t)ti * d + i] * w; }
}


// ---------- per-layer n-gram embeddings (PLE) ------------------------------------------------------
// ple_rows, qwen4exp_gguf.rs:1390-1407
bool ple_rows(const OrcCfg& c, const OrcTensor& tab, const uint32_t* tokens, int start, int t, float* emb) {
  const int ng = c.ple_ngram, nh = (ng - 1) * c.ple_per_gram, hd = c.ple_dim;
  int qk, bs; if (!geom(tab.ty, &qk, &bs) || hd % qk || (int)tab.cols != hd) return false; const size_t rb = (size_t)hd / qk * bs;
  for (int ti = 0; ti < t; ++ti) {
    const int p = start + ti;
    uint64_t ctx[8]; for (int s = 0; s < ng; ++s) ctx[s] = tokens[p];
    bool cut = false;
    for (int s = 1; s < ng; ++s) {
      const bool none = cut || p < s; const uint32_t tk = none ? 0 : tokens[p - s];
      cut = cut || none || tk == c.ple_eos; ctx[s] = cut ? (uint64_t)c.ple_eos : (uint64_t)tk;
    }
    for (int n = 2; n <= ng; ++n) {
      uint64_t mixed = ctx[0] * c.ple_mult[0];                       // wrapping
      for (int j = 1; j < n; ++j) mixed ^= ctx[j] * c.ple_mult[j];
      for (int gi = 0; gi < c.ple_per_gram; ++gi) {
        const int h = (n - 2) * c.ple_per_gram + gi; const uint64_t row = mixed % c.ple_vocab[h] + c.ple_off[h];
        if (row >= tab.rows) return false;
        if (!dequant(tab.ty, (const uint8_t*)tab.data + row * rb, hd, emb + ((size_t)ti * nh + h) * hd)) return false;
      }
    }
  }
  return true;
}
// ple, qwen4exp_gguf.rs:1409-1434
bool ple_apply(const OrcCfg& c, const OrcTensor* key, const OrcTensor* value, const float* nk, const float* nq, const float* nc, const float* conv,
               std::vector<float>& hist, const float* emb, float* x, int t, int th) {
  const int d = c.d, hc = c.hc, w = hc * d, dil = c.ple_ngram, K = c.ple_conv_k, hl = (K - 1) * dil;
  if ((int)key->rows != w || (int)value->rows != d || key->cols != value->cols || (int)hist.size() != hl * w) return false;
  std::vector<float> kt((size_t)t * w), vt((size_t)t * d);
  if (!mm(key, emb, t, kt.data(), th) || !mm(value, emb, t, vt.data(), th)) return false;
  std::vector<float> gated(w), nrm(w), kk(d), q(d);
  for (int ti = 0; ti < t; ++ti) {
    float* xt = x + (size_t)ti * w;
    for (int s = 0; s < hc; ++s) {
      memcpy(kk.data(), &kt[(size_t)ti * w + (size_t)s * d], sizeof(float) * d); rms_inplace(kk.data(), nk + (size_t)s * d, c.eps, d);
      rms(xt + (size_t)s * d, nq + (size_t)s * d, c.eps, q.data(), d);
      const float sc = dot(kk.data(), q.data(), d) / sqrtf((float)d);
      const float g = sc != sc ? sc : sigm(copysignf(1.0f, sc) * sqrtf(fmaxf(fabsf(sc), 1e-6f)));      // f32::signum: +-1 by the sign bit (also of zero), NaN for NaN
      for (int i = 0; i < d; ++i) gated[(size_t)s * d + i] = vt[(size_t)ti * d + i] * g;
    }
    nrm = gated;
    for (int s = 0; s < hc; ++s) rms_inplace(nrm.data() + (size_t)s * d, nc + (size_t)s * d, c.eps, d);
    // depthwise causal conv, dilation = n-gram length: taps K-1 (now), then (K-1-k)*dil rows back; hist oldest first
    for (int ch = 0; ch < w; ++ch) {
      float o = conv[(size_t)ch * K + K - 1] * nrm[ch];
      for (int k = 0; k < K - 1; ++k) { const int back = (K - 1 - k) * dil; o += conv[(size_t)ch * K + k] * hist[(size_t)(hl - back) * w + ch]; }
      xt[ch] += gated[ch] + silu(o);
    }
    hist.erase(hist.begin(), hist.begin() + w); hist.insert(hist.end(), nrm.begin(), nrm.end());
  }
  return true;
}

}  // namespace

// ---------- model ------------------------------------------------------------------------------
struct OrcModel {
  OrcCfg c; std::vector<OrcTensor> lt; OrcTensor g[ORC_GLOBAL_SLOTS]; int threads;
  std::vector<float> rope_inv; float mscale = 1.0f;
  bool has_idx(int il) const { return c.idx_nh > 0 && T(il, ORC_IDX_Q).data != nullptr; }
  std::vector<std::vector<float>> vec;  // dequantized small tensors, indexed like lt (empty when unused)
  std::vector<float> head_norm;
  const OrcTensor& T(int il, int slot) const { return lt[(size_t)il * ORC_LAYER_SLOTS + slot]; }
  const float* V(int il, int slot) const { return vec[(size_t)il * ORC_LAYER_SLOTS + slot].data(); }
  bool full(int il) const { return (il + 1) % c.full_every == 0; }
  bool has_ple(int il) const { return c.ple_ngram > 1 && T(il, ORC_PLE_KEY).data != nullptr; }
};
struct OrcCkpt { std::vector<std::vector<float>> conv, ssm, ple_hist; };
struct OrcState {
  std::vector<uint32_t> tokens;
  std::vector<std::vector<float>> conv, ssm, k, v, ik, ib;   // ik / ib: raw index keys [pos][idx_hd], pooled block keys [block][idx_hd]
  std::vector<std::vector<float>> ple_hist;                  // per PLE layer: the last (conv_k-1)*ngram normalised rows [hc*d], oldest first (:196)
  std::vector<OrcCkpt> ck;  // state after each token of the last forward_multi
  // MTP drafter (mtp_r / mtp_kv, qwen4exp_gguf.rs:206): the last final residuals by position; the drafter's own K/V cells
  int mtp_window = 0; std::deque<std::pair<int, std::vector<float>>> mtp_r;
  int mtp_c0 = 0, mtp_n = 0; std::vector<float> mtp_k, mtp_v;
};

static bool to_vec(const OrcTensor& t, std::vector<float>& out) {
  if (!t.data) return true; out.resize(t.rows * t.cols); int qk, bs; if (!geom(t.ty, &qk, &bs)) return false;
  return dequant(t.ty, (const uint8_t*)t.data, t.rows * t.cols, out.data());
}

extern "C" {

int orc_type_geom(uint32_t ty, int* e, int* b) { return geom(ty, e, b) ? 0 : -1; }
int orc_dequant(uint32_t ty, const uint8_t* x, size_t n, float* y) { int qk, bs; if (!geom(ty, &qk, &bs) || n % qk) return -1; return dequant(ty, x, n, y) ? 0 : -1; }
float orc_dot(const float* a, const float* b, size_t n) { return dot(a, b, n); }
int orc_matmul(uint32_t ty, const uint8_t* w, size_t rows, size_t cols, const float* x, int t, float* y, int threads) { return matmul(ty, w, rows, cols, x, t, y, threads) ? 0 : -1; }
void orc_expand_iq3s(uint32_t* o) { memcpy(o, tables().iq3s, sizeof(uint32_t) * 512); }
void orc_expand_iq2xs(uint64_t* o) { memcpy(o, tables().iq2xs, sizeof(uint64_t) * 512); }
uint8_t orc_ksigns(int i) { return tables().ksigns[i & 127]; }

void orc_kv4_pack(const float* x, size_t n, uint32_t* w, float* sc) { kv4_pack(x, n, w, sc); }
float orc_kv4_get(const uint32_t* w, const float* sc, size_t i) { return kv4_get(w, sc, i); }
void orc_kvq_roundtrip(float* x, size_t n, int bits) { kvq_roundtrip(x, n, bits); }
size_t orc_kv_packed_boundary(size_t n, int kv_bits, int recent) { return packed_boundary(n, kv_bits, recent); }

// rope_inv, qn_ctx.rs:164-170 (unscaled branch): inv[i] = base.powf(-(2 i) / n_rot)
void orc_rope_inv(int n_rot, float base, float* inv) { for (int i = 0; i < n_rot / 2; ++i) inv[i] = powf(base, -(2.0f * (float)i) / (float)n_rot); }
// rope_inv, qn_ctx.rs:164-185, both branches
float orc_rope_inv_yarn(int n_rot, float base, int ctx_train, int ctx, float* inv) {
  int half = n_rot / 2;
  float scale = (ctx_train > 0 && ctx > ctx_train) ? (float)ctx / (float)ctx_train : 1.0f;
  if (scale <= 1.0f) { orc_rope_inv(n_rot, base, inv); return 1.0f; }
  float dim = (float)n_rot;
  auto corr = [&](float rot) { return (dim * logf((float)ctx_train / (rot * 2.0f * 3.14159265358979323846f))) / (2.0f * logf(base)); };
  float low = fmaxf(floorf(corr(32.0f)), 0.0f);
  float high = fminf(ceilf(corr(1.0f)), (float)(half > 0 ? half - 1 : 0));
  for (int i = 0; i < half; ++i) {
    float extrap = powf(base, -(2.0f * (float)i) / dim), interp = extrap / scale;
    float ramp = fabsf(high - low) < 1e-6f ? 1.0f : fminf(fmaxf(((float)i - low) / (high - low), 0.0f), 1.0f);
    inv[i] = interp * (1.0f - ramp) + extrap * ramp;
  }
  return 1.0f + 0.1f * logf(scale);
}
// sampler::argmax, sampler.rs:142-148: first index of the maximum (strict >)
uint32_t orc_argmax(const float* l, size_t n) { size_t best = 0; for (size_t i = 1; i < n; ++i) if (l[i] > l[best]) best = i; return (uint32_t)best; }
int orc_top_k(const float* r, int n, int k, int32_t* idx, float* w) { return top_k(r, n, k, idx, w) ? 0 : -1; }
void orc_rms(const float* x, const float* w, float eps, float* y, size_t n) { rms(x, w, eps, y, n); }
void orc_rms_inplace(float* x, const float* w, float eps, size_t n) { rms_inplace(x, w, eps, n); }
float orc_sigm(float x) { return sigm(x); }
float orc_silu(float x) { return silu(x); }
float orc_softplus(float x) { return softplus(x); }

void orc_gdn_core(int nk, int nv, int dk, int dv, int conv_k, float eps, const float* a, const float* dt, const float* conv_w, const float* norm_w,
                  const float* qkv, const float* z, const float* beta, const float* alpha, int t, float* conv_state, float* ssm, float* out) {
  gdn_core(nk, nv, dk, dv, conv_k, eps, a, dt, conv_w, norm_w, qkv, z, beta, alpha, t, conv_state, ssm, out);
}
void orc_attn_core(int nh, int nkv, int hd, int n_rot, float eps, const float* inv, const float* qn, const float* kn, const float* q, const float* k, const float* v,
                   int start, int t, int kv_bits, int kv_recent, float* kc, float* vc, float* out) {
  attn_core(nh, nkv, hd, n_rot, eps, inv, 1.0f, qn, kn, q, k, v, start, t, kv_bits, kv_recent, kc, vc, out);
}
void orc_attn_core_qsa(int nh, int nkv, int hd, int n_rot, float eps, const float* inv, float mscale, const float* qn, const float* kn, const float* q, const float* k, const float* v,
                       int start, int t, int kv_bits, int kv_recent, float* kc, float* vc, int idx_nh, int idx_hd, int idx_ratio, int idx_budget, const float* iqn, const float* ikn,
                       const float* iq, const float* ik, float* ikc, float* ibc, float* out, int32_t* sel, int32_t* sel_n, int sel_stride) {
  Qsa qs; qs.nh = idx_nh; qs.hd = idx_hd; qs.ratio = idx_ratio < 1 ? 1 : idx_ratio; qs.budget = idx_budget; qs.iqn = iqn; qs.ikn = ikn; qs.iq = iq; qs.ik = ik; qs.ikc = ikc; qs.ibc = ibc;
  qs.sel = sel; qs.sel_n = sel_n; qs.sel_stride = sel_stride;
  attn_core(nh, nkv, hd, n_rot, eps, inv, mscale, qn, kn, q, k, v, start, t, kv_bits, kv_recent, kc, vc, out, qs);
}
int orc_moe_ffn(int d, int n_exp, int top_k_, int ff, const OrcTensor* router, const OrcTensor* gate_e, const OrcTensor* up_e, const OrcTensor* down_e,
                const float* sh_gate_inp, const OrcTensor* sh_gate, const OrcTensor* sh_up, const OrcTensor* sh_down,
                const float* x, int t, float* y, int32_t* sel_idx, float* sel_w, int threads) {
  return moe_ffn(d, n_exp, top_k_, ff, router, gate_e, up_e, down_e, sh_gate_inp, sh_gate, sh_up, sh_down, x, t, y, sel_idx, sel_w, threads) ? 0 : -1;
}
int orc_hc_mix(int d, int hc, float eps, const float* norm, const OrcTensor* down, const OrcTensor* inject, const OrcTensor* up,
               const float* x, int t, float* mixed, float* inj, int threads) { return hc_mix(d, hc, eps, norm, down, inject, up, x, t, mixed, inj, threads) ? 0 : -1; }
void orc_hc_combine(int d, int hc, float* x, const float* out, const float* inj, int t) { hc_combine(d, hc, x, out, inj, t); }

OrcModel* orc_model_create(const OrcCfg* cfg, const OrcTensor* lt, const OrcTensor* globals, int threads) {
  OrcModel* m = new OrcModel(); m->c = *cfg; m->threads = threads;
  m->lt.assign(lt, lt + (size_t)cfg->n_layers * ORC_LAYER_SLOTS); for (int i = 0; i < ORC_GLOBAL_SLOTS; ++i) m->g[i] = globals[i];
  m->vec.resize(m->lt.size());
  if (cfg->ple_ngram > 8 || (cfg->ple_ngram > 1 && ((cfg->ple_ngram - 1) * cfg->ple_per_gram > 16 || cfg->ple_conv_k < 1))) { delete m; return nullptr; }
  static const int vs[] = {ORC_HCA_NORM, ORC_HCF_NORM, ORC_ATTN_QN, ORC_ATTN_KN, ORC_LIN_A, ORC_LIN_DT, ORC_LIN_CONV, ORC_LIN_NORM, ORC_SH_GATE_INP, ORC_IDX_QN, ORC_IDX_KN,
                           ORC_PLE_NK, ORC_PLE_NQ, ORC_PLE_NC, ORC_PLE_CONV};
  for (int il = 0; il < cfg->n_layers; ++il) for (int s : vs) if (!to_vec(m->T(il, s), m->vec[(size_t)il * ORC_LAYER_SLOTS + s])) { delete m; return nullptr; }
  if (!to_vec(m->g[ORC_G_HEAD_NORM], m->head_norm)) { delete m; return nullptr; }
  m->rope_inv.resize(cfg->n_rot / 2); m->mscale = orc_rope_inv_yarn(cfg->n_rot, cfg->rope_base, cfg->ctx_train, cfg->ctx, m->rope_inv.data());
  return m;
}
void orc_model_destroy(OrcModel* m) { delete m; }

OrcState* orc_state_create(const OrcModel* m) {  // new_state, qwen4exp_gguf.rs:1345-1353
  OrcState* s = new OrcState(); const OrcCfg& c = m->c; int ch = 2 * c.lin_nk * c.lin_dk + c.lin_nv * c.lin_dv;
  for (int il = 0; il < c.n_layers; ++il) {
    if (m->full(il)) { s->k.emplace_back(); s->v.emplace_back(); s->ik.emplace_back(); s->ib.emplace_back(); }
    else { s->conv.emplace_back((size_t)(c.conv_k - 1) * ch, 0.0f); s->ssm.emplace_back((size_t)c.lin_nv * c.lin_dk * c.lin_dv, 0.0f); }
    if (m->has_ple(il)) s->ple_hist.emplace_back((size_t)(c.ple_conv_k - 1) * c.ple_ngram * c.hc * c.d, 0.0f);      // :1350
  }
  return s;
}
void orc_state_destroy(OrcState* s) { delete s; }
int orc_state_len(const OrcState* s) { return (int)s->tokens.size(); }
float* orc_state_conv(OrcState* s, int li) { return s->conv[li].data(); }
float* orc_state_ssm(OrcState* s, int li) { return s->ssm[li].data(); }
float* orc_state_k(OrcState* s, int ai) { return s->k[ai].data(); }
float* orc_state_v(OrcState* s, int ai) { return s->v[ai].data(); }
float* orc_state_ik(OrcState* s, int ai) { return s->ik[ai].data(); }
float* orc_state_ib(OrcState* s, int ai) { return s->ib[ai].data(); }
float* orc_state_ple_hist(OrcState* s, int pi) { return s->ple_hist[pi].data(); }
int orc_ple_rows(const OrcCfg* c, const OrcTensor* tab, const uint32_t* tokens, int start, int t, float* emb) { return ple_rows(*c, *tab, tokens, start, t, emb) ? 0 : -1; }
int orc_ple(const OrcCfg* c, const OrcTensor* key, const OrcTensor* value, const float* nk, const float* nq, const float* nc, const float* conv,
            float* hist, const float* emb, float* x, int t, int threads) {
  const size_t n = (size_t)(c->ple_conv_k - 1) * c->ple_ngram * c->hc * c->d; std::vector<float> h(hist, hist + n);
  if (!ple_apply(*c, key, value, nk, nq, nc, conv, h, emb, x, t, threads)) return -1;
  memcpy(hist, h.data(), n * sizeof(float)); return 0;
}

// forward_inner, qwen4exp_gguf.rs:2087-2157 (host branch :2134-2142, head :2150-2153)
int orc_forward(const OrcModel* m, OrcState* st, const uint32_t* ids, int t, float* logits) {
  const OrcCfg& c = m->c; int d = c.d, hc = c.hc; int start = (int)st->tokens.size(); int th = m->threads;
  for (int i = 0; i < t; ++i) if (ids[i] >= (uint32_t)c.vocab) return -1;
  st->tokens.insert(st->tokens.end(), ids, ids + t);
  std::vector<float> x((size_t)t * hc * d), e(d);
  const OrcTensor& embd = m->g[ORC_G_EMBD]; int qk, bs; if (!geom(embd.ty, &qk, &bs)) return -1; size_t erb = (size_t)d / qk * bs;
  for (int ti = 0; ti < t; ++ti) { dequant(embd.ty, (const uint8_t*)embd.data + ids[ti] * erb, d, e.data()); for (int s = 0; s < hc; ++s) memcpy(&x[((size_t)ti * hc + s) * d], e.data(), sizeof(float) * d); }
  int li = 0, ai = 0, pi = 0;
  std::vector<float> mixed((size_t)t * d), inj((size_t)t * hc), o((size_t)t * d), emb;
  if (c.ple_ngram > 1 && m->g[ORC_G_PLE_TAB].data) {      // :2093
    emb.resize((size_t)t * (c.ple_ngram - 1) * c.ple_per_gram * c.ple_dim);
    if (!ple_rows(c, m->g[ORC_G_PLE_TAB], st->tokens.data(), start, t, emb.data())) return -9;
  }
  for (int il = 0; il < c.n_layers; ++il) {
    if (m->has_ple(il)) {                                   // :2112
      if (emb.empty() || !ple_apply(c, &m->T(il, ORC_PLE_KEY), &m->T(il, ORC_PLE_VALUE), m->V(il, ORC_PLE_NK), m->V(il, ORC_PLE_NQ), m->V(il, ORC_PLE_NC), m->V(il, ORC_PLE_CONV),
                                    st->ple_hist[pi], emb.data(), x.data(), t, th)) return -9;
      ++pi;
    }
    if (hc_mix(d, hc, c.eps, m->V(il, ORC_HCA_NORM), &m->T(il, ORC_HCA_DOWN), &m->T(il, ORC_HCA_INJECT), &m->T(il, ORC_HCA_UP), x.data(), t, mixed.data(), inj.data(), th) == false) return -2;
    if (m->full(il)) {  // attn, :1441-1446
      int nh = c.n_head, nkv = c.n_kv, hd = c.hd; size_t row = (size_t)nkv * hd;
      std::vector<float> q((size_t)t * nh * 2 * hd), k(t * row), v(t * row), att((size_t)t * nh * hd);
      if (!mm(&m->T(il, ORC_ATTN_Q), mixed.data(), t, q.data(), th) || !mm(&m->T(il, ORC_ATTN_K), mixed.data(), t, k.data(), th) || !mm(&m->T(il, ORC_ATTN_V), mixed.data(), t, v.data(), th)) return -3;
      st->k[ai].resize((size_t)(start + t) * row); st->v[ai].resize((size_t)(start + t) * row);
      Qsa qs; std::vector<float> iq, ik;
      if (m->has_idx(il)) {
        int ihd = c.idx_hd, ir = c.idx_ratio < 1 ? 1 : c.idx_ratio; iq.resize((size_t)t * c.idx_nh * ihd); ik.resize((size_t)t * ihd);
        if (!mm(&m->T(il, ORC_IDX_Q), mixed.data(), t, iq.data(), th) || !mm(&m->T(il, ORC_IDX_K), mixed.data(), t, ik.data(), th)) return -3;
        st->ik[ai].resize((size_t)(start + t) * ihd); st->ib[ai].resize((size_t)((start + t) / ir) * ihd);
        qs.nh = c.idx_nh; qs.hd = ihd; qs.ratio = ir; qs.budget = c.idx_budget; qs.iqn = m->V(il, ORC_IDX_QN); qs.ikn = m->V(il, ORC_IDX_KN); qs.iq = iq.data(); qs.ik = ik.data();
        qs.ikc = st->ik[ai].data(); qs.ibc = st->ib[ai].data();
      }
      attn_core(nh, nkv, hd, c.n_rot, c.eps, m->rope_inv.data(), m->mscale, m->V(il, ORC_ATTN_QN), m->V(il, ORC_ATTN_KN), q.data(), k.data(), v.data(), start, t, c.kv_bits, c.kv_recent, st->k[ai].data(), st->v[ai].data(), att.data(), qs);
      if (!mm(&m->T(il, ORC_ATTN_O), att.data(), t, o.data(), th)) return -3;
      ++ai;
    } else {  // linear, :1617-1621
      int nk = c.lin_nk, nv = c.lin_nv, dk = c.lin_dk, dv = c.lin_dv; int ch = 2 * nk * dk + nv * dv;
      std::vector<float> qkv((size_t)t * ch), z((size_t)t * nv * dv), be((size_t)t * nv), al((size_t)t * nv), oa((size_t)t * nv * dv);
      if (!mm(&m->T(il, ORC_LIN_QKV), mixed.data(), t, qkv.data(), th) || !mm(&m->T(il, ORC_LIN_Z), mixed.data(), t, z.data(), th) || !mm(&m->T(il, ORC_LIN_BETA), mixed.data(), t, be.data(), th) || !mm(&m->T(il, ORC_LIN_ALPHA), mixed.data(), t, al.data(), th)) return -4;
      gdn_core(nk, nv, dk, dv, c.conv_k, c.eps, m->V(il, ORC_LIN_A), m->V(il, ORC_LIN_DT), m->V(il, ORC_LIN_CONV), m->V(il, ORC_LIN_NORM), qkv.data(), z.data(), be.data(), al.data(), t, st->conv[li].data(), st->ssm[li].data(), oa.data());
      if (!mm(&m->T(il, ORC_LIN_OUT), oa.data(), t, o.data(), th)) return -4;
      ++li;
    }
    hc_combine(d, hc, x.data(), o.data(), inj.data(), t);
    if (!hc_mix(d, hc, c.eps, m->V(il, ORC_HCF_NORM), &m->T(il, ORC_HCF_DOWN), &m->T(il, ORC_HCF_INJECT), &m->T(il, ORC_HCF_UP), x.data(), t, mixed.data(), inj.data(), th)) return -5;
    if (!moe_ffn(d, c.n_exp, c.top_k, c.ff_exp, &m->T(il, ORC_ROUTER), &m->T(il, ORC_GATE_E), &m->T(il, ORC_UP_E), &m->T(il, ORC_DOWN_E), m->V(il, ORC_SH_GATE_INP),
                 &m->T(il, ORC_SH_GATE), &m->T(il, ORC_SH_UP), &m->T(il, ORC_SH_DOWN), mixed.data(), t, o.data(), nullptr, nullptr, th)) return -6;
    hc_combine(d, hc, x.data(), o.data(), inj.data(), t);
  }
  if (st->mtp_window > 0) {      // mtp_keep_r for the last `window` tokens of the call, :2148-2150, :2279-2285
    for (int ti = std::max(0, t - st->mtp_window); ti < t; ++ti) {
      const int pos = start + ti;
      while (!st->mtp_r.empty() && st->mtp_r.back().first >= pos) st->mtp_r.pop_back();
      if (!st->mtp_r.empty() && st->mtp_r.back().first + 1 != pos) st->mtp_r.clear();
      st->mtp_r.emplace_back(pos, std::vector<float>(x.begin() + (size_t)ti * hc * d, x.begin() + (size_t)(ti + 1) * hc * d));
      while ((int)st->mtp_r.size() > st->mtp_window + 16) st->mtp_r.pop_front();
    }
  }
  std::vector<float> h(d), dummy(hc);
  if (!hc_mix(d, hc, c.eps, m->head_norm.data(), &m->g[ORC_G_HEAD_DOWN], nullptr, &m->g[ORC_G_HEAD_UP], x.data() + (size_t)(t - 1) * hc * d, 1, h.data(), dummy.data(), th)) return -7;
  if (!mm(&m->g[ORC_G_OUT], h.data(), 1, logits, th)) return -8;  // head_logits, :2361-2364
  return 0;
}

// forward_multi, qwen4exp_gguf.rs:2365-2480: logits after each token, every token's arithmetic equal to one-token
// decode (:2357-2360), recurrent-state checkpoints after each token for spec_keep.
int orc_forward_multi(const OrcModel* m, OrcState* st, const uint32_t* ids, int n, float* logits) {
  st->ck.clear();
  for (int i = 0; i < n; ++i) { int rc = orc_forward(m, st, ids + i, 1, logits + (size_t)i * m->c.vocab); if (rc) return rc; st->ck.push_back({st->conv, st->ssm, st->ple_hist}); }
  return 0;
}
// spec_keep, qwen4exp_gguf.rs:2495-2515
int orc_spec_keep(const OrcModel* m, OrcState* st, int t, int keep) {
  if (keep >= t || t < 2) return 0; if (keep < 1) keep = 1; if ((int)st->ck.size() < t) return -1;
  size_t n = st->tokens.size() - t + keep; st->tokens.resize(n);
  st->conv = st->ck[keep - 1].conv; st->ssm = st->ck[keep - 1].ssm; st->ple_hist = st->ck[keep - 1].ple_hist;      // ple_ck, :2417
  size_t row = (size_t)m->c.n_kv * m->c.hd; for (auto& k : st->k) k.resize(n * row); for (auto& v : st->v) v.resize(n * row);
  size_t ihd = m->c.idx_hd, ir = m->c.idx_ratio < 1 ? 1 : m->c.idx_ratio;       // :2509-2513
  for (auto& k : st->ik) if (!k.empty()) k.resize(n * ihd);
  for (auto& b : st->ib) if (!b.empty()) b.resize((n / ir) * ihd);
  return 0;
}
// spec::generate, greedy branch (spec.rs:156-267; accept loop :229-238, keep :249), drafts from a fixed stream:
// the round that starts with `produced` tokens emitted proposes draft_stream[produced .. produced+kk).
int orc_generate_greedy(const OrcModel* m, OrcState* st, const float* first_logits, int n_out, uint32_t* out, int n_draft, const uint32_t* draft_stream) {
  size_t V = m->c.vocab; std::vector<float> lg(first_logits, first_logits + V), ls; int produced = 0, rounds = 0;
  uint32_t pending = orc_argmax(lg.data(), V);
  for (;;) {
    out[produced++] = pending; if (produced >= n_out) break;
    int left = n_out - produced; int kk = std::min(std::min(n_draft, left - 1), 8); if (!draft_stream) kk = 0;
    if (kk <= 0) { if (orc_forward(m, st, &pending, 1, lg.data())) return -1; pending = orc_argmax(lg.data(), V); continue; }
    std::vector<uint32_t> toks{pending}; for (int j = 0; j < kk; ++j) toks.push_back(draft_stream[produced + j]);
    ls.resize(toks.size() * V); if (orc_forward_multi(m, st, toks.data(), (int)toks.size(), ls.data())) return -1;
    int acc = 0; bool have = false; uint32_t nx = 0;
    for (int i = 0; i < kk; ++i) { uint32_t tk = orc_argmax(ls.data() + (size_t)i * V, V); if (tk == toks[i + 1]) { ++acc; continue; } nx = tk; have = true; break; }
    if (!have) nx = orc_argmax(ls.data() + (size_t)kk * V, V);
    orc_spec_keep(m, st, (int)toks.size(), acc + 1); ++rounds;
    bool stop = false; for (int i = 0; i < acc; ++i) { out[produced++] = toks[i + 1]; if (produced >= n_out) { stop = true; break; } }
    if (stop) break; pending = nx;
  }
  return rounds;
}

}  // extern "C"

// ---------- MTP drafter, src/model/mtp.rs ------------------------------------------------------------------------------
struct OrcMtp {
  OrcMtpCfg c; OrcTensor t[ORC_MTP_SLOTS]; std::vector<uint32_t> ids; const OrcModel* main;
  std::vector<float> pre_e, pre_h, hca_norm, hcf_norm, mix_norm, qn, kn, sgate, rope_inv;
};
namespace {
const float* mtp_r_get(const OrcState* st, int pos) {      // mtp_r_get, :2286
  if (st->mtp_r.empty()) return nullptr; const int f = st->mtp_r.front().first; if (pos < f || pos - f >= (int)st->mtp_r.size()) return nullptr;
  const auto& e = st->mtp_r[pos - f]; return e.first == pos ? e.second.data() : nullptr;
}
// input, mtp.rs:151-160: t rows of main-model residuals r [t][hc*d] and token embeddings emb [t][d] -> [t][hc][d]
bool mtp_input(const OrcMtp* m, const float* r, const float* emb, int t, std::vector<float>& out) {
  const OrcCfg& c = m->main->c; const int d = c.d, hc = c.hc, w = hc * d, th = m->main->threads;
  std::vector<float> en((size_t)t * d), e2((size_t)t * d), hn((size_t)t * w);
  for (int ti = 0; ti < t; ++ti) rms(emb + (size_t)ti * d, m->pre_e.data(), c.eps, en.data() + (size_t)ti * d, d);
  if (!mm(&m->t[ORC_MTP_FC_E], en.data(), t, e2.data(), th)) return false;
  for (int ti = 0; ti < t; ++ti) rms(r + (size_t)ti * w, m->pre_h.data(), c.eps, hn.data() + (size_t)ti * w, w);
  out.assign((size_t)t * w, 0.0f);
  if (!mm(&m->t[ORC_MTP_FC_H], hn.data(), t * hc, out.data(), th)) return false;
  for (int ti = 0; ti < t; ++ti) for (int s = 0; s < hc; ++s) for (int i = 0; i < d; ++i) out[((size_t)ti * hc + s) * d + i] += e2[(size_t)ti * d + i];
  return true;
}
// kv_append, mtp.rs:163-176: K/V of t cells starting at pos0 appended (window kept); returns R after input, mixed, inject
bool mtp_kv_append(const OrcMtp* m, OrcState* st, const float* r, const float* emb, int t, int pos0, std::vector<float>& rr, std::vector<float>& mixed, std::vector<float>& inj) {
  const OrcCfg& c = m->main->c; const int d = c.d, hc = c.hc, row = c.n_kv * c.hd, th = m->main->threads;
  if (st->mtp_c0 + st->mtp_n != pos0) { st->mtp_c0 = pos0; st->mtp_n = 0; st->mtp_k.clear(); st->mtp_v.clear(); }
  if (!mtp_input(m, r, emb, t, rr)) return false;
  mixed.assign((size_t)t * d, 0.0f); inj.assign((size_t)t * hc, 0.0f);
  if (!hc_mix(d, hc, c.eps, m->hca_norm.data(), &m->t[ORC_MTP_HCA_DOWN], &m->t[ORC_MTP_HCA_INJECT], &m->t[ORC_MTP_HCA_UP], rr.data(), t, mixed.data(), inj.data(), th)) return false;
  std::vector<float> kf((size_t)t * row), vf((size_t)t * row), y(c.hd);
  if (!mm(&m->t[ORC_MTP_K], mixed.data(), t, kf.data(), th) || !mm(&m->t[ORC_MTP_V], mixed.data(), t, vf.data(), th)) return false;
  for (int ti = 0; ti < t; ++ti) for (int h = 0; h < c.n_kv; ++h) { float* kh = kf.data() + (size_t)ti * row + (size_t)h * c.hd; rms(kh, m->kn.data(), c.eps, y.data(), c.hd); memcpy(kh, y.data(), sizeof(float) * c.hd); rope(kh, pos0 + ti, c.n_rot, m->rope_inv.data()); }
  st->mtp_k.insert(st->mtp_k.end(), kf.begin(), kf.end()); st->mtp_v.insert(st->mtp_v.end(), vf.begin(), vf.end()); st->mtp_n += t;
  if (st->mtp_n > m->c.window) { const int drop = st->mtp_n - m->c.window; st->mtp_k.erase(st->mtp_k.begin(), st->mtp_k.begin() + (size_t)drop * row); st->mtp_v.erase(st->mtp_v.begin(), st->mtp_v.begin() + (size_t)drop * row); st->mtp_c0 += drop; st->mtp_n -= drop; }
  return true;
}
// step, mtp.rs:190-236: one draft step at cell pos; s = the final mixer's output for the head, rr = the drafter's residual.
// The routed experts go through the main model's MoE statement (chosen experts summed in ascending id; the reference's
// select_nth_unstable leaves their order open).
bool mtp_step(const OrcMtp* m, OrcState* st, const float* r, const float* emb, int pos, std::vector<float>& s_out, std::vector<float>& rr) {
  const OrcCfg& c = m->main->c; const int d = c.d, hc = c.hc, nh = c.n_head, hd = c.hd, row = c.n_kv * hd, grp = nh / c.n_kv, th = m->main->threads;
  std::vector<float> mx, inj;
  if (!mtp_kv_append(m, st, r, emb, 1, pos, rr, mx, inj)) return false;
  std::vector<float> qf((size_t)nh * 2 * hd), att((size_t)nh * hd, 0.0f), qh(hd), sc;
  if (!mm(&m->t[ORC_MTP_Q], mx.data(), 1, qf.data(), th)) return false;
  const int n = st->mtp_n; const float scale = 1.0f / sqrtf((float)hd);
  for (int h = 0; h < nh; ++h) {
    const size_t base = (size_t)h * 2 * hd; rms(qf.data() + base, m->qn.data(), c.eps, qh.data(), hd); rope(qh.data(), pos, c.n_rot, m->rope_inv.data());
    const int kvh = h / grp; sc.assign(n, 0.0f); float mxs = -INFINITY;
    for (int p = 0; p < n; ++p) { const float* k = st->mtp_k.data() + (size_t)p * row + (size_t)kvh * hd; float a = 0.0f; for (int i = 0; i < hd; ++i) a += qh[i] * k[i]; sc[p] = a * scale; mxs = fmaxf(mxs, sc[p]); }
    float sum = 0.0f; for (int p = 0; p < n; ++p) { sc[p] = expf(sc[p] - mxs); sum += sc[p]; }
    float* o = att.data() + (size_t)h * hd;
    for (int p = 0; p < n; ++p) { const float wgt = sc[p] / sum; const float* v = st->mtp_v.data() + (size_t)p * row + (size_t)kvh * hd; for (int i = 0; i < hd; ++i) o[i] += wgt * v[i]; }
    for (int i = 0; i < hd; ++i) o[i] *= sigm(qf[base + hd + i]);
  }
  std::vector<float> bo(d), m2(d), inj2(hc), y(d), dummy(hc);
  if (!mm(&m->t[ORC_MTP_O], att.data(), 1, bo.data(), th)) return false;
  hc_combine(d, hc, rr.data(), bo.data(), inj.data(), 1);
  if (!hc_mix(d, hc, c.eps, m->hcf_norm.data(), &m->t[ORC_MTP_HCF_DOWN], &m->t[ORC_MTP_HCF_INJECT], &m->t[ORC_MTP_HCF_UP], rr.data(), 1, m2.data(), inj2.data(), th)) return false;
  if (!moe_ffn(d, m->c.n_exp, m->c.top_k, m->c.ff, &m->t[ORC_MTP_ROUTER], &m->t[ORC_MTP_GATE_E], &m->t[ORC_MTP_UP_E], &m->t[ORC_MTP_DOWN_E], m->sgate.data(),
               &m->t[ORC_MTP_SH_GATE], &m->t[ORC_MTP_SH_UP], &m->t[ORC_MTP_SH_DOWN], m2.data(), 1, y.data(), nullptr, nullptr, th)) return false;
  hc_combine(d, hc, rr.data(), y.data(), inj2.data(), 1);
  s_out.assign(d, 0.0f);
  return hc_mix(d, hc, c.eps, m->mix_norm.data(), &m->t[ORC_MTP_MIX_DOWN], nullptr, &m->t[ORC_MTP_MIX_UP], rr.data(), 1, s_out.data(), dummy.data(), th);
}
bool embd_row(const OrcModel* m, uint32_t id, float* e) { const OrcTensor& embd = m->g[ORC_G_EMBD]; int qk, bs; if (!geom(embd.ty, &qk, &bs)) return false; return dequant(embd.ty, (const uint8_t*)embd.data + (size_t)id * ((size_t)m->c.d / qk * bs), m->c.d, e); }
}  // namespace

extern "C" {
OrcMtp* orc_mtp_create(const OrcModel* main, const OrcMtpCfg* cfg, const OrcTensor* tensors, const uint32_t* draft_ids) {
  OrcMtp* m = new OrcMtp(); m->c = *cfg; m->main = main; for (int i = 0; i < ORC_MTP_SLOTS; ++i) m->t[i] = tensors[i];
  m->ids.assign(draft_ids, draft_ids + cfg->n_draft_vocab);
  bool ok = to_vec(m->t[ORC_MTP_PRE_E], m->pre_e) && to_vec(m->t[ORC_MTP_PRE_H], m->pre_h) && to_vec(m->t[ORC_MTP_HCA_NORM], m->hca_norm) && to_vec(m->t[ORC_MTP_HCF_NORM], m->hcf_norm) &&
            to_vec(m->t[ORC_MTP_MIX_NORM], m->mix_norm) && to_vec(m->t[ORC_MTP_QN], m->qn) && to_vec(m->t[ORC_MTP_KN], m->kn) && to_vec(m->t[ORC_MTP_SH_GATE_INP], m->sgate);
  if (!ok || (int)m->t[ORC_MTP_HEAD].rows != cfg->n_draft_vocab) { delete m; return nullptr; }
  m->rope_inv.resize(main->c.n_rot / 2); orc_rope_inv(main->c.n_rot, main->c.rope_base, m->rope_inv.data());      // mtp.rs:111: the unscaled table
  return m;
}
void orc_mtp_destroy(OrcMtp* m) { delete m; }
void orc_state_attach_mtp(OrcState* st, const OrcMtp* m) { st->mtp_window = m->c.window; }
const float* orc_mtp_r(const OrcState* st, int pos) { return mtp_r_get(st, pos); }
int orc_mtp_kv(const OrcState* st, int* c0, const float** k, const float** v) { *c0 = st->mtp_c0; *k = st->mtp_k.data(); *v = st->mtp_v.data(); return st->mtp_n; }

int orc_mtp_draft(const OrcMtp* m, const OrcModel* main, OrcState* st, uint32_t pending, int k, float min_p, uint32_t* ids, float* probs) {
  const OrcCfg& c = main->c; const int n = (int)st->tokens.size(), d = c.d, w = c.hc * d, row = c.n_kv * c.hd;
  if (n == 0 || k <= 0) return 0;
  // kv.truncate(n - 1)
  if (n - 1 < st->mtp_c0 + st->mtp_n) { const int keep = std::max(0, n - 1 - st->mtp_c0); st->mtp_n = keep; st->mtp_k.resize((size_t)keep * row); st->mtp_v.resize((size_t)keep * row); }
  // catch-up over the cells whose residual is known and whose token is committed, :2194-2217
  const int first = st->mtp_r.empty() ? n : st->mtp_r.front().first;
  const int end = st->mtp_c0 + st->mtp_n;
  const int lo = (st->mtp_n > 0 && end >= first) ? end : std::max(first, std::max(0, (n - 1) - m->c.window));
  if (lo < n - 1) {
    const int nc = n - 1 - lo; std::vector<float> rs((size_t)nc * w), es((size_t)nc * d); bool ok = true;
    for (int j = 0; j < nc; ++j) { const float* r = mtp_r_get(st, lo + j); if (!r) { ok = false; break; } memcpy(&rs[(size_t)j * w], r, sizeof(float) * w); if (!embd_row(main, st->tokens[lo + j + 1], &es[(size_t)j * d])) return -1; }
    if (ok) { std::vector<float> rr, mx, inj; for (int c0 = 0; c0 < nc; c0 += 64) { const int nn = std::min(64, nc - c0); if (!mtp_kv_append(m, st, &rs[(size_t)c0 * w], &es[(size_t)c0 * d], nn, lo + c0, rr, mx, inj)) return -1; } }
    else { st->mtp_c0 = 0; st->mtp_n = 0; st->mtp_k.clear(); st->mtp_v.clear(); }
  }
  const float* r0 = mtp_r_get(st, n - 1); if (!r0) return 0;
  std::vector<float> r(r0, r0 + w), e(d), s, r2, lg(m->c.n_draft_vocab); uint32_t tok = pending; int out = 0;
  for (int j = 0; j < k; ++j) {
    if (!embd_row(main, tok, e.data())) return -1;
    if (!mtp_step(m, st, r.data(), e.data(), n - 1 + j, s, r2)) return -1;
    if (!mm(&m->t[ORC_MTP_HEAD], s.data(), 1, lg.data(), main->threads)) return -1;
    size_t bi = 0; float bv = -INFINITY; for (size_t i = 0; i < lg.size(); ++i) if (lg[i] > bv) { bv = lg[i]; bi = i; }      // best, mtp.rs:424-427
    float z = 0.0f; for (float v : lg) z += expf(v - bv); const float p = 1.0f / z;
    if (j > 0 && p < min_p) break;                                                        // draft_gate with the policy off
    ids[out] = m->ids[bi]; probs[out] = p; ++out; r = r2; tok = ids[out - 1];
  }
  // kv.truncate(n)
  if (n < st->mtp_c0 + st->mtp_n) { const int keep = std::max(0, n - st->mtp_c0); st->mtp_n = keep; st->mtp_k.resize((size_t)keep * row); st->mtp_v.resize((size_t)keep * row); }
  return out;
}

int orc_generate_greedy_mtp(const OrcModel* m, const OrcMtp* mtp, OrcState* st, const float* first_logits, int n_out, uint32_t* out, int k, float min_p, int* drafted, int* accepted) {
  const size_t V = m->c.vocab; int produced = 0, nd = 0, na = 0; uint32_t pending = orc_argmax(first_logits, V); std::vector<float> ls;
  for (;;) {
    out[produced++] = pending; if (produced >= n_out) break;
    const int left = n_out - produced; const int kk = std::min(k, left - 1);
    uint32_t dr[8]; float dp[8]; int got = kk > 0 ? orc_mtp_draft(mtp, m, st, pending, std::min(kk, 7), min_p, dr, dp) : 0; if (got < 0) return -1;
    std::vector<uint32_t> toks{pending}; for (int j = 0; j < got; ++j) toks.push_back(dr[j]);
    ls.resize(toks.size() * V); if (orc_forward_multi(m, st, toks.data(), (int)toks.size(), ls.data())) return -1;
    int acc = 0; bool have = false; uint32_t nx = 0;
    for (int i = 0; i < got; ++i) { const uint32_t tk = orc_argmax(&ls[(size_t)i * V], V); if (tk == toks[i + 1]) { ++acc; continue; } nx = tk; have = true; break; }
    if (!have) nx = orc_argmax(&ls[(size_t)got * V], V);
    orc_spec_keep(m, st, (int)toks.size(), acc + 1); nd += got; na += acc;
    bool stop = false; for (int i = 0; i < acc; ++i) { out[produced++] = toks[i + 1]; if (produced >= n_out) { stop = true; break; } }
    if (stop) break;
    pending = nx;
  }
  if (drafted) *drafted = nd; if (accepted) *accepted = na; return 0;
}
}  // extern "C"
