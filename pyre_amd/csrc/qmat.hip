// Quantized matrix operator: GGUF blocks -> lane=row planes (repack), bit-exact dequant export, dequant-GEMV.
// Drop-in for QMat / QMat::matmul of the reference (src/model/gguf_q.rs:201-247).
#include "formats.h"
#include <stdlib.h>
PYRE_TS_DECL(qmat_ts) PYRE_TS_EXPORT(qmat_ts, pyre_debug_ts_qmat)

// ---- repack: raw GGUF rows -> planes --------------------------------------------------------------------------------
// One thread per (padded row, unit).  Rows beyond m.rows are written as zeros (they decode to 0 and are never stored).
__global__ void k_repack(QMatDev m, const uint8_t* __restrict__ raw, size_t row_bytes, uint8_t* p0, uint8_t* p1, uint8_t* p2, uint8_t* p3, uint8_t* pb, const uint32_t* __restrict__ g3, const uint16_t* __restrict__ cb) {
  size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t total = (size_t)m.tiles * 64 * m.U;
  if (gid >= total) return;
  int ku = (int)(gid % m.U); size_t r = gid / m.U; int tile = (int)(r / 64), lane = (int)(r % 64);
  bool live = r < (size_t)m.rows;
  const uint8_t* row = raw + r * row_bytes;
  FmtGeom g = qmat_geom(m.fmt, m.ty);
  size_t e = ((size_t)tile * m.U + ku) * 64 + lane;              // entry index in per-unit planes
  uint8_t* v = p0 + ((size_t)tile * m.U + ku) * g.V * 64 * 16;     // chunk c of this lane at v + (c*64 + lane)*16
  auto put_vec = [&](int chunk, const uint8_t* src) { uint8_t* d = v + ((size_t)chunk * 64 + lane) * 16; for (int i = 0; i < 16; ++i) d[i] = live ? src[i] : 0; };
  switch (m.fmt) {
    case FMT_F32: for (int c = 0; c < 16; ++c) put_vec(c, row + (size_t)ku * 256 + 16 * c); break;
    case FMT_F16: case FMT_BF16: for (int c = 0; c < 8; ++c) put_vec(c, row + (size_t)ku * 128 + 16 * c); break;
    case FMT_Q8_0: {
      const uint8_t* b0 = row + (size_t)(2 * ku) * 34; const uint8_t* b1 = b0 + 34;
      put_vec(0, b0 + 2); put_vec(1, b0 + 18); put_vec(2, b1 + 2); put_vec(3, b1 + 18);
      uint8_t* d = p1 + e * 4; d[0] = live ? b0[0] : 0; d[1] = live ? b0[1] : 0; d[2] = live ? b1[0] : 0; d[3] = live ? b1[1] : 0;
    } break;
    case FMT_Q4_K: {
      const uint8_t* b = row + (size_t)(ku >> 2) * 144; int j = ku & 3;
      put_vec(0, b + 16 + 32 * j); put_vec(1, b + 32 + 32 * j);
      if (j == 0) { uint8_t* d = pb + (((size_t)tile * (m.U >> 2) + (ku >> 2)) * 64 + lane) * 16; for (int i = 0; i < 16; ++i) d[i] = live ? b[i] : 0; }
    } break;
    case FMT_IQ2_XS: {   // IQ2_XS / IQ2_XXS / IQ2_S (gguf_q.rs:122-135): grid and sign lookups resolved here, once; cb holds 2-bit magnitude indices per grid byte
      uint32_t M[4] = {0, 0, 0, 0}, S[2] = {0, 0}; uint32_t scb = 0; int j = ku & 3;
      auto ks = [](uint32_t i) { return i | ((__popc(i) & 1u) << 7); };
      auto put = [&](int ev, uint32_t idx, uint32_t neg) { int gq = ev >> 4, e16 = ev & 15, r = e16 >> 2, bb = e16 & 3; M[gq] |= (idx & 3) << (8 * bb + 2 * r); S[gq >> 1] |= (neg & 1) << (8 * bb + r + 4 * (gq & 1)); };
      const uint8_t* b = row; uint32_t dbits = 0;
      if (live) {
        if (m.ty == PYRE_IQ2_XS) {
          b = row + (size_t)(ku >> 2) * 74; dbits = b[0] | (b[1] << 8); scb = b[66 + 2 * j] | (b[67 + 2 * j] << 8);
          for (int l = 0; l < 8; ++l) { uint32_t q = b[2 + 16 * j + 2 * l] | (b[3 + 16 * j + 2 * l] << 8), gcode = cb[1536 + (q & 511)], sg = ks(q >> 9);
            for (int jj = 0; jj < 8; ++jj) put(8 * l + jj, (gcode >> (2 * jj)) & 3, (sg >> jj) & 1); }
        } else if (m.ty == PYRE_IQ2_XXS) {
          b = row + (size_t)(ku >> 2) * 66; dbits = b[0] | (b[1] << 8);
          for (int c = 0; c < 2; ++c) { int ib = 2 * j + c; const uint8_t* a0 = b + 2 + 8 * ib; uint32_t a1 = a0[4] | (a0[5] << 8) | (a0[6] << 16) | ((uint32_t)a0[7] << 24), nib = a1 >> 28;
            scb |= (nib | (nib << 4)) << (8 * c);
            for (int l = 0; l < 4; ++l) { uint32_t gcode = cb[a0[l]], sg = ks((a1 >> (7 * l)) & 127); for (int jj = 0; jj < 8; ++jj) put(32 * c + 8 * l + jj, (gcode >> (2 * jj)) & 3, (sg >> jj) & 1); } }
        } else {           // IQ2_S
          b = row + (size_t)(ku >> 2) * 82; dbits = b[0] | (b[1] << 8);
          for (int c = 0; c < 2; ++c) { int ib = 2 * j + c; uint32_t qh = b[66 + ib]; scb |= (uint32_t)b[74 + ib] << (8 * c);
            for (int l = 0; l < 4; ++l) { uint32_t gcode = cb[256 + (b[2 + 4 * ib + l] | ((qh << (8 - 2 * l)) & 0x300))], sg = b[34 + 4 * ib + l];
              for (int jj = 0; jj < 8; ++jj) put(32 * c + 8 * l + jj, (gcode >> (2 * jj)) & 3, (sg >> jj) & 1); } }
        }
      }
      uint32_t* dst = (uint32_t*)(v + (size_t)lane * 16); for (int i = 0; i < 4; ++i) dst[i] = M[i];
      uint8_t* d1 = p1 + e * 2; d1[0] = (uint8_t)(scb & 0xFF); d1[1] = (uint8_t)(scb >> 8);
      uint32_t* d2 = (uint32_t*)(p2 + e * 8); d2[0] = S[0]; d2[1] = S[1];
      if (j == 0) { uint8_t* dd = pb + (((size_t)tile * (m.U >> 2) + (ku >> 2)) * 64 + lane) * 2; dd[0] = (uint8_t)(dbits & 0xFF); dd[1] = (uint8_t)(dbits >> 8); }
    } break;
    case FMT_C4: case FMT_C8: {
      // cb: compact codebooks [iq2xxs 256 | iq2s 1024 | iq3xxs 256 | iq2xs 512 | iq1s 2048]; code(e) and scale(e / 16) of the unit's 64 values e
      uint32_t words[16]; float sc[4], off[4];
      for (int i = 0; i < 16; ++i) words[i] = 0;
      for (int i = 0; i < 4; ++i) { sc[i] = 0.0f; off[i] = 0.0f; }
      auto h2 = [](const uint8_t* q) { return __half2float(__ushort_as_half((unsigned short)(q[0] | (q[1] << 8)))); };
      auto put4 = [&](int e, uint32_t code) { words[e >> 3] |= (code & 0xF) << (4 * (e & 7)); };
      auto put8b = [&](int e, int q) { words[e >> 2] |= (uint32_t)(q & 0xFF) << (8 * (e & 3)); };
      auto ks = [](uint32_t i) { return i | ((__popc(i) & 1u) << 7); };
      if (live) switch (m.ty) {          // padding rows lie past the end of the raw buffer: never read them
        case PYRE_Q4_0: case PYRE_IQ4_NL:                              // gguf_q.rs:74-75, 82-83: unit = two 32-value blocks
          for (int h = 0; h < 2; ++h) { const uint8_t* b = row + (size_t)(2 * ku + h) * 18; sc[2 * h] = sc[2 * h + 1] = h2(b);
            for (int j = 0; j < 16; ++j) { put4(32 * h + j, b[2 + j] & 0xF); put4(32 * h + 16 + j, b[2 + j] >> 4); } }
          break;
        case PYRE_Q5_0:                                                // gguf_q.rs:76-78
          for (int h = 0; h < 2; ++h) { const uint8_t* b = row + (size_t)(2 * ku + h) * 22; sc[2 * h] = sc[2 * h + 1] = h2(b);
            uint32_t qh = b[2] | (b[3] << 8) | (b[4] << 16) | ((uint32_t)b[5] << 24);
            for (int j = 0; j < 16; ++j) { put8b(32 * h + j, (int)((b[6 + j] & 0xF) | (((qh >> j) << 4) & 0x10)) - 16); put8b(32 * h + 16 + j, (int)((b[6 + j] >> 4) | ((qh >> (j + 12)) & 0x10)) - 16); } }
          break;
        case PYRE_IQ4_XS: {                                            // gguf_q.rs:84-89
          const uint8_t* b = row + (size_t)(ku >> 2) * 136; float d = h2(b); uint32_t sh = b[2] | (b[3] << 8);
          for (int c = 0; c < 2; ++c) { int ib = 2 * (ku & 3) + c; int ls = (int)((b[4 + ib / 2] >> (4 * (ib % 2))) & 0xF) | (int)(((sh >> (2 * ib)) & 3) << 4);
            sc[2 * c] = sc[2 * c + 1] = d * (float)(ls - 32); const uint8_t* q = b + 8 + 16 * ib;
            for (int j = 0; j < 16; ++j) { put4(32 * c + j, q[j] & 0xF); put4(32 * c + 16 + j, q[j] >> 4); } }
        } break;
        case PYRE_Q6_K: {                                              // gguf_q.rs:114-121
          const uint8_t* b = row + (size_t)(ku >> 2) * 210; float d = h2(b + 208); int n = (ku & 3) >> 1;
          for (int c = 0; c < 2; ++c) { int qd = 2 * (ku & 1) + c;      // quarter of the 128-value half
            for (int l = 0; l < 32; ++l) { uint32_t qlb = b[64 * n + l + ((qd & 1) ? 32 : 0)], nib = qd < 2 ? (qlb & 0xF) : (qlb >> 4), hi2 = (b[128 + 32 * n + l] >> (2 * qd)) & 3;
              put8b(32 * c + l, (int)(nib | (hi2 << 4)) - 32); }
            for (int g = 0; g < 2; ++g) sc[2 * c + g] = d * (float)(int)(int8_t)b[192 + 8 * n + 2 * qd + g]; }
        } break;
        case PYRE_Q2_0: {                                              // gguf_q.rs:80-81, lut q2 :50: one 64-value block per unit
          const uint8_t* b = row + (size_t)ku * 18; const float d = h2(b);
          for (int i = 0; i < 4; ++i) sc[i] = d;
          for (int k = 0; k < 16; ++k) for (int j = 0; j < 4; ++j) put4(4 * k + j, (b[2 + k] >> (2 * j)) & 3);
        } break;
        case PYRE_Q3_K: {                                              // gguf_q.rs:90-102
          const uint8_t* b = row + (size_t)(ku >> 2) * 110; const uint8_t* hm = b; const uint8_t* s12 = b + 96; const float d = h2(b + 108);
          auto a = [&](int k) { return (uint32_t)s12[4 * k] | ((uint32_t)s12[4 * k + 1] << 8) | ((uint32_t)s12[4 * k + 2] << 16) | ((uint32_t)s12[4 * k + 3] << 24); };
          const uint32_t a0 = a(0), a1 = a(1), tmp = a(2), k1 = 0x03030303u, k2 = 0x0f0f0f0fu;
          const uint32_t aux[4] = {(a0 & k2) | ((tmp & k1) << 4), (a1 & k2) | (((tmp >> 2) & k1) << 4), ((a0 >> 4) & k2) | (((tmp >> 4) & k1) << 4), ((a1 >> 4) & k2) | (((tmp >> 6) & k1) << 4)};
          const int u = ku & 3, n = u >> 1; const uint8_t* q = b + 32 + 32 * n;
          for (int g4 = 0; g4 < 4; ++g4) {                             // 16 values: j = 2*(u&1) + g4/2, half = g4&1
            const int j = 2 * (u & 1) + (g4 >> 1), half = g4 & 1, is = 8 * n + 2 * j + half, shift = 2 * j; const uint32_t mbit = 1u << (4 * n + j);
            sc[g4] = d * (float)((int)(int8_t)((aux[is >> 2] >> (8 * (is & 3))) & 0xFF) - 32);
            for (int l = 0; l < 16; ++l) { const int o = l + 16 * half; put4(16 * g4 + l, ((q[o] >> shift) & 3) | ((hm[o] & mbit) ? 4u : 0u)); }
          }
        } break;
        case PYRE_IQ1_M: {                                             // gguf_q.rs:152-165
          const uint8_t* b = row + (size_t)(ku >> 2) * 56; const uint8_t* scb = b + 48;
          const uint32_t s16[4] = {(uint32_t)scb[0] | (scb[1] << 8), (uint32_t)scb[2] | (scb[3] << 8), (uint32_t)scb[4] | (scb[5] << 8), (uint32_t)scb[6] | (scb[7] << 8)};
          const uint32_t su = (s16[0] >> 12) | ((s16[1] >> 8) & 0x00f0) | ((s16[2] >> 4) & 0x0f00) | (s16[3] & 0xf000);
          const float d = __half2float(__ushort_as_half((unsigned short)su));
          for (int c = 0; c < 2; ++c) { const int ib = 2 * (ku & 3) + c; const uint8_t* qs = b + 4 * ib; const uint8_t* qh = b + 32 + 2 * ib;
            const float dl1 = d * (float)(2 * ((s16[ib / 2] >> (6 * (ib % 2))) & 7) + 1), dl2 = d * (float)(2 * ((s16[ib / 2] >> (6 * (ib % 2) + 3)) & 7) + 1);
            sc[2 * c] = dl1 * 0.125f; sc[2 * c + 1] = dl2 * 0.125f;
            const uint32_t idx[4] = {(uint32_t)qs[0] | (((uint32_t)qh[0] << 8) & 0x700), (uint32_t)qs[1] | (((uint32_t)qh[0] << 4) & 0x700), (uint32_t)qs[2] | (((uint32_t)qh[1] << 8) & 0x700), (uint32_t)qs[3] | (((uint32_t)qh[1] << 4) & 0x700)};
            const uint32_t neg[4] = {(uint32_t)(qh[0] >> 3) & 1, (uint32_t)(qh[0] >> 7) & 1, (uint32_t)(qh[1] >> 3) & 1, (uint32_t)(qh[1] >> 7) & 1};
            for (int l = 0; l < 4; ++l) { const uint32_t gc = cb[2048 + idx[l]]; for (int j = 0; j < 8; ++j) put4(32 * c + 8 * l + j, ((gc >> (2 * j)) & 3) | (neg[l] << 2)); } }
        } break;
        case PYRE_Q5_K: {                                              // gguf_q.rs:108-113
          const uint8_t* b = row + (size_t)(ku >> 2) * 176; const float d = h2(b), mn = h2(b + 2); const int j = ku & 3;
          auto w32 = [&](int k) { return (uint32_t)b[4 + 4 * k] | ((uint32_t)b[5 + 4 * k] << 8) | ((uint32_t)b[6 + 4 * k] << 16) | ((uint32_t)b[7 + 4 * k] << 24); };
          uint32_t s1, m1, s2, m2; scale_min_k4(2 * j, w32(0), w32(1), w32(2), s1, m1); scale_min_k4(2 * j + 1, w32(0), w32(1), w32(2), s2, m2);
          sc[0] = sc[1] = d * (float)s1; off[0] = off[1] = mn * (float)m1; sc[2] = sc[3] = d * (float)s2; off[2] = off[3] = mn * (float)m2;
          const uint8_t* qh = b + 16; const uint8_t* ql = b + 48 + 32 * j; const uint32_t u1 = 1u << (2 * j), u2 = 2u << (2 * j);
          for (int l = 0; l < 32; ++l) { put8b(l, (int)((ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0))); put8b(32 + l, (int)((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0))); }
        } break;
        case PYRE_IQ3_XXS: {                                           // gguf_q.rs:136-140
          const uint8_t* b = row + (size_t)(ku >> 2) * 98; float d = h2(b);
          for (int c = 0; c < 2; ++c) { int ib = 2 * (ku & 3) + c; const uint8_t* ss = b + 66 + 4 * ib; uint32_t a = ss[0] | (ss[1] << 8) | (ss[2] << 16) | ((uint32_t)ss[3] << 24);
            sc[2 * c] = sc[2 * c + 1] = d * (0.5f + (float)(a >> 28)) * 0.5f;
            for (int l = 0; l < 4; ++l) { uint32_t g1 = cb[1280 + b[2 + 8 * ib + 2 * l]], g2 = cb[1280 + b[2 + 8 * ib + 2 * l + 1]], sg = ks((a >> (7 * l)) & 127);
              for (int j = 0; j < 4; ++j) { put4(32 * c + 8 * l + j, ((g1 >> (3 * j)) & 7) | (((sg >> j) & 1) << 3)); put4(32 * c + 8 * l + 4 + j, ((g2 >> (3 * j)) & 7) | (((sg >> (4 + j)) & 1) << 3)); } } }
        } break;
        default: break;
      }
      for (int c = 0; c < g.V; ++c) { uint32_t* dst = (uint32_t*)(v + ((size_t)c * 64 + lane) * 16); for (int i = 0; i < 4; ++i) dst[i] = words[4 * c + i]; }
      float* sd = (float*)(p1 + e * 16); for (int i = 0; i < 4; ++i) sd[i] = sc[i];
      if (g.e2 == 16) { float* od = (float*)(p2 + e * 16); for (int i = 0; i < 4; ++i) od[i] = off[i]; }
    } break;
    default: {   // IQ3_S: codebook lookups and signs are resolved here, once (gguf_q.rs:141-151), into 4-bit codes
      const uint8_t* b = row + (size_t)(ku >> 2) * 110; int j = ku & 3;
      for (int c = 0; c < 2; ++c) {              // chunk c = sub-block 2j + c of the super-block: 32 values
        int ib = 2 * j + c; uint32_t words[4] = {0, 0, 0, 0}; uint32_t h = live ? b[66 + ib] : 0;
        for (int l = 0; live && l < 4; ++l) {      // padding rows lie past the end of the raw buffer: never read them
          uint32_t gA = g3[b[2 + 8 * ib + 2 * l] | ((h << (8 - 2 * l)) & 256)], gB = g3[b[2 + 8 * ib + 2 * l + 1] | ((h << (7 - 2 * l)) & 256)];
          uint32_t sg = b[74 + 4 * ib + l], wd = 0;
          for (int jj = 0; jj < 4; ++jj) { wd |= iq3s_code((gA >> (8 * jj)) & 0xFF, (sg >> jj) & 1) << (4 * jj); wd |= iq3s_code((gB >> (8 * jj)) & 0xFF, (sg >> (4 + jj)) & 1) << (16 + 4 * jj); }
          words[l] = wd;
        }
        uint32_t* dst = (uint32_t*)(v + ((size_t)c * 64 + lane) * 16); for (int i = 0; i < 4; ++i) dst[i] = words[i];
      }
      p3[e] = live ? b[106 + j] : 0;
      if (j == 0) { uint8_t* dd = pb + (((size_t)tile * (m.U >> 2) + (ku >> 2)) * 64 + lane) * 2; dd[0] = live ? b[0] : 0; dd[1] = live ? b[1] : 0; }
    }
  }
}

// IQ3_S into the matrix-core layout (QMatDev::mq / mh): one thread per (row of the padded row groups, super-block).
__global__ __launch_bounds__(256) void k_repack_m(int rows, int rows_pad, int SB, const uint8_t* __restrict__ raw, size_t row_bytes, uint32_t* __restrict__ mq, uint2* __restrict__ mh, const uint32_t* __restrict__ g3) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; if (idx >= (size_t)rows_pad * SB) return;
  const int row = (int)(idx / SB), sb = (int)(idx % SB); const bool live = row < rows;      // padding rows lie past the end of the raw buffer: never read them
  const size_t rg = (size_t)(row >> 4); const int j = row & 15; const size_t K128 = (size_t)SB * 2;
  const uint8_t* b = raw + (size_t)row * row_bytes + (size_t)sb * 110;
  for (int ib = 0; ib < 8; ++ib) {               // sub-block ib: 32 values = step ib & 3 of 128-column chunk 2 sb + ib / 4
    const uint32_t h = live ? b[66 + ib] : 0;
    for (int l = 0; l < 4; ++l) {                // eight consecutive values = the share of lane group l
      uint32_t wd = 0;
      if (live) {
        const uint32_t gA = g3[b[2 + 8 * ib + 2 * l] | ((h << (8 - 2 * l)) & 256)], gB = g3[b[2 + 8 * ib + 2 * l + 1] | ((h << (7 - 2 * l)) & 256)], sg = b[74 + 4 * ib + l];
        for (int e = 0; e < 8; ++e) { const uint32_t gb = ((e < 4 ? gA : gB) >> (8 * (e & 3))) & 0xFF; wd |= iq3s_code(gb, (sg >> e) & 1) << (4 * ((e >> 1) + 4 * (e & 1))); }
      }
      mq[(mq_slot(rg, 2 * sb + (ib >> 2), (int)K128) + l * 16 + j) * 4 + (ib & 3)] = wd;
    }
  }
  uint2 hd{0u, 0u};
  if (live) {       // sub-block i's scale at field i/2 + 4*(i&1) of the scale word, the order the codes of a step are in
    hd.x = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
    for (int i = 0; i < 8; ++i) hd.y |= (uint32_t)((b[106 + (i >> 1)] >> (4 * (i & 1))) & 0xF) << (4 * ((i >> 1) + 4 * (i & 1)));
  }
  mh[mh_slot(rg, sb, SB) + j] = hd;
}

// ---- bit-exact dequant export -----------------------------------------------------------------------------------------
// grid (U, tiles), 64 threads: lane l decodes unit ku of row tile*64+l, the tile is transposed through LDS so that
// each row's 64 values leave as one contiguous 256-byte store.
template <int FMT> __global__ __launch_bounds__(64) void k_dequant(QMatDev m, const uint64_t* g2, float* __restrict__ out) {
  __shared__ float tile_buf[64][65];
  int ku = blockIdx.x, tile = blockIdx.y, lane = threadIdx.x;
  float y[64];
  decode_exact<FMT>(m, g2, tile, ku, lane, y);
  for (int i = 0; i < 64; ++i) tile_buf[lane][i] = y[i];
  __syncthreads();
  for (int r = 0; r < 64; ++r) { size_t row = (size_t)tile * 64 + r; if (row < (size_t)m.rows) out[row * m.cols + (size_t)ku * 64 + lane] = tile_buf[r][lane]; }
}

// rows by index (embedding lookup, QMat::row): grid (ceil(U/64), n), 64 threads, thread = unit
template <int FMT> __global__ __launch_bounds__(64) void k_rows(QMatDev m, const uint64_t* g2, const uint32_t* __restrict__ idx, float* __restrict__ out, int out_stride) {
  int ku = blockIdx.x * 64 + threadIdx.x; if (ku >= m.U) return;
  uint32_t r = idx[blockIdx.y]; if (r >= (uint32_t)m.rows) return;
  float y[64];
  decode_exact<FMT>(m, g2, (int)(r >> 6), ku, (int)(r & 63), y);
  float* o = out + (size_t)blockIdx.y * out_stride + (size_t)ku * 64;
  for (int i = 0; i < 64; ++i) o[i] = y[i];
}

// ---- dequant-GEMV -----------------------------------------------------------------------------------------------------
// grid (tiles, ksplit), NW waves.  Wave w of K-slice ks walks units [(ks*NW+w)*upw, +upw).  Lane l owns row tile*64+l:
// weights come from coalesced per-lane loads, activations from wave-uniform (scalar) loads, so there is no cross-lane
// reduction at all; the NW partial sums meet in LDS and are added in wave order.
//   ksplit == 1: y[t*rows + row] = sum.
//   ksplit  > 1: y is a partial buffer, y[(ks*T + t)*tiles*64 + row] = slice sum; the consumer kernel adds the slices in
//                slice order (no in-kernel cross-workgroup reduction: a device-scope fence per workgroup costs about a
//                microsecond of serialized L2 write-back per XCD on this part).
//   best != nullptr (T == 1, ksplit == 1): best[2*tile] = bits of the tile's maximum, best[2*tile+1] = its first row.
template <int FMT, int T, int NW>
__global__ __launch_bounds__(NW * 64) void k_gemv(QMatDev m, const float* __restrict__ x, float* __restrict__ y, int upw,
                                                  GemvEpi ep, const uint2* __restrict__ g2) {
  const uint2* lds2 = nullptr;          // no format needs a codebook in shared memory any more
  PYRE_TS_VARS PYRE_TS(0);
  __shared__ float red[NW][T][64];
  const int tile = blockIdx.x, ks = blockIdx.y, ksplit = gridDim.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  // conv epilogue: wave 0 fetches its rows' taps and state first, so the loads overlap the dot products
  float cw[8], chist[8]; const bool conv_row = ep.co != nullptr && wave == 0 && tile * 64 + lane < ep.ch;
  if (conv_row) {
    const size_t row = (size_t)tile * 64 + lane;
#pragma unroll
    for (int k = 0; k < 8; ++k) { cw[k] = k < ep.kk ? ep.conv_w[row * ep.kk + k] : 0.0f; chist[k] = k < ep.kk - 1 ? ep.conv_in[(size_t)k * ep.ch + row] : 0.0f; }
  }
  const int k0 = (ks * NW + wave) * upw; const int k1 = min(m.U, k0 + upw);
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.0f;
  if constexpr (T == 1) {
    // One token: a unit's 64 activations reach all lanes as scalar loads, and every multiply-add takes its activation
    // straight from a scalar register.  (Copying the K range into shared memory first, all loads in flight at once, was
    // measured slower: 4.2 against 2.3 us for a 2048-column projection -- 64 shared-memory reads per unit and vector
    // operands cost more than the units' scalar round trips save.)
    for (int ku = k0; ku < k1; ++ku) unit_dot<FMT, T>(m, lds2, tile, ku, lane, x + (size_t)ku * 64, m.cols, acc);
  } else {
    // Several tokens: T x 64 activations per unit do not fit the scalar registers, and scalar loads in pieces cost one
    // memory round trip per piece.  Each wave stages the activations of two units at a time in its own slice of shared
    // memory ([token][unit][64], vector loads issued together with the units' weights) and takes them from there; a
    // wave's shared-memory operations execute in order, so no workgroup barrier is involved.  The arithmetic per token
    // is the single-token sequence.
    extern __shared__ __align__(16) float xsm[];
    float* xw = xsm + (size_t)wave * (2 * 64 * T);
    for (int ku = k0; ku < k1; ku += 2) {
      const bool two = ku + 1 < k1;
      UnitRaw<FMT> r0 = unit_load<FMT>(m, tile, ku, lane), r1 = unit_load<FMT>(m, tile, two ? ku + 1 : ku, lane);
      float xa[T], xb[T];
#pragma unroll
      for (int t = 0; t < T; ++t) { xa[t] = x[(size_t)t * m.cols + (size_t)ku * 64 + lane]; xb[t] = x[(size_t)t * m.cols + (size_t)(two ? ku + 1 : ku) * 64 + lane]; }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < T; ++t) { xw[(t * 2 + 0) * 64 + lane] = xa[t]; xw[(t * 2 + 1) * 64 + lane] = xb[t]; }
      __builtin_amdgcn_wave_barrier();
      unit_fma<FMT, T>(m, r0, ku, lds2, lane, xw, 128, acc);
      if (two) unit_fma<FMT, T>(m, r1, ku + 1, lds2, lane, xw + 64, 128, acc);
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t) red[wave][t][lane] = acc[t];
  PYRE_TS(1);
  lds_barrier(); PYRE_TS(2);
  const size_t r64 = (size_t)m.tiles * 64;
  for (int i = threadIdx.x; i < T * 64; i += NW * 64) {
    int t = i >> 6, l = i & 63; float s = red[0][t][l];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][t][l];
    size_t row = (size_t)tile * 64 + l;
    if (ksplit == 1) { if (row < (size_t)m.rows) y[(size_t)t * m.rows + row] = s; }
    else y[((size_t)ks * T + t) * r64 + row] = s;
    if (T == 1 && ep.best != nullptr) {       // threads 0..63 = wave 0: first maximum of the tile (sampler::argmax order)
      float bv = row < (size_t)m.rows ? s : -INFINITY; uint32_t bi = (uint32_t)row;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) { float ov = __shfl_xor(bv, o); uint32_t oi = __shfl_xor(bi, o); if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; } }
      if (l == 0) { ep.best[2 * tile] = __float_as_uint(bv); ep.best[2 * tile + 1] = bi; }
    }
  }
  if (conv_row) {      // linear_core's conv1d + SiLU for this row, tokens in order (qwen4exp_gguf.rs:1643-1647)
    const size_t row = (size_t)tile * 64 + lane;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float cur = red[0][t][lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) cur += red[w][t][lane];
      float o = 0.0f;
#pragma unroll
      for (int k = 0; k < 8; ++k) if (k == ep.kk - 1) o = cw[k] * cur;
#pragma unroll
      for (int k = 0; k < 7; ++k) if (k < ep.kk - 1) o += cw[k] * chist[k];
      ep.co[(size_t)t * ep.ch + row] = o * (1.0f / (1.0f + expf(-o)));
#pragma unroll
      for (int k = 0; k < 7; ++k) if (k + 1 < ep.kk - 1) chist[k] = chist[k + 1];
#pragma unroll
      for (int k = 0; k < 7; ++k) if (k == ep.kk - 2) chist[k] = cur;
    }
#pragma unroll
    for (int k = 0; k < 7; ++k) if (k < ep.kk - 1) ep.conv_out[(size_t)k * ep.ch + row] = chist[k];
  }
  PYRE_TS(3); PYRE_TS_FLUSH(qmat_ts, (NW == 16 ? 0 : (gridDim.y > 1 ? 8 : 16)));
}

namespace {
int env_int(const char* n, int dflt) { const char* v = getenv(n); return v && *v ? atoi(v) : dflt; }

int gemv_nw(const QMatDev& m, int ksplit) {
  static const int force = env_int("PYRE_GEMV_NW", 0);
  int per_wg = (m.U + ksplit - 1) / ksplit;
  int nw = m.tiles >= 1024 ? 4 : (m.tiles >= 256 ? 8 : 16);
  while (nw > 1 && nw / 2 >= per_wg) nw /= 2;          // no idle waves
  if (nw < 4) nw = 4;
  if (force == 4 || force == 8 || force == 16) nw = force;
  return nw;
}
template <int FMT, int T, int NW> int gemv_launch_nw(pyre_ctx* ctx, const QMatDev& m, const float* x, float* y, int ksplit, const GemvEpi& ep) {
  int per_wg = (m.U + ksplit - 1) / ksplit, upw = (per_wg + NW - 1) / NW; if (upw < 1) upw = 1;
  static const char* fn[FMT_COUNT] = {"f32", "f16", "bf16", "q8_0", "q4_k", "iq2_xs", "iq3_s", "c4", "c8", "iq3_s", "q4_k", "iq2_xs", "q8_0"};
  static const std::string name = std::string("gemv_") + fn[FMT] + "_t" + std::to_string(T);
  ProfScope ps(ctx, name.c_str(), qmat_gguf_bytes(m, m.rows) + 4.0 * T * ((double)m.cols + m.rows));
  hipLaunchKernelGGL((k_gemv<FMT, T, NW>), dim3(m.tiles, ksplit), dim3(NW * 64), T > 1 ? (size_t)NW * 2 * 64 * T * 4 : 0, ctx->stream, m, x, y, upw, ep, (const uint2*)ctx->d_iq2xs);
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
// Waves per workgroup: enough that a row tile's whole K range is covered by one workgroup with few units per wave,
// fewer when there are so many tiles that the chip is full anyway.
template <int FMT, int T> int gemv_t(pyre_ctx* ctx, const QMatDev& m, const float* x, float* y, int ksplit, const GemvEpi& ep) {
  int nw = ep.four_waves ? 4 : gemv_nw(m, ksplit);
  if (nw == 4) return gemv_launch_nw<FMT, T, 4>(ctx, m, x, y, ksplit, ep);
  if (nw == 8) return gemv_launch_nw<FMT, T, 8>(ctx, m, x, y, ksplit, ep);
  return gemv_launch_nw<FMT, T, 16>(ctx, m, x, y, ksplit, ep);
}
template <int FMT> int gemv_f(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y, int ksplit, const GemvEpi& ep) {
  switch (t) { case 1: return gemv_t<FMT, 1>(ctx, m, x, y, ksplit, ep); case 2: return gemv_t<FMT, 2>(ctx, m, x, y, ksplit, ep); case 3: return gemv_t<FMT, 3>(ctx, m, x, y, ksplit, ep);
    case 4: return gemv_t<FMT, 4>(ctx, m, x, y, ksplit, ep); case 5: return gemv_t<FMT, 5>(ctx, m, x, y, ksplit, ep); case 6: return gemv_t<FMT, 6>(ctx, m, x, y, ksplit, ep);
    case 7: return gemv_t<FMT, 7>(ctx, m, x, y, ksplit, ep); case 8: return gemv_t<FMT, 8>(ctx, m, x, y, ksplit, ep); }
  return pyre_fail(ctx, PYRE_E_ARG, "qmatmul: t = %d outside 1..8", t);
}
#define FMT_DISPATCH(fmt, CALL) \
  switch (fmt) { case FMT_F32: { constexpr int F = FMT_F32; CALL; } break; case FMT_F16: { constexpr int F = FMT_F16; CALL; } break; case FMT_BF16: { constexpr int F = FMT_BF16; CALL; } break; \
    case FMT_Q8_0: { constexpr int F = FMT_Q8_0; CALL; } break; case FMT_Q4_K: { constexpr int F = FMT_Q4_K; CALL; } break; case FMT_IQ2_XS: { constexpr int F = FMT_IQ2_XS; CALL; } break; \
    case FMT_C4: { constexpr int F = FMT_C4; CALL; } break; case FMT_C8: { constexpr int F = FMT_C8; CALL; } break; \
    default: { constexpr int F = FMT_IQ3_S; CALL; } break; }
// the kernels that only decode (export, rows by index, the greedy pick) also read the matrix-core layout
#define FMT_DISPATCH_X(fmt, CALL) \
  switch (fmt) { case FMT_F32: { constexpr int F = FMT_F32; CALL; } break; case FMT_F16: { constexpr int F = FMT_F16; CALL; } break; case FMT_BF16: { constexpr int F = FMT_BF16; CALL; } break; \
    case FMT_Q8_0: { constexpr int F = FMT_Q8_0; CALL; } break; case FMT_Q4_K: { constexpr int F = FMT_Q4_K; CALL; } break; case FMT_IQ2_XS: { constexpr int F = FMT_IQ2_XS; CALL; } break; \
    case FMT_C4: { constexpr int F = FMT_C4; CALL; } break; case FMT_C8: { constexpr int F = FMT_C8; CALL; } break; case FMT_IQ3_S_M: { constexpr int F = FMT_IQ3_S_M; CALL; } break; \
    default: { constexpr int F = FMT_IQ3_S; CALL; } break; }

// A matrix in the matrix-core layout whose caller has no f16 operand at hand: the activations are split into the
// context's operand buffer first (sized by pyre_gemm_m_scratch; grows only outside stream capture).
int gemm_m_from_f32(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y, int ksplit, const GemvEpi& ep, const PyreAop* a) {
  if (a && a->op) return pyre_gemm_m_launch(ctx, m, *a, t, y, ksplit, ep);
  if (ctx->batch_n > 1) return pyre_fail(ctx, PYRE_E_ARG, "gemv: a launch for several windows needs the windows' own operands");
  if (pyre_gemm_m_x_ok(m, t, ep)) return pyre_gemm_m_launch(ctx, m, PyreAop{nullptr, nullptr}, 1, y, ksplit, ep, x);          // few row tiles: the product converts x itself, a launch less
  uint4* op; float* ainv; int rc = pyre_gemm_m_scratch(ctx, m.cols, &op, &ainv); if (rc) return rc;
  if ((rc = pyre_act_split_launch(ctx, x, t, m.cols, op, ainv))) return rc;
  return pyre_gemm_m_launch(ctx, m, PyreAop{op, ainv}, t, y, ksplit, ep);
}
}  // namespace

void pyre_gemv_plan(const QMatDev& m, int* nw, int* upw) { *nw = gemv_nw(m, 1); *upw = (m.U + *nw - 1) / *nw; if (*upw < 1) *upw = 1; }
int pyre_gemv_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y, const PyreAop* a) {
  if (m.fmt == FMT_IQ3_S_M) return gemm_m_from_f32(ctx, m, x, t, y, 1, GemvEpi{}, a);
  if (ctx->batch_n > 1) return pyre_fail(ctx, PYRE_E_ARG, "gemv: only the matrix-core GEMM serves several windows a launch");
  int rc = PYRE_OK;
  FMT_DISPATCH(m.fmt, rc = gemv_f<F>(ctx, m, x, t, y, 1, GemvEpi{}));
  return rc;
}
int pyre_gemv_split_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* partial, int ksplit, const PyreAop* a) {
  if (m.fmt == FMT_IQ3_S_M) return gemm_m_from_f32(ctx, m, x, t, partial, ksplit, GemvEpi{}, a);
  int rc = PYRE_OK;
  FMT_DISPATCH(m.fmt, rc = gemv_f<F>(ctx, m, x, t, partial, ksplit, GemvEpi{}));
  return rc;
}
bool pyre_gemv_parts_ok(const QMatDev& m) {
  static const int off = env_int("PYRE_GEMV_PARTS", 1) == 0;
  if (m.fmt == FMT_IQ3_S_M) return !off && m.tiles <= 64 && m.cols % (128 * PYRE_GEMV_PARTS * 4) == 0 && m.rows == m.tiles * 64;
  return !off && m.tiles <= 64 && gemv_nw(m, 1) == 16 && m.U % 16 == 0 && m.U / 16 >= 2 && m.rows == m.tiles * 64;
}
int pyre_gemv_parts_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* parts, const PyreAop* a) {
  if (!pyre_gemv_parts_ok(m)) return pyre_fail(ctx, PYRE_E_SHAPE, "gemv: the four-part form needs few row tiles and rows of a multiple of 32 units");
  int rc = PYRE_OK;
  GemvEpi ep{}; ep.four_waves = 1;
  if (m.fmt == FMT_IQ3_S_M) return gemm_m_from_f32(ctx, m, x, t, parts, PYRE_GEMV_PARTS, ep, a);
  if (ctx->batch_n > 1) return pyre_fail(ctx, PYRE_E_ARG, "gemv: only the matrix-core GEMM serves several windows a launch");
  FMT_DISPATCH(m.fmt, rc = gemv_f<F>(ctx, m, x, t, parts, PYRE_GEMV_PARTS, ep));
  return rc;
}
int pyre_gemv_best_count(const QMatDev& m) { return m.fmt == FMT_IQ3_S_M ? pyre_gemm_m_best_count(m) : m.tiles; }
int pyre_gemv_argmax_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, float* y, uint32_t* best, const PyreAop* a) {
  int rc = PYRE_OK;
  GemvEpi ep{}; ep.best = best;
  if (m.fmt == FMT_IQ3_S_M) return gemm_m_from_f32(ctx, m, x, 1, y, 1, ep, a);
  FMT_DISPATCH(m.fmt, rc = gemv_f<F>(ctx, m, x, 1, y, 1, ep));
  return rc;
}
int pyre_gemv_conv_launch(pyre_ctx* ctx, const QMatDev& m, const float* x, int t, float* y, const GemvEpi& conv, const PyreAop* a) {
  if (!conv.co || !conv.conv_w || !conv.conv_in || !conv.conv_out || conv.kk < 2 || conv.kk > 8 || conv.ch < 1 || conv.ch > m.rows) return pyre_fail(ctx, PYRE_E_ARG, "gemv: bad conv epilogue (kernel %d, %d channels of %d rows)", conv.kk, conv.ch, m.rows);
  GemvEpi ep = conv; ep.best = nullptr; int rc = PYRE_OK;
  if (m.fmt == FMT_IQ3_S_M) return gemm_m_from_f32(ctx, m, x, t, y, 1, ep, a);
  FMT_DISPATCH(m.fmt, rc = gemv_f<F>(ctx, m, x, t, y, 1, ep));
  return rc;
}

// 256 threads per block: every block redoes the (tiny) scan of the per-tile maxima -- a thread's candidates are all fetched
// before the first is looked at, so the scan is one memory round trip up to 4096 tiles -- block 0 publishes the id, and when
// a matrix is given thread u < 64 of block b then dequantizes unit 64*b+u of the chosen row.
__device__ __forceinline__ void pick_better(float& bv, uint32_t& bi, float v, uint32_t r) {          // larger value, then lower row; 0xFFFFFFFF = no candidate yet
  if (r != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || v > bv || (v == bv && r < bi))) { bv = v; bi = r; }
}
template <int FMT> __global__ __launch_bounds__(256) void k_pick(const uint32_t* __restrict__ best, int n_tiles, uint32_t* id_out, uint32_t* mirror, QMatDev m, int have_m,
                                                                const uint64_t* g2, float* __restrict__ out, int* step, uint32_t* hist) {
  __shared__ float wv[4]; __shared__ uint32_t wi[4];
  const int tid = threadIdx.x;
  float bv = -INFINITY; uint32_t bi = 0xFFFFFFFFu;
  const uint2* b2 = (const uint2*)best;
  for (int i0 = tid; i0 < n_tiles; i0 += 256 * 16) {
    uint2 e[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) e[q] = b2[min(i0 + 256 * q, n_tiles - 1)];
#pragma unroll
    for (int q = 0; q < 16; ++q) if (i0 + 256 * q < n_tiles) pick_better(bv, bi, __uint_as_float(e[q].x), e[q].y);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { float ov = __shfl_xor(bv, o); uint32_t oi = __shfl_xor(bi, o); pick_better(bv, bi, ov, oi); }
  if ((tid & 63) == 0) { wv[tid >> 6] = bv; wi[tid >> 6] = bi; }
  __syncthreads();
  bv = wv[0]; bi = wi[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) pick_better(bv, bi, wv[w], wi[w]);
  if (bi == 0xFFFFFFFFu) bi = 0;
  if (blockIdx.x == 0 && tid == 0) { int slot = 0; if (step) { int p = step[0] + 1; step[0] = p; slot = p - step[1]; if (hist) hist[p] = bi; } id_out[0] = bi; if (mirror) mirror[slot] = bi; }
  if (!have_m || tid >= 64) return;
  int ku = blockIdx.x * 64 + tid; if (ku >= m.U || bi >= (uint32_t)m.rows) return;
  float y[64];
  decode_exact<FMT>(m, g2, (int)(bi >> 6), ku, (int)(bi & 63), y);
  float4* o = (float4*)(out + (size_t)ku * 64);
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] = float4{y[4 * i], y[4 * i + 1], y[4 * i + 2], y[4 * i + 3]};
}

int pyre_pick_launch(pyre_ctx* ctx, const uint32_t* best, int n_tiles, uint32_t* id_out, uint32_t* mirror, const QMatDev* m, float* out, int* step, uint32_t* hist) {
  ProfScope ps(ctx, "pick_embed", 8.0 * n_tiles);
  if (!m) { QMatDev z{}; hipLaunchKernelGGL((k_pick<FMT_F32>), dim3(1), dim3(256), 0, ctx->stream, best, n_tiles, id_out, mirror, z, 0, (const uint64_t*)ctx->d_iq2xs, out, step, hist); }
  else { dim3 grid((m->U + 63) / 64);
    FMT_DISPATCH_X(m->fmt, hipLaunchKernelGGL((k_pick<F>), grid, dim3(256), 0, ctx->stream, best, n_tiles, id_out, mirror, *m, 1, (const uint64_t*)ctx->d_iq2xs, out, step, hist)); }
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

int pyre_row_launch(pyre_ctx* ctx, const QMatDev& m, const uint32_t* idx, int n, float* out, int out_stride) {
  if (n <= 0) return PYRE_OK;
  dim3 grid((m.U + 63) / 64, n);
  ProfScope ps(ctx, "embed_rows", 0.0);
  FMT_DISPATCH_X(m.fmt, hipLaunchKernelGGL((k_rows<F>), grid, dim3(64), 0, ctx->stream, m, (const uint64_t*)ctx->d_iq2xs, idx, out, out_stride));
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}

int pyre_qmat_create_layout(pyre_ctx* ctx, uint32_t ty, size_t rows, size_t cols, const void* blocks, bool on_device, size_t nbytes, int layout, pyre_qmat** out) {
  if (!ctx || !out) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmat_create: null argument");
  *out = nullptr;
  int fmt = fmt_from_ggml(ty); if (fmt < 0) return pyre_fail(ctx, PYRE_E_TYPE, "pyre_qmat_create: unsupported ggml type %u", ty);
  FmtGeom g = qmat_geom(fmt, ty); int gel = 1, gbytes = 4; ggml_geom(ty, &gel, &gbytes);
  if (rows == 0 || cols == 0 || cols % PYRE_UNIT != 0 || cols % gel != 0) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmat_create: %zu x %zu: cols must be a non-zero multiple of 64 and of the block size %d", rows, cols, gel);
  if (rows > (size_t)1 << 30 || cols > (size_t)1 << 24) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmat_create: %zu x %zu too large", rows, cols);
  size_t row_bytes = cols / gel * gbytes;
  if (!blocks || nbytes != rows * row_bytes) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmat_create: expected %zu bytes of blocks, got %zu", rows * row_bytes, nbytes);
  const bool want_n = layout == PYRE_LAYOUT_ALL && (fmt == FMT_IQ3_S || fmt == FMT_IQ2_XS || (fmt == FMT_Q4_K && ty == PYRE_Q4_K)) && cols % 256 == 0;      // the single token's native-format layout
  const bool want_q4m = layout == PYRE_LAYOUT_ALL && fmt == FMT_Q4_K && ty == PYRE_Q4_K && cols % 256 == 0;      // Q4_K for the matrix cores: the operator's windows
  const bool want_q2m = layout == PYRE_LAYOUT_ALL && fmt == FMT_IQ2_XS && ty == PYRE_IQ2_XS && cols % 256 == 0;      // IQ2_XS likewise
  const bool want_q8m = layout == PYRE_LAYOUT_ALL && fmt == FMT_Q8_0 && ty == PYRE_Q8_0 && cols % 256 == 0;      // Q8_0 likewise
  if (layout == PYRE_LAYOUT_ALL) layout = PYRE_LAYOUT_BOTH;
  if (fmt != FMT_IQ3_S) layout = PYRE_LAYOUT_ROWS;       // in a model only IQ3_S has a matrix-core layout
  const bool want_rows = layout != PYRE_LAYOUT_M, want_m = layout != PYRE_LAYOUT_ROWS;
  PYRE_HIP(ctx, hipSetDevice(ctx->device));
  pyre_qmat* m = new pyre_qmat(); m->ctx = ctx; m->ty = ty; m->rows = rows; m->cols = cols; m->gguf_bytes = nbytes;
  auto drop = [&]() { if (m->base) (void)hipFree(m->base); if (m->base_m) (void)hipFree(m->base_m); if (m->base_n) (void)hipFree(m->base_n); delete m; };
  int U = (int)(cols / PYRE_UNIT), tiles = (int)((rows + 63) / 64);
  size_t ent = (size_t)tiles * U * 64;
  auto al = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const uint8_t* src = (const uint8_t*)blocks; void* tmp = nullptr; hipError_t e = hipSuccess;
  if (!on_device) {
    e = hipMalloc(&tmp, nbytes);
    if (e == hipSuccess) e = hipMemcpyAsync(tmp, blocks, nbytes, hipMemcpyHostToDevice, ctx->stream);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmat_create: upload failed: %s", hipGetErrorString(e)); }
    src = (const uint8_t*)tmp;
  }
  const QMatDev shape{nullptr, nullptr, nullptr, nullptr, nullptr, (int)rows, (int)cols, U, tiles, fmt, ty, gel, gbytes, {0, 0, 0, 0}, 0, nullptr, nullptr, 0};
  if (want_rows) {
    size_t s0 = al(ent * g.V * 16), s1 = al(ent * g.e1), s2 = al(ent * g.e2), s3 = al(ent * g.e3), sb = al(ent / 4 * g.eb + 256);
    m->dev_bytes = s0 + s1 + s2 + s3 + sb;
    e = hipMalloc(&m->base, m->dev_bytes);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_qmat_create: hipMalloc(%zu) failed: %s", s0 + s1 + s2 + s3 + sb, hipGetErrorString(e)); }
    uint8_t* b = (uint8_t*)m->base;
    m->dv = shape; m->dv.p0 = b; m->dv.p1 = b + s0; m->dv.p2 = b + s0 + s1; m->dv.p3 = b + s0 + s1 + s2; m->dv.pb = b + s0 + s1 + s2 + s3;
    if (fmt == FMT_C4) c4_table(ty, m->dv.lut, &m->dv.bias);
    size_t total = ent * 1; unsigned nblk = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(k_repack, dim3(nblk), dim3(256), 0, ctx->stream, m->dv, src, row_bytes, b, b + s0, b + s0 + s1, b + s0 + s1 + s2, b + s0 + s1 + s2 + s3, (const uint32_t*)ctx->d_iq3s, (const uint16_t*)ctx->d_cb);
    e = hipGetLastError();
  }
  if (want_m && e == hipSuccess) {
    if (cols % 256) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmat_create: IQ3_S rows are whole super-blocks of 256 columns, got %zu", cols); }
    const int SB = (int)(cols / 256); const size_t rows_pad = (size_t)tiles * 64;
    const size_t sq = al(rows_pad * cols / 2), sh = al(rows_pad * SB * 8);
    m->dev_bytes_m = sq + sh;
    e = hipMalloc(&m->base_m, m->dev_bytes_m);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_qmat_create: hipMalloc(%zu) failed: %s", sq + sh, hipGetErrorString(e)); }
    uint8_t* b = (uint8_t*)m->base_m;
    m->dvm = shape; m->dvm.fmt = FMT_IQ3_S_M; m->dvm.mq = b; m->dvm.mh = b + sq; m->dvm.SB = SB;
    const size_t total = rows_pad * SB;
    hipLaunchKernelGGL(k_repack_m, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, (int)rows, (int)rows_pad, SB, src, row_bytes, (uint32_t*)b, (uint2*)(b + sq), (const uint32_t*)ctx->d_iq3s);
    e = hipGetLastError();
    if (!want_rows) m->dv = m->dvm;         // the only layout the matrix has is the one every user sees
  }
  if (want_q4m && e == hipSuccess) {
    size_t sq; m->dev_bytes_m = pyre_gemm_q4_bytes(rows, cols, &sq);
    e = hipMalloc(&m->base_m, m->dev_bytes_m);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_qmat_create: hipMalloc(%zu) failed: %s", m->dev_bytes_m, hipGetErrorString(e)); }
    m->dvm = shape; m->dvm.fmt = FMT_Q4_K_M; m->dvm.mq = (const uint8_t*)m->base_m; m->dvm.mh = (const uint8_t*)m->base_m + sq; m->dvm.SB = (int)(cols / 256);
    if (pyre_gemm_q4_repack(ctx, rows, cols, src, row_bytes, m->base_m) != PYRE_OK) e = hipErrorLaunchFailure;
  }
  if (want_q2m && e == hipSuccess) {
    size_t sq; m->dev_bytes_m = pyre_gemm_q2_bytes(rows, cols, &sq);
    e = hipMalloc(&m->base_m, m->dev_bytes_m);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_qmat_create: hipMalloc(%zu) failed: %s", m->dev_bytes_m, hipGetErrorString(e)); }
    m->dvm = shape; m->dvm.fmt = FMT_IQ2_XS_M; m->dvm.mq = (const uint8_t*)m->base_m; m->dvm.mh = (const uint8_t*)m->base_m + sq; m->dvm.SB = (int)(cols / 256);
    if (pyre_gemm_q2_repack(ctx, rows, cols, src, row_bytes, m->base_m) != PYRE_OK) e = hipErrorLaunchFailure;
  }
  if (want_q8m && e == hipSuccess) {
    size_t sq; m->dev_bytes_m = pyre_gemm_q8_bytes(rows, cols, &sq);
    e = hipMalloc(&m->base_m, m->dev_bytes_m);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_qmat_create: hipMalloc(%zu) failed: %s", m->dev_bytes_m, hipGetErrorString(e)); }
    m->dvm = shape; m->dvm.fmt = FMT_Q8_0_M; m->dvm.mq = (const uint8_t*)m->base_m; m->dvm.mh = (const uint8_t*)m->base_m + sq; m->dvm.SB = (int)(cols / 256);
    if (pyre_gemm_q8_repack(ctx, rows, cols, src, row_bytes, m->base_m) != PYRE_OK) e = hipErrorLaunchFailure;
  }
  if (want_n && e == hipSuccess) {      // the stand-alone operator's single-token kernel streams (close to) the file's bits per weight
    m->dev_bytes_n = pyre_gemv_n_bytes(rows, cols, fmt);
    e = hipMalloc(&m->base_n, m->dev_bytes_n);
    if (e != hipSuccess) { if (tmp) (void)hipFree(tmp); drop(); return pyre_fail(ctx, PYRE_E_NOMEM, "pyre_qmat_create: hipMalloc(%zu) failed: %s", m->dev_bytes_n, hipGetErrorString(e)); }
    if (pyre_gemv_n_repack(ctx, rows, cols, src, row_bytes, m->base_n, fmt) != PYRE_OK) e = hipErrorLaunchFailure;
  }
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (tmp) (void)hipFree(tmp);
  if (e != hipSuccess) { drop(); return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmat_create: repack failed: %s", hipGetErrorString(e)); }
  *out = m; return PYRE_OK;
}
// the stand-alone operator keeps an IQ3_S matrix in both layouts: pyre_qmatmul runs on the matrix cores, pyre_qmatmul_f32
// on the lane = row GEMV that the model's expert matrices use
static int qmat_create_common(pyre_ctx* ctx, uint32_t ty, size_t rows, size_t cols, const void* blocks, bool on_device, size_t nbytes, pyre_qmat** out) {
  return pyre_qmat_create_layout(ctx, ty, rows, cols, blocks, on_device, nbytes, PYRE_LAYOUT_ALL, out);
}

extern "C" {

int pyre_qmat_create(pyre_ctx* ctx, uint32_t ty, size_t rows, size_t cols, const void* host_blocks, size_t nbytes, pyre_qmat** out) { return qmat_create_common(ctx, ty, rows, cols, host_blocks, false, nbytes, out); }
int pyre_qmat_create_dev(pyre_ctx* ctx, uint32_t ty, size_t rows, size_t cols, const void* dev_blocks, size_t nbytes, pyre_qmat** out) { return qmat_create_common(ctx, ty, rows, cols, dev_blocks, true, nbytes, out); }
void pyre_qmat_destroy(pyre_qmat* m) { if (!m) return; (void)hipSetDevice(m->ctx->device); (void)hipStreamSynchronize(m->ctx->stream); if (m->base) (void)hipFree(m->base); if (m->base_m) (void)hipFree(m->base_m); if (m->base_n) (void)hipFree(m->base_n); delete m; }
size_t pyre_qmat_rows(const pyre_qmat* m) { return m ? m->rows : 0; }
size_t pyre_qmat_cols(const pyre_qmat* m) { return m ? m->cols : 0; }
size_t pyre_qmat_gguf_bytes(const pyre_qmat* m) { return m ? m->gguf_bytes : 0; }
size_t pyre_qmat_device_bytes(const pyre_qmat* m) { return m ? m->dev_bytes + m->dev_bytes_m + m->dev_bytes_n : 0; }
size_t pyre_qmat_layout_bytes(const pyre_qmat* m, int which) { return !m ? 0 : (which == 2 ? m->dev_bytes_n : (which ? m->dev_bytes_m : m->dev_bytes)); }

int pyre_qmat_dequant_dev(pyre_ctx* ctx, const pyre_qmat* m, float* out_dev) {
  if (!ctx || !m || !out_dev) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmat_dequant: null argument");
  dim3 grid(m->dv.U, m->dv.tiles);
  FMT_DISPATCH_X(m->dv.fmt, hipLaunchKernelGGL((k_dequant<F>), grid, dim3(64), 0, ctx->stream, m->dv, (const uint64_t*)ctx->d_iq2xs, out_dev));
  PYRE_CHECK_LAUNCH(ctx); return PYRE_OK;
}
int pyre_qmat_dequant(pyre_ctx* ctx, const pyre_qmat* m, float* out_host) {
  if (!ctx || !m || !out_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmat_dequant: null argument");
  size_t n = m->rows * m->cols * sizeof(float); void* tmp = nullptr;
  PYRE_HIP(ctx, hipMalloc(&tmp, n));
  int rc = pyre_qmat_dequant_dev(ctx, m, (float*)tmp);
  hipError_t e = hipSuccess;
  if (!rc) { e = hipMemcpyAsync(out_host, tmp, n, hipMemcpyDeviceToHost, ctx->stream); if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream); }
  (void)hipFree(tmp);
  if (rc) return rc; if (e != hipSuccess) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmat_dequant: %s", hipGetErrorString(e));
  return PYRE_OK;
}
int pyre_qmat_row(pyre_ctx* ctx, const pyre_qmat* m, size_t row, float* out_host) {
  if (!ctx || !m || !out_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmat_row: null argument");
  if (row >= m->rows) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmat_row: row %zu of %zu", row, m->rows);
  void* st; int rc = pyre_stage(ctx, m->cols * sizeof(float) + 256, &st); if (rc) return rc;
  uint32_t r = (uint32_t)row; uint32_t* idx = (uint32_t*)((uint8_t*)st + m->cols * sizeof(float));
  PYRE_HIP(ctx, hipMemcpyAsync(idx, &r, 4, hipMemcpyHostToDevice, ctx->stream));
  rc = pyre_row_launch(ctx, (m->dvm.mq && m->dvm.fmt == FMT_IQ3_S_M) ? m->dvm : m->dv, idx, 1, (float*)st, (int)m->cols); if (rc) return rc;      // a matrix held in both layouts: rows come from the matrix-core one, pyre_qmat_dequant from the other
  PYRE_HIP(ctx, hipMemcpyAsync(out_host, st, m->cols * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}

// The operator's own launch: an IQ3_S matrix goes through the matrix-core GEMM (for every t, so a token's result does not
// depend on the window width); f32_path (or PYRE_QMATMUL_F32=1) takes the f32 lane = row GEMV the model's expert matrices use.
static bool qmat_small_one_token(const pyre_qmat* m, int t) {
  const int on = env_int("PYRE_QMATMUL_SMALL", 1);          // read at every call: tests switch it to reach the native-format kernel with small shapes
  return on && t == 1 && m->dvm.fmt == FMT_IQ3_S_M && m->base != nullptr && m->dv.fmt == FMT_IQ3_S && m->dv.tiles <= 128;
}
static int qmatmul_launch(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev, bool f32_path) {
  static const int f32_only = env_int("PYRE_QMATMUL_F32", 0), native = env_int("PYRE_QMATMUL_NATIVE", 1);
  // one token of a small IQ3_S matrix (at most 128 row tiles): the lane = row f32 GEMV -- one launch where the other two
  // paths need a second one for the activations, and a call of this size is its launches, not its bytes
  if (qmat_small_one_token(m, t) && !f32_path && !f32_only) return pyre_gemv_launch(ctx, m->dv, x_dev, t, y_dev);
  // one token of an IQ3_S matrix: the kernel that streams the file's 3.44 bit/weight (PYRE_QMATMUL_NATIVE=0: the matrix cores as for a window)
  // (IQ2_XS and Q4_K have the same kernel over their own layouts, 2.5 and 4.5 bit/weight; a small matrix of them stays with the one-launch f32 GEMV likewise)
  const bool rows_only = m->dv.fmt == FMT_IQ2_XS || m->dv.fmt == FMT_Q4_K;          // (the formats without a matrix-core layout)
  if (t == 1 && m->base_n && native && !f32_path && !f32_only && !(rows_only && m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) return pyre_gemv_n_launch(ctx, m->base_n, m->rows, m->cols, x_dev, y_dev, nullptr, rows_only ? m->dv.fmt : FMT_IQ3_S);
  // a window of a large Q4_K matrix: the matrix cores, where eight tokens cost what two do (PYRE_QMATMUL_Q4M=0: the lane = row GEMV);
  // small matrices stay with the one-launch GEMV, as above
  if (t >= 2 && env_int("PYRE_QMATMUL_Q4M", 1) && m->dvm.fmt == FMT_Q4_K_M && m->dvm.mq && !f32_path && !f32_only && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) return pyre_gemm_q4_launch(ctx, m->dvm, x_dev, t, y_dev);
  // a window of a large Q8_0 matrix likewise (PYRE_QMATMUL_Q8M=0: the lane = row GEMV)
  if (t >= 2 && env_int("PYRE_QMATMUL_Q8M", 1) && m->dvm.fmt == FMT_Q8_0_M && m->dvm.mq && !f32_path && !f32_only && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) return pyre_gemm_q8_launch(ctx, m->dvm, x_dev, t, y_dev);
  // a window of a large IQ2_XS matrix likewise (PYRE_QMATMUL_Q2M=0: the lane = row GEMV)
  if (t >= 2 && env_int("PYRE_QMATMUL_Q2M", 1) && m->dvm.fmt == FMT_IQ2_XS_M && m->dvm.mq && !f32_path && !f32_only && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) return pyre_gemm_q2_launch(ctx, m->dvm, x_dev, t, y_dev);
  const bool has_m = m->dvm.fmt == FMT_IQ3_S_M && m->dvm.mq, has_rows = m->base != nullptr;
  if (has_m && (!has_rows || (!f32_path && !f32_only))) return pyre_gemv_launch(ctx, m->dvm, x_dev, t, y_dev);
  return pyre_gemv_launch(ctx, m->dv, x_dev, t, y_dev);
}
static int qmatmul_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev, bool f32_path) {
  if (!ctx || !m || !x_dev || !y_dev) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul: null argument");
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul: t = %d outside 1..8", t);
  return qmatmul_launch(ctx, m, x_dev, t, y_dev, f32_path);
}
static int qmatmul_host(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host, bool f32_path) {
  if (!ctx || !m || !x_host || !y_host) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul: null argument");
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul: t = %d outside 1..8", t);
  size_t xb = (size_t)t * m->cols * sizeof(float), yb = (size_t)t * m->rows * sizeof(float), xo = (xb + 255) & ~(size_t)255;
  void* st; int rc = pyre_stage(ctx, xo + yb, &st); if (rc) return rc;
  float* xd = (float*)st; float* yd = (float*)((uint8_t*)st + xo);
  PYRE_HIP(ctx, hipMemcpyAsync(xd, x_host, xb, hipMemcpyHostToDevice, ctx->stream));
  rc = qmatmul_launch(ctx, m, xd, t, yd, f32_path); if (rc) return rc;
  PYRE_HIP(ctx, hipMemcpyAsync(y_host, yd, yb, hipMemcpyDeviceToHost, ctx->stream));
  PYRE_HIP(ctx, hipStreamSynchronize(ctx->stream)); return PYRE_OK;
}
int pyre_qmatmul_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev) { return qmatmul_dev(ctx, m, x_dev, t, y_dev, false); }
int pyre_qmatmul(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host) { return qmatmul_host(ctx, m, x_host, t, y_host, false); }
int pyre_qmatmul_static_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev) {
  if (!ctx || !m || !x_dev || !y_dev) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul_static_dev: null argument");
  if (t < 1 || t > 8) return pyre_fail(ctx, PYRE_E_ARG, "pyre_qmatmul_static_dev: t = %d outside 1..8", t);
  if ((m->dv.fmt == FMT_IQ2_XS || m->dv.fmt == FMT_Q4_K) && m->base_n) {      // IQ2_XS, Q4_K: only the single token of a large matrix uses scratch (the native-format kernel's activation digits)
    if (m->cols > PYRE_QMATMUL_STATIC_MAX_COLS) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmatmul_static_dev: %zu columns exceed the static scratch of %d columns; use pyre_qmatmul_dev", m->cols, PYRE_QMATMUL_STATIC_MAX_COLS);
    if (t == 1 && env_int("PYRE_QMATMUL_NATIVE", 1) && !env_int("PYRE_QMATMUL_F32", 0) && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) {
      if (!ctx->aop_static) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the device array was not resolved at context creation");
      return pyre_gemv_n_launch(ctx, m->base_n, m->rows, m->cols, x_dev, y_dev, ctx->aop_static, m->dv.fmt);
    }
    if (t >= 2 && env_int("PYRE_QMATMUL_Q4M", 1) && m->dvm.fmt == FMT_Q4_K_M && m->dvm.mq && !env_int("PYRE_QMATMUL_F32", 0) && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) {      // a Q4_K window on the matrix cores, as in pyre_qmatmul_dev
      if (!ctx->aop_static) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the device array was not resolved at context creation");
      return pyre_gemm_q4_launch(ctx, m->dvm, x_dev, t, y_dev, ctx->aop_static);
    }
    if (t >= 2 && env_int("PYRE_QMATMUL_Q2M", 1) && m->dvm.fmt == FMT_IQ2_XS_M && m->dvm.mq && !env_int("PYRE_QMATMUL_F32", 0) && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) {      // an IQ2_XS window likewise
      if (!ctx->aop_static) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the device array was not resolved at context creation");
      return pyre_gemm_q2_launch(ctx, m->dvm, x_dev, t, y_dev, ctx->aop_static);
    }
    return pyre_gemv_launch(ctx, m->dv, x_dev, t, y_dev);
  }
  if (m->dvm.fmt == FMT_Q8_0_M && m->dvm.mq) {      // Q8_0: only a window of a large matrix uses scratch (the matrix-core kernel's operand rows)
    if (m->cols > PYRE_QMATMUL_STATIC_MAX_COLS) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmatmul_static_dev: %zu columns exceed the static scratch of %d columns; use pyre_qmatmul_dev", m->cols, PYRE_QMATMUL_STATIC_MAX_COLS);
    if (t >= 2 && env_int("PYRE_QMATMUL_Q8M", 1) && !env_int("PYRE_QMATMUL_F32", 0) && !(m->dv.tiles <= 128 && env_int("PYRE_QMATMUL_SMALL", 1))) {
      if (!ctx->aop_static) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the device array was not resolved at context creation");
      return pyre_gemm_q8_launch(ctx, m->dvm, x_dev, t, y_dev, ctx->aop_static);
    }
    return pyre_gemv_launch(ctx, m->dv, x_dev, t, y_dev);
  }
  if (m->dvm.fmt != FMT_IQ3_S_M || !m->dvm.mq) return pyre_fail(ctx, PYRE_E_TYPE, "pyre_qmatmul_static_dev: IQ3_S, IQ2_XS, Q4_K and Q8_0 matrices only (the other types' GEMV uses no scratch: pyre_qmatmul_dev allocates nothing for them)");
  if (m->cols > PYRE_QMATMUL_STATIC_MAX_COLS) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmatmul_static_dev: %zu columns exceed the static scratch of %d columns; use pyre_qmatmul_dev", m->cols, PYRE_QMATMUL_STATIC_MAX_COLS);
  if (qmat_small_one_token(m, t) && !env_int("PYRE_QMATMUL_F32", 0)) return pyre_gemv_launch(ctx, m->dv, x_dev, t, y_dev);      // as pyre_qmatmul_dev (a launch that happens to need no scratch; the limit above holds for every call alike)
  if (t == 1 && m->base_n && env_int("PYRE_QMATMUL_NATIVE", 1)) {      // one token: the native-format kernel, as in pyre_qmatmul_dev, its activation digits in the static array
    if (m->cols > PYRE_QMATMUL_STATIC_MAX_COLS) return pyre_fail(ctx, PYRE_E_SHAPE, "pyre_qmatmul_static_dev: %zu columns exceed the static scratch of %d columns; use pyre_qmatmul_dev", m->cols, PYRE_QMATMUL_STATIC_MAX_COLS);
    if (!ctx->aop_static) return pyre_fail(ctx, PYRE_E_HIP, "pyre_qmatmul_static_dev: the device array was not resolved at context creation");
    return pyre_gemv_n_launch(ctx, m->base_n, m->rows, m->cols, x_dev, y_dev, ctx->aop_static);
  }
  return pyre_gemm_m_static(ctx, m->dvm, x_dev, t, y_dev);
}
int pyre_qmatmul_f32_dev(pyre_ctx* ctx, const pyre_qmat* m, const float* x_dev, int t, float* y_dev) { return qmatmul_dev(ctx, m, x_dev, t, y_dev, true); }
int pyre_qmatmul_f32(pyre_ctx* ctx, const pyre_qmat* m, const float* x_host, int t, float* y_host) { return qmatmul_host(ctx, m, x_host, t, y_host, true); }

}  // extern "C"
