"""Pins the CPU oracle's wire formats (no GPU): codebooks, the four block dequantizers, dot / matmul, KV4, RoPE
table, argmax, top-k.  Known answers are derived from the format definitions (gguf_q.rs:79,103-107,126-129,141-151
of the reference), not from the oracle's own code."""
import numpy as np
import pytest

import np_ref
import orc
from pyre_amd import synth

FMTS = [orc.Q8_0, orc.Q4_K, orc.IQ2_XS, orc.IQ3_S]
# the other block types real files of this architecture use (gguf_q.rs:74-78,82-89,114-125,130-140)
FMTS_MORE = [orc.Q4_0, orc.Q5_0, orc.Q6_K, orc.IQ2_XXS, orc.IQ3_XXS, orc.IQ4_NL, orc.IQ2_S, orc.IQ4_XS, orc.Q3_K, orc.Q2_0, orc.Q5_K, orc.IQ1_M]


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_codebook_digests_match_reference_tables():
    for hdr in ("oracle/iq_codebooks.h", "pyre_amd/csrc/iq_codebooks.h"):
        import os
        p = os.path.join(np_ref._ROOT, hdr)
        assert np_ref.codebook_digests(p) == (np_ref.IQ3S_SHA256, np_ref.IQ2XS_SHA256, np_ref.KSIGNS_SHA256)
        assert np_ref.codebook_digests_more(p) == (np_ref.IQ2XXS_SHA256, np_ref.IQ2S_SHA256, np_ref.IQ3XXS_SHA256, np_ref.IQ4NL_VALUES)
        import hashlib
        assert hashlib.sha256(np_ref.codebook_iq1s(p).tobytes()).hexdigest() == np_ref.IQ1S_SHA256


def test_oracle_expansion_equals_numpy_expansion():
    import ctypes as C
    g3, g2, ks = np_ref.codebooks()
    o3 = np.empty(512, dtype=np.uint32); o2 = np.empty(512, dtype=np.uint64)
    orc.lib().orc_expand_iq3s(o3.ctypes.data_as(C.c_void_p)); orc.lib().orc_expand_iq2xs(o2.ctypes.data_as(C.c_void_p))
    assert np.array_equal(o3.view(np.uint8).reshape(512, 4), g3)
    assert np.array_equal(o2.view(np.uint8).reshape(512, 8), g2)
    assert [orc.lib().orc_ksigns(i) for i in range(128)] == list(ks)
    # structural facts of the published codebooks
    assert set(np.unique(g3)) == {1, 3, 5, 7, 9, 11, 13, 15}
    assert set(np.unique(g2)) == {8, 25, 43}
    assert np.array_equal(g3[0], [1, 1, 1, 1]) and np.array_equal(g2[0], [8] * 8)


# ---- known-answer blocks --------------------------------------------------------------------------------------
def test_iq3s_zero_payload_is_all_d():
    # indices 0 -> grid entry 0 = (1,1,1,1); scale nibble 0 -> factor 1; no sign bits
    b = np_ref.pack_iq3s(1.0, np.zeros(64, np.uint8), np.zeros(8, np.uint8), np.zeros(32, np.uint8), np.zeros(4, np.uint8))
    assert np.array_equal(orc.dequant(orc.IQ3_S, b, 256), np.ones(256, np.float32))


def test_iq3s_scale_sign_and_high_bit_fields():
    g3, _, _ = np_ref.codebooks()
    qs = np.zeros(64, np.uint8); qh = np.zeros(8, np.uint8); sg = np.zeros(32, np.uint8); sc = np.zeros(4, np.uint8)
    sc[1] = 0x5 | (0xC << 4)            # sub-block 2 -> 1+2*5 = 11, sub-block 3 -> 1+2*12 = 25
    sg[4 * 2 + 1] = 0b00100100          # sub-block 2, group 1: elements 2 and 5 negative
    qs[8 * 3 + 5] = 77; qh[3] = 1 << 5  # sub-block 3, index byte 5 -> entry 77 + 256
    qs[8 * 5 + 0] = 200                 # sub-block 5, index byte 0 -> entry 200 (no high bit)
    y = orc.dequant(orc.IQ3_S, np_ref.pack_iq3s(0.5, qs, qh, sg, sc), 256).reshape(8, 4, 8)
    exp = np.full((8, 4, 8), 0.5, np.float32)
    exp[2] = 0.5 * 11; exp[3] = 0.5 * 25
    exp[2, 1, 2] *= -1; exp[2, 1, 5] *= -1
    exp[3, 2, 4:8] = 0.5 * 25 * g3[77 + 256].astype(np.float32)      # index byte 5 = second entry of group 2
    exp[5, 0, 0:4] = 0.5 * g3[200].astype(np.float32)
    assert np.array_equal(y, exp)


def test_iq2xs_zero_payload_and_fields():
    _, g2, ks = np_ref.codebooks()
    # q = 0 -> grid entry 0 = eight 8s, scale nibble 0 -> d * 0.5 * 0.25 * 8 = d
    b = np_ref.pack_iq2xs(2.0, np.zeros(32, np.uint16), np.zeros(8, np.uint8))
    assert np.array_equal(orc.dequant(orc.IQ2_XS, b, 256), np.full(256, 2.0, np.float32))
    qs = np.zeros(32, np.uint16); sc = np.zeros(8, np.uint8)
    sc[2] = 0x3 | (0x9 << 4)            # ib 2: groups 0,1 -> (0.5+3)/4, groups 2,3 -> (0.5+9)/4
    qs[4 * 2 + 3] = 300 | (5 << 9)      # ib 2, group 3: grid 300, sign index 5 -> ksigns[5] = 0b00000101
    y = orc.dequant(orc.IQ2_XS, np_ref.pack_iq2xs(1.0, qs, sc), 256).reshape(8, 4, 8)
    exp = np.full((8, 4, 8), 1.0, np.float32)
    exp[2, 0:2] = 3.5 * 0.25 * 8; exp[2, 2:4] = 9.5 * 0.25 * 8
    sgn = np.where((ks[5] >> np.arange(8)) & 1, -1.0, 1.0).astype(np.float32)
    assert ks[5] == 5
    exp[2, 3] = np.float32(9.5 * 0.25) * g2[300].astype(np.float32) * sgn
    assert np.array_equal(y, exp)


def test_q4k_both_scale_branches_and_nibbles():
    s = [1, 2, 3, 4, 33, 47, 63, 17]; m = [5, 6, 7, 8, 21, 62, 9, 40]   # j>=4 values need the split 4+2 bit encoding
    q = (np.arange(256) * 7 + 3) % 16
    y = orc.dequant(orc.Q4_K, np_ref.pack_q4k(0.25, 0.5, s, m, q), 256).reshape(8, 32)
    for j in range(8):
        exp = np.float32(0.25 * s[j]) * q.reshape(8, 32)[j].astype(np.float32) - np.float32(0.5 * m[j])
        assert np.array_equal(y[j], exp.astype(np.float32)), j


def test_q8_0_full_range():
    q = np.concatenate([np.arange(-128, -112), np.arange(112, 128)])
    y = orc.dequant(orc.Q8_0, np_ref.pack_q8_0(0.125, q), 32)
    assert np.array_equal(y, q.astype(np.float32) * 0.125)


def test_bf16_f16_f32_passthrough():
    x = np.array([1.5, -2.25, 3.0e-5, 1024.0], dtype=np.float32)
    assert np.array_equal(orc.dequant(orc.F32, x.view(np.uint8), 4), x)
    assert np.array_equal(orc.dequant(orc.F16, x.astype(np.float16).view(np.uint8), 4), x.astype(np.float16).astype(np.float32))
    bf = (x.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(orc.dequant(orc.BF16, bf.view(np.uint8), 4), (bf.astype(np.uint32) << 16).view(np.float32))


def _blk(n, d, off=0):
    b = np.zeros(n, np.uint8); b[off:off + 2] = np_ref.f16_bytes(d); return b


def test_q4_0_and_q5_0_known_answers():
    b = _blk(18, 0.5); b[2:] = np.arange(16) | ((15 - np.arange(16)) << 4)       # low nibble j, high nibble 15 - j
    y = orc.dequant(orc.Q4_0, b, 32)
    assert np.array_equal(y[:16], (np.arange(16) - 8) * 0.5) and np.array_equal(y[16:], (7 - np.arange(16)) * 0.5)
    b = _blk(22, 0.25); b[2:6] = np.array([(1 << 3) | (1 << 20)], np.uint32).view(np.uint8)   # fifth bit of elements 3 and 20
    b[6:] = 0x21                                                                      # low nibble 1, high nibble 2
    y = orc.dequant(orc.Q5_0, b, 32)
    exp = np.concatenate([np.full(16, 1 - 16.0), np.full(16, 2 - 16.0)]); exp[3] += 16; exp[20] += 16
    assert np.array_equal(y, (exp * 0.25).astype(np.float32))


def test_q2_0_and_q3_k_known_answers():
    # Q2_0 (gguf_q.rs:80-81, :50): byte 0b11100100 holds the codes 0, 1, 2, 3 from the low bits up -> values -1, 0, 1, 2
    b = _blk(18, 0.5); b[2:] = 0b11100100
    assert np.array_equal(orc.dequant(orc.Q2_0, b, 64), np.tile(np.array([-1, 0, 1, 2], np.float32) * 0.5, 16))
    # Q3_K (gguf_q.rs:90-102): zero payload -> scale 0 - 32, low bits 0, mask clear -> -4: every value d * -32 * -4
    assert np.array_equal(orc.dequant(orc.Q3_K, _blk(110, 0.5, 108), 256), np.full(256, 0.5 * -32 * -4, np.float32))
    b = _blk(110, 1.0, 108)
    b[96 + 3] = 0x5 | (0xA << 4)          # low 4 bits of scale 3 = 5, of scale 11 = 10
    b[96 + 8 + 3] = 0b00100001            # high 2 bits: scale 3 (bits 0-1) = 1, scale 11 (bits 4-5) = 2
    b[32 + 20] = 0b00001100               # first 128 values, byte o = 20: code 3 at shift 2 (j = 1) -> value index 32 + 20
    b[0 + 20] = 0b00000010                # high-mask bit 1 (n = 0, j = 1) of byte 20 set: no -4
    b[32 + 32 + 7] = 0b01000000           # second 128 values, byte o = 7: code 1 at shift 6 (j = 3) -> value index 128 + 96 + 7
    y = orc.dequant(orc.Q3_K, b, 256)
    exp = np.full(256, -32.0 * -4, np.float32)
    exp[48:64] = ((5 | (1 << 4)) - 32) * -4.0           # scale 3 covers values 48..63
    exp[176:192] = ((10 | (2 << 4)) - 32) * -4.0        # scale 11 covers values 176..191
    exp[52] = ((5 | (1 << 4)) - 32) * 3.0               # value 32 + 20 lies in scale 3's group: code 3, mask set
    exp[128 + 96 + 7] = -32.0 * (1 - 4)
    assert np.array_equal(y, exp)


def test_iq1_m_known_answers():
    # gguf_q.rs:152-165.  The IQ1S grid is ggml's; its expansion is pinned by digest like the other grids.
    g1 = np_ref.codebook_iq1s()
    import hashlib
    assert hashlib.sha256(g1.tobytes()).hexdigest() == np_ref.IQ1S_SHA256
    assert set(np.unique(g1)) == {-1, 0, 1}

    def blk(d):
        b = np.zeros(56, np.uint8); h = int(np.array([d], np.float16).view(np.uint16)[0])
        for k in range(4):
            b[49 + 2 * k] = ((h >> (4 * k)) & 0xF) << 4
        return b
    # zero payload: index 0, 3-bit scales 0 -> d * 1, delta +0.125: every value d * (grid[0] + 0.125)
    y = orc.dequant(orc.IQ1_M, blk(2.0), 256).reshape(32, 8)
    assert np.array_equal(y, np.tile(2.0 * (g1[0].astype(np.float32) + 0.125), (32, 1)))
    # sub-block 5 (second half of scale word 2): first scale 3 -> x7, second scale 6 -> x13; group 1 of it: index 0x2A5 (high bits 2 from
    # qh[0] bits 4-6), delta negative (qh[0] bit 7); group 2: index 0x733 (high bits 7 from qh[1] bits 0-2), delta positive
    b = blk(0.5)
    w2 = (3 << 6) | (6 << 9); b[48 + 4] |= w2 & 0xFF; b[48 + 5] |= (w2 >> 8) & 0x0F
    b[4 * 5 + 1] = 0xA5; b[32 + 2 * 5 + 0] = (2 << 4) | 0x80
    b[4 * 5 + 2] = 0x33; b[32 + 2 * 5 + 1] = 7
    y = orc.dequant(orc.IQ1_M, b, 256).reshape(8, 4, 8)
    assert np.array_equal(y[5, 1], (0.5 * 7) * (g1[0x2A5].astype(np.float32) - 0.125))
    assert np.array_equal(y[5, 2], (0.5 * 13) * (g1[0x733].astype(np.float32) + 0.125))
    assert np.array_equal(y[5, 0], (0.5 * 7) * (g1[0].astype(np.float32) + 0.125)) and np.array_equal(y[5, 3], (0.5 * 13) * (g1[0].astype(np.float32) + 0.125))
    assert np.array_equal(y[4, 0], 0.5 * (g1[0].astype(np.float32) + 0.125))       # first half of the same scale word: 3-bit scales 0


def test_q5_k_known_answers():
    # gguf_q.rs:108-113.  scales bytes: sub-block 0 -> (s, m) = (3, 5) through the j < 4 branch; sub-block 5 -> (s, m) = (0x2B, 0x1C)
    # through the j >= 4 branch: low 4 bits in byte 9 (s low nibble, m high nibble), high 2 bits in bits 6-7 of bytes 1 (s) and 5 (m)
    b = _blk(176, 0.5); b[2:4] = np_ref.f16_bytes(0.25)
    b[4 + 0] = 3; b[4 + 4] = 5
    b[4 + 9] = (0x2B & 0xF) | ((0x1C & 0xF) << 4); b[4 + 1] = (0x2B >> 4) << 6; b[4 + 5] = (0x1C >> 4) << 6
    b[48 + 7] = 0x9                      # sub-block 0 (low nibbles of the first 32 bytes), value 7: nibble 9
    b[16 + 7] = 0b00000001               # ... with its fifth bit (bit 0 of qh[7]) set -> 25
    b[48 + 64 + 3] = 0xC0                # sub-block 5 (high nibbles of the third 32 bytes), value 3: nibble 12
    b[16 + 3] = 1 << 5                   # ... fifth bit = bit 5 of qh[3] -> 28
    y = orc.dequant(orc.Q5_K, b, 256).reshape(8, 32)
    exp = np.zeros((8, 32), np.float32)
    exp[0] = 0.5 * 3 * 0 - 0.25 * 5; exp[0, 7] = 0.5 * 3 * 25 - 0.25 * 5
    exp[5] = -0.25 * 0x1C; exp[5, 3] = 0.5 * 0x2B * 28 - 0.25 * 0x1C
    exp[1, 7] = 0.0                      # bytes 1 and 5 also carry the 6-bit (s, m) of sub-block 1: both 0 in their low bits
    assert np.array_equal(y, exp)


def test_iq4_nl_and_iq4_xs_known_answers():
    kv = np.array(np_ref.IQ4NL_VALUES, np.float32)
    b = _blk(18, 2.0); b[2:] = np.arange(16) | ((15 - np.arange(16)) << 4)
    y = orc.dequant(orc.IQ4_NL, b, 32)
    assert np.array_equal(y[:16], 2.0 * kv) and np.array_equal(y[16:], 2.0 * kv[::-1])
    # IQ4_XS: zero payload -> 6-bit scale 0 -> d * (0 - 32), level 0 = -127
    assert np.array_equal(orc.dequant(orc.IQ4_XS, _blk(136, 0.5), 256), np.full(256, -127 * (0.5 * -32), np.float32))
    b = _blk(136, 1.0)
    b[2:4] = np.array([(2 << (2 * 5)) | (3 << (2 * 6))], np.uint16).view(np.uint8)   # high bits: sub-block 5 -> 2, sub-block 6 -> 3
    b[4 + 2] = 0x9 << 4                                                               # low bits of sub-block 5 (high nibble of byte 2) = 9
    b[4 + 3] = 0x4                                                                    # low bits of sub-block 6 = 4
    b[8 + 16 * 5:8 + 16 * 6] = np.arange(16) | ((15 - np.arange(16)) << 4)
    y = orc.dequant(orc.IQ4_XS, b, 256).reshape(8, 32)
    assert np.array_equal(y[5, :16], kv * float((9 | (2 << 4)) - 32)) and np.array_equal(y[5, 16:], kv[::-1] * float(41 - 32))
    assert np.array_equal(y[6], np.full(32, -127.0 * ((4 | (3 << 4)) - 32), np.float32))
    assert np.array_equal(y[0], np.full(32, -127.0 * -32, np.float32))


def test_q6_k_known_answers():
    b = _blk(210, 0.5, off=208); b[192:208] = 1
    assert np.array_equal(orc.dequant(orc.Q6_K, b, 256), np.full(256, 0.5 * 1 * -32, np.float32))     # all six-bit values 0 -> -32
    b = _blk(210, 1.0, off=208)
    b[192:208] = np.array([1, 2, 3, 4, 5, 6, 7, 8, -1, -2, -3, -4, -5, -6, -7, -8], np.int8).view(np.uint8)
    # second half (elements 128..255): element 128 + 64 + 17 is quarter 2, l = 17 -> high nibble of ql[64 + 17], bits 4..5 of qh[32 + 17],
    # scale index 8 + 2*2 + 17 // 16 = 13 (-6)
    b[64 + 17] = 0xB << 4; b[128 + 32 + 17] = 0x2 << 4
    y = orc.dequant(orc.Q6_K, b, 256)
    assert y[128 + 64 + 17] == -6.0 * ((0xB | (2 << 4)) - 32)
    # element 33 is quarter 1, l = 1 -> low nibble of ql[32 + 1], bits 2..3 of qh[1], scale index 2
    b[32 + 1] = 0x7; b[128 + 1] = 0x3 << 2
    y = orc.dequant(orc.Q6_K, b, 256)
    assert y[33] == 3.0 * ((7 | (3 << 4)) - 32)
    assert y[0] == 1.0 * -32 and y[16] == 2.0 * -32 and y[255] == -8.0 * -32


def test_iq2_xxs_iq2_s_iq3_xxs_known_answers():
    gxx, gs, g3x, _ = np_ref.codebooks_more()
    _, _, ks = np_ref.codebooks()
    assert np.array_equal(gxx[0], [8] * 8) and np.array_equal(gs[0], [8] * 8) and np.array_equal(g3x[0], [4] * 4)
    assert set(np.unique(gxx)) == {8, 25, 43} and set(np.unique(gs)) == {8, 25, 43} and set(np.unique(g3x)) == {4, 12, 20, 28, 36, 44, 52, 62}
    # zero payload: entry 0, scale bits 0, no signs -> d*(0.5)*0.25*8 = d, and d*(0.5)*0.5*4 = d
    for ty, n in ((orc.IQ2_XXS, 66), (orc.IQ2_S, 82), (orc.IQ3_XXS, 98)):
        assert np.array_equal(orc.dequant(ty, _blk(n, 3.0), 256), np.full(256, 3.0, np.float32)), ty
    # IQ2_XXS: sub-block 3: grid bytes (10, 0, 200, 0), sign index 9 for group 2, scale bits 6
    b = _blk(66, 1.0); b[2 + 8 * 3 + 0] = 10; b[2 + 8 * 3 + 2] = 200
    b[2 + 8 * 3 + 4:2 + 8 * 3 + 8] = np.array([(9 << 14) | (6 << 28)], np.uint32).view(np.uint8)
    y = orc.dequant(orc.IQ2_XXS, b, 256).reshape(8, 4, 8)
    db = np.float32(6.5 * 0.25)
    sgn = np.where((ks[9] >> np.arange(8)) & 1, -1.0, 1.0).astype(np.float32)
    assert np.array_equal(y[3, 0], db * gxx[10].astype(np.float32)) and np.array_equal(y[3, 2], db * gxx[200].astype(np.float32) * sgn)
    assert np.array_equal(y[3, 1], np.full(8, db * 8)) and np.array_equal(y[2], np.full((4, 8), 1.0, np.float32))
    # IQ2_S: sub-block 6: index byte 1 = 0x55 with high bits 2 (qh bits 2..3) -> entry 0x255; sign byte for group 1; scale nibbles 3 / 12
    b = _blk(82, 1.0); b[2 + 4 * 6 + 1] = 0x55; b[66 + 6] = 2 << 2; b[34 + 4 * 6 + 1] = 0b10000001; b[74 + 6] = 3 | (12 << 4)
    y = orc.dequant(orc.IQ2_S, b, 256).reshape(8, 4, 8)
    lo, hi = np.float32(3.5 * 0.25), np.float32(12.5 * 0.25)
    exp1 = lo * gs[0x255].astype(np.float32); exp1[0] *= -1; exp1[7] *= -1
    assert np.array_equal(y[6, 1], exp1) and np.array_equal(y[6, 0], np.full(8, lo * 8)) and np.array_equal(y[6, 2], np.full(8, hi * 8))
    # IQ3_XXS: sub-block 2: index bytes 4, 5 (group 2) = 100, 255; sign index 3 for group 2; scale bits 15
    b = _blk(98, 1.0); b[2 + 8 * 2 + 4] = 100; b[2 + 8 * 2 + 5] = 255
    b[66 + 4 * 2:66 + 4 * 2 + 4] = np.array([(3 << 14) | (15 << 28)], np.uint32).view(np.uint8)
    y = orc.dequant(orc.IQ3_XXS, b, 256).reshape(8, 4, 8)
    db = np.float32(15.5 * 0.5)
    exp = db * np.concatenate([g3x[100], g3x[255]]).astype(np.float32); exp[0] *= -1; exp[1] *= -1
    assert np.array_equal(y[2, 2], exp) and np.array_equal(y[2, 0], np.full(8, db * 4))


@pytest.mark.parametrize("ty", FMTS + FMTS_MORE)
def test_oracle_dequant_bit_equal_to_numpy_on_random_blocks(ty):
    el, bs, _ = synth.GEOM[ty]
    nb = 4096
    raw = synth.blocks(ty, nb, seed=1000 + ty)
    a = orc.dequant(ty, raw, nb * el); b = np_ref.dequant(ty, raw, nb * el)
    assert np.array_equal(bits(a), bits(b))
    # fully random bytes, including the f16 scale fields (inf/nan/subnormal patterns), must agree too
    raw2 = np.random.Generator(np.random.PCG64(7)).integers(0, 256, nb * bs, dtype=np.uint8)
    with np.errstate(all="ignore"):
        a = orc.dequant(ty, raw2, nb * el); b = np_ref.dequant(ty, raw2, nb * el)
    ok = (bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b))
    assert ok.all()


@pytest.mark.parametrize("ty", [orc.IQ3_S, orc.IQ2_XS])
def test_value_bounds_follow_from_codebooks(ty):
    raw = synth.blocks(ty, 2048, seed=5, d_lo=1.0, d_hi=1.0)
    y = np.abs(orc.dequant(ty, raw, 2048 * 256))
    assert y.max() <= (31 * 15 if ty == orc.IQ3_S else 3.875 * 43)
    assert y.min() >= (1.0 if ty == orc.IQ3_S else 0.125 * 8)


# ---- dot / matmul --------------------------------------------------------------------------------------------
def test_dot_small_integers_exact_and_tail():
    for n in (1, 7, 8, 31, 32, 33, 40, 100, 4096):
        a = (np.arange(n) % 13 - 6).astype(np.float32); b = (np.arange(n) % 7 - 3).astype(np.float32)
        assert orc.dot(a, b) == float(np.dot(a.astype(np.float64), b.astype(np.float64)))


@pytest.mark.parametrize("ty", FMTS + FMTS_MORE + [orc.BF16])
def test_matmul_index_contract_and_accuracy(ty):
    rows, cols, t = 48, 512, 3
    raw = synth.matrix(ty, rows, cols, seed=33) if ty != orc.BF16 else synth.bf16_normal(rows, cols, 3, 0.02)
    x = synth.normal((t, cols), seed=9)
    y = orc.matmul(ty, raw, rows, cols, x)
    W = np_ref.dequant(ty, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    truth = x.astype(np.float64) @ W.T                               # y[ti][r] = sum_c W[r,c] x[ti][c]
    assert y.shape == (t, rows)
    assert np.abs(y - truth).max() / np.abs(truth).max() <= 1e-5


# ---- KV4 (reference tests kv4.rs:52-104) -----------------------------------------------------------------------
def test_kv4_reference_roundtrip_vector():
    i = np.arange(256, dtype=np.float32)
    t = (i * np.float32(0.017) - np.float32(1.3)).astype(np.float32)
    x = np.where(np.arange(256) % 32 == 7, t * np.float32(4.0), t * np.float32(0.15)).astype(np.float32)
    w, s = orc.kv4_pack(x)
    assert w.size == 32 and s.size == 8
    y = orc.kv4_unpack(w, s, 256)
    z = orc.kvq_roundtrip(x, 4)
    assert (np.abs(y - z) <= 1e-5 * np.maximum(np.abs(z), 1.0)).all()
    assert (np.abs(y - x) <= np.repeat(s, 32) * 0.5 + 1e-6).all()
    e4 = np.abs(x - y).mean(); e8 = np.abs(x - orc.kvq_roundtrip(x, 8)).mean()
    assert e8 < e4 and e4 > 2 * e8 and e4 < 0.2
    # independent numpy statement, bit for bit (codes and scales too)
    rt, q, sc = np_ref.kv4_roundtrip(x)
    assert np.array_equal(bits(rt), bits(y)) and np.array_equal(bits(sc), bits(s))
    nib = np.array([(w[i // 8] >> (4 * (i % 8))) & 0xF for i in range(256)])
    assert np.array_equal(np.where(nib >= 8, nib.astype(int) - 16, nib), q)


def test_kv4_zero_block_extremes_and_sign_extension():
    w0, s0 = orc.kv4_pack(np.zeros(32, np.float32))
    assert np.array_equal(orc.kv4_unpack(w0, s0, 32), np.zeros(32, np.float32))
    ext = np.ones(32, np.float32); ext[31] = -1.0
    we, se = orc.kv4_pack(ext)
    back = orc.kv4_unpack(we, se, 32)
    assert abs(back[31] + 1.0) < 1e-5 and (we[3] >> 28) == 0x9      # -7 stored as two's complement nibble 9
    x = np.zeros(32, np.float32); x[0] = -0.7; x[1] = 0.7
    w, s = orc.kv4_pack(x)
    assert s[0] > 0 and (w[0] & 0xF) >= 8 and ((w[0] >> 4) & 0xF) < 8
    y = orc.kv4_unpack(w, s, 32)
    assert abs(y[0] - x[0]) <= s[0] * 0.5 + 1e-6 and abs(y[1] - x[1]) <= s[0] * 0.5 + 1e-6
    bad = np.ones(32, np.float32); bad[3] = np.inf
    wb, sb = orc.kv4_pack(bad)
    assert sb[0] == 0.0 and not wb.any()


def test_kv4_random_matches_numpy():
    x = synth.normal((64 * 32,), seed=4, std=3.0)
    w, s = orc.kv4_pack(x)
    rt, _, sc = np_ref.kv4_roundtrip(x)
    assert np.array_equal(bits(orc.kv4_unpack(w, s, x.size)), bits(rt))
    assert np.array_equal(orc.kvq_roundtrip(x, 4), rt)   # value equality: the in-place round trip keeps -0.0


def test_packed_boundary_rule():
    assert orc.packed_boundary(1024 + 64) == 0
    assert orc.packed_boundary(1024 + 65) == 64
    assert orc.packed_boundary(32768) == 31744
    assert orc.packed_boundary(32769) == 31744
    assert orc.packed_boundary(32768, kv_bits=0) == 0


# ---- rope table, argmax, top-k -----------------------------------------------------------------------------------
def test_rope_inv_closed_form():
    inv = orc.rope_inv(64, 1e7)                       # qn_ctx.rs:406-411
    assert inv[0] == 1.0 and inv.size == 32
    exp = np.float64(1e7) ** (-2.0 * np.arange(32) / 64.0)
    assert np.abs(inv - exp).max() / exp.max() < 1e-6 and (np.diff(inv) < 0).all()


def test_argmax_first_max():
    assert orc.argmax([1.0, 3.0, 2.0, 0.5, 2.9]) == 1      # sampler.rs:154-159
    assert orc.argmax([2.0, 5.0, 5.0, 1.0]) == 1
    assert orc.argmax([np.nan, 1.0, 0.0]) == 0             # comparisons with NaN are false: index 0 stays


def test_top_k_bruteforce_ties_and_nan():
    g = np.random.Generator(np.random.PCG64(3))
    for n, k in ((8, 2), (64, 10), (512, 10)):
        r = g.standard_normal(n).astype(np.float32)
        idx, w = orc.top_k(r, k); ridx, rw = np_ref.top_k(r, k)
        assert np.array_equal(idx, ridx) and np.abs(w - rw).max() < 1e-6 and abs(w.sum() - 1) < 1e-6
    r = np.array([1.0, 2.0, 2.0, 2.0, 0.0, 2.0], np.float32)
    idx, w = orc.top_k(r, 3)
    assert list(idx) == [1, 2, 3] and np.allclose(w, 1 / 3)
    r = np.array([np.nan, 0.5, np.nan, 0.25], np.float32)
    idx, w = orc.top_k(r, 2)
    assert list(idx) == [1, 3]
    idx, w = orc.top_k(np.full(4, np.nan, np.float32), 2)
    assert list(idx) == [0, 1] and np.allclose(w, 0.5)
