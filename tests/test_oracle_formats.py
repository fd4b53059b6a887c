"""Pins the CPU oracle's wire formats (no GPU): codebooks, the four block dequantizers, dot / matmul, KV4, RoPE
table, argmax, top-k.  Known answers are derived from the format definitions (gguf_q.rs:79,103-107,126-129,141-151
of the reference), not from the oracle's own code."""
import numpy as np
import pytest

import np_ref
import orc
from pyre_amd import synth

FMTS = [orc.Q8_0, orc.Q4_K, orc.IQ2_XS, orc.IQ3_S]


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_codebook_digests_match_reference_tables():
    for hdr in ("oracle/iq_codebooks.h", "pyre_amd/csrc/iq_codebooks.h"):
        import os
        p = os.path.join(np_ref._ROOT, hdr)
        assert np_ref.codebook_digests(p) == (np_ref.IQ3S_SHA256, np_ref.IQ2XS_SHA256, np_ref.KSIGNS_SHA256)


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


@pytest.mark.parametrize("ty", FMTS)
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


@pytest.mark.parametrize("ty", FMTS + [orc.BF16])
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
