"""The oracle's per-layer n-gram embeddings (ple_rows / ple, qwen4exp_gguf.rs:1390-1434) pinned by cases whose answer the
definition fixes: hashes that reduce to a single token of the context, the cut at the start of the sequence and at the
eos token, 64-bit wrap-around; a zero value matrix (only the conv over the history remains, one tap at a time), a zero
key (the gate's floor), one-hot keys and streams (the gate in closed form), constant gated streams (the normalised row
is the norm weight), and the shift of the history."""
import math

import numpy as np

import orc
from pyre_amd import synth


def cfg(d=64, hc=2, ngram=3, per_gram=1, conv_k=3, dim=32, eos=5, mult=(1, 0, 0), off=(0, 0), vocab=(1000, 1000), eps=1e-6):
    c = orc.Cfg(); c.d = d; c.hc = hc; c.eps = eps
    c.ple_ngram = ngram; c.ple_per_gram = per_gram; c.ple_conv_k = conv_k; c.ple_dim = dim; c.ple_eos = eos
    for i, v in enumerate(mult): c.ple_mult[i] = v
    for i, v in enumerate(off): c.ple_off[i] = v
    for i, v in enumerate(vocab): c.ple_vocab[i] = v
    return c


def table(rows, dim):
    t = (np.arange(rows, dtype=np.float32)[:, None] * 100.0 + np.arange(dim, dtype=np.float32)[None, :]).copy()      # row r = 100 r + column
    return t, orc.Tensor(synth.F32, rows, dim, t.ctypes.data)


def test_rows_pick_the_token_the_multipliers_single_out():
    tab, tt = table(64, 32)
    toks = np.array([11, 3, 5, 9, 20, 21], dtype=np.uint32)          # eos = 5 at position 2
    # head 0: 2-grams, head 1: 3-grams; only the current token counts: row = token % 40 + offset
    c = cfg(mult=(1, 0, 0), off=(0, 10), vocab=(40, 40))
    e = orc.ple_rows(c, tt, toks, 0, 6).reshape(6, 2, 32)
    for p, tk in enumerate(toks):
        assert e[p, 0, 0] == 100.0 * (tk % 40) and e[p, 1, 0] == 100.0 * (tk % 40 + 10) and e[p, 0, 7] == e[p, 0, 0] + 7
    # only the previous token counts (both heads): position 0 has none -> eos; the token after the eos sees the eos itself
    c = cfg(mult=(0, 1, 0), off=(0, 0), vocab=(64, 64))
    e = orc.ple_rows(c, tt, toks, 0, 6).reshape(6, 2, 32)
    assert [int(e[p, 0, 0] / 100) for p in range(6)] == [5, 11, 3, 5, 9, 20]
    # only the token two back counts, in the 3-gram head; the 2-gram head (j < 2) never sees it -> row 0
    c = cfg(mult=(0, 0, 1), off=(0, 0), vocab=(64, 64))
    e = orc.ple_rows(c, tt, toks, 0, 6).reshape(6, 2, 32)
    assert [int(e[p, 0, 0] / 100) for p in range(6)] == [0] * 6
    # p = 0, 1: cut by the start; p = 2: two back = 11; p = 3: one back is the eos -> cut, everything further is eos;
    # p = 4: two back is the eos (an eos in the context reads as itself); p = 5: two back = 9
    assert [int(e[p, 1, 0] / 100) for p in range(6)] == [5, 5, 11, 5, 5, 9]
    # a window that starts inside the history sees the same rows
    assert np.array_equal(orc.ple_rows(c, tt, toks, 3, 3), e.reshape(6, -1)[3:6])


def test_rows_hash_wraps_at_64_bits_and_combines_by_xor():
    tab, tt = table(64, 32)
    toks = np.array([3, 6], dtype=np.uint32)
    m0 = (1 << 63) + 1
    c = cfg(ngram=2, mult=(m0, 0), off=(0,), vocab=(61,))
    want = ((3 * m0) % (1 << 64)) % 61                       # 3 * (2^63 + 1) wraps to 2^63 + 3
    assert ((3 * m0) % (1 << 64)) == (1 << 63) + 3
    e = orc.ple_rows(c, tt, toks, 0, 1)
    assert e[0, 0] == 100.0 * want
    c = cfg(ngram=2, mult=(1, 1), off=(0,), vocab=(64,))      # xor of the two tokens: 6 ^ 3 = 5, not 9
    assert orc.ple_rows(c, tt, toks, 1, 1)[0, 0] == 500.0


def mats(c, key, value):
    key = np.ascontiguousarray(key, dtype=np.float32); value = np.ascontiguousarray(value, dtype=np.float32)
    ein = (c.ple_ngram - 1) * c.ple_per_gram * c.ple_dim
    assert key.shape == (c.hc * c.d, ein) and value.shape == (c.d, ein)
    return key, value, orc.Tensor(synth.F32, key.shape[0], ein, key.ctypes.data), orc.Tensor(synth.F32, c.d, ein, value.ctypes.data)


def test_zero_value_leaves_only_the_conv_over_the_history_one_tap_at_a_time():
    c = cfg(ngram=2, conv_k=3, dim=32)          # dilation 2, history of 4 rows
    w = c.hc * c.d; ein = 32
    k, v, kt, vt = mats(c, np.ones((w, ein)), np.zeros((c.d, ein)))
    ones = np.ones(w, np.float32); emb = np.ones((1, ein), np.float32)
    x0 = np.linspace(-1, 1, w, dtype=np.float32)
    silu = lambda o: o / (1.0 + math.exp(-o))
    for tap, row in ((0, 0), (1, 2)):            # tap k lies (K-1-k) * 2 positions back: rows hl - 4 = 0 and hl - 2 = 2 of the oldest-first history
        hist = np.stack([np.full(w, r + 1.0, np.float32) for r in range(4)])
        conv = np.zeros((w, 3), np.float32); conv[:, tap] = 0.5
        y = orc.ple(c, kt, vt, ones, ones, ones, conv.reshape(-1), hist, emb, x0)
        assert np.allclose(y[0] - x0, silu(0.5 * (row + 1.0)), rtol=0, atol=1e-6), tap
        # the history moved up by one row and took the new (zero) normalised row at the end
        assert np.array_equal(hist[:3], np.stack([np.full(w, r + 2.0, np.float32) for r in range(3)])) and not hist[3].any()
    hist = np.ones((4, w), np.float32); conv = np.zeros((w, 3), np.float32); conv[:, 2] = 9.0      # the tap on the current row: that row is zero here
    y = orc.ple(c, kt, vt, ones, ones, ones, conv.reshape(-1), hist, emb, x0)
    assert np.array_equal(y[0], x0)              # silu(0) = 0, gated = 0


def test_zero_key_gives_the_gate_floor_and_constant_streams_normalise_to_the_norm_weight():
    c = cfg(ngram=2, conv_k=2, dim=32)           # history of 2 rows... (conv_k - 1) * ngram
    w = c.hc * c.d; ein = 32
    k, v, kt, vt = mats(c, np.zeros((w, ein)), np.full((c.d, ein), 1.0 / ein))       # value . emb = 1 in every channel
    emb = np.ones((1, ein), np.float32)
    nc = np.linspace(0.5, 1.5, w).astype(np.float32)
    conv = np.zeros((w, 2), np.float32); conv[:, 1] = 2.0                             # current row only
    hist = np.zeros((2, w), np.float32)
    x0 = np.random.Generator(np.random.PCG64(1)).standard_normal(w).astype(np.float32)
    y = orc.ple(c, kt, vt, np.ones(w, np.float32), np.ones(w, np.float32), nc, conv.reshape(-1), hist, emb, x0)
    g = 1.0 / (1.0 + math.exp(-1e-3))            # key = 0 -> score +0 -> sign +1, |score| floored at 1e-6, sqrt -> 1e-3
    # gated = g in every channel; a constant stream normalises to 1 (times the norm weight); conv = 2 * nrm
    nrm = nc.astype(np.float64) / math.sqrt(1.0 + c.eps / (g * g))
    o = 2.0 * nrm
    want = x0 + (g + o / (1.0 + np.exp(-o)))
    assert np.allclose(y[0], want, rtol=0, atol=2e-6)
    assert np.allclose(hist[1], nrm, rtol=0, atol=1e-6) and not hist[0].any()


def test_one_hot_key_and_stream_give_the_gate_in_closed_form_per_stream():
    c = cfg(d=64, hc=2, ngram=2, conv_k=2, dim=32)
    d, w, ein = c.d, c.hc * c.d, 32
    key = np.zeros((w, ein), np.float32); key[0 * d + 3, 0] = 2.0; key[1 * d + 9, 0] = -4.0      # stream 0: channel 3, stream 1: channel 9 (negative)
    k, v, kt, vt = mats(c, key, np.full((d, ein), 1.0 / ein))
    emb = np.ones((1, ein), np.float32)
    nk = np.full(w, 0.5, np.float32); nq = np.full(w, 2.0, np.float32)
    x0 = np.zeros(w, np.float32); x0[0 * d + 3] = 7.0; x0[1 * d + 9] = 3.0
    conv = np.zeros((w, 2), np.float32); hist = np.zeros((2, w), np.float32)
    y = orc.ple(c, kt, vt, nk, nq, np.ones(w, np.float32), conv.reshape(-1), hist, emb, x0)
    # rms of a one-hot vector a e_i is sign(a) sqrt(d) e_i (eps negligible): key -> +-sqrt(d) * 0.5, stream -> sqrt(d) * 2,
    # dot = +-d, score = +-sqrt(d) = +-8, gate = sigmoid(+-sqrt(8))
    g0 = 1.0 / (1.0 + math.exp(-math.sqrt(8.0))); g1 = 1.0 / (1.0 + math.exp(math.sqrt(8.0)))
    assert np.allclose(y[0, :d] - x0[:d], g0, rtol=0, atol=1e-5) and np.allclose(y[0, d:] - x0[d:], g1, rtol=0, atol=1e-5)


def test_tokens_of_a_window_are_processed_in_order_against_the_shifting_history():
    # two tokens in one call == two calls of one token
    c = cfg(ngram=2, conv_k=3, dim=32)
    w = c.hc * c.d; ein = 32
    g = np.random.Generator(np.random.PCG64(5))
    k, v, kt, vt = mats(c, g.standard_normal((w, ein)), g.standard_normal((c.d, ein)))
    nk, nq, nc = (1 + 0.1 * g.standard_normal(w).astype(np.float32) for _ in range(3))
    conv = g.standard_normal(w * 3).astype(np.float32); emb = g.standard_normal((2, ein)).astype(np.float32)
    x0 = g.standard_normal((2, w)).astype(np.float32); h0 = g.standard_normal((4, w)).astype(np.float32)
    ha = h0.copy(); ya = orc.ple(c, kt, vt, nk, nq, nc, conv, ha, emb, x0)
    hb = h0.copy(); yb0 = orc.ple(c, kt, vt, nk, nq, nc, conv, hb, emb[:1], x0[:1]); yb1 = orc.ple(c, kt, vt, nk, nq, nc, conv, hb, emb[1:], x0[1:])
    assert np.array_equal(ya[0], yb0[0]) and np.array_equal(ya[1], yb1[0]) and np.array_equal(ha, hb)
    assert np.array_equal(ha[:2], h0[2:])        # two rows left, two came in
