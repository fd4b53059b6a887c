"""The vectors the reference's own unit tests hold for this path (tests/golden/reference_vectors.json), against the
oracle and the library's host-only entry points.  No GPU."""
import json
import os

import numpy as np

import orc
from pyre_amd import lib

G = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.json")))


def test_sampler_argmax_vector():
    for c in G["sampler_argmax"]["cases"]:
        assert orc.argmax(c["logits"]) == c["expect"]


def test_ngram_draft_vectors():
    for c in G["ngram_draft"]["cases"]:
        assert lib.ngram_draft(c["history"], c["k"], c["min_n"], c["max_n"]).tolist() == c["expect"]


def test_rope_inv_vector():
    r = G["rope_inv"]
    inv = orc.rope_inv(r["n_rot"], r["base"])
    assert inv[0] == r["expect_first"] and inv.size == r["n_rot"] // 2
    exp = np.float64(r["base"]) ** (-2.0 * np.arange(r["n_rot"] // 2) / r["n_rot"])
    assert np.abs(inv - exp).max() / exp.max() < r["rel_tol"]


def test_kv4_roundtrip_vector():
    k = G["kv4_roundtrip"]
    i = np.arange(k["n"], dtype=np.float32)
    t = (i * np.float32(0.017) - np.float32(1.3)).astype(np.float32)
    x = np.where(np.arange(k["n"]) % 32 == 7, t * np.float32(4.0), t * np.float32(0.15)).astype(np.float32)
    w, s = orc.kv4_pack(x)
    assert w.size == k["words"] and s.size == k["scales"]
    y = orc.kv4_unpack(w, s, k["n"]); z = orc.kvq_roundtrip(x, 4)
    assert (np.abs(y - z) <= 1e-5 * np.maximum(np.abs(z), 1.0)).all()
    assert (np.abs(y - x) <= np.repeat(s, 32) * 0.5 + 1e-6).all()
    e4 = np.abs(x - y).mean(); e8 = np.abs(x - orc.kvq_roundtrip(x, 8)).mean()
    assert e4 > 2 * e8 and e4 < 0.2
    ext = np.ones(32, np.float32); ext[31] = -1.0
    we, se = orc.kv4_pack(ext)
    assert abs(orc.kv4_unpack(we, se, 32)[31] + 1.0) < 1e-5 and (we[3] >> 28) == 0x9
    w0, s0 = orc.kv4_pack(np.zeros(32, np.float32))
    assert not orc.kv4_unpack(w0, s0, 32).any() and s0[0] == 0.0
