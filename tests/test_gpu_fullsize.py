"""The benchmark's real dimensions (d 2048, 512 experts top-10, 16/32 DeltaNet heads, 16/2 attention heads of 256,
vocabulary 151936, IQ3_S) on a few layers: size-independent properties at full width, and one comparison with the
oracle on a two-layer slice (one Gated DeltaNet + one attention layer), the size it finishes in seconds."""
import os

import numpy as np
import pytest

import orc
from helpers import orc_model, relerr
from pyre_amd import lib
from pyre_amd import modelgen as mg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def model4(ctx):
    cfg = mg.a3b_config(n_layers=4)
    layers, globals_, raw = mg.build_device(ctx, cfg, seed=5)
    m = lib.Model(ctx, cfg, layers, globals_)
    for p in raw:
        ctx.free(p)
    return cfg, m


def test_verify_window_equals_single_steps_and_rollback_at_full_width(model4):
    cfg, gm = model4
    g = np.random.Generator(np.random.PCG64(3))
    prompt = g.integers(0, cfg.vocab, 37, dtype=np.uint32)
    sa, sb = gm.new_state(128), gm.new_state(128)
    gm.forward(prompt, sa, want_logits=False); gm.forward(prompt, sb, want_logits=False)
    toks = g.integers(0, cfg.vocab, 5, dtype=np.uint32)
    lv = gm.forward_multi(toks, sa)
    singles = np.array([gm.forward(toks[i:i + 1], sb) for i in range(5)])
    assert np.array_equal(lv.view(np.uint32), singles.view(np.uint32))
    gm.spec_keep(sa, 5, 2)                                                   # keep two of the five
    sc = gm.new_state(128); gm.forward(np.concatenate([prompt, toks[:2]]), sc, want_logits=False)
    nxt = np.array([toks[2] ^ 1], dtype=np.uint32)
    la, lc = gm.forward(nxt, sa), gm.forward(nxt, sc)                         # rolled back == never drafted
    assert len(sa) == len(sc) == 40 and np.array_equal(la.view(np.uint32), lc.view(np.uint32))


def test_device_loop_host_loop_and_snapshot_agree_at_full_width(model4):
    cfg, gm = model4
    g = np.random.Generator(np.random.PCG64(4))
    prompt = g.integers(0, cfg.vocab, 21, dtype=np.uint32)
    st = gm.new_state(128)
    lg = gm.forward(prompt, st); first = int(np.argmax(lg))
    snap = st.snapshot()
    a = gm.decode_greedy_dev(st, first, 24)
    st.restore(snap)
    host = []; tok = first                                                    # the host-driven loop: forward + argmax per token
    for _ in range(24):
        lg = gm.forward(np.array([tok], dtype=np.uint32), st); tok = int(orc.argmax(lg)); host.append(tok)
    assert np.array_equal(a, np.array(host, dtype=np.uint32))
    st.restore(snap)
    os.environ["PYRE_NO_GRAPH"] = "1"                                         # the same step as ordinary launches instead of a replayed graph
    try:
        b = gm.decode_greedy_dev(st, first, 24)
    finally:
        os.environ.pop("PYRE_NO_GRAPH", None)
    assert np.array_equal(a, b)


def test_two_layer_slice_matches_the_oracle_at_full_width(ctx):
    cfg = mg.a3b_config(n_layers=2, full_every=2)
    hw = mg.build_host(cfg, seed=8)
    gm = lib.Model(ctx, cfg, hw.layers, hw.globals_); om = orc_model(hw, threads=min(os.cpu_count() or 1, 16))
    g = np.random.Generator(np.random.PCG64(9))
    prompt = g.integers(0, cfg.vocab, 10, dtype=np.uint32)
    gs, os_ = gm.new_state(64), om.new_state()
    lg, lo = gm.forward(prompt, gs), om.forward(prompt, os_)
    assert relerr(lg, lo) <= 1e-3 and relerr(lg, lo) <= 1e-4
    tg, _ = gm.generate_greedy(gs, lg, 6); to, _ = om.generate_greedy(os_, lo, 6)
    assert np.array_equal(tg, to)
    conv, ssm = gs.gdn(0)
    assert relerr(ssm, os_.ssm(0)) <= 1e-4 and relerr(conv, os_.conv(0)) <= 1e-5


def test_drafter_matches_the_oracle_at_full_width(ctx):
    # the drafter block at the benchmark's width (4 streams of 2048, 512 experts top-10 of width 512, 16 / 2 heads of
    # 256) over a two-layer model; a 4096-row draft head
    import helpers
    cfg = mg.a3b_config(n_layers=2, full_every=2)
    hw = mg.build_host(cfg, seed=8)
    ids = (np.arange(4096, dtype=np.uint32) * 37) % cfg.vocab
    mt = mg.build_mtp_host(cfg, hw, 512, 512, ids, seed=18)
    gm = lib.Model(ctx, cfg, hw.layers, hw.globals_); om = orc_model(hw, threads=min(os.cpu_count() or 1, 16))
    gd = lib.Mtp(gm, 512, 10, 512, 128, mt, ids); od = helpers.orc_mtp(om, mt, 512, 10, 512, 128, ids)
    g = np.random.Generator(np.random.PCG64(19))
    prompt = g.integers(0, cfg.vocab, 11, dtype=np.uint32)
    gs, os_ = gm.new_state(64), om.new_state(); gd.attach(gs); od.attach(os_)
    lg, lo = gm.forward(prompt, gs), om.forward(prompt, os_)
    assert relerr(lg, lo) <= 1e-3
    pending = int(orc.argmax(lo))
    gi, gp = gd.draft(gs, pending, 3); oi, op = od.draft(os_, pending, 3)
    assert list(gi) == list(oi) and np.allclose(gp, op, rtol=2e-3, atol=0)
    gc0, gk, gv = gd.kv(gs); oc0, ok, ov = od.kv(os_)
    assert (gc0, len(gk)) == (oc0, len(ok)) == (0, 11) and relerr(gk, ok) <= 1e-5 and relerr(gv, ov) <= 1e-5
    out, rounds, drafted, accepted = gd.generate_greedy(gs, lg, 9, k=3)
    oo, od_n, oa_n = od.generate_greedy(os_, lo, 9, k=3)
    assert np.array_equal(out, oo) and (drafted, accepted) == (od_n, oa_n)


def test_prompt_in_blocks_with_the_ffn_grouped_by_expert_agrees_with_the_windows_path(ctx, model4, monkeypatch):
    """A long prompt takes blocks of up to 128 windows layer by layer, the FFN of a block's tokens grouped by expert on the
    matrix cores: logits agree with the windows' path (PYRE_PROMPT_WINDOWS=1 at run time) to rounding, the tokens that follow
    and the state's length are the same, for a call that is whole blocks plus a ragged tail, and for a state that continues
    with a second long call."""
    cfg, gm = model4
    g = np.random.Generator(np.random.PCG64(21))
    prompt = g.integers(0, cfg.vocab, 2 * 256 + 45, dtype=np.uint32)
    more = g.integers(0, cfg.vocab, 256 + 100 + 9, dtype=np.uint32)          # a full block and a shorter one
    out = {}
    modes = ("0", "1", "1 one block at a time", "1 groups of 5", "1 a launch a window", "1 projection in the chain", "1 attention in the chain", "1 router riding")
    for mode in modes:
        monkeypatch.setenv("PYRE_PROMPT_WINDOWS", "1" if mode == "0" else "0")
        monkeypatch.setenv("PYRE_PROMPT_PAIRS", "0" if mode == "1 one block at a time" else "1")     # two blocks in flight, one's FFN beside the other's windows
        monkeypatch.setenv("PYRE_PROMPT_GROUP", "5" if mode == "1 groups of 5" else "0")              # consecutive windows a stream takes together
        monkeypatch.setenv("PYRE_PROMPT_BATCH", "0" if mode == "1 a launch a window" else "1")        # a group's mixes, projections, convolution and recurrences in one launch each
        monkeypatch.setenv("PYRE_PROMPT_PROJ_EARLY", "0" if mode == "1 projection in the chain" else "1")     # projection (and convolution) outside the chain through the layer's state
        monkeypatch.setenv("PYRE_PROMPT_ATTN_SPLIT", "0" if mode == "1 attention in the chain" else "1")      # the pass over the cache outside it
        monkeypatch.setenv("PYRE_PROMPT_ROUTER_APART", "0" if mode == "1 router riding" else "1")           # the router's sums with the block's FFN launches, not on every window's FFN mix
        st = gm.new_state(1024)
        n0 = gm.prompt_blocks()
        lg = gm.forward(prompt, st)
        assert gm.prompt_blocks() - n0 == (0 if mode == "0" else 1 if mode == "1 one block at a time" else 2)          # the path under test is the one that ran (68 whole windows: a pair of blocks, or one)
        toks = gm.decode_greedy_dev(st, int(np.argmax(lg)), 6)
        lg2 = gm.forward(more, st)                                           # (starts at a position that is no multiple of eight)
        toks2 = gm.decode_greedy_dev(st, int(np.argmax(lg2)), 4)
        out[mode] = (lg.copy(), toks.copy(), lg2.copy(), toks2.copy(), len(st))
        st.close()
    a, b = out["0"], out["1"]
    for other in modes[2:]:          # the order and the grouping of the launches do not change a bit
        for i in range(4):
            assert np.array_equal(np.asarray(b[i]).view(np.uint32), np.asarray(out[other][i]).view(np.uint32)), (other, i)
    assert a[4] == b[4] == prompt.size + 6 + more.size + 4
    assert relerr(b[0], a[0]) <= 1e-4 and np.array_equal(a[1], b[1])
    assert relerr(b[2], a[2]) <= 1e-4 and np.array_equal(a[3], b[3])


def test_prompt_in_blocks_at_a_long_context_agrees_with_the_windows_path(model4, monkeypatch):
    """20 000 tokens (the 4-bit boundary of the caches moves some three hundred times, the attention passes cover many chunks,
    twenty blocks in ten calls' worth of pairs): logits within 1e-4 of the windows' path, the same tokens after it."""
    cfg, gm = model4
    prompt = np.random.Generator(np.random.PCG64(27)).integers(0, cfg.vocab, 20000, dtype=np.uint32)
    out = {}
    for mode in ("1", "0"):
        monkeypatch.setenv("PYRE_PROMPT_WINDOWS", mode)
        st = gm.new_state(20000 + 32); n0 = gm.prompt_blocks()
        lg = gm.forward(prompt, st)
        out[mode] = (lg.copy(), gm.decode_greedy_dev(st, int(np.argmax(lg)), 8).copy(), gm.prompt_blocks() - n0)
        st.close()
    assert out["1"][2] == 0 and out["0"][2] == 20
    assert relerr(out["0"][0], out["1"][0]) <= 1e-4 and np.array_equal(out["0"][1], out["1"][1])


def test_prompt_in_blocks_matches_the_oracle_at_full_width(ctx):
    """256 tokens in a pair of blocks plus a tail through the two-layer slice against the oracle's token-by-token prompt."""
    cfg = mg.a3b_config(n_layers=2, full_every=2)
    hw = mg.build_host(cfg, seed=8)
    gm = lib.Model(ctx, cfg, hw.layers, hw.globals_); om = orc_model(hw, threads=min(os.cpu_count() or 1, 16))
    g = np.random.Generator(np.random.PCG64(23))
    prompt = g.integers(0, cfg.vocab, 256 + 19, dtype=np.uint32)
    gs, os_ = gm.new_state(512), om.new_state()
    lg = gm.forward(prompt, gs)
    assert gm.prompt_blocks() == 2          # 33 whole windows in front of the last tokens: a pair of blocks
    lo = om.forward(prompt, os_)
    assert relerr(lg, lo) <= 1e-3
    tg, _ = gm.generate_greedy(gs, lg, 4); to, _ = om.generate_greedy(os_, lo, 4)
    assert np.array_equal(tg, to)
    conv, ssm = gs.gdn(0)
    assert relerr(ssm, os_.ssm(0)) <= 1e-3 and relerr(conv, os_.conv(0)) <= 1e-4
