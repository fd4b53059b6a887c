"""GPU parity of the layer API (forward / forward_multi / spec_keep / greedy generation) against the CPU oracle on
small configurations the oracle finishes in seconds.  Logits: max|d| / max|logit| <= 1e-3 (in practice ~1e-6),
greedy token streams identical."""
import numpy as np
import pytest

import orc
from helpers import orc_model, relerr
from pyre_amd import lib, synth
from pyre_amd import modelgen as mg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


def small_cfg(**kw):
    c = mg.Config(n_layers=4, d=256, hc=2, hc_lr=64, n_exp=8, top_k=2, ff_exp=256, vocab=512, kv_recent=64)
    for k, v in kw.items():
        setattr(c, k, v)
    return c


def pair(ctx, c, seed, max_ctx=512):
    hw = mg.build_host(c, seed=seed)
    gm = lib.Model(ctx, c, hw.layers, hw.globals_)
    om = orc_model(hw)
    return hw, gm, om


@pytest.mark.parametrize("qtype,hc_type", [(synth.IQ3_S, synth.BF16), (synth.IQ3_S, synth.IQ3_S), (synth.Q4_K, synth.F32), (synth.IQ2_XS, synth.F16), (synth.Q8_0, synth.BF16),
                                           (synth.IQ4_XS, synth.BF16), (synth.IQ2_S, synth.Q6_K), (synth.IQ3_XXS, synth.IQ4_XS), (synth.Q6_K, synth.F32), (synth.IQ2_XXS, synth.BF16),
                                           (synth.Q5_K, synth.Q3_K), (synth.Q3_K, synth.Q5_K)])
def test_forward_logits_and_state_match_oracle(ctx, qtype, hc_type):
    c = small_cfg(qtype=qtype, hc_type=hc_type, hc_lr=256 if synth.GEOM[hc_type][0] == 256 else 64)
    hw, gm, om = pair(ctx, c, 5)
    ids = np.array([3, 77, 500, 12, 9, 311, 4, 4, 250, 17, 88], dtype=np.uint32)
    gs, os_ = gm.new_state(64), om.new_state()
    lg = gm.forward(ids, gs); lo = om.forward(ids, os_)            # prefill of 11 tokens (windows of 8 + 3)
    assert relerr(lg, lo) <= 1e-3 and relerr(lg, lo) <= 1e-4
    assert orc.argmax(lg) == orc.argmax(lo) and len(gs) == len(os_) == 11
    for i in range(4):                                              # then token by token
        tok = np.array([orc.argmax(lo)], dtype=np.uint32)
        lg = gm.forward(tok, gs); lo = om.forward(tok, os_)
        assert relerr(lg, lo) <= 1e-4, i
    conv, ssm = gs.gdn(0)
    assert relerr(ssm, os_.ssm(0)) <= 1e-4 and relerr(conv, os_.conv(0)) <= 1e-5
    k, v = gs.kv(0)
    assert relerr(k.reshape(-1), os_.kcache(0)) <= 1e-4 and relerr(v.reshape(-1), os_.vcache(0)) <= 1e-4


def test_matrix_core_layout_equals_the_lane_per_row_layout_and_the_separate_operand_split(ctx, monkeypatch):
    # the same IQ3_S model three ways: projections, head and embedding on the matrix cores with the operand left by the
    # producer kernels (default); the same with every GEMV splitting its own input; every matrix in the lane = row layout.
    # All three against the oracle, single steps and a verify window, and the same greedy stream.
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.IQ3_S, hc_lr=256)
    hw = mg.build_host(c, seed=41); om = orc_model(hw)
    prompt = np.random.Generator(np.random.PCG64(42)).integers(0, c.vocab, 21, dtype=np.uint32)
    os_ = om.new_state(); lo = om.forward(prompt, os_)
    want = []; tok = int(orc.argmax(lo))
    for _ in range(12):
        want.append(tok); tok = int(orc.argmax(om.forward(np.array([tok], dtype=np.uint32), os_)))
    outs = {}
    for name, env in (("default", {}), ("split", {"PYRE_AOP_SPLIT": "1"}), ("rows", {"PYRE_MODEL_ROWS": "1"})):
        for k in ("PYRE_AOP_SPLIT", "PYRE_MODEL_ROWS"):
            monkeypatch.delenv(k, raising=False)
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        gm = lib.Model(ctx, c, hw.layers, hw.globals_); st = gm.new_state(128)
        lg = gm.forward(prompt, st)
        assert relerr(lg, lo) <= 1e-3, name
        got = gm.decode_greedy_dev(st, int(orc.argmax(lg)), 12)
        assert [int(orc.argmax(lg))] + [int(x) for x in got[:11]] == want, name
        win = gm.forward_multi(np.array(want[:5], dtype=np.uint32), st)          # a verify window on top
        outs[name] = (lg, win)
        st.close(); gm.close()
    for name in ("split", "rows"):
        assert relerr(outs[name][0], outs["default"][0]) <= 1e-4 and relerr(outs[name][1], outs["default"][1]) <= 1e-4, name


@pytest.mark.parametrize("router_type,hc_type,rides", [(synth.BF16, synth.IQ3_S, True), (synth.F32, synth.BF16, True), (synth.F32, synth.F32, True), (synth.BF16, synth.F16, True),
                                                       (synth.F16, synth.BF16, False), (synth.BF16, synth.Q8_0, False)])
def test_router_riding_on_the_mix_equals_the_separate_router_launch(ctx, router_type, hc_type, rides, monkeypatch):
    """The router GEMV as K slices left by the mix's second launch (bf16 / f32 routers behind IQ3_S / bf16 / f16 / f32
    mixes) against the separate launch: same experts, logits within 1e-5 of each other and of the oracle's 1e-4; other
    type pairs keep the separate launch."""
    c = small_cfg(qtype=synth.IQ3_S, hc_type=hc_type, hc_lr=256 if synth.GEOM[hc_type][0] == 256 else 64, router_type=router_type, n_exp=64, top_k=6)
    hw, gm, om = pair(ctx, c, 31)
    ids = np.array([3, 77, 500, 12, 9, 311, 4, 4, 250, 17, 88, 5, 6], dtype=np.uint32)
    out = {}
    for on in ("1", "0"):
        monkeypatch.setenv("PYRE_ROUTER_RIDES", on)
        st = gm.new_state(64)
        ctx.prof_reset(); ctx.prof_enable(True)
        lg = [gm.forward(ids[:8], st), gm.forward(ids[8:], st)] + [gm.forward(ids[i:i + 1], st) for i in range(3)]
        prof = ctx.prof_report(); ctx.prof_enable(False)
        out[on] = (lg, prof)
    assert ("hc_up_mix_router" in out["1"][1]) == rides and "hc_up_mix_router" not in out["0"][1]
    os_ = om.new_state()
    lo = [om.forward(ids[:8], os_), om.forward(ids[8:], os_)] + [om.forward(ids[i:i + 1], os_) for i in range(3)]
    for a, b, o in zip(out["1"][0], out["0"][0], lo):
        assert relerr(a, b) <= 1e-5 and relerr(a, o) <= 1e-4 and orc.argmax(a) == orc.argmax(b) == orc.argmax(o)
        if not rides:
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_greedy_stream_identical_to_oracle_across_the_packing_boundary(ctx):
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 6)
    prompt = (np.arange(100, dtype=np.uint32) * 37 + 11) % c.vocab
    gs, os_ = gm.new_state(300), om.new_state()
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)
    assert relerr(lg, lo) <= 1e-4
    n = 96                                                            # context grows to 195 > recent + 64: packed region active
    out_g, _ = gm.generate_greedy(gs, lg, n)
    out_o, _ = om.generate_greedy(os_, lo, n)
    # report the oracle's top-2 margins if the streams ever split
    assert np.array_equal(out_g, out_o), "first split at %d" % int(np.argmax(out_g != out_o))
    assert len(gs) == len(os_) == 100 + n - 1 and orc.packed_boundary(len(os_), 4, 64) == 128


def test_device_loop_identical_to_oracle_across_the_packing_boundary(ctx):
    # the device-resident loop (replayed step, position on the device): the 64-position packing step rides on the
    # attention prep launch there; the stream must cross the boundary (context 129) exactly as the oracle's does
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 6)
    prompt = (np.arange(100, dtype=np.uint32) * 37 + 11) % c.vocab
    gs, os_ = gm.new_state(300), om.new_state()
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)
    n = 96
    out_o, _ = om.generate_greedy(os_, lo, n)
    first = int(np.argmax(lg))
    assert first == int(out_o[0])
    out_d = gm.decode_greedy_dev(gs, first, n - 1)
    assert np.array_equal(out_d, out_o[1:]), "first split at %d" % int(np.argmax(out_d != out_o[1:]))
    assert orc.packed_boundary(len(os_), 4, 64) == 128
    # and the state it leaves continues like the oracle's
    l2 = gm.forward(np.array([out_d[-1]], dtype=np.uint32), gs); o2 = om.forward(np.array([out_o[-1]], dtype=np.uint32), os_)
    assert relerr(l2, o2) <= 1e-3 and orc.argmax(l2) == orc.argmax(o2)


def test_device_argmax_rows_follows_the_host_scan(ctx):
    # sampler::argmax (src/sampler.rs:142-148): b = 0; for i: if l[i] > l[b] { b = i }
    def host(l):
        b = 0
        for i in range(len(l)):
            if l[i] > l[b]:
                b = i
        return b
    g = np.random.Generator(np.random.PCG64(4))
    V = 5003                                                             # not a multiple of the workgroup width
    rows = g.standard_normal((8, V)).astype(np.float32)
    rows[0, [17, 4000, 4999]] = 9.0                                      # equal maxima: the first wins
    rows[1, 0] = np.nan                                                  # a NaN at index 0 is never replaced
    rows[2, [5, 1024, 3000]] = np.nan; rows[2, 2048] = 50.0              # NaNs elsewhere are never chosen
    rows[3, :] = -np.inf                                                 # nothing is greater than the first element
    rows[4, :] = np.nan
    rows[5, 1023] = 7.0; rows[5, 1024] = 7.0                             # a tie across two threads' strides
    rows[6, V - 1] = 99.0                                                # the last element
    rows[7, 0] = 99.0
    picks = np.empty(8, dtype=np.uint32)
    ctx.check(ctx.L.pyre_argmax_rows(ctx.h, rows.ctypes.data_as(lib.C.c_void_p), 8, V, picks.ctypes.data_as(lib.C.c_void_p)), "argmax_rows")
    with np.errstate(invalid="ignore"):
        assert picks.tolist() == [host(r) for r in rows] == [17, 0, 2048, 0, 0, 1023, V - 1, 0]


def test_ngram_drafted_generation_equals_plain_greedy(ctx):
    # spec::generate with the prompt-lookup drafter (src/spec.rs:207): whatever the drafts, the stream is plain greedy's
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 8)
    pat = np.array([5, 9, 200, 31, 77, 12, 64, 3], dtype=np.uint32)
    prompt = np.concatenate([pat, pat, pat, pat[:5]])                   # a repetitive prompt: the drafter finds matches from the first round
    ga, gb, os_ = gm.new_state(200), gm.new_state(200), om.new_state()
    la = gm.forward(prompt, ga); lb = gm.forward(prompt, gb); lo = om.forward(prompt, os_)
    plain, _ = gm.generate_greedy(ga, la, 60)
    drafted, rounds, nd, na = gm.generate_greedy_ngram(gb, prompt, lb, 60, k=4, ng_min=2, ng_max=8)
    oracle, _ = om.generate_greedy(os_, lo, 60)
    assert np.array_equal(plain, oracle)
    assert np.array_equal(drafted, plain), "first split at %d" % int(np.argmax(drafted != plain))
    assert rounds > 0 and nd >= rounds and 0 <= na <= nd
    assert len(gb) == len(ga)
    # and both states continue alike
    t = np.array([plain[-1]], dtype=np.uint32)
    assert np.array_equal(gm.forward(t, ga).view(np.uint32), gm.forward(t, gb).view(np.uint32))


def test_verify_window_equals_single_steps_and_rollback(ctx):
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 7)
    prompt = np.array([5, 6, 7, 8, 9, 10, 11, 12, 13, 14], dtype=np.uint32)
    sa, sb = gm.new_state(64), gm.new_state(64)
    gm.forward(prompt, sa); gm.forward(prompt, sb)
    toks = np.array([9, 100, 11, 212, 13], dtype=np.uint32)
    lv = gm.forward_multi(toks, sa)
    singles = np.array([gm.forward(toks[i:i + 1], sb) for i in range(5)])
    assert np.array_equal(lv.view(np.uint32), singles.view(np.uint32))       # every token's arithmetic = one-token decode
    so = om.new_state(); om.forward(prompt, so); lo = om.forward_multi(toks, so)
    assert relerr(lv, lo) <= 1e-4
    # keep 2 of 5, continue: identical to a state that only ever saw those 2
    gm.spec_keep(sa, 5, 2)
    sc = gm.new_state(64); gm.forward(prompt, sc); gm.forward(toks[0:1], sc); gm.forward(toks[1:2], sc)
    assert len(sa) == len(sc) == 12
    nxt = np.array([40], dtype=np.uint32)
    assert np.array_equal(gm.forward(nxt, sa).view(np.uint32), gm.forward(nxt, sc).view(np.uint32))
    assert np.array_equal(sa.gdn(1)[1].view(np.uint32), sc.gdn(1)[1].view(np.uint32))
    with pytest.raises(lib.PyreError):
        gm.spec_keep(sa, 5, 2)                                        # not armed any more


@pytest.mark.parametrize("kind", ["plain", "iq3s_mixes", "ple", "indexer"])
def test_long_prompt_on_several_streams_equals_short_calls_on_one(ctx, kind, monkeypatch):
    monkeypatch.setenv("PYRE_PROMPT_WINDOWS", "1")          # (the windows' path: a model whose experts qualify would take the long call in blocks, equal to rounding only)
    # A call of 2 * 3 windows or more runs its windows on three streams, a window entering a layer when the previous one has
    # left that layer's state; shorter calls run on the model's own stream.  Same logits, recurrent state, caches and
    # continuation, bit for bit (250 tokens: the 4-bit boundary moves several times, ragged last window).
    if kind == "plain": c = small_cfg()
    elif kind == "iq3s_mixes": c = small_cfg(hc_lr=256, qtype=synth.IQ3_S, hc_type=synth.IQ3_S, n_exp=16, top_k=10)
    elif kind == "ple": c = mg.with_ple(small_cfg(), layers=(0, 2, 3), ngram=3, per_gram=2, conv_k=3, dim=64, eos=7)
    else: c = idx_cfg(); c.ctx = 512
    hw = mg.build_host(c, seed=41)
    gm = lib.Model(ctx, c, hw.layers, hw.globals_)
    g = np.random.Generator(np.random.PCG64(42))
    prompt = g.integers(0, c.vocab, 250, dtype=np.uint32)
    sa, sb = gm.new_state(320), gm.new_state(320)
    la = gm.forward(prompt, sa)                                     # 32 windows: three in flight
    for i in range(0, 250, 40): lb = gm.forward(prompt[i:i + 40], sb)      # 5 windows a call: one stream
    assert np.array_equal(la.view(np.uint32), lb.view(np.uint32))
    n_lin = sum(1 for il in range(c.n_layers) if not c.full(il))
    for li in range(n_lin):
        ca, xa = sa.gdn(li); cb, xb = sb.gdn(li)
        assert np.array_equal(ca.view(np.uint32), cb.view(np.uint32)) and np.array_equal(xa.view(np.uint32), xb.view(np.uint32)), li
    for ai in range(c.n_layers - n_lin):
        ka, va = sa.kv(ai); kb, vb = sb.kv(ai)
        assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32)) and np.array_equal(va.view(np.uint32), vb.view(np.uint32)), ai
    more = g.integers(0, c.vocab, 60, dtype=np.uint32)              # and again on top of the state a long call left
    la = gm.forward(more, sa)
    for i in range(0, 60, 30): lb = gm.forward(more[i:i + 30], sb)
    assert np.array_equal(la.view(np.uint32), lb.view(np.uint32)) and len(sa) == len(sb) == 310
    assert np.array_equal(gm.decode_greedy_dev(sa, int(np.argmax(la)), 12), gm.decode_greedy_dev(sb, int(np.argmax(lb)), 12))


@pytest.mark.parametrize("kind", ["iq3s_mixes", "indexer"])
def test_long_prompt_in_blocks_matches_the_oracle(ctx, kind):
    # A long call of a model whose experts qualify (IQ3_S, equal widths in multiples of 256) takes the whole windows in front of
    # its last tokens in blocks, layer by layer, the FFN of a block grouped by expert on the matrix cores: logits, recurrent
    # state and the tokens that follow against the oracle's token-by-token prompt; with a sparse indexer in the attention
    # layers as well; a second long call continues the state (ragged tails, a position that is no multiple of eight).
    kw = dict(hc_lr=256, qtype=synth.IQ3_S, hc_type=synth.IQ3_S, n_exp=16, top_k=10)
    if kind == "iq3s_mixes": c = small_cfg(**kw)
    else: c = idx_cfg(**kw); c.ctx = 512
    hw, gm, om = pair(ctx, c, 43)
    g = np.random.Generator(np.random.PCG64(44))
    prompt = g.integers(0, c.vocab, 250, dtype=np.uint32)
    gs, os_ = gm.new_state(480), om.new_state()
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)
    assert gm.prompt_blocks() == 2                                     # 30 whole windows: a pair of blocks
    assert relerr(lg, lo) <= 1e-3 and int(np.argmax(lg)) == int(np.argmax(lo))
    n_lin = sum(1 for il in range(c.n_layers) if not c.full(il))
    for li in range(n_lin):
        conv, ssm = gs.gdn(li)
        assert relerr(ssm, os_.ssm(li)) <= 1e-3 and relerr(conv, os_.conv(li)) <= 1e-4, li
    tg, _ = gm.generate_greedy(gs, lg, 6); to, _ = om.generate_greedy(os_, lo, 6)
    assert np.array_equal(tg, to)
    more = g.integers(0, c.vocab, 131, dtype=np.uint32)
    lg = gm.forward(more, gs); lo = om.forward(more, os_)
    assert gm.prompt_blocks() == 3 and len(gs) == 250 + 5 + 131     # 15 whole windows: one block (the sixth generated token has not been fed)
    assert relerr(lg, lo) <= 1e-3 and int(np.argmax(lg)) == int(np.argmax(lo))
    tg, _ = gm.generate_greedy(gs, lg, 6); to, _ = om.generate_greedy(os_, lo, 6)
    assert np.array_equal(tg, to)


@pytest.mark.parametrize("n_exp,top_k,ff_sh,qtype", [(32, 13, 512, synth.IQ3_S), (16, 3, 0, synth.IQ3_S), (16, 2, 0, synth.IQ3_S), (16, 10, 0, synth.Q4_K), (16, 11, 512, synth.Q8_0)])
def test_window_ffn_output_as_group_sums_equals_single_steps_and_the_oracle(ctx, n_exp, top_k, ff_sh, qtype):
    # With IQ3_S hyper-connection matrices a window's FFN output reaches the next mix as four group sums a token (groups of
    # (k + 4) / 4 experts, the shared expert in the last; here groups of 4, 1, 1, 3 and 3 experts, an empty third group, a
    # shared expert wider than the routed ones); a single token leaves the unreduced terms and the mix forms the same sums.
    c = small_cfg(n_exp=n_exp, top_k=top_k, ff_sh=ff_sh, hc_lr=256, qtype=qtype, hc_type=synth.IQ3_S)
    hw, gm, om = pair(ctx, c, 31)
    g = np.random.Generator(np.random.PCG64(32))
    prompt = g.integers(0, c.vocab, 11, dtype=np.uint32)
    sa, sb, so = gm.new_state(64), gm.new_state(64), om.new_state()
    la = gm.forward(prompt, sa); lo = om.forward(prompt, so)
    for tok in prompt: lb = gm.forward(np.array([tok], dtype=np.uint32), sb)
    assert relerr(la, lo) <= 1e-3 and np.array_equal(la.view(np.uint32), lb.view(np.uint32))
    for t in (8, 5, 2):
        toks = g.integers(0, c.vocab, t, dtype=np.uint32)
        lv = gm.forward_multi(toks, sa)
        singles = np.array([gm.forward(toks[i:i + 1], sb) for i in range(t)])
        assert np.array_equal(lv.view(np.uint32), singles.view(np.uint32)), t
        assert relerr(lv, om.forward_multi(toks, so)) <= 1e-3, t


@pytest.mark.parametrize("d,hc,rows", [(256, 2, False), (512, 4, False), (1024, 2, False), (512, 4, True)])
def test_matrix_core_hyper_connection_mixes_windows_equal_steps_and_the_oracle(ctx, monkeypatch, d, hc, rows):
    # IQ3_S hyper-connection matrices with a low rank of 256: the mixes run on the matrix cores (slices of 256 or 512
    # columns, 2 or 4 streams); every window width gives a token the bits of a single step, and the oracle's logits.
    # rows: the same through the lane = row kernels (PYRE_HC_ROWS) -- the two agree within the logits' bound.
    monkeypatch.delenv("PYRE_HC_ROWS", raising=False)
    c = small_cfg(d=d, hc=hc, hc_lr=256, qtype=synth.IQ3_S, hc_type=synth.IQ3_S, n_layers=4)
    hw, gm, om = pair(ctx, c, 23)
    g = np.random.Generator(np.random.PCG64(24))
    prompt = g.integers(0, c.vocab, 13, dtype=np.uint32)
    sa, sb, so = gm.new_state(64), gm.new_state(64), om.new_state()
    la = gm.forward(prompt, sa); gm.forward(prompt, sb); lo = om.forward(prompt, so)
    assert relerr(la, lo) <= 1e-3
    for t in (8, 5, 3, 2):
        toks = g.integers(0, c.vocab, t, dtype=np.uint32)
        lv = gm.forward_multi(toks, sa)
        singles = np.array([gm.forward(toks[i:i + 1], sb) for i in range(t)])
        assert np.array_equal(lv.view(np.uint32), singles.view(np.uint32)), t
        assert relerr(lv, om.forward_multi(toks, so)) <= 1e-3, t
    if rows:          # one of the geometries again through the other kernels (the switch is read once per process: a fresh one)
        import subprocess, sys, os
        code = ("import numpy as np, sys; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
                "from pyre_amd import lib, synth, modelgen as mg\n"
                "c = mg.Config(n_layers=4, d=%d, hc=%d, hc_lr=256, n_exp=8, top_k=2, ff_exp=256, vocab=512, kv_recent=64, qtype=synth.IQ3_S, hc_type=synth.IQ3_S)\n"
                "ctx = lib.Context(0); hw = mg.build_host(c, seed=23); gm = lib.Model(ctx, c, hw.layers, hw.globals_); st = gm.new_state(64)\n"
                "lg = gm.forward(np.frombuffer(bytes.fromhex(%r), dtype=np.uint32), st); sys.stdout.write(lg.tobytes().hex())\n") % (
                    os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)), d, hc, prompt.tobytes().hex())
        env = dict(os.environ, PYRE_HC_ROWS="1")
        out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr[-2000:]
        lr = np.frombuffer(bytes.fromhex(out.stdout.strip()), dtype=np.float32)
        assert relerr(lr, lo) <= 1e-3 and relerr(lr, la) <= 1e-3 and int(np.argmax(lr)) == int(np.argmax(la))


@pytest.mark.parametrize("scale,mixes", [(1.0e5, False), (1.0e4, False), (1.0e5, True), (1.0e-6, True), (1.0e-9, True)])
def test_large_and_tiny_activations_through_the_producer_operands(ctx, scale, mixes):
    # The kernels that produce a matrix-core GEMV's input (attention-side mix -> projections, Gated DeltaNet -> ssm_out,
    # head mix -> vocabulary head) leave it as that GEMV's f16 operand, every token scaled by a power of two.  With the
    # DeltaNet norm weights and the head's norm weights (and, `mixes`, the attention-side hyper-connection norm weights)
    # multiplied by 1e5 .. 1e-9 those inputs leave the range an unscaled f16 half could hold (65504 overflows, below 6e-5
    # loses bits): the logits must be finite and the oracle's, and a window must still equal single steps bit for bit.
    # (Large hyper-connection norm weights also saturate the mixes' sigmoid gates, which makes the network itself
    # ill-conditioned -- the oracle's f32 evaluation and any other f32 evaluation part by percents, with the operand split
    # exactly as with the producers' operands -- so that case checks finiteness and the bit equality only.)
    c = small_cfg(d=512, hc=4, hc_lr=256, qtype=synth.IQ3_S, hc_type=synth.IQ3_S, n_layers=4)
    hw = mg.build_host(c, seed=29)
    def mul(e):
        ty, rows, cols, b = e; assert ty == synth.F32
        return (ty, rows, cols, (b.view(np.float32) * np.float32(scale)).view(np.uint8).copy())
    for L in hw.layers:
        if mixes: L[mg.HCA_NORM] = mul(L[mg.HCA_NORM])
        if mg.LIN_NORM in L: L[mg.LIN_NORM] = mul(L[mg.LIN_NORM])
    hw.globals_[mg.G_HEAD_NORM] = mul(hw.globals_[mg.G_HEAD_NORM])
    gm = lib.Model(ctx, c, hw.layers, hw.globals_); om = orc_model(hw)
    well_conditioned = not (mixes and scale > 1.0)
    g = np.random.Generator(np.random.PCG64(30))
    prompt = g.integers(0, c.vocab, 11, dtype=np.uint32)
    sa, sb, so = gm.new_state(64), gm.new_state(64), om.new_state()
    la = gm.forward(prompt, sa); gm.forward(prompt, sb); lo = om.forward(prompt, so)
    assert np.isfinite(la).all() and np.isfinite(lo).all() and np.abs(la).max() > 0
    if well_conditioned:
        assert relerr(la, lo) <= 1e-3, relerr(la, lo)
    for t in (5, 2):
        toks = g.integers(0, c.vocab, t, dtype=np.uint32)
        lv = gm.forward_multi(toks, sa)
        singles = np.array([gm.forward(toks[i:i + 1], sb) for i in range(t)])
        assert np.isfinite(lv).all() and np.array_equal(lv.view(np.uint32), singles.view(np.uint32)), t
        lw = om.forward_multi(toks, so)
        if well_conditioned:
            assert relerr(lv, lw) <= 1e-3, t
    sa.close(); sb.close(); gm.close()


def test_drafted_generation_identical_to_plain_and_to_oracle(ctx):
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 8)
    prompt = np.array([5, 6, 7, 8], dtype=np.uint32)
    s0 = gm.new_state(128); f0 = gm.forward(prompt, s0)
    plain, _ = gm.generate_greedy(s0, f0, 24)
    so = om.new_state(); fo = om.forward(prompt, so)
    assert np.array_equal(plain, om.generate_greedy(so, fo, 24)[0])
    for corrupt in (False, True):
        ds = np.concatenate([plain, np.zeros(8, np.uint32)]).astype(np.uint32)
        if corrupt:
            ds[3::4] = (ds[3::4] + 1) % c.vocab
        s1 = gm.new_state(128); f1 = gm.forward(prompt, s1)
        out, rounds = gm.generate_greedy(s1, f1, 24, n_draft=4, draft_stream=ds)
        assert np.array_equal(out, plain) and rounds > 0
        so = om.new_state(); fo = om.forward(prompt, so)
        oo, orounds = om.generate_greedy(so, fo, 24, n_draft=4, draft_stream=ds)
        assert np.array_equal(oo, plain) and orounds == rounds


# ---- per-layer n-gram embeddings (PLE) -----------------------------------------------------------------------------------
def ple_pair(ctx, seed, **kw):
    c = mg.with_ple(small_cfg(**kw), layers=(0, 2, 3), ngram=3, per_gram=2, conv_k=3, dim=64, eos=7)
    return (c,) + pair(ctx, c, seed)


def test_ple_model_matches_oracle_steps_window_rollback_device_loop_and_snapshot(ctx, tmp_path):
    c, hw, gm, om = ple_pair(ctx, 61)
    g = np.random.Generator(np.random.PCG64(62))
    prompt = g.integers(0, c.vocab, 27, dtype=np.uint32); prompt[[4, 5, 13]] = c.ple_eos          # eos tokens cut the n-gram contexts
    gs, os_ = gm.new_state(160), om.new_state()
    lg, lo = gm.forward(prompt, gs), om.forward(prompt, os_)                                  # windows of 8, 8, 8, 3 against the oracle's one call
    assert relerr(lg, lo) <= 1e-3
    for pi in range(3):
        assert relerr(gs.ple_hist(pi), os_.ple_hist(pi)) <= 1e-4, pi
    # single steps: the same greedy stream
    toks = []
    for _ in range(10):
        tg, to = int(orc.argmax(lg)), int(orc.argmax(lo)); assert tg == to
        toks.append(to); t1 = np.array([to], dtype=np.uint32); lg, lo = gm.forward(t1, gs), om.forward(t1, os_)
        assert relerr(lg, lo) <= 1e-3
    # a verify window equals single steps bit for bit, and a rollback equals never having drafted
    snap = gs.snapshot()
    win = np.array([int(orc.argmax(lg)), 3, c.ple_eos, 200, 41], dtype=np.uint32)
    lv = gm.forward_multi(win, gs)
    sb = gm.new_state(160); sb.restore(snap)
    singles = np.array([gm.forward(win[i:i + 1], sb) for i in range(5)])
    assert np.array_equal(lv.view(np.uint32), singles.view(np.uint32))
    so = om.new_state(); om.forward(np.concatenate([prompt, np.array(toks, np.uint32)]), so)
    assert relerr(lv, om.forward_multi(win, so)) <= 1e-3
    gm.spec_keep(gs, 5, 2); om.spec_keep(so, 5, 2)
    sc = gm.new_state(160); sc.restore(snap); gm.forward(win[0:1], sc); gm.forward(win[1:2], sc)
    nxt = np.array([77], dtype=np.uint32)
    la = gm.forward(nxt, gs)
    assert np.array_equal(la.view(np.uint32), gm.forward(nxt, sc).view(np.uint32)) and relerr(la, om.forward(nxt, so)) <= 1e-3
    for pi in range(3):
        assert np.array_equal(gs.ple_hist(pi).view(np.uint32), sc.ple_hist(pi).view(np.uint32)) and relerr(gs.ple_hist(pi), so.ple_hist(pi)) <= 1e-4
    # the device-resident loop (token history and position on the device, replayed) against the oracle's loop
    first = int(orc.argmax(la)); dev = gm.decode_greedy_dev(gs, first, 30)
    want = []; tok = first
    for _ in range(30):
        tok = int(orc.argmax(om.forward(np.array([tok], dtype=np.uint32), so))); want.append(tok)
    assert np.array_equal(dev, np.array(want, dtype=np.uint32))
    # and once more from a restored snapshot, eagerly replayed
    sd = gm.new_state(160); sd.restore(snap)
    gm.forward(win[0:1], sd); gm.forward(win[1:2], sd); gm.forward(nxt, sd)
    assert np.array_equal(gm.decode_greedy_dev(sd, first, 30), dev)
    # the same model through a GGUF file with the ple.* keys
    import gguf_writer as gw
    p = str(tmp_path / "ple.gguf")
    gw.write(p, gw.model_meta(c), gw.model_tensors(c, hw))
    gg = lib.Model.from_gguf(ctx, p, kv_bits=c.kv_bits, kv_recent=c.kv_recent)
    sg = gg.new_state(64)
    assert np.array_equal(gg.forward(prompt, sg).view(np.uint32), gm.forward(prompt, gm.new_state(64)).view(np.uint32))


def test_ple_table_rows_outside_the_table_are_refused(ctx):
    c = mg.with_ple(small_cfg(), layers=(1,))
    hw = mg.build_host(c, seed=63)
    c.ple_vocab = tuple(v + 1000 for v in c.ple_vocab)
    with pytest.raises(lib.PyreError, match="per_layer_token_embd"):
        lib.Model(ctx, c, hw.layers, hw.globals_)


def test_errors(ctx):
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 9)
    st = gm.new_state(16)
    with pytest.raises(lib.PyreError):
        gm.forward(np.array([c.vocab], dtype=np.uint32), st)                 # id outside the vocabulary
    with pytest.raises(lib.PyreError):
        gm.forward_multi(np.arange(9, dtype=np.uint32), st)                  # window > 8
    with pytest.raises(lib.PyreError):
        gm.forward(np.zeros(400, dtype=np.uint32), st)                       # beyond the state's capacity
    bad = [dict(l) for l in hw.layers]; bad[0].pop(mg.ROUTER)
    with pytest.raises(lib.PyreError):
        lib.Model(ctx, c, bad, hw.globals_)                                  # missing tensor


def test_model_loaded_from_gguf_shards_equals_the_model_built_from_the_same_tensors(ctx, tmp_path):
    import gguf_writer as gw
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 9)
    tens = gw.model_tensors(c, hw); half = len(tens) // 2
    p1 = str(tmp_path / "tiny-00001-of-00002.gguf"); p2 = str(tmp_path / "tiny-00002-of-00002.gguf")
    gw.write(p1, gw.model_meta(c), tens[:half]); gw.write(p2, [("split.no", gw.U16, 1)], tens[half:], alignment=128)
    gg = lib.Model.from_gguf(ctx, p2, kv_bits=c.kv_bits, kv_recent=c.kv_recent)
    skip = ("rope_base", "eps", "ctx_train", "ctx")        # floats; the file's trained context (262144 by default) is the model's context unless one is asked for
    val = lambda cfg, f: list(getattr(cfg, f)) if f in ("ple_mult", "ple_off", "ple_vocab") else getattr(cfg, f)
    assert [val(gg.cfg, f) for f, _ in lib.ModelCfg._fields_ if f not in skip] == [val(gm.cfg, f) for f, _ in lib.ModelCfg._fields_ if f not in skip]
    ids = np.array([3, 77, 500, 12, 9, 311, 4, 4, 250, 17, 88], dtype=np.uint32)
    sa, sb = gm.new_state(64), gg.new_state(64)
    la, lb = gm.forward(ids, sa), gg.forward(ids, sb)
    assert np.array_equal(la.view(np.uint32), lb.view(np.uint32))
    assert relerr(lb, om.forward(ids, om.new_state())) <= 1e-4
    # a file of another architecture, and one with a tensor missing, are refused with the reference's messages
    bad = str(tmp_path / "other.gguf")
    gw.write(bad, [("general.architecture", gw.STR, "llama")], [])
    with pytest.raises(lib.PyreError, match="is not qwen4exp"):
        lib.Model.from_gguf(ctx, bad)
    gw.write(bad, gw.model_meta(c), [t for t in tens if t[0] != "blk.2.ssm_out.weight"])
    with pytest.raises(lib.PyreError, match="missing tensor blk.2.ssm_out.weight"):
        lib.Model.from_gguf(ctx, bad)
    gw.write(bad, [m for m in gw.model_meta(c) if "expert_count" not in m[0]], tens)
    with pytest.raises(lib.PyreError, match="gguf key qwen4exp.expert_count"):
        lib.Model.from_gguf(ctx, bad)


def idx_cfg(**kw):
    # one attention layer with an indexer: dense up to 16 + 4 - 1 = 19 visible positions, 4 blocks + tail beyond; YaRN x2
    return small_cfg(idx_nh=2, idx_hd=128, idx_ratio=4, idx_budget=16, ctx_train=64, ctx=128, **kw)


def test_indexer_and_yarn_model_matches_oracle_greedy_verify_rollback_snapshot_and_device_loop(ctx, tmp_path):
    c = idx_cfg()
    hw, gm, om = pair(ctx, c, 12)
    prompt = (np.arange(37, dtype=np.uint32) * 31 + 3) % c.vocab            # 37 > 19: the prompt itself already runs sparse
    gs, os_ = gm.new_state(300), om.new_state()
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)
    assert relerr(lg, lo) <= 1e-4 and orc.argmax(lg) == orc.argmax(lo)
    snap = gs.snapshot()
    out_g, _ = gm.generate_greedy(gs, lg, 100)                               # host-driven loop; crosses the packing boundary at 128 + 64
    out_o, _ = om.generate_greedy(os_, lo, 100)
    assert np.array_equal(out_g, out_o), "first split at %d" % int(np.argmax(out_g != out_o))
    # the device-resident loop (captured step, position on the device) from the snapshot gives the same stream
    s2 = gm.new_state(200); s2.restore(snap)
    assert np.array_equal(gm.decode_greedy_dev(s2, int(out_g[0]), 99), out_g[1:])
    # verify window == single steps, rollback == never drafted (indexer keys and block keys included)
    sa, sb = gm.new_state(64), gm.new_state(64)
    gm.forward(prompt[:30], sa); gm.forward(prompt[:30], sb)
    toks = np.array([9, 100, 11, 212, 13, 77], dtype=np.uint32)
    lv = gm.forward_multi(toks, sa)
    singles = np.array([gm.forward(toks[i:i + 1], sb) for i in range(6)])
    assert np.array_equal(lv.view(np.uint32), singles.view(np.uint32))
    gm.spec_keep(sa, 6, 3)
    sc = gm.new_state(64); gm.forward(prompt[:30], sc)
    for i in range(3):
        gm.forward(toks[i:i + 1], sc)
    nxt = np.array([40, 41, 42, 43, 44], dtype=np.uint32)
    assert np.array_equal(gm.forward(nxt, sa).view(np.uint32), gm.forward(nxt, sc).view(np.uint32))
    # the same model through a GGUF file (indexer metadata and tensors by name; context 128 -> YaRN)
    import gguf_writer as gw
    p = str(tmp_path / "idx.gguf")
    gw.write(p, gw.model_meta(c), gw.model_tensors(c, hw))
    gg = lib.Model.from_gguf(ctx, p, kv_bits=c.kv_bits, kv_recent=c.kv_recent, ctx_tokens=128)
    assert (gg.cfg.idx_nh, gg.cfg.idx_hd, gg.cfg.idx_ratio, gg.cfg.idx_budget, gg.cfg.ctx_train, gg.cfg.ctx) == (2, 128, 4, 16, 64, 128)
    sg = gg.new_state(64)
    assert np.array_equal(gg.forward(prompt, sg).view(np.uint32), lg.view(np.uint32))
    # without the requested context the rotation table is the trained one: different logits
    g0 = lib.Model.from_gguf(ctx, p, kv_bits=c.kv_bits, kv_recent=c.kv_recent)
    assert relerr(g0.forward(prompt, g0.new_state(64)), lg) > 1e-4


def test_snapshot_restore_reproduces_the_continuation_bit_for_bit(ctx):
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 10)
    prompt = (np.arange(150, dtype=np.uint32) * 29 + 5) % c.vocab          # 150 > recent + 64: the packed region exists
    sa = gm.new_state(400)
    lg = gm.forward(prompt, sa)
    snap = sa.snapshot()
    assert len(snap) == 150 and snap.nbytes > 0 and sa.capacity >= 400 and ctx.L.pyre_model_max_window(gm.h) == 8
    first = int(np.argmax(lg))
    ta = gm.decode_greedy_dev(sa, first, 40)                               # the original state moves on (and packs more positions)
    sb = gm.new_state(200)                                                 # another capacity: the blocked key planes are prefix-compatible
    sb.restore(snap)
    assert len(sb) == 150
    tb = gm.decode_greedy_dev(sb, first, 40)
    assert np.array_equal(ta, tb)
    sa.restore(snap)                                                       # and back onto the state it came from
    tc = gm.decode_greedy_dev(sa, first, 40)
    assert np.array_equal(ta, tc)
    for li in range(3):
        for x, y in zip(sa.gdn(li), sb.gdn(li)):
            assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
    ka, va = sa.kv(0); kb, vb = sb.kv(0)
    assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32)) and np.array_equal(va.view(np.uint32), vb.view(np.uint32))
    gm.decode_greedy_dev(sa, int(tc[-1]), 80)                              # 270 positions: more than a 256-position state holds
    small = gm.new_state(100)
    with pytest.raises(lib.PyreError, match="do not fit"):
        small.restore(sa.snapshot())


def test_device_greedy_loop_called_repeatedly_on_one_state_continues_the_same_stream(ctx):
    """The captured decode step must follow the state through several calls and through forward calls in between."""
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 11)
    prompt = np.array([5, 6, 7, 8, 9, 10, 11, 12, 13, 14], dtype=np.uint32)
    sa, sb = gm.new_state(200), gm.new_state(200)
    lg = gm.forward(prompt, sa); gm.forward(prompt, sb)
    first = int(np.argmax(lg))
    whole = gm.decode_greedy_dev(sb, first, 60)
    parts = [gm.decode_greedy_dev(sa, first, 7)]
    parts.append(gm.decode_greedy_dev(sa, int(parts[-1][-1]), 13))
    lg2 = gm.forward(np.array([parts[-1][-1]], dtype=np.uint32), sa)          # a host-driven step in between flips the double buffers
    parts.append(np.array([int(np.argmax(lg2))], dtype=np.uint32))
    parts.append(gm.decode_greedy_dev(sa, int(parts[-1][-1]), 19))
    parts.append(gm.decode_greedy_dev(sa, int(parts[-1][-1]), 20))
    assert np.array_equal(np.concatenate(parts), whole)
    os_ = om.new_state(); lo = om.forward(prompt, os_)
    ref, _ = om.generate_greedy(os_, lo, 61)
    assert np.array_equal(ref[1:], whole)


def test_session_chunk_grid_prefill_and_prefix_cache_give_the_state_of_a_full_prefill(ctx):
    """engine_qn::run: continue the previous state, resume from the longest grid snapshot, cut at the common prefix."""
    c = small_cfg()
    hw, gm, om = pair(ctx, c, 13)
    rng = np.random.Generator(np.random.PCG64(5))
    A = rng.integers(0, c.vocab, 150, dtype=np.uint32)
    full = lambda ids: gm.forward(ids, gm.new_state(400))
    se = lib.Session(gm, 400, chunk=32, cache_bytes=64 << 20)
    la, cached, snap = se.prefill(A)
    assert cached == 0 and not snap and np.array_equal(la.view(np.uint32), full(A).view(np.uint32))
    assert se.stats()[3] == [32, 64, 96, 128] and se.stats()[2] == 150                  # grid snapshots, none at the prompt's end
    out, _ = se.generate_greedy(la, 10)
    so = om.new_state(); lo = om.forward(A, so)
    assert np.array_equal(out, om.generate_greedy(so, lo, 10)[0]) and se.stats()[2] == 159     # the last token is pending
    # 1. a prompt that strictly extends what the state consumed continues it
    B = np.concatenate([A, out[:9], rng.integers(0, c.vocab, 20, dtype=np.uint32)]).astype(np.uint32)
    lb, cached, snap = se.prefill(B)
    assert cached == 159 and not snap and np.array_equal(lb.view(np.uint32), full(B).view(np.uint32))
    # 2. a prompt that shares 100 tokens with A: longest snapshot it extends is 96; a snapshot is cut at the common prefix with
    #    the previous prompt (B: 100 tokens) as well as on the grid
    C2 = np.concatenate([A[:100], rng.integers(0, c.vocab, 70, dtype=np.uint32)]).astype(np.uint32)
    lc, cached, snap = se.prefill(C2)
    assert cached == 96 and snap and np.array_equal(lc.view(np.uint32), full(C2).view(np.uint32))
    lens = se.stats()[3]
    assert 100 in lens and 128 in lens and 160 in lens and lens.count(128) == 2          # A's and C2's 128-token prefixes differ
    # 3. the same prompt again: every snapshot it strictly extends is a candidate -> the 160-token one
    lc2, cached, snap = se.prefill(C2)
    assert cached == 160 and snap and np.array_equal(lc2.view(np.uint32), lc.view(np.uint32))
    # 4. an unrelated prompt starts from an empty state
    D = rng.integers(0, c.vocab, 40, dtype=np.uint32)
    ld, cached, snap = se.prefill(D)
    assert cached == 0 and not snap and np.array_equal(ld.view(np.uint32), full(D).view(np.uint32))
    # 5. the byte cap drops the oldest snapshots first; a prompt at or beyond the context size is refused
    one = se.stats()[1] // se.stats()[0]
    small = lib.Session(gm, 400, chunk=32, cache_bytes=3 * one)
    small.prefill(A)
    n, b, _, lens = small.stats()
    assert b <= 3 * one and lens == sorted(lens) and lens[-1] == 128 and n < 4
    with pytest.raises(lib.PyreError, match="exceeds context size"):
        se.prefill(np.zeros(400, np.uint32))
    off = lib.Session(gm, 400, chunk=32, cache_bytes=0)                                 # PYRE_QN_PCACHE=0
    off.prefill(A); assert off.stats()[0] == 0
    se.close(); small.close(); off.close()
