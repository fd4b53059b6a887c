"""GPU parity against the CPU oracle at the benchmark's own sizes, through the C ABI: gated attention over a
32 768-position 4-bit cache (the second pass of the chunk merge), a full-width model of three 3 + 1 layer groups against
the oracle's token loop, the 4096 x 4096 IQ3_S GEMV, the 151 936-row head in every format of the sweep, and the
4096-token chunked Gated DeltaNet prefill against the sequential recurrence."""
import os

import numpy as np
import pytest

import orc
from helpers import orc_cfg, relerr
from pyre_amd import lib, synth
from pyre_amd import modelgen as mg

pytestmark = pytest.mark.gpu
THREADS = min(os.cpu_count() or 1, 16)


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


def rnd(seed):
    return np.random.Generator(np.random.PCG64(seed))


# ---- attention at the benchmark's context ---------------------------------------------------------------------------------
@pytest.mark.parametrize("start,t", [(32768, 1), (32768 + 77, 5), (33000, 3)])
def test_attention_over_32k_packed_cache_matches_oracle(ctx, start, t):
    # 16 query heads, 2 KV heads of 256, 4-bit cache with the newest 1024 positions in f32: more than 256 chunks of 128
    # positions per head, so the chunk merge runs its second pass; about 31 700 positions are read from the packed planes
    nh, nkv, recent = 16, 2, 1024
    row = nkv * 256
    g = rnd(1000 + start + t)
    kc = g.standard_normal((start, row), dtype=np.float32); vc = g.standard_normal((start, row), dtype=np.float32)
    q = g.standard_normal((t, nh * 512), dtype=np.float32); k = g.standard_normal((t, row), dtype=np.float32); v = g.standard_normal((t, row), dtype=np.float32)
    qn = (1 + 0.1 * g.standard_normal(256)).astype(np.float32); kn = (1 + 0.1 * g.standard_normal(256)).astype(np.float32)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, qn, kn, 4, recent, start + 16)
    att.load_cache(kc, vc)
    out = att.decode(q, k, v)
    K = np.zeros((start + t, row), np.float32); V = np.zeros_like(K); K[:start] = kc; V[:start] = vc
    ref = orc.attn_core(nh, nkv, 256, 64, 1e-6, orc.rope_inv(64, 1e7), qn, kn, q, k, v, start, 4, recent, K, V)
    assert orc.packed_boundary(start + 1, 4, recent) >= 31680
    assert relerr(out, ref) <= 2e-5
    for h in range(nh):             # per head as well: no head hides behind a larger one
        assert relerr(out.reshape(t, nh, 256)[:, h], ref.reshape(t, nh, 256)[:, h]) <= 5e-5, h
    assert len(att) == start + t
    att.close()


# ---- the model at full width, three layer groups, against the oracle's token loop -----------------------------------------
def host_weights_from_device(ctx, cfg, layers, globals_):
    """The oracle's view of a device-generated weight set: every device tensor is downloaded once."""
    def pull(e):
        ty, rows, cols, data = e
        if isinstance(data, np.ndarray):
            return e
        el, bs, _ = synth.GEOM[ty]
        return (ty, rows, cols, ctx.download(data, (rows * (cols // el) * bs,), np.uint8))
    return [{s: pull(e) for s, e in L.items()} for L in layers], {s: pull(e) for s, e in globals_.items()}


def test_twelve_layer_full_width_greedy_stream_matches_oracle(ctx):
    cfg = mg.a3b_config(n_layers=12)
    layers, globals_, raw = mg.build_device(ctx, cfg, seed=21)
    gm = lib.Model(ctx, cfg, layers, globals_)
    hl, hg = host_weights_from_device(ctx, cfg, layers, globals_)
    for p in raw:
        ctx.free(p)
    lt = []
    for il in range(cfg.n_layers):
        for slot in range(mg.LAYER_SLOTS):
            e = hl[il].get(slot)
            lt.append(orc.tensor(*e) if e is not None else orc.Tensor(0, 0, 0, None))
    om = orc.Model(orc_cfg(cfg), lt, [orc.tensor(*hg[s]) if s in hg else orc.Tensor(0, 0, 0, None) for s in range(mg.GLOBAL_SLOTS)], threads=THREADS, keep=(hl, hg))
    prompt = rnd(22).integers(0, cfg.vocab, 24, dtype=np.uint32)
    gs, os_ = gm.new_state(128), om.new_state()
    lg, lo = gm.forward(prompt, gs), om.forward(prompt, os_)
    worst = relerr(lg, lo); rows = []
    for i in range(32):
        tg, to = int(orc.argmax(lg)), int(orc.argmax(lo))
        top2 = np.partition(lo, -2)[-2:]; margin = float(top2[1] - top2[0]); dl = float(np.abs(lg - lo).max())
        rows.append((i, to, margin, dl))
        assert tg == to, "token %d: device %d, oracle %d, oracle top-2 margin %.3e, max |dlogit| %.3e" % (i, tg, to, margin, dl)
        tok = np.array([to], dtype=np.uint32)
        lg, lo = gm.forward(tok, gs), om.forward(tok, os_)
        worst = max(worst, relerr(lg, lo))
    print("\n12-layer full-width greedy stream: token, id, oracle top-2 margin, max |dlogit|")
    for r in rows:
        print("  %2d %6d  %.3e  %.3e" % r)
    assert worst <= 1e-3
    # the recurrent state and the cache of the last attention layer after 56 tokens
    _, ssm = gs.gdn(0)
    assert relerr(ssm, os_.ssm(0)) <= 1e-4
    kd, vd = gs.kv(2)
    assert relerr(kd, os_.kcache(2).reshape(kd.shape)) <= 1e-4 and relerr(vd, os_.vcache(2).reshape(vd.shape)) <= 1e-4
    gs.close(); gm.close()


def test_all_48_layers_full_width_greedy_stream_matches_oracle(ctx, capsys):
    # the benchmark's own depth and width: 48 layers (36 Gated DeltaNet + 12 attention, 512 experts each), an 8-token prompt
    # and 16 greedy tokens against the oracle's token loop on the same weights (generated on the device, downloaded once)
    # (PYRE_TEST_48L_TOKENS=256 runs the 256 tokens the oracle needs about five minutes for)
    n_new = int(os.environ.get("PYRE_TEST_48L_TOKENS", "16"))
    def say(msg):
        with capsys.disabled():
            print(msg, flush=True)
    cfg = mg.a3b_config(n_layers=48)
    layers, globals_, raw = mg.build_device(ctx, cfg, seed=23)
    gm = lib.Model(ctx, cfg, layers, globals_)
    say("\n48-layer model on the device; downloading the weights for the oracle")
    hl, hg = host_weights_from_device(ctx, cfg, layers, globals_)
    for p in raw:
        ctx.free(p)
    lt = []
    for il in range(cfg.n_layers):
        for slot in range(mg.LAYER_SLOTS):
            e = hl[il].get(slot)
            lt.append(orc.tensor(*e) if e is not None else orc.Tensor(0, 0, 0, None))
    om = orc.Model(orc_cfg(cfg), lt, [orc.tensor(*hg[s]) if s in hg else orc.Tensor(0, 0, 0, None) for s in range(mg.GLOBAL_SLOTS)], threads=THREADS, keep=(hl, hg))
    prompt = rnd(24).integers(0, cfg.vocab, 8, dtype=np.uint32)
    gs, os_ = gm.new_state(64 + n_new), om.new_state()
    lg, lo = gm.forward(prompt, gs), om.forward(prompt, os_)
    say("prompt done: logits rel err %.3e" % relerr(lg, lo))
    worst = relerr(lg, lo); rows = []
    for i in range(n_new):
        tg, to = int(orc.argmax(lg)), int(orc.argmax(lo))
        top2 = np.partition(lo, -2)[-2:]; margin = float(top2[1] - top2[0]); dl = float(np.abs(lg - lo).max())
        rows.append((i, to, margin, dl))
        assert tg == to, "token %d: device %d, oracle %d, oracle top-2 margin %.3e, max |dlogit| %.3e" % (i, tg, to, margin, dl)
        tok = np.array([to], dtype=np.uint32)
        lg, lo = gm.forward(tok, gs), om.forward(tok, os_)
        worst = max(worst, relerr(lg, lo))
        if i % 4 == 3:
            say("  %d tokens identical, worst logits rel err so far %.3e" % (i + 1, worst))
    say("48-layer full-width greedy stream: token, id, oracle top-2 margin, max |dlogit|")
    for r in rows:
        say("  %2d %6d  %.3e  %.3e" % r)
    assert worst <= 1e-3
    gs.close()
    # the same depth through a long prompt: 1100 tokens in blocks (the FFN grouped by expert on the matrix cores) against
    # the same prompt in windows of eight: logits within 1e-3, the sixteen greedy tokens that follow identical
    longp = rnd(25).integers(0, cfg.vocab, 1100, dtype=np.uint32); res = {}
    for mode in ("1", "0"):
        os.environ["PYRE_PROMPT_WINDOWS"] = mode
        try:
            st = gm.new_state(1100 + 32); b0 = gm.prompt_blocks()
            lgl = gm.forward(longp, st)
            res[mode] = (lgl.copy(), gm.decode_greedy_dev(st, int(np.argmax(lgl)), 16).copy(), gm.prompt_blocks() - b0)
            st.close()
        finally:
            os.environ.pop("PYRE_PROMPT_WINDOWS", None)
    assert res["1"][2] == 0 and res["0"][2] == 2          # 136 whole windows: a pair of blocks
    say("1100-token prompt at 48 layers, blocks against windows: logits rel err %.3e" % relerr(res["0"][0], res["1"][0]))
    assert relerr(res["0"][0], res["1"][0]) <= 1e-3 and np.array_equal(res["0"][1], res["1"][1])
    gm.close()


def test_device_loop_equals_host_loop_beyond_32k_context(ctx):
    # one layer group (3 Gated DeltaNet + 1 attention layer) at full width with a 32 800-token prompt: the replayed
    # device-resident step (positions read from device memory, packing check folded into the prep launch) against the
    # host-facing step on the same state, across a packing-boundary move (32 832 = 513 * 64)
    cfg = mg.a3b_config(n_layers=4)
    layers, globals_, raw = mg.build_device(ctx, cfg, seed=5)
    gm = lib.Model(ctx, cfg, layers, globals_)
    for p in raw:
        ctx.free(p)
    prompt = rnd(31).integers(0, cfg.vocab, 32800, dtype=np.uint32)
    st = gm.new_state(32800 + 64)
    lg = gm.forward(prompt, st); first = int(orc.argmax(lg))
    snap = st.snapshot()
    dev = gm.decode_greedy_dev(st, first, 40)
    st.restore(snap)
    host = []; tok = first
    for _ in range(40):
        lg = gm.forward(np.array([tok], dtype=np.uint32), st); tok = int(orc.argmax(lg)); host.append(tok)
    assert np.array_equal(dev, np.array(host, dtype=np.uint32))
    st.close(); gm.close()


# ---- GEMV: the single 4096 x 4096 IQ3_S case and the vocabulary head in every format of the sweep ---------------------------
def test_iq3s_gemv_4096_by_4096(ctx):
    rows = cols = 4096
    raw = synth.matrix(lib.IQ3_S, rows, cols, 4096)
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, raw)
    W = orc.dequant(lib.IQ3_S, raw, rows * cols).reshape(rows, cols)
    assert np.array_equal(m.to_f32().view(np.uint32), W.view(np.uint32))
    x = synth.normal((1, cols), 4097)
    truth = x.astype(np.float64) @ W.astype(np.float64).T
    assert relerr(m.matmul(x), truth) <= 1e-5 and relerr(m.matmul_f32(x), truth) <= 1e-5
    assert relerr(orc.matmul(lib.IQ3_S, raw, rows, cols, x, threads=THREADS), truth) <= 1e-5
    m.close()


@pytest.mark.parametrize("ty", [lib.IQ2_XS, lib.IQ3_S, lib.Q4_K, lib.Q8_0])
def test_vocab_head_every_sweep_format_and_width(ctx, ty):
    rows, cols = 151936, 2048
    el, bs, _ = synth.GEOM[ty]
    nb = rows * cols // el; rb = cols // el * bs
    dev = ctx.alloc(nb * bs)
    ctx.synth_blocks(ty, nb, 5000 + ty, dev_out=dev)
    m = lib.QMat(ctx, ty, rows, cols, dev_blocks=dev, nbytes=nb * bs)
    sel = np.r_[0:64, 40000:40064, 75000 + 13:75064 + 13, rows - 64:rows]
    rawsel = np.stack([ctx.download(dev + int(r) * rb, (rb,), np.uint8) for r in sel])
    ctx.free(dev)
    Wsel = np.stack([orc.dequant(ty, rawsel[i], cols) for i in range(len(sel))]).astype(np.float64)
    for r in (0, 3):
        assert np.array_equal(m.row(int(sel[r])).view(np.uint32), Wsel[r].astype(np.float32).view(np.uint32))
    y8 = None
    for t in (8, 4, 2, 1):
        x = synth.normal((8, cols), 93)[:t]
        y = m.matmul(x)
        truth = x.astype(np.float64) @ Wsel.T
        assert np.abs(y[:, sel] - truth).max() / np.abs(truth).max() <= 1e-5, t
        assert np.isfinite(y).all()
        if y8 is None:
            y8 = y
        elif ty in (lib.IQ3_S, lib.IQ2_XS, lib.Q4_K, lib.Q8_0) and t == 1:        # (one token of an IQ3_S, IQ2_XS or Q4_K matrix takes the native-format kernel, of a Q8_0 matrix the lane = row one, windows the matrix cores: equal to rounding)
            assert relerr(y, y8[:1]) <= 2e-6
        else:                                   # a token's row does not depend on the window it was computed in
            assert np.array_equal(y.view(np.uint32), y8[:t].view(np.uint32)), t
    m.close()


# ---- the 4096-token chunked prefill against the sequential recurrence -------------------------------------------------------
@pytest.mark.parametrize("dt_bias", [0.0, 0.3])
def test_gdn_chunked_prefill_4096_tokens_matches_sequential_oracle(ctx, dt_bias):
    nk, nv, T = 16, 32, 4096
    ch = 2 * nk * 128 + nv * 128
    g = rnd(900 + int(dt_bias * 10))
    a = (-np.exp(g.uniform(0.0, np.log(16.0), nv))).astype(np.float32)
    dt = (dt_bias * g.standard_normal(nv)).astype(np.float32)
    conv_w = (0.5 * g.standard_normal(ch * 4)).astype(np.float32); norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    gd = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, a, dt, conv_w, norm_w)
    S0 = (0.01 * g.standard_normal((nv, 128, 128))).astype(np.float32); cs0 = (0.3 * g.standard_normal((3, ch))).astype(np.float32)
    gd.set_state(cs0, S0)
    qkv = g.standard_normal((T, ch), dtype=np.float32); z = g.standard_normal((T, nv * 128), dtype=np.float32)
    beta = g.standard_normal((T, nv), dtype=np.float32); alpha = g.standard_normal((T, nv), dtype=np.float32)
    out = gd.prefill_chunked(qkv, z, beta, alpha)
    so, co = S0.copy().reshape(-1), cs0.copy().reshape(-1)
    ref = orc.gdn_core(nk, nv, 128, 128, 4, 1e-6, a, dt, conv_w, norm_w, qkv, z, beta, alpha, co, so)
    assert relerr(out, ref) <= 1e-5
    for lo in range(0, T, 512):             # and per stretch of the sequence: late tokens are held to the same bound as early ones
        assert relerr(out[lo:lo + 512], ref[lo:lo + 512]) <= 2e-5, lo
    conv, ssm = gd.get_state()
    assert relerr(ssm, so) <= 1e-5 and np.array_equal(conv.reshape(-1), co)
    gd.close()
