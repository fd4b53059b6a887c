"""GPU parity of the block-level entry points (MoE FFN, Gated DeltaNet step, gated attention over the 4-bit cache)
against the CPU oracle, through the C ABI.  Tolerance 1e-5 on max|d| / max|ref| unless stated."""
import numpy as np
import pytest

import np_ref
import orc
from helpers import orc_tensor, relerr
from pyre_amd import lib, synth
from pyre_amd import modelgen as mg

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


# ---- MoE --------------------------------------------------------------------------------------------------------------
def moe_pair(ctx, c, seed):
    hw = mg.build_host(c, seed=seed); L = hw.layers[0]
    qm = {s: lib.QMat(ctx, L[s][0], L[s][1], L[s][2], L[s][3]) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E, mg.SH_GATE, mg.SH_UP, mg.SH_DOWN)}
    moe = lib.Moe(ctx, c.top_k, qm[mg.ROUTER], qm[mg.GATE_E], qm[mg.UP_E], qm[mg.DOWN_E], hw.f32(0, mg.SH_GATE_INP), qm[mg.SH_GATE], qm[mg.SH_UP], qm[mg.SH_DOWN])

    def oracle(x):
        return orc.moe_ffn(c.d, c.n_exp, c.top_k, c.ff_exp, *(orc_tensor(L[s]) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E)),
                           hw.f32(0, mg.SH_GATE_INP), *(orc_tensor(L[s]) for s in (mg.SH_GATE, mg.SH_UP, mg.SH_DOWN)), x)
    return moe, oracle, hw


@pytest.mark.parametrize("qtype", [synth.IQ3_S, synth.IQ2_XS, synth.Q4_K, synth.Q8_0, synth.IQ2_S, synth.IQ4_NL, synth.Q6_K, synth.Q5_K, synth.Q3_K])
@pytest.mark.parametrize("t", [1, 4])
def test_moe_ffn_small(ctx, qtype, t):
    c = mg.Config(n_layers=1, full_every=4, d=512, n_exp=16, top_k=4, ff_exp=256, qtype=qtype)
    moe, oracle, _ = moe_pair(ctx, c, 7)
    x = synth.normal((t, c.d), 100 + t)
    y, idx, w = moe.ffn(x)
    yo, io, wo = oracle(x)
    assert np.array_equal(idx, io) and np.abs(w - wo).max() < 1e-6
    assert relerr(y, yo) <= TOL


@pytest.mark.parametrize("qtype,d", [(synth.Q4_K, 2048), (synth.Q8_0, 2048), (synth.IQ2_XS, 2048), (synth.IQ4_NL, 2048), (synth.IQ3_S, 4096)])
def test_moe_gate_up_in_two_k_parts(ctx, qtype, d):
    # rows of a multiple of 32 units: the gate/up dot products are summed in two K parts -- one workgroup per part for a
    # single token, both parts in one workgroup for a window -- and a token's bits must not depend on which (d = 4096:
    # two units per wave and part)
    c = mg.Config(n_layers=1, full_every=4, d=d, n_exp=16, top_k=4, ff_exp=256, qtype=qtype)
    moe, oracle, _ = moe_pair(ctx, c, 11)
    x = synth.normal((3, c.d), 300)
    y, idx, w = moe.ffn(x)
    yo, io, wo = oracle(x)
    assert np.array_equal(idx, io) and np.abs(w - wo).max() < 1e-6
    assert relerr(y, yo) <= TOL
    for ti in range(3):
        y1, i1, _ = moe.ffn(x[ti:ti + 1])
        assert np.array_equal(i1, idx[ti:ti + 1]) and relerr(y1, yo[ti:ti + 1]) <= TOL
        assert np.array_equal(y1.view(np.uint32), y[ti:ti + 1].view(np.uint32))


def test_moe_iq3s_gate_up_in_the_integer_form_over_the_activation_range(ctx):
    # IQ3_S experts multiply gate/up in integers: per 64 columns the activations become a power of two and three signed-byte
    # digits.  Activations whose 64-column stretches sit on powers of two of their own, outliers, tiny and huge values must
    # still give the oracle's result; a window equals its single steps bit for bit; PYRE_MOE_IDOT=0 (the f32 multiply-add
    # form, read once per process: a fresh one) agrees to rounding and chooses the same experts.
    c = mg.Config(n_layers=1, full_every=4, d=2048, n_exp=16, top_k=4, ff_exp=256, qtype=synth.IQ3_S)
    moe, oracle, _ = moe_pair(ctx, c, 13)
    g = np.random.Generator(np.random.PCG64(77))
    xs = []
    for case in range(5):
        x = synth.normal((3, c.d), 700 + case)
        if case == 1: x *= np.exp2(g.integers(-20, 20, c.d // 64).repeat(64)).astype(np.float32)
        if case == 2: x[0, 5] = 3.0e3; x[1, c.d - 3] = -2.0e4
        if case == 3: x *= 1e-20
        if case == 4: x[:, ::2] = 0.0; x[:, :64] = 0.0
        xs.append(x)
        y, idx, w = moe.ffn(x)
        yo, io, wo = oracle(x)
        assert np.array_equal(idx, io), case
        assert relerr(y, yo) <= TOL, case
        for ti in range(3):
            y1, _, _ = moe.ffn(x[ti:ti + 1])
            assert np.array_equal(y1.view(np.uint32), y[ti:ti + 1].view(np.uint32)), (case, ti)
    import subprocess, sys, os
    if os.environ.get("PYRE_MOE_IDOT", "") == "0":
        return                                                              # this process already runs the f32 form: nothing to compare
    code = ("import numpy as np, sys; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
            "from pyre_amd import lib, synth, modelgen as mg\n"
            "import test_gpu_blocks as tb\n"
            "ctx = lib.Context(0); c = mg.Config(n_layers=1, full_every=4, d=2048, n_exp=16, top_k=4, ff_exp=256, qtype=synth.IQ3_S)\n"
            "moe, _, _ = tb.moe_pair(ctx, c, 13)\n"
            "x = np.frombuffer(bytes.fromhex(sys.stdin.read()), dtype=np.float32).reshape(3, 2048)\n"
            "y, idx, w = moe.ffn(x); sys.stdout.write(y.tobytes().hex() + ' ' + idx.astype(np.int32).tobytes().hex())\n") % (
                os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, PYRE_MOE_IDOT="0"), input=xs[1].tobytes().hex(), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    yh, ih = out.stdout.strip().split(" ")
    yf = np.frombuffer(bytes.fromhex(yh), dtype=np.float32).reshape(3, c.d)
    y, idx, _ = moe.ffn(xs[1])
    assert np.array_equal(np.frombuffer(bytes.fromhex(ih), dtype=np.int32).reshape(idx.shape), idx.astype(np.int32))
    assert relerr(y, yf) <= 2e-6 and not np.array_equal(y.view(np.uint32), yf.view(np.uint32))          # (two forms: equal to rounding, not bit for bit)


@pytest.mark.parametrize("t", [1, 4])
def test_moe_ffn_benchmark_geometry(ctx, t):
    # 512 routed experts + 1 shared, d 2048, expert ff 512, top-10, IQ3_S (reduced to 64 resident experts' worth of
    # distinct routing by the seed; all 512 experts exist)
    c = mg.Config(n_layers=1, full_every=4, d=2048, n_exp=512, top_k=10, ff_exp=512, qtype=synth.IQ3_S)
    moe, oracle, _ = moe_pair(ctx, c, 9)
    x = synth.normal((t, c.d), 200 + t)
    y, idx, w = moe.ffn(x)
    yo, io, wo = oracle(x)
    assert np.array_equal(idx, io) and np.abs(w - wo).max() < 1e-6 and (np.diff(idx, axis=1) > 0).all()
    assert relerr(y, yo) <= TOL
    # each token's result does not depend on its companions in the window
    y1, _, _ = moe.ffn(x[:1])
    assert np.array_equal(y1.view(np.uint32), y[:1].view(np.uint32))


def test_router_ties_and_nan(ctx):
    c = mg.Config(n_layers=1, full_every=4, d=256, n_exp=8, top_k=3, ff_exp=256, qtype=synth.Q8_0)
    moe, oracle, hw = moe_pair(ctx, c, 11)
    # x = 0 -> all router logits equal (0): ties resolve to the lowest expert ids, uniform weights
    y, idx, w = moe.ffn(np.zeros((1, c.d), np.float32))
    assert list(idx[0]) == [0, 1, 2] and np.allclose(w, 1 / 3) and not y.any()
    xn = synth.normal((1, c.d), 5); xn[0, 3] = np.nan
    y, idx, w = moe.ffn(xn)          # every logit NaN -> -inf -> lowest ids, uniform weights (nan_clean / soft_top)
    assert list(idx[0]) == [0, 1, 2] and np.allclose(w, 1 / 3)


# ---- Gated DeltaNet ------------------------------------------------------------------------------------------------------
def gdn_params(nk, nv, seed, conv_k=4):
    ch = 2 * nk * 128 + nv * 128
    a = -np.exp(synth.uniform((nv,), seed + 1, 0.0, np.log(16.0)))
    return dict(a=a, dt=synth.normal((nv,), seed + 8, 0.1), conv_w=synth.normal((ch * conv_k,), seed + 2, 0.5), norm_w=1 + synth.normal((128,), seed + 3, 0.1)), ch


def gdn_inputs(nv, ch, t, seed):
    return synth.normal((t, ch), seed + 4), synth.normal((t, nv * 128), seed + 5), synth.normal((t, nv), seed + 6), synth.normal((t, nv), seed + 7)


@pytest.mark.parametrize("nk,nv", [(2, 4), (16, 32)])
def test_gdn_step_matches_oracle(ctx, nk, nv):
    p, ch = gdn_params(nk, nv, 300 + nv)
    g = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    S0 = synth.normal((nv, 128, 128), 77, 0.01); cs0 = synth.normal((3, ch), 78, 0.3)
    g.set_state(cs0, S0)
    so, co = S0.copy().reshape(-1), cs0.copy().reshape(-1)
    for rnd, t in enumerate((1, 1, 5, 8, 13)):
        qkv, z, beta, alpha = gdn_inputs(nv, ch, t, 1000 * rnd)
        out = g.step(qkv, z, beta, alpha)
        ref = orc.gdn_core(nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"], qkv, z, beta, alpha, co, so)
        assert relerr(out, ref) <= TOL, (rnd, t)
    conv, ssm = g.get_state()
    assert relerr(ssm, so) <= TOL and np.array_equal(conv.reshape(-1), co)


def test_gdn_benchmark_config_state_and_closed_forms(ctx):
    # 16 QK heads, 32 V heads, head dim 128, conv 4, state N(0, 0.01), A_log ~ U(0, ln 16), dt_bias 0
    nk, nv = 16, 32
    p, ch = gdn_params(nk, nv, 400); p["dt"] = np.zeros(nv, np.float32)
    g = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    S0 = synth.normal((nv, 128, 128), 79, 0.01)
    g.set_state(None, S0)
    qkv, z, beta, alpha = gdn_inputs(nv, ch, 1, 5000)
    # delta-rule property: g = 1, beta = 1 -> afterwards S^T k = v
    alpha[:] = -40.0; beta[:] = 40.0
    g.step(qkv, z, beta, alpha)
    _, S = g.get_state()
    w = p["conv_w"].reshape(ch, 4).astype(np.float64)
    o = w[:, 3] * qkv[0]; co = o / (1 + np.exp(-o))
    k = co[nk * 128:2 * nk * 128].reshape(nk, 128); k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6); v = co[2 * nk * 128:].reshape(nv, 128)
    for h in (0, 7, 31):
        assert relerr(S[h].astype(np.float64).T @ k[h % nk], v[h]) < 1e-5
    # pure decay: beta = 0 -> S' = g S
    g.set_state(None, S0); beta[:] = -200.0; alpha = synth.normal((1, nv), 9)
    g.step(qkv, z, beta, alpha)
    _, S = g.get_state()
    for h in (0, 13, 31):
        gg = np.exp(np.log1p(np.exp(float(alpha[0, h]))) * float(p["a"][h]))
        assert relerr(S[h], gg * S0[h].astype(np.float64)) < 1e-6


def test_gdn_window_equals_single_steps(ctx):
    nk, nv = 2, 4
    p, ch = gdn_params(nk, nv, 500)
    g1 = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    g2 = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    qkv, z, beta, alpha = gdn_inputs(nv, ch, 6, 6000)
    a = g1.step(qkv, z, beta, alpha)
    b = np.concatenate([g2.step(qkv[i:i + 1], z[i:i + 1], beta[i:i + 1], alpha[i:i + 1]) for i in range(6)])
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(g1.get_state()[1].view(np.uint32), g2.get_state()[1].view(np.uint32))


# ---- attention -------------------------------------------------------------------------------------------------------------
def attn_inputs(nh, nkv, seed, t):
    g = lambda s, shape, std=1.0: synth.normal(shape, seed * 100 + s, std)
    return dict(q=g(1, (t, nh * 2 * 256)), k=g(2, (t, nkv * 256)), v=g(3, (t, nkv * 256)), qn=1 + g(4, (256,), 0.1), kn=1 + g(5, (256,), 0.1))


@pytest.mark.parametrize("nh,nkv", [(4, 2), (16, 2)])
@pytest.mark.parametrize("kv_bits,recent,start", [(0, 1024, 0), (0, 1024, 300), (4, 64, 200), (4, 64, 700), (4, 1024, 1500)])
def test_attention_matches_oracle(ctx, nh, nkv, kv_bits, recent, start):
    t = 3
    p = attn_inputs(nh, nkv, 3 + start, t)
    row = nkv * 256
    kc = synth.normal((start, row), 6); vc = synth.normal((start, row), 7)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], kv_bits, recent, start + 16)
    att.load_cache(kc, vc)
    out = att.decode(p["q"], p["k"], p["v"])
    K = np.zeros((start + t, row), np.float32); V = np.zeros_like(K); K[:start] = kc; V[:start] = vc
    ref = orc.attn_core(nh, nkv, 256, 64, 1e-6, orc.rope_inv(64, 1e7), p["qn"], p["kn"], p["q"], p["k"], p["v"], start, kv_bits, recent, K, V)
    assert relerr(out, ref) <= 2e-5
    k2, v2 = att.read_cache()
    assert len(att) == start + t and relerr(k2, K) <= 1e-6 and np.array_equal(v2, V)


@pytest.mark.parametrize("nh", [4, 16])          # 2 and 8 heads per KV head: eight and two tokens of a window share a pass over the cache
def test_attention_token_by_token_growth_crosses_the_packing_boundary(ctx, nh):
    nkv, recent = 2, 64
    row = nkv * 256
    p = attn_inputs(nh, nkv, 9, 200)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 4, recent, 256)
    K = np.zeros((200, row), np.float32); V = np.zeros_like(K)
    inv = orc.rope_inv(64, 1e7)
    worst = 0.0
    i = 0
    for t in [1] * 130 + [8] * 8 + [3, 3]:
        out = att.decode(p["q"][i:i + t], p["k"][i:i + t], p["v"][i:i + t])
        ref = orc.attn_core(nh, nkv, 256, 64, 1e-6, inv, p["qn"], p["kn"], p["q"][i:i + t], p["k"][i:i + t], p["v"][i:i + t], i, 4, recent, K, V)
        worst = max(worst, relerr(out, ref)); i += t
    assert i == 200 and orc.packed_boundary(200, 4, recent) == 128 and worst <= 2e-5
    # the windows' rows are bit for bit what single steps give (the window 186..193 spans the move of the 4-bit boundary at 192)
    att2 = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 4, recent, 256)
    att2.load_cache(*[x[:186] for x in att.read_cache()])
    att3 = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 4, recent, 256)
    att3.load_cache(*[x[:186] for x in att.read_cache()])
    win = att2.decode(p["q"][186:194], p["k"][186:194], p["v"][186:194])
    one = np.concatenate([att3.decode(p["q"][j:j + 1], p["k"][j:j + 1], p["v"][j:j + 1]) for j in range(186, 194)])
    assert np.array_equal(win.view(np.uint32), one.view(np.uint32))


def test_attention_closed_forms(ctx):
    nh, nkv = 16, 2
    p = attn_inputs(nh, nkv, 11, 1)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 4, 1024, 64)
    out = att.decode(p["q"], p["k"], p["v"])       # a single position: out = v * sigmoid(gate)
    for h in range(nh):
        gate = p["q"][0].reshape(nh, 512)[h, 256:].astype(np.float64)
        assert relerr(out[0].reshape(nh, 256)[h], p["v"][0].reshape(nkv, 256)[h // 8] / (1 + np.exp(-gate))) < 1e-6
    # all keys zero -> uniform softmax -> mean of the values
    att2 = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 0, 1024, 64)
    n = 9; vc = synth.normal((n, nkv * 256), 5)
    att2.load_cache(np.zeros((n, nkv * 256), np.float32), vc)
    p["k"][:] = 0
    out = att2.decode(p["q"], p["k"], p["v"])
    allv = np.concatenate([vc, p["v"]]).astype(np.float64).reshape(n + 1, nkv, 256).mean(0)
    for h in (0, 9, 15):
        gate = p["q"][0].reshape(nh, 512)[h, 256:].astype(np.float64)
        assert relerr(out[0].reshape(nh, 256)[h], allv[h // 8] / (1 + np.exp(-gate))) < 1e-5


# ---- QSA sparse indexer + YaRN ------------------------------------------------------------------------------------------------
INH, IHD, IR, IBUD = 3, 128, 4, 64          # dense up to 67 visible positions


def qsa_inputs(nh, nkv, seed, t):
    g = lambda s, shape, std=1.0: synth.normal(shape, seed * 100 + s, std)
    p = attn_inputs(nh, nkv, seed, t)
    p.update(iq=g(11, (t, INH * IHD)), ik=g(12, (t, IHD)), iqn=1 + g(13, (IHD,), 0.1), ikn=1 + g(14, (IHD,), 0.1))
    return p


def pooled(ik, ikn, inv, mscale=1.0):
    nb = ik.shape[0] // IR
    return np.stack([np_ref.qsa_pool(ik[b * IR:(b + 1) * IR], ikn, 1e-6, b * IR, 64, inv, mscale) for b in range(nb)]).astype(np.float32) if nb else np.zeros((0, IHD), np.float32)


@pytest.mark.parametrize("kv_bits,recent,start,t", [(0, 1024, 150, 5), (4, 64, 300, 8), (0, 1024, 64, 6), (4, 64, 1000, 3), (0, 1024, 20, 8)])
def test_qsa_attention_selection_and_output_match_oracle(ctx, kv_bits, recent, start, t):
    nh, nkv = 16, 2
    row = nkv * 256
    p = qsa_inputs(nh, nkv, 7 + start, t)
    kc = synth.normal((start, row), 6); vc = synth.normal((start, row), 7); ikc = synth.normal((start, IHD), 8)
    inv = orc.rope_inv(64, 1e7)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], kv_bits, recent, start + 16)
    att.set_indexer(INH, IHD, IR, IBUD, p["iqn"], p["ikn"])
    att.load_cache(kc, vc); att.load_index(ikc)
    ik0, ib0 = att.read_index()
    ibc = pooled(ikc, p["ikn"], inv)
    assert np.array_equal(ik0, ikc) and relerr(ib0, ibc) <= 1e-6 and ib0.shape == (start // IR, IHD)
    out = att.decode(p["q"], p["k"], p["v"], p["iq"], p["ik"])
    K = np.zeros((start + t, row), np.float32); V = np.zeros_like(K); K[:start] = kc; V[:start] = vc
    IK = np.zeros((start + t, IHD), np.float32); IK[:start] = ikc
    IB = np.zeros(((start + t) // IR, IHD), np.float32); IB[:start // IR] = ib0          # the device's own pooled keys: same selection inputs on both sides
    ref, sel = orc.attn_core_qsa(nh, nkv, 256, 64, 1e-6, inv, 1.0, p["qn"], p["kn"], p["q"], p["k"], p["v"], start, kv_bits, recent, K, V,
                                 INH, IHD, IR, IBUD, p["iqn"], p["ikn"], p["iq"], p["ik"], IK, IB)
    for ti in range(t):
        got = att.selection(ti)
        if sel[ti] is None:
            assert got is None, ti
        else:
            assert got is not None and np.array_equal(got, sel[ti]), ti
    assert relerr(out, ref) <= 2e-5
    ik2, ib2 = att.read_index()
    assert np.array_equal(ik2, IK) and relerr(ib2, IB) <= 1e-6
    if start + t > IBUD + IR - 1:
        assert sel[t - 1] is not None and len(sel[t - 1]) == IBUD + (start + t) % IR


def test_qsa_growth_from_empty_crosses_dense_limit_and_packing_boundary(ctx):
    nh, nkv, recent = 4, 2, 64
    row = nkv * 256; N = 200
    p = qsa_inputs(nh, nkv, 19, N)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 4, recent, 256)
    att.set_indexer(INH, IHD, IR, IBUD, p["iqn"], p["ikn"])
    K = np.zeros((N, row), np.float32); V = np.zeros_like(K); IK = np.zeros((N, IHD), np.float32); IB = np.zeros((N // IR, IHD), np.float32)
    inv = orc.rope_inv(64, 1e7)
    worst = 0.0; i = 0; sparse_seen = 0
    for t in [1] * 75 + [8] * 10 + [3, 5, 7, 1, 1, 1, 2, 8, 8, 8, 1]:
        sl = slice(i, i + t)
        out = att.decode(p["q"][sl], p["k"][sl], p["v"][sl], p["iq"][sl], p["ik"][sl])
        ref, sel = orc.attn_core_qsa(nh, nkv, 256, 64, 1e-6, inv, 1.0, p["qn"], p["kn"], p["q"][sl], p["k"][sl], p["v"][sl], i, 4, recent, K, V,
                                     INH, IHD, IR, IBUD, p["iqn"], p["ikn"], p["iq"][sl], p["ik"][sl], IK, IB)
        for ti in range(t):
            got = att.selection(ti)
            assert (got is None) == (sel[ti] is None) and (got is None or np.array_equal(got, sel[ti])), (i, ti)
            sparse_seen += got is not None
        worst = max(worst, relerr(out, ref)); i += t
    assert i == N and sparse_seen == N - (IBUD + IR - 1) and worst <= 2e-5
    _, ib = att.read_index()
    assert relerr(ib, IB) <= 1e-6


def test_qsa_equal_scores_take_the_lowest_blocks_and_yarn_changes_the_rotation(ctx):
    nh, nkv = 4, 2
    row = nkv * 256; start = 160
    p = qsa_inputs(nh, nkv, 23, 1)
    # index queries whose dot with every block key is negative: all scores are exactly zero -> blocks 0..15 + tail
    u = np.zeros(IHD, np.float32); u[64:] = 1.0
    ikc = np.tile(u, (start, 1)).astype(np.float32); p["iq"] = np.tile(-u, (1, INH)).astype(np.float32); p["iqn"] = np.ones(IHD, np.float32); p["ikn"] = np.ones(IHD, np.float32)
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, p["qn"], p["kn"], 0, 1024, 256)
    att.set_indexer(INH, IHD, IR, IBUD, p["iqn"], p["ikn"])
    att.set_context(128, 256)                                      # YaRN x2
    kc = synth.normal((start, row), 6); vc = synth.normal((start, row), 7)
    att.load_cache(kc, vc); att.load_index(ikc)
    out = att.decode(p["q"], p["k"], p["v"], p["iq"], p["ik"])
    assert list(att.selection(0)) == list(range(IBUD)) + [start]
    inv, ms = orc.rope_inv_yarn(64, 1e7, 128, 256)
    assert ms > 1.0
    K = np.zeros((start + 1, row), np.float32); V = np.zeros_like(K); K[:start] = kc; V[:start] = vc
    IK = np.zeros((start + 1, IHD), np.float32); IK[:start] = ikc; IB = np.zeros(((start + 1) // IR, IHD), np.float32); IB[:start // IR] = pooled(ikc, p["ikn"], inv, ms)
    ref, sel = orc.attn_core_qsa(nh, nkv, 256, 64, 1e-6, inv, ms, p["qn"], p["kn"], p["q"], p["k"], p["v"], start, 0, 1024, K, V,
                                 INH, IHD, IR, IBUD, p["iqn"], p["ikn"], p["iq"], p["ik"], IK, IB)
    assert list(sel[0]) == list(range(IBUD)) + [start] and relerr(out, ref) <= 2e-5
    k2, _ = att.read_cache()
    assert relerr(k2[start], K[start]) <= 1e-6
    _, ib = att.read_index()
    assert relerr(ib, IB[:start // IR]) <= 1e-6
    # without the factor and the scaled frequencies the new key row differs
    plain = orc.attn_core(nh, nkv, 256, 64, 1e-6, orc.rope_inv(64, 1e7), p["qn"], p["kn"], p["q"], p["k"], p["v"], start, 0, 1024, K.copy(), V.copy())
    assert relerr(out, plain) > 1e-3


# ---- chunked DeltaNet prefill (matrix cores) against the sequential recurrence ---------------------------------------------
@pytest.mark.parametrize("nk,nv,T", [(2, 4, 64), (2, 4, 200), (16, 32, 512)])
def test_gdn_chunked_prefill_matches_sequential_oracle(ctx, nk, nv, T):
    p, ch = gdn_params(nk, nv, 700 + nv); p["dt"] = np.zeros(nv, np.float32)
    g = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    S0 = synth.normal((nv, 128, 128), 81, 0.01); cs0 = synth.normal((3, ch), 82, 0.3)
    g.set_state(cs0, S0)
    qkv, z, beta, alpha = gdn_inputs(nv, ch, T, 9000)
    out = g.prefill_chunked(qkv, z, beta, alpha)
    so, co = S0.copy().reshape(-1), cs0.copy().reshape(-1)
    ref = orc.gdn_core(nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"], qkv, z, beta, alpha, co, so)
    assert relerr(out, ref) <= TOL
    conv, ssm = g.get_state()
    assert relerr(ssm, so) <= TOL and np.array_equal(conv.reshape(-1), co)
    # and the chunked state continues exactly like the recurrent one would: one more decode step on top
    q1, z1, b1, a1 = gdn_inputs(nv, ch, 1, 9100)
    o1 = g.step(q1, z1, b1, a1)
    r1 = orc.gdn_core(nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"], q1, z1, b1, a1, co, so)
    assert relerr(o1, r1) <= TOL


def test_gdn_chunked_prefill_benchmark_length_against_the_step_kernels(ctx):
    # 4096 tokens, 16 QK / 32 V heads, chunk 64: the sequential device kernels (themselves pinned against the oracle)
    # are the reference at this length
    nk, nv, T = 16, 32, 4096
    p, ch = gdn_params(nk, nv, 800); p["dt"] = np.zeros(nv, np.float32)
    ga = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    gb = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"])
    S0 = synth.normal((nv, 128, 128), 83, 0.01)
    ga.set_state(None, S0); gb.set_state(None, S0)
    qkv, z, beta, alpha = gdn_inputs(nv, ch, T, 9500)
    a = ga.prefill_chunked(qkv, z, beta, alpha)
    b = gb.step(qkv, z, beta, alpha)
    assert relerr(a, b) <= TOL
    assert relerr(ga.get_state()[1], gb.get_state()[1]) <= TOL
