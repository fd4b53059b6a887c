"""Closed-form pins of the oracle's hyper-connection mixer, hyper-connection combine, MoE FFN body and token-step
composition (qwen4exp_gguf.rs:1357-1388, 1675-1684, 1721-1793, 2087-2157): special cases whose answer can be written
down by hand, chosen so that a plausible misreading -- the divide by hc on the wrong side of silu, a missing 2 in the
combine weight, softmax over all experts instead of the chosen ones, an expert matrix indexed the wrong way round, a
mix whose inject factors are applied to the wrong combine -- fails at least one of them.  Nothing here re-states the
oracle's formulas as a second implementation: every expected value is an explicit number or a one-line closed form."""
import numpy as np

import orc
from helpers import orc_model, orc_tensor, relerr
from pyre_amd import modelgen as mg
from pyre_amd import synth


def f32t(a):
    """F32 tensor (rows x cols) for the oracle, kept alive by the returned array."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    return orc.tensor(orc.F32, a.shape[0], a.shape[1], a), a


def sig(v):
    return 1.0 / (1.0 + np.exp(-np.asarray(v, dtype=np.float64)))


def silu(v):
    v = np.asarray(v, dtype=np.float64)
    return v * sig(v)


def rms64(x, w, eps):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean() + eps) * np.asarray(w, dtype=np.float64)


D, HC, LR, EPS = 8, 4, 3, 1e-6


def streams(seed=1):
    g = np.random.Generator(np.random.PCG64(seed))
    x = g.standard_normal((1, HC * D)).astype(np.float32)
    norm = (1 + 0.2 * g.standard_normal(HC * D)).astype(np.float32)
    xn = np.concatenate([rms64(x[0, s * D:(s + 1) * D], norm[s * D:(s + 1) * D], EPS) for s in range(HC)])
    return g, x, norm, xn


# ---- hc_mix ---------------------------------------------------------------------------------------------------------------
def test_rms_of_a_constant_vector():
    # x = c everywhere: x / sqrt(c^2 + eps) * w -- the mean of squares (not the sum) under the root, eps inside it
    w = np.array([1.0, 2.0, -0.5, 3.0], np.float32); y = np.empty(4, np.float32)
    x = np.full(4, 3.0, np.float32)
    orc.lib().orc_rms(orc._p(x), orc._p(w), orc.C.c_float(0.25), orc._p(y), orc.C.c_size_t(4))
    assert relerr(y, 3.0 / np.sqrt(9.25) * w.astype(np.float64)) < 1e-6


def test_hc_mix_with_zero_up_is_half_the_stream_mean():
    g, x, norm, xn = streams(1)
    down, _d = f32t(g.standard_normal((LR, HC * D))); inject, _i = f32t(g.standard_normal((HC, HC * D))); up, _u = f32t(np.zeros((HC * D, LR)))
    mixed, inj = orc.hc_mix(D, HC, EPS, norm, down, inject, up, x)
    # gate = 0 -> sigmoid = 1/2 -> mixed = (sum_s xn_s / 2) / hc
    assert relerr(mixed[0], 0.5 * xn.reshape(HC, D).mean(0)) < 1e-6
    # inject rows are plain dot products with the normalised streams, divided by hc, with no activation
    assert relerr(inj[0], (_i.astype(np.float64) @ xn) / HC) < 1e-6


def test_hc_mix_with_zero_down_has_zero_gate_whatever_up_is():
    g, x, norm, xn = streams(2)
    down, _d = f32t(np.zeros((LR, HC * D))); up, _u = f32t(10 * g.standard_normal((HC * D, LR)))
    mixed, inj = orc.hc_mix(D, HC, EPS, norm, down, None, up, x)
    assert relerr(mixed[0], 0.5 * xn.reshape(HC, D).mean(0)) < 1e-6     # silu(0 / hc) = 0 -> gate = 0
    assert not inj.any()                                                # no inject matrix (the head mixer): zeros


def test_hc_mix_one_hot_rows_pin_the_order_of_divide_and_silu_and_the_gate_layout():
    g, x, norm, xn = streams(3)
    # down row i picks element j_i of the flattened normalised streams; inject row s picks element m_s;
    # up row k (stream-major, k = s*d + i) picks low-rank element (k % LR) scaled by 3
    j = [5, 17, 30]; m = [2, 9, 20, 31]
    dn = np.zeros((LR, HC * D)); dn[np.arange(LR), j] = 1.0
    ij = np.zeros((HC, HC * D)); ij[np.arange(HC), m] = 1.0
    upm = np.zeros((HC * D, LR)); upm[np.arange(HC * D), np.arange(HC * D) % LR] = 3.0
    down, _d = f32t(dn); inject, _i = f32t(ij); up, _u = f32t(upm)
    mixed, inj = orc.hc_mix(D, HC, EPS, norm, down, inject, up, x)
    assert relerr(inj[0], xn[m] / HC) < 1e-6
    lo = silu(xn[j] / HC)                         # silu of (o / hc): silu(o) / hc would differ, silu is not linear
    assert np.abs(lo - silu(xn[j]) / HC).max() > 1e-3
    gate = 3.0 * lo[np.arange(HC * D) % LR]
    expect = (xn * sig(gate)).reshape(HC, D).sum(0) / HC
    assert relerr(mixed[0], expect) < 1e-6
    # the same gate read token-major (k = i*hc + s) gives something else: the layout is pinned
    wrong = (xn.reshape(HC, D) * sig(gate).reshape(D, HC).T).sum(0) / HC
    assert relerr(mixed[0], wrong) > 1e-3


def test_hc_mix_windows_are_per_token():
    g, x, norm, xn = streams(4)
    down, _d = f32t(g.standard_normal((LR, HC * D))); inject, _i = f32t(g.standard_normal((HC, HC * D))); up, _u = f32t(g.standard_normal((HC * D, LR)))
    x2 = np.concatenate([x, g.standard_normal((2, HC * D)).astype(np.float32)])
    m3, i3 = orc.hc_mix(D, HC, EPS, norm, down, inject, up, x2)
    for ti in range(3):
        m1, i1 = orc.hc_mix(D, HC, EPS, norm, down, inject, up, x2[ti:ti + 1])
        assert np.array_equal(m1[0], m3[ti]) and np.array_equal(i1[0], i3[ti])


# ---- hc_combine -------------------------------------------------------------------------------------------------------------
def test_hc_combine_weights():
    g = np.random.Generator(np.random.PCG64(5))
    x = g.standard_normal((1, HC * D)).astype(np.float32); out = g.standard_normal((1, D)).astype(np.float32)
    # inject = 0: weight 2 * sigmoid(0) = 1, every stream gets the same vector added, exactly
    y = orc.hc_combine(D, HC, x, out, np.zeros((1, HC), np.float32)).reshape(HC, D)
    assert np.array_equal(y, x.reshape(HC, D) + out[0])
    # inject -> -inf: unchanged; inject -> +inf: plus twice the vector; one stream at ln 3: weight 2 * 3/4 = 1.5
    inj = np.array([[-200.0, 200.0, np.log(3.0), 0.0]], np.float32)
    y = orc.hc_combine(D, HC, x, out, inj).reshape(HC, D).astype(np.float64)
    xs = x.reshape(HC, D).astype(np.float64); o = out[0].astype(np.float64)
    assert relerr(y[0], xs[0]) < 1e-7 and relerr(y[1], xs[1] + 2 * o) < 1e-6 and relerr(y[2], xs[2] + 1.5 * o) < 1e-6 and relerr(y[3], xs[3] + o) < 1e-6


# ---- MoE FFN ------------------------------------------------------------------------------------------------------------------
MD, MFF, ME, MK = 8, 4, 4, 2


def moe_call(W, x, sgi):
    t = {k: f32t(v) for k, v in W.items()}
    y, idx, w = orc.moe_ffn(MD, ME, MK, MFF, t["router"][0], t["gate_e"][0], t["up_e"][0], t["down_e"][0], np.asarray(sgi, np.float32),
                            t["sh_gate"][0], t["sh_up"][0], t["sh_down"][0], x)
    return y, idx, w


def zero_moe():
    return {"router": np.zeros((ME, MD)), "gate_e": np.zeros((ME * MFF, MD)), "up_e": np.zeros((ME * MFF, MD)), "down_e": np.zeros((ME * MD, MFF)),
            "sh_gate": np.zeros((MFF, MD)), "sh_up": np.zeros((MFF, MD)), "sh_down": np.zeros((MD, MFF))}


def test_moe_shared_expert_alone_with_zero_gate_vector_is_halved():
    x = np.array([[0.5, -1.0, 2.0, 0.25, 1.5, -0.75, 3.0, -2.0]], np.float32)
    W = zero_moe()
    for i in range(MFF):
        W["sh_gate"][i, i] = 1.0; W["sh_up"][i, MFF + i] = 1.0; W["sh_down"][i, i] = 1.0     # g_i = x_i, u_i = x_{4+i}, y_i = h_i
    W["sh_down"][7, 2] = -2.0                                                               # y_7 = -2 h_2
    y, _, _ = moe_call(W, x, np.zeros(MD))
    h = silu(x[0, :MFF]) * x[0, MFF:].astype(np.float64)           # silu on the gate branch, the up branch plain
    expect = np.zeros(MD); expect[:MFF] = 0.5 * h; expect[7] = 0.5 * -2.0 * h[2]
    assert relerr(y[0], expect) < 1e-6
    assert np.abs(h - x[0, :MFF] * silu(x[0, MFF:])).max() > 1e-2   # the roles of the two branches are not interchangeable here
    # a gate vector: sigmoid(sh_gate_inp . x), e.g. picks x_2 = 2 -> sigmoid(2)
    sgi = np.zeros(MD); sgi[2] = 1.0
    y, _, _ = moe_call(W, x, sgi)
    assert relerr(y[0], expect * 2 * sig(2.0)) < 1e-6


def test_moe_routing_renormalises_over_the_chosen_experts_and_a_zero_expert_adds_nothing():
    x = np.array([[1.0, 0.0, 0.0, 0.0, 0.5, -1.5, 2.0, 0.0]], np.float32)
    W = zero_moe()
    logits = np.array([0.3, 1.7, -0.4, 0.9])
    W["router"][:, 0] = logits                                          # logit_e = router[e] . x = logits[e] * x_0
    g = np.random.Generator(np.random.PCG64(6))
    W["gate_e"] = g.standard_normal((ME * MFF, MD)); W["up_e"] = g.standard_normal((ME * MFF, MD)); W["down_e"] = g.standard_normal((ME * MD, MFF))
    W["down_e"][3 * MD:4 * MD] = 0.0                                    # expert 3 is chosen but projects to zero
    y, idx, w = moe_call(W, x, np.zeros(MD))
    assert list(idx[0]) == [1, 3]                                       # the two largest logits, ascending expert id
    w1 = 1.0 / (1.0 + np.exp(0.9 - 1.7))                                # softmax over the two chosen logits only
    assert abs(w[0, 0] - w1) < 1e-6 and abs(w[0, 1] - (1 - w1)) < 1e-6
    assert abs(w1 - np.exp(1.7) / np.exp(logits).sum()) > 0.1           # (a softmax over all four would be something else)
    x64 = x[0].astype(np.float64)
    G1 = W["gate_e"][1 * MFF:2 * MFF]; U1 = W["up_e"][1 * MFF:2 * MFF]; D1 = W["down_e"][1 * MD:2 * MD]     # expert e = rows e*ff.. / e*d..
    expect = w1 * (D1 @ (silu(G1 @ x64) * (U1 @ x64)))
    assert relerr(y[0], expect) < 1e-6
    # the shared expert is zero here, so its sigmoid gate must not leak into the routed sum
    y2, _, _ = moe_call(W, x, 5 * np.ones(MD))
    assert np.array_equal(y2, y)


def test_moe_of_all_ones_q8_0_matrices():
    # Q8_0 blocks with d = 1 and every code +1: each row of every matrix is all ones, so gate . x = up . x = S = sum(x),
    # every hidden unit is silu(S) S, and a down row sums ff of them.  Router logits are all S: ties -> experts 0..k-1,
    # weights 1/k each, so y_r = sigmoid(sgi . x) sf silu(S) S + ff silu(S) S.
    d, ff, E, k = 64, 32, 4, 2
    def ones(rows, cols):
        b = np.zeros((rows * cols // 32, 34), np.uint8); b[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8); b[:, 2:] = 1
        b = b.reshape(-1).copy()
        return orc.tensor(orc.Q8_0, rows, cols, b), b
    x = (np.arange(d, dtype=np.float32) - 20.0) / 64.0
    S = float(x.astype(np.float64).sum()); hval = float(silu(S) * S)
    router, _r = ones(E, d); ge, _g = ones(E * ff, d); ue, _u = ones(E * ff, d); de, _d = ones(E * d, ff); sg, _a = ones(ff, d); su, _b = ones(ff, d); sd, _c = ones(d, ff)
    sgi = np.zeros(d, np.float32); sgi[0] = 1.0                          # sigmoid(x_0)
    y, idx, w = orc.moe_ffn(d, E, k, ff, router, ge, ue, de, sgi, sg, su, sd, x[None])
    assert list(idx[0]) == [0, 1] and np.allclose(w, 0.5)
    assert relerr(y[0], np.full(d, ff * hval * float(sig(x[0])) + ff * hval)) < 1e-5


# ---- the token step's composition -------------------------------------------------------------------------------------------
def tiny_model(seed, zero_slots=()):
    c = mg.Config(n_layers=4, d=256, hc=2, hc_lr=32, n_exp=8, top_k=2, ff_exp=256, vocab=512, kv_recent=64)
    hw = mg.build_host(c, seed=seed)
    for L in hw.layers:
        for s in zero_slots:
            if s in L:
                ty, rows, cols, b = L[s]; L[s] = (ty, rows, cols, np.zeros_like(b))      # all-zero blocks decode to zero (d = 0)
    return c, hw


def head_of(c, hw, xs):
    G = hw.globals_
    h, _ = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(-1, mg.G_HEAD_NORM), orc_tensor(G[mg.G_HEAD_DOWN]), None, orc_tensor(G[mg.G_HEAD_UP]), xs)
    ty, rows, cols, b = G[mg.G_OUT]
    return orc.matmul(ty, b, rows, cols, h)[0]


def embedding(c, hw, tok):
    ty, rows, cols, b = hw.globals_[mg.G_EMBD]
    el, bs, _ = synth.GEOM[ty]; rb = cols // el * bs
    return orc.dequant(ty, b[tok * rb:(tok + 1) * rb], cols)


def test_forward_with_every_block_output_zeroed_is_the_head_of_the_tiled_embedding():
    # zero output projections (attention, DeltaNet) and zero down projections (experts, shared expert): every layer adds
    # zero to the streams, so the logits are head(hc_mix_head(embedding tiled over the streams)) of the LAST token
    c, hw = tiny_model(31, zero_slots=(mg.ATTN_O, mg.LIN_OUT, mg.DOWN_E, mg.SH_DOWN))
    m = orc_model(hw); st = m.new_state()
    ids = np.array([7, 400, 33], dtype=np.uint32)
    lg = m.forward(ids, st)
    e = embedding(c, hw, 33)
    assert np.array_equal(lg, head_of(c, hw, np.tile(e, c.hc)[None]))
    assert not np.array_equal(lg, head_of(c, hw, np.tile(embedding(c, hw, 7), c.hc)[None]))
    assert len(st) == 3


def test_forward_with_one_live_ffn_is_mix_ffn_combine_on_that_layer():
    # only layer 2's FFN writes to the streams: x = tile(e); (m, inj) = mix_f(x); x += ffn(m) * 2 sigmoid(inj); logits =
    # head(x) -- from the block entry points pinned above.  A combine that used the attention-side inject factors, or a
    # layer that fed the FFN the un-mixed stream, would not reproduce it.
    c, hw = tiny_model(32, zero_slots=(mg.ATTN_O, mg.LIN_OUT))
    for il, L in enumerate(hw.layers):
        if il != 2:
            for s in (mg.DOWN_E, mg.SH_DOWN):
                ty, rows, cols, b = L[s]; L[s] = (ty, rows, cols, np.zeros_like(b))
    m = orc_model(hw); st = m.new_state()
    lg = m.forward(np.array([99], dtype=np.uint32), st)
    L = hw.layers[2]
    x = np.tile(embedding(c, hw, 99), c.hc)[None]
    mixed, inj = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(2, mg.HCF_NORM), orc_tensor(L[mg.HCF_DOWN]), orc_tensor(L[mg.HCF_INJECT]), orc_tensor(L[mg.HCF_UP]), x)
    o, _, _ = orc.moe_ffn(c.d, c.n_exp, c.top_k, c.ff_exp, *(orc_tensor(L[s]) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E)),
                          hw.f32(2, mg.SH_GATE_INP), *(orc_tensor(L[s]) for s in (mg.SH_GATE, mg.SH_UP, mg.SH_DOWN)), mixed)
    x1 = orc.hc_combine(c.d, c.hc, x, o, inj).reshape(1, -1)
    assert np.abs(o).max() > 0 and np.array_equal(lg, head_of(c, hw, x1))
    # with the attention-side mixer's inject factors instead the result differs
    _, inj_a = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(2, mg.HCA_NORM), orc_tensor(L[mg.HCA_DOWN]), orc_tensor(L[mg.HCA_INJECT]), orc_tensor(L[mg.HCA_UP]), x)
    assert not np.array_equal(lg, head_of(c, hw, orc.hc_combine(c.d, c.hc, x, o, inj_a).reshape(1, -1)))


def test_forward_with_one_live_deltanet_layer_is_mix_projections_core_out_combine():
    # only layer 0's Gated DeltaNet writes to the streams (every FFN is zeroed, the other mixers' outputs too)
    c, hw = tiny_model(33, zero_slots=(mg.ATTN_O, mg.DOWN_E, mg.SH_DOWN))
    for il, L in enumerate(hw.layers):
        if il != 0 and mg.LIN_OUT in L:
            ty, rows, cols, b = L[mg.LIN_OUT]; L[mg.LIN_OUT] = (ty, rows, cols, np.zeros_like(b))
    m = orc_model(hw); st = m.new_state()
    ids = np.array([5, 250], dtype=np.uint32)
    L = hw.layers[0]
    conv = np.zeros((c.conv_k - 1) * c.ch, np.float32); ssm = np.zeros(c.lin_nv * c.lin_dk * c.lin_dv, np.float32)
    for tok in ids:
        lg = m.forward(np.array([tok], dtype=np.uint32), st)
        x = np.tile(embedding(c, hw, int(tok)), c.hc)[None]
        mixed, inj = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(0, mg.HCA_NORM), orc_tensor(L[mg.HCA_DOWN]), orc_tensor(L[mg.HCA_INJECT]), orc_tensor(L[mg.HCA_UP]), x)
        pr = {s: orc.matmul(L[s][0], L[s][3], L[s][1], L[s][2], mixed) for s in (mg.LIN_QKV, mg.LIN_Z, mg.LIN_BETA, mg.LIN_ALPHA)}
        oa = orc.gdn_core(c.lin_nk, c.lin_nv, c.lin_dk, c.lin_dv, c.conv_k, c.eps, hw.f32(0, mg.LIN_A), hw.f32(0, mg.LIN_DT), hw.f32(0, mg.LIN_CONV), hw.f32(0, mg.LIN_NORM),
                          pr[mg.LIN_QKV], pr[mg.LIN_Z], pr[mg.LIN_BETA], pr[mg.LIN_ALPHA], conv, ssm)       # the state carries over the two tokens
        o = orc.matmul(L[mg.LIN_OUT][0], L[mg.LIN_OUT][3], L[mg.LIN_OUT][1], L[mg.LIN_OUT][2], oa)
        x1 = orc.hc_combine(c.d, c.hc, x, o, inj).reshape(1, -1)
        assert np.abs(o).max() > 0 and np.array_equal(lg, head_of(c, hw, x1)), tok
    assert np.array_equal(st.ssm(0), ssm) and np.array_equal(st.conv(0), conv)


def test_forward_with_one_live_attention_layer_is_mix_projections_core_out_combine():
    # only layer 3's gated attention writes to the streams (every FFN and every DeltaNet output projection is zeroed): over
    # three tokens the logits are head(combine(tile(e), attn_output(attn_core(q, k, v over the layer's own cache)), inject))
    # with the attention-side mix, the [q ; k ; v] projections of the mixed vector, the cache carried across the tokens and
    # the token's own position -- from the block entry points pinned in test_oracle_blocks.py.
    c, hw = tiny_model(34, zero_slots=(mg.LIN_OUT, mg.DOWN_E, mg.SH_DOWN))
    m = orc_model(hw); st = m.new_state()
    L = hw.layers[3]; assert mg.ATTN_O in L
    row = c.n_kv * c.hd
    K = np.zeros((16, row), np.float32); V = np.zeros((16, row), np.float32)
    inv = orc.rope_inv(c.n_rot, c.rope_base)
    mm = lambda s, x: orc.matmul(L[s][0], L[s][3], L[s][1], L[s][2], x)
    for pos, tok in enumerate((5, 250, 77)):
        lg = m.forward(np.array([tok], dtype=np.uint32), st)
        x = np.tile(embedding(c, hw, tok), c.hc)[None]
        mixed, inj = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(3, mg.HCA_NORM), orc_tensor(L[mg.HCA_DOWN]), orc_tensor(L[mg.HCA_INJECT]), orc_tensor(L[mg.HCA_UP]), x)
        q, k, v = mm(mg.ATTN_Q, mixed), mm(mg.ATTN_K, mixed), mm(mg.ATTN_V, mixed)
        oa = orc.attn_core(c.n_head, c.n_kv, c.hd, c.n_rot, c.eps, inv, hw.f32(3, mg.ATTN_QN), hw.f32(3, mg.ATTN_KN), q, k, v, pos, c.kv_bits, c.kv_recent, K, V)
        o = mm(mg.ATTN_O, oa)
        x1 = orc.hc_combine(c.d, c.hc, x, o, inj).reshape(1, -1)
        assert np.abs(o).max() > 0 and np.array_equal(lg, head_of(c, hw, x1)), pos
        # the FFN-side mixer's inject factors, or a cache that forgot the earlier tokens, give something else
        _, inj_f = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(3, mg.HCF_NORM), orc_tensor(L[mg.HCF_DOWN]), orc_tensor(L[mg.HCF_INJECT]), orc_tensor(L[mg.HCF_UP]), x)
        assert not np.array_equal(lg, head_of(c, hw, orc.hc_combine(c.d, c.hc, x, o, inj_f).reshape(1, -1)))
        if pos > 0:
            K0 = np.zeros_like(K); V0 = np.zeros_like(V)
            o0 = mm(mg.ATTN_O, orc.attn_core(c.n_head, c.n_kv, c.hd, c.n_rot, c.eps, inv, hw.f32(3, mg.ATTN_QN), hw.f32(3, mg.ATTN_KN), q, k, v, 0, c.kv_bits, c.kv_recent, K0, V0))
            assert not np.array_equal(o0, o)
    assert np.array_equal(st.kcache(0).reshape(-1, row)[:3], K[:3]) and np.array_equal(st.vcache(0).reshape(-1, row)[:3], V[:3])
