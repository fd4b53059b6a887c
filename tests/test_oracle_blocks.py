"""Pins the oracle's block-level math (no GPU): Gated DeltaNet step, gated attention, MoE FFN, hyper-connections and
the whole token step, through closed forms and the independent float64 numpy statements of np_ref."""
import numpy as np
import pytest

import np_ref
import orc
from helpers import dense, np_forward_tokens, orc_model, orc_tensor, relerr
from pyre_amd import modelgen as mg
from pyre_amd import synth

NK, NV, DK, DV, CK = 2, 4, 128, 128, 4
CH = 2 * NK * DK + NV * DV


def gdn_inputs(seed, t=1):
    g = lambda s, shape, std=1.0: synth.normal(shape, seed * 100 + s, std)
    a = -np.exp(synth.uniform((NV,), seed * 100 + 1, 0.0, np.log(16.0)))
    return dict(a=a, dt=np.zeros(NV, np.float32), conv_w=g(2, (CH * CK,), 0.5), norm_w=1 + g(3, (DV,), 0.1),
                qkv=g(4, (t, CH)), z=g(5, (t, NV * DV)), beta=g(6, (t, NV)), alpha=g(7, (t, NV)))


def run_gdn(p, conv_state, S, eps=1e-6):
    cs = np.ascontiguousarray(conv_state, np.float32).copy(); s = np.ascontiguousarray(S, np.float32).copy()
    out = orc.gdn_core(NK, NV, DK, DV, CK, eps, p["a"], p["dt"], p["conv_w"], p["norm_w"], p["qkv"], p["z"], p["beta"], p["alpha"], cs, s)
    return out, cs, s


def test_gdn_matches_numpy_over_several_tokens():
    p = gdn_inputs(1, t=5)
    S0 = synth.normal((NV, DK, DV), 77, 0.01); cs0 = synth.normal((CK - 1, CH), 78, 0.3)
    out, cs, s = run_gdn(p, cs0, S0)
    cn, Sn = cs0.astype(np.float64), S0.astype(np.float64)
    for ti in range(5):
        on, cn, Sn = np_ref.gdn_step(NK, NV, DK, DV, CK, 1e-6, p["a"], p["dt"], p["conv_w"], p["norm_w"], p["qkv"][ti], p["z"][ti], p["beta"][ti], p["alpha"][ti], cn, Sn)
        assert relerr(out[ti], on) < 1e-5, ti
    assert relerr(s, Sn.reshape(-1)) < 1e-5 and relerr(cs, cn.reshape(-1)) == 0.0


def test_gdn_zero_state_closed_form():
    # S = 0, conv = identity on the newest tap: o_h = (k.q) * beta * v before the gated norm
    p = gdn_inputs(2)
    w = np.zeros((CH, CK), np.float32); w[:, CK - 1] = 1.0; p["conv_w"] = w.reshape(-1)
    out, cs, S = run_gdn(p, np.zeros((CK - 1, CH)), np.zeros((NV, DK, DV)))
    co = np_ref.silu(p["qkv"][0].astype(np.float64))
    q = co[:NK * DK].reshape(NK, DK); k = co[NK * DK:2 * NK * DK].reshape(NK, DK); v = co[2 * NK * DK:].reshape(NV, DV)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) / np.sqrt(DK); k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    for h in range(NV):
        b = np_ref.sigm(float(p["beta"][0, h]))
        o = (k[h % NK] @ q[h % NK]) * b * v[h]
        exp = np_ref.rms(o, p["norm_w"].astype(np.float64), 1e-6) * np_ref.sigm(p["z"][0, h * DV:(h + 1) * DV].astype(np.float64))
        assert relerr(out[0, h * DV:(h + 1) * DV], exp) < 1e-5
        assert relerr(S.reshape(NV, DK, DV)[h], np.outer(k[h % NK], b * v[h])) < 1e-5
    assert np.array_equal(cs.reshape(CK - 1, CH)[-1], p["qkv"][0]) and not cs.reshape(CK - 1, CH)[:-1].any()


def test_gdn_delta_rule_overwrites_key_direction_and_pure_decay():
    p = gdn_inputs(3)
    S0 = synth.normal((NV, DK, DV), 5, 0.05)
    # g = 1 (softplus(-40) = 0 in f32), beta = 1 (sigmoid(40) = 1 in f32): afterwards S^T k = v exactly up to rounding
    p["alpha"] = np.full((1, NV), -40.0, np.float32); p["beta"] = np.full((1, NV), 40.0, np.float32)
    _, _, S = run_gdn(p, np.zeros((CK - 1, CH)), S0)
    w = p["conv_w"].reshape(CH, CK).astype(np.float64)
    co = np_ref.silu(w[:, CK - 1] * p["qkv"][0])
    k = co[NK * DK:2 * NK * DK].reshape(NK, DK); k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6); v = co[2 * NK * DK:].reshape(NV, DV)
    S = S.reshape(NV, DK, DV).astype(np.float64)
    for h in range(NV):
        assert relerr(S[h].T @ k[h % NK], v[h]) < 1e-5
        u = np.random.Generator(np.random.PCG64(h)).standard_normal(DK); u -= (u @ k[h % NK]) * k[h % NK]      # orthogonal to k
        assert relerr(S[h].T @ u, S0[h].astype(np.float64).T @ u) < 1e-5
    # beta = 0: S' = g * S
    p["beta"] = np.full((1, NV), -200.0, np.float32); p["alpha"] = synth.normal((1, NV), 9)
    _, _, S = run_gdn(p, np.zeros((CK - 1, CH)), S0)
    for h in range(NV):
        g = np.exp(np_ref.softplus(float(p["alpha"][0, h])) * float(p["a"][h]))
        assert relerr(S.reshape(NV, DK, DV)[h], g * S0[h].astype(np.float64)) < 1e-6


def test_gdn_one_hot_conv_is_a_delay():
    p = gdn_inputs(4, t=4)
    for tap in range(CK):
        w = np.zeros((CH, CK), np.float32); w[:, tap] = 1.0; p["conv_w"] = w.reshape(-1)
        hist = synth.normal((CK - 1, CH), 11)
        # run 4 tokens; conv output of token ti is silu(input delayed by (CK-1-tap)); read it back through the state rows
        _, cs, _ = run_gdn(p, hist, np.zeros((NV, DK, DV)))
        assert np.array_equal(cs.reshape(CK - 1, CH), p["qkv"][1:4])
    # the delayed value itself: tap 0 sees hist[0] at the first token -> q/k/v built from silu(hist[0])
    w = np.zeros((CH, CK), np.float32); w[:, 0] = 1.0
    p1 = gdn_inputs(4); p1["conv_w"] = w.reshape(-1)
    hist = synth.normal((CK - 1, CH), 11)
    out_a, _, _ = run_gdn(p1, hist, np.zeros((NV, DK, DV)))
    w2 = np.zeros((CH, CK), np.float32); w2[:, CK - 1] = 1.0
    p2 = dict(p1); p2["conv_w"] = w2.reshape(-1); p2["qkv"] = hist[0:1].copy()
    out_b, _, _ = run_gdn(p2, np.zeros((CK - 1, CH)), np.zeros((NV, DK, DV)))
    assert np.array_equal(out_a, out_b)


# ---- attention --------------------------------------------------------------------------------------------------
NH, NKV, HD, NROT = 4, 2, 256, 64


def attn_inputs(seed, t):
    g = lambda s, shape, std=1.0: synth.normal(shape, seed * 100 + s, std)
    return dict(q=g(1, (t, NH * 2 * HD)), k=g(2, (t, NKV * HD)), v=g(3, (t, NKV * HD)), qn=1 + g(4, (HD,), 0.1), kn=1 + g(5, (HD,), 0.1))


def run_attn(p, start, kc, vc, kv_bits=0, recent=1024):
    t = p["q"].shape[0]
    K = np.zeros((start + t, NKV * HD), np.float32); V = np.zeros_like(K); K[:start] = kc; V[:start] = vc
    inv = orc.rope_inv(NROT, 1e7)
    out = orc.attn_core(NH, NKV, HD, NROT, 1e-6, inv, p["qn"], p["kn"], p["q"], p["k"], p["v"], start, kv_bits, recent, K, V)
    return out, K, V


def test_attention_single_position_is_value_times_gate_and_rope_identity_at_zero():
    p = attn_inputs(1, 1)
    out, K, V = run_attn(p, 0, np.zeros((0, NKV * HD)), np.zeros((0, NKV * HD)))
    for h in range(NH):
        gate = p["q"][0].reshape(NH, 2 * HD)[h, HD:]
        exp = p["v"][0].reshape(NKV, HD)[h // (NH // NKV)] * np_ref.sigm(gate.astype(np.float64))
        assert relerr(out[0].reshape(NH, HD)[h], exp) < 1e-6
    kexp = np_ref.rms(p["k"][0].reshape(NKV, HD).astype(np.float64), p["kn"].astype(np.float64), 1e-6)   # pos 0: rope = identity
    assert relerr(K[0], kexp.reshape(-1)) < 1e-6 and np.array_equal(V[0], p["v"][0])


def test_attention_uniform_keys_average_the_values():
    p = attn_inputs(2, 1)
    n = 9
    vc = synth.normal((n, NKV * HD), 5); kc = np.zeros((n, NKV * HD), np.float32)
    p["k"] = np.zeros((1, NKV * HD), np.float32)          # all keys zero -> all scores equal -> softmax uniform
    out, _, _ = run_attn(p, n, kc, vc)
    allv = np.concatenate([vc, p["v"]]).astype(np.float64).reshape(n + 1, NKV, HD).mean(0)
    for h in range(NH):
        gate = p["q"][0].reshape(NH, 2 * HD)[h, HD:].astype(np.float64)
        assert relerr(out[0].reshape(NH, HD)[h], allv[h // (NH // NKV)] * np_ref.sigm(gate)) < 1e-5


@pytest.mark.parametrize("kv_bits,recent", [(0, 1024), (4, 64)])
def test_attention_matches_numpy_incl_packed_region(kv_bits, recent):
    start, t = 200, 3
    p = attn_inputs(3, t)
    kc = synth.normal((start, NKV * HD), 6); vc = synth.normal((start, NKV * HD), 7)
    out, K, V = run_attn(p, start, kc, vc, kv_bits, recent)
    inv = orc.rope_inv(NROT, 1e7)
    Kn, Vn = kc.copy(), vc.copy()
    for ti in range(t):
        pb = orc.packed_boundary(start + ti + 1, kv_bits, recent)
        if kv_bits:
            assert pb == ((start + ti + 1 - recent) // 64) * 64 and pb > 0
        o, kr, vr = np_ref.attn_step(NH, NKV, HD, NROT, 1e-6, inv, p["qn"], p["kn"], p["q"][ti], p["k"][ti], p["v"][ti], start + ti, Kn, Vn, pb)
        Kn = np.concatenate([Kn, kr[None]]); Vn = np.concatenate([Vn, vr[None]])
        assert relerr(out[ti], o) < 2e-5, ti
    assert relerr(K, Kn) < 1e-6 and np.array_equal(V, Vn)


def test_rope_rotates_pairs_i_and_i_plus_half_only_below_n_rot():
    inv = orc.rope_inv(NROT, 1e7)
    p = attn_inputs(4, 1); p["kn"] = np.ones(HD, np.float32)
    _, K, _ = run_attn(p, 5, np.zeros((5, NKV * HD)), np.zeros((5, NKV * HD)))
    k0 = np_ref.rms(p["k"][0].reshape(NKV, HD).astype(np.float64), np.ones(HD), 1e-6)
    got = K[5].reshape(NKV, HD).astype(np.float64)
    assert relerr(got[:, NROT:], k0[:, NROT:]) < 1e-6                                        # untouched dims
    ang = 5.0 * inv.astype(np.float64)
    assert relerr(got[:, :NROT // 2], k0[:, :NROT // 2] * np.cos(ang) - k0[:, NROT // 2:NROT] * np.sin(ang)) < 1e-5
    assert relerr(got[:, NROT // 2:NROT], k0[:, NROT // 2:NROT] * np.cos(ang) + k0[:, :NROT // 2] * np.sin(ang)) < 1e-5


# ---- QSA sparse indexer + YaRN ---------------------------------------------------------------------------------------
INH, IHD, IR, IBUD = 3, 128, 4, 64          # dense up to 64 + 4 - 1 = 67 visible positions


def qsa_inputs(seed, t):
    g = lambda s, shape, std=1.0: synth.normal(shape, seed * 100 + s, std)
    p = attn_inputs(seed, t)
    p.update(iq=g(11, (t, INH * IHD)), ik=g(12, (t, IHD)), iqn=1 + g(13, (IHD,), 0.1), ikn=1 + g(14, (IHD,), 0.1))
    return p


def run_qsa(p, start, kc, vc, ikc, ibc, kv_bits=0, recent=1024, inv=None, mscale=1.0, budget=IBUD):
    t = p["q"].shape[0]
    K = np.zeros((start + t, NKV * HD), np.float32); V = np.zeros_like(K); K[:start] = kc; V[:start] = vc
    IK = np.zeros((start + t, IHD), np.float32); IK[:start] = ikc
    IB = np.zeros(((start + t) // IR, IHD), np.float32); IB[:start // IR] = ibc
    inv = orc.rope_inv(NROT, 1e7) if inv is None else inv
    out, sel = orc.attn_core_qsa(NH, NKV, HD, NROT, 1e-6, inv, mscale, p["qn"], p["kn"], p["q"], p["k"], p["v"], start, kv_bits, recent, K, V,
                                 INH, IHD, IR, budget, p["iqn"], p["ikn"], p["iq"], p["ik"], IK, IB)
    return out, sel, K, V, IK, IB


def feed(seed, n, chunk=5, **kw):
    """n positions through the oracle in windows of `chunk`; returns the per-token inputs and the final caches."""
    kc = np.zeros((0, NKV * HD), np.float32); vc = kc.copy(); ikc = np.zeros((0, IHD), np.float32); ibc = ikc.copy()
    ps, outs, sels = [], [], []
    start = 0
    while start < n:
        t = min(chunk, n - start)
        p = qsa_inputs(seed * 1000 + start, t)
        out, sel, kc, vc, ikc, ibc = run_qsa(p, start, kc, vc, ikc, ibc, **kw)
        ps.append(p); outs += list(out); sels += sel; start += t
    return ps, outs, sels, kc, vc, ikc, ibc


def test_qsa_is_dense_up_to_budget_plus_ratio_minus_one_and_equals_the_dense_branch():
    n = IBUD + IR - 1
    ps, outs, sels, kc, vc, ikc, ibc = feed(1, n)
    assert all(s is None for s in sels)
    # the dense entry point on the same inputs gives the same bits
    kd = np.zeros((0, NKV * HD), np.float32); vd = kd.copy(); start = 0
    for p in ps:
        t = p["q"].shape[0]
        o, kd, vd = run_attn(p, start, kd, vd)
        assert np.array_equal(o, np.array(outs[start:start + t])); start += t
    assert np.array_equal(kd, kc)
    # one more position switches the selection on: budget/ratio blocks + tail
    p = qsa_inputs(77, 1)
    _, sel, *_ = run_qsa(p, n, kc, vc, ikc, ibc)
    assert sel[0] is not None and len(sel[0]) == IBUD + (n + 1) % IR and (np.diff(sel[0]) > 0).all() and sel[0][-1] == n


def test_qsa_block_keys_are_pooled_normalised_rotated_and_indexed_by_block():
    n = 23
    ps, _, _, _, _, ikc, ibc = feed(2, n, chunk=3)
    assert ikc.shape == (n, IHD) and ibc.shape == (n // IR, IHD)
    raw = np.concatenate([p["ik"] for p in ps]); assert np.array_equal(ikc, raw)       # raw keys stored as projected
    inv = orc.rope_inv(NROT, 1e7); ikn = ps[0]["ikn"]
    # all windows use differently seeded norm weights in feed(); re-run with one weight set to check the closed form
    kc = np.zeros((0, NKV * HD), np.float32); vc = kc.copy(); ikc = np.zeros((0, IHD), np.float32); ibc = ikc.copy(); start = 0
    rows = []
    for w in range(6):
        p = qsa_inputs(500 + w, 4); p["ikn"] = ikn; rows.append(p["ik"])
        _, _, kc, vc, ikc, ibc = run_qsa(p, start, kc, vc, ikc, ibc); start += 4
    for b in range(6):
        exp = np_ref.qsa_pool(rows[b], ikn, 1e-6, b * IR, NROT, inv)
        assert relerr(ibc[b], exp) < 1e-6, b
    # identical keys in a block: the mean is the key itself
    p = qsa_inputs(600, 4); p["ikn"] = ikn; p["ik"][:] = p["ik"][0]
    _, _, _, _, _, ibc2 = run_qsa(p, start, kc, vc, ikc, ibc)
    assert relerr(ibc2[6], np_ref.rope(np_ref.rms(p["ik"][0].astype(np.float64), ikn.astype(np.float64), 1e-6), 24, NROT, inv)) < 1e-6


@pytest.mark.parametrize("kv_bits,recent", [(0, 1024), (4, 64)])
def test_qsa_selection_and_sparse_attention_match_numpy(kv_bits, recent):
    n0, t = 150, 6
    ps, _, _, kc, vc, ikc, ibc = feed(3, n0, chunk=8, kv_bits=kv_bits, recent=recent)
    p = qsa_inputs(9, t); p["iqn"] = ps[0]["iqn"]
    out, sel, K, V, IK, IB = run_qsa(p, n0, kc, vc, ikc, ibc, kv_bits, recent)
    inv = orc.rope_inv(NROT, 1e7)
    Kn, Vn = kc.copy(), vc.copy()
    for ti in range(t):
        pos = n0 + ti; n = pos + 1
        iq = np.stack([np_ref.rope(np_ref.rms(p["iq"][ti].reshape(INH, IHD)[h].astype(np.float64), p["iqn"].astype(np.float64), 1e-6), pos, NROT, inv) for h in range(INH)])
        want = np_ref.qsa_select(iq, IB.astype(np.float64), n, IR, IBUD)
        assert want is not None and np.array_equal(sel[ti], want), ti
        assert len(want) == IBUD + n % IR
        pb = orc.packed_boundary(n, kv_bits, recent)
        o, kr, vr = np_ref.attn_step(NH, NKV, HD, NROT, 1e-6, inv, p["qn"], p["kn"], p["q"][ti], p["k"][ti], p["v"][ti], pos, Kn, Vn, pb, positions=want)
        Kn = np.concatenate([Kn, kr[None]]); Vn = np.concatenate([Vn, vr[None]])
        assert relerr(out[ti], o) < 2e-5, ti
    if kv_bits:
        assert orc.packed_boundary(n0 + t, kv_bits, recent) > 0


def test_qsa_picks_the_blocks_whose_keys_point_along_the_query():
    # block keys are pooled from raw keys; plant raw keys proportional to a direction u in chosen blocks and to -u elsewhere:
    # with norm weights 1 and positions where RoPE leaves the planted (non-rotated) dims alone, relu(q.k) is positive only there
    n0 = 200; nb = n0 // IR; chosen = sorted([3, 17, 18, 40, 41, 42, 5, 11, 29, 30, 31, 33, 36, 44, 47, 49])     # = budget / ratio = 16 blocks
    u = np.zeros(IHD, np.float32); u[NROT:] = synth.normal((IHD - NROT,), 5)                                      # outside the rotated dims
    kc = synth.normal((n0, NKV * HD), 6); vc = synth.normal((n0, NKV * HD), 7)
    ikc = np.tile(-u, (n0, 1)).astype(np.float32)
    for b in chosen:
        ikc[b * IR:(b + 1) * IR] = u * (1.0 + 0.1 * b)          # distinct positive scores
    ones = np.ones(IHD, np.float32)
    inv = orc.rope_inv(NROT, 1e7)
    ibc = np.stack([np_ref.qsa_pool(ikc[b * IR:(b + 1) * IR], ones, 1e-6, b * IR, NROT, inv) for b in range(nb)]).astype(np.float32)
    p = qsa_inputs(4, 1); p["iqn"] = ones; p["ikn"] = ones; p["iq"] = np.tile(u, (1, INH)).astype(np.float32)
    _, sel, *_ = run_qsa(p, n0, kc, vc, ikc, ibc)
    want = [q for b in chosen for q in range(b * IR, (b + 1) * IR)] + [n0]
    assert list(sel[0]) == want


def test_yarn_table_reference_properties_and_closed_form():
    inv, ms = orc.rope_inv_yarn(64, 1e7, 262144, 131072)                 # qn_ctx.rs:406-411
    plain = orc.rope_inv(64, 1e7)
    assert ms == 1.0 and inv[0] == 1.0 and np.array_equal(inv, plain)
    assert np.array_equal(orc.rope_inv_yarn(64, 1e7, 0, 524288)[0], plain)
    y, ym = orc.rope_inv_yarn(64, 1e7, 262144, 524288)                   # qn_ctx.rs:412-419
    assert abs(ym - (1.0 + 0.1 * np.log(2.0))) < 1e-5 and ym > 1.0
    assert y[0] < plain[0] and (abs(y[31] - plain[31]) / plain[31] < 0.05 or y[31] <= plain[31])
    for train, ctx in ((262144, 524288), (262144, 300000), (32768, 1048576), (4096, 6000)):
        got, gm = orc.rope_inv_yarn(64, 1e7, train, ctx)
        exp, em = np_ref.yarn_inv(64, 1e7, train, ctx)
        assert relerr(got, exp) < 1e-5 and abs(gm - em) < 1e-6, (train, ctx)
        s = ctx / train
        assert abs(got[0] * s - 1.0) < 1e-6 and abs(got[-1] / plain[-1] - 1.0) < 1e-6        # pure interpolation / pure extrapolation ends


def test_yarn_magnitude_factor_scales_rotated_dims_only():
    y, ym = orc.rope_inv_yarn(NROT, 1e7, 128, 256)
    p = qsa_inputs(8, 1); p["kn"] = np.ones(HD, np.float32)
    _, _, K, *_ = run_qsa(p, 7, np.zeros((7, NKV * HD)), np.zeros((7, NKV * HD)), np.zeros((7, IHD)), np.zeros((1, IHD)), inv=y, mscale=ym)
    k0 = np_ref.rms(p["k"][0].reshape(NKV, HD).astype(np.float64), np.ones(HD), 1e-6)
    got = K[7].reshape(NKV, HD).astype(np.float64)
    assert relerr(got[:, NROT:], k0[:, NROT:]) < 1e-6
    assert relerr(got, np_ref.rope(k0, 7, NROT, y, ym)) < 1e-5
    assert relerr((got[:, :NROT] ** 2).sum(-1), (k0[:, :NROT] ** 2).sum(-1) * ym * ym) < 1e-5


# ---- MoE / hyper-connections / token step --------------------------------------------------------------------------
def small_cfg(**kw):
    c = mg.Config(n_layers=4, d=256, hc=2, hc_lr=32, n_exp=8, top_k=2, ff_exp=256, vocab=512, kv_recent=64)
    for k, v in kw.items():
        setattr(c, k, v)
    return c


@pytest.mark.parametrize("qtype", [synth.IQ3_S, synth.Q4_K])
def test_moe_ffn_matches_numpy(qtype):
    c = small_cfg(qtype=qtype)
    hw = mg.build_host(c, seed=3); L = hw.layers[0]
    x = synth.normal((3, c.d), 17)
    y, idx, w = orc.moe_ffn(c.d, c.n_exp, c.top_k, c.ff_exp, *(orc_tensor(L[s]) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E)),
                            hw.f32(0, mg.SH_GATE_INP), *(orc_tensor(L[s]) for s in (mg.SH_GATE, mg.SH_UP, mg.SH_DOWN)), x)
    W = {"router": dense(L[mg.ROUTER]), "gate_e": dense(L[mg.GATE_E]).reshape(c.n_exp, c.ff_exp, c.d), "up_e": dense(L[mg.UP_E]).reshape(c.n_exp, c.ff_exp, c.d),
         "down_e": dense(L[mg.DOWN_E]).reshape(c.n_exp, c.d, c.ff_exp), "sh_gate_inp": hw.f32(0, mg.SH_GATE_INP).astype(np.float64),
         "sh_gate": dense(L[mg.SH_GATE]), "sh_up": dense(L[mg.SH_UP]), "sh_down": dense(L[mg.SH_DOWN])}
    for ti in range(3):
        yn, idn, wn = np_ref.moe_ffn(c.d, c.n_exp, c.top_k, c.ff_exp, W, x[ti])
        assert np.array_equal(idx[ti], idn) and np.abs(w[ti] - wn).max() < 1e-6
        assert relerr(y[ti], yn) < 1e-5


def test_hc_mix_and_combine_match_numpy():
    c = small_cfg()
    hw = mg.build_host(c, seed=4); L = hw.layers[1]
    x = synth.normal((2, c.hc * c.d), 21)
    mixed, inj = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(1, mg.HCA_NORM), orc_tensor(L[mg.HCA_DOWN]), orc_tensor(L[mg.HCA_INJECT]), orc_tensor(L[mg.HCA_UP]), x)
    for ti in range(2):
        mn, jn = np_ref.hc_mix(c.d, c.hc, c.eps, hw.f32(1, mg.HCA_NORM), dense(L[mg.HCA_DOWN]), dense(L[mg.HCA_INJECT]), dense(L[mg.HCA_UP]), x[ti])
        assert relerr(mixed[ti], mn) < 1e-5 and relerr(inj[ti], jn) < 1e-5
    out = synth.normal((2, c.d), 22)
    xc = orc.hc_combine(c.d, c.hc, x, out, inj).reshape(2, -1)
    for ti in range(2):
        assert relerr(xc[ti], np_ref.hc_combine(c.d, c.hc, x[ti], out[ti].astype(np.float64), inj[ti].astype(np.float64))) < 1e-6
    # head mixer: no inject
    G = hw.globals_
    mixed, inj = orc.hc_mix(c.d, c.hc, c.eps, hw.f32(-1, mg.G_HEAD_NORM), orc_tensor(G[mg.G_HEAD_DOWN]), None, orc_tensor(G[mg.G_HEAD_UP]), x[:1])
    mn, _ = np_ref.hc_mix(c.d, c.hc, c.eps, hw.f32(-1, mg.G_HEAD_NORM), dense(G[mg.G_HEAD_DOWN]), None, dense(G[mg.G_HEAD_UP]), x[0])
    assert relerr(mixed[0], mn) < 1e-5 and not inj.any()


def test_token_step_matches_numpy_and_prefill_equals_steps():
    c = small_cfg()
    hw = mg.build_host(c, seed=5)
    m = orc_model(hw)
    ids = np.array([3, 77, 500, 12, 9, 311], dtype=np.uint32)
    st = m.new_state()
    lg = np.array([m.forward(ids[i:i + 1], st) for i in range(ids.size)])
    ref = np_forward_tokens(hw, ids)
    for i in range(ids.size):
        assert relerr(lg[i], ref[i]) < 1e-4, i
    assert [orc.argmax(l) for l in lg] == [int(np.argmax(r)) for r in ref]
    st2 = m.new_state()
    lg2 = m.forward(ids, st2)                      # one prefill chunk: same arithmetic per token
    assert relerr(lg2, lg[-1]) < 1e-6
    assert relerr(st2.ssm(0), st.ssm(0)) < 1e-6 and np.array_equal(st2.kcache(0), st.kcache(0))


def test_token_step_with_indexer_and_yarn_matches_numpy_and_rollback_restores_the_indexer_state():
    # 4 layers (one attention layer with an indexer): dense up to 8 + 4 - 1 = 11 positions, sparse beyond; YaRN x2
    c = small_cfg(idx_nh=2, idx_hd=128, idx_ratio=4, idx_budget=8, ctx_train=32, ctx=64)
    hw = mg.build_host(c, seed=8)
    m = orc_model(hw)
    ids = ((np.arange(22, dtype=np.uint32) * 29 + 7) % c.vocab).astype(np.uint32)
    st = m.new_state()
    lg = np.array([m.forward(ids[i:i + 1], st) for i in range(ids.size)])
    ref = np_forward_tokens(hw, ids)
    for i in range(ids.size):
        assert relerr(lg[i], ref[i]) < 1e-4, i
    assert st.ikeys(0).size == 22 * 128 and st.iblocks(0).size == 5 * 128
    # windows (prefill chunks) give the same per-token arithmetic
    st2 = m.new_state(); m.forward(ids[:13], st2); lg2 = m.forward(ids[13:], st2)
    assert relerr(lg2, lg[-1]) < 1e-6 and np.array_equal(st2.iblocks(0), st.iblocks(0)) and np.array_equal(st2.ikeys(0), st.ikeys(0))
    # verify window + rollback: 5 tokens, keep 2 -> indexer state truncated to 15 + 2 = 17 positions, 4 blocks; continuing
    # from there equals never having drafted
    st3 = m.new_state(); m.forward(ids[:15], st3)
    bad = ids[15:20].copy(); bad[2:] = (bad[2:] + 1) % c.vocab
    m.forward_multi(bad, st3); m.spec_keep(st3, 5, 2)
    assert len(st3) == 17 and st3.ikeys(0).size == 17 * 128 and st3.iblocks(0).size == 4 * 128
    lg3 = np.array([m.forward(ids[i:i + 1], st3) for i in range(17, 22)])
    assert np.array_equal(lg3, lg[17:22])


def test_verify_rollback_and_drafted_generation_are_identical_to_plain_decode():
    c = small_cfg(n_layers=4)
    hw = mg.build_host(c, seed=6)
    m = orc_model(hw)
    prompt = np.array([5, 6, 7, 8], dtype=np.uint32)
    st = m.new_state(); first = m.forward(prompt, st)
    plain, _ = m.generate_greedy(st, first, 12)
    # drafts = the true continuation (all accepted) and a corrupted continuation (forces rollbacks)
    for corrupt in (False, True):
        ds = np.concatenate([plain, np.zeros(8, np.uint32)]).astype(np.uint32)
        if corrupt:
            ds[3::4] = (ds[3::4] + 1) % c.vocab
        st2 = m.new_state(); f2 = m.forward(prompt, st2)
        out, rounds = m.generate_greedy(st2, f2, 12, n_draft=4, draft_stream=ds)
        assert np.array_equal(out, plain) and rounds > 0
        # the rolled-back state continues exactly like the never-drafted one
        nxt = np.array([out[-1]], dtype=np.uint32)
    # explicit spec_keep: verify 5 tokens, keep 2, continue == feeding those 2 tokens one by one
    sa = m.new_state(); m.forward(prompt, sa); sb = m.new_state(); m.forward(prompt, sb)
    toks = np.array([9, 10, 11, 12, 13], dtype=np.uint32)
    lv = m.forward_multi(toks, sa); m.spec_keep(sa, 5, 2)
    l1 = m.forward(toks[0:1], sb); l2 = m.forward(toks[1:2], sb)
    assert np.array_equal(lv[0], l1) and np.array_equal(lv[1], l2) and len(sa) == len(sb) == 6
    assert np.array_equal(m.forward(np.array([40], np.uint32), sa), m.forward(np.array([40], np.uint32), sb))
