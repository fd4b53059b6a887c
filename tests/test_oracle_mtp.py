"""The oracle's MTP drafter (src/model/mtp.rs; Model::mtp_draft, qwen4exp_gguf.rs:2180-2277) pinned by what the
definition fixes:
  * a zero head: every logit equal -> the first draft-vocabulary id with probability exactly 1 / n, and the min_p gate
    that spares the first draft only;
  * a zero fc_hidden: a cell depends on nothing but the token one position ahead (the pairing R_i with token i + 1),
    and its key is that token's key turned by the rope of the cell's own index with the unscaled table;
  * a zero fc_embedding: a cell depends on nothing but the main model's residual of its own position;
  * the cell bookkeeping (catch-up start, window, the two truncations) as numbers worked out by hand from the rules;
  * the draft step as the composition of the block entry points that have pins of their own (matmul, hc_mix,
    hc_combine, attn_core, moe_ffn), cell by cell;
  * generation with the drafter proposing equals plain greedy decoding."""
import numpy as np

import helpers
import np_ref
import orc
from pyre_amd import modelgen as mg, synth

N_EXP, TOP_K, FF = 4, 2, 256
DRAFT_IDS = np.array([5, 9, 17, 33, 64, 65, 100, 101, 200, 300, 301, 302, 400, 410, 500, 511], dtype=np.uint32)


def setup(window=16, zero=(), cfg_kw=None, seed=3):
    c = mg.Config(**(cfg_kw or {}))
    hw = mg.build_host(c, seed)
    mt = mg.build_mtp_host(c, hw, N_EXP, FF, DRAFT_IDS, seed=seed + 10)
    for slot in zero:
        ty, rows, cols, b = mt[slot]
        mt[slot] = (synth.F32, rows, cols, np.zeros(rows * cols, dtype=np.float32).view(np.uint8))
    om = helpers.orc_model(hw, threads=2)
    dr = helpers.orc_mtp(om, mt, N_EXP, TOP_K, FF, window, DRAFT_IDS)
    return c, hw, mt, om, dr


def prompt(n, seed, vocab=512):
    return synth.ids(n, vocab, seed) if hasattr(synth, "ids") else np.random.default_rng(seed).integers(0, vocab, n).astype(np.uint32)


def test_zero_head_gives_the_first_id_with_probability_one_over_n_and_the_gate_spares_only_the_first_draft():
    c, hw, mt, om, dr = setup(zero=(mg.MTP_HEAD,))
    st = om.new_state(); dr.attach(st)
    om.forward(prompt(5, 1), st)
    ids, ps = dr.draft(st, 42, 4)
    assert list(ids) == [5, 5, 5, 5] and np.all(ps == np.float32(1.0 / 16))
    ids, ps = dr.draft(st, 42, 4, min_p=0.07)          # 1/16 = 0.0625 < 0.07: draft 0 is never gated, draft 1 is
    assert list(ids) == [5]
    ids, ps = dr.draft(st, 42, 4, min_p=0.0625)        # p >= min_p passes
    assert len(ids) == 4
    assert len(dr.draft(st, 42, 0)[0]) == 0


def test_without_a_kept_residual_there_is_no_draft():
    c, hw, mt, om, dr = setup()
    st = om.new_state()
    om.forward(prompt(5, 1), st)                          # not attached yet: nothing was kept
    dr.attach(st)
    assert len(dr.draft(st, 42, 3)[0]) == 0
    om.forward(prompt(1, 2), st)                          # now the last position's residual is there
    assert len(dr.draft(st, 42, 3)[0]) == 3
    c0, k, v = dr.kv(st)
    assert (c0, len(k)) == (5, 1)                         # cell 5 only: the earlier residuals are unknown


def test_zero_fc_hidden_a_cell_sees_only_the_next_token_and_its_key_turns_with_the_cell_index():
    # the main model runs with a stretched context (YaRN): the drafter must still use the plain table
    c, hw, mt, om, dr = setup(zero=(mg.MTP_FC_H,), cfg_kw=dict(ctx_train=64, ctx=256))
    a = np.array([7, 11, 300, 11, 45, 11, 90], dtype=np.uint32)
    b = np.array([8, 11, 301, 11, 46, 12, 91], dtype=np.uint32)           # positions 1 and 3 hold the same token as in a
    sa = om.new_state(); dr.attach(sa); om.forward(a, sa); dr.draft(sa, 11, 1)
    sb = om.new_state(); dr.attach(sb); om.forward(b, sb); dr.draft(sb, 77, 1)
    c0a, ka, va = dr.kv(sa); c0b, kb, vb = dr.kv(sb)
    assert c0a == 0 and c0b == 0 and len(ka) == 7 and len(kb) == 7        # cells 0..5 caught up, cell 6 from the draft step
    # cell i pairs with token i + 1: cells 0 and 2 agree between the prompts, the others do not
    for cell in range(7):
        same = cell in (0, 2)
        assert np.array_equal(va[cell], vb[cell]) == same, cell
        assert np.array_equal(ka[cell], kb[cell]) == same, cell
    # within prompt a the cells 0, 2, 4 and 6 (pending = 11) all pair with token 11: equal values, keys equal after
    # turning each back by its own index with inv_i = base^(-2i / n_rot)
    inv = c.rope_base ** (-2.0 * np.arange(c.n_rot // 2) / c.n_rot)
    for cell in (2, 4, 6):
        assert np.array_equal(va[cell], va[0])
    base = [np_ref.rope(ka[0].reshape(c.n_kv, c.hd)[h].astype(np.float64), 0, c.n_rot, inv) for h in range(c.n_kv)]
    for cell in (2, 4, 6):
        assert not np.array_equal(ka[cell], ka[0])
        for h in range(c.n_kv):
            back = np_ref.rope(ka[cell].reshape(c.n_kv, c.hd)[h].astype(np.float64), -cell, c.n_rot, inv)
            assert np.abs(back - base[h]).max() <= 2e-5 * np.abs(base[h]).max()


def test_zero_fc_embedding_a_cell_sees_only_the_residual_of_its_position():
    c, hw, mt, om, dr = setup(zero=(mg.MTP_FC_E,))
    a = np.array([7, 11, 300, 13, 45], dtype=np.uint32)
    b = np.array([7, 11, 300, 99, 46], dtype=np.uint32)                   # same prefix through position 2
    sa = om.new_state(); dr.attach(sa); om.forward(a, sa); dr.draft(sa, 1, 1)
    sb = om.new_state(); dr.attach(sb); om.forward(b, sb); dr.draft(sb, 2, 1)
    _, ka, va = dr.kv(sa); _, kb, vb = dr.kv(sb)
    for cell in range(5):
        assert np.array_equal(va[cell], vb[cell]) == (cell <= 2) and np.array_equal(ka[cell], kb[cell]) == (cell <= 2), cell


def test_cell_bookkeeping_by_hand():
    # window 8, a prompt of 40 tokens in one call: the residuals of positions 32..39 are kept (the last `window` tokens
    # of the call).  draft(k = 3) at n = 40: nothing cached, first = 32 -> lo = max(32, 39 - 8) = 32; catch-up cells
    # 32..38; steps at cells 39, 40, 41 -> 10 cells, the window keeps 34..41; truncate(40) -> cells 34..39.
    c, hw, mt, om, dr = setup(window=8)
    st = om.new_state(); dr.attach(st)
    om.forward(prompt(40, 4), st)
    assert dr.residual(st, 31) is None and dr.residual(st, 32) is not None and dr.residual(st, 39) is not None
    ids, _ = dr.draft(st, 3, 3)
    assert len(ids) == 3
    c0, k, v = dr.kv(st)
    assert (c0, len(k)) == (34, 6)
    # two tokens more (a verify window of pending + 1 accepted draft, say): n = 42; truncate(41) keeps 34..39; the
    # cache ends at 40 >= first -> lo = 40: one catch-up cell (40), then steps at 41, 42 -> cells 34..42 = 9, window ->
    # 35..42; truncate(42) -> 35..41
    om.forward_multi(np.array([3, int(ids[0])], dtype=np.uint32), st)
    k_before = k.copy()
    dr.draft(st, 9, 2)
    c0, k, v = dr.kv(st)
    assert (c0, len(k)) == (35, 7)
    assert np.array_equal(k[:5], k_before[1:6])           # cells 35..39 were not recomputed
    # a rollback: spec_keep drops position 41's residual on the next push only; a draft at n = 41 truncates to cells < 40
    om.forward_multi(np.array([9, 1, 2], dtype=np.uint32), st); om.spec_keep(st, 3, 1)       # n = 43
    dr.draft(st, 5, 1)
    c0, k, v = dr.kv(st)
    assert c0 + len(k) == 43 and len(k) == 8


def np_rms(x, w, eps):
    x = np.asarray(x, dtype=np.float32); s = np.float32(1.0) / np.sqrt(np.float32(np.sum(x.astype(np.float64) ** 2) / x.size) + np.float32(eps))
    return (x * s * w).astype(np.float32)


def test_draft_steps_are_the_composition_of_the_pinned_blocks():
    c, hw, mt, om, dr = setup(window=16)
    d, hc, w, row = c.d, c.hc, c.hc * c.d, c.n_kv * c.hd
    ids = prompt(6, 9); pending, k = 123, 3
    st = om.new_state(); dr.attach(st); om.forward(ids, st)
    R = [dr.residual(st, p) for p in range(6)]
    got_ids, got_p = dr.draft(st, pending, k)
    c0, gk, gv = dr.kv(st)
    assert c0 == 0 and len(gk) == 6                         # cells 0..5 after the final truncation

    T = lambda s: mt[s]
    vec = lambda s: mt[s][3].view(np.float32)
    mm = lambda s, x: orc.matmul(T(s)[0], T(s)[3], T(s)[1], T(s)[2], x, threads=2)
    ot = lambda s: helpers.orc_tensor(T(s))
    emb_rows = orc.dequant(hw.globals_[mg.G_EMBD][0], hw.globals_[mg.G_EMBD][3], c.vocab * d).reshape(c.vocab, d)
    inv = orc.rope_inv(c.n_rot, c.rope_base)
    kc = np.zeros((32, row), np.float32); vc = np.zeros((32, row), np.float32)

    def cell(r, tok, pos, full):
        en = np_rms(emb_rows[tok], vec(mg.MTP_PRE_E), c.eps); hn = np_rms(r, vec(mg.MTP_PRE_H), c.eps)
        rr = (mm(mg.MTP_FC_H, hn.reshape(hc, d)) + mm(mg.MTP_FC_E, en)[0][None, :]).reshape(-1)
        mixed, inj = orc.hc_mix(d, hc, c.eps, vec(mg.MTP_HCA_NORM), ot(mg.MTP_HCA_DOWN), ot(mg.MTP_HCA_INJECT), ot(mg.MTP_HCA_UP), rr, threads=2)
        q = mm(mg.MTP_Q, mixed); kk = mm(mg.MTP_K, mixed); vv = mm(mg.MTP_V, mixed)
        att = orc.attn_core(c.n_head, c.n_kv, c.hd, c.n_rot, c.eps, inv, vec(mg.MTP_QN), vec(mg.MTP_KN), q, kk, vv, pos, 0, 0, kc, vc)      # appends the cell, attends to cells 0..pos
        if not full:
            return None, None
        rr = orc.hc_combine(d, hc, rr, mm(mg.MTP_O, att.reshape(1, -1)), inj)
        m2, inj2 = orc.hc_mix(d, hc, c.eps, vec(mg.MTP_HCF_NORM), ot(mg.MTP_HCF_DOWN), ot(mg.MTP_HCF_INJECT), ot(mg.MTP_HCF_UP), rr, threads=2)
        y = orc.moe_ffn(d, N_EXP, TOP_K, FF, ot(mg.MTP_ROUTER), ot(mg.MTP_GATE_E), ot(mg.MTP_UP_E), ot(mg.MTP_DOWN_E), vec(mg.MTP_SH_GATE_INP),
                        ot(mg.MTP_SH_GATE), ot(mg.MTP_SH_UP), ot(mg.MTP_SH_DOWN), m2, threads=2)
        y = y[0] if isinstance(y, tuple) else y
        rr = orc.hc_combine(d, hc, rr, y, inj2)
        s, _ = orc.hc_mix(d, hc, c.eps, vec(mg.MTP_MIX_NORM), ot(mg.MTP_MIX_DOWN), None, ot(mg.MTP_MIX_UP), rr, threads=2)
        lg = mm(mg.MTP_HEAD, s)[0]
        bi = int(np.argmax(lg)); p = 1.0 / np.sum(np.exp((lg - lg[bi]).astype(np.float64)))
        return (int(DRAFT_IDS[bi]), p), np.asarray(rr, dtype=np.float32).reshape(-1)

    for i in range(5):                                       # catch-up: cell i = (R_i, token i + 1)
        cell(R[i], int(ids[i + 1]), i, False)
    r, tok, want = R[5], pending, []
    for j in range(k):
        (tok, p), r = cell(r, tok, 5 + j, True)
        want.append((tok, p))
    assert [t for t, _ in want] == list(got_ids)
    assert np.allclose([p for _, p in want], got_p, rtol=2e-5)
    assert helpers.relerr(gk, kc[:6]) <= 1e-6 and helpers.relerr(gv, vc[:6]) <= 1e-6


def test_generation_with_the_drafter_equals_plain_greedy():
    c, hw, mt, om, dr = setup(window=8)
    ids = prompt(12, 21)
    s0 = om.new_state(); fl = om.forward(ids, s0); plain, _ = om.generate_greedy(s0, fl, 24)
    s1 = om.new_state(); dr.attach(s1); fl1 = om.forward(ids, s1)
    out, drafted, accepted = dr.generate_greedy(s1, fl1, 24, k=3)
    assert np.array_equal(out, plain) and drafted > 0 and 0 <= accepted <= drafted
    assert len(s1) == len(s0)
