"""GPU parity of the MTP drafter (pyre_mtp_*: src/model/mtp.rs, Model::mtp_draft) against the CPU oracle through the C
ABI: draft ids identical, draft probabilities within 2e-3 relative (a probability is the exponential of logit
differences, so an error of 1e-3 of the largest logit, the bar for logits, shows up as a relative error of that size),
the drafter's K / V cells within 1e-5 of the largest value, the cell bookkeeping identical, and generation with the drafter proposing identical to plain greedy
decoding on the device and in the oracle."""
import numpy as np
import pytest

import helpers
import orc
from helpers import orc_model, relerr
from pyre_amd import lib, synth
from pyre_amd import modelgen as mg

pytestmark = pytest.mark.gpu

N_EXP, TOP_K, FF = 4, 2, 256
DRAFT_IDS = np.array([5, 9, 17, 33, 64, 65, 100, 101, 200, 300, 301, 302, 400, 410, 500, 511], dtype=np.uint32)


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


def pair(ctx, c, seed, window, zero=(), draft_ids=DRAFT_IDS):
    hw = mg.build_host(c, seed=seed)
    mt = mg.build_mtp_host(c, hw, N_EXP, FF, draft_ids, seed=seed + 10)
    for slot in zero:
        ty, rows, cols, b = mt[slot]
        mt[slot] = (synth.F32, rows, cols, np.zeros(rows * cols, dtype=np.float32).view(np.uint8))
    gm = lib.Model(ctx, c, hw.layers, hw.globals_); om = orc_model(hw)
    gd = lib.Mtp(gm, N_EXP, TOP_K, FF, window, mt, draft_ids); od = helpers.orc_mtp(om, mt, N_EXP, TOP_K, FF, window, draft_ids)
    return gm, gd, om, od


def same_drafts(gd, gs, od, os_, pending, k, min_p=0.0):
    gi, gp = gd.draft(gs, pending, k, min_p); oi, op = od.draft(os_, pending, k, min_p)
    assert list(gi) == list(oi), (gi, oi)
    assert np.allclose(gp, op, rtol=2e-3, atol=0), (gp, op)
    gc0, gk, gv = gd.kv(gs); oc0, ok, ov = od.kv(os_)
    assert (gc0, len(gk)) == (oc0, len(ok))
    if len(ok):
        assert relerr(gk, ok) <= 1e-5 and relerr(gv, ov) <= 1e-5
    return gi


@pytest.mark.parametrize("qtype,hc_type,hc,env", [(synth.IQ3_S, synth.IQ3_S, 2, {}), (synth.IQ3_S, synth.BF16, 4, {}), (synth.Q8_0, synth.BF16, 2, {}),
                                                  (synth.IQ3_S, synth.IQ3_S, 2, {"PYRE_MODEL_ROWS": "1"}), (synth.Q4_K, synth.F32, 1, {})])
def test_drafts_and_cells_match_the_oracle_over_prompt_windows_rollback_and_the_device_loop(ctx, monkeypatch, qtype, hc_type, hc, env):
    monkeypatch.delenv("PYRE_MODEL_ROWS", raising=False)
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    c = small_cfg(qtype=qtype, hc_type=hc_type, hc=hc, hc_lr=256 if synth.GEOM.get(hc_type, (1,))[0] == 256 else 64)
    gm, gd, om, od = pair(ctx, c, 51, window=16)
    gs, os_ = gm.new_state(128), om.new_state(); gd.attach(gs); od.attach(os_)
    prompt = np.random.Generator(np.random.PCG64(52)).integers(0, c.vocab, 21, dtype=np.uint32)
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)              # windows of 8, 8, 5; the last 16 positions keep their residual
    assert relerr(lg, lo) <= 1e-3
    pending = int(orc.argmax(lo))
    drafts = same_drafts(gd, gs, od, os_, pending, 4)
    assert len(drafts) == 4
    # the verify window, one draft accepted, the rest rolled back
    toks = np.array([pending] + [int(x) for x in drafts], dtype=np.uint32)
    wg = gm.forward_multi(toks, gs); wo = om.forward_multi(toks, os_)
    assert relerr(wg, wo) <= 1e-3
    gm.spec_keep(gs, 5, 2); om.spec_keep(os_, 5, 2)
    pending = int(orc.argmax(wo[1]))
    same_drafts(gd, gs, od, os_, pending, 3)
    # the device loop stores each step's residual itself (captured step); the oracle walks the same tokens one by one
    got = gm.decode_greedy_dev(gs, pending, 6)
    tok = pending
    for i in range(6):
        tok = int(orc.argmax(om.forward(np.array([tok], dtype=np.uint32), os_)))
        assert tok == int(got[i])
    same_drafts(gd, gs, od, os_, tok, 7)
    # a second run of the loop replays the step captured with the drafter attached
    got = gm.decode_greedy_dev(gs, tok, 3)
    for i in range(3):
        tok = int(orc.argmax(om.forward(np.array([tok], dtype=np.uint32), os_)))
        assert tok == int(got[i])
    same_drafts(gd, gs, od, os_, tok, 2, min_p=0.5)
    for o in (gd, gs, gm):
        o.close()


def test_window_shorter_than_the_prompt_and_than_a_verify_window(ctx):
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.IQ3_S, hc_lr=256)
    gm, gd, om, od = pair(ctx, c, 61, window=8)
    gs, os_ = gm.new_state(128), om.new_state(); gd.attach(gs); od.attach(os_)
    prompt = np.random.Generator(np.random.PCG64(62)).integers(0, c.vocab, 40, dtype=np.uint32)
    gm.forward(prompt, gs, want_logits=False); om.forward(prompt, os_)
    d = same_drafts(gd, gs, od, os_, 3, 3)
    assert (gd.kv(gs)[0], len(gd.kv(gs)[1])) == (34, 6)        # by hand: residuals 32..39 kept, cells 32..41 computed, window -> 34..41, cells >= 40 dropped
    toks = np.array([3, int(d[0])], dtype=np.uint32)
    gm.forward_multi(toks, gs); om.forward_multi(toks, os_)
    same_drafts(gd, gs, od, os_, 9, 2)
    assert (gd.kv(gs)[0], len(gd.kv(gs)[1])) == (35, 7)
    for o in (gd, gs, gm):
        o.close()
    # a window of 3 cells under verify windows of 5 tokens: only the last 3 residuals of each call are kept
    gm, gd, om, od = pair(ctx, c, 63, window=3)
    gs, os_ = gm.new_state(128), om.new_state(); gd.attach(gs); od.attach(os_)
    p = prompt[:11]
    gm.forward(p, gs); om.forward(p, os_)
    same_drafts(gd, gs, od, os_, 1, 2)
    w5 = prompt[11:16]
    gm.forward_multi(w5, gs); om.forward_multi(w5, os_)
    same_drafts(gd, gs, od, os_, 2, 4)
    for o in (gd, gs, gm):
        o.close()


def test_drafter_after_a_long_prompt_on_several_streams(ctx):
    # 123 tokens = 16 windows, three in flight on three streams; the last 16 residual rows come from the last three windows
    # (the last one ragged), i.e. from all three streams; the drafts are the oracle's
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.IQ3_S, hc_lr=256)
    gm, gd, om, od = pair(ctx, c, 65, window=16)
    gs, os_ = gm.new_state(192), om.new_state(); gd.attach(gs); od.attach(os_)
    prompt = np.random.Generator(np.random.PCG64(66)).integers(0, c.vocab, 123, dtype=np.uint32)
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)
    assert gm.prompt_blocks() == 1          # (the twelve whole windows in front of the drafter's rows and the last window: one block, the FFN grouped by expert)
    assert relerr(lg, lo) <= 1e-3 and int(np.argmax(lg)) == int(np.argmax(lo))
    same_drafts(gd, gs, od, os_, int(np.argmax(lo)), 3)
    for o in (gd, gs, gm):
        o.close()


def test_zero_head_closed_form_and_the_probability_gate(ctx):
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.BF16)
    gm, gd, om, od = pair(ctx, c, 71, window=16, zero=(mg.MTP_HEAD,))
    gs = gm.new_state(64); gd.attach(gs)
    gm.forward(np.array([1, 2, 3, 4, 5], dtype=np.uint32), gs)
    ids, ps = gd.draft(gs, 42, 4)
    assert list(ids) == [5, 5, 5, 5] and np.all(ps == np.float32(1.0 / 16))      # equal logits: the first row's id, probability exactly 1/16
    assert list(gd.draft(gs, 42, 4, min_p=0.07)[0]) == [5]                        # the first draft is never gated
    assert len(gd.draft(gs, 42, 4, min_p=0.0625)[0]) == 4
    assert len(gd.draft(gs, 42, 0)[0]) == 0
    for o in (gd, gs, gm):
        o.close()


def test_generation_with_the_drafter_equals_plain_greedy_on_the_device_and_in_the_oracle(ctx):
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.IQ3_S, hc_lr=256)
    gm, gd, om, od = pair(ctx, c, 81, window=8)
    prompt = np.random.Generator(np.random.PCG64(82)).integers(0, c.vocab, 13, dtype=np.uint32)
    s0 = gm.new_state(128); fl = gm.forward(prompt, s0); plain, _ = gm.generate_greedy(s0, fl, 30)
    s1 = gm.new_state(128); gd.attach(s1); fl1 = gm.forward(prompt, s1)
    assert np.array_equal(fl.view(np.uint32), fl1.view(np.uint32))                # keeping the residuals changes no logit
    out, rounds, drafted, accepted = gd.generate_greedy(s1, fl1, 30, k=3)
    assert np.array_equal(out, plain) and len(s1) == len(s0)
    os_ = om.new_state(); od.attach(os_); flo = om.forward(prompt, os_)
    oo, od_n, oa_n = od.generate_greedy(os_, flo, 30, k=3)
    assert np.array_equal(oo, plain) and (drafted, accepted) == (od_n, oa_n) and drafted > 0 and rounds > 0
    # with a gate no draft passes beyond the first of a round
    s2 = gm.new_state(128); gd.attach(s2); fl2 = gm.forward(prompt, s2)
    out2, r2, d2, a2 = gd.generate_greedy(s2, fl2, 30, k=3, min_p=1.5)
    assert np.array_equal(out2, plain) and d2 == r2
    for o in (gd, s0, s1, s2, gm):
        o.close()


def test_a_drafter_that_predicts_the_model_is_accepted(ctx):
    # the model's own greedy continuation of a prompt, fed back as the prompt's continuation, makes the n-gram of
    # accepted drafts observable: here the drafter's head is the full output matrix and its block is the real one, so
    # acceptance is whatever it is; what must hold is the count identity drafted >= accepted and the output equality
    c = small_cfg(qtype=synth.Q8_0, hc_type=synth.BF16)
    ids = np.arange(c.vocab, dtype=np.uint32)
    gm, gd, om, od = pair(ctx, c, 91, window=16, draft_ids=ids)
    prompt = np.random.Generator(np.random.PCG64(92)).integers(0, c.vocab, 9, dtype=np.uint32)
    s0 = gm.new_state(96); fl = gm.forward(prompt, s0); plain, _ = gm.generate_greedy(s0, fl, 20)
    s1 = gm.new_state(96); gd.attach(s1); fl1 = gm.forward(prompt, s1)
    out, rounds, drafted, accepted = gd.generate_greedy(s1, fl1, 20, k=7)
    assert np.array_equal(out, plain) and 0 <= accepted <= drafted
    for o in (gd, s0, s1, gm):
        o.close()


def test_restore_starts_the_drafter_over_and_errors_are_reported(ctx):
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.BF16)
    gm, gd, om, od = pair(ctx, c, 95, window=16)
    gs = gm.new_state(64)
    with pytest.raises(lib.PyreError, match="not attached"):
        gd.draft(gs, 1, 2)
    gd.attach(gs)
    with pytest.raises(lib.PyreError, match="already"):
        gd.attach(gs)
    gm.forward(np.array([1, 2, 3, 4, 5, 6], dtype=np.uint32), gs)
    snap = gs.snapshot()
    assert len(gd.draft(gs, 7, 3)[0]) == 3
    with pytest.raises(lib.PyreError, match="above 7"):
        gd.draft(gs, 7, 8)
    with pytest.raises(lib.PyreError, match="vocabulary"):
        gd.draft(gs, 9999, 2)
    gm.forward(np.array([7, 8], dtype=np.uint32), gs)
    gs.restore(snap)
    assert len(gd.draft(gs, 7, 3)[0]) == 0                  # the residual of position 5 went with the restore
    gm.forward(np.array([7], dtype=np.uint32), gs)
    ids, _ = gd.draft(gs, 8, 3)
    assert len(ids) == 3 and gd.kv(gs)[0] == 6              # cells start at the first position whose residual is known again
    other = lib.Model(ctx, c, mg.build_host(c, seed=96).layers, mg.build_host(c, seed=96).globals_)
    so = other.new_state(32)
    with pytest.raises(lib.PyreError, match="another model"):
        gd.attach(so)
    for o in (so, other, snap, gd, gs, gm):
        o.close()


def test_drafter_beside_a_model_with_per_layer_ngram_embeddings(ctx):
    # both keep a token history by position on the device: the state's one serves the n-gram hashes and the drafter's catch-up
    c = mg.with_ple(small_cfg(qtype=synth.IQ3_S, hc_type=synth.IQ3_S, hc_lr=256), layers=(0, 2))
    gm, gd, om, od = pair(ctx, c, 97, window=8)
    gs, os_ = gm.new_state(128), om.new_state(); gd.attach(gs); od.attach(os_)
    prompt = np.random.Generator(np.random.PCG64(98)).integers(0, c.vocab, 19, dtype=np.uint32)
    lg = gm.forward(prompt, gs); lo = om.forward(prompt, os_)
    assert relerr(lg, lo) <= 1e-3
    pending = int(orc.argmax(lo))
    d = same_drafts(gd, gs, od, os_, pending, 3)
    toks = np.array([pending] + [int(x) for x in d], dtype=np.uint32)
    gm.forward_multi(toks, gs); om.forward_multi(toks, os_); gm.spec_keep(gs, 4, 1); om.spec_keep(os_, 4, 1)
    same_drafts(gd, gs, od, os_, 5, 2)
    s0 = gm.new_state(128); fl = gm.forward(prompt, s0); plain, _ = gm.generate_greedy(s0, fl, 16)
    s1 = gm.new_state(128); gd.attach(s1); fl1 = gm.forward(prompt, s1)
    out, rounds, drafted, accepted = gd.generate_greedy(s1, fl1, 16, k=3)
    assert np.array_equal(out, plain)
    for o in (gd, gs, s0, s1, gm):
        o.close()


def test_drafter_loaded_from_its_safetensors_checkpoint_equals_the_drafter_given_the_same_tensors(ctx, tmp_path):
    """Mtp::load (mtp.rs:99-118): names with their prefixes, norms as 1 + w, the fused gate_up_proj split per expert."""
    import copy
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.BF16)
    hw = mg.build_host(c, seed=101)
    cd = copy.copy(c); cd.qtype = synth.BF16; cd.router_type = synth.BF16
    mt = mg.build_mtp_host(cd, hw, N_EXP, FF, DRAFT_IDS, seed=111)

    def bf16_bits(x):      # round to nearest even, as numpy has no bf16
        u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)

    def f32_of(bits):
        return (bits.astype(np.uint32) << 16).view(np.float32)
    names = {mg.MTP_PRE_E: "mtp.pre_fc_norm_embedding.weight", mg.MTP_PRE_H: "mtp.pre_fc_norm_hidden.weight", mg.MTP_FC_E: "mtp.fc_embedding.weight", mg.MTP_FC_H: "mtp.fc_hidden.weight",
             mg.MTP_Q: "mtp.layers.0.self_attn.q_proj.weight", mg.MTP_K: "mtp.layers.0.self_attn.k_proj.weight", mg.MTP_V: "mtp.layers.0.self_attn.v_proj.weight",
             mg.MTP_O: "mtp.layers.0.self_attn.o_proj.weight", mg.MTP_QN: "mtp.layers.0.self_attn.q_norm.weight", mg.MTP_KN: "mtp.layers.0.self_attn.k_norm.weight",
             mg.MTP_ROUTER: "mtp.layers.0.mlp.gate.weight", mg.MTP_SH_GATE_INP: "mtp.layers.0.mlp.shared_expert_gate.weight", mg.MTP_SH_GATE: "mtp.layers.0.mlp.shared_expert.gate_proj.weight",
             mg.MTP_SH_UP: "mtp.layers.0.mlp.shared_expert.up_proj.weight", mg.MTP_SH_DOWN: "mtp.layers.0.mlp.shared_expert.down_proj.weight"}
    for base, pre, inj in ((mg.MTP_HCA_NORM, "attn_hyper_connection", True), (mg.MTP_HCF_NORM, "mlp_hyper_connection", True), (mg.MTP_MIX_NORM, "hyper_connection_mixer", False)):
        names[base] = "mtp.layers.0.%s.hc_norm.weight" % pre; names[base + 1] = "mtp.layers.0.%s.input_mix_weight_down.weight" % pre
        if inj:
            names[base + 2] = "mtp.layers.0.%s.block_inject_weight.weight" % pre
        names[base + (3 if inj else 2)] = "mtp.layers.0.%s.input_mix_weight_up.weight" % pre
    norms = (mg.MTP_PRE_E, mg.MTP_PRE_H, mg.MTP_HCA_NORM, mg.MTP_HCF_NORM, mg.MTP_MIX_NORM, mg.MTP_QN, mg.MTP_KN)
    file = {}
    for slot, name in names.items():
        ty, rows, cols, b = mt[slot]
        if ty == synth.F32:      # a vector: the file holds bf16(w - 1) for a norm, bf16(w) otherwise; the drafter built from tensors gets what the loader must form
            w = np.ascontiguousarray(b).view(np.float32)
            bits = bf16_bits(w - np.float32(1.0) if slot in norms else w)
            file[name] = bits
            mt[slot] = (synth.F32, rows, cols, (f32_of(bits) + np.float32(1.0 if slot in norms else 0.0)).astype(np.float32).view(np.uint8))
        else:
            assert ty == synth.BF16
            file[name] = np.ascontiguousarray(b).view(np.uint16).reshape(rows, cols)
    g3 = lambda s, r, q: np.ascontiguousarray(mt[s][3]).view(np.uint16).reshape(N_EXP, r, q)
    file["mtp.layers.0.mlp.experts.gate_up_proj"] = np.concatenate([g3(mg.MTP_GATE_E, FF, c.d), g3(mg.MTP_UP_E, FF, c.d)], axis=1)
    file["mtp.layers.0.mlp.experts.down_proj"] = g3(mg.MTP_DOWN_E, c.d, FF)
    path = str(tmp_path / "mtp.safetensors")
    helpers.write_safetensors(path, file, meta={"format": "pt"})
    gm = lib.Model(ctx, c, hw.layers, hw.globals_)
    ga = lib.Mtp(gm, N_EXP, TOP_K, FF, 16, mt, DRAFT_IDS)
    gb = lib.Mtp.from_safetensors(gm, path, DRAFT_IDS, top_k=TOP_K, window=16, head=mt[mg.MTP_HEAD])
    gc = lib.Mtp.from_safetensors(gm, path, DRAFT_IDS, top_k=TOP_K, window=16)            # head: rows of the main output matrix as f32
    prompt = np.random.Generator(np.random.PCG64(102)).integers(0, c.vocab, 21, dtype=np.uint32)
    res = []
    for gd in (ga, gb, gc):
        gs = gm.new_state(96); gd.attach(gs); lg = gm.forward(prompt, gs)
        ids, ps = gd.draft(gs, int(np.argmax(lg)), 4); c0, k, v = gd.kv(gs)
        res.append((ids, ps, c0, k, v)); gs.close()
    assert len(res[0][0]) == 4
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1].view(np.uint32), res[1][1].view(np.uint32))
    assert res[0][2] == res[1][2] and np.array_equal(res[0][3].view(np.uint32), res[1][3].view(np.uint32)) and np.array_equal(res[0][4].view(np.uint32), res[1][4].view(np.uint32))
    assert np.array_equal(res[0][0], res[2][0]) and np.allclose(res[0][1], res[2][1], rtol=1e-4, atol=0)
    # the experts per token are capped by the main model's (PYRE_MTP_TOPK, mtp.rs:108); a missing tensor is named
    gd = lib.Mtp.from_safetensors(gm, path, DRAFT_IDS, top_k=99, window=16); gd.close()
    del file["mtp.layers.0.self_attn.k_norm.weight"]
    helpers.write_safetensors(path, file)
    with pytest.raises(lib.PyreError, match="mtp tensor self_attn.k_norm.weight"):
        lib.Mtp.from_safetensors(gm, path, DRAFT_IDS)
    for o in (ga, gb, gc, gm):
        o.close()


def test_adaptive_draft_length_changes_which_drafts_are_verified_not_the_tokens(ctx):
    """spec::generate's adaptive plan (spec.rs:162-217): with it on, the drafted loops still produce the plain greedy stream;
    a drafter whose drafts are never accepted is verified less often once a plain step has been timed."""
    c = small_cfg(qtype=synth.IQ3_S, hc_type=synth.IQ3_S, hc_lr=256)
    gm, gd, om, od = pair(ctx, c, 121, window=8)
    prompt = np.random.Generator(np.random.PCG64(122)).integers(0, c.vocab, 13, dtype=np.uint32)
    s0 = gm.new_state(160); fl = gm.forward(prompt, s0); plain, _ = gm.generate_greedy(s0, fl, 60)
    ctx.set_spec_adapt(1)
    try:
        s1 = gm.new_state(160); gd.attach(s1); fl1 = gm.forward(prompt, s1)
        out, rounds, drafted, accepted = gd.generate_greedy(s1, fl1, 60, k=3)
        assert np.array_equal(out, plain) and 0 <= accepted <= drafted
        # the prompt-lookup drafter misses often, so plain steps get timed and the plan engages
        s2 = gm.new_state(160); fl2 = gm.forward(prompt, s2)
        out2, r2, d2, a2 = gm.generate_greedy_ngram(s2, prompt, fl2, 60, k=4, ng_min=1, ng_max=4)
        assert np.array_equal(out2, plain) and 0 <= a2 <= d2
        ctx.set_spec_adapt(0)
        s3 = gm.new_state(160); fl3 = gm.forward(prompt, s3)
        out3, r3, d3, a3 = gm.generate_greedy_ngram(s3, prompt, fl3, 60, k=4, ng_min=1, ng_max=4)
        assert np.array_equal(out3, plain) and 0 <= a3 <= d3
    finally:
        ctx.set_spec_adapt(-1)
    for o in (gd, s0, s1, s2, s3, gm):
        o.close()
