"""The persistent-kernel decode (one launch for a run of tokens, grid barriers between stages) against the
launch-per-stage path: token stream, recurrent state, KV cache and the follow-up logits must be bit-identical."""
import os

import numpy as np
import pytest

from pyre_amd import lib, synth
from pyre_amd import modelgen as mg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


def run(gm, prompt, first, n, mega):
    os.environ["PYRE_MEGA"] = "2" if mega else "0"
    os.environ["PYRE_ROUTER_RIDES"] = "0"          # the persistent kernel mirrors the stage path with a separate router GEMV
    try:
        st = gm.new_state(len(prompt) + n + 8)
        gm.forward(prompt, st, want_logits=False)
        toks = gm.decode_greedy_dev(st, first, n)
        conv, ssm = st.gdn(0)
        k, v = st.kv(0)
        nxt = gm.forward(np.array([toks[-1]], dtype=np.uint32), st)
        return toks, conv, ssm, k, v, nxt, len(st)
    finally:
        os.environ.pop("PYRE_MEGA", None); os.environ.pop("PYRE_ROUTER_RIDES", None)


@pytest.mark.parametrize("n_prompt,n", [(10, 24), (100, 96)])
def test_persistent_decode_is_bit_identical_to_the_stage_launches(ctx, n_prompt, n):
    c = mg.Config(n_layers=4, d=256, hc=2, hc_lr=256, n_exp=8, top_k=2, ff_exp=256, vocab=512, kv_recent=64, qtype=synth.IQ3_S, hc_type=synth.IQ3_S)
    hw = mg.build_host(c, seed=21)
    gm = lib.Model(ctx, c, hw.layers, hw.globals_)
    prompt = (np.arange(n_prompt, dtype=np.uint32) * 37 + 11) % c.vocab
    a = run(gm, prompt, 7, n, mega=False)
    b = run(gm, prompt, 7, n, mega=True)
    assert np.array_equal(a[0], b[0]), "first split at %d" % int(np.argmax(a[0] != b[0]))
    for i in (1, 2, 3, 4, 5):
        assert np.array_equal(a[i].view(np.uint32), b[i].view(np.uint32)), i
    assert a[6] == b[6] == n_prompt + n + 1
