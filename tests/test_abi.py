"""No-GPU checks of the C-ABI library: it loads, and it exports every symbol include/pyre_hip.h declares."""
import ctypes as C
import os

import pytest

import helpers
from pyre_amd import lib


def test_library_is_built_and_exports_every_declared_symbol():
    assert os.path.exists(lib.LIB_PATH), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    L = C.CDLL(lib.LIB_PATH)
    names = lib.exported_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing


def test_python_binding_declares_every_header_symbol():
    L = C.CDLL(lib.LIB_PATH)
    declared = set(lib._declare(L))
    assert declared == set(lib.exported_symbols())


def test_ngram_drafter_reference_vectors_and_brute_force():
    # the reference's own test (src/spec.rs:346-349)
    h = [1, 2, 3, 9, 1, 2, 3, 4, 5, 7, 1, 2, 3]
    assert lib.ngram_draft(h, 2, 2, 4).tolist() == [4, 5]
    assert lib.ngram_draft([1, 2, 3], 2, 2, 4).tolist() == []
    # longest suffix wins over a more recent shorter one; the most recent occurrence of that length wins; k caps the copy
    h = [7, 8, 9, 1, 5, 8, 9, 2, 6, 7, 8, 9]
    assert lib.ngram_draft(h, 3, 2, 4).tolist() == [1, 5, 8]            # suffix (7, 8, 9) occurred at 0 -> what followed
    assert lib.ngram_draft(h, 3, 2, 2).tolist() == [2, 6, 7]            # only n = 2: (8, 9) most recently at 5..6
    assert lib.ngram_draft(h, 1, 2, 2).tolist() == [2]
    assert lib.ngram_draft(h, 0, 2, 4).tolist() == [] and lib.ngram_draft(h, 3, 5, 8).tolist() == []
    # against a plain restatement of the definition on random small-alphabet histories
    import numpy as np
    g = np.random.Generator(np.random.PCG64(3))

    def brute(h, k, lo, hi):
        n_h = len(h)
        if k == 0 or n_h < lo + 1:
            return []
        for n in range(min(hi, n_h - 1), lo - 1, -1):
            suf = h[n_h - n:]
            for i in range(n_h - n - 1, -1, -1):
                if h[i:i + n] == suf and i + n < n_h:
                    return h[i + n:min(i + n + k, n_h)]
        return []
    for _ in range(300):
        h = g.integers(0, 4, int(g.integers(1, 40))).tolist(); k = int(g.integers(0, 6)); lo = int(g.integers(1, 4)); hi = lo + int(g.integers(0, 5))
        assert lib.ngram_draft(h, k, lo, hi).tolist() == brute(h, k, lo, hi), (h, k, lo, hi)


def test_adapt_plan_reference_vectors_and_brute_force():
    # the reference's own test (src/spec.rs:362-370)
    tv = [0.0] * 10
    assert lib.adapt_plan(2, 0.1, tv, 0.7, 0.0) == 0            # a 2-token verify at 1.75 plain steps with 70 % acceptance does not pay
    tv2 = list(tv); tv2[2] = 0.12; tv2[3] = 0.14
    assert lib.adapt_plan(2, 0.1, tv2, 0.75, 0.0) >= 1
    assert lib.adapt_plan(2, 0.1, tv2, 0.75, 0.1) == 0          # a draft cost as large as a plain step kills it again
    # values worked out from the definition: gain(k) = (1 + p + .. + p^k) ts / (tv[k + 1] + td), best k with gain > 1, first on ties
    assert lib.adapt_plan(2, 0.1, tv2, 0.75, 0.0) == 2          # 1.75 / 1.2 = 1.458 < (1.75 + 0.5625) / 1.4 = 1.652
    assert lib.adapt_plan(1, 0.1, tv2, 0.75, 0.0) == 1
    assert lib.adapt_plan(3, 1.0, tv, 1.0, 0.0) == 3            # unmeasured windows: (k + 1) / (1 + 0.75 k) = 1.143, 1.2, 1.231
    assert lib.adapt_plan(9, 1.0, tv, 1.0, 0.0) == 8            # never more than eight drafts
    assert lib.adapt_plan(3, 1.0, tv, 0.0, 0.0) == 0 and lib.adapt_plan(0, 1.0, tv, 1.0, 0.0) == 0
    import numpy as np
    g = np.random.Generator(np.random.PCG64(11))

    def brute(n, ts, tv, p, td):
        best, bk = 1.0, 0
        for k in range(1, min(n, 8) + 1):
            e = sum(p ** i for i in range(k + 1))
            est = tv[k + 1] if tv[k + 1] > 0 else ts * (1 + 0.75 * k)
            gain = e * ts / (est + td)
            if gain > best * (1 + 1e-12):
                best, bk = gain, k
        return bk
    for _ in range(500):
        n = int(g.integers(0, 10)); ts = float(g.uniform(0.001, 0.1)); p = float(g.uniform(0, 1)); td = float(g.uniform(0, 0.02))
        tv = [0.0] * 10
        for t in range(2, 10):
            if g.random() < 0.6:
                tv[t] = ts * float(g.uniform(0.8, 3.0))
        got = lib.adapt_plan(n, ts, tv, p, td)
        assert 0 <= got <= min(n, 8)
        # the brute force sums the series afresh (the library accumulates it): accept either side of a numerical tie
        want = brute(n, ts, tv, p, td)
        if got != want:
            def gain(k):
                e = sum(p ** i for i in range(k + 1)); est = tv[k + 1] if tv[k + 1] > 0 else ts * (1 + 0.75 * k); return e * ts / (est + td) if k else 1.0
            assert abs(gain(got) - gain(want)) <= 1e-9 * gain(want), (n, ts, tv, p, td, got, want)


def test_safetensors_reader_names_shapes_bytes_and_errors(tmp_path):
    import numpy as np
    g = np.random.Generator(np.random.PCG64(5))
    ts = {"mtp.layers.0.self_attn.q_proj.weight": g.integers(0, 65536, (6, 4), dtype=np.uint16),
          "mtp.fc_embedding.weight": g.integers(0, 65536, (4, 4), dtype=np.uint16),
          "mtp.layers.0.mlp.experts.down_proj": g.integers(0, 65536, (3, 4, 2), dtype=np.uint16),
          "plain \"quoted\" \u00e9 name": g.integers(0, 65536, (5,), dtype=np.uint16)}
    p = str(tmp_path / "mtp.safetensors")
    helpers.write_safetensors(p, ts, meta={"format": "pt", "nested": {"a": [1, 2, {"b": None}], "c": True}})
    st = lib.Safetensors(p)
    assert st.names() == ["self_attn.q_proj.weight", "fc_embedding.weight", "mlp.experts.down_proj", 'plain "quoted" \u00e9 name']      # prefixes trimmed (mtp.rs:37)
    for k, a in ts.items():
        nm = k.replace("mtp.", "", 1).replace("layers.0.", "", 1)
        shape, bits = st.tensor(nm)
        assert shape == list(a.shape) and np.array_equal(bits, a.reshape(-1))
    with pytest.raises(lib.PyreError, match="mtp tensor nope"):
        st.tensor("nope")
    st.close()
    # anything but BF16 is refused (mtp.rs:34); offsets that do not match the shape, a header longer than the file
    helpers.write_safetensors(p, {"a": np.zeros((2, 2), dtype=np.uint16)}, dtype="F16")
    with pytest.raises(lib.PyreError, match="dtype F16"):
        lib.Safetensors(p)
    import json
    h = json.dumps({"a": {"dtype": "BF16", "shape": [2, 3], "data_offsets": [0, 8]}}).encode()
    open(p, "wb").write(len(h).to_bytes(8, "little") + h + b"\0" * 12)
    with pytest.raises(lib.PyreError, match="data_offsets"):
        lib.Safetensors(p)
    open(p, "wb").write((1 << 40).to_bytes(8, "little") + b"{}")
    with pytest.raises(lib.PyreError, match="header length"):
        lib.Safetensors(p)
    with pytest.raises(lib.PyreError, match="open"):
        lib.Safetensors(str(tmp_path / "missing.safetensors"))


def test_safetensors_reader_against_files_the_safetensors_library_writes(tmp_path):
    """The container as the reference's checkpoint comes (scripts/mtp_fetch.py writes it with the safetensors library): BF16
    tensors saved by safetensors.torch.save_file, with metadata, read back name by name, shape by shape, bit by bit."""
    import numpy as np
    torch = pytest.importorskip("torch")
    st_torch = pytest.importorskip("safetensors.torch")
    g = torch.Generator().manual_seed(7)
    ts = {"mtp.fc_embedding.weight": torch.randn(6, 8, generator=g).to(torch.bfloat16),
          "mtp.layers.0.mlp.experts.gate_up_proj": torch.randn(3, 4, 8, generator=g).to(torch.bfloat16),
          "mtp.layers.0.self_attn.q_norm.weight": torch.randn(5, generator=g).to(torch.bfloat16),
          "mtp.pre_fc_norm_hidden.weight": torch.zeros(0, dtype=torch.bfloat16)}
    p = str(tmp_path / "lib.safetensors")
    st_torch.save_file(ts, p, metadata={"format": "pt", "note": "written by the safetensors library"})
    st = lib.Safetensors(p)
    assert sorted(st.names()) == sorted(["fc_embedding.weight", "mlp.experts.gate_up_proj", "self_attn.q_norm.weight", "pre_fc_norm_hidden.weight"])
    for k, t in ts.items():
        nm = k.replace("mtp.", "", 1).replace("layers.0.", "", 1)
        shape, bits = st.tensor(nm)
        want = t.contiguous().view(torch.int16).numpy().view(np.uint16).reshape(-1)
        assert shape == list(t.shape) and np.array_equal(bits[:want.size], want)
    st.close()
    st_torch.save_file({"a": torch.zeros(2, 2, dtype=torch.float16)}, p)
    with pytest.raises(lib.PyreError, match="dtype F16"):
        lib.Safetensors(p)


def test_create_without_gpu_fails_loudly_not_silently():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(lib.PyreError):
        lib.Context(0)
