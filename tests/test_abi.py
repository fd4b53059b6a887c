"""No-GPU checks of the C-ABI library: it loads, and it exports every symbol include/pyre_hip.h declares."""
import ctypes as C
import os

import pytest

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


def test_create_without_gpu_fails_loudly_not_silently():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(lib.PyreError):
        lib.Context(0)
