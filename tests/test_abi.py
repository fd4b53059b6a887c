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


def test_create_without_gpu_fails_loudly_not_silently():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(lib.PyreError):
        lib.Context(0)
