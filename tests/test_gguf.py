"""GGUF container reader (host only): every metadata value type, alignment, N-D flattening, shards, and the refusals.
The expected values are what the writer put in, i.e. the container format itself is the oracle."""
import os
import struct

import numpy as np
import pytest

import gguf_writer as gw
from pyre_amd import lib, synth


def test_metadata_types_alignment_and_matrix_views(tmp_path):
    p = str(tmp_path / "m.gguf")
    meta = [("k.u8", gw.U8, 200), ("k.i8", gw.I8, -5), ("k.u16", gw.U16, 60000), ("k.i16", gw.I16, -1234), ("k.u32", gw.U32, 4000000000), ("k.i32", gw.I32, -7),
            ("k.f32", gw.F32, 1.5), ("k.bool", gw.BOOL, 1), ("k.str", gw.STR, "héllo"), ("k.u64", gw.U64, 2 ** 40 + 3), ("k.i64", gw.I64, -(2 ** 40)), ("k.f64", gw.F64, 1e-300),
            ("k.arr", gw.ARR, (gw.U32, [3, 1, 4, 1, 5])), ("k.arr_s", gw.ARR, (gw.STR, ["x", "yy"])), ("k.nested", gw.ARR, (gw.ARR, [(gw.I16, [1, -2]), (gw.I16, [])]))]
    a = synth.matrix(synth.IQ3_S, 6, 512, 1); b = np.arange(24, dtype=np.float32); c3 = synth.matrix(synth.Q8_0, 2 * 3, 64, 2)
    gw.write(p, meta, [("a.weight", [512, 6], synth.IQ3_S, a), ("b", [24], synth.F32, b), ("c3", [64, 2, 3], synth.Q8_0, c3)], alignment=64)
    g = lib.Gguf(p)
    assert g.n_shards == 1 and g.names() == ["a.weight", "b", "c3"] and g.has("b") and not g.has("nope")
    assert g.u64("k.u8") == 200 and g.u64("k.u16") == 60000 and g.u64("k.u32") == 4000000000 and g.u64("k.u64") == 2 ** 40 + 3 and g.u64("k.bool") == 1
    assert g.u64("k.i8") == (-5) % 2 ** 64 and g.u64("k.i64") == (-(2 ** 40)) % 2 ** 64           # Meta::as_u64 casts signed values
    assert g.f64("k.f32") == 1.5 and g.f64("k.f64") == 1e-300 and g.f64("k.i16") == -1234.0 and g.f64("k.u32") == 4000000000.0
    assert g.string("k.str") == "héllo" and g.arr_u64("k.arr") == [3, 1, 4, 1, 5] and g.arr_u64("k.arr_s") == [] and g.u64("general.alignment") == 64
    with pytest.raises(KeyError):
        g.u64("k.str")
    with pytest.raises(KeyError):
        g.f64("k.bool")
    ty, rows, cols, shape, data = g.tensor("a.weight")
    assert (ty, rows, cols, shape) == (synth.IQ3_S, 6, 512, (512, 6)) and np.array_equal(data, a.reshape(-1))
    ty, rows, cols, shape, data = g.tensor("b")
    assert (ty, rows, cols, shape) == (synth.F32, 1, 24, (24,)) and np.array_equal(data.view(np.float32), b)
    ty, rows, cols, shape, data = g.tensor("c3")                                                   # N-D: rows = prod(shape[1:])
    assert (ty, rows, cols, shape) == (synth.Q8_0, 6, 64, (64, 2, 3)) and np.array_equal(data, c3.reshape(-1))
    raw = open(p, "rb").read()
    assert raw.find(a.tobytes()) % 64 == 0                                                          # data section honours general.alignment
    g.close()


def test_shards_are_found_from_any_member_and_first_metadata_wins(tmp_path):
    a = np.arange(8, dtype=np.float32); b = np.arange(8, 16, dtype=np.float32)
    p1 = str(tmp_path / "w-00001-of-00002.gguf"); p2 = str(tmp_path / "w-00002-of-00002.gguf")
    gw.write(p1, [("x", gw.U32, 1), ("only1", gw.U32, 11)], [("a", [8], synth.F32, a)])
    gw.write(p2, [("x", gw.U32, 2), ("only2", gw.U32, 22)], [("b", [8], synth.F32, b)])
    for p in (p1, p2):
        g = lib.Gguf(p)
        assert g.n_shards == 2 and g.u64("x") == 1 and g.u64("only1") == 11 and g.u64("only2") == 22
        assert np.array_equal(g.tensor("a")[4].view(np.float32), a) and np.array_equal(g.tensor("b")[4].view(np.float32), b)
        g.close()
    os.remove(p2)
    with pytest.raises(lib.PyreError, match="missing shard"):
        lib.Gguf(p1)


def test_refusals(tmp_path):
    p = str(tmp_path / "bad.gguf")
    open(p, "wb").write(b"GGML" + b"\0" * 64)
    with pytest.raises(lib.PyreError, match="not GGUF"):
        lib.Gguf(p)
    good = str(tmp_path / "g.gguf")
    gw.write(good, [("k", gw.STR, "v" * 100)], [("q2k", [256], 10, np.zeros(84, np.uint8)), ("q6", [256], synth.Q6_K, np.zeros(210, np.uint8)), ("odd", [48], synth.Q8_0, np.zeros(51, np.uint8)),
                                                 ("t", [64, 8], synth.Q8_0, synth.matrix(synth.Q8_0, 8, 64, 1))])
    raw = open(good, "rb").read()
    for cut in (10, 30, 60, 150, len(raw) - 100):                                                   # truncated header, key, tensor info, data
        open(p, "wb").write(raw[:cut])
        try:
            g = lib.Gguf(p)
        except lib.PyreError:
            continue
        with pytest.raises(lib.PyreError, match="past the end"):                                    # header intact, data cut off
            g.tensor("t")
    open(p, "wb").write(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13))
    with pytest.raises(lib.PyreError, match="bad value type"):
        lib.Gguf(p)
    open(p, "wb").write(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 4, 2 ** 60))   # absurd array length
    with pytest.raises(lib.PyreError):
        lib.Gguf(p)
    g = lib.Gguf(good)
    with pytest.raises(lib.PyreError, match="Q2_K.*not supported"):
        g.tensor("q2k")
    assert g.tensor("q6")[0] == synth.Q6_K
    with pytest.raises(lib.PyreError, match="not a multiple of block"):
        g.tensor("odd")
    with pytest.raises(lib.PyreError, match="missing tensor"):
        g.tensor("nope")
    with pytest.raises(lib.PyreError):
        lib.Gguf(str(tmp_path / "absent.gguf"))
