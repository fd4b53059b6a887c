"""The entry point that allocates nothing (pyre_qmatmul_static_dev): its output against pyre_qmatmul_dev's, bit for
bit, through the C ABI, on calls in a row that share the library's fixed scratch array (the second smaller than the
first), and the size limit's error."""
import numpy as np
import pytest

from pyre_amd import lib, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


def both(ctx, m, rows, cols, x):
    t = x.shape[0]
    xd = ctx.upload(x); ya = ctx.alloc(t * rows * 4); yb = ctx.alloc(t * rows * 4)
    m.matmul_dev(xd, t, ya)
    m.matmul_static_dev(xd, t, yb)
    a = ctx.download(ya, (t, rows)); b = ctx.download(yb, (t, rows))
    for p in (xd, ya, yb):
        ctx.free(p)
    return a, b


def test_static_scratch_entry_point_equals_the_allocating_one_on_consecutive_calls(ctx):
    big = lib.QMat(ctx, lib.IQ3_S, 4096, 4096, synth.matrix(lib.IQ3_S, 4096, 4096, 501))
    small = lib.QMat(ctx, lib.IQ3_S, 320, 512, synth.matrix(lib.IQ3_S, 320, 512, 502))
    xa = synth.normal((8, 4096), 503); xb = synth.normal((1, 512), 504)
    a, b = both(ctx, big, 4096, 4096, xa)                  # first call: 4096 columns of sixteen operand rows
    assert np.isfinite(a).all() and np.abs(a).max() > 0
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    a, b = both(ctx, small, 320, 512, xb)                  # second call, smaller: the array still holds the first call's operand beyond its own
    assert np.abs(a).max() > 0 and np.array_equal(a.view(np.uint32), b.view(np.uint32))
    a, b = both(ctx, big, 4096, 4096, xa[:3])              # and back to a larger one, another width
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # a second context on the same GPU resolves the same array and gives the same bits
    c2 = lib.Context(0)
    m2 = lib.QMat(c2, lib.IQ3_S, 320, 512, synth.matrix(lib.IQ3_S, 320, 512, 502))
    a2, b2 = both(c2, m2, 320, 512, xb)
    assert np.array_equal(b2.view(np.uint32), a2.view(np.uint32))
    m2.close(); c2.close()
    big.close(); small.close()


@pytest.mark.parametrize("ty", [lib.IQ2_XS, lib.Q4_K, lib.Q8_0])
def test_static_scratch_entry_point_iq2xs_q4k_single_token(ctx, ty):          # (Q8_0: its window alone uses scratch)
    big = lib.QMat(ctx, ty, 8256, 2048, synth.matrix(ty, 8256, 2048, 511))          # 129 row tiles: the native-format kernel, digits in the array
    small = lib.QMat(ctx, ty, 320, 512, synth.matrix(ty, 320, 512, 512))          # one launch, no scratch
    for m, rows, cols, t in ((big, 8256, 2048, 1), (small, 320, 512, 1), (big, 8256, 2048, 4), (big, 8256, 2048, 1)):
        a, b = both(ctx, m, rows, cols, synth.normal((t, cols), 513 + t))
        assert np.abs(a).max() > 0 and np.array_equal(a.view(np.uint32), b.view(np.uint32))
    big.close(); small.close()


def test_static_scratch_entry_point_rejects_what_does_not_fit_and_other_types(ctx):
    rows = 64
    wide = lib.QMat(ctx, lib.IQ3_S, rows, 65536, synth.matrix(lib.IQ3_S, rows, 65536, 505))      # twice the 32 768 columns the array holds
    edge = lib.QMat(ctx, lib.IQ3_S, rows, 32768, synth.matrix(lib.IQ3_S, rows, 32768, 508))      # exactly the limit
    xd = ctx.upload(synth.normal((8, 65536), 506)); yd = ctx.alloc(8 * rows * 4); ya = ctx.alloc(8 * rows * 4)
    for t in (1, 8):
        with pytest.raises(lib.PyreError, match="static scratch"):
            wide.matmul_static_dev(xd, t, yd)
    edge.matmul_static_dev(xd, 8, yd); edge.matmul_dev(xd, 8, ya)
    assert np.array_equal(ctx.download(yd, (8, rows)).view(np.uint32), ctx.download(ya, (8, rows)).view(np.uint32))
    with pytest.raises(lib.PyreError):
        edge.matmul_static_dev(xd, 9, yd)
    q8 = lib.QMat(ctx, lib.Q6_K, 64, 256, synth.matrix(lib.Q6_K, 64, 256, 507))
    with pytest.raises(lib.PyreError, match="IQ3_S"):
        q8.matmul_static_dev(xd, 1, yd)
    for p in (xd, yd, ya):
        ctx.free(p)
    wide.close(); edge.close(); q8.close()


def test_static_entry_point_under_stream_capture(ctx):
    """The claim 'no allocation, no event, no synchronisation' checked by the runtime itself: a stream capture fails on any
    of them.  The call is captured for one token of a large matrix (the native-format kernel, activation digits in the
    array) and for a window (operand rows in the array), the graphs are replayed with other calls on the array in between,
    and every replay gives the bits of pyre_qmatmul_dev."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]; hip.hipGraphDestroy.argtypes = [C.c_void_p]
    stream = C.c_void_p(ctx.stream)
    rows, cols = 8320, 2048          # 130 row tiles: a single token takes the native-format kernel
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, synth.matrix(lib.IQ3_S, rows, cols, 601))
    other = lib.QMat(ctx, lib.IQ3_S, 320, 4096, synth.matrix(lib.IQ3_S, 320, 4096, 602))
    x = synth.normal((8, cols), 603); xo = ctx.upload(synth.normal((8, 4096), 604)); yo = ctx.alloc(8 * 320 * 4)
    xd = ctx.upload(x)
    for t in (1, 5):
        yref = ctx.alloc(t * rows * 4); ycap = ctx.alloc(t * rows * 4)
        m.matmul_dev(xd, t, yref); ctx.sync()
        want = ctx.download(yref, (t, rows)).view(np.uint32)
        assert hip.hipStreamBeginCapture(stream, 0) == 0          # hipStreamCaptureModeGlobal: unsafe calls from any thread fail
        try:
            m.matmul_static_dev(xd, t, ycap)
        finally:
            graph = C.c_void_p(); rc = hip.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0 and graph.value
        ex = C.c_void_p()
        assert hip.hipGraphInstantiate(C.byref(ex), graph, None, None, 0) == 0
        for rep in range(3):
            other.matmul_static_dev(xo, 8 if rep else 1, yo)          # eager work on the same array between the replays
            z = ctx.upload(np.zeros((t, rows), np.float32)); ctx.sync()
            assert hip.hipGraphLaunch(ex, stream) == 0
            ctx.sync()
            got = ctx.download(ycap, (t, rows)).view(np.uint32)
            assert np.array_equal(got, want), (t, rep)
            ctx.free(z)
        assert hip.hipGraphExecDestroy(ex) == 0 and hip.hipGraphDestroy(graph) == 0
        ctx.free(yref); ctx.free(ycap)
    for p_ in (xd, xo, yo):
        ctx.free(p_)
    m.close(); other.close()
