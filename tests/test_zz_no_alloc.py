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
    q8 = lib.QMat(ctx, lib.Q8_0, 64, 256, synth.matrix(lib.Q8_0, 64, 256, 507))
    with pytest.raises(lib.PyreError, match="IQ3_S"):
        q8.matmul_static_dev(xd, 1, yd)
    for p in (xd, yd, ya):
        ctx.free(p)
    wide.close(); edge.close(); q8.close()
