"""GPU parity of the quantized-matrix operator through the C ABI: dequant bit-exact with the oracle, GEMV within
1e-5 of the f64-accumulated truth (max|dy| / max|y|, the reference's own normalisation, kquant.rs:203-206)."""
import numpy as np
import pytest

import np_ref
import orc
from helpers import relerr
from pyre_amd import lib, synth

pytestmark = pytest.mark.gpu
FMTS = [lib.Q8_0, lib.Q4_K, lib.IQ2_XS, lib.IQ3_S, lib.Q4_0, lib.Q5_0, lib.Q6_K, lib.IQ2_XXS, lib.IQ3_XXS, lib.IQ4_NL, lib.IQ2_S, lib.IQ4_XS, lib.Q3_K, lib.Q2_0, lib.Q5_K, lib.IQ1_M]
ALL = FMTS + [lib.BF16, lib.F16, lib.F32]
TOL = 1e-5


@pytest.fixture(scope="module")
def ctx():
    c = lib.Context(0)
    yield c
    c.close()


def raw_matrix(ty, rows, cols, seed):
    if ty == lib.BF16:
        return synth.bf16_normal(rows, cols, seed, 0.02)
    if ty == lib.F16:
        return synth.normal((rows, cols), seed, 0.05).astype(np.float16).view(np.uint8).reshape(-1)
    if ty == lib.F32:
        return synth.normal((rows, cols), seed, 0.05).view(np.uint8).reshape(-1)
    return synth.matrix(ty, rows, cols, seed)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("ty", ALL)
@pytest.mark.parametrize("rows,cols", [(64, 256), (100, 512), (513, 2048)])
def test_dequant_bit_exact(ctx, ty, rows, cols):
    raw = raw_matrix(ty, rows, cols, 11 + ty)
    m = lib.QMat(ctx, ty, rows, cols, raw)
    got = m.to_f32()
    exp = orc.dequant(ty, raw, rows * cols).reshape(rows, cols)
    assert np.array_equal(bits(got), bits(exp))
    for r in (0, rows // 2, rows - 1):
        assert np.array_equal(bits(m.row(r)), bits(exp[r]))
    assert m.gguf_bytes == raw.nbytes


@pytest.mark.parametrize("ty", FMTS)
def test_dequant_bit_exact_on_arbitrary_bytes_and_known_answers(ctx, ty):
    el, bs, _ = synth.GEOM[ty]
    rows, cols = 96, 512
    raw = np.random.Generator(np.random.PCG64(99 + ty)).integers(0, 256, rows * cols // el * bs, dtype=np.uint8)
    m = lib.QMat(ctx, ty, rows, cols, raw)
    with np.errstate(all="ignore"):
        got = m.to_f32(); exp = orc.dequant(ty, raw, rows * cols).reshape(rows, cols)
    ok = (bits(got) == bits(exp)) | (np.isnan(got) & np.isnan(exp))
    assert ok.all()


def test_known_answer_blocks_on_device(ctx):
    z = np_ref.pack_iq3s(1.0, np.zeros(64, np.uint8), np.zeros(8, np.uint8), np.zeros(32, np.uint8), np.zeros(4, np.uint8))
    m = lib.QMat(ctx, lib.IQ3_S, 1, 256, z)
    assert np.array_equal(m.to_f32(), np.ones((1, 256), np.float32))
    z2 = np_ref.pack_iq2xs(2.0, np.zeros(32, np.uint16), np.zeros(8, np.uint8))
    assert np.array_equal(lib.QMat(ctx, lib.IQ2_XS, 1, 256, z2).to_f32(), np.full((1, 256), 2.0, np.float32))


def test_known_answer_blocks_of_the_recoded_types(ctx):
    def blk(n, d, off=0):
        b = np.zeros(n, np.uint8); b[off:off + 2] = np_ref.f16_bytes(d); return b
    # zero payload: first codebook entry, scale bits 0, no signs -> every value equals d (see the oracle's known answers)
    for ty, n in ((lib.IQ2_XXS, 66), (lib.IQ2_S, 82), (lib.IQ3_XXS, 98)):
        assert np.array_equal(lib.QMat(ctx, ty, 1, 256, blk(n, 3.0)).to_f32(), np.full((1, 256), 3.0, np.float32)), ty
    assert np.array_equal(lib.QMat(ctx, lib.IQ4_XS, 1, 256, blk(136, 0.5)).to_f32(), np.full((1, 256), -127 * (0.5 * -32), np.float32))
    b = blk(210, 0.5, off=208); b[192:208] = 1
    assert np.array_equal(lib.QMat(ctx, lib.Q6_K, 1, 256, b).to_f32(), np.full((1, 256), -16.0, np.float32))
    kv = np.array(np_ref.IQ4NL_VALUES, np.float32)
    b = np.concatenate([blk(18, 2.0), blk(18, 1.0)]); b[2:18] = np.arange(16) | ((15 - np.arange(16)) << 4); b[20:36] = 0x88
    y = lib.QMat(ctx, lib.IQ4_NL, 1, 64, b).to_f32()[0]
    assert np.array_equal(y[:16], 2.0 * kv) and np.array_equal(y[16:32], 2.0 * kv[::-1]) and np.array_equal(y[32:], np.full(32, kv[8]))


@pytest.mark.parametrize("ty", FMTS)
def test_device_generator_equals_host_generator(ctx, ty):
    el, bs, _ = synth.GEOM[ty]
    nb = 3000
    dev = ctx.alloc(nb * bs)
    ctx.synth_blocks(ty, nb, 777 + ty, dev_out=dev)
    got = ctx.download(dev, (nb * bs,), np.uint8); ctx.free(dev)
    assert np.array_equal(got, synth.blocks(ty, nb, 777 + ty))


@pytest.mark.parametrize("ty", ALL)
@pytest.mark.parametrize("t", [1, 2, 3, 4, 5, 8])
def test_gemv_matches_truth_and_oracle(ctx, ty, t):
    rows, cols = 320, 2048
    raw = raw_matrix(ty, rows, cols, 21 + ty)
    m = lib.QMat(ctx, ty, rows, cols, raw)
    x = synth.normal((t, cols), 31 + t)
    y = m.matmul(x)
    W = orc.dequant(ty, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    truth = x.astype(np.float64) @ W.T
    assert relerr(y, truth) <= TOL
    assert relerr(orc.matmul(ty, raw, rows, cols, x), truth) <= TOL


# the shapes of the benchmark sweep: rows <- cols
SHAPES = [(4096, 2048), (2048, 4096), (512, 2048), (2048, 512)]


@pytest.mark.parametrize("ty", FMTS)
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_gemv_sweep_shapes(ctx, ty, rows, cols):
    raw = synth.matrix(ty, rows, cols, 41 + ty)
    m = lib.QMat(ctx, ty, rows, cols, raw)
    W = orc.dequant(ty, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    for t in (1, 2, 4, 8):
        x = synth.normal((t, cols), 51 + t)
        assert relerr(m.matmul(x), x.astype(np.float64) @ W.T) <= TOL, t


@pytest.mark.parametrize("ty", FMTS)
def test_result_for_a_token_does_not_depend_on_batch_width(ctx, ty):
    rows, cols = 1024, 2048
    m = lib.QMat(ctx, ty, rows, cols, synth.matrix(ty, rows, cols, 61 + ty))
    x = synth.normal((8, cols), 71)
    y8 = m.matmul(x)
    for t in (1, 2, 4):
        yt = m.matmul(x[:t])
        if ty == lib.IQ3_S and t == 1:          # one token of an IQ3_S matrix has a kernel of its own: equal to rounding, and to itself
            assert relerr(yt, y8[:1]) <= 2e-6 and np.array_equal(bits(yt), bits(m.matmul(x[:1])))
        else:
            assert np.array_equal(bits(yt), bits(y8[:t])), t
    if ty == lib.IQ3_S:
        assert relerr(m.matmul(x[3:4]), y8[3:4]) <= 2e-6 and np.array_equal(bits(m.matmul(x[2:4])[1:]), bits(y8[3:4]))
    else:
        assert np.array_equal(bits(m.matmul(x[3:4])), bits(y8[3:4]))
    # and it is reproducible run to run (split-K partials are added in a fixed order)
    assert np.array_equal(bits(m.matmul(x)), bits(y8))
    y8f = m.matmul_f32(x)
    for t in (1, 3):
        assert np.array_equal(bits(m.matmul_f32(x[:t])), bits(y8f[:t])), t


# ---- IQ3_S: the operator's integer-dot path (matmul) beside the f32 multiply-add path the layers use (matmul_f32) ------
@pytest.mark.parametrize("rows,cols", [(320, 2048), (4096, 2048), (2048, 4096), (2048, 512), (100, 256)])
def test_iq3s_both_paths_match_truth_and_each_other(ctx, rows, cols):
    raw = synth.matrix(lib.IQ3_S, rows, cols, 131)
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, raw)
    W = orc.dequant(lib.IQ3_S, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    for t in (1, 2, 3, 5, 8):
        x = synth.normal((t, cols), 141 + t)
        truth = x.astype(np.float64) @ W.T
        yi, yf = m.matmul(x), m.matmul_f32(x)
        assert relerr(yi, truth) <= TOL and relerr(yf, truth) <= TOL, t
        assert relerr(yi, yf) <= 2e-6, t
        for i in range(t):           # per token, whatever the window width (a single token of `matmul` runs the native-format kernel: equal to rounding)
            if t >= 2:
                pair = x[[i, (i + 1) % t]]
                assert np.array_equal(bits(m.matmul(pair)[:1]), bits(yi[i:i + 1]))
            assert relerr(m.matmul(x[i:i + 1]), yi[i:i + 1]) <= 2e-6
            assert np.array_equal(bits(m.matmul_f32(x[i:i + 1])), bits(yf[i:i + 1]))


def test_iq3s_matrix_core_path_operand_scaling_edge_cases(ctx):
    rows, cols = 256, 1024
    raw = synth.matrix(lib.IQ3_S, rows, cols, 151)
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, raw)
    W = orc.dequant(lib.IQ3_S, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    g = np.random.Generator(np.random.PCG64(152))
    x = synth.normal((6, cols), 153)
    x[0, 5] = 3.0e4; x[0, 700] = -2.0e4                       # outliers: only their own 256-column stretches are scaled down
    x[1] *= np.exp2(g.integers(-40, 40, cols // 64).repeat(64)).astype(np.float32)      # every 64 columns on their own power of two
    x[2] = 0.0; x[2, 64:128] = synth.normal((64,), 154)       # all-zero units beside one live unit
    x[3] *= 1e-30                                             # tiny but normal magnitudes
    x[4] *= 1e30
    x[5, ::2] = 0.0
    with np.errstate(all="ignore"):
        truth = x.astype(np.float64) @ W.T
    y = m.matmul(x)
    for i in range(6):
        assert relerr(y[i], truth[i]) <= TOL, i
    # activations that fit one f16 half (small integers): exact products, only the f32 sums round
    xi = g.integers(-1000, 1000, (1, cols)).astype(np.float32)
    assert relerr(m.matmul(xi), xi.astype(np.float64) @ W.T) <= 2e-7
    # a power-of-two scaling of the input scales the output exactly
    a = synth.normal((1, cols), 155)
    assert np.array_equal(bits(m.matmul(a * 1024.0)), bits(m.matmul(a) * 1024.0))
    # a non-finite activation: every output of that token is NaN (the f32 path gives inf or NaN row by row)
    bad = synth.normal((1, cols), 156); bad[0, 3] = np.inf
    assert np.isnan(m.matmul(bad)).all()
    bad[0, 3] = np.nan
    assert np.isnan(m.matmul(bad)).all()


def test_linearity_and_zero_input(ctx):
    rows, cols = 2048, 2048
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, synth.matrix(lib.IQ3_S, rows, cols, 81))
    a = synth.normal((1, cols), 82); b = synth.normal((1, cols), 83)
    ya, yb, yab = m.matmul(a), m.matmul(b), m.matmul(2 * a - b)
    assert relerr(yab, 2 * ya.astype(np.float64) - yb) <= 1e-5
    assert not m.matmul(np.zeros((1, cols), np.float32)).any()
    assert not m.matmul_f32(np.zeros((1, cols), np.float32)).any()
    assert relerr(m.matmul_f32(2 * a - b), 2 * m.matmul_f32(a).astype(np.float64) - m.matmul_f32(b)) <= 1e-5


def test_vocab_head_shape_against_sampled_rows(ctx):
    rows, cols = 151936, 2048
    ty = lib.IQ3_S
    el, bs, _ = synth.GEOM[ty]
    nb = rows * cols // el
    dev = ctx.alloc(nb * bs)
    ctx.synth_blocks(ty, nb, 4242, dev_out=dev)
    m = lib.QMat(ctx, ty, rows, cols, dev_blocks=dev, nbytes=nb * bs)
    ctx.free(dev)
    raw = synth.matrix(ty, rows, cols, 4242)
    x = synth.normal((2, cols), 91)
    y = m.matmul(x)
    yf = m.matmul_f32(x)
    sel = np.r_[0:64, 75000:75064, rows - 64:rows]
    rb = cols // el * bs
    Wsel = np.stack([orc.dequant(ty, raw[r * rb:(r + 1) * rb], cols) for r in sel]).astype(np.float64)
    truth = x.astype(np.float64) @ Wsel.T
    assert np.abs(y[:, sel] - truth).max() / np.abs(truth).max() <= TOL
    assert np.abs(yf[:, sel] - truth).max() / np.abs(truth).max() <= TOL
    assert relerr(y, yf) <= 2e-6
    # device generator == host generator, through the bit-exact dequant of a few rows
    for r in (0, 12345, rows - 1):
        assert np.array_equal(bits(m.row(r)), bits(orc.dequant(ty, raw[r * rb:(r + 1) * rb], cols)))


def test_argument_errors_are_reported(ctx):
    with pytest.raises(lib.PyreError):
        lib.QMat(ctx, 99, 64, 256, np.zeros(16, np.uint8))               # unknown type
    with pytest.raises(lib.PyreError):
        lib.QMat(ctx, lib.IQ3_S, 64, 200, np.zeros(16, np.uint8))        # cols not a block multiple
    with pytest.raises(lib.PyreError):
        lib.QMat(ctx, lib.IQ3_S, 64, 256, np.zeros(16, np.uint8))        # wrong byte count
    m = lib.QMat(ctx, lib.Q8_0, 64, 256, synth.matrix(lib.Q8_0, 64, 256, 1))
    with pytest.raises(lib.PyreError):
        m.matmul(np.zeros((9, 256), np.float32))                         # t outside 1..8
    with pytest.raises(lib.PyreError):
        m.row(64)


# ---- the verify window on the matrix cores (IQ3_S, t >= 2) and the native-format kernel (t = 1) ------------------------------
@pytest.mark.parametrize("t", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("rows,cols", [(320, 2048), (4096, 2048), (2048, 4096), (2048, 512), (100, 256)])
def test_verify_gemm_on_matrix_cores_matches_truth(ctx, rows, cols, t):
    raw = synth.matrix(lib.IQ3_S, rows, cols, 61 + t)
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, raw)
    W = orc.dequant(lib.IQ3_S, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    x = synth.normal((t, cols), 71 + t)
    x[0] *= 3000.0                                   # a token far outside the half range: the exact power-of-two rescaling
    x[-1] *= 1e-6
    truth = x.astype(np.float64) @ W.T
    y = m.matmul(x)
    for i in range(t):                               # per token: the tokens differ by nine orders of magnitude
        assert relerr(y[i], truth[i]) <= TOL, i
    yf = m.matmul_f32(x)
    for i in range(t):
        assert relerr(y[i], yf[i]) <= 2e-6, i


# ---- one token of an IQ3_S matrix: the file's bits per weight, codebook with signs in shared memory, integer dots --------------
@pytest.mark.parametrize("rows,cols", [(64, 256), (100, 256), (65, 512), (320, 2048), (4096, 2048), (2048, 4096), (1000, 768), (130, 8192)])
def test_iq3s_native_format_single_token(ctx, rows, cols, monkeypatch):
    monkeypatch.setenv("PYRE_QMATMUL_SMALL", "0")          # small shapes too through the native-format kernel (the operator sends them to the one-launch f32 GEMV otherwise)
    raw = synth.matrix(lib.IQ3_S, rows, cols, 300 + rows % 97)
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, raw)
    assert m.layout_bytes(2) == (rows + 63) // 64 * 64 * (cols // 256) * 112
    W = orc.dequant(lib.IQ3_S, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    g = np.random.Generator(np.random.PCG64(rows + cols))
    for case in range(6):
        x = synth.normal((1, cols), 400 + case)
        if case == 1: x *= np.exp2(g.integers(-40, 40, cols // 64).repeat(64)).astype(np.float32)      # every 64 columns on their own power of two
        if case == 2: x[0, 5] = 3.0e4; x[0, cols - 3] = -2.0e7                                          # outliers
        if case == 3: x *= 1e-30
        if case == 4: x *= 1e30
        if case == 5: x[0, ::2] = 0.0; x[0, :64] = 0.0                                                  # an all-zero unit
        with np.errstate(all="ignore"):
            truth = x.astype(np.float64) @ W.T
        y = m.matmul(x)
        assert relerr(y, truth) <= TOL, case
        assert np.array_equal(bits(y), bits(m.matmul(x)))          # run to run
        assert relerr(y, m.matmul(np.concatenate([x, x]))[:1]) <= 2e-6          # the window's kernel agrees to rounding
    xi = g.integers(-1000, 1000, (1, cols)).astype(np.float32)          # integers: exact digits, exact sums, only the f32 scaling rounds
    assert relerr(m.matmul(xi), xi.astype(np.float64) @ W.T) <= 2e-7
    a = synth.normal((1, cols), 155)
    assert np.array_equal(bits(m.matmul(a * 1024.0)), bits(m.matmul(a) * 1024.0))          # a power of two scales the result exactly
    bad = synth.normal((1, cols), 156); bad[0, 3] = np.inf
    assert np.isnan(m.matmul(bad)).all()
    bad[0, 3] = np.nan
    assert np.isnan(m.matmul(bad)).all()
    assert not m.matmul(np.zeros((1, cols), np.float32)).any()


# ---- one token of an IQ2_XS matrix: 80 bytes per 256 weights, two signed codebook tables in shared memory, integer dots;
# ---- of a Q4_K matrix: the file's 144 bytes, nibbles straight into the integer dots, the minima through the digit sums ----------
@pytest.mark.gpu
@pytest.mark.parametrize("ty,piece_bytes", [(lib.IQ2_XS, 80), (lib.Q4_K, 144)])
@pytest.mark.parametrize("rows,cols", [(64, 256), (100, 256), (65, 512), (320, 2048), (4096, 2048), (1000, 768), (130, 8192), (8256, 1024)])
def test_iq2xs_q4k_native_format_single_token(ctx, rows, cols, ty, piece_bytes, monkeypatch):
    monkeypatch.setenv("PYRE_QMATMUL_SMALL", "0")          # small shapes too through the native-format kernel
    raw = synth.matrix(ty, rows, cols, 500 + rows % 97)
    m = lib.QMat(ctx, ty, rows, cols, raw)
    assert m.layout_bytes(2) == (rows + 63) // 64 * 64 * (cols // 256) * piece_bytes
    W = orc.dequant(ty, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    g = np.random.Generator(np.random.PCG64(rows + cols + 1))
    for case in range(6):
        x = synth.normal((1, cols), 600 + case)
        if case == 1: x *= np.exp2(g.integers(-40, 40, cols // 64).repeat(64)).astype(np.float32)
        if case == 2: x[0, 5] = 3.0e4; x[0, cols - 3] = -2.0e7
        if case == 3: x *= 1e-30
        if case == 4: x *= 1e30
        if case == 5: x[0, ::2] = 0.0; x[0, :64] = 0.0
        with np.errstate(all="ignore"):
            truth = x.astype(np.float64) @ W.T
        y = m.matmul(x)
        assert relerr(y, truth) <= TOL, case
        assert np.array_equal(bits(y), bits(m.matmul(x)))          # run to run
        assert relerr(y, m.matmul_f32(x)) <= 2e-6                  # the f32 GEMV agrees to rounding
        assert relerr(y, m.matmul(np.concatenate([x, x]))[:1]) <= 2e-6
    xi = g.integers(-1000, 1000, (1, cols)).astype(np.float32)          # integers: exact digits, exact sums, only the f32 scaling rounds
    assert relerr(m.matmul(xi), xi.astype(np.float64) @ W.T) <= 4e-7          # (sixteen f32 additions a super-block: two scales a sub-block)
    a = synth.normal((1, cols), 155)
    assert np.array_equal(bits(m.matmul(a * 1024.0)), bits(m.matmul(a) * 1024.0))
    bad = synth.normal((1, cols), 156); bad[0, 3] = np.inf
    assert np.isnan(m.matmul(bad)).all()
    assert not m.matmul(np.zeros((1, cols), np.float32)).any()
    monkeypatch.setenv("PYRE_QMATMUL_SMALL", "1")
    if (rows + 63) // 64 <= 128:                                        # a small matrix: the one-launch f32 GEMV
        assert np.array_equal(bits(m.matmul(a)), bits(m.matmul_f32(a)))


@pytest.mark.gpu
def test_small_iq3s_single_token_takes_one_launch(ctx):
    """A single token of an IQ3_S matrix of at most 128 row tiles goes through the lane = row f32 GEMV (one launch): the
    result is bit for bit pyre_qmatmul_f32's; a window and a large matrix are unaffected."""
    rows, cols = 4096, 4096
    raw = synth.matrix(lib.IQ3_S, rows, cols, 77)
    m = lib.QMat(ctx, lib.IQ3_S, rows, cols, raw)
    x = synth.normal((1, cols), 78)
    y = m.matmul(x)
    assert np.array_equal(bits(y), bits(m.matmul_f32(x)))
    W = orc.dequant(lib.IQ3_S, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    assert relerr(y, x.astype(np.float64) @ W.T) <= TOL
    ctx.prof_reset(); ctx.prof_enable(True)
    m.matmul(x); ctx.sync()
    rep = ctx.prof_report(); ctx.prof_enable(False)
    assert sum(v[0] for v in rep.values()) == 1, rep          # one kernel launch for the call


# ---- a window of a Q4_K matrix on the matrix cores: codes -> f16 by or-ing, scales folded before the product, minima through
# ---- the sub-block sums of the activations; of an IQ2_XS matrix: codes -> f16 by byte permutes through a table in registers;
# ---- of a Q8_0 matrix: bytes -> f16 by one byte permute and an addition, the block's d after the product ----------------------
@pytest.mark.gpu
@pytest.mark.parametrize("ty,switch", [(lib.Q4_K, "PYRE_QMATMUL_Q4M"), (lib.IQ2_XS, "PYRE_QMATMUL_Q2M"), (lib.Q8_0, "PYRE_QMATMUL_Q8M")], ids=["q4_k", "iq2_xs", "q8_0"])
@pytest.mark.parametrize("rows,cols", [(64, 256), (100, 512), (320, 2048), (8256, 1024), (1000, 768), (130, 8192)])
def test_q4k_window_on_the_matrix_cores(ctx, rows, cols, ty, switch, monkeypatch):
    monkeypatch.setenv("PYRE_QMATMUL_SMALL", "0")          # small shapes too through the matrix-core kernel
    raw = synth.matrix(ty, rows, cols, 900 + rows % 97)
    m = lib.QMat(ctx, ty, rows, cols, raw)
    assert m.layout_bytes(1) >= (rows + 63) // 64 * 64 * (cols // 256) * (272 if ty == lib.Q8_0 else 144)          # 4.5 bit/weight: 128 bytes of codes + a 16-byte header (Q8_0: 8.5: 256 + 16)
    W = orc.dequant(ty, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    g = np.random.Generator(np.random.PCG64(rows + cols + 3))
    for case in range(6):
        x = synth.normal((8, cols), 910 + case)
        if case == 1: x *= np.exp2(g.integers(-30, 30, cols // 256).repeat(256)).astype(np.float32)
        if case == 2: x[0, 5] = 3.0e4; x[3, cols - 3] = -2.0e7
        if case == 3: x *= 1e-25
        if case == 4: x[5] *= 1e20
        if case == 5: x[:, ::2] = 0.0; x[:, :64] = 0.0
        with np.errstate(all="ignore"):
            truth = x.astype(np.float64) @ W.T
        y = m.matmul(x)
        for ti in range(8):                                     # per token: each has its own largest magnitude
            assert relerr(y[ti], truth[ti]) <= TOL, (case, ti)
        assert np.array_equal(bits(y), bits(m.matmul(x)))          # run to run
        for t in (2, 3, 5):                                     # a token's bits do not depend on the window's width
            assert np.array_equal(bits(m.matmul(x[:t])), bits(y[:t])), (case, t)
        assert relerr(y[:2], m.matmul_f32(x[:2])) <= 4e-6       # the f32 GEMV agrees to rounding
    assert not m.matmul(np.zeros((4, cols), np.float32)).any()
    bad = synth.normal((3, cols), 920); bad[1, 7] = np.nan
    yb = m.matmul(bad)
    assert np.isnan(yb[1]).all() and np.isfinite(yb[0]).all() and np.isfinite(yb[2]).all()          # a token's NaN stays its own
    ctx.prof_reset(); ctx.prof_enable(True)
    m.matmul(x[:4]); ctx.sync()
    assert any(k.startswith({lib.Q4_K: "gemm_q4k_t4", lib.IQ2_XS: "gemm_iq2xs_t4", lib.Q8_0: "gemm_q8_0_t4"}[ty]) for k in ctx.prof_report()), ctx.prof_report()          # the kernel under test is the one that ran
    ctx.prof_enable(False)
    monkeypatch.setenv(switch, "0")
    assert relerr(m.matmul(x), truth) <= TOL                     # (the lane = row window path stays available)
