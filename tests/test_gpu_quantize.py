"""Parity of the HIP quantizer against the CPU oracle, through the C ABI. Needs an MI355X.

Mirrors the structure of the reference's own test (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp:239-402):
for every bit width and, at 1 bit, both threshold modes, several iterations with the residual carried over and
the output accumulated from the second iteration on; each iteration is checked against the oracle on the same
(gradient, residual-in), which the oracle chain supplies (teacher forcing), and the free-running GPU chain is
checked through the conservation law.
"""
import sys

import numpy as np
import pytest
import torch

import cntk_amd
import datagen
import oracle
import parity
from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

pytestmark = pytest.mark.gpu

VARIANTS = [(1, False), (1, True), (2, False), (4, False), (8, False), (16, False), (32, False)]
PATH_AUTO, PATH_TILE, PATH_TALL, PATH_COL, PATH_REG, PATH_REG_SCALAR, PATH_STRIP, PATH_STRIP_PASSES = 0, 1, 2, 3, 4, 5, 6, 7


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def quantizer():
    assert torch.cuda.is_available(), "these tests need the GPU"
    q = MatrixQuantizerImpl.Create(0, False)
    yield q
    torch.cuda.synchronize()


def gpu_quantize(qz, g, r_in, nbits, zt, in_place=True, host_q=False):
    rows, cols = g.shape
    G = Matrix.from_numpy(g)
    R = Matrix.from_numpy(r_in)
    Rout = R if in_place else Matrix(rows, cols)
    Q = QuantizedMatrix(rows, cols, nbits, cntk_amd.CPUDEVICE if host_q else 0)
    qz.QuantizeAsync(G, R, Q, Rout, zt)
    qz.WaitQuantizeAsyncDone()
    if not host_q:
        torch.cuda.synchronize()
    return Q, Rout.to_numpy()


def run_chain(qz, rows, cols, nbits, zt, make_input, iterations, report, in_place=True, host_q=False):
    """Teacher-forced chain: the oracle's residual feeds both sides at every step."""
    res_o = np.zeros((rows, cols), np.float32, order="F")
    out_o = np.zeros((rows, cols), np.float32, order="F")
    Out = Matrix(rows, cols)
    for it in range(iterations):
        g = make_input(it)
        Q, r_gpu = gpu_quantize(qz, g, res_o, nbits, zt, in_place=in_place, host_q=host_q)
        q_gpu = Q.to_numpy()
        parity.check_quantize(g, res_o, q_gpu, r_gpu, nbits, zt, report=report)
        # unquantize what the GPU packed, accumulating like the reference test does
        prev = Out.to_numpy()
        qz.UnquantizeAsync(Q, Out, add=(it > 0))
        qz.WaitUnquantizeAsyncDone()
        parity.check_unquantize(q_gpu, rows, cols, nbits, Out.to_numpy(), prev_out=prev if it > 0 else None)
        # carry the ORACLE's state forward so that both sides keep seeing identical inputs
        q_or, _ = oracle.quantize(g, res_o, nbits, zt, r_out=res_o, threads=8)
        oracle.unquantize(q_or, rows, cols, nbits, out=out_o, add=(it > 0), threads=8)
        Out = Matrix.from_numpy(out_o)


# ---- the reference unit test's shapes ------------------------------------------------------------------

UNIT_SHAPES = [
    (25, 13, -1.0, 1.0, 2015), (25, 13, -0.005, 0.005, 2115), (13, 25, -0.00001, 0.00001, 2215),
    (13, 25, -10.0, 10.0, 2315), (25, 13, -1.0, 2.05, 2415), (489, 1, -0.5, 0.5, 2515), (1, 135, -0.5, 0.5, 2615),
    (89, 23, -0.5, 0.5, 2715), (15, 35, -0.5, 0.5, 2815), (100, 50, -0.5, 0.5, 2915),
    # the sizes the reference test was first written with (MatrixQuantizerTests.cpp:474-487)
    (256, 135, -1.0, 2.05, 2415), (737, 373, -0.5, 0.5, 2915),
]


@pytest.mark.parametrize("shape", UNIT_SHAPES, ids=["%dx%d_%d" % (s[0], s[1], s[4]) for s in UNIT_SHAPES])
def test_reference_unit_shapes(quantizer, shape):
    rows, cols, lo, hi, seed = shape
    rep = parity.Report()
    for nbits, zt in VARIANTS:
        say("unit shape", shape, "nbits", nbits, "zeroThr", zt)
        run_chain(quantizer, rows, cols, nbits, zt, lambda it: datagen.uniform(seed + it, rows, cols, lo, hi), 5, rep)
    say("  ", rep)


def test_free_running_conservation(quantizer):
    """GPU chain on its own state: g + r_in + prev_out == r_out + out (MatrixQuantizerTests.cpp:327-338)."""
    rows, cols, lo, hi = 100, 50, -0.5, 0.5
    for nbits, zt in VARIANTS:
        say("conservation nbits", nbits, "zeroThr", zt)
        R, Out = Matrix(rows, cols), Matrix(rows, cols)
        for it in range(5):
            g = datagen.uniform(2915 + it, rows, cols, lo, hi)
            r_in, prev = R.to_numpy(), Out.to_numpy()
            Q = QuantizedMatrix(rows, cols, nbits, 0)
            quantizer.QuantizeAsync(Matrix.from_numpy(g), R, Q, R, zt)
            quantizer.WaitQuantizeAsyncDone()
            quantizer.UnquantizeAsync(Q, Out, add=(it > 0))
            quantizer.WaitUnquantizeAsyncDone()
            tol = (hi - lo) * 1e-4 if nbits != 32 else 1e-6
            parity.conservation(g, r_in, prev, R.to_numpy(), Out.to_numpy(), tol)


# ---- every kernel path on shapes that stress its indexing ------------------------------------------------

PATH_CASES = [
    # rows, cols, path, tile_gs
    (1, 1, PATH_TILE, 0), (3, 70, PATH_TILE, 0), (31, 5, PATH_TILE, 8), (33, 67, PATH_TILE, 0), (64, 64, PATH_TILE, 16),
    (147, 64, PATH_TILE, 0), (429, 37, PATH_TILE, 0), (429, 37, PATH_TILE, 64), (576, 64, PATH_TILE, 0),
    (1023, 9, PATH_TILE, 0), (1024, 33, PATH_TILE, 0), (2048, 19, PATH_TILE, 0), (2048, 19, PATH_TILE, 256),
    (2304, 5, PATH_TILE, 0), (4608, 3, PATH_TILE, 0), (9304, 2, PATH_TILE, 0), (14336, 1, PATH_TILE, 0),
    (1, 5, PATH_TALL, 0), (70, 3, PATH_TALL, 0), (1025, 3, PATH_TALL, 0), (20001, 2, PATH_TALL, 0),
    (33000, 2, PATH_AUTO, 0),
    # one workgroup per column: any height that is a multiple of 4
    (4, 3, PATH_COL, 0), (36, 70, PATH_COL, 0), (128, 9, PATH_COL, 0), (1000, 5, PATH_COL, 0), (1028, 7, PATH_COL, 0),
    (2048, 19, PATH_COL, 0), (2304, 5, PATH_COL, 0), (4100, 3, PATH_COL, 0), (9304, 2, PATH_COL, 0), (14336, 2, PATH_COL, 0),
    (9304, 3, PATH_AUTO, 0), (1152, 40, PATH_AUTO, 0), (100000, 2, PATH_AUTO, 0), (14340, 3, PATH_AUTO, 0),
    # one workgroup per column, the column in registers: 256 threads up to 14336 rows, 1024 above
    (4, 3, PATH_REG, 0), (36, 70, PATH_REG, 0), (1000, 5, PATH_REG, 0), (4100, 3, PATH_REG, 0), (6148, 5, PATH_REG, 0),
    (9304, 2, PATH_REG, 0), (12292, 3, PATH_REG, 0), (14336, 2, PATH_REG, 0), (14340, 3, PATH_REG, 0), (20000, 3, PATH_REG, 0),
    (40964, 2, PATH_REG, 0), (65540, 2, PATH_REG, 0), (102400, 1, PATH_REG, 0), (102404, 2, PATH_AUTO, 0),
    # the same one float at a time: any height up to 98304 rows (the automatic choice for tall columns the piece-wise
    # kernel cannot take)
    (1, 3, PATH_REG_SCALAR, 0), (37, 5, PATH_REG_SCALAR, 0), (1001, 3, PATH_REG_SCALAR, 0), (14337, 3, PATH_AUTO, 0),
    (20001, 2, PATH_AUTO, 0), (32769, 2, PATH_REG_SCALAR, 0), (50257, 2, PATH_AUTO, 0), (65537, 1, PATH_AUTO, 0), (98303, 1, PATH_AUTO, 0),
    (98304, 1, PATH_REG_SCALAR, 0), (98305, 1, PATH_AUTO, 0),
    # the piece-wise kernel with edge elements (heights that are not a multiple of 4; the automatic choice for them above
    # 14336 rows when the three matrices share their alignment)
    (9, 5, PATH_REG, 0), (37, 5, PATH_REG, 0), (1001, 3, PATH_REG, 0), (4099, 2, PATH_REG, 0), (14338, 3, PATH_REG, 0),
    (50257, 2, PATH_REG, 0), (102365, 1, PATH_REG, 0),
    # several workgroups per column, a strip of QWords each: any height and alignment, one strip or many, full or ragged
    (1, 3, PATH_STRIP, 0), (37, 5, PATH_STRIP, 0), (1000, 3, PATH_STRIP, 0), (8192, 3, PATH_STRIP, 0), (8193, 2, PATH_STRIP, 0),
    (16384, 2, PATH_STRIP, 0),
    (9304, 3, PATH_STRIP, 0), (16385, 2, PATH_STRIP, 0), (32768, 2, PATH_STRIP, 0), (50257, 3, PATH_STRIP, 0), (100000, 5, PATH_STRIP, 0),
    (102401, 2, PATH_AUTO, 0), (200000, 3, PATH_AUTO, 0), (262147, 2, PATH_STRIP, 0), (524288, 9, PATH_STRIP, 0), (524289, 1, PATH_AUTO, 0),
    (600000, 9, PATH_STRIP, 0), (655361, 1, PATH_AUTO, 0), (1000003, 1, PATH_AUTO, 0), (1500001, 2, PATH_STRIP, 0),
    # the strips in two or three launches (nothing waits, nothing need be resident together): any height of two strips or
    # more, and the automatic choice for columns of more strips than the device holds at once
    (9304, 3, PATH_STRIP_PASSES, 0), (16385, 2, PATH_STRIP_PASSES, 0), (50257, 3, PATH_STRIP_PASSES, 0), (102401, 2, PATH_STRIP_PASSES, 0),
    (262147, 2, PATH_STRIP_PASSES, 0), (6000001, 1, PATH_AUTO, 0),
]


def strip_words(nbits):
    """QWords of a float column that one strip holds."""
    return 512 if nbits == 1 else 1024 if nbits == 2 else 2048


@pytest.mark.parametrize("case", PATH_CASES, ids=["%dx%d_p%d_g%d" % c for c in PATH_CASES])
def test_kernel_paths(case):
    rows, cols, path, gs = case
    qz = MatrixQuantizerImpl.Create(0, False)
    rep = parity.Report()
    for nbits, zt in VARIANTS:
        say("path case", case, "nbits", nbits, "zeroThr", zt)
        if (path == PATH_STRIP and (nbits == 32 or oracle.qwords_per_col(rows, nbits) > qz._strip_max_strips(nbits, zt) * strip_words(nbits))) or \
                (path == PATH_STRIP_PASSES and (nbits == 32 or oracle.qwords_per_col(rows, nbits) <= strip_words(nbits))):
            # whole-QWord codes need no assembling, a column's strips must be resident on the device together, and a single
            # strip has nothing to cut into passes
            qz._set_tuning(quantize_path=path)
            with pytest.raises(cntk_amd.QuantizerLogicError):
                gpu_quantize(qz, datagen.normal(1, rows, cols), np.zeros((rows, cols), np.float32, order="F"), nbits, zt)
            continue
        if path in (PATH_REG, PATH_REG_SCALAR) and (nbits == 32 or (50 + 2 * oracle.qwords_per_col(rows, nbits)) * 4 > 163840):
            # whole-QWord codes and columns whose QWords (twice, as the stripe reduction keeps them) exceed the LDS of a compute
            # unit are not the register kernels' business
            qz._set_tuning(quantize_path=path)
            with pytest.raises(cntk_amd.QuantizerLogicError):
                gpu_quantize(qz, datagen.normal(1, rows, cols), np.zeros((rows, cols), np.float32, order="F"), nbits, zt)
            continue
        # alternate between the two ways a tile kernel writes its residual
        qz._set_tuning(quantize_path=path, tile_gs=gs, tile_stage=(nbits + rows) % 2 if path == PATH_TILE else -1)
        # a shifted mean, one all-zero column and outliers exercise every branch of the statistics
        def make(it):
            a = datagen.normal_with_outliers(1000 * rows + cols + it, rows, cols, 0.01) + np.float32(0.004 * (it % 2))
            a = np.asfortranarray(a.astype(np.float32))
            if cols > 1:
                a[:, cols // 2] = 0.0
            return a
        run_chain(qz, rows, cols, nbits, zt, make, 2, rep)
    say("  ", rep)


@pytest.mark.parametrize("rows,cols", [(9000, 7), (40000, 5), (150001, 5), (262144, 3)])
def test_strips_in_passes_give_the_strip_kernels_bytes(rows, cols):
    """The strip kernel cut into launches at the points where its workgroups would wait for each other adds the same
    partial sums in the same order: packed bytes and residuals are identical, for floats and doubles."""
    qz = MatrixQuantizerImpl.Create(0, False)
    for dtype, npdt in ((torch.float32, np.float32), (torch.float64, np.float64)):
        g, r = datagen.normal_with_outliers(rows, rows, cols, 0.01, dtype=npdt), datagen.normal(rows + 1, rows, cols, 0.002, dtype=npdt)
        for nbits, zt in VARIANTS:
            per_strip = (64 // nbits if npdt == np.float64 else 32 // nbits) * (strip_words(nbits) if npdt == np.float32 else
                                                                                 {1: 128, 2: 256, 4: 512}.get(nbits, 1024))
            if nbits == 32 or rows <= per_strip:
                continue
            say("strips in one launch and in passes", rows, cols, npdt.__name__, nbits, zt)
            outs = []
            for path in (PATH_STRIP, PATH_STRIP_PASSES):
                qz._set_tuning(quantize_path=path)
                G, R = Matrix.from_numpy(g), Matrix.from_numpy(r)
                Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=dtype)
                qz.QuantizeAsync(G, R, Q, R, zt)
                qz.WaitQuantizeAsyncDone()
                torch.cuda.synchronize()
                outs.append((Q.to_numpy(), R.to_numpy()))
            assert np.array_equal(outs[0][0], outs[1][0]) and parity.bits_equal(outs[0][1], outs[1][1])
        qz._set_tuning(quantize_path=PATH_AUTO)


def test_tall_columns_that_never_wait():
    """A handle told that its tall columns must never wait runs them as the strips in passes (the bytes of the single launch),
    keeps doing so for the tall member of a batched call, and no longer offers the fused reduction of tall stripes."""
    rows, cols = 150001, 4
    a, b = MatrixQuantizerImpl.Create(0, False), MatrixQuantizerImpl.Create(0, False)
    b.SetTallColumnsNeverWait(True)
    assert a.StripeReduceTakes(rows, cols, 1) and not b.StripeReduceTakes(rows, cols, 1) and b.StripeReduceTakes(9304, cols, 1)
    g, r = datagen.normal_with_outliers(3, rows, cols, 0.01), datagen.normal(4, rows, cols, 0.002)
    small = datagen.normal(5, 2048, 6)
    outs = []
    for qz in (a, b):
        G, R, Q = Matrix.from_numpy(g), Matrix.from_numpy(r), QuantizedMatrix(rows, cols, 1, 0)
        qz.QuantizeAsync(G, R, Q, R, False)
        qz.WaitQuantizeAsyncDone()
        G2, R2, Q2 = Matrix.from_numpy(g), Matrix.from_numpy(r), QuantizedMatrix(rows, cols, 1, 0)
        S, RS, QS = Matrix.from_numpy(small), Matrix(2048, 6), QuantizedMatrix(2048, 6, 1, 0)
        S3, RS3, QS3 = Matrix.from_numpy(small), Matrix(2048, 6), QuantizedMatrix(2048, 6, 1, 0)
        qz.QuantizeBatchAsync([(G2, R2, Q2, R2), (S, RS, QS, RS), (S3, RS3, QS3, RS3)], False)
        qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        assert np.array_equal(Q.to_numpy(), Q2.to_numpy()) and parity.bits_equal(R.to_numpy(), R2.to_numpy())
        outs.append((Q.to_numpy(), R.to_numpy()))
    assert np.array_equal(outs[0][0], outs[1][0]) and parity.bits_equal(outs[0][1], outs[1][1])
    parity.check_quantize(g, r, outs[1][0], outs[1][1], 1, False)
    # with no patience at all for another workgroup's partial sum (every wait that does not find its record at the first
    # look gives up) the launches that never wait still give the right bytes
    b._set_strip_spin_limit(0)
    G, R, Q = Matrix.from_numpy(g), Matrix.from_numpy(r), QuantizedMatrix(rows, cols, 1, 0)
    b.QuantizeAsync(G, R, Q, R, False)
    b.WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
    assert np.array_equal(Q.to_numpy(), outs[0][0]) and parity.bits_equal(R.to_numpy(), outs[0][1])
    b._set_strip_spin_limit(1 << 17)
    b.SetTallColumnsNeverWait(False)
    assert b.StripeReduceTakes(rows, cols, 1)


@pytest.mark.parametrize("rows", [2048, 4100, 9304, 14336])
def test_register_and_lds_column_kernels_give_the_same_bytes(rows):
    """Up to 14336 rows the register kernels sum the column statistics in the order of the LDS kernels (which the
    stripe reduction uses at these heights): packed bytes and residuals are identical for every bit width."""
    qz = MatrixQuantizerImpl.Create(0, False)
    cols = 5
    g, r = datagen.normal_with_outliers(rows, rows, cols, 0.01), datagen.normal(rows + 1, rows, cols, 0.002)
    for nbits, zt in VARIANTS:
        if nbits == 32:
            continue
        say("register vs LDS column kernel", rows, nbits, zt)
        qz._set_tuning(quantize_path=PATH_COL)
        Qa, ra = gpu_quantize(qz, g, r, nbits, zt)
        qz._set_tuning(quantize_path=PATH_REG)
        Qb, rb = gpu_quantize(qz, g, r, nbits, zt)
        assert np.array_equal(Qa.to_numpy(), Qb.to_numpy()) and parity.bits_equal(ra, rb)
    # matrices that all start 16, 48 or 112 bytes into a 128-byte line (and once at different offsets, where no shift
    # is used): still the same bytes from both kernels, and right by the oracle
    for og, orr in ((4, 4), (12, 12), (28, 28), (4, 8)):
        def place(a, off):
            buf = torch.zeros(rows * cols + 64, dtype=torch.float32, device="cuda:0")
            buf[off:off + rows * cols] = torch.from_numpy(a.reshape(-1, order="F").copy()).cuda()
            return Matrix(rows, cols, 0, buf[off:off + rows * cols])
        outs = []
        for path in (PATH_COL, PATH_REG):
            qz._set_tuning(quantize_path=path)
            G, R, Q = place(g, og), place(r, orr), QuantizedMatrix(rows, cols, 1, 0)
            assert G.Data() % 128 == 4 * og and R.Data() % 128 == 4 * orr
            qz.QuantizeAsync(G, R, Q, R, False)
            qz.WaitQuantizeAsyncDone()
            outs.append((Q.to_numpy(), R.to_numpy()))
        assert np.array_equal(outs[0][0], outs[1][0]) and parity.bits_equal(outs[0][1], outs[1][1])
        parity.check_quantize(g, r, outs[1][0], outs[1][1], 1, False)
    # beyond 25 pieces for each of 1024 threads the forced path refuses
    with pytest.raises(cntk_amd.QuantizerLogicError):
        gpu_quantize(qz, datagen.normal(1, 102404, 1), np.zeros((102404, 1), np.float32, order="F"), 1, False)


@pytest.mark.parametrize("rows", [1024, 2048, 4096])
def test_workgroup_per_column_path(rows):
    """The 1-bit kernel that keeps one column per workgroup in LDS: the path the automatic choice takes for these
    heights, here also forced, against the oracle and against the general tile kernel's codes."""
    qz = MatrixQuantizerImpl.Create(0, False)
    rep = parity.Report()
    for path in (PATH_COL, PATH_AUTO):
        qz._set_tuning(quantize_path=path)
        for cols in (1, 4, 7, 130):
            for zt in (False, True):
                say("column kernel", rows, cols, zt, "path", path)
                def make(it):
                    a = datagen.normal(rows + cols + it, rows, cols) + np.float32(0.003 * it)
                    a = np.asfortranarray(a.astype(np.float32))
                    if cols > 2:
                        a[:, 1] = 0.0
                    return a
                run_chain(qz, rows, cols, 1, zt, make, 3, rep)
    say("  ", rep)
    qz._set_tuning(quantize_path=PATH_COL)
    # shapes and alignments the path does not cover are refused when forced, not mis-computed
    with pytest.raises(cntk_amd.QuantizerLogicError):
        gpu_quantize(qz, datagen.normal(1, 513, 4), np.zeros((513, 4), np.float32, order="F"), 1, False)
    # a packed buffer that is only 4-byte aligned takes the general (not unrolled) column kernel: same bytes
    cols = 6
    g, r = datagen.normal(8, rows, cols), datagen.normal(9, rows, cols, 0.002)
    for zt in (False, True):
        Qa, ra = gpu_quantize(qz, g, r, 1, zt)
        raw = torch.zeros(Qa.GetSize() + 4, dtype=torch.uint8, device="cuda:0")
        Qb = QuantizedMatrix(rows, cols, 1, 0, raw[4:])
        assert Qb.Buffer() % 8 == 4
        G, R = Matrix.from_numpy(g), Matrix.from_numpy(r)
        qz.QuantizeAsync(G, R, Qb, R, zt)
        qz.WaitQuantizeAsyncDone()
        assert np.array_equal(Qa.to_numpy(), Qb.to_numpy()) and parity.bits_equal(ra, R.to_numpy())
    # a gradient that starts 4 bytes off a 16-byte boundary: refused when forced, served by the tile kernel otherwise
    cols = 5
    g = datagen.normal(5, rows, cols)
    big = torch.zeros(rows * cols + 4, dtype=torch.float32, device="cuda:0")
    big[1:1 + rows * cols] = torch.from_numpy(g.reshape(-1, order="F").copy()).cuda()
    G = Matrix(rows, cols, 0, big[1:1 + rows * cols])
    R, Q = Matrix(rows, cols), QuantizedMatrix(rows, cols, 1, 0)
    with pytest.raises(cntk_amd.QuantizerLogicError):
        qz.QuantizeAsync(G, R, Q, R, False)
    qz._set_tuning(quantize_path=PATH_AUTO)
    qz.QuantizeAsync(G, R, Q, R, False)
    qz.WaitQuantizeAsyncDone()
    parity.check_quantize(g, np.zeros_like(g, order="F"), Q.to_numpy(), R.to_numpy(), 1, False, report=rep)


def test_unquantize_variants(quantizer):
    """Scalar and 16-byte-store decoders, every slot split, add and overwrite: all bit-exact."""
    # QWord-major decoder with 16-byte stores, its 4-byte variant, and the segment decoder for long odd columns
    for rows, cols in [(5, 3), (37, 2), (128, 9), (429, 5), (2048, 6), (4100, 2), (1001, 5), (3003, 3), (100000, 2)]:
        for nbits, zt in VARIANTS:
            g = datagen.normal(rows * 7 + nbits, rows, cols)
            q, _ = oracle.quantize(g, np.zeros_like(g, order="F"), nbits, zt)
            prev = datagen.normal(rows * 9 + nbits, rows, cols, 1.0)
            for slots in (0, 1, 3, 32):
                for scalar in (0, 1):
                    say("unquantize", rows, cols, nbits, "slots", slots, "scalar", scalar)
                    qz = MatrixQuantizerImpl.Create(0, False)
                    qz._set_tuning(unq_slots=slots, unq_mode=scalar)
                    Q = QuantizedMatrix(rows, cols, nbits, 0)
                    Q.from_numpy(q)
                    for add in (False, True):
                        Out = Matrix.from_numpy(prev)
                        qz.UnquantizeAsync(Q, Out, add=add)
                        qz.WaitUnquantizeAsyncDone()
                        parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)


TILE_DECODER_SHAPES = [(1, 1), (1, 9), (2, 7), (3, 5), (5, 3), (31, 13), (32, 8), (33, 41), (64, 100), (147, 64), (256, 1031),
                       (429, 37), (512, 24), (1000, 9), (1001, 5), (1024, 3), (2047, 2), (2048, 7), (4096, 5), (4095, 3), (4097, 3), (9305, 2), (16383, 2), (16385, 2), (1025, 7), (1026, 5), (1027, 3), (50257, 2), (100001, 2),
                       # heights and QWord counts in whole 16-byte groups: the decoder that treats the matrix as one run of such groups
                       (4, 3), (12, 50), (128, 4099), (576, 50), (1152, 33), (4608, 3)]


@pytest.mark.parametrize("shape", TILE_DECODER_SHAPES, ids=["%dx%d" % s for s in TILE_DECODER_SHAPES])
def test_tile_decoder(shape):
    """The decoder that takes several short columns per workgroup: forced on every height it accepts (groups of four
    values that straddle columns, matrices whose size is not a multiple of four, a last tile with fewer columns), and
    as the automatic choice; add and overwrite; bit-exact. A misaligned output falls back to another decoder."""
    rows, cols = shape
    for nbits, zt in VARIANTS:
        g = datagen.normal_with_outliers(rows * 11 + nbits, rows, cols, 0.01)
        q, _ = oracle.quantize(g, np.zeros_like(g, order="F"), nbits, zt)
        prev = datagen.normal(rows * 13 + nbits, rows, cols, 1.0)
        for mode in (2, 0, 3, 5, 6):
            say("tile decoder", rows, cols, nbits, "mode", mode)
            qz = MatrixQuantizerImpl.Create(0, False)
            qz._set_tuning(unq_mode=mode)
            Q = QuantizedMatrix(rows, cols, nbits, 0)
            Q.from_numpy(q)
            for add in (False, True):
                Out = Matrix.from_numpy(prev)
                qz.UnquantizeAsync(Q, Out, add=add)
                qz.WaitUnquantizeAsyncDone()
                parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)
        # output 4 bytes off a 16-byte boundary
        big = torch.zeros(rows * cols + 4, dtype=torch.float32, device="cuda:0")
        Out = Matrix(rows, cols, 0, big[1:1 + rows * cols])
        qz.UnquantizeAsync(Q, Out)
        qz.WaitUnquantizeAsyncDone()
        parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy())
        assert float(big[0]) == 0.0 and float(big[-1]) == 0.0 and float(big[-2]) == 0.0 and float(big[-3]) == 0.0


DIRECT_DECODER_SHAPES = [(2048, 5), (2049, 3), (4096, 3), (6143, 2), (8192, 3), (9304, 3), (16384, 2), (20001, 2), (32770, 2), (100000, 2),
                         (150001, 2), (600000, 1)]


@pytest.mark.parametrize("shape", DIRECT_DECODER_SHAPES, ids=["%dx%d" % s for s in DIRECT_DECODER_SHAPES])
def test_row_major_decoder_that_fetches_its_qwords(shape):
    """The row-major decoder without a copy of the packed column in LDS, forced (mode 5) and as the automatic choice:
    one chunk and many per column, a last chunk of a few rows, groups of four that wrap to the next bit position,
    outputs at every offset within 16 bytes; add and overwrite; bit-exact, and nothing written outside the matrix."""
    rows, cols = shape
    for nbits, zt in VARIANTS:
        g = datagen.normal_with_outliers(rows * 17 + nbits, rows, cols, 0.01)
        q, _ = oracle.quantize(g, np.zeros_like(g, order="F"), nbits, zt, threads=8)
        prev = datagen.normal(rows * 19 + nbits, rows, cols, 1.0)
        Q = QuantizedMatrix(rows, cols, nbits, 0)
        Q.from_numpy(q)
        for mode in (5, 0):
            qz = MatrixQuantizerImpl.Create(0, False)
            qz._set_tuning(unq_mode=mode)
            for offset in (0, 1, 2, 3):
                say("decoder without LDS", rows, cols, nbits, "mode", mode, "offset", offset)
                for add in (False, True):
                    big = torch.full((rows * cols + 8,), 7.0, dtype=torch.float32, device="cuda:0")
                    big[offset:offset + rows * cols] = torch.from_numpy(np.ascontiguousarray(prev.reshape(-1, order="F"))).cuda()
                    Out = Matrix(rows, cols, 0, big[offset:offset + rows * cols])
                    qz.UnquantizeAsync(Q, Out, add=add)
                    qz.WaitUnquantizeAsyncDone()
                    parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)
                    assert bool((big[:offset] == 7.0).all()) and bool((big[offset + rows * cols:] == 7.0).all())


# ---- boundary behaviour ------------------------------------------------------------------------------


def test_out_of_place_residual_and_host_buffer(quantizer):
    """Distinct in/out residual buffers (first call of the v2 communicator, QuantizedDistributedCommunicator.h:246-252)
    and a host-resident packed matrix (the reference always stages through pinned host memory) give the same bytes."""
    rows, cols = 429, 37
    for nbits, zt in VARIANTS:
        say("out-of-place / host", nbits, zt)
        rep = parity.Report()
        make = lambda it: datagen.student_t(50 + it, rows, cols)
        run_chain(quantizer, rows, cols, nbits, zt, make, 2, rep, in_place=False)
        run_chain(quantizer, rows, cols, nbits, zt, make, 2, rep, host_q=True)


def test_column_slices_are_packed_matrices(quantizer):
    """ColumnSlice of gradient, residual and packed matrix addresses the same bytes as the whole
    (Source/Math/QuantizedMatrix.cpp:102-107) -- also exercises tiles that start at unaligned addresses."""
    rows, cols, nbits = 429, 23, 1
    g = datagen.normal(11, rows, cols)
    r = datagen.normal(12, rows, cols, 0.002)
    G, R, Q = Matrix.from_numpy(g), Matrix.from_numpy(r), QuantizedMatrix(rows, cols, nbits, 0)
    for start, n in [(0, 5), (5, 1), (6, 17)]:
        quantizer.QuantizeAsync(G.ColumnSlice(start, n), R.ColumnSlice(start, n), Q.ColumnSlice(start, n),
                                R.ColumnSlice(start, n), False)
    quantizer.WaitQuantizeAsyncDone()
    parity.check_quantize(g, r, Q.to_numpy(), R.to_numpy(), nbits, False)
    Out = Matrix(rows, cols)
    quantizer.UnquantizeAsync(Q.ColumnSlice(3, 11), Out.ColumnSlice(3, 11))
    quantizer.WaitUnquantizeAsyncDone()
    ref = oracle.unquantize(Q.to_numpy(), rows, cols, nbits)
    out = Out.to_numpy()
    assert parity.bits_equal(np.asfortranarray(out[:, 3:14]), np.asfortranarray(ref[:, 3:14]))
    assert not out[:, :3].any() and not out[:, 14:].any()


def test_special_columns(quantizer):
    """All-zero columns: lower = upper = 0, every valid bit 1, padding 0, residual 0 -- in both threshold modes."""
    z = np.zeros((70, 3), np.float32, order="F")
    for zt in (False, True):
        Q, r = gpu_quantize(quantizer, z, z.copy(order="F"), 1, zt)
        w = oracle.words(Q.to_numpy(), 70, 3, 1)
        assert [hex(x) for x in w[0]] == ["0xffffff", "0x7fffff", "0x7fffff"]
        lo, hi = oracle.headers(Q.to_numpy(), 70, 3, 1)
        assert not lo.any() and not hi.any() and not r.any()
    # the five-element column worked by hand
    g = np.asfortranarray(np.array([[0.1], [-0.2], [0.3], [-0.4], [0.05]], np.float32))
    Q, r = gpu_quantize(quantizer, g, np.zeros_like(g, order="F"), 1, False)
    lo, hi = oracle.headers(Q.to_numpy(), 5, 1, 1)
    assert abs(lo[0] + 0.462) < 1e-6 and abs(hi[0] - 0.402) < 1e-6
    assert oracle.words(Q.to_numpy(), 5, 1, 1)[0, 0] == 0b10101


@pytest.mark.parametrize("rows,cols", [(70, 9), (429, 8), (2048, 12), (1152, 10), (20000, 6)])
def test_non_finite_columns_stay_in_their_columns(rows, cols):
    """A NaN or an infinity in one column must not disturb any other column (columns are independent in the reference,
    Source/Math/MatrixQuantizerCPU.cpp:28-59), and the call must complete. What the poisoned column itself holds is
    not compared: the reference converts a NaN to an integer there, which C leaves undefined."""
    qz = MatrixQuantizerImpl.Create(0, False)
    g = datagen.normal(4242 + rows, rows, cols)
    r = datagen.normal(4243 + rows, rows, cols, 0.002)
    bad = [1, cols - 2, cols - 1]
    g[rows // 2, bad[0]] = np.nan
    g[0, bad[1]] = np.inf
    r[rows - 1, bad[2]] = -np.inf
    good = [j for j in range(cols) if j not in bad]
    for nbits, zt in VARIANTS:
        say("non-finite", rows, cols, nbits, zt)
        Q, r_out = gpu_quantize(qz, g, r, nbits, zt)
        q = Q.to_numpy()
        qcol = oracle.qcol_bytes(nbits, rows)
        q_good = np.concatenate([q[j * qcol:(j + 1) * qcol] for j in good])
        parity.check_quantize(np.asfortranarray(g[:, good]), np.asfortranarray(r[:, good]), q_good,
                              np.asfortranarray(r_out[:, good]), nbits, zt)
        Out = Matrix(rows, cols)
        qz.UnquantizeAsync(Q, Out)
        qz.WaitUnquantizeAsyncDone()
        out = Out.to_numpy()
        ref = oracle.unquantize(q_good, rows, len(good), nbits)
        assert parity.bits_equal(np.asfortranarray(out[:, good]), ref)
        if nbits < 32:
            # the poisoned values do not come back as ordinary numbers in the error feedback
            assert not np.isfinite(r_out[rows // 2, bad[0]]) and not np.isfinite(r_out[0, bad[1]])


def test_error_behaviour(quantizer):
    g = Matrix(8, 4)
    with pytest.raises(cntk_amd.QuantizerLogicError):  # dimension mismatch (asserts in the reference)
        quantizer.QuantizeAsync(g, Matrix(8, 5), QuantizedMatrix(8, 4, 1, 0), g, False)
    with pytest.raises(cntk_amd.QuantizerLogicError):  # packed size does not match the output matrix
        quantizer.UnquantizeAsync(QuantizedMatrix(8, 4, 1, 0), Matrix(8, 5))
    with pytest.raises(cntk_amd.QuantizerLogicError):
        quantizer.UnquantizeAsync(QuantizedMatrix(8, 4, 2, 0), Matrix(16, 4))
    with pytest.raises(cntk_amd.QuantizerLogicError):  # same dimensions, packed buffer of another bit width
        cntk_amd._check(cntk_amd.lib().cntkq_unquantize_async(quantizer._h, QuantizedMatrix(8, 4, 2, 0).Buffer(), 48, 0,
                                                              Matrix(8, 4).Data(), 8, 4, 8, 0))
    # empty matrices are silent no-ops
    quantizer.QuantizeAsync(Matrix(0, 4), Matrix(0, 4), QuantizedMatrix(0, 4, 1, 0), Matrix(0, 4), False)
    quantizer.UnquantizeAsync(QuantizedMatrix(5, 0, 1, 0), Matrix(5, 0))
    quantizer.WaitQuantizeAsyncDone()
    quantizer.WaitUnquantizeAsyncDone()
    assert quantizer.GetDeviceId() == 0


def test_wait_event_orders_the_quantizer_stream():
    """A dedicated-stream quantizer that is told to wait for the caller's event sees the data written before it."""
    rows, cols = 2048, 256
    q = MatrixQuantizerImpl.Create(0, True)
    side = torch.cuda.Stream()
    G, R, Q = Matrix(rows, cols), Matrix(rows, cols), QuantizedMatrix(rows, cols, 1, 0)
    g = datagen.normal(21, rows, cols)
    src = torch.from_numpy(g.reshape(-1, order="F").copy()).cuda()
    torch.cuda.synchronize()
    ev = torch.cuda.Event()
    with torch.cuda.stream(side):
        for _ in range(20):  # keep the side stream busy so that the copy really is pending when the quantizer is called
            G.data.mul_(1.0)
        G.data.copy_(src)
        ev.record(side)
    q.WaitEvent(ev.cuda_event)
    q.QuantizeAsync(G, R, Q, R, False)
    q.WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
    parity.check_quantize(g, np.zeros_like(g, order="F"), Q.to_numpy(), R.to_numpy(), 1, False)
    with pytest.raises(cntk_amd.QuantizerLogicError):
        q.WaitEvent(None)


def test_dedicated_stream_handles_share_one_stream():
    """Handles created with useAsync share one process-wide stream, so work issued through different quantizer
    objects is sequenced without waits -- callers rely on it (AllReduceDistGradAggregator.h:426-428)."""
    a = MatrixQuantizerImpl.Create(0, True)
    b = MatrixQuantizerImpl.Create(0, True)
    c = MatrixQuantizerImpl.Create(0, False)
    assert a.stream() == b.stream() and a.stream() is not None and a.stream() != c.stream()
    rows, cols = 2048, 64
    g = datagen.normal(3, rows, cols)
    G = Matrix.from_numpy(g)
    R, Out, Q = Matrix(rows, cols), Matrix(rows, cols), QuantizedMatrix(rows, cols, 1, 0)
    torch.cuda.synchronize()
    a.SynchronizeWithMainStream()
    a.QuantizeAsync(G, R, Q, R, False)
    b.UnquantizeAsync(Q, Out)  # no wait in between: same stream
    b.WaitUnquantizeAsyncDone()
    parity.check_quantize(g, np.zeros_like(g, order="F"), Q.to_numpy(), R.to_numpy(), 1, False)
    parity.check_unquantize(Q.to_numpy(), rows, cols, 1, Out.to_numpy())


@pytest.mark.parametrize("rows,cols,nbits", [(2048, 96, 1), (429, 40, 4), (20000, 8, 1)])
def test_calls_replayed_from_a_hip_graph(rows, cols, nbits):
    """QuantizeAsync, UnquantizeAsync and the fused stripe reduction issued on a capturing stream become graph nodes
    (no allocation, no host wait, no memset in them); every replay, with eager work and synchronisations in between,
    must give the bytes of the same calls issued eagerly on the same inputs, residuals carried."""
    k, owner = 3, 1
    qz = MatrixQuantizerImpl.Create(0, False)

    class Set:
        def __init__(self):
            self.G, self.R, self.Out = Matrix(rows, cols), Matrix(rows, cols), Matrix(rows, cols)
            self.Q = QuantizedMatrix(rows, cols, nbits, 0)
            self.S, self.Agg = Matrix(rows, cols), Matrix(rows, cols)
            self.stripes = [QuantizedMatrix(rows, cols, nbits, 0) for _ in range(k)]

        def run(self):
            qz.QuantizeAsync(self.G, self.R, self.Q, self.R, False)
            qz.UnquantizeAsync(self.Q, self.Out)
            qz.StripeReduceAsync(self.stripes, owner, self.S, self.stripes[owner], False, agg_out=self.Agg)

        def load(self, g, packed):
            self.G.data.copy_(g)
            for q, p in zip(self.stripes, packed):
                q.buffer.copy_(p)

    graphed, eager = Set(), Set()
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(80, nbits) + rows)

    def inputs():
        g = torch.randn(rows * cols, generator=gen, device="cuda:0") * 0.01
        packed = []
        for w in range(k):  # valid packed stripes: quantize random matrices
            T, Tr, Tq = Matrix(rows, cols, 0, torch.randn(rows * cols, generator=gen, device="cuda:0") * 0.01), Matrix(rows, cols), \
                QuantizedMatrix(rows, cols, nbits, 0)
            qz.QuantizeAsync(T, Tr, Tq, Tr, False)
            packed.append(Tq.buffer)
        torch.cuda.synchronize()
        return g, packed

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        qz.SetMainStream(torch.cuda.current_stream().cuda_stream)
        graphed.run()
    qz.SetMainStream(torch.cuda.current_stream().cuda_stream)
    for step in range(4):
        g, packed = inputs()
        graphed.load(g, packed)
        eager.load(g, packed)
        eager.run()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name in ("R", "Out", "S", "Agg"):
            assert torch.equal(getattr(graphed, name).data, getattr(eager, name).data), "replay %d: %s differs" % (step, name)
        assert torch.equal(graphed.Q.buffer, eager.Q.buffer), "replay %d: packed matrix differs" % step
        assert torch.equal(graphed.stripes[owner].buffer, eager.stripes[owner].buffer), "replay %d: reduced stripe differs" % step


@pytest.mark.parametrize("rows,cols,nbits", [(150001, 3, 1), (120000, 2, 4), (6000001, 1, 1)])
def test_strip_kernel_replayed_from_a_hip_graph(rows, cols, nbits):
    """Columns taller than any workgroup holds are cut into strips whose workgroups exchange partial sums through a
    scratch buffer that carries a launch count from one launch to the next. A captured launch must find that state
    right at every replay, with eager launches of the same and of another shape in between, and give the eager bytes.
    (The tallest case has more strips than the device holds at once: three launches, recorded as three kernel nodes.)"""
    qz = MatrixQuantizerImpl.Create(0, False)
    other_rows = 110000
    graphed = (Matrix(rows, cols), Matrix(rows, cols), QuantizedMatrix(rows, cols, nbits, 0))
    eager = (Matrix(rows, cols), Matrix(rows, cols), QuantizedMatrix(rows, cols, nbits, 0))
    other = (Matrix(other_rows, 5), Matrix(other_rows, 5), QuantizedMatrix(other_rows, 5, nbits, 0))
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        qz.SetMainStream(torch.cuda.current_stream().cuda_stream)
        qz.QuantizeAsync(graphed[0], graphed[1], graphed[2], graphed[1], False)
    qz.SetMainStream(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(81, nbits) + rows)
    rep = parity.Report()
    res = np.zeros((rows, cols), np.float32, order="F")
    for step in range(4):
        g = torch.randn(rows * cols, generator=gen, device="cuda:0") * 0.01
        graphed[0].data.copy_(g)
        eager[0].data.copy_(g)
        qz.QuantizeAsync(eager[0], eager[1], eager[2], eager[1], False)
        other[0].data.copy_(torch.randn(other_rows * 5, generator=gen, device="cuda:0"))
        qz.QuantizeAsync(other[0], other[1], other[2], other[1], False)  # another geometry on the same scratch buffer
        qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        qz.WaitQuantizeAsyncDone()  # reports a strip kernel whose workgroups gave up on each other, replays included
        assert torch.equal(graphed[1].data, eager[1].data), "replay %d: residual differs" % step
        assert torch.equal(graphed[2].buffer, eager[2].buffer), "replay %d: packed matrix differs" % step
        if step in (0, 3):
            parity.check_quantize(np.asfortranarray(g.cpu().numpy().reshape((rows, cols), order="F")), res, graphed[2].to_numpy(),
                                  graphed[1].to_numpy(), nbits, False, report=rep)
        res = graphed[1].to_numpy().copy(order="F")
    say("  ", rep)


def columns_untouched_or_right(g, r_in, q_before, q_after, r_after, nbits, zt):
    """What a strip launch may leave behind when some of its workgroups gave up: every column is either as it was (packed
    column and residual untouched) or quantized right. Returns the number of untouched columns."""
    rows, cols = g.shape
    qcol = q_after.size // cols
    untouched = 0
    for j in range(cols):
        qa, qb = q_after[j * qcol:(j + 1) * qcol], q_before[j * qcol:(j + 1) * qcol]
        if np.array_equal(qa, qb) and parity.bits_equal(r_after[:, j], r_in[:, j]):
            untouched += 1
            continue
        parity.check_quantize(np.asfortranarray(g[:, j:j + 1]), np.asfortranarray(r_in[:, j:j + 1]), qa.copy(),
                              np.asfortranarray(r_after[:, j:j + 1]), nbits, zt)
    return untouched


@pytest.mark.parametrize("host_q", [False, True], ids=["device_q", "host_q"])
def test_strip_kernel_reports_workgroups_that_give_up(host_q):
    """The workgroups of a column wait for each other's partial sums a bounded number of polls. With that number set to
    zero from the host every wait that does not find its record at the first look gives up: the kernel still runs to its
    end, the column is left as it was (packed column and in-place residual untouched, so the error feedback survives),
    the next wait reports the call as failed -- also where the packed matrix lives in host memory and the wait is for
    the copy -- and the handle goes on working afterwards."""
    # (7 strips per column: below 8 a strip looks for the others' records the moment it has published its own, and the
    # first one of a column to do so cannot find them)
    rows, cols = 110000, 4
    qz = MatrixQuantizerImpl.Create(0, False)
    g = datagen.normal(5, rows, cols)
    r0 = datagen.normal(6, rows, cols, 0.002)
    G, R = Matrix.from_numpy(g), Matrix.from_numpy(r0)
    Q = QuantizedMatrix(rows, cols, 1, cntk_amd.CPUDEVICE if host_q else 0)
    Q.buffer.fill_(0xA5)
    q_before = Q.to_numpy()
    torch.cuda.synchronize()
    qz._set_strip_spin_limit(0)
    qz.QuantizeAsync(G, R, Q, R, False)
    with pytest.raises(cntk_amd.QuantizerError, match="left as they were"):
        qz.WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
    if not host_q:  # (the copy to the host takes the staging buffer's bytes, which nothing preset)
        n = columns_untouched_or_right(g, r0, q_before, Q.to_numpy(), R.to_numpy(), 1, False)
        say("   columns left untouched: %d of %d" % (n, cols))
        assert n >= 1
    else:
        r_after = R.to_numpy()
        assert any(parity.bits_equal(r_after[:, j], r0[:, j]) for j in range(cols))
    qz._set_strip_spin_limit(1 << 17)
    R.data.zero_()
    qz.QuantizeAsync(G, R, Q, R, False)
    qz.WaitQuantizeAsyncDone()
    parity.check_quantize(g, np.zeros_like(g, order="F"), Q.to_numpy(), R.to_numpy(), 1, False)


def test_strip_kernel_beside_other_work_on_the_device():
    """The strips of a column wait for each other, which needs all of them resident together. Here the device is kept busy
    by long fill and copy kernels on another stream while tall matrices are quantized on the quantizer's dedicated stream:
    whatever the scheduler does, every kernel ends (the wait is bounded), and the outcome is the right bytes or a reported
    error with every column either untouched or right -- never silently wrong."""
    rows, cols, nbits = 200000, 96, 1
    qz = MatrixQuantizerImpl.Create(0, True)
    g = datagen.normal(9, rows, cols)
    r0 = datagen.normal(10, rows, cols, 0.002)
    G = Matrix.from_numpy(g)
    side = torch.cuda.Stream()
    big = torch.empty(1 << 30, dtype=torch.float32, device="cuda:0")  # 4 GB: a fill takes about a millisecond
    big2 = torch.empty_like(big)
    reported = 0
    for rep in range(3):
        R = Matrix.from_numpy(r0)
        Q = QuantizedMatrix(rows, cols, nbits, 0)
        Q.buffer.fill_(0xA5)
        q_before = Q.to_numpy()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            for i in range(6):
                big.fill_(float(i))
                big2.copy_(big)
        qz.QuantizeAsync(G, R, Q, R, False)
        try:
            qz.WaitQuantizeAsyncDone()
            failed = False
        except cntk_amd.QuantizerError:
            failed = True
            reported += 1
        torch.cuda.synchronize()
        if failed:
            columns_untouched_or_right(g, r0, q_before, Q.to_numpy(), R.to_numpy(), nbits, False)
        else:
            parity.check_quantize(g, r0, Q.to_numpy(), R.to_numpy(), nbits, False)
    say("   launches that reported strips giving up: %d of 3" % reported)
    # told that its tall columns must never wait, the same handle beside the same work cannot fail that way
    qz.SetTallColumnsNeverWait(True)
    for rep in range(2):
        R = Matrix.from_numpy(r0)
        Q = QuantizedMatrix(rows, cols, nbits, 0)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            for i in range(6):
                big.fill_(float(i))
                big2.copy_(big)
        qz.QuantizeAsync(G, R, Q, R, False)
        qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        parity.check_quantize(g, r0, Q.to_numpy(), R.to_numpy(), nbits, False)


def test_strip_scratch_outgrown_after_a_recorded_launch():
    """A recorded strip launch has the scratch buffer's addresses in its graph node. A later, larger launch makes the handle
    take a larger buffer; the old one must stay alive for the replays (it is freed with the handle): replays after the
    growth still give the eager bytes."""
    rows, cols, nbits = 150001, 3, 1
    wide_rows, wide_cols = 110000, 2400  # 14 strips x 2400 columns: more records than the starting buffer holds
    qz = MatrixQuantizerImpl.Create(0, False)
    graphed = (Matrix(rows, cols), Matrix(rows, cols), QuantizedMatrix(rows, cols, nbits, 0))
    eager = (Matrix(rows, cols), Matrix(rows, cols), QuantizedMatrix(rows, cols, nbits, 0))
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        qz.SetMainStream(torch.cuda.current_stream().cuda_stream)
        qz.QuantizeAsync(graphed[0], graphed[1], graphed[2], graphed[1], False)
    qz.SetMainStream(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(4711)
    wide = (Matrix(wide_rows, wide_cols), Matrix(wide_rows, wide_cols), QuantizedMatrix(wide_rows, wide_cols, nbits, 0))
    wide[0].data.copy_(torch.randn(wide_rows * wide_cols, generator=gen, device="cuda:0") * 0.01)
    for step in range(3):
        g = torch.randn(rows * cols, generator=gen, device="cuda:0") * 0.01
        graphed[0].data.copy_(g)
        eager[0].data.copy_(g)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        if step == 0:
            say("   the wide launch that outgrows the buffer")
            qz.QuantizeAsync(wide[0], wide[1], wide[2], wide[1], False)
            qz.WaitQuantizeAsyncDone()
            torch.cuda.synchronize()
            # the conservation law on the wide matrix: g + r_in (zero) == unquantize(q) + r_out
            back = Matrix(wide_rows, wide_cols)
            qz.UnquantizeAsync(wide[2], back)
            qz.WaitUnquantizeAsyncDone()
            torch.cuda.synchronize()
            assert torch.equal(back.data + wide[1].data, wide[0].data) or \
                float((back.data + wide[1].data - wide[0].data).abs().max()) <= 1e-6
        qz.QuantizeAsync(eager[0], eager[1], eager[2], eager[1], False)
        qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        assert torch.equal(graphed[1].data, eager[1].data), "replay %d: residual differs" % step
        assert torch.equal(graphed[2].buffer, eager[2].buffer), "replay %d: packed matrix differs" % step


def test_strip_kernel_across_a_stream_change():
    """Strip launches of one handle share its scratch buffer, so a launch on a new main stream must wait for the last one
    on the old stream: two tall matrices quantized back to back on two streams, several times over, both right."""
    rows, cols = 140000, 24
    qz = MatrixQuantizerImpl.Create(0, False)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    gs = [datagen.normal(7 + i, rows, cols) for i in range(2)]
    G = [Matrix.from_numpy(g) for g in gs]
    R = [Matrix(rows, cols) for _ in range(2)]
    Q = [QuantizedMatrix(rows, cols, 1, 0) for _ in range(2)]
    torch.cuda.synchronize()
    for rep in range(3):
        for i in range(2):
            R[i].data.zero_()
        torch.cuda.synchronize()
        for i in range(2):
            qz.SetMainStream(streams[i].cuda_stream)
            qz.QuantizeAsync(G[i], R[i], Q[i], R[i], False)
        torch.cuda.synchronize()
        qz.WaitQuantizeAsyncDone()
        for i in range(2):
            parity.check_quantize(gs[i], np.zeros_like(gs[i], order="F"), Q[i].to_numpy(), R[i].to_numpy(), 1, False)


def test_force_sync_mode_waits_inside_the_calls():
    """MatrixQuantizerGPU(deviceId, useDedicatedComputeStream, forceSync = true) (Source/Math/MatrixQuantizerGPU.h:20,
    Source/Math/MatrixQuantizerGPU.cu:118-122, 137-141, 237-240): every call has finished its own work, kernel and copy to
    the host, when it returns -- no Wait call needed before the results are read."""
    rows, cols = 2048, 512
    g = datagen.normal(17, rows, cols)
    for dedicated in (False, True):
        qz = MatrixQuantizerImpl(0, dedicated, force_sync=True)
        G, R = Matrix.from_numpy(g), Matrix(rows, cols)
        Qhost = QuantizedMatrix(rows, cols, 1, cntk_amd.CPUDEVICE)
        torch.cuda.synchronize()
        qz.QuantizeAsync(G, R, Qhost, R, False)
        # no WaitQuantizeAsyncDone: the packed matrix is in host memory and the residual written already
        q_now = Qhost.to_numpy().copy()
        stream = torch.cuda.ExternalStream(qz.stream()) if qz.stream() else torch.cuda.current_stream()
        assert stream.query(), "the work stream still has work after a call in forceSync mode"
        parity.check_quantize(g, np.zeros_like(g, order="F"), q_now, R.to_numpy(), 1, False)
        qz.WaitQuantizeAsyncDone()
        assert np.array_equal(q_now, Qhost.to_numpy())
        Out = Matrix(rows, cols)
        qz.UnquantizeAsync(Qhost, Out)
        # the call has waited for its kernel too (RecordQuantizeCompleteEvent at the end of UnquantizeAsync)
        assert stream.query(), "the work stream still has work after UnquantizeAsync in forceSync mode"
        out_now = Out.to_numpy().copy()
        qz.WaitUnquantizeAsyncDone()
        parity.check_unquantize(q_now, rows, cols, 1, out_now)


OFFSET_SHAPES = [(147, 300), (512, 200), (1000, 90), (2048, 40), (2049, 37), (4100, 24), (9304, 16), (20001, 9), (50257, 5)]


@pytest.mark.parametrize("shape", OFFSET_SHAPES, ids=["%dx%d" % s for s in OFFSET_SHAPES])
def test_matrices_at_different_offsets_within_16_bytes(shape):
    """Gradient, residual and residual output that start at different 4-byte offsets within 16 bytes (slices of larger
    buffers, the gradient views of a flat communication bucket beside separately allocated residuals): the kernels read and
    write such matrices in 16-byte accesses at whatever alignment that leaves them -- the tile kernels up to 2048 rows, the
    register kernels with edge elements above (their aligned pieces are the residual input's) -- and the tile decoder
    writes to an output at any offset. Checked against the oracle; nothing may be written outside the matrices."""
    rows, cols = shape
    qz = MatrixQuantizerImpl.Create(0, False)
    rep = parity.Report()

    def place(a, off):
        buf = torch.zeros(a.size + 64, dtype=torch.float32, device="cuda:0")
        buf[off:off + a.size] = torch.from_numpy(a.reshape(-1, order="F").copy()).cuda()
        return Matrix(a.shape[0], a.shape[1], 0, buf[off:off + a.size]), buf

    n = 0
    for offs in ((1, 0, 0), (0, 2, 0), (1, 2, 3), (3, 3, 1), (5, 7, 6)):
        for nbits, zt in ((1, False), (1, True), (4, False)):
            n += 1
            say("offsets", shape, offs, "nbits", nbits, "zeroThr", zt)
            g = datagen.normal_with_outliers(100 * rows + n, rows, cols, 0.01)
            r = datagen.normal(200 * rows + n, rows, cols, 0.002)
            G, _gbuf = place(g, offs[0])
            R, rbuf = place(r, offs[1])
            in_place = n % 2 == 0
            Rout, obuf = (R, rbuf) if in_place else place(np.zeros_like(g, order="F"), offs[2])
            Q = QuantizedMatrix(rows, cols, nbits, 0)
            qz.QuantizeAsync(G, R, Q, Rout, zt)
            qz.WaitQuantizeAsyncDone()
            torch.cuda.synchronize()
            q_gpu = Q.to_numpy()
            parity.check_quantize(g, r, q_gpu, Rout.to_numpy(), nbits, zt, report=rep)
            off_o = offs[1] if in_place else offs[2]
            assert float(obuf[:off_o].abs().sum()) == 0.0 and float(obuf[off_o + rows * cols:].abs().sum()) == 0.0
            prev = datagen.normal(300 * rows + n, rows, cols, 1.0)
            add = n % 3 == 0
            Out, outbuf = place(prev, offs[2])
            qz.UnquantizeAsync(Q, Out, add=add)
            qz.WaitUnquantizeAsyncDone()
            torch.cuda.synchronize()
            parity.check_unquantize(q_gpu, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)
            assert float(outbuf[:offs[2]].abs().sum()) == 0.0 and float(outbuf[offs[2] + rows * cols:].abs().sum()) == 0.0
    say("  ", rep)


@pytest.mark.parametrize("shape", [(1000, 60), (4100, 24), (9304, 16), (20001, 9)], ids=lambda s: "%dx%d" % s)
def test_double_matrices_at_different_offsets_within_16_bytes(shape):
    """The same for doubles: gradient, residual and residual output 8 bytes apart in their 16-byte phase."""
    rows, cols = shape
    qz = MatrixQuantizerImpl.Create(0, False)
    rep = parity.Report()

    def place(a, off):
        buf = torch.zeros(a.size + 64, dtype=torch.float64, device="cuda:0")
        buf[off:off + a.size] = torch.from_numpy(a.reshape(-1, order="F").copy()).cuda()
        return Matrix(a.shape[0], a.shape[1], 0, buf[off:off + a.size], dtype=torch.float64), buf

    n = 0
    for offs in ((1, 0, 0), (0, 1, 0), (1, 0, 1), (3, 2, 5)):
        for nbits, zt in ((1, False), (4, False)):
            n += 1
            say("double offsets", shape, offs, "nbits", nbits, "zeroThr", zt)
            g = datagen.normal_with_outliers(100 * rows + n, rows, cols, 0.01, dtype=np.float64)
            r = datagen.normal(200 * rows + n, rows, cols, 0.002, dtype=np.float64)
            G, _gbuf = place(g, offs[0])
            R, rbuf = place(r, offs[1])
            in_place = n % 2 == 0
            Rout, obuf = (R, rbuf) if in_place else place(np.zeros_like(g, order="F"), offs[2])
            Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
            qz.QuantizeAsync(G, R, Q, Rout, zt)
            qz.WaitQuantizeAsyncDone()
            torch.cuda.synchronize()
            q_gpu = Q.to_numpy()
            parity.check_quantize(g, r, q_gpu, Rout.to_numpy(), nbits, zt, report=rep)
            off_o = offs[1] if in_place else offs[2]
            assert float(obuf[:off_o].abs().sum()) == 0.0 and float(obuf[off_o + rows * cols:].abs().sum()) == 0.0
            prev = datagen.normal(300 * rows + n, rows, cols, 1.0, dtype=np.float64)
            Out, outbuf = place(prev, offs[2])
            qz.UnquantizeAsync(Q, Out, add=False)
            qz.WaitUnquantizeAsyncDone()
            torch.cuda.synchronize()
            parity.check_unquantize(q_gpu, rows, cols, nbits, Out.to_numpy())
            assert float(outbuf[:offs[2]].abs().sum()) == 0.0 and float(outbuf[offs[2] + rows * cols:].abs().sum()) == 0.0
    say("  ", rep)
