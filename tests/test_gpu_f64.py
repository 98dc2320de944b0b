"""Parity of the double-precision instantiation (MatrixQuantizerImpl<double>, 64-bit QWords) against the CPU oracle,
through the C ABI (the _f64 entry points). Needs an MI355X.

Same structure as the float tests: the reference unit test's shapes (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp
runs every case for double as well, :420-431), every bit width 1..64, both 1-bit threshold modes, teacher-forced
chains with carried residual, every kernel path, the unquantize variants, the fused stripe reduction.
Tolerances: bit-exact under the GPU's own headers; headers within 1e-12 of the column scale, codes different only
within 1e-13 of a threshold, other residuals within 1e-12 (both sides sum in double).
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

F64 = np.float64
VARIANTS = [(1, False), (1, True), (2, False), (4, False), (8, False), (16, False), (32, False), (64, False)]
PATH_AUTO, PATH_TILE, PATH_TALL, PATH_COL, PATH_REG, PATH_REGS, PATH_STRIP, PATH_STRIP_PASSES = 0, 1, 2, 3, 4, 5, 6, 7


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def zeros(rows, cols):
    return np.zeros((rows, cols), F64, order="F")


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
    assert G.dtype == torch.float64
    Rout = R if in_place else Matrix(rows, cols, dtype=torch.float64)
    Q = QuantizedMatrix(rows, cols, nbits, cntk_amd.CPUDEVICE if host_q else 0, dtype=torch.float64)
    qz.QuantizeAsync(G, R, Q, Rout, zt)
    qz.WaitQuantizeAsyncDone()
    if not host_q:
        torch.cuda.synchronize()
    return Q, Rout.to_numpy()


def run_chain(qz, rows, cols, nbits, zt, make_input, iterations, report, in_place=True, host_q=False):
    """Teacher-forced chain: the oracle's residual feeds both sides at every step."""
    res_o, out_o = zeros(rows, cols), zeros(rows, cols)
    Out = Matrix(rows, cols, dtype=torch.float64)
    for it in range(iterations):
        g = make_input(it)
        assert g.dtype == F64
        Q, r_gpu = gpu_quantize(qz, g, res_o, nbits, zt, in_place=in_place, host_q=host_q)
        q_gpu = Q.to_numpy()
        parity.check_quantize(g, res_o, q_gpu, r_gpu, nbits, zt, report=report)
        prev = Out.to_numpy()
        qz.UnquantizeAsync(Q, Out, add=(it > 0))
        qz.WaitUnquantizeAsyncDone()
        parity.check_unquantize(q_gpu, rows, cols, nbits, Out.to_numpy(), prev_out=prev if it > 0 else None)
        q_or, _ = oracle.quantize(g, res_o, nbits, zt, r_out=res_o, threads=8)
        oracle.unquantize(q_or, rows, cols, nbits, out=out_o, add=(it > 0), threads=8)
        Out = Matrix.from_numpy(out_o)


UNIT_SHAPES = [
    (25, 13, -1.0, 1.0, 2015), (25, 13, -0.005, 0.005, 2115), (13, 25, -0.00001, 0.00001, 2215),
    (13, 25, -10.0, 10.0, 2315), (25, 13, -1.0, 2.05, 2415), (489, 1, -0.5, 0.5, 2515), (1, 135, -0.5, 0.5, 2615),
    (89, 23, -0.5, 0.5, 2715), (15, 35, -0.5, 0.5, 2815), (100, 50, -0.5, 0.5, 2915), (737, 373, -0.5, 0.5, 2915),
]


@pytest.mark.parametrize("shape", UNIT_SHAPES, ids=["%dx%d_%d" % (s[0], s[1], s[4]) for s in UNIT_SHAPES])
def test_reference_unit_shapes_f64(quantizer, shape):
    rows, cols, lo, hi, seed = shape
    rep = parity.Report()
    for nbits, zt in VARIANTS:
        say("f64 unit shape", shape, "nbits", nbits, "zeroThr", zt)
        run_chain(quantizer, rows, cols, nbits, zt, lambda it: datagen.uniform(seed + it, rows, cols, lo, hi, dtype=F64), 3, rep)
    say("  ", rep)


def test_golden_vectors_f64(quantizer):
    """Against the packed bytes the reference's own headers wrote for double (tests/golden/unit_shapes_f64.npz): the
    oracle reproduces them byte for byte, and the GPU result is held to the parity rules against that same result.
    Byte-identical GPU output is counted, not required: the sums behind a header are taken in another order."""
    import os
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "unit_shapes_f64.npz"))
    from golden.make_golden import UNIT_SHAPES as GOLD_SHAPES
    same = total = 0
    for si, (rows, cols, lo, hi, seed) in enumerate(GOLD_SHAPES):
        g = np.asfortranarray(gold["s%d_inputs" % si][0].reshape((rows, cols), order="F"))
        for nbits, zt in VARIANTS:
            Q, r = gpu_quantize(quantizer, g, zeros(rows, cols), nbits, zt)
            ref_q = gold["s%d_b%d_z%d_q" % (si, nbits, int(zt))][0]
            assert np.array_equal(oracle.quantize(g, zeros(rows, cols), nbits, zt)[0], ref_q)
            parity.check_quantize(g, zeros(rows, cols), Q.to_numpy(), r, nbits, zt)
            total += 1
            same += int(np.array_equal(Q.to_numpy(), ref_q))
    say("f64 golden: %d of %d packed matrices byte-identical to the reference's" % (same, total))
    assert same > 0


def test_free_running_conservation_f64(quantizer):
    rows, cols, lo, hi = 100, 50, -0.5, 0.5
    for nbits, zt in VARIANTS:
        R, Out = Matrix(rows, cols, dtype=torch.float64), Matrix(rows, cols, dtype=torch.float64)
        for it in range(4):
            g = datagen.uniform(2915 + it, rows, cols, lo, hi, dtype=F64)
            r_in, prev = R.to_numpy(), Out.to_numpy()
            Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
            quantizer.QuantizeAsync(Matrix.from_numpy(g), R, Q, R, zt)
            quantizer.WaitQuantizeAsyncDone()
            quantizer.UnquantizeAsync(Q, Out, add=(it > 0))
            quantizer.WaitUnquantizeAsyncDone()
            parity.conservation(g, r_in, prev, R.to_numpy(), Out.to_numpy(), 1e-14)


PATH_CASES = [
    # rows, cols, path, tile_gs
    (1, 1, PATH_TILE, 0), (3, 70, PATH_TILE, 0), (31, 5, PATH_TILE, 8), (65, 67, PATH_TILE, 0), (64, 64, PATH_TILE, 16),
    (147, 64, PATH_TILE, 0), (429, 37, PATH_TILE, 0), (429, 37, PATH_TILE, 64), (1023, 9, PATH_TILE, 0),
    (2048, 19, PATH_TILE, 0), (2048, 19, PATH_TILE, 256), (4608, 3, PATH_TILE, 0), (7168, 2, PATH_TILE, 0),
    (1, 5, PATH_TALL, 0), (70, 3, PATH_TALL, 0), (1025, 3, PATH_TALL, 0), (20001, 2, PATH_TALL, 0), (9304, 2, PATH_AUTO, 0),
    # one workgroup of 1024 threads per column, the column in registers: even heights; the automatic choice above 7168 rows
    (4, 3, PATH_REG, 0), (70, 3, PATH_REG, 0), (1000, 5, PATH_REG, 0), (7170, 3, PATH_REG, 0), (9304, 3, PATH_REG, 0),
    (20000, 3, PATH_AUTO, 0), (32770, 2, PATH_REG, 0), (51200, 1, PATH_AUTO, 0), (51202, 1, PATH_AUTO, 0),
    (5, 3, PATH_REG, 0), (1001, 3, PATH_REG, 0), (9305, 3, PATH_AUTO, 0), (20001, 2, PATH_AUTO, 0), (50257, 1, PATH_AUTO, 0),
    # one workgroup of 256 threads per column, the column in registers element by element: 1025 to 6144 rows
    (1025, 3, PATH_REGS, 0), (2048, 5, PATH_REGS, 0), (2049, 3, PATH_AUTO, 0), (3073, 3, PATH_REGS, 0), (4096, 3, PATH_AUTO, 0),
    (4991, 2, PATH_AUTO, 0), (5120, 2, PATH_REGS, 0), (4099, 2, PATH_REGS, 0), (6144, 2, PATH_AUTO, 0), (6143, 2, PATH_AUTO, 0),
    (6146, 2, PATH_AUTO, 0),
    # several workgroups per column, a strip of QWords each: any height, one strip or many, full or ragged; the automatic
    # choice above what one workgroup's registers hold (51184 rows), on one die or, from 33 strips on, on all of them
    (1, 3, PATH_STRIP, 0), (37, 5, PATH_STRIP, 0), (1000, 3, PATH_STRIP, 0), (4096, 3, PATH_STRIP, 0), (4097, 2, PATH_STRIP, 0),
    (9304, 3, PATH_STRIP, 0), (16385, 2, PATH_STRIP, 0), (50257, 3, PATH_STRIP, 0), (51201, 2, PATH_AUTO, 0), (102401, 2, PATH_AUTO, 0),
    (200000, 3, PATH_AUTO, 0), (262147, 2, PATH_STRIP, 0), (330001, 1, PATH_AUTO, 0), (400000, 9, PATH_STRIP, 0),
    # the strips in two or three launches: any height of two strips or more; the automatic choice above what the device holds
    (9304, 3, PATH_STRIP_PASSES, 0), (51201, 2, PATH_STRIP_PASSES, 0), (3000001, 1, PATH_AUTO, 0),
]


def strip_words_f64(nbits):
    """QWords of a double column that one strip holds."""
    return {1: 128, 2: 256, 4: 512}.get(nbits, 1024)


@pytest.mark.parametrize("case", PATH_CASES, ids=["%dx%d_p%d_g%d" % c for c in PATH_CASES])
def test_kernel_paths_f64(case):
    rows, cols, path, gs = case
    qz = MatrixQuantizerImpl.Create(0, False)
    qz._set_tuning(quantize_path=path, tile_gs=gs)
    rep = parity.Report()
    for nbits, zt in VARIANTS:
        say("f64 path case", case, "nbits", nbits, "zeroThr", zt)
        if (path == PATH_REGS and nbits == 64) or \
                (path == PATH_REG and (nbits == 64 or (50 + 2 * oracle.qwords_per_col(rows, nbits, F64)) * 8 > 163840)) or \
                (path == PATH_STRIP and (nbits == 64 or oracle.qwords_per_col(rows, nbits, F64) >
                                         qz._strip_max_strips(nbits, zt, torch.float64) * strip_words_f64(nbits))) or \
                (path == PATH_STRIP_PASSES and (nbits == 64 or oracle.qwords_per_col(rows, nbits, F64) <= strip_words_f64(nbits))):
            # whole-QWord codes, columns whose QWords (twice, as the stripe reduction keeps them) exceed the LDS of a compute unit
            # and columns of more strips than the device holds at once are refused when forced
            with pytest.raises(cntk_amd.QuantizerLogicError):
                gpu_quantize(qz, datagen.normal(1, rows, cols, dtype=F64), zeros(rows, cols), nbits, zt)
            continue

        def make(it):
            a = datagen.normal_with_outliers(1000 * rows + cols + it, rows, cols, 0.01, dtype=F64) + 0.004 * (it % 2)
            a = np.asfortranarray(a)
            if cols > 1:
                a[:, cols // 2] = 0.0
            return a
        run_chain(qz, rows, cols, nbits, zt, make, 2, rep)
    say("  ", rep)


@pytest.mark.parametrize("rows,cols", [(1025, 7), (2048, 9), (3000, 5), (4097, 4), (4990, 3), (5120, 3), (6144, 2)])
def test_element_register_kernel_gives_the_tile_kernels_bytes_f64(rows, cols):
    """The 256-thread register kernel adds in the order of the one-column tile, so both give the same bytes (which is what
    lets the tile stripe reduction reproduce a call sequence that quantizes with either); matrices 8 bytes off a 16-byte
    boundary included."""
    qa, qb = MatrixQuantizerImpl.Create(0, False), MatrixQuantizerImpl.Create(0, False)
    qa._set_tuning(quantize_path=PATH_TILE)
    qb._set_tuning(quantize_path=PATH_REGS)
    for nbits, zt in VARIANTS:
        if nbits == 64:
            continue
        for off in (0, 1):
            say("tile against element registers", rows, cols, nbits, zt, "offset", off)
            g = datagen.normal_with_outliers(17 * rows + nbits + off, rows, cols, 0.01, dtype=F64)
            r = datagen.normal(19 * rows + nbits + off, rows, cols, 0.003, dtype=F64)
            outs = []
            for qz in (qa, qb):
                n = rows * cols
                gbuf = torch.zeros(n + 2, dtype=torch.float64, device="cuda:0")
                rbuf = torch.zeros(n + 2, dtype=torch.float64, device="cuda:0")
                gbuf[off:off + n].copy_(torch.from_numpy(np.ascontiguousarray(g.T).reshape(-1)))
                rbuf[off:off + n].copy_(torch.from_numpy(np.ascontiguousarray(r.T).reshape(-1)))
                G, R = Matrix(rows, cols, 0, gbuf[off:off + n]), Matrix(rows, cols, 0, rbuf[off:off + n])
                Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
                qz.QuantizeAsync(G, R, Q, R, zt)
                qz.WaitQuantizeAsyncDone()
                torch.cuda.synchronize()
                outs.append((Q.to_numpy(), R.to_numpy()))
            assert np.array_equal(outs[0][0], outs[1][0]), ("packed", rows, cols, nbits, zt, off)
            assert parity.bits_equal(outs[0][1], outs[1][1]), ("residual", rows, cols, nbits, zt, off)


def test_unsupported_paths_are_refused_f64():
    qz = MatrixQuantizerImpl.Create(0, False)
    qz._set_tuning(quantize_path=PATH_COL)  # exists for float only
    with pytest.raises(cntk_amd.QuantizerLogicError):
        gpu_quantize(qz, datagen.normal(1, 2048, 4, dtype=F64), zeros(2048, 4), 1, False)
    qz._set_tuning(quantize_path=PATH_TILE)
    with pytest.raises(cntk_amd.QuantizerLogicError):
        gpu_quantize(qz, datagen.normal(1, 7169, 2, dtype=F64), zeros(7169, 2), 1, False)
    qz._set_tuning(quantize_path=PATH_REGS)  # 1025 to 6144 rows
    for rows in (1024, 6145):
        with pytest.raises(cntk_amd.QuantizerLogicError):
            gpu_quantize(qz, datagen.normal(1, rows, 2, dtype=F64), zeros(rows, 2), 1, False)


def test_unquantize_variants_f64(quantizer):
    for rows, cols in [(5, 3), (37, 2), (128, 9), (429, 5), (2048, 6), (4100, 2), (1001, 5), (100000, 2)]:
        for nbits, zt in VARIANTS:
            g = datagen.normal(rows * 7 + nbits, rows, cols, dtype=F64)
            q, _ = oracle.quantize(g, zeros(rows, cols), nbits, zt)
            prev = datagen.normal(rows * 9 + nbits, rows, cols, 1.0, dtype=F64)
            for slots in (0, 1, 3, 64):
                for scalar in (0, 1):
                    say("f64 unquantize", rows, cols, nbits, "slots", slots, "scalar", scalar)
                    qz = MatrixQuantizerImpl.Create(0, False)
                    qz._set_tuning(unq_slots=slots, unq_mode=scalar)
                    Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
                    Q.from_numpy(q)
                    for add in (False, True):
                        Out = Matrix.from_numpy(prev)
                        qz.UnquantizeAsync(Q, Out, add=add)
                        qz.WaitUnquantizeAsyncDone()
                        parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)


DECODER_SHAPES_F64 = [(1, 1), (1, 9), (3, 5), (31, 13), (64, 100), (147, 64), (429, 37), (512, 24), (1000, 9), (1001, 5), (2048, 7),
                      (4095, 3), (4096, 2), (4097, 3), (9304, 3), (9305, 2), (16383, 2), (20000, 2), (20001, 3), (50257, 2), (100000, 2),
                      (2, 3), (128, 4099), (576, 50), (1152, 33), (1536, 9)]


@pytest.mark.parametrize("shape", DECODER_SHAPES_F64, ids=["%dx%d" % s for s in DECODER_SHAPES_F64])
def test_tile_and_row_major_decoders_f64(shape):
    """The decoders for columns whose QWord-major stores would not be whole lines: several short columns per workgroup
    (mode 2), row-major with the packed column in LDS (mode 4), row-major with every thread fetching its own QWords
    (mode 5), and the automatic choice; add and overwrite; bit-exact."""
    rows, cols = shape
    for nbits, zt in VARIANTS:
        g = datagen.normal_with_outliers(rows * 11 + nbits, rows, cols, 0.01, dtype=F64)
        q, _ = oracle.quantize(g, zeros(rows, cols), nbits, zt)
        prev = datagen.normal(rows * 13 + nbits, rows, cols, 1.0, dtype=F64)
        for mode in (2, 4, 5, 6, 0):
            say("f64 decoder", rows, cols, nbits, "mode", mode)
            qz = MatrixQuantizerImpl.Create(0, False)
            qz._set_tuning(unq_mode=mode)
            Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
            Q.from_numpy(q)
            for add in (False, True):
                Out = Matrix.from_numpy(prev)
                qz.UnquantizeAsync(Q, Out, add=add)
                qz.WaitUnquantizeAsyncDone()
                parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)
        # output 8 bytes off a 16-byte boundary: another decoder serves it
        big = torch.zeros(rows * cols + 2, dtype=torch.float64, device="cuda:0")
        Out = Matrix(rows, cols, 0, big[1:1 + rows * cols], dtype=torch.float64)
        qz.UnquantizeAsync(Q, Out)
        qz.WaitUnquantizeAsyncDone()
        parity.check_unquantize(q, rows, cols, nbits, Out.to_numpy())
        assert float(big[0]) == 0.0 and float(big[-1]) == 0.0


def test_out_of_place_host_buffer_and_slices_f64(quantizer):
    rows, cols = 429, 37
    for nbits, zt in VARIANTS:
        rep = parity.Report()
        make = lambda it: datagen.student_t(50 + it, rows, cols, dtype=F64)
        run_chain(quantizer, rows, cols, nbits, zt, make, 2, rep, in_place=False)
        run_chain(quantizer, rows, cols, nbits, zt, make, 2, rep, host_q=True)
    # column slices of gradient, residual and packed matrix
    rows, cols, nbits = 429, 23, 1
    g, r = datagen.normal(11, rows, cols, dtype=F64), datagen.normal(12, rows, cols, 0.002, dtype=F64)
    G, R, Q = Matrix.from_numpy(g), Matrix.from_numpy(r), QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
    for start, n in [(0, 5), (5, 1), (6, 17)]:
        quantizer.QuantizeAsync(G.ColumnSlice(start, n), R.ColumnSlice(start, n), Q.ColumnSlice(start, n),
                                R.ColumnSlice(start, n), False)
    quantizer.WaitQuantizeAsyncDone()
    parity.check_quantize(g, r, Q.to_numpy(), R.to_numpy(), nbits, False)
    Out = Matrix(rows, cols, dtype=torch.float64)
    quantizer.UnquantizeAsync(Q.ColumnSlice(3, 11), Out.ColumnSlice(3, 11))
    quantizer.WaitUnquantizeAsyncDone()
    ref = oracle.unquantize(Q.to_numpy(), rows, cols, nbits, dtype=F64)
    out = Out.to_numpy()
    assert parity.bits_equal(np.asfortranarray(out[:, 3:14]), np.asfortranarray(ref[:, 3:14]))
    assert not out[:, :3].any() and not out[:, 14:].any()


def test_special_columns_and_errors_f64(quantizer):
    z = zeros(70, 3)
    for zt in (False, True):
        Q, r = gpu_quantize(quantizer, z, z.copy(order="F"), 1, zt)
        w = oracle.words(Q.to_numpy(), 70, 3, 1, dtype=F64)  # 70 rows -> 2 QWords: 35 valid bits each
        assert [hex(int(x)) for x in w[0]] == ["0x7ffffffff", "0x7ffffffff"]
        lo, hi = oracle.headers(Q.to_numpy(), 70, 3, 1, dtype=F64)
        assert not lo.any() and not hi.any() and not r.any()
    g = np.asfortranarray(np.array([[0.1], [-0.2], [0.3], [-0.4], [0.05]], F64))
    Q, r = gpu_quantize(quantizer, g, zeros(5, 1), 1, False)
    lo, hi = oracle.headers(Q.to_numpy(), 5, 1, 1, dtype=F64)
    assert abs(lo[0] + 0.462) < 1e-15 and abs(hi[0] - 0.402) < 1e-15
    assert int(oracle.words(Q.to_numpy(), 5, 1, 1, dtype=F64)[0, 0]) == 0b10101
    # element types may not be mixed; 64 bits does not exist for float
    with pytest.raises(cntk_amd.QuantizerLogicError):
        quantizer.QuantizeAsync(Matrix(8, 4, dtype=torch.float64), Matrix(8, 4), QuantizedMatrix(8, 4, 1, 0, dtype=torch.float64),
                                Matrix(8, 4, dtype=torch.float64), False)
    with pytest.raises(cntk_amd.QuantizerLogicError):
        quantizer.UnquantizeAsync(QuantizedMatrix(8, 4, 1, 0), Matrix(8, 4, dtype=torch.float64))
    with pytest.raises(cntk_amd.QuantizerLogicError):
        QuantizedMatrix(8, 4, 64, 0)
    with pytest.raises(cntk_amd.QuantizerLogicError):  # packed size of the float layout handed to the double call
        cntk_amd._check(cntk_amd.lib().cntkq_unquantize_async_f64(quantizer._h, QuantizedMatrix(8, 4, 1, 0).Buffer(), 48, 0,
                                                                  Matrix(8, 4, dtype=torch.float64).Data(), 8, 4, 1, 0))
    quantizer.QuantizeAsync(Matrix(0, 4, dtype=torch.float64), Matrix(0, 4, dtype=torch.float64),
                            QuantizedMatrix(0, 4, 1, 0, dtype=torch.float64), Matrix(0, 4, dtype=torch.float64), False)
    quantizer.WaitQuantizeAsyncDone()


# ---- fused stripe reduction ---------------------------------------------------------------------------------


def unfused_reference(qz, stripes_np, owner, rows, n, nbits, sres, zt):
    """The reference's call sequence on the GPU: unquantize own stripe, add the others in ascending order, requantize."""
    Agg = Matrix(rows, n, dtype=torch.float64)
    order = [owner] + [w for w in range(len(stripes_np)) if w != owner]
    for pos, w in enumerate(order):
        Q = QuantizedMatrix(rows, n, nbits, 0, dtype=torch.float64)
        Q.from_numpy(stripes_np[w])
        qz.UnquantizeAsync(Q, Agg, add=(pos > 0))
    S = Matrix.from_numpy(sres)
    Qo = QuantizedMatrix(rows, n, nbits, 0, dtype=torch.float64)
    qz.QuantizeAsync(Agg, S, Qo, S, zt)
    qz.WaitQuantizeAsyncDone()
    return Agg.to_numpy(), Qo.to_numpy(), S.to_numpy()


def stripe_max_rows_f64(nbits):
    L = cntk_amd.lib()
    return L.cntkq_stripe_reduce_max_rows_f64(nbits)


@pytest.mark.parametrize("rows,n,k", [(70, 9, 3), (429, 12, 4), (2048, 20, 8), (4096, 3, 2), (4988, 3, 3), (4992, 3, 3), (5003, 2, 2),
                                      (6144, 2, 3), (6145, 2, 2), (6148, 3, 3), (7168, 2, 5), (64, 40, 64), (8000, 2, 3), (20001, 2, 2), (51184, 1, 2),
                                      # on strips: the heights that no single workgroup holds
                                      (51201, 2, 2), (102401, 2, 3), (330001, 1, 2),
                                      # the register kernel's tallest stripes at 16 and 32 bits (all of a compute unit's LDS)
                                      (40860, 2, 2), (20430, 2, 3)])
def test_stripe_reduce_f64(quantizer, rows, n, k):
    for nbits, zt in VARIANTS:
        if not quantizer.StripeReduceTakes(rows, n, nbits, zt, torch.float64):
            assert rows > stripe_max_rows_f64(nbits)
            continue
        say("f64 stripe reduce", rows, n, k, nbits, zt)
        stripes = [oracle.quantize(datagen.normal(31 * w + rows + nbits, rows, n, dtype=F64), zeros(rows, n), nbits, zt, threads=8)[0]
                   for w in range(k)]
        sres = datagen.normal(977 + rows, rows, n, 0.002, dtype=F64)
        for owner in sorted({0, k - 1, k // 2}):
            # the oracle's aggregate: owner first, then ascending
            agg_o = oracle.unquantize(stripes[owner], rows, n, nbits, dtype=F64, threads=8)
            for w in range(k):
                if w != owner:
                    oracle.unquantize(stripes[w], rows, n, nbits, out=agg_o, add=True, threads=8)
            Qs = []
            for w in range(k):
                Q = QuantizedMatrix(rows, n, nbits, 0, dtype=torch.float64)
                Q.from_numpy(stripes[w])
                Qs.append(Q)
            S = Matrix.from_numpy(sres)
            Agg = Matrix(rows, n, dtype=torch.float64)
            quantizer.StripeReduceAsync(Qs, owner, S, Qs[owner], zt, agg_out=Agg)  # in place over the owner's stripe
            quantizer.WaitStripeReduceDone()
            assert parity.bits_equal(Agg.to_numpy(), agg_o), "aggregate differs from the ordered sum"
            parity.check_quantize(agg_o, sres, Qs[owner].to_numpy(), S.to_numpy(), nbits, zt)
            # the fused call gives the very bytes of the reference's unquantize ... quantize call sequence
            agg_u, q_u, s_u = unfused_reference(quantizer, stripes, owner, rows, n, nbits, sres, zt)
            assert parity.bits_equal(agg_u, agg_o)
            assert np.array_equal(q_u, Qs[owner].to_numpy()) and parity.bits_equal(s_u, S.to_numpy())


def test_end_to_end_allreduce_f64(quantizer):
    """K = 4 workers through quantize -> fused stripe reduction -> unquantize against the staged oracle."""
    k, rows, cols = 4, 512, 37
    for nbits, zt in [(1, False), (1, True), (4, False)]:
        gs = [datagen.normal(700 + w, rows, cols, dtype=F64) for w in range(k)]
        res = [datagen.normal(750 + w, rows, cols, 0.002, dtype=F64) for w in range(k)]
        sres = [datagen.normal(770 + s, rows, oracle.stripe_range(cols, s, k)[1], 0.002, dtype=F64) for s in range(k)]
        res_o = [r.copy(order="F") for r in res]
        sres_o = [s.copy(order="F") for s in sres]
        q1_o, aggs_o, qagg_o, out_o = parity.oracle_allreduce_staged(gs, res_o, sres_o, nbits, zt)
        rep = parity.Report()
        Qw, tainted = [], np.zeros(cols, dtype=bool)
        for w in range(k):
            Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
            R = Matrix.from_numpy(res[w])
            quantizer.QuantizeAsync(Matrix.from_numpy(gs[w]), R, Q, R, zt)
            quantizer.WaitQuantizeAsyncDone()
            parity.check_quantize(gs[w], res[w], Q.to_numpy(), R.to_numpy(), nbits, zt, report=rep)
            tainted |= rep.last_mismatch_cols
            Qw.append(Q)
        Qagg = QuantizedMatrix(rows, cols, nbits, 0, dtype=torch.float64)
        sres_gpu = []
        for s in range(k):
            st, n = oracle.stripe_range(cols, s, k)
            S = Matrix.from_numpy(sres[s])
            quantizer.StripeReduceAsync([Q.ColumnSlice(st, n) for Q in Qw], s, S, Qagg.ColumnSlice(st, n), zt)
            quantizer.WaitStripeReduceDone()
            sres_gpu.append(S.to_numpy())
        Out = Matrix(rows, cols, dtype=torch.float64)
        quantizer.UnquantizeAsync(Qagg, Out)
        quantizer.WaitUnquantizeAsyncDone()
        worst, ntaint = parity.check_end_to_end(aggs_o, sres, Qagg.to_numpy(), sres_gpu, Out.to_numpy(), qagg_o, out_o, rows, cols,
                                                nbits, zt, tainted, report=rep)
        say("f64 all-reduce nbits", nbits, "zt", zt, "worst", worst, "tainted columns", ntaint, rep)


# ---- the batched calls on doubles ---------------------------------------------------------------------------------------

MIXED64 = [(147, 64), (64, 64), (576, 33), (1, 5), (5, 1), (429, 37), (2048, 33), (2304, 5), (4608, 3), (0, 4), (1000, 1), (1152, 40),
           (4096, 6), (5120, 3), (7168, 2), (8000, 2), (20001, 2), (512, 100), (33, 67)]


@pytest.mark.parametrize("nbits,zt", [(1, False), (1, True), (4, False), (16, False), (64, False)])
def test_batch_equals_per_matrix_calls_f64(quantizer, nbits, zt):
    """One call for a whole set of double matrices (tile members, register-kernel and tall matrices with launches of
    their own, an empty one) gives the bytes of one call per matrix; the oracle checks the result as well."""
    qz = quantizer
    gs = [datagen.normal_with_outliers(100 * i + nbits, r, c, dtype=F64) for i, (r, c) in enumerate(MIXED64)]
    rs = [datagen.normal(300 * i + nbits, r, c, 0.003, dtype=F64) for i, (r, c) in enumerate(MIXED64)]
    new = lambda: [QuantizedMatrix(r, c, nbits, 0, dtype=torch.float64) for r, c in MIXED64]
    for step in range(2):
        say("f64 batch", nbits, zt, "step", step)
        G = [Matrix.from_numpy(g) for g in gs]
        R1, Q1, O1 = [Matrix.from_numpy(r) for r in rs], new(), [Matrix.from_numpy(r) for r in rs]
        for g, r, q in zip(G, R1, Q1):
            qz.QuantizeAsync(g, r, q, r, zt)
        for q, o in zip(Q1, O1):
            qz.UnquantizeAsync(q, o, add=(step == 1))
        qz.WaitUnquantizeAsyncDone()
        R2, Q2, O2 = [Matrix.from_numpy(r) for r in rs], new(), [Matrix.from_numpy(r) for r in rs]
        qz.QuantizeBatchAsync([(g, r, q, r) for g, r, q in zip(G, R2, Q2)], zt)
        qz.WaitQuantizeAsyncDone()
        qz.UnquantizeBatchAsync(list(zip(Q2, O2)), add=(step == 1))
        qz.WaitUnquantizeAsyncDone()
        torch.cuda.synchronize()
        for i, (r, c) in enumerate(MIXED64):
            assert np.array_equal(Q1[i].to_numpy(), Q2[i].to_numpy()), ("packed", MIXED64[i])
            assert parity.bits_equal(R1[i].to_numpy(), R2[i].to_numpy()), ("residual", MIXED64[i])
            assert parity.bits_equal(O1[i].to_numpy(), O2[i].to_numpy()), ("output", MIXED64[i])
            if r and c:
                parity.check_quantize(gs[i], rs[i], Q2[i].to_numpy(), R2[i].to_numpy(), nbits, zt)
        rs = [m.to_numpy() for m in R2]
    with pytest.raises(cntk_amd.QuantizerLogicError):  # element types may not be mixed within a call
        qz.QuantizeBatchAsync([(G[0], R2[0], Q2[0], R2[0]), (Matrix(4, 4), Matrix(4, 4), QuantizedMatrix(4, 4, nbits if nbits <= 32 else 32, 0),
                                                             Matrix(4, 4))], zt)


STRIPE_SETS64 = [(147, 8), (64, 16), (576, 9), (1, 5), (429, 7), (2048, 12), (4608, 3), (1000, 4), (4096, 6), (7168, 2), (0, 3), (33, 9)]


@pytest.mark.parametrize("nbits,zt,k", [(1, False, 8), (1, True, 3), (4, False, 4), (64, False, 2)])
def test_stripe_batch_equals_per_matrix_calls_f64(quantizer, nbits, zt, k):
    qz = quantizer
    owner = k // 2
    # (and a stripe that no single workgroup holds: a launch of its own, on strips)
    sets = STRIPE_SETS64 + ([(60000, 2)] if nbits < 64 else [])
    packed = [[oracle.quantize(datagen.normal(50 * i + 7 * w + nbits, r, c, dtype=F64), zeros(r, c), nbits, zt, threads=8)[0] if r and c
               else np.zeros(0, np.uint8) for w in range(k)] for i, (r, c) in enumerate(sets)]
    sres = [datagen.normal(900 + i, r, c, 0.003, dtype=F64) for i, (r, c) in enumerate(sets)]

    def device_state():
        Qs = []
        for i, (r, c) in enumerate(sets):
            row = []
            for w in range(k):
                Q = QuantizedMatrix(r, c, nbits, 0, dtype=torch.float64)
                if r and c:
                    Q.from_numpy(packed[i][w])
                row.append(Q)
            Qs.append(row)
        return Qs, [Matrix.from_numpy(s) for s in sres], [Matrix(r, c, dtype=torch.float64) for r, c in sets]

    Q1, S1, A1 = device_state()
    for i in range(len(sets)):
        if sets[i][0]:
            qz.StripeReduceAsync(Q1[i], owner, S1[i], Q1[i][owner], zt, agg_out=A1[i])
    qz.WaitStripeReduceDone()
    Q2, S2, A2 = device_state()
    for rep in range(2):  # the second call finds the cached table
        if rep == 1:
            for i, (r, c) in enumerate(sets):
                S2[i].data.copy_(Matrix.from_numpy(sres[i]).data)
                if r and c:
                    Q2[i][owner].from_numpy(packed[i][owner])
        qz.StripeReduceBatchAsync([(Q2[i], S2[i], Q2[i][owner], A2[i]) for i in range(len(sets))], owner, zt)
        qz.WaitStripeReduceDone()
        torch.cuda.synchronize()
        for i, (r, c) in enumerate(sets):
            if r == 0:
                continue
            assert np.array_equal(Q1[i][owner].to_numpy(), Q2[i][owner].to_numpy()), ("packed", sets[i])
            assert parity.bits_equal(S1[i].to_numpy(), S2[i].to_numpy()), ("stripe residual", sets[i])
            assert parity.bits_equal(A1[i].to_numpy(), A2[i].to_numpy()), ("aggregate", sets[i])


def test_stripe_reduce_height_limit_f64(quantizer):
    """The limit the library reports per bit width is the tallest column the fused call takes."""
    assert stripe_max_rows_f64(64) == 7168 and stripe_max_rows_f64(1) == 51184 and stripe_max_rows_f64(3) == 0
    assert stripe_max_rows_f64(16) == 40860 and stripe_max_rows_f64(32) == 20430 and stripe_max_rows_f64(8) == 51184
    rows, n, k = 7170, 2, 2  # (codes as wide as a QWord: the tile kernels' heights only)
    Qs = [QuantizedMatrix(rows, n, 64, 0, dtype=torch.float64) for _ in range(k)]
    S = Matrix(rows, n, dtype=torch.float64)
    with pytest.raises(cntk_amd.QuantizerLogicError, match="up to 7168 rows"):
        quantizer.StripeReduceAsync(Qs, 0, S, Qs[0], False)
    takes = lambda rows, nbits: quantizer.StripeReduceTakes(rows, 2, nbits, False, torch.float64)
    # (the register kernels quantize and reduce the same heights; whatever is taller goes to the strips, both of them)
    assert takes(40860, 16) and takes(40862, 16) and takes(20430, 32) and takes(20432, 32)
    assert takes(51184, 1) and takes(51185, 1) and takes(400000, 4) and not takes(20000, 64) and not takes(50000000, 1)
