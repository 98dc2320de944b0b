"""Seeded random shapes through the automatic kernel choice, fp32 and fp64: heights drawn around every boundary of the
kernel selection (multiples of 4 and 32 and their neighbours, 1024, 4096, 7168, 14336, 51200, 102400), few columns, every
bit width, matrices at random offsets inside their allocations, residual in place or not. Every case: quantize against the
oracle (codes under the GPU's own headers bit-exact, bounds and residuals within tolerance), unquantize bit-exact."""
import sys

import numpy as np
import pytest
import torch

import datagen
import oracle
import parity
from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

pytestmark = pytest.mark.gpu

BOUNDARIES = [1, 4, 31, 32, 33, 64, 128, 255, 256, 1000, 1023, 1024, 1028, 2048, 2304, 4095, 4096, 4100, 4128, 6148, 7168, 7170, 9304,
              12288, 14332, 14336, 14340, 16384, 20000, 32768, 51198, 51200, 51204, 65540, 102396, 102400, 102404]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


TALL = [102401, 110000, 131072, 131073, 147456, 200000, 262144, 262145, 300001, 524288, 524289, 600000, 655361, 700001, 1048577, 2800001,
        6000001]


def draw_case(rng, is64, tall=False):
    r = rng.random()
    if tall:
        # above what one workgroup holds: strips of a column on several workgroups (on one die, or on all), then the
        # same strips in several launches
        rows = int(rng.choice(TALL)) if r < 0.6 else int(rng.integers(102401, 540000))
    elif r < 0.5:
        rows = int(rng.choice(BOUNDARIES))
    elif r < 0.8:
        rows = int(rng.integers(1, 3000))
    else:
        rows = int(rng.integers(1, 26000)) * 4
    rows = max(1, rows + int(rng.choice([0, 0, 0, -1, 1, 2])))
    max_cols = max(1, min(40, 400000 // rows))
    cols = int(rng.integers(1, max_cols + 1))
    nbits = int(rng.choice([1, 1, 1, 2, 4, 8, 16, 32] + ([64] if is64 else [])))
    zt = bool(rng.integers(0, 2)) and nbits == 1
    # element offsets of gradient, residual and output inside their allocations: mostly equal (then the kernels may
    # align their accesses to cache lines), sometimes not
    unit = 2 if is64 else 4
    off = int(rng.integers(0, 8)) * unit if rng.random() < 0.5 else 0
    offs = (off, off, off) if rng.random() < 0.7 else tuple(int(rng.integers(0, 9)) for _ in range(3))
    in_place = bool(rng.integers(0, 2))
    return rows, cols, nbits, zt, offs, in_place


def place(a, off, tdt):
    n = a.size
    buf = torch.zeros(n + 64, dtype=tdt, device="cuda:0")
    buf[off:off + n] = torch.from_numpy(a.reshape(-1, order="F").copy()).cuda()
    return Matrix(a.shape[0], a.shape[1], 0, buf[off:off + n], dtype=tdt), buf


@pytest.mark.parametrize("dtype,seed,count,tall", [("f32", 11, 150, False), ("f32", 12, 150, False), ("f64", 13, 120, False), ("f64", 14, 120, False),
                                                   ("f32", 15, 40, True), ("f64", 16, 12, True)])
def test_random_shapes(dtype, seed, count, tall):
    is64 = dtype == "f64"
    ndt, tdt = (np.float64, torch.float64) if is64 else (np.float32, torch.float32)
    rng = np.random.default_rng(seed)
    qz = MatrixQuantizerImpl.Create(0, False)
    rep = parity.Report()
    for n in range(count):
        rows, cols, nbits, zt, offs, in_place = draw_case(rng, is64, tall)
        say("random case", dtype, seed, n, "rows", rows, "cols", cols, "nbits", nbits, "zeroThr", zt, "offsets", offs, "in place", in_place)
        g = datagen.normal_with_outliers(seed * 1000 + n, rows, cols, 0.01, dtype=ndt)
        r = datagen.normal(seed * 2000 + n, rows, cols, 0.002, dtype=ndt)
        G, _g = place(g, offs[0], tdt)
        R, rbuf = place(r, offs[1], tdt)
        if in_place:
            Rout, obuf = R, rbuf
        else:
            Rout, obuf = place(np.zeros_like(g, order="F"), offs[2], tdt)
        Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=tdt)
        qz.QuantizeAsync(G, R, Q, Rout, zt)
        qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        q_gpu = Q.to_numpy()
        parity.check_quantize(g, r, q_gpu, Rout.to_numpy(), nbits, zt, report=rep)
        # nothing written outside the residual
        off_o = offs[1] if in_place else offs[2]
        assert float(obuf[:off_o].abs().sum()) == 0.0 and float(obuf[off_o + rows * cols:].abs().sum()) == 0.0
        prev = datagen.normal(seed * 3000 + n, rows, cols, 1.0, dtype=ndt)
        add = bool(n % 2)
        Out, outbuf = place(prev, offs[2], tdt)
        qz.UnquantizeAsync(Q, Out, add=add)
        qz.WaitUnquantizeAsyncDone()
        torch.cuda.synchronize()
        parity.check_unquantize(q_gpu, rows, cols, nbits, Out.to_numpy(), prev_out=prev if add else None)
        assert float(outbuf[:offs[2]].abs().sum()) == 0.0 and float(outbuf[offs[2] + rows * cols:].abs().sum()) == 0.0
    say("  ", rep)


@pytest.mark.parametrize("seed,count,tall", [(21, 60, False), (22, 60, False), (23, 40, True), (24, 24, 2)])
def test_random_stripe_reductions(seed, count, tall):
    """Random stripes through the fused reduction: the fp32 aggregate bit-exact against the oracle (owner first, then
    ascending rank), the requantized stripe like any quantize result, and the bytes of the reference's call sequence
    (unquantize own stripe, add the others, quantize the aggregate) on the same handle."""
    from test_gpu_stripe_reduce import gpu_stripe_reduce

    rng = np.random.default_rng(seed)
    qz = MatrixQuantizerImpl.Create(0, False)
    rep = parity.Report()
    heights = [h for h in BOUNDARIES if h <= 14336]
    for n in range(count):
        nbits = int(rng.choice([1, 1, 1, 2, 4, 8, 16, 32]))
        if tall == 2:
            # what no single workgroup holds: the reduction on strips, on one die and (above some 524288 rows) on all
            nbits = int(rng.choice([1, 1, 2, 4, 8, 16]))
            least = {1: 102401, 2: 102401, 4: 102401, 8: 81821, 16: 40911}[nbits]
            most = {1: 1000000, 2: 800000, 4: 500000, 8: 300000, 16: 150000}[nbits]
            k = int(rng.choice([1, 2, 3, 5, 6, 8, 11]))
            cols = int(rng.integers(1, 4)) + k - 1  # every owner has a column
            most = max(least + 4, min(most, 16000000 // (cols * k)))  # bounds what the oracle quantizes per case
            rows = int(rng.choice([least, least + 3, 131072, 200000, 262147, int(rng.integers(least, most))]))
            rows = max(least, min(most, rows))
            assert qz.StripeReduceTakes(rows, 1, nbits)
        elif tall:
            # above the LDS kernels' heights: the register kernel of the stripe reduction, up to its limit per bit width
            nbits = int(rng.choice([1, 1, 2, 4, 8, 16]))
            limit = {1: 102368, 2: 102368, 4: 102368, 8: 81820, 16: 40910}[nbits]
            rows = int(rng.choice([14337, 14340, 16334, 20000, 32668, 40910, 50257, 65536, 81820, 102368, int(rng.integers(14337, 102369))]))
            rows = max(14337, min(limit, rows + int(rng.choice([0, 0, -1, 1, 2]))))
            k = int(rng.choice([1, 2, 3, 5, 8]))
            cols = int(rng.integers(1, max(2, min(8, 240000 // rows)) + 1))
        else:
            rows = int(rng.choice(heights)) if rng.random() < 0.6 else int(rng.integers(1, 3600)) * 4
            rows = max(1, min(14336, rows + int(rng.choice([0, 0, 0, -1, 1]))))
            k = int(rng.choice([1, 2, 3, 5, 8, 8, 13, 64]))
            cols = int(rng.integers(1, max(2, min(48, 120000 // rows)) + 1))
        zt = bool(rng.integers(0, 2)) and nbits == 1
        owner = int(rng.integers(0, k))
        start, ncols = oracle.stripe_range(cols, owner, k)
        say("random stripe", seed, n, "rows", rows, "cols", cols, "workers", k, "owner", owner, "stripe", start, ncols, "nbits", nbits, "zeroThr", zt)
        if ncols == 0:
            continue
        gs = [datagen.normal(seed * 5000 + 70 * n + w, rows, cols) for w in range(k)]
        zeros = np.zeros((rows, cols), np.float32, order="F")
        qs = [oracle.quantize(g, zeros, nbits, zt, threads=8)[0] for g in gs]
        sres = datagen.normal(seed * 7000 + n, rows, ncols, 0.003)
        q_new, s_new, agg = gpu_stripe_reduce(qz, qs, owner, rows, cols, nbits, sres, zt, alias_out=bool(n % 2))
        s_o = sres.copy(order="F")
        agg_o = oracle.stripe_reduce([q.copy() for q in qs], owner, rows, cols, nbits, s_o, zt, threads=8)
        assert parity.bits_equal(agg, agg_o), "fp32 aggregate differs from the oracle"
        parity.check_quantize(agg_o, sres, q_new, s_new, nbits, zt, report=rep)
        Agg = Matrix(rows, ncols)
        qcol = oracle.qcol_bytes(nbits, rows)
        for pos, w in enumerate([owner] + [w for w in range(k) if w != owner]):
            Qw = QuantizedMatrix(rows, ncols, nbits, 0)
            Qw.from_numpy(qs[w][start * qcol:(start + ncols) * qcol])
            qz.UnquantizeAsync(Qw, Agg, add=(pos > 0))
        S = Matrix.from_numpy(sres)
        Qo = QuantizedMatrix(rows, ncols, nbits, 0)
        qz.QuantizeAsync(Agg, S, Qo, S, zt)
        qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        assert np.array_equal(Qo.to_numpy(), q_new), "fused != call sequence (codes)"
        assert parity.bits_equal(S.to_numpy(), s_new), "fused != call sequence (residual)"
    say("  ", rep)
