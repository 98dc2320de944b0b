"""Parity of the fused stripe reduction and of the whole simulated K-worker quantized all-reduce
(Source/1BitSGD/AllReduceDistGradAggregator.h:268-531) against the CPU oracle. Needs an MI355X.

All K workers live in one GPU's memory. The fp32 sum inside the stripe reduction has a fixed order (owner
first, then ascending rank), so the fp32 aggregate must equal the oracle's bit for bit; the requantized
stripe is then checked like any quantize result.
"""
import ctypes
import sys

import numpy as np
import pytest
import torch

import cntk_amd
import datagen
import oracle
import parity
from cntk_amd import Matrix, MatrixQuantizer, MatrixQuantizerImpl, QuantizedMatrix

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def gpu_stripe_reduce(qz, q_workers, owner, rows, cols, nbits, stripe_res, zt, alias_out=True):
    """q_workers: list of numpy packed FULL matrices; returns (new packed stripe, new stripe residual, aggregate)."""
    k = len(q_workers)
    start, n = cntk_amd.stripe_range(cols, owner, k)
    Qs = []
    for q in q_workers:
        Q = QuantizedMatrix(rows, cols, nbits, 0)
        Q.from_numpy(q)
        Qs.append(Q)
    stripes = [Q.ColumnSlice(start, n) for Q in Qs]
    S = Matrix.from_numpy(stripe_res)
    Agg = Matrix(rows, n)
    out_q = stripes[owner] if alias_out else QuantizedMatrix(rows, n, nbits, 0)
    qz.StripeReduceAsync(stripes, owner, S, out_q, zt, agg_out=Agg)
    qz.WaitStripeReduceDone()
    torch.cuda.synchronize()
    return out_q.to_numpy(), S.to_numpy(), Agg.to_numpy()


CASES = [
    # rows, cols, workers, nbits, zeroThr
    (5, 7, 2, 1, False), (37, 11, 3, 2, False), (70, 10, 4, 1, True), (429, 40, 8, 1, False), (429, 40, 8, 1, True),
    (147, 64, 8, 4, False), (576, 24, 5, 8, False), (100, 9, 3, 16, False), (64, 12, 4, 32, False),
    (2048, 48, 8, 1, False), (2048, 48, 8, 1, True), (2048, 16, 8, 2, False), (4608, 8, 2, 1, False),
    (9304, 3, 3, 1, True), (33, 5, 8, 1, False), (512, 64, 64, 1, False), (4096, 7, 3, 1, False), (4096, 4, 12, 1, True),
    (2048, 20, 11, 1, False), (1024, 24, 4, 1, False), (1024, 9, 64, 1, True), (4096, 5, 64, 1, False),
    # tall columns: 1024 threads per column in the stripe reduction, register kernels in the call sequence
    (9304, 6, 4, 1, False), (8192, 4, 3, 4, False), (12000, 4, 5, 2, False), (14336, 2, 2, 8, False),
    # above 14336 rows: the register kernel's shape (the running sum in registers, one worker's record at a time in LDS)
    (14340, 6, 4, 1, False), (14337, 3, 2, 2, False), (20000, 5, 3, 1, True), (32768, 4, 5, 4, False), (50257, 3, 8, 1, False),
    (100000, 2, 2, 1, False), (102365, 2, 3, 2, False), (16332, 2, 2, 16, False), (32668, 2, 2, 8, False), (40910, 2, 2, 16, False),
    (81820, 2, 3, 8, False), (100000, 2, 2, 4, False),
    # heights that are not a multiple of 4: the tile kernels up to 2048 rows, above them the register kernels with edge
    # elements (256 threads per column up to 7168 rows, 1024 above)
    (1023, 6, 3, 1, False), (1025, 6, 3, 1, False), (2049, 8, 8, 1, False), (2050, 5, 2, 1, True), (4097, 4, 3, 4, False), (6001, 3, 5, 2, False),
    (7167, 4, 3, 1, False), (7169, 3, 2, 4, False), (7170, 4, 3, 1, True), (8001, 4, 2, 2, False), (9305, 3, 3, 1, False),
    (14335, 2, 8, 1, False), (9305, 2, 2, 32, False),
    # stripes of more than 256 columns above 6144 rows: 512 threads per column in the LDS column kernel
    (6400, 600, 2, 2, False), (8192, 540, 2, 8, False), (6148, 2320, 9, 1, False),
    # more than eight workers at 2 and 4 bits: the second batch of workers reads its levels from the table too
    (2048, 26, 13, 2, False), (4096, 20, 10, 4, False), (1152, 22, 11, 4, False),
    # six pieces per thread in the table-driven kernels (256 threads: 4100 to 6144 rows, 1024 threads: 16388 to 24576)
    (6144, 16, 8, 1, False), (5000, 16, 8, 1, True), (24576, 8, 8, 1, False), (20000, 6, 12, 1, False),
    # taller than any workgroup holds: the reduction on strips, several workgroups per column (on one die, and -- the last
    # case -- on all of them), wherever the call sequence's quantize step runs on strips too
    (102401, 4, 2, 1, False), (110000, 3, 3, 1, True), (150001, 4, 4, 2, False), (131072, 2, 2, 4, False), (81822, 2, 2, 8, False),
    (40912, 2, 2, 16, False), (90000, 2, 2, 16, False), (262147, 2, 8, 1, False), (700000, 2, 2, 1, False),
    # worker counts that are no multiple of the four workers whose QWords a strip requests together, up to the most workers
    (120001, 5, 5, 1, False), (102403, 13, 13, 2, False), (110000, 3, 64, 1, True), (131075, 2, 7, 4, False),
]


@pytest.mark.parametrize("case", CASES, ids=["%dx%d_k%d_b%d_z%d" % (c[0], c[1], c[2], c[3], int(c[4])) for c in CASES])
def test_stripe_reduce(case):
    rows, cols, k, nbits, zt = case
    qz = MatrixQuantizerImpl.Create(0, False)
    gs = [datagen.normal(datagen.case_seed(4, 0, 0, w) + rows, rows, cols) for w in range(k)]
    zeros = np.zeros((rows, cols), np.float32, order="F")
    qs = [oracle.quantize(g, zeros, nbits, zt, threads=8)[0] for g in gs]
    rep = parity.Report()
    for owner in sorted({0, k // 2, k - 1}):
        start, n = oracle.stripe_range(cols, owner, k)
        if n == 0:
            continue
        say("stripe reduce", case, "owner", owner, "cols", start, n)
        sres = datagen.normal(900 + owner, rows, n, 0.003)
        # heights that are a multiple of 4 can take the kernels with one workgroup per column (path 3; the automatic
        # choice from 1024 rows on) as well as the tile kernels (path 1)
        variants = [(True, 0), (False, 0)] + ([(True, 1), (True, 3)] if rows % 4 == 0 and rows <= 14336 else [])
        for alias, path in variants:
            qz._set_tuning(quantize_path=path)
            q_new, s_new, agg = gpu_stripe_reduce(qz, qs, owner, rows, cols, nbits, sres, zt, alias_out=alias)
            # oracle on copies
            qs_o = [q.copy() for q in qs]
            s_o = sres.copy(order="F")
            agg_o = oracle.stripe_reduce(qs_o, owner, rows, cols, nbits, s_o, zt, threads=8)
            assert parity.bits_equal(agg, agg_o), "fp32 aggregate differs from the oracle (order: owner, then ascending)"
            # the requantization sees (aggregate, stripe residual) as (gradient, residual)
            parity.check_quantize(agg_o, sres, q_new, s_new, nbits, zt, report=rep)
            # and the fused call gives the very bytes of the reference's call sequence on the same handle:
            # unquantize own stripe, add the others in ascending order, quantize the aggregate
            if alias:
                Agg = Matrix(rows, n)
                order = [owner] + [w for w in range(k) if w != owner]
                qcol = oracle.qcol_bytes(nbits, rows)
                for pos, w in enumerate(order):
                    Qw = QuantizedMatrix(rows, n, nbits, 0)
                    Qw.from_numpy(qs[w][start * qcol:(start + n) * qcol])
                    qz.UnquantizeAsync(Qw, Agg, add=(pos > 0))
                S = Matrix.from_numpy(sres)
                Qo = QuantizedMatrix(rows, n, nbits, 0)
                qz.QuantizeAsync(Agg, S, Qo, S, zt)
                qz.WaitQuantizeAsyncDone()
                assert parity.bits_equal(Agg.to_numpy(), agg)
                assert np.array_equal(Qo.to_numpy(), q_new), "fused != call sequence (codes)"
                assert parity.bits_equal(S.to_numpy(), s_new), "fused != call sequence (residual)"
    say("  ", rep)


def test_stripe_reduce_of_few_valued_columns_6144_rows():
    """The recorded miss of the 1e-5 bound tolerance: a 6144-row stripe at K = 2, 1 bit, zero threshold. The aggregate
    holds four distinct values, the oracle's term-by-term fp32 sum of such a column is off by more than 1e-5 of the
    column scale, the device's pairwise sums are not. The comparison accepts exactly those columns against the
    float64 bounds and counts them."""
    rows, cols, k = 6144, 32, 2
    a, b, s = datagen.few_valued_stripe_sum(rows, cols)
    zeros = np.zeros((rows, cols), np.float32, order="F")
    qs = [oracle.quantize(g, zeros, 1, True, threads=8)[0] for g in (a, b)]
    # one stripe of all columns: the second worker's packed matrix stands in for a stripe of the same width
    qz = MatrixQuantizerImpl.Create(0, False)
    Qs = []
    for q in qs:
        Q = QuantizedMatrix(rows, cols, 1, 0)
        Q.from_numpy(q)
        Qs.append(Q)
    S, Agg = Matrix(rows, cols), Matrix(rows, cols)
    qz.StripeReduceAsync(Qs, 0, S, Qs[0], True, agg_out=Agg)
    qz.WaitStripeReduceDone()
    torch.cuda.synchronize()
    assert parity.bits_equal(Agg.to_numpy(), s)
    rep = parity.check_quantize(s, zeros, Qs[0].to_numpy(), S.to_numpy(), 1, True, strict=True)
    say("few-valued 6144-row stripe:", rep)
    lo_g, hi_g = oracle.headers(Qs[0].to_numpy(), rows, cols, 1)
    lo_x, hi_x = parity.exact_headers(s, zeros, 1, True)
    assert np.max(np.maximum(np.abs(lo_g - lo_x), np.abs(hi_g - hi_x)) / (hi_x - lo_x)) < 1e-6
    assert 3 <= rep.fallback_cols <= cols


@pytest.mark.parametrize("rows,off", [(2048, 1), (1024, 3), (4096, 2), (9304, 1), (1028, 5), (20000, 1), (20001, 2)])
@pytest.mark.parametrize("batched", [False, True], ids=["plain", "batched"])
def test_stripe_residual_at_4_byte_offsets(rows, off, batched):
    """A stripe residual that is only 4-byte aligned (a view `off` elements into an allocation): the fused reduction
    must still give the bytes of the call sequence whose aggregate and residual sit at that same offset, i.e. pick the
    kernel family a quantize call on such matrices picks. Also through the batched call, alone and beside a second item."""
    from test_gpu_random_shapes import place

    cols, k, nbits, zt = 6, 3, 1, False
    qz = MatrixQuantizerImpl.Create(0, False)
    gs = [datagen.normal(3100 + w + rows, rows, cols) for w in range(k)]
    zeros = np.zeros((rows, cols), np.float32, order="F")
    qs = [oracle.quantize(g, zeros, nbits, zt, threads=8)[0] for g in gs]
    sres = datagen.normal(3200 + rows, rows, cols, 0.003)
    Qs = []
    for q in qs:
        Q = QuantizedMatrix(rows, cols, nbits, 0)
        Q.from_numpy(q)
        Qs.append(Q)
    S, _sbuf = place(sres, off, torch.float32)
    Out = QuantizedMatrix(rows, cols, nbits, 0)
    if batched:
        # a second, ordinary item makes the call a real shared grid; then the item alone (the call falls back to the plain one)
        g2 = [datagen.normal(3300 + w, 2048, 4) for w in range(k)]
        Q2 = []
        for g in g2:
            Q = QuantizedMatrix(2048, 4, nbits, 0)
            Q.from_numpy(oracle.quantize(g, np.zeros((2048, 4), np.float32, order="F"), nbits, zt)[0])
            Q2.append(Q)
        S2, Out2 = Matrix(2048, 4), QuantizedMatrix(2048, 4, nbits, 0)
        qz.StripeReduceBatchAsync([(Qs, S, Out, None), (Q2, S2, Out2, None)], 0, zt)
        qz.WaitStripeReduceDone()
        torch.cuda.synchronize()
        first = (Out.to_numpy().copy(), S.to_numpy().copy())
        S, _sbuf = place(sres, off, torch.float32)
        qz.StripeReduceBatchAsync([(Qs, S, Out, None)], 0, zt)
    else:
        first = None
        qz.StripeReduceAsync(Qs, 0, S, Out, zt)
    qz.WaitStripeReduceDone()
    torch.cuda.synchronize()
    q_new, s_new = Out.to_numpy(), S.to_numpy()
    if first is not None:
        assert np.array_equal(first[0], q_new) and parity.bits_equal(first[1], s_new), "batch member != item alone"
    # the call sequence with aggregate and residual at the same offset
    Agg, _abuf = place(zeros, off, torch.float32)
    for w in range(k):
        qz.UnquantizeAsync(Qs[w], Agg, add=(w > 0))
    S2, _s2buf = place(sres, off, torch.float32)
    Qo = QuantizedMatrix(rows, cols, nbits, 0)
    qz.QuantizeAsync(Agg, S2, Qo, S2, zt)
    qz.WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
    assert np.array_equal(Qo.to_numpy(), q_new), "fused != call sequence (codes)"
    assert parity.bits_equal(S2.to_numpy(), s_new), "fused != call sequence (residual)"
    # (the packed matrices stand in for stripes of their full width: the aggregate is their decoded sum, worker 0 first)
    agg_o = oracle.unquantize(qs[0], rows, cols, nbits, threads=8)
    for w in range(1, k):
        agg_o = oracle.unquantize(qs[w], rows, cols, nbits, out=agg_o, add=True, threads=8)
    assert parity.bits_equal(agg_o, Agg.to_numpy())
    parity.check_quantize(agg_o, sres, q_new, s_new, nbits, zt)


def test_stripe_reduce_height_limit():
    """The tallest stripe the fused call takes with one workgroup per column depends on the bit width (its LDS holds the
    output QWords and one worker's record); the limit can be asked for, and so can whether a taller stripe is taken."""
    L = cntk_amd.lib()
    L.cntkq_stripe_reduce_max_rows.restype = ctypes.c_size_t
    L.cntkq_stripe_reduce_max_rows.argtypes = [ctypes.c_size_t]
    assert L.cntkq_stripe_reduce_max_rows(1) == 102368 and L.cntkq_stripe_reduce_max_rows(32) == 14336
    assert L.cntkq_stripe_reduce_max_rows(16) == 40910 and L.cntkq_stripe_reduce_max_rows(8) == 81820 and L.cntkq_stripe_reduce_max_rows(3) == 0
    assert L.cntkq_stripe_reduce_max_rows(4) == 102368 and L.cntkq_stripe_reduce_max_rows(2) == 102368
    qz = MatrixQuantizerImpl.Create(0, False)
    rows, cols, k = 14340, 2, 2  # (codes as wide as a QWord: the LDS kernels' heights only)
    zeros = np.zeros((rows, cols), np.float32, order="F")
    qs = [oracle.quantize(datagen.normal(5 + w, rows, cols), zeros, 32, False)[0] for w in range(k)]
    with pytest.raises(cntk_amd.QuantizerLogicError):
        gpu_stripe_reduce(qz, qs, 0, rows, cols, 32, np.zeros((rows, 1), np.float32, order="F"), False)
    # Taller stripes are taken where a quantize call on the same shape runs on strips (what no single workgroup holds): the
    # library says which. (Between 102369 and 102400 rows a quantize call still runs in registers: the call sequence.)
    assert qz.StripeReduceTakes(40910, 1, 16) and qz.StripeReduceTakes(40912, 1, 16) and qz.StripeReduceTakes(81822, 1, 8)
    assert qz.StripeReduceTakes(102368, 5, 1) and qz.StripeReduceTakes(102401, 5, 1, True) and qz.StripeReduceTakes(1000000, 5, 2)
    assert not qz.StripeReduceTakes(102369, 5, 1)  # (a height the register kernels still take)
    assert not qz.StripeReduceTakes(20000, 5, 32) and not qz.StripeReduceTakes(50000000, 1, 1) and not qz.StripeReduceTakes(0, 1, 1)


def test_stripe_reduce_32bit_equals_plain_sum():
    """The reference's own known-answer trick (32 bits: Tests/EndToEndTests/CNTKv2Library/EndToEndTests/FrameMode.cpp:112-116)."""
    rows, cols, k = 129, 24, 4
    qz = MatrixQuantizerImpl.Create(0, False)
    gs = [datagen.normal(70 + w, rows, cols, 1.0) for w in range(k)]
    zeros = np.zeros((rows, cols), np.float32, order="F")
    qs = [oracle.quantize(g, zeros, 32, False)[0] for g in gs]
    for owner in range(k):
        start, n = oracle.stripe_range(cols, owner, k)
        q_new, s_new, agg = gpu_stripe_reduce(qz, qs, owner, rows, cols, 32, np.zeros((rows, n), np.float32, order="F"), False)
        acc = gs[owner][:, start:start + n].copy()
        for w in range(k):
            if w != owner:
                acc = gs[w][:, start:start + n] + acc
        assert parity.bits_equal(np.asfortranarray(acc), agg)
        assert not s_new.any()
        assert parity.bits_equal(oracle.unquantize(q_new, rows, n, 32), np.asfortranarray(acc))


def simulated_allreduce_gpu(gs, res, sres, nbits, zt, use_async):
    """The aggregator's dataflow on one GPU: per-worker MatrixQuantizer objects, stripes exchanged by pointer.
    Returns (worker residuals, stripe residuals, packed matrices before the reduction, assembled packed
    aggregate, output)."""
    k = len(gs)
    rows, cols = gs[0].shape
    workers = [MatrixQuantizer(rows, cols, 0, use_async) for _ in range(k)]
    G = [Matrix.from_numpy(g) for g in gs]
    Q = [QuantizedMatrix(rows, cols, nbits, 0) for _ in range(k)]
    S = [Matrix.from_numpy(s) for s in sres]
    for w in range(k):
        workers[w].GetResidualMatrix().data.copy_(Matrix.from_numpy(res[w]).data)
    torch.cuda.synchronize()
    for w in range(k):
        workers[w].impl.SynchronizeWithMainStream()
        workers[w].QuantizeAsync(G[w], Q[w], zt)
    for w in range(k):
        workers[w].WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
    q_before = [q.to_numpy() for q in Q]
    for s in range(k):
        start, n = cntk_amd.stripe_range(cols, s, k)
        if n == 0:
            continue
        stripes = [Q[w].ColumnSlice(start, n) for w in range(k)]
        # the owner's requantized stripe overwrites its own slice, as in the reference
        workers[s].impl.StripeReduceAsync(stripes, s, S[s], stripes[s], zt)
    for s in range(k):
        workers[s].impl.WaitStripeReduceDone()
    torch.cuda.synchronize()
    # "broadcast": assemble the requantized stripes; every worker would unquantize this same buffer
    Qagg = QuantizedMatrix(rows, cols, nbits, 0)
    for s in range(k):
        start, n = cntk_amd.stripe_range(cols, s, k)
        if n:
            Qagg.ColumnSlice(start, n).buffer.copy_(Q[s].ColumnSlice(start, n).buffer)
    torch.cuda.synchronize()
    Out = Matrix(rows, cols)
    workers[0].impl.SynchronizeWithMainStream()
    workers[0].UnquantizeAsync(Qagg, Out)
    workers[0].WaitUnquantizeAsyncDone()
    torch.cuda.synchronize()
    return ([w.GetResidualMatrix().to_numpy() for w in workers], [s.to_numpy() for s in S], q_before,
            Qagg.to_numpy(), Out.to_numpy())


ALLREDUCE_SHAPES = [(429, 37, 8, 1, True), (2048, 64, 8, 1, False), (576, 20, 3, 4, False), (64, 5, 8, 1, False)]


@pytest.mark.parametrize("shape", ALLREDUCE_SHAPES, ids=lambda s: "%dx%d_k%d_b%d" % (s[0], s[1], s[2], s[3]))
@pytest.mark.parametrize("use_async", [False, True], ids=["mainstream", "dedicated"])
def test_simulated_allreduce(shape, use_async):
    """Two carried steps of the whole all-reduce. Every stage is checked against the oracle applied to the
    GPU's own previous stage (so each comparison sees identical inputs); the end-to-end aggregate is then
    compared with the free-standing oracle run."""
    rows, cols, k, nbits, zt = shape
    res_o = [np.zeros((rows, cols), np.float32, order="F") for _ in range(k)]
    sres_o = [np.zeros((rows, oracle.stripe_range(cols, s, k)[1]), np.float32, order="F") for s in range(k)]
    qcol = oracle.qcol_bytes(nbits, rows)
    rep = parity.Report()
    for step in range(2):
        say("all-reduce", shape, "async", use_async, "step", step)
        gs = [datagen.normal(datagen.case_seed(4, 1, step, w), rows, cols) for w in range(k)]
        res_in = [r.copy(order="F") for r in res_o]
        sres_in = [s.copy(order="F") for s in sres_o]
        res_g, sres_g, q1_g, qagg_g, out_g = simulated_allreduce_gpu(gs, res_in, sres_in, nbits, zt, use_async)
        _, aggs_o, qagg_o, out_o = parity.oracle_allreduce_staged(gs, res_o, sres_o, nbits, zt, threads=8)

        # stage 1: every worker's own quantization
        tainted = np.zeros(cols, dtype=bool)
        for w in range(k):
            parity.check_quantize(gs[w], res_in[w], q1_g[w], res_g[w], nbits, zt, report=rep)
            tainted |= rep.last_mismatch_cols
        # stage 2: each owner's stripe reduction, given the GPU's stage-1 buffers
        for s in range(k):
            start, n = oracle.stripe_range(cols, s, k)
            if n == 0:
                continue
            q_copy = [q.copy() for q in q1_g]
            s_copy = sres_in[s].copy(order="F")
            agg = oracle.stripe_reduce(q_copy, s, rows, cols, nbits, s_copy, zt, threads=8)
            parity.check_quantize(agg, sres_in[s], qagg_g[start * qcol:(start + n) * qcol], sres_g[s], nbits, zt,
                                  report=rep)
            tainted[start:start + n] |= rep.last_mismatch_cols
        # stage 3: unquantize is exact given the packed buffer
        parity.check_unquantize(qagg_g, rows, cols, nbits, out_g)
        worst, ntaint = parity.check_end_to_end(aggs_o, sres_in, qagg_g, sres_g, out_g, qagg_o, out_o, rows, cols, nbits, zt,
                                                tainted, report=rep)
        say("   aggregated gradient: max err %.3g of column scale; %d of %d columns hold a near-threshold flip"
            % (worst, ntaint, cols))
        assert ntaint <= max(1, cols // 100)
    say("  ", rep)


def test_config4_shape_one_stripe():
    """The 8-worker all-reduce workload at its real shape, one owner: 8 workers x 2048x9304, stripe 2048x1163."""
    rows, cols, k, nbits = 2048, 9304, 8, 1
    qz = MatrixQuantizerImpl.Create(0, False)
    zeros = np.zeros((rows, cols), np.float32, order="F")
    qs = []
    for w in range(k):
        g = datagen.normal(datagen.case_seed(4, 0, 0, w), rows, cols)
        qs.append(oracle.quantize(g, zeros, nbits, False, threads=8)[0])
    owner = 3
    start, n = oracle.stripe_range(cols, owner, k)
    assert (start, n) == (3 * 1163, 1163)
    sres = datagen.normal(4242, rows, n, 0.004)
    say("config 4 stripe", owner)
    q_new, s_new, agg = gpu_stripe_reduce(qz, qs, owner, rows, cols, nbits, sres, False)
    qs_o = [q.copy() for q in qs]
    s_o = sres.copy(order="F")
    agg_o = oracle.stripe_reduce(qs_o, owner, rows, cols, nbits, s_o, False, threads=8)
    assert parity.bits_equal(agg, agg_o)
    rep = parity.check_quantize(agg_o, sres, q_new, s_new, nbits, False)
    say("  ", rep)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
def test_stripe_reduce_on_strips_reports_workgroups_that_give_up(dtype):
    """A stripe taller than any workgroup holds is reduced by several workgroups per column that wait for each other's
    partial sums a bounded number of polls. With that number set to zero from the host every wait that does not find its
    record at the first look gives up: the kernel still runs to its end, such a column is left as it was (output stripe
    and stripe residual untouched), the wait reports the call as failed, and the handle goes on working afterwards."""
    # (seven strips per column, fewer than 8: the first look at the other strips' records then follows a strip's own sum at once)
    rows, n, k, nbits = (110000 if dtype == torch.float32 else 57000), 3, 2, 1
    npdt = np.float32 if dtype == torch.float32 else np.float64
    qz = MatrixQuantizerImpl.Create(0, False)
    assert qz.StripeReduceTakes(rows, n, nbits, False, dtype)
    zeros = np.zeros((rows, n), npdt, order="F")
    stripes = [oracle.quantize(datagen.normal(50 + w, rows, n, dtype=npdt), zeros, nbits, False, threads=8)[0] for w in range(k)]
    sres = datagen.normal(60, rows, n, 0.002, dtype=npdt)
    agg_o = oracle.unquantize(stripes[0], rows, n, nbits, dtype=npdt, threads=8)
    oracle.unquantize(stripes[1], rows, n, nbits, out=agg_o, add=True, threads=8)
    qcol = oracle.qcol_bytes(nbits, rows, npdt)

    def run():
        Qs = []
        for w in range(k):
            Q = QuantizedMatrix(rows, n, nbits, 0, dtype=dtype)
            Q.from_numpy(stripes[w])
            Qs.append(Q)
        S = Matrix.from_numpy(sres)
        Out = QuantizedMatrix(rows, n, nbits, 0, dtype=dtype)
        Out.buffer.fill_(0xA5)
        before = Out.to_numpy()
        torch.cuda.synchronize()
        qz.StripeReduceAsync(Qs, 0, S, Out, False)
        return before, Out, S

    qz._set_strip_spin_limit(0)
    before, Out, S = run()
    with pytest.raises(cntk_amd.QuantizerError, match="left as they were"):
        qz.WaitStripeReduceDone()
    torch.cuda.synchronize()
    q_after, s_after = Out.to_numpy(), S.to_numpy()
    untouched = 0
    for j in range(n):
        qa = q_after[j * qcol:(j + 1) * qcol]
        if np.array_equal(qa, before[j * qcol:(j + 1) * qcol]) and parity.bits_equal(s_after[:, j], sres[:, j]):
            untouched += 1
            continue
        parity.check_quantize(np.asfortranarray(agg_o[:, j:j + 1]), np.asfortranarray(sres[:, j:j + 1]), qa.copy(),
                              np.asfortranarray(s_after[:, j:j + 1]), nbits, False)
    say("   columns left untouched: %d of %d" % (untouched, n))
    assert untouched >= 1
    qz._set_strip_spin_limit(1 << 17)
    _, Out, S = run()
    qz.WaitStripeReduceDone()
    parity.check_quantize(agg_o, sres, Out.to_numpy(), S.to_numpy(), nbits, False)
