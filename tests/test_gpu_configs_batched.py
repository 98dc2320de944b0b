"""The benchmark workloads through the calls that `bench.py --config N` measures: the gradient-set calls on the real
16-, 161- and 6-matrix lists, and the three calls of the simulated 8-worker all-reduce. Needs an MI355X.

Every step is checked twice: against the CPU oracle on the very (gradient, residual-in) the device saw (the 1e-6 threshold
rule taken literally, columns resting on the float64 bounds counted and bounded per workload), and byte for byte against
the per-matrix / per-owner calls of the boundary on the same inputs. Residuals are carried on the device over three
steps. (Source/1BitSGD/AllReduceDistGradAggregator.h:288-300, 339-436, 517-531 are the loops these calls replace.)
"""
import sys

import numpy as np
import pytest
import torch

import cntk_amd
import oracle
import parity
from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix
from cntk_amd.config_bench import LSTM_LM, SPEECH_DNN, resnet50_shapes

pytestmark = pytest.mark.gpu

STEPS = 3


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def same_bits(a, b):
    return torch.equal(a.view(torch.int32), b.view(torch.int32))


def gradient(gen, rows, cols, kind):
    n = rows * cols
    if kind == "student_t3":
        z = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32)
        chi = torch.randn(3, n, generator=gen, device="cuda:0", dtype=torch.float32).square_().sum(0)
        return z / torch.sqrt(chi / 3.0) * 1e-3
    if kind == "outliers":
        a = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32) * 0.01
        return torch.where(torch.rand(n, generator=gen, device="cuda:0") < 0.01, a * 50.0, a)
    g = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32) * 0.01
    if kind == "sparse_columns" and rows >= 100000:
        keep = (torch.rand(cols, generator=gen, device="cuda:0") >= 0.9).to(torch.float32)
        g.view(cols, rows).mul_(keep[:, None])
    return g


def as_np(flat, rows, cols):
    return np.asfortranarray(flat.detach().cpu().numpy().reshape((rows, cols), order="F"))


def gradient_set(shapes, nbits, zt, kind, seed, fallback_bound, label):
    """quantize the set + unquantize the set, one gradient-set call each (what `bench.py --config 2 / 3 / 5` times),
    beside the per-matrix calls on the same inputs."""
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(seed)
    batched, single = MatrixQuantizerImpl.Create(0, False), MatrixQuantizerImpl.Create(0, False)
    n = len(shapes)
    G = [Matrix(r, c) for r, c in shapes]
    R = [[Matrix(r, c) for r, c in shapes] for _ in range(2)]
    Q = [[QuantizedMatrix(r, c, nbits, 0) for r, c in shapes] for _ in range(2)]
    Out = [[Matrix(r, c) for r, c in shapes] for _ in range(2)]
    pq = batched.PrepareQuantizeBatch([(G[i], R[0][i], Q[0][i], R[0][i]) for i in range(n)])
    pu = batched.PrepareUnquantizeBatch([(Q[0][i], Out[0][i]) for i in range(n)])
    rep = parity.Report()
    for step in range(STEPS):
        say(label, "step", step)
        for i, (r, c) in enumerate(shapes):
            G[i].data.copy_(gradient(gen, r, c, kind))
            Q[0][i].buffer.fill_(0xA5)
            Out[0][i].data.fill_(float("nan"))
        r_in = [m.data.clone() for m in R[0]]
        torch.cuda.synchronize()
        batched.QuantizeBatchAsync(pq, zt)
        batched.UnquantizeBatchAsync(pu, False)
        batched.WaitQuantizeAsyncDone()
        batched.WaitUnquantizeAsyncDone()
        for i in range(n):
            single.QuantizeAsync(G[i], R[1][i], Q[1][i], R[1][i], zt)
            single.UnquantizeAsync(Q[1][i], Out[1][i])
        single.WaitUnquantizeAsyncDone()
        torch.cuda.synchronize()
        for i, (r, c) in enumerate(shapes):
            assert torch.equal(Q[0][i].buffer, Q[1][i].buffer), (label, step, "packed matrix differs from the per-matrix call", i, (r, c))
            assert same_bits(R[0][i].data, R[1][i].data), (label, step, "residual differs from the per-matrix call", i, (r, c))
            assert same_bits(Out[0][i].data, Out[1][i].data), (label, step, "output differs from the per-matrix call", i, (r, c))
            q = Q[0][i].to_numpy()
            parity.check_quantize(as_np(G[i].data, r, c), as_np(r_in[i], r, c), q, R[0][i].to_numpy(), nbits, zt, threads=16,
                                  report=rep, strict=True)
            parity.check_unquantize(q, r, c, nbits, Out[0][i].to_numpy(), threads=16)
    say(label + ":", rep)
    say(label + ": fallback columns = %d of %d" % (rep.fallback_cols, rep.cols))
    rep.assert_fallback_at_most(fallback_bound)


@pytest.mark.parametrize("zt", [False, True], ids=["meanThr", "zeroThr"])
def test_config2_speech_dnn_gradient_set_calls(zt):
    assert len(SPEECH_DNN) == 16
    gradient_set(SPEECH_DNN, 1, zt, "student_t3", 0xC2 + int(zt), 0, "config 2 (gradient-set calls) zeroThr=%s" % zt)


@pytest.mark.parametrize("nbits", [2, 4, 8])
def test_config3_resnet50_gradient_set_calls(nbits):
    shapes = resnet50_shapes()
    assert len(shapes) == 161 and sum(r * c for r, c in shapes) == 25557032
    gradient_set(shapes, nbits, False, "outliers", 0xC3 + nbits, 0, "config 3 (gradient-set calls) nbits=%d" % nbits)


def test_config5_lstm_lm_gradient_set_calls():
    assert len(LSTM_LM) == 6
    # (the 100000-row embedding columns that received a gradient are long enough for the oracle's own fp32 sum to use up
    # the tolerance: the same bound as the per-matrix test of this workload)
    gradient_set(LSTM_LM, 1, True, "sparse_columns", 0xC5, 8, "config 5 (gradient-set calls)")


def test_config4_allreduce_three_calls():
    """8 workers x 2048 x 9304 in one GPU's memory, as `bench.py --config 4` issues it: all workers' quantizations in one
    call, all owners' stripe reductions in one call (an owner per item, each writing over its own packed stripe), the
    packed aggregate unquantized into worker 0's gradient from the owners' stripes in one call."""
    rows, cols, k, nbits, zt = 2048, 9304, 8, 1, False
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(0xC4)
    ranges = [cntk_amd.stripe_range(cols, s, k) for s in range(k)]
    qcol = oracle.qcol_bytes(nbits, rows)

    class Side:
        def __init__(self):
            self.qz = MatrixQuantizerImpl.Create(0, False)
            self.G = [Matrix(rows, cols) for _ in range(k)]
            self.R = [Matrix(rows, cols) for _ in range(k)]
            self.Q = [QuantizedMatrix(rows, cols, nbits, 0) for _ in range(k)]
            self.S = [Matrix(rows, n) for _, n in ranges]
            self.stripes = [[self.Q[w].ColumnSlice(start, n) for w in range(k)] for start, n in ranges]
            self.views = [(self.stripes[s][s], self.G[0].ColumnSlice(start, n)) for s, (start, n) in enumerate(ranges)]

    a, b = Side(), Side()
    pq = a.qz.PrepareQuantizeBatch([(a.G[w], a.R[w], a.Q[w], a.R[w]) for w in range(k)])
    ps = a.qz.PrepareStripeReduceBatch([(a.stripes[s], a.S[s], a.stripes[s][s], None) for s in range(k)])
    pu = a.qz.PrepareUnquantizeBatch(a.views)
    owners = list(range(k))
    rep = parity.Report()
    for step in range(STEPS):
        say("config 4 (three calls) step", step)
        for w in range(k):
            g = gradient(gen, rows, cols, "normal")
            a.G[w].data.copy_(g)
            b.G[w].data.copy_(g)
        gs = [m.to_numpy() for m in a.G]
        res_in = [m.to_numpy() for m in a.R]
        sres_in = [m.to_numpy() for m in a.S]
        torch.cuda.synchronize()
        # the three calls
        a.qz.QuantizeBatchAsync(pq, zt)
        a.qz.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        q1 = [q.to_numpy() for q in a.Q]  # (the owners' reductions write over their own stripes: looked at before)
        a.qz.StripeReduceBatchAsync(ps, owners, zt)
        a.qz.UnquantizeBatchAsync(pu, False)
        a.qz.WaitStripeReduceDone()
        a.qz.WaitUnquantizeAsyncDone()
        # the same through one call per worker, per owner and per stripe
        for w in range(k):
            b.qz.QuantizeAsync(b.G[w], b.R[w], b.Q[w], b.R[w], zt)
        for s in range(k):
            b.qz.StripeReduceAsync(b.stripes[s], s, b.S[s], b.stripes[s][s], zt)
        for q, out in b.views:
            b.qz.UnquantizeAsync(q, out)
        b.qz.WaitUnquantizeAsyncDone()
        torch.cuda.synchronize()
        for w in range(k):
            assert torch.equal(a.Q[w].buffer, b.Q[w].buffer), (step, "packed matrix differs from the per-call sequence", w)
            assert same_bits(a.R[w].data, b.R[w].data), (step, "residual differs from the per-call sequence", w)
            assert same_bits(a.S[w].data, b.S[w].data), (step, "stripe residual differs from the per-call sequence", w)
        assert same_bits(a.G[0].data, b.G[0].data), (step, "aggregated gradient differs from the per-call sequence")
        # against the oracle, stage by stage on what the device saw
        for w in range(k):
            parity.check_quantize(gs[w], res_in[w], q1[w], a.R[w].to_numpy(), nbits, zt, threads=16, report=rep, strict=True)
        qagg = np.empty(qcol * cols, np.uint8)
        for s, (start, n) in enumerate(ranges):
            s_copy = sres_in[s].copy(order="F")
            agg = oracle.stripe_reduce([q.copy() for q in q1], s, rows, cols, nbits, s_copy, zt, threads=16)
            q_s = a.stripes[s][s].to_numpy()
            parity.check_quantize(agg, sres_in[s], q_s, a.S[s].to_numpy(), nbits, zt, threads=16, report=rep, strict=True)
            qagg[start * qcol:(start + n) * qcol] = q_s
        parity.check_unquantize(qagg, rows, cols, nbits, a.G[0].to_numpy(), threads=16)
    say("config 4 (three calls):", rep)
    say("config 4 (three calls): fallback columns = %d of %d" % (rep.fallback_cols, rep.cols))
    rep.assert_fallback_at_most(0)
