"""The quantized all-reduce on torch gradient tensors (cntk_amd.torch_hook): K workers in one process against the CPU
oracle's all-reduce, stage by stage; the DistributedDataParallel hook on a stand-in bucket and, in a child process,
under a real one-rank process group. Needs an MI355X."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import datagen
import oracle
import parity
from cntk_amd import QuantizerLogicError
from cntk_amd.torch_hook import (InProcessGroup, QuantizedGradientAggregator, make_hook_state, matrix_view,
                                 quantized_allreduce_hook)

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def say(*a):
    print(*a, flush=True)


def as_matrix(t):
    """(rows, cols) Fortran-order numpy view of what matrix_view makes of the tensor."""
    m = matrix_view(t)
    return np.asfortranarray(t.detach().cpu().numpy().reshape(-1).reshape((m.rows, m.cols), order="F"))


def flat_matrix(flat, rows, cols):
    return np.asfortranarray(flat.detach().cpu().numpy().reshape((rows, cols), order="F"))


def packed_of(agg, buf, slot_of_owner, i, K):
    """Gradient i's whole packed matrix, assembled from the owners' stripes in `buf`."""
    parts = []
    for s in range(K):
        if agg._stripe[s][i][1]:
            parts.append(agg._packed(buf, slot_of_owner(s), s, i).to_numpy())
    return np.concatenate(parts) if parts else np.zeros(0, np.uint8)


SHAPES = [((96, 300), torch.float32),       # Linear weight: 96 columns of 300 rows
          ((40, 16, 3, 3), torch.float32),  # convolution: 40 columns of 144 rows
          ((96,), torch.float32),           # bias: one column
          ((3, 2048), torch.float32),       # fewer columns than workers: some stripes are empty
          ((24, 130), torch.float64),
          ((2, 110000), torch.float32),     # columns too tall for the fused stripe reduction: the reference's call sequence
          ((3, 52000), torch.float64)]      # the same for doubles (limit 51184 rows)


@pytest.mark.parametrize("K,nbits,zt", [(1, 1, True), (4, 1, False), (4, 1, True), (3, 4, False), (8, 2, False)])
def test_in_process_workers_against_the_oracle(K, nbits, zt):
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(70 + K, nbits))
    group = InProcessGroup(K, nbits, zt)
    rep = parity.Report()
    for step in range(3):
        say("torch hook K=%d nbits=%d zt=%s step %d" % (K, nbits, zt, step))
        grads = [[torch.randn(shape, generator=gen, device="cuda:0", dtype=dt) * 0.01 for shape, dt in SHAPES]
                 for _ in range(K)]
        gs = [[as_matrix(g) for g in grads[w]] for w in range(K)]
        if step == 0:
            res_in = [[np.zeros_like(m) for m in gs[w]] for w in range(K)]
            sres_in = None
        else:
            res_in = [[flat_matrix(group.workers[w]._residual[i], *gs[w][i].shape) for i in range(len(SHAPES))] for w in range(K)]
        # the phases one by one, as InProcessGroup.aggregate runs them, with the packed buffers read in between
        for w in range(K):
            group.workers[w].quantize(grads[w])
        torch.cuda.synchronize()
        W0 = group.workers[0]
        if sres_in is None:
            sres_in = [[np.zeros((gs[0][i].shape[0], W0._stripe[s][i][1]), gs[0][i].dtype, order="F") for i in range(len(SHAPES))]
                       for s in range(K)]
        else:
            sres_in = [[flat_matrix(group.workers[s]._stripe_residual[i], gs[0][i].shape[0], W0._stripe[s][i][1])
                        for i in range(len(SHAPES))] for s in range(K)]
        q1 = [[packed_of(group.workers[w], group.workers[w]._send, lambda s: s, i, K) for i in range(len(SHAPES))] for w in range(K)]
        res_out = [[flat_matrix(group.workers[w]._residual[i], *gs[w][i].shape) for i in range(len(SHAPES))] for w in range(K)]
        group.aggregate_after_quantize()
        torch.cuda.synchronize()
        for i, (shape, dt) in enumerate(SHAPES):
            rows, cols = gs[0][i].shape
            qcol = oracle.qcol_bytes(nbits, rows, gs[0][i].dtype)
            # every worker must hold the same aggregated gradient
            outs = [as_matrix(grads[w][i]) for w in range(K)]
            for w in range(1, K):
                assert parity.bits_equal(outs[0], outs[w]), "workers disagree on gradient %d" % i
            qagg_g = packed_of(W0, W0._gathered if K > 1 else W0._mine, lambda s: s, i, K)
            sres_out = [flat_matrix(group.workers[s]._stripe_residual[i], rows, W0._stripe[s][i][1]) for s in range(K)]
            ro = [r[i].copy(order="F") for r in res_in]
            so = [sres_in[s][i].copy(order="F") for s in range(K)]
            _, aggs_o, qagg_o, out_o = parity.oracle_allreduce_staged([gs[w][i] for w in range(K)], ro, so, nbits, zt, threads=8)
            tainted = np.zeros(cols, dtype=bool)
            for w in range(K):
                parity.check_quantize(gs[w][i], res_in[w][i], q1[w][i], res_out[w][i], nbits, zt, threads=8, report=rep, strict=rows <= 16384)
                tainted |= rep.last_mismatch_cols
            aggs_g = [None] * K
            for s in range(K):
                start, n = oracle.stripe_range(cols, s, K)
                if n == 0:
                    continue
                q_copy = [q[i].copy() for q in q1]
                s_copy = sres_in[s][i].copy(order="F")
                agg = oracle.stripe_reduce(q_copy, s, rows, cols, nbits, s_copy, zt, threads=8)
                aggs_g[s] = agg
                parity.check_quantize(agg, sres_in[s][i], qagg_g[start * qcol:(start + n) * qcol], sres_out[s], nbits, zt,
                                      threads=8, report=rep, strict=rows <= 16384)
                tainted[start:start + n] |= rep.last_mismatch_cols
            parity.check_unquantize(qagg_g, rows, cols, nbits, outs[0], threads=8)
            parity.check_end_to_end(aggs_o, [sres_in[s][i] for s in range(K)], qagg_g, sres_out, outs[0], qagg_o, out_o, rows, cols,
                                    nbits, zt, tainted, threads=8, report=rep, aggs_gpu=aggs_g)
            if rows <= 16384:  # (a column of 100000 elements is likelier than not to hold one element at a threshold)
                assert tainted.sum() <= max(1, cols // 50)
    say("torch hook K=%d nbits=%d:" % (K, nbits), rep)


def test_aggregate_equals_the_phases_and_reset_state():
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(77))
    a, b = QuantizedGradientAggregator(1, True), QuantizedGradientAggregator(1, True)
    for step in range(2):
        g = [torch.randn(shape, generator=gen, device="cuda:0", dtype=dt) * 0.01 for shape, dt in SHAPES]
        h = [x.clone() for x in g]
        a.aggregate(g)
        b.quantize(h), b.exchange_stripes(), b.reduce(), b.exchange_reduced(), b.unquantize()
        torch.cuda.synchronize()
        for x, y in zip(g, h):
            assert torch.equal(x, y)
    assert any(float(r.abs().max()) > 0 for r in a._residual)
    a.reset_state()
    assert all(float(r.abs().max()) == 0 for r in a._residual + a._stripe_residual)
    with pytest.raises(QuantizerLogicError):
        a.aggregate(g[:-1])
    with pytest.raises(QuantizerLogicError):
        QuantizedGradientAggregator().aggregate([torch.zeros(4, 4, device="cuda:0", dtype=torch.float16)])


class FakeBucket:
    """What the hook uses of torch.distributed.GradBucket: views of one flat buffer."""

    def __init__(self, index, shapes, gen):
        n = sum(int(np.prod(s)) for s in shapes)
        self._buf = torch.randn(n, generator=gen, device="cuda:0") * 0.01
        self._views, o = [], 0
        for s in shapes:
            k = int(np.prod(s))
            self._views.append(self._buf[o:o + k].view(s))
            o += k
        self._index = index

    def index(self):
        return self._index

    def buffer(self):
        return self._buf

    def gradients(self):
        return self._views


def test_hook_on_a_stand_in_bucket():
    """Gradients at arbitrary 4-byte offsets inside the bucket's buffer; one aggregator (and residual set) per bucket."""
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(78))
    shapes = [(33, 301), (33,), (7, 33), (7,)]
    state = make_hook_state(None, nbits=1, zero_threshold_for_1bit=True)
    ref = QuantizedGradientAggregator(1, True)
    for step in range(3):
        bucket = FakeBucket(0, shapes, gen)
        alone = [v.clone() for v in bucket.gradients()]
        fut = quantized_allreduce_hook(state, bucket)
        ref.aggregate(alone)
        torch.cuda.synchronize()
        assert fut.done() and fut.value().data_ptr() == bucket.buffer().data_ptr()
        for v, x in zip(bucket.gradients(), alone):
            # same arithmetic on differently aligned copies: kernels may differ in summation order, so compare within
            # the bound tolerance of the column scale
            scale = float(x.abs().max())
            assert float((v - x).abs().max()) <= 1e-5 * scale
    assert list(state.aggregators) == [0]
    other = FakeBucket(1, shapes[:2], gen)
    quantized_allreduce_hook(state, other)
    torch.cuda.synchronize()
    assert sorted(state.aggregators) == [0, 1]


def test_hook_under_distributed_data_parallel():
    """A real DistributedDataParallel model on a one-rank process group, in a child process (a process group is
    process-wide state). Skipped only if the process group itself cannot be created on this machine."""
    p = subprocess.run([sys.executable, "-u", os.path.join(HERE, "ddp_hook_worker.py")], capture_output=True, text=True, timeout=240)
    say(p.stdout[-2000:], p.stderr[-2000:])
    lines = [ln for ln in p.stdout.splitlines() if ln.startswith("{")]
    assert lines, "the worker printed no result (exit code %d)" % p.returncode
    out = json.loads(lines[-1])
    if out.get("skipped"):
        pytest.skip(out["skipped"])
    assert p.returncode == 0
    assert out["steps"] == 3 and out["max_err"] <= 1e-5 and out["aggregators"] >= 1 and out["transport_ok"]


def test_aggregate_replayed_from_a_hip_graph():
    """The three batched launches of a step captured once (after a warm-up step has built the argument tables) and
    replayed: every replay, with eager work and synchronisations in between, must give the bytes of an eager twin
    that sees the same gradients, residuals carried from replay to replay."""
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(79))
    shapes = [s for s, dt in SHAPES if dt == torch.float32] + [(2048, 512), (9304, 64)]
    fresh = lambda: [torch.randn(s, generator=gen, device="cuda:0") * 0.01 for s in shapes]
    graphed, twin = QuantizedGradientAggregator(1, True), QuantizedGradientAggregator(1, True)
    g = fresh()
    graphed.aggregate(g)  # warm-up: buffers, residuals and the cached tables of the batched calls come into being
    torch.cuda.synchronize()
    graphed.reset_state()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        graphed.aggregate(g)
    graphed.reset_state()
    torch.cuda.synchronize()
    for step in range(5):
        new = fresh()
        ref = [x.clone() for x in new]
        twin.aggregate(ref)
        for a, b in zip(g, new):
            a.copy_(b)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(g, ref)):
            assert torch.equal(a, b), "replay %d, gradient %d differs from the eager step" % (step, i)
        for a, b in zip(graphed._residual + graphed._stripe_residual, twin._residual + twin._stripe_residual):
            assert torch.equal(a, b), "replay %d: residuals differ from the eager step's" % step


def test_average_divides_the_sum_by_the_number_of_workers():
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(82))
    shapes = [(96, 300), (96,), (24, 130)]
    src = [[torch.randn(s, generator=gen, device="cuda:0") * 0.01 for s in shapes] for _ in range(4)]
    summed = [[x.clone() for x in w] for w in src]
    averaged = [[x.clone() for x in w] for w in src]
    InProcessGroup(4, 1, True, average=False).aggregate(summed)
    InProcessGroup(4, 1, True, average=True).aggregate(averaged)
    torch.cuda.synchronize()
    for w in range(4):
        for a, b in zip(summed[w], averaged[w]):
            assert torch.equal(a / 4, b)


def test_caller_owned_residues():
    """The v2 communicator's shape of the call: the learner owns the residual tensors and hands them in; the result and
    the residues are those of an aggregator that keeps its own."""
    from cntk_amd.torch_hook import stripe_residue_numel

    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(83))
    shapes = [(96, 300), (96,), (24, 130)]
    res = [torch.zeros(int(np.prod(s)), device="cuda:0") for s in shapes]
    sres = [torch.zeros(stripe_residue_numel(torch.empty(s), 0, 1), device="cuda:0") for s in shapes]
    mine, own = QuantizedGradientAggregator(1, True, residues=res, stripe_residues=sres), QuantizedGradientAggregator(1, True)
    for step in range(3):
        g = [torch.randn(s, generator=gen, device="cuda:0") * 0.01 for s in shapes]
        h = [x.clone() for x in g]
        mine.aggregate(g)
        own.aggregate(h)
        torch.cuda.synchronize()
        for a, b in zip(g, h):
            assert torch.equal(a, b)
    for a, b in zip(res + sres, own._residual + own._stripe_residual):
        assert torch.equal(a, b) and float(a.abs().max()) > 0
    with pytest.raises(QuantizerLogicError):
        QuantizedGradientAggregator(1, True, residues=res[:2]).aggregate(g)
