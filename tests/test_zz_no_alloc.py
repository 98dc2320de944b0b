"""cntkq_quantize_batch_noalloc (the gradient-set quantize that allocates nothing: its argument table lives in a fixed
array in the library's device image) gives exactly the bytes of cntkq_quantize_batch_async. Needs an MI355X.

Two calls in a row on one handle, the second with a smaller item list, so that the fixed array is reused while it
still holds the first call's table; then the first list again (its table must be uploaded anew), a second handle in
between (the array is shared by all handles of a GPU), a call recorded into a graph mixed with eager calls, and the limits."""
import sys

import numpy as np
import pytest
import torch

import cntk_amd
import datagen
import parity
from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

pytestmark = pytest.mark.gpu

LARGE = [(147, 64), (64, 64), (576, 64), (64, 256), (1, 5), (5, 1), (429, 37), (2048, 33), (2304, 5), (4608, 3), (9304, 1),
         (2048, 1), (0, 4), (1000, 1), (1152, 128), (4096, 6), (20000, 2), (512, 100), (33, 67), (14336, 1), (2048, 1100),
         (1028, 9), (12000, 2), (150001, 3)]
SMALL = [(429, 37), (64, 256), (2048, 7), (33, 67), (1152, 16)]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_pair(qz_ref, qz_new, shapes, seed, nbits, zt, rs=None):
    """Quantizes the same gradient set through both entry points; returns the new residuals (numpy) after checking that
    packed matrices and residuals agree bit for bit."""
    gs = [datagen.normal_with_outliers(seed + 100 * i, r, c) for i, (r, c) in enumerate(shapes)]
    if rs is None:
        rs = [datagen.normal(seed + 300 * i + 1, r, c, 0.003) for i, (r, c) in enumerate(shapes)]
    G = [Matrix.from_numpy(g) for g in gs]
    R1 = [Matrix.from_numpy(r) for r in rs]
    R2 = [Matrix.from_numpy(r) for r in rs]
    Q1 = [QuantizedMatrix(r, c, nbits, 0) for r, c in shapes]
    Q2 = [QuantizedMatrix(r, c, nbits, 0) for r, c in shapes]
    for q, (r, c) in zip(Q2, shapes):
        if r and c:  # (an empty matrix is a no-op for both entry points)
            q.buffer.fill_(0xA5)  # every byte of the packed matrices must be written by the call
    torch.cuda.synchronize()
    qz_ref.QuantizeBatchAsync([(g, r, q, r) for g, r, q in zip(G, R1, Q1)], zt)
    qz_ref.WaitQuantizeAsyncDone()
    qz_new.QuantizeBatchNoAlloc([(g, r, q, r) for g, r, q in zip(G, R2, Q2)], zt)
    qz_new.WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
    for i, (r, c) in enumerate(shapes):
        assert np.array_equal(Q1[i].to_numpy(), Q2[i].to_numpy()), ("packed", shapes[i], nbits, zt)
        assert parity.bits_equal(R1[i].to_numpy(), R2[i].to_numpy()), ("residual", shapes[i], nbits, zt)
        if r and c:
            parity.check_quantize(gs[i], rs[i], Q2[i].to_numpy(), R2[i].to_numpy(), nbits, zt)
    return [m.to_numpy() for m in R2]


@pytest.mark.parametrize("nbits,zt", [(1, False), (1, True), (4, False)])
def test_noalloc_equals_batch_call(nbits, zt):
    ref = MatrixQuantizerImpl.Create(0, False)
    new = MatrixQuantizerImpl.Create(0, False)
    other = MatrixQuantizerImpl.Create(0, False)
    say("no-alloc: large list", nbits, zt)
    rs = run_pair(ref, new, LARGE, 11, nbits, zt)
    say("no-alloc: smaller list right after", nbits, zt)
    run_pair(ref, new, SMALL, 23, nbits, zt)
    say("no-alloc: large list again, residual carried", nbits, zt)
    rs = run_pair(ref, new, LARGE, 37, nbits, zt, rs)
    say("no-alloc: another handle overwrites the array, then the first handle repeats its list", nbits, zt)
    run_pair(ref, other, SMALL, 41, nbits, zt)
    run_pair(ref, new, LARGE, 53, nbits, zt, rs)


def test_noalloc_same_list_twice_skips_nothing_visible():
    """The same item list (same addresses) called twice in a row: the second call may skip the upload; results must
    still be those of the batched call on the same inputs."""
    ref = MatrixQuantizerImpl.Create(0, False)
    new = MatrixQuantizerImpl.Create(0, False)
    shapes = SMALL
    gs = [datagen.normal(7 + i, r, c) for i, (r, c) in enumerate(shapes)]
    G = [Matrix.from_numpy(g) for g in gs]
    R1, R2 = [Matrix(r, c) for r, c in shapes], [Matrix(r, c) for r, c in shapes]
    Q1, Q2 = [QuantizedMatrix(r, c, 1, 0) for r, c in shapes], [QuantizedMatrix(r, c, 1, 0) for r, c in shapes]
    items1 = ref.PrepareQuantizeBatch([(g, r, q, r) for g, r, q in zip(G, R1, Q1)])
    items2 = new.PrepareQuantizeBatch([(g, r, q, r) for g, r, q in zip(G, R2, Q2)])
    for step in range(4):
        say("no-alloc: repeated list, step", step)
        ref.QuantizeBatchAsync(items1, False)
        new.QuantizeBatchNoAlloc(items2, False)
        ref.WaitQuantizeAsyncDone()
        new.WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        for i in range(len(shapes)):
            assert np.array_equal(Q1[i].to_numpy(), Q2[i].to_numpy()), ("packed", shapes[i], step)
            assert parity.bits_equal(R1[i].to_numpy(), R2[i].to_numpy()), ("residual", shapes[i], step)


class _Pair:
    """One gradient set twice: for the no-alloc entry point and for the batched call it must equal."""

    def __init__(self, shapes, nbits, seed):
        self.shapes, self.nbits = shapes, nbits
        self.gen = torch.Generator(device="cuda:0")
        self.gen.manual_seed(seed)
        self.G = [Matrix(r, c) for r, c in shapes]
        self.R = [[Matrix(r, c) for r, c in shapes] for _ in range(2)]
        self.Q = [[QuantizedMatrix(r, c, nbits, 0) for r, c in shapes] for _ in range(2)]
        self.items = [MatrixQuantizerImpl.PrepareQuantizeBatch([(g, r, q, r) for g, r, q in zip(self.G, self.R[k], self.Q[k])])
                      for k in range(2)]

    def new_gradients(self):
        for g in self.G:
            g.data.copy_(torch.randn(g.data.numel(), generator=self.gen, device="cuda:0") * 0.01)
        for q in self.Q[0]:
            q.buffer.fill_(0xA5)
        torch.cuda.synchronize()

    def check(self, what):
        torch.cuda.synchronize()
        for i, shape in enumerate(self.shapes):
            assert torch.equal(self.Q[0][i].buffer, self.Q[1][i].buffer), (what, "packed", shape)
            assert torch.equal(self.R[0][i].data.view(torch.int32), self.R[1][i].data.view(torch.int32)), (what, "residual", shape)


def test_noalloc_recorded_call_among_eager_calls():
    """A recorded call has not run when the recording ends, and its replays rewrite the shared array at times the
    library does not see: an eager call may never take its table for uploaded because of either. List A is recorded;
    then: eager A before the first replay, replay, eager B, replay, eager B again -- every result equal to the batched
    call's on the same inputs, residuals carried."""
    nbits = 1
    new, ref = MatrixQuantizerImpl.Create(0, False), MatrixQuantizerImpl.Create(0, False)
    a = _Pair([(429, 37), (64, 256), (2048, 7), (33, 67), (1152, 16)], nbits, 901)
    b = _Pair([(147, 64), (2048, 33), (576, 64), (4608, 3)], nbits, 902)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    a.new_gradients()
    with torch.cuda.graph(graph, stream=side):
        new.SetMainStream(torch.cuda.current_stream().cuda_stream)
        new.QuantizeBatchNoAlloc(a.items[0], False)
    new.SetMainStream(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    def eager(pair, what):
        say("no-alloc:", what)
        pair.new_gradients()
        new.QuantizeBatchNoAlloc(pair.items[0], False)
        ref.QuantizeBatchAsync(pair.items[1], False)
        new.WaitQuantizeAsyncDone()
        ref.WaitQuantizeAsyncDone()
        pair.check(what)

    def replay(what):
        say("no-alloc:", what)
        a.new_gradients()
        graph.replay()
        ref.QuantizeBatchAsync(a.items[1], False)
        ref.WaitQuantizeAsyncDone()
        a.check(what)

    eager(a, "eager call with the recorded list before the first replay")
    replay("first replay")
    eager(b, "eager call with another list")
    replay("second replay")
    eager(b, "the other list again, right after a replay")
    replay("third replay")
    eager(a, "the recorded list, eager, after the replays")


def test_noalloc_limits():
    qz = MatrixQuantizerImpl.Create(0, False)
    n = 257  # one more than CNTKQ_NOALLOC_MAX_ITEMS
    G = [Matrix(8, 2) for _ in range(n)]
    R = [Matrix(8, 2) for _ in range(n)]
    Q = [QuantizedMatrix(8, 2, 1, 0) for _ in range(n)]
    with pytest.raises(cntk_amd.QuantizerLogicError, match="exceed the limit"):
        qz.QuantizeBatchNoAlloc([(g, r, q, r) for g, r, q in zip(G, R, Q)], False)
    # at the limit it runs
    qz.QuantizeBatchNoAlloc([(g, r, q, r) for g, r, q in zip(G[:256], R[:256], Q[:256])], False)
    qz.WaitQuantizeAsyncDone()
    torch.cuda.synchronize()
