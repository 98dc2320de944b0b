"""cntkq_quantize_batch_noalloc (the gradient-set quantize that allocates nothing: its argument table lives in a fixed
array in the library's device image) gives exactly the bytes of cntkq_quantize_batch_async. Needs an MI355X.

Two calls in a row on one handle, the second with a smaller item list, so that the fixed array is reused while it
still holds the first call's table; then the first list again (its table must be uploaded anew), a second handle in
between (the array is shared by all handles of a GPU), and the limits."""
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
         (1028, 9), (12000, 2)]
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
