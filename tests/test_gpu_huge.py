"""Matrices of more than 2^32 elements (byte offsets beyond 16 GiB): every index in the kernels and in the C ABI must be
64 bits wide where it counts elements or bytes of the whole matrix. Checked through properties that do not depend on
the size (conservation of the error feedback, chunk by chunk on the device) and against the CPU oracle on a few
columns at the start, in the middle and at the very end of the matrix. Needs an MI355X (about 60 GB of device memory)."""
import sys

import numpy as np
import pytest
import torch

import datagen
import oracle
import parity
from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def columns_to_numpy(flat, rows, first, n):
    return np.asfortranarray(flat[first * rows:(first + n) * rows].cpu().numpy().reshape((rows, n), order="F"))


CASES = [
    # rows, cols, nbits: 4.5e9 elements each
    (4096, 1100000, 1),   # register kernel with 256 threads, QWord-major decoder
    (100000, 45000, 1),   # register kernel with 1024 threads, row-major decoder
    (429, 10500000, 4),   # tile kernel and tile decoder
]


@pytest.mark.parametrize("rows,cols,nbits", CASES, ids=["%dx%d_b%d" % c for c in CASES])
def test_more_than_2_to_32_elements(rows, cols, nbits):
    n = rows * cols
    assert n > 2 ** 32
    free, _ = torch.cuda.mem_get_info(0)
    need = 3 * 4 * n + 2 * n // 8 * nbits + (8 << 30)
    if free < need:
        pytest.skip("needs %.0f GB of free device memory, %.0f GB are free" % (need / 1e9, free / 1e9))
    say("huge matrix", rows, cols, nbits, "elements", n)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(90, nbits))
    g = torch.empty(n, device="cuda:0", dtype=torch.float32)
    step = 1 << 28
    for o in range(0, n, step):  # in pieces: the generator's own temporaries stay small
        g[o:o + step].normal_(0.0, 0.01, generator=gen)
    G, R, Out = Matrix(rows, cols, 0, g), Matrix(rows, cols), Matrix(rows, cols)
    Q = QuantizedMatrix(rows, cols, nbits, 0)
    assert Q.GetSize() == oracle.qcol_bytes(nbits, rows) * cols
    qz = MatrixQuantizerImpl.Create(0, False)
    qz.QuantizeAsync(G, R, Q, R, False)   # residual in place, zero at the start
    qz.WaitQuantizeAsyncDone()
    qz.UnquantizeAsync(Q, Out)
    qz.WaitUnquantizeAsyncDone()
    torch.cuda.synchronize()
    # conservation: g (+ 0) == unquantize(q) + residual up to the rounding of the two fp32 operations, everywhere
    bad = 0
    for o in range(0, n, step):
        v, back, r = g[o:o + step], Out.data[o:o + step], R.data[o:o + step]
        bad += int(((v - (back + r)).abs() > 4e-7 * (v.abs() + back.abs()) + 1e-37).sum().item())
    assert bad == 0, "%d elements violate the conservation law" % bad
    # the oracle on columns from both ends and the middle
    qcol = oracle.qcol_bytes(nbits, rows)
    rep = parity.Report()
    for first in (0, cols // 2 - 1, cols - 3):
        gc = columns_to_numpy(g, rows, first, 3)
        qc = Q.buffer[first * qcol:(first + 3) * qcol].cpu().numpy()
        rc = columns_to_numpy(R.data, rows, first, 3)
        oc = columns_to_numpy(Out.data, rows, first, 3)
        parity.check_quantize(gc, np.zeros_like(gc, order="F"), qc, rc, nbits, False, report=rep, strict=True)
        parity.check_unquantize(qc, rows, 3, nbits, oc)
    say("   ", rep)
    del g, G, R, Out, Q
    torch.cuda.empty_cache()
