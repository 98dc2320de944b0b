"""QuantizedMatrix.Decode / Print of the Python mirror read a packed matrix by its layout alone; checked on the CPU against
the oracle's codes and reconstructed values (packed matrices in host memory need no GPU)."""
import io

import numpy as np
import pytest
import torch

import cntk_amd
import datagen
import oracle
from cntk_amd import QuantizedMatrix


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("rows,cols,nbits", [(37, 5, 1), (37, 5, 2), (100, 3, 4), (70, 4, 8), (33, 2, 16), (9, 3, 32), (1, 4, 1), (300, 2, 1)])
def test_decode_matches_the_oracle(dtype, rows, cols, nbits):
    tdt = torch.float64 if dtype == np.float64 else torch.float32
    g = datagen.normal(5 + rows + nbits, rows, cols, dtype=dtype)
    g[:, cols - 1] = 0  # an all-zero column: bounds 0, every code 1 at one bit
    q, _ = oracle.quantize(g, np.zeros_like(g, order="F"), nbits, False, threads=2)
    Q = QuantizedMatrix(rows, cols, nbits, cntk_amd.CPUDEVICE, dtype=tdt)
    Q.from_numpy(q)
    lower, upper, codes, values = Q.Decode(0, rows - 1, 0, cols - 1)
    lo_o, hi_o = oracle.headers(q, rows, cols, nbits, dtype=dtype)
    assert np.array_equal(lower, lo_o) and np.array_equal(upper, hi_o)
    assert np.array_equal(codes.astype(np.uint64), oracle.codes(q, rows, cols, nbits, dtype=dtype).astype(np.uint64))
    out_o = oracle.unquantize(q, rows, cols, nbits, threads=2, dtype=dtype)
    assert np.array_equal(values.view(np.uint8), np.ascontiguousarray(out_o).view(np.uint8)), "reconstructed values differ"
    # a sub-range is the same numbers
    if rows > 4 and cols > 2:
        _, _, c2, v2 = Q.Decode(2, 4, 1, 2)
        assert np.array_equal(c2, codes[2:5, 1:3]) and np.array_equal(v2, values[2:5, 1:3])
    with pytest.raises(cntk_amd.QuantizerLogicError):
        Q.Decode(0, rows, 0, 0)


def test_print_format():
    g = np.asfortranarray(np.array([[0.1], [-0.2], [0.3], [-0.4], [0.05]], np.float32))
    q, _ = oracle.quantize(g, np.zeros_like(g, order="F"), 1, False, threads=1)
    Q = QuantizedMatrix(5, 1, 1, cntk_amd.CPUDEVICE)
    Q.from_numpy(q)
    buf = io.StringIO()
    Q.Print("grad", 0, 4, 0, 0, file=buf)
    text = buf.getvalue()
    assert "###### grad (5, 1) ######" in text and "Print Range (0:4, 0:0)" in text
    assert "Lower=-0.46" in text and "Upper=0.40" in text  # the hand example: lower -0.462, upper 0.402
    lines = [ln for ln in text.splitlines() if "(" in ln and "Print" not in ln and "#" not in ln]
    assert [int(ln.split()[0]) for ln in lines] == [1, 0, 1, 0, 1]  # bits 0b10101
