"""The comparison rules of tests/parity.py themselves, on the CPU: what they accept, what they refuse, and what they
count. The inputs are the recorded case where the oracle's own term-by-term fp32 sum misses the float64 bounds by more
than the 1e-5 tolerance at only 6144 rows (a K = 2 stripe sum of one-bit reconstructions: four distinct values)."""
import numpy as np
import pytest

import datagen
import oracle
import parity

ROWS, COLS = 6144, 32


def packed_with_bounds(s, lower, upper):
    """The packed matrix an implementation with the given column bounds produces (codes and residual from the oracle's
    element arithmetic under those bounds)."""
    rows, cols = s.shape
    qcol = oracle.qcol_bytes(1, rows)
    q = np.zeros(cols * qcol, np.uint8)
    hdr = q.reshape(cols, qcol)[:, :8].view(np.float32)
    hdr[:, 0] = lower
    hdr[:, 1] = upper
    return oracle.pack_with_headers(s, np.zeros_like(s, order="F"), q, 1, True, threads=4)


@pytest.fixture(scope="module")
def case():
    _, _, s = datagen.few_valued_stripe_sum(ROWS, COLS)
    z = np.zeros_like(s, order="F")
    q_or, _ = oracle.quantize(s, z, 1, True, threads=4)
    lo_o, hi_o = oracle.headers(q_or, ROWS, COLS, 1)
    lo_x, hi_x = parity.exact_headers(s, z, 1, True)
    scale = hi_o.astype(np.float64) - lo_o
    dev_o = np.maximum(np.abs(lo_o - lo_x), np.abs(hi_o - hi_x)) / scale
    return s, z, lo_o, hi_o, lo_x, hi_x, scale, dev_o


def test_the_oracle_itself_misses_the_float64_bounds_at_6144_rows(case):
    s, z, lo_o, hi_o, lo_x, hi_x, scale, dev_o = case
    assert len(np.unique(s[:, 0])) == 4
    assert (dev_o > 1e-5).sum() >= 3, dev_o.max()  # seeds 4, 13, 27 ... of the recorded search


def test_accurate_bounds_are_accepted_and_counted(case):
    s, z, lo_o, hi_o, lo_x, hi_x, scale, dev_o = case
    q, r = packed_with_bounds(s, lo_x.astype(np.float32), hi_x.astype(np.float32))
    rep = parity.check_quantize(s, z, q, r, 1, True, threads=4, strict=True)
    # every column the oracle has off by more than the tolerance (plus the fp32 rounding of the exact bounds) took the
    # fallback, no other did
    assert rep.fallback_cols == int((dev_o > 1e-5 + 2e-7).sum()) or rep.fallback_cols == int((dev_o > 1e-5 - 2e-7).sum())
    assert 3 <= rep.fallback_cols <= COLS and rep.cols == COLS
    assert "fallback columns = %d of %d" % (rep.fallback_cols, COLS) in repr(rep)
    rep.assert_fallback_at_most(COLS)
    with pytest.raises(AssertionError, match="fallback columns"):
        rep.assert_fallback_at_most(rep.fallback_cols - 1)


def test_bounds_off_from_both_are_refused(case):
    s, z, lo_o, hi_o, lo_x, hi_x, scale, dev_o = case
    # 3e-5 of the scale away from the float64 bounds, on the side away from the oracle's
    side = np.where(hi_o >= hi_x, -1.0, 1.0)
    q, r = packed_with_bounds(s, lo_x.astype(np.float32), (hi_x + side * 3e-5 * scale).astype(np.float32))
    with pytest.raises(AssertionError, match="column bounds off"):
        parity.check_quantize(s, z, q, r, 1, True, threads=4)


def test_bounds_further_from_float64_than_the_oracle_are_refused(case):
    """Within the tolerance of the float64 bounds, but further from them than the oracle is and more than the tolerance
    from the oracle: the oracle's inexactness does not explain such a result."""
    s, z, lo_o, hi_o, lo_x, hi_x, scale, dev_o = case
    dev_hi = np.abs(hi_o - hi_x) / scale
    ok = np.nonzero((dev_hi > 5e-7) & (dev_o < 4e-6))[0]
    assert ok.size, "no column whose oracle bounds are between 5e-7 and 4e-6 from the float64 ones"
    j = int(ok[0])
    lo, hi = lo_o.copy(), hi_o.copy()
    side = 1.0 if hi_o[j] >= hi_x[j] else -1.0
    # upper bound 1e-5 - dev/2 from float64 on the far side of the oracle, hence 1e-5 + dev/2 from the oracle
    hi[j] = np.float32(hi_x[j] - side * (1e-5 - 0.5 * dev_hi[j]) * scale[j])
    assert abs(float(hi[j]) - hi_x[j]) / scale[j] <= 1e-5 < abs(float(hi[j]) - float(hi_o[j])) / scale[j]
    q, r = packed_with_bounds(s, lo, hi)
    with pytest.raises(AssertionError, match="column bounds off"):
        parity.check_quantize(s, z, q, r, 1, True, threads=4)


def test_no_fallback_on_ordinary_data():
    g = datagen.normal(11, 2048, 24)
    r = datagen.normal(12, 2048, 24, 0.002)
    q, r_out = oracle.quantize(g, r, 1, False, threads=4)
    rep = parity.check_quantize(g, r, q, r_out, 1, False, threads=4, strict=True)
    assert rep.fallback_cols == 0 and rep.fallback_elements == 0 and rep.cols == 24


def test_inputs_that_all_moved_one_way_explain_as_much_on_the_bounds():
    """A second-stage quantization whose inputs (the aggregates) are themselves equal only within a tolerance: a shift
    of every input moves the bounds by as much, and is allowed only when the caller states it."""
    g = datagen.normal(13, 2048, 8)
    r = datagen.normal(14, 2048, 8, 0.002)
    shift = np.float32(4e-7)  # about 2e-5 of the column scale of 0.02
    q, r_out = oracle.quantize(np.asfortranarray(g + shift), r, 1, False, threads=4)
    with pytest.raises(AssertionError, match="column bounds off"):
        parity.check_quantize(g, r, q, r_out, 1, False, threads=4, exact=False)
    parity.check_quantize(g, r, q, r_out, 1, False, threads=4, exact=False, input_dev=np.full(8, float(shift)))


def test_a_column_without_spread_whose_inputs_moved_a_little():
    """The whole-run comparison on a column that is all zero on the oracle's side (bounds 0, 0) and off by the inputs'
    difference on the other: exact agreement is asked for only where the inputs are the same."""
    g = np.zeros((64, 3), np.float32, order="F")
    r = np.zeros((64, 3), np.float32, order="F")
    moved = g.copy(order="F")
    moved[:, 1] = np.float32(3e-9)
    for nbits in (1, 2):
        q, r_out = oracle.quantize(moved, r, nbits, False, threads=2)
        with pytest.raises(AssertionError):
            parity.check_quantize(g, r, q, r_out, nbits, False, threads=2, exact=False)
        dev = np.array([0.0, 3e-9, 0.0])
        parity.check_quantize(g, r, q, r_out, nbits, False, threads=2, exact=False, input_dev=dev)
        with pytest.raises(AssertionError, match="without spread"):
            parity.check_quantize(g, r, q, r_out, nbits, False, threads=2, exact=False, input_dev=dev * 1e-3)


def test_an_element_on_the_other_side_of_zero_leaves_its_column_out_of_the_whole_run():
    """With the zero threshold the bounds are the means of the two sides: one element at -2e-8 here and 0.0 there moves
    both by mean / count (1e-4 of the scale at 2000 rows). The whole-run comparison leaves such a column out, and counts
    it, when it is given the aggregates of both sides; without them it must refuse."""
    rows, cols = 2000, 6
    a = datagen.normal(15, rows, cols)
    a[7, 2] = np.float32(-2e-8)
    b = a.copy(order="F")
    b[7, 2] = np.float32(0.0)
    z = np.zeros_like(a, order="F")
    q_or, _ = oracle.quantize(a, z, 1, True, threads=4)
    q_gpu, s_gpu = oracle.quantize(b, z, 1, True, threads=4)
    out_or = oracle.unquantize(q_or, rows, cols, 1, threads=4)
    out_gpu = oracle.unquantize(q_gpu, rows, cols, 1, threads=4)
    none = np.zeros(cols, dtype=bool)
    with pytest.raises(AssertionError, match="column bounds off"):
        parity.check_end_to_end([a], [z], q_gpu, [s_gpu], out_gpu, q_or, out_or, rows, cols, 1, True, none, threads=4)
    _, left_out = parity.check_end_to_end([a], [z], q_gpu, [s_gpu], out_gpu, q_or, out_or, rows, cols, 1, True, none, threads=4,
                                          aggs_gpu=[b])
    assert left_out == 1 and not none.any()
