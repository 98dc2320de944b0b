"""Comparison rules for HIP results against the CPU oracle.

Two layers:
  exact     -- under the headers the GPU produced, codes and residuals must equal the oracle's bit for bit
               (the only freedom a parallel implementation has is the order of the fp32 sums behind the header);
  tolerance -- the GPU headers against the sequential-sum oracle headers: lower/upper within 1e-5 of the column
               scale (upper - lower); a code may differ only for an element within 1e-6 * scale of a decision
               threshold (their number is reported); residuals of all other elements within 1e-5 * scale -- or, where
               that is more, within what the (accepted) deviation of the bounds does to the top reconstruction level,
               2^nbits / (2^nbits - 1) times that deviation above 1 bit -- plus one unit in the last place of the
               residual itself (both sides round value - reconstruction once, and an outlier many column scales large
               rounds coarser than 1e-5 * scale). Residuals beyond 1e-5 * scale are counted (Report.rounding_elements).

A decision threshold lies between lower and upper, so it can move by as much as the header moved. Where the header
of a column deviates by more than 1e-6 of its scale (long columns: the oracle's own sequential fp32 sum is that
inexact; fine code grids: 16 bits), a differing code is accepted within 1.5 x that column's observed header
deviation instead, and counted separately as "beyond 1e-6"; callers that must hold the 1e-6 rule literally pass
strict=True, which makes any such element a failure.

Where the oracle itself is inexact: the oracle adds a column term by term in the element type, as the reference's CPU
path does, and that sum is itself off by up to about sqrt(rows) * 2^-24 of the sum for fp32 (2e-5 at 100000 rows; more
than 1e-5 already at 6144 rows when a column holds few distinct values, so that every addition rounds the same way).
No height limit separates such columns from the others, so the rule looks at the data: a column whose bounds miss the
oracle's by more than the tolerance is accepted only if (a) its bounds are within the tolerance of the bounds computed
from the same values in float64 (exact_headers) and (b) the oracle's own bounds are further from those float64 bounds
than the column's, i.e. the oracle's deviation is what used up the tolerance. Such columns are counted
(Report.fallback_cols out of Report.cols); their residuals may differ from the oracle's by 1.5 x the observed
deviation of the bounds (a residual is value - reconstruction, so it moves with them), and the elements that needed
that are counted too (Report.fallback_elements). Callers state how many they allow (Report.assert_fallback_at_most).

The figures above are for float32 matrices. For float64 matrices (64-bit QWords) the same rules apply with 1e-12 /
1e-13 / 1e-12: both sides sum in double and differ in the order of the additions only.
"""
import numpy as np

import oracle

BOUND_RTOL = 1e-5
THRESH_RTOL = 1e-6
VALUE_RTOL = 1e-5


def tolerances(dtype):
    """(bound, threshold, value, floor of the relaxed rule), relative to the column scale."""
    if np.dtype(dtype) == np.float64:
        return 1e-12, 1e-13, 1e-12, 1e-14
    return BOUND_RTOL, THRESH_RTOL, VALUE_RTOL, 1e-7


def bits_equal(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


class Report:
    def __init__(self):
        self.elements = 0
        self.near_threshold_mismatches = 0
        self.beyond_1e6 = 0
        self.last_mismatch_cols = None  # per column of the last check: did any code differ from the oracle's
        self.max_bound_err = 0.0
        self.max_residual_err = 0.0
        self.cols = 0  # columns compared with the oracle in the tolerance layer
        self.fallback_cols = 0  # of those: accepted against the float64 bounds because the oracle's own were further off
        self.fallback_elements = 0  # residuals in such columns that differ from the oracle's by more than the tolerance
        # residuals beyond the tolerance by no more than the bounds' own (accepted) deviation carried to the top
        # reconstruction level, plus one unit in the residual's own last place
        self.rounding_elements = 0

    def __repr__(self):
        return ("elements=%d near-threshold code mismatches=%d (of which beyond 1e-6 of scale: %d) max bound err=%.3g "
                "max residual err=%.3g (relative to column scale) fallback columns = %d of %d (fallback elements = %d) "
                "residuals over the tolerance as far as the accepted bounds and their own last place explain = %d"
                % (self.elements, self.near_threshold_mismatches, self.beyond_1e6, self.max_bound_err,
                   self.max_residual_err, self.fallback_cols, self.cols, self.fallback_elements, self.rounding_elements))

    def assert_fallback_at_most(self, cols, elements=None):
        """The caller's bound on how much of the comparison rested on the float64 bounds instead of the oracle's."""
        assert self.fallback_cols <= cols, "fallback columns = %d, more than the %d allowed" % (self.fallback_cols, cols)
        if elements is not None:
            assert self.fallback_elements <= elements, \
                "fallback elements = %d, more than the %d allowed" % (self.fallback_elements, elements)


def exact_headers(g, r_in, nbits, zt):
    """(lower, upper) per column from the statistics of Source/Math/ColumnQuantizer.h:209-341 evaluated in float64 on
    v = g + r_in (the sum itself rounded in the element type, as every implementation does)."""
    v = (g + r_in).astype(np.float64)
    rows = v.shape[0]
    if nbits > 1:
        half = 4.0 * np.sqrt((v * v).sum(axis=0) / rows)
        return -half, half
    mean = np.zeros(v.shape[1]) if zt else v.sum(axis=0) / rows
    below = v < mean[None, :]
    s0 = np.where(below, v, 0.0).sum(axis=0)
    s1 = np.where(below, 0.0, v).sum(axis=0)
    n0 = below.sum(axis=0)
    n1 = rows - n0
    if zt:
        m0, m1 = s0 / np.maximum(n0, 1), s1 / np.maximum(n1, 1)
        centre = 0.5 * (m0 + m1)
        radius = 2.0 * (m1 - centre)
    else:
        radius = 2.0 * ((n0 * mean - s0) + (s1 - n1 * mean)) / rows
        centre = mean
    return centre - radius, centre + radius


def check_quantize(g, r_in, q_gpu, r_gpu, nbits, zero_threshold, threads=8, report=None, strict=False, exact=True,
                   skip_cols=None, input_dev=None):
    """g, r_in: inputs (F-order float32); q_gpu: packed bytes from the GPU; r_gpu: residual from the GPU.
    exact=False skips the bit-exact layer (for inputs that are themselves only equal within tolerance);
    skip_cols (bool per column) leaves columns out of the tolerance layer; input_dev (per column, absolute): by how much
    the values that the GPU quantized may differ from g + r_in -- a residual is value - reconstruction, so it may differ
    by that much more."""
    rows, cols = g.shape
    dt = g.dtype
    bound_rtol, thresh_rtol, value_rtol, relaxed_floor = tolerances(dt)
    word_bits = 8 * dt.itemsize
    zt = bool(zero_threshold) and nbits == 1
    rep = report if report is not None else Report()
    rep.elements += rows * cols
    keep = np.ones(cols, dtype=bool) if skip_cols is None else ~np.asarray(skip_cols, dtype=bool)

    # ---- exact layer
    if exact:
        q_ex, r_ex = oracle.pack_with_headers(g, r_in, q_gpu, nbits, zt, threads=threads)
        assert np.array_equal(q_ex, q_gpu), "codes differ from the oracle's under the GPU's own headers"
        assert bits_equal(r_ex, r_gpu), "residual differs from the oracle's under the GPU's own headers"

    # ---- tolerance layer
    q_or, r_or = oracle.quantize(g, r_in, nbits, zt, threads=threads)
    lo_g, hi_g = oracle.headers(q_gpu, rows, cols, nbits, dtype=dt)
    lo_o, hi_o = oracle.headers(q_or, rows, cols, nbits, dtype=dt)
    scale = (hi_o.astype(np.float64) - lo_o.astype(np.float64))
    tiny = np.finfo(dt).tiny
    denom = np.maximum(np.abs(scale), tiny)
    abs_dev = np.maximum(np.abs(lo_g.astype(np.float64) - lo_o), np.abs(hi_g.astype(np.float64) - hi_o))
    err = abs_dev / denom
    # columns without any spread (all-zero) must agree exactly -- unless the caller states that this side's inputs differ
    # from the oracle's (input_dev): a column that is all zero there is then all within input_dev here, and bounds made
    # of such values (a mean and a deviation, or a few standard deviations) lie within a small multiple of it
    flat = (scale == 0) & keep
    if input_dev is None:
        assert np.array_equal(lo_g[flat], lo_o[flat]) and np.array_equal(hi_g[flat], hi_o[flat])
    else:
        assert (abs_dev[flat] <= 8.0 * np.asarray(input_dev, dtype=np.float64)[flat]).all(), \
            "bounds of a column without spread are further from the oracle's than the inputs' difference explains"
    err[flat] = 0.0
    err[~keep] = 0.0
    # A reconstruction level is lower + (code + 1/2) * (upper - lower) / (2^nbits - 1) (one step fewer than codes above 1
    # bit): the top level lies half a step beyond `upper`, so when the bounds move by d in opposite directions (the
    # symmetric range of the multi-bit quantizer always does) that level, and the residual against it, moves by
    # d * 2^nbits / (2^nbits - 1): 4/3 at 2 bits. Bounds within the tolerance therefore allow that much on a residual.
    reach = 1.0 if nbits == 1 or nbits >= 32 else float(2 ** nbits) / float(2 ** nbits - 1)
    res_allow = np.maximum(value_rtol, reach * err)
    slack = np.zeros(cols) if input_dev is None else np.asarray(input_dev, dtype=np.float64) / denom
    res_allow = res_allow + slack
    # A column's bounds are averages of its values (1 bit) or of their squares: inputs that all moved one way by up to
    # input_dev move the bounds by up to as much, so that part of a deviation is the inputs', not this quantization's.
    err = np.maximum(err - slack, 0.0)
    rep.cols += int(keep.sum())
    fallback = np.zeros(cols, dtype=bool)
    if err.max(initial=0.0) > bound_rtol:
        # The oracle's term-by-term sum in the element type is itself inexact. A column that misses the oracle's bounds
        # is accepted if it is within the tolerance of the bounds computed from the same values in float64 AND the
        # oracle's own bounds are further from those than the column's (the oracle's deviation used up the tolerance).
        lo_x, hi_x = exact_headers(g, r_in, nbits, zt)
        err_x = np.maximum(np.abs(lo_g.astype(np.float64) - lo_x), np.abs(hi_g.astype(np.float64) - hi_x)) / denom
        err_x = np.maximum(err_x - slack, 0.0)
        err_ox = np.maximum(np.abs(lo_o.astype(np.float64) - lo_x), np.abs(hi_o.astype(np.float64) - hi_x)) / denom
        fallback = (err > bound_rtol) & (err_x <= bound_rtol) & (err_x <= err_ox) & keep & ~flat
        # a residual is value - reconstruction: it moves with the bounds
        res_allow = np.where(fallback, np.maximum(value_rtol, 1.5 * err) + slack, res_allow)
        err = np.where(fallback, err_x, err)
        rep.fallback_cols += int(fallback.sum())
    rep.max_bound_err = max(rep.max_bound_err, float(err.max(initial=0.0)))
    if err.max(initial=0.0) > bound_rtol:
        j = int(np.argmax(err))
        lo_x, hi_x = exact_headers(g[:, j:j + 1], r_in[:, j:j + 1], nbits, zt)
        raise AssertionError("column bounds off by %.3g of the column scale (column %d of %d, %d rows: [%r, %r] against the oracle's "
                             "[%r, %r]; from the same values in float64 [%r, %r]; inputs moved by %.3g of the scale)"
                             % (err.max(), j, cols, rows, lo_g[j], hi_g[j], lo_o[j], hi_o[j], float(lo_x[0]), float(hi_x[0]),
                                slack[j]))

    if nbits == word_bits:
        assert np.array_equal(q_or[:], q_gpu[:]) or np.array_equal(oracle.words(q_or, rows, cols, nbits, dtype=dt),
                                                                   oracle.words(q_gpu, rows, cols, nbits, dtype=dt))
        assert bits_equal(r_or, r_gpu)
        rep.last_mismatch_cols = np.zeros(cols, dtype=bool)
        return rep

    c_g = oracle.codes(q_gpu, rows, cols, nbits, dtype=dt)
    c_o = oracle.codes(q_or, rows, cols, nbits, dtype=dt)
    diff = (c_g != c_o) & keep[None, :]
    ndiff = int(diff.sum())
    rep.last_mismatch_cols = diff.any(axis=0)
    if ndiff:
        v = (g + r_in).astype(np.float64)  # one add rounded in the element type, then widened
        ii, jj = np.nonzero(diff)
        vv = v[ii, jj]
        sc = denom[jj]
        if nbits == 1:
            thr = np.zeros_like(vv) if zt else 0.5 * (hi_o[jj].astype(np.float64) + lo_o[jj])
            dist = np.abs(vv - thr)
        else:
            used = float((1 << nbits) - 1)
            lo = lo_o[jj].astype(np.float64)
            pos = (vv - lo) * (used / sc)
            dist = np.abs(pos - np.round(pos)) * (sc / used)
            dist = np.minimum(dist, np.minimum(np.abs(vv - lo), np.abs(vv - hi_o[jj].astype(np.float64))))
            # one level, plus however many levels the bounds themselves moved (fine grids under long columns)
            levels = 1 + np.floor(1.5 * abs_dev[jj] * used / sc)
            assert np.all(np.abs(c_g[ii, jj].astype(np.int64) - c_o[ii, jj].astype(np.int64)) <= levels), \
                "codes differ by more levels than the bounds moved"
        far = dist > thresh_rtol * sc
        allowed = np.maximum(thresh_rtol * sc, 1.5 * abs_dev[jj] + relaxed_floor * sc)
        if strict:
            allowed = thresh_rtol * sc
        assert np.all(dist <= allowed), \
            "%d codes differ away from a threshold (worst %.3g of scale)" % (ndiff, float((dist / sc).max()))
        rep.near_threshold_mismatches += ndiff
        rep.beyond_1e6 += int(far.sum())

    same = ~diff & keep[None, :]
    rerr = np.abs(r_gpu.astype(np.float64) - r_or) / denom[None, :]
    rerr = np.where(same, rerr, 0.0)
    rep.max_residual_err = max(rep.max_residual_err, float(rerr.max(initial=0.0)))
    rep.fallback_elements += int((rerr[:, fallback] > value_rtol).sum())
    # Both residuals are value - reconstruction rounded once in the element type; under bounds that differ within the
    # tolerance the two exact differences round separately, so one unit in the last place of the residual itself comes
    # on top of the tolerance (it matters for outliers many column scales large: heavy-tailed gradients).
    # (and each side evaluates its reconstruction level in three rounded operations on numbers as large as the bounds)
    level = 4.0 * np.maximum(np.abs(lo_o.astype(np.float64)), np.abs(hi_o.astype(np.float64)))
    ulp = (np.abs(r_or.astype(np.float64)) + level[None, :]) * float(np.finfo(dt).eps) / denom[None, :]
    over = (rerr > value_rtol) & ~fallback[None, :]
    rep.rounding_elements += int(over.sum())
    bad = rerr > res_allow[None, :] + ulp
    if bad.any():
        i, j = np.unravel_index(int(np.argmax(np.where(bad, rerr, 0.0))), rerr.shape)
        raise AssertionError("residual off by %.3g of the column scale (row %d, column %d: value %.3g, column scale %.3g, bounds off "
                             "by %.3g of it)" % (rerr[i, j], i, j, float(g[i, j]) + float(r_in[i, j]), denom[j], err[j]))
    return rep


def check_unquantize(q, rows, cols, nbits, out_gpu, prev_out=None, threads=8):
    """Unquantize has no reductions: bit-exact against the oracle."""
    add = prev_out is not None
    out = np.array(prev_out, dtype=out_gpu.dtype, order="F", copy=True) if add else None
    ref = oracle.unquantize(q, rows, cols, nbits, out=out, add=add, threads=threads, dtype=out_gpu.dtype)
    assert bits_equal(ref, out_gpu), "unquantized output differs from the oracle"


def conservation(g, r_in, prev_out, r_out, out, tol):
    """Error feedback loses nothing: g + r_in + prev_out == r_out + out (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp:327-338)."""
    lhs = g.astype(np.float64) + r_in + prev_out
    rhs = r_out.astype(np.float64) + out
    assert np.abs(lhs - rhs).max(initial=0.0) <= tol


def oracle_allreduce_staged(gs, res, sres, nbits, zt, threads=8):
    """The oracle's all-reduce, stage by stage, keeping the intermediates. Updates res[w], sres[s] in place.
    Returns (packed matrices after stage 1, fp32 aggregates per stripe, assembled packed aggregate, output)."""
    k = len(gs)
    rows, cols = gs[0].shape
    dt = gs[0].dtype
    qcol = oracle.qcol_bytes(nbits, rows, dt)
    q1 = [oracle.quantize(gs[w], res[w], nbits, zt, r_out=res[w], threads=threads)[0] for w in range(k)]
    qagg = np.zeros_like(q1[0])
    aggs = []
    for s in range(k):
        start, n = oracle.stripe_range(cols, s, k)
        if n == 0:
            aggs.append(np.zeros((rows, 0), dt, order="F"))
            continue
        qc = [q.copy() for q in q1]
        aggs.append(oracle.stripe_reduce(qc, s, rows, cols, nbits, sres[s], zt, threads=threads))
        qagg[start * qcol:(start + n) * qcol] = qc[s][start * qcol:(start + n) * qcol]
    out = oracle.unquantize(qagg, rows, cols, nbits, threads=threads, dtype=dt)
    return q1, aggs, qagg, out


def check_end_to_end(aggs_or, sres_in, qagg_gpu, sres_gpu, out_gpu, qagg_or, out_or, rows, cols, nbits, zt, tainted_cols,
                     threads=8, report=None, aggs_gpu=None):
    """Whole all-reduce against the free-standing oracle run (oracle_allreduce_staged). A first-stage code that flips
    at its threshold moves that element's aggregate by a whole reconstruction level, hence the second-stage header
    of that column by about level / rows; such columns (tainted_cols) are left out and counted. Everywhere else the
    second stage must agree with the oracle's under the usual tolerance rules (its inputs, the aggregates, are
    themselves equal only within the first-stage header tolerance: with aggs_gpu, the exact aggregates of the GPU's
    first-stage codes, the residuals are allowed that difference on top), and the aggregated gradient must be within 1e-5
    of the column scale wherever the final codes agree."""
    k = len(aggs_or)
    dt = out_or.dtype
    qcol = oracle.qcol_bytes(nbits, rows, dt)
    rep = report if report is not None else Report()
    tainted_cols = np.array(tainted_cols, dtype=bool)
    for s in range(k):
        start, n = oracle.stripe_range(cols, s, k)
        if n == 0:
            continue
        dev = None
        if aggs_gpu is not None:
            dev = np.abs(np.asarray(aggs_gpu[s], dtype=np.float64) - aggs_or[s]).max(axis=0, initial=0.0)
            if zt and nbits == 1:
                # With the zero threshold a column's bounds are the means of its negative and of its other values
                # (the zero-threshold branch of Source/Math/ColumnQuantizer.h:209-341): an element within that difference of zero may be on one
                # side here and on the other there, and one such element moves both means by mean / count, far more
                # than the inputs differ (met: -2.6e-8 against 0.0 in 7650 rows moved the bounds by 6.8e-5 of the
                # scale). Such columns are left out like those a first-stage code flipped in.
                v = (aggs_or[s] + sres_in[s]).astype(np.float64)
                tainted_cols[start:start + n] |= (np.abs(v) <= dev[None, :]).any(axis=0)
        check_quantize(aggs_or[s], sres_in[s], qagg_gpu[start * qcol:(start + n) * qcol], sres_gpu[s], nbits, zt,
                       threads=threads, report=rep, exact=False, skip_cols=tainted_cols[start:start + n], input_dev=dev)
    clean = ~tainted_cols
    lo, hi = oracle.headers(qagg_or, rows, cols, nbits, dtype=dt)
    scale = np.maximum(np.abs(hi.astype(np.float64) - lo), np.finfo(dt).tiny)
    # elements whose final code differs sit a whole level apart; the check above has vetted each of them
    same = oracle.codes(qagg_gpu, rows, cols, nbits, dtype=dt) == oracle.codes(qagg_or, rows, cols, nbits, dtype=dt)
    err = np.where(same, np.abs(out_gpu.astype(np.float64) - out_or) / scale[None, :], 0.0)
    tol = tolerances(dt)[2]
    # a value reconstructed from equal codes moves with the bounds; where the bounds moved by more than the tolerance,
    # check_quantize above has accepted the column against the float64 statistics (and counted it)
    lo_g, hi_g = oracle.headers(qagg_gpu, rows, cols, nbits, dtype=dt)
    moved = np.maximum(np.abs(lo_g.astype(np.float64) - lo), np.abs(hi_g.astype(np.float64) - hi)) / scale
    # ... and within the tolerance it moves as a residual does in check_quantize: the top level of a multi-bit quantizer by
    # 2^nbits / (2^nbits - 1) times what the bounds moved (met at 2 bits on a 20000-row column: bounds off by 0.96e-5 of
    # the column scale, the top level by 1.28e-5)
    reach = 1.0 if nbits == 1 or nbits >= 32 else float(2 ** nbits) / float(2 ** nbits - 1)
    allow = np.where(moved > tol, 1.5 * moved, np.maximum(tol, reach * moved))
    # (each side evaluates its reconstruction level in three rounded operations on numbers as large as the bounds)
    allow = allow + 4.0 * np.maximum(np.abs(lo.astype(np.float64)), np.abs(hi.astype(np.float64))) * float(np.finfo(dt).eps) / scale
    over = err - allow[None, :]
    worst = float(err[:, clean].max(initial=0.0))
    if float(over[:, clean].max(initial=-1.0)) > 0.0:
        bad = np.where(clean, over.max(axis=0), -1.0)
        j = int(np.argmax(bad))
        i = int(np.argmax(over[:, j]))
        raise AssertionError("aggregated gradient off by %.3g of the column scale (column %d of %d, row %d of %d: %r against the "
                             "oracle's %r; bounds [%r, %r] against [%r, %r], moved by %.3g of the scale %.3g)"
                             % (float(err[i, j]), j, cols, i, rows, out_gpu[i, j], out_or[i, j], lo_g[j], hi_g[j], lo[j], hi[j],
                                float(moved[j]), float(scale[j])))
    return worst, int(tainted_cols.sum())
