"""Comparison rules for HIP results against the CPU oracle.

Two layers:
  exact     -- under the headers the GPU produced, codes and residuals must equal the oracle's bit for bit
               (the only freedom a parallel implementation has is the order of the fp32 sums behind the header);
  tolerance -- the GPU headers against the sequential-sum oracle headers: lower/upper within 1e-5 of the column
               scale (upper - lower); a code may differ only for an element within 1e-6 * scale of a decision
               threshold (their number is reported); residuals of all other elements within 1e-5 * scale.
"""
import numpy as np

import oracle

BOUND_RTOL = 1e-5
THRESH_RTOL = 1e-6
VALUE_RTOL = 1e-5


def bits_equal(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


class Report:
    def __init__(self):
        self.elements = 0
        self.near_threshold_mismatches = 0
        self.max_bound_err = 0.0
        self.max_residual_err = 0.0

    def __repr__(self):
        return ("elements=%d near-threshold code mismatches=%d max bound err=%.3g max residual err=%.3g (relative to column scale)"
                % (self.elements, self.near_threshold_mismatches, self.max_bound_err, self.max_residual_err))


def check_quantize(g, r_in, q_gpu, r_gpu, nbits, zero_threshold, threads=8, report=None):
    """g, r_in: inputs (F-order float32); q_gpu: packed bytes from the GPU; r_gpu: residual from the GPU."""
    rows, cols = g.shape
    zt = bool(zero_threshold) and nbits == 1
    rep = report if report is not None else Report()
    rep.elements += rows * cols

    # ---- exact layer
    q_ex, r_ex = oracle.pack_with_headers(g, r_in, q_gpu, nbits, zt, threads=threads)
    assert np.array_equal(q_ex, q_gpu), "codes differ from the oracle's under the GPU's own headers"
    assert bits_equal(r_ex, r_gpu), "residual differs from the oracle's under the GPU's own headers"

    # ---- tolerance layer
    q_or, r_or = oracle.quantize(g, r_in, nbits, zt, threads=threads)
    lo_g, hi_g = oracle.headers(q_gpu, rows, cols, nbits)
    lo_o, hi_o = oracle.headers(q_or, rows, cols, nbits)
    scale = (hi_o.astype(np.float64) - lo_o.astype(np.float64))
    tiny = np.finfo(np.float32).tiny
    denom = np.maximum(np.abs(scale), tiny)
    err = np.maximum(np.abs(lo_g.astype(np.float64) - lo_o), np.abs(hi_g.astype(np.float64) - hi_o)) / denom
    # columns without any spread (all-zero) must agree exactly
    flat = scale == 0
    assert np.array_equal(lo_g[flat], lo_o[flat]) and np.array_equal(hi_g[flat], hi_o[flat])
    err[flat] = 0.0
    rep.max_bound_err = max(rep.max_bound_err, float(err.max(initial=0.0)))
    assert err.max(initial=0.0) <= BOUND_RTOL, "column bounds off by %.3g of the column scale" % err.max()

    if nbits == 32:
        assert np.array_equal(q_or[:], q_gpu[:]) or np.array_equal(oracle.words(q_or, rows, cols, 32),
                                                                   oracle.words(q_gpu, rows, cols, 32))
        assert bits_equal(r_or, r_gpu)
        return rep

    c_g = oracle.codes(q_gpu, rows, cols, nbits)
    c_o = oracle.codes(q_or, rows, cols, nbits)
    diff = c_g != c_o
    ndiff = int(diff.sum())
    if ndiff:
        v = (g + r_in).astype(np.float64)  # one rounded fp32 add, then widened
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
            assert np.all(np.abs(c_g[ii, jj].astype(np.int64) - c_o[ii, jj].astype(np.int64)) == 1), \
                "codes differ by more than one level"
        assert np.all(dist <= THRESH_RTOL * sc), \
            "%d codes differ away from a threshold (worst %.3g of scale)" % (ndiff, float((dist / sc).max()))
        rep.near_threshold_mismatches += ndiff

    same = ~diff
    rerr = np.abs(r_gpu.astype(np.float64) - r_or) / denom[None, :]
    rerr = np.where(same, rerr, 0.0)
    rep.max_residual_err = max(rep.max_residual_err, float(rerr.max(initial=0.0)))
    assert rerr.max(initial=0.0) <= VALUE_RTOL, "residual off by %.3g of the column scale" % rerr.max()
    return rep


def check_unquantize(q, rows, cols, nbits, out_gpu, prev_out=None, threads=8):
    """Unquantize has no reductions: bit-exact against the oracle."""
    add = prev_out is not None
    out = np.array(prev_out, dtype=np.float32, order="F", copy=True) if add else None
    ref = oracle.unquantize(q, rows, cols, nbits, out=out, add=add, threads=threads)
    assert bits_equal(ref, out_gpu), "unquantized output differs from the oracle"


def conservation(g, r_in, prev_out, r_out, out, tol):
    """Error feedback loses nothing: g + r_in + prev_out == r_out + out (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp:327-338)."""
    lhs = g.astype(np.float64) + r_in + prev_out
    rhs = r_out.astype(np.float64) + out
    assert np.abs(lhs - rhs).max(initial=0.0) <= tol
