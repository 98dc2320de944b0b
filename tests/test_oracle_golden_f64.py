"""Pins the double-precision instantiation of the CPU oracle (ELEM = double, 64-bit QWords) -- runs without a GPU.

Same three layers as for float: golden vectors written by the reference's own headers instantiated for double
(tests/golden/make_golden.py), the reference headers directly where oracle/_ref is built, and what the mathematics
fixes (hand-computed column, closed forms, brute-force placement in 64-bit words, 64 bits = identity, the
reference unit test's inline checker, Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp:54-237, which the
reference itself runs for double at :420-431).
"""
import hashlib
import os

import numpy as np
import pytest

import datagen
import oracle
from golden.make_golden import BELL_F64, ITERATIONS_F64, UNIT_SHAPES, VARIANTS_F64
from test_oracle_golden import _inline_checker

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F64 = np.float64


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def flat(a):
    return np.asfortranarray(a).reshape(-1, order="F")


def unflat(v, rows, cols):
    return np.asfortranarray(v.reshape((rows, cols), order="F"))


def bits_eq(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint64), np.ascontiguousarray(b).view(np.uint64))


def zeros(rows, cols):
    return np.zeros((rows, cols), F64, order="F")


@pytest.mark.parametrize("si", range(len(UNIT_SHAPES)))
def test_unit_shapes_golden_f64(si):
    gold = np.load(os.path.join(GOLD, "unit_shapes_f64.npz"))
    rows, cols, lo, hi, seed = UNIT_SHAPES[si]
    inputs = [unflat(v, rows, cols) for v in gold["s%d_inputs" % si]]
    assert len(inputs) == ITERATIONS_F64 and inputs[0].dtype == F64
    for nbits, zt in VARIANTS_F64:
        key = "s%d_b%d_z%d" % (si, nbits, int(zt))
        res, out = zeros(rows, cols), zeros(rows, cols)
        for it, g in enumerate(inputs):
            q, _ = oracle.quantize(g, res, nbits, zt, r_out=res)
            oracle.unquantize(q, rows, cols, nbits, out=out, add=(it > 0))
            assert np.array_equal(q, gold[key + "_q"][it]), (key, it)
        assert bits_eq(flat(res), gold[key + "_res_last"]), key
        assert bits_eq(flat(out), gold[key + "_out_last"]), key


@pytest.mark.parametrize("case", BELL_F64, ids=[c[0] for c in BELL_F64])
def test_bell_golden_f64(case):
    gold = np.load(os.path.join(GOLD, "unit_shapes_f64.npz"))
    name, rows, cols, seed = case
    inputs = [datagen.exact_bell(seed * 10 + it, rows, cols, dtype=F64) for it in range(2)]
    assert [sha(flat(g)) for g in inputs] == [str(s) for s in gold[name + "_in_sha"]]
    # the values really use bits below float32's mantissa
    assert not np.array_equal(inputs[0], inputs[0].astype(np.float32).astype(F64))
    for nbits, zt in [(1, False), (1, True), (4, False)]:
        key = "%s_b%d_z%d" % (name, nbits, int(zt))
        res, out = zeros(rows, cols), zeros(rows, cols)
        for it, g in enumerate(inputs):
            q, _ = oracle.quantize(g, res, nbits, zt, r_out=res, threads=4)
            oracle.unquantize(q, rows, cols, nbits, out=out, add=(it > 0), threads=4)
            assert sha(q) == str(gold[key + "_q_sha"][it]), (key, it)
            assert sha(flat(res)) == str(gold[key + "_res_sha"][it]), (key, it)
            assert sha(flat(out)) == str(gold[key + "_out_sha"][it]), (key, it)
        lo, hi = oracle.headers(q, rows, cols, nbits, dtype=F64)
        assert bits_eq(lo, gold[key + "_lower"]) and bits_eq(hi, gold[key + "_upper"])


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref needs the reference tree")
def test_against_reference_headers_f64():
    rng = np.random.default_rng(6)
    for rows, cols in [(33, 7), (64, 5), (65, 3), (257, 3), (2048, 4), (1, 9), (4097, 2)]:
        assert oracle.qwords_per_col(rows, 1, F64) == oracle.ref_lib().ref_qwords_per_col_f64(rows, 1)
        for nbits, zt in VARIANTS_F64:
            r1, r2, o1, o2 = zeros(rows, cols), zeros(rows, cols), zeros(rows, cols), zeros(rows, cols)
            for it in range(3):
                g = np.asfortranarray(rng.standard_normal((rows, cols)) * 0.01 + 0.004 * (it % 2))
                if it == 1:
                    g[:, 0] = 0
                q1, _ = oracle.quantize(g, r1, nbits, zt, r_out=r1)
                q2, _ = oracle.quantize(g, r2, nbits, zt, r_out=r2, use_ref=True)
                assert np.array_equal(q1, q2) and bits_eq(r1, r2)
                oracle.unquantize(q1, rows, cols, nbits, out=o1, add=it > 0)
                oracle.unquantize(q2, rows, cols, nbits, out=o2, add=it > 0, use_ref=True)
                assert bits_eq(o1, o2)


def test_layout_helpers_f64():
    # record = 16-byte header + 8-byte QWords; 64 values per QWord at 1 bit
    assert oracle.qwords_per_col(2048, 1, F64) == 32 and oracle.qcol_bytes(1, 2048, F64) == 16 + 32 * 8
    assert oracle.qwords_per_col(65, 1, F64) == 2 and oracle.qcol_bytes(1, 65, F64) == 32
    assert oracle.qwords_per_col(100, 4, F64) == 7 and oracle.qcol_bytes(4, 100, F64) == 16 + 7 * 8
    assert oracle.qcol_bytes(64, 5, F64) == 16 + 5 * 8 and oracle.qcol_bytes(32, 5, F64) == 16 + 3 * 8
    assert oracle.check_nbits(64, F64) and not oracle.check_nbits(64, np.float32)
    assert not oracle.check_nbits(3, F64) and not oracle.check_nbits(128, F64) and not oracle.check_nbits(0, F64)


def test_hand_computed_column_f64():
    # same column as the float test; in double the closed-form values hold to 1e-15
    g = np.asfortranarray(np.array([[0.1], [-0.2], [0.3], [-0.4], [0.05]], F64))
    q, r = oracle.quantize(g, zeros(5, 1), 1, False)
    lo, hi = oracle.headers(q, 5, 1, 1, dtype=F64)
    assert abs(lo[0] + 0.462) < 1e-15 and abs(hi[0] - 0.402) < 1e-15
    assert int(oracle.words(q, 5, 1, 1, dtype=F64)[0, 0]) == 0b10101
    out = oracle.unquantize(q, 5, 1, 1, dtype=F64)
    np.testing.assert_allclose(out[:, 0], [0.186, -0.246, 0.186, -0.246, 0.186], atol=1e-15)
    np.testing.assert_allclose(r[:, 0], g[:, 0] - out[:, 0], atol=1e-16)
    q, r = oracle.quantize(g, zeros(5, 1), 1, True)
    out = oracle.unquantize(q, 5, 1, 1, dtype=F64)
    np.testing.assert_allclose(out[:, 0], [0.15, -0.3, 0.15, -0.3, 0.15], atol=1e-15)


def test_value_quantizer_closed_forms_f64():
    lo, hi = -0.5, 1.5
    for nbits in (2, 4, 8, 16, 32):  # 32 bits is a real quantizer for double: 2^32 - 1 steps
        top = (1 << nbits) - 1
        uf = (hi - lo) / top
        assert oracle.quantize_value(-0.5, nbits, lo, hi, 0, F64) == 0
        assert oracle.quantize_value(-7.0, nbits, lo, hi, 0, F64) == 0
        assert oracle.quantize_value(1.5, nbits, lo, hi, 0, F64) == top
        assert oracle.quantize_value(1.5 - 1e-12, nbits, lo, hi, 0, F64) == top - 1
        assert abs(oracle.unquantize_value(top, nbits, lo, hi, F64) - (hi + 0.5 * uf)) < 1e-14
        assert abs(oracle.unquantize_value(0, nbits, lo, hi, F64) - (lo + 0.5 * uf)) < 1e-15
        assert oracle.quantize_value(0.5, nbits, lo, hi, 0, F64) == int((0.5 + 0.5) * (top / (hi - lo)))
    assert oracle.quantize_value(0.5 - 1e-15, 1, lo, hi, 0, F64) == 0 and oracle.quantize_value(0.5, 1, lo, hi, 0, F64) == 1
    assert oracle.quantize_value(-1e-300, 1, lo, hi, 1, F64) == 0 and oracle.quantize_value(0.0, 1, lo, hi, 1, F64) == 1
    assert oracle.unquantize_value(0, 1, lo, hi, F64) == 0.0 and oracle.unquantize_value(1, 1, lo, hi, F64) == 1.0
    # the futility guard compares the span with the float literal 1e-36f: a span of 1e-37 gives factor 0,
    # a span of 1e-35 does not
    assert oracle.unquantize_value(1, 2, 0.0, 1e-37, F64) == 0.0
    assert oracle.unquantize_value(1, 2, 0.0, 1e-35, F64) > 0.0
    # 64 bits: identity on the bit pattern
    x = np.float64(-3.141592653589793)
    code = oracle.quantize_value(x, 64, lo, hi, 0, F64)
    assert code == int(np.array([x]).view(np.uint64)[0])
    assert oracle.unquantize_value(code, 64, lo, hi, F64) == x


@pytest.mark.parametrize("nbits", [1, 2, 4, 8, 16, 32, 64])
def test_brute_force_placement_f64(nbits):
    """Element i of a column sits in 64-bit word i % nq at bit (i // nq) * nbits; padding bits are zero."""
    for rows, cols in [(1, 3), (5, 2), (37, 2), (70, 1), (131, 2), (200, 1)]:
        g = datagen.uniform(90 + rows, rows, cols, -1.0, 2.0, dtype=F64)
        r = datagen.uniform(91 + rows, rows, cols, -0.1, 0.1, dtype=F64)
        for zt in ((False, True) if nbits == 1 else (False,)):
            q, r_out = oracle.quantize(g, r, nbits, zt)
            nq = oracle.qwords_per_col(rows, nbits, F64)
            assert nq == -(-rows // (64 // nbits))
            w = oracle.words(q, rows, cols, nbits, dtype=F64)
            for j in range(cols):
                lo, hi = oracle.column_stats(g, r, j, nbits, zt)
                expect = [0] * nq
                for i in range(rows):
                    v = g[i, j] + r[i, j]
                    code = oracle.quantize_value(v, nbits, lo, hi, zt, F64)
                    expect[i % nq] |= code << ((i // nq) * nbits)
                    back = oracle.unquantize_value(code, nbits, lo, hi, F64)
                    assert v - back == r_out[i, j]
                assert [int(x) for x in w[j]] == expect


@pytest.mark.parametrize("si", range(len(UNIT_SHAPES)))
def test_against_inline_checker_f64(si):
    rows, cols, lo, hi, seed = UNIT_SHAPES[si]
    for nbits, zt in VARIANTS_F64:
        if nbits == 64:
            continue
        res, out = zeros(rows, cols), zeros(rows, cols)
        # both sides compute in double; they differ in summation order only (at 32 bits a code is 2^-32 of the
        # range wide, so a last-bit difference of the header can move a value by one code)
        tol = (hi - lo) * (1e-11 if nbits < 32 else 1e-8)
        allowed = max(1, int(rows * cols * 1e-3))
        for it in range(ITERATIONS_F64):
            g = datagen.uniform(seed + it, rows, cols, lo, hi, dtype=F64)
            prev_res, prev_out = res.copy(order="F"), out.copy(order="F")
            q, _ = oracle.quantize(g, res, nbits, zt, r_out=res)
            oracle.unquantize(q, rows, cols, nbits, out=out, add=(it > 0))
            assert np.abs((g + prev_res + prev_out) - (res + out)).max() <= 1e-14 * max(1.0, hi - lo)
            ref_out, ref_res = _inline_checker(nbits, g, prev_res, prev_out, zt, passthrough_bits=64)
            assert int((np.abs(out - ref_out) > tol).sum()) <= allowed, (nbits, zt, it)
            assert int((np.abs(res - ref_res) > tol).sum()) <= allowed, (nbits, zt, it)


def test_64bit_allreduce_is_plain_sum():
    k, rows, cols = 4, 19, 11
    gs = [datagen.normal(300 + w, rows, cols, 1.0, dtype=F64) for w in range(k)]
    res = [zeros(rows, cols) for _ in range(k)]
    sres = [zeros(rows, oracle.stripe_range(cols, s, k)[1]) for s in range(k)]
    qs, qagg, out = oracle.allreduce(gs, res, sres, 64, False)
    for s in range(k):
        st, n = oracle.stripe_range(cols, s, k)
        acc = gs[s][:, st:st + n].copy()
        for w in range(k):
            if w != s:
                acc = gs[w][:, st:st + n] + acc
        assert bits_eq(np.asfortranarray(out[:, st:st + n]), np.asfortranarray(acc))
    assert not any(r.any() for r in res) and not any(s.any() for s in sres)


@pytest.mark.parametrize("nbits,zt", [(1, False), (1, True), (4, False)])
def test_allreduce_composition_f64(nbits, zt):
    k, rows, cols = 3, 70, 10
    gs = [datagen.normal(400 + w, rows, cols, dtype=F64) for w in range(k)]
    res = [datagen.normal(450 + w, rows, cols, 0.002, dtype=F64) for w in range(k)]
    sres = [datagen.normal(470 + s, rows, oracle.stripe_range(cols, s, k)[1], 0.002, dtype=F64) for s in range(k)]
    res2 = [r.copy(order="F") for r in res]
    sres2 = [s.copy(order="F") for s in sres]
    _, qagg, out = oracle.allreduce(gs, res, sres, nbits, zt)
    qs = [oracle.quantize(gs[w], res2[w], nbits, zt, r_out=res2[w])[0] for w in range(k)]
    qcol = oracle.qcol_bytes(nbits, rows, F64)
    final = np.zeros_like(qagg)
    for s in range(k):
        st, n = oracle.stripe_range(cols, s, k)
        sl = slice(st * qcol, (st + n) * qcol)
        agg = oracle.unquantize(qs[s][sl].copy(), rows, n, nbits, dtype=F64)
        for w in range(k):
            if w != s:
                oracle.unquantize(qs[w][sl].copy(), rows, n, nbits, out=agg, add=True)
        q2, _ = oracle.quantize(agg, sres2[s], nbits, zt, r_out=sres2[s])
        final[sl] = q2
    assert np.array_equal(final, qagg)
    assert bits_eq(oracle.unquantize(final, rows, cols, nbits, dtype=F64), out)
    assert all(bits_eq(a, b) for a, b in zip(res, res2)) and all(bits_eq(a, b) for a, b in zip(sres, sres2))
