"""Pins the CPU oracle (oracle/quantizer_oracle.c) -- runs without a GPU.

1. against golden vectors written by the reference's own headers (tests/golden/make_golden.py);
2. against the reference headers directly, where oracle/_ref is built;
3. against what the mathematics fixes: a hand-computed column, closed forms of the reconstruction levels,
   a brute-force element -> (word, shift) placement, the conservation law, 32 bits = identity, and an
   independent float64 restatement that follows the reference unit test's inline checker
   (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp:54-237).
"""
import hashlib
import os

import numpy as np
import pytest

import datagen
import oracle
from golden.make_golden import BELL_CASES, ITERATIONS, UNIT_SHAPES, VARIANTS

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def flat(a):
    return np.asfortranarray(a).reshape(-1, order="F")


def unflat(v, rows, cols):
    return np.asfortranarray(v.reshape((rows, cols), order="F"))


def bits_eq(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint32), np.ascontiguousarray(b).view(np.uint32))


# ---- 1. golden vectors from the reference headers -------------------------------------------------


@pytest.mark.parametrize("si", range(len(UNIT_SHAPES)))
def test_unit_shapes_golden(si):
    gold = np.load(os.path.join(GOLD, "unit_shapes.npz"))
    rows, cols, lo, hi, seed = UNIT_SHAPES[si]
    inputs = [unflat(v, rows, cols) for v in gold["s%d_inputs" % si]]
    assert len(inputs) == ITERATIONS
    for nbits, zt in VARIANTS:
        key = "s%d_b%d_z%d" % (si, nbits, int(zt))
        res = np.zeros((rows, cols), np.float32, order="F")
        out = np.zeros((rows, cols), np.float32, order="F")
        for it, g in enumerate(inputs):
            q, _ = oracle.quantize(g, res, nbits, zt, r_out=res)
            oracle.unquantize(q, rows, cols, nbits, out=out, add=(it > 0))
            assert np.array_equal(q, gold[key + "_q"][it]), (key, it)
            assert sha(flat(res)) == str(gold[key + "_res_sha"][it]), (key, it)
            assert sha(flat(out)) == str(gold[key + "_out_sha"][it]), (key, it)
        assert bits_eq(flat(res), gold[key + "_res_last"])
        assert bits_eq(flat(out), gold[key + "_out_last"])


def test_special_golden():
    gold = np.load(os.path.join(GOLD, "special.npz"))
    g = np.asfortranarray(np.array([[0.1], [-0.2], [0.3], [-0.4], [0.05]], np.float32))
    q, r = oracle.quantize(g, np.zeros_like(g, order="F"), 1, False)
    assert np.array_equal(q, gold["hand_q"]) and bits_eq(flat(r), gold["hand_res"])
    z = np.zeros((70, 3), np.float32, order="F")
    for zt in (False, True):
        q, r = oracle.quantize(z, z.copy(order="F"), 1, zt)
        assert np.array_equal(q, gold["zero_z%d_q" % int(zt)])
        assert bits_eq(flat(r), gold["zero_z%d_res" % int(zt)])
    for nb in (2, 8):
        q, _ = oracle.quantize(z, z.copy(order="F"), nb, False)
        assert np.array_equal(q, gold["zero_b%d_q" % nb])
    g = datagen.exact_bell(7, 37, 2)
    q, r = oracle.quantize(g, np.zeros_like(g, order="F"), 2, False)
    assert np.array_equal(q, gold["lay2_q"]) and bits_eq(flat(r), gold["lay2_res"])
    assert bits_eq(flat(oracle.unquantize(q, 37, 2, 2)), gold["lay2_out"])


@pytest.mark.parametrize("case", BELL_CASES, ids=[c[0] for c in BELL_CASES])
def test_bell_golden(case):
    gold = np.load(os.path.join(GOLD, "bell.npz"))
    name, rows, cols, seed, variants, steps = case
    inputs = [datagen.exact_bell(seed * 10 + it, rows, cols) for it in range(steps)]
    # the integer-only generator must give the very same inputs on this machine
    assert [sha(flat(g)) for g in inputs] == [str(s) for s in gold[name + "_in_sha"]]
    for nbits, zt in variants:
        key = "%s_b%d_z%d" % (name, nbits, int(zt))
        res = np.zeros((rows, cols), np.float32, order="F")
        out = np.zeros((rows, cols), np.float32, order="F")
        for it, g in enumerate(inputs):
            q, _ = oracle.quantize(g, res, nbits, zt, r_out=res, threads=4)
            oracle.unquantize(q, rows, cols, nbits, out=out, add=(it > 0), threads=4)
            assert sha(q) == str(gold[key + "_q_sha"][it]), (key, it)
            assert sha(flat(res)) == str(gold[key + "_res_sha"][it]), (key, it)
            assert sha(flat(out)) == str(gold[key + "_out_sha"][it]), (key, it)
        lo, hi = oracle.headers(q, rows, cols, nbits)
        assert bits_eq(lo, gold[key + "_lower"]) and bits_eq(hi, gold[key + "_upper"])
        head = gold[key + "_q_head"]
        assert np.array_equal(q[: head.size], head)


# ---- 2. the reference headers themselves, where they could be built ---------------------------------


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref needs the reference tree")
def test_against_reference_headers():
    rng = np.random.default_rng(5)
    for rows, cols in [(33, 7), (64, 5), (257, 3), (2048, 4), (1, 9), (4097, 2)]:
        for nbits, zt in VARIANTS:
            r1 = np.zeros((rows, cols), np.float32, order="F")
            r2 = r1.copy(order="F")
            o1, o2 = r1.copy(order="F"), r1.copy(order="F")
            for it in range(3):
                g = np.asfortranarray((rng.standard_normal((rows, cols)) * 0.01 + 0.004 * (it % 2)).astype(np.float32))
                if it == 1:
                    g[:, 0] = 0
                q1, _ = oracle.quantize(g, r1, nbits, zt, r_out=r1)
                q2, _ = oracle.quantize(g, r2, nbits, zt, r_out=r2, use_ref=True)
                assert np.array_equal(q1, q2) and bits_eq(r1, r2)
                oracle.unquantize(q1, rows, cols, nbits, out=o1, add=it > 0)
                oracle.unquantize(q2, rows, cols, nbits, out=o2, add=it > 0, use_ref=True)
                assert bits_eq(o1, o2)


# ---- 3. what the mathematics fixes ------------------------------------------------------------------


def test_hand_computed_column():
    # mean = -0.03; below: {-0.2, -0.4}, above: {0.1, 0.3, 0.05}; both deviations sum to 0.54;
    # dev = 1.08 / 5 = 0.216, radius = 0.432 -> lower = -0.462, upper = 0.402; levels mean -/+ dev
    g = np.asfortranarray(np.array([[0.1], [-0.2], [0.3], [-0.4], [0.05]], np.float32))
    z = np.zeros_like(g, order="F")
    q, r = oracle.quantize(g, z, 1, False)
    lo, hi = oracle.headers(q, 5, 1, 1)
    assert abs(lo[0] + 0.462) < 1e-6 and abs(hi[0] - 0.402) < 1e-6
    assert oracle.words(q, 5, 1, 1)[0, 0] == 0b10101
    out = oracle.unquantize(q, 5, 1, 1)
    np.testing.assert_allclose(out[:, 0], [0.186, -0.246, 0.186, -0.246, 0.186], atol=1e-6)
    np.testing.assert_allclose(r[:, 0], g[:, 0] - out[:, 0], atol=1e-7)
    # zero-threshold mode: levels are the plain means of the negative and non-negative parts
    q, r = oracle.quantize(g, z, 1, True)
    out = oracle.unquantize(q, 5, 1, 1)
    np.testing.assert_allclose(out[:, 0], [0.15, -0.3, 0.15, -0.3, 0.15], atol=1e-6)


def test_value_quantizer_closed_forms():
    L = oracle.lib()
    lo, hi = np.float32(-0.5), np.float32(1.5)
    for nbits in (2, 4, 8, 16):
        top = (1 << nbits) - 1
        uf = (float(hi) - float(lo)) / top
        assert L.oracle_quantize_value(-0.5, nbits, lo, hi, 0) == 0
        assert L.oracle_quantize_value(-7.0, nbits, lo, hi, 0) == 0
        assert L.oracle_quantize_value(1.5, nbits, lo, hi, 0) == top  # the top code is reached only at/above upper
        assert L.oracle_quantize_value(1.5 - 1e-6, nbits, lo, hi, 0) == top - 1
        # codes reconstruct to bin centres; the top code lands half a step above upper
        assert abs(L.oracle_unquantize_value(top, nbits, lo, hi) - (float(hi) + 0.5 * uf)) < 1e-5
        assert abs(L.oracle_unquantize_value(0, nbits, lo, hi) - (float(lo) + 0.5 * uf)) < 1e-6
        mid_code = L.oracle_quantize_value(0.5, nbits, lo, hi, 0)
        assert mid_code == int((0.5 + 0.5) / uf)
    # 1 bit: threshold is the midpoint of the stored header, or 0 in zero-threshold mode
    assert L.oracle_quantize_value(0.49, 1, lo, hi, 0) == 0 and L.oracle_quantize_value(0.5, 1, lo, hi, 0) == 1
    assert L.oracle_quantize_value(-1e-9, 1, lo, hi, 1) == 0 and L.oracle_quantize_value(0.0, 1, lo, hi, 1) == 1
    assert abs(L.oracle_unquantize_value(0, 1, lo, hi) - 0.0) < 1e-7 and abs(L.oracle_unquantize_value(1, 1, lo, hi) - 1.0) < 1e-7
    # degenerate range: factors are 0, everything reconstructs to lower
    assert L.oracle_unquantize_value(1, 1, np.float32(0.25), np.float32(0.25)) == np.float32(0.25)
    # 32 bits: identity on the bit pattern
    x = np.float32(-3.1415927)
    code = L.oracle_quantize_value(x, 32, lo, hi, 0)
    assert code == int(np.array([x]).view(np.uint32)[0])
    assert np.float32(L.oracle_unquantize_value(code, 32, lo, hi)) == x


def test_layout_helpers():
    assert oracle.qwords_per_col(2048, 1) == 64 and oracle.qcol_bytes(1, 2048) == 264
    assert oracle.qwords_per_col(429, 1) == 14 and oracle.qcol_bytes(1, 429) == 64
    assert oracle.qcol_bytes(1, 512) == 72 and oracle.qcol_bytes(1, 100000) == 12508
    assert oracle.qcol_bytes(8, 2048) == 2056 and oracle.qcol_bytes(2, 147) == 48
    assert oracle.qwords_per_col(147, 2) == 10 and oracle.qwords_per_col(37, 2) == 3
    assert oracle.qcol_bytes(32, 5) == 28
    assert oracle.lib().oracle_check_nbits(3) != 0 and oracle.lib().oracle_check_nbits(64) != 0
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros((4, 4), np.float32, order="F"), np.zeros((4, 4), np.float32, order="F"), 3, False)


@pytest.mark.parametrize("nbits", [1, 2, 4, 8, 16, 32])
def test_brute_force_placement(nbits):
    """Element i of a column sits in word i % nq at bit (i // nq) * nbits; padding bits are zero."""
    L = oracle.lib()
    for rows, cols in [(1, 3), (5, 2), (37, 2), (70, 1), (131, 2)]:
        g = datagen.uniform(90 + rows, rows, cols, -1.0, 2.0)
        r = datagen.uniform(91 + rows, rows, cols, -0.1, 0.1)
        for zt in ((False, True) if nbits == 1 else (False,)):
            q, r_out = oracle.quantize(g, r, nbits, zt)
            nq = oracle.qwords_per_col(rows, nbits)
            w = oracle.words(q, rows, cols, nbits)
            for j in range(cols):
                lo, hi = oracle.column_stats(g, r, j, nbits, zt)
                expect = [0] * nq
                for i in range(rows):
                    v = np.float32(g[i, j] + r[i, j])
                    code = L.oracle_quantize_value(v, nbits, lo, hi, int(zt))
                    expect[i % nq] |= code << ((i // nq) * nbits)
                    back = np.float32(L.oracle_unquantize_value(code, nbits, lo, hi))
                    assert np.float32(v - back) == r_out[i, j] or (np.isnan(r_out[i, j]))
                assert [int(x) for x in w[j]] == expect


def _inline_checker(nbits, g, prev_res, prev_out, zt, passthrough_bits=32):
    """Independent float64 restatement after the reference unit test's ReferenceCPUQuantizer: row-major loops,
    `val < mean` decisions for 1 bit, no packing at all. passthrough_bits = width of the QWord."""
    rows, cols = g.shape
    out = np.zeros((rows, cols))
    res = np.zeros((rows, cols))
    for j in range(cols):
        v = g[:, j].astype(np.float64) + prev_res[:, j]
        if nbits == passthrough_bits:
            out[:, j] = prev_out[:, j] + v
            continue
        mean = v.sum() / rows if (not zt and nbits == 1) else 0.0
        if nbits == 1:
            below = v < mean
            s0, s1, n0, n1 = v[below].sum(), v[~below].sum(), int(below.sum()), int((~below).sum())
            if not zt:
                dev = ((n0 * mean - s0) + (s1 - n1 * mean)) / rows
                radius, centre = 2 * dev, mean
            else:
                m0, m1 = s0 / max(n0, 1), s1 / max(n1, 1)
                centre = 0.5 * (m0 + m1)
                radius = 2 * (m1 - centre)
            qv = np.where(below, centre - 0.5 * radius, centre + 0.5 * radius)
        else:
            sd = np.sqrt((v * v).sum() / rows)
            lo, hi = -4 * sd, 4 * sd
            rng = 1 << nbits
            if hi - lo < 1e-36:
                qf = uf = 0.0
            else:
                qf, uf = (rng - 1) / (hi - lo), (hi - lo) / (rng - 1)
            code = np.where(v <= lo, 0, np.where(v >= hi, rng - 1, np.trunc((v - lo) * qf)))
            qv = (code + 0.5) * uf + lo
        out[:, j] = prev_out[:, j] + qv
        res[:, j] = v - qv
    return out, res


@pytest.mark.parametrize("si", range(len(UNIT_SHAPES)))
def test_against_inline_checker(si):
    rows, cols, lo, hi, seed = UNIT_SHAPES[si]
    for nbits, zt in VARIANTS:
        res = np.zeros((rows, cols), np.float32, order="F")
        out = np.zeros((rows, cols), np.float32, order="F")
        tol = (hi - lo) * 1e-4 if nbits != 32 else 0.0
        allowed = max(1, int(rows * cols * 1e-3))  # elements that may fall on the other side of a decision
        for it in range(ITERATIONS):
            g = datagen.uniform(seed + it, rows, cols, lo, hi)
            prev_res, prev_out = res.copy(order="F"), out.copy(order="F")
            q, _ = oracle.quantize(g, res, nbits, zt, r_out=res)
            oracle.unquantize(q, rows, cols, nbits, out=out, add=(it > 0))
            # conservation of the error feedback (MatrixQuantizerTests.cpp:327-338)
            lhs = g.astype(np.float64) + prev_res + prev_out
            assert np.abs(lhs - (res.astype(np.float64) + out)).max() <= max(tol, 1e-5 * (hi - lo))
            ref_out, ref_res = _inline_checker(nbits, g, prev_res, prev_out, zt)
            if nbits == 32:
                np.testing.assert_allclose(out, ref_out, rtol=1e-6, atol=1e-12)
                assert not res.any()
                continue
            assert int((np.abs(out - ref_out) > tol).sum()) <= allowed
            assert int((np.abs(res - ref_res) > tol).sum()) <= allowed


def test_stripe_ranges():
    assert oracle.stripe_range(9304, 0, 8) == (0, 1163) and oracle.stripe_range(9304, 7, 8) == (8141, 1163)
    for cols, k in [(10, 4), (3, 8), (0, 2), (135, 7)]:
        pos = 0
        for r in range(k):
            s, n = oracle.stripe_range(cols, r, k)
            assert s == pos and n in (cols // k, cols // k + 1)
            pos += n
        assert pos == cols


def test_stripe_reduce_32bit_is_plain_sum():
    """With 32 bits nothing is lost: the aggregate is the fp32 sum, owner first, then ascending rank."""
    k, rows, cols = 4, 19, 11
    gs = [datagen.normal(300 + w, rows, cols, 1.0) for w in range(k)]
    res = [np.zeros((rows, cols), np.float32, order="F") for _ in range(k)]
    sres = [np.zeros((rows, oracle.stripe_range(cols, s, k)[1]), np.float32, order="F") for s in range(k)]
    qs, qagg, out = oracle.allreduce(gs, res, sres, 32, False)
    for s in range(k):
        st, n = oracle.stripe_range(cols, s, k)
        acc = gs[s][:, st:st + n].copy()
        for w in range(k):
            if w != s:
                acc = gs[w][:, st:st + n] + acc
        assert bits_eq(np.asfortranarray(out[:, st:st + n]), np.asfortranarray(acc))
    assert not any(r.any() for r in res) and not any(s.any() for s in sres)


@pytest.mark.parametrize("nbits,zt", [(1, False), (1, True), (4, False)])
def test_allreduce_composition(nbits, zt):
    """The all-reduce is exactly the composition of quantize / unquantize calls the aggregator makes
    (Source/1BitSGD/AllReduceDistGradAggregator.h:299, 373, 407, 434, 521)."""
    k, rows, cols = 3, 70, 10
    gs = [datagen.normal(400 + w, rows, cols) for w in range(k)]
    res = [datagen.normal(450 + w, rows, cols, 0.002) for w in range(k)]
    sres = [datagen.normal(470 + s, rows, oracle.stripe_range(cols, s, k)[1], 0.002) for s in range(k)]
    res2 = [r.copy(order="F") for r in res]
    sres2 = [s.copy(order="F") for s in sres]
    _, qagg, out = oracle.allreduce(gs, res, sres, nbits, zt)

    qs = [oracle.quantize(gs[w], res2[w], nbits, zt, r_out=res2[w])[0] for w in range(k)]
    qcol = oracle.qcol_bytes(nbits, rows)
    final = np.zeros_like(qagg)
    for s in range(k):
        st, n = oracle.stripe_range(cols, s, k)
        sl = slice(st * qcol, (st + n) * qcol)
        agg = oracle.unquantize(qs[s][sl].copy(), rows, n, nbits)
        for w in range(k):
            if w != s:
                oracle.unquantize(qs[w][sl].copy(), rows, n, nbits, out=agg, add=True)
        q2, _ = oracle.quantize(agg, sres2[s], nbits, zt, r_out=sres2[s])
        final[sl] = q2
    assert np.array_equal(final, qagg)
    assert bits_eq(oracle.unquantize(final, rows, cols, nbits), out)
    assert all(bits_eq(a, b) for a, b in zip(res, res2)) and all(bits_eq(a, b) for a, b in zip(sres, sres2))
    # one worker: aggregate = unquantize(quantize(unquantize(quantize(G))))
    g1, r1 = [gs[0]], [np.zeros((rows, cols), np.float32, order="F")]
    s1 = [np.zeros((rows, cols), np.float32, order="F")]
    _, _, out1 = oracle.allreduce(g1, r1, s1, nbits, zt)
    z = np.zeros((rows, cols), np.float32, order="F")
    qa, _ = oracle.quantize(gs[0], z, nbits, zt)
    qb, _ = oracle.quantize(oracle.unquantize(qa, rows, cols, nbits), z, nbits, zt)
    assert bits_eq(oracle.unquantize(qb, rows, cols, nbits), out1)


def test_in_place_equals_out_of_place():
    g = datagen.normal(77, 429, 37)
    r = datagen.normal(78, 429, 37, 0.003)
    for nbits, zt in VARIANTS:
        q1, r1 = oracle.quantize(g, r, nbits, zt)
        r2 = r.copy(order="F")
        q2, _ = oracle.quantize(g, r2, nbits, zt, r_out=r2)
        assert np.array_equal(q1, q2) and bits_eq(r1, r2)
