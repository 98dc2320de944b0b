"""Seeded synthetic gradients for the parity tests and the benchmark (column-major numpy arrays, float32 unless
`dtype=np.float64` is asked for).

`exact_bell` uses integer arithmetic only, so its output is bit-identical on every machine and numpy
version; the golden vectors whose inputs are not stored are generated from it. The other generators
go through numpy's Generator and are used where both sides of a comparison see the same array.
"""
import numpy as np

BASE_SEED = 0x1B17


def case_seed(config, matrix=0, step=0, worker=0):
    return BASE_SEED + 1000 * config + 100 * matrix + step + 10000 * worker


def _f(a, dtype=np.float32):
    return np.asfortranarray(a.astype(dtype))


def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15)) & np.uint64(0xFFFFFFFFFFFFFFFF)
    z = x
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def exact_bell(seed, rows, cols, shift=22, dtype=np.float32):
    """Bell-shaped values (sum of four 16-bit uniforms, centred) times 2^-shift; exact in fp32.
    Standard deviation = 2^-shift * 65536 / sqrt(3), e.g. about 0.009 for shift = 22.
    With dtype=float64 a second 16-bit uniform times 2^-52 is added (still exact), so that the values
    use mantissa bits a float32 does not have."""
    n = rows * cols
    with np.errstate(over="ignore"):
        idx = np.arange(n, dtype=np.uint64)
        z = _splitmix64(idx * np.uint64(0x632BE59BD9B4E019) + np.uint64(seed) * np.uint64(0xD1342543DE82EF95))
    parts = [(z >> np.uint64(16 * k)) & np.uint64(0xFFFF) for k in range(4)]
    total = (parts[0] + parts[1] + parts[2] + parts[3]).astype(np.int64) - 2 * 65535
    vals = np.ldexp(total.astype(np.float64), -shift)
    if np.dtype(dtype) == np.float64:
        with np.errstate(over="ignore"):
            z2 = _splitmix64(z + np.uint64(0x2545F4914F6CDD1D))
        vals = vals + np.ldexp((z2 & np.uint64(0xFFFF)).astype(np.float64), -52)
    return _f(vals.reshape((rows, cols), order="F"), dtype)


def uniform(seed, rows, cols, lo, hi, dtype=np.float32):
    rng = np.random.default_rng(seed)
    return _f(lo + (hi - lo) * rng.random((rows, cols)), dtype)


def normal(seed, rows, cols, sigma=0.01, dtype=np.float32):
    rng = np.random.default_rng(seed)
    return _f(rng.standard_normal((rows, cols)) * sigma, dtype)


def student_t(seed, rows, cols, nu=3.0, scale=1e-3, dtype=np.float32):
    rng = np.random.default_rng(seed)
    return _f(rng.standard_t(nu, (rows, cols)) * scale, dtype)


def normal_with_outliers(seed, rows, cols, sigma=0.01, frac=0.01, mult=50.0, dtype=np.float32):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((rows, cols)) * sigma
    mask = rng.random((rows, cols)) < frac
    a[mask] *= mult
    return _f(a, dtype)


def zero_columns(a, seed, frac=0.9):
    """Zeroes a fixed (seed-dependent) subset of whole columns, in place; returns the mask of zeroed columns."""
    rng = np.random.default_rng(seed)
    mask = rng.random(a.shape[1]) < frac
    a[:, mask] = 0.0
    return mask


def few_valued_stripe_sum(rows, cols, seed0=90000, seed1=95000):
    """What the owner of a stripe requantizes at K = 2, 1 bit, zeroThresholdFor1Bit on: the sum of two workers'
    reconstructions, i.e. columns that hold only four distinct values. The fp32 term-by-term sum of such a column
    rounds the same way at every addition; at 6144 rows the bounds it gives are off by more than 1e-5 of the column
    scale for many seeds (the recorded case: a 6144-row stripe of the two-worker aggregator run).
    Returns (a, b, sum): the two gradients (exact bell-shaped values) and the fp32 sum of their reconstructions."""
    import oracle

    a = np.asfortranarray(np.concatenate([exact_bell(seed0 + j, rows, 1) for j in range(cols)], axis=1))
    b = np.asfortranarray(np.concatenate([exact_bell(seed1 + j, rows, 1) for j in range(cols)], axis=1))
    z = np.zeros_like(a, order="F")
    qa, _ = oracle.quantize(a, z, 1, True, threads=4)
    qb, _ = oracle.quantize(b, z, 1, True, threads=4)
    s = oracle.unquantize(qa, rows, cols, 1, threads=4)
    s = oracle.unquantize(qb, rows, cols, 1, out=s, add=True, threads=4)
    return a, b, s
