"""ctypes front end of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only the tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this package; the shipped library (``cntk_amd``) never does.

Matrices are float32 (or float64) numpy arrays in column-major (Fortran) order, shape ``(rows, cols)``,
exactly the memory layout the reference's ``Matrix<ElemType>::Data()`` hands to its quantizer. Packed
matrices are flat ``uint8`` arrays of ``cols * qcol_bytes(nbits, rows)`` bytes. The element type of the
arrays selects the instantiation (float32: 32-bit QWords; float64: 64-bit QWords); helpers that see no
matrix take ``dtype`` (default float32).

``lib()`` is the plain-C restatement (``quantizer_oracle.c``).  ``ref_lib()`` is the reference's own
headers compiled into ``oracle/_ref`` -- present only where that was built (it cannot be built on a
machine without the reference tree) and used only to validate the restatement and to write the
golden vectors.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

_f32p = ctypes.POINTER(ctypes.c_float)
_sz = ctypes.c_size_t


def build(ref=False):
    """Compile liboracle.so (and oracle/_ref when asked and the reference tree is mounted)."""
    targets = ["all"] + (["ref"] if ref else [])
    subprocess.run(["make", "-C", _HERE, "-B"] + targets, check=True, capture_output=True)


def build_flags():
    """The compiler flags the two CPU libraries are built with, as the Makefile states them ({"CFLAGS": ..., "CXXFLAGS": ...})."""
    out = {}
    with open(os.path.join(_HERE, "Makefile")) as f:
        for line in f:
            name, eq, value = line.partition("=")
            if eq and name.strip() in ("CFLAGS", "CXXFLAGS"):
                out[name.strip()] = value.strip()
    return out


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)
        L = ctypes.CDLL(path)
        L.oracle_check_nbits.argtypes = [_sz]
        L.oracle_check_nbits.restype = ctypes.c_int
        L.oracle_qwords_per_col.argtypes = [_sz, _sz]
        L.oracle_qwords_per_col.restype = _sz
        L.oracle_qcol_bytes.argtypes = [_sz, _sz]
        L.oracle_qcol_bytes.restype = _sz
        L.oracle_quantize_value.argtypes = [ctypes.c_float, _sz, ctypes.c_float, ctypes.c_float, ctypes.c_int]
        L.oracle_quantize_value.restype = ctypes.c_uint32
        L.oracle_unquantize_value.argtypes = [ctypes.c_uint32, _sz, ctypes.c_float, ctypes.c_float]
        L.oracle_unquantize_value.restype = ctypes.c_float
        L.oracle_column_stats.argtypes = [ctypes.c_void_p, ctypes.c_void_p, _sz, _sz, _sz, ctypes.c_int, _f32p, _f32p]
        L.oracle_column_stats.restype = None
        L.oracle_quantize.argtypes = [ctypes.c_void_p, ctypes.c_void_p, _sz, _sz, ctypes.c_void_p, _sz,
                                      ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        L.oracle_quantize.restype = ctypes.c_int
        L.oracle_pack_with_headers.argtypes = L.oracle_quantize.argtypes
        L.oracle_pack_with_headers.restype = ctypes.c_int
        L.oracle_unquantize.argtypes = [ctypes.c_void_p, _sz, _sz, _sz, ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        L.oracle_unquantize.restype = ctypes.c_int
        L.oracle_stripe_range.argtypes = [_sz, _sz, _sz, ctypes.POINTER(_sz), ctypes.POINTER(_sz)]
        L.oracle_stripe_range.restype = None
        L.oracle_stripe_reduce.argtypes = [ctypes.POINTER(ctypes.c_void_p), _sz, _sz, _sz, _sz, _sz,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        L.oracle_stripe_reduce.restype = ctypes.c_int
        L.oracle_allreduce.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p),
                                       ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p),
                                       _sz, _sz, _sz, _sz, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                       ctypes.c_int]
        L.oracle_allreduce.restype = ctypes.c_int
        for name in ("check_nbits", "qwords_per_col", "qcol_bytes", "quantize", "pack_with_headers", "unquantize",
                     "stripe_reduce", "allreduce"):
            f32, f64 = getattr(L, "oracle_" + name), getattr(L, "oracle_%s_f64" % name)
            f64.argtypes, f64.restype = f32.argtypes, f32.restype
        _f64p = ctypes.POINTER(ctypes.c_double)
        L.oracle_quantize_value_f64.argtypes = [ctypes.c_double, _sz, ctypes.c_double, ctypes.c_double, ctypes.c_int]
        L.oracle_quantize_value_f64.restype = ctypes.c_uint64
        L.oracle_unquantize_value_f64.argtypes = [ctypes.c_uint64, _sz, ctypes.c_double, ctypes.c_double]
        L.oracle_unquantize_value_f64.restype = ctypes.c_double
        L.oracle_column_stats_f64.argtypes = [ctypes.c_void_p, ctypes.c_void_p, _sz, _sz, _sz, ctypes.c_int, _f64p, _f64p]
        L.oracle_column_stats_f64.restype = None
        _LIB = L
    return _LIB


def ref_available():
    return os.path.exists(os.path.join(_HERE, "_ref", "libref_quantizer.so"))


def ref_lib():
    global _REF
    if _REF is None:
        L = ctypes.CDLL(os.path.join(_HERE, "_ref", "libref_quantizer.so"))
        L.ref_qwords_per_col.argtypes = [_sz, _sz]
        L.ref_qwords_per_col.restype = _sz
        L.ref_quantize.argtypes = [ctypes.c_void_p, ctypes.c_void_p, _sz, _sz, ctypes.c_void_p, _sz,
                                   ctypes.c_void_p, ctypes.c_int]
        L.ref_quantize.restype = ctypes.c_int
        L.ref_unquantize.argtypes = [ctypes.c_void_p, _sz, _sz, _sz, ctypes.c_void_p, ctypes.c_int]
        L.ref_unquantize.restype = ctypes.c_int
        for name in ("qwords_per_col", "quantize", "unquantize"):
            f32, f64 = getattr(L, "ref_" + name), getattr(L, "ref_%s_f64" % name)
            f64.argtypes, f64.restype = f32.argtypes, f32.restype
        _REF = L
    return _REF


# ---------------------------------------------------------------------------------------------


def _is64(dtype):
    dt = np.dtype(dtype)
    if dt == np.float32:
        return False
    if dt == np.float64:
        return True
    raise ValueError("element type must be float32 or float64")


def _fn(handle, name, dtype):
    return getattr(handle, name + ("_f64" if _is64(dtype) else ""))


def _word_dtype(dtype):
    return np.uint64 if _is64(dtype) else np.uint32


def _colmajor(a, name, dtype=None):
    if a.dtype not in (np.float32, np.float64) or a.ndim != 2 or not a.flags.f_contiguous:
        raise ValueError("%s must be a 2-D float32 or float64 array in column-major (order='F') layout" % name)
    if dtype is not None and a.dtype != np.dtype(dtype):
        raise ValueError("%s must have element type %s" % (name, np.dtype(dtype)))
    return a


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _bad_nbits(dtype):
    return ValueError("nbits must be one of 1, 2, 4, 8, 16, 32" + (", 64" if _is64(dtype) else ""))


def check_nbits(nbits, dtype=np.float32):
    return _fn(lib(), "oracle_check_nbits", dtype)(nbits) == 0


def qwords_per_col(rows, nbits, dtype=np.float32):
    return _fn(lib(), "oracle_qwords_per_col", dtype)(rows, nbits)


def qcol_bytes(nbits, rows, dtype=np.float32):
    return _fn(lib(), "oracle_qcol_bytes", dtype)(nbits, rows)


def stripe_range(cols, rank, workers):
    s, n = _sz(), _sz()
    lib().oracle_stripe_range(cols, rank, workers, ctypes.byref(s), ctypes.byref(n))
    return s.value, n.value


def quantize_value(u, nbits, lower, upper, zero_threshold, dtype=np.float32):
    return int(_fn(lib(), "oracle_quantize_value", dtype)(u, nbits, lower, upper, int(zero_threshold)))


def unquantize_value(q, nbits, lower, upper, dtype=np.float32):
    return np.dtype(dtype).type(_fn(lib(), "oracle_unquantize_value", dtype)(q, nbits, lower, upper))


def column_stats(g, r, j, nbits, zero_threshold):
    _colmajor(g, "g"), _colmajor(r, "r", g.dtype)
    ct = ctypes.c_double if _is64(g.dtype) else ctypes.c_float
    lo, hi = ct(), ct()
    _fn(lib(), "oracle_column_stats", g.dtype)(_ptr(g), _ptr(r), g.shape[0], j, nbits, int(zero_threshold),
                                               ctypes.byref(lo), ctypes.byref(hi))
    return g.dtype.type(lo.value), g.dtype.type(hi.value)


def quantize(g, r_in, nbits, zero_threshold, r_out=None, threads=1, use_ref=False):
    """Returns (packed uint8 buffer, new residual). r_out=None allocates; r_out=r_in is in place."""
    _colmajor(g, "g"), _colmajor(r_in, "r_in", g.dtype)
    rows, cols = g.shape
    if r_in.shape != g.shape:
        raise ValueError("residual shape mismatch")
    if not check_nbits(nbits, g.dtype):
        raise _bad_nbits(g.dtype)
    if r_out is None:
        r_out = np.zeros_like(g, order="F")
    _colmajor(r_out, "r_out", g.dtype)
    q = np.zeros(cols * qcol_bytes(nbits, rows, g.dtype), dtype=np.uint8)
    if use_ref:
        rc = _fn(ref_lib(), "ref_quantize", g.dtype)(_ptr(g), _ptr(r_in), rows, cols, _ptr(q), nbits, _ptr(r_out),
                                                     int(zero_threshold))
    else:
        rc = _fn(lib(), "oracle_quantize", g.dtype)(_ptr(g), _ptr(r_in), rows, cols, _ptr(q), nbits, _ptr(r_out),
                                                    int(zero_threshold), threads)
    if rc != 0:
        raise _bad_nbits(g.dtype)
    return q, r_out


def pack_with_headers(g, r_in, q_with_headers, nbits, zero_threshold, threads=1):
    """Codes and residual under the headers already stored in q_with_headers (not modified).
    Returns (packed buffer, residual)."""
    _colmajor(g, "g"), _colmajor(r_in, "r_in", g.dtype)
    rows, cols = g.shape
    if not check_nbits(nbits, g.dtype):
        raise _bad_nbits(g.dtype)
    q = np.array(q_with_headers, dtype=np.uint8, copy=True)
    if q.size != cols * qcol_bytes(nbits, rows, g.dtype):
        raise ValueError("packed buffer has the wrong size")
    r_out = np.zeros_like(g, order="F")
    rc = _fn(lib(), "oracle_pack_with_headers", g.dtype)(_ptr(g), _ptr(r_in), rows, cols, _ptr(q), nbits,
                                                         _ptr(r_out), int(zero_threshold), threads)
    if rc != 0:
        raise _bad_nbits(g.dtype)
    return q, r_out


def unquantize(q, rows, cols, nbits, out=None, add=False, threads=1, use_ref=False, dtype=None):
    """dtype: element type of the packed matrix; taken from `out` when that is given, else float32."""
    if dtype is None:
        dtype = out.dtype if out is not None else np.float32
    if not check_nbits(nbits, dtype):
        raise _bad_nbits(dtype)
    if q.dtype != np.uint8 or q.size != cols * qcol_bytes(nbits, rows, dtype):
        raise ValueError("packed buffer has the wrong size")
    if out is None:
        out = np.zeros((rows, cols), dtype=dtype, order="F")
    _colmajor(out, "out", dtype)
    if use_ref:
        rc = _fn(ref_lib(), "ref_unquantize", dtype)(_ptr(q), rows, cols, nbits, _ptr(out), int(add))
    else:
        rc = _fn(lib(), "oracle_unquantize", dtype)(_ptr(q), rows, cols, nbits, _ptr(out), int(add), threads)
    if rc != 0:
        raise _bad_nbits(dtype)
    return out


def headers(q, rows, cols, nbits, dtype=np.float32):
    """(lower, upper) arrays read from a packed buffer."""
    stride = qcol_bytes(nbits, rows, dtype)
    hb = 2 * np.dtype(dtype).itemsize
    h = np.lib.stride_tricks.as_strided(q.view(np.uint8), shape=(cols, hb), strides=(stride, 1))
    h = np.ascontiguousarray(h).view(dtype)
    return h[:, 0].copy(), h[:, 1].copy()


def words(q, rows, cols, nbits, dtype=np.float32):
    """(cols, nq) array of the packed QWords (uint32, or uint64 for float64 matrices)."""
    stride = qcol_bytes(nbits, rows, dtype)
    nq = qwords_per_col(rows, nbits, dtype)
    wt = np.dtype(_word_dtype(dtype))
    hb = 2 * np.dtype(dtype).itemsize
    w = np.lib.stride_tricks.as_strided(q[hb:].view(np.uint8), shape=(cols, nq * wt.itemsize), strides=(stride, 1))
    return np.ascontiguousarray(w).view(wt)


def codes(q, rows, cols, nbits, dtype=np.float32):
    """(rows, cols) array of per-element codes, undoing the interleaved packing:
    element i lives in word i % nq at bit (i // nq) * nbits (Source/Math/QuantizedMatrix.cpp:143-169)."""
    w = words(q, rows, cols, nbits, dtype)
    wt = w.dtype.type
    nq = w.shape[1]
    i = np.arange(rows)
    full = 8 * w.dtype.itemsize
    mask = wt((1 << full) - 1) if nbits == full else wt((1 << nbits) - 1)
    c = (w[:, i % nq] >> ((i // nq) * nbits).astype(w.dtype)) & mask
    return np.asfortranarray(c.T)


def stripe_reduce(qs, owner, rows, cols, nbits, stripe_res, zero_threshold, threads=1):
    """In place on qs[owner]'s stripe and stripe_res; returns the aggregate (rows x len)."""
    k = len(qs)
    dtype = stripe_res.dtype
    _, n = stripe_range(cols, owner, k)
    agg = np.zeros((rows, n), dtype=dtype, order="F")
    arr = (ctypes.c_void_p * k)(*[q.ctypes.data for q in qs])
    rc = _fn(lib(), "oracle_stripe_reduce", dtype)(arr, k, owner, rows, cols, nbits, _ptr(stripe_res), _ptr(agg),
                                                   int(zero_threshold), threads)
    if rc != 0:
        raise _bad_nbits(dtype)
    return agg


def allreduce(gs, res, stripe_res, nbits, zero_threshold, threads=1):
    """Simulated K-worker quantized all-reduce. Updates res[w] and stripe_res[s] in place.
    Returns (per-worker packed buffers after the stripe reduction, assembled packed buffer, out)."""
    k = len(gs)
    rows, cols = gs[0].shape
    dtype = gs[0].dtype
    if not check_nbits(nbits, dtype):
        raise _bad_nbits(dtype)
    nbytes = cols * qcol_bytes(nbits, rows, dtype)
    qs = [np.zeros(nbytes, dtype=np.uint8) for _ in range(k)]
    qagg = np.zeros(nbytes, dtype=np.uint8)
    out = np.zeros((rows, cols), dtype=dtype, order="F")
    vp = ctypes.c_void_p * k
    rc = _fn(lib(), "oracle_allreduce", dtype)(vp(*[g.ctypes.data for g in gs]), vp(*[r.ctypes.data for r in res]),
                                               vp(*[q.ctypes.data for q in qs]), vp(*[s.ctypes.data for s in stripe_res]),
                                               k, rows, cols, nbits, int(zero_threshold), _ptr(qagg), _ptr(out), threads)
    if rc != 0:
        raise _bad_nbits(dtype)
    return qs, qagg, out
