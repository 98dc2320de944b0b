"""ctypes front end of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only the tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this package; the shipped library (``cntk_amd``) never does.

Matrices are float32 numpy arrays in column-major (Fortran) order, shape ``(rows, cols)``, exactly
the memory layout the reference's ``Matrix<float>::Data()`` hands to its quantizer. Packed matrices
are flat ``uint8`` arrays of ``cols * qcol_bytes(nbits, rows)`` bytes.

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
        _REF = L
    return _REF


# ---------------------------------------------------------------------------------------------


def _colmajor(a, name):
    if a.dtype != np.float32 or a.ndim != 2 or not a.flags.f_contiguous:
        raise ValueError("%s must be a 2-D float32 array in column-major (order='F') layout" % name)
    return a


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def qwords_per_col(rows, nbits):
    return lib().oracle_qwords_per_col(rows, nbits)


def qcol_bytes(nbits, rows):
    return lib().oracle_qcol_bytes(nbits, rows)


def stripe_range(cols, rank, workers):
    s, n = _sz(), _sz()
    lib().oracle_stripe_range(cols, rank, workers, ctypes.byref(s), ctypes.byref(n))
    return s.value, n.value


def column_stats(g, r, j, nbits, zero_threshold):
    _colmajor(g, "g"), _colmajor(r, "r")
    lo, hi = ctypes.c_float(), ctypes.c_float()
    lib().oracle_column_stats(_ptr(g), _ptr(r), g.shape[0], j, nbits, int(zero_threshold),
                              ctypes.byref(lo), ctypes.byref(hi))
    return np.float32(lo.value), np.float32(hi.value)


def quantize(g, r_in, nbits, zero_threshold, r_out=None, threads=1, use_ref=False):
    """Returns (packed uint8 buffer, new residual). r_out=None allocates; r_out=r_in is in place."""
    _colmajor(g, "g"), _colmajor(r_in, "r_in")
    rows, cols = g.shape
    if r_in.shape != g.shape:
        raise ValueError("residual shape mismatch")
    if r_out is None:
        r_out = np.zeros_like(g, order="F")
    _colmajor(r_out, "r_out")
    q = np.zeros(cols * qcol_bytes(nbits, rows), dtype=np.uint8)
    if use_ref:
        rc = ref_lib().ref_quantize(_ptr(g), _ptr(r_in), rows, cols, _ptr(q), nbits, _ptr(r_out), int(zero_threshold))
    else:
        rc = lib().oracle_quantize(_ptr(g), _ptr(r_in), rows, cols, _ptr(q), nbits, _ptr(r_out),
                                   int(zero_threshold), threads)
    if rc != 0:
        raise ValueError("nbits must be one of 1, 2, 4, 8, 16, 32")
    return q, r_out


def pack_with_headers(g, r_in, q_with_headers, nbits, zero_threshold, threads=1):
    """Codes and residual under the headers already stored in q_with_headers (not modified).
    Returns (packed buffer, residual)."""
    _colmajor(g, "g"), _colmajor(r_in, "r_in")
    rows, cols = g.shape
    q = np.array(q_with_headers, dtype=np.uint8, copy=True)
    if q.size != cols * qcol_bytes(nbits, rows):
        raise ValueError("packed buffer has the wrong size")
    r_out = np.zeros_like(g, order="F")
    rc = lib().oracle_pack_with_headers(_ptr(g), _ptr(r_in), rows, cols, _ptr(q), nbits, _ptr(r_out),
                                        int(zero_threshold), threads)
    if rc != 0:
        raise ValueError("nbits must be one of 1, 2, 4, 8, 16, 32")
    return q, r_out


def unquantize(q, rows, cols, nbits, out=None, add=False, threads=1, use_ref=False):
    if q.dtype != np.uint8 or q.size != cols * qcol_bytes(nbits, rows):
        raise ValueError("packed buffer has the wrong size")
    if out is None:
        out = np.zeros((rows, cols), dtype=np.float32, order="F")
    _colmajor(out, "out")
    if use_ref:
        rc = ref_lib().ref_unquantize(_ptr(q), rows, cols, nbits, _ptr(out), int(add))
    else:
        rc = lib().oracle_unquantize(_ptr(q), rows, cols, nbits, _ptr(out), int(add), threads)
    if rc != 0:
        raise ValueError("nbits must be one of 1, 2, 4, 8, 16, 32")
    return out


def headers(q, rows, cols, nbits):
    """(lower, upper) float32 arrays read from a packed buffer."""
    stride = qcol_bytes(nbits, rows)
    h = np.lib.stride_tricks.as_strided(q.view(np.uint8), shape=(cols, 8), strides=(stride, 1))
    h = np.ascontiguousarray(h).view(np.float32)
    return h[:, 0].copy(), h[:, 1].copy()


def words(q, rows, cols, nbits):
    """(cols, nq) uint32 array of the packed QWords."""
    stride = qcol_bytes(nbits, rows)
    nq = qwords_per_col(rows, nbits)
    w = np.lib.stride_tricks.as_strided(q[8:].view(np.uint8), shape=(cols, nq * 4), strides=(stride, 1))
    return np.ascontiguousarray(w).view(np.uint32)


def codes(q, rows, cols, nbits):
    """(rows, cols) uint32 array of per-element codes, undoing the interleaved packing:
    element i lives in word i % nq at bit (i // nq) * nbits (Source/Math/QuantizedMatrix.cpp:143-169)."""
    w = words(q, rows, cols, nbits)
    nq = w.shape[1]
    i = np.arange(rows)
    mask = np.uint32(0xFFFFFFFF) if nbits == 32 else np.uint32((1 << nbits) - 1)
    c = (w[:, i % nq] >> ((i // nq) * nbits).astype(np.uint32)) & mask
    return np.asfortranarray(c.T)


def stripe_reduce(qs, owner, rows, cols, nbits, stripe_res, zero_threshold, threads=1):
    """In place on qs[owner]'s stripe and stripe_res; returns the fp32 aggregate (rows x len)."""
    k = len(qs)
    _, n = stripe_range(cols, owner, k)
    agg = np.zeros((rows, n), dtype=np.float32, order="F")
    arr = (ctypes.c_void_p * k)(*[q.ctypes.data for q in qs])
    rc = lib().oracle_stripe_reduce(arr, k, owner, rows, cols, nbits, _ptr(stripe_res), _ptr(agg),
                                    int(zero_threshold), threads)
    if rc != 0:
        raise ValueError("nbits must be one of 1, 2, 4, 8, 16, 32")
    return agg


def allreduce(gs, res, stripe_res, nbits, zero_threshold, threads=1):
    """Simulated K-worker quantized all-reduce. Updates res[w] and stripe_res[s] in place.
    Returns (per-worker packed buffers after the stripe reduction, assembled packed buffer, out)."""
    k = len(gs)
    rows, cols = gs[0].shape
    nbytes = cols * qcol_bytes(nbits, rows)
    qs = [np.zeros(nbytes, dtype=np.uint8) for _ in range(k)]
    qagg = np.zeros(nbytes, dtype=np.uint8)
    out = np.zeros((rows, cols), dtype=np.float32, order="F")
    vp = ctypes.c_void_p * k
    rc = lib().oracle_allreduce(vp(*[g.ctypes.data for g in gs]), vp(*[r.ctypes.data for r in res]),
                                vp(*[q.ctypes.data for q in qs]), vp(*[s.ctypes.data for s in stripe_res]),
                                k, rows, cols, nbits, int(zero_threshold), _ptr(qagg), _ptr(out), threads)
    if rc != 0:
        raise ValueError("nbits must be one of 1, 2, 4, 8, 16, 32")
    return qs, qagg, out
