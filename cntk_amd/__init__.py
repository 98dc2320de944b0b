"""cntk_amd -- MI355X (gfx950) implementation of CNTK's quantized-gradient hot path.

Python mirror of the reference's quantizer interface on top of the C ABI in
``include/cntk_amd_quantizer.h`` (``libcntk_amd_quantizer.so``):

    MatrixQuantizerImpl  <->  Source/Math/MatrixQuantizerImpl.h:19-49
    QuantizedMatrix      <->  Source/Math/QuantizedMatrix.h:54-124
    MatrixQuantizer      <->  Source/1BitSGD/MatrixQuantizer.h:24-85
    Matrix               <->  the little of Source/Math/Matrix.h the path needs (dense, column-major)

Both instantiations of the reference are served: float32 matrices with 32-bit QWords and float64 matrices with
64-bit QWords (Source/Math/ValueQuantizer.h:36-57); the element type of the matrices selects the entry points.

torch is used only as the owner of device memory. There is no CPU implementation and no fallback:
if the HIP library is missing, importing the bindings raises.
"""
import ctypes
import os

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcntk_amd_quantizer.so")

CPUDEVICE = -1

_sz = ctypes.c_size_t
_vp = ctypes.c_void_p
_lib = None


class QuantizerError(RuntimeError):
    """RuntimeError of the reference (a failed device call)."""


class QuantizerLogicError(ValueError):
    """LogicError / InvalidArgument of the reference (bad nbits, mismatching sizes)."""


class _QuantizeItem(ctypes.Structure):
    _fields_ = [("in_", _vp), ("res_in", _vp), ("res_out", _vp), ("qbuf", _vp), ("rows", _sz), ("cols", _sz), ("qbuf_bytes", _sz)]


class _UnquantizeItem(ctypes.Structure):
    _fields_ = [("qbuf", _vp), ("out", _vp), ("rows", _sz), ("cols", _sz), ("qbuf_bytes", _sz)]


class _StripeReduceItem(ctypes.Structure):
    _fields_ = [("stripes", ctypes.POINTER(_vp)), ("stripe_res", _vp), ("q_out", _vp), ("agg_out", _vp), ("rows", _sz),
                ("stripe_cols", _sz)]


def lib():
    """The loaded C-ABI library. Raises if it has not been built (python -m cntk_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m cntk_amd.build` "
                              "(there is no CPU fallback)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.cntkq_last_error.restype = ctypes.c_char_p
        L.cntkq_qwords_per_col.argtypes = [_sz, _sz]
        L.cntkq_qwords_per_col.restype = _sz
        L.cntkq_qcol_bytes.argtypes = [_sz, _sz]
        L.cntkq_qcol_bytes.restype = _sz
        L.cntkq_qmatrix_bytes.argtypes = [_sz, _sz, _sz]
        L.cntkq_qmatrix_bytes.restype = _sz
        L.cntkq_stripe_range.argtypes = [_sz, _sz, _sz, ctypes.POINTER(_sz), ctypes.POINTER(_sz)]
        L.cntkq_create.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(_vp)]
        L.cntkq_destroy.argtypes = [_vp]
        L.cntkq_device_id.argtypes = [_vp]
        L.cntkq_stream.argtypes = [_vp]
        L.cntkq_stream.restype = _vp
        L.cntkq_set_main_stream.argtypes = [_vp, _vp]
        L.cntkq_sync_with_main_stream.argtypes = [_vp]
        L.cntkq_stream_wait_event.argtypes = [_vp, _vp]
        L.cntkq_quantize_async.argtypes = [_vp, _vp, _vp, _sz, _sz, _vp, _sz, ctypes.c_int, _sz, _vp, ctypes.c_int]
        L.cntkq_wait_quantize_done.argtypes = [_vp]
        L.cntkq_unquantize_async.argtypes = [_vp, _vp, _sz, ctypes.c_int, _vp, _sz, _sz, _sz, ctypes.c_int]
        L.cntkq_wait_unquantize_done.argtypes = [_vp]
        L.cntkq_stripe_reduce_async.argtypes = [_vp, ctypes.POINTER(_vp), _sz, _sz, _sz, _sz, _sz, _vp, _vp, _vp,
                                                ctypes.c_int]
        L.cntkq_wait_stripe_reduce_done.argtypes = [_vp]
        L.cntkq_quantize_batch_async.argtypes = [_vp, ctypes.POINTER(_QuantizeItem), _sz, _sz, ctypes.c_int]
        L.cntkq_unquantize_batch_async.argtypes = [_vp, ctypes.POINTER(_UnquantizeItem), _sz, _sz, ctypes.c_int]
        L.cntkq_quantize_batch_noalloc.argtypes = L.cntkq_quantize_batch_async.argtypes
        L.cntkq_qwords_per_col_f64.argtypes = [_sz, _sz]
        L.cntkq_qwords_per_col_f64.restype = _sz
        L.cntkq_qcol_bytes_f64.argtypes = [_sz, _sz]
        L.cntkq_qcol_bytes_f64.restype = _sz
        L.cntkq_qmatrix_bytes_f64.argtypes = [_sz, _sz, _sz]
        L.cntkq_qmatrix_bytes_f64.restype = _sz
        L.cntkq_quantize_async_f64.argtypes = L.cntkq_quantize_async.argtypes
        L.cntkq_unquantize_async_f64.argtypes = L.cntkq_unquantize_async.argtypes
        L.cntkq_stripe_reduce_async_f64.argtypes = L.cntkq_stripe_reduce_async.argtypes
        L.cntkq_stripe_reduce_batch_async.argtypes = [_vp, ctypes.POINTER(_StripeReduceItem), _sz, _sz, _sz, _sz, ctypes.c_int]
        L.cntkq_quantize_batch_async_f64.argtypes = L.cntkq_quantize_batch_async.argtypes
        L.cntkq_unquantize_batch_async_f64.argtypes = L.cntkq_unquantize_batch_async.argtypes
        L.cntkq_stripe_reduce_batch_async_f64.argtypes = L.cntkq_stripe_reduce_batch_async.argtypes
        L.cntkq_stripe_reduce_batch_owners_async.argtypes = [_vp, ctypes.POINTER(_StripeReduceItem), ctypes.POINTER(_sz), _sz, _sz, _sz,
                                                             ctypes.c_int]
        L.cntkq_stripe_reduce_batch_owners_async_f64.argtypes = L.cntkq_stripe_reduce_batch_owners_async.argtypes
        for name in ("cntkq_stripe_reduce_max_rows", "cntkq_stripe_reduce_max_rows_f64"):
            getattr(L, name).argtypes = [_sz]
            getattr(L, name).restype = _sz
        for name in ("cntkq_stripe_reduce_takes", "cntkq_stripe_reduce_takes_f64"):
            getattr(L, name).argtypes = [_vp, _sz, _sz, _sz, ctypes.c_int]
        L.cntkq_debug_set_tuning.argtypes = [_vp, ctypes.c_int, ctypes.c_uint, ctypes.c_uint, ctypes.c_int, ctypes.c_int]
        L.cntkq_debug_set_strip_spin_limit.argtypes = [_vp, ctypes.c_uint]
        L.cntkq_debug_strip_max_strips.argtypes = [_vp, _sz, ctypes.c_int]
        L.cntkq_debug_strip_max_strips.restype = ctypes.c_uint
        L.cntkq_debug_strip_max_strips_f64.argtypes = [_vp, _sz, ctypes.c_int]
        L.cntkq_debug_strip_max_strips_f64.restype = ctypes.c_uint
        L.cntkq_set_force_sync.argtypes = [_vp, ctypes.c_int]
        L.cntkq_set_tall_columns_never_wait.argtypes = [_vp, ctypes.c_int]
        _lib = L
    return _lib


def _check(rc):
    if rc == 0:
        return
    msg = lib().cntkq_last_error().decode("utf-8", "replace")
    if rc == 3:
        raise QuantizerError(msg)
    raise QuantizerLogicError(msg)


def _is64(dtype):
    """True for float64, False for float32 (numpy or torch dtype); anything else is refused."""
    if dtype in (np.float32, torch.float32) or dtype == np.dtype(np.float32):
        return False
    if dtype in (np.float64, torch.float64) or dtype == np.dtype(np.float64):
        return True
    raise QuantizerLogicError("element type must be float32 or float64")


def _fn(name, dtype):
    return getattr(lib(), name + ("_f64" if _is64(dtype) else ""))


def qwords_per_col(rows, nbits, dtype=np.float32):
    return _fn("cntkq_qwords_per_col", dtype)(rows, nbits)


def qcol_bytes(nbits, rows, dtype=np.float32):
    return _fn("cntkq_qcol_bytes", dtype)(nbits, rows)


def stripe_range(cols, rank, workers):
    """GetStripeForNode (Source/1BitSGD/AllReduceDistGradAggregator.h:56-65) -> (start_col, num_cols)."""
    s, n = _sz(), _sz()
    _check(lib().cntkq_stripe_range(cols, rank, workers, ctypes.byref(s), ctypes.byref(n)))
    return s.value, n.value


# ---------------------------------------------------------------------------------------------------


class Matrix:
    """Dense float32 or float64 matrix in column-major storage on one device (Source/Math/Matrix.h, the part used
    here: Matrix<float> / Matrix<double>).

    ``data`` is a flat torch tensor of rows * cols elements: element (i, j) is data[j * rows + i].
    """

    def __init__(self, rows, cols, device_id=0, data=None, dtype=torch.float32):
        self.rows, self.cols, self.device_id = int(rows), int(cols), device_id
        if data is None:
            dev = "cpu" if device_id < 0 else "cuda:%d" % device_id
            data = torch.zeros(self.rows * self.cols, dtype=torch.float64 if _is64(dtype) else torch.float32, device=dev)
        if data.dtype not in (torch.float32, torch.float64) or data.dim() != 1 or data.numel() != self.rows * self.cols:
            raise QuantizerLogicError("Matrix data must be a flat float32 or float64 tensor of rows * cols elements")
        if not data.is_contiguous():
            raise QuantizerLogicError("Matrix data must be contiguous")
        self.data = data

    @property
    def dtype(self):
        return self.data.dtype

    @classmethod
    def from_numpy(cls, a, device_id=0):
        """From a (rows, cols) float32 / float64 numpy array (anything else becomes float32); the values are laid
        out column-major on the device."""
        a = np.asarray(a)
        a = np.asfortranarray(a, dtype=a.dtype if a.dtype == np.float64 else np.float32)
        flat = torch.from_numpy(a.reshape(-1, order="F").copy())
        if device_id >= 0:
            flat = flat.to("cuda:%d" % device_id)
        return cls(a.shape[0], a.shape[1], device_id, flat)

    def to_numpy(self):
        """(rows, cols) numpy array in Fortran order."""
        return np.asfortranarray(self.data.detach().cpu().numpy().reshape((self.rows, self.cols), order="F"))

    def GetNumRows(self):
        return self.rows

    def GetNumCols(self):
        return self.cols

    def GetDeviceId(self):
        return self.device_id

    def Data(self):
        return self.data.data_ptr()

    def ColumnSlice(self, start_col, num_cols):
        """Zero-copy view of columns [start_col, start_col + num_cols) (Source/Math/Matrix.h:194)."""
        if start_col + num_cols > self.cols:
            raise QuantizerLogicError("ColumnSlice out of range")
        view = self.data[start_col * self.rows:(start_col + num_cols) * self.rows]
        return Matrix(self.rows, num_cols, self.device_id, view)

    def SetValue(self, v):
        self.data.fill_(v)


class QuantizedMatrix:
    """Packed matrix: per column {lower, upper, bits[nq]} (Source/Math/QuantizedMatrix.h:27-124); float and 32-bit
    QWords for dtype float32, double and 64-bit QWords for float64.

    device_id >= 0 keeps the buffer on that GPU; CPUDEVICE keeps it in pinned host memory, as the
    reference's v1 aggregator does through its page-locked allocator
    (Source/1BitSGD/AllReduceDistGradAggregator.h:76-77, 88).
    """

    def __init__(self, num_rows, num_cols, nbits, device_id=0, _buffer=None, dtype=torch.float32):
        self.is64 = _is64(dtype)
        word_bits = 64 if self.is64 else 32
        if nbits not in (1, 2, 4, 8, 16, 32, 64) or nbits > word_bits:
            # Source/Math/QuantizedMatrix.cpp:12-15
            raise QuantizerLogicError("Quantization: 'nbits' must be a power of two that divides %d" % word_bits)
        self.num_rows, self.num_cols, self.nbits, self.device_id = int(num_rows), int(num_cols), int(nbits), device_id
        self.dtype = torch.float64 if self.is64 else torch.float32
        self.qcol_size = qcol_bytes(nbits, self.num_rows, self.dtype)
        size = self.qcol_size * self.num_cols
        if _buffer is None:
            if device_id < 0:
                _buffer = torch.zeros(size, dtype=torch.uint8, pin_memory=torch.cuda.is_available())
            else:
                _buffer = torch.zeros(size, dtype=torch.uint8, device="cuda:%d" % device_id)
        self.buffer = _buffer

    def GetNumRows(self):
        return self.num_rows

    def GetNumCols(self):
        return self.num_cols

    def GetNumBits(self):
        return self.nbits

    def GetDeviceId(self):
        return self.device_id

    def GetSize(self):
        return self.buffer.numel()

    def Buffer(self):
        return self.buffer.data_ptr()

    def ColumnSlice(self, start_col, num_cols):
        """Non-owning view of a run of columns (Source/Math/QuantizedMatrix.cpp:102-107)."""
        if start_col + num_cols > self.num_cols:
            raise QuantizerLogicError("ColumnSlice out of range")
        view = self.buffer[start_col * self.qcol_size:(start_col + num_cols) * self.qcol_size]
        return QuantizedMatrix(self.num_rows, num_cols, self.nbits, self.device_id, view, dtype=self.dtype)

    def to_numpy(self):
        return self.buffer.detach().cpu().numpy().copy()

    def Decode(self, row_start, row_end, col_start, col_end):
        """Host-side reading of a range of the packed matrix, by the layout alone (the index arithmetic of
        QuantizedMatrix::Print, Source/Math/QuantizedMatrix.cpp:143-169): returns (lower, upper, codes, values) with
        lower / upper per column and codes / values of shape (rows, cols) of the inclusive range. A debugging aid: the
        values are reconstructed on the host in the element type, value = (code + 0.5) * ufactor + lower
        (Source/Math/ValueQuantizer.h:68-97, 131-141)."""
        if not (row_start <= row_end < self.num_rows and col_start <= col_end < self.num_cols):
            raise QuantizerLogicError("Index out of range.")  # Source/Math/QuantizedMatrix.cpp:116-120
        ft, wt = (np.float64, np.uint64) if self.is64 else (np.float32, np.uint32)
        word_bits, hdr = (64, 16) if self.is64 else (32, 8)
        raw = self.to_numpy()
        nq = qwords_per_col(self.num_rows, self.nbits, self.dtype)
        ncols, nrows = col_end - col_start + 1, row_end - row_start + 1
        lower, upper = np.empty(ncols, ft), np.empty(ncols, ft)
        codes, values = np.empty((nrows, ncols), wt), np.empty((nrows, ncols), ft)
        rows = np.arange(row_start, row_end + 1)
        word_idx, slot = rows % nq, (rows // nq).astype(wt)
        for jj, j in enumerate(range(col_start, col_end + 1)):
            col = raw[j * self.qcol_size:(j + 1) * self.qcol_size]
            lo, hi = col[:hdr].view(ft)
            bits = col[hdr:].view(wt)
            lower[jj], upper[jj] = lo, hi
            if self.nbits == word_bits:  # pass-through: the code is the value's bit pattern
                codes[:, jj] = bits[word_idx]
                values[:, jj] = bits[word_idx].view(ft)
                continue
            mask = wt((1 << self.nbits) - 1)
            c = (bits[word_idx] >> (slot * wt(self.nbits))) & mask
            used = ft((1 << self.nbits) - (1 if self.nbits > 1 else 0))
            with np.errstate(invalid="ignore", over="ignore"):
                spread = ft(hi - lo)
                ufactor = ft(0) if not (spread >= ft(1e-36)) else ft(spread / used)
                values[:, jj] = (c.astype(ft) + ft(0.5)) * ufactor + lo
            codes[:, jj] = c
        return lower, upper, codes, values

    def Print(self, matrix_name, row_start, row_end, col_start, col_end, file=None):
        """QuantizedMatrix::Print (Source/Math/QuantizedMatrix.cpp:109-171): the column bounds, then code and
        reconstructed value of every element of the range, to stderr."""
        import sys
        out = file if file is not None else sys.stderr
        lower, upper, codes, values = self.Decode(row_start, row_end, col_start, col_end)
        name = matrix_name if matrix_name is not None else "Unnamed Matrix"
        print("\n###### %s (%d, %d) ######" % (name, self.num_rows, self.num_cols), file=out)
        print("\n------ Print Range (%d:%d, %d:%d) ------" % (row_start, row_end, col_start, col_end), file=out)
        print("".join("Lower=%.10f,Upper=%.10f\t" % (lo, hi) for lo, hi in zip(lower, upper)), file=out)
        for i in range(codes.shape[0]):
            print("".join("%10d (%.10f)          \t" % (int(codes[i, j]), values[i, j]) for j in range(codes.shape[1])), file=out)

    def from_numpy(self, a):
        self.buffer.copy_(torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint8)))


class PreparedBatch:
    """The argument block of one batched call, built once by MatrixQuantizerImpl.Prepare...Batch. It holds addresses,
    not matrices: the caller keeps the matrices alive and in place for as long as it uses the block."""

    def __init__(self, kind, array, count, nbits, keep, workers=0, dtype=torch.float32):
        self.kind, self.array, self.count, self.nbits, self.keep, self.workers = kind, array, count, nbits, keep, workers
        self.dtype = dtype


class MatrixQuantizerImpl:
    """The quantizer object (Source/Math/MatrixQuantizerImpl.h:19-49) for one GPU."""

    def __init__(self, device_id, use_async, force_sync=False):
        if device_id < 0:
            # the reference returns its CPU quantizer here; this library has none
            raise QuantizerError("MatrixQuantizerImpl.Create: no CPU quantizer in this library (device %d)" % device_id)
        h = _vp()
        _check(lib().cntkq_create(device_id, int(bool(use_async)), ctypes.byref(h)))
        self._h = h
        self._device_id = device_id
        if force_sync:
            # MatrixQuantizerGPU(deviceId, useDedicatedComputeStream, forceSync) (Source/Math/MatrixQuantizerGPU.h:20)
            _check(lib().cntkq_set_force_sync(h, 1))

    @staticmethod
    def Create(device_id, use_async):
        return MatrixQuantizerImpl(device_id, use_async)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.cntkq_destroy(h)

    def GetDeviceId(self):
        return self._device_id

    def stream(self):
        return lib().cntkq_stream(self._h)

    def SetMainStream(self, hip_stream):
        """The stream a quantizer without a dedicated stream issues on, and the one SynchronizeWithMainStream orders
        against (the reference's GetStream(), Source/Math/MatrixQuantizerGPU.cu:248-252); a hipStream_t as an integer,
        e.g. torch.cuda.current_stream().cuda_stream."""
        _check(lib().cntkq_set_main_stream(self._h, hip_stream))

    def SynchronizeWithMainStream(self):
        """MatrixComputeStreamEvent::SynchronizeQuantizationComputeStreamWithEvent
        (Source/Math/MatrixQuantizerGPU.cu:347-371)."""
        _check(lib().cntkq_sync_with_main_stream(self._h))

    def WaitEvent(self, hip_event):
        """Work issued through this quantizer from now on starts only after `hip_event` (a hipEvent_t as an integer,
        e.g. torch.cuda.Event(...).cuda_event after record()) has completed."""
        _check(lib().cntkq_stream_wait_event(self._h, hip_event))

    def QuantizeAsync(self, in_matrix, in_residual, out_qmatrix, out_residual, zero_threshold_for_1bit):
        rows, cols = in_matrix.GetNumRows(), in_matrix.GetNumCols()
        # the reference asserts these (Source/Math/MatrixQuantizerGPU.cu:229-232)
        for m in (in_residual, out_residual, out_qmatrix):
            if m.GetNumRows() != rows or m.GetNumCols() != cols:
                raise QuantizerLogicError("QuantizeAsync: matrix dimensions do not match")
            if m.dtype != in_matrix.dtype:
                raise QuantizerLogicError("QuantizeAsync: element types do not match")
        _check(_fn("cntkq_quantize_async", in_matrix.dtype)(self._h, in_matrix.Data(), in_residual.Data(), rows, cols,
                                          out_qmatrix.Buffer(), out_qmatrix.GetSize(),
                                          int(out_qmatrix.GetDeviceId() < 0), out_qmatrix.GetNumBits(),
                                          out_residual.Data(), int(bool(zero_threshold_for_1bit))))

    def WaitQuantizeAsyncDone(self):
        _check(lib().cntkq_wait_quantize_done(self._h))

    def UnquantizeAsync(self, in_qmatrix, out_matrix, add=False):
        rows, cols = out_matrix.GetNumRows(), out_matrix.GetNumCols()
        # the reference asserts this (Source/Math/MatrixQuantizerGPU.cu:297)
        if in_qmatrix.GetNumRows() != rows or in_qmatrix.GetNumCols() != cols:
            raise QuantizerLogicError("UnquantizeAsync: matrix dimensions do not match")
        if in_qmatrix.dtype != out_matrix.dtype:
            raise QuantizerLogicError("UnquantizeAsync: element types do not match")
        _check(_fn("cntkq_unquantize_async", out_matrix.dtype)(self._h, in_qmatrix.Buffer(), in_qmatrix.GetSize(),
                                            int(in_qmatrix.GetDeviceId() < 0), out_matrix.Data(), rows, cols,
                                            in_qmatrix.GetNumBits(), int(bool(add))))

    def WaitUnquantizeAsyncDone(self):
        _check(lib().cntkq_wait_unquantize_done(self._h))

    def QuantizeBatchAsync(self, items, zero_threshold_for_1bit):
        """The aggregator's loop over its gradient matrices as one call (Source/1BitSGD/AllReduceDistGradAggregator.h:288-300).
        items: sequence of (in_matrix, in_residual, out_qmatrix, out_residual); all packed matrices on the device, of
        one bit width and one element type."""
        if isinstance(items, PreparedBatch):
            if items.kind != "quantize":
                raise QuantizerLogicError("QuantizeBatchAsync: prepared for another call")
            if items.count:
                _check(_fn("cntkq_quantize_batch_async", items.dtype)(self._h, items.array, items.count, items.nbits,
                                                                      int(bool(zero_threshold_for_1bit))))
            return
        self.QuantizeBatchAsync(self.PrepareQuantizeBatch(items), zero_threshold_for_1bit)

    def QuantizeBatchNoAlloc(self, items, zero_threshold_for_1bit):
        """QuantizeBatchAsync through the entry point that allocates nothing (float32 only): the argument table lives in
        a fixed array in the library's device image; at most 256 items. No counterpart in the reference."""
        prep = items if isinstance(items, PreparedBatch) else self.PrepareQuantizeBatch(items)
        if prep.kind != "quantize" or _is64(prep.dtype):
            raise QuantizerLogicError("QuantizeBatchNoAlloc: needs a float32 quantize item list")
        if prep.count:
            _check(lib().cntkq_quantize_batch_noalloc(self._h, prep.array, prep.count, prep.nbits, int(bool(zero_threshold_for_1bit))))

    @staticmethod
    def PrepareQuantizeBatch(items):
        """Checks the items of QuantizeBatchAsync and lays them out for the call once; the result can be passed to
        QuantizeBatchAsync in place of the item list for as long as the matrices stay where they are."""
        if not items:
            return PreparedBatch("quantize", None, 0, 0, ())
        nbits = items[0][2].GetNumBits()
        arr = (_QuantizeItem * len(items))()
        for k, (g, r_in, q, r_out) in enumerate(items):
            rows, cols = g.GetNumRows(), g.GetNumCols()
            for m in (r_in, r_out, q):
                if m.GetNumRows() != rows or m.GetNumCols() != cols:
                    raise QuantizerLogicError("QuantizeBatchAsync: matrix dimensions do not match")
            if q.GetNumBits() != nbits or q.GetDeviceId() < 0:
                raise QuantizerLogicError("QuantizeBatchAsync: packed matrices must share one bit width and live on the device")
            if any(m.dtype != items[0][0].dtype for m in (g, r_in, r_out, q)):
                raise QuantizerLogicError("QuantizeBatchAsync: all matrices of a call must have one element type")
            arr[k] = _QuantizeItem(g.Data(), r_in.Data(), r_out.Data(), q.Buffer(), rows, cols, q.GetSize())
        return PreparedBatch("quantize", arr, len(items), nbits, (), dtype=items[0][0].dtype)

    def UnquantizeBatchAsync(self, items, add=False):
        """The aggregator's final loop (Source/1BitSGD/AllReduceDistGradAggregator.h:517-522) as one call.
        items: sequence of (in_qmatrix, out_matrix)."""
        if isinstance(items, PreparedBatch):
            if items.kind != "unquantize":
                raise QuantizerLogicError("UnquantizeBatchAsync: prepared for another call")
            if items.count:
                _check(_fn("cntkq_unquantize_batch_async", items.dtype)(self._h, items.array, items.count, items.nbits, int(bool(add))))
            return
        self.UnquantizeBatchAsync(self.PrepareUnquantizeBatch(items), add)

    @staticmethod
    def PrepareUnquantizeBatch(items):
        """The items of UnquantizeBatchAsync, checked and laid out once (see PrepareQuantizeBatch)."""
        if not items:
            return PreparedBatch("unquantize", None, 0, 0, ())
        nbits = items[0][0].GetNumBits()
        arr = (_UnquantizeItem * len(items))()
        for k, (q, out) in enumerate(items):
            if q.GetNumRows() != out.GetNumRows() or q.GetNumCols() != out.GetNumCols():
                raise QuantizerLogicError("UnquantizeBatchAsync: matrix dimensions do not match")
            if q.GetNumBits() != nbits or q.GetDeviceId() < 0:
                raise QuantizerLogicError("UnquantizeBatchAsync: packed matrices must share one bit width and live on the device")
            if q.dtype != items[0][1].dtype or out.dtype != items[0][1].dtype:
                raise QuantizerLogicError("UnquantizeBatchAsync: all matrices of a call must have one element type")
            arr[k] = _UnquantizeItem(q.Buffer(), out.Data(), out.GetNumRows(), out.GetNumCols(), q.GetSize())
        return PreparedBatch("unquantize", arr, len(items), nbits, (), dtype=items[0][1].dtype)

    def StripeReduceAsync(self, stripes, owner, stripe_residual, out_qstripe, zero_threshold_for_1bit, agg_out=None):
        """Fused stripe reduction of the quantized all-reduce (dataflow of
        Source/1BitSGD/AllReduceDistGradAggregator.h:365-436): stripes[w] is worker w's packed stripe."""
        k = len(stripes)
        rows, cols, nbits = out_qstripe.GetNumRows(), out_qstripe.GetNumCols(), out_qstripe.GetNumBits()
        for s in stripes:
            if s.GetNumRows() != rows or s.GetNumCols() != cols or s.GetNumBits() != nbits or s.GetDeviceId() < 0:
                raise QuantizerLogicError("StripeReduceAsync: stripes must be device-resident and of equal shape")
            if s.dtype != out_qstripe.dtype:
                raise QuantizerLogicError("StripeReduceAsync: element types do not match")
        if stripe_residual.GetNumRows() != rows or stripe_residual.GetNumCols() != cols:
            raise QuantizerLogicError("StripeReduceAsync: stripe residual has the wrong shape")
        if stripe_residual.dtype != out_qstripe.dtype or (agg_out is not None and agg_out.dtype != out_qstripe.dtype):
            raise QuantizerLogicError("StripeReduceAsync: element types do not match")
        arr = (_vp * k)(*[s.Buffer() for s in stripes])
        _check(_fn("cntkq_stripe_reduce_async", out_qstripe.dtype)(self._h, arr, k, owner, rows, cols, nbits, stripe_residual.Data(),
                                               out_qstripe.Buffer(), agg_out.Data() if agg_out is not None else None,
                                               int(bool(zero_threshold_for_1bit))))

    def SetTallColumnsNeverWait(self, never_wait):
        """Columns taller than one workgroup holds: several launches whose workgroups never wait for each other instead of one
        launch whose workgroups do (for handles whose stream shares the device with other work)."""
        _check(lib().cntkq_set_tall_columns_never_wait(self._h, int(bool(never_wait))))

    def StripeReduceTakes(self, rows, cols, nbits, zero_threshold_for_1bit=False, dtype=torch.float32):
        """Whether StripeReduceAsync takes stripes of this shape; where not, the caller runs the reference's sequence of
        UnquantizeAsync ... QuantizeAsync calls (Source/1BitSGD/AllReduceDistGradAggregator.h:365-436)."""
        return bool(_fn("cntkq_stripe_reduce_takes", dtype)(self._h, rows, cols, nbits, int(bool(zero_threshold_for_1bit))))

    def StripeReduceBatchAsync(self, items, owner, zero_threshold_for_1bit):
        """The owner's stripe reductions of a whole gradient set as one call. items: sequence of
        (stripes, stripe_residual, out_qstripe, agg_out or None), one per gradient matrix, one element type."""
        if isinstance(items, PreparedBatch):
            if items.kind != "stripe_reduce":
                raise QuantizerLogicError("StripeReduceBatchAsync: prepared for another call")
            if items.count and isinstance(owner, (list, tuple)):
                # an owner per item: the stripes of all the ranks of a cluster simulated on one GPU
                if len(owner) != items.count:
                    raise QuantizerLogicError("StripeReduceBatchAsync: one owner per item")
                owners = (_sz * items.count)(*owner)
                _check(_fn("cntkq_stripe_reduce_batch_owners_async", items.dtype)(self._h, items.array, owners, items.count, items.workers,
                                                                                  items.nbits, int(bool(zero_threshold_for_1bit))))
            elif items.count:
                _check(_fn("cntkq_stripe_reduce_batch_async", items.dtype)(self._h, items.array, items.count, items.workers, owner,
                                                                           items.nbits, int(bool(zero_threshold_for_1bit))))
            return
        self.StripeReduceBatchAsync(self.PrepareStripeReduceBatch(items), owner, zero_threshold_for_1bit)

    @staticmethod
    def PrepareStripeReduceBatch(items):
        """The items of StripeReduceBatchAsync, checked and laid out once (see PrepareQuantizeBatch)."""
        if not items:
            return PreparedBatch("stripe_reduce", None, 0, 0, ())
        k = len(items[0][0])
        nbits = items[0][2].GetNumBits()
        arr = (_StripeReduceItem * len(items))()
        keep = []
        for n, (stripes, stripe_residual, out_qstripe, agg_out) in enumerate(items):
            rows, cols = out_qstripe.GetNumRows(), out_qstripe.GetNumCols()
            if len(stripes) != k or out_qstripe.GetNumBits() != nbits:
                raise QuantizerLogicError("StripeReduceBatchAsync: items must share the worker count and the bit width")
            for s in stripes:
                if s.GetNumRows() != rows or s.GetNumCols() != cols or s.GetNumBits() != nbits or s.GetDeviceId() < 0:
                    raise QuantizerLogicError("StripeReduceBatchAsync: stripes must be device-resident and of equal shape")
            if stripe_residual.GetNumRows() != rows or stripe_residual.GetNumCols() != cols:
                raise QuantizerLogicError("StripeReduceBatchAsync: stripe residual has the wrong shape")
            mats = list(stripes) + [stripe_residual, out_qstripe] + ([agg_out] if agg_out is not None else [])
            if any(m.dtype != items[0][1].dtype for m in mats):
                raise QuantizerLogicError("StripeReduceBatchAsync: all matrices of a call must have one element type")
            ptrs = (_vp * k)(*[s.Buffer() for s in stripes])
            keep.append(ptrs)
            arr[n] = _StripeReduceItem(ptrs, stripe_residual.Data(), out_qstripe.Buffer(),
                                       agg_out.Data() if agg_out is not None else None, rows, cols)
        return PreparedBatch("stripe_reduce", arr, len(items), nbits, keep, workers=k, dtype=items[0][1].dtype)

    def WaitStripeReduceDone(self):
        _check(lib().cntkq_wait_stripe_reduce_done(self._h))

    def _set_tuning(self, quantize_path=0, tile_gs=0, unq_slots=0, unq_mode=0, tile_stage=-1):
        _check(lib().cntkq_debug_set_tuning(self._h, quantize_path, tile_gs, unq_slots, unq_mode, tile_stage))

    def _set_strip_spin_limit(self, limit):
        _check(lib().cntkq_debug_set_strip_spin_limit(self._h, limit))

    def _strip_max_strips(self, nbits, zero_threshold_for_1bit=False, dtype=torch.float32):
        """Most strips per column that the strip kernels take on this device at this bit width (0: none)."""
        f = lib().cntkq_debug_strip_max_strips_f64 if dtype == torch.float64 else lib().cntkq_debug_strip_max_strips
        return int(f(self._h, nbits, 1 if zero_threshold_for_1bit else 0))


class MatrixQuantizer:
    """Quantizer that owns its error-feedback residual (Source/1BitSGD/MatrixQuantizer.h:24-85)."""

    def __init__(self, num_rows, num_cols, device_id, use_async, dtype=torch.float32):
        self._impl = MatrixQuantizerImpl.Create(device_id, use_async)
        self._residual = Matrix(num_rows, num_cols, device_id, dtype=dtype)

    def QuantizeAsync(self, in_matrix, out_qmatrix, zero_threshold_for_1bit, in_residual=None, out_residual=None):
        if in_residual is None:
            in_residual = out_residual = self._residual
        self._impl.QuantizeAsync(in_matrix, in_residual, out_qmatrix, out_residual, zero_threshold_for_1bit)

    def WaitQuantizeAsyncDone(self):
        self._impl.WaitQuantizeAsyncDone()

    def UnquantizeAsync(self, in_qmatrix, out_matrix, add=False):
        self._impl.UnquantizeAsync(in_qmatrix, out_matrix, add)

    def WaitUnquantizeAsyncDone(self):
        self._impl.WaitUnquantizeAsyncDone()

    def GetDeviceId(self):
        return self._impl.GetDeviceId()

    def ResetResidue(self):
        self._residual.SetValue(0.0)

    def GetResidualMatrix(self):
        return self._residual

    @property
    def impl(self):
        return self._impl
