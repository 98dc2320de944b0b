// C++ host side of the MI355X gradient quantizer: the reference's class shapes on top of the C ABI.
//
//   cntk_amd::MatrixQuantizerImpl<E>       <->  Source/Math/MatrixQuantizerImpl.h:19-49
//   cntk_amd::QuantizedMatrix<E>           <->  Source/Math/QuantizedMatrix.h:54-124, Source/Math/QuantizedMatrix.cpp
//   cntk_amd::QuantizedColumn<E>           <->  Source/Math/QuantizedMatrix.h:27-48
//   cntk_amd::MatrixQuantizer<E>           <->  Source/1BitSGD/MatrixQuantizer.h:24-85
//   cntk_amd::MatrixComputeStreamEvent     <->  Source/Math/MatrixQuantizerImpl.h:53-72
//   cntk_amd::Matrix<E>                         the little of Source/Math/Matrix.h this path needs
//
// Same method names, argument meaning and error behaviour (LogicError / RuntimeError / InvalidArgument become
// std::logic_error / std::runtime_error / std::invalid_argument). ElemType is float or double (the batched calls: float
// only). Header-only; link with
// libcntk_amd_quantizer.so and the HIP runtime. There is no CPU quantizer: Create(deviceId < 0) throws.
#pragma once

#include "../../include/cntk_amd_quantizer.h"

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

namespace cntk_amd {

constexpr int CPUDEVICE = -1;

namespace detail {
inline void Check(int rc)
{
    if (rc == CNTKQ_OK)
        return;
    const std::string msg = cntkq_last_error();
    if (rc == CNTKQ_RUNTIME_ERROR)
        throw std::runtime_error(msg);
    if (rc == CNTKQ_INVALID_ARGUMENT)
        throw std::invalid_argument(msg);
    throw std::logic_error(msg);
}

inline void HipCheck(hipError_t rc, const char* what)
{
    if (rc != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(rc));
}

// What differs between the two instantiations the reference has (Source/Math/MatrixQuantizerImpl.cpp:28-29): the QWord
// (Source/Math/ValueQuantizer.h:36-57) and the entry points of the C ABI.
template <class ElemType>
struct Abi;

template <>
struct Abi<float>
{
    typedef uint32_t QWord;
    static size_t QColBytes(size_t bits, size_t rows) { return cntkq_qcol_bytes(bits, rows); }
    static size_t StripeReduceMaxRows(size_t bits) { return cntkq_stripe_reduce_max_rows(bits); }
    static bool StripeReduceTakes(cntkq_quantizer* h, size_t rows, size_t cols, size_t bits, int zt)
    {
        return cntkq_stripe_reduce_takes(h, rows, cols, bits, zt) != 0;
    }
    static int Quantize(cntkq_quantizer* h, const float* in, const float* resIn, size_t rows, size_t cols, void* q, size_t qBytes, int onHost,
                        size_t bits, float* resOut, int zt)
    {
        return cntkq_quantize_async(h, in, resIn, rows, cols, q, qBytes, onHost, bits, resOut, zt);
    }
    static int Unquantize(cntkq_quantizer* h, const void* q, size_t qBytes, int onHost, float* out, size_t rows, size_t cols, size_t bits, int add)
    {
        return cntkq_unquantize_async(h, q, qBytes, onHost, out, rows, cols, bits, add);
    }
    static int StripeReduce(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner, size_t rows, size_t cols,
                            size_t bits, float* stripeRes, void* qOut, float* agg, int zt)
    {
        return cntkq_stripe_reduce_async(h, stripes, workers, owner, rows, cols, bits, stripeRes, qOut, agg, zt);
    }
    typedef cntkq_quantize_item QuantizeItem;
    typedef cntkq_unquantize_item UnquantizeItem;
    typedef cntkq_stripe_reduce_item StripeReduceItem;
    static int QuantizeBatch(cntkq_quantizer* h, const QuantizeItem* items, size_t n, size_t bits, int zt)
    {
        return cntkq_quantize_batch_async(h, items, n, bits, zt);
    }
    static int UnquantizeBatch(cntkq_quantizer* h, const UnquantizeItem* items, size_t n, size_t bits, int add)
    {
        return cntkq_unquantize_batch_async(h, items, n, bits, add);
    }
    static int StripeReduceBatch(cntkq_quantizer* h, const StripeReduceItem* items, size_t n, size_t workers, size_t owner, size_t bits, int zt)
    {
        return cntkq_stripe_reduce_batch_async(h, items, n, workers, owner, bits, zt);
    }
    static int StripeReduceBatchOwners(cntkq_quantizer* h, const StripeReduceItem* items, const size_t* owners, size_t n, size_t workers,
                                       size_t bits, int zt)
    {
        return cntkq_stripe_reduce_batch_owners_async(h, items, owners, n, workers, bits, zt);
    }
};

template <>
struct Abi<double>
{
    typedef uint64_t QWord;
    static size_t QColBytes(size_t bits, size_t rows) { return cntkq_qcol_bytes_f64(bits, rows); }
    static size_t StripeReduceMaxRows(size_t bits) { return cntkq_stripe_reduce_max_rows_f64(bits); }
    static bool StripeReduceTakes(cntkq_quantizer* h, size_t rows, size_t cols, size_t bits, int zt)
    {
        return cntkq_stripe_reduce_takes_f64(h, rows, cols, bits, zt) != 0;
    }
    static int Quantize(cntkq_quantizer* h, const double* in, const double* resIn, size_t rows, size_t cols, void* q, size_t qBytes,
                        int onHost, size_t bits, double* resOut, int zt)
    {
        return cntkq_quantize_async_f64(h, in, resIn, rows, cols, q, qBytes, onHost, bits, resOut, zt);
    }
    static int Unquantize(cntkq_quantizer* h, const void* q, size_t qBytes, int onHost, double* out, size_t rows, size_t cols, size_t bits,
                          int add)
    {
        return cntkq_unquantize_async_f64(h, q, qBytes, onHost, out, rows, cols, bits, add);
    }
    static int StripeReduce(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner, size_t rows, size_t cols,
                            size_t bits, double* stripeRes, void* qOut, double* agg, int zt)
    {
        return cntkq_stripe_reduce_async_f64(h, stripes, workers, owner, rows, cols, bits, stripeRes, qOut, agg, zt);
    }
    typedef cntkq_quantize_item_f64 QuantizeItem;
    typedef cntkq_unquantize_item_f64 UnquantizeItem;
    typedef cntkq_stripe_reduce_item_f64 StripeReduceItem;
    static int QuantizeBatch(cntkq_quantizer* h, const QuantizeItem* items, size_t n, size_t bits, int zt)
    {
        return cntkq_quantize_batch_async_f64(h, items, n, bits, zt);
    }
    static int UnquantizeBatch(cntkq_quantizer* h, const UnquantizeItem* items, size_t n, size_t bits, int add)
    {
        return cntkq_unquantize_batch_async_f64(h, items, n, bits, add);
    }
    static int StripeReduceBatch(cntkq_quantizer* h, const StripeReduceItem* items, size_t n, size_t workers, size_t owner, size_t bits, int zt)
    {
        return cntkq_stripe_reduce_batch_async_f64(h, items, n, workers, owner, bits, zt);
    }
    static int StripeReduceBatchOwners(cntkq_quantizer* h, const StripeReduceItem* items, const size_t* owners, size_t n, size_t workers,
                                       size_t bits, int zt)
    {
        return cntkq_stripe_reduce_batch_owners_async_f64(h, items, owners, n, workers, bits, zt);
    }
};
} // namespace detail

// Dense column-major matrix on one GPU: element (i, j) at Data()[j * GetNumRows() + i]. Owning, or a view of columns.
template <class ElemType>
class Matrix
{
    static_assert(std::is_same<ElemType, float>::value || std::is_same<ElemType, double>::value, "float or double");

public:
    Matrix(size_t numRows, size_t numCols, int deviceId) : m_rows(numRows), m_cols(numCols), m_device(deviceId), m_owner(true)
    {
        if (deviceId < 0)
            throw std::invalid_argument("Matrix: this library keeps matrices on a GPU");
        detail::HipCheck(hipSetDevice(deviceId), "hipSetDevice");
        const size_t bytes = numRows * numCols * sizeof(ElemType);
        if (bytes != 0)
        {
            detail::HipCheck(hipMalloc(reinterpret_cast<void**>(&m_data), bytes), "hipMalloc");
            detail::HipCheck(hipMemset(m_data, 0, bytes), "hipMemset"); // matrices start as zeros, like the reference's
        }
    }
    Matrix(Matrix&& o) noexcept : m_data(o.m_data), m_rows(o.m_rows), m_cols(o.m_cols), m_device(o.m_device), m_owner(o.m_owner)
    {
        o.m_data = nullptr;
        o.m_owner = false;
    }
    Matrix(const Matrix&) = delete;
    Matrix& operator=(const Matrix&) = delete;
    ~Matrix()
    {
        if (m_owner && m_data != nullptr)
            (void) hipFree(m_data);
    }

    size_t GetNumRows() const { return m_rows; }
    size_t GetNumCols() const { return m_cols; }
    size_t GetNumElements() const { return m_rows * m_cols; }
    int GetDeviceId() const { return m_device; }
    ElemType* Data() const { return m_data; }

    // zero-copy view of columns [startColumn, startColumn + numCols) (Source/Math/Matrix.h:194)
    Matrix ColumnSlice(size_t startColumn, size_t numCols) const
    {
        if (startColumn + numCols > m_cols)
            throw std::logic_error("ColumnSlice: out of range");
        return Matrix(m_data + startColumn * m_rows, m_rows, numCols, m_device);
    }

    // exchange of contents (std::swap of two matrices in the reference's double-buffered aggregation)
    void Swap(Matrix& o) noexcept
    {
        std::swap(m_data, o.m_data);
        std::swap(m_rows, o.m_rows);
        std::swap(m_cols, o.m_cols);
        std::swap(m_device, o.m_device);
        std::swap(m_owner, o.m_owner);
    }

    void SetValue(ElemType v)
    {
        std::vector<ElemType> host(GetNumElements(), v);
        SetValue(host.data());
    }
    void SetValue(const ElemType* hostColumnMajor)
    {
        if (GetNumElements() != 0)
            detail::HipCheck(hipMemcpy(m_data, hostColumnMajor, GetNumElements() * sizeof(ElemType), hipMemcpyHostToDevice), "hipMemcpy");
    }
    // Matrix::Print of an inclusive range (Source/Math/CPUMatrixImpl.h:4097-4149, the form the aggregator's debug peeks
    // use: a corner that starts at the first row and column): name and shape, the range where it is not the whole matrix,
    // then the values row by row with "..." where rows or columns are left out. Reads the range back from the device.
    void Print(const char* matrixName, size_t rowFirst, size_t rowLast, size_t colFirst, size_t colLast, FILE* out = stderr) const
    {
        std::fprintf(out, "\n###### ");
        if (matrixName != nullptr)
            std::fprintf(out, "%s ", matrixName);
        std::fprintf(out, "(%lu, %lu)", (unsigned long) m_rows, (unsigned long) m_cols);
        if (rowFirst != 0 || colFirst != 0 || rowLast + 1 != m_rows || colLast + 1 != m_cols)
            std::fprintf(out, " [%ld:%ld, %ld:%ld]", (long) rowFirst, (long) rowLast, (long) colFirst, (long) colLast);
        std::fprintf(out, " ######\n\n");
        if (GetNumElements() == 0 || rowFirst > rowLast || colFirst > colLast || rowLast >= m_rows || colLast >= m_cols)
        {
            std::fprintf(out, "(empty)\n");
            return;
        }
        const size_t nr = rowLast - rowFirst + 1, nc = colLast - colFirst + 1;
        std::vector<ElemType> host(nr * nc);
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        for (size_t j = 0; j < nc; ++j)
            detail::HipCheck(hipMemcpy(host.data() + j * nr, m_data + (colFirst + j) * m_rows + rowFirst, nr * sizeof(ElemType), hipMemcpyDeviceToHost),
                             "hipMemcpy");
        if (rowFirst > 0)
            std::fprintf(out, "...\n");
        for (size_t i = 0; i < nr; ++i)
        {
            if (colFirst > 0)
                std::fprintf(out, "...\t");
            for (size_t j = 0; j < nc; ++j)
                std::fprintf(out, "%.10f\t", (double) host[j * nr + i]);
            if (colLast + 1 < m_cols)
                std::fprintf(out, "...");
            std::fprintf(out, "\n");
        }
        if (rowLast + 1 < m_rows)
            std::fprintf(out, "...\n");
    }

    // host copy in column-major order (Matrix::CopyToArray)
    std::unique_ptr<ElemType[]> CopyToArray() const
    {
        std::unique_ptr<ElemType[]> host(new ElemType[GetNumElements() ? GetNumElements() : 1]);
        if (GetNumElements() != 0)
            detail::HipCheck(hipMemcpy(host.get(), m_data, GetNumElements() * sizeof(ElemType), hipMemcpyDeviceToHost), "hipMemcpy");
        return host;
    }

private:
    Matrix(ElemType* data, size_t rows, size_t cols, int device) : m_data(data), m_rows(rows), m_cols(cols), m_device(device), m_owner(false) {}

    ElemType* m_data = nullptr;
    size_t m_rows, m_cols;
    int m_device;
    bool m_owner;
};

// One packed column: { lower; upper; bits[nq] } (Source/Math/QuantizedMatrix.h:27-48)
template <class ElemType>
struct QuantizedColumn
{
    typedef typename detail::Abi<ElemType>::QWord QWord;
    static const size_t QWordNumBits = 8 * sizeof(QWord);
    ElemType lower;
    ElemType upper;
    QWord bits[1];

    static size_t QuantizedColumnSize(size_t bits, size_t rows) { return detail::Abi<ElemType>::QColBytes(bits, rows); }
};

// Packed matrix; on a GPU (deviceId >= 0) or in pinned host memory (CPUDEVICE), which is how the reference's v1
// aggregator keeps it (Source/1BitSGD/AllReduceDistGradAggregator.h:76-77, 88). Move-only; ColumnSlice is a view.
template <class ElemType>
class QuantizedMatrix
{
    static_assert(std::is_same<ElemType, float>::value || std::is_same<ElemType, double>::value, "float or double");

public:
    QuantizedMatrix(size_t numRows, size_t numCols, size_t nbits, int deviceId)
        : m_rows(numRows), m_cols(numCols), m_bits(nbits), m_device(deviceId), m_owner(true)
    {
        m_qColSize = detail::Abi<ElemType>::QColBytes(nbits, numRows);
        if (m_qColSize == 0) // Source/Math/QuantizedMatrix.cpp:12-15
            throw std::logic_error("Quantization: 'nbits' must be a power of two that divides the QWord width");
        const size_t bytes = m_qColSize * numCols;
        if (bytes == 0)
            return;
        if (deviceId >= 0)
        {
            detail::HipCheck(hipSetDevice(deviceId), "hipSetDevice");
            detail::HipCheck(hipMalloc(reinterpret_cast<void**>(&m_buffer), bytes), "hipMalloc");
            detail::HipCheck(hipMemset(m_buffer, 0, bytes), "hipMemset");
        }
        else
        {
            detail::HipCheck(hipHostMalloc(reinterpret_cast<void**>(&m_buffer), bytes, hipHostMallocDefault), "hipHostMalloc");
            std::memset(m_buffer, 0, bytes);
        }
    }
    QuantizedMatrix(QuantizedMatrix&& o) noexcept
        : m_buffer(o.m_buffer), m_rows(o.m_rows), m_cols(o.m_cols), m_bits(o.m_bits), m_qColSize(o.m_qColSize), m_device(o.m_device), m_owner(o.m_owner)
    {
        o.m_buffer = nullptr;
        o.m_owner = false;
    }
    QuantizedMatrix(const QuantizedMatrix&) = delete;
    QuantizedMatrix& operator=(const QuantizedMatrix&) = delete;
    ~QuantizedMatrix()
    {
        if (m_owner && m_buffer != nullptr)
        {
            if (m_device >= 0)
                (void) hipFree(m_buffer);
            else
                (void) hipHostFree(m_buffer);
        }
    }

    int GetDeviceId() const { return m_device; }
    size_t GetNumRows() const { return m_rows; }
    size_t GetNumCols() const { return m_cols; }
    size_t GetNumBits() const { return m_bits; }
    size_t GetSize() const { return m_qColSize * m_cols; }
    char* Buffer() const { return m_buffer; }

    // valid to dereference only for a host-resident matrix
    QuantizedColumn<ElemType>* GetQuantizedColumn(size_t colIdx)
    {
        return reinterpret_cast<QuantizedColumn<ElemType>*>(m_buffer + m_qColSize * colIdx);
    }

    QuantizedMatrix ColumnSlice(size_t startColumn, size_t numCols) const
    {
        if (startColumn + numCols > m_cols)
            throw std::logic_error("ColumnSlice: out of range");
        return QuantizedMatrix(m_buffer + startColumn * m_qColSize, m_rows, numCols, m_bits, m_qColSize, m_device);
    }

    // host copy of the packed bytes, wherever they live
    std::vector<char> CopyToHost() const
    {
        std::vector<char> host(GetSize());
        if (!host.empty())
        {
            if (m_device >= 0)
                detail::HipCheck(hipMemcpy(host.data(), m_buffer, host.size(), hipMemcpyDeviceToHost), "hipMemcpy");
            else
                std::memcpy(host.data(), m_buffer, host.size());
        }
        return host;
    }

    // QuantizedMatrix::Print (Source/Math/QuantizedMatrix.cpp:109-171): the column bounds, then code and reconstructed
    // value of every element of the inclusive range, to stderr (or `out`). Reads a host copy; element i of a column is in
    // QWord i % nq at bit (i / nq) * nbits; value = (code + 0.5) * ufactor + lower (Source/Math/ValueQuantizer.h:68-97, 131-141).
    void Print(const char* matrixName, size_t rowStart, size_t rowEnd, size_t colStart, size_t colEnd, FILE* out = stderr) const
    {
        typedef typename detail::Abi<ElemType>::QWord QWord;
        if (rowStart > rowEnd || rowEnd >= m_rows || colStart > colEnd || colEnd >= m_cols)
            throw std::invalid_argument("Index out of range.");
        const std::vector<char> host = CopyToHost();
        const size_t wordBits = 8 * sizeof(QWord);
        const size_t nq = (m_qColSize - 2 * sizeof(ElemType)) / sizeof(QWord);
        if (matrixName != nullptr)
            std::fprintf(out, "\n###### %s (%lu, %lu) ######\n", matrixName, (unsigned long) m_rows, (unsigned long) m_cols);
        else
            std::fprintf(out, "\n###### Unnamed Matrix (%lu, %lu) ######\n", (unsigned long) m_rows, (unsigned long) m_cols);
        std::fprintf(out, "\n------ Print Range (%lu:%lu, %lu:%lu) ------\n", (unsigned long) rowStart, (unsigned long) rowEnd,
                     (unsigned long) colStart, (unsigned long) colEnd);
        auto header = [&](size_t j, int which) {
            ElemType v;
            std::memcpy(&v, host.data() + j * m_qColSize + which * sizeof(ElemType), sizeof v);
            return v;
        };
        for (size_t j = colStart; j <= colEnd; ++j)
            std::fprintf(out, "Lower=%.10f,Upper=%.10f\t", (double) header(j, 0), (double) header(j, 1));
        std::fprintf(out, "\n");
        for (size_t i = rowStart; i <= rowEnd; ++i)
        {
            for (size_t j = colStart; j <= colEnd; ++j)
            {
                const ElemType lower = header(j, 0), upper = header(j, 1);
                QWord word;
                std::memcpy(&word, host.data() + j * m_qColSize + 2 * sizeof(ElemType) + (i % nq) * sizeof(QWord), sizeof word);
                QWord code;
                ElemType value;
                if (m_bits == wordBits)
                {
                    code = word; // pass-through: the code is the value's bit pattern
                    std::memcpy(&value, &word, sizeof value);
                }
                else
                {
                    code = (word >> ((i / nq) * m_bits)) & ((QWord(1) << m_bits) - 1);
                    const ElemType spread = upper - lower;
                    const ElemType used = (ElemType) ((QWord(1) << m_bits) - (m_bits > 1 ? 1 : 0));
                    const ElemType ufactor = spread >= (ElemType) 1e-36f ? spread / used : (ElemType) 0;
                    value = ((ElemType) code + (ElemType) 0.5) * ufactor + lower;
                }
                std::fprintf(out, "%10d (%.10f)          \t", (int) code, (double) value);
            }
            std::fprintf(out, "\n");
        }
    }

private:
    QuantizedMatrix(char* buffer, size_t rows, size_t cols, size_t bits, size_t qColSize, int device)
        : m_buffer(buffer), m_rows(rows), m_cols(cols), m_bits(bits), m_qColSize(qColSize), m_device(device), m_owner(false)
    {
    }

    char* m_buffer = nullptr;
    size_t m_rows, m_cols, m_bits;
    size_t m_qColSize = 0;
    int m_device;
    bool m_owner;
};

// The quantizer boundary (Source/Math/MatrixQuantizerImpl.h:19-49)
template <class ElemType>
class MatrixQuantizerImpl
{
    static_assert(std::is_same<ElemType, float>::value || std::is_same<ElemType, double>::value, "float or double");

public:
    // deviceId >= 0: the GPU quantizer, useAsync = dedicated compute stream (Source/Math/MatrixQuantizerImpl.cpp:10-26)
    static MatrixQuantizerImpl<ElemType>* Create(int deviceId, bool useAsync);
    virtual ~MatrixQuantizerImpl() {}
    MatrixQuantizerImpl(const MatrixQuantizerImpl&) = delete;
    MatrixQuantizerImpl& operator=(const MatrixQuantizerImpl&) = delete;

    virtual void QuantizeAsync(const Matrix<ElemType>& inMatrix, const Matrix<ElemType>& inResidual, QuantizedMatrix<ElemType>& outQMatrix,
                               Matrix<ElemType>& outResidual, bool zeroThresholdFor1Bit) = 0;
    virtual void WaitQuantizeAsyncDone() = 0;
    virtual void UnquantizeAsync(QuantizedMatrix<ElemType>& inQMatrix, Matrix<ElemType>& outMatrix, bool add = false) = 0;
    virtual void WaitUnquantizeAsyncDone() = 0;

    int GetDeviceId() const { return m_deviceId; }

protected:
    explicit MatrixQuantizerImpl(int deviceId) : m_deviceId(deviceId) {}

private:
    int m_deviceId;
};

// Replaces MatrixQuantizerGPU (Source/Math/MatrixQuantizerGPU.h:17-95)
template <class ElemType>
class MatrixQuantizerGPU final : public MatrixQuantizerImpl<ElemType>
{
public:
    // forceSync: every call waits for its own work (Source/Math/MatrixQuantizerGPU.h:20), for time measurements
    MatrixQuantizerGPU(int deviceId, bool useDedicatedComputeStream, bool forceSync = false) : MatrixQuantizerImpl<ElemType>(deviceId)
    {
        detail::Check(cntkq_create(deviceId, useDedicatedComputeStream ? 1 : 0, &m_handle));
        if (forceSync)
            detail::Check(cntkq_set_force_sync(m_handle, 1));
    }
    ~MatrixQuantizerGPU() override { (void) cntkq_destroy(m_handle); }

    // No counterpart in the reference: columns taller than one workgroup holds as several launches whose workgroups never wait
    // for one another, instead of one launch whose workgroups do (for quantizers whose stream shares the device with other work).
    void SetTallColumnsNeverWait(bool neverWait) { detail::Check(cntkq_set_tall_columns_never_wait(m_handle, neverWait ? 1 : 0)); }

    void QuantizeAsync(const Matrix<ElemType>& inMatrix, const Matrix<ElemType>& inResidual, QuantizedMatrix<ElemType>& outQMatrix,
                       Matrix<ElemType>& outResidual, bool zeroThresholdFor1Bit) override
    {
        const size_t rows = inMatrix.GetNumRows(), cols = inMatrix.GetNumCols();
        // asserts in the reference (Source/Math/MatrixQuantizerGPU.cu:229-232)
        if (outQMatrix.GetNumRows() != rows || outQMatrix.GetNumCols() != cols || inResidual.GetNumRows() != rows ||
            inResidual.GetNumCols() != cols || outResidual.GetNumRows() != rows || outResidual.GetNumCols() != cols)
            throw std::invalid_argument("QuantizeAsync: matrix dimensions do not match");
        detail::Check(detail::Abi<ElemType>::Quantize(m_handle, inMatrix.Data(), inResidual.Data(), rows, cols, outQMatrix.Buffer(),
                                                      outQMatrix.GetSize(), outQMatrix.GetDeviceId() == CPUDEVICE, outQMatrix.GetNumBits(),
                                                      outResidual.Data(), zeroThresholdFor1Bit ? 1 : 0));
    }
    void WaitQuantizeAsyncDone() override { detail::Check(cntkq_wait_quantize_done(m_handle)); }

    void UnquantizeAsync(QuantizedMatrix<ElemType>& inQMatrix, Matrix<ElemType>& outMatrix, bool add = false) override
    {
        if (inQMatrix.GetNumRows() != outMatrix.GetNumRows() || inQMatrix.GetNumCols() != outMatrix.GetNumCols())
            throw std::invalid_argument("UnquantizeAsync: matrix dimensions do not match");
        detail::Check(detail::Abi<ElemType>::Unquantize(m_handle, inQMatrix.Buffer(), inQMatrix.GetSize(), inQMatrix.GetDeviceId() == CPUDEVICE,
                                                        outMatrix.Data(), outMatrix.GetNumRows(), outMatrix.GetNumCols(), inQMatrix.GetNumBits(),
                                                        add ? 1 : 0));
    }
    void WaitUnquantizeAsyncDone() override { detail::Check(cntkq_wait_unquantize_done(m_handle)); }

    // A whole gradient set per call: the aggregator's loops over its matrices
    // (Source/1BitSGD/AllReduceDistGradAggregator.h:288-300 and :517-522) as one launch each.
    struct QuantizeItem
    {
        const Matrix<ElemType>* inMatrix;
        const Matrix<ElemType>* inResidual;
        QuantizedMatrix<ElemType>* outQMatrix;
        Matrix<ElemType>* outResidual;
    };
    void QuantizeBatchAsync(const std::vector<QuantizeItem>& items, bool zeroThresholdFor1Bit)
    {
        if (items.empty())
            return;
        const size_t nbits = items[0].outQMatrix->GetNumBits();
        std::vector<typename detail::Abi<ElemType>::QuantizeItem> raw;
        for (const auto& it : items)
        {
            const size_t rows = it.inMatrix->GetNumRows(), cols = it.inMatrix->GetNumCols();
            if (it.outQMatrix->GetNumRows() != rows || it.outQMatrix->GetNumCols() != cols || it.inResidual->GetNumRows() != rows ||
                it.inResidual->GetNumCols() != cols || it.outResidual->GetNumRows() != rows || it.outResidual->GetNumCols() != cols)
                throw std::invalid_argument("QuantizeBatchAsync: matrix dimensions do not match");
            if (it.outQMatrix->GetNumBits() != nbits || it.outQMatrix->GetDeviceId() < 0)
                throw std::invalid_argument("QuantizeBatchAsync: packed matrices must share one bit width and live on the device");
            raw.push_back(typename detail::Abi<ElemType>::QuantizeItem{it.inMatrix->Data(), it.inResidual->Data(), it.outResidual->Data(), it.outQMatrix->Buffer(), rows, cols, it.outQMatrix->GetSize()});
        }
        detail::Check(detail::Abi<ElemType>::QuantizeBatch(m_handle, raw.data(), raw.size(), nbits, zeroThresholdFor1Bit ? 1 : 0));
    }
    struct UnquantizeItem
    {
        const QuantizedMatrix<ElemType>* inQMatrix;
        Matrix<ElemType>* outMatrix;
    };
    void UnquantizeBatchAsync(const std::vector<UnquantizeItem>& items, bool add = false)
    {
        if (items.empty())
            return;
        const size_t nbits = items[0].inQMatrix->GetNumBits();
        std::vector<typename detail::Abi<ElemType>::UnquantizeItem> raw;
        for (const auto& it : items)
        {
            if (it.inQMatrix->GetNumRows() != it.outMatrix->GetNumRows() || it.inQMatrix->GetNumCols() != it.outMatrix->GetNumCols())
                throw std::invalid_argument("UnquantizeBatchAsync: matrix dimensions do not match");
            if (it.inQMatrix->GetNumBits() != nbits || it.inQMatrix->GetDeviceId() < 0)
                throw std::invalid_argument("UnquantizeBatchAsync: packed matrices must share one bit width and live on the device");
            raw.push_back(typename detail::Abi<ElemType>::UnquantizeItem{it.inQMatrix->Buffer(), it.outMatrix->Data(), it.outMatrix->GetNumRows(), it.outMatrix->GetNumCols(), it.inQMatrix->GetSize()});
        }
        detail::Check(detail::Abi<ElemType>::UnquantizeBatch(m_handle, raw.data(), raw.size(), nbits, add ? 1 : 0));
    }

    // Whether StripeReduceAsync takes stripes of this shape on this quantizer; where not, the caller keeps the reference's
    // sequence of UnquantizeAsync ... QuantizeAsync calls (Source/1BitSGD/AllReduceDistGradAggregator.h:365-436).
    bool StripeReduceTakes(size_t numRows, size_t numStripeCols, size_t nbits, bool zeroThresholdFor1Bit) const
    {
        return detail::Abi<ElemType>::StripeReduceTakes(m_handle, numRows, numStripeCols, nbits, zeroThresholdFor1Bit ? 1 : 0);
    }

    // Fused stripe reduction of the quantized all-reduce (dataflow of Source/1BitSGD/AllReduceDistGradAggregator.h:365-436):
    // stripes[w] is worker w's packed stripe; the requantized aggregate goes to outQStripe (may be stripes[owner]).
    void StripeReduceAsync(const std::vector<const QuantizedMatrix<ElemType>*>& stripes, size_t owner, Matrix<ElemType>& stripeResidual,
                           QuantizedMatrix<ElemType>& outQStripe, bool zeroThresholdFor1Bit, Matrix<ElemType>* aggregate = nullptr)
    {
        std::vector<const void*> ptrs;
        for (const auto* s : stripes)
        {
            if (s->GetNumRows() != outQStripe.GetNumRows() || s->GetNumCols() != outQStripe.GetNumCols() || s->GetNumBits() != outQStripe.GetNumBits() ||
                s->GetDeviceId() < 0)
                throw std::invalid_argument("StripeReduceAsync: stripes must be device-resident and of equal shape");
            ptrs.push_back(s->Buffer());
        }
        detail::Check(detail::Abi<ElemType>::StripeReduce(m_handle, ptrs.data(), ptrs.size(), owner, outQStripe.GetNumRows(),
                                                          outQStripe.GetNumCols(), outQStripe.GetNumBits(), stripeResidual.Data(),
                                                          outQStripe.Buffer(), aggregate ? aggregate->Data() : nullptr,
                                                          zeroThresholdFor1Bit ? 1 : 0));
    }
    // The owner's stripe reductions of a whole gradient set as one call (one item per gradient matrix).
    struct StripeReduceItem
    {
        std::vector<const QuantizedMatrix<ElemType>*> stripes;
        Matrix<ElemType>* stripeResidual;
        QuantizedMatrix<ElemType>* outQStripe;
        Matrix<ElemType>* aggregate; // may be null
    };
    void StripeReduceBatchAsync(const std::vector<StripeReduceItem>& items, size_t owner, bool zeroThresholdFor1Bit)
    {
        StripeReduceBatchAsync(items, owner, nullptr, zeroThresholdFor1Bit);
    }
    // owners[i]: the rank whose stripe item i is (all ranks of a cluster simulated on one GPU in one call)
    void StripeReduceBatchAsync(const std::vector<StripeReduceItem>& items, const std::vector<size_t>& owners, bool zeroThresholdFor1Bit)
    {
        if (owners.size() != items.size())
            throw std::invalid_argument("StripeReduceBatchAsync: one owner per item");
        StripeReduceBatchAsync(items, 0, owners.data(), zeroThresholdFor1Bit);
    }
    void StripeReduceBatchAsync(const std::vector<StripeReduceItem>& items, size_t owner, const size_t* owners, bool zeroThresholdFor1Bit)
    {
        if (items.empty())
            return;
        const size_t workers = items[0].stripes.size();
        const size_t nbits = items[0].outQStripe->GetNumBits();
        std::vector<std::vector<const void*>> ptrs(items.size());
        std::vector<typename detail::Abi<ElemType>::StripeReduceItem> raw;
        for (size_t i = 0; i < items.size(); ++i)
        {
            const auto& it = items[i];
            if (it.stripes.size() != workers || it.outQStripe->GetNumBits() != nbits)
                throw std::invalid_argument("StripeReduceBatchAsync: items must share the worker count and the bit width");
            for (const auto* s : it.stripes)
            {
                if (s->GetNumRows() != it.outQStripe->GetNumRows() || s->GetNumCols() != it.outQStripe->GetNumCols() ||
                    s->GetNumBits() != nbits || s->GetDeviceId() < 0)
                    throw std::invalid_argument("StripeReduceBatchAsync: stripes must be device-resident and of equal shape");
                ptrs[i].push_back(s->Buffer());
            }
            raw.push_back(typename detail::Abi<ElemType>::StripeReduceItem{ptrs[i].data(), it.stripeResidual->Data(), it.outQStripe->Buffer(),
                                                   it.aggregate ? it.aggregate->Data() : nullptr, it.outQStripe->GetNumRows(),
                                                   it.outQStripe->GetNumCols()});
        }
        if (owners != nullptr)
            detail::Check(detail::Abi<ElemType>::StripeReduceBatchOwners(m_handle, raw.data(), owners, raw.size(), workers, nbits,
                                                                         zeroThresholdFor1Bit ? 1 : 0));
        else
            detail::Check(detail::Abi<ElemType>::StripeReduceBatch(m_handle, raw.data(), raw.size(), workers, owner, nbits, zeroThresholdFor1Bit ? 1 : 0));
    }
    void WaitStripeReduceDone() { detail::Check(cntkq_wait_stripe_reduce_done(m_handle)); }

    cntkq_quantizer* Handle() const { return m_handle; }

private:
    cntkq_quantizer* m_handle = nullptr;
};

template <class ElemType>
MatrixQuantizerImpl<ElemType>* MatrixQuantizerImpl<ElemType>::Create(int deviceId, bool useAsync)
{
    if (deviceId >= 0)
        return new MatrixQuantizerGPU<ElemType>(deviceId, useAsync);
    // the reference returns its CPU quantizer here; a build without one throws, as CPUONLY builds do for GPUs
    throw std::runtime_error("CreateMatrixQuantizer: this library has no CPU quantizer");
}

// Orders the quantizer's stream after everything already issued on the main stream
// (Source/Math/MatrixQuantizerImpl.h:53-72, Source/Math/MatrixQuantizerGPU.cu:347-371)
class MatrixComputeStreamEvent
{
public:
    static MatrixComputeStreamEvent* Create(int deviceId) { return new MatrixComputeStreamEvent(deviceId); }
    virtual ~MatrixComputeStreamEvent() {}
    virtual void SynchronizeEvent() { detail::HipCheck(hipStreamSynchronize(nullptr), "hipStreamSynchronize"); }

    template <typename ElemType>
    void SynchronizeQuantizationComputeStreamWithEvent(MatrixQuantizerImpl<ElemType>& quantizer)
    {
        auto* gpu = dynamic_cast<MatrixQuantizerGPU<ElemType>*>(&quantizer);
        if (gpu != nullptr)
            detail::Check(cntkq_sync_with_main_stream(gpu->Handle()));
    }

protected:
    explicit MatrixComputeStreamEvent(int deviceId) : m_deviceId(deviceId) {}
    int m_deviceId;
};

// Quantizer that owns the error-feedback residual (Source/1BitSGD/MatrixQuantizer.h:24-85)
class MatrixQuantizerBase
{
};

template <class ElemType>
class MatrixQuantizer final : public MatrixQuantizerBase
{
public:
    MatrixQuantizer(size_t numRows, size_t numCols, int deviceId, bool useAsync) : MatrixQuantizer(deviceId, useAsync)
    {
        m_residual = std::make_shared<Matrix<ElemType>>(numRows, numCols, deviceId);
    }
    MatrixQuantizer(int deviceId, bool useAsync) : m_residual(nullptr)
    {
        m_quantizerImpl.reset(MatrixQuantizerImpl<ElemType>::Create(deviceId, useAsync));
    }
    MatrixQuantizer(const MatrixQuantizer&) = delete;
    MatrixQuantizer& operator=(const MatrixQuantizer&) = delete;

    void QuantizeAsync(const Matrix<ElemType>& inMatrix, QuantizedMatrix<ElemType>& outQMatrix, bool zeroThresholdFor1Bit)
    {
        m_quantizerImpl->QuantizeAsync(inMatrix, *m_residual, outQMatrix, *m_residual, zeroThresholdFor1Bit);
    }
    void QuantizeAsync(const Matrix<ElemType>& inMatrix, const Matrix<ElemType>& inResidual, QuantizedMatrix<ElemType>& outQMatrix,
                       Matrix<ElemType>& outResidual, bool zeroThresholdFor1Bit)
    {
        m_quantizerImpl->QuantizeAsync(inMatrix, inResidual, outQMatrix, outResidual, zeroThresholdFor1Bit);
    }
    void WaitQuantizeAsyncDone() { m_quantizerImpl->WaitQuantizeAsyncDone(); }
    void UnquantizeAsync(QuantizedMatrix<ElemType>& inQMatrix, Matrix<ElemType>& outMatrix, bool add = false)
    {
        m_quantizerImpl->UnquantizeAsync(inQMatrix, outMatrix, add);
    }
    void WaitUnquantizeAsyncDone() { m_quantizerImpl->WaitUnquantizeAsyncDone(); }
    int GetDeviceId() const { return m_quantizerImpl->GetDeviceId(); }
    void ResetResidue() { m_residual->SetValue((ElemType) 0); }
    const Matrix<ElemType>& GetResidualMatrix() const { return *m_residual; }
    MatrixQuantizerImpl<ElemType>& Impl() { return *m_quantizerImpl; }

private:
    std::unique_ptr<MatrixQuantizerImpl<ElemType>> m_quantizerImpl;
    std::shared_ptr<Matrix<ElemType>> m_residual;
};

} // namespace cntk_amd
