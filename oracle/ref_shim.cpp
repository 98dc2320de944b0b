// Thin C-ABI wrapper around the reference's OWN quantizer headers -- TEST INFRASTRUCTURE ONLY.
//
// Nothing of the reference is copied here: this file is compiled together with
// /root/reference/Source/Math/{ColumnQuantizer,ValueQuantizer}.h where they lie, and the result
// goes to oracle/_ref/ (git-ignored). It exists to prove the plain-C oracle bit-identical to the
// reference arithmetic and to write the golden vectors under tests/golden/.
//
// The per-matrix driver below is the two-calls-per-column loop of
// Source/Math/MatrixQuantizerCPU.cpp:28-59 and :87-96 (that file itself needs the full Matrix
// library, BLAS and Boost, so it cannot be built here; it adds no arithmetic of its own).
#include "ColumnQuantizer.h"

#include <cstddef>
#include <cstdint>

using Microsoft::MSR::CNTK::ColumnQuantizer;
using Microsoft::MSR::CNTK::ValueQuantizer;

namespace {
// same bytes as QuantizedColumn<ElemType> (Source/Math/QuantizedMatrix.h:27-48)
template <class E>
struct PackedColumn
{
    typedef typename ValueQuantizer<E>::QWord QWord;
    E lower;
    E upper;
    QWord bits[1];
};

template <class E>
size_t ColumnBytes(size_t nbits, size_t rows)
{
    typedef typename ValueQuantizer<E>::QWord QWord;
    const size_t wordBits = 8 * sizeof(QWord);
    return 2 * sizeof(E) + ((rows * nbits + wordBits - 1) / wordBits) * sizeof(QWord);
}

template <class E>
int Quantize(const E* g, const E* r_in, size_t rows, size_t cols, void* qbuf, size_t nbits, E* r_out, int zero_threshold)
{
    try
    {
        const size_t ld = ValueQuantizer<E>::ld(nbits);
        const size_t stride = ColumnBytes<E>(nbits, rows);
        for (size_t j = 0; j < cols; j++)
        {
            PackedColumn<E>& col = *reinterpret_cast<PackedColumn<E>*>(static_cast<char*>(qbuf) + j * stride);
            if (zero_threshold)
                ColumnQuantizer<E>::template ComputeRangeStatColj<true>(g, r_in, (long) rows, j, nbits, col.lower, col.upper);
            else
                ColumnQuantizer<E>::template ComputeRangeStatColj<false>(g, r_in, (long) rows, j, nbits, col.lower, col.upper);
            ColumnQuantizer<E> cq(ld, col.lower, col.upper);
            if (zero_threshold)
                cq.template Quantize<true>(g, r_in, (long) rows, j, col.bits, r_out);
            else
                cq.template Quantize<false>(g, r_in, (long) rows, j, col.bits, r_out);
        }
        return 0;
    }
    catch (...)
    {
        return -1;
    }
}

template <class E>
int Unquantize(const void* qbuf, size_t rows, size_t cols, size_t nbits, E* out, int add)
{
    try
    {
        const size_t ld = ValueQuantizer<E>::ld(nbits);
        const size_t stride = ColumnBytes<E>(nbits, rows);
        for (size_t j = 0; j < cols; j++)
        {
            const PackedColumn<E>& col =
                *reinterpret_cast<const PackedColumn<E>*>(static_cast<const char*>(qbuf) + j * stride);
            ColumnQuantizer<E> cq(ld, col.lower, col.upper);
            cq.Unquantize(out, (long) rows, j, col.bits, add != 0);
        }
        return 0;
    }
    catch (...)
    {
        return -1;
    }
}
} // namespace

extern "C" {

size_t ref_qwords_per_col(size_t rows, size_t nbits)
{
    return ColumnQuantizer<float>::QWordsPerCol(rows, nbits);
}

size_t ref_qwords_per_col_f64(size_t rows, size_t nbits)
{
    return ColumnQuantizer<double>::QWordsPerCol(rows, nbits);
}

int ref_quantize(const float* g, const float* r_in, size_t rows, size_t cols, void* qbuf, size_t nbits,
                 float* r_out, int zero_threshold)
{
    return Quantize<float>(g, r_in, rows, cols, qbuf, nbits, r_out, zero_threshold);
}

int ref_quantize_f64(const double* g, const double* r_in, size_t rows, size_t cols, void* qbuf, size_t nbits,
                     double* r_out, int zero_threshold)
{
    return Quantize<double>(g, r_in, rows, cols, qbuf, nbits, r_out, zero_threshold);
}

int ref_unquantize(const void* qbuf, size_t rows, size_t cols, size_t nbits, float* out, int add)
{
    return Unquantize<float>(qbuf, rows, cols, nbits, out, add);
}

int ref_unquantize_f64(const void* qbuf, size_t rows, size_t cols, size_t nbits, double* out, int add)
{
    return Unquantize<double>(qbuf, rows, cols, nbits, out, add);
}

} // extern "C"
