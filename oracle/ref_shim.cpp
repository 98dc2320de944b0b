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
struct PackedColumn // same bytes as QuantizedColumn<float> (Source/Math/QuantizedMatrix.h:27-48)
{
    float lower;
    float upper;
    unsigned int bits[1];
};

size_t ColumnBytes(size_t nbits, size_t rows)
{
    return 2 * sizeof(float) + ((rows * nbits + 31) / 32) * sizeof(unsigned int);
}
} // namespace

extern "C" {

size_t ref_qwords_per_col(size_t rows, size_t nbits)
{
    return ColumnQuantizer<float>::QWordsPerCol(rows, nbits);
}

int ref_quantize(const float* g, const float* r_in, size_t rows, size_t cols, void* qbuf, size_t nbits,
                 float* r_out, int zero_threshold)
{
    try
    {
        const size_t ld = ValueQuantizer<float>::ld(nbits);
        const size_t stride = ColumnBytes(nbits, rows);
        for (size_t j = 0; j < cols; j++)
        {
            PackedColumn& col = *reinterpret_cast<PackedColumn*>(static_cast<char*>(qbuf) + j * stride);
            if (zero_threshold)
                ColumnQuantizer<float>::ComputeRangeStatColj<true>(g, r_in, (long) rows, j, nbits, col.lower, col.upper);
            else
                ColumnQuantizer<float>::ComputeRangeStatColj<false>(g, r_in, (long) rows, j, nbits, col.lower, col.upper);
            ColumnQuantizer<float> cq(ld, col.lower, col.upper);
            if (zero_threshold)
                cq.Quantize<true>(g, r_in, (long) rows, j, col.bits, r_out);
            else
                cq.Quantize<false>(g, r_in, (long) rows, j, col.bits, r_out);
        }
        return 0;
    }
    catch (...)
    {
        return -1;
    }
}

int ref_unquantize(const void* qbuf, size_t rows, size_t cols, size_t nbits, float* out, int add)
{
    try
    {
        const size_t ld = ValueQuantizer<float>::ld(nbits);
        const size_t stride = ColumnBytes(nbits, rows);
        for (size_t j = 0; j < cols; j++)
        {
            const PackedColumn& col = *reinterpret_cast<const PackedColumn*>(static_cast<const char*>(qbuf) + j * stride);
            ColumnQuantizer<float> cq(ld, col.lower, col.upper);
            cq.Unquantize(out, (long) rows, j, col.bits, add != 0);
        }
        return 0;
    }
    catch (...)
    {
        return -1;
    }
}

} // extern "C"
