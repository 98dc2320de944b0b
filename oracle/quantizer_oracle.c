/*
 * CPU oracle for the per-column gradient quantizer -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the reference CPU quantizer's arithmetic. Used by the tests as the
 * checker for the HIP kernels and by the benchmark as the timed CPU baseline. The shipped
 * library never links, loads or calls anything in this file.
 *
 * What pins each function (so that a dropped term, wrong sign or transposed index fails):
 * The arithmetic is in quantizer_oracle_body.inc, compiled here once per element type.
 *
 *   - every function: bit-exact agreement with the reference's own headers, compiled from
 *     /root/reference into oracle/_ref, on the committed golden vectors (all six bit widths,
 *     both 1-bit threshold modes, carried residuals, the reference unit test's ten shapes);
 *   - value quantizer: closed forms (1-bit levels are newmean -/+ radius/2; the top code of a
 *     multi-bit column reconstructs to upper + ufactor/2; 32 bits is the identity);
 *   - statistics: a hand-computed column and an independent restatement following the
 *     reference unit test's inline checker;
 *   - packing: brute-force element -> (word, shift) mapping on tiny matrices and the
 *     conservation law  g + r_in == unquantize(q) + r_out;
 *   - stripe reduction: with 32 bits it must equal the plain fp32 sum in the stated order.
 * Parity unpinned: only the ORDER of the fp32 additions in the stripe reduction, which the
 * reference leaves to message arrival; this file fixes "owner first, then ascending rank".
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp (never -ffast-math): the reference CPU build has
 * no fused multiply-add and every operation is rounded to fp32 separately.
 */
#include "quantizer_oracle.h"

#include <math.h>
#include <string.h>

#define ORACLE_PASTE2(a, b) a##b
#define ORACLE_PASTE(a, b) ORACLE_PASTE2(a, b)

/* ---- MatrixQuantizerImpl<float>: QWord = 32 bits ---- */
#define ELEM float
#define QWORD uint32_t
#define SQWORD int32_t
#define QWORD_BITS 32u
#define ELEM_SQRT sqrtf
#define FN(name) oracle_##name
#define LOCAL(name) name##_f32
#define ORACLE_DEFINE_SHARED
#include "quantizer_oracle_body.inc"
#undef ORACLE_DEFINE_SHARED
#undef ELEM
#undef QWORD
#undef SQWORD
#undef QWORD_BITS
#undef ELEM_SQRT
#undef FN
#undef LOCAL

/* ---- MatrixQuantizerImpl<double>: QWord = 64 bits ---- */
#define ELEM double
#define QWORD uint64_t
#define SQWORD int64_t
#define QWORD_BITS 64u
#define ELEM_SQRT sqrt
#define FN(name) oracle_##name##_f64
#define LOCAL(name) name##_f64
#include "quantizer_oracle_body.inc"
