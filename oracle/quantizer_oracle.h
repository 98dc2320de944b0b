/*
 * CPU oracle for the per-column gradient quantizer -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the arithmetic of the reference CPU quantizer.
 * It exists to check the HIP kernels and to serve as the timed CPU baseline; the
 * shipped library never links, loads or calls it.
 *
 * All arithmetic is IEEE fp32, every operation separately rounded (build with
 * -ffp-contract=off, no fast-math), sums taken strictly in increasing row order.
 */
#ifndef CNTK_AMD_QUANTIZER_ORACLE_H
#define CNTK_AMD_QUANTIZER_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 0 when nbits is one of 1,2,4,8,16,32, else -1
 * (Source/Math/ValueQuantizer.h:177-191, Source/Math/QuantizedMatrix.cpp:12-15). */
int oracle_check_nbits(size_t nbits);

/* Number of 32-bit QWords in one packed column (Source/Math/ColumnQuantizer.h:36-40). */
size_t oracle_qwords_per_col(size_t rows, size_t nbits);

/* Bytes of one packed column record {f32 lower; f32 upper; u32 bits[nq]}
 * (Source/Math/QuantizedMatrix.h:42-47). */
size_t oracle_qcol_bytes(size_t nbits, size_t rows);

/* Scalar quantize / unquantize for one value under a column header
 * (Source/Math/ValueQuantizer.h:68-97, 101-128, 131-141, 144-156). */
uint32_t oracle_quantize_value(float u, size_t nbits, float lower, float upper, int zero_threshold);
float oracle_unquantize_value(uint32_t q, size_t nbits, float lower, float upper);

/* Range statistics of column j of (g + r) (Source/Math/ColumnQuantizer.h:209-341). */
void oracle_column_stats(const float* g, const float* r, size_t rows, size_t j, size_t nbits,
                         int zero_threshold, float* lower, float* upper);

/* Quantize a whole column-major rows x cols matrix into qbuf (cols packed column records),
 * writing the new residual to r_out (r_out may alias r_in)
 * (Source/Math/MatrixQuantizerCPU.cpp:12-63, Source/Math/ColumnQuantizer.h:50-65, 90-147).
 * threads > 1 splits the (independent) columns over OpenMP threads. Returns 0, or -1 for bad nbits. */
int oracle_quantize(const float* g, const float* r_in, size_t rows, size_t cols, void* qbuf,
                    size_t nbits, float* r_out, int zero_threshold, int threads);

/* Packing step of oracle_quantize alone (Source/Math/ColumnQuantizer.h:50-65, 90-147): the column
 * headers already present in qbuf are used as they are, only codes and residual are produced. Lets a
 * test check codes and residuals bit for bit under headers that came from somewhere else. */
int oracle_pack_with_headers(const float* g, const float* r_in, size_t rows, size_t cols, void* qbuf,
                             size_t nbits, float* r_out, int zero_threshold, int threads);

/* Inverse: out = (add ? out : 0) + unquantize(qbuf)
 * (Source/Math/MatrixQuantizerCPU.cpp:72-100, Source/Math/ColumnQuantizer.h:68-78, 149-203). */
int oracle_unquantize(const void* qbuf, size_t rows, size_t cols, size_t nbits, float* out,
                      int add, int threads);

/* Column stripe owned by worker `rank` of `workers`
 * (Source/1BitSGD/AllReduceDistGradAggregator.h:56-65). */
void oracle_stripe_range(size_t cols, size_t rank, size_t workers, size_t* start, size_t* len);

/* One owner's stripe reduction (Source/1BitSGD/AllReduceDistGradAggregator.h:339-436):
 *   A  = unquantize(q[owner] stripe)            (add = false; self stripe first)
 *   A += unquantize(q[r] stripe), r != owner    in ascending r (the reference's order is arrival order)
 *   q[owner] stripe = quantize(A, stripe_res -> stripe_res)
 * q[w] points at worker w's full packed matrix (cols columns); stripe_res is rows x len.
 * agg_scratch (rows x len floats) receives A. */
int oracle_stripe_reduce(void* const* q, size_t workers, size_t owner, size_t rows, size_t cols,
                         size_t nbits, float* stripe_res, float* agg_scratch,
                         int zero_threshold, int threads);

/* Whole simulated K-worker quantized all-reduce of one gradient matrix
 * (Source/1BitSGD/AllReduceDistGradAggregator.h:268-531):
 *   every worker w: q[w] = quantize(g[w], res[w] -> res[w])
 *   every owner s : stripe reduction into q[s]'s own stripe, with stripe_res[s]
 *   assembled     : qagg = [q[0] stripe 0 | ... | q[K-1] stripe K-1];  out = unquantize(qagg)
 * qagg (cols packed columns) and out (rows x cols) are outputs. */
int oracle_allreduce(const float* const* g, float* const* res, void* const* q, float* const* stripe_res,
                     size_t workers, size_t rows, size_t cols, size_t nbits, int zero_threshold,
                     void* qagg, float* out, int threads);

/* ---- MatrixQuantizerImpl<double> (QWord = uint64_t, nbits in 1..64, record {f64 lower; f64 upper; u64 bits[nq]}) ----
 * Same functions, same citations; only the element and QWord types differ. */
int oracle_check_nbits_f64(size_t nbits);
size_t oracle_qwords_per_col_f64(size_t rows, size_t nbits);
size_t oracle_qcol_bytes_f64(size_t nbits, size_t rows);
uint64_t oracle_quantize_value_f64(double u, size_t nbits, double lower, double upper, int zero_threshold);
double oracle_unquantize_value_f64(uint64_t q, size_t nbits, double lower, double upper);
void oracle_column_stats_f64(const double* g, const double* r, size_t rows, size_t j, size_t nbits,
                             int zero_threshold, double* lower, double* upper);
int oracle_quantize_f64(const double* g, const double* r_in, size_t rows, size_t cols, void* qbuf,
                        size_t nbits, double* r_out, int zero_threshold, int threads);
int oracle_pack_with_headers_f64(const double* g, const double* r_in, size_t rows, size_t cols, void* qbuf,
                                 size_t nbits, double* r_out, int zero_threshold, int threads);
int oracle_unquantize_f64(const void* qbuf, size_t rows, size_t cols, size_t nbits, double* out,
                          int add, int threads);
int oracle_stripe_reduce_f64(void* const* q, size_t workers, size_t owner, size_t rows, size_t cols,
                             size_t nbits, double* stripe_res, double* agg_scratch,
                             int zero_threshold, int threads);
int oracle_allreduce_f64(const double* const* g, double* const* res, void* const* q, double* const* stripe_res,
                         size_t workers, size_t rows, size_t cols, size_t nbits, int zero_threshold,
                         void* qagg, double* out, int threads);

#ifdef __cplusplus
}
#endif
#endif
