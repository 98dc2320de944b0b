/*
 * CPU oracle for the per-column gradient quantizer -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the reference CPU quantizer's arithmetic. Used by the tests as the
 * checker for the HIP kernels and by the benchmark as the timed CPU baseline. The shipped
 * library never links, loads or calls anything in this file.
 *
 * What pins each function (so that a dropped term, wrong sign or transposed index fails):
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

#define QWORD_BITS 32u

/* ---- layout (Source/Math/ColumnQuantizer.h:36-40, Source/Math/QuantizedMatrix.h:42-47) ---- */

int oracle_check_nbits(size_t nbits)
{
    return (nbits == 1 || nbits == 2 || nbits == 4 || nbits == 8 || nbits == 16 || nbits == 32) ? 0 : -1;
}

size_t oracle_qwords_per_col(size_t rows, size_t nbits)
{
    size_t per_word = QWORD_BITS / nbits;
    return (rows + per_word - 1) / per_word;
}

size_t oracle_qcol_bytes(size_t nbits, size_t rows)
{
    size_t payload = ((rows * nbits + (QWORD_BITS - 1)) / QWORD_BITS) * sizeof(uint32_t);
    return 2 * sizeof(float) + payload;
}

/* ---- per-value quantizer state (Source/Math/ValueQuantizer.h:68-97) ---- */

typedef struct
{
    size_t nbits;
    uint32_t rangeend; /* 2^nbits, or 0 in the 32-bit pass-through mode */
    float lo, hi, mid;
    float qfactor, ufactor;
} vq_t;

static vq_t vq_make(size_t nbits, float lower, float upper)
{
    vq_t v;
    v.nbits = nbits;
    v.lo = lower;
    v.hi = upper;
    v.rangeend = (nbits >= QWORD_BITS) ? 0u : ((uint32_t) 1 << nbits);
    if (((upper - lower) < 1e-36f) || (v.rangeend == 0))
    {
        v.qfactor = 0.0f;
        v.ufactor = 0.0f;
    }
    else
    {
        /* one code fewer than 2^nbits is spread over the range when nbits > 1 */
        size_t used = (size_t) v.rangeend - (nbits > 1 ? 1 : 0);
        v.qfactor = (float) used / (upper - lower);
        v.ufactor = (upper - lower) / (float) used;
    }
    v.mid = 0.5f * (upper + lower);
    return v;
}

/* Source/Math/ValueQuantizer.h:101-128, 144-156 */
static uint32_t vq_quantize(const vq_t* v, float u, int zero_threshold)
{
    if (v->nbits == QWORD_BITS)
    {
        uint32_t raw;
        memcpy(&raw, &u, sizeof raw);
        return raw;
    }
    if (v->nbits == 1)
        return zero_threshold ? (u >= 0.0f) : (u >= v->mid);
    if (u <= v->lo)
        return 0;
    if (u >= v->hi)
        return v->rangeend - 1;
    return (uint32_t) (int32_t) ((u - v->lo) * v->qfactor);
}

/* Source/Math/ValueQuantizer.h:131-141 */
static float vq_unquantize(const vq_t* v, uint32_t q)
{
    if (v->nbits == QWORD_BITS)
    {
        float f;
        memcpy(&f, &q, sizeof f);
        return f;
    }
    float t = (float) q + 0.5f;
    t = t * v->ufactor;
    return t + v->lo;
}

uint32_t oracle_quantize_value(float u, size_t nbits, float lower, float upper, int zero_threshold)
{
    vq_t v = vq_make(nbits, lower, upper);
    return vq_quantize(&v, u, zero_threshold);
}

float oracle_unquantize_value(uint32_t q, size_t nbits, float lower, float upper)
{
    vq_t v = vq_make(nbits, lower, upper);
    return vq_unquantize(&v, q);
}

/* ---- per-column range statistics (Source/Math/ColumnQuantizer.h:209-341, serial case) ---- */

void oracle_column_stats(const float* g, const float* r, size_t rows, size_t j, size_t nbits,
                         int zero_threshold, float* lower, float* upper)
{
    const float* gc = g + j * rows;
    const float* rc = r + j * rows;
    float mean = 0.0f;

    if (!zero_threshold && nbits == 1)
    {
        float acc = 0.0f;
        for (size_t i = 0; i < rows; i++)
            acc += gc[i] + rc[i];
        mean = acc / (float) rows;
    }

    if (nbits == 1)
    {
        /* two reconstruction levels: means of the part below / not below the threshold */
        float acc0 = 0.0f, acc1 = 0.0f;
        unsigned int n0 = 0, n1 = 0;
        for (size_t i = 0; i < rows; i++)
        {
            float v = gc[i] + rc[i];
            if (v < mean)
            {
                acc0 += v;
                n0++;
            }
            else
            {
                acc1 += v;
                n1++;
            }
        }

        float radius, centre;
        if (!zero_threshold)
        {
            /* both sides tied to one mean absolute deviation around the column mean */
            float dev0 = ((float) n0 * mean) - acc0;
            float dev1 = acc1 - ((float) n1 * mean);
            float dev = (dev0 + dev1) / (float) rows;
            radius = 2.0f * dev;
            centre = mean;
        }
        else
        {
            /* threshold pinned at 0, separate level means; empty sides count as one element */
            if (n0 == 0)
                n0 = 1;
            if (n1 == 0)
                n1 = 1;
            float m0 = acc0 / (float) n0;
            float m1 = acc1 / (float) n1;
            centre = 0.5f * (m0 + m1);
            radius = 2.0f * (m1 - centre);
        }
        *lower = centre - radius;
        *upper = centre + radius;
    }
    else
    {
        /* linear range of +/- 4 standard deviations about a mean that is taken to be 0 */
        const float stddevs = 4.0f;
        float acc = 0.0f;
        for (size_t i = 0; i < rows; i++)
        {
            float v = gc[i] + rc[i];
            float d = v - mean;
            acc += d * d;
        }
        float sd = sqrtf(acc / (float) rows);
        float half = stddevs * sd;
        *lower = mean - half;
        *upper = mean + half;
    }
}

/* ---- pack / unpack one column (Source/Math/ColumnQuantizer.h:90-147, 149-203) ----
 * Word w of a column holds rows w, w + nq, w + 2 nq, ...; the k-th of them sits at bit k * nbits. */

static void quantize_column(const float* g, const float* r_in, size_t rows, size_t j, size_t nbits,
                            int zero_threshold, float lower, float upper, uint32_t* words, float* r_out)
{
    const vq_t v = vq_make(nbits, lower, upper);
    const size_t nq = oracle_qwords_per_col(rows, nbits);
    const size_t base = j * rows;
    for (size_t w = 0; w < nq; w++)
    {
        uint32_t word = 0;
        size_t i = w;
        for (size_t shift = 0; shift < QWORD_BITS && i < rows; shift += nbits, i += nq)
        {
            float val = g[base + i] + r_in[base + i];
            uint32_t q = vq_quantize(&v, val, zero_threshold);
            float back = vq_unquantize(&v, q);
            r_out[base + i] = val - back;
            word |= q << shift;
        }
        words[w] = word;
    }
}

static void unquantize_column(const uint32_t* words, size_t rows, size_t j, size_t nbits, float lower,
                              float upper, float* out, int add)
{
    const vq_t v = vq_make(nbits, lower, upper);
    const size_t nq = oracle_qwords_per_col(rows, nbits);
    const uint32_t mask = v.rangeend - 1; /* all ones in pass-through mode */
    const size_t base = j * rows;
    for (size_t w = 0; w < nq; w++)
    {
        const uint32_t word = words[w];
        size_t i = w;
        for (size_t shift = 0; shift < QWORD_BITS && i < rows; shift += nbits, i += nq)
        {
            float val = vq_unquantize(&v, (word >> shift) & mask);
            if (add)
                val += out[base + i];
            out[base + i] = val;
        }
    }
}

/* ---- whole matrix (Source/Math/MatrixQuantizerCPU.cpp:12-63, 72-100) ---- */

int oracle_quantize(const float* g, const float* r_in, size_t rows, size_t cols, void* qbuf,
                    size_t nbits, float* r_out, int zero_threshold, int threads)
{
    if (oracle_check_nbits(nbits) != 0)
        return -1;
    const size_t qcol = oracle_qcol_bytes(nbits, rows);
    char* q = (char*) qbuf;
    long long n = (long long) cols;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (long long jj = 0; jj < n; jj++)
    {
        size_t j = (size_t) jj;
        float* hdr = (float*) (q + j * qcol);
        float lower, upper;
        oracle_column_stats(g, r_in, rows, j, nbits, zero_threshold, &lower, &upper);
        hdr[0] = lower;
        hdr[1] = upper;
        quantize_column(g, r_in, rows, j, nbits, zero_threshold, lower, upper, (uint32_t*) (hdr + 2), r_out);
    }
    return 0;
}

int oracle_pack_with_headers(const float* g, const float* r_in, size_t rows, size_t cols, void* qbuf,
                             size_t nbits, float* r_out, int zero_threshold, int threads)
{
    /* second half of oracle_quantize alone: the (lower, upper) already stored in qbuf are kept */
    if (oracle_check_nbits(nbits) != 0)
        return -1;
    const size_t qcol = oracle_qcol_bytes(nbits, rows);
    char* q = (char*) qbuf;
    long long n = (long long) cols;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (long long jj = 0; jj < n; jj++)
    {
        size_t j = (size_t) jj;
        float* hdr = (float*) (q + j * qcol);
        quantize_column(g, r_in, rows, j, nbits, zero_threshold, hdr[0], hdr[1], (uint32_t*) (hdr + 2), r_out);
    }
    return 0;
}

int oracle_unquantize(const void* qbuf, size_t rows, size_t cols, size_t nbits, float* out, int add,
                      int threads)
{
    if (oracle_check_nbits(nbits) != 0)
        return -1;
    const size_t qcol = oracle_qcol_bytes(nbits, rows);
    const char* q = (const char*) qbuf;
    long long n = (long long) cols;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (long long jj = 0; jj < n; jj++)
    {
        size_t j = (size_t) jj;
        const float* hdr = (const float*) (q + j * qcol);
        unquantize_column((const uint32_t*) (hdr + 2), rows, j, nbits, hdr[0], hdr[1], out, add);
    }
    return 0;
}

/* ---- simulated K-worker all-reduce (Source/1BitSGD/AllReduceDistGradAggregator.h) ---- */

void oracle_stripe_range(size_t cols, size_t rank, size_t workers, size_t* start, size_t* len)
{
    size_t per = cols / workers;
    size_t extra = cols % workers;
    *start = per * rank + (extra < rank ? extra : rank);
    *len = per + (rank < extra ? 1 : 0);
}

int oracle_stripe_reduce(void* const* q, size_t workers, size_t owner, size_t rows, size_t cols,
                         size_t nbits, float* stripe_res, float* agg_scratch, int zero_threshold,
                         int threads)
{
    if (oracle_check_nbits(nbits) != 0)
        return -1;
    size_t start, len;
    oracle_stripe_range(cols, owner, workers, &start, &len);
    if (len == 0)
        return 0;
    const size_t qcol = oracle_qcol_bytes(nbits, rows);
    /* the owner's own quantized stripe seeds the aggregate (lines 365-375) */
    oracle_unquantize((const char*) q[owner] + start * qcol, rows, len, nbits, agg_scratch, 0, threads);
    /* then every other worker's stripe is decoded on top of it (lines 385-436) */
    for (size_t w = 0; w < workers; w++)
    {
        if (w == owner)
            continue;
        oracle_unquantize((const char*) q[w] + start * qcol, rows, len, nbits, agg_scratch, 1, threads);
    }
    /* requantize with the stripe's own residual, over the owner's slice of its packed matrix */
    return oracle_quantize(agg_scratch, stripe_res, rows, len, (char*) q[owner] + start * qcol, nbits,
                           stripe_res, zero_threshold, threads);
}

int oracle_allreduce(const float* const* g, float* const* res, void* const* q, float* const* stripe_res,
                     size_t workers, size_t rows, size_t cols, size_t nbits, int zero_threshold,
                     void* qagg, float* out, int threads)
{
    if (oracle_check_nbits(nbits) != 0)
        return -1;
    const size_t qcol = oracle_qcol_bytes(nbits, rows);
    for (size_t w = 0; w < workers; w++)
        oracle_quantize(g[w], res[w], rows, cols, q[w], nbits, res[w], zero_threshold, threads);
    for (size_t s = 0; s < workers; s++)
    {
        size_t start, len;
        oracle_stripe_range(cols, s, workers, &start, &len);
        if (len == 0)
            continue;
        /* `out` doubles as the fp32 aggregate: the reference aggregates into the owner's slice of
         * the gradient matrix itself, which the final unquantize then overwrites (lines 268-300). */
        oracle_stripe_reduce(q, workers, s, rows, cols, nbits, stripe_res[s], out + start * rows,
                             zero_threshold, threads);
        memcpy((char*) qagg + start * qcol, (const char*) q[s] + start * qcol, len * qcol);
    }
    return oracle_unquantize(qagg, rows, cols, nbits, out, 0, threads);
}
