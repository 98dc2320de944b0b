/*
 * cntk_amd_quantizer.h -- C ABI of the MI355X (gfx950) gradient quantizer.
 *
 * This is the boundary a CNTK build binds in place of MatrixQuantizerGPU: one opaque handle per
 * MatrixQuantizerImpl<float> (or <double>, see the _f64 calls at the end) object, plain pointers and sizes, no C++ or torch types. Every call
 * returns a status code; cntkq_last_error() gives the text the reference would have thrown.
 *
 * Data contracts (identical to the reference):
 *   - gradients / residuals / outputs: dense fp32, column-major, rows x cols, leading dimension = rows
 *     (Source/Math/ColumnQuantizer.h:10);
 *   - packed matrix: cols records of cntkq_qcol_bytes(nbits, rows) bytes each, back to back:
 *         { float lower; float upper; uint32_t bits[nq]; }      nq = cntkq_qwords_per_col(rows, nbits)
 *     element i of a column is stored in bits[i % nq] at bit (i / nq) * nbits
 *     (Source/Math/QuantizedMatrix.h:27-48, Source/Math/QuantizedMatrix.cpp:143-169).
 *     A contiguous run of columns of a packed matrix is itself a packed matrix (ColumnSlice,
 *     Source/Math/QuantizedMatrix.cpp:102-107): pass  buffer + first_col * qcol_bytes.
 *   - nbits is one of 1, 2, 4, 8, 16, 32 (32 = pass-through, Source/Math/ValueQuantizer.h:104-107).
 *
 * Ordering: all work of a handle is issued on ONE HIP stream (cntkq_stream). Handles created with
 * use_dedicated_stream != 0 on the same device share one process-wide non-blocking stream, exactly
 * like the reference's static compute stream (Source/Math/MatrixQuantizerGPU.cu:83-90, 197-206), so
 * work issued through different handles is implicitly sequenced. Handles created with
 * use_dedicated_stream == 0 issue on the caller's main stream (the null stream unless
 * cntkq_set_main_stream was called). A handle is not re-entrant; distinct handles may be used
 * from distinct threads.
 *
 * HIP graphs: the quantize, unquantize and stripe-reduction calls (plain and batched) may be issued while the handle's
 * stream is being captured; each becomes kernel nodes only (no allocation, no copy, no memset, no host wait). The
 * matching cntkq_wait_* call then has nothing to wait for and returns at once: order against a replay with the graph's
 * own launch stream. A batched call must have run once outside the capture with the same item list (its argument
 * table is built and uploaded then); after a capture that table is never written again -- a later call with another
 * list builds a new one -- so graphs stay valid until the handle is destroyed. The same holds for the scratch buffer of
 * the kernels that cut very tall columns into strips: once a launch on it has been recorded, the buffer is kept until the
 * handle is destroyed, and a later launch that needs a larger one takes a new buffer. A graph must not be replayed after
 * the handle it was recorded from has been destroyed. Packed matrices in host memory (qbuf_on_host) are refused during
 * capture.
 */
#ifndef CNTK_AMD_QUANTIZER_H
#define CNTK_AMD_QUANTIZER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cntkq_quantizer cntkq_quantizer;

enum
{
    CNTKQ_OK = 0,
    CNTKQ_INVALID_ARGUMENT = 1, /* reference: InvalidArgument / failed assert on dimensions */
    CNTKQ_LOGIC_ERROR = 2,      /* reference: LogicError (bad nbits, packed-size mismatch) */
    CNTKQ_RUNTIME_ERROR = 3     /* reference: RuntimeError from a failed device call */
};

/* Text of the last failure on the calling thread ("" if none). */
const char* cntkq_last_error(void);

/* ---- layout helpers ------------------------------------------------------------------------ */

/* ColumnQuantizer<float>::QWordsPerCol (Source/Math/ColumnQuantizer.h:36-45). 0 if nbits is invalid. */
size_t cntkq_qwords_per_col(size_t rows, size_t nbits);

/* QuantizedColumn<float>::QuantizedColumnSize (Source/Math/QuantizedMatrix.h:42-47). 0 if nbits is invalid. */
size_t cntkq_qcol_bytes(size_t nbits, size_t rows);

/* QuantizedMatrix<float>::GetSize (Source/Math/QuantizedMatrix.cpp:90-94): cols * qcol_bytes. */
size_t cntkq_qmatrix_bytes(size_t rows, size_t cols, size_t nbits);

/* AllReduceDistGradAggregator::GetStripeForNode (Source/1BitSGD/AllReduceDistGradAggregator.h:56-65). */
int cntkq_stripe_range(size_t cols, size_t rank, size_t workers, size_t* start_col, size_t* num_cols);

/* Tallest column the fused stripe reduction (cntkq_stripe_reduce_async / _batch_async, an optional fast path without a
 * counterpart in the reference) accepts on any device at this bit width (0 for an invalid width). Taller stripes: ask
 * cntkq_stripe_reduce_takes; where it says no, the caller keeps the reference's sequence of UnquantizeAsync ...
 * QuantizeAsync calls (Source/1BitSGD/AllReduceDistGradAggregator.h:365-436). */
size_t cntkq_stripe_reduce_max_rows(size_t nbits);

/* ---- the quantizer object -------------------------------------------------------------------- */

/* MatrixQuantizerImpl<float>::Create(deviceId, useAsync) (Source/Math/MatrixQuantizerImpl.cpp:10-26) for
 * deviceId >= 0, i.e. the MatrixQuantizerGPU constructor (Source/Math/MatrixQuantizerGPU.cu:183-207).
 * device_id < 0 (the reference's CPU quantizer) is refused: this library has no CPU path. */
int cntkq_create(int device_id, int use_dedicated_stream, cntkq_quantizer** out);

/* ~MatrixQuantizerGPU (Source/Math/MatrixQuantizerGPU.cu:209-223). Waits for the handle's own work. */
int cntkq_destroy(cntkq_quantizer* h);

/* MatrixQuantizerImpl::GetDeviceId (Source/Math/MatrixQuantizerImpl.h:36-39). */
int cntkq_device_id(const cntkq_quantizer* h);

/* The hipStream_t the handle issues on (MatrixQuantizerGPU::GetComputeStream,
 * Source/Math/MatrixQuantizerGPU.cu:92-96). */
void* cntkq_stream(const cntkq_quantizer* h);

/* Sets the main stream used by handles without a dedicated stream (the reference's GetStream(),
 * Source/Math/MatrixQuantizerGPU.cu:248-252) and by cntkq_sync_with_main_stream. Work already issued on the previous
 * main stream is not ordered against work issued on the new one: that is the caller's to arrange. */
int cntkq_set_main_stream(cntkq_quantizer* h, void* hip_stream);

/* The forceSync argument of the reference's constructor (Source/Math/MatrixQuantizerGPU.h:20,
 * Source/Math/MatrixQuantizerGPU.cu:118-122, 137-141, 237-240, 318-321): when set, cntkq_quantize_async and
 * cntkq_unquantize_async run serialised, for time measurements -- the device is synchronised before a quantization starts,
 * and the host waits for the kernel and for the copy to or from a host-resident packed matrix before the call returns.
 * Off by default. Calls recorded into a graph ignore it. */
int cntkq_set_force_sync(cntkq_quantizer* h, int force_sync);

/* No counterpart in the reference. Columns taller than one workgroup holds (above 102400 rows; doubles 51184) are cut into
 * strips on several workgroups, which by default run as ONE launch whose workgroups wait for each other's partial sums:
 * gradient and residual are read once, but all strips of a column must be running on the device together, which other work
 * on the device at the same time (a training step's kernels on another stream) can prevent -- such a column is then left
 * untouched and the next wait reports it. With never_wait set, the handle runs the strips as two or three launches that
 * read the matrix once each instead: about 1.6 times the time, the same bytes, and no workgroup ever waits for another;
 * cntkq_stripe_reduce_takes then answers 0 for such heights (the caller's sequence of calls, whose QuantizeAsync step runs in
 * those launches). Off by default. */
int cntkq_set_tall_columns_never_wait(cntkq_quantizer* h, int never_wait);

/* MatrixComputeStreamEvent::Create + SynchronizeQuantizationComputeStreamWithEvent
 * (Source/Math/MatrixQuantizerImpl.h:53-72, Source/Math/MatrixQuantizerGPU.cu:347-371): work issued on the
 * handle's stream after this call starts only after everything already issued on the main stream. */
int cntkq_sync_with_main_stream(cntkq_quantizer* h);

/* The same hand-over for a caller that has its own event: work issued on the handle's stream after this call starts
 * only after `hip_event` (a hipEvent_t recorded by the caller, on any stream of the device) has completed. This is what
 * MatrixComputeStreamEvent does with its event (Source/Math/MatrixQuantizerGPU.cu:353-371). */
int cntkq_stream_wait_event(cntkq_quantizer* h, void* hip_event);

/* MatrixQuantizerImpl::QuantizeAsync (Source/Math/MatrixQuantizerImpl.h:30, Source/Math/MatrixQuantizerGPU.cu:226-269).
 *   in, res_in, res_out : device, rows x cols fp32; res_out may be the same pointer as res_in (in place),
 *                         no other overlap is allowed.
 *   qbuf                : packed matrix, qbuf_bytes == cntkq_qmatrix_bytes(rows, cols, nbits);
 *                         device memory, or (qbuf_on_host != 0) host memory, in which case the packed
 *                         data is produced in a device staging buffer owned by the handle and copied
 *                         out asynchronously (pinned host memory keeps that copy asynchronous).
 *   zero_threshold_for_1bit : the reference's zeroThresholdFor1Bit; ignored unless nbits == 1.
 * rows == 0 or cols == 0 is a no-op. */
int cntkq_quantize_async(cntkq_quantizer* h, const float* in, const float* res_in, size_t rows, size_t cols,
                         void* qbuf, size_t qbuf_bytes, int qbuf_on_host, size_t nbits, float* res_out,
                         int zero_threshold_for_1bit);

/* MatrixQuantizerImpl::WaitQuantizeAsyncDone (Source/Math/MatrixQuantizerGPU.cu:271-284): blocks the host
 * until the last quantize of this handle (including its copy to the host, if any) has finished.
 * CNTKQ_RUNTIME_ERROR here can also mean that a launch on columns of more than 102400 rows did not complete: the
 * workgroups that share such a column wait for each other a bounded time, and a column whose workgroups gave up is left
 * as it was -- no header, no codes, residual not updated, also when res_out == res_in -- so the call may be repeated.
 * The error text says how many columns. The other columns of the call are complete and right. */
int cntkq_wait_quantize_done(cntkq_quantizer* h);

/* MatrixQuantizerImpl::UnquantizeAsync (Source/Math/MatrixQuantizerImpl.h:33, Source/Math/MatrixQuantizerGPU.cu:286-334).
 *   out = (add ? out : 0) + unquantize(qbuf).  qbuf_bytes must equal cntkq_qmatrix_bytes(rows, cols, nbits),
 *   else CNTKQ_LOGIC_ERROR (Source/Math/MatrixQuantizer_kernel.cu:287-289); an empty buffer is a no-op (:290-291).
 *   With qbuf_on_host != 0 the packed data is first copied to the handle's staging buffer. */
int cntkq_unquantize_async(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, float* out,
                           size_t rows, size_t cols, size_t nbits, int add);

/* MatrixQuantizerImpl::WaitUnquantizeAsyncDone (Source/Math/MatrixQuantizerGPU.cu:336-341). */
int cntkq_wait_unquantize_done(cntkq_quantizer* h);

/* A whole gradient set in one piece of stream work.
 *
 * The reference's aggregator quantizes (and later unquantizes) its gradient matrices one call each, in a loop
 * (Source/1BitSGD/AllReduceDistGradAggregator.h:288-300 and :517-522; v2: Source/1BitSGD/QuantizedDistributedCommunicator.h:356-366
 * and :516-521), all with the same bit width and threshold mode. On MI355X each launch has a floor of several
 * microseconds, which dominates sets of many small matrices (ResNet-50: 161 matrices); these two calls take the whole
 * loop at once and run it as one launch (plus one per very large matrix). Results are identical to the per-matrix calls.
 *   items : host array, read during the call only. All buffers device-resident, same alignment rules as the
 *           per-matrix calls; res_out may equal res_in; the matrices must not overlap one another.
 *   cntkq_wait_quantize_done / cntkq_wait_unquantize_done wait for the whole batch. */
typedef struct cntkq_quantize_item
{
    const float* in;
    const float* res_in;
    float* res_out;
    void* qbuf;
    size_t rows;
    size_t cols;
    size_t qbuf_bytes; /* must be cntkq_qmatrix_bytes(rows, cols, nbits): the packed-size LogicError of the plain call */
} cntkq_quantize_item;

typedef struct cntkq_unquantize_item
{
    const void* qbuf;
    float* out;
    size_t rows;
    size_t cols;
    size_t qbuf_bytes; /* must be cntkq_qmatrix_bytes(rows, cols, nbits) */
} cntkq_unquantize_item;

int cntkq_quantize_batch_async(cntkq_quantizer* h, const cntkq_quantize_item* items, size_t count, size_t nbits,
                               int zero_threshold_for_1bit);
int cntkq_unquantize_batch_async(cntkq_quantizer* h, const cntkq_unquantize_item* items, size_t count, size_t nbits, int add);

/* cntkq_quantize_batch_async for callers that cannot allocate. It has no counterpart in the reference; it is for code
 * under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc. Same arguments, same kernels and the
 * same bytes as cntkq_quantize_batch_async (one exception below), but the call touches no allocator, device or host: the argument table that
 * the batched kernels read (the only memory of that call beyond its inputs and outputs) lives in a fixed array in the
 * library's device image -- 32 KB, held by every GPU the library runs on until the process ends -- and reaches it as
 * kernel arguments of a small store kernel, not through a copy.
 *   Limits: count <= CNTKQ_NOALLOC_MAX_ITEMS, and the table (CNTKQ_NOALLOC_ENTRY_BYTES + 4 bytes per matrix that shares
 *   the grid, + 8) must fit the array -- it always does within that count; beyond the limit the call fails with
 *   CNTKQ_INVALID_ARGUMENT and does nothing.
 *   The array is shared by every call on that GPU and keeps the last call's contents. Calls on one stream are ordered
 *   like any other stream work; calls that can overlap on one GPU (other streams, other handles on other streams) race
 *   for the array and must be ordered by the caller. A call recorded into a graph writes the array at every replay; from
 *   the first such call on a GPU every call on that GPU uploads its table (a few small launches) instead of trusting
 *   what the array held last.
 *   Columns above 102400 rows: the batched call cuts them into strips whose workgroups meet in a scratch buffer that it
 *   grows on demand. This call uses that buffer only as it stands (created with the handle: enough for about 30000
 *   column-strips, e.g. 150000 x 1500 at 1 bit); a matrix beyond that runs the kernel that re-reads its columns, whose
 *   sums are added in another order, so its column bounds may differ from the batched call's in their last bits.
 *   cntkq_wait_quantize_done waits for the whole batch. */
#define CNTKQ_NOALLOC_MAX_ITEMS 256
#define CNTKQ_NOALLOC_ENTRY_BYTES 112
int cntkq_quantize_batch_noalloc(cntkq_quantizer* h, const cntkq_quantize_item* items, size_t count, size_t nbits,
                                 int zero_threshold_for_1bit);

/* One owner's stripe reduction of the quantized all-reduce, fused into one pass
 * (dataflow of Source/1BitSGD/AllReduceDistGradAggregator.h:365-375 and :385-436; v2:
 * Source/1BitSGD/QuantizedDistributedCommunicator.h:423-471), replacing the reference's sequence
 * UnquantizeAsync(own, add=false); (workers-1) x UnquantizeAsync(peer, add=true); QuantizeAsync(aggregate).
 *   stripes      : host array of `workers` device pointers; stripes[w] is worker w's packed stripe
 *                  (stripe_cols columns of height rows), all quantized with the same nbits.
 *   owner        : index of the worker that owns this stripe. The fp32 sum is taken in the order
 *                  owner first, then the other workers in ascending index (the reference adds them in
 *                  message-arrival order).
 *   stripe_res   : device, rows x stripe_cols fp32, the owner's aggregation residual; updated in place.
 *   q_out        : device, packed stripe that receives the requantized aggregate; may be stripes[owner]
 *                  (the reference overwrites the owner's own slice), must not overlap any other input.
 *   agg_out      : optional (may be NULL) device rows x stripe_cols fp32 that receives the fp32 aggregate
 *                  before requantization (the reference leaves it in the owner's slice of the gradient).
 * Limits: 1 <= workers <= CNTKQ_MAX_WORKERS. */
#define CNTKQ_MAX_WORKERS 64
int cntkq_stripe_reduce_async(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner,
                              size_t rows, size_t stripe_cols, size_t nbits, float* stripe_res, void* q_out,
                              float* agg_out, int zero_threshold_for_1bit);

/* The owner's stripe reductions for a whole gradient set (one item per gradient matrix) as one piece of stream work:
 * the loop over the gradient matrices around the calls above (Source/1BitSGD/AllReduceDistGradAggregator.h:339-436 runs
 * per matrix i). Same workers, owner, bit width and threshold mode for all items; results identical to
 * cntkq_stripe_reduce_async item by item. items and the stripes arrays are host memory, read during the call only.
 * cntkq_wait_stripe_reduce_done waits for the whole batch. */
typedef struct cntkq_stripe_reduce_item
{
    const void* const* stripes; /* `workers` device pointers: worker w's packed stripe of this matrix */
    float* stripe_res;          /* rows x stripe_cols, updated in place */
    void* q_out;                /* packed stripe receiving the requantized aggregate; may be stripes[owner] */
    float* agg_out;             /* optional (may be NULL) */
    size_t rows;
    size_t stripe_cols;
} cntkq_stripe_reduce_item;

int cntkq_stripe_reduce_batch_async(cntkq_quantizer* h, const cntkq_stripe_reduce_item* items, size_t count, size_t workers,
                                    size_t owner, size_t nbits, int zero_threshold_for_1bit);

/* The same with an owner per item: item i is reduced as rank owners[i] reduces its stripe, i.e. the loop of
 * Source/1BitSGD/AllReduceDistGradAggregator.h:339-436 as EVERY rank runs it, in one call. For K workers simulated in
 * one GPU's memory (all K ranks' stripes then form one grid instead of K launches that each fill a fraction of the chip);
 * results identical to cntkq_stripe_reduce_async item by item with owner = owners[i]. owners: `count` entries, host
 * memory, read during the call only. */
int cntkq_stripe_reduce_batch_owners_async(cntkq_quantizer* h, const cntkq_stripe_reduce_item* items, const size_t* owners,
                                           size_t count, size_t workers, size_t nbits, int zero_threshold_for_1bit);

/* Blocks until the last stripe reduction of this handle has finished (the reference waits on the stripe
 * quantizer's WaitQuantizeAsyncDone, Source/1BitSGD/AllReduceDistGradAggregator.h:494). A reduction that ran on strips
 * (see cntkq_stripe_reduce_takes) reports here, as CNTKQ_RUNTIME_ERROR, columns whose workgroups gave up waiting for one
 * another; those columns are left as they were. */
int cntkq_wait_stripe_reduce_done(cntkq_quantizer* h);

/* Whether the fused stripe reduction of this handle takes stripes of this shape (1) or the caller keeps the reference's
 * sequence of UnquantizeAsync ... QuantizeAsync calls for them (0). No counterpart in the reference: the fused call is
 * an optional fast path. Always 1 up to cntkq_stripe_reduce_max_rows(nbits). Taller stripes run with several workgroups per
 * column where a QuantizeAsync call on the same shape does too (heights that no single workgroup holds: above 102400
 * rows, 81820 at 8 bits, 40910 at 16) and the device holds all of a column's workgroups at once: 1 to 16 bits, up to some 4
 * million rows at 1 to 4 bits on an MI355X. The answer holds for the handle's current stream; under stream capture it is
 * 0 where the call would have to allocate. */
int cntkq_stripe_reduce_takes(cntkq_quantizer* h, size_t rows, size_t stripe_cols, size_t nbits, int zero_threshold_for_1bit);

/* ---- the double instantiation: MatrixQuantizerImpl<double> -----------------------------------------------
 *
 * The reference instantiates the whole path for ElemType = double as well (Source/Math/MatrixQuantizerImpl.cpp:28-29,
 * Source/Math/MatrixQuantizerGPU.cu:344-345, Source/Math/QuantizedMatrix.cpp:183-184); its QWord is then the 64-bit
 * unsigned integer (Source/Math/ValueQuantizer.h:50-57). Same handle type, same streams, same waits
 * (cntkq_wait_quantize_done etc.), same semantics as the float calls above, with
 *   - matrices: dense fp64, column-major, 8-byte aligned;
 *   - packed matrix: cols records { double lower; double upper; uint64_t bits[nq]; }, nq = ceil(rows / (64 / nbits)),
 *     element i in bits[i % nq] at bit (i / nq) * nbits; the buffer must be 8-byte aligned;
 *   - nbits one of 1, 2, 4, 8, 16, 32, 64 (64 = pass-through; 32 is a real quantizer with 2^32 - 1 steps);
 *   - stripe reduction: rows <= cntkq_stripe_reduce_max_rows_f64(nbits), or a shape cntkq_stripe_reduce_takes_f64 accepts.
 * The gradient-set (batch) calls have their _f64 forms further down. */

/* ColumnQuantizer<double>::QWordsPerCol, QuantizedColumn<double>::QuantizedColumnSize, QuantizedMatrix<double>::GetSize. */
size_t cntkq_qwords_per_col_f64(size_t rows, size_t nbits);
size_t cntkq_qcol_bytes_f64(size_t nbits, size_t rows);
size_t cntkq_qmatrix_bytes_f64(size_t rows, size_t cols, size_t nbits);

/* MatrixQuantizerImpl<double>::QuantizeAsync (Source/Math/MatrixQuantizerImpl.h:30, Source/Math/MatrixQuantizerGPU.cu:226-269). */
int cntkq_quantize_async_f64(cntkq_quantizer* h, const double* in, const double* res_in, size_t rows, size_t cols,
                             void* qbuf, size_t qbuf_bytes, int qbuf_on_host, size_t nbits, double* res_out,
                             int zero_threshold_for_1bit);

/* MatrixQuantizerImpl<double>::UnquantizeAsync (Source/Math/MatrixQuantizerImpl.h:33, Source/Math/MatrixQuantizerGPU.cu:286-334). */
int cntkq_unquantize_async_f64(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, double* out,
                               size_t rows, size_t cols, size_t nbits, int add);

/* cntkq_stripe_reduce_async for double stripes (same dataflow and summation order). */
int cntkq_stripe_reduce_async_f64(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner,
                                  size_t rows, size_t stripe_cols, size_t nbits, double* stripe_res, void* q_out,
                                  double* agg_out, int zero_threshold_for_1bit);
size_t cntkq_stripe_reduce_max_rows_f64(size_t nbits);
/* cntkq_stripe_reduce_takes for double stripes (taller than cntkq_stripe_reduce_max_rows_f64: from 51185 rows, 1 to 32 bits). */
int cntkq_stripe_reduce_takes_f64(cntkq_quantizer* h, size_t rows, size_t stripe_cols, size_t nbits, int zero_threshold_for_1bit);

/* The gradient-set calls (cntkq_quantize_batch_async, cntkq_unquantize_batch_async, cntkq_stripe_reduce_batch_async) for
 * double matrices: the same loops of the aggregator (Source/1BitSGD/AllReduceDistGradAggregator.h:288-300, 339-436,
 * 517-522) as one call each; results identical to the _f64 plain calls item by item. Pointers 8-byte aligned. */
typedef struct cntkq_quantize_item_f64
{
    const double* in;
    const double* res_in;
    double* res_out; /* may be res_in */
    void* qbuf;      /* device memory */
    size_t rows;
    size_t cols;
    size_t qbuf_bytes; /* must be cols * cntkq_qcol_bytes_f64(nbits, rows) */
} cntkq_quantize_item_f64;

typedef struct cntkq_unquantize_item_f64
{
    const void* qbuf;
    double* out;
    size_t rows;
    size_t cols;
    size_t qbuf_bytes; /* must be cols * cntkq_qcol_bytes_f64(nbits, rows) */
} cntkq_unquantize_item_f64;

typedef struct cntkq_stripe_reduce_item_f64
{
    const void* const* stripes; /* `workers` device pointers: worker w's packed stripe of this matrix */
    double* stripe_res;         /* rows x stripe_cols, updated in place */
    void* q_out;                /* packed stripe receiving the requantized aggregate; may be stripes[owner] */
    double* agg_out;            /* optional (may be NULL) */
    size_t rows;                /* a height cntkq_stripe_reduce_takes_f64 accepts */
    size_t stripe_cols;
} cntkq_stripe_reduce_item_f64;

int cntkq_quantize_batch_async_f64(cntkq_quantizer* h, const cntkq_quantize_item_f64* items, size_t count, size_t nbits,
                                   int zero_threshold_for_1bit);
int cntkq_unquantize_batch_async_f64(cntkq_quantizer* h, const cntkq_unquantize_item_f64* items, size_t count, size_t nbits, int add);
int cntkq_stripe_reduce_batch_async_f64(cntkq_quantizer* h, const cntkq_stripe_reduce_item_f64* items, size_t count, size_t workers,
                                        size_t owner, size_t nbits, int zero_threshold_for_1bit);
int cntkq_stripe_reduce_batch_owners_async_f64(cntkq_quantizer* h, const cntkq_stripe_reduce_item_f64* items, const size_t* owners,
                                               size_t count, size_t workers, size_t nbits, int zero_threshold_for_1bit);

#ifdef __cplusplus
}
#endif
#endif /* CNTK_AMD_QUANTIZER_H */
