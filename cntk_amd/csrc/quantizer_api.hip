// C ABI of the MI355X gradient quantizer: handles, streams, events, argument checks.
// Replaces the host side of the reference's GPU quantizer (Source/Math/MatrixQuantizerGPU.cu:83-341).
#include "../../include/cntk_amd_quantizer.h"
#include "quantizer_internal.h"
#include "quantizer_launch.h"
#include "quantizer_launch_f64.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

using namespace cntkq;

namespace {

thread_local char g_last_error[1024] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(call, what)                                                                                          \
    do                                                                                                               \
    {                                                                                                                \
        hipError_t rc__ = (call);                                                                                    \
        if (rc__ != hipSuccess)                                                                                      \
            return fail(CNTKQ_RUNTIME_ERROR, "%s: %s (hip error %d)", what, hipGetErrorString(rc__), (int) rc__);    \
    } while (0)

// Process-wide streams per device, created on first use and never destroyed, like the reference's
// static compute / fetch / assign streams (Source/Math/MatrixQuantizerGPU.cu:83-90, 197-206).
constexpr int kMaxDevices = 64;
struct DeviceStreams
{
    hipStream_t compute = nullptr;
    hipStream_t fetch = nullptr;
    hipStream_t assign = nullptr;
};
DeviceStreams g_streams[kMaxDevices];
std::mutex g_streams_mutex;

class DeviceGuard // PrepareDevice (Source/Math/MatrixQuantizerGPU.cu:186, 234): make the handle's device current
{
public:
    explicit DeviceGuard(int device) : m_prev(-1), m_changed(false)
    {
        if (hipGetDevice(&m_prev) == hipSuccess && m_prev != device)
            m_changed = (hipSetDevice(device) == hipSuccess);
    }
    ~DeviceGuard()
    {
        if (m_changed)
            (void) hipSetDevice(m_prev);
    }

private:
    int m_prev;
    bool m_changed;
};

bool aligned4(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 3u) == 0;
}

// What differs between the two instantiations of the boundary (MatrixQuantizerImpl<float> / <double>).
template <typename E>
struct Elem;

template <>
struct Elem<float>
{
    static constexpr size_t kAlign = 4;
    static constexpr size_t kWordBits = 32;
    static size_t stripe_max_rows(size_t nbits) { return cntkq::stripe_reduce_max_rows(nbits); }
    static bool valid_nbits(size_t nbits) { return cntkq::valid_nbits(nbits); }
    static size_t qcol_bytes(size_t nbits, size_t rows) { return cntkq::qcol_bytes(nbits, rows); }
    static hipError_t quantize(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, void* q, size_t rows,
                               size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
    {
        return cntkq::launch_quantize(s, ev, g, r_in, r_out, q, rows, cols, nbits, zt, tune);
    }
    static hipError_t unquantize(hipStream_t s, LaunchEvents ev, const void* q, float* out, size_t rows, size_t cols, size_t nbits,
                                 bool add, const LaunchTuning& tune)
    {
        return cntkq::launch_unquantize(s, ev, q, out, rows, cols, nbits, add, tune);
    }
    static hipError_t stripe_reduce(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, void* q_out,
                                    float* agg_out, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
    {
        return cntkq::launch_stripe_reduce(s, ev, src, stripe_res, q_out, agg_out, rows, cols, nbits, zt, tune);
    }
};

template <>
struct Elem<double>
{
    static constexpr size_t kAlign = 8;
    static constexpr size_t kWordBits = 64;
    static size_t stripe_max_rows(size_t) { return cntkq::f64::kTileMaxRows; }
    static bool valid_nbits(size_t nbits) { return cntkq::f64::valid_nbits(nbits); }
    static size_t qcol_bytes(size_t nbits, size_t rows) { return cntkq::f64::qcol_bytes(nbits, rows); }
    static hipError_t quantize(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, void* q, size_t rows,
                               size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
    {
        return cntkq::f64::launch_quantize(s, ev, g, r_in, r_out, q, rows, cols, nbits, zt, tune);
    }
    static hipError_t unquantize(hipStream_t s, LaunchEvents ev, const void* q, double* out, size_t rows, size_t cols, size_t nbits,
                                 bool add, const LaunchTuning& tune)
    {
        return cntkq::f64::launch_unquantize(s, ev, q, out, rows, cols, nbits, add, tune);
    }
    static hipError_t stripe_reduce(hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, void* q_out,
                                    double* agg_out, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
    {
        return cntkq::f64::launch_stripe_reduce(s, ev, src, stripe_res, q_out, agg_out, rows, cols, nbits, zt, tune);
    }
};

template <typename E>
bool aligned_for(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & (Elem<E>::kAlign - 1)) == 0;
}

} // namespace

struct BatchTable
{
    std::vector<char> key;   // the item list and parameters the table was built for
    char* host = nullptr;    // pinned
    char* dev = nullptr;
    size_t capacity = 0;
    hipEvent_t event = nullptr; // set when the last kernel that reads the table has finished
    bool in_flight = false;
    // A launch that reads the table was recorded into a graph (stream capture): the graph may be replayed at any time
    // from then on, so the buffers are never written again; a rebuild retires them (freed with the handle) and takes
    // fresh ones.
    bool captured = false;
    std::vector<std::pair<char*, char*>> retired;
    // launch parameters of the two LDS classes and the matrices that get a launch of their own
    size_t members[2] = {0, 0};
    uint32_t blocks[2] = {0, 0};
    size_t lds[2] = {0, 0};
    size_t first_entry[2] = {0, 0};
    size_t first_begin[2] = {0, 0};
    size_t entries_bytes = 0;
    std::vector<size_t> own;
};

struct cntkq_quantizer
{
    int device = 0;
    bool dedicated = false;
    hipStream_t main_stream = nullptr;
    hipStream_t compute = nullptr; // == main_stream when !dedicated
    hipStream_t fetch = nullptr;
    hipStream_t assign = nullptr;
    hipEvent_t ev_quantize = nullptr;
    hipEvent_t ev_fetch = nullptr;
    hipEvent_t ev_assign = nullptr;
    hipEvent_t ev_unquantize = nullptr;
    hipEvent_t ev_stripe = nullptr;
    hipEvent_t ev_main = nullptr;
    // the event each Wait call waits on: the handle's own, or one attached through the debug hook
    hipEvent_t last_quantize = nullptr;
    hipEvent_t last_unquantize = nullptr;
    hipEvent_t last_stripe = nullptr;
    hipEvent_t attach_start = nullptr; // one-shot: tied to the next kernel this handle launches
    hipEvent_t attach_stop = nullptr;
    bool quantize_included_fetch = false;
    bool fetch_pending = false;   // a device-to-host copy out of the staging buffer may still be running
    bool staging_read_pending = false; // a kernel reading the staging buffer may still be running
    char* staging = nullptr;      // device buffer used when the packed matrix lives in host memory
    size_t staging_bytes = 0;
    // entry tables of the batched calls, one for quantize and one for unquantize. A gradient set is the same list of
    // matrices step after step, so the table built for a list is kept (host key, pinned host copy, device copy, launch
    // parameters) and a call with the same list only launches. A table is rebuilt only after the last kernel that
    // reads it has finished (its event).
    BatchTable quantize_table;
    BatchTable unquantize_table;
    BatchTable stripe_table;
    BatchTable quantize_table64; // the same for the _f64 batched calls
    BatchTable unquantize_table64;
    BatchTable stripe_table64;
    LaunchTuning tune;
};

namespace {

hipStream_t work_stream(const cntkq_quantizer* h)
{
    return h->dedicated ? h->compute : h->main_stream;
}

// Completion is signalled by the kernel dispatch itself (no separate event record in the stream).
LaunchEvents take_events(cntkq_quantizer* h, hipEvent_t own)
{
    LaunchEvents ev;
    ev.start = h->attach_start;
    ev.stop = h->attach_stop != nullptr ? h->attach_stop : own;
    h->attach_start = nullptr;
    h->attach_stop = nullptr;
    return ev;
}

// Temp device buffer for a host-resident packed matrix (GetTempGPUQuantizedMatrix,
// Source/Math/MatrixQuantizerGPU.cu:158-179). Grows only; waits for everything that may still use the old one.
int ensure_staging(cntkq_quantizer* h, size_t bytes)
{
    if (h->staging_bytes >= bytes)
        return CNTKQ_OK;
    if (h->staging != nullptr)
    {
        HIP_TRY(hipStreamSynchronize(work_stream(h)), "hipStreamSynchronize failed");
        HIP_TRY(hipStreamSynchronize(h->fetch), "hipStreamSynchronize failed");
        HIP_TRY(hipStreamSynchronize(h->assign), "hipStreamSynchronize failed");
        HIP_TRY(hipFree(h->staging), "hipFree failed");
        h->staging = nullptr;
        h->staging_bytes = 0;
        h->fetch_pending = false;
        h->staging_read_pending = false;
    }
    void* p = nullptr;
    HIP_TRY(hipMalloc(&p, bytes), "hipMalloc of the packed staging buffer failed");
    h->staging = static_cast<char*>(p);
    h->staging_bytes = bytes;
    return CNTKQ_OK;
}

// Whether work issued on `s` is being recorded into a graph instead of executed.
bool stream_capturing(hipStream_t s)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess)
    {
        (void) hipGetLastError();
        return false;
    }
    return st == hipStreamCaptureStatusActive;
}

// True when `t` was built for exactly this item list and parameters.
bool table_matches(const BatchTable& t, const void* items, size_t items_bytes, const size_t (&params)[3])
{
    if (t.key.size() != items_bytes + sizeof params)
        return false;
    return std::memcmp(t.key.data(), params, sizeof params) == 0 && std::memcmp(t.key.data() + sizeof params, items, items_bytes) == 0;
}

// Makes `t` writable with room for `bytes`: waits for the kernels that still read it, grows the buffers.
int table_begin_rebuild(BatchTable& t, size_t bytes)
{
    t.key.clear();
    if (t.event == nullptr)
        HIP_TRY(hipEventCreateWithFlags(&t.event, hipEventDisableTiming), "hipEventCreateWithFlags failed");
    if (t.captured)
    {
        t.retired.emplace_back(t.host, t.dev);
        t.host = t.dev = nullptr;
        t.capacity = 0;
        t.captured = false;
    }
    if (t.in_flight)
    {
        HIP_TRY(hipEventSynchronize(t.event), "hipEventSynchronize failed");
        t.in_flight = false;
    }
    if (bytes > t.capacity)
    {
        if (t.host != nullptr)
            HIP_TRY(hipHostFree(t.host), "hipHostFree failed");
        if (t.dev != nullptr)
            HIP_TRY(hipFree(t.dev), "hipFree failed");
        t.host = t.dev = nullptr;
        t.capacity = 0;
        const size_t cap = (bytes * 2 + 4095) & ~(size_t) 4095;
        void* p = nullptr;
        HIP_TRY(hipHostMalloc(&p, cap, hipHostMallocDefault), "hipHostMalloc of the batch table failed");
        t.host = static_cast<char*>(p);
        HIP_TRY(hipMalloc(&p, cap), "hipMalloc of the batch table failed");
        t.dev = static_cast<char*>(p);
        t.capacity = cap;
    }
    return CNTKQ_OK;
}

void table_set_key(BatchTable& t, const void* items, size_t items_bytes, const size_t (&params)[3])
{
    t.key.resize(items_bytes + sizeof params);
    std::memcpy(t.key.data(), params, sizeof params);
    std::memcpy(t.key.data() + sizeof params, items, items_bytes);
}

void table_destroy(BatchTable& t)
{
    if (t.event != nullptr)
    {
        if (t.in_flight)
            (void) hipEventSynchronize(t.event);
        (void) hipEventDestroy(t.event);
    }
    if (t.host != nullptr)
        (void) hipHostFree(t.host);
    if (t.dev != nullptr)
        (void) hipFree(t.dev);
    for (auto& r : t.retired)
    {
        (void) hipHostFree(r.first);
        (void) hipFree(r.second);
    }
}

int sync_event(hipEvent_t ev) // SyncEvent (Source/Math/MatrixQuantizerGPU.cu:68-80)
{
    hipError_t rc = hipEventQuery(ev);
    if (rc == hipSuccess)
        return CNTKQ_OK;
    if (rc != hipErrorNotReady)
        return fail(CNTKQ_RUNTIME_ERROR, "hipEventQuery failed: %s (hip error %d)", hipGetErrorString(rc), (int) rc);
    HIP_TRY(hipEventSynchronize(ev), "hipEventSynchronize failed");
    return CNTKQ_OK;
}


// ---- the three asynchronous calls, written once for both element types ----------------------------------

template <typename E>
int quantize_async_impl(cntkq_quantizer* h, const E* in, const E* res_in, size_t rows, size_t cols, void* qbuf, size_t qbuf_bytes,
                        int qbuf_on_host, size_t nbits, E* res_out, int zero_threshold_for_1bit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_async: null handle");
    if (!Elem<E>::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides %zu (got %zu)", Elem<E>::kWordBits, nbits);
    if (rows >= (1ull << 31) || cols >= (1ull << 31))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_async: rows and cols must be below 2^31");
    const size_t need = Elem<E>::qcol_bytes(nbits, rows) * cols;
    if (qbuf_bytes != need)
        return fail(CNTKQ_LOGIC_ERROR,
                    "quantize: packed buffer of %zu bytes does not match %zu x %zu at %zu bits (%zu bytes)", qbuf_bytes,
                    rows, cols, nbits, need);
    h->quantize_included_fetch = false;
    if (rows == 0 || cols == 0)
        return CNTKQ_OK;
    if (in == nullptr || res_in == nullptr || res_out == nullptr || qbuf == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_async: null matrix pointer");
    if (!aligned_for<E>(in) || !aligned_for<E>(res_in) || !aligned_for<E>(res_out) || !aligned_for<E>(qbuf))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_async: pointers must be %zu-byte aligned", Elem<E>::kAlign);

    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    char* qdev = static_cast<char*>(qbuf);
    const bool capturing = stream_capturing(s);
    if (capturing && qbuf_on_host)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_async: a host-resident packed matrix needs copies on other streams and cannot "
                                            "be recorded into a graph");
    if (qbuf_on_host)
    {
        int rc = ensure_staging(h, need);
        if (rc != CNTKQ_OK)
            return rc;
        // a copy out of the staging buffer issued earlier must have drained before it is overwritten
        if (h->fetch_pending)
            HIP_TRY(hipStreamWaitEvent(s, h->ev_fetch, 0), "hipStreamWaitEvent failed");
        qdev = h->staging;
    }

    LaunchEvents ev = take_events(h, h->ev_quantize);
    if (capturing)
        ev.stop = nullptr; // recorded, not executed: nothing to wait for
    hipError_t lrc = Elem<E>::quantize(s, ev, in, res_in, res_out, qdev, rows, cols, nbits, zero_threshold_for_1bit != 0, h->tune);
    if (lrc == hipErrorInvalidValue)
        return fail(CNTKQ_INVALID_ARGUMENT, "quantize: the forced kernel path does not support %zu x %zu at %zu bits", rows, cols, nbits);
    HIP_TRY(lrc, "quantize kernel launch failed");
    h->last_quantize = ev.stop;

    if (qbuf_on_host)
    {
        HIP_TRY(hipStreamWaitEvent(h->fetch, ev.stop, 0), "hipStreamWaitEvent failed");
        HIP_TRY(hipMemcpyAsync(qbuf, qdev, need, hipMemcpyDeviceToHost, h->fetch), "hipMemcpyAsync failed");
        HIP_TRY(hipEventRecord(h->ev_fetch, h->fetch), "hipEventRecord failed");
        h->quantize_included_fetch = true;
        h->fetch_pending = true;
    }
    return CNTKQ_OK;
}

template <typename E>
int unquantize_async_impl(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, E* out, size_t rows, size_t cols,
                          size_t nbits, int add)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_async: null handle");
    if (!Elem<E>::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides %zu (got %zu)", Elem<E>::kWordBits, nbits);
    if (rows >= (1ull << 31) || cols >= (1ull << 31))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_async: rows and cols must be below 2^31");
    const size_t need = Elem<E>::qcol_bytes(nbits, rows) * cols;
    if (qbuf_bytes != need)
        return fail(CNTKQ_LOGIC_ERROR,
                    "unquantizestripe: dimension of patch to be unquantized does not match size of quantized data "
                    "(%zu bytes given, %zu x %zu at %zu bits needs %zu)", qbuf_bytes, rows, cols, nbits, need);
    if (qbuf_bytes == 0 || rows == 0 || cols == 0)
        return CNTKQ_OK; // empty buffer: empty matrix, nothing to do
    if (qbuf == nullptr || out == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_async: null matrix pointer");
    if (!aligned_for<E>(qbuf) || !aligned_for<E>(out))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_async: pointers must be %zu-byte aligned", Elem<E>::kAlign);

    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    const char* qdev = static_cast<const char*>(qbuf);
    if (qbuf_on_host && stream_capturing(s))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_async: a host-resident packed matrix needs copies on other streams and "
                                            "cannot be recorded into a graph");
    if (qbuf_on_host)
    {
        int rc = ensure_staging(h, need);
        if (rc != CNTKQ_OK)
            return rc;
        // the staging buffer may still be read by an earlier kernel or copied out by an earlier fetch
        HIP_TRY(hipEventRecord(h->ev_assign, s), "hipEventRecord failed");
        HIP_TRY(hipStreamWaitEvent(h->assign, h->ev_assign, 0), "hipStreamWaitEvent failed");
        if (h->fetch_pending)
            HIP_TRY(hipStreamWaitEvent(h->assign, h->ev_fetch, 0), "hipStreamWaitEvent failed");
        HIP_TRY(hipMemcpyAsync(h->staging, qbuf, need, hipMemcpyHostToDevice, h->assign), "hipMemcpyAsync failed");
        HIP_TRY(hipEventRecord(h->ev_assign, h->assign), "hipEventRecord failed");
        HIP_TRY(hipStreamWaitEvent(s, h->ev_assign, 0), "hipStreamWaitEvent failed");
        qdev = h->staging;
    }
    LaunchEvents ev = take_events(h, h->ev_unquantize);
    if (stream_capturing(s))
        ev.stop = nullptr; // recorded, not executed: nothing to wait for
    hipError_t lrc = Elem<E>::unquantize(s, ev, qdev, out, rows, cols, nbits, add != 0, h->tune);
    if (lrc == hipErrorInvalidValue)
        return fail(CNTKQ_INVALID_ARGUMENT, "unquantize: %zu x %zu at %zu bits is too large for one launch", rows, cols, nbits);
    HIP_TRY(lrc, "unquantize kernel launch failed");
    h->last_unquantize = ev.stop;
    return CNTKQ_OK;
}

template <typename E>
int stripe_reduce_async_impl(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner, size_t rows,
                             size_t stripe_cols, size_t nbits, E* stripe_res, void* q_out, E* agg_out, int zero_threshold_for_1bit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_async: null handle");
    if (!Elem<E>::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides %zu (got %zu)", Elem<E>::kWordBits, nbits);
    if (workers == 0 || workers > CNTKQ_MAX_WORKERS || owner >= workers || stripes == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_async: need 1 <= workers <= %d and owner < workers",
                    CNTKQ_MAX_WORKERS);
    if (rows >= (1ull << 31) || stripe_cols >= (1ull << 31))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_async: rows and cols must be below 2^31");
    if (rows == 0 || stripe_cols == 0)
        return CNTKQ_OK;
    if (rows > Elem<E>::stripe_max_rows(nbits))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_async: columns taller than %zu rows are not supported at %zu bits",
                    Elem<E>::stripe_max_rows(nbits), nbits);
    if (stripe_res == nullptr || q_out == nullptr || !aligned_for<E>(stripe_res) || !aligned_for<E>(q_out) || !aligned_for<E>(agg_out))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_async: null or misaligned matrix pointer");
    StripeSources src;
    std::memset(&src, 0, sizeof src);
    for (size_t w = 0; w < workers; ++w)
    {
        if (stripes[w] == nullptr || !aligned_for<E>(stripes[w]))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_async: stripe %zu is null or misaligned", w);
        src.q[w] = static_cast<const char*>(stripes[w]);
    }
    src.workers = (uint32_t) workers;
    src.owner = (uint32_t) owner;

    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    LaunchEvents ev = take_events(h, h->ev_stripe);
    if (stream_capturing(s))
        ev.stop = nullptr; // recorded, not executed: nothing to wait for
    hipError_t lrc = Elem<E>::stripe_reduce(s, ev, src, stripe_res, q_out, agg_out, rows, stripe_cols, nbits,
                                            zero_threshold_for_1bit != 0, h->tune);
    if (lrc == hipErrorInvalidValue)
        return fail(CNTKQ_INVALID_ARGUMENT, "stripe reduction: %zu rows with %zu workers at %zu bits does not fit the kernel", rows, workers,
                    nbits);
    HIP_TRY(lrc, "stripe reduction kernel launch failed");
    h->last_stripe = ev.stop;
    return CNTKQ_OK;
}

} // namespace

extern "C" {

const char* cntkq_last_error(void)
{
    return g_last_error;
}

size_t cntkq_qwords_per_col(size_t rows, size_t nbits)
{
    return valid_nbits(nbits) ? qwords_per_col(rows, nbits) : 0;
}

size_t cntkq_qcol_bytes(size_t nbits, size_t rows)
{
    return valid_nbits(nbits) ? qcol_bytes(nbits, rows) : 0;
}

size_t cntkq_qmatrix_bytes(size_t rows, size_t cols, size_t nbits)
{
    return valid_nbits(nbits) ? qcol_bytes(nbits, rows) * cols : 0;
}

size_t cntkq_qwords_per_col_f64(size_t rows, size_t nbits)
{
    return f64::valid_nbits(nbits) ? f64::qwords_per_col(rows, nbits) : 0;
}

size_t cntkq_qcol_bytes_f64(size_t nbits, size_t rows)
{
    return f64::valid_nbits(nbits) ? f64::qcol_bytes(nbits, rows) : 0;
}

size_t cntkq_qmatrix_bytes_f64(size_t rows, size_t cols, size_t nbits)
{
    return f64::valid_nbits(nbits) ? f64::qcol_bytes(nbits, rows) * cols : 0;
}

size_t cntkq_stripe_reduce_max_rows(size_t nbits)
{
    return valid_nbits(nbits) ? Elem<float>::stripe_max_rows(nbits) : 0;
}

size_t cntkq_stripe_reduce_max_rows_f64(size_t nbits)
{
    return cntkq::f64::valid_nbits(nbits) ? Elem<double>::stripe_max_rows(nbits) : 0;
}

int cntkq_stripe_range(size_t cols, size_t rank, size_t workers, size_t* start_col, size_t* num_cols)
{
    if (workers == 0 || rank >= workers || start_col == nullptr || num_cols == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_range: need 0 <= rank < workers and non-null outputs");
    const size_t per = cols / workers;
    const size_t extra = cols % workers;
    *start_col = per * rank + (extra < rank ? extra : rank);
    *num_cols = per + (rank < extra ? 1 : 0);
    return CNTKQ_OK;
}

int cntkq_create(int device_id, int use_dedicated_stream, cntkq_quantizer** out)
{
    if (out == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_create: out is null");
    *out = nullptr;
    if (device_id < 0)
        return fail(CNTKQ_RUNTIME_ERROR, "cntkq_create: device %d requested, but this library has no CPU quantizer", device_id);
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count), "hipGetDeviceCount failed");
    if (device_id >= count || device_id >= kMaxDevices)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_create: device %d out of range (%d devices)", device_id, count);

    DeviceGuard guard(device_id);
    cntkq_quantizer* h = new (std::nothrow) cntkq_quantizer();
    if (h == nullptr)
        return fail(CNTKQ_RUNTIME_ERROR, "cntkq_create: out of host memory");
    h->device = device_id;
    h->dedicated = use_dedicated_stream != 0;
    {
        std::lock_guard<std::mutex> lock(g_streams_mutex);
        DeviceStreams& ds = g_streams[device_id];
        // all streams keep the default priority
        if (h->dedicated && ds.compute == nullptr)
        {
            hipError_t rc = hipStreamCreateWithFlags(&ds.compute, hipStreamNonBlocking);
            if (rc != hipSuccess)
            {
                delete h;
                return fail(CNTKQ_RUNTIME_ERROR, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(rc));
            }
        }
        if (ds.fetch == nullptr)
        {
            hipError_t rc = hipStreamCreateWithFlags(&ds.fetch, hipStreamNonBlocking);
            if (rc == hipSuccess)
                rc = hipStreamCreateWithFlags(&ds.assign, hipStreamNonBlocking);
            if (rc != hipSuccess)
            {
                delete h;
                return fail(CNTKQ_RUNTIME_ERROR, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(rc));
            }
        }
        h->compute = ds.compute;
        h->fetch = ds.fetch;
        h->assign = ds.assign;
    }
    hipEvent_t* evs[] = {&h->ev_quantize, &h->ev_fetch, &h->ev_assign, &h->ev_unquantize, &h->ev_stripe, &h->ev_main};
    for (hipEvent_t* e : evs)
    {
        // no blocking-sync flag: waiting spins, as the reference found blocking events to stall for tens of ms
        hipError_t rc = hipEventCreateWithFlags(e, hipEventDisableTiming);
        if (rc != hipSuccess)
        {
            cntkq_destroy(h);
            return fail(CNTKQ_RUNTIME_ERROR, "hipEventCreateWithFlags failed: %s", hipGetErrorString(rc));
        }
    }
    *out = h;
    return CNTKQ_OK;
}

int cntkq_destroy(cntkq_quantizer* h)
{
    if (h == nullptr)
        return CNTKQ_OK;
    DeviceGuard guard(h->device);
    if (h->ev_quantize) (void) hipEventSynchronize(h->ev_quantize);
    if (h->ev_fetch) (void) hipEventSynchronize(h->ev_fetch);
    if (h->ev_assign) (void) hipEventSynchronize(h->ev_assign);
    if (h->ev_unquantize) (void) hipEventSynchronize(h->ev_unquantize);
    if (h->ev_stripe) (void) hipEventSynchronize(h->ev_stripe);
    if (h->staging != nullptr)
        (void) hipFree(h->staging);
    table_destroy(h->quantize_table);
    table_destroy(h->unquantize_table);
    table_destroy(h->stripe_table);
    table_destroy(h->quantize_table64);
    table_destroy(h->unquantize_table64);
    table_destroy(h->stripe_table64);
    hipEvent_t evs[] = {h->ev_quantize, h->ev_fetch, h->ev_assign, h->ev_unquantize, h->ev_stripe, h->ev_main};
    for (hipEvent_t e : evs)
        if (e != nullptr)
            (void) hipEventDestroy(e);
    delete h;
    return CNTKQ_OK;
}

int cntkq_device_id(const cntkq_quantizer* h)
{
    return h ? h->device : -1;
}

void* cntkq_stream(const cntkq_quantizer* h)
{
    return h ? static_cast<void*>(work_stream(h)) : nullptr;
}

int cntkq_set_main_stream(cntkq_quantizer* h, void* hip_stream)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_set_main_stream: null handle");
    h->main_stream = static_cast<hipStream_t>(hip_stream);
    return CNTKQ_OK;
}

int cntkq_sync_with_main_stream(cntkq_quantizer* h)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_sync_with_main_stream: null handle");
    if (!h->dedicated)
        return CNTKQ_OK; // the work stream is the main stream
    DeviceGuard guard(h->device);
    HIP_TRY(hipEventRecord(h->ev_main, h->main_stream), "hipEventRecord failed");
    HIP_TRY(hipStreamWaitEvent(h->compute, h->ev_main, 0), "hipStreamWaitEvent failed");
    return CNTKQ_OK;
}

int cntkq_stream_wait_event(cntkq_quantizer* h, void* hip_event)
{
    if (h == nullptr || hip_event == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stream_wait_event: null handle or event");
    DeviceGuard guard(h->device);
    HIP_TRY(hipStreamWaitEvent(work_stream(h), static_cast<hipEvent_t>(hip_event), 0), "hipStreamWaitEvent failed");
    return CNTKQ_OK;
}

int cntkq_quantize_async(cntkq_quantizer* h, const float* in, const float* res_in, size_t rows, size_t cols, void* qbuf,
                         size_t qbuf_bytes, int qbuf_on_host, size_t nbits, float* res_out, int zero_threshold_for_1bit)
{
    return quantize_async_impl<float>(h, in, res_in, rows, cols, qbuf, qbuf_bytes, qbuf_on_host, nbits, res_out, zero_threshold_for_1bit);
}

int cntkq_quantize_async_f64(cntkq_quantizer* h, const double* in, const double* res_in, size_t rows, size_t cols, void* qbuf,
                             size_t qbuf_bytes, int qbuf_on_host, size_t nbits, double* res_out, int zero_threshold_for_1bit)
{
    return quantize_async_impl<double>(h, in, res_in, rows, cols, qbuf, qbuf_bytes, qbuf_on_host, nbits, res_out, zero_threshold_for_1bit);
}

int cntkq_wait_quantize_done(cntkq_quantizer* h)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_wait_quantize_done: null handle");
    DeviceGuard guard(h->device);
    if (h->quantize_included_fetch)
    {
        int rc = sync_event(h->ev_fetch);
        if (rc == CNTKQ_OK)
            h->fetch_pending = false;
        return rc;
    }
    return h->last_quantize != nullptr ? sync_event(h->last_quantize) : CNTKQ_OK;
}

int cntkq_unquantize_async(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, float* out,
                           size_t rows, size_t cols, size_t nbits, int add)
{
    return unquantize_async_impl<float>(h, qbuf, qbuf_bytes, qbuf_on_host, out, rows, cols, nbits, add);
}

int cntkq_unquantize_async_f64(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, double* out,
                               size_t rows, size_t cols, size_t nbits, int add)
{
    return unquantize_async_impl<double>(h, qbuf, qbuf_bytes, qbuf_on_host, out, rows, cols, nbits, add);
}

int cntkq_wait_unquantize_done(cntkq_quantizer* h)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_wait_unquantize_done: null handle");
    DeviceGuard guard(h->device);
    return h->last_unquantize != nullptr ? sync_event(h->last_unquantize) : CNTKQ_OK;
}

int cntkq_quantize_batch_async(cntkq_quantizer* h, const cntkq_quantize_item* items, size_t count, size_t nbits,
                               int zero_threshold_for_1bit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async: null handle");
    if (!valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 32 (got %zu)", nbits);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr || count > 0xFFFFFF)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async: bad item list");
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_quantize_item& it = items[i];
        if (it.rows >= (1ull << 31) || it.cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.cols == 0)
            continue;
        if (it.in == nullptr || it.res_in == nullptr || it.res_out == nullptr || it.qbuf == nullptr || !aligned4(it.in) ||
            !aligned4(it.res_in) || !aligned4(it.res_out) || !aligned4(it.qbuf))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async: item %zu: null or misaligned pointer", i);
    }
    const bool zt = zero_threshold_for_1bit != 0;
    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    BatchTable& tb = h->quantize_table;
    const size_t params[3] = {count, nbits, (size_t) (zt ? 1 : 0)};
    const size_t items_bytes = count * sizeof(cntkq_quantize_item);

    const bool capturing = stream_capturing(s);
    if (capturing && !table_matches(tb, items, items_bytes, params))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async: the stream is being captured into a graph and this item list "
                                            "has not been seen: call once outside the capture first (the argument table is built and uploaded then)");
    if (!table_matches(tb, items, items_bytes, params))
    {
        // Every matrix is a member of one of two grid-wide launches (small / large LDS need), as a run of column
        // tiles or of single columns; only columns too tall for LDS get a launch of their own. Large matrices gain
        // from sharing a grid too: their workgroups fill the gaps the others leave.
        constexpr size_t kSmallLds = 20 * 1024;
        constexpr size_t kOwnLaunchElements = (size_t) 8 << 20;
        struct Plan
        {
            int kind; // -1 skip, 0 tiles in a batch, 1 columns in a batch, 2 own launch
            int cls;  // LDS class of a batch member
            size_t lds;
            uint64_t blocks;
            TileGeom t;
            ColGeom c;
        };
        std::vector<Plan> plans(count);
        size_t members[2] = {0, 0};
        for (size_t i = 0; i < count; ++i)
        {
            const cntkq_quantize_item& it = items[i];
            Plan& p = plans[i];
            std::memset(&p, 0, sizeof p);
            p.kind = -1;
            if (it.rows == 0 || it.cols == 0)
                continue;
            const int path = quantize_auto_path(it.in, it.res_in, it.res_out, it.qbuf, it.rows, nbits);
            if (path == kPathTile)
            {
                p.kind = 0;
                p.t = make_tile_geom(it.rows, it.cols, nbits, 0, -1, 0);
                p.lds = tile_lds_bytes(p.t, 0);
                p.blocks = (p.t.cols + p.t.cols_per_tile - 1) / p.t.cols_per_tile;
            }
            else if (path == kPathCol || (path == kPathReg && it.rows <= kTileMaxRows && it.rows * it.cols < kOwnLaunchElements))
            {
                // (a register-kernel matrix of modest size gives the same bytes as a member: a launch costs more than it gains)
                p.kind = 1;
                p.c = make_col_geom(it.rows, nbits, quantize_line_shift(it.in, it.res_in, it.res_out, it.rows));
                p.lds = colg_lds_bytes_rt(p.c, nbits);
                p.blocks = it.cols;
            }
            else
            {
                p.kind = 2;
                continue;
            }
            p.cls = p.lds <= kSmallLds ? 0 : 1;
            members[p.cls]++;
        }
        if (members[0] + members[1] == 1)
        {
            // a grid of its own is nothing to share: the plain launch picks the best kernel for the matrix
            for (size_t i = 0; i < count; ++i)
                if (plans[i].kind == 0 || plans[i].kind == 1)
                    plans[i].kind = 2;
            members[0] = members[1] = 0;
        }
        const size_t total = members[0] + members[1];
        const size_t entries_bytes = total * sizeof(QuantizeBatchEntry);
        int rc = table_begin_rebuild(tb, entries_bytes + (total + 2) * sizeof(uint32_t) + 64);
        if (rc != CNTKQ_OK)
            return rc;
        QuantizeBatchEntry* he = reinterpret_cast<QuantizeBatchEntry*>(tb.host);
        uint32_t* hb = reinterpret_cast<uint32_t*>(tb.host + entries_bytes);
        size_t e = 0, bpos = 0;
        tb.own.clear();
        for (int cls = 0; cls < 2; ++cls)
        {
            tb.first_entry[cls] = e;
            tb.first_begin[cls] = bpos;
            tb.lds[cls] = 0;
            uint64_t acc = 0;
            for (size_t i = 0; i < count; ++i)
            {
                const Plan& p = plans[i];
                if ((p.kind != 0 && p.kind != 1) || p.cls != cls)
                    continue;
                he[e].g = items[i].in;
                he[e].r_in = items[i].res_in;
                he[e].r_out = items[i].res_out;
                he[e].q = static_cast<char*>(items[i].qbuf);
                he[e].kind = (uint32_t) p.kind;
                he[e].pad = 0;
                he[e].t = p.t;
                he[e].c = p.c;
                hb[bpos++] = (uint32_t) acc;
                acc += p.blocks;
                if (acc > 0x7FFFFFFFull)
                    return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async: too many workgroups in one batch");
                if (p.lds > tb.lds[cls])
                    tb.lds[cls] = p.lds;
                e++;
            }
            if (members[cls] != 0)
                hb[bpos++] = (uint32_t) acc; // sentinel
            tb.members[cls] = members[cls];
            tb.blocks[cls] = (uint32_t) acc;
        }
        for (size_t i = 0; i < count; ++i)
            if (plans[i].kind == 2)
                tb.own.push_back(i);
        tb.entries_bytes = entries_bytes;
        if (total != 0)
            HIP_TRY(hipMemcpyAsync(tb.dev, tb.host, entries_bytes + bpos * sizeof(uint32_t), hipMemcpyHostToDevice, s),
                    "hipMemcpyAsync of the batch table failed");
        table_set_key(tb, items, items_bytes, params);
    }

    size_t launches_left = (tb.members[0] ? 1 : 0) + (tb.members[1] ? 1 : 0) + tb.own.size();
    if (launches_left == 0)
        return CNTKQ_OK;
    // the last kernel of the call carries the table's event: the kernels before it run on the same stream
    // (none when the call is recorded into a graph: there is nothing to wait for, and the table is frozen instead)
    hipEvent_t done = capturing ? nullptr : tb.event;
    if (capturing)
        tb.captured = true;
    for (int cls = 0; cls < 2; ++cls)
    {
        if (tb.members[cls] == 0)
            continue;
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 ? done : nullptr;
        const QuantizeBatchEntry* de = reinterpret_cast<const QuantizeBatchEntry*>(tb.dev) + tb.first_entry[cls];
        const uint32_t* db = reinterpret_cast<const uint32_t*>(tb.dev + tb.entries_bytes) + tb.first_begin[cls];
        HIP_TRY(launch_quantize_batch(s, ev, de, db, (uint32_t) tb.members[cls], tb.blocks[cls], tb.lds[cls], nbits, zt),
                "batched quantize kernel launch failed");
        tb.in_flight = tb.in_flight || !capturing;
    }
    LaunchTuning autotune;
    for (size_t i : tb.own)
    {
        const cntkq_quantize_item& it = items[i];
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 ? done : nullptr;
        HIP_TRY(launch_quantize(s, ev, it.in, it.res_in, it.res_out, it.qbuf, it.rows, it.cols, nbits, zt, autotune),
                "quantize kernel launch failed");
        tb.in_flight = tb.in_flight || !capturing;
    }
    h->last_quantize = done;
    h->quantize_included_fetch = false;
    return CNTKQ_OK;
}

int cntkq_unquantize_batch_async(cntkq_quantizer* h, const cntkq_unquantize_item* items, size_t count, size_t nbits, int add)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: null handle");
    if (!valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 32 (got %zu)", nbits);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr || count > 0xFFFFFF)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: bad item list");
    size_t n = 0;
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_unquantize_item& it = items[i];
        if (it.rows >= (1ull << 31) || it.cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.cols == 0)
            continue;
        if (it.qbuf == nullptr || it.out == nullptr || !aligned4(it.qbuf) || !aligned4(it.out))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: item %zu: null or misaligned pointer", i);
        n++;
    }
    if (n == 0)
        return CNTKQ_OK;
    if (n == 1)
    {
        for (size_t i = 0; i < count; ++i)
            if (items[i].rows != 0 && items[i].cols != 0)
                return cntkq_unquantize_async(h, items[i].qbuf, qcol_bytes(nbits, items[i].rows) * items[i].cols, 0, items[i].out,
                                              items[i].rows, items[i].cols, nbits, add);
    }
    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    BatchTable& tb = h->unquantize_table;
    const size_t params[3] = {count, nbits, 0};
    const size_t items_bytes = count * sizeof(cntkq_unquantize_item);
    const bool capturing = stream_capturing(s);
    if (capturing && !table_matches(tb, items, items_bytes, params))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: the stream is being captured into a graph and this item "
                                            "list has not been seen: call once outside the capture first");
    if (!table_matches(tb, items, items_bytes, params))
    {
        const size_t entries_bytes = n * sizeof(UnquantizeBatchEntry);
        int rc = table_begin_rebuild(tb, entries_bytes + (n + 1) * sizeof(uint32_t) + 64);
        if (rc != CNTKQ_OK)
            return rc;
        UnquantizeBatchEntry* he = reinterpret_cast<UnquantizeBatchEntry*>(tb.host);
        uint32_t* hb = reinterpret_cast<uint32_t*>(tb.host + entries_bytes);
        tb.lds[0] = 0;
        LaunchTuning autotune;
        uint64_t blocks = 0;
        size_t e = 0;
        for (size_t i = 0; i < count; ++i)
        {
            const cntkq_unquantize_item& it = items[i];
            if (it.rows == 0 || it.cols == 0)
                continue;
            const UnquantizePlan p = plan_unquantize(it.qbuf, it.out, it.rows, it.cols, nbits, autotune);
            if (!p.ok)
                return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: item %zu is too large", i);
            he[e].q = static_cast<const char*>(it.qbuf);
            he[e].out = it.out;
            he[e].kind = p.kind;
            he[e].pad = 0;
            he[e].qw = p.qw;
            he[e].seg = p.seg;
            he[e].rowg = p.rowg;
            he[e].tile = p.tile;
            if (p.lds > tb.lds[0])
                tb.lds[0] = p.lds;
            hb[e] = (uint32_t) blocks;
            blocks += p.blocks;
            if (blocks > 0x7FFFFFFFull)
                return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async: too much work in one batch");
            e++;
        }
        hb[e] = (uint32_t) blocks;
        tb.members[0] = n;
        tb.blocks[0] = (uint32_t) blocks;
        tb.entries_bytes = entries_bytes;
        HIP_TRY(hipMemcpyAsync(tb.dev, tb.host, entries_bytes + (n + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, s),
                "hipMemcpyAsync of the batch table failed");
        table_set_key(tb, items, items_bytes, params);
    }
    LaunchEvents ev;
    ev.stop = capturing ? nullptr : tb.event;
    HIP_TRY(launch_unquantize_batch(s, ev, reinterpret_cast<const UnquantizeBatchEntry*>(tb.dev),
                                    reinterpret_cast<const uint32_t*>(tb.dev + tb.entries_bytes), (uint32_t) tb.members[0], tb.blocks[0],
                                    nbits, add != 0, tb.lds[0]),
            "batched unquantize kernel launch failed");
    if (capturing)
        tb.captured = true;
    else
        tb.in_flight = true;
    h->last_unquantize = ev.stop;
    return CNTKQ_OK;
}

int cntkq_stripe_reduce_async(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner, size_t rows,
                              size_t stripe_cols, size_t nbits, float* stripe_res, void* q_out, float* agg_out,
                              int zero_threshold_for_1bit)
{
    return stripe_reduce_async_impl<float>(h, stripes, workers, owner, rows, stripe_cols, nbits, stripe_res, q_out, agg_out,
                                           zero_threshold_for_1bit);
}

int cntkq_stripe_reduce_async_f64(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner, size_t rows,
                                  size_t stripe_cols, size_t nbits, double* stripe_res, void* q_out, double* agg_out,
                                  int zero_threshold_for_1bit)
{
    return stripe_reduce_async_impl<double>(h, stripes, workers, owner, rows, stripe_cols, nbits, stripe_res, q_out, agg_out,
                                            zero_threshold_for_1bit);
}

int cntkq_stripe_reduce_batch_async(cntkq_quantizer* h, const cntkq_stripe_reduce_item* items, size_t count, size_t workers,
                                    size_t owner, size_t nbits, int zero_threshold_for_1bit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: null handle");
    if (!valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 32 (got %zu)", nbits);
    if (workers == 0 || workers > CNTKQ_MAX_WORKERS || owner >= workers)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: need 1 <= workers <= %d and owner < workers",
                    CNTKQ_MAX_WORKERS);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr || count > 0xFFFFFF)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: bad item list");
    size_t n = 0, only = 0, tall = 0;
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_stripe_reduce_item& it = items[i];
        if (it.rows >= (1ull << 31) || it.stripe_cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.stripe_cols == 0)
            continue;
        if (it.rows > stripe_reduce_max_rows(nbits))
            return fail(CNTKQ_INVALID_ARGUMENT,
                        "cntkq_stripe_reduce_batch_async: item %zu: columns taller than %zu rows are not supported at %zu bits", i,
                        stripe_reduce_max_rows(nbits), nbits);
        if (it.stripes == nullptr || it.stripe_res == nullptr || it.q_out == nullptr || !aligned4(it.stripe_res) || !aligned4(it.q_out) ||
            !aligned4(it.agg_out))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: item %zu: null or misaligned pointer", i);
        for (size_t w = 0; w < workers; ++w)
            if (it.stripes[w] == nullptr || !aligned4(it.stripes[w]))
                return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: item %zu: stripe %zu is null or misaligned", i, w);
        if (it.rows > kTileMaxRows)
        {
            tall++; // a launch of its own, below
            continue;
        }
        only = i;
        n++;
    }
    // tall stripes (1024 threads per column, registers) do not fit the shared grid: each is a plain call on the same stream
    for (size_t i = 0; i < count && tall != 0; ++i)
    {
        const cntkq_stripe_reduce_item& it = items[i];
        if (it.rows <= kTileMaxRows || it.stripe_cols == 0)
            continue;
        const int rc = cntkq_stripe_reduce_async(h, it.stripes, workers, owner, it.rows, it.stripe_cols, nbits, it.stripe_res, it.q_out,
                                                 it.agg_out, zero_threshold_for_1bit);
        if (rc != CNTKQ_OK)
            return rc;
    }
    if (n == 0)
        return CNTKQ_OK;
    if (n == 1) // a grid of its own is nothing to share: the plain call picks the best kernel for the stripe
        return cntkq_stripe_reduce_async(h, items[only].stripes, workers, owner, items[only].rows, items[only].stripe_cols, nbits,
                                         items[only].stripe_res, items[only].q_out, items[only].agg_out, zero_threshold_for_1bit);
    const bool zt = zero_threshold_for_1bit != 0;
    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    BatchTable& tb = h->stripe_table;

    // the key is the item list with the workers' stripe pointers written out
    const size_t params[3] = {count, nbits | (workers << 8) | (owner << 16), (size_t) (zt ? 1 : 0)};
    std::vector<size_t> flat;
    flat.reserve(count * (5 + workers));
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_stripe_reduce_item& it = items[i];
        flat.push_back(reinterpret_cast<size_t>(it.stripe_res));
        flat.push_back(reinterpret_cast<size_t>(it.q_out));
        flat.push_back(reinterpret_cast<size_t>(it.agg_out));
        flat.push_back(it.rows);
        flat.push_back(it.stripe_cols);
        if (it.rows != 0 && it.stripe_cols != 0)
            for (size_t w = 0; w < workers; ++w)
                flat.push_back(reinterpret_cast<size_t>(it.stripes[w]));
    }
    const size_t flat_bytes = flat.size() * sizeof(size_t);

    const bool capturing = stream_capturing(s);
    if (capturing && !table_matches(tb, flat.data(), flat_bytes, params))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: the stream is being captured into a graph and this item "
                                            "list has not been seen: call once outside the capture first");
    if (!table_matches(tb, flat.data(), flat_bytes, params))
    {
        constexpr size_t kSmallLds = 20 * 1024;
        const size_t entries_bytes = n * sizeof(StripeBatchEntry);
        int rc = table_begin_rebuild(tb, entries_bytes + (n + 2) * sizeof(uint32_t) + 64);
        if (rc != CNTKQ_OK)
            return rc;
        StripeBatchEntry* he = reinterpret_cast<StripeBatchEntry*>(tb.host);
        uint32_t* hb = reinterpret_cast<uint32_t*>(tb.host + entries_bytes);
        size_t e = 0, bpos = 0;
        for (int cls = 0; cls < 2; ++cls)
        {
            tb.first_entry[cls] = e;
            tb.first_begin[cls] = bpos;
            tb.lds[cls] = 0;
            tb.members[cls] = 0;
            uint64_t acc = 0;
            for (size_t i = 0; i < count; ++i)
            {
                const cntkq_stripe_reduce_item& it = items[i];
                if (it.rows == 0 || it.stripe_cols == 0 || it.rows > kTileMaxRows)
                    continue;
                // the kernel family the plain call would take, so that both give the same bytes
                const bool col = stripe_auto_col(it.rows);
                StripeBatchEntry en;
                std::memset(&en, 0, sizeof en);
                size_t lds, blocks;
                if (col)
                {
                    en.kind = 1;
                    en.c = make_col_geom(it.rows, nbits, !columns_start_on_lines(it.stripe_res, it.rows));
                    lds = colg_lds_bytes_rt(en.c, nbits) + 2 * workers * sizeof(float);
                    blocks = it.stripe_cols;
                }
                else
                {
                    en.kind = 0;
                    en.t = make_tile_geom(it.rows, it.stripe_cols, nbits, 0, -1, 0);
                    lds = tile_lds_bytes(en.t, (uint32_t) workers);
                    blocks = (en.t.cols + en.t.cols_per_tile - 1) / en.t.cols_per_tile;
                }
                if ((lds <= kSmallLds ? 0 : 1) != cls)
                    continue;
                for (size_t w = 0; w < workers; ++w)
                    en.src.q[w] = static_cast<const char*>(it.stripes[w]);
                en.src.workers = (uint32_t) workers;
                en.src.owner = (uint32_t) owner;
                en.stripe_res = it.stripe_res;
                en.q_out = static_cast<char*>(it.q_out);
                en.agg_out = it.agg_out;
                he[e] = en;
                hb[bpos++] = (uint32_t) acc;
                acc += blocks;
                if (acc > 0x7FFFFFFFull)
                    return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async: too many workgroups in one batch");
                if (lds > tb.lds[cls])
                    tb.lds[cls] = lds;
                tb.members[cls]++;
                e++;
            }
            if (tb.members[cls] != 0)
                hb[bpos++] = (uint32_t) acc; // sentinel
            tb.blocks[cls] = (uint32_t) acc;
        }
        tb.entries_bytes = entries_bytes;
        HIP_TRY(hipMemcpyAsync(tb.dev, tb.host, entries_bytes + bpos * sizeof(uint32_t), hipMemcpyHostToDevice, s),
                "hipMemcpyAsync of the batch table failed");
        table_set_key(tb, flat.data(), flat_bytes, params);
    }
    size_t launches_left = (tb.members[0] ? 1 : 0) + (tb.members[1] ? 1 : 0);
    for (int cls = 0; cls < 2; ++cls)
    {
        if (tb.members[cls] == 0)
            continue;
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 && !capturing ? tb.event : nullptr;
        const StripeBatchEntry* de = reinterpret_cast<const StripeBatchEntry*>(tb.dev) + tb.first_entry[cls];
        const uint32_t* db = reinterpret_cast<const uint32_t*>(tb.dev + tb.entries_bytes) + tb.first_begin[cls];
        HIP_TRY(launch_stripe_reduce_batch(s, ev, de, db, (uint32_t) tb.members[cls], tb.blocks[cls], tb.lds[cls], nbits, zt),
                "batched stripe reduction kernel launch failed");
        if (capturing)
            tb.captured = true;
        else
            tb.in_flight = true;
    }
    h->last_stripe = capturing ? nullptr : tb.event;
    return CNTKQ_OK;
}

int cntkq_wait_stripe_reduce_done(cntkq_quantizer* h)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_wait_stripe_reduce_done: null handle");
    DeviceGuard guard(h->device);
    return h->last_stripe != nullptr ? sync_event(h->last_stripe) : CNTKQ_OK;
}

// ---- the batched calls on doubles ----------------------------------------------------------------------------------
//
// Same construction as the float calls: members of the quantize and stripe-reduction grids are runs of column tiles
// (every double matrix the tile kernel serves; the register / tall kernels' matrices get launches of their own), members
// of the unquantize grid keep their decoder. Two LDS classes per call, tables cached per handle, frozen once captured.

namespace {

bool aligned8(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 7u) == 0;
}

constexpr size_t kSmallLds64 = 20 * 1024;

} // namespace

int cntkq_quantize_batch_async_f64(cntkq_quantizer* h, const cntkq_quantize_item_f64* items, size_t count, size_t nbits,
                                   int zero_threshold_for_1bit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async_f64: null handle");
    if (!f64::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 64 (got %zu)", nbits);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr || count > 0xFFFFFF)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async_f64: bad item list");
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_quantize_item_f64& it = items[i];
        if (it.rows >= (1ull << 31) || it.cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async_f64: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.cols == 0)
            continue;
        if (it.in == nullptr || it.res_in == nullptr || it.res_out == nullptr || it.qbuf == nullptr || !aligned8(it.in) ||
            !aligned8(it.res_in) || !aligned8(it.res_out) || !aligned8(it.qbuf))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async_f64: item %zu: null or misaligned pointer", i);
    }
    const bool zt = zero_threshold_for_1bit != 0;
    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    BatchTable& tb = h->quantize_table64;
    const size_t params[3] = {count, nbits, (size_t) (zt ? 1 : 0)};
    const size_t items_bytes = count * sizeof(cntkq_quantize_item_f64);
    const bool capturing = stream_capturing(s);
    if (capturing && !table_matches(tb, items, items_bytes, params))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async_f64: the stream is being captured into a graph and this item "
                                            "list has not been seen: call once outside the capture first");
    LaunchTuning autotune;
    if (!table_matches(tb, items, items_bytes, params))
    {
        struct Plan
        {
            int cls; // -1 skip, 0 / 1 member of that LDS class, 2 own launch
            size_t lds;
            uint64_t blocks;
            f64::TileGeom t;
        };
        std::vector<Plan> plans(count);
        size_t members[2] = {0, 0};
        for (size_t i = 0; i < count; ++i)
        {
            const cntkq_quantize_item_f64& it = items[i];
            Plan& p = plans[i];
            std::memset(&p, 0, sizeof p);
            p.cls = -1;
            if (it.rows == 0 || it.cols == 0)
                continue;
            p.cls = 2;
            if (f64::quantize_auto_path(it.in, it.res_in, it.res_out, it.rows, nbits) != kPathTile)
                continue;
            p.t = f64::make_tile_geom(it.rows, it.cols, nbits, 0);
            p.lds = f64::tile_lds_bytes(p.t, 0);
            if (p.lds > f64::kMaxLdsBytes)
                continue;
            p.blocks = (p.t.cols + p.t.cols_per_tile - 1) / p.t.cols_per_tile;
            p.cls = p.lds <= kSmallLds64 ? 0 : 1;
            members[p.cls]++;
        }
        if (members[0] + members[1] == 1)
        {
            for (size_t i = 0; i < count; ++i)
                if (plans[i].cls == 0 || plans[i].cls == 1)
                    plans[i].cls = 2;
            members[0] = members[1] = 0;
        }
        const size_t total = members[0] + members[1];
        const size_t entries_bytes = total * sizeof(f64::QuantizeBatchEntry64);
        int rc = table_begin_rebuild(tb, entries_bytes + (total + 2) * sizeof(uint32_t) + 64);
        if (rc != CNTKQ_OK)
            return rc;
        f64::QuantizeBatchEntry64* he = reinterpret_cast<f64::QuantizeBatchEntry64*>(tb.host);
        uint32_t* hb = reinterpret_cast<uint32_t*>(tb.host + entries_bytes);
        size_t e = 0, bpos = 0;
        tb.own.clear();
        for (int cls = 0; cls < 2; ++cls)
        {
            tb.first_entry[cls] = e;
            tb.first_begin[cls] = bpos;
            tb.lds[cls] = 0;
            uint64_t acc = 0;
            for (size_t i = 0; i < count; ++i)
            {
                const Plan& p = plans[i];
                if (p.cls != cls)
                    continue;
                he[e].g = items[i].in;
                he[e].r_in = items[i].res_in;
                he[e].r_out = items[i].res_out;
                he[e].q = static_cast<char*>(items[i].qbuf);
                he[e].t = p.t;
                hb[bpos++] = (uint32_t) acc;
                acc += p.blocks;
                if (acc > 0x7FFFFFFFull)
                    return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_async_f64: too many workgroups in one batch");
                if (p.lds > tb.lds[cls])
                    tb.lds[cls] = p.lds;
                e++;
            }
            if (members[cls] != 0)
                hb[bpos++] = (uint32_t) acc; // sentinel
            tb.members[cls] = members[cls];
            tb.blocks[cls] = (uint32_t) acc;
        }
        for (size_t i = 0; i < count; ++i)
            if (plans[i].cls == 2)
                tb.own.push_back(i);
        tb.entries_bytes = entries_bytes;
        if (total != 0)
            HIP_TRY(hipMemcpyAsync(tb.dev, tb.host, entries_bytes + bpos * sizeof(uint32_t), hipMemcpyHostToDevice, s),
                    "hipMemcpyAsync of the batch table failed");
        table_set_key(tb, items, items_bytes, params);
    }
    size_t launches_left = (tb.members[0] ? 1 : 0) + (tb.members[1] ? 1 : 0) + tb.own.size();
    if (launches_left == 0)
        return CNTKQ_OK;
    hipEvent_t done = capturing ? nullptr : tb.event;
    if (capturing)
        tb.captured = true;
    for (int cls = 0; cls < 2; ++cls)
    {
        if (tb.members[cls] == 0)
            continue;
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 ? done : nullptr;
        const f64::QuantizeBatchEntry64* de = reinterpret_cast<const f64::QuantizeBatchEntry64*>(tb.dev) + tb.first_entry[cls];
        const uint32_t* db = reinterpret_cast<const uint32_t*>(tb.dev + tb.entries_bytes) + tb.first_begin[cls];
        HIP_TRY(f64::dispatch_nbits64<f64::QuantizeBatchLauncher64>(nbits, zt && nbits == 1, s, ev, de, db, (uint32_t) tb.members[cls],
                                                                     tb.blocks[cls], tb.lds[cls]),
                "batched quantize kernel launch failed");
        tb.in_flight = tb.in_flight || !capturing;
    }
    for (size_t i : tb.own)
    {
        const cntkq_quantize_item_f64& it = items[i];
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 ? done : nullptr;
        HIP_TRY(f64::launch_quantize(s, ev, it.in, it.res_in, it.res_out, it.qbuf, it.rows, it.cols, nbits, zt, autotune),
                "quantize kernel launch failed");
        tb.in_flight = tb.in_flight || !capturing;
    }
    h->last_quantize = done;
    h->quantize_included_fetch = false;
    return CNTKQ_OK;
}

int cntkq_unquantize_batch_async_f64(cntkq_quantizer* h, const cntkq_unquantize_item_f64* items, size_t count, size_t nbits, int add)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: null handle");
    if (!f64::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 64 (got %zu)", nbits);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr || count > 0xFFFFFF)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: bad item list");
    size_t n = 0;
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_unquantize_item_f64& it = items[i];
        if (it.rows >= (1ull << 31) || it.cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.cols == 0)
            continue;
        if (it.qbuf == nullptr || it.out == nullptr || !aligned8(it.qbuf) || !aligned8(it.out))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: item %zu: null or misaligned pointer", i);
        n++;
    }
    if (n == 0)
        return CNTKQ_OK;
    if (n == 1)
    {
        for (size_t i = 0; i < count; ++i)
            if (items[i].rows != 0 && items[i].cols != 0)
                return cntkq_unquantize_async_f64(h, items[i].qbuf, f64::qcol_bytes(nbits, items[i].rows) * items[i].cols, 0, items[i].out,
                                                  items[i].rows, items[i].cols, nbits, add);
    }
    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    BatchTable& tb = h->unquantize_table64;
    const size_t params[3] = {count, nbits, 0};
    const size_t items_bytes = count * sizeof(cntkq_unquantize_item_f64);
    const bool capturing = stream_capturing(s);
    if (capturing && !table_matches(tb, items, items_bytes, params))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: the stream is being captured into a graph and this item "
                                            "list has not been seen: call once outside the capture first");
    if (!table_matches(tb, items, items_bytes, params))
    {
        const size_t entries_bytes = n * sizeof(f64::UnquantizeBatchEntry64);
        int rc = table_begin_rebuild(tb, entries_bytes + (n + 1) * sizeof(uint32_t) + 64);
        if (rc != CNTKQ_OK)
            return rc;
        f64::UnquantizeBatchEntry64* he = reinterpret_cast<f64::UnquantizeBatchEntry64*>(tb.host);
        uint32_t* hb = reinterpret_cast<uint32_t*>(tb.host + entries_bytes);
        tb.lds[0] = 0;
        LaunchTuning autotune;
        uint64_t blocks = 0;
        size_t e = 0;
        for (size_t i = 0; i < count; ++i)
        {
            const cntkq_unquantize_item_f64& it = items[i];
            if (it.rows == 0 || it.cols == 0)
                continue;
            const f64::UnquantizePlan64 p = f64::plan_unquantize(it.out, it.rows, it.cols, nbits, autotune);
            if (!p.ok)
                return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: item %zu is too large", i);
            he[e].q = static_cast<const char*>(it.qbuf);
            he[e].out = it.out;
            he[e].kind = p.kind;
            he[e].pad = 0;
            he[e].qw = p.qw;
            he[e].rowg = p.rowg;
            he[e].tile = p.tile;
            if (p.lds > tb.lds[0])
                tb.lds[0] = p.lds;
            hb[e] = (uint32_t) blocks;
            blocks += p.blocks;
            if (blocks > 0x7FFFFFFFull)
                return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_unquantize_batch_async_f64: too much work in one batch");
            e++;
        }
        hb[e] = (uint32_t) blocks;
        tb.members[0] = n;
        tb.blocks[0] = (uint32_t) blocks;
        tb.entries_bytes = entries_bytes;
        HIP_TRY(hipMemcpyAsync(tb.dev, tb.host, entries_bytes + (n + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, s),
                "hipMemcpyAsync of the batch table failed");
        table_set_key(tb, items, items_bytes, params);
    }
    LaunchEvents ev;
    ev.stop = capturing ? nullptr : tb.event;
    HIP_TRY(f64::launch_unquantize_batch(s, ev, reinterpret_cast<const f64::UnquantizeBatchEntry64*>(tb.dev),
                                         reinterpret_cast<const uint32_t*>(tb.dev + tb.entries_bytes), (uint32_t) tb.members[0], tb.blocks[0],
                                         nbits, add != 0, tb.lds[0]),
            "batched unquantize kernel launch failed");
    if (capturing)
        tb.captured = true;
    else
        tb.in_flight = true;
    h->last_unquantize = ev.stop;
    return CNTKQ_OK;
}

int cntkq_stripe_reduce_batch_async_f64(cntkq_quantizer* h, const cntkq_stripe_reduce_item_f64* items, size_t count, size_t workers,
                                        size_t owner, size_t nbits, int zero_threshold_for_1bit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: null handle");
    if (!f64::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 64 (got %zu)", nbits);
    if (workers == 0 || workers > CNTKQ_MAX_WORKERS || owner >= workers)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: need 1 <= workers <= %d and owner < workers",
                    CNTKQ_MAX_WORKERS);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr || count > 0xFFFFFF)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: bad item list");
    size_t n = 0, only = 0;
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_stripe_reduce_item_f64& it = items[i];
        if (it.rows >= (1ull << 31) || it.stripe_cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.stripe_cols == 0)
            continue;
        if (it.rows > f64::kTileMaxRows)
            return fail(CNTKQ_INVALID_ARGUMENT,
                        "cntkq_stripe_reduce_batch_async_f64: item %zu: columns taller than %zu rows are not supported", i,
                        (size_t) f64::kTileMaxRows);
        if (it.stripes == nullptr || it.stripe_res == nullptr || it.q_out == nullptr || !aligned8(it.stripe_res) || !aligned8(it.q_out) ||
            !aligned8(it.agg_out))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: item %zu: null or misaligned pointer", i);
        for (size_t w = 0; w < workers; ++w)
            if (it.stripes[w] == nullptr || !aligned8(it.stripes[w]))
                return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: item %zu: stripe %zu is null or misaligned", i, w);
        only = i;
        n++;
    }
    if (n == 0)
        return CNTKQ_OK;
    if (n == 1)
        return cntkq_stripe_reduce_async_f64(h, items[only].stripes, workers, owner, items[only].rows, items[only].stripe_cols, nbits,
                                             items[only].stripe_res, items[only].q_out, items[only].agg_out, zero_threshold_for_1bit);
    const bool zt = zero_threshold_for_1bit != 0;
    DeviceGuard guard(h->device);
    hipStream_t s = work_stream(h);
    BatchTable& tb = h->stripe_table64;
    const size_t params[3] = {count, nbits | (workers << 8) | (owner << 16), (size_t) (zt ? 1 : 0)};
    std::vector<size_t> flat;
    flat.reserve(count * (5 + workers));
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_stripe_reduce_item_f64& it = items[i];
        flat.push_back(reinterpret_cast<size_t>(it.stripe_res));
        flat.push_back(reinterpret_cast<size_t>(it.q_out));
        flat.push_back(reinterpret_cast<size_t>(it.agg_out));
        flat.push_back(it.rows);
        flat.push_back(it.stripe_cols);
        if (it.rows != 0 && it.stripe_cols != 0)
            for (size_t w = 0; w < workers; ++w)
                flat.push_back(reinterpret_cast<size_t>(it.stripes[w]));
    }
    const size_t flat_bytes = flat.size() * sizeof(size_t);
    const bool capturing = stream_capturing(s);
    if (capturing && !table_matches(tb, flat.data(), flat_bytes, params))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: the stream is being captured into a graph and this "
                                            "item list has not been seen: call once outside the capture first");
    if (!table_matches(tb, flat.data(), flat_bytes, params))
    {
        const size_t entries_bytes = n * sizeof(f64::StripeBatchEntry64);
        int rc = table_begin_rebuild(tb, entries_bytes + (n + 2) * sizeof(uint32_t) + 64);
        if (rc != CNTKQ_OK)
            return rc;
        f64::StripeBatchEntry64* he = reinterpret_cast<f64::StripeBatchEntry64*>(tb.host);
        uint32_t* hb = reinterpret_cast<uint32_t*>(tb.host + entries_bytes);
        size_t e = 0, bpos = 0;
        for (int cls = 0; cls < 2; ++cls)
        {
            tb.first_entry[cls] = e;
            tb.first_begin[cls] = bpos;
            tb.lds[cls] = 0;
            tb.members[cls] = 0;
            uint64_t acc = 0;
            for (size_t i = 0; i < count; ++i)
            {
                const cntkq_stripe_reduce_item_f64& it = items[i];
                if (it.rows == 0 || it.stripe_cols == 0)
                    continue;
                f64::StripeBatchEntry64 en;
                std::memset(&en, 0, sizeof en);
                en.t = f64::make_tile_geom(it.rows, it.stripe_cols, nbits, 0); // the plain call's geometry: same bytes
                const size_t lds = f64::tile_lds_bytes(en.t, (uint32_t) workers);
                if (lds > f64::kMaxLdsBytes)
                    return fail(CNTKQ_INVALID_ARGUMENT,
                                "cntkq_stripe_reduce_batch_async_f64: item %zu: %zu rows with %zu workers at %zu bits does not fit the kernel", i,
                                it.rows, workers, nbits);
                if ((lds <= kSmallLds64 ? 0 : 1) != cls)
                    continue;
                for (size_t w = 0; w < workers; ++w)
                    en.src.q[w] = static_cast<const char*>(it.stripes[w]);
                en.src.workers = (uint32_t) workers;
                en.src.owner = (uint32_t) owner;
                en.stripe_res = it.stripe_res;
                en.q_out = static_cast<char*>(it.q_out);
                en.agg_out = it.agg_out;
                he[e] = en;
                hb[bpos++] = (uint32_t) acc;
                acc += (en.t.cols + en.t.cols_per_tile - 1) / en.t.cols_per_tile;
                if (acc > 0x7FFFFFFFull)
                    return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_async_f64: too many workgroups in one batch");
                if (lds > tb.lds[cls])
                    tb.lds[cls] = lds;
                tb.members[cls]++;
                e++;
            }
            if (tb.members[cls] != 0)
                hb[bpos++] = (uint32_t) acc; // sentinel
            tb.blocks[cls] = (uint32_t) acc;
        }
        tb.entries_bytes = entries_bytes;
        HIP_TRY(hipMemcpyAsync(tb.dev, tb.host, entries_bytes + bpos * sizeof(uint32_t), hipMemcpyHostToDevice, s),
                "hipMemcpyAsync of the batch table failed");
        table_set_key(tb, flat.data(), flat_bytes, params);
    }
    size_t launches_left = (tb.members[0] ? 1 : 0) + (tb.members[1] ? 1 : 0);
    for (int cls = 0; cls < 2; ++cls)
    {
        if (tb.members[cls] == 0)
            continue;
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 && !capturing ? tb.event : nullptr;
        const f64::StripeBatchEntry64* de = reinterpret_cast<const f64::StripeBatchEntry64*>(tb.dev) + tb.first_entry[cls];
        const uint32_t* db = reinterpret_cast<const uint32_t*>(tb.dev + tb.entries_bytes) + tb.first_begin[cls];
        HIP_TRY(f64::dispatch_nbits64<f64::StripeBatchLauncher64>(nbits, zt && nbits == 1, s, ev, de, db, (uint32_t) tb.members[cls],
                                                                   tb.blocks[cls], tb.lds[cls]),
                "batched stripe reduction kernel launch failed");
        if (capturing)
            tb.captured = true;
        else
            tb.in_flight = true;
    }
    h->last_stripe = capturing ? nullptr : tb.event;
    return CNTKQ_OK;
}

// ---- hooks for tests and tuning runs (not part of the public header) --------------------------------

int cntkq_debug_set_tuning(cntkq_quantizer* h, int quantize_path, unsigned tile_gs, unsigned unq_slots, int unq_mode,
                           int tile_stage)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_debug_set_tuning: null handle");
    if (quantize_path < kPathAuto || quantize_path > kPathRegScalar)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_debug_set_tuning: unknown quantize path %d", quantize_path);
    if (tile_gs != 0 && (tile_gs < 8 || tile_gs > kTileThreads || (tile_gs & (tile_gs - 1)) != 0))
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_debug_set_tuning: tile_gs must be a power of two in [8, 256]");
    h->tune.quantize_path = quantize_path;
    h->tune.tile_gs = tile_gs;
    h->tune.unq_slots = unq_slots;
    h->tune.unq_mode = unq_mode;
    h->tune.tile_stage = tile_stage;
    return CNTKQ_OK;
}

int cntkq_debug_attach_events(cntkq_quantizer* h, void* start_event, void* stop_event)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_debug_attach_events: null handle");
    h->attach_start = static_cast<hipEvent_t>(start_event);
    h->attach_stop = static_cast<hipEvent_t>(stop_event);
    return CNTKQ_OK;
}

} // extern "C"
