// Host side of the C ABI shared by the two source files of the library (quantizer_api.hip: float matrices and everything
// that is independent of the element type; quantizer_api_f64.hip: double matrices): error text, process-wide streams,
// the handle, the cached argument tables, and the asynchronous calls written once as templates on the element type.
// The two files are compiled separately (their kernels share nothing), which halves the build time.
// Replaces the host side of the reference's GPU quantizer (Source/Math/MatrixQuantizerGPU.cu:83-341).
#pragma once

#include "../../include/cntk_amd_quantizer.h"
#include "quantizer_internal.h"
#include "quantizer_launch.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

namespace cntkq_api {

using namespace cntkq;

inline thread_local char g_last_error[1024] = "";

inline int fail(int code, const char* fmt, ...)
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
inline DeviceStreams g_streams[kMaxDevices];
inline std::mutex g_streams_mutex;

// the fixed device array of cntkq_quantize_batch_noalloc (defined in quantizer_api.hip) and the handle's mirror of it
constexpr size_t kNoAllocScratchBytes = 32 * 1024;

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

inline bool aligned4(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 3u) == 0;
}

// What differs between the two instantiations of the boundary (MatrixQuantizerImpl<float> / <double>).
template <typename E>
struct Elem;

template <typename E>
bool aligned_for(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & (Elem<E>::kAlign - 1)) == 0;
}


} // namespace cntkq_api

struct BatchTable
{
    std::vector<char> key;   // the item list and parameters the table was built for
    char* host = nullptr;    // pinned
    char* dev = nullptr;
    size_t capacity = 0;
    hipEvent_t event = nullptr; // set when the last kernel that reads the table has finished
    bool in_flight = false;
    // The upload is an asynchronous copy on the stream of the call that built the table. A later call may run on another
    // stream (the caller changed the handle's main stream): it is ordered after the upload, and after the kernels of
    // the other stream that still read the table, by table_before_launch.
    hipEvent_t upload_event = nullptr;
    hipStream_t upload_stream = nullptr;
    bool upload_known_done = true;
    hipStream_t last_stream = nullptr; // stream of the last launch that read the table
    // A launch that reads the table was recorded into a graph (stream capture): the graph may be replayed at any time
    // from then on, so the buffers are never written again; a rebuild retires them (freed with the handle) and takes
    // fresh ones.
    bool captured = false;
    std::vector<std::pair<char*, char*>> retired;
    // launch parameters of the two LDS classes and the matrices that get a launch of their own
    size_t members[2] = {0, 0};
    uint32_t blocks[2] = {0, 0};
    size_t lds[2] = {0, 0};
    bool wide[2] = {false, false}; // a member of the class needs the kernel variant compiled for more registers
    size_t first_entry[2] = {0, 0};
    size_t first_begin[2] = {0, 0};
    size_t entries_bytes = 0;
    std::vector<size_t> own;
};

// Host-side state of cntkq_quantize_batch_noalloc: everything the call needs besides the device array, at fixed size,
// so that the call itself touches no allocator (host or device).
struct NoAllocState
{
    static constexpr size_t kMaxItems = CNTKQ_NOALLOC_MAX_ITEMS;
    static constexpr size_t kTableWords = cntkq_api::kNoAllocScratchBytes / sizeof(uint32_t);
    // the table as uploaded: entries of the two LDS classes, then the first-workgroup lists (with sentinels)
    alignas(16) uint32_t table[kTableWords];
    size_t table_words = 0;
    // launch parameters
    size_t members[2] = {0, 0};
    uint32_t blocks[2] = {0, 0};
    size_t lds[2] = {0, 0};
    bool wide[2] = {false, false}; // a member of the class needs the kernel variant compiled for more registers
    size_t first_entry[2] = {0, 0};
    size_t first_begin[2] = {0, 0};
    size_t entries_bytes = 0;
    size_t own[kMaxItems];
    size_t own_count = 0;
    // what the table was built for, and the upload of it that the device array last received from this handle
    cntkq_quantize_item key_items[kMaxItems];
    size_t key_count = 0, key_nbits = 0, key_zt = 0;
    bool key_valid = false;
    uint64_t uploaded_generation = 0;
    hipStream_t uploaded_stream = nullptr; // later launches on another stream would not be ordered after that upload
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
    cntkq::LaunchTuning tune;
    bool force_sync = false; // the host waits after every step of a call (the reference's m_forceSync, for time measurements)
    cntkq::StripScratchOwner strip_scratch; // partial sums and launch count of the strip kernels (tune.strip points here)
    struct NoAllocState* noalloc = nullptr; // fixed-size host state of cntkq_quantize_batch_noalloc (created with the handle)
};

namespace cntkq_api {

inline hipStream_t work_stream(const cntkq_quantizer* h)
{
    return h->dedicated ? h->compute : h->main_stream;
}

// Completion is signalled by the kernel dispatch itself (no separate event record in the stream).
inline LaunchEvents take_events(cntkq_quantizer* h, hipEvent_t own)
{
    LaunchEvents ev;
    ev.start = h->attach_start;
    ev.stop = h->attach_stop != nullptr ? h->attach_stop : own;
    h->attach_start = nullptr;
    h->attach_stop = nullptr;
    return ev;
}

// The same for a call of several launches (the gradient-set calls): the first launch starts the one event, the last ends
// the other. Nothing is attached to launches that are only recorded into a graph.
struct AttachedEvents
{
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};
inline AttachedEvents take_attached(cntkq_quantizer* h, bool capturing)
{
    AttachedEvents a;
    if (!capturing)
    {
        a.start = h->attach_start;
        a.stop = h->attach_stop;
    }
    h->attach_start = nullptr;
    h->attach_stop = nullptr;
    return a;
}

// Temp device buffer for a host-resident packed matrix (GetTempGPUQuantizedMatrix,
// Source/Math/MatrixQuantizerGPU.cu:158-179). Grows only; waits for everything that may still use the old one.
inline int ensure_staging(cntkq_quantizer* h, size_t bytes)
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
inline bool stream_capturing(hipStream_t s)
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
inline bool table_matches(const BatchTable& t, const void* items, size_t items_bytes, const size_t (&params)[3])
{
    if (t.key.size() != items_bytes + sizeof params)
        return false;
    return std::memcmp(t.key.data(), params, sizeof params) == 0 && std::memcmp(t.key.data() + sizeof params, items, items_bytes) == 0;
}

// Makes `t` writable with room for `bytes`: waits for the kernels that still read it, grows the buffers.
inline int table_begin_rebuild(BatchTable& t, size_t bytes)
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
    if (!t.upload_known_done)
    {
        // the copy out of the pinned host table may still be running (a table built and never read, or read on another stream)
        HIP_TRY(hipEventSynchronize(t.upload_event), "hipEventSynchronize failed");
        t.upload_known_done = true;
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

// After the upload of a freshly built table has been issued on `s`.
inline int table_uploaded(BatchTable& t, hipStream_t s)
{
    if (t.upload_event == nullptr)
        HIP_TRY(hipEventCreateWithFlags(&t.upload_event, hipEventDisableTiming), "hipEventCreateWithFlags failed");
    HIP_TRY(hipEventRecord(t.upload_event, s), "hipEventRecord failed");
    t.upload_stream = s;
    t.upload_known_done = false;
    t.last_stream = s;
    return CNTKQ_OK;
}

// Before the launches of a call that reads `t` on stream `s`. The same stream as the upload and the last reader: nothing
// to do (stream order). Another stream: the host waits once for the upload (a few microseconds, and legal while `s` is
// being captured, since the event belongs to no capture), and `s` is made to wait for the last reader on the other
// stream, so that the event of this call's last kernel again covers every reader.
inline int table_before_launch(BatchTable& t, hipStream_t s, bool capturing)
{
    if (!t.upload_known_done && s != t.upload_stream)
    {
        HIP_TRY(hipEventSynchronize(t.upload_event), "hipEventSynchronize failed");
        t.upload_known_done = true;
    }
    if (!capturing)
    {
        if (t.in_flight && t.last_stream != s)
            HIP_TRY(hipStreamWaitEvent(s, t.event, 0), "hipStreamWaitEvent failed");
        t.last_stream = s;
    }
    return CNTKQ_OK;
}

// A launch of a batched call failed after earlier ones of the same call were issued on `s`: the table's event is
// recorded behind them, so that a rebuild and the Wait call still cover the work that was issued.
inline hipEvent_t table_partial_failure(BatchTable& t, hipStream_t s, bool issued, bool capturing)
{
    if (!issued || capturing || t.event == nullptr)
        return nullptr;
    if (hipEventRecord(t.event, s) != hipSuccess)
    {
        (void) hipGetLastError();
        return nullptr;
    }
    t.in_flight = true;
    return t.event;
}

inline void table_set_key(BatchTable& t, const void* items, size_t items_bytes, const size_t (&params)[3])
{
    t.key.resize(items_bytes + sizeof params);
    std::memcpy(t.key.data(), params, sizeof params);
    std::memcpy(t.key.data() + sizeof params, items, items_bytes);
}

inline void table_destroy(BatchTable& t)
{
    if (t.event != nullptr)
    {
        if (t.in_flight)
            (void) hipEventSynchronize(t.event);
        (void) hipEventDestroy(t.event);
    }
    if (t.upload_event != nullptr)
    {
        (void) hipEventSynchronize(t.upload_event);
        (void) hipEventDestroy(t.upload_event);
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

// After a wait: a strip kernel whose workgroups gave up waiting for one another has raised the error word (launches
// replayed from a graph included, so the word is looked at whenever it exists).
inline int check_strip_error(cntkq_quantizer* h)
{
    cntkq::StripScratchOwner& o = h->strip_scratch;
    if (o.error_host == nullptr)
        return CNTKQ_OK;
    if (*static_cast<volatile uint32_t*>(o.error_host) != 0u)
    {
        *o.error_host = 0u;
        // how many columns: the buffer's count only ever goes up, so the difference to what was seen last is this call's
        // (a launch replayed on a retired buffer counted there: then the figure is a lower bound)
        uint32_t now = o.abandoned_seen;
        // (copied on one of the handle's own streams: the legacy default stream stays out of it)
        if (o.dev != nullptr &&
            (hipMemcpyAsync(&now, o.dev + offsetof(cntkq::StripHeader, abandoned), sizeof now, hipMemcpyDeviceToHost, h->fetch) != hipSuccess ||
             hipStreamSynchronize(h->fetch) != hipSuccess))
            (void) hipGetLastError();
        const uint32_t columns = now - o.abandoned_seen;
        o.abandoned_seen = now;
        return fail(CNTKQ_RUNTIME_ERROR,
                    "quantize: the workgroups of %s%u column(s) gave up waiting for each other's partial sums; those columns were left as "
                    "they were (no header, no codes, residual not updated) and the result of the call is invalid",
                    columns == 0 ? "at least " : "", columns == 0 ? 1u : columns);
    }
    return CNTKQ_OK;
}

inline int sync_event(hipEvent_t ev) // SyncEvent (Source/Math/MatrixQuantizerGPU.cu:68-80)
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

    // serialised mode (Source/Math/MatrixQuantizerGPU.cu:237-240, 118-122, 137-141): the device is idle before the kernel
    // starts, and the host waits for the kernel and for the copy
    const bool force_sync = h->force_sync && !capturing;
    if (force_sync)
        HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize failed");
    LaunchEvents ev = take_events(h, h->ev_quantize);
    if (capturing)
        ev.stop = nullptr; // recorded, not executed: nothing to wait for
    hipError_t lrc = Elem<E>::quantize(s, ev, in, res_in, res_out, qdev, rows, cols, nbits, zero_threshold_for_1bit != 0, h->tune);
    if (lrc == hipErrorInvalidValue)
        return fail(CNTKQ_INVALID_ARGUMENT, "quantize: the forced kernel path does not support %zu x %zu at %zu bits", rows, cols, nbits);
    HIP_TRY(lrc, "quantize kernel launch failed");
    h->last_quantize = ev.stop;
    if (force_sync)
        HIP_TRY(hipStreamSynchronize(s), "hipStreamSynchronize failed");

    if (qbuf_on_host)
    {
        HIP_TRY(hipStreamWaitEvent(h->fetch, ev.stop, 0), "hipStreamWaitEvent failed");
        HIP_TRY(hipMemcpyAsync(qbuf, qdev, need, hipMemcpyDeviceToHost, h->fetch), "hipMemcpyAsync failed");
        HIP_TRY(hipEventRecord(h->ev_fetch, h->fetch), "hipEventRecord failed");
        h->quantize_included_fetch = true;
        h->fetch_pending = true;
        if (force_sync)
            HIP_TRY(hipStreamSynchronize(h->fetch), "hipStreamSynchronize failed");
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
        if (h->force_sync) // Source/Math/MatrixQuantizerGPU.cu:318-321
            HIP_TRY(hipStreamSynchronize(h->assign), "hipStreamSynchronize failed");
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
    // serialised mode: the host waits for the kernel before the call returns (RecordQuantizeCompleteEvent,
    // Source/Math/MatrixQuantizerGPU.cu:118-122, called at the end of UnquantizeAsync, :338)
    if (h->force_sync && !stream_capturing(s))
        HIP_TRY(hipStreamSynchronize(s), "hipStreamSynchronize failed");
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
    {
        // taller stripes run on strips where the device holds a column's strips at once (cntkq_stripe_reduce_takes)
        DeviceGuard guard(h->device);
        if (!Elem<E>::stripe_takes_strips(work_stream(h), rows, stripe_cols, nbits, zero_threshold_for_1bit != 0, h->tune))
            return fail(CNTKQ_INVALID_ARGUMENT,
                        "cntkq_stripe_reduce_async: columns of %zu rows are not supported at %zu bits (up to %zu rows, and on strips the "
                        "heights that cntkq_stripe_reduce_takes reports)",
                        rows, nbits, Elem<E>::stripe_max_rows(nbits));
    }
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

#include "quantizer_api_batch.inc"

} // namespace cntkq_api
