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

// ---- the argument table of cntkq_quantize_batch_noalloc ----------------------------------------------------------
//
// That entry point must not allocate, so its table (entries, then the first workgroup of every member) lives in this
// fixed array in the library's device image: every GPU the library runs on holds its own copy, at its own address,
// until the process ends. Host code never uses the array's name as an address (in host code it is only a stand-in for
// the symbol): scratch_for_device() asks the runtime for the copy's address on the current device, once per device, and
// everything -- kernel arguments included -- goes through that pointer.
constexpr size_t kNoAllocScratchBytes = 32 * 1024;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

struct DeviceScratch
{
    unsigned char* ptr = nullptr;        // address of `scratch` on this device
    const void* writer = nullptr;        // the handle whose table the array holds (host-side bookkeeping)
    uint64_t generation = 0;             // bumped on every upload
};
DeviceScratch g_scratch[kMaxDevices];

// Call with `device` current. Returns hipSuccess once the device's address of `scratch` is known.
hipError_t scratch_for_device(int device)
{
    std::lock_guard<std::mutex> lock(g_streams_mutex);
    if (g_scratch[device].ptr != nullptr)
        return hipSuccess;
    void* p = nullptr;
    hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (rc != hipSuccess)
        return rc;
    if (p == nullptr)
        return hipErrorInvalidSymbol;
    g_scratch[device].ptr = static_cast<unsigned char*>(p);
    return hipSuccess;
}

// The table travels to the device as kernel arguments, 2 KB per launch: no copy engine, no staging memory.
constexpr uint32_t kChunkWords = 512;
struct TableChunk
{
    uint32_t w[kChunkWords];
};

__global__ __launch_bounds__(256) void table_store_kernel(TableChunk chunk, uint32_t* dst, uint32_t words)
{
    for (uint32_t i = threadIdx.x; i < words; i += 256)
        dst[i] = chunk.w[i];
}

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
    static size_t stripe_max_rows(size_t nbits) { return cntkq::f64::stripe_reduce_max_rows(nbits); }
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

// Host-side state of cntkq_quantize_batch_noalloc: everything the call needs besides the device array, at fixed size,
// so that the call itself touches no allocator (host or device).
struct NoAllocState
{
    static constexpr size_t kMaxItems = CNTKQ_NOALLOC_MAX_ITEMS;
    static constexpr size_t kTableWords = kNoAllocScratchBytes / sizeof(uint32_t);
    // the table as uploaded: entries of the two LDS classes, then the first-workgroup lists (with sentinels)
    alignas(16) uint32_t table[kTableWords];
    size_t table_words = 0;
    // launch parameters
    size_t members[2] = {0, 0};
    uint32_t blocks[2] = {0, 0};
    size_t lds[2] = {0, 0};
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
    LaunchTuning tune;
    struct NoAllocState* noalloc = nullptr; // fixed-size host state of cntkq_quantize_batch_noalloc (created with the handle)
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

#include "quantizer_api_batch.inc"

// ---- the gradient-set quantize that allocates nothing -----------------------------------------------------------------
//
// Same planning, same kernels and hence the same bytes as quantize_batch_impl<float>; what differs is where the argument
// table lives (the fixed device array `scratch`, reached through the per-device pointer) and how it gets there (as kernel
// arguments of table_store_kernel). Nothing on this path calls an allocator: no hipMalloc / hipHostMalloc / hipFree, no
// host heap (the plan is built in the handle's NoAllocState), no copy that would need staging memory.
int quantize_batch_noalloc_impl(cntkq_quantizer* h, const cntkq_quantize_item* items, size_t count, size_t nbits, int zero_threshold_for_1bit)
{
    typedef BatchAbi<float> A;
    typedef QuantizeBatchEntry Entry;
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: null handle");
    if (!cntkq::valid_nbits(nbits))
        return fail(CNTKQ_LOGIC_ERROR, "Quantization: 'nbits' must be a power of two that divides 32 (got %zu)", nbits);
    if (count == 0)
        return CNTKQ_OK;
    if (items == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: bad item list");
    if (count > NoAllocState::kMaxItems)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: %zu items exceed the limit of %zu (CNTKQ_NOALLOC_MAX_ITEMS)", count,
                    NoAllocState::kMaxItems);
    for (size_t i = 0; i < count; ++i)
    {
        const cntkq_quantize_item& it = items[i];
        if (it.rows >= (1ull << 31) || it.cols >= (1ull << 31))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: item %zu: rows and cols must be below 2^31", i);
        if (it.rows == 0 || it.cols == 0)
            continue;
        if (it.in == nullptr || it.res_in == nullptr || it.res_out == nullptr || it.qbuf == nullptr || !aligned4(it.in) || !aligned4(it.res_in) ||
            !aligned4(it.res_out) || !aligned4(it.qbuf))
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: item %zu: null or misaligned pointer", i);
    }
    const bool zt = zero_threshold_for_1bit != 0;
    DeviceGuard guard(h->device);
    DeviceScratch& ds = g_scratch[h->device];
    if (ds.ptr == nullptr || h->noalloc == nullptr)
        return fail(CNTKQ_RUNTIME_ERROR, "cntkq_quantize_batch_noalloc: the device array was not set up when the handle was created");
    NoAllocState& st = *h->noalloc;
    hipStream_t s = work_stream(h);
    const bool capturing = stream_capturing(s);

    const bool same_list = st.key_valid && st.key_count == count && st.key_nbits == nbits && st.key_zt == (size_t) zt &&
                           std::memcmp(st.key_items, items, count * sizeof(cntkq_quantize_item)) == 0;
    if (!same_list)
    {
        st.key_valid = false;
        // plan: the class of every item (-1 skip, 0 / 1 member of that LDS class, 2 a launch of its own), kept in `own`
        // until the table is laid out
        Entry* he = reinterpret_cast<Entry*>(st.table);
        static_assert(sizeof(Entry) % sizeof(uint32_t) == 0 && alignof(Entry) <= 16, "table layout");
        static_assert(sizeof(Entry) == CNTKQ_NOALLOC_ENTRY_BYTES, "the public header states the size of a table entry");
        static_assert(CNTKQ_NOALLOC_MAX_ITEMS * (sizeof(Entry) + sizeof(uint32_t)) + 2 * sizeof(uint32_t) <= kNoAllocScratchBytes,
                      "a list of the largest permitted size fits the fixed array");
        // pass 1: count the members, so that the two classes can be laid out one after the other
        size_t members[2] = {0, 0};
        for (size_t i = 0; i < count; ++i)
        {
            const cntkq_quantize_item& it = items[i];
            if (it.rows == 0 || it.cols == 0)
                continue;
            Entry e;
            std::memset(&e, 0, sizeof e);
            size_t lds = 0;
            uint64_t blocks = 0;
            if (A::quantize_member(it, nbits, e, lds, blocks))
                members[lds <= kBatchSmallLds ? 0 : 1]++;
        }
        const bool single = members[0] + members[1] == 1; // a grid of its own is nothing to share: plain launch
        if (single)
            members[0] = members[1] = 0;
        const size_t total = members[0] + members[1];
        const size_t entries_bytes = total * sizeof(Entry);
        const size_t need = entries_bytes + (total + 2) * sizeof(uint32_t);
        if (need > kNoAllocScratchBytes)
            return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: the argument table of %zu matrices (%zu bytes) exceeds the fixed "
                                                "device array of %zu bytes", total, need, kNoAllocScratchBytes);
        uint32_t* hb = st.table + entries_bytes / sizeof(uint32_t);
        size_t e = 0, bpos = 0;
        st.own_count = 0;
        for (int cls = 0; cls < 2; ++cls)
        {
            st.first_entry[cls] = e;
            st.first_begin[cls] = bpos;
            st.lds[cls] = 0;
            uint64_t acc = 0;
            for (size_t i = 0; i < count && !single; ++i)
            {
                const cntkq_quantize_item& it = items[i];
                if (it.rows == 0 || it.cols == 0)
                    continue;
                Entry en;
                std::memset(&en, 0, sizeof en);
                size_t lds = 0;
                uint64_t blocks = 0;
                if (!A::quantize_member(it, nbits, en, lds, blocks) || (lds <= kBatchSmallLds ? 0 : 1) != cls)
                    continue;
                en.g = it.in;
                en.r_in = it.res_in;
                en.r_out = it.res_out;
                en.q = static_cast<char*>(it.qbuf);
                he[e++] = en;
                hb[bpos++] = (uint32_t) acc;
                acc += blocks;
                if (acc > 0x7FFFFFFFull)
                    return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_quantize_batch_noalloc: too many workgroups in one batch");
                if (lds > st.lds[cls])
                    st.lds[cls] = lds;
            }
            if (members[cls] != 0)
                hb[bpos++] = (uint32_t) acc; // sentinel
            st.members[cls] = members[cls];
            st.blocks[cls] = (uint32_t) acc;
        }
        for (size_t i = 0; i < count; ++i)
        {
            const cntkq_quantize_item& it = items[i];
            if (it.rows == 0 || it.cols == 0)
                continue;
            Entry en;
            size_t lds = 0;
            uint64_t blocks = 0;
            if (single || !A::quantize_member(it, nbits, en, lds, blocks))
                st.own[st.own_count++] = i;
        }
        st.entries_bytes = entries_bytes;
        st.table_words = total != 0 ? entries_bytes / sizeof(uint32_t) + bpos : 0;
        std::memcpy(st.key_items, items, count * sizeof(cntkq_quantize_item));
        st.key_count = count;
        st.key_nbits = nbits;
        st.key_zt = (size_t) zt;
        st.key_valid = true;
        st.uploaded_generation = 0; // whatever the device array holds, it is not this table
    }

    // The device array is shared by every handle on this GPU and keeps the last call's contents: upload unless this very
    // table is what it received last. (A recorded call always uploads: a replay must not depend on what ran before it.)
    bool upload = st.table_words != 0;
    {
        std::lock_guard<std::mutex> lock(g_streams_mutex);
        if (upload && !capturing && ds.writer == h && st.uploaded_generation != 0 && ds.generation == st.uploaded_generation &&
            st.uploaded_stream == s)
            upload = false;
        if (upload)
        {
            ds.writer = h;
            st.uploaded_generation = ++ds.generation;
            st.uploaded_stream = s;
        }
    }
    if (upload)
    {
        for (size_t w0 = 0; w0 < st.table_words; w0 += kChunkWords)
        {
            const uint32_t words = (uint32_t) (st.table_words - w0 < kChunkWords ? st.table_words - w0 : kChunkWords);
            TableChunk chunk;
            std::memcpy(chunk.w, st.table + w0, words * sizeof(uint32_t));
            hipLaunchKernelGGL(table_store_kernel, dim3(1), dim3(256), 0, s, chunk, reinterpret_cast<uint32_t*>(ds.ptr) + w0, words);
            HIP_TRY(hipGetLastError(), "table_store_kernel launch failed");
        }
    }

    size_t launches_left = (st.members[0] ? 1 : 0) + (st.members[1] ? 1 : 0) + st.own_count;
    if (launches_left == 0)
        return CNTKQ_OK;
    hipEvent_t done = capturing ? nullptr : h->ev_quantize;
    for (int cls = 0; cls < 2; ++cls)
    {
        if (st.members[cls] == 0)
            continue;
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 ? done : nullptr;
        const Entry* de = reinterpret_cast<const Entry*>(ds.ptr) + st.first_entry[cls];
        const uint32_t* db = reinterpret_cast<const uint32_t*>(ds.ptr + st.entries_bytes) + st.first_begin[cls];
        HIP_TRY(A::launch_quantize_members(s, ev, de, db, (uint32_t) st.members[cls], st.blocks[cls], st.lds[cls], nbits, zt),
                "batched quantize kernel launch failed");
    }
    for (size_t k = 0; k < st.own_count; ++k)
    {
        LaunchEvents ev;
        launches_left--;
        ev.stop = launches_left == 0 ? done : nullptr;
        HIP_TRY(A::launch_quantize_own(s, ev, items[st.own[k]], nbits, zt), "quantize kernel launch failed");
    }
    h->last_quantize = done;
    h->quantize_included_fetch = false;
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
    {
        // the no-allocation entry point's fixed state: the address of the device array on this GPU (looked up once per
        // device, with the device current) and the handle's host-side plan space
        hipError_t rc = scratch_for_device(device_id);
        if (rc != hipSuccess)
        {
            delete h;
            return fail(CNTKQ_RUNTIME_ERROR, "hipGetSymbolAddress of the fixed device array failed: %s (hip error %d)", hipGetErrorString(rc),
                        (int) rc);
        }
        h->noalloc = new (std::nothrow) NoAllocState();
        if (h->noalloc == nullptr)
        {
            delete h;
            return fail(CNTKQ_RUNTIME_ERROR, "cntkq_create: out of host memory");
        }
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
    {
        std::lock_guard<std::mutex> lock(g_streams_mutex);
        if (g_scratch[h->device].writer == h)
            g_scratch[h->device].writer = nullptr; // a later handle at the same address must upload again
    }
    delete h->noalloc;
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
    return quantize_batch_impl<float>(h, items, count, nbits, zero_threshold_for_1bit);
}

int cntkq_unquantize_batch_async(cntkq_quantizer* h, const cntkq_unquantize_item* items, size_t count, size_t nbits, int add)
{
    return unquantize_batch_impl<float>(h, items, count, nbits, add);
}

int cntkq_quantize_batch_noalloc(cntkq_quantizer* h, const cntkq_quantize_item* items, size_t count, size_t nbits,
                                 int zero_threshold_for_1bit)
{
    return quantize_batch_noalloc_impl(h, items, count, nbits, zero_threshold_for_1bit);
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
    return stripe_reduce_batch_impl<float>(h, items, count, workers, owner, nbits, zero_threshold_for_1bit);
}

int cntkq_wait_stripe_reduce_done(cntkq_quantizer* h)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_wait_stripe_reduce_done: null handle");
    DeviceGuard guard(h->device);
    return h->last_stripe != nullptr ? sync_event(h->last_stripe) : CNTKQ_OK;
}

// ---- the gradient-set calls on doubles (same implementation, see quantizer_api_batch.inc) ----------------------------

int cntkq_quantize_batch_async_f64(cntkq_quantizer* h, const cntkq_quantize_item_f64* items, size_t count, size_t nbits,
                                   int zero_threshold_for_1bit)
{
    return quantize_batch_impl<double>(h, items, count, nbits, zero_threshold_for_1bit);
}

int cntkq_unquantize_batch_async_f64(cntkq_quantizer* h, const cntkq_unquantize_item_f64* items, size_t count, size_t nbits, int add)
{
    return unquantize_batch_impl<double>(h, items, count, nbits, add);
}

int cntkq_stripe_reduce_batch_async_f64(cntkq_quantizer* h, const cntkq_stripe_reduce_item_f64* items, size_t count, size_t workers,
                                        size_t owner, size_t nbits, int zero_threshold_for_1bit)
{
    return stripe_reduce_batch_impl<double>(h, items, count, workers, owner, nbits, zero_threshold_for_1bit);
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
