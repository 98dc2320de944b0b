// C ABI of the MI355X gradient quantizer: handles, streams, events, argument checks; the calls on float matrices.
// Replaces the host side of the reference's GPU quantizer (Source/Math/MatrixQuantizerGPU.cu:83-341).
#include "quantizer_api_shared.h"

using namespace cntkq;
using namespace cntkq_api;

namespace cntkq_api {

template <>
struct Elem<float>
{
    static constexpr size_t kAlign = 4;
    static constexpr size_t kWordBits = 32;
    static size_t stripe_max_rows(size_t nbits) { return cntkq::stripe_reduce_max_rows(nbits); }
    static bool stripe_takes_strips(hipStream_t s, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
    {
        return cntkq::stripe_takes_strips(s, rows, cols, nbits, zt, tune);
    }
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
struct BatchAbi<float>
{
    typedef cntkq_quantize_item QItem;
    typedef cntkq_unquantize_item UItem;
    typedef cntkq_stripe_reduce_item SItem;
    typedef QuantizeBatchEntry QEntry;
    typedef UnquantizeBatchEntry UEntry;
    typedef StripeBatchEntry SEntry;
    static const char* suffix() { return ""; }
    static unsigned word_bits() { return 32; }
    static bool valid_nbits(size_t nbits) { return cntkq::valid_nbits(nbits); }
    static bool aligned(const void* p) { return aligned4(p); }
    static BatchTable& quantize_table(cntkq_quantizer* h) { return h->quantize_table; }
    static BatchTable& unquantize_table(cntkq_quantizer* h) { return h->unquantize_table; }
    static BatchTable& stripe_table(cntkq_quantizer* h) { return h->stripe_table; }

    // Fills the geometry of a member of the quantize grid; false: the matrix gets a launch of its own.
    static bool quantize_member(const QItem& it, size_t nbits, QEntry& e, size_t& lds, uint64_t& blocks)
    {
        const int path = quantize_auto_path(it.in, it.res_in, it.res_out, it.qbuf, it.rows, nbits);
        if (path == kPathTile)
        {
            e.kind = 0;
            e.t = make_tile_geom(it.rows, it.cols, nbits, 0, -1, 0);
            lds = tile_lds_bytes(e.t, 0);
            blocks = (e.t.cols + e.t.cols_per_tile - 1) / e.t.cols_per_tile;
            return true;
        }
        // (a register-kernel matrix of modest size gives the same bytes as a member: a launch costs more than it gains)
        if (path == kPathCol || (path == kPathReg && it.rows <= kTileMaxRows && it.rows * it.cols < kOwnLaunchElements &&
                                 reg_applicable(it.in, it.res_in, it.res_out, it.qbuf, it.rows, nbits)))
        {
            const bool line_shift = quantize_line_shift(it.in, it.res_in, it.res_out, it.rows);
            e.kind = 1;
            e.c = make_col_geom(it.rows, nbits, line_shift);
            lds = colg_lds_bytes_rt(e.c, nbits);
            blocks = it.cols;
            // a few tall columns (a bias vector) do not get a launch with more LDS to themselves: they stage the column in
            // the residual's memory and join the other members (same bytes)
            if (lds > kBatchSmallLds && it.cols <= kStagedInResidualMaxCols)
            {
                e.kind = 5;
                lds = ((nbits <= 2 ? e.c.nq : 0) + kColgRedSlots) * sizeof(float);
            }
            // 1 bit, 1024 / 2048 / 4096 rows, columns on 128-byte lines, 8-byte aligned records: the unrolled body (same bytes)
            if (!line_shift && col_unrolled(it.qbuf, it.rows, nbits))
            {
                e.kind = it.rows == 1024 ? 2 : (it.rows == 2048 ? 3 : 4);
                lds = it.rows == 1024 ? col_lds_bytes<1>() : (it.rows == 2048 ? col_lds_bytes<2>() : col_lds_bytes<4>());
            }
            else if (path == kPathReg && e.kind == 1)
            {
                // what the plain call runs for this matrix, where a thread holds at most 6 pieces (6144 rows): the column in
                // registers, with the slots dealt as the plain call deals them (same bytes as the LDS body either way)
                const RegGeom r = make_reg_geom(it.rows, nbits, kTileThreads, line_shift);
                const uint32_t per = (r.pieces + (r.line_shift ? 7u : 0u) + kTileThreads - 1) / kTileThreads;
                if (per <= 6)
                {
                    e.kind = per <= 3 ? 6 : 7;
                    e.r = r;
                    lds = reg_lds_bytes(r);
                }
            }
            return true;
        }
        return false;
    }
    static bool first_in_grid(const QEntry& e) { return e.kind == 5; }
    static hipError_t launch_quantize_members(hipStream_t s, LaunchEvents ev, const QEntry* de, const uint32_t* db, uint32_t members,
                                              uint32_t blocks, size_t lds, size_t nbits, bool zt)
    {
        return launch_quantize_batch(s, ev, de, db, members, blocks, lds, nbits, zt);
    }
    static hipError_t launch_quantize_own(cntkq_quantizer* h, hipStream_t s, LaunchEvents ev, const QItem& it, size_t nbits, bool zt)
    {
        LaunchTuning autotune;
        autotune.strip = &h->strip_scratch;
        autotune.strip_never_waits = h->tune.strip_never_waits;
        return launch_quantize(s, ev, it.in, it.res_in, it.res_out, it.qbuf, it.rows, it.cols, nbits, zt, autotune);
    }

    static int unquantize_one(cntkq_quantizer* h, const UItem& it, size_t nbits, int add)
    {
        return cntkq_unquantize_async(h, it.qbuf, qcol_bytes(nbits, it.rows) * it.cols, 0, it.out, it.rows, it.cols, nbits, add);
    }
    static bool unquantize_member(const UItem& it, size_t nbits, UEntry& e, size_t& lds, uint64_t& blocks)
    {
        LaunchTuning autotune;
        autotune.unq_member = true;
        const UnquantizePlan p = plan_unquantize(it.qbuf, it.out, it.rows, it.cols, nbits, autotune);
        if (!p.ok)
            return false;
        e.kind = p.kind;
        e.qw = p.qw;
        e.seg = p.seg;
        e.rowg = p.rowg;
        e.flat = p.flat;
        e.tile = p.tile;
        lds = p.lds;
        blocks = p.blocks;
        return true;
    }
    static hipError_t launch_unquantize_members(hipStream_t s, LaunchEvents ev, const UEntry* de, const uint32_t* db, uint32_t members,
                                                uint32_t blocks, size_t nbits, bool add, size_t lds)
    {
        return launch_unquantize_batch(s, ev, de, db, members, blocks, nbits, add, lds);
    }

    static size_t stripe_max_rows(size_t nbits) { return stripe_reduce_max_rows(nbits); }
    static bool stripe_takes_strips(cntkq_quantizer* h, size_t rows, size_t cols, size_t nbits, bool zt)
    {
        DeviceGuard guard(h->device);
        return cntkq::stripe_takes_strips(work_stream(h), rows, cols, nbits, zt, h->tune);
    }
    // taller stripes run 1024 threads per column, or on strips: a launch of their own
    // (so do stripes that the table-driven register kernel takes with more than six pieces per thread: the shared launch is
    // compiled for what its largest member needs)
    static bool stripe_is_member(const SItem& it, size_t workers, size_t nbits)
    {
        if (stripe_uses_reg(it.rows, it.stripe_res, nbits))
            return false;
        if (stripe_auto_col(it.rows, it.stripe_res) && stripe_looks_up(it.rows, nbits, workers))
            return stripe_lookup_per(it.rows, !columns_start_on_lines(it.stripe_res, it.rows)) <= 6;
        return true;
    }
    static int stripe_one(cntkq_quantizer* h, const SItem& it, size_t workers, size_t owner, size_t nbits, int zt)
    {
        return cntkq_stripe_reduce_async(h, it.stripes, workers, owner, it.rows, it.stripe_cols, nbits, it.stripe_res, it.q_out, it.agg_out, zt);
    }
    // the kernel family the plain call would take, so that both give the same bytes; false: does not fit the kernel
    static bool stripe_member(const SItem& it, size_t workers, size_t nbits, SEntry& e, size_t& lds, uint64_t& blocks)
    {
        if (stripe_auto_col(it.rows, it.stripe_res))
        {
            const bool line_shift = !columns_start_on_lines(it.stripe_res, it.rows);
            e.kind = 1;
            e.c = make_col_geom(it.rows, nbits, line_shift);
            lds = colg_lds_bytes_rt(e.c, nbits) + stripe_dec_bytes(nbits, workers);
            blocks = it.stripe_cols;
            // as launch_stripe_reduce chooses: the unrolled body where every packed stripe is 8-byte aligned
            bool aligned = (reinterpret_cast<uintptr_t>(it.q_out) & 7u) == 0;
            for (size_t w = 0; w < workers; ++w)
                aligned = aligned && (reinterpret_cast<uintptr_t>(it.stripes[w]) & 7u) == 0;
            if (!line_shift && aligned && it.rows <= 2048 && col_unrolled(it.q_out, it.rows, nbits))
            {
                e.kind = it.rows == 1024 ? 2 : 3;
                lds = (it.rows == 1024 ? col_lds_bytes<1>() : col_lds_bytes<2>()) + kStripeColExtraLds;
            }
            else if (stripe_looks_up(it.rows, nbits, workers))
            {
                // as launch_stripe_reduce chooses (stripe_is_member has left those with more than six pieces per thread out)
                e.r = make_reg_geom(it.rows, nbits, 256, line_shift);
                e.kind = stripe_lookup_per(it.rows, line_shift) <= 3 ? 4 : 5;
                lds = stripe_lut_lds_bytes(e.r);
            }
        }
        else
        {
            e.kind = 0;
            e.t = make_tile_geom(it.rows, it.stripe_cols, nbits, 0, -1, 0);
            lds = tile_lds_bytes(e.t, (uint32_t) workers);
            blocks = (e.t.cols + e.t.cols_per_tile - 1) / e.t.cols_per_tile;
        }
        return true;
    }
    // members that look their sums up need 76 registers where the others need 44: a launch without them keeps eight
    // wavefronts per SIMD
    static bool stripe_entry_wide(const SEntry& e) { return e.kind >= 4; }
    // he / hb: the host's copy of the entries and first workgroups that de / db hold on the device
    static hipError_t launch_stripe_members(hipStream_t s, LaunchEvents ev, const SEntry* de, const uint32_t* db, const SEntry* he,
                                            const uint32_t* hb, uint32_t members, uint32_t blocks, size_t lds, size_t nbits, bool zt, bool wide)
    {
        // a few stripes of one shape that all run the unrolled 1-bit column body with up to eight workers (the ranks of a
        // small cluster simulated on one GPU): described in the kernel's arguments instead of the table in device memory
        bool as_set = members <= kStripeSetMax && nbits == 1 && (he[0].kind == 2 || he[0].kind == 3) && he[0].src.workers <= kStripeSetMax;
        for (uint32_t i = 1; i < members && as_set; ++i)
            as_set = he[i].kind == he[0].kind && he[i].src.workers == he[0].src.workers;
        if (as_set)
        {
            StripeColSet set;
            std::memset(&set, 0, sizeof set);
            for (uint32_t i = 0; i <= kStripeSetMax; ++i)
                set.begin[i] = i <= members ? hb[i] : 0xFFFFFFFFu;
            for (uint32_t i = 0; i < members; ++i)
            {
                for (uint32_t w = 0; w < he[i].src.workers; ++w)
                    set.q[i][w] = he[i].src.q[w];
                set.stripe_res[i] = he[i].stripe_res;
                set.q_out[i] = he[i].q_out;
                set.agg_out[i] = he[i].agg_out;
                set.owner[i] = he[i].src.owner;
            }
            set.count = members;
            set.workers = he[0].src.workers;
            set.qcol = he[0].c.qcol;
            return family_col_stripe_set(zt && nbits == 1, he[0].kind == 2 ? 1 : 2, s, ev, set);
        }
        return launch_stripe_reduce_batch(s, ev, de, db, members, blocks, lds, nbits, zt, wide);
    }
};


} // namespace cntkq_api

namespace {

// ---- the argument table of cntkq_quantize_batch_noalloc ----------------------------------------------------------
//
// That entry point must not allocate, so its table (entries, then the first workgroup of every member) lives in this
// fixed array in the library's device image: every GPU the library runs on holds its own copy, at its own address,
// until the process ends. Host code never uses the array's name as an address (in host code it is only a stand-in for
// the symbol): scratch_for_device() asks the runtime for the copy's address on the current device, once per device, and
// everything -- kernel arguments included -- goes through that pointer.
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

struct DeviceScratch
{
    unsigned char* ptr = nullptr;        // address of `scratch` on this device
    const void* writer = nullptr;        // the handle whose table the array holds (host-side bookkeeping)
    uint64_t generation = 0;             // bumped on every upload
    // A call recorded into a graph (stream capture) writes the array whenever the graph is replayed, which no host-side
    // bookkeeping sees: once there is such a call on the device, every call uploads its table.
    bool recorded_call = false;
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
        if (it.qbuf_bytes != qcol_bytes(nbits, it.rows) * it.cols)
            return fail(CNTKQ_LOGIC_ERROR, "cntkq_quantize_batch_noalloc: item %zu: packed buffer of %zu bytes does not match %zu x %zu at %zu bits (%zu bytes)",
                        i, it.qbuf_bytes, it.rows, it.cols, nbits, qcol_bytes(nbits, it.rows) * it.cols);
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
    // table is what it received last. A recorded call always uploads (a replay must not depend on what ran before it) and
    // is never taken for an upload that has happened: nothing ran yet, and from then on replays rewrite the array at times
    // the host does not know of.
    bool upload = st.table_words != 0;
    {
        std::lock_guard<std::mutex> lock(g_streams_mutex);
        if (capturing)
            ds.recorded_call = true;
        if (upload && !capturing && !ds.recorded_call && ds.writer == h && st.uploaded_generation != 0 &&
            ds.generation == st.uploaded_generation && st.uploaded_stream == s)
            upload = false;
        if (upload)
        {
            ++ds.generation;
            ds.writer = capturing ? nullptr : h;
            st.uploaded_generation = capturing ? 0 : ds.generation;
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
        // (the strip kernels only where the handle's scratch buffer, made when the handle was created, holds the matrix
        // as it stands: this call allocates nothing. A taller or wider matrix runs the kernel that re-reads its columns,
        // whose sums are added in another order: its column bounds may differ from the batched call's in their last bits.)
        const cntkq_quantize_item& it = items[st.own[k]];
        LaunchTuning fixed;
        fixed.strip = h->strip_scratch.order_event != nullptr ? &h->strip_scratch : nullptr;
        fixed.strip_may_allocate = false;
        fixed.strip_never_waits = h->tune.strip_never_waits;
        HIP_TRY(launch_quantize(s, ev, it.in, it.res_in, it.res_out, it.qbuf, it.rows, it.cols, nbits, zt, fixed), "quantize kernel launch failed");
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




size_t cntkq_stripe_reduce_max_rows(size_t nbits)
{
    return valid_nbits(nbits) ? Elem<float>::stripe_max_rows(nbits) : 0;
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
    h->tune.strip = &h->strip_scratch;
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
    {
        // The strip kernels' scratch buffer at its starting size, so that a first call under graph capture (which cannot
        // allocate) finds it. A failure here is not one of the handle: the first call that needs the buffer tries again.
        // (cleared on one of the handle's own streams and waited for there: the legacy default stream stays out of it)
        StripScratch unused;
        if (strip_scratch_for(h->strip_scratch, h->fetch, 1, 2, strip_records<double>(), unused) != hipSuccess ||
            hipEventCreateWithFlags(&h->strip_scratch.order_event, hipEventDisableTiming) != hipSuccess)
            (void) hipGetLastError();
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
    if (h->strip_scratch.dev != nullptr)
        (void) hipFree(h->strip_scratch.dev);
    for (char* p : h->strip_scratch.retired)
        (void) hipFree(p);
    if (h->strip_scratch.error_host != nullptr)
        (void) hipHostFree(h->strip_scratch.error_host);
    if (h->strip_scratch.order_event != nullptr)
        (void) hipEventDestroy(h->strip_scratch.order_event);
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

int cntkq_set_force_sync(cntkq_quantizer* h, int force_sync)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_set_force_sync: null handle");
    h->force_sync = force_sync != 0;
    return CNTKQ_OK;
}

int cntkq_set_tall_columns_never_wait(cntkq_quantizer* h, int never_wait)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_set_tall_columns_never_wait: null handle");
    h->tune.strip_never_waits = never_wait != 0;
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
        // (the copy ran after the kernel: whatever the kernel reported is there by now)
        return rc != CNTKQ_OK ? rc : check_strip_error(h);
    }
    const int rc = h->last_quantize != nullptr ? sync_event(h->last_quantize) : CNTKQ_OK;
    return rc != CNTKQ_OK ? rc : check_strip_error(h);
}

int cntkq_unquantize_async(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, float* out,
                           size_t rows, size_t cols, size_t nbits, int add)
{
    return unquantize_async_impl<float>(h, qbuf, qbuf_bytes, qbuf_on_host, out, rows, cols, nbits, add);
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


int cntkq_stripe_reduce_batch_async(cntkq_quantizer* h, const cntkq_stripe_reduce_item* items, size_t count, size_t workers,
                                    size_t owner, size_t nbits, int zero_threshold_for_1bit)
{
    return stripe_reduce_batch_impl<float>(h, items, count, workers, owner, nbits, zero_threshold_for_1bit);
}

int cntkq_stripe_reduce_batch_owners_async(cntkq_quantizer* h, const cntkq_stripe_reduce_item* items, const size_t* owners, size_t count,
                                           size_t workers, size_t nbits, int zero_threshold_for_1bit)
{
    if (owners == nullptr && count != 0)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_owners_async: null owner list");
    return stripe_reduce_batch_impl<float>(h, items, count, workers, 0, nbits, zero_threshold_for_1bit, owners);
}

int cntkq_wait_stripe_reduce_done(cntkq_quantizer* h)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_wait_stripe_reduce_done: null handle");
    DeviceGuard guard(h->device);
    const int rc = h->last_stripe != nullptr ? sync_event(h->last_stripe) : CNTKQ_OK;
    // (a reduction on strips reports workgroups that gave up on each other like a quantize call on strips)
    return rc != CNTKQ_OK ? rc : check_strip_error(h);
}

int cntkq_stripe_reduce_takes(cntkq_quantizer* h, size_t rows, size_t stripe_cols, size_t nbits, int zero_threshold_for_1bit)
{
    if (h == nullptr || !valid_nbits(nbits) || rows == 0 || stripe_cols == 0 || rows >= (1ull << 31) || stripe_cols >= (1ull << 31))
        return 0;
    if (rows <= Elem<float>::stripe_max_rows(nbits))
        return 1;
    DeviceGuard guard(h->device);
    return cntkq::stripe_takes_strips(work_stream(h), rows, stripe_cols, nbits, zero_threshold_for_1bit != 0, h->tune) ? 1 : 0;
}




// ---- hooks for tests and tuning runs (not part of the public header) --------------------------------

int cntkq_debug_set_tuning(cntkq_quantizer* h, int quantize_path, unsigned tile_gs, unsigned unq_slots, int unq_mode,
                           int tile_stage)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_debug_set_tuning: null handle");
    if (quantize_path < kPathAuto || quantize_path > kPathStripPasses)
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

// How often a lane of a strip kernel polls for another workgroup's partial sum before it gives up (tests of the error path
// set it to zero: every kernel still runs to its end).
int cntkq_debug_set_strip_spin_limit(cntkq_quantizer* h, unsigned limit)
{
    if (h == nullptr)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_debug_set_strip_spin_limit: null handle");
    h->tune.strip_spin_limit = limit;
    return CNTKQ_OK;
}

unsigned cntkq_debug_strip_max_strips(cntkq_quantizer* h, size_t nbits, int zero_threshold_for_1bit)
{
    if (h == nullptr || !valid_nbits(nbits) || nbits >= 32)
        return 0;
    DeviceGuard guard(h->device);
    return strip_max_strips<float>(nbits, zero_threshold_for_1bit != 0 && nbits == 1);
}

unsigned cntkq_debug_strip_max_strips_f64(cntkq_quantizer* h, size_t nbits, int zero_threshold_for_1bit)
{
    if (h == nullptr || nbits == 0 || nbits >= 64 || (nbits & (nbits - 1)) != 0)
        return 0;
    DeviceGuard guard(h->device);
    return strip_max_strips<double>(nbits, zero_threshold_for_1bit != 0 && nbits == 1);
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
