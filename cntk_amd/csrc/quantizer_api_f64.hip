// C ABI of the MI355X gradient quantizer: the calls on double matrices (MatrixQuantizerImpl<double>, 64-bit QWords).
// Same handle, streams and waits as the float calls; see quantizer_api_shared.h.
#include "quantizer_api_shared.h"
#include "quantizer_launch_f64.h"

using namespace cntkq;
using namespace cntkq_api;

namespace cntkq_api {

template <>
struct Elem<double>
{
    static constexpr size_t kAlign = 8;
    static constexpr size_t kWordBits = 64;
    static size_t stripe_max_rows(size_t nbits) { return cntkq::f64::stripe_reduce_max_rows(nbits); }
    static bool stripe_takes_strips(hipStream_t s, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
    {
        return cntkq::f64::stripe_takes_strips(s, rows, cols, nbits, zt, tune);
    }
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

template <>
struct BatchAbi<double>
{
    typedef cntkq_quantize_item_f64 QItem;
    typedef cntkq_unquantize_item_f64 UItem;
    typedef cntkq_stripe_reduce_item_f64 SItem;
    typedef f64::QuantizeBatchEntry64 QEntry;
    typedef f64::UnquantizeBatchEntry64 UEntry;
    typedef f64::StripeBatchEntry64 SEntry;
    static const char* suffix() { return "_f64"; }
    static unsigned word_bits() { return 64; }
    static bool valid_nbits(size_t nbits) { return f64::valid_nbits(nbits); }
    static bool aligned(const void* p) { return aligned8(p); }
    static BatchTable& quantize_table(cntkq_quantizer* h) { return h->quantize_table64; }
    static BatchTable& unquantize_table(cntkq_quantizer* h) { return h->unquantize_table64; }
    static BatchTable& stripe_table(cntkq_quantizer* h) { return h->stripe_table64; }

    // members are runs of column tiles; the register and tall kernels' matrices get launches of their own, except small
    // matrices of the element-wise register kernel, which stay members and run the tile body (the same bytes)
    static bool quantize_member(const QItem& it, size_t nbits, QEntry& e, size_t& lds, uint64_t& blocks)
    {
        const int path = f64::quantize_auto_path(it.in, it.res_in, it.res_out, it.rows, nbits);
        if (path != kPathTile && !(path == kPathRegScalar && it.rows * it.cols < kOwnLaunchElements))
            return false;
        e.t = f64::make_tile_geom(it.rows, it.cols, nbits, 0);
        lds = f64::tile_lds_bytes(e.t, 0);
        if (lds > f64::kMaxLdsBytes)
            return false;
        blocks = (e.t.cols + e.t.cols_per_tile - 1) / e.t.cols_per_tile;
        return true;
    }
    static bool first_in_grid(const QEntry&) { return false; }
    static hipError_t launch_quantize_members(hipStream_t s, LaunchEvents ev, const QEntry* de, const uint32_t* db, uint32_t members,
                                              uint32_t blocks, size_t lds, size_t nbits, bool zt)
    {
        return f64::dispatch_nbits64<f64::QuantizeBatchLauncher64>(nbits, zt && nbits == 1, s, ev, de, db, members, blocks, lds);
    }
    static hipError_t launch_quantize_own(cntkq_quantizer* h, hipStream_t s, LaunchEvents ev, const QItem& it, size_t nbits, bool zt)
    {
        LaunchTuning autotune;
        autotune.strip = &h->strip_scratch;
        autotune.strip_never_waits = h->tune.strip_never_waits;
        return f64::launch_quantize(s, ev, it.in, it.res_in, it.res_out, it.qbuf, it.rows, it.cols, nbits, zt, autotune);
    }

    static int unquantize_one(cntkq_quantizer* h, const UItem& it, size_t nbits, int add)
    {
        return cntkq_unquantize_async_f64(h, it.qbuf, f64::qcol_bytes(nbits, it.rows) * it.cols, 0, it.out, it.rows, it.cols, nbits, add);
    }
    static bool unquantize_member(const UItem& it, size_t nbits, UEntry& e, size_t& lds, uint64_t& blocks)
    {
        LaunchTuning autotune;
        autotune.unq_member = true;
        const f64::UnquantizePlan64 p = f64::plan_unquantize(it.out, it.rows, it.cols, nbits, autotune);
        if (!p.ok)
            return false;
        e.kind = p.kind;
        e.qw = p.qw;
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
        return f64::launch_unquantize_batch(s, ev, de, db, members, blocks, nbits, add, lds);
    }

    static size_t stripe_max_rows(size_t nbits) { return f64::stripe_reduce_max_rows(nbits); }
    static bool stripe_takes_strips(cntkq_quantizer* h, size_t rows, size_t cols, size_t nbits, bool zt)
    {
        DeviceGuard guard(h->device);
        return f64::stripe_takes_strips(work_stream(h), rows, cols, nbits, zt, h->tune);
    }
    // stripes of the register kernel's heights run 1024 threads per column, taller ones on strips: a launch of their own
    static bool stripe_is_member(const SItem& it, size_t, size_t nbits)
    {
        return it.rows <= f64::stripe_reduce_max_rows(nbits) && !f64::stripe_uses_reg(it.rows, nbits);
    }
    static int stripe_one(cntkq_quantizer* h, const SItem& it, size_t workers, size_t owner, size_t nbits, int zt)
    {
        return cntkq_stripe_reduce_async_f64(h, it.stripes, workers, owner, it.rows, it.stripe_cols, nbits, it.stripe_res, it.q_out, it.agg_out,
                                             zt);
    }
    static bool stripe_member(const SItem& it, size_t workers, size_t nbits, SEntry& e, size_t& lds, uint64_t& blocks)
    {
        e.t = f64::make_tile_geom(it.rows, it.stripe_cols, nbits, 0); // the plain call's geometry: same bytes
        lds = f64::tile_lds_bytes(e.t, (uint32_t) workers);
        blocks = (e.t.cols + e.t.cols_per_tile - 1) / e.t.cols_per_tile;
        return lds <= f64::kMaxLdsBytes;
    }
    static bool stripe_entry_wide(const SEntry&) { return false; }
    static hipError_t launch_stripe_members(hipStream_t s, LaunchEvents ev, const SEntry* de, const uint32_t* db, const SEntry*, const uint32_t*,
                                            uint32_t members, uint32_t blocks, size_t lds, size_t nbits, bool zt, bool)
    {
        return f64::dispatch_nbits64<f64::StripeBatchLauncher64>(nbits, zt && nbits == 1, s, ev, de, db, members, blocks, lds);
    }
};


} // namespace cntkq_api

extern "C" {

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

size_t cntkq_stripe_reduce_max_rows_f64(size_t nbits)
{
    return cntkq::f64::valid_nbits(nbits) ? Elem<double>::stripe_max_rows(nbits) : 0;
}

int cntkq_stripe_reduce_takes_f64(cntkq_quantizer* h, size_t rows, size_t stripe_cols, size_t nbits, int zero_threshold_for_1bit)
{
    if (h == nullptr || !cntkq::f64::valid_nbits(nbits) || rows == 0 || stripe_cols == 0 || rows >= (1ull << 31) || stripe_cols >= (1ull << 31))
        return 0;
    if (rows <= Elem<double>::stripe_max_rows(nbits))
        return 1;
    DeviceGuard guard(h->device);
    return cntkq::f64::stripe_takes_strips(work_stream(h), rows, stripe_cols, nbits, zero_threshold_for_1bit != 0, h->tune) ? 1 : 0;
}

int cntkq_quantize_async_f64(cntkq_quantizer* h, const double* in, const double* res_in, size_t rows, size_t cols, void* qbuf,
                             size_t qbuf_bytes, int qbuf_on_host, size_t nbits, double* res_out, int zero_threshold_for_1bit)
{
    return quantize_async_impl<double>(h, in, res_in, rows, cols, qbuf, qbuf_bytes, qbuf_on_host, nbits, res_out, zero_threshold_for_1bit);
}

int cntkq_unquantize_async_f64(cntkq_quantizer* h, const void* qbuf, size_t qbuf_bytes, int qbuf_on_host, double* out,
                               size_t rows, size_t cols, size_t nbits, int add)
{
    return unquantize_async_impl<double>(h, qbuf, qbuf_bytes, qbuf_on_host, out, rows, cols, nbits, add);
}

int cntkq_stripe_reduce_async_f64(cntkq_quantizer* h, const void* const* stripes, size_t workers, size_t owner, size_t rows,
                                  size_t stripe_cols, size_t nbits, double* stripe_res, void* q_out, double* agg_out,
                                  int zero_threshold_for_1bit)
{
    return stripe_reduce_async_impl<double>(h, stripes, workers, owner, rows, stripe_cols, nbits, stripe_res, q_out, agg_out,
                                            zero_threshold_for_1bit);
}

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

int cntkq_stripe_reduce_batch_owners_async_f64(cntkq_quantizer* h, const cntkq_stripe_reduce_item_f64* items, const size_t* owners,
                                               size_t count, size_t workers, size_t nbits, int zero_threshold_for_1bit)
{
    if (owners == nullptr && count != 0)
        return fail(CNTKQ_INVALID_ARGUMENT, "cntkq_stripe_reduce_batch_owners_async_f64: null owner list");
    return stripe_reduce_batch_impl<double>(h, items, count, workers, 0, nbits, zero_threshold_for_1bit, owners);
}

} // extern "C"
