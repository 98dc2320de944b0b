// Kernel family of the per-column gradient quantizer (gfx950): column tiles in LDS (short and odd columns) and the re-reading kernel for the tallest columns.
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT>
struct TileLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, TileGeom t)
    {
        const uint32_t tiles = (t.cols + t.cols_per_tile - 1) / t.cols_per_tile;
        const size_t lds = tile_lds_bytes(t, 0);
        hipExtLaunchKernelGGL((quantize_tile_kernel<NBITS, ZT>), dim3(tiles), dim3(t.threads), lds, s, ev.start, ev.stop, 0, g, r_in, r_out, q, t);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct TallLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t rows,
                          uint32_t cols, uint32_t nq, uint64_t qcol)
    {
        hipExtLaunchKernelGGL((quantize_tall_kernel<NBITS, ZT, float>), dim3(cols), dim3(kTallThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out, q, rows,
                           nq, qcol);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct StripeLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                          TileGeom t)
    {
        const uint32_t tiles = (t.cols + t.cols_per_tile - 1) / t.cols_per_tile;
        const size_t lds = tile_lds_bytes(t, src.workers);
        hipExtLaunchKernelGGL((stripe_reduce_tile_kernel<NBITS, ZT>), dim3(tiles), dim3(t.threads), lds, s, ev.start, ev.stop, 0, src, stripe_res,
                           q_out, agg_out, t);
        return hipGetLastError();
    }
};

hipError_t family_tile_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, TileGeom t)
{
    return dispatch_nbits<TileLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, t);
}

hipError_t family_tile_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                              float* agg_out, TileGeom t)
{
    return dispatch_nbits<StripeLauncher>(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, t);
}

hipError_t family_tall_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t rows, uint32_t cols, uint32_t nq, uint64_t qcol)
{
    return dispatch_nbits<TallLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, rows, cols, nq, qcol);
}

} // namespace cntkq
