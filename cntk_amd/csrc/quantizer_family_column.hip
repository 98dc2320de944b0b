// Kernel family of the per-column gradient quantizer (gfx950): one workgroup per column, the column in LDS (quantize and stripe reduction).
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT>
struct ColLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, ColGeom c)
    {
        hipExtLaunchKernelGGL((quantize_colg_kernel<NBITS, ZT>), dim3(cols), dim3(kColThreads), colg_lds_bytes<NBITS>(c, 0), s, ev.start,
                              ev.stop, 0, g, r_in, r_out, q, c);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct StripeColLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                          uint32_t cols, ColGeom c)
    {
        // Every work item (a QWord, or a chunk of its bit positions) is a chain of dependent loads, and the column's LDS
        // limits how many workgroups a CU holds: from 24 KB per column on (6 workgroups or fewer per CU) 512 threads keep
        // the CU's wavefront slots filled, and where the stripe has no more columns than the device has CUs, 1024 do.
        // Measured at 8 workers, 256 / 512 / 1024 threads: 9304 x 2048 at 2 bits 62 / 58 / 84 us, 14336 x 1328 at 4 bits
        // 91 / 68 / 80, 4096 x 4652 at 8 bits 67 / 75 / 114, 6144 x 3101 at 2 bits 55 / 59 / 99, 14336 x 256 at 2 bits
        // 28 / 19 / 15, 8192 x 300 at 8 bits 23 / 16 / 20.
        uint32_t wg = 256u;
        if (c.nq * PackShape<NBITS>::CHUNKS >= kStripeWideItems)
            wg = cols <= kStripeWideMaxCols ? 1024u : (c.rows > kStripeMidMinRows ? 512u : 256u);
        if (wg == 1024)
            hipExtLaunchKernelGGL((stripe_reduce_colg_kernel<NBITS, ZT, 1024>), dim3(cols), dim3(1024), colg_lds_bytes<NBITS>(c, src.workers),
                                  s, ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, c);
        else if (wg == 512)
            hipExtLaunchKernelGGL((stripe_reduce_colg_kernel<NBITS, ZT, 512>), dim3(cols), dim3(512), colg_lds_bytes<NBITS>(c, src.workers),
                                  s, ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, c);
        else
            hipExtLaunchKernelGGL((stripe_reduce_colg_kernel<NBITS, ZT, kColThreads>), dim3(cols), dim3(kColThreads),
                                  colg_lds_bytes<NBITS>(c, src.workers), s, ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, c);
        return hipGetLastError();
    }
};

template <bool ZT, int PER>
inline void launch_quantize_col(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols,
                                uint64_t qcol)
{
    hipExtLaunchKernelGGL((quantize_col_kernel<ZT, PER>), dim3(cols), dim3(kColThreads), col_lds_bytes<PER>(), s, ev.start, ev.stop, 0, g,
                          r_in, r_out, q, qcol);
}

template <bool ZT, int PER>
inline void launch_stripe_col(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                              uint32_t cols, uint64_t qcol)
{
    hipExtLaunchKernelGGL((stripe_reduce_col_kernel<ZT, PER>), dim3(cols), dim3(kColThreads), col_lds_bytes<PER>() + kStripeColExtraLds, s,
                          ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, qcol);
}

hipError_t family_col_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, ColGeom c)
{
    return dispatch_nbits<ColLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c);
}

hipError_t family_col_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                             float* agg_out, uint32_t cols, ColGeom c)
{
    return dispatch_nbits<StripeColLauncher>(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, cols, c);
}

hipError_t family_col_quantize_unrolled(bool zt, int per, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, uint64_t qcol)
{
    if (per == 1)
        zt ? launch_quantize_col<true, 1>(s, ev, g, r_in, r_out, q, cols, qcol) : launch_quantize_col<false, 1>(s, ev, g, r_in, r_out, q, cols, qcol);
    else if (per == 2)
        zt ? launch_quantize_col<true, 2>(s, ev, g, r_in, r_out, q, cols, qcol) : launch_quantize_col<false, 2>(s, ev, g, r_in, r_out, q, cols, qcol);
    else if (per == 4)
        zt ? launch_quantize_col<true, 4>(s, ev, g, r_in, r_out, q, cols, qcol) : launch_quantize_col<false, 4>(s, ev, g, r_in, r_out, q, cols, qcol);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t family_col_stripe_unrolled(bool zt, int per, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                                      float* agg_out, uint32_t cols, uint64_t qcol)
{
    if (per == 1)
        zt ? launch_stripe_col<true, 1>(s, ev, src, stripe_res, q_out, agg_out, cols, qcol) : launch_stripe_col<false, 1>(s, ev, src, stripe_res, q_out, agg_out, cols, qcol);
    else if (per == 2)
        zt ? launch_stripe_col<true, 2>(s, ev, src, stripe_res, q_out, agg_out, cols, qcol) : launch_stripe_col<false, 2>(s, ev, src, stripe_res, q_out, agg_out, cols, qcol);
    else if (per == 4)
        zt ? launch_stripe_col<true, 4>(s, ev, src, stripe_res, q_out, agg_out, cols, qcol) : launch_stripe_col<false, 4>(s, ev, src, stripe_res, q_out, agg_out, cols, qcol);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t family_col_stripe_set(bool zt, int per, hipStream_t s, LaunchEvents ev, const StripeColSet& set)
{
    const uint32_t grid = set.begin[set.count];
    if (per == 1)
    {
        if (zt)
            hipExtLaunchKernelGGL((stripe_reduce_col_set_kernel<true, 1>), dim3(grid), dim3(kColThreads), col_lds_bytes<1>() + kStripeColExtraLds, s, ev.start, ev.stop, 0, set);
        else
            hipExtLaunchKernelGGL((stripe_reduce_col_set_kernel<false, 1>), dim3(grid), dim3(kColThreads), col_lds_bytes<1>() + kStripeColExtraLds, s, ev.start, ev.stop, 0, set);
    }
    else if (per == 2)
    {
        if (zt)
            hipExtLaunchKernelGGL((stripe_reduce_col_set_kernel<true, 2>), dim3(grid), dim3(kColThreads), col_lds_bytes<2>() + kStripeColExtraLds, s, ev.start, ev.stop, 0, set);
        else
            hipExtLaunchKernelGGL((stripe_reduce_col_set_kernel<false, 2>), dim3(grid), dim3(kColThreads), col_lds_bytes<2>() + kStripeColExtraLds, s, ev.start, ev.stop, 0, set);
    }
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

} // namespace cntkq
