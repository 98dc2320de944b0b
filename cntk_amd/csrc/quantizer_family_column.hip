// Kernel family of the per-column gradient quantizer (gfx950): one workgroup per column, the column in LDS (quantize and stripe reduction).
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

#include <algorithm>

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
        // How many threads a column gets. The work items of a column (a QWord, or a chunk of its bit positions) are dealt to
        // the threads in rounds, each a chain of dependent loads; the column's LDS limits how many workgroups a compute unit
        // holds, and a workgroup's sums are taken by its first 256 threads whatever its size (their order is part of the
        // result), so larger workgroups pay for idle threads in those phases. The size is the one of 256, 512 and 768 (whole
        // wavefronts on every SIMD: 576 and 640 threads measure a third slower than 512) with the most busy threads per
        // compute unit: resident workgroups x threads x the fill of the last round of items, times 0.8 for 512 and 0.75 for
        // 768 threads. Measured at 8 workers over 256 / 512 / 768 / 1024 threads: 9304 x 2048 at 2 bits 54 / 49 / 52 / 74 us,
        // at 8 bits 77 / 69 / 69 / 83; 14336 x 1328 at 2 bits 70 / 53 / 49 / 66, at 8 bits 93 / 70 / 68 / 80; 6144 x 3101 at 2
        // bits 44 / 50 / 51 / 82, at 8 bits 66 / 63 / 66 / 97; 4096 x 4652 at 2 bits 41 / 48 / 59 / 97. Where the stripe has no
        // more columns than the device has compute units, 1024 threads (14336 x 256 at 2 bits: 28 / 19 / - / 15 us).
        const uint32_t items = c.nq * PackShape<NBITS>::CHUNKS;
        uint32_t wg = 256u;
        if (items >= kStripeWideItems && cols <= kStripeWideMaxCols)
            wg = 1024u;
        else if (items >= kStripeWideItems)
        {
            const size_t lds = colg_lds_bytes<NBITS>(c, src.workers);
            double best = 0.0;
            for (uint32_t t = 256; t <= 768; t += 256)
            {
                const uint32_t resident = (uint32_t) std::max<size_t>(1, std::min<size_t>(2048 / t, (160 * 1024) / lds));
                const uint32_t rounds = (items + t - 1) / t;
                const double busy = (double) std::min(2048u, resident * t) * ((double) items / (double) (rounds * t)) *
                                    (t == 256 ? 1.0 : (t == 512 ? 0.8 : 0.75));
                if (busy > best)
                {
                    best = busy;
                    wg = t;
                }
            }
        }
        if (wg == kColThreads)
            hipExtLaunchKernelGGL((stripe_reduce_colg_kernel<NBITS, ZT, kColThreads>), dim3(cols), dim3(kColThreads),
                                  colg_lds_bytes<NBITS>(c, src.workers), s, ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, c);
        else
            hipExtLaunchKernelGGL((stripe_reduce_colg_kernel<NBITS, ZT, 0>), dim3(cols), dim3(wg), colg_lds_bytes<NBITS>(c, src.workers), s,
                                  ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, c);
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
