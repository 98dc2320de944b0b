// Kernel family of the per-column gradient quantizer (gfx950): columns of any height cut into strips on several workgroups,
// for float and for double matrices. The launchers of one family, instantiated here and nowhere else; quantizer_launch.h
// declares the functions and chooses between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <typename E>
struct StripFor
{
    template <int NBITS, bool ZT>
    struct Launcher
    {
        static hipError_t run(hipStream_t s, LaunchEvents ev, const E* g, const E* r_in, E* r_out, char* q, uint32_t cols, StripGeom c,
                              StripScratch scratch)
        {
            if constexpr (NBITS >= Word<E>::kBits)
                return hipErrorInvalidValue;
            else
            {
                hipExtLaunchKernelGGL((quantize_strip_kernel<NBITS, ZT, E>), dim3(strip_grid(cols, c)), dim3(kStripThreads),
                                      strip_lds_bytes<E>(NBITS), s, ev.start, ev.stop, 0, g, r_in, r_out, q, c, scratch);
                return hipGetLastError();
            }
        }
    };

    // the quantization cut into launches that follow each other on the stream (columns of more strips than the device holds)
    template <int NBITS, bool ZT>
    struct PassLauncher
    {
        template <int PASS>
        static hipError_t one(hipStream_t s, hipEvent_t start, hipEvent_t stop, const E* g, const E* r_in, E* r_out, char* q, uint32_t cols,
                              const StripGeom& c, const StripScratch& scratch)
        {
            hipExtLaunchKernelGGL((quantize_strip_kernel<NBITS, ZT, E, PASS>), dim3(strip_grid(cols, c)), dim3(kStripThreads),
                                  strip_lds_bytes<E>(NBITS), s, start, stop, 0, g, r_in, r_out, q, c, scratch);
            return hipGetLastError();
        }
        static hipError_t run(hipStream_t s, LaunchEvents ev, const E* g, const E* r_in, E* r_out, char* q, uint32_t cols, StripGeom c,
                              StripScratch scratch)
        {
            if constexpr (NBITS >= Word<E>::kBits)
                return hipErrorInvalidValue;
            else
            {
                hipError_t rc = hipSuccess;
                hipEvent_t start = ev.start;
                if constexpr (NBITS != 1 || !ZT)
                {
                    rc = one<kStripPassStat>(s, start, nullptr, g, r_in, r_out, q, cols, c, scratch);
                    start = nullptr;
                }
                if constexpr (NBITS == 1)
                {
                    if (rc == hipSuccess)
                        rc = one<kStripPassSplit>(s, start, nullptr, g, r_in, r_out, q, cols, c, scratch);
                    start = nullptr;
                }
                if (rc == hipSuccess)
                    rc = one<kStripPassPack>(s, start, ev.stop, g, r_in, r_out, q, cols, c, scratch);
                return rc;
            }
        }
    };

    template <int NBITS, bool ZT>
    struct StripeLauncher
    {
        static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, E* stripe_res, char* q_out, E* agg_out, uint32_t cols,
                              StripGeom c, StripScratch scratch)
        {
            if constexpr (NBITS >= Word<E>::kBits)
                return hipErrorInvalidValue;
            else
            {
                hipExtLaunchKernelGGL((stripe_reduce_strip_kernel<NBITS, ZT, E>), dim3(strip_grid(cols, c)), dim3(kStripThreads),
                                      strip_lds_bytes<E>(NBITS), s, ev.start, ev.stop, 0, src, stripe_res, q_out, agg_out, c, scratch);
                return hipGetLastError();
            }
        }
    };

    template <int NBITS, bool ZT>
    struct Occupancy
    {
        static hipError_t run(bool stripe, int* per_cu)
        {
            if constexpr (NBITS >= Word<E>::kBits)
                return hipErrorInvalidValue;
            else if (stripe)
                return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, stripe_reduce_strip_kernel<NBITS, ZT, E>, (int) kStripThreads,
                                                                    strip_lds_bytes<E>(NBITS));
            else
                return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, quantize_strip_kernel<NBITS, ZT, E>, (int) kStripThreads,
                                                                    strip_lds_bytes<E>(NBITS));
        }
    };
};

hipError_t family_strip_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripFor<float>::Launcher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, scratch);
}

hipError_t family_strip_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripFor<double>::Launcher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, scratch);
}

hipError_t family_strip_quantize_passes(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripFor<float>::PassLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, scratch);
}

hipError_t family_strip_quantize_passes(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripFor<double>::PassLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, scratch);
}

hipError_t family_strip_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripFor<float>::StripeLauncher>(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, cols, c, scratch);
}

hipError_t family_strip_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, char* q_out, double* agg_out, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripFor<double>::StripeLauncher>(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, cols, c, scratch);
}

hipError_t family_strip_occupancy(size_t nbits, bool zt, bool stripe, int* per_cu, const float*)
{
    return dispatch_nbits<StripFor<float>::Occupancy>(nbits, zt, stripe, per_cu);
}

hipError_t family_strip_occupancy(size_t nbits, bool zt, bool stripe, int* per_cu, const double*)
{
    return dispatch_nbits<StripFor<double>::Occupancy>(nbits, zt, stripe, per_cu);
}

} // namespace cntkq
