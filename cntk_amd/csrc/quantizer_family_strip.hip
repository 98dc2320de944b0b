// Kernel family of the per-column gradient quantizer (gfx950): columns of any height cut into strips on several workgroups.
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT>
struct StripLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, StripGeom c,
                          StripScratch scratch)
    {
        if constexpr (NBITS >= 32)
            return hipErrorInvalidValue;
        else
        {
            hipExtLaunchKernelGGL((quantize_strip_kernel<NBITS, ZT>), dim3(strip_grid(cols, c)), dim3(kStripThreads), strip_lds_bytes(NBITS), s,
                                  ev.start, ev.stop, 0, g, r_in, r_out, q, c, scratch);
            return hipGetLastError();
        }
    }
};

template <int NBITS, bool ZT>
struct StripOccupancy
{
    static hipError_t run(int* per_cu)
    {
        if constexpr (NBITS >= 32)
            return hipErrorInvalidValue;
        else
            return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, quantize_strip_kernel<NBITS, ZT>, (int) kStripThreads, strip_lds_bytes(NBITS));
    }
};

hipError_t family_strip_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, StripGeom c, StripScratch scratch)
{
    return dispatch_nbits<StripLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, scratch);
}

hipError_t family_strip_occupancy(size_t nbits, bool zt, int* per_cu)
{
    return dispatch_nbits<StripOccupancy>(nbits, zt, per_cu);
}

} // namespace cntkq
