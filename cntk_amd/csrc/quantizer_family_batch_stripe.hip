// Kernel family of the per-column gradient quantizer (gfx950): the stripe reductions of a whole gradient set in one grid.
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT>
struct StripeBatchLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeBatchEntry* entries, const uint32_t* begins, uint32_t count,
                          uint32_t total_blocks, size_t lds, bool wide)
    {
        if constexpr (NBITS == 1)
        {
            if (wide)
            {
                hipExtLaunchKernelGGL((stripe_reduce_batch_lookup_kernel<ZT>), dim3(total_blocks), dim3(kTileThreads), lds, s, ev.start, ev.stop,
                                      0, entries, begins, count);
                return hipGetLastError();
            }
        }
        hipExtLaunchKernelGGL((stripe_reduce_batch_kernel<NBITS, ZT>), dim3(total_blocks), dim3(kTileThreads), lds, s, ev.start, ev.stop, 0,
                              entries, begins, count);
        return hipGetLastError();
    }
};

hipError_t family_batch_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeBatchEntry* entries, const uint32_t* begins, uint32_t count, uint32_t total_blocks, size_t lds, bool wide)
{
    return dispatch_nbits<StripeBatchLauncher>(nbits, zt, s, ev, entries, begins, count, total_blocks, lds, wide);
}

} // namespace cntkq
