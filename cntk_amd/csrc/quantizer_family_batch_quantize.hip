// Kernel family of the per-column gradient quantizer (gfx950): a whole gradient set quantized by one grid.
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT>
struct BatchLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const QuantizeBatchEntry* entries, const uint32_t* begins, uint32_t count,
                          uint32_t total_blocks, size_t lds)
    {
        static_assert(kTileThreads == kColThreads, "tiles and columns share one workgroup size in a batch");
        hipExtLaunchKernelGGL((quantize_batch_kernel<NBITS, ZT>), dim3(total_blocks), dim3(kTileThreads), lds, s, ev.start, ev.stop, 0,
                              entries, begins, count);
        return hipGetLastError();
    }
};

hipError_t family_batch_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const QuantizeBatchEntry* entries, const uint32_t* begins, uint32_t count, uint32_t total_blocks, size_t lds)
{
    return dispatch_nbits<BatchLauncher>(nbits, zt, s, ev, entries, begins, count, total_blocks, lds);
}

} // namespace cntkq
