// Kernel family of the per-column gradient quantizer (gfx950): the decoders (QWord-major, row-major, tile, segment) and the gradient-set decoder.
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS>
inline hipError_t launch_unquantize_plan(hipStream_t s, LaunchEvents ev, const char* q, float* out, const UnquantizePlan& p, int add)
{
    if (p.kind == kUnqTile)
        hipExtLaunchKernelGGL((unquantize_tile_kernel<NBITS, float>), dim3(p.blocks), dim3(256), p.lds, s, ev.start, ev.stop, 0, q, out, p.tile, add);
    else if (p.kind == kUnqRows)
        hipExtLaunchKernelGGL((unquantize_rows_kernel<NBITS, float>), dim3(p.blocks), dim3(256), p.lds, s, ev.start, ev.stop, 0, q, out, p.rowg, add);
    else if (p.kind == kUnqDirect)
        hipExtLaunchKernelGGL((unquantize_direct_kernel<NBITS, float>), dim3(p.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.rowg, add);
    else if (p.kind == kUnqFlat)
        hipExtLaunchKernelGGL((unquantize_flat_kernel<NBITS, float>), dim3(p.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.flat, add);
    else if (p.kind == kUnqSegment)
        hipExtLaunchKernelGGL((unquantize_segment_kernel<NBITS>), dim3(p.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.seg, add);
    else if (p.kind == kUnqVec4)
        hipExtLaunchKernelGGL((unquantize_kernel<NBITS, 4, float>), dim3(p.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.qw, add);
    else
        hipExtLaunchKernelGGL((unquantize_kernel<NBITS, 1, float>), dim3(p.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.qw, add);
    return hipGetLastError();
}

hipError_t launch_unquantize_batch(hipStream_t s, LaunchEvents ev, const UnquantizeBatchEntry* entries, const uint32_t* begins,
                                          uint32_t count, uint32_t total_blocks, size_t nbits, bool add, size_t lds)
{
    const int a = add ? 1 : 0;
    switch (nbits)
    {
    case 1: hipExtLaunchKernelGGL((unquantize_batch_kernel<1>), dim3(total_blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count, a); break;
    case 2: hipExtLaunchKernelGGL((unquantize_batch_kernel<2>), dim3(total_blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count, a); break;
    case 4: hipExtLaunchKernelGGL((unquantize_batch_kernel<4>), dim3(total_blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count, a); break;
    case 8: hipExtLaunchKernelGGL((unquantize_batch_kernel<8>), dim3(total_blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count, a); break;
    case 16: hipExtLaunchKernelGGL((unquantize_batch_kernel<16>), dim3(total_blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count, a); break;
    case 32: hipExtLaunchKernelGGL((unquantize_batch_kernel<32>), dim3(total_blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count, a); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}


hipError_t family_unquantize(size_t nbits, hipStream_t s, LaunchEvents ev, const char* q, float* out, const UnquantizePlan& p, int add)
{
    switch (nbits)
    {
    case 1: return launch_unquantize_plan<1>(s, ev, q, out, p, add);
    case 2: return launch_unquantize_plan<2>(s, ev, q, out, p, add);
    case 4: return launch_unquantize_plan<4>(s, ev, q, out, p, add);
    case 8: return launch_unquantize_plan<8>(s, ev, q, out, p, add);
    case 16: return launch_unquantize_plan<16>(s, ev, q, out, p, add);
    case 32: return launch_unquantize_plan<32>(s, ev, q, out, p, add);
    default: return hipErrorInvalidValue;
    }
}

} // namespace cntkq
