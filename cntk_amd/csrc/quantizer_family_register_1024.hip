// Kernel family of the per-column gradient quantizer (gfx950): one workgroup of 1024 threads per column, the column in registers (whole 16-byte pieces).
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT, int T, int PER>
inline hipError_t launch_reg_one(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols,
                                 const RegGeom& c)
{
    hipExtLaunchKernelGGL((quantize_reg_kernel<NBITS, ZT, T, PER>), dim3(cols), dim3(T), reg_lds_bytes(c), s, ev.start, ev.stop, 0, g, r_in,
                          r_out, q, c);
    return hipGetLastError();
}

template <int NBITS, bool ZT>
struct Reg1024Launcher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c,
                          uint32_t threads)
    {
        if constexpr (NBITS >= 32)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t per = (c.pieces + (c.line_shift ? 7u : 0u) + threads - 1) / threads; // up to 7 slots lie before the column
#define CNTKQ_REG(T, P) if (threads == T && per <= P) return launch_reg_one<NBITS, ZT, T, P>(s, ev, g, r_in, r_out, q, cols, c)
            CNTKQ_REG(1024, 4);
            CNTKQ_REG(1024, 6);
            CNTKQ_REG(1024, 8);
            CNTKQ_REG(1024, 10);
            CNTKQ_REG(1024, 13);
            CNTKQ_REG(1024, 16);
            CNTKQ_REG(1024, 20);
            CNTKQ_REG(1024, 25);
#undef CNTKQ_REG
            return hipErrorInvalidValue;
        }
    }
};

hipError_t family_reg1024_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c)
{
    return dispatch_nbits<Reg1024Launcher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, 1024u);
}

hipError_t family_reg256_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c);

hipError_t family_reg_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c, uint32_t threads)
{
    if (threads == 256)
        return family_reg256_quantize(nbits, zt, s, ev, g, r_in, r_out, q, cols, c);
    if (threads == 1024)
        return family_reg1024_quantize(nbits, zt, s, ev, g, r_in, r_out, q, cols, c);
    return hipErrorInvalidValue;
}

} // namespace cntkq
