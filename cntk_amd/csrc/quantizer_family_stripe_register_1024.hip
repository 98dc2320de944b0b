// Kernel family of the per-column gradient quantizer (gfx950): stripe reductions with the sums in registers, 1024 threads per column.
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT, int PER, int T = 1024>
inline hipError_t launch_stripe_reg_one(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                                        uint32_t cols, const RegGeom& c)
{
    if constexpr (NBITS == 1)
    {
        // up to eight workers: the row sums looked up in a table of 256 (the same additions, made once per column)
        if (src.workers <= 8 && stripe_lut_lds_bytes(c) <= 160 * 1024)
        {
            hipExtLaunchKernelGGL((stripe_reduce_lut_kernel<ZT, PER, T>), dim3(cols), dim3(T), stripe_lut_lds_bytes(c), s, ev.start, ev.stop, 0, src,
                                  stripe_res, q_out, agg_out, c);
            return hipGetLastError();
        }
    }
    if constexpr (NBITS == 1 && T == 1024)
    {
        // 1 bit: eight workers at a time from the worker-minor table, where a CU's LDS holds it (always, up to 102400 rows)
        // (it always decodes eight slots: with four workers or fewer the kernel below does less work)
        if (src.workers > 4 && stripe_reg8_lds_bytes(c) <= 160 * 1024)
        {
            hipExtLaunchKernelGGL((stripe_reduce_reg8_kernel<ZT, PER>), dim3(cols), dim3(1024), stripe_reg8_lds_bytes(c), s, ev.start, ev.stop, 0,
                                  src, stripe_res, q_out, agg_out, c);
            return hipGetLastError();
        }
    }
    const uint32_t group = stripe_reg_group(c, src.workers);
    hipExtLaunchKernelGGL((stripe_reduce_reg_kernel<NBITS, ZT, PER, T>), dim3(cols), dim3(T), stripe_reg_lds_bytes(c, group), s, ev.start,
                          ev.stop, 0, src, stripe_res, q_out, agg_out, c, group);
    return hipGetLastError();
}

template <int NBITS, bool ZT>
struct StripeReg1024Launcher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint32_t cols,
                          RegGeom c, uint32_t threads)
    {
        if constexpr (NBITS >= 32)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t per = (c.pieces + (c.line_shift ? 7u : 0u) + threads - 1) / threads;
            if (threads != 1024)
                return hipErrorInvalidValue;
#define CNTKQ_SREG(P) if (per <= P) return launch_stripe_reg_one<NBITS, ZT, P>(s, ev, src, stripe_res, q_out, agg_out, cols, c)
            CNTKQ_SREG(4);
            CNTKQ_SREG(6);
            CNTKQ_SREG(8);
            CNTKQ_SREG(10);
            CNTKQ_SREG(13);
            CNTKQ_SREG(16);
            CNTKQ_SREG(20);
            CNTKQ_SREG(25);
#undef CNTKQ_SREG
            return hipErrorInvalidValue;
        }
    }
};

hipError_t family_reg1024_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint32_t cols, RegGeom c)
{
    return dispatch_nbits<StripeReg1024Launcher>(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, cols, c, 1024u);
}

hipError_t family_reg256_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint32_t cols, RegGeom c);

hipError_t family_reg_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint32_t cols, RegGeom c, uint32_t threads)
{
    if (threads == 256)
        return family_reg256_stripe(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, cols, c);
    if (threads == 1024)
        return family_reg1024_stripe(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, cols, c);
    return hipErrorInvalidValue;
}

} // namespace cntkq
