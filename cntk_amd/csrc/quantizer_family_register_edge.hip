// Kernel family of the per-column gradient quantizer (gfx950): the column in registers with edge elements (odd heights, slices at a 4-byte offset) or one element per access (any alignment).
// The launchers of one family, instantiated here and nowhere else; quantizer_launch.h declares the functions and chooses
// between the families.
#include "quantizer_launch.h"

namespace cntkq {

template <int NBITS, bool ZT, int PER, int T = 1024>
inline hipError_t launch_reg_edge_one(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols,
                                      const RegGeom& c)
{
    hipExtLaunchKernelGGL((quantize_reg_kernel<NBITS, ZT, T, PER, true>), dim3(cols), dim3(T), reg_lds_bytes(c), s, ev.start, ev.stop, 0,
                          g, r_in, r_out, q, c);
    return hipGetLastError();
}

// The variant for columns that start anywhere and have any height: c.pieces is an upper bound. 256 threads up to
// kRegEdgeMinRows rows (2049 x 9304: the tile kernel's 57 us), 1024 above.
template <int NBITS, bool ZT>
struct RegEdgeLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c,
                          uint32_t threads)
    {
        if constexpr (NBITS >= 32)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t per = (c.pieces + (c.line_shift ? 7u : 0u) + threads - 1) / threads;
#define CNTKQ_REGE256(P) if (threads == 256 && per <= P) return launch_reg_edge_one<NBITS, ZT, P, 256>(s, ev, g, r_in, r_out, q, cols, c)
            CNTKQ_REGE256(3);
            CNTKQ_REGE256(4);
            CNTKQ_REGE256(6);
            CNTKQ_REGE256(8);
#undef CNTKQ_REGE256
            if (threads != 1024)
                return hipErrorInvalidValue;
#define CNTKQ_REGE(P) if (per <= P) return launch_reg_edge_one<NBITS, ZT, P>(s, ev, g, r_in, r_out, q, cols, c)
            CNTKQ_REGE(4);
            CNTKQ_REGE(6);
            CNTKQ_REGE(8);
            CNTKQ_REGE(10);
            CNTKQ_REGE(13);
            CNTKQ_REGE(16);
            CNTKQ_REGE(20);
            CNTKQ_REGE(25);
#undef CNTKQ_REGE
            return hipErrorInvalidValue;
        }
    }
};

template <int NBITS, bool ZT, int EPT>
inline hipError_t launch_regs_one(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols,
                                  const RegGeom& c)
{
    hipExtLaunchKernelGGL((quantize_regs_kernel<NBITS, ZT, EPT>), dim3(cols), dim3(kRegsThreads), reg_lds_bytes(c), s, ev.start, ev.stop, 0, g,
                          r_in, r_out, q, c);
    return hipGetLastError();
}

template <int NBITS, bool ZT>
struct RegsLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c)
    {
        if constexpr (NBITS >= 32)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t ept = (c.rows + kRegsThreads - 1) / kRegsThreads;
#define CNTKQ_REGS(E) if (ept <= E) return launch_regs_one<NBITS, ZT, E>(s, ev, g, r_in, r_out, q, cols, c)
            CNTKQ_REGS(16);
            CNTKQ_REGS(24);
            CNTKQ_REGS(32);
            CNTKQ_REGS(48);
            CNTKQ_REGS(64);
            CNTKQ_REGS(80);
            CNTKQ_REGS(96);
#undef CNTKQ_REGS
            return hipErrorInvalidValue;
        }
    }
};

hipError_t family_reg_edge_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c, uint32_t threads)
{
    return dispatch_nbits<RegEdgeLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c, threads);
}

hipError_t family_regs_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t cols, RegGeom c)
{
    return dispatch_nbits<RegsLauncher>(nbits, zt, s, ev, g, r_in, r_out, q, cols, c);
}

} // namespace cntkq
