// gfx950 kernels of the per-column gradient quantizer: columns too tall for LDS and registers.
#pragma once

#include "quantizer_kernels_common.h"

namespace cntkq {

// ---- quantize, columns too tall for LDS: one workgroup per column, global memory re-read -------------

template <typename T>
__device__ __forceinline__ T tall_block_sum(T v, T* scratch)
{
    v = wave_sum(v);
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0)
        scratch[wave] = v;
    __syncthreads();
    T t = scratch[0];
    for (uint32_t x = 1; x < kTallThreads / 64; ++x)
        t += scratch[x];
    __syncthreads();
    return t;
}

// 16-byte accesses at the element's own alignment: four floats or two doubles
template <typename E>
struct TallVec;
template <>
struct TallVec<float>
{
    typedef f32x4 V;
    typedef f32x4_u VU;
    typedef u32x4 Q;
    typedef u32x4_u QU;
    static constexpr uint32_t N = 4;
};
template <>
struct TallVec<double>
{
    typedef f64x2 V;
    typedef f64x2 VU __attribute__((aligned(8)));
    typedef uint64_t Q __attribute__((ext_vector_type(2)));
    typedef Q QU __attribute__((aligned(8)));
    static constexpr uint32_t N = 2;
};

// E: float with 32-bit QWords or double with 64-bit QWords; one source for both.
template <int NBITS, bool ZT, typename E>
__global__ __launch_bounds__(kTallThreads) void quantize_tall_kernel(const E* __restrict__ g, const E* r_in, E* r_out, char* __restrict__ q,
                                                                     uint32_t rows, uint32_t nq, uint64_t qcol)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    __shared__ E scratch_f[kTallThreads / 64];
    __shared__ uint32_t scratch_u[kTallThreads / 64];

    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * rows;
    const E* gp = g + base;
    const E* rp = r_in + base;
    char* qc = q + (size_t) blockIdx.x * qcol;
    QWord* bits = reinterpret_cast<QWord*>(qc + 2 * sizeof(E));
    E* op = r_out + base;
    E lo, hi;

    if constexpr (NBITS == Word<E>::kBits)
    {
        // A code as wide as the element is the value itself and its residual the value minus itself, whatever the range in
        // the header: one pass computes the header's sum of squares while it writes both (16 bytes per access at the
        // element's alignment; a thread reads an element before it writes it and nobody else does either, so r_out may
        // be r_in).
        using TV = TallVec<E>;
        const uint32_t pieces = rows / TV::N;
        E s = (E) 0;
#pragma unroll 4
        for (uint32_t x = tid; x < pieces; x += kTallThreads)
        {
            const typename TV::V v = __builtin_nontemporal_load(reinterpret_cast<const typename TV::VU*>(gp) + x) +
                                     __builtin_nontemporal_load(reinterpret_cast<const typename TV::VU*>(rp) + x);
            typename TV::Q code;
#pragma unroll
            for (uint32_t e = 0; e < TV::N; ++e)
            {
                s += v[e] * v[e];
                code[e] = Word<E>::bits_of(v[e]);
            }
            __builtin_nontemporal_store(code, reinterpret_cast<typename TV::QU*>(bits) + x);
            __builtin_nontemporal_store(v - v, reinterpret_cast<typename TV::VU*>(op) + x);
        }
        const uint32_t i = TV::N * pieces + tid;
        if (i < rows)
        {
            const E v = gp[i] + rp[i];
            s += v * v;
            bits[i] = Word<E>::bits_of(v);
            op[i] = v - v;
        }
        s = tall_block_sum(s, scratch_f);
        finish_stats_multibit(s, rows, lo, hi);
        if (tid == 0)
        {
            E* gh = reinterpret_cast<E*>(qc);
            gh[0] = lo;
            gh[1] = hi;
        }
        return;
    }
    else if constexpr (NBITS == 1)
    {
        E mean = (E) 0;
        if constexpr (!ZT)
        {
            E s = (E) 0;
            for (uint32_t i = tid; i < rows; i += kTallThreads)
                s += gp[i] + rp[i];
            s = tall_block_sum(s, scratch_f);
            mean = s / (E) rows;
        }
        E s0 = (E) 0, s1 = (E) 0;
        uint32_t n0 = 0, n1 = 0;
        for (uint32_t i = tid; i < rows; i += kTallThreads)
        {
            const E v = gp[i] + rp[i];
            if (v < mean)
            {
                s0 += v;
                n0++;
            }
            else
            {
                s1 += v;
                n1++;
            }
        }
        s0 = tall_block_sum(s0, scratch_f);
        s1 = tall_block_sum(s1, scratch_f);
        n0 = tall_block_sum(n0, scratch_u);
        n1 = tall_block_sum(n1, scratch_u);
        finish_stats_1bit<ZT>(mean, s0, s1, n0, n1, rows, lo, hi);
    }
    else
    {
        E s = (E) 0;
        for (uint32_t i = tid; i < rows; i += kTallThreads)
        {
            const E v = gp[i] + rp[i];
            s += v * v;
        }
        s = tall_block_sum(s, scratch_f);
        finish_stats_multibit(s, rows, lo, hi);
    }
    // every thread has passed the last barrier of tall_block_sum, so all statistics reads of r_in are done
    // before any residual is written (r_out may be r_in)

    if (tid == 0)
    {
        E* gh = reinterpret_cast<E*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQOf<E> vq = make_vq<NBITS>(lo, hi);
    const E val0 = unquantize_value<NBITS>(vq, 0u);
    const E val1 = unquantize_value<NBITS>(vq, 1u);
    for (uint32_t w = tid; w < nq; w += kTallThreads)
    {
        QWord word = 0;
#pragma unroll
        for (uint32_t k = 0; k < PS::VPW; ++k)
        {
            const uint32_t i = w + k * nq;
            if (i < rows)
            {
                // last use of these values: streaming loads and stores
                const E v = __builtin_nontemporal_load(gp + i) + __builtin_nontemporal_load(rp + i);
                const QWord code = quantize_value<NBITS, ZT>(vq, v);
                E back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                __builtin_nontemporal_store(v - back, op + i);
                word |= code << (k * PS::SHIFT);
            }
        }
        bits[w] = word;
    }
}

} // namespace cntkq
