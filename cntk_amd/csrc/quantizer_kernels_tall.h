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

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTallThreads) void quantize_tall_kernel(const float* __restrict__ g, const float* r_in,
                                                                     float* r_out, char* __restrict__ q, uint32_t rows,
                                                                     uint32_t nq, uint64_t qcol)
{
    constexpr uint32_t VPW = 32 / NBITS;
    constexpr uint32_t MASKBITS = NBITS & 31;
    __shared__ float scratch_f[kTallThreads / 64];
    __shared__ uint32_t scratch_u[kTallThreads / 64];

    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * rows;
    const float* gp = g + base;
    const float* rp = r_in + base;
    float lo, hi;

    if constexpr (NBITS == 32)
    {
        // A 32-bit code is the value itself and its residual the value minus itself, whatever the range in the header: one
        // pass computes the header's sum of squares while it writes both (four elements per access at any 4-byte alignment;
        // a thread reads an element before it writes it and nobody else does either, so r_out may be r_in).
        char* qc = q + (size_t) blockIdx.x * qcol;
        uint32_t* bits = reinterpret_cast<uint32_t*>(qc + 8);
        float* op = r_out + base;
        const uint32_t quads = rows / 4;
        float s = 0.0f;
#pragma unroll 4
        for (uint32_t x = tid; x < quads; x += kTallThreads)
        {
            const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(gp) + x) +
                            __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(rp) + x);
            s += v[0] * v[0];
            s += v[1] * v[1];
            s += v[2] * v[2];
            s += v[3] * v[3];
            const u32x4 code = {__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
            __builtin_nontemporal_store(code, reinterpret_cast<u32x4_u*>(bits) + x);
            __builtin_nontemporal_store(v - v, reinterpret_cast<f32x4_u*>(op) + x);
        }
        const uint32_t i = 4 * quads + tid;
        if (i < rows)
        {
            const float v = gp[i] + rp[i];
            s += v * v;
            bits[i] = __float_as_uint(v);
            op[i] = v - v;
        }
        s = tall_block_sum(s, scratch_f);
        finish_stats_multibit(s, rows, lo, hi);
        if (tid == 0)
        {
            float* gh = reinterpret_cast<float*>(qc);
            gh[0] = lo;
            gh[1] = hi;
        }
        return;
    }
    else if constexpr (NBITS == 1)
    {
        float mean = 0.0f;
        if constexpr (!ZT)
        {
            float s = 0.0f;
            for (uint32_t i = tid; i < rows; i += kTallThreads)
                s += gp[i] + rp[i];
            s = tall_block_sum(s, scratch_f);
            mean = s / (float) rows;
        }
        float s0 = 0.0f, s1 = 0.0f;
        uint32_t n0 = 0, n1 = 0;
        for (uint32_t i = tid; i < rows; i += kTallThreads)
        {
            const float v = gp[i] + rp[i];
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
        float s = 0.0f;
        for (uint32_t i = tid; i < rows; i += kTallThreads)
        {
            const float v = gp[i] + rp[i];
            s += v * v;
        }
        s = tall_block_sum(s, scratch_f);
        finish_stats_multibit(s, rows, lo, hi);
    }
    // every thread has passed the last barrier of tall_block_sum, so all statistics reads of r_in are done
    // before any residual is written (r_out may be r_in)

    char* qc = q + (size_t) blockIdx.x * qcol;
    if (tid == 0)
    {
        float* gh = reinterpret_cast<float*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const float val0 = unquantize_value<NBITS>(vq, 0u);
    const float val1 = unquantize_value<NBITS>(vq, 1u);
    float* op = r_out + base;
    uint32_t* bits = reinterpret_cast<uint32_t*>(qc + 8);
    for (uint32_t w = tid; w < nq; w += kTallThreads)
    {
        uint32_t word = 0;
#pragma unroll
        for (uint32_t k = 0; k < VPW; ++k)
        {
            const uint32_t i = w + k * nq;
            if (i < rows)
            {
                // last use of these values: streaming loads and stores
                const float v = __builtin_nontemporal_load(gp + i) + __builtin_nontemporal_load(rp + i);
                const uint32_t code = quantize_value<NBITS, ZT>(vq, v);
                float back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                __builtin_nontemporal_store(v - back, op + i);
                word |= code << (k * MASKBITS);
            }
        }
        bits[w] = word;
    }
}

} // namespace cntkq
