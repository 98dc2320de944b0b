// Device-side arithmetic of the per-column quantizer for gfx950.
//
// Every floating-point operation here is a separately rounded IEEE fp32 operation; the file must be
// compiled with -ffp-contract=off (no fused multiply-add) and without fast-math so that, given the
// same column header, codes and residuals are bit-identical to the reference CPU quantizer
// (Source/Math/ValueQuantizer.h, Source/Math/ColumnQuantizer.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cntkq {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef f32x4 f32x4_u __attribute__((aligned(4))); // a 16-byte access at any 4-byte alignment
typedef u32x4 u32x4_u __attribute__((aligned(4)));

constexpr int kWave = 64;

// ---- per-value quantizer (Source/Math/ValueQuantizer.h:68-97) ------------------------------------

struct ValueQ
{
    float lo, hi; // reconstruction range as stored in the column header
    float mid;    // 1-bit decision threshold derived from the STORED header, not from the column mean
    float qf, uf; // value -> code and code -> value scale factors
};

template <int NBITS>
__device__ __forceinline__ ValueQ make_vq(float lo, float hi)
{
    constexpr uint32_t rangeend = (NBITS >= 32) ? 0u : (1u << (NBITS & 31));
    ValueQ v;
    v.lo = lo;
    v.hi = hi;
    const float span = hi - lo;
    if ((span < 1e-36f) || (rangeend == 0))
    {
        v.qf = 0.0f;
        v.uf = 0.0f;
    }
    else
    {
        // one code fewer than 2^NBITS spans the range when NBITS > 1, which leaves a code for 0
        constexpr float used = (float) (rangeend - (NBITS > 1 ? 1u : 0u));
        v.qf = used / span;
        v.uf = span / used;
    }
    v.mid = 0.5f * (hi + lo);
    return v;
}

// Only what decoding needs: the code -> value step of the same quantizer state (identical arithmetic to make_vq).
template <int NBITS>
__device__ __forceinline__ float make_ufactor(float lo, float hi)
{
    constexpr uint32_t rangeend = (NBITS >= 32) ? 0u : (1u << (NBITS & 31));
    const float span = hi - lo;
    if ((span < 1e-36f) || (rangeend == 0))
        return 0.0f;
    constexpr float used = (float) (rangeend - (NBITS > 1 ? 1u : 0u));
    return span / used;
}

// x / d and x % d for 32-bit operands through one double-precision multiply by a host-computed reciprocal
// (exact after the single correction step: the product is off by less than 2^-20).
__device__ __forceinline__ void divmod_u32(uint32_t x, uint32_t d, double inv_d, uint32_t& quot, uint32_t& rem)
{
    uint32_t qv = (uint32_t) ((double) x * inv_d);
    uint32_t r = x - qv * d;
    if ((int32_t) r < 0)
    {
        qv--;
        r += d;
    }
    else if (r >= d)
    {
        qv++;
        r -= d;
    }
    quot = qv;
    rem = r;
}

// Source/Math/ValueQuantizer.h:101-128, 144-156
template <int NBITS, bool ZT>
__device__ __forceinline__ uint32_t quantize_value(const ValueQ& v, float u)
{
    if constexpr (NBITS == 32)
    {
        return __float_as_uint(u);
    }
    else if constexpr (NBITS == 1)
    {
        return ZT ? (u >= 0.0f ? 1u : 0u) : (u >= v.mid ? 1u : 0u);
    }
    else
    {
        constexpr uint32_t top = (1u << (NBITS & 31)) - 1u;
        if (u <= v.lo)
            return 0u;
        if (u >= v.hi)
            return top;
        return (uint32_t) (int32_t) ((u - v.lo) * v.qf);
    }
}

// Source/Math/ValueQuantizer.h:131-141.  (q + 0.5) * uf + lo, multiply and add rounded separately.
template <int NBITS>
__device__ __forceinline__ float unquantize_value(float uf, float lo, uint32_t q)
{
    if constexpr (NBITS == 32)
    {
        return __uint_as_float(q);
    }
    else
    {
        float t = (float) q + 0.5f;
        t = t * uf;
        return t + lo;
    }
}

// 1-bit decoding of bit `pos` of a QWord: val1 where the bit is set, val0 elsewhere, as a bit-field extract (the bit
// sign-extended to a mask) and a bitwise select, i.e. two instructions and no condition register. Written with compare
// and conditional move the same choice takes three and a wait for the condition register each time; the stripe
// reductions, which decode workers x elements values per column, are bound by instruction issue.
__device__ __forceinline__ float pick_level(uint32_t bits, uint32_t pos, float val0, float val1)
{
    const int32_t mask = __builtin_amdgcn_sbfe((int32_t) bits, pos, 1u);
    float x;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(x) : "v"(mask), "v"(val1), "v"(val0));
    return x;
}

template <int NBITS>
__device__ __forceinline__ float unquantize_value(const ValueQ& v, uint32_t q)
{
    return unquantize_value<NBITS>(v.uf, v.lo, q);
}

// ---- column header from reduced sums (Source/Math/ColumnQuantizer.h:265-340) ---------------------

// 1 bit: the two reconstruction levels are  centre -/+ radius/2;  the header stores centre -/+ radius.
template <bool ZT>
__device__ __forceinline__ void finish_stats_1bit(float mean, float s0, float s1, uint32_t n0, uint32_t n1,
                                                  uint32_t rows, float& lo, float& hi)
{
    float radius, centre;
    if constexpr (!ZT)
    {
        const float dev0 = ((float) n0 * mean) - s0;
        const float dev1 = s1 - ((float) n1 * mean);
        const float dev = (dev0 + dev1) / (float) rows;
        radius = 2.0f * dev;
        centre = mean;
    }
    else
    {
        if (n0 == 0)
            n0 = 1;
        if (n1 == 0)
            n1 = 1;
        const float m0 = s0 / (float) n0;
        const float m1 = s1 / (float) n1;
        centre = 0.5f * (m0 + m1);
        radius = 2.0f * (m1 - centre);
    }
    lo = centre - radius;
    hi = centre + radius;
}

// more than 1 bit: +/- 4 standard deviations around a mean that is taken to be 0
__device__ __forceinline__ void finish_stats_multibit(float sumsq, uint32_t rows, float& lo, float& hi)
{
    const float mean = 0.0f;
    const float sd = sqrtf(sumsq / (float) rows);
    const float half = 4.0f * sd;
    lo = mean - half;
    hi = mean + half;
}

// ---- cross-lane sums ----------------------------------------------------------------------------

// Sum over aligned groups of `width` lanes (power of two, <= 64); every lane of a group gets the
// same bits because each butterfly step adds the same two operands on both partner lanes.
template <typename T>
__device__ __forceinline__ T lanes_sum(T v, uint32_t width)
{
    for (uint32_t off = width >> 1; off > 0; off >>= 1)
        v += __shfl_xor(v, (int) off, kWave);
    return v;
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1)
        v += __shfl_xor(v, off, kWave);
    return v;
}

// Sum over aligned groups of `gs` consecutive threads of a workgroup (power of two, 8..blockDim.x).
// `scratch` holds one T per wave of the workgroup. gs is uniform over the workgroup, so the barriers
// are reached by all threads. The cross-wave part adds the wave sums in ascending wave order.
template <typename T>
__device__ __forceinline__ T group_sum(T v, uint32_t gs, T* scratch)
{
    v = lanes_sum(v, gs < (uint32_t) kWave ? gs : (uint32_t) kWave);
    if (gs > (uint32_t) kWave)
    {
        const uint32_t wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63u) == 0)
            scratch[wave] = v;
        __syncthreads();
        const uint32_t per = gs >> 6;
        const uint32_t first = (threadIdx.x / gs) * per;
        T t = scratch[first];
        for (uint32_t x = 1; x < per; ++x)
            t += scratch[first + x];
        __syncthreads();
        v = t;
    }
    return v;
}

// The three sums of the 1-bit split (sum below, sum not below, count below) over aligned groups of `gs` threads in
// one exchange: same order of additions as three group_sum calls, one pair of barriers instead of three.
// scratch_f holds two T per wave (a of every wave, then b of every wave), scratch_u one uint32 per wave.
template <typename T>
__device__ __forceinline__ void group_sum3(T& a, T& b, uint32_t& c, uint32_t gs, T* scratch_f, uint32_t* scratch_u)
{
    const uint32_t width = gs < (uint32_t) kWave ? gs : (uint32_t) kWave;
    a = lanes_sum(a, width);
    b = lanes_sum(b, width);
    c = lanes_sum(c, width);
    if (gs > (uint32_t) kWave)
    {
        const uint32_t wave = threadIdx.x >> 6;
        const uint32_t waves = blockDim.x >> 6;
        if ((threadIdx.x & 63u) == 0)
        {
            scratch_f[wave] = a;
            scratch_f[waves + wave] = b;
            scratch_u[wave] = c;
        }
        __syncthreads();
        const uint32_t per = gs >> 6;
        const uint32_t first = (threadIdx.x / gs) * per;
        T ta = scratch_f[first], tb = scratch_f[waves + first];
        uint32_t tc = scratch_u[first];
        for (uint32_t x = 1; x < per; ++x)
        {
            ta += scratch_f[first + x];
            tb += scratch_f[waves + first + x];
            tc += scratch_u[first + x];
        }
        __syncthreads();
        a = ta;
        b = tb;
        c = tc;
    }
}

} // namespace cntkq
