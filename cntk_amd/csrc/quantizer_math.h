// Device-side arithmetic of the per-column quantizer for gfx950.
//
// Every floating-point operation here is a separately rounded IEEE operation in the element type; the file must be
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

// floor(a / d) for a below 2^20, given inv = small_divisor(d): four instructions where the integer division takes thirty.
// (a + 0.5) / d lies at least 0.5 / d away from every integer, the reciprocal and the product are off by less than
// 2^-22 of the quotient together, and (a + 0.5) * 2^-21 stays below 1.
__device__ __forceinline__ float small_divisor(uint32_t d)
{
    return __builtin_amdgcn_rcpf((float) d);
}
__device__ __forceinline__ uint32_t small_div(uint32_t a, float inv)
{
    return (uint32_t) (((float) a + 0.5f) * inv);
}

// For kernels meant to run eight wavefronts per SIMD. A SIMD's 800 scalar registers are dealt in blocks of 16, and every
// wavefront gets 16 more than its kernel asks for (measured with a kernel that does nothing but hold registers: up to 80
// scalar registers eight wavefronts per SIMD are resident, up to 96 seven, beyond that six); the compiler counts without
// those 16 and would take up to 96. The kernels that get a set of stripes by value are the ones that reach that many.
#define CNTKQ_SGPRS_FOR_8_WAVES __attribute__((amdgpu_num_sgpr(80)))

// LDS by byte address, for kernels that declare no LDS of their own and get all of theirs from the launch (theirs starts
// at address 0). Through an `extern __shared__` array that start reaches the compiler too late to be folded into the
// instructions: every access at a computed offset then carries an addition of zero, which these do not.
template <typename T>
__device__ __forceinline__ T lds_read(uint32_t byte_address)
{
    return *(const __attribute__((address_space(3))) T*) byte_address;
}
template <typename T>
__device__ __forceinline__ void lds_write(uint32_t byte_address, T v)
{
    *(__attribute__((address_space(3))) T*) byte_address = v;
}
typedef u32x4 u32x4_u __attribute__((aligned(4)));
typedef f32x2 f32x2_u __attribute__((aligned(4)));

constexpr int kWave = 64;

// ---- element types and their QWords (Source/Math/ValueQuantizer.h:48-57) -------------------------

typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef f64x2 f64x2_u __attribute__((aligned(8))); // a 16-byte access at any 8-byte alignment

// What differs between MatrixQuantizerImpl<float> and <double>: the QWord a column is packed into (as wide as the element),
// its signed twin for the float -> code conversion, the raw bits of a value (the "code" when NBITS is the QWord's width) and
// the square root of the header statistics. Everything below is written once over this.
template <typename E>
struct Word;
template <>
struct Word<float>
{
    typedef uint32_t Q;
    typedef int32_t S;
    static constexpr int kBits = 32;
    static __device__ __forceinline__ Q bits_of(float x) { return __float_as_uint(x); }
    static __device__ __forceinline__ float value_of(Q q) { return __uint_as_float(q); }
    static __device__ __forceinline__ float root(float x) { return sqrtf(x); }
};
template <>
struct Word<double>
{
    typedef uint64_t Q;
    typedef int64_t S;
    static constexpr int kBits = 64;
    static __device__ __forceinline__ Q bits_of(double x) { return (Q) __double_as_longlong(x); }
    static __device__ __forceinline__ double value_of(Q q) { return __longlong_as_double((long long) q); }
    static __device__ __forceinline__ double root(double x) { return sqrt(x); }
};

// ---- per-value quantizer (Source/Math/ValueQuantizer.h:68-97) ------------------------------------

template <typename E>
struct ValueQOf
{
    E lo, hi; // reconstruction range as stored in the column header
    E mid;    // 1-bit decision threshold derived from the STORED header, not from the column mean
    E qf, uf; // value -> code and code -> value scale factors
};
typedef ValueQOf<float> ValueQ;

// the number of codes that span the range: one fewer than 2^NBITS when NBITS > 1, which leaves a code for 0; 0 when a code
// is the value itself (exact in either element type: at most 2^32 - 1 where it is used)
template <int NBITS, typename E>
__device__ __forceinline__ constexpr uint64_t codes_in_range()
{
    return NBITS >= Word<E>::kBits ? 0ull : (1ull << (NBITS & 63)) - (NBITS > 1 ? 1ull : 0ull);
}

template <int NBITS, typename E>
__device__ __forceinline__ ValueQOf<E> make_vq(E lo, E hi)
{
    constexpr uint64_t codes = codes_in_range<NBITS, E>();
    ValueQOf<E> v;
    v.lo = lo;
    v.hi = hi;
    const E span = hi - lo;
    // the reference compares with the float literal 1e-36f in either precision
    if ((span < (E) 1e-36f) || (codes == 0))
    {
        v.qf = (E) 0;
        v.uf = (E) 0;
    }
    else
    {
        constexpr E used = (E) codes;
        v.qf = used / span;
        v.uf = span / used;
    }
    v.mid = (E) 0.5 * (hi + lo);
    return v;
}

// Only what decoding needs: the code -> value step of the same quantizer state (identical arithmetic to make_vq).
template <int NBITS, typename E>
__device__ __forceinline__ E make_ufactor(E lo, E hi)
{
    constexpr uint64_t codes = codes_in_range<NBITS, E>();
    const E span = hi - lo;
    if ((span < (E) 1e-36f) || (codes == 0))
        return (E) 0;
    constexpr E used = (E) codes;
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
template <int NBITS, bool ZT, typename E>
__device__ __forceinline__ typename Word<E>::Q quantize_value(const ValueQOf<E>& v, E u)
{
    typedef typename Word<E>::Q Q;
    if constexpr (NBITS == Word<E>::kBits)
    {
        return Word<E>::bits_of(u);
    }
    else if constexpr (NBITS == 1)
    {
        return ZT ? (u >= (E) 0 ? (Q) 1 : (Q) 0) : (u >= v.mid ? (Q) 1 : (Q) 0);
    }
    else
    {
        // (written as selects: with early returns the compiler branches around the conversion for every value, and the
        // kernels that code many values per thread spend more on the branches than on the arithmetic; a value outside the
        // range converts to something that is not used)
        constexpr Q top = ((Q) 1 << (NBITS & 63)) - (Q) 1;
        const Q inside = (Q) (typename Word<E>::S)((u - v.lo) * v.qf);
        return u <= v.lo ? (Q) 0 : (u >= v.hi ? top : inside);
    }
}

// Source/Math/ValueQuantizer.h:131-141.  (q + 0.5) * uf + lo, multiply and add rounded separately.
template <int NBITS, typename E>
__device__ __forceinline__ E unquantize_value(E uf, E lo, typename Word<E>::Q q)
{
    if constexpr (NBITS == Word<E>::kBits)
    {
        return Word<E>::value_of(q);
    }
    else
    {
        // codes are below 2^32 here, so the conversion is exact whichever way it is done
        E t = (E) (uint32_t) q + (E) 0.5;
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

template <int NBITS, typename E>
__device__ __forceinline__ E unquantize_value(const ValueQOf<E>& v, typename Word<E>::Q q)
{
    return unquantize_value<NBITS>(v.uf, v.lo, q);
}

// ---- column header from reduced sums (Source/Math/ColumnQuantizer.h:265-340) ---------------------

// 1 bit: the two reconstruction levels are  centre -/+ radius/2;  the header stores centre -/+ radius.
template <bool ZT, typename E>
__device__ __forceinline__ void finish_stats_1bit(E mean, E s0, E s1, uint32_t n0, uint32_t n1, uint32_t rows, E& lo, E& hi)
{
    E radius, centre;
    if constexpr (!ZT)
    {
        const E dev0 = ((E) n0 * mean) - s0;
        const E dev1 = s1 - ((E) n1 * mean);
        const E dev = (dev0 + dev1) / (E) rows;
        radius = (E) 2 * dev;
        centre = mean;
    }
    else
    {
        if (n0 == 0)
            n0 = 1;
        if (n1 == 0)
            n1 = 1;
        const E m0 = s0 / (E) n0;
        const E m1 = s1 / (E) n1;
        centre = (E) 0.5 * (m0 + m1);
        radius = (E) 2 * (m1 - centre);
    }
    lo = centre - radius;
    hi = centre + radius;
}

// more than 1 bit: +/- 4 standard deviations around a mean that is taken to be 0
template <typename E>
__device__ __forceinline__ void finish_stats_multibit(E sumsq, uint32_t rows, E& lo, E& hi)
{
    const E mean = (E) 0;
    const E sd = Word<E>::root(sumsq / (E) rows);
    const E half = (E) 4 * sd;
    lo = mean - half;
    hi = mean + half;
}

// ---- bit matrices -------------------------------------------------------------------------------

// Transposes an 8 x 8 bit matrix held as two dwords (row r = byte r, lo holds rows 0-3): three rounds of swapping
// off-diagonal blocks. After it byte r has, as bit g, bit r of the former byte g.
__device__ __forceinline__ void transpose_bits_8x8(uint32_t& lo, uint32_t& hi)
{
    uint32_t t;
    // 1 x 1 blocks within 2 x 2: bit c of row r <-> bit r of row c for neighbours (rows 8 bits apart: shift 7)
    t = (lo ^ (lo >> 7)) & 0x00AA00AAu;
    lo = lo ^ t ^ (t << 7);
    t = (hi ^ (hi >> 7)) & 0x00AA00AAu;
    hi = hi ^ t ^ (t << 7);
    // 2 x 2 blocks within 4 x 4 (rows 16 bits apart: shift 14)
    t = (lo ^ (lo >> 14)) & 0x0000CCCCu;
    lo = lo ^ t ^ (t << 14);
    t = (hi ^ (hi >> 14)) & 0x0000CCCCu;
    hi = hi ^ t ^ (t << 14);
    // 4 x 4 blocks: the high nibbles of rows 0-3 <-> the low nibbles of rows 4-7
    t = ((lo >> 4) ^ hi) & 0x0F0F0F0Fu;
    hi = hi ^ t;
    lo = lo ^ (t << 4);
}

// ---- cross-lane sums ----------------------------------------------------------------------------
//
// A butterfly over the lanes of a wavefront, nearest partners first: lane ^ 1, ^ 2, ^ 4, ^ 8, then the rows of 16 lanes in
// pairs, then the pairs. Each step adds the same two operands on both partner lanes, so all lanes of a group hold the same
// bits after it, and the tree -- which decides the last bits of a column's bounds -- is the same in every kernel. The
// steps are data-parallel-primitive modifiers of the addition itself (a permutation within four lanes; the mirror image
// of a half row and of a row, which is the partner's value once groups of four and eight lanes agree; the last lane of
// the row before, and lane 31, broadcast to the rows that follow): no trip through the LDS crossbar, which costs an
// index computation and some hundred cycles of latency per step, six steps per sum and four sums per column.

constexpr int kDppXor1 = 0xB1;       // quad_perm [1, 0, 3, 2]
constexpr int kDppXor2 = 0x4E;       // quad_perm [2, 3, 0, 1]
constexpr int kDppHalfMirror = 0x141; // lane 7 - i of each half row
constexpr int kDppMirror = 0x140;     // lane 15 - i of each row
constexpr int kDppBcast15 = 0x142;    // lane 15 of a row to every lane of the next row
constexpr int kDppBcast31 = 0x143;    // lane 31 to every lane of rows 2 and 3

// the value another lane holds, chosen by a DPP control (a lane without a source reads zero bits; written so that the
// compiler folds the move into the addition that follows)
template <int CTRL, typename T>
__device__ __forceinline__ T dpp_lane(T v)
{
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- and 64-bit values");
    int w[sizeof(T) / 4];
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 4; ++i)
        w[i] = __builtin_amdgcn_update_dpp(0, w[i], CTRL, 0xF, 0xF, true);
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

// the value lane `lane` (the same for the whole wavefront) holds
template <typename T>
__device__ __forceinline__ T read_lane(T v, int lane)
{
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- and 64-bit values");
    int w[sizeof(T) / 4];
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 4; ++i)
        w[i] = __builtin_amdgcn_readlane(w[i], lane);
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

// Sum over the 64 lanes of a wavefront (all of them active); every lane gets the same bits.
template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
    v += dpp_lane<kDppXor1>(v);
    v += dpp_lane<kDppXor2>(v);
    v += dpp_lane<kDppHalfMirror>(v);
    v += dpp_lane<kDppMirror>(v);  // every lane: the sum of its row
    v += dpp_lane<kDppBcast15>(v); // rows 1 and 3: rows 0 + 1 and 2 + 3 (rows 0 and 2 hold nothing of use from here on)
    v += dpp_lane<kDppBcast31>(v); // row 3: (2 + 3) + (0 + 1)
    return read_lane(v, 63);
}

// Sum over aligned groups of `width` lanes (power of two, <= 64; the same for the whole wavefront, all lanes active);
// every lane of a group gets the same bits. lanes_sum(v, 64) and wave_sum(v) are the same tree.
template <typename T>
__device__ __forceinline__ T lanes_sum(T v, uint32_t width)
{
    if (width >= 2)
        v += dpp_lane<kDppXor1>(v);
    if (width >= 4)
        v += dpp_lane<kDppXor2>(v);
    if (width >= 8)
        v += dpp_lane<kDppHalfMirror>(v);
    if (width >= 16)
        v += dpp_lane<kDppMirror>(v);
    if (width >= 32)
    {
        T t = v + dpp_lane<kDppBcast15>(v);
        if (width == 32)
        {
            const T first = read_lane(t, 31), second = read_lane(t, 63);
            v = (threadIdx.x & 32u) ? second : first;
        }
        else
        {
            t += dpp_lane<kDppBcast31>(t);
            v = read_lane(t, 63);
        }
    }
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
