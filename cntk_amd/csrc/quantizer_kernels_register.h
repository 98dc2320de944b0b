// gfx950 kernels of the per-column gradient quantizer: one workgroup per column, the column in registers,
// for quantize and for the stripe reduction of tall columns.
#pragma once

#include "quantizer_kernels_column.h"

namespace cntkq {

// ---- one workgroup per column, the column in registers ------------------------------------------------------
//
// Thread tid of T loads the 16-byte pieces tid, tid + T, ... (at most PER of them) of gradient and residual and keeps
// their sum in registers through statistics, coding and the residual store; LDS holds only the column's QWords, which
// the threads assemble with atomic OR (element i is bit position i / nq of QWord i % nq). With no column in LDS the
// number of resident workgroups no longer falls with the column height. Statistics are summed in the piece order of
// the LDS kernels above, so with T = 256 the bytes are theirs.

struct RegGeom
{
    uint32_t rows;   // multiple of 4, at most 4 * T * PER
    uint32_t nq;
    uint32_t pieces; // rows / 4
    uint32_t step_k; // (4 * T) / nq: a thread's next piece lies this many bit positions ...
    uint32_t step_w; // (4 * T) % nq: ... and this many QWords further on
    uint32_t line_shift; // non-zero: slots are dealt so that wavefronts cover whole 128-byte lines (see column_shift)
    uint64_t qcol;
};

// The value of x, but unknown to the compiler. The register kernels use the same indices and bounds checks in every
// phase (loads of the gradient, loads of the residual, sums, stores); recognised as common subexpressions they would
// all be kept in registers from the first phase to the last (a 64-bit address pair for every piece), which costs more
// registers than the column itself. Recomputing them from an opaque copy of the thread index is a few instructions.
__device__ __forceinline__ uint32_t opaque(uint32_t x)
{
    asm volatile("" : "+v"(x));
    return x;
}

constexpr uint32_t kRegRedSlots = 48; // three partial results for each of up to 16 waves
constexpr int kRegMaxShiftPer = 25;   // most pieces per thread of a register kernel that deals its slots by lines (all of them)

__host__ __device__ inline size_t reg_lds_bytes(const RegGeom& c)
{
    return ((size_t) kRegRedSlots + c.nq) * 4;
}

// Waves per SIMD the register allocator is asked to keep possible: the column's 4 * PER registers, one batch of
// residual pieces and about 40 more for addresses, statistics and coding.
template <int T, int PER>
constexpr int reg_waves()
{
    // (a looser budget does not help: given 128 registers the compiler hoists work until it spills)
    if (T == 1024)
        return PER <= 6 ? 8 : 4; // a workgroup is 4 waves on every SIMD: two of them fit, or one
    int w = 512 / (4 * PER + 40);
    return w > 8 ? 8 : (w < T / 256 ? T / 256 : w);
}

// Second half of the register kernels: statistics, header, codes, residual and packed QWords of the column a thread
// block holds in registers (a: the slots' pieces; edge: this thread's edge element if has_edge). words[0 .. nq) must be
// zero; the first barrier inside also orders everything the callers did before it.
template <int NBITS, bool ZT, int T, int PER>
__device__ __forceinline__ void reg_stats_pack(f32x4 (&a)[PER], float edge, bool has_edge, uint32_t edge_at, uint32_t head, uint32_t pieces,
                                               uint32_t shift, const RegGeom& c, float* red, uint32_t* red_u, uint32_t* words,
                                               float* r_out_col, char* qc)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t NW = T / 64;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    float total = 0.0f;
    if constexpr (need_stat)
    {
        float stat = 0.0f;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            const float with = colg_add_piece<NBITS>(stat, a[u]);
            stat = slot_valid(t + T * u, shift, pieces) ? with : stat;
        }
        if (has_edge)
            stat += NBITS == 1 ? edge : edge * edge;
        stat = wave_sum(stat);
        if (lane == 0)
            red[wave] = stat;
    }
    // the whole column has been read before this barrier, so r_out may be r_in
    __syncthreads();
    if constexpr (need_stat)
    {
        total = red[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
            total += red[x];
    }
    float lo, hi;
    if constexpr (NBITS == 1)
    {
        const float mean = ZT ? 0.0f : total / (float) c.rows;
        float s0 = 0.0f, s1 = 0.0f;
        uint32_t n0 = 0;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            float t0 = s0, t1 = s1;
            uint32_t tn = n0;
            split_add_piece(a[u], mean, t0, t1, tn);
            const bool valid = slot_valid(t + T * u, shift, pieces);
            s0 = valid ? t0 : s0;
            s1 = valid ? t1 : s1;
            n0 = valid ? tn : n0;
        }
        if (has_edge)
        {
            const bool below = edge < mean;
            s0 += below ? edge : 0.0f;
            s1 += below ? 0.0f : edge;
            n0 += below ? 1u : 0u;
        }
        s0 = wave_sum(s0);
        s1 = wave_sum(s1);
        n0 = wave_sum(n0);
        __syncthreads(); // everyone has read the wave sums of the mean
        if (lane == 0)
        {
            red[wave] = s0;
            red[NW + wave] = s1;
            red_u[wave] = n0;
        }
        __syncthreads();
        float S0 = red[0], S1 = red[NW];
        uint32_t N0 = red_u[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
        {
            S0 += red[x];
            S1 += red[NW + x];
            N0 += red_u[x];
        }
        finish_stats_1bit<ZT>(mean, S0, S1, N0, c.rows - N0, c.rows, lo, hi);
    }
    else
    {
        finish_stats_multibit(total, c.rows, lo, hi);
    }
    if (tid == 0)
    {
        float* gh = reinterpret_cast<float*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const float val0 = unquantize_value<NBITS>(vq, 0u);
    const float val1 = unquantize_value<NBITS>(vq, 1u);
    f32x4* o4 = reinterpret_cast<f32x4*>(r_out_col + head);
    // the first element of this thread's first slot inside the column is bit position k of QWord w; the elements after it
    // are the following QWords, the slots after it lie 4 * T elements further on
    const uint32_t ufirst = tid < shift ? 1u : 0u;
    const uint32_t e0 = head + 4 * (tid + T * ufirst - shift);
    uint32_t k = e0 / c.nq;
    uint32_t w = e0 - k * c.nq;
    const uint32_t to = opaque(tid);
#pragma unroll
    for (int u = 0; u < PER; ++u)
    {
        const uint32_t p = to + T * u - shift;
        if (slot_valid(to + T * u, shift, pieces))
        {
            f32x4 res;
            uint32_t kk = k, ww = w;
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                const float v = a[u][e];
                const uint32_t code = quantize_value<NBITS, ZT>(vq, v);
                float back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                res[e] = v - back;
                atomicOr(&words[ww], code << (kk * PS::SHIFT));
                if (++ww == c.nq)
                {
                    ww = 0;
                    ++kk;
                }
            }
            __builtin_nontemporal_store(res, o4 + p);
        }
        if ((uint32_t) u >= ufirst)
        {
            w += c.step_w;
            k += c.step_k;
            if (w >= c.nq)
            {
                w -= c.nq;
                ++k;
            }
        }
    }
    if (has_edge)
    {
        const uint32_t code = quantize_value<NBITS, ZT>(vq, edge);
        float back;
        if constexpr (NBITS == 1)
            back = code ? val1 : val0;
        else
            back = unquantize_value<NBITS>(vq, code);
        r_out_col[edge_at] = edge - back;
        const uint32_t ek = edge_at / c.nq;
        atomicOr(&words[edge_at - ek * c.nq], code << (ek * PS::SHIFT));
    }
    __syncthreads();
    uint32_t* bits = reinterpret_cast<uint32_t*>(qc + 8);
    for (uint32_t x = tid; x < c.nq; x += T)
        bits[x] = words[x];
}

// EDGE: the column need not start on a 16-byte boundary nor hold a multiple of 4 elements: up to 3 elements before the
// first aligned piece and up to 3 after the last are held, one each, by threads 0..5 and take part in every phase after
// the thread's pieces. (c.pieces then only bounds the pieces; the count is taken from the column's address.)
template <int NBITS, bool ZT, int T, int PER, bool EDGE = false>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(reg_waves<T, PER>(), reg_waves<T, PER>()))) void quantize_reg_kernel(
    const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q, RegGeom c)
{
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * c.rows;
    char* qc = q + (size_t) blockIdx.x * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0u;
    uint32_t head = 0, tail = 0, pieces = c.pieces;
    if constexpr (EDGE)
    {
        head = (4u - (uint32_t) ((reinterpret_cast<uintptr_t>(r_in + base) >> 2) & 3u)) & 3u; // elements before the first aligned piece
        pieces = (c.rows - head) >> 2;
        tail = c.rows - head - 4 * pieces;
    }
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g + base + head);
    const f32x4* r4 = reinterpret_cast<const f32x4*>(r_in + base + head);
    // the edge element of this thread, if it has one
    const bool has_edge = EDGE && tid < head + tail;
    const uint32_t edge_at = tid < head ? tid : c.rows - tail + (tid - head);
    float edge = 0.0f;
    if (has_edge)
        edge = g[base + edge_at] + r_in[base + edge_at];
    // Slot v = tid + T * u holds piece v - shift, where shift (0..7) is the column's offset into its 128-byte line in
    // pieces: every wavefront's 64 slots then cover whole lines, also in columns that start inside a line (9304 rows: every
    // column but each fourth). Slots before the column or past its end read a piece of the column all the same (no
    // branch, all loads in flight together) and are left out of every sum and store.
    const uint32_t shift = PER <= kRegMaxShiftPer ? column_shift(r_in + base + head, c.line_shift) : 0u;
    const uint32_t last = pieces - 1;
    f32x4 a[PER];
    {
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
            a[u] = __builtin_nontemporal_load(g4 + slot_piece(t + T * u, shift, last));
    }
#pragma unroll
    for (int u0 = 0; u0 < PER; u0 += 4)
    {
        const uint32_t t = opaque(tid);
        f32x4 b[4];
#pragma unroll
        for (int u = u0; u < u0 + 4 && u < PER; ++u)
            b[u - u0] = __builtin_nontemporal_load(r4 + slot_piece(t + T * u, shift, last));
#pragma unroll
        for (int u = u0; u < u0 + 4 && u < PER; ++u)
            a[u] = a[u] + b[u - u0];
    }
    reg_stats_pack<NBITS, ZT, T, PER>(a, edge, has_edge, edge_at, head, pieces, shift, c, red, red_u, words, r_out + base, qc);
}

// Stripe reduction for tall columns (above the LDS kernels' 14336 rows), in the register kernel's shape: 1024 threads per
// owned column, the running sum of the decoded stripes in registers. The workers are taken one at a time in the fixed
// order (owner first, then ascending rank): the worker's packed record goes to LDS in one coalesced copy (every QWord
// serves up to 32 rows), each thread decodes its slots' elements from it and adds them to its sums. Then the stripe
// residual is added and reg_stats_pack requantizes, so that the result is, byte for byte, what the sequence
// "unquantize own stripe, add the others, quantize_reg_kernel on (aggregate, stripe residual)" gives.
// LDS: [48 reduction slots | nq output QWords | nq + 2 words of one worker's record].
__host__ __device__ inline size_t stripe_reg_lds_bytes(const RegGeom& c)
{
    return ((size_t) kRegRedSlots + 2 * (size_t) c.nq + 2) * 4;
}

template <int NBITS, bool ZT, int PER>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(reg_waves<1024, PER>(), reg_waves<1024, PER>()))) void stripe_reduce_reg_kernel(
    StripeSources src, float* stripe_res, char* q_out, float* agg_out, RegGeom c)
{
    using PS = PackShape<NBITS>;
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t T = 1024, NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    uint32_t* pw = words + c.nq; // one worker's record: lower, upper, QWords
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * c.rows;
    const size_t rec = (size_t) blockIdx.x * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0u;
    // the column as the quantize kernel would see it: head elements, aligned pieces, tail elements
    float* sres = stripe_res + base;
    const uint32_t head = (4u - (uint32_t) ((reinterpret_cast<uintptr_t>(sres) >> 2) & 3u)) & 3u;
    const uint32_t pieces = (c.rows - head) >> 2;
    const uint32_t tail = c.rows - head - 4 * pieces;
    const bool has_edge = tid < head + tail;
    const uint32_t edge_at = tid < head ? tid : c.rows - tail + (tid - head);
    const uint32_t shift = column_shift(sres + head, c.line_shift);
    const uint32_t ufirst = tid < shift ? 1u : 0u;
    const uint32_t e0 = head + 4 * (tid + T * ufirst - shift);
    const uint32_t k_first = e0 / c.nq;
    const uint32_t w_first = e0 - k_first * c.nq;
    const uint32_t edge_k = edge_at / c.nq;
    const uint32_t edge_w = edge_at - edge_k * c.nq;

    f32x4 a[PER];
    float edge = 0.0f;
    const uint32_t K = src.workers;
    const uint32_t rec_words = c.nq + 2;
    for (uint32_t n = 0; n < K; ++n)
    {
        const uint32_t* from = reinterpret_cast<const uint32_t*>(src.q[stripe_order(n, src.owner)] + rec);
        if (n != 0)
            __syncthreads(); // everyone has decoded the previous worker's record
        for (uint32_t x = tid; x < rec_words; x += 8 * T)
        {
            uint32_t v[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                v[u] = from[(x + T * u < rec_words) ? x + T * u : x];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                if (x + T * u < rec_words)
                    pw[x + T * u] = v[u];
        }
        __syncthreads();
        const float lo = __uint_as_float(pw[0]);
        const float uf = make_ufactor<NBITS>(lo, __uint_as_float(pw[1]));
        const float val0 = unquantize_value<NBITS>(uf, lo, 0u);
        const float val1 = unquantize_value<NBITS>(uf, lo, 1u);
        const uint32_t* bits = pw + 2;
        // (opaque: the positions of all slots do not depend on the worker, and hoisted out of this loop they would be held
        // in registers for its whole duration)
        uint32_t k = opaque(k_first), w = opaque(w_first);
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            if (slot_valid(t + T * u, shift, pieces))
            {
                uint32_t kk = k, ww = w;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    float x;
                    if constexpr (NBITS == 1)
                        x = pick_level(bits[ww], kk, val0, val1);
                    else
                        x = unquantize_value<NBITS>(uf, lo, (bits[ww] >> (kk * PS::SHIFT)) & PS::CODEMASK);
                    // the first term (the owner's) seeds the sum; afterwards: decoded value + running sum
                    a[u][e] = (n == 0) ? x : x + a[u][e];
                    if (++ww == c.nq)
                    {
                        ww = 0;
                        ++kk;
                    }
                }
            }
            if ((uint32_t) u >= ufirst)
            {
                w += c.step_w;
                k += c.step_k;
                if (w >= c.nq)
                {
                    w -= c.nq;
                    ++k;
                }
            }
        }
        if (has_edge)
        {
            const uint32_t code = (bits[edge_w] >> (edge_k * PS::SHIFT)) & PS::CODEMASK;
            float x;
            if constexpr (NBITS == 1)
                x = code ? val1 : val0;
            else
                x = unquantize_value<NBITS>(uf, lo, code);
            edge = (n == 0) ? x : x + edge;
        }
    }
    // aggregate out (optional), then the stripe residual in
    {
        const f32x4* r4 = reinterpret_cast<const f32x4*>(sres + head);
        float* ag = agg_out != nullptr ? agg_out + base : nullptr;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            const uint32_t v = t + T * u;
            if (slot_valid(v, shift, pieces))
            {
                const uint32_t p = v - shift;
                if (ag != nullptr)
                {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        ag[head + 4 * p + e] = a[u][e];
                }
                a[u] = a[u] + __builtin_nontemporal_load(r4 + p);
            }
        }
        if (has_edge)
        {
            if (ag != nullptr)
                ag[edge_at] = edge;
            edge = edge + sres[edge_at];
        }
    }
    reg_stats_pack<NBITS, ZT, T, PER>(a, edge, has_edge, edge_at, head, pieces, shift, c, red, red_u, words, sres, q_out + rec);
}

// ---- the same for tall columns of any height and alignment: elements instead of pieces ----------------------
//
// Thread tid of 1024 keeps elements tid, tid + 1024, ... (at most EPT) of the column in registers, loaded and stored one
// float at a time: consecutive lanes touch consecutive floats, so nothing depends on the height being a multiple of 4
// or on the matrices being 16-byte aligned (columns of 50257 or 100001 rows, unaligned slices). One read of the
// inputs, like the piece-wise kernel above; step_k / step_w describe a stride of 1024 elements.

constexpr int kRegsThreads = 1024;

template <int EPT>
constexpr int regs_waves()
{
    return EPT <= 24 ? 8 : 4; // two workgroups per CU where 64 registers are enough, else one
}

template <int NBITS, bool ZT, int EPT>
__global__ __launch_bounds__(kRegsThreads) __attribute__((amdgpu_waves_per_eu(regs_waves<EPT>(), regs_waves<EPT>()))) void quantize_regs_kernel(
    const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q, RegGeom c)
{
    using PS = PackShape<NBITS>;
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t T = kRegsThreads, NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const size_t base = (size_t) blockIdx.x * c.rows;
    char* qc = q + (size_t) blockIdx.x * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0u;
    const float* gc = g + base;
    const float* rc = r_in + base;
    // branch-free loads: an element beyond the column is replaced by the column's last one and left out of every sum and store
    const uint32_t last = c.rows - 1;
    float a[EPT];
    {
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int j = 0; j < EPT; ++j)
        {
            const uint32_t e = t + T * j;
            a[j] = gc[e < c.rows ? e : last];
        }
    }
#pragma unroll
    for (int j0 = 0; j0 < EPT; j0 += 8)
    {
        const uint32_t t = opaque(tid);
        float b[8];
#pragma unroll
        for (int j = j0; j < j0 + 8 && j < EPT; ++j)
        {
            const uint32_t e = t + T * j;
            b[j - j0] = rc[e < c.rows ? e : last];
        }
#pragma unroll
        for (int j = j0; j < j0 + 8 && j < EPT; ++j)
            a[j] = a[j] + b[j - j0];
    }
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    float total = 0.0f;
    if constexpr (need_stat)
    {
        float stat = 0.0f;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int j = 0; j < EPT; ++j)
        {
            const float with = stat + (NBITS == 1 ? a[j] : a[j] * a[j]);
            stat = (t + T * j < c.rows) ? with : stat;
        }
        stat = wave_sum(stat);
        if (lane == 0)
            red[wave] = stat;
    }
    // the whole column has been read before this barrier, so r_out may be r_in
    __syncthreads();
    if constexpr (need_stat)
    {
        total = red[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
            total += red[x];
    }
    float lo, hi;
    if constexpr (NBITS == 1)
    {
        const float mean = ZT ? 0.0f : total / (float) c.rows;
        float s0 = 0.0f, s1 = 0.0f;
        uint32_t n0 = 0;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int j = 0; j < EPT; ++j)
        {
            const float x = a[j];
            const bool below = x < mean;
            const bool valid = t + T * j < c.rows;
            s0 = valid ? s0 + (below ? x : 0.0f) : s0;
            s1 = valid ? s1 + (below ? 0.0f : x) : s1;
            n0 += (valid && below) ? 1u : 0u;
        }
        s0 = wave_sum(s0);
        s1 = wave_sum(s1);
        n0 = wave_sum(n0);
        __syncthreads(); // everyone has read the wave sums of the mean
        if (lane == 0)
        {
            red[wave] = s0;
            red[NW + wave] = s1;
            red_u[wave] = n0;
        }
        __syncthreads();
        float S0 = red[0], S1 = red[NW];
        uint32_t N0 = red_u[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
        {
            S0 += red[x];
            S1 += red[NW + x];
            N0 += red_u[x];
        }
        finish_stats_1bit<ZT>(mean, S0, S1, N0, c.rows - N0, c.rows, lo, hi);
    }
    else
    {
        finish_stats_multibit(total, c.rows, lo, hi);
    }
    if (tid == 0)
    {
        float* gh = reinterpret_cast<float*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const float val0 = unquantize_value<NBITS>(vq, 0u);
    const float val1 = unquantize_value<NBITS>(vq, 1u);
    float* oc = r_out + base;
    // element tid is bit position k of QWord w; this thread's next element lies 1024 elements further on
    uint32_t k = tid / c.nq;
    uint32_t w = tid - k * c.nq;
    const uint32_t to = opaque(tid);
#pragma unroll
    for (int j = 0; j < EPT; ++j)
    {
        const uint32_t e = to + T * j;
        if (e < c.rows)
        {
            const float v = a[j];
            const uint32_t code = quantize_value<NBITS, ZT>(vq, v);
            float back;
            if constexpr (NBITS == 1)
                back = code ? val1 : val0;
            else
                back = unquantize_value<NBITS>(vq, code);
            oc[e] = v - back;
            atomicOr(&words[w], code << (k * PS::SHIFT));
        }
        w += c.step_w;
        k += c.step_k;
        if (w >= c.nq)
        {
            w -= c.nq;
            ++k;
        }
    }
    __syncthreads();
    uint32_t* bits = reinterpret_cast<uint32_t*>(qc + 8);
    for (uint32_t x = tid; x < c.nq; x += T)
        bits[x] = words[x];
}

} // namespace cntkq
