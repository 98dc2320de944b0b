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
    // (with edge elements the residual output may lie at another offset within 16 bytes than the input that the pieces follow)
    f32x4_u* o4 = reinterpret_cast<f32x4_u*>(r_out_col + head);
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

// EDGE: the column need not start on a 16-byte boundary nor hold a multiple of 4 elements, and the three matrices need
// not share their offset within 16 bytes (the aligned pieces are the residual input's): up to 3 elements before the
// first aligned piece and up to 3 after the last are held, one each, by threads 0..5 and take part in every phase after
// the thread's pieces. (c.pieces then only bounds the pieces; the count is taken from the column's address.)
template <int NBITS, bool ZT, int T, int PER, bool EDGE = false>
__device__ __forceinline__ void quantize_reg_body(const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q, const RegGeom& c,
                                                  uint32_t column, f32x4* smem_v4)
{
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t NW = T / 64;
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * c.rows;
    char* qc = q + (size_t) column * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0u;
    uint32_t head = 0, tail = 0, pieces = c.pieces;
    if constexpr (EDGE)
    {
        head = (4u - (uint32_t) ((reinterpret_cast<uintptr_t>(r_in + base) >> 2) & 3u)) & 3u; // elements before the first aligned piece
        pieces = (c.rows - head) >> 2;
        tail = c.rows - head - 4 * pieces;
    }
    // (the pieces follow the residual input; with edge elements the gradient may lie at another offset within 16 bytes)
    using GradientPiece = typename std::conditional<EDGE, f32x4_u, f32x4>::type;
    const GradientPiece* g4 = reinterpret_cast<const GradientPiece*>(g + base + head);
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

template <int NBITS, bool ZT, int T, int PER, bool EDGE = false>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(reg_waves<T, PER>(), reg_waves<T, PER>()))) void quantize_reg_kernel(
    const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q, RegGeom c)
{
    extern __shared__ f32x4 smem_v4[];
    quantize_reg_body<NBITS, ZT, T, PER, EDGE>(g, r_in, r_out, q, c, blockIdx.x, smem_v4);
}

// Stripe reduction for tall columns (above the LDS kernels' 14336 rows), in the register kernel's shape: 1024 threads per
// owned column, the running sum of the decoded stripes in registers. The workers are taken in the fixed order (owner
// first, then ascending rank), `group` of them at a time (as many as the CU's 160 KB of LDS hold; all 8 of a 100000-row
// 1-bit stripe): their packed columns go to LDS in coalesced copies (every QWord serves up to 32 rows), and each thread
// walks its slots once per group -- the position of a slot's elements (QWord, bit) is worked out once and serves every
// worker of the group; a piece's four elements sit in four consecutive QWords at one bit position unless the piece
// straddles the end of the QWord run, which takes an element-wise path. The kernel is bound by instruction issue, not by
// memory: one worker at a time with every position recomputed per worker and element cost 11,500 vector instructions
// per wavefront at 100000 rows and 8 workers, 14.7 per decoded value. Then the stripe residual is added and
// reg_stats_pack requantizes, so that the result is, byte for byte, what the sequence "unquantize own stripe, add the
// others, quantize_reg_kernel on (aggregate, stripe residual)" gives.
// LDS: [48 reduction slots | nq output QWords | 2 decoding constants per worker of a group | group x nq QWords].
__host__ __device__ inline size_t stripe_reg_lds_bytes(const RegGeom& c, uint32_t group)
{
    return ((size_t) kRegRedSlots + (size_t) c.nq + 2 * (size_t) group + (size_t) group * c.nq) * 4;
}

// how many workers' packed columns are decoded together: what fits the LDS of a CU beside the output QWords
__host__ __device__ inline uint32_t stripe_reg_group(const RegGeom& c, uint32_t workers, size_t lds_limit = 160 * 1024)
{
    const size_t fixed = ((size_t) kRegRedSlots + c.nq) * 4;
    const size_t per = ((size_t) c.nq + 2) * 4;
    size_t g = lds_limit > fixed ? (lds_limit - fixed) / per : 0;
    if (g < 1)
        g = 1;
    return (uint32_t) (g < workers ? g : workers);
}

template <int NBITS, bool ZT, int PER, int TT = 1024>
__global__ __launch_bounds__(TT) __attribute__((amdgpu_waves_per_eu(reg_waves<TT, PER>(), reg_waves<TT, PER>()))) void stripe_reduce_reg_kernel(
    StripeSources src, float* stripe_res, char* q_out, float* agg_out, RegGeom c, uint32_t group)
{
    using PS = PackShape<NBITS>;
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t T = TT, NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    float* dec = reinterpret_cast<float*>(words + c.nq); // per worker of the group: 1 bit -> the two levels, else (ufactor, lower)
    uint32_t* pw = words + c.nq + 2 * group;             // the group's packed columns, nq QWords each
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

    // -0 is the additive identity (x + -0 = x for every x, signed zeros included): the first worker's values seed the sums
    // through the same addition as the others
    f32x4 a[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u)
        a[u] = f32x4{-0.0f, -0.0f, -0.0f, -0.0f};
    float edge = -0.0f;
    const uint32_t K = src.workers;
    for (uint32_t n0 = 0; n0 < K; n0 += group)
    {
        const uint32_t G = min(group, K - n0);
        if (n0 != 0)
            __syncthreads(); // everyone has decoded the previous group
        // decoding constants: one lane of a wavefront of its own per worker
        for (uint32_t g = 0; g < G; ++g)
        {
            if (tid == 64 * (g & (NW - 1u)))
            {
                const float* h = reinterpret_cast<const float*>(src.q[stripe_order(n0 + g, src.owner)] + rec);
                const float lo = h[0];
                const float uf = make_ufactor<NBITS>(lo, h[1]);
                if constexpr (NBITS == 1)
                {
                    dec[2 * g] = unquantize_value<NBITS>(uf, lo, 0u);
                    dec[2 * g + 1] = unquantize_value<NBITS>(uf, lo, 1u);
                }
                else
                {
                    dec[2 * g] = uf;
                    dec[2 * g + 1] = lo;
                }
            }
        }
        // the packed columns, four workers and four QWords per thread in flight together (one round trip for eight workers
        // of a 100000-row column takes two passes, where a worker at a time took eight)
        for (uint32_t g0 = 0; g0 < G; g0 += 4)
        {
            const uint32_t* from[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                from[j] = reinterpret_cast<const uint32_t*>(src.q[stripe_order(n0 + min(g0 + j, G - 1), src.owner)] + rec) + 2;
            for (uint32_t x = tid; x < c.nq; x += 4 * T)
            {
                uint32_t v[4][4];
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j)
#pragma unroll
                    for (uint32_t u = 0; u < 4; ++u)
                        v[j][u] = from[j][(x + T * u < c.nq) ? x + T * u : x];
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j)
                    if (g0 + j < G)
                    {
                        uint32_t* to = pw + (size_t) (g0 + j) * c.nq;
#pragma unroll
                        for (uint32_t u = 0; u < 4; ++u)
                            if (x + T * u < c.nq)
                                to[x + T * u] = v[j][u];
                    }
            }
        }
        __syncthreads();
        // (opaque: the positions of all slots do not depend on the group, and hoisted out of this loop they would be held
        // in registers for its whole duration; the sums alone take 100 of a thread's 128 registers at 100000 rows)
        const uint32_t t = opaque(tid);
        const uint32_t ufirst = t < shift ? 1u : 0u;
        uint32_t k, w;
        {
            const uint32_t e0 = head + 4 * (t + T * ufirst - shift);
            k = e0 / c.nq;
            w = e0 - k * c.nq;
        }
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            if (slot_valid(t + T * u, shift, pieces))
            {
                if (w + 3 < c.nq)
                {
                    // the common case: four consecutive QWords, one bit position
                    const uint32_t* bp = pw + w;
                    const uint32_t sh = k * PS::SHIFT;
                    for (uint32_t g = 0; g < G; ++g)
                    {
                        const uint32_t b0 = bp[0], b1 = bp[1], b2 = bp[2], b3 = bp[3];
                        const float d0 = dec[2 * g], d1 = dec[2 * g + 1];
                        bp += c.nq;
                        if constexpr (NBITS == 1)
                        {
                            a[u].x = pick_level(b0, sh, d0, d1) + a[u].x;
                            a[u].y = pick_level(b1, sh, d0, d1) + a[u].y;
                            a[u].z = pick_level(b2, sh, d0, d1) + a[u].z;
                            a[u].w = pick_level(b3, sh, d0, d1) + a[u].w;
                        }
                        else
                        {
                            a[u].x = unquantize_value<NBITS>(d0, d1, (b0 >> sh) & PS::CODEMASK) + a[u].x;
                            a[u].y = unquantize_value<NBITS>(d0, d1, (b1 >> sh) & PS::CODEMASK) + a[u].y;
                            a[u].z = unquantize_value<NBITS>(d0, d1, (b2 >> sh) & PS::CODEMASK) + a[u].z;
                            a[u].w = unquantize_value<NBITS>(d0, d1, (b3 >> sh) & PS::CODEMASK) + a[u].w;
                        }
                    }
                }
                else
                {
                    // the piece runs past the last QWord: its later elements are the next bit position of the first QWords
                    for (uint32_t g = 0; g < G; ++g)
                    {
                        const uint32_t* bits = pw + (size_t) g * c.nq;
                        const float d0 = dec[2 * g], d1 = dec[2 * g + 1];
                        uint32_t kk = k, ww = w;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            float x;
                            if constexpr (NBITS == 1)
                                x = pick_level(bits[ww], kk, d0, d1);
                            else
                                x = unquantize_value<NBITS>(d0, d1, (bits[ww] >> (kk * PS::SHIFT)) & PS::CODEMASK);
                            a[u][e] = x + a[u][e];
                            if (++ww == c.nq)
                            {
                                ww = 0;
                                ++kk;
                            }
                        }
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
            const uint32_t at = opaque(edge_at);
            const uint32_t edge_k = at / c.nq;
            const uint32_t edge_w = at - edge_k * c.nq;
            for (uint32_t g = 0; g < G; ++g)
            {
                const uint32_t bits = pw[(size_t) g * c.nq + edge_w];
                float x;
                if constexpr (NBITS == 1)
                    x = pick_level(bits, edge_k, dec[2 * g], dec[2 * g + 1]);
                else
                    x = unquantize_value<NBITS>(dec[2 * g], dec[2 * g + 1], (bits >> (edge_k * PS::SHIFT)) & PS::CODEMASK);
                edge = x + edge;
            }
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

// The 1-bit tall stripe reduction with up to eight workers decoded together from a worker-minor table in LDS. The kernel
// above reads a piece's four QWords of one worker at a time (lanes 16 bytes apart, 4 bytes each: a quarter of the LDS
// banks serve every access, and counters put the kernel at 122 us of LDS time for a 219 us run at 100000 x 512, K = 8).
// Here QWord w of the group's worker g sits at dword (w / 4) * 36 + (w % 4) * 8 + g: the eight workers' copies of one QWord
// are 32 consecutive bytes, fetched by two 16-byte reads, and the 4 padding dwords per row of 32 turn consecutive lanes
// (QWords 4 apart) by 4 banks, so that every read and every fill of the table is free of bank conflicts. One worker's
// level for a cleared bit is kept per thread, the level for a set bit per wavefront (scalar registers): a decoded value
// costs a bit-field extract, a bitwise select and the addition.
// LDS: [48 reduction slots | nq output QWords | 16 levels | padding to 16 bytes | ceil(nq / 4) rows of 36 dwords].
constexpr uint32_t kStripe8Row = 36; // dwords; the decoder below spells 36 * 4 bytes out as shifts

__host__ __device__ inline uint32_t stripe_reg8_table_offset(const RegGeom& c) // in dwords
{
    return (kRegRedSlots + c.nq + 16u + 3u) & ~3u;
}

__host__ __device__ inline size_t stripe_reg8_lds_bytes(const RegGeom& c)
{
    return ((size_t) stripe_reg8_table_offset(c) + (size_t) ((c.nq + 3) / 4) * kStripe8Row) * 4;
}

__device__ __forceinline__ float pick_level_s(uint32_t bits, uint32_t pos, float val0, float val1_uniform)
{
    const int32_t mask = __builtin_amdgcn_sbfe((int32_t) bits, pos, 1u);
    float x;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(x) : "v"(mask), "s"(val1_uniform), "v"(val0));
    return x;
}

// (six pieces per thread do not fit the 64 registers that two workgroups per CU leave: one workgroup without spills does
// 20000 x 1024, K = 12, in 93 us, two with 50 spilled registers in 108 us)
template <int PER>
constexpr int reg8_waves()
{
    return PER == 6 ? 4 : reg_waves<1024, PER>();
}

template <bool ZT, int PER>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(reg8_waves<PER>(), reg8_waves<PER>()))) void stripe_reduce_reg8_kernel(
    StripeSources src, float* stripe_res, char* q_out, float* agg_out, RegGeom c)
{
    constexpr uint32_t T = 1024, NW = T / 64, S = 8;
    extern __shared__ f32x4 smem_v4[];
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    float* dec = reinterpret_cast<float*>(words + c.nq); // [0, 8): level of a cleared bit per worker slot, [8, 16): of a set bit
    uint32_t* tab = reinterpret_cast<uint32_t*>(red) + stripe_reg8_table_offset(c);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * c.rows;
    const size_t rec = (size_t) blockIdx.x * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0u;
    float* sres = stripe_res + base;
    const uint32_t head = (4u - (uint32_t) ((reinterpret_cast<uintptr_t>(sres) >> 2) & 3u)) & 3u;
    const uint32_t pieces = (c.rows - head) >> 2;
    const uint32_t tail = c.rows - head - 4 * pieces;
    const bool has_edge = tid < head + tail;
    const uint32_t edge_at = tid < head ? tid : c.rows - tail + (tid - head);
    const uint32_t shift = column_shift(sres + head, c.line_shift);

    // -0 is the additive identity (x + -0 = x for every x, signed zeros included)
    f32x4 a[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u)
        a[u] = f32x4{-0.0f, -0.0f, -0.0f, -0.0f};
    float edge = -0.0f;
    const uint32_t K = src.workers;
    for (uint32_t n0 = 0; n0 < K; n0 += S)
    {
        const uint32_t G = min(S, K - n0);
        if (n0 != 0)
            __syncthreads(); // everyone has decoded the previous group
        for (uint32_t g = 0; g < S; ++g)
        {
            if (tid == 64 * g) // one lane of a wavefront of its own per worker slot; an empty slot decodes to -0
            {
                float v0 = -0.0f, v1 = -0.0f;
                if (g < G)
                {
                    const float* h = reinterpret_cast<const float*>(src.q[stripe_order(n0 + g, src.owner)] + rec);
                    const float lo = h[0];
                    const float uf = make_ufactor<1>(lo, h[1]);
                    v0 = unquantize_value<1>(uf, lo, 0u);
                    v1 = unquantize_value<1>(uf, lo, 1u);
                }
                dec[g] = v0;
                dec[S + g] = v1;
            }
        }
        for (uint32_t g0 = 0; g0 < G; g0 += 4)
        {
            const uint32_t* from[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                from[j] = reinterpret_cast<const uint32_t*>(src.q[stripe_order(n0 + min(g0 + j, G - 1), src.owner)] + rec) + 2;
            for (uint32_t x = tid; x < c.nq; x += 4 * T)
            {
                uint32_t v[4][4];
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j)
#pragma unroll
                    for (uint32_t u = 0; u < 4; ++u)
                        v[j][u] = from[j][(x + T * u < c.nq) ? x + T * u : x];
#pragma unroll
                for (uint32_t u = 0; u < 4; ++u)
                {
                    const uint32_t w = x + T * u;
                    if (w < c.nq)
                    {
                        uint32_t* to = tab + (w >> 2) * kStripe8Row + (w & 3u) * S + g0;
#pragma unroll
                        for (uint32_t j = 0; j < 4; ++j)
                            if (g0 + j < G)
                                to[j] = v[j][u];
                    }
                }
            }
        }
        __syncthreads();
        float val0[S], val1[S];
#pragma unroll
        for (uint32_t g = 0; g < S; ++g)
        {
            val0[g] = dec[g];
            val1[g] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(dec[S + g])));
        }
        // (opaque: the positions of all slots do not depend on the group, and hoisted out of this loop they would be held
        // in registers for its whole duration; the sums alone take 100 of a thread's 128 registers at 100000 rows)
        const uint32_t t = opaque(tid);
        const uint32_t ufirst = t < shift ? 1u : 0u;
        uint32_t k, w;
        {
            const uint32_t e0 = head + 4 * (t + T * ufirst - shift);
            k = e0 / c.nq;
            w = e0 - k * c.nq;
        }
        // With the last group the stripe residual is added piece by piece: a piece's residual is requested before its
        // decoding and used after it, so that the memory latency runs under the arithmetic of this and the other
        // wavefronts (one workgroup fills a CU: nothing else would overlap the two phases).
        const bool last = n0 + S >= K;
        const f32x4* r4 = reinterpret_cast<const f32x4*>(sres + head);
        float* ag = agg_out != nullptr ? agg_out + base : nullptr;
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            if (slot_valid(t + T * u, shift, pieces))
            {
                f32x4 rr = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                if (last)
                    rr = __builtin_nontemporal_load(r4 + (t + T * u - shift));
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    // element e of the piece: QWord w + e at bit k, or past the last QWord the next bit of the first ones
                    uint32_t we = w + e, ke = k;
                    if (we >= c.nq)
                    {
                        we -= c.nq;
                        ++ke;
                    }
                    // byte offset of the eight workers' copies of QWord we: row (we / 4) of 144 bytes, 32 bytes per QWord
                    const uint32_t row = we >> 2;
                    const uint32_t off = (row << 7) + (row << 4) + ((we & 3u) << 5);
                    const char* at = reinterpret_cast<const char*>(tab) + off;
                    const u32x4 lo4 = *reinterpret_cast<const u32x4*>(at);
                    const u32x4 hi4 = *reinterpret_cast<const u32x4*>(at + 16);
                    // all eight slots, always: an empty slot's levels are both -0 and leave the sum as it is
                    float acc = a[u][e];
                    acc = pick_level_s(lo4.x, ke, val0[0], val1[0]) + acc;
                    acc = pick_level_s(lo4.y, ke, val0[1], val1[1]) + acc;
                    acc = pick_level_s(lo4.z, ke, val0[2], val1[2]) + acc;
                    acc = pick_level_s(lo4.w, ke, val0[3], val1[3]) + acc;
                    acc = pick_level_s(hi4.x, ke, val0[4], val1[4]) + acc;
                    acc = pick_level_s(hi4.y, ke, val0[5], val1[5]) + acc;
                    acc = pick_level_s(hi4.z, ke, val0[6], val1[6]) + acc;
                    acc = pick_level_s(hi4.w, ke, val0[7], val1[7]) + acc;
                    a[u][e] = acc;
                }
                if (last)
                {
                    if (ag != nullptr)
                    {
                        const uint32_t p = t + T * u - shift;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            ag[head + 4 * p + e] = a[u][e];
                    }
                    a[u] = a[u] + rr;
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
            const uint32_t at = opaque(edge_at);
            const uint32_t edge_k = at / c.nq;
            const uint32_t edge_w = at - edge_k * c.nq;
            const uint32_t* p = tab + (edge_w >> 2) * kStripe8Row + (edge_w & 3u) * S;
            for (uint32_t g = 0; g < G; ++g)
                edge = pick_level(p[g], edge_k, dec[g], dec[S + g]) + edge;
        }
    }
    if (has_edge)
    {
        if (agg_out != nullptr)
            agg_out[base + edge_at] = edge;
        edge = edge + sres[edge_at];
    }
    reg_stats_pack<1, ZT, T, PER>(a, edge, has_edge, edge_at, head, pieces, shift, c, red, red_u, words, sres, q_out + rec);
}

// ---- 1 bit, up to eight workers: the sum of a row looked up, not added up ----------------------------------------------
//
// With K <= 8 workers the aggregate of an element is one of 256 values: the levels of the K columns' headers added up in
// the summation order (owner first), picked by the K bits of the element. A workgroup builds that table once per column
// (256 entries, each with the additions of the decoding loop in their order, hence the same bits) and turns the workers'
// QWords into one byte per element: bit g of the byte = the element's bit in the stripe of the g-th worker of the order.
// The bytes lie in element order (QWord w of bit position k holds element k * nq + w), so the four elements of a piece are
// one aligned dword (the table is shifted by the column's `head`) and need no position arithmetic at all. Decoding an
// element is a bit-field extract, an address and an LDS read where the kernels above spend three instructions per worker;
// the transposition costs about five per element (8 x 8 bit blocks, three exchange steps each).
// LDS: [48 reduction slots | nq output QWords | 256 sums | rows + 8 bytes].

__host__ __device__ inline uint32_t stripe_lut_bytes_offset(const RegGeom& c) // in dwords
{
    return (kRegRedSlots + c.nq + 256u + 3u) & ~3u;
}

__host__ __device__ inline size_t stripe_lut_lds_bytes(const RegGeom& c)
{
    return (size_t) stripe_lut_bytes_offset(c) * 4 + (((size_t) c.rows + 8 + 15) & ~(size_t) 15);
}

template <bool ZT, int PER, int TT = 1024>
__device__ __forceinline__ void stripe_reduce_lut_body(const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, const RegGeom& c,
                                                       uint32_t column, f32x4* smem_v4)
{
    constexpr uint32_t T = TT, NW = T / 64, S = 8;
    static_assert(T >= 256, "one thread per table entry");
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    float* lut = reinterpret_cast<float*>(words + c.nq);
    uint8_t* pat = reinterpret_cast<uint8_t*>(reinterpret_cast<uint32_t*>(red) + stripe_lut_bytes_offset(c));
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * c.rows;
    const size_t rec = (size_t) column * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0u;
    float* sres = stripe_res + base;
    const uint32_t head = (4u - (uint32_t) ((reinterpret_cast<uintptr_t>(sres) >> 2) & 3u)) & 3u;
    const uint32_t pieces = (c.rows - head) >> 2;
    const uint32_t tail = c.rows - head - 4 * pieces;
    const bool has_edge = tid < head + tail;
    const uint32_t edge_at = tid < head ? tid : c.rows - tail + (tid - head);
    const uint32_t shift = column_shift(sres + head, c.line_shift);
    const uint32_t K = src.workers; // at most 8
    // element i has its byte at pat[i + lead]: piece p (elements head + 4 p ...) is the aligned dword 4 p + lead + head
    const uint32_t lead = (4u - head) & 3u;

    // The stripe residual is requested first: its latency runs under the table building below (one workgroup fills a CU,
    // nothing else would overlap the two), and a sum plus its residual is the same bits in either order. The tallest
    // columns, whose residual would leave the table building no registers, request it piece by piece at the look-ups,
    // and so does the one shape that has two workgroups per CU only within 64 registers.
    constexpr bool EARLY = PER <= 20 && !(PER == 6 && TT == 1024);
    f32x4 a[PER];
    const f32x4* r4 = reinterpret_cast<const f32x4*>(sres + head);
    if constexpr (EARLY)
    {
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            a[u] = f32x4{-0.0f, -0.0f, -0.0f, -0.0f};
            if (slot_valid(t + T * u, shift, pieces))
                a[u] = __builtin_nontemporal_load(r4 + (t + T * u - shift));
        }
    }

    // this thread's first QWords are requested before the table of sums is built, so that headers and QWords cost one round
    // trip to memory, not two
    const uint32_t* from[S];
#pragma unroll
    for (uint32_t g = 0; g < S; ++g)
        from[g] = reinterpret_cast<const uint32_t*>(src.q[stripe_order(min(g, K - 1), src.owner)] + rec) + 2;
    uint32_t first[S];
#pragma unroll
    for (uint32_t g = 0; g < S; ++g)
        first[g] = from[g][min(tid, c.nq - 1)];

    // the 256 sums: entry x adds, in the order of the summation, the level each worker's header gives for its bit of x,
    // starting from -0 (x + -0 = x for every x, signed zeros included), as unquantize ... unquantize-and-add would
    if (tid < 256)
    {
        // (all headers requested together: a loop over the K workers would wait for each in turn)
        f32x2 h[S];
#pragma unroll
        for (uint32_t g = 0; g < S; ++g)
            h[g] = *reinterpret_cast<const f32x2_u*>(src.q[stripe_order(min(g, K - 1), src.owner)] + rec);
        float acc = -0.0f;
#pragma unroll
        for (uint32_t g = 0; g < S; ++g)
        {
            if (g < K)
            {
                const float uf = make_ufactor<1>(h[g].x, h[g].y);
                acc = unquantize_value<1>(uf, h[g].x, (tid >> g) & 1u) + acc;
            }
        }
        lut[tid] = acc;
    }
    // the workers' QWords, transposed into one byte per element
    {
        for (uint32_t x = tid; x < c.nq; x += T)
        {
            uint32_t d[S];
#pragma unroll
            for (uint32_t g = 0; g < S; ++g)
                d[g] = x == tid ? first[g] : from[g][x];
#pragma unroll
            for (uint32_t g = 0; g < S; ++g)
                d[g] = g < K ? d[g] : 0u;
            uint8_t* to = pat + lead + x;
#pragma unroll 1 // (one block at a time: most registers are taken by the residual by now)
            for (uint32_t j = 0; j < 4; ++j)
            {
                // byte j of every worker's QWord: an 8 x 8 block of (worker, bit position 8 j ...)
                const uint32_t sel = 0x0C0C0000u | ((4u + j) << 8) | j; // byte 0: byte j of the second operand, byte 1: of the first
                uint32_t lo = __builtin_amdgcn_perm(d[1], d[0], sel) | (__builtin_amdgcn_perm(d[3], d[2], sel) << 16);
                uint32_t hi = __builtin_amdgcn_perm(d[5], d[4], sel) | (__builtin_amdgcn_perm(d[7], d[6], sel) << 16);
                transpose_bits_8x8(lo, hi);
#pragma unroll
                for (uint32_t r = 0; r < 8; ++r)
                {
                    const uint32_t k = 8 * j + r;
                    const uint32_t i = k * c.nq + x;
                    if (i < c.rows)
                        to[k * c.nq] = (uint8_t) ((r < 4 ? lo : hi) >> (8 * (r & 3u)));
                }
            }
        }
    }
    __syncthreads();

    float edge = -0.0f;
    {
        const uint32_t t = opaque(tid);
        const uint32_t* pat4 = reinterpret_cast<const uint32_t*>(pat + lead + head);
        float* ag = agg_out != nullptr ? agg_out + base : nullptr;
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            if constexpr (!EARLY)
                a[u] = f32x4{-0.0f, -0.0f, -0.0f, -0.0f};
            if (slot_valid(t + T * u, shift, pieces))
            {
                const uint32_t p = t + T * u - shift;
                if constexpr (!EARLY)
                    a[u] = __builtin_nontemporal_load(r4 + p); // requested before the look-ups, used after them
                const uint32_t four = pat4[p];
                f32x4 v;
                v[0] = lut[four & 255u];
                v[1] = lut[(four >> 8) & 255u];
                v[2] = lut[(four >> 16) & 255u];
                v[3] = lut[four >> 24];
                if (ag != nullptr)
                {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        ag[head + 4 * p + e] = v[e];
                }
                a[u] = v + a[u];
            }
        }
        if (has_edge)
        {
            edge = lut[pat[lead + edge_at]];
            if (agg_out != nullptr)
                agg_out[base + edge_at] = edge;
            edge = edge + sres[edge_at];
        }
    }
    reg_stats_pack<1, ZT, T, PER>(a, edge, has_edge, edge_at, head, pieces, shift, c, red, red_u, words, sres, q_out + rec);
}

// The register budget of the look-up kernel: that of the other register kernels, except at six pieces per thread, where
// their eight wavefronts per SIMD (64 registers) made it spill 512 registers' worth (6144 x 3101, K = 8: 548 us instead of
// 39 us). With 256 threads it gets the 74 it needs (six wavefronts); with 1024 threads it keeps eight -- two workgroups per
// CU -- and fits by requesting the residual at the look-ups (20000 x 2048, K = 8: 83 us; 113 us with one workgroup per CU).
template <int T, int PER>
constexpr int lut_waves()
{
    return PER == 6 && T != 1024 ? 6 : reg_waves<T, PER>();
}

template <bool ZT, int PER, int TT = 1024>
__global__ __launch_bounds__(TT) __attribute__((amdgpu_waves_per_eu(lut_waves<TT, PER>(), lut_waves<TT, PER>()))) void stripe_reduce_lut_kernel(
    StripeSources src, float* stripe_res, char* q_out, float* agg_out, RegGeom c)
{
    extern __shared__ f32x4 smem_v4[];
    stripe_reduce_lut_body<ZT, PER, TT>(src, stripe_res, q_out, agg_out, c, blockIdx.x, smem_v4);
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
