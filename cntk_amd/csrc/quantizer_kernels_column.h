// gfx950 kernels of the per-column gradient quantizer: one workgroup per column, the column in LDS,
// for quantize and for the stripe reduction.
#pragma once

#include "quantizer_kernels_tile.h"

namespace cntkq {

// ---- quantize, 1 bit, one workgroup per column, rows = 1024 * PER (PER = 1, 2, 4) ---------------------------
//
// 256 threads own one column: each loads PER 16-byte pieces of gradient and residual, adds them into an LDS copy
// of the column and sums its own values on the way, so the column mean needs no second pass. The split sums are
// then taken from LDS (thread t takes rows t, t + 256, ...), and the codes are packed from LDS by work items of
// (QWord, run of 4 * PER bit positions), whose partial words meet in LDS. Few registers and 4..16 KB of LDS per
// workgroup keep 8 workgroups resident per CU; that, not wider stores, is what brings this kernel to the rate of a
// plain read-read-write stream.

constexpr uint32_t kColThreads = 256;

struct ColLds
{
    float* tile;      // 1024 * PER floats, 16-byte aligned
    uint32_t* words;  // 32 * PER partial QWords
    float* red_f;     // 2 * 4 floats: the split sums of the four wavefronts
    uint32_t* red_u;  // 4: their counts
    float* red_m;     // 4: the wavefronts' sums for the mean (slots of their own: no barrier between reading these and writing the others)
};

template <int PER>
__device__ __forceinline__ ColLds col_lds(f32x4* smem)
{
    ColLds l;
    l.tile = reinterpret_cast<float*>(smem);
    l.words = reinterpret_cast<uint32_t*>(l.tile + 1024 * PER);
    l.red_f = reinterpret_cast<float*>(l.words + 32 * PER);
    l.red_u = reinterpret_cast<uint32_t*>(l.red_f + 8);
    l.red_m = reinterpret_cast<float*>(l.red_u + 4);
    return l;
}

template <int PER>
constexpr size_t col_lds_bytes()
{
    return (size_t) (1024 * PER + 32 * PER + 8 + 4 + 4) * 4;
}

// LDS of the stripe reduction beyond col_lds_bytes: two levels per worker (up to kMaxWorkers), or, with up to eight
// workers, their sixteen levels and the 256 sums they can add up to
constexpr size_t kStripeColExtraLds = (2 * 8 + 256) * 4 > 2 * kMaxWorkers * 4 ? (2 * 8 + 256) * 4 : 2 * kMaxWorkers * 4;

// The 1-bit split sums of one 16-byte piece (x y z w in order): values below the mean go to s0 / n0, the others to s1.
// Like the column sum, the split sums are taken piece by piece by every column kernel, whether it keeps the column in
// LDS or in registers, so that all of them give the same header for the same column.
__device__ __forceinline__ void split_add_piece(const f32x4& v, float mean, float& s0, float& s1, uint32_t& n0)
{
#pragma unroll
    for (int c = 0; c < 4; ++c)
    {
        const float x = v[c];
        const bool below = x < mean;
        s0 += below ? x : 0.0f;
        s1 += below ? 0.0f : x;
        n0 += below ? 1u : 0u;
    }
}

// Sum of the values thread tid holds when the column is cut into 16-byte pieces tid, tid + 256, ...: in that order,
// x y z w within a piece. Both the quantize and the stripe-reduction kernel take the column mean from these
// per-thread sums, so they produce identical headers for identical columns.
template <int PER>
__device__ __forceinline__ float col_thread_sum(const f32x4 (&v)[PER])
{
    float s = 0.0f;
#pragma unroll
    for (int u = 0; u < PER; ++u)
    {
        s += v[u].x;
        s += v[u].y;
        s += v[u].z;
        s += v[u].w;
    }
    return s;
}

// Statistics, header, codes and residual of the column held in l.tile. csum: this thread's col_thread_sum
// (ignored when ZT). l.words[0 .. 32 * PER) must be zero; no barrier is needed between writing l.tile / l.words
// and calling this. res_col: the column of the residual output; qc: the packed column record (8-byte aligned).
template <bool ZT, int PER>
__device__ __forceinline__ void col_stats_pack(const ColLds& l, float csum, float* res_col, char* qc)
{
    constexpr uint32_t ROWS = 1024 * PER, NQ = 32 * PER, T = kColThreads, NW = T / 64;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    float mean = 0.0f;
    if constexpr (!ZT)
    {
        const float s = wave_sum(csum);
        if (lane == 0)
            l.red_m[wave] = s;
    }
    __syncthreads(); // the column and the wave sums are visible
    if constexpr (!ZT)
    {
        float s = l.red_m[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
            s += l.red_m[x];
        mean = s / (float) ROWS;
    }
    float s0 = 0.0f, s1 = 0.0f;
    uint32_t n0 = 0;
    {
        const f32x4* t4 = reinterpret_cast<const f32x4*>(l.tile);
#pragma unroll
        for (uint32_t u = 0; u < PER; ++u)
            split_add_piece(t4[tid + T * u], mean, s0, s1, n0);
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    n0 = wave_sum(n0);
    if (lane == 0)
    {
        l.red_f[wave] = s0;
        l.red_f[4 + wave] = s1;
        l.red_u[wave] = n0;
    }
    __syncthreads();
    float S0 = l.red_f[0], S1 = l.red_f[4];
    uint32_t N0 = l.red_u[0];
#pragma unroll
    for (uint32_t x = 1; x < NW; ++x)
    {
        S0 += l.red_f[x];
        S1 += l.red_f[4 + x];
        N0 += l.red_u[x];
    }
    float lo, hi;
    finish_stats_1bit<ZT>(mean, S0, S1, N0, ROWS - N0, ROWS, lo, hi);
    if (tid == 0)
    {
        f32x2 h;
        h.x = lo;
        h.y = hi;
        *reinterpret_cast<f32x2*>(qc) = h;
    }
    const ValueQ vq = make_vq<1>(lo, hi);
    const float val0 = unquantize_value<1>(vq, 0u);
    const float val1 = unquantize_value<1>(vq, 1u);
    // work item = (QWord p, chunk of KS bit positions); NQ * (32 / KS) = 256 items
    constexpr uint32_t KS = 4 * PER;
    const uint32_t p = tid % NQ, chunk = tid / NQ;
    uint32_t word = 0;
#pragma unroll
    for (uint32_t kk = 0; kk < KS; ++kk)
    {
        const uint32_t k = chunk * KS + kk;
        const uint32_t i = p + NQ * k;
        const float x = l.tile[i];
        const uint32_t code = quantize_value<1, ZT>(vq, x);
        __builtin_nontemporal_store(x - (code ? val1 : val0), res_col + i);
        word |= code << k;
    }
    atomicOr(&l.words[p], word);
    __syncthreads();
    if (tid < NQ)
        reinterpret_cast<uint32_t*>(qc + 8)[tid] = l.words[tid];
}

template <bool ZT, int PER>
__device__ __forceinline__ void quantize_col_body(const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q,
                                                  uint64_t qcol, uint32_t column, f32x4* smem_v4)
{
    constexpr uint32_t ROWS = 1024 * PER, T = kColThreads;
    const ColLds l = col_lds<PER>(smem_v4);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * ROWS;
    if (tid < 32 * PER)
        l.words[tid] = 0u;
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g + base);
    const f32x4* r4 = reinterpret_cast<const f32x4*>(r_in + base);
    f32x4* t4 = reinterpret_cast<f32x4*>(l.tile);
    f32x4 a[PER], b[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u)
    {
        a[u] = __builtin_nontemporal_load(g4 + tid + T * u);
        b[u] = __builtin_nontemporal_load(r4 + tid + T * u);
    }
#pragma unroll
    for (int u = 0; u < PER; ++u)
    {
        a[u] = a[u] + b[u];
        t4[tid + T * u] = a[u];
    }
    // the whole column has been read before col_stats_pack's first barrier, so r_out may be r_in
    col_stats_pack<ZT, PER>(l, col_thread_sum<PER>(a), r_out + base, q + (size_t) column * qcol);
}

template <bool ZT, int PER>
__global__ __launch_bounds__(kColThreads) void quantize_col_kernel(const float* __restrict__ g, const float* r_in, float* r_out,
                                                                   char* __restrict__ q, uint64_t qcol)
{
    extern __shared__ f32x4 smem_v4[];
    quantize_col_body<ZT, PER>(g, r_in, r_out, q, qcol, blockIdx.x, smem_v4);
}

// Consecutive workgroups go to the device's eight dies in turn, each die with an L2 of its own. A packed column record is
// not a whole number of 128-byte lines (264 bytes at 2048 rows), so neighbouring columns share lines, and neighbours on
// different dies fetch such a line into two L2s (2048 x 9304, eight workers: 29 MB read for 19.6 MB of packed stripes).
// Runs of 16 consecutive columns therefore go to one die; the eight dies still walk through memory side by side, a
// megabyte of residual at a time. Maps workgroup b of n to its column (the last n % 128 keep their index).
__device__ __forceinline__ uint32_t column_of_workgroup(uint32_t b, uint32_t n)
{
    constexpr uint32_t RUN = 16, DIES = 8;
    const uint32_t whole = n - n % (RUN * DIES);
    if (b >= whole)
        return b;
    const uint32_t die = b % DIES, slot = b / DIES;
    return ((slot / RUN) * DIES + die) * RUN + slot % RUN;
}

// Stripe reduction in the same shape, up to eight workers: the sum of an element is one of 256 values, picked by the
// workers' bits of the element. The work item that will pack (QWord p, chunk) turns that QWord of every worker into one
// byte per bit position (bit u = worker u) by an 8 x 8 bit transposition and looks the sums up in a table that the
// workgroup's 256 threads build, one entry each, by the additions of the plain decoding loop in its order (owner first,
// then ascending rank; seeded with -0, and -0 for a worker that is skipped: x + -0 = x for every x): a bit-field extract
// and an LDS read per element instead of three instructions per worker and element.
// A stripe can be one GPU's share of a matrix, a single round of workgroups whose time is the length of one workgroup's
// chain of dependent steps, so everything a thread needs from memory is requested at once, before the first barrier, and
// nothing in those requests depends on anything but the kernel's arguments: the workers' records are read in worker
// order (whoever the owner is; the order of the additions is the table's business), so that their addresses come from
// one scalar load instead of eight dependent ones, and the lane that decodes worker u's header picks that worker's
// address out of registers instead of loading it.
template <bool ZT, int PER>
__device__ __forceinline__ void stripe_reduce_col_lookup(const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint64_t qcol,
                                                         uint32_t column, f32x4* smem_v4)
{
    constexpr uint32_t ROWS = 1024 * PER, NQ = 32 * PER, T = kColThreads, KS = 4 * PER, W = 8;
    const ColLds l = col_lds<PER>(smem_v4);
    float* dec = l.red_m + 4; // two reconstruction levels per worker, in worker order
    float* lut = dec + 2 * W;
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * ROWS;
    const size_t rec = (size_t) column * qcol;
    const uint32_t K = src.workers, owner = src.owner;
    if (tid < NQ)
        l.words[tid] = 0u;
    const uint32_t p = tid % NQ, chunk = tid / NQ;
    const uint32_t sh0 = chunk * KS;
    // (beyond the last worker: worker 0's record, fetched and not used)
    const char* record[W];
#pragma unroll
    for (uint32_t u = 0; u < W; ++u)
        record[u] = (u < K ? src.q[u] : src.q[0]) + rec;
    uint32_t word[W];
#pragma unroll
    for (uint32_t u = 0; u < W; ++u)
        word[u] = reinterpret_cast<const uint32_t*>(record[u] + 8)[p];
    const float* sp = stripe_res + base;
    float resid[KS];
#pragma unroll
    for (uint32_t kk = 0; kk < KS; ++kk)
        resid[kk] = __builtin_nontemporal_load(sp + p + NQ * (sh0 + kk));
    if (tid < K)
    {
        const char* mine = record[0];
#pragma unroll
        for (uint32_t u = 1; u < W; ++u)
            mine = tid == u ? record[u] : mine;
        const float* h = reinterpret_cast<const float*>(mine);
        const ValueQ vq = make_vq<1>(h[0], h[1]);
        dec[2 * tid] = unquantize_value<1>(vq, 0u);
        dec[2 * tid + 1] = unquantize_value<1>(vq, 1u);
    }
    __syncthreads();
    {
        float a = dec[2 * owner + ((tid >> owner) & 1u)] + -0.0f;
#pragma unroll
        for (uint32_t u = 0; u < W; ++u)
        {
            const float x = dec[2 * u + ((tid >> u) & 1u)];
            a = ((u < K && u != owner) ? x : -0.0f) + a;
        }
        lut[tid] = a;
    }
    // the bytes that index the table do not need it yet
    uint32_t index[(KS + 7) / 8][2];
#pragma unroll
    for (uint32_t b = 0; b < (KS + 7) / 8; ++b)
    {
        uint32_t row[W];
#pragma unroll
        for (uint32_t u = 0; u < W; ++u)
            row[u] = word[u] >> (sh0 + 8 * b);
        // byte 0 of the second operand, byte 0 of the first, zeros
        uint32_t lo = __builtin_amdgcn_perm(row[1], row[0], 0x0C0C0400u) | (__builtin_amdgcn_perm(row[3], row[2], 0x0C0C0400u) << 16);
        uint32_t hi = __builtin_amdgcn_perm(row[5], row[4], 0x0C0C0400u) | (__builtin_amdgcn_perm(row[7], row[6], 0x0C0C0400u) << 16);
        transpose_bits_8x8(lo, hi);
        index[b][0] = lo;
        index[b][1] = hi;
    }
    __syncthreads();
    float acc[KS];
#pragma unroll
    for (uint32_t kk = 0; kk < KS; ++kk)
        acc[kk] = lut[(index[kk / 8][(kk & 7u) < 4 ? 0 : 1] >> (8 * (kk & 3u))) & 255u];
#pragma unroll
    for (uint32_t kk = 0; kk < KS; ++kk)
    {
        const uint32_t i = p + NQ * (sh0 + kk);
        if (agg_out != nullptr)
            agg_out[base + i] = acc[kk];
        l.tile[i] = acc[kk] + resid[kk];
    }
    float csum = 0.0f;
    if constexpr (!ZT)
    {
        __syncthreads();
        const f32x4* t4 = reinterpret_cast<const f32x4*>(l.tile);
        f32x4 v[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u)
            v[u] = t4[tid + T * u];
        csum = col_thread_sum<PER>(v);
    }
    col_stats_pack<ZT, PER>(l, csum, stripe_res + base, q_out + rec);
}

// More than eight workers: the work item that will pack (QWord p, chunk) decodes those bit positions from every worker's
// packed stripe, eight workers at a time, sums them (owner first, then ascending) and adds the stripe residual.
template <bool ZT, int PER>
__device__ __forceinline__ void stripe_reduce_col_body(const StripeSources& src, float* stripe_res, char* q_out, float* agg_out, uint64_t qcol,
                                                       uint32_t column, f32x4* smem_v4)
{
    constexpr uint32_t ROWS = 1024 * PER, NQ = 32 * PER, T = kColThreads, KS = 4 * PER, BATCH = 8;
    const uint32_t K = src.workers;
    if (K <= BATCH)
    {
        stripe_reduce_col_lookup<ZT, PER>(src, stripe_res, q_out, agg_out, qcol, column, smem_v4);
        return;
    }
    const ColLds l = col_lds<PER>(smem_v4);
    float* dec = l.red_m + 4; // two reconstruction levels per worker, in summation order
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * ROWS;
    const size_t rec = (size_t) column * qcol;
    if (tid < NQ)
        l.words[tid] = 0u;
    const uint32_t p = tid % NQ, chunk = tid / NQ;
    const uint32_t sh0 = chunk * KS;
    uint32_t word[BATCH];
#pragma unroll
    for (uint32_t u = 0; u < BATCH; ++u)
        word[u] = reinterpret_cast<const uint32_t*>(src.q[stripe_order(u, src.owner)] + rec + 8)[p];
    const float* sp = stripe_res + base;
    float resid[KS];
#pragma unroll
    for (uint32_t kk = 0; kk < KS; ++kk)
        resid[kk] = __builtin_nontemporal_load(sp + p + NQ * (sh0 + kk));
    if (tid < K)
    {
        const float* h = reinterpret_cast<const float*>(src.q[stripe_order(tid, src.owner)] + rec);
        const ValueQ vq = make_vq<1>(h[0], h[1]);
        dec[2 * tid] = unquantize_value<1>(vq, 0u);
        dec[2 * tid + 1] = unquantize_value<1>(vq, 1u);
    }
    __syncthreads();

    float acc[KS];
    for (uint32_t n0 = 0; n0 < K; n0 += BATCH)
    {
        if (n0 != 0)
        {
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
                if (n0 + u < K)
                    word[u] = reinterpret_cast<const uint32_t*>(src.q[stripe_order(n0 + u, src.owner)] + rec + 8)[p];
        }
#pragma unroll
        for (uint32_t u = 0; u < BATCH; ++u)
        {
            if (n0 + u < K)
            {
                const float val0 = dec[2 * (n0 + u)], val1 = dec[2 * (n0 + u) + 1];
                const uint32_t bits = word[u] >> sh0;
#pragma unroll
                for (uint32_t kk = 0; kk < KS; ++kk)
                {
                    const float x = pick_level(bits, kk, val0, val1);
                    // the first term (the owner's) seeds the sum; afterwards: decoded value + running sum
                    acc[kk] = (n0 + u == 0) ? x : x + acc[kk];
                }
            }
        }
    }
#pragma unroll
    for (uint32_t kk = 0; kk < KS; ++kk)
    {
        const uint32_t i = p + NQ * (sh0 + kk);
        if (agg_out != nullptr)
            agg_out[base + i] = acc[kk];
        l.tile[i] = acc[kk] + resid[kk];
    }
    float csum = 0.0f;
    if constexpr (!ZT)
    {
        __syncthreads();
        const f32x4* t4 = reinterpret_cast<const f32x4*>(l.tile);
        f32x4 v[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u)
            v[u] = t4[tid + T * u];
        csum = col_thread_sum<PER>(v);
    }
    col_stats_pack<ZT, PER>(l, csum, stripe_res + base, q_out + rec);
}

template <bool ZT, int PER>
__global__ __launch_bounds__(kColThreads) void stripe_reduce_col_kernel(StripeSources src, float* stripe_res, char* q_out,
                                                                        float* agg_out, uint64_t qcol)
{
    extern __shared__ f32x4 smem_v4[];
    stripe_reduce_col_body<ZT, PER>(src, stripe_res, q_out, agg_out, qcol, column_of_workgroup(blockIdx.x, gridDim.x), smem_v4);
}

// A few stripes of one shape in one grid, everything a workgroup needs to find its column in the kernel's arguments: the
// stripes of all the ranks of a small cluster simulated in one GPU's memory. The table-driven launch for whole gradient
// sets (stripe_reduce_batch_kernel) finds a workgroup's stripe by two dependent reads of device memory before the first
// load of data goes out, which a workgroup that lives a few microseconds notices (8 x 1163 columns of 2048 rows: 38 us
// against 32 us for the same columns as one stripe).
constexpr uint32_t kStripeSetMax = 8; // stripes per launch, and workers per stripe
struct StripeColSet
{
    const char* q[kStripeSetMax][kStripeSetMax]; // [stripe][worker]; beyond the last worker: null
    float* stripe_res[kStripeSetMax];
    char* q_out[kStripeSetMax];
    float* agg_out[kStripeSetMax];
    uint32_t begin[kStripeSetMax + 1]; // first workgroup of every stripe; begin[count] = the grid; beyond: 0xFFFFFFFF
    uint32_t owner[kStripeSetMax];
    uint32_t count;
    uint32_t workers;
    uint64_t qcol;
};

template <bool ZT, int PER>
__global__ __launch_bounds__(kColThreads) void stripe_reduce_col_set_kernel(StripeColSet set)
{
    extern __shared__ f32x4 smem_v4[];
    uint32_t e = 0;
#pragma unroll
    for (uint32_t i = 1; i < kStripeSetMax; ++i)
        e += blockIdx.x >= set.begin[i] ? 1u : 0u;
    StripeSources src;
#pragma unroll
    for (uint32_t u = 0; u < kStripeSetMax; ++u)
        src.q[u] = set.q[e][u];
    src.workers = set.workers;
    src.owner = set.owner[e];
    const uint32_t column = column_of_workgroup(blockIdx.x - set.begin[e], set.begin[e + 1] - set.begin[e]);
    stripe_reduce_col_lookup<ZT, PER>(src, set.stripe_res[e], set.q_out[e], set.agg_out[e], set.qcol, column, smem_v4);
}

// ---- the same decomposition for any bit width and any column height that is a multiple of 4 ----------------
//
// One workgroup of 256 threads per column, the column in LDS. The running statistic (sum for 1 bit, sum of squares
// otherwise) is taken piece by piece while loading, in the order col_thread_sum defines, so for 1 bit and 1024 * PER
// rows these kernels give the very bytes of the unrolled ones above.

// How a column's 16-byte pieces are dealt to the slots of a workgroup (slot v = thread + T * u). With line_shift set,
// slot v holds piece v - shift, shift = the column's offset into its 128-byte line in pieces (the residual input's
// address decides; the launch sets line_shift only when gradient and residual output share that offset).
__device__ __forceinline__ uint32_t column_shift(const void* column, uint32_t line_shift)
{
    return line_shift ? (uint32_t) ((reinterpret_cast<uintptr_t>(column) >> 4) & 7u) : 0u;
}

__device__ __forceinline__ bool slot_valid(uint32_t v, uint32_t shift, uint32_t pieces)
{
    return v >= shift && v - shift < pieces;
}

// the piece a slot loads: its own, or (outside the column) the column's first or last
__device__ __forceinline__ uint32_t slot_piece(uint32_t v, uint32_t shift, uint32_t last)
{
    const uint32_t p = v < shift ? 0u : v - shift;
    return p < last ? p : last;
}

struct ColGeom
{
    uint32_t rows;   // multiple of 4
    uint32_t nq;
    uint32_t pieces; // rows / 4
    uint32_t line_shift; // non-zero: statistics are summed in the order of line-aligned slots (see column_shift)
    uint64_t qcol;
};

// LDS: [stripe reductions: the first workers' decoding tables | column | partial QWords (nq when a QWord has several work
// items) | kColgRedSlots reduction slots | stripe reductions: further workers' tables]; workers = 0: a quantize kernel
// Columns from this height on hand their residual back through LDS where a bit position's runs do not start on 128-byte
// lines (stripe reduction over 8 workers, staged against direct: 1152 x 16384 at 1 bit 63 against 60 us, 1536 x 12288 52
// against 48, 2304 x 8192 at 2 bits 48 against 46, 3000 x 6300 45.5 against 45.2, 4100 x 4600 at 4 bits 52 against 55,
// 5000 x 3800 46 against 48, 7000 x 2700 48 against 50, 9304 x 2048 at 2 bits 42 against 45)
constexpr uint32_t kColStageMinRows = 3073;
constexpr uint32_t kColgRedSlots = 16; // 4 + 4 split sums, 4 counts, 4 sums for the mean or the sum of squares
template <int NBITS>
__host__ __device__ inline size_t colg_lds_bytes(const ColGeom& c, uint32_t workers)
{
    return ((size_t) c.rows + (PackShape<NBITS>::CHUNKS > 1 ? c.nq : 0) + kColgRedSlots) * sizeof(float) + (workers != 0 ? stripe_dec_bytes(NBITS, workers) : 0);
}

template <int NBITS>
__device__ __forceinline__ float colg_add_piece(float s, const f32x4& v)
{
    if constexpr (NBITS == 1)
    {
        s += v.x;
        s += v.y;
        s += v.z;
        s += v.w;
    }
    else
    {
        s += v.x * v.x;
        s += v.y * v.y;
        s += v.z * v.z;
        s += v.w * v.w;
    }
    return s;
}

// which chunk of bit positions work item `it` of a column of nq QWords belongs to (chunk-major numbering), without a division
template <uint32_t CHUNKS>
__device__ __forceinline__ uint32_t chunk_of_item(uint32_t it, uint32_t nq)
{
    static_assert(CHUNKS <= 4, "up to four chunks per QWord");
    uint32_t chunk = 0;
    if constexpr (CHUNKS > 1)
        chunk += it >= nq ? 1u : 0u;
    if constexpr (CHUNKS > 2)
        chunk += it >= 2 * nq ? 1u : 0u;
    if constexpr (CHUNKS > 3)
        chunk += it >= 3 * nq ? 1u : 0u;
    return chunk;
}

// stat: this thread's running statistic over its pieces (unused for 1 bit with ZT). tile = the column, words = zeroed
// partial QWords, red = kColgRedSlots reduction slots. No barrier is needed between writing the column and calling this.
// WGT: threads in the workgroup, or 0 for "as launched" (any multiple of 64 from 256 on). The sums are always taken by the first 256 threads (their order is part of the result);
// coding and packing use all of them.
template <int NBITS, bool ZT, int WGT = kColThreads>
__device__ __forceinline__ void colg_stats_pack(float* tile, uint32_t* words, float* red, const ColGeom& c, float stat,
                                                uint32_t shift, float* res_col, char* qc)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t T = kColThreads, NW = T / 64;
    static_assert(WGT == 0 || (WGT >= (int) T && WGT % 64 == 0), "workgroup size");
    const uint32_t WG = WGT == 0 ? blockDim.x : (uint32_t) WGT;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 8);
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    float total = 0.0f;
    if constexpr (need_stat)
    {
        // (slots of their own: the split sums below are written without a barrier after these have been read)
        const float s = wave_sum(stat);
        if (lane == 0 && wave < NW)
            red[12 + wave] = s;
    }
    __syncthreads(); // the column and the wave sums are visible
    if constexpr (need_stat)
    {
        total = red[12];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
            total += red[12 + x];
    }
    float lo, hi;
    if constexpr (NBITS == 1)
    {
        const float mean = ZT ? 0.0f : total / (float) c.rows;
        float s0 = 0.0f, s1 = 0.0f;
        uint32_t n0 = 0;
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile);
        if (WGT == (int) T || tid < T)
            for (uint32_t v = tid; v < c.pieces + shift; v += T)
                if (v >= shift)
                    split_add_piece(t4[v - shift], mean, s0, s1, n0);
        s0 = wave_sum(s0);
        s1 = wave_sum(s1);
        n0 = wave_sum(n0);
        if (lane == 0 && wave < NW)
        {
            red[wave] = s0;
            red[4 + wave] = s1;
            red_u[wave] = n0;
        }
        __syncthreads();
        float S0 = red[0], S1 = red[4];
        uint32_t N0 = red_u[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
        {
            S0 += red[x];
            S1 += red[4 + x];
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
        // a record is only 4-byte aligned when the column has an odd number of QWords
        float* gh = reinterpret_cast<float*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const float val0 = unquantize_value<NBITS>(vq, 0u);
    const float val1 = unquantize_value<NBITS>(vq, 1u);
    uint32_t* bits = reinterpret_cast<uint32_t*>(qc + 8);
    const uint32_t items = c.nq * PS::CHUNKS;
    // A QWord's bit positions are nq elements apart; element i lies 4 * i bytes into the column, in LDS as in memory, so
    // one byte offset serves the read and the store (the column's address is the same for all threads and stays in scalar
    // registers). In a column of more than VPW * VPW rows only a QWord's last bit position can lie beyond the end: a work
    // item with all of its elements inside runs without a branch per element.
    const uint32_t step = c.nq * 4u, end = c.rows * 4u;
    // A wavefront's store of one bit position is a run of 256 bytes; where the runs of a column do not all start on 128-byte
    // lines (the column starts inside a line, or its QWords are not a multiple of 32) they end in partial lines, which the
    // memory writes by reading the line first: 9304 x 2048 then moves 24 MB more than its 195 MB. There the residual goes
    // back into the LDS column instead (an element is read by the one thread that replaces it) and leaves afterwards in
    // whole lines -- from kColStageMinRows rows on: shorter columns lose more by the barrier and the second pass than
    // they gain. (A column staged in memory is its own residual: nothing to stage.)
    const bool staged = c.rows >= kColStageMinRows && reinterpret_cast<const void*>(tile) != reinterpret_cast<const void*>(res_col) &&
                        ((c.nq & 31u) != 0 || (reinterpret_cast<uintptr_t>(res_col) & 127u) != 0);
    auto pack_item = [&](uint32_t off, auto guard, auto to_lds) {
        uint32_t word = 0;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            if (!decltype(guard)::value || off < end)
            {
                float* at = reinterpret_cast<float*>(reinterpret_cast<char*>(tile) + off);
                const float v = *at;
                const uint32_t code = quantize_value<NBITS, ZT>(vq, v);
                float back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                if constexpr (decltype(to_lds)::value)
                    *at = v - back;
                else
                    __builtin_nontemporal_store(v - back, reinterpret_cast<float*>(reinterpret_cast<char*>(res_col) + off));
                word |= code << (kk * PS::SHIFT);
            }
            off += step;
        }
        return word;
    };
    for (uint32_t it = tid; it < items; it += WG)
    {
        // chunk-major: consecutive threads take consecutive QWords, hence consecutive rows
        const uint32_t chunk = chunk_of_item<PS::CHUNKS>(it, c.nq);
        const uint32_t w = it - chunk * c.nq;
        const uint32_t off = (w + chunk * PS::SLOTS * c.nq) * 4u;
        uint32_t word;
        const bool whole = off + (PS::SLOTS - 1u) * step < end;
        if (staged)
            word = whole ? pack_item(off, std::false_type(), std::true_type()) : pack_item(off, std::true_type(), std::true_type());
        else
            word = whole ? pack_item(off, std::false_type(), std::false_type()) : pack_item(off, std::true_type(), std::false_type());
        word <<= chunk * PS::SLOTS * PS::SHIFT;
        if constexpr (PS::CHUNKS == 1)
            bits[w] = word;
        else
            atomicOr(&words[w], word);
    }
    if (PS::CHUNKS > 1 || staged)
        __syncthreads();
    if constexpr (PS::CHUNKS > 1)
    {
        for (uint32_t w = tid; w < c.nq; w += WG)
            bits[w] = words[w];
    }
    if (staged)
    {
        // slot v holds piece v - shift: wavefronts cover whole lines (see column_shift)
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile);
        f32x4* r4 = reinterpret_cast<f32x4*>(res_col);
        for (uint32_t v = tid; v < c.pieces + shift; v += WG)
            if (v >= shift)
                __builtin_nontemporal_store(t4[v - shift], r4 + (v - shift));
    }
}

// IN_RESIDUAL: the column v = g + r is staged in the residual output's own column in memory instead of LDS (every
// element is then read back and replaced by its residual by the thread that coded it; all phases are separated by
// workgroup barriers). Twice the traffic, served by L2 -- for the few tall columns of a gradient set (a 9304-row bias
// vector) that would otherwise need a launch with more LDS per workgroup all to themselves: 12 us for one workgroup.
template <int NBITS, bool ZT, bool IN_RESIDUAL = false>
__device__ __forceinline__ void quantize_colg_body(const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q,
                                                   const ColGeom& c, uint32_t column, f32x4* smem)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t T = kColThreads;
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * c.rows;
    float* tile = IN_RESIDUAL ? r_out + base : reinterpret_cast<float*>(smem);
    uint32_t* words = reinterpret_cast<uint32_t*>(smem) + (IN_RESIDUAL ? 0u : c.rows);
    float* red = reinterpret_cast<float*>(words + (PS::CHUNKS > 1 ? c.nq : 0));
    if constexpr (PS::CHUNKS > 1)
        for (uint32_t x = tid; x < c.nq; x += T)
            words[x] = 0u;
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g + base);
    const f32x4* r4 = reinterpret_cast<const f32x4*>(r_in + base);
    f32x4* t4 = reinterpret_cast<f32x4*>(tile);
    float stat = 0.0f;
    // slot v holds piece v - shift (see column_shift): the order the register kernels sum in, and whole lines per wavefront
    const uint32_t shift = column_shift(r_in + base, c.line_shift);
    const uint32_t slots = c.pieces + shift;
    for (uint32_t v0 = tid; v0 < slots; v0 += 4 * T)
    {
        f32x4 a[4], b[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
        {
            const uint32_t v = v0 + u * T;
            if (v >= shift && v < slots)
            {
                a[u] = __builtin_nontemporal_load(g4 + (v - shift));
                b[u] = __builtin_nontemporal_load(r4 + (v - shift));
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
        {
            const uint32_t v = v0 + u * T;
            if (v >= shift && v < slots)
            {
                const f32x4 x = a[u] + b[u];
                t4[v - shift] = x;
                stat = colg_add_piece<NBITS>(stat, x);
            }
        }
    }
    // the whole column has been read before the first barrier of colg_stats_pack, so r_out may be r_in
    colg_stats_pack<NBITS, ZT>(tile, words, red, c, stat, shift, r_out + base, q + (size_t) column * c.qcol);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kColThreads) void quantize_colg_kernel(const float* __restrict__ g, const float* r_in, float* r_out,
                                                                    char* __restrict__ q, ColGeom c)
{
    extern __shared__ f32x4 smem_v4[];
    quantize_colg_body<NBITS, ZT>(g, r_in, r_out, q, c, blockIdx.x, smem_v4);
}

// One group of up to eight workers (n0 ... n0 + 7 of the summation order) added to the running sums of a work item's SLOTS
// elements. word[u]: worker n0 + u's QWord; dec: the group's decoding tables. FIRST: the group that holds the owner, whose
// value seeds the sum, and whose tables start at LDS address 0 (see lds_read). FULL: count is 8 (nothing to branch around,
// and the look-ups of all eight workers can be in flight together).
template <int NBITS, bool FIRST, bool FULL>
__device__ __forceinline__ void stripe_add_group(float (&acc)[PackShape<NBITS>::SLOTS], const uint32_t (&word)[8], uint32_t sh0, uint32_t count,
                                                 const float* dec)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t DEC = stripe_dec_floats(NBITS);
#pragma unroll
    for (uint32_t u = 0; u < 8; ++u)
    {
        if (FULL || u < count)
        {
            const uint32_t bits = word[u] >> sh0;
            const float* lev = dec + u * DEC;
            if constexpr (NBITS == 2)
            {
                // two codes at a time: their four bits, times 8 bytes, are the offset of the pair of levels
                static_assert(PS::SLOTS % 2 == 0, "pairs of bit positions");
#pragma unroll
                for (uint32_t j = 0; j < PS::SLOTS / 2; ++j)
                {
                    const uint32_t off = j == 0 ? (bits << 3) & 0x78u : (bits >> (4 * j - 3)) & 0x78u;
                    f32x2 x;
                    if constexpr (FIRST)
                        x = lds_read<f32x2>(off + u * DEC * 4u);
                    else
                        x = *reinterpret_cast<const f32x2*>(reinterpret_cast<const char*>(lev) + off);
                    acc[2 * j] = (FIRST && u == 0) ? x.x : x.x + acc[2 * j];
                    acc[2 * j + 1] = (FIRST && u == 0) ? x.y : x.y + acc[2 * j + 1];
                }
            }
            else if constexpr (NBITS == 4)
            {
#pragma unroll
                for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
                {
                    const uint32_t off = kk == 0 ? (bits << 2) & 0x3Cu : (bits >> (4 * kk - 2)) & 0x3Cu;
                    float x;
                    if constexpr (FIRST)
                        x = lds_read<float>(off + u * DEC * 4u);
                    else
                        x = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(lev) + off);
                    acc[kk] = (FIRST && u == 0) ? x : x + acc[kk];
                }
            }
            else
            {
                const float a = lev[0];
                const float b = lev[1];
#pragma unroll
                for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
                {
                    float x;
                    if constexpr (NBITS == 1)
                        x = pick_level(bits, kk, a, b);
                    else
                        x = unquantize_value<NBITS>(a, b, (bits >> (kk * PS::SHIFT)) & PS::CODEMASK);
                    // the first term (the owner's) seeds the sum; afterwards: decoded value + running sum
                    acc[kk] = (FIRST && u == 0) ? x : x + acc[kk];
                }
            }
        }
    }
}

// The sums' results for one work item: SLOTS elements, nq apart, from byte offset off0 of the column on; the aggregate
// (when asked for) to memory, aggregate plus stripe residual to the column in LDS (which starts at LDS address tile_at, see
// lds_write). GUARD: some may lie beyond the column.
template <int NBITS, bool GUARD>
__device__ __forceinline__ void stripe_store_item(const float (&acc)[PackShape<NBITS>::SLOTS], const float (&resid)[PackShape<NBITS>::SLOTS],
                                                  uint32_t tile_at, float* agg_col, uint32_t off0, uint32_t step, uint32_t end)
{
    uint32_t off = off0;
#pragma unroll
    for (uint32_t kk = 0; kk < PackShape<NBITS>::SLOTS; ++kk)
    {
        if (!GUARD || off < end)
        {
            if (agg_col != nullptr)
                *reinterpret_cast<float*>(reinterpret_cast<char*>(agg_col) + off) = acc[kk];
            lds_write<float>(tile_at + off, acc[kk] + resid[kk]);
        }
        off += step;
    }
}

// WGT: threads in the workgroup, or 0 for what the launch says (tall columns: many work items would otherwise be a long
// chain of dependent loads for each of few threads).
// LDS: the decoding tables of the first eight workers of the summation order (at offsets the compiler knows, which the
// look-ups then carry in the instruction), the column, its QWords under assembly (when a QWord's bit positions are
// dealt to several work items), the sums' slots, the tables of any further workers.
template <int NBITS, bool ZT, int WGT = kColThreads>
__device__ __forceinline__ void stripe_reduce_colg_body(const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                                                        const ColGeom& c, uint32_t column, f32x4* smem)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t T = kColThreads, BATCH = kStripeDecGroup;
    constexpr uint32_t DEC = stripe_dec_floats(NBITS);
    static_assert(WGT == 0 || WGT >= (int) T, "workgroup size");
    static_assert(BATCH * DEC % 4 == 0, "the column starts on a 16-byte boundary");
    const uint32_t WG = WGT == 0 ? blockDim.x : (uint32_t) WGT;
    float* dec = reinterpret_cast<float*>(smem);
    float* tile = dec + BATCH * DEC;
    uint32_t* words = reinterpret_cast<uint32_t*>(tile + c.rows);
    float* red = tile + c.rows + (PS::CHUNKS > 1 ? c.nq : 0);
    // from an 8-byte boundary on
    float* dec_more = red + kColgRedSlots + ((c.rows + (PS::CHUNKS > 1 ? c.nq : 0)) & 1u);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * c.rows;
    const size_t rec = (size_t) column * c.qcol;
    const uint32_t K = src.workers;
    if constexpr (PS::CHUNKS > 1)
        for (uint32_t x = tid; x < c.nq; x += WG)
            words[x] = 0u;
    // what this thread's first work item needs from memory is requested before the first barrier: one round trip for
    // headers, QWords and stripe residual instead of three (see stripe_reduce_col_kernel)
    const float* sp = stripe_res + base;
    float* agg_col = agg_out != nullptr ? agg_out + base : nullptr;
    const uint32_t items = c.nq * PS::CHUNKS;
    // A QWord's bit positions are nq elements apart; element i lies 4 * i bytes into the column, in memory as in LDS, and
    // all of a column's addresses are a base that every thread shares plus a 32-bit offset.
    const uint32_t step = c.nq * 4u, end = c.rows * 4u;
    // the QWords of this column in the first BATCH workers' records, in summation order (beyond the last worker: the last
    // one's again, fetched and not used). Looked up once: inside the loop over the work items every worker's pointer
    // would be fetched from the kernel's arguments again, one after the other, before the loads that need it go out.
    const char* first[BATCH];
#pragma unroll
    for (uint32_t u = 0; u < BATCH; ++u)
        first[u] = src.q[stripe_order(min(u, K - 1u), src.owner)] + rec + 8;
    uint32_t word[BATCH], word_next[BATCH];
    float resid[PS::SLOTS], resid_next[PS::SLOTS];
    // (a row beyond the column reads the last row instead, and is not used: no branch around any of the loads)
    auto fetch = [&](uint32_t it, uint32_t (&wd)[BATCH], float (&rs)[PS::SLOTS]) {
        const uint32_t chunk = chunk_of_item<PS::CHUNKS>(it, c.nq);
        const uint32_t w = it - chunk * c.nq;
#pragma unroll
        for (uint32_t u = 0; u < BATCH; ++u)
            wd[u] = *reinterpret_cast<const uint32_t*>(first[u] + w * 4u);
        uint32_t off = (w + chunk * PS::SLOTS * c.nq) * 4u;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            rs[kk] = __builtin_nontemporal_load(reinterpret_cast<const float*>(reinterpret_cast<const char*>(sp) + min(off, end - 4u)));
            off += step;
        }
    };
    if (tid < items)
        fetch(tid, word, resid);
    auto table_of = [&](uint32_t n) { return n < BATCH ? dec + n * DEC : dec_more + (n - BATCH) * DEC; };
    if constexpr (NBITS == 2)
    {
        // entry x of a worker: the levels of codes x & 3 and x >> 2, side by side
        for (uint32_t x = tid; x < K * 16u; x += WG)
        {
            const uint32_t n = x / 16u, e = x % 16u;
            const float* h = reinterpret_cast<const float*>(src.q[stripe_order(n, src.owner)] + rec);
            const ValueQ vq = make_vq<NBITS>(h[0], h[1]);
            float* t = table_of(n);
            t[2 * e] = unquantize_value<NBITS>(vq, e & 3u);
            t[2 * e + 1] = unquantize_value<NBITS>(vq, e >> 2);
        }
    }
    else if constexpr (NBITS == 4)
    {
        for (uint32_t x = tid; x < K * DEC; x += WG)
        {
            const uint32_t n = x / DEC, e = x % DEC;
            const float* h = reinterpret_cast<const float*>(src.q[stripe_order(n, src.owner)] + rec);
            table_of(n)[e] = unquantize_value<NBITS>(make_vq<NBITS>(h[0], h[1]), e);
        }
    }
    else if (tid < K)
    {
        const float* h = reinterpret_cast<const float*>(src.q[stripe_order(tid, src.owner)] + rec);
        const ValueQ vq = make_vq<NBITS>(h[0], h[1]);
        float* t = table_of(tid);
        if constexpr (NBITS == 1)
        {
            t[0] = unquantize_value<NBITS>(vq, 0u);
            t[1] = unquantize_value<NBITS>(vq, 1u);
        }
        else
        {
            t[0] = vq.uf;
            t[1] = vq.lo;
        }
    }
    __syncthreads();

    for (uint32_t it = tid; it < items; it += WG)
    {
        const uint32_t chunk = chunk_of_item<PS::CHUNKS>(it, c.nq);
        const uint32_t w = it - chunk * c.nq;
        const uint32_t off0 = (w + chunk * PS::SLOTS * c.nq) * 4u;
        const uint32_t sh0 = chunk * PS::SLOTS * PS::SHIFT;
        // the next work item's inputs are on their way while this one's are summed
        if (it + WG < items)
            fetch(it + WG, word_next, resid_next);
        float acc[PS::SLOTS];
        // up to eight workers (the tables at offsets the compiler knows), then the others eight at a time
        if (K >= BATCH)
            stripe_add_group<NBITS, true, true>(acc, word, sh0, BATCH, dec);
        else
            stripe_add_group<NBITS, true, false>(acc, word, sh0, K, dec);
        for (uint32_t n0 = BATCH; n0 < K; n0 += BATCH)
        {
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
                word[u] = *reinterpret_cast<const uint32_t*>(src.q[stripe_order(min(n0 + u, K - 1u), src.owner)] + rec + 8 + w * 4u);
            stripe_add_group<NBITS, false, false>(acc, word, sh0, min(K - n0, BATCH), dec_more + (n0 - BATCH) * DEC);
        }
        // only the last of a QWord's bit positions can lie beyond the end of a column of more than VPW * VPW rows
        if (off0 + (PS::SLOTS - 1u) * step < end)
            stripe_store_item<NBITS, false>(acc, resid, BATCH * DEC * 4u, agg_col, off0, step, end);
        else
            stripe_store_item<NBITS, true>(acc, resid, BATCH * DEC * 4u, agg_col, off0, step, end);
#pragma unroll
        for (uint32_t u = 0; u < BATCH; ++u)
            word[u] = word_next[u];
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
            resid[kk] = resid_next[kk];
    }
    float stat = 0.0f;
    // the quantize kernels' summation order for a residual at this address
    const uint32_t shift = column_shift(stripe_res + base, c.line_shift);
    if constexpr ((NBITS != 1) || !ZT)
    {
        __syncthreads();
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile);
        if (WGT == (int) T || tid < T)
            for (uint32_t v = tid; v < c.pieces + shift; v += T)
                if (v >= shift)
                    stat = colg_add_piece<NBITS>(stat, t4[v - shift]);
    }
    colg_stats_pack<NBITS, ZT, WGT>(tile, words, red, c, stat, shift, stripe_res + base, q_out + rec);
}

// WGT: the workgroup's size, or 0 for any multiple of 64 from 256 to 1024 (the launch says)
template <int NBITS, bool ZT, int WGT>
__global__ __launch_bounds__(WGT == 0 ? 1024 : WGT) CNTKQ_SGPRS_FOR_8_WAVES void stripe_reduce_colg_kernel(StripeSources src, float* stripe_res, char* q_out, float* agg_out,
                                                                                   ColGeom c)
{
    extern __shared__ f32x4 smem_v4[];
    stripe_reduce_colg_body<NBITS, ZT, WGT>(src, stripe_res, q_out, agg_out, c, blockIdx.x, smem_v4);
}

} // namespace cntkq
