// gfx950 kernels of the per-column gradient quantizer, double-precision instantiation
// (MatrixQuantizerImpl<double>: QWord = 64-bit, Source/Math/ValueQuantizer.h:50-57).
//
// Packed layout (Source/Math/QuantizedMatrix.h:27-48 with ElemType = double):
//   column j = { f64 lower; f64 upper; u64 bits[nq] } at byte j * qcol,  nq = ceil(rows / (64 / NBITS));
//   element i of the column is in bits[i % nq] at bit (i / nq) * NBITS. NBITS is 1, 2, 4, ..., 64 (64 = pass-through).
// Every record is a multiple of 8 bytes, so all headers and QWords are naturally aligned.
//
// Work decomposition mirrors the fp32 tile kernels: a workgroup owns a run of consecutive columns, reads gradient and
// residual once, keeps v = g + r in LDS as doubles, takes the statistics from LDS, packs, writes the residual.
// Columns too tall for LDS take the one-workgroup-per-column kernel that re-reads global memory.
// All arithmetic is separately rounded IEEE fp64 (compile with -ffp-contract=off).
#pragma once

#include "quantizer_kernels.h"

namespace cntkq {
namespace f64 {

constexpr uint32_t kThreads = 256;
constexpr uint32_t kMaxTileCols = 32;
// LDS prefix in 8-byte units: 8 double + 2 (four uint32) for the reductions of up to 4 wavefronts, then (lower, upper) per column
constexpr uint32_t kPrefixWords = 10 + 2 * kMaxTileCols;

// The per-value quantizer, the header statistics and the pack shape are the element-type templates of quantizer_math.h
// and quantizer_kernels_common.h, here on doubles and 64-bit QWords.
typedef ValueQOf<double> ValueQ;
template <int NBITS>
using PackShape = PackShapeOf<NBITS, 64>;

struct TileGeom
{
    uint32_t rows;
    uint32_t cols;
    uint32_t nq;
    uint32_t cols_per_tile; // kThreads / gs
    uint32_t gs;            // threads per column in the statistics phase: power of two in [8, kThreads]
    uint32_t gs_log2;
    uint32_t tile_words;    // LDS doubles reserved for the tile
    uint32_t words_words;   // LDS QWords for partial words (cols_per_tile * nq when a QWord has several work items)
    uint64_t qcol;
};

// LDS layout in 8-byte units: [prefix | tile | partial QWords | decode constants (2 * workers * cols_per_tile)]
__host__ __device__ inline size_t tile_lds_bytes(const TileGeom& t, uint32_t workers)
{
    return ((size_t) kPrefixWords + t.tile_words + t.words_words + (size_t) 2 * workers * t.cols_per_tile) * 8;
}

// ---- statistics + packing of a tile in LDS (same contract as the fp32 tile_stats / tile_pack) ----------

// (tile_stats is the fp32 tile kernels' function, written over the element type)

// Columns of fewer QWords than this hand their new residual back through the LDS tile.
constexpr uint32_t kStagedResidualBelowQWords = 16;

// (tile_pack is the fp32 tile kernels' function too.) For a fixed bit position consecutive threads hold consecutive rows of a
// column, nq of them: where that run is at least a 128-byte line the new residual goes straight to global memory; shorter
// runs (a 147-row column at 1 bit: 3 doubles) would reach memory as fragments, so there the residual replaces the value in
// the tile and the tile leaves in consecutive stores.
__device__ __forceinline__ bool tile_residual_staged(const TileGeom& t)
{
    return t.nq < kStagedResidualBelowQWords;
}

// after tile_pack with a staged residual: the tile to global memory
__device__ __forceinline__ void tile_store(const double* tile, double* res_out, uint32_t total)
{
    for (uint32_t e = threadIdx.x; e < total; e += kThreads)
        __builtin_nontemporal_store(tile[e], res_out + e);
}

struct TileLds
{
    double* scratch_f;
    uint32_t* scratch_u;
    double* hdr;
    double* tile;
    uint64_t* words;
    double* dec;
};

__device__ __forceinline__ TileLds tile_lds(double* smem, const TileGeom& t)
{
    TileLds l;
    l.scratch_f = smem;
    l.scratch_u = reinterpret_cast<uint32_t*>(smem + 8);
    l.hdr = smem + 10;
    l.tile = smem + kPrefixWords;
    l.words = reinterpret_cast<uint64_t*>(smem + kPrefixWords + t.tile_words);
    l.dec = smem + kPrefixWords + t.tile_words + t.words_words;
    return l;
}

// ---- quantize ---------------------------------------------------------------------------------------------

// (block: the tile's index within the matrix; smem: the workgroup's dynamic LDS -- a kernel of its own below, and a member
// of the batched launch)
template <int NBITS, bool ZT>
__device__ __forceinline__ void quantize_tile_body(const double* __restrict__ g, const double* r_in, double* r_out, char* __restrict__ q,
                                                   const TileGeom& t, uint32_t block, double* smem)
{
    const TileLds l = tile_lds(smem, t);
    const uint32_t tid = threadIdx.x;
    const uint32_t j0 = block * t.cols_per_tile;
    const uint32_t nc = min(t.cols_per_tile, t.cols - j0);
    const size_t base = (size_t) j0 * t.rows;
    const uint32_t total = nc * t.rows;
    const double* gp = g + base;
    const double* rp = r_in + base;

    if constexpr (PackShape<NBITS>::CHUNKS > 1)
        for (uint32_t x = tid; x < nc * t.nq; x += kThreads)
            l.words[x] = 0ull;

    // four loads of each operand in flight per thread
    for (uint32_t e0 = tid; e0 < total; e0 += 4 * kThreads)
    {
        double a[4], b[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
        {
            const uint32_t e = e0 + u * kThreads;
            if (e < total)
            {
                a[u] = __builtin_nontemporal_load(gp + e);
                b[u] = __builtin_nontemporal_load(rp + e);
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
        {
            const uint32_t e = e0 + u * kThreads;
            if (e < total)
                l.tile[e] = a[u] + b[u];
        }
    }
    __syncthreads(); // from here on r_in is no longer read by this workgroup, so r_out may be r_in

    char* qtile = q + (size_t) j0 * t.qcol;
    tile_stats<NBITS, ZT>(l.tile, l.hdr, l.scratch_f, l.scratch_u, t, nc, qtile);
    const bool staged = tile_residual_staged(t);
    tile_pack<NBITS, ZT>(l.tile, l.hdr, l.words, t, staged, nc, qtile, r_out + base);
    if (staged)
        tile_store(l.tile, r_out + base, nc * t.rows);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kThreads) void quantize_tile_kernel(const double* __restrict__ g, const double* r_in, double* r_out,
                                                                 char* __restrict__ q, TileGeom t)
{
    extern __shared__ f64x2 smem_f64[];
    quantize_tile_body<NBITS, ZT>(g, r_in, r_out, q, t, blockIdx.x, reinterpret_cast<double*>(smem_f64));
}

// ---- one 256-thread workgroup per column, the column in registers element by element ------------------------
//
// For the heights at which the tile kernel holds a single column per tile (more than 1024 rows) and that column starts to
// crowd LDS (16 KB at 2048 rows, 48 KB at 6144): thread t keeps rows t, t + 256, ... (at most EPT of them) from the loads
// to the residual store, LDS holds only the reduction slots and the column's QWords (assembled by atomic OR), and the
// occupancy no longer falls with the height. Nothing depends on alignment: every access is one double, consecutive
// threads on consecutive rows. The sums are taken exactly as tile_stats takes them for a one-column tile -- a thread adds
// its rows in ascending order, then group_sum over the 256 threads -- so the bytes are those of the tile kernel, and the
// tile stripe reduction still reproduces the call sequence. A row beyond the column is replaced by the last row on
// loading and masked out of every sum and store, so the load and statistics phases have no branches.
template <int EPT>
constexpr int colreg_waves()
{
    int w = 512 / (2 * EPT + 40); // (with 8 registers fewer one instantiation spills)
    return w > 8 ? 8 : w;
}

constexpr uint32_t kColRegPrefixWords = 10; // 8 doubles + four uint32 for the reductions, as in the tile kernels

__host__ __device__ inline size_t colreg_lds_bytes(uint32_t nq)
{
    return ((size_t) kColRegPrefixWords + nq) * 8;
}

template <int NBITS, bool ZT, int EPT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(colreg_waves<EPT>(), colreg_waves<EPT>()))) void quantize_colreg_kernel(
    const double* __restrict__ g, const double* r_in, double* r_out, char* __restrict__ q, uint32_t rows, uint32_t nq, uint64_t qcol)
{
    static_assert(NBITS < 64, "64-bit codes are whole QWords: nothing to assemble");
    using PS = PackShape<NBITS>;
    extern __shared__ f64x2 smem_f64[];
    double* scratch_f = reinterpret_cast<double*>(smem_f64);
    uint32_t* scratch_u = reinterpret_cast<uint32_t*>(scratch_f + 8);
    unsigned long long* words = reinterpret_cast<unsigned long long*>(scratch_f + kColRegPrefixWords);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * rows;
    char* qc = q + (size_t) blockIdx.x * qcol;
    for (uint32_t x = tid; x < nq; x += kThreads)
        words[x] = 0ull;
    const double* gp = g + base;
    const double* rp = r_in + base;
    const uint32_t last = rows - 1;
    double a[EPT];
    {
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < EPT; ++u)
            a[u] = __builtin_nontemporal_load(gp + min(t + kThreads * u, last));
    }
#pragma unroll
    for (int u0 = 0; u0 < EPT; u0 += 4)
    {
        const uint32_t t = opaque(tid);
        double b[4];
#pragma unroll
        for (int u = u0; u < u0 + 4 && u < EPT; ++u)
            b[u - u0] = __builtin_nontemporal_load(rp + min(t + kThreads * u, last));
#pragma unroll
        for (int u = u0; u < u0 + 4 && u < EPT; ++u)
            a[u] = a[u] + b[u - u0];
    }
    // a thread stores only rows it has loaded itself, so r_out may be r_in without a barrier in between

    double lo, hi;
    if constexpr (NBITS == 1)
    {
        double mean = 0.0;
        if constexpr (!ZT)
        {
            double sum = 0.0;
            const uint32_t t = opaque(tid);
#pragma unroll
            for (int u = 0; u < EPT; ++u)
                sum = (t + kThreads * u < rows) ? sum + a[u] : sum;
            sum = group_sum(sum, kThreads, scratch_f);
            mean = sum / (double) rows;
        }
        double s0 = 0.0, s1 = 0.0;
        uint32_t n0 = 0;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < EPT; ++u)
        {
            const bool valid = t + kThreads * u < rows;
            const bool below = a[u] < mean;
            s0 = (valid && below) ? s0 + a[u] : s0;
            s1 = (valid && !below) ? s1 + a[u] : s1;
            n0 += (valid && below) ? 1u : 0u;
        }
        group_sum3(s0, s1, n0, kThreads, scratch_f, scratch_u);
        finish_stats_1bit<ZT>(mean, s0, s1, n0, rows - n0, rows, lo, hi);
    }
    else
    {
        double sum = 0.0;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < EPT; ++u)
        {
            const double sq = a[u] * a[u];
            sum = (t + kThreads * u < rows) ? sum + sq : sum;
        }
        sum = group_sum(sum, kThreads, scratch_f);
        finish_stats_multibit(sum, rows, lo, hi);
    }
    if (tid == 0)
    {
        double* gh = reinterpret_cast<double*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const double val0 = unquantize_value<NBITS>(vq.uf, vq.lo, 0ull);
    const double val1 = unquantize_value<NBITS>(vq.uf, vq.lo, 1ull);
    double* ro = r_out + base;
    // row i is bit position i / nq of QWord i % nq; a thread's rows lie 256 apart
    const uint32_t step_k = kThreads / nq, step_w = kThreads - step_k * nq;
    uint32_t k = tid / nq;
    uint32_t w = tid - k * nq;
    const uint32_t to = opaque(tid);
#pragma unroll
    for (int u = 0; u < EPT; ++u)
    {
        const uint32_t i = to + kThreads * u;
        if (i < rows)
        {
            const double v = a[u];
            const uint64_t code = quantize_value<NBITS, ZT>(vq, v);
            double back;
            if constexpr (NBITS == 1)
                back = code ? val1 : val0;
            else
                back = unquantize_value<NBITS>(vq.uf, vq.lo, code);
            __builtin_nontemporal_store(v - back, ro + i);
            atomicOr(&words[w], (unsigned long long) (code << (k * PS::SHIFT)));
        }
        w += step_w;
        k += step_k;
        if (w >= nq)
        {
            w -= nq;
            ++k;
        }
    }
    __syncthreads();
    unsigned long long* bits = reinterpret_cast<unsigned long long*>(qc + 16);
    for (uint32_t x = tid; x < nq; x += kThreads)
        bits[x] = words[x];
}

// (columns too tall for these take quantize_tall_kernel of quantizer_kernels_tall.h, written over the element type)

// ---- stripe reduction: K packed stripes -> fp64 sum (owner first, then ascending) -> requantize ------------

template <int NBITS, bool ZT>
__device__ __forceinline__ void stripe_reduce_tile_body(const StripeSources& src, double* stripe_res, char* q_out, double* agg_out,
                                                        const TileGeom& t, uint32_t block, double* smem)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t BATCH = 8; // packed words fetched together, so their latencies overlap

    const TileLds l = tile_lds(smem, t);
    const uint32_t tid = threadIdx.x;
    const uint32_t j0 = block * t.cols_per_tile;
    const uint32_t nc = min(t.cols_per_tile, t.cols - j0);
    const size_t base = (size_t) j0 * t.rows;
    const uint32_t K = src.workers;
    const uint32_t nwords = nc * t.nq;
    double* sp = stripe_res + base;

    if constexpr (PS::CHUNKS > 1)
        for (uint32_t x = tid; x < nwords; x += kThreads)
            l.words[x] = 0ull;

    // short columns: the stripe residual comes in as one consecutive run (see tile_pack), not as runs of nq rows
    const bool staged = tile_residual_staged(t);
    if (staged)
        for (uint32_t e = tid; e < nc * t.rows; e += kThreads)
            l.tile[e] = __builtin_nontemporal_load(sp + e);

    // decode constants from every worker's column header, in summation order: 1 bit -> the two levels, else (ufactor, lower)
    for (uint32_t x = tid; x < nc * K; x += kThreads)
    {
        const uint32_t c = x / K;
        const uint32_t n = x - c * K;
        const double* h = reinterpret_cast<const double*>(src.q[stripe_order(n, src.owner)] + (size_t) (j0 + c) * t.qcol);
        const ValueQ vq = make_vq<NBITS>(h[0], h[1]);
        if constexpr (NBITS == 1)
        {
            l.dec[2 * x] = unquantize_value<NBITS>(vq.uf, vq.lo, 0ull);
            l.dec[2 * x + 1] = unquantize_value<NBITS>(vq.uf, vq.lo, 1ull);
        }
        else
        {
            l.dec[2 * x] = vq.uf;
            l.dec[2 * x + 1] = vq.lo;
        }
    }
    __syncthreads();

    const uint32_t items = nwords * PS::CHUNKS;
    for (uint32_t it = tid; it < items; it += kThreads)
    {
        const uint32_t chunk = (PS::CHUNKS == 1) ? 0u : it / nwords;
        const uint32_t qi = it - chunk * nwords;
        const uint32_t c = (nc == 1) ? 0u : qi / t.nq;
        const uint32_t w = qi - c * t.nq;
        const size_t word_off = (size_t) (j0 + c) * t.qcol + 16 + (size_t) w * 8;
        const uint32_t sh0 = chunk * PS::SLOTS * PS::SHIFT;
        const double* d = l.dec + 2 * (size_t) c * K;
        double acc[PS::SLOTS];
        for (uint32_t n0 = 0; n0 < K; n0 += BATCH)
        {
            uint64_t word[BATCH];
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
                if (n0 + u < K)
                    word[u] = *reinterpret_cast<const uint64_t*>(src.q[stripe_order(n0 + u, src.owner)] + word_off);
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
            {
                if (n0 + u < K)
                {
                    const double a = d[2 * (n0 + u)];
                    const double b = d[2 * (n0 + u) + 1];
                    const uint64_t bits = word[u] >> sh0;
#pragma unroll
                    for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
                    {
                        const uint64_t code = (bits >> (kk * PS::SHIFT)) & PS::CODEMASK;
                        double x;
                        if constexpr (NBITS == 1)
                            x = code ? b : a;
                        else
                            x = unquantize_value<NBITS>(a, b, code);
                        // the first term seeds the sum; afterwards: decoded value + running sum
                        acc[kk] = (n0 + u == 0) ? x : x + acc[kk];
                    }
                }
            }
        }
        double* colv = l.tile + (size_t) c * t.rows;
        const double* sc = sp + (size_t) c * t.rows;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t i = w + (chunk * PS::SLOTS + kk) * t.nq;
            if (i < t.rows)
            {
                if (agg_out != nullptr)
                    agg_out[base + (size_t) c * t.rows + i] = acc[kk];
                colv[i] = acc[kk] + (staged ? colv[i] : __builtin_nontemporal_load(sc + i));
            }
        }
    }
    __syncthreads();

    char* qtile = q_out + (size_t) j0 * t.qcol;
    tile_stats<NBITS, ZT>(l.tile, l.hdr, l.scratch_f, l.scratch_u, t, nc, qtile);
    tile_pack<NBITS, ZT>(l.tile, l.hdr, l.words, t, staged, nc, qtile, sp);
    if (staged)
        tile_store(l.tile, sp, nc * t.rows);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kThreads) CNTKQ_SGPRS_FOR_8_WAVES void stripe_reduce_tile_kernel(StripeSources src, double* stripe_res, char* q_out,
                                                                      double* agg_out, TileGeom t)
{
    extern __shared__ f64x2 smem_f64[];
    stripe_reduce_tile_body<NBITS, ZT>(src, stripe_res, q_out, agg_out, t, blockIdx.x, reinterpret_cast<double*>(smem_f64));
}

// ---- unquantize ----------------------------------------------------------------------------------------------
//
// The QWord-major decoder (UnqGeom, unquantize_body, unquantize_kernel) is the fp32 source, written over the element type:
// two QWords and two rows per thread and bit position where rows and QWords per column are even, else one.

// The row-major decoder (unquantize_rows_kernel) and the tile decoder (unquantize_tile_kernel) are the fp32 sources too: a
// 16-byte store holds two doubles, QWords are 64-bit, a packed record is nq + 2 QWords (lower, upper, bits).


// ---- one workgroup per column, the column in registers (the fp32 quantize_reg_kernel on doubles) ------------
//
// Thread tid of T keeps the 16-byte pieces (two doubles) of its slots tid, tid + T, ... through statistics, coding and
// the residual store; LDS holds only the column's 64-bit QWords, assembled by atomic OR. Slots are dealt by 128-byte
// lines (column_shift). For columns too tall for the tile kernels: up to 25 pieces for each of 1024 threads.

template <int NBITS>
__device__ __forceinline__ double reg_add_piece(double s, const f64x2& v)
{
    if constexpr (NBITS == 1)
    {
        s += v.x;
        s += v.y;
    }
    else
    {
        s += v.x * v.x;
        s += v.y * v.y;
    }
    return s;
}

__host__ __device__ inline size_t reg_lds_bytes64(const RegGeom& c)
{
    return ((size_t) kRegRedSlots + c.nq) * 8;
}

// Second half of the register kernel: statistics, header, codes, residual and packed QWords of the column a workgroup
// holds in registers (a: the slots' pieces; edge: this thread's edge element if has_edge). words[0 .. nq) must be zero;
// the first barrier inside also orders everything the caller did before it. Shared with the stripe reduction below.
template <int NBITS, bool ZT, int T, int PER>
__device__ __forceinline__ void reg_stats_pack(f64x2 (&a)[PER], double edge, bool has_edge, uint32_t edge_at, uint32_t head, uint32_t pieces,
                                               uint32_t shift, const RegGeom& c, double* red, uint32_t* red_u, unsigned long long* words,
                                               double* r_out_col, char* qc)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t NW = T / 64;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    double total = 0.0;
    if constexpr (need_stat)
    {
        double stat = 0.0;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            const double with = reg_add_piece<NBITS>(stat, a[u]);
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
    double lo, hi;
    if constexpr (NBITS == 1)
    {
        const double mean = ZT ? 0.0 : total / (double) c.rows;
        double s0 = 0.0, s1 = 0.0;
        uint32_t n0 = 0;
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            double t0 = s0, t1 = s1;
            uint32_t tn = n0;
#pragma unroll
            for (int e = 0; e < 2; ++e)
            {
                const double x = a[u][e];
                const bool below = x < mean;
                t0 += below ? x : 0.0;
                t1 += below ? 0.0 : x;
                tn += below ? 1u : 0u;
            }
            const bool valid = slot_valid(t + T * u, shift, pieces);
            s0 = valid ? t0 : s0;
            s1 = valid ? t1 : s1;
            n0 = valid ? tn : n0;
        }
        if (has_edge)
        {
            const bool below = edge < mean;
            s0 += below ? edge : 0.0;
            s1 += below ? 0.0 : edge;
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
        double S0 = red[0], S1 = red[NW];
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
        double* gh = reinterpret_cast<double*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const double val0 = unquantize_value<NBITS>(vq.uf, vq.lo, 0ull);
    const double val1 = unquantize_value<NBITS>(vq.uf, vq.lo, 1ull);
    // (the residual output may lie 8 bytes off the residual input that the pieces follow)
    f64x2_u* o2 = reinterpret_cast<f64x2_u*>(r_out_col + head);
    // the first element of this thread's first slot inside the column is bit position k of QWord w; the element after it
    // is the following QWord, the slots after it lie 2 * T elements further on (step_k, step_w)
    const uint32_t ufirst = tid < shift ? 1u : 0u;
    const uint32_t e0 = head + 2 * (tid + T * ufirst - shift);
    uint32_t k = e0 / c.nq;
    uint32_t w = e0 - k * c.nq;
    const uint32_t to = opaque(tid);
#pragma unroll
    for (int u = 0; u < PER; ++u)
    {
        const uint32_t p = to + T * u - shift;
        if (slot_valid(to + T * u, shift, pieces))
        {
            f64x2 res;
            uint32_t kk = k, ww = w;
#pragma unroll
            for (int e = 0; e < 2; ++e)
            {
                const double v = a[u][e];
                const uint64_t code = quantize_value<NBITS, ZT>(vq, v);
                double back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq.uf, vq.lo, code);
                res[e] = v - back;
                atomicOr(&words[ww], (unsigned long long) (code << (kk * PS::SHIFT)));
                if (++ww == c.nq)
                {
                    ww = 0;
                    ++kk;
                }
            }
            __builtin_nontemporal_store(res, o2 + p);
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
        const uint64_t code = quantize_value<NBITS, ZT>(vq, edge);
        double back;
        if constexpr (NBITS == 1)
            back = code ? val1 : val0;
        else
            back = unquantize_value<NBITS>(vq.uf, vq.lo, code);
        r_out_col[edge_at] = edge - back;
        const uint32_t ek = edge_at / c.nq;
        atomicOr(&words[edge_at - ek * c.nq], (unsigned long long) (code << (ek * PS::SHIFT)));
    }
    __syncthreads();
    unsigned long long* bits = reinterpret_cast<unsigned long long*>(qc + 16);
    for (uint32_t x = tid; x < c.nq; x += T)
        bits[x] = words[x];
}

template <int NBITS, bool ZT, int T, int PER>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(reg_waves<T, PER>(), reg_waves<T, PER>()))) void quantize_reg_kernel(
    const double* __restrict__ g, const double* r_in, double* r_out, char* __restrict__ q, RegGeom c)
{
    static_assert(NBITS < 64, "64-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    double* red = reinterpret_cast<double*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    unsigned long long* words = reinterpret_cast<unsigned long long*>(red + kRegRedSlots);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * c.rows;
    char* qc = q + (size_t) blockIdx.x * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0ull;
    // the column may start 8 bytes off a 16-byte boundary and have an odd height: one element before the first aligned
    // pair (held by thread 0) and one after the last (thread 1) then take part in every phase after the thread's pieces
    const uint32_t head = (uint32_t) ((reinterpret_cast<uintptr_t>(r_in + base) >> 3) & 1u);
    const uint32_t pieces = (c.rows - head) >> 1;
    const uint32_t tail = c.rows - head - 2 * pieces;
    // (the aligned pairs are the residual input's; the gradient may lie 8 bytes off them)
    const f64x2_u* g2 = reinterpret_cast<const f64x2_u*>(g + base + head);
    const f64x2* r2 = reinterpret_cast<const f64x2*>(r_in + base + head);
    const bool has_edge = (tid == 0 && head != 0) || (tid == 1 && tail != 0);
    const uint32_t edge_at = tid == 0 ? 0u : c.rows - 1;
    double edge = 0.0;
    if (has_edge)
        edge = g[base + edge_at] + r_in[base + edge_at];
    const uint32_t shift = PER <= kRegMaxShiftPer ? column_shift(r_in + base + head, c.line_shift) : 0u;
    const uint32_t last = pieces - 1;
    f64x2 a[PER];
    {
        const uint32_t t = opaque(tid);
#pragma unroll
        for (int u = 0; u < PER; ++u)
            a[u] = __builtin_nontemporal_load(g2 + slot_piece(t + T * u, shift, last));
    }
#pragma unroll
    for (int u0 = 0; u0 < PER; u0 += 4)
    {
        const uint32_t t = opaque(tid);
        f64x2 b[4];
#pragma unroll
        for (int u = u0; u < u0 + 4 && u < PER; ++u)
            b[u - u0] = __builtin_nontemporal_load(r2 + slot_piece(t + T * u, shift, last));
#pragma unroll
        for (int u = u0; u < u0 + 4 && u < PER; ++u)
            a[u] = a[u] + b[u - u0];
    }
    reg_stats_pack<NBITS, ZT, T, PER>(a, edge, has_edge, edge_at, head, pieces, shift, c, red, red_u, words, r_out + base, qc);
}

// Stripe reduction in the register kernel's shape (the fp32 stripe_reduce_reg_kernel on doubles): 1024 threads per owned
// column, the running sum of the decoded stripes in registers. The workers are taken one at a time in the fixed order
// (owner first, then ascending rank): the worker's packed record goes to LDS in one coalesced copy, each thread decodes
// its slots' elements from it and adds them to its sums. Then the stripe residual is added and reg_stats_pack
// requantizes: byte for byte what "unquantize own stripe, add the others, quantize_reg_kernel on (aggregate, stripe
// residual)" gives. LDS: [reduction slots | nq output QWords | lower, upper and nq QWords of one worker's record].
__host__ __device__ inline size_t stripe_reg_lds_bytes64(const RegGeom& c)
{
    return ((size_t) kRegRedSlots + 2 * (size_t) c.nq + 2) * 8;
}

template <int NBITS, bool ZT, int PER>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(reg_waves<1024, PER>(), reg_waves<1024, PER>()))) void stripe_reduce_reg_kernel(
    StripeSources src, double* stripe_res, char* q_out, double* agg_out, RegGeom c)
{
    using PS = PackShape<NBITS>;
    static_assert(NBITS < 64, "64-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t T = 1024, NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    double* red = reinterpret_cast<double*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    unsigned long long* words = reinterpret_cast<unsigned long long*>(red + kRegRedSlots);
    unsigned long long* pw = words + c.nq; // one worker's record: lower, upper, QWords
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * c.rows;
    const size_t rec = (size_t) blockIdx.x * c.qcol;
    for (uint32_t x = tid; x < c.nq; x += T)
        words[x] = 0ull;
    // the column as the quantize kernel would see it: an element before the first aligned pair, pairs, an element after
    double* sres = stripe_res + base;
    const uint32_t head = (uint32_t) ((reinterpret_cast<uintptr_t>(sres) >> 3) & 1u);
    const uint32_t pieces = (c.rows - head) >> 1;
    const uint32_t tail = c.rows - head - 2 * pieces;
    const bool has_edge = (tid == 0 && head != 0) || (tid == 1 && tail != 0);
    const uint32_t edge_at = tid == 0 ? 0u : c.rows - 1;
    const uint32_t shift = PER <= kRegMaxShiftPer ? column_shift(sres + head, c.line_shift) : 0u;
    const uint32_t ufirst = tid < shift ? 1u : 0u;
    const uint32_t e0 = head + 2 * (tid + T * ufirst - shift);
    const uint32_t k_first = e0 / c.nq;
    const uint32_t w_first = e0 - k_first * c.nq;
    const uint32_t edge_k = edge_at / c.nq;
    const uint32_t edge_w = edge_at - edge_k * c.nq;

    f64x2 a[PER];
    double edge = 0.0;
    const uint32_t K = src.workers;
    const uint32_t rec_words = c.nq + 2;
    for (uint32_t n = 0; n < K; ++n)
    {
        const unsigned long long* from = reinterpret_cast<const unsigned long long*>(src.q[stripe_order(n, src.owner)] + rec);
        if (n != 0)
            __syncthreads(); // everyone has decoded the previous worker's record
        for (uint32_t x = tid; x < rec_words; x += 8 * T)
        {
            unsigned long long v[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                v[u] = from[(x + T * u < rec_words) ? x + T * u : x];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                if (x + T * u < rec_words)
                    pw[x + T * u] = v[u];
        }
        __syncthreads();
        const ValueQ vq = make_vq<NBITS>(__longlong_as_double((long long) pw[0]), __longlong_as_double((long long) pw[1]));
        const double val0 = unquantize_value<NBITS>(vq.uf, vq.lo, 0ull);
        const double val1 = unquantize_value<NBITS>(vq.uf, vq.lo, 1ull);
        const unsigned long long* bits = pw + 2;
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
                for (int e = 0; e < 2; ++e)
                {
                    const uint64_t code = (bits[ww] >> (kk * PS::SHIFT)) & PS::CODEMASK;
                    double x;
                    if constexpr (NBITS == 1)
                        x = code ? val1 : val0;
                    else
                        x = unquantize_value<NBITS>(vq.uf, vq.lo, code);
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
            const uint64_t code = (bits[edge_w] >> (edge_k * PS::SHIFT)) & PS::CODEMASK;
            double x;
            if constexpr (NBITS == 1)
                x = code ? val1 : val0;
            else
                x = unquantize_value<NBITS>(vq.uf, vq.lo, code);
            edge = (n == 0) ? x : x + edge;
        }
    }
    // aggregate out (optional), then the stripe residual in
    {
        const f64x2* r2 = reinterpret_cast<const f64x2*>(sres + head);
        double* ag = agg_out != nullptr ? agg_out + base : nullptr;
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
                    ag[head + 2 * p] = a[u][0];
                    ag[head + 2 * p + 1] = a[u][1];
                }
                a[u] = a[u] + __builtin_nontemporal_load(r2 + p);
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

// ---- whole gradient sets in one launch (the fp32 batch kernels on doubles) ------------------------------------------
//
// The workgroups of all member matrices form one grid; `begins` (count + 1 entries, ascending) gives the first workgroup
// of every matrix. Members of the quantize and stripe-reduction launches are runs of column tiles; members of the
// unquantize launch keep the decoder the plain call would choose.

struct QuantizeBatchEntry64
{
    const double* g;
    const double* r_in;
    double* r_out;
    char* q;
    TileGeom t;
};

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kThreads) void quantize_batch_kernel64(const QuantizeBatchEntry64* __restrict__ entries,
                                                                    const uint32_t* __restrict__ begins, uint32_t count)
{
    extern __shared__ f64x2 smem_f64[];
    const uint32_t e = batch_find(begins, count, blockIdx.x);
    const TileGeom t = entries[e].t; // by value: read once, then held in registers whatever the kernel stores
    quantize_tile_body<NBITS, ZT>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, t, blockIdx.x - begins[e],
                                  reinterpret_cast<double*>(smem_f64));
}

struct StripeBatchEntry64
{
    StripeSources src;
    double* stripe_res;
    char* q_out;
    double* agg_out;
    TileGeom t;
};

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kThreads) CNTKQ_SGPRS_FOR_8_WAVES void stripe_reduce_batch_kernel64(const StripeBatchEntry64* __restrict__ entries,
                                                                         const uint32_t* __restrict__ begins, uint32_t count)
{
    extern __shared__ f64x2 smem_f64[];
    const uint32_t e = batch_find(begins, count, blockIdx.x);
    const StripeBatchEntry64& en = entries[e]; // the table is read-only while the kernel runs
    const TileGeom t = en.t;
    stripe_reduce_tile_body<NBITS, ZT>(en.src, en.stripe_res, en.q_out, en.agg_out, t, blockIdx.x - begins[e],
                                       reinterpret_cast<double*>(smem_f64));
}

struct UnquantizeBatchEntry64
{
    const char* q;
    double* out;
    uint32_t kind; // kUnqVec4 (here: 16-byte stores of two doubles), kUnqScalar, kUnqRows, kUnqDirect, kUnqFlat or kUnqTile
    uint32_t pad;
    UnqGeom qw;
    UnqRowGeom rowg;
    UnqTileGeom tile;
    UnqFlatGeom flat;
};

template <int NBITS>
__global__ __launch_bounds__(256) void unquantize_batch_kernel64(const UnquantizeBatchEntry64* __restrict__ entries,
                                                                 const uint32_t* __restrict__ begins, uint32_t count, int add)
{
    extern __shared__ f32x4 smem_v4[];
    const uint32_t e = batch_find(begins, count, blockIdx.x);
    const UnquantizeBatchEntry64& en = entries[e];
    const uint32_t block = blockIdx.x - begins[e];
    if (en.kind == kUnqVec4)
        unquantize_body<NBITS, 2>(en.q, en.out, en.qw, add, block);
    else if (en.kind == kUnqScalar)
        unquantize_body<NBITS, 1>(en.q, en.out, en.qw, add, block);
    else if (en.kind == kUnqRows)
    {
        const UnqRowGeom t = en.rowg; // by value: the loop below stores between its uses
        unquantize_rows_body<NBITS>(en.q, en.out, t, add, block, reinterpret_cast<uint64_t*>(smem_v4));
    }
    else if (en.kind == kUnqDirect)
    {
        const UnqRowGeom t = en.rowg;
        unquantize_direct_body<NBITS>(en.q, en.out, t, add, block);
    }
    else if (en.kind == kUnqFlat)
    {
        const UnqFlatGeom t = en.flat;
        unquantize_flat_body<NBITS>(en.q, en.out, t, add, block);
    }
    else
    {
        const UnqTileGeom t = en.tile;
        unquantize_tile_body<NBITS>(en.q, en.out, t, add, block, reinterpret_cast<uint64_t*>(smem_v4));
    }
}

} // namespace f64
} // namespace cntkq
