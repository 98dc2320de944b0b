// gfx950 kernels of the per-column gradient quantizer.
//
// Work decomposition (fp32, QWord = uint32):
//   * quantize_tile_kernel / stripe_reduce_tile_kernel: one workgroup owns a run of consecutive columns
//     (a contiguous piece of the column-major matrix). It reads gradient and residual ONCE with
//     coalesced 16-byte loads, keeps v = g + r in LDS, takes the column statistics from LDS
//     (wavefront shuffles, LDS across wavefronts), then packs codes and writes the new residual.
//   * quantize_col_kernel / stripe_reduce_col_kernel: 1-bit columns of 1024, 2048 or 4096 rows; one workgroup
//     owns one column, 16-byte loads, column sum taken while loading.
//   * quantize_tall_kernel: columns too tall for LDS; statistics and packing re-read global memory.
//   * unquantize_kernel: streams codes back to fp32 (optionally accumulating).
//
// Packed layout (Source/Math/QuantizedMatrix.h:27-48): column j = { f32 lower; f32 upper; u32 bits[nq] }
// at byte j * qcol; element i of the column is in bits[i % nq] at bit (i / nq) * NBITS
// (Source/Math/ColumnQuantizer.h:90-147).
#pragma once

#include "quantizer_math.h"

namespace cntkq {

constexpr uint32_t kTileThreads = 256;
constexpr uint32_t kTallThreads = 1024;
constexpr uint32_t kMaxWorkers = 64;

// floats of LDS in front of the column tile: 12 reduction slots (8 float + 4 uint: up to 4 wavefronts),
// then (lower, upper) per tile column (at most 32 columns)
constexpr uint32_t kTileScratchFloats = 12;
constexpr uint32_t kTileMaxCols = 32;
constexpr uint32_t kTilePrefixFloats = kTileScratchFloats + 2 * kTileMaxCols; // 76 floats = 304 B (16-B multiple)

// A QWord is assembled from work items of at most 8 bit positions each, so that a tile with few QWords
// still keeps every thread busy; the partial words meet in LDS (atomic OR).
template <int NBITS>
struct PackShape
{
    static constexpr uint32_t VPW = 32 / NBITS;              // values per QWord
    static constexpr uint32_t SLOTS = VPW < 8 ? VPW : 8;     // bit positions per work item
    static constexpr uint32_t CHUNKS = VPW / SLOTS;          // work items per QWord (4, 2, 1, 1, 1, 1)
    static constexpr uint32_t SHIFT = NBITS & 31;
    static constexpr uint32_t CODEMASK = (NBITS >= 32) ? 0xFFFFFFFFu : ((1u << SHIFT) - 1u);
};

struct TileGeom
{
    uint32_t rows;
    uint32_t cols;
    uint32_t nq;            // QWords per column
    uint32_t threads;       // workgroup size: 64, 128 or 256
    uint32_t cols_per_tile; // threads / gs, <= kTileMaxCols
    uint32_t gs;            // threads per column in the statistics phase: power of two in [8, threads]
    uint32_t gs_log2;
    uint32_t tile_floats;   // LDS floats reserved for the tile: cols_per_tile * rows + alignment slack, multiple of 4
    uint32_t words_floats;  // LDS words for partial QWords: cols_per_tile * nq when a QWord has several work items, else 0
    uint32_t stage_residual; // non-zero: the new residual goes back through LDS and leaves in 16-byte stores
    uint64_t qcol;          // bytes per packed column
};

// LDS layout in floats: [prefix | tile | partial QWords | decode constants (2 * workers * cols_per_tile)]
__host__ __device__ inline size_t tile_lds_bytes(const TileGeom& t, uint32_t workers)
{
    return ((size_t) kTilePrefixFloats + t.tile_floats + t.words_floats + (size_t) 2 * workers * t.cols_per_tile) *
           sizeof(float);
}

// ---- statistics + packing of a tile that already sits in LDS --------------------------------------
//
// tile[c * rows + i] holds v(i, c) = value to quantize for tile column c. On return the column headers are
// in global memory and in hdr[], codes are in global memory and the new residual v - unquantize(code) has
// been written to res_out (dense, column-major, tile-relative).

template <int NBITS, bool ZT>
__device__ __forceinline__ void tile_stats(const float* tile, float* hdr, float* scratch_f, uint32_t* scratch_u,
                                           const TileGeom& t, uint32_t nc, char* qtile)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t c = tid >> t.gs_log2;
    const uint32_t lg = tid & (t.gs - 1);
    const bool col_ok = c < nc;
    const float* colv = tile + (size_t) c * t.rows;
    float lo = 0.0f, hi = 0.0f;

    if constexpr (NBITS == 1)
    {
        float mean = 0.0f;
        if constexpr (!ZT)
        {
            float s = 0.0f;
            if (col_ok)
                for (uint32_t i = lg; i < t.rows; i += t.gs)
                    s += colv[i];
            s = group_sum(s, t.gs, scratch_f);
            mean = s / (float) t.rows;
        }
        float s0 = 0.0f, s1 = 0.0f;
        uint32_t n0 = 0;
        if (col_ok)
        {
            for (uint32_t i = lg; i < t.rows; i += t.gs)
            {
                const float v = colv[i];
                if (v < mean)
                {
                    s0 += v;
                    n0++;
                }
                else
                {
                    s1 += v;
                }
            }
        }
        group_sum3(s0, s1, n0, t.gs, scratch_f, scratch_u);
        finish_stats_1bit<ZT>(mean, s0, s1, n0, t.rows - n0, t.rows, lo, hi);
    }
    else
    {
        float s = 0.0f;
        if (col_ok)
        {
            for (uint32_t i = lg; i < t.rows; i += t.gs)
            {
                const float v = colv[i];
                s += v * v;
            }
        }
        s = group_sum(s, t.gs, scratch_f);
        finish_stats_multibit(s, t.rows, lo, hi);
    }

    if (col_ok && lg == 0)
    {
        hdr[2 * c] = lo;
        hdr[2 * c + 1] = hi;
        // a record is only 4-byte aligned when the column has an odd number of QWords
        float* gh = reinterpret_cast<float*>(qtile + (size_t) c * t.qcol);
        gh[0] = lo;
        gh[1] = hi;
    }
    __syncthreads();
}

// words[] (LDS, nc * nq entries) must be zero on entry when PackShape<NBITS>::CHUNKS > 1.
template <int NBITS, bool ZT>
__device__ __forceinline__ void tile_pack(float* tile, const float* hdr, uint32_t* words, const TileGeom& t,
                                          uint32_t nc, char* qtile, float* res_out)
{
    using PS = PackShape<NBITS>;
    const uint32_t nwords = nc * t.nq;
    const uint32_t items = nwords * PS::CHUNKS;
    const bool stage = t.stage_residual != 0;
    for (uint32_t it = threadIdx.x; it < items; it += t.threads)
    {
        // chunk-major: consecutive threads take consecutive QWords, hence consecutive rows
        const uint32_t chunk = (PS::CHUNKS == 1) ? 0u : it / nwords;
        const uint32_t qi = it - chunk * nwords;
        const uint32_t c = (nc == 1) ? 0u : qi / t.nq;
        const uint32_t w = qi - c * t.nq;
        const ValueQ vq = make_vq<NBITS>(hdr[2 * c], hdr[2 * c + 1]);
        const float val0 = unquantize_value<NBITS>(vq, 0u);
        const float val1 = unquantize_value<NBITS>(vq, 1u);
        float* colv = tile + (size_t) c * t.rows;
        float* ro = res_out + (size_t) c * t.rows;
        uint32_t word = 0;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t k = chunk * PS::SLOTS + kk;
            const uint32_t i = w + k * t.nq;
            if (i < t.rows)
            {
                const float v = colv[i];
                const uint32_t code = quantize_value<NBITS, ZT>(vq, v);
                float back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                const float res = v - back;
                if (stage)
                    colv[i] = res; // this element belongs to this work item alone
                else
                    __builtin_nontemporal_store(res, ro + i);
                word |= code << (k * PS::SHIFT);
            }
        }
        if constexpr (PS::CHUNKS == 1)
            reinterpret_cast<uint32_t*>(qtile + (size_t) c * t.qcol + 8)[w] = word;
        else
            atomicOr(&words[qi], word);
    }
    if constexpr (PS::CHUNKS > 1)
    {
        __syncthreads();
        for (uint32_t qi = threadIdx.x; qi < nwords; qi += t.threads)
        {
            const uint32_t c = (nc == 1) ? 0u : qi / t.nq;
            const uint32_t w = qi - c * t.nq;
            reinterpret_cast<uint32_t*>(qtile + (size_t) c * t.qcol + 8)[w] = words[qi];
        }
    }
    else if (stage)
    {
        __syncthreads();
    }
}

// Coalesced copy of the tile (now holding the new residual) to global memory; 16-byte stores where the
// destination shares the tile's 16-byte phase (`mis` = floats by which the tile start is off a 16-byte boundary).
__device__ __forceinline__ void tile_store(const float* tile, uint32_t mis, float* dst, uint32_t total,
                                           const TileGeom& t)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t mis_d = (uint32_t) ((reinterpret_cast<uintptr_t>(dst) >> 2) & 3u);
    if (mis_d == mis)
    {
        uint32_t head = (4u - mis) & 3u;
        if (head > total)
            head = total;
        const uint32_t nvec = (total - head) >> 2;
        const uint32_t tail0 = head + (nvec << 2);
        if (tid < head)
            dst[tid] = tile[tid];
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile + head);
        f32x4* d4 = reinterpret_cast<f32x4*>(dst + head);
        for (uint32_t e = tid; e < nvec; e += t.threads)
            __builtin_nontemporal_store(t4[e], d4 + e);
        for (uint32_t e = tail0 + tid; e < total; e += t.threads)
            dst[e] = tile[e];
    }
    else
    {
        for (uint32_t e = tid; e < total; e += t.threads)
            __builtin_nontemporal_store(tile[e], dst + e);
    }
}

// ---- quantize: gradient + residual -> packed codes + new residual -----------------------------------

template <int NBITS, bool ZT>
__device__ __forceinline__ void quantize_tile_body(const float* __restrict__ g, const float* r_in, float* r_out,
                                                   char* __restrict__ q, const TileGeom& t, uint32_t tile_index)
{
    extern __shared__ f32x4 smem_v4[];
    float* smem = reinterpret_cast<float*>(smem_v4);
    float* scratch_f = smem;
    uint32_t* scratch_u = reinterpret_cast<uint32_t*>(smem + 8);
    float* hdr = smem + kTileScratchFloats;
    uint32_t* words = reinterpret_cast<uint32_t*>(smem + kTilePrefixFloats + t.tile_floats);

    const uint32_t tid = threadIdx.x;
    const uint32_t j0 = tile_index * t.cols_per_tile;
    const uint32_t nc = min(t.cols_per_tile, t.cols - j0);
    const size_t base = (size_t) j0 * t.rows;
    const uint32_t total = nc * t.rows;
    const float* gp = g + base;
    const float* rp = r_in + base;

    if constexpr (PackShape<NBITS>::CHUNKS > 1)
        for (uint32_t x = tid; x < nc * t.nq; x += t.threads)
            words[x] = 0u;

    // The tile starts `mis` floats into its LDS area so that LDS and global addresses share 16-byte phase.
    const uint32_t mis_g = (uint32_t) ((reinterpret_cast<uintptr_t>(gp) >> 2) & 3u);
    const uint32_t mis_r = (uint32_t) ((reinterpret_cast<uintptr_t>(rp) >> 2) & 3u);
    float* tile = smem + kTilePrefixFloats + mis_g;

    if (mis_g == mis_r)
    {
        uint32_t head = (4u - mis_g) & 3u;
        if (head > total)
            head = total;
        const uint32_t nvec = (total - head) >> 2;
        const uint32_t tail0 = head + (nvec << 2);
        if (tid < head)
            tile[tid] = gp[tid] + rp[tid];
        const f32x4* g4 = reinterpret_cast<const f32x4*>(gp + head);
        const f32x4* r4 = reinterpret_cast<const f32x4*>(rp + head);
        f32x4* t4 = reinterpret_cast<f32x4*>(tile + head);
        for (uint32_t e0 = tid; e0 < nvec; e0 += 4 * t.threads)
        {
            f32x4 a[4], b[4];
#pragma unroll
            for (uint32_t u = 0; u < 4; ++u)
            {
                const uint32_t e = e0 + u * t.threads;
                if (e < nvec)
                {
                    a[u] = __builtin_nontemporal_load(g4 + e);
                    b[u] = __builtin_nontemporal_load(r4 + e);
                }
            }
#pragma unroll
            for (uint32_t u = 0; u < 4; ++u)
            {
                const uint32_t e = e0 + u * t.threads;
                if (e < nvec)
                    t4[e] = a[u] + b[u];
            }
        }
        for (uint32_t e = tail0 + tid; e < total; e += t.threads)
            tile[e] = gp[e] + rp[e];
    }
    else
    {
        for (uint32_t e = tid; e < total; e += t.threads)
            tile[e] = __builtin_nontemporal_load(gp + e) + __builtin_nontemporal_load(rp + e);
    }
    __syncthreads();

    char* qtile = q + (size_t) j0 * t.qcol;
    tile_stats<NBITS, ZT>(tile, hdr, scratch_f, scratch_u, t, nc, qtile);
    tile_pack<NBITS, ZT>(tile, hdr, words, t, nc, qtile, r_out + base);
    if (t.stage_residual)
        tile_store(tile, mis_g, r_out + base, total, t);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) void quantize_tile_kernel(const float* __restrict__ g, const float* r_in,
                                                                     float* r_out, char* __restrict__ q, TileGeom t)
{
    quantize_tile_body<NBITS, ZT>(g, r_in, r_out, q, t, blockIdx.x);
}

// largest e with begins[e] <= b; b and everything derived from it is uniform over the workgroup
__device__ __forceinline__ uint32_t batch_find(const uint32_t* __restrict__ begins, uint32_t count, uint32_t b)
{
    uint32_t lo = 0, hi = count;
    while (hi - lo > 1)
    {
        const uint32_t mid = (lo + hi) >> 1;
        if (begins[mid] <= b)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// ---- stripe reduction: K packed stripes -> fp32 sum -> requantize with the stripe residual ----------

struct StripeSources
{
    const char* q[kMaxWorkers]; // packed stripes, one per worker
    uint32_t workers;
    uint32_t owner;
};

// Position n of the summation order: the owner first, then the other workers in ascending index.
__device__ __forceinline__ uint32_t stripe_order(uint32_t n, uint32_t owner)
{
    return n == 0 ? owner : (n - 1 < owner ? n - 1 : n);
}

template <int NBITS, bool ZT>
__device__ __forceinline__ void stripe_reduce_tile_body(const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                                                        const TileGeom& t, uint32_t tile_index)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t BATCH = 8; // packed words fetched together, so their latencies overlap

    extern __shared__ f32x4 smem_v4[];
    float* smem = reinterpret_cast<float*>(smem_v4);
    float* scratch_f = smem;
    uint32_t* scratch_u = reinterpret_cast<uint32_t*>(smem + 8);
    float* hdr = smem + kTileScratchFloats;
    uint32_t* words = reinterpret_cast<uint32_t*>(smem + kTilePrefixFloats + t.tile_floats);
    float* dec = smem + kTilePrefixFloats + t.tile_floats + t.words_floats;

    const uint32_t tid = threadIdx.x;
    const uint32_t j0 = tile_index * t.cols_per_tile;
    const uint32_t nc = min(t.cols_per_tile, t.cols - j0);
    const size_t base = (size_t) j0 * t.rows;
    const uint32_t K = src.workers;
    const uint32_t nwords = nc * t.nq;
    const uint32_t total = nc * t.rows;
    float* sp = stripe_res + base;
    const uint32_t mis_s = (uint32_t) ((reinterpret_cast<uintptr_t>(sp) >> 2) & 3u);
    float* tile = smem + kTilePrefixFloats + mis_s;

    if constexpr (PS::CHUNKS > 1)
        for (uint32_t x = tid; x < nwords; x += t.threads)
            words[x] = 0u;

    // decode constants from every worker's column header, stored in summation order:
    // 1 bit -> the two levels, else (ufactor, lower)
    for (uint32_t x = tid; x < nc * K; x += t.threads)
    {
        const uint32_t c = x / K;
        const uint32_t n = x - c * K;
        const float* h = reinterpret_cast<const float*>(src.q[stripe_order(n, src.owner)] + (size_t) (j0 + c) * t.qcol);
        const ValueQ vq = make_vq<NBITS>(h[0], h[1]);
        if constexpr (NBITS == 1)
        {
            dec[2 * x] = unquantize_value<NBITS>(vq, 0u);
            dec[2 * x + 1] = unquantize_value<NBITS>(vq, 1u);
        }
        else
        {
            dec[2 * x] = vq.uf;
            dec[2 * x + 1] = vq.lo;
        }
    }
    __syncthreads();

    const uint32_t items = nwords * PS::CHUNKS;
    for (uint32_t it = tid; it < items; it += t.threads)
    {
        const uint32_t chunk = (PS::CHUNKS == 1) ? 0u : it / nwords;
        const uint32_t qi = it - chunk * nwords;
        const uint32_t c = (nc == 1) ? 0u : qi / t.nq;
        const uint32_t w = qi - c * t.nq;
        const size_t word_off = (size_t) (j0 + c) * t.qcol + 8 + (size_t) w * 4;
        const uint32_t sh0 = chunk * PS::SLOTS * PS::SHIFT;
        const float* d = dec + 2 * (size_t) c * K;
        float acc[PS::SLOTS];
        for (uint32_t n0 = 0; n0 < K; n0 += BATCH)
        {
            uint32_t word[BATCH];
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
                if (n0 + u < K)
                    word[u] = *reinterpret_cast<const uint32_t*>(src.q[stripe_order(n0 + u, src.owner)] + word_off);
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
            {
                if (n0 + u < K)
                {
                    const float a = d[2 * (n0 + u)];
                    const float b = d[2 * (n0 + u) + 1];
                    const uint32_t bits = word[u] >> sh0;
#pragma unroll
                    for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
                    {
                        const uint32_t code = (bits >> (kk * PS::SHIFT)) & PS::CODEMASK;
                        float x;
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
        float* colv = tile + (size_t) c * t.rows;
        const float* sc = sp + (size_t) c * t.rows;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t i = w + (chunk * PS::SLOTS + kk) * t.nq;
            if (i < t.rows)
            {
                if (agg_out != nullptr)
                    agg_out[base + (size_t) c * t.rows + i] = acc[kk];
                colv[i] = acc[kk] + __builtin_nontemporal_load(sc + i);
            }
        }
    }
    __syncthreads();

    char* qtile = q_out + (size_t) j0 * t.qcol;
    tile_stats<NBITS, ZT>(tile, hdr, scratch_f, scratch_u, t, nc, qtile);
    tile_pack<NBITS, ZT>(tile, hdr, words, t, nc, qtile, sp);
    if (t.stage_residual)
        tile_store(tile, mis_s, sp, total, t);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) void stripe_reduce_tile_kernel(StripeSources src, float* stripe_res,
                                                                          char* q_out, float* agg_out, TileGeom t)
{
    stripe_reduce_tile_body<NBITS, ZT>(src, stripe_res, q_out, agg_out, t, blockIdx.x);
}

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
    float* red_f;     // 2 * 4 floats
    uint32_t* red_u;  // 4
};

template <int PER>
__device__ __forceinline__ ColLds col_lds(f32x4* smem)
{
    ColLds l;
    l.tile = reinterpret_cast<float*>(smem);
    l.words = reinterpret_cast<uint32_t*>(l.tile + 1024 * PER);
    l.red_f = reinterpret_cast<float*>(l.words + 32 * PER);
    l.red_u = reinterpret_cast<uint32_t*>(l.red_f + 8);
    return l;
}

template <int PER>
constexpr size_t col_lds_bytes()
{
    return (size_t) (1024 * PER + 32 * PER + 8 + 4) * 4;
}

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
            l.red_f[wave] = s;
    }
    __syncthreads(); // the column and the wave sums are visible
    if constexpr (!ZT)
    {
        float s = l.red_f[0];
#pragma unroll
        for (uint32_t x = 1; x < NW; ++x)
            s += l.red_f[x];
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
    __syncthreads(); // everyone has read the wave sums of the mean
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
__global__ __launch_bounds__(kColThreads) void quantize_col_kernel(const float* __restrict__ g, const float* r_in, float* r_out,
                                                                   char* __restrict__ q, uint64_t qcol)
{
    constexpr uint32_t ROWS = 1024 * PER, T = kColThreads;
    extern __shared__ f32x4 smem_v4[];
    const ColLds l = col_lds<PER>(smem_v4);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * ROWS;
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
    col_stats_pack<ZT, PER>(l, col_thread_sum<PER>(a), r_out + base, q + (size_t) blockIdx.x * qcol);
}

// Stripe reduction in the same shape: the work item that will pack (QWord p, chunk) first decodes those bit positions
// from every worker's packed stripe, sums them (owner first, then ascending) and adds the stripe residual.
template <bool ZT, int PER>
__global__ __launch_bounds__(kColThreads) void stripe_reduce_col_kernel(StripeSources src, float* stripe_res, char* q_out,
                                                                        float* agg_out, uint64_t qcol)
{
    constexpr uint32_t ROWS = 1024 * PER, NQ = 32 * PER, T = kColThreads, KS = 4 * PER, BATCH = 8;
    extern __shared__ f32x4 smem_v4[];
    const ColLds l = col_lds<PER>(smem_v4);
    float* dec = reinterpret_cast<float*>(l.red_u + 4); // two reconstruction levels per worker, in summation order
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) blockIdx.x * ROWS;
    const size_t rec = (size_t) blockIdx.x * qcol;
    const uint32_t K = src.workers;
    if (tid < NQ)
        l.words[tid] = 0u;
    // Everything this thread will need from memory is requested before the first barrier, so that the headers, the
    // first eight workers' QWords and the stripe residual cost one round trip, not three: a stripe is one GPU's share
    // of a matrix, a single round of workgroups, and its time is the length of this dependent chain.
    const uint32_t p = tid % NQ, chunk = tid / NQ;
    const uint32_t sh0 = chunk * KS;
    uint32_t word[BATCH];
#pragma unroll
    for (uint32_t u = 0; u < BATCH; ++u)
        if (u < K)
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
                    const float x = ((bits >> kk) & 1u) ? val1 : val0;
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

// LDS in floats: [column | partial QWords (nq when a QWord has several work items) | 12 reduction slots | decode constants]
template <int NBITS>
__host__ __device__ inline size_t colg_lds_bytes(const ColGeom& c, uint32_t workers)
{
    return ((size_t) c.rows + (PackShape<NBITS>::CHUNKS > 1 ? c.nq : 0) + 12 + (size_t) 2 * workers) * sizeof(float);
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

// stat: this thread's running statistic over its pieces (unused for 1 bit with ZT). tile = the column, words = zeroed
// partial QWords, red = 12 reduction slots. No barrier is needed between writing the column and calling this.
// WG: threads in the workgroup. The sums are always taken by the first 256 threads (their order is part of the result);
// coding and packing use all of them.
template <int NBITS, bool ZT, int WG = kColThreads>
__device__ __forceinline__ void colg_stats_pack(float* tile, uint32_t* words, float* red, const ColGeom& c, float stat,
                                                uint32_t shift, float* res_col, char* qc)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t T = kColThreads, NW = T / 64;
    static_assert(WG >= (int) T && WG % 64 == 0, "workgroup size");
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 8);
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    float total = 0.0f;
    if constexpr (need_stat)
    {
        const float s = wave_sum(stat);
        if (lane == 0 && wave < NW)
            red[wave] = s;
    }
    __syncthreads(); // the column and the wave sums are visible
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
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile);
        if (WG == T || tid < T)
            for (uint32_t v = tid; v < c.pieces + shift; v += T)
                if (v >= shift)
                    split_add_piece(t4[v - shift], mean, s0, s1, n0);
        s0 = wave_sum(s0);
        s1 = wave_sum(s1);
        n0 = wave_sum(n0);
        __syncthreads(); // everyone has read the wave sums of the mean
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
    for (uint32_t it = tid; it < items; it += WG)
    {
        // chunk-major: consecutive threads take consecutive QWords, hence consecutive rows
        const uint32_t chunk = (PS::CHUNKS == 1) ? 0u : it / c.nq;
        const uint32_t w = it - chunk * c.nq;
        uint32_t word = 0;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t k = chunk * PS::SLOTS + kk;
            const uint32_t i = w + k * c.nq;
            if (i < c.rows)
            {
                const float v = tile[i];
                const uint32_t code = quantize_value<NBITS, ZT>(vq, v);
                float back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                __builtin_nontemporal_store(v - back, res_col + i);
                word |= code << (k * PS::SHIFT);
            }
        }
        if constexpr (PS::CHUNKS == 1)
            bits[w] = word;
        else
            atomicOr(&words[w], word);
    }
    if constexpr (PS::CHUNKS > 1)
    {
        __syncthreads();
        for (uint32_t w = tid; w < c.nq; w += WG)
            bits[w] = words[w];
    }
}

template <int NBITS, bool ZT>
__device__ __forceinline__ void quantize_colg_body(const float* __restrict__ g, const float* r_in, float* r_out, char* __restrict__ q,
                                                   const ColGeom& c, uint32_t column, f32x4* smem)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t T = kColThreads;
    float* tile = reinterpret_cast<float*>(smem);
    uint32_t* words = reinterpret_cast<uint32_t*>(tile + c.rows);
    float* red = tile + c.rows + (PS::CHUNKS > 1 ? c.nq : 0);
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t) column * c.rows;
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

// WG: threads in the workgroup (256, or 1024 for tall columns, whose many work items would otherwise be a long chain of
// dependent loads for each of few threads)
template <int NBITS, bool ZT, int WG = kColThreads>
__device__ __forceinline__ void stripe_reduce_colg_body(const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                                                        const ColGeom& c, uint32_t column, f32x4* smem)
{
    using PS = PackShape<NBITS>;
    constexpr uint32_t T = kColThreads, BATCH = 8;
    static_assert(WG >= (int) T, "workgroup size");
    float* tile = reinterpret_cast<float*>(smem);
    uint32_t* words = reinterpret_cast<uint32_t*>(tile + c.rows);
    float* red = tile + c.rows + (PS::CHUNKS > 1 ? c.nq : 0);
    float* dec = red + 12; // per worker, in summation order: 1 bit -> the two levels, else (ufactor, lower)
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
    const uint32_t items = c.nq * PS::CHUNKS;
    uint32_t word[BATCH];
    float resid[PS::SLOTS];
    if (tid < items)
    {
        const uint32_t chunk = (PS::CHUNKS == 1) ? 0u : tid / c.nq;
        const uint32_t w = tid - chunk * c.nq;
#pragma unroll
        for (uint32_t u = 0; u < BATCH; ++u)
            if (u < K)
                word[u] = *reinterpret_cast<const uint32_t*>(src.q[stripe_order(u, src.owner)] + rec + 8 + (size_t) w * 4);
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t i = w + (chunk * PS::SLOTS + kk) * c.nq;
            if (i < c.rows)
                resid[kk] = __builtin_nontemporal_load(sp + i);
        }
    }
    if (tid < K)
    {
        const float* h = reinterpret_cast<const float*>(src.q[stripe_order(tid, src.owner)] + rec);
        const ValueQ vq = make_vq<NBITS>(h[0], h[1]);
        if constexpr (NBITS == 1)
        {
            dec[2 * tid] = unquantize_value<NBITS>(vq, 0u);
            dec[2 * tid + 1] = unquantize_value<NBITS>(vq, 1u);
        }
        else
        {
            dec[2 * tid] = vq.uf;
            dec[2 * tid + 1] = vq.lo;
        }
    }
    __syncthreads();

    for (uint32_t it = tid; it < items; it += WG)
    {
        const uint32_t chunk = (PS::CHUNKS == 1) ? 0u : it / c.nq;
        const uint32_t w = it - chunk * c.nq;
        const size_t word_off = rec + 8 + (size_t) w * 4;
        const uint32_t sh0 = chunk * PS::SLOTS * PS::SHIFT;
        if (it != tid)
        {
#pragma unroll
            for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
            {
                const uint32_t i = w + (chunk * PS::SLOTS + kk) * c.nq;
                if (i < c.rows)
                    resid[kk] = __builtin_nontemporal_load(sp + i);
            }
        }
        float acc[PS::SLOTS];
        for (uint32_t n0 = 0; n0 < K; n0 += BATCH)
        {
            if (it != tid || n0 != 0)
            {
#pragma unroll
                for (uint32_t u = 0; u < BATCH; ++u)
                    if (n0 + u < K)
                        word[u] = *reinterpret_cast<const uint32_t*>(src.q[stripe_order(n0 + u, src.owner)] + word_off);
            }
#pragma unroll
            for (uint32_t u = 0; u < BATCH; ++u)
            {
                if (n0 + u < K)
                {
                    const float a = dec[2 * (n0 + u)];
                    const float b = dec[2 * (n0 + u) + 1];
                    const uint32_t bits = word[u] >> sh0;
#pragma unroll
                    for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
                    {
                        const uint32_t code = (bits >> (kk * PS::SHIFT)) & PS::CODEMASK;
                        float x;
                        if constexpr (NBITS == 1)
                            x = code ? b : a;
                        else
                            x = unquantize_value<NBITS>(a, b, code);
                        // the first term (the owner's) seeds the sum; afterwards: decoded value + running sum
                        acc[kk] = (n0 + u == 0) ? x : x + acc[kk];
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t i = w + (chunk * PS::SLOTS + kk) * c.nq;
            if (i < c.rows)
            {
                if (agg_out != nullptr)
                    agg_out[base + i] = acc[kk];
                tile[i] = acc[kk] + resid[kk];
            }
        }
    }
    float stat = 0.0f;
    // the quantize kernels' summation order for a residual at this address
    const uint32_t shift = column_shift(stripe_res + base, c.line_shift);
    if constexpr ((NBITS != 1) || !ZT)
    {
        __syncthreads();
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile);
        if (WG == T || tid < T)
            for (uint32_t v = tid; v < c.pieces + shift; v += T)
                if (v >= shift)
                    stat = colg_add_piece<NBITS>(stat, t4[v - shift]);
    }
    colg_stats_pack<NBITS, ZT, WG>(tile, words, red, c, stat, shift, stripe_res + base, q_out + rec);
}

template <int NBITS, bool ZT, int WG>
__global__ __launch_bounds__(WG) void stripe_reduce_colg_kernel(StripeSources src, float* stripe_res, char* q_out, float* agg_out,
                                                                ColGeom c)
{
    extern __shared__ f32x4 smem_v4[];
    stripe_reduce_colg_body<NBITS, ZT, WG>(src, stripe_res, q_out, agg_out, c, blockIdx.x, smem_v4);
}

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
    using PS = PackShape<NBITS>;
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    constexpr uint32_t NW = T / 64;
    extern __shared__ f32x4 smem_v4[];
    float* red = reinterpret_cast<float*>(smem_v4);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(red + 2 * NW);
    uint32_t* words = reinterpret_cast<uint32_t*>(red + kRegRedSlots);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
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
                    const uint32_t code = (bits[ww] >> (kk * PS::SHIFT)) & PS::CODEMASK;
                    float x;
                    if constexpr (NBITS == 1)
                        x = code ? val1 : val0;
                    else
                        x = unquantize_value<NBITS>(uf, lo, code);
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

// Many matrices in one launch: the workgroups of all matrices form one grid; `begins` (count + 1 entries, ascending)
// gives the first workgroup of every matrix. A matrix is a run of column tiles (quantize_tile_body) or of single columns
// (quantize_colg_body). Removes the per-launch floor (several microseconds) that dominates gradient sets made of many
// small matrices.
struct QuantizeBatchEntry
{
    const float* g;
    const float* r_in;
    float* r_out;
    char* q;
    uint32_t kind; // 0: tiles (t), 1: columns (c)
    uint32_t pad;
    TileGeom t;
    ColGeom c;
};

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) void quantize_batch_kernel(const QuantizeBatchEntry* __restrict__ entries,
                                                                      const uint32_t* __restrict__ begins, uint32_t count)
{
    extern __shared__ f32x4 smem_v4[];
    const uint32_t e = batch_find(begins, count, blockIdx.x);
    const uint32_t index = blockIdx.x - begins[e];
    // geometry by value: read once, then held in registers whatever the kernel stores
    if (entries[e].kind == 0)
    {
        const TileGeom t = entries[e].t;
        quantize_tile_body<NBITS, ZT>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, t, index);
    }
    else
    {
        const ColGeom c = entries[e].c;
        quantize_colg_body<NBITS, ZT>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, c, index, smem_v4);
    }
}

// The owner's stripe reductions of a whole gradient set in one launch: same grid construction as quantize_batch_kernel.
struct StripeBatchEntry
{
    StripeSources src;
    float* stripe_res;
    char* q_out;
    float* agg_out;
    uint32_t kind; // 0: tiles (t), 1: columns (c)
    uint32_t pad;
    TileGeom t;
    ColGeom c;
};

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) void stripe_reduce_batch_kernel(const StripeBatchEntry* __restrict__ entries,
                                                                           const uint32_t* __restrict__ begins, uint32_t count)
{
    extern __shared__ f32x4 smem_v4[];
    const uint32_t e = batch_find(begins, count, blockIdx.x);
    const uint32_t index = blockIdx.x - begins[e];
    const StripeBatchEntry& en = entries[e]; // the table is read-only while the kernel runs
    if (en.kind == 0)
    {
        const TileGeom t = en.t;
        stripe_reduce_tile_body<NBITS, ZT>(en.src, en.stripe_res, en.q_out, en.agg_out, t, index);
    }
    else
    {
        const ColGeom c = en.c;
        stripe_reduce_colg_body<NBITS, ZT>(en.src, en.stripe_res, en.q_out, en.agg_out, c, index, smem_v4);
    }
}

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

    if constexpr (NBITS == 1)
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

// ---- unquantize ---------------------------------------------------------------------------------------
//
// One thread decodes WV consecutive QWords of a column (WV = 4: 16-byte stores; WV = 1: any shape) for a
// chunk of `slots` consecutive bit positions. For fixed bit position k the rows w + k * nq of
// consecutive QWords are consecutive in memory, so stores coalesce.

struct UnqGeom
{
    uint32_t rows;
    uint32_t cols;
    uint32_t nq;
    uint32_t groups;  // ceil(nq / WV) word groups per column
    uint32_t chunks;  // ceil(VPW / slots)
    uint32_t slots;   // bit positions per thread
    uint32_t per_col; // groups * chunks work items per column
    uint32_t items;   // per_col * cols (the host refuses matrices that need more than 2^32 - 1)
    uint32_t swz_members; // > 1: workgroups are regrouped by XCD, this many share the same QWords (see unq_xcd_block)
    uint32_t swz_gw;      // workgroups side by side along the QWords of one column (1 when one workgroup spans them all)
    uint64_t qcol;
};

// The workgroups of a column that decode different bit positions of the same QWords read the same packed bytes.
// Consecutive workgroups go to the 8 XCDs in turn, each with its own L2; this permutation of the workgroup index puts
// the `members` workgroups of such a set 8 apart, i.e. on one XCD, so that the QWords are fetched once (measured
// without it: 4 to 4.5 times the packed bytes at 8192 and 65536 rows). Sets are taken in groups of 8; the remainder at
// the end keeps its order. Returns the logical workgroup index (column-major, then chunk of bit positions, then QWords).
__device__ __forceinline__ uint32_t unq_xcd_block(uint32_t b, uint32_t blocks, uint32_t members, uint32_t gw)
{
    const uint32_t per_group = 8 * members;
    const uint32_t grouped = (blocks / per_group) * per_group;
    uint32_t set, m;
    if (b < grouped)
    {
        const uint32_t grp = b / per_group;
        const uint32_t rem = b - grp * per_group;
        m = rem >> 3;
        set = grp * 8 + (rem & 7u);
    }
    else
    {
        const uint32_t r = b - grouped;
        const uint32_t ss = r / members;
        m = r - ss * members;
        set = grouped / members + ss;
    }
    const uint32_t c = set / gw;
    const uint32_t g = set - c * gw;
    return (c * members + m) * gw + g;
}

template <int NBITS, int WV>
__device__ __forceinline__ void unquantize_body(const char* __restrict__ q, float* out, const UnqGeom& t, int add, uint32_t block)
{
    constexpr uint32_t VPW = 32 / NBITS;
    constexpr uint32_t MASKBITS = NBITS & 31;
    constexpr uint32_t CODEMASK = (NBITS >= 32) ? 0xFFFFFFFFu : ((1u << MASKBITS) - 1u);

    if (t.swz_members > 1)
        block = unq_xcd_block(block, t.items / 256, t.swz_members, t.swz_gw);
    const uint64_t id64 = (uint64_t) block * 256 + threadIdx.x;
    if (id64 >= t.items)
        return;
    const uint32_t id = (uint32_t) id64;
    const uint32_t c = id / t.per_col;
    const uint32_t rem = id - c * t.per_col;
    const uint32_t chunk = rem / t.groups;
    const uint32_t grp = rem - chunk * t.groups;
    const uint32_t w0 = grp * WV;

    const char* qc = q + (size_t) c * t.qcol;
    const float* gh = reinterpret_cast<const float*>(qc);
    ValueQ vq; // decoding needs only the code -> value factor and the lower bound
    vq.lo = gh[0];
    vq.uf = make_ufactor<NBITS>(gh[0], gh[1]);
    const float val0 = unquantize_value<NBITS>(vq, 0u);
    const float val1 = unquantize_value<NBITS>(vq, 1u);
    const uint32_t* bits = reinterpret_cast<const uint32_t*>(qc + 8);
    float* oc = out + (size_t) c * t.rows;

    uint32_t word[WV];
    if constexpr (WV == 4)
    {
        // the word group starts 8 bytes past a 16-byte boundary or on one: two 8-byte loads are always aligned
        const u32x2 a = *reinterpret_cast<const u32x2*>(bits + w0);
        const u32x2 b = *reinterpret_cast<const u32x2*>(bits + w0 + 2);
        word[0] = a.x;
        word[1] = a.y;
        word[2] = b.x;
        word[3] = b.y;
    }
    else
    {
        word[0] = bits[w0];
    }

    const uint32_t k0 = chunk * t.slots;
    const uint32_t k1 = min(k0 + t.slots, VPW);
    for (uint32_t k = k0; k < k1; ++k)
    {
        const uint32_t i = w0 + k * t.nq;
        if (i >= t.rows)
            break; // rows only grow with k
        const uint32_t sh = k * MASKBITS;
        if constexpr (WV == 4)
        {
            // rows % 4 == 0 and i % 4 == 0: the four rows are all inside the column
            f32x4 x;
            if constexpr (NBITS == 1)
            {
                x.x = ((word[0] >> sh) & 1u) ? val1 : val0;
                x.y = ((word[1] >> sh) & 1u) ? val1 : val0;
                x.z = ((word[2] >> sh) & 1u) ? val1 : val0;
                x.w = ((word[3] >> sh) & 1u) ? val1 : val0;
            }
            else
            {
                x.x = unquantize_value<NBITS>(vq, (word[0] >> sh) & CODEMASK);
                x.y = unquantize_value<NBITS>(vq, (word[1] >> sh) & CODEMASK);
                x.z = unquantize_value<NBITS>(vq, (word[2] >> sh) & CODEMASK);
                x.w = unquantize_value<NBITS>(vq, (word[3] >> sh) & CODEMASK);
            }
            f32x4* dst = reinterpret_cast<f32x4*>(oc + i);
            if (add)
                x = x + *dst; // unquantized value + previous content
            __builtin_nontemporal_store(x, dst);
        }
        else
        {
            float x;
            if constexpr (NBITS == 1)
                x = ((word[0] >> sh) & 1u) ? val1 : val0;
            else
                x = unquantize_value<NBITS>(vq, (word[0] >> sh) & CODEMASK);
            if (add)
                x = x + oc[i];
            oc[i] = x;
        }
    }
}

template <int NBITS, int WV>
__global__ __launch_bounds__(256) void unquantize_kernel(const char* __restrict__ q, float* out, UnqGeom t, int add)
{
    unquantize_body<NBITS, WV>(q, out, t, add, blockIdx.x);
}

// Decoder with 16-byte stores for shapes the QWord-major decoder above can only serve with 4-byte stores
// (nq or rows not a multiple of 4, e.g. 100000 rows -> 3125 QWords). For one column and one bit position k the
// rows k * nq ... (k + 1) * nq - 1 are consecutive in memory: such a segment is cut into groups of four elements
// aligned to 16 bytes in the OUTPUT (the first and last group of a segment may be partial and use 4-byte stores).
struct UnqSegGeom
{
    uint32_t rows;
    uint32_t nq;
    uint32_t segs;    // bit positions in use per column: ceil(rows / nq)
    uint32_t gps;     // groups per segment
    uint32_t items;   // cols * segs * gps (the host refuses more than 2^32 - 1)
    double inv_gps;
    double inv_segs;
    uint64_t qcol;
};

template <int NBITS>
__device__ __forceinline__ void unquantize_segment_body(const char* __restrict__ q, float* out, const UnqSegGeom& t, int add,
                                                        uint32_t block)
{
    constexpr uint32_t SHIFT = NBITS & 31;
    constexpr uint32_t CODEMASK = (NBITS >= 32) ? 0xFFFFFFFFu : ((1u << SHIFT) - 1u);
    const uint64_t id64 = (uint64_t) block * 256 + threadIdx.x;
    if (id64 >= t.items)
        return;
    uint32_t seg, g, c, k;
    divmod_u32((uint32_t) id64, t.gps, t.inv_gps, seg, g);
    divmod_u32(seg, t.segs, t.inv_segs, c, k);
    const uint32_t row0 = k * t.nq;
    const uint32_t seg_len = min(t.nq, t.rows - row0);
    const size_t obase = (size_t) c * t.rows + row0;       // out is 16-byte aligned (checked by the host)
    const int32_t first = (int32_t) (4u * g) - (int32_t) (obase & 3u); // QWord index of this group's first element
    if (first >= (int32_t) seg_len)
        return;

    const char* qc = q + (size_t) c * t.qcol;
    const float* gh = reinterpret_cast<const float*>(qc);
    const float lo = gh[0];
    const float uf = make_ufactor<NBITS>(lo, gh[1]);
    const uint32_t* bits = reinterpret_cast<const uint32_t*>(qc + 8);
    const uint32_t sh = k * SHIFT;
    float* dst = out + obase;

    if (first >= 0 && first + 3 < (int32_t) seg_len)
    {
        f32x4 v;
        v.x = unquantize_value<NBITS>(uf, lo, (bits[first] >> sh) & CODEMASK);
        v.y = unquantize_value<NBITS>(uf, lo, (bits[first + 1] >> sh) & CODEMASK);
        v.z = unquantize_value<NBITS>(uf, lo, (bits[first + 2] >> sh) & CODEMASK);
        v.w = unquantize_value<NBITS>(uf, lo, (bits[first + 3] >> sh) & CODEMASK);
        f32x4* d4 = reinterpret_cast<f32x4*>(dst + first);
        if (add)
            v = v + *d4;
        __builtin_nontemporal_store(v, d4);
    }
    else
    {
        for (int32_t e = 0; e < 4; ++e)
        {
            const int32_t w = first + e;
            if (w >= 0 && w < (int32_t) seg_len)
            {
                const float x = unquantize_value<NBITS>(uf, lo, (bits[w] >> sh) & CODEMASK);
                dst[w] = add ? x + dst[w] : x;
            }
        }
    }
}

template <int NBITS>
__global__ __launch_bounds__(256) void unquantize_segment_kernel(const char* __restrict__ q, float* out, UnqSegGeom t, int add)
{
    unquantize_segment_body<NBITS>(q, out, t, add, blockIdx.x);
}

// Row-major decoder for columns of 1024 rows and more whose QWord-major stores would not be whole lines (9304 rows -> 291
// QWords, 100000 -> 3125, 50257 -> 1571): a workgroup copies the packed column into LDS once (every QWord is used by
// up to 32 rows) and then walks a chunk of consecutive rows, four per thread and store, so that all stores are aligned
// 16-byte stores whatever the QWord count, the height and the alignment of the output.
struct UnqRowGeom
{
    uint32_t rows;
    uint32_t nq;
    uint32_t chunk;  // rows per workgroup, multiple of 4 (the last workgroup of a column also takes the remainder)
    uint32_t chunks; // workgroups per column
    uint32_t blocks; // cols * chunks
    uint32_t pad;
    uint64_t qcol;
};

// Which (column, chunk) a workgroup of the row-major decoder takes. Consecutive workgroups go to the 8 XCDs in turn and
// every XCD has its own L2, so the chunks of one column are given to workgroups 8 apart: they then read the column's
// packed record through one L2 instead of fetching it once per XCD. Columns are taken in groups of 8; what is left over
// at the end is dealt column by column.
__device__ __forceinline__ void unq_rows_block_to_chunk(uint32_t block, uint32_t chunks, uint32_t blocks, uint32_t& c, uint32_t& ch)
{
    const uint32_t per_group = 8 * chunks;
    const uint32_t grouped = (blocks / per_group) * per_group;
    if (block < grouped)
    {
        const uint32_t grp = block / per_group;
        const uint32_t rem = block - grp * per_group;
        ch = rem >> 3;
        c = grp * 8 + (rem & 7u);
    }
    else
    {
        const uint32_t b = block - grouped;
        const uint32_t cc = b / chunks;
        ch = b - cc * chunks;
        c = grouped / chunks + cc;
    }
}

template <int NBITS>
__device__ __forceinline__ void unquantize_rows_body(const char* __restrict__ q, float* out, const UnqRowGeom& t, int add, uint32_t block,
                                                     uint32_t* words)
{
    constexpr uint32_t SHIFT = NBITS & 31;
    constexpr uint32_t CODEMASK = (NBITS >= 32) ? 0xFFFFFFFFu : ((1u << SHIFT) - 1u);
    const uint32_t tid = threadIdx.x;
    uint32_t c, ch;
    unq_rows_block_to_chunk(block, t.chunks, t.blocks, c, ch);
    const char* qc = q + (size_t) c * t.qcol;
    const float* gh = reinterpret_cast<const float*>(qc);
    const float lo = gh[0];
    const float uf = make_ufactor<NBITS>(lo, gh[1]);
    const uint32_t* bits = reinterpret_cast<const uint32_t*>(qc + 8);
    if (t.nq <= 1024)
    {
        for (uint32_t w = tid; w < t.nq; w += 256)
            words[w] = bits[w];
    }
    else
    {
        // eight loads in flight per thread: a tall column has thousands of QWords, and one round trip for every 256 of
        // them would cost more than the decoding
        for (uint32_t w = tid; w < t.nq; w += 8 * 256)
        {
            uint32_t v[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                v[u] = bits[(w + 256 * u < t.nq) ? w + 256 * u : w];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                if (w + 256 * u < t.nq)
                    words[w + 256 * u] = v[u];
        }
    }
    __syncthreads();
    // The column need not start on a 16-byte boundary nor hold a multiple of 4 rows: `head` rows (0..3) lie before its
    // first aligned group of four and `tail` rows (0..3) after the last; chunks are counted from the first aligned row,
    // the first chunk's workgroup also writes the head rows, the last one's the tail rows, one row per thread.
    float* oc = out + (size_t) c * t.rows;
    const uint32_t head = (4u - (uint32_t) ((reinterpret_cast<uintptr_t>(oc) >> 2) & 3u)) & 3u;
    const uint32_t body = (t.rows - head) & ~3u; // rows in aligned groups of four
    const uint32_t tail = t.rows - head - body;
    const uint32_t r0 = ch * t.chunk;
    const uint32_t pieces = ((ch + 1 == t.chunks ? body : r0 + t.chunk) - r0) >> 2; // the last chunk runs to the end
    f32x4* o4 = reinterpret_cast<f32x4*>(oc + head + r0);
    const float val0 = unquantize_value<NBITS>(uf, lo, 0u);
    const float val1 = unquantize_value<NBITS>(uf, lo, 1u);
    {
        uint32_t row = t.rows; // none
        if (ch == 0 && tid < head)
            row = tid;
        else if (ch + 1 == t.chunks && tid >= 4 && tid < 4 + tail)
            row = head + body + (tid - 4);
        if (row < t.rows)
        {
            const uint32_t k = row / t.nq;
            const uint32_t code = (words[row - k * t.nq] >> (k * SHIFT)) & CODEMASK;
            float x;
            if constexpr (NBITS == 1)
                x = code ? val1 : val0;
            else
                x = unquantize_value<NBITS>(uf, lo, code);
            oc[row] = add ? x + oc[row] : x;
        }
    }
    // Slot v = tid, tid + 256, ... holds piece v - shift, shift = the chunk's offset into its 128-byte line in pieces, so
    // that every wavefront's 64 stores cover whole lines also where columns do not start on one (9304 rows).
    const uint32_t shift = (uint32_t) ((reinterpret_cast<uintptr_t>(o4) >> 4) & 7u);
    const uint32_t vfirst = tid < shift ? tid + 256 : tid;
    // row i sits in QWord i % nq at bit position i / nq; a thread's pieces are 1024 rows apart
    const uint32_t i0 = head + r0 + 4 * (vfirst - shift);
    uint32_t k0 = i0 / t.nq;
    uint32_t w0 = i0 - k0 * t.nq;
    const uint32_t dk = 1024u / t.nq;
    const uint32_t dw = 1024u - dk * t.nq;
    for (uint32_t p = vfirst - shift; p < pieces; p += 256)
    {
        uint32_t k = k0, w = w0;
        f32x4 x;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            const uint32_t code = (words[w] >> (k * SHIFT)) & CODEMASK;
            if constexpr (NBITS == 1)
                x[e] = code ? val1 : val0;
            else
                x[e] = unquantize_value<NBITS>(uf, lo, code);
            if (++w == t.nq)
            {
                w = 0;
                ++k;
            }
        }
        if (add)
            x = x + o4[p]; // unquantized value + previous content
        __builtin_nontemporal_store(x, o4 + p);
        k0 += dk;
        w0 += dw;
        if (w0 >= t.nq)
        {
            w0 -= t.nq;
            ++k0;
        }
    }
}

template <int NBITS>
__global__ __launch_bounds__(256) void unquantize_rows_kernel(const char* __restrict__ q, float* out, UnqRowGeom t, int add)
{
    extern __shared__ f32x4 smem_v4[];
    unquantize_rows_body<NBITS>(q, out, t, add, blockIdx.x, reinterpret_cast<uint32_t*>(smem_v4));
}

// Tile decoder for short columns. Consecutive columns are adjacent in the packed matrix and in the output, so a
// workgroup takes `cpt` columns at once: their packed records (one contiguous run) go to LDS in coalesced loads, each
// column's decoding constants are computed once, and the cpt * rows values (one contiguous run) leave in aligned
// 16-byte stores, four consecutive elements per thread and store, whatever the column height: a group of four may
// straddle columns. cpt is a multiple of 4, so every tile starts on a 16-byte boundary of an aligned output.
struct UnqTileGeom
{
    uint32_t rows;
    uint32_t cols;
    uint32_t nq;
    uint32_t cpt;        // columns per workgroup
    uint32_t rec_words;  // nq + 2: 32-bit words per packed record
    uint32_t rows_magic; // ceil(2^32 / rows) (unused when rows == 1)
    uint32_t nq_magic;   // ceil(2^32 / nq) (unused when nq == 1)
    uint32_t blocks;
};

__host__ __device__ inline size_t unq_tile_lds_bytes(const UnqTileGeom& t)
{
    return (size_t) t.cpt * (t.rec_words + 2) * 4;
}

// x / d for x * d < 2^32 with magic = ceil(2^32 / d)
__device__ __forceinline__ uint32_t small_div(uint32_t x, uint32_t d, uint32_t magic)
{
    return d == 1 ? x : __umulhi(x, magic);
}

template <int NBITS>
__device__ __forceinline__ void unquantize_tile_body(const char* __restrict__ q, float* out, const UnqTileGeom& t, int add, uint32_t block,
                                                     uint32_t* smem)
{
    constexpr uint32_t SHIFT = NBITS & 31;
    constexpr uint32_t CODEMASK = (NBITS >= 32) ? 0xFFFFFFFFu : ((1u << SHIFT) - 1u);
    const uint32_t tid = threadIdx.x;
    const uint32_t col0 = block * t.cpt;
    const uint32_t ncols = (t.cols - col0 < t.cpt) ? t.cols - col0 : t.cpt;
    uint32_t* words = smem;                                          // ncols packed records
    float* dec = reinterpret_cast<float*>(smem + t.cpt * t.rec_words); // per column: the two levels (1 bit) or (ufactor, lower)
    const uint32_t* src = reinterpret_cast<const uint32_t*>(q + (size_t) col0 * t.rec_words * 4);
    const uint32_t total_words = ncols * t.rec_words;
    for (uint32_t x = tid; x < total_words; x += 256)
        words[x] = __builtin_nontemporal_load(src + x);
    __syncthreads();
    for (uint32_t c = tid; c < ncols; c += 256)
    {
        const float lo = __uint_as_float(words[c * t.rec_words]);
        const float hi = __uint_as_float(words[c * t.rec_words + 1]);
        const float uf = make_ufactor<NBITS>(lo, hi);
        if constexpr (NBITS == 1)
        {
            dec[2 * c] = unquantize_value<NBITS>(uf, lo, 0u);
            dec[2 * c + 1] = unquantize_value<NBITS>(uf, lo, 1u);
        }
        else
        {
            dec[2 * c] = uf;
            dec[2 * c + 1] = lo;
        }
    }
    __syncthreads();
    const uint32_t elems = ncols * t.rows;
    float* o = out + (size_t) col0 * t.rows;
    // slots dealt by 128-byte lines: slot v = tid, tid + 256, ... holds the group of four that starts at element
    // 4 * (v - shift), shift = the tile's offset into its line in 16-byte pieces
    const uint32_t shift = (uint32_t) ((reinterpret_cast<uintptr_t>(o) >> 4) & 7u);
    for (uint32_t i = 4 * ((tid < shift ? tid + 256 : tid) - shift); i < elems; i += 1024)
    {
        uint32_t c = small_div(i, t.rows, t.rows_magic);
        uint32_t r = i - c * t.rows;
        uint32_t k = small_div(r, t.nq, t.nq_magic);
        uint32_t w = r - k * t.nq;
        const uint32_t* cw = words + c * t.rec_words + 2;
        float d0 = dec[2 * c], d1 = dec[2 * c + 1];
        f32x4 x;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            // (past the end of the matrix c == ncols: the reads stay inside the LDS block and the value is not stored)
            const uint32_t code = (cw[w] >> (k * SHIFT)) & CODEMASK;
            if constexpr (NBITS == 1)
                x[e] = code ? d1 : d0;
            else
                x[e] = unquantize_value<NBITS>(d0, d1, code);
            ++r;
            if (++w == t.nq)
            {
                w = 0;
                ++k;
            }
            if (r == t.rows)
            {
                r = 0;
                k = 0;
                w = 0;
                c = (c + 1 < t.cpt) ? c + 1 : c;
                cw = words + c * t.rec_words + 2;
                d0 = dec[2 * c];
                d1 = dec[2 * c + 1];
            }
        }
        if (i + 4 <= elems)
        {
            f32x4* o4 = reinterpret_cast<f32x4*>(o + i);
            if (add)
                x = x + *o4; // unquantized value + previous content
            __builtin_nontemporal_store(x, o4);
        }
        else
        {
            for (uint32_t e = 0; i + e < elems; ++e)
                o[i + e] = add ? x[e] + o[i + e] : x[e];
        }
    }
}

template <int NBITS>
__global__ __launch_bounds__(256) void unquantize_tile_kernel(const char* __restrict__ q, float* out, UnqTileGeom t, int add)
{
    extern __shared__ f32x4 smem_v4[];
    unquantize_tile_body<NBITS>(q, out, t, add, blockIdx.x, reinterpret_cast<uint32_t*>(smem_v4));
}

// Many matrices in one launch (see quantize_batch_kernel): the 256-thread blocks of all matrices form one grid.
enum UnqKind : uint32_t
{
    kUnqVec4 = 0,    // QWord-major, 16-byte stores
    kUnqScalar = 1,  // QWord-major, 4-byte stores
    kUnqSegment = 2, // segment decoder
    kUnqRows = 3,    // row-major decoder, packed column in LDS
    kUnqTile = 4     // several short columns per workgroup, packed records in LDS
};

struct UnquantizeBatchEntry
{
    const char* q;
    float* out;
    uint32_t kind;
    uint32_t pad;
    UnqGeom qw;      // valid for kUnqVec4 / kUnqScalar
    UnqSegGeom seg;  // valid for kUnqSegment
    UnqRowGeom rowg; // valid for kUnqRows
    UnqTileGeom tile; // valid for kUnqTile
};

template <int NBITS>
__global__ __launch_bounds__(256) void unquantize_batch_kernel(const UnquantizeBatchEntry* __restrict__ entries,
                                                               const uint32_t* __restrict__ begins, uint32_t count, int add)
{
    extern __shared__ f32x4 smem_v4[];
    const uint32_t e = batch_find(begins, count, blockIdx.x);
    const UnquantizeBatchEntry& en = entries[e];
    const uint32_t block = blockIdx.x - begins[e];
    if (en.kind == kUnqVec4)
        unquantize_body<NBITS, 4>(en.q, en.out, en.qw, add, block);
    else if (en.kind == kUnqScalar)
        unquantize_body<NBITS, 1>(en.q, en.out, en.qw, add, block);
    else if (en.kind == kUnqSegment)
        unquantize_segment_body<NBITS>(en.q, en.out, en.seg, add, block);
    else if (en.kind == kUnqRows)
    {
        const UnqRowGeom t = en.rowg; // by value: the loop below stores between its uses
        unquantize_rows_body<NBITS>(en.q, en.out, t, add, block, reinterpret_cast<uint32_t*>(smem_v4));
    }
    else
    {
        const UnqTileGeom t = en.tile;
        unquantize_tile_body<NBITS>(en.q, en.out, t, add, block, reinterpret_cast<uint32_t*>(smem_v4));
    }
}

} // namespace cntkq
