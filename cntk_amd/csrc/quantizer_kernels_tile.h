// gfx950 kernels of the per-column gradient quantizer: column tiles in LDS (several short columns per workgroup),
// for quantize and for the stripe reduction.
#pragma once

#include "quantizer_kernels_common.h"

namespace cntkq {

// ---- statistics + packing of a tile that already sits in LDS --------------------------------------
//
// tile[c * rows + i] holds v(i, c) = value to quantize for tile column c. On return the column headers are
// in global memory and in hdr[], codes are in global memory and the new residual v - unquantize(code) has
// been written to res_out (dense, column-major, tile-relative).

template <int NBITS, bool ZT, typename E, typename Geom>
__device__ __forceinline__ void tile_stats(const E* tile, E* hdr, E* scratch_f, uint32_t* scratch_u, const Geom& t, uint32_t nc, char* qtile)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t c = tid >> t.gs_log2;
    const uint32_t lg = tid & (t.gs - 1);
    const bool col_ok = c < nc;
    const E* colv = tile + (size_t) c * t.rows;
    E lo = (E) 0, hi = (E) 0;

    if constexpr (NBITS == 1)
    {
        E mean = (E) 0;
        if constexpr (!ZT)
        {
            E s = (E) 0;
            if (col_ok)
                for (uint32_t i = lg; i < t.rows; i += t.gs)
                    s += colv[i];
            s = group_sum(s, t.gs, scratch_f);
            mean = s / (E) t.rows;
        }
        E s0 = (E) 0, s1 = (E) 0;
        uint32_t n0 = 0;
        if (col_ok)
        {
            for (uint32_t i = lg; i < t.rows; i += t.gs)
            {
                const E v = colv[i];
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
        E s = (E) 0;
        if (col_ok)
        {
            for (uint32_t i = lg; i < t.rows; i += t.gs)
            {
                const E v = colv[i];
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
        // (a float record is only 4-byte aligned when the column has an odd number of QWords)
        E* gh = reinterpret_cast<E*>(qtile + (size_t) c * t.qcol);
        gh[0] = lo;
        gh[1] = hi;
    }
    __syncthreads();
}

__device__ __forceinline__ void lds_or(uint32_t* p, uint32_t v) { atomicOr(p, v); }
__device__ __forceinline__ void lds_or(uint64_t* p, uint64_t v) { atomicOr(reinterpret_cast<unsigned long long*>(p), (unsigned long long) v); }

// words[] (LDS, nc * nq entries) must be zero on entry when a QWord has several work items (PackShape CHUNKS > 1).
// stage: the new residual replaces the value in the tile (every value is read by exactly one work item) and the caller
// writes the tile out afterwards; otherwise it goes straight to res_out. Written over the element type (E, its QWord) and
// the tile geometry of either precision; the workgroup's size is blockDim.x.
template <int NBITS, bool ZT, typename E, typename Geom>
__device__ __forceinline__ void tile_pack(E* tile, const E* hdr, typename Word<E>::Q* words, const Geom& t, bool stage, uint32_t nc, char* qtile,
                                          E* res_out)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    const uint32_t threads = blockDim.x;
    const uint32_t nwords = nc * t.nq;
    const uint32_t items = nwords * PS::CHUNKS;
    // (a tile lives in LDS, so its item numbers are far below the 2^20 that small_div takes)
    const float inv_nwords = small_divisor(nwords), inv_nq = small_divisor(t.nq);
    for (uint32_t it = threadIdx.x; it < items; it += threads)
    {
        // chunk-major: consecutive threads take consecutive QWords, hence consecutive rows
        const uint32_t chunk = (PS::CHUNKS == 1 || nc == 1) ? (PS::CHUNKS == 1 ? 0u : it / nwords) : small_div(it, inv_nwords);
        const uint32_t qi = it - chunk * nwords;
        const uint32_t c = (nc == 1) ? 0u : small_div(qi, inv_nq);
        const uint32_t w = qi - c * t.nq;
        const ValueQOf<E> vq = make_vq<NBITS>(hdr[2 * c], hdr[2 * c + 1]);
        const E val0 = unquantize_value<NBITS>(vq, 0u);
        const E val1 = unquantize_value<NBITS>(vq, 1u);
        E* colv = tile + (size_t) c * t.rows;
        E* ro = res_out + (size_t) c * t.rows;
        QWord word = 0;
#pragma unroll
        for (uint32_t kk = 0; kk < PS::SLOTS; ++kk)
        {
            const uint32_t k = chunk * PS::SLOTS + kk;
            const uint32_t i = w + k * t.nq;
            if (i < t.rows)
            {
                const E v = colv[i];
                const QWord code = quantize_value<NBITS, ZT>(vq, v);
                E back;
                if constexpr (NBITS == 1)
                    back = code ? val1 : val0;
                else
                    back = unquantize_value<NBITS>(vq, code);
                const E res = v - back;
                if (stage)
                    colv[i] = res; // this element belongs to this work item alone
                else
                    __builtin_nontemporal_store(res, ro + i);
                word |= code << (k * PS::SHIFT);
            }
        }
        if constexpr (PS::CHUNKS == 1)
            reinterpret_cast<QWord*>(qtile + (size_t) c * t.qcol + 2 * sizeof(E))[w] = word;
        else
            lds_or(&words[qi], word);
    }
    if constexpr (PS::CHUNKS > 1)
    {
        __syncthreads();
        for (uint32_t qi = threadIdx.x; qi < nwords; qi += threads)
        {
            const uint32_t c = (nc == 1) ? 0u : small_div(qi, inv_nq);
            const uint32_t w = qi - c * t.nq;
            reinterpret_cast<QWord*>(qtile + (size_t) c * t.qcol + 2 * sizeof(E))[w] = words[qi];
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
        // the destination at another phase: 16-byte stores all the same, at the 4-byte alignment that leaves them (a
        // store per element costs four times the instructions; quantize + unquantize of 2048 x 9304 with the gradient one
        // float off the residual: 73 -> 58 us, 512 x 37216: 71 -> 58 us)
        uint32_t head = (4u - mis) & 3u;
        if (head > total)
            head = total;
        const uint32_t nvec = (total - head) >> 2;
        const uint32_t tail0 = head + (nvec << 2);
        if (tid < head)
            dst[tid] = tile[tid];
        const f32x4* t4 = reinterpret_cast<const f32x4*>(tile + head);
        f32x4_u* d4 = reinterpret_cast<f32x4_u*>(dst + head);
        for (uint32_t e = tid; e < nvec; e += t.threads)
            __builtin_nontemporal_store(t4[e], d4 + e);
        for (uint32_t e = tail0 + tid; e < total; e += t.threads)
            dst[e] = tile[e];
    }
}

// The reverse: a coalesced copy of `total` floats into the tile (same phase rule).
__device__ __forceinline__ void tile_load(float* tile, uint32_t mis, const float* src, uint32_t total, const TileGeom& t)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t mis_s = (uint32_t) ((reinterpret_cast<uintptr_t>(src) >> 2) & 3u);
    if (mis_s == mis)
    {
        uint32_t head = (4u - mis) & 3u;
        if (head > total)
            head = total;
        const uint32_t nvec = (total - head) >> 2;
        const uint32_t tail0 = head + (nvec << 2);
        if (tid < head)
            tile[tid] = src[tid];
        f32x4* t4 = reinterpret_cast<f32x4*>(tile + head);
        const f32x4* s4 = reinterpret_cast<const f32x4*>(src + head);
        for (uint32_t e = tid; e < nvec; e += t.threads)
            t4[e] = __builtin_nontemporal_load(s4 + e);
        for (uint32_t e = tail0 + tid; e < total; e += t.threads)
            tile[e] = src[e];
    }
    else
    {
        for (uint32_t e = tid; e < total; e += t.threads)
            tile[e] = __builtin_nontemporal_load(src + e);
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
        // the residual at another phase than the gradient: the gradient in aligned pieces, the residual in 16-byte loads at
        // the 4-byte alignment that leaves them
        uint32_t head = (4u - mis_g) & 3u;
        if (head > total)
            head = total;
        const uint32_t nvec = (total - head) >> 2;
        const uint32_t tail0 = head + (nvec << 2);
        if (tid < head)
            tile[tid] = gp[tid] + rp[tid];
        const f32x4* g4 = reinterpret_cast<const f32x4*>(gp + head);
        const f32x4_u* r4 = reinterpret_cast<const f32x4_u*>(rp + head);
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
    __syncthreads();

    char* qtile = q + (size_t) j0 * t.qcol;
    tile_stats<NBITS, ZT>(tile, hdr, scratch_f, scratch_u, t, nc, qtile);
    tile_pack<NBITS, ZT>(tile, hdr, words, t, t.stage_residual != 0, nc, qtile, r_out + base);
    if (t.stage_residual)
        tile_store(tile, mis_g, r_out + base, total, t);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) void quantize_tile_kernel(const float* __restrict__ g, const float* r_in,
                                                                     float* r_out, char* __restrict__ q, TileGeom t)
{
    quantize_tile_body<NBITS, ZT>(g, r_in, r_out, q, t, blockIdx.x);
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

    // the stripe residual comes in as one consecutive run where it also leaves as one: a work item's rows lie nq apart, and
    // short columns (few QWords) would otherwise be read in fragments
    const bool staged = t.stage_residual != 0;
    if (staged)
        tile_load(tile, mis_s, sp, total, t);

    // decode constants from every worker's column header, stored in summation order:
    // 1 bit -> the two levels, else (ufactor, lower)
    const float inv_k = small_divisor(K);
    for (uint32_t x = tid; x < nc * K; x += t.threads)
    {
        const uint32_t c = small_div(x, inv_k);
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
    const float inv_nwords = small_divisor(nwords), inv_nq = small_divisor(t.nq);
    for (uint32_t it = tid; it < items; it += t.threads)
    {
        const uint32_t chunk = (PS::CHUNKS == 1 || nc == 1) ? (PS::CHUNKS == 1 ? 0u : it / nwords) : small_div(it, inv_nwords);
        const uint32_t qi = it - chunk * nwords;
        const uint32_t c = (nc == 1) ? 0u : small_div(qi, inv_nq);
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
                        float x;
                        if constexpr (NBITS == 1)
                            x = pick_level(bits, kk, a, b);
                        else
                            x = unquantize_value<NBITS>(a, b, (bits >> (kk * PS::SHIFT)) & PS::CODEMASK);
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
                colv[i] = acc[kk] + (staged ? colv[i] : __builtin_nontemporal_load(sc + i));
            }
        }
    }
    __syncthreads();

    char* qtile = q_out + (size_t) j0 * t.qcol;
    tile_stats<NBITS, ZT>(tile, hdr, scratch_f, scratch_u, t, nc, qtile);
    tile_pack<NBITS, ZT>(tile, hdr, words, t, t.stage_residual != 0, nc, qtile, sp);
    if (t.stage_residual)
        tile_store(tile, mis_s, sp, total, t);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) CNTKQ_SGPRS_FOR_8_WAVES void stripe_reduce_tile_kernel(StripeSources src, float* stripe_res,
                                                                          char* q_out, float* agg_out, TileGeom t)
{
    stripe_reduce_tile_body<NBITS, ZT>(src, stripe_res, q_out, agg_out, t, blockIdx.x);
}

} // namespace cntkq
