// Host-side kernel selection and launch for the per-column quantizer (gfx950).
// Shared by the C-ABI library and by stand-alone timing programs; no allocation happens here.
#pragma once

#include "quantizer_kernels.h"

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace cntkq {

// which quantize kernel to use
enum QuantizePath
{
    kPathAuto = 0,
    kPathTile = 1,    // LDS-staged column tile (rows <= kTileMaxRows)
    kPathTall = 2,    // one workgroup per column, global re-read (any rows)
    kPathWaveCol = 3  // 1 bit, rows in {2048, 4096}, one wavefront per column in registers
};

constexpr uint32_t kTileMaxRows = 14336; // 56 KB of LDS for a one-column tile

struct LaunchTuning
{
    int quantize_path = kPathAuto;
    uint32_t tile_gs = 0;   // 0 = pick from rows; else threads per column (power of two, 8..256)
    int tile_stage = -1;    // -1 = automatic; 0 / 1 = residual written straight to memory / staged through LDS
    uint32_t tile_threads = 0; // 0 = automatic; else workgroup size of the tile kernels (64, 128, 256)
    uint32_t unq_slots = 0; // 0 = default; else bit positions per thread in unquantize
    int unq_force_scalar = 0;
};

// Events tied to the kernel dispatch itself (its completion signal), not recorded as separate stream
// commands: a separate record after every kernel costs about 3 us of idle GPU per launch on MI355X.
struct LaunchEvents
{
    hipEvent_t start = nullptr; // optional: set when the kernel starts
    hipEvent_t stop = nullptr;  // optional: set when the kernel has finished
};

inline bool valid_nbits(size_t nbits)
{
    return nbits == 1 || nbits == 2 || nbits == 4 || nbits == 8 || nbits == 16 || nbits == 32;
}

inline size_t qwords_per_col(size_t rows, size_t nbits)
{
    const size_t per = 32 / nbits;
    return (rows + per - 1) / per;
}

inline size_t qcol_bytes(size_t nbits, size_t rows)
{
    return 8 + ((rows * nbits + 31) / 32) * 4;
}

inline TileGeom make_tile_geom(size_t rows, size_t cols, size_t nbits, uint32_t gs_override, int stage = -1,
                               uint32_t threads_override = 0)
{
    TileGeom t;
    t.rows = (uint32_t) rows;
    t.cols = (uint32_t) cols;
    t.nq = (uint32_t) qwords_per_col(rows, nbits);
    uint32_t threads = threads_override != 0 ? threads_override : kTileThreads;
    uint32_t gs = 8;
    if (gs_override != 0)
        gs = gs_override;
    else
        while (gs < threads && rows > (size_t) gs * 32)
            gs <<= 1;
    if (gs > threads)
        gs = threads;
    // a tile may not exceed 4096 floats (16 KB) unless it is a single column: small tiles keep many
    // workgroups resident per CU, which is what hides the barrier-separated phases of each of them
    while (gs < threads && (size_t) (threads / gs) * rows > 4096)
        gs <<= 1;
    t.threads = threads;
    t.gs = gs;
    t.gs_log2 = 0;
    while ((1u << t.gs_log2) < gs)
        t.gs_log2++;
    t.cols_per_tile = threads / gs;
    t.tile_floats = (uint32_t) (((size_t) t.cols_per_tile * rows + 4 + 3) & ~(size_t) 3);
    t.words_floats = (nbits <= 2) ? t.cols_per_tile * t.nq : 0;
    t.stage_residual = (stage < 0) ? 1u : (uint32_t) (stage != 0);
    t.qcol = qcol_bytes(nbits, rows);
    return t;
}

template <template <int, bool> class Launcher, typename... Args>
inline hipError_t dispatch_nbits(size_t nbits, bool zt, Args... args)
{
    switch (nbits)
    {
    case 1: return zt ? Launcher<1, true>::run(args...) : Launcher<1, false>::run(args...);
    case 2: return Launcher<2, false>::run(args...);
    case 4: return Launcher<4, false>::run(args...);
    case 8: return Launcher<8, false>::run(args...);
    case 16: return Launcher<16, false>::run(args...);
    case 32: return Launcher<32, false>::run(args...);
    default: return hipErrorInvalidValue;
    }
}

template <int NBITS, bool ZT>
struct TileLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, TileGeom t)
    {
        const uint32_t tiles = (t.cols + t.cols_per_tile - 1) / t.cols_per_tile;
        const size_t lds = tile_lds_bytes(t, 0);
        hipExtLaunchKernelGGL((quantize_tile_kernel<NBITS, ZT>), dim3(tiles), dim3(t.threads), lds, s, ev.start, ev.stop, 0, g, r_in, r_out, q, t);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct TallLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, uint32_t rows,
                          uint32_t cols, uint32_t nq, uint64_t qcol)
    {
        hipExtLaunchKernelGGL((quantize_tall_kernel<NBITS, ZT>), dim3(cols), dim3(kTallThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out, q, rows,
                           nq, qcol);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct StripeLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out, float* agg_out,
                          TileGeom t)
    {
        const uint32_t tiles = (t.cols + t.cols_per_tile - 1) / t.cols_per_tile;
        const size_t lds = tile_lds_bytes(t, src.workers);
        hipExtLaunchKernelGGL((stripe_reduce_tile_kernel<NBITS, ZT>), dim3(tiles), dim3(t.threads), lds, s, ev.start, ev.stop, 0, src, stripe_res,
                           q_out, agg_out, t);
        return hipGetLastError();
    }
};

inline bool wavecol_applicable(const float* g, const float* r_in, const float* r_out, const void* q, size_t rows,
                               size_t nbits)
{
    (void) g, (void) r_in, (void) r_out;
    return nbits == 1 && (rows == 2048 || rows == 4096) && (reinterpret_cast<uintptr_t>(q) & 7u) == 0;
}

// Launches the quantize kernel(s) for one matrix. rows, cols > 0; pointers 4-byte aligned (checked by caller).
inline hipError_t launch_quantize(hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, void* q, size_t rows,
                                  size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    char* qc = static_cast<char*>(q);
    int path = tune.quantize_path;
    if (path == kPathAuto)
    {
        if (rows > kTileMaxRows)
            path = kPathTall;
        else if (wavecol_applicable(g, r_in, r_out, q, rows, nbits))
            path = kPathWaveCol;
        else
            path = kPathTile;
    }
    if (path == kPathWaveCol)
    {
        if (!wavecol_applicable(g, r_in, r_out, q, rows, nbits))
            return hipErrorInvalidValue;
        constexpr uint32_t per_block = kWaveColThreads / 64;
        const uint32_t blocks = (uint32_t) ((cols + per_block - 1) / per_block);
        const uint64_t qcol = qcol_bytes(nbits, rows);
        if (rows == 2048)
        {
            if (zt)
                hipExtLaunchKernelGGL((quantize_wavecol_kernel<true, 1>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out, qc, (uint32_t) cols, qcol);
            else
                hipExtLaunchKernelGGL((quantize_wavecol_kernel<false, 1>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out, qc, (uint32_t) cols, qcol);
        }
        else
        {
            if (zt)
                hipExtLaunchKernelGGL((quantize_wavecol_kernel<true, 2>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out, qc, (uint32_t) cols, qcol);
            else
                hipExtLaunchKernelGGL((quantize_wavecol_kernel<false, 2>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out, qc, (uint32_t) cols, qcol);
        }
        return hipGetLastError();
    }
    if (path == kPathTile)
    {
        if (rows > kTileMaxRows)
            return hipErrorInvalidValue;
        const TileGeom t = make_tile_geom(rows, cols, nbits, tune.tile_gs, tune.tile_stage, tune.tile_threads);
        return dispatch_nbits<TileLauncher>(nbits, zt, s, ev, g, r_in, r_out, qc, t);
    }
    return dispatch_nbits<TallLauncher>(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) rows, (uint32_t) cols,
                                        (uint32_t) qwords_per_col(rows, nbits), (uint64_t) qcol_bytes(nbits, rows));
}

inline hipError_t launch_stripe_reduce(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, void* q_out,
                                       float* agg_out, size_t rows, size_t cols, size_t nbits, bool zt,
                                       const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    if (rows > kTileMaxRows)
        return hipErrorInvalidValue;
    bool aligned8 = (reinterpret_cast<uintptr_t>(q_out) & 7u) == 0;
    for (uint32_t w = 0; w < src.workers; ++w)
        aligned8 = aligned8 && (reinterpret_cast<uintptr_t>(src.q[w]) & 7u) == 0;
    if (tune.quantize_path != kPathTile && nbits == 1 && (rows == 2048 || rows == 4096) && aligned8)
    {
        constexpr uint32_t per_block = kWaveColThreads / 64;
        const uint32_t blocks = (uint32_t) ((cols + per_block - 1) / per_block);
        const uint64_t qcol = qcol_bytes(nbits, rows);
        char* qo = static_cast<char*>(q_out);
        if (rows == 2048)
        {
            if (zt)
                hipExtLaunchKernelGGL((stripe_reduce_wavecol_kernel<true, 1>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, src, stripe_res, qo, agg_out, (uint32_t) cols, qcol);
            else
                hipExtLaunchKernelGGL((stripe_reduce_wavecol_kernel<false, 1>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, src, stripe_res, qo, agg_out, (uint32_t) cols, qcol);
        }
        else
        {
            if (zt)
                hipExtLaunchKernelGGL((stripe_reduce_wavecol_kernel<true, 2>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, src, stripe_res, qo, agg_out, (uint32_t) cols, qcol);
            else
                hipExtLaunchKernelGGL((stripe_reduce_wavecol_kernel<false, 2>), dim3(blocks), dim3(kWaveColThreads), 0, s, ev.start, ev.stop, 0, src, stripe_res, qo, agg_out, (uint32_t) cols, qcol);
        }
        return hipGetLastError();
    }
    // A stripe is small (one GPU's share of the columns), so the kernel is latency-bound: take the smallest
    // tile that still gives every thread of a workgroup a work item, to spread the stripe over all CUs.
    uint32_t gs = tune.tile_gs;
    if (gs == 0)
    {
        const size_t chunks = nbits == 1 ? 4 : (nbits == 2 ? 2 : 1);
        const size_t items_per_col = qwords_per_col(rows, nbits) * chunks;
        gs = kTileThreads;
        while (gs > 8 && items_per_col * (kTileThreads / gs) < kTileThreads)
            gs >>= 1;
    }
    const TileGeom t = make_tile_geom(rows, cols, nbits, gs, tune.tile_stage, tune.tile_threads);
    return dispatch_nbits<StripeLauncher>(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, t);
}

template <int NBITS, int WV>
inline hipError_t launch_unquantize_t(hipStream_t s, LaunchEvents ev, const char* q, float* out, size_t rows, size_t cols, uint32_t slots,
                                      int add)
{
    constexpr uint32_t VPW = 32 / NBITS;
    UnqGeom t;
    t.rows = (uint32_t) rows;
    t.cols = (uint32_t) cols;
    t.nq = (uint32_t) qwords_per_col(rows, NBITS);
    t.groups = (t.nq + WV - 1) / WV;
    if (slots == 0)
        slots = VPW < 2 ? VPW : 2;
    if (slots > VPW)
        slots = VPW;
    t.slots = slots;
    t.chunks = (VPW + slots - 1) / slots;
    const uint64_t per_col = (uint64_t) t.groups * t.chunks;
    const uint64_t items = per_col * cols;
    if (items > 0xFFFFFFFFull)
        return hipErrorInvalidValue;
    t.per_col = (uint32_t) per_col;
    t.items = (uint32_t) items;
    t.qcol = qcol_bytes(NBITS, rows);
    const uint32_t blocks = (uint32_t) ((items + 255) / 256);
    hipExtLaunchKernelGGL((unquantize_kernel<NBITS, WV>), dim3(blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, t, add);
    return hipGetLastError();
}

template <int NBITS>
inline hipError_t launch_unquantize_segment_t(hipStream_t s, LaunchEvents ev, const char* q, float* out, size_t rows, size_t cols, int add)
{
    UnqSegGeom t;
    t.rows = (uint32_t) rows;
    t.nq = (uint32_t) qwords_per_col(rows, NBITS);
    t.segs = (uint32_t) ((rows + t.nq - 1) / t.nq);
    t.gps = (t.nq + 3 + 3) / 4;
    const uint64_t items = (uint64_t) cols * t.segs * t.gps;
    if (items > 0xFFFFFFFFull)
        return hipErrorInvalidValue;
    t.items = (uint32_t) items;
    t.inv_gps = 1.0 / (double) t.gps;
    t.inv_segs = 1.0 / (double) t.segs;
    t.qcol = qcol_bytes(NBITS, rows);
    const uint32_t blocks = (uint32_t) ((items + 255) / 256);
    hipExtLaunchKernelGGL((unquantize_segment_kernel<NBITS>), dim3(blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, t, add);
    return hipGetLastError();
}

inline hipError_t launch_unquantize(hipStream_t s, LaunchEvents ev, const void* q, float* out, size_t rows, size_t cols, size_t nbits,
                                    bool add, const LaunchTuning& tune)
{
    const char* qc = static_cast<const char*>(q);
    const size_t nq = qwords_per_col(rows, nbits);
    const bool vec = !tune.unq_force_scalar && (nq % 4 == 0) && (rows % 4 == 0) &&
                     (reinterpret_cast<uintptr_t>(out) & 15u) == 0 && (reinterpret_cast<uintptr_t>(q) & 7u) == 0;
    const int a = add ? 1 : 0;
    const uint32_t sl = tune.unq_slots;
    // long columns that the QWord-major decoder could only serve with 4-byte stores go to the segment decoder
    const bool seg = !vec && !tune.unq_force_scalar && (reinterpret_cast<uintptr_t>(out) & 15u) == 0 && nq >= 32 &&
                     (uint64_t) cols * (32 / nbits) * ((nq + 6) / 4) <= 0xFFFFFFFFull;
    if (seg)
    {
        switch (nbits)
        {
        case 1: return launch_unquantize_segment_t<1>(s, ev, qc, out, rows, cols, a);
        case 2: return launch_unquantize_segment_t<2>(s, ev, qc, out, rows, cols, a);
        case 4: return launch_unquantize_segment_t<4>(s, ev, qc, out, rows, cols, a);
        case 8: return launch_unquantize_segment_t<8>(s, ev, qc, out, rows, cols, a);
        case 16: return launch_unquantize_segment_t<16>(s, ev, qc, out, rows, cols, a);
        case 32: return launch_unquantize_segment_t<32>(s, ev, qc, out, rows, cols, a);
        default: return hipErrorInvalidValue;
        }
    }
    switch (nbits)
    {
    case 1: return vec ? launch_unquantize_t<1, 4>(s, ev, qc, out, rows, cols, sl, a) : launch_unquantize_t<1, 1>(s, ev, qc, out, rows, cols, sl, a);
    case 2: return vec ? launch_unquantize_t<2, 4>(s, ev, qc, out, rows, cols, sl, a) : launch_unquantize_t<2, 1>(s, ev, qc, out, rows, cols, sl, a);
    case 4: return vec ? launch_unquantize_t<4, 4>(s, ev, qc, out, rows, cols, sl, a) : launch_unquantize_t<4, 1>(s, ev, qc, out, rows, cols, sl, a);
    case 8: return vec ? launch_unquantize_t<8, 4>(s, ev, qc, out, rows, cols, sl, a) : launch_unquantize_t<8, 1>(s, ev, qc, out, rows, cols, sl, a);
    case 16: return vec ? launch_unquantize_t<16, 4>(s, ev, qc, out, rows, cols, sl, a) : launch_unquantize_t<16, 1>(s, ev, qc, out, rows, cols, sl, a);
    case 32: return vec ? launch_unquantize_t<32, 4>(s, ev, qc, out, rows, cols, sl, a) : launch_unquantize_t<32, 1>(s, ev, qc, out, rows, cols, sl, a);
    default: return hipErrorInvalidValue;
    }
}

} // namespace cntkq
