// Host-side kernel selection and launch for the double-precision instantiation (gfx950). No allocation happens here.
#pragma once

#include "quantizer_kernels_f64.h"
#include "quantizer_launch.h"

namespace cntkq {
namespace f64 {

constexpr uint32_t kTileMaxRows = 7168; // 56 KB of LDS for a one-column tile of doubles
constexpr size_t kMaxLdsBytes = 64 * 1024;

inline bool valid_nbits(size_t nbits)
{
    return nbits >= 1 && nbits <= 64 && (nbits & (nbits - 1)) == 0;
}

// ColumnQuantizer<double>::QWordsPerCol (Source/Math/ColumnQuantizer.h:36-45)
inline size_t qwords_per_col(size_t rows, size_t nbits)
{
    const size_t per = 64 / nbits;
    return (rows + per - 1) / per;
}

// QuantizedColumn<double>::QuantizedColumnSize (Source/Math/QuantizedMatrix.h:42-47)
inline size_t qcol_bytes(size_t nbits, size_t rows)
{
    return 16 + ((rows * nbits + 63) / 64) * 8;
}

inline TileGeom make_tile_geom(size_t rows, size_t cols, size_t nbits, uint32_t gs_override)
{
    TileGeom t;
    t.rows = (uint32_t) rows;
    t.cols = (uint32_t) cols;
    t.nq = (uint32_t) qwords_per_col(rows, nbits);
    uint32_t gs = 8;
    if (gs_override != 0)
        gs = gs_override;
    else
        while (gs < kThreads && rows > (size_t) gs * 32)
            gs <<= 1;
    if (gs > kThreads)
        gs = kThreads;
    // a tile may not exceed 2048 doubles (16 KB) unless it is a single column
    while (gs < kThreads && (size_t) (kThreads / gs) * rows > 2048)
        gs <<= 1;
    t.gs = gs;
    t.gs_log2 = 0;
    while ((1u << t.gs_log2) < gs)
        t.gs_log2++;
    t.cols_per_tile = kThreads / gs;
    t.tile_words = (uint32_t) (((size_t) t.cols_per_tile * rows + 1) & ~(size_t) 1);
    t.words_words = (nbits <= 4) ? t.cols_per_tile * t.nq : 0; // a QWord has several work items below 8 bits
    t.qcol = qcol_bytes(nbits, rows);
    return t;
}

template <template <int, bool> class Launcher, typename... Args>
inline hipError_t dispatch_nbits64(size_t nbits, bool zt, Args... args)
{
    switch (nbits)
    {
    case 1: return zt ? Launcher<1, true>::run(args...) : Launcher<1, false>::run(args...);
    case 2: return Launcher<2, false>::run(args...);
    case 4: return Launcher<4, false>::run(args...);
    case 8: return Launcher<8, false>::run(args...);
    case 16: return Launcher<16, false>::run(args...);
    case 32: return Launcher<32, false>::run(args...);
    case 64: return Launcher<64, false>::run(args...);
    default: return hipErrorInvalidValue;
    }
}

template <int NBITS, bool ZT>
struct TileLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, TileGeom t)
    {
        const uint32_t tiles = (t.cols + t.cols_per_tile - 1) / t.cols_per_tile;
        hipExtLaunchKernelGGL((quantize_tile_kernel<NBITS, ZT>), dim3(tiles), dim3(kThreads), tile_lds_bytes(t, 0), s, ev.start, ev.stop, 0,
                              g, r_in, r_out, q, t);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct TallLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, uint32_t rows,
                          uint32_t cols, uint32_t nq, uint64_t qcol)
    {
        hipExtLaunchKernelGGL((quantize_tall_kernel<NBITS, ZT>), dim3(cols), dim3(kTallThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out,
                              q, rows, nq, qcol);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct StripeLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, char* q_out, double* agg_out,
                          TileGeom t)
    {
        const uint32_t tiles = (t.cols + t.cols_per_tile - 1) / t.cols_per_tile;
        hipExtLaunchKernelGGL((stripe_reduce_tile_kernel<NBITS, ZT>), dim3(tiles), dim3(kThreads), tile_lds_bytes(t, src.workers), s, ev.start,
                              ev.stop, 0, src, stripe_res, q_out, agg_out, t);
        return hipGetLastError();
    }
};

// rows, cols > 0; pointers 8-byte aligned (checked by the caller). tune.quantize_path may force the tile or tall kernel.
inline hipError_t launch_quantize(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, void* q, size_t rows,
                                  size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    char* qc = static_cast<char*>(q);
    int path = tune.quantize_path;
    if (path == kPathAuto)
        path = rows > kTileMaxRows ? kPathTall : kPathTile;
    if (path == kPathTile)
    {
        if (rows > kTileMaxRows)
            return hipErrorInvalidValue;
        const TileGeom t = make_tile_geom(rows, cols, nbits, tune.tile_gs);
        if (tile_lds_bytes(t, 0) > kMaxLdsBytes)
            return hipErrorInvalidValue;
        return dispatch_nbits64<TileLauncher>(nbits, zt, s, ev, g, r_in, r_out, qc, t);
    }
    if (path != kPathTall)
        return hipErrorInvalidValue;
    return dispatch_nbits64<TallLauncher>(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) rows, (uint32_t) cols,
                                        (uint32_t) qwords_per_col(rows, nbits), (uint64_t) qcol_bytes(nbits, rows));
}

// Same tile geometry as launch_quantize, so that the fused call gives the bytes of the unquantize ... quantize call sequence.
inline hipError_t launch_stripe_reduce(hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, void* q_out,
                                       double* agg_out, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    if (rows > kTileMaxRows)
        return hipErrorInvalidValue;
    const TileGeom t = make_tile_geom(rows, cols, nbits, tune.tile_gs);
    if (tile_lds_bytes(t, src.workers) > kMaxLdsBytes)
        return hipErrorInvalidValue;
    return dispatch_nbits64<StripeLauncher>(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, t);
}

template <int NBITS>
inline hipError_t launch_unquantize_n(hipStream_t s, LaunchEvents ev, const char* q, double* out, const UnqGeom& t, bool vec, int add)
{
    const uint32_t blocks = (uint32_t) (((uint64_t) t.items + 255) / 256);
    if (vec)
        hipExtLaunchKernelGGL((unquantize_kernel<NBITS, 2>), dim3(blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, t, add);
    else
        hipExtLaunchKernelGGL((unquantize_kernel<NBITS, 1>), dim3(blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, t, add);
    return hipGetLastError();
}

inline hipError_t launch_unquantize(hipStream_t s, LaunchEvents ev, const void* q, double* out, size_t rows, size_t cols, size_t nbits,
                                    bool add, const LaunchTuning& tune)
{
    const size_t vpw = 64 / nbits;
    const size_t nq = qwords_per_col(rows, nbits);
    const bool vec = !tune.unq_force_scalar && (nq % 2 == 0) && (rows % 2 == 0) && (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    const uint32_t wv = vec ? 2 : 1;
    UnqGeom t;
    t.rows = (uint32_t) rows;
    t.cols = (uint32_t) cols;
    t.nq = (uint32_t) nq;
    t.groups = (uint32_t) ((nq + wv - 1) / wv);
    uint32_t slots = tune.unq_slots;
    if (slots == 0)
        slots = vpw < 4 ? (uint32_t) vpw : 4;
    if (slots > vpw)
        slots = (uint32_t) vpw;
    t.slots = slots;
    t.chunks = (uint32_t) ((vpw + slots - 1) / slots);
    const uint64_t per_col = (uint64_t) t.groups * t.chunks;
    const uint64_t items = per_col * cols;
    if (items > 0xFFFFFFFFull)
        return hipErrorInvalidValue;
    t.per_col = (uint32_t) per_col;
    t.items = (uint32_t) items;
    t.qcol = qcol_bytes(nbits, rows);
    const char* qc = static_cast<const char*>(q);
    const int a = add ? 1 : 0;
    switch (nbits)
    {
    case 1: return launch_unquantize_n<1>(s, ev, qc, out, t, vec, a);
    case 2: return launch_unquantize_n<2>(s, ev, qc, out, t, vec, a);
    case 4: return launch_unquantize_n<4>(s, ev, qc, out, t, vec, a);
    case 8: return launch_unquantize_n<8>(s, ev, qc, out, t, vec, a);
    case 16: return launch_unquantize_n<16>(s, ev, qc, out, t, vec, a);
    case 32: return launch_unquantize_n<32>(s, ev, qc, out, t, vec, a);
    case 64: return launch_unquantize_n<64>(s, ev, qc, out, t, vec, a);
    default: return hipErrorInvalidValue;
    }
}

} // namespace f64
} // namespace cntkq
