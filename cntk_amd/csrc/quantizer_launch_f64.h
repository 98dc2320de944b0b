// Host-side kernel selection and launch for the double-precision instantiation (gfx950). No allocation happens here.
#pragma once

#include "quantizer_kernels_f64.h"
#include "quantizer_launch.h"

namespace cntkq {
namespace f64 {

constexpr uint32_t kTileMaxRows = 7168; // 56 KB of LDS for a one-column tile of doubles
constexpr size_t kMaxLdsBytes = 64 * 1024;
// the register kernels may have all of a compute unit's LDS; quantize and fused stripe reduction take the same heights (see
// reg_lds_fits of the float kernels)
constexpr size_t kRegMaxLdsBytes = 160 * 1024;

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
        hipExtLaunchKernelGGL((quantize_tall_kernel<NBITS, ZT, double>), dim3(cols), dim3(kTallThreads), 0, s, ev.start, ev.stop, 0, g, r_in, r_out,
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

// The register kernel: for columns the tile kernel cannot hold, below 64 bits,
// at most 25 pieces of two doubles for each of 1024 threads, QWords within 64 KB of LDS.
constexpr uint32_t kRegThreads = 1024;
constexpr size_t kRegMaxRows = 2 * 1024 * 25;
constexpr size_t kRegMinRows = 6145; // up to 6144 rows the element-wise register kernel and the tile stripe reduction are faster

inline bool reg_applicable(const double* g, const double* r_in, const double* r_out, size_t rows, size_t nbits)
{
    // any height from 4 rows on, any 8-byte alignment: the aligned pairs are the residual input's, gradient and residual
    // output are read and written in 16-byte accesses wherever they lie
    (void) g;
    (void) r_in;
    (void) r_out;
    if (rows < 4 || rows > kRegMaxRows - 16 || nbits >= 64)
        return false;
    return ((size_t) kRegRedSlots + 2 * qwords_per_col(rows, nbits) + 2) * 8 <= kRegMaxLdsBytes;
}

// Slots are dealt by 128-byte lines where some column of the residual starts inside one and the registers allow it. Only
// the residual's address enters (the slot dealing is part of the summation order, and the stripe reduction, which must
// reproduce it, knows only the stripe residual).
inline bool reg_line_shift(const double* r_in, size_t rows)
{
    return !columns_start_on_lines(r_in, rows, 16) && rows / 2 + 7 <= (size_t) kRegThreads * kRegMaxShiftPer;
}

inline RegGeom make_reg_geom(size_t rows, size_t nbits, bool line_shift)
{
    RegGeom c;
    c.rows = (uint32_t) rows;
    c.nq = (uint32_t) qwords_per_col(rows, nbits);
    c.pieces = (uint32_t) (rows / 2);
    c.step_k = (2 * kRegThreads) / c.nq;
    c.step_w = (2 * kRegThreads) % c.nq;
    c.line_shift = line_shift ? 1u : 0u;
    c.qcol = qcol_bytes(nbits, rows);
    return c;
}

template <int NBITS, bool ZT, int PER>
inline hipError_t launch_reg_one(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, uint32_t cols,
                                 const RegGeom& c)
{
    hipExtLaunchKernelGGL((quantize_reg_kernel<NBITS, ZT, (int) kRegThreads, PER>), dim3(cols), dim3(kRegThreads), reg_lds_bytes64(c), s,
                          ev.start, ev.stop, 0, g, r_in, r_out, q, c);
    return hipGetLastError();
}

template <int NBITS, bool ZT>
struct RegLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, uint32_t cols, RegGeom c)
    {
        if constexpr (NBITS >= 64)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t per = (c.pieces + (c.line_shift ? 7u : 0u) + kRegThreads - 1) / kRegThreads;
#define CNTKQ_REG64(P) if (per <= P) return launch_reg_one<NBITS, ZT, P>(s, ev, g, r_in, r_out, q, cols, c)
            CNTKQ_REG64(4);
            CNTKQ_REG64(6);
            CNTKQ_REG64(8);
            CNTKQ_REG64(10);
            CNTKQ_REG64(13);
            CNTKQ_REG64(16);
            CNTKQ_REG64(20);
            CNTKQ_REG64(25);
#undef CNTKQ_REG64
            return hipErrorInvalidValue;
        }
    }
};

// The element-wise register kernel (256 threads, up to 24 rows each): the heights at which the tile kernel holds one column
// per tile, any alignment, below 64 bits. Same bytes as the tile kernel in its default geometry.
constexpr size_t kColRegMaxRows = 256 * 24;
constexpr size_t kColRegMinRows = 1025; // the whole range: 1028 rows 87 us against 108 us on 18.5 M elements, 4096: 76 against 86

inline bool colreg_applicable(size_t rows, size_t nbits)
{
    return rows > 1024 && rows <= kColRegMaxRows && nbits < 64;
}

template <int NBITS, bool ZT>
struct ColRegLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q, uint32_t rows,
                          uint32_t cols, uint32_t nq, uint64_t qcol)
    {
        if constexpr (NBITS >= 64)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t ept = (rows + kThreads - 1) / kThreads;
#define CNTKQ_COLREG64(E)                                                                                                              \
    if (ept <= E)                                                                                                                      \
    {                                                                                                                                  \
        hipExtLaunchKernelGGL((quantize_colreg_kernel<NBITS, ZT, E>), dim3(cols), dim3(kThreads), colreg_lds_bytes(nq), s, ev.start,   \
                              ev.stop, 0, g, r_in, r_out, q, rows, nq, qcol);                                                          \
        return hipGetLastError();                                                                                                      \
    }
            CNTKQ_COLREG64(8)
            CNTKQ_COLREG64(12)
            CNTKQ_COLREG64(16)
            CNTKQ_COLREG64(20)
            CNTKQ_COLREG64(24)
#undef CNTKQ_COLREG64
            return hipErrorInvalidValue;
        }
    }
};

// The kernel family a matrix gets when nothing is forced.
inline int quantize_auto_path(const double* g, const double* r_in, const double* r_out, size_t rows, size_t nbits)
{
    // from 1025 to 6144 rows the column stays in registers element by element (256 threads); above, the 1024-thread
    // register kernel is faster (7168 rows on 19 M elements: 78 us against 81 us, and the stripe reduction that has to
    // follow the quantize kernel's order of additions 161 us against 202 us; at 6144 rows 77 against 75 and 164 against 126)
    if (rows >= kRegMinRows && reg_applicable(g, r_in, r_out, rows, nbits))
        return kPathReg;
    if (rows >= kColRegMinRows && colreg_applicable(rows, nbits))
        return kPathRegScalar;
    return rows <= kTileMaxRows ? kPathTile : kPathTall;
}

// rows, cols > 0; pointers 8-byte aligned (checked by the caller). tune.quantize_path may force a kernel family.
inline hipError_t launch_quantize(hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, void* q, size_t rows,
                                  size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    char* qc = static_cast<char*>(q);
    int path = tune.quantize_path;
    if (path == kPathAuto)
    {
        path = quantize_auto_path(g, r_in, r_out, rows, nbits);
        // columns that no workgroup's registers hold: strips of the column on several workgroups, which read their inputs
        // once, where the device holds all strips of a column at once and the scratch buffer is there or may be made
        if (path == kPathTall && nbits < 64 && !tune.strip_never_waits && strip_ready<double>(s, rows, cols, nbits, zt, tune))
            path = kPathStrip;
        // ... and of more strips than that: the strips in passes (two or three reads, on the whole device)
        if (path == kPathTall && nbits < 64 && strip_passes_ready<double>(s, rows, cols, nbits, tune))
            path = kPathStripPasses;
    }
    if (path == kPathStrip)
        return launch_strip_quantize<double>(s, ev, g, r_in, r_out, qc, rows, cols, nbits, zt, tune);
    if (path == kPathStripPasses)
        return launch_strip_quantize_passes<double>(s, ev, g, r_in, r_out, qc, rows, cols, nbits, zt, tune);
    if (path == kPathReg)
    {
        if (!reg_applicable(g, r_in, r_out, rows, nbits))
            return hipErrorInvalidValue;
        return dispatch_nbits64<RegLauncher>(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols,
                                             make_reg_geom(rows, nbits, reg_line_shift(r_in, rows)));
    }
    if (path == kPathRegScalar)
    {
        if (!colreg_applicable(rows, nbits))
            return hipErrorInvalidValue;
        return dispatch_nbits64<ColRegLauncher>(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) rows, (uint32_t) cols,
                                                (uint32_t) qwords_per_col(rows, nbits), (uint64_t) qcol_bytes(nbits, rows));
    }
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

template <int NBITS, bool ZT, int PER>
inline hipError_t launch_stripe_reg_one(hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, char* q_out,
                                        double* agg_out, uint32_t cols, const RegGeom& c)
{
    hipExtLaunchKernelGGL((stripe_reduce_reg_kernel<NBITS, ZT, PER>), dim3(cols), dim3(kRegThreads), stripe_reg_lds_bytes64(c), s, ev.start,
                          ev.stop, 0, src, stripe_res, q_out, agg_out, c);
    return hipGetLastError();
}

template <int NBITS, bool ZT>
struct StripeRegLauncher
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, char* q_out, double* agg_out,
                          uint32_t cols, RegGeom c)
    {
        if constexpr (NBITS >= 64)
            return hipErrorInvalidValue;
        else
        {
            const uint32_t per = (c.pieces + (c.line_shift ? 7u : 0u) + kRegThreads - 1) / kRegThreads;
#define CNTKQ_SREG64(P) if (per <= P) return launch_stripe_reg_one<NBITS, ZT, P>(s, ev, src, stripe_res, q_out, agg_out, cols, c)
            CNTKQ_SREG64(4);
            CNTKQ_SREG64(6);
            CNTKQ_SREG64(8);
            CNTKQ_SREG64(10);
            CNTKQ_SREG64(13);
            CNTKQ_SREG64(16);
            CNTKQ_SREG64(20);
            CNTKQ_SREG64(25);
#undef CNTKQ_SREG64
            return hipErrorInvalidValue;
        }
    }
};

// Whether the stripe reduction of such a stripe runs in the register kernel's shape: the heights where a quantize call on
// (aggregate, stripe residual) takes the register kernel, as far as two packed columns fit LDS.
inline bool stripe_uses_reg(size_t rows, size_t nbits)
{
    if (rows < kRegMinRows || rows > kRegMaxRows - 16 || nbits >= 64)
        return false;
    return ((size_t) kRegRedSlots + 2 * qwords_per_col(rows, nbits) + 2) * 8 <= kRegMaxLdsBytes;
}

// Tallest column the fused stripe reduction takes at this bit width.
inline size_t stripe_reduce_max_rows(size_t nbits)
{
    if (nbits >= 64)
        return kTileMaxRows;
    const size_t max_nq = (kRegMaxLdsBytes / 8 - kRegRedSlots - 2) / 2;
    const size_t by_lds = max_nq * (64 / nbits);
    const size_t by_regs = kRegMaxRows - 16;
    const size_t tall = by_lds < by_regs ? by_lds : by_regs;
    return tall > kTileMaxRows ? tall : kTileMaxRows;
}

// The kernel family, and within it the geometry, that a quantize call on (aggregate, stripe residual) would take, so that the
// fused call gives the bytes of the unquantize ... quantize call sequence (the sequence's aggregate must sit at the stripe
// residual's offset within 16 bytes for that, as whole allocations do).
// Heights at which the automatic choice of a quantize call is the strip kernels (or, without them, the kernel that re-reads
// its columns): what no workgroup's registers hold.
inline bool strip_only_height(size_t rows, size_t nbits)
{
    return nbits < 64 && rows > kTileMaxRows && quantize_auto_path(nullptr, nullptr, nullptr, rows, nbits) == kPathTall;
}

// Whether the fused stripe reduction takes a stripe taller than stripe_reduce_max_rows: on strips, where a quantize call
// on (aggregate, stripe residual) would run on strips as well (same bytes), with the scratch buffer there or obtainable.
inline bool stripe_takes_strips(hipStream_t s, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && nbits == 1;
    return !tune.strip_never_waits && strip_only_height(rows, nbits) && strip_ready<double>(s, rows, cols, nbits, zt, tune, false) &&
           strip_ready<double>(s, rows, cols, nbits, zt, tune, true);
}

inline hipError_t launch_stripe_reduce(hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, void* q_out,
                                       double* agg_out, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    if (rows > stripe_reduce_max_rows(nbits))
    {
        if (!f64::stripe_takes_strips(s, rows, cols, nbits, zt, tune))
            return hipErrorInvalidValue;
        return launch_strip_stripe<double>(s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, rows, cols, nbits, zt, tune);
    }
    if (stripe_uses_reg(rows, nbits))
        return dispatch_nbits64<StripeRegLauncher>(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, (uint32_t) cols,
                                                   make_reg_geom(rows, nbits, reg_line_shift(stripe_res, rows)));
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
        hipExtLaunchKernelGGL((unquantize_kernel<NBITS, 2, double>), dim3(blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, t, add);
    else
        hipExtLaunchKernelGGL((unquantize_kernel<NBITS, 1, double>), dim3(blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, t, add);
    return hipGetLastError();
}

constexpr size_t kUnqRowsMinRows64 = 512;  // from this height on a column keeps the 256 threads of the row-major decoder busy
constexpr size_t kUnqTileMaxRows64 = 16384;
constexpr size_t kUnqTileElems64 = 2048;   // values per workgroup the tile decoder aims for

template <int NBITS>
inline hipError_t launch_unquantize_rows(hipStream_t s, LaunchEvents ev, const char* q, double* out, const UnqRowGeom& t, int add)
{
    hipExtLaunchKernelGGL((unquantize_rows_kernel<NBITS, double>), dim3(t.blocks), dim3(256), (size_t) t.nq * 8, s, ev.start, ev.stop, 0, q, out, t, add);
    return hipGetLastError();
}

template <int NBITS>
inline hipError_t launch_unquantize_tile(hipStream_t s, LaunchEvents ev, const char* q, double* out, const UnqTileGeom& t, int add)
{
    hipExtLaunchKernelGGL((unquantize_tile_kernel<NBITS, double>), dim3(t.blocks), dim3(256), (size_t) t.cpt * (t.rec_words + 2) * 8, s, ev.start,
                          ev.stop, 0, q, out, t, add);
    return hipGetLastError();
}

#define CNTKQ_NBITS64_SWITCH(FN, ...)                                                                                  \
    switch (nbits)                                                                                                     \
    {                                                                                                                  \
    case 1: return FN<1>(__VA_ARGS__);                                                                                 \
    case 2: return FN<2>(__VA_ARGS__);                                                                                 \
    case 4: return FN<4>(__VA_ARGS__);                                                                                 \
    case 8: return FN<8>(__VA_ARGS__);                                                                                 \
    case 16: return FN<16>(__VA_ARGS__);                                                                               \
    case 32: return FN<32>(__VA_ARGS__);                                                                               \
    case 64: return FN<64>(__VA_ARGS__);                                                                               \
    default: return hipErrorInvalidValue;                                                                              \
    }

// Which decoder unquantizes a matrix, and its geometry; shared by the plain call and the batched one.
struct UnquantizePlan64
{
    uint32_t kind = kUnqScalar; // kUnqVec4 (16-byte stores of two doubles), kUnqScalar, kUnqRows, kUnqTile
    UnqGeom qw;
    UnqRowGeom rowg;
    UnqTileGeom tile;
    UnqFlatGeom flat;
    uint32_t blocks = 0; // 256-thread blocks
    size_t lds = 0;      // dynamic LDS (kUnqRows, kUnqTile)
    bool ok = false;
};

inline UnquantizePlan64 plan_unquantize(const double* out, size_t rows, size_t cols, size_t nbits, const LaunchTuning& tune)
{
    UnquantizePlan64 p;
    std::memset(&p.qw, 0, sizeof p.qw);
    std::memset(&p.rowg, 0, sizeof p.rowg);
    std::memset(&p.tile, 0, sizeof p.tile);
    std::memset(&p.flat, 0, sizeof p.flat);
    const size_t vpw = 64 / nbits;
    const size_t nq = qwords_per_col(rows, nbits);
    const bool out16 = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    const int mode = tune.unq_mode; // 0 automatic, 1 QWord-major 8-byte stores, 2 / 4 tile / row-major decoder wherever it can run, 3 QWord-major
    // The QWord-major decoder is at its best when every bit position of a column is a run of whole 128-byte lines. Other
    // columns: row-major decoder from 512 rows on, tile decoder for shorter ones (the choices of the fp32 side).
    const bool vec_ideal = nq % 16 == 0 && rows % 16 == 0 && rows * nbits == nq * 64 && out16;
    const bool rows_can = tune.unq_slots == 0 && rows >= 16 && nq >= 16 && nq * 8 <= 48 * 1024; // any height, any alignment
    const bool tile_can = tune.unq_slots == 0 && out16 && rows <= kUnqTileMaxRows64;
    const bool direct_can = tune.unq_slots == 0 && rows >= 16 && nq >= 16; // any height, any alignment
    // (the automatic choice from 16384 rows on, for 1- and 2-bit columns of whole chunks of 1024 rows in a launch of their
    // own -- as members of a gradient-set launch they measured slower than with the QWord-major decoder --, and from 8192 rows
    // at 2 bits and more where the QWord-major stores would not be whole lines and the last chunk is not mostly empty)
    const size_t direct_chunk = 256 * kUnqDirectPieces * 2;
    const bool direct_full = (((rows + direct_chunk - 1) / direct_chunk) * direct_chunk - rows) * 8 <= rows;
    const bool direct_auto = direct_can && (rows >= 16384 || (nbits <= 2 && rows % direct_chunk == 0 && !tune.unq_member) ||
                                            (!vec_ideal && nbits >= 2 && rows >= 8192 && direct_full));
    // (the LDS-free decoder for short columns: the rule of the float side, up to 2048 rows -- 512 x 50000 38.0 -> 32.4 us,
    // 576 x 16384 at 2 bits 15.6 -> 12.8 us, 1536 x 6144 13.7 -> 12.0 us, even at 2048 x 4652 at 4 bits; 4608 x 2048 at 4 bits
    // is 13 % slower with it than with the packed column in LDS)
    // (QWord counts that are odd stay with the tile and row-major decoders here: 1000 x 10000 at 8 bits and 200 x 100000 at 2
    // bits were 11 % slower with it, 576 x 16384 at 1 bit 10 % faster)
    const bool flat_auto = mode == 0 && !direct_auto && rows <= 2048 && nq % 2 == 0 &&
                           (!tune.unq_member || (uint64_t) rows * cols >= ((uint64_t) 1 << 22));
    if ((mode == 6 || flat_auto) && tune.unq_slots == 0 && out16 && make_unq_flat_geom(p.flat, rows, cols, nq, qcol_bytes(nbits, rows), 2))
    {
        p.kind = kUnqFlat;
        p.blocks = p.flat.blocks;
        p.ok = true;
        return p;
    }
    bool use_rows = false, use_tile = false;
    if ((mode == 5 && direct_can) || (mode == 0 && direct_auto))
    {
        if (make_unq_direct_geom(p.rowg, rows, cols, nq, qcol_bytes(nbits, rows), 2))
        {
            p.kind = kUnqDirect;
            p.blocks = p.rowg.blocks;
            p.ok = true;
            return p;
        }
    }
    else if (mode == 2 && tile_can)
        use_tile = true;
    else if (mode == 4 && rows_can)
        use_rows = true;
    else if (mode == 0 && tune.unq_slots == 0 && !vec_ideal)
    {
        if (rows_can && rows >= kUnqRowsMinRows64)
            use_rows = true;
        else if (tile_can)
            use_tile = true;
        else if (rows_can)
            use_rows = true;
    }
    if (use_rows)
    {
        UnqRowGeom& t = p.rowg;
        t.rows = (uint32_t) rows;
        t.nq = (uint32_t) nq;
        const size_t mult = nq > 512 ? 2 : 4;
        size_t chunk = ((mult * nq + 511) / 512) * 512;
        if (chunk < 1024)
            chunk = 1024;
        t.chunk = (uint32_t) chunk;
        t.chunks = rows >= chunk ? (uint32_t) ((rows + chunk / 2) / chunk) : 1u;
        t.pad = 0;
        t.qcol = qcol_bytes(nbits, rows);
        const uint64_t blocks = (uint64_t) cols * t.chunks;
        if (blocks <= 0x7FFFFFFFull)
        {
            t.blocks = (uint32_t) blocks;
            p.kind = kUnqRows;
            p.blocks = t.blocks;
            p.lds = (size_t) t.nq * 8;
            p.ok = true;
            return p;
        }
    }
    if (use_tile)
    {
        UnqTileGeom& t = p.tile;
        t.rows = (uint32_t) rows;
        t.cols = (uint32_t) cols;
        t.nq = (uint32_t) nq;
        size_t cpt = (kUnqTileElems64 / rows) & ~(size_t) 1;
        if (cpt < 2)
            cpt = 2;
        t.cpt = (uint32_t) cpt;
        t.rec_words = (uint32_t) nq + 2;
        t.rows_magic = rows > 1 ? (uint32_t) ((((uint64_t) 1 << 32) + rows - 1) / rows) : 0u;
        t.nq_magic = nq > 1 ? (uint32_t) ((((uint64_t) 1 << 32) + nq - 1) / nq) : 0u;
        const uint64_t blocks = (cols + cpt - 1) / cpt;
        if (blocks <= 0x7FFFFFFFull && (size_t) t.cpt * (t.rec_words + 2) * 8 <= kMaxLdsBytes)
        {
            t.blocks = (uint32_t) blocks;
            p.kind = kUnqTile;
            p.blocks = t.blocks;
            p.lds = (size_t) t.cpt * (t.rec_words + 2) * 8;
            p.ok = true;
            return p;
        }
    }
    const bool vec = mode != 1 && (nq % 2 == 0) && (rows % 2 == 0) && out16;
    const uint32_t wv = vec ? 2 : 1;
    UnqGeom& t = p.qw;
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
        return p; // not ok
    t.per_col = (uint32_t) per_col;
    t.items = (uint32_t) items;
    // several workgroups per column that read the same QWords: regroup them by XCD (whole workgroups per column only)
    t.swz_members = 0;
    t.swz_gw = 1;
    if (per_col % 256 == 0 && per_col > 256)
    {
        if (t.groups <= 256)
            t.swz_members = (uint32_t) (per_col / 256);
        else if (t.groups % 256 == 0)
        {
            t.swz_members = t.chunks;
            t.swz_gw = t.groups / 256;
        }
    }
    t.qcol = qcol_bytes(nbits, rows);
    p.kind = vec ? kUnqVec4 : kUnqScalar;
    p.blocks = (uint32_t) (((uint64_t) t.items + 255) / 256);
    p.ok = true;
    return p;
}

template <int NBITS>
inline hipError_t launch_unquantize_plan(hipStream_t s, LaunchEvents ev, const char* q, double* out, const UnquantizePlan64& p, int add)
{
    if (p.kind == kUnqRows)
        return launch_unquantize_rows<NBITS>(s, ev, q, out, p.rowg, add);
    if (p.kind == kUnqDirect)
    {
        hipExtLaunchKernelGGL((unquantize_direct_kernel<NBITS, double>), dim3(p.rowg.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.rowg, add);
        return hipGetLastError();
    }
    if (p.kind == kUnqFlat)
    {
        hipExtLaunchKernelGGL((unquantize_flat_kernel<NBITS, double>), dim3(p.flat.blocks), dim3(256), 0, s, ev.start, ev.stop, 0, q, out, p.flat, add);
        return hipGetLastError();
    }
    if (p.kind == kUnqTile)
        return launch_unquantize_tile<NBITS>(s, ev, q, out, p.tile, add);
    return launch_unquantize_n<NBITS>(s, ev, q, out, p.qw, p.kind == kUnqVec4, add);
}

inline hipError_t launch_unquantize(hipStream_t s, LaunchEvents ev, const void* q, double* out, size_t rows, size_t cols, size_t nbits,
                                    bool add, const LaunchTuning& tune)
{
    const UnquantizePlan64 p = plan_unquantize(out, rows, cols, nbits, tune);
    if (!p.ok)
        return hipErrorInvalidValue;
    const char* qc = static_cast<const char*>(q);
    const int a = add ? 1 : 0;
    CNTKQ_NBITS64_SWITCH(launch_unquantize_plan, s, ev, qc, out, p, a)
}

template <int NBITS, bool ZT>
struct QuantizeBatchLauncher64
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const QuantizeBatchEntry64* entries, const uint32_t* begins, uint32_t count,
                          uint32_t blocks, size_t lds)
    {
        hipExtLaunchKernelGGL((quantize_batch_kernel64<NBITS, ZT>), dim3(blocks), dim3(kThreads), lds, s, ev.start, ev.stop, 0, entries, begins,
                              count);
        return hipGetLastError();
    }
};

template <int NBITS, bool ZT>
struct StripeBatchLauncher64
{
    static hipError_t run(hipStream_t s, LaunchEvents ev, const StripeBatchEntry64* entries, const uint32_t* begins, uint32_t count,
                          uint32_t blocks, size_t lds)
    {
        hipExtLaunchKernelGGL((stripe_reduce_batch_kernel64<NBITS, ZT>), dim3(blocks), dim3(kThreads), lds, s, ev.start, ev.stop, 0, entries,
                              begins, count);
        return hipGetLastError();
    }
};

template <int NBITS>
inline hipError_t launch_unquantize_batch_n(hipStream_t s, LaunchEvents ev, const UnquantizeBatchEntry64* entries, const uint32_t* begins,
                                            uint32_t count, uint32_t blocks, int add, size_t lds)
{
    hipExtLaunchKernelGGL((unquantize_batch_kernel64<NBITS>), dim3(blocks), dim3(256), lds, s, ev.start, ev.stop, 0, entries, begins, count,
                          add);
    return hipGetLastError();
}

inline hipError_t launch_unquantize_batch(hipStream_t s, LaunchEvents ev, const UnquantizeBatchEntry64* entries, const uint32_t* begins,
                                          uint32_t count, uint32_t blocks, size_t nbits, bool add, size_t lds)
{
    const int a = add ? 1 : 0;
    CNTKQ_NBITS64_SWITCH(launch_unquantize_batch_n, s, ev, entries, begins, count, blocks, a, lds)
}

} // namespace f64
} // namespace cntkq
