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

#include <type_traits>

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
// still keeps every thread busy; the partial words meet in LDS (atomic OR). WORD_BITS: 32 for float columns, 64 for double.
template <int NBITS, int WORD_BITS>
struct PackShapeOf
{
    typedef typename std::conditional<WORD_BITS == 64, uint64_t, uint32_t>::type Q;
    static constexpr uint32_t VPW = WORD_BITS / NBITS;       // values per QWord
    static constexpr uint32_t SLOTS = VPW < 8 ? VPW : 8;     // bit positions per work item
    static constexpr uint32_t CHUNKS = VPW / SLOTS;          // work items per QWord (fp32: 4, 2, 1, 1, 1, 1; fp64: 8, 4, 2, 1, 1, 1, 1)
    static constexpr uint32_t SHIFT = NBITS & (WORD_BITS - 1);
    static constexpr Q CODEMASK = (NBITS >= WORD_BITS) ? ~(Q) 0 : (((Q) 1 << SHIFT) - (Q) 1);
};
template <int NBITS>
using PackShape = PackShapeOf<NBITS, 32>;

// What a stripe reduction keeps in LDS per worker and column to decode that worker's codes: at 4 bits every level of the
// column (a decoded value is then one LDS read at the code's offset: three vector instructions per value and worker instead
// of six); at 2 bits the levels of two neighbouring codes side by side, for each of their 16 combinations (one 8-byte
// LDS read at the offset that the four bits make decodes two values); at 1 bit the two levels; else (ufactor, lower).
__host__ __device__ constexpr uint32_t stripe_dec_floats(size_t nbits)
{
    return nbits == 2 ? 32u : (nbits == 4 ? 16u : 2u);
}

// The workers whose tables sit at the front of LDS (room for them is always there), at offsets the compiler knows
constexpr uint32_t kStripeDecGroup = 8;

// ... in bytes for `workers` workers, with room to start the later workers' tables on an 8-byte boundary
__host__ __device__ constexpr size_t stripe_dec_bytes(size_t nbits, size_t workers)
{
    return (size_t) stripe_dec_floats(nbits) * (workers < kStripeDecGroup ? kStripeDecGroup : workers) * sizeof(float) + 8;
}

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

} // namespace cntkq
