// Host-side kernel selection and launch for the per-column quantizer (gfx950).
// Shared by the C-ABI library and by stand-alone timing programs; no allocation happens here.
#pragma once

#include "quantizer_kernels.h"

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <cstring>
#include <vector>

namespace cntkq {

// which quantize kernel to use
enum QuantizePath
{
    kPathAuto = 0,
    kPathTile = 1,    // LDS-staged column tile (rows <= kTileMaxRows)
    kPathTall = 2,    // one workgroup per column, global re-read (any rows)
    kPathCol = 3,     // one workgroup per column, column in LDS: rows a multiple of 4, matrices 16-byte aligned
    kPathReg = 4,     // one workgroup per column, column in registers: same conditions, 1 to 16 bits
    kPathRegScalar = 5, // the same with one float per load and store: any height up to 98304 rows, any alignment, 1 to 16 bits
    kPathStrip = 6,     // several workgroups per column, a strip of QWords with all its bit positions each: any height, any alignment, 1 to 16 bits
    kPathStripPasses = 7 // the same cut into two or three launches that read the matrix once each: columns of more strips than the device holds at once
};

constexpr uint32_t kTileMaxRows = 14336; // 56 KB of LDS for a one-column tile
constexpr size_t kTileMaxFloats = 5120;   // ... and 20 KB for a tile of several columns
constexpr uint32_t kStripPollPause = 64;           // strip kernel: 64-cycle pauses between two polls of a partial sum
constexpr uint32_t kStripFirstPauseMinStrips = 8; // ... strips per column from which a pause of 2 x strips precedes the first poll
constexpr uint32_t kStripeWideItems = 768;   // work items per column from which the stripe reduction may use more than 256 threads
constexpr uint32_t kStripeWideMaxCols = 256; // ... 1024 threads up to this many columns
constexpr uint32_t kColMinRows = 1024;   // shorter columns are better served several to a workgroup (tile kernels)

// The scratch buffer of the strip kernels (partial sums of the columns' workgroups and the launch count), owned by a handle: one
// launch stream at a time uses it. The error word lives in pinned host memory, where the host reads it without a copy.
struct StripScratchOwner
{
    char* dev = nullptr;
    size_t bytes = 0;        // header, finish counters, records
    size_t groups_bytes = 0; // the part of it set aside for finish counters: 1/256 of the whole
    uint32_t* error_host = nullptr;
    // Launches that share the buffer must not overlap. One stream orders them by itself; when the handle's stream changes,
    // the new stream first waits for the last launch on the old one (an event recorded after every launch).
    hipEvent_t order_event = nullptr;
    hipStream_t last_stream = nullptr;
    bool launched = false;
    // A launch recorded into a graph (stream capture) has the buffer's addresses in its kernel node and may be replayed at
    // any time from then on: such a buffer is never freed while the handle lives. When a later launch needs a larger one,
    // the old buffer is retired (freed with the handle) instead. Graphs must not outlive the handle.
    bool captured = false;
    std::vector<char*> retired;
    uint32_t abandoned_seen = 0; // what the buffer's count of abandoned columns read when the host last looked
};

struct LaunchTuning
{
    StripScratchOwner* strip = nullptr; // null: the strip kernels are not available to this launch
    uint32_t strip_spin_limit = 1u << 17; // polls of a partial sum (two microseconds or so each) before a lane gives up
    bool strip_may_allocate = true; // false: the strip kernels only where the scratch buffer as it stands holds the launch
    bool strip_never_waits = false; // true: tall columns take the strips in passes, whose workgroups never wait for one another
    int quantize_path = kPathAuto;
    uint32_t tile_gs = 0;   // 0 = pick from rows; else threads per column (power of two, 8..256)
    int tile_stage = -1;    // -1 = automatic; 0 / 1 = residual written straight to memory / staged through LDS
    uint32_t tile_threads = 0; // 0 = automatic; else workgroup size of the tile kernels (64, 128, 256)
    uint32_t unq_slots = 0; // 0 = default; else bit positions per thread in unquantize
    int unq_mode = 0; // 0 automatic, 1 QWord-major with 4-byte stores, 2 / 4 / 5 tile / row-major / LDS-free row-major decoder wherever it can run, 3 automatic without the tile decoder
    bool unq_member = false; // the matrix is decoded as a member of a gradient-set launch
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
    // a tile may not exceed 5120 floats (20 KB) unless it is a single column: eight workgroups, all that a compute unit's
    // wavefront slots take, then still find room in its LDS, and it is the number of resident workgroups that hides the
    // barrier-separated phases of each of them. (Measured over limits of 2048 / 4096 / 5120 / 8192 floats, quantize and
    // stripe reduction over 4 workers: 147 x 100000 37 / 34 / 34 / 34 and 58 / 49 / 45 / 45 us, 576 x 30000 46 / 37 / 37 / 38
    // and 70 / 57 / 49 / 49 us, 1000 x 18000 - / 39 / 39 / 47 and - / 49 / 48 / 72 us.)
    while (gs < threads && (size_t) (threads / gs) * rows > kTileMaxFloats)
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

// ---- the kernel families ----------------------------------------------------------------------------------------------
// Each family of kernels is instantiated in a source file of its own (quantizer_family_*.hip), so that the families
// compile side by side and a source file that only plans launches (the C ABI, the double-precision instantiation) carries
// no copy of them. nbits is 1, 2, 4, 8, 16 or 32; zt only matters at 1 bit. hipErrorInvalidValue: the family has no
// kernel for the arguments.
struct UnquantizePlan;
hipError_t family_tile_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q, TileGeom t);
hipError_t family_tile_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                              float* agg_out, TileGeom t);
hipError_t family_tall_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                                uint32_t rows, uint32_t cols, uint32_t nq, uint64_t qcol);
hipError_t family_col_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                               uint32_t cols, ColGeom c);
// per: 1, 2 or 4 pieces per thread (1024, 2048, 4096 rows at 1 bit)
hipError_t family_col_quantize_unrolled(bool zt, int per, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                                        uint32_t cols, uint64_t qcol);
hipError_t family_col_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                             float* agg_out, uint32_t cols, ColGeom c);
hipError_t family_col_stripe_unrolled(bool zt, int per, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                                      float* agg_out, uint32_t cols, uint64_t qcol);
// up to kStripeSetMax stripes of 1024 (per = 1) or 2048 (per = 2) rows at 1 bit with up to eight workers each, described in the arguments
hipError_t family_col_stripe_set(bool zt, int per, hipStream_t s, LaunchEvents ev, const StripeColSet& set);
// threads: 256 or 1024 per column
hipError_t family_reg_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                               uint32_t cols, RegGeom c, uint32_t threads);
hipError_t family_reg_edge_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                                    uint32_t cols, RegGeom c, uint32_t threads);
hipError_t family_regs_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                                uint32_t cols, RegGeom c);
hipError_t family_reg_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                             float* agg_out, uint32_t cols, RegGeom c, uint32_t threads);
hipError_t family_strip_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out, char* q,
                                 uint32_t cols, StripGeom c, StripScratch scratch);
hipError_t family_strip_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out, char* q,
                                 uint32_t cols, StripGeom c, StripScratch scratch);
// workgroups of the strip kernel that the runtime says a compute unit holds at once
hipError_t family_strip_quantize_passes(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const float* g, const float* r_in, float* r_out,
                                        char* q, uint32_t cols, StripGeom c, StripScratch scratch);
hipError_t family_strip_quantize_passes(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const double* g, const double* r_in, double* r_out,
                                        char* q, uint32_t cols, StripGeom c, StripScratch scratch);
hipError_t family_strip_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, char* q_out,
                               float* agg_out, uint32_t cols, StripGeom c, StripScratch scratch);
hipError_t family_strip_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeSources& src, double* stripe_res, char* q_out,
                               double* agg_out, uint32_t cols, StripGeom c, StripScratch scratch);
// (stripe: of the stripe-reduction kernel instead of the quantize kernel; the last argument only names the element type)
hipError_t family_strip_occupancy(size_t nbits, bool zt, bool stripe, int* per_cu, const float*);
hipError_t family_strip_occupancy(size_t nbits, bool zt, bool stripe, int* per_cu, const double*);
hipError_t family_unquantize(size_t nbits, hipStream_t s, LaunchEvents ev, const char* q, float* out, const UnquantizePlan& p, int add);
hipError_t family_batch_quantize(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const QuantizeBatchEntry* entries, const uint32_t* begins,
                                 uint32_t count, uint32_t total_blocks, size_t lds);
hipError_t family_batch_stripe(size_t nbits, bool zt, hipStream_t s, LaunchEvents ev, const StripeBatchEntry* entries, const uint32_t* begins,
                               uint32_t count, uint32_t total_blocks, size_t lds, bool wide);
hipError_t launch_unquantize_batch(hipStream_t s, LaunchEvents ev, const UnquantizeBatchEntry* entries, const uint32_t* begins, uint32_t count,
                                   uint32_t total_blocks, size_t nbits, bool add, size_t lds);

// forced = the caller insists on the column kernels: any height they can handle; otherwise only where they pay
inline bool col_applicable(const float* g, const float* r_in, const float* r_out, const void* q, size_t rows, size_t nbits,
                           bool forced = false)
{
    (void) nbits;
    const uintptr_t m = reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(r_in) | reinterpret_cast<uintptr_t>(r_out);
    return rows % 4 == 0 && rows <= kTileMaxRows && (forced ? rows >= 4 : rows >= kColMinRows) && (m & 15u) == 0 &&
           (reinterpret_cast<uintptr_t>(q) & 3u) == 0;
}

// Whether the three matrices sit at the same offset within a 128-byte line (then so do their columns), and whether any
// column can start inside a line at all.
inline bool same_line_offset(const void* g, const void* r_in, const void* r_out)
{
    const uintptr_t a = reinterpret_cast<uintptr_t>(g) & 127u, b = reinterpret_cast<uintptr_t>(r_in) & 127u,
                    c = reinterpret_cast<uintptr_t>(r_out) & 127u;
    return a == b && b == c;
}

inline bool columns_start_on_lines(const void* r_in, size_t rows, size_t rows_per_line = 32)
{
    return (reinterpret_cast<uintptr_t>(r_in) & 127u) == 0 && rows % rows_per_line == 0;
}

// Column kernels sum their statistics in the order of line-aligned slots when some column of the residual starts
// inside a 128-byte line.
inline bool quantize_line_shift(const float* g, const float* r_in, const float* r_out, size_t rows)
{
    // The residual's address alone decides (the slot dealing is part of the summation order, and the stripe reduction,
    // which must reproduce it, knows only the stripe residual); a gradient at another offset within a line is then
    // simply read across line boundaries.
    (void) g;
    (void) r_out;
    return !columns_start_on_lines(r_in, rows);
}

// the unrolled 1-bit kernels: 1024, 2048 or 4096 rows and 8-byte aligned packed buffers
inline bool col_unrolled(const void* q, size_t rows, size_t nbits)
{
    return nbits == 1 && (rows == 1024 || rows == 2048 || rows == 4096) && (reinterpret_cast<uintptr_t>(q) & 7u) == 0;
}

inline ColGeom make_col_geom(size_t rows, size_t nbits, bool line_shift)
{
    ColGeom c;
    c.rows = (uint32_t) rows;
    c.nq = (uint32_t) qwords_per_col(rows, nbits);
    c.pieces = (uint32_t) (rows / 4);
    c.line_shift = line_shift ? 1u : 0u;
    c.qcol = qcol_bytes(nbits, rows);
    return c;
}

inline RegGeom make_reg_geom(size_t rows, size_t nbits, uint32_t threads, bool line_shift)
{
    RegGeom c;
    c.rows = (uint32_t) rows;
    c.nq = (uint32_t) qwords_per_col(rows, nbits);
    c.pieces = (uint32_t) (rows / 4);
    c.step_k = (4 * threads) / c.nq;
    c.step_w = (4 * threads) % c.nq;
    c.line_shift = line_shift ? 1u : 0u;
    c.qcol = qcol_bytes(nbits, rows);
    return c;
}

// The register kernels: above 1024 rows (unless forced; 37.7 M elements at 1152 / 1536 / 2000 rows: 95 / 76 / 72 us against
// 102 / 81 / 80 us with the LDS column kernels, the same bytes), up to 25 pieces for each of
// 1024 threads, the column's QWords in LDS (reg_lds_fits). 256 threads up to the height the stripe reduction handles (whose
// LDS kernels then sum in the same order), 1024 above.
constexpr uint32_t kRegMinRows = 1024;
constexpr uint32_t kRegMaxRows = 4 * 1024 * 25;

inline uint32_t reg_threads(size_t rows)
{
    return rows <= kTileMaxRows ? 256u : 1024u;
}

// LDS of the register kernels: a workgroup may have all 160 KB of its compute unit. The quantize kernels keep the column's
// QWords there, the fused stripe reduction the output QWords and at least one worker's packed record: both families take
// the heights at which the latter fits, so that every stripe whose quantize step runs in registers can be reduced in
// registers too.
constexpr size_t kRegMaxLdsBytes = 160 * 1024;
inline bool reg_lds_fits(size_t rows, size_t nbits)
{
    return ((size_t) kRegRedSlots + 2 * qwords_per_col(rows, nbits) + 2) * 4 <= kRegMaxLdsBytes;
}

inline bool reg_applicable(const float* g, const float* r_in, const float* r_out, const void* q, size_t rows, size_t nbits,
                           bool forced = false)
{
    const uintptr_t m = reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(r_in) | reinterpret_cast<uintptr_t>(r_out);
    if (rows % 4 != 0 || rows < 4 || rows > kRegMaxRows || nbits >= 32 || (m & 15u) != 0 || (reinterpret_cast<uintptr_t>(q) & 3u) != 0)
        return false;
    if (!forced && rows <= kRegMinRows)
        return false;
    return reg_lds_fits(rows, nbits);
}

// The piece-wise register kernel with edge elements: matrices only 4-byte aligned, any height from 8 rows on. The aligned
// pieces are those of the residual input; a gradient or residual output at another offset within 16 bytes is read and
// written in 16-byte accesses at the 4-byte alignment that leaves them (quantize + unquantize of 50257 x 512 with the three
// matrices at three offsets: 81 us like the matrices at one offset, against 118 us one element per access; 9304 x 2048:
// 56.5 against 90 us).
inline bool reg_edge_applicable(const float* g, const float* r_in, const float* r_out, const void* q, size_t rows, size_t nbits)
{
    (void) g;
    (void) r_in;
    (void) r_out;
    if (rows < 8 || rows > kRegMaxRows - 32 || nbits >= 32 || (reinterpret_cast<uintptr_t>(q) & 3u) != 0)
        return false;
    return reg_lds_fits(rows, nbits);
}

// Matrices that are not whole aligned pieces (odd heights, slices at a 4-byte offset) above kRegEdge256MinRows rows: the
// register kernels with edge elements. From this height on with 1024 threads per column (9305 x 2048 44 us against the tile kernel's
// 57 us, 14335 x 1400 44 us against 82 us; at 4097 x 4652 the 1024 threads take 73 us against 48 us). The fused stripe
// reduction follows with its register kernel of the same workgroup size, which sums in the same order.
constexpr uint32_t kRegEdgeMinRows = 7168;

// ... and below it the same kernels with 256 threads per column, down to 2049 rows: 2049 x 9304 38.5 us against the tile
// kernel's 56 us, 4097 x 4652 40 us against 47 us, 6001 x 3000 38 us against 48 us. The stripe reduction that has to follow
// is slower than the tile one at these heights (full width, K = 8: 90 us against 86 us, 84 against 74, 78 against 63), but
// an all-reduce runs it on one K-th of the columns. At 1026 x 18000 the quantize kernels measure the same (49 us) and the
// stripe reductions 126 us against 85 us: up to 2048 rows the tile kernels stay.
constexpr uint32_t kRegEdge256MinRows = 2048;

inline uint32_t reg_edge_threads(size_t rows)
{
    return rows <= kRegEdgeMinRows ? 256u : 1024u;
}

constexpr uint32_t kRegsMaxRows = 1024 * 96;

inline bool regs_applicable(size_t rows, size_t nbits)
{
    return rows >= 1 && rows <= kRegsMaxRows && nbits < 32 && reg_lds_fits(rows, nbits);
}

// ---- strip kernels: any height, several workgroups per column ------------------------------------------------------


// The workgroups of a column wait for each other, so all of them must be resident at once: on one die at most half of
// what the die holds of the kernel (strip_resident_limit, asked from the runtime: 32 strips at 1 to 4 bits, i.e. 524288
// rows, on a die of 32 compute units at two workgroups each) and never more than this many; a column of more strips has
// them on all eight dies, up to eight times as many (4.2 M rows at 1 to 8 bits). Taller columns run the same strips in
// several launches.
constexpr uint32_t kStripMaxPerColumn = 128;

// (written over the element type: E's QWord has Word<E>::kBits bits)
template <typename E>
inline size_t strip_qwords_per_col(size_t rows, size_t nbits)
{
    const size_t vpw = Word<E>::kBits / nbits;
    return (rows + vpw - 1) / vpw;
}

template <typename E>
inline bool strip_applicable(size_t rows, size_t nbits, const LaunchTuning& tune)
{
    return tune.strip != nullptr && nbits < (size_t) Word<E>::kBits && rows >= 1 &&
           (strip_qwords_per_col<E>(rows, nbits) + strip_words<E>(nbits) - 1) / strip_words<E>(nbits) <= kStripMaxPerColumn * kStripDies;
}

// per_die: the most strips of a column that one die takes (strip_resident_limit); a column of more has its strips on all
// dies (StripGeom::spread), up to kStripDies times as many
template <typename E>
inline StripGeom make_strip_geom(size_t rows, size_t cols, size_t nbits, uint32_t spin_limit, uint32_t per_die)
{
    StripGeom c;
    c.rows = (uint32_t) rows;
    c.cols = (uint32_t) cols;
    c.nq = (uint32_t) strip_qwords_per_col<E>(rows, nbits);
    c.strips = (c.nq + strip_words<E>(nbits) - 1) / strip_words<E>(nbits);
    c.spin_limit = spin_limit;
    c.poll_pause = kStripPollPause;
    c.poll_first = c.strips >= kStripFirstPauseMinStrips ? 2u * std::min(c.strips, kStripMaxPerColumn) : 0u;
    c.inv_strips = 1.0 / (double) c.strips;
    c.spread = c.strips > per_die ? 1u : 0u;
    c.whole_positions = (uint32_t) (rows / c.nq);
    c.last_words = (uint32_t) (rows % c.nq);
    c.pad = 0;
    c.qcol = (uint64_t) (2 + c.nq) * sizeof(E); // the header's two bounds, then the QWords
    return c;
}

// records_each: records per (column, strip) of the element type (strip_records<E>())
inline bool strip_scratch_fits(const StripScratchOwner& o, size_t cols, size_t strips, size_t records_each)
{
    return o.dev != nullptr && strip_groups_bytes(cols, strips) <= o.groups_bytes &&
           sizeof(StripHeader) + o.groups_bytes + strip_records_bytes(cols, strips, records_each) <= o.bytes;
}

// Makes the owner's buffer large enough for this launch (growing waits for the stream and clears the new buffer: the launch
// count and every record's tag start at zero). Not possible while the stream is being captured.
inline hipError_t strip_scratch_for(StripScratchOwner& o, hipStream_t s, size_t cols, size_t strips, size_t records_each, StripScratch& out)
{
    if (o.error_host == nullptr)
    {
        void* p = nullptr;
        hipError_t rc = hipHostMalloc(&p, 64, hipHostMallocDefault);
        if (rc != hipSuccess)
            return rc;
        o.error_host = static_cast<uint32_t*>(p);
        *o.error_host = 0u;
    }
    if (!strip_scratch_fits(o, cols, strips, records_each))
    {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &st) == hipSuccess && st == hipStreamCaptureStatusActive)
            return hipErrorStreamCaptureUnsupported;
        hipError_t rc = hipStreamSynchronize(s);
        if (rc != hipSuccess)
            return rc;
        if (o.dev != nullptr)
        {
            if (o.captured)
                o.retired.push_back(o.dev); // a recorded launch may still be replayed on it
            else
                (void) hipFree(o.dev);
        }
        o.dev = nullptr;
        o.bytes = 0;
        o.captured = false;
        o.abandoned_seen = 0;
        const size_t need = sizeof(StripHeader) + strip_records_bytes(cols, strips, records_each);
        const size_t cap = std::max<size_t>((need * 2 + 8191) & ~(size_t) 4095, (size_t) 1 << 20);
        void* p = nullptr;
        rc = hipMalloc(&p, cap);
        if (rc != hipSuccess)
            return rc;
        rc = hipMemsetAsync(p, 0, cap, s);
        if (rc == hipSuccess)
            rc = hipStreamSynchronize(s); // whichever stream launches next finds the buffer cleared
        if (rc != hipSuccess)
        {
            (void) hipFree(p);
            return rc;
        }
        o.dev = static_cast<char*>(p);
        o.bytes = cap;
        o.groups_bytes = (cap / 256 + 63) & ~(size_t) 63; // counters need 1/512 of what the records need
    }
    out.error = o.error_host;
    out.header = reinterpret_cast<StripHeader*>(o.dev);
    out.groups = reinterpret_cast<uint32_t*>(o.dev + sizeof(StripHeader));
    out.records = reinterpret_cast<uint64_t*>(o.dev + sizeof(StripHeader) + o.groups_bytes);
    return hipSuccess;
}

// whether this launch finds its scratch buffer without allocating, or may allocate (the caller permits it and the stream
// is not being captured)
inline bool strip_scratch_ready(const StripScratchOwner& o, hipStream_t s, size_t cols, size_t strips, size_t records_each, bool may_allocate = true)
{
    if (o.error_host != nullptr && strip_scratch_fits(o, cols, strips, records_each))
        return true;
    if (!may_allocate)
        return false;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &st) == hipSuccess && st == hipStreamCaptureStatusNone;
}

inline uint32_t strip_grid(size_t cols, const StripGeom& c)
{
    return (uint32_t) (c.spread ? cols * c.strips : (cols + kStripDies - 1) / kStripDies * kStripDies * c.strips);
}

// How many strips a column may have for the automatic choice to take the strip kernels: the strips of a column wait for
// each other on one die, so all of them must be resident there together, next to the strips of the columns around them.
// Half of what the die holds by the runtime's own occupancy figure for the kernel (workgroups per compute unit x compute
// units of the device / 8 dies); 0 where the runtime cannot say. Asked once per kernel variant and device.
template <typename E>
inline uint32_t strip_resident_limit(size_t nbits, bool zt, bool stripe = false)
{
    static int cache[64][6][2][2]; // 0: not asked yet; -1: unknown (one table per element type)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 0;
    const int b = nbits == 1 ? 0 : nbits == 2 ? 1 : nbits == 4 ? 2 : nbits == 8 ? 3 : nbits == 16 ? 4 : 5;
    int& slot = cache[dev][b][zt ? 1 : 0][stripe ? 1 : 0];
    if (slot == 0)
    {
        int per_cu = 0, cus = 0;
        hipError_t rc = family_strip_occupancy(nbits, zt, stripe, &per_cu, (const E*) nullptr);
        if (rc == hipSuccess)
            rc = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (rc != hipSuccess)
            (void) hipGetLastError();
        slot = (rc == hipSuccess && per_cu > 0 && cus >= (int) kStripDies) ? per_cu * (cus / (int) kStripDies) / 2 : -1;
    }
    return slot > 0 ? (uint32_t) slot : 0u;
}

// ... the same, never more than kStripMaxPerColumn
template <typename E>
inline uint32_t strip_per_die(size_t nbits, bool zt, bool stripe = false)
{
    return std::min(strip_resident_limit<E>(nbits, zt, stripe), kStripMaxPerColumn);
}

// the most strips per column that the strip kernels take on the current device, spread over all dies
template <typename E>
inline uint32_t strip_max_strips(size_t nbits, bool zt, bool stripe = false)
{
    return strip_per_die<E>(nbits, zt, stripe) * kStripDies;
}

// Whether the automatic choice may hand this matrix to the strip kernels right now: a column within what the device holds
// of strips, and a scratch buffer that is there or may be made (a stream under capture cannot wait for a larger one).
// Whether the strip kernels cut into passes may take this matrix right now: any number of strips (nothing waits, so nothing
// need be resident together), at least two, a grid the launch can express, and the scratch buffer there or obtainable.
template <typename E>
inline bool strip_passes_ready(hipStream_t s, size_t rows, size_t cols, size_t nbits, const LaunchTuning& tune)
{
    if (tune.strip == nullptr || nbits >= (size_t) Word<E>::kBits || rows < 1)
        return false;
    const size_t strips = (strip_qwords_per_col<E>(rows, nbits) + strip_words<E>(nbits) - 1) / strip_words<E>(nbits);
    return strips >= 2 && (uint64_t) (cols + kStripDies) * strips <= 0x7FFFFFFFull &&
           strip_scratch_ready(*tune.strip, s, cols, strips, strip_records<E>(), tune.strip_may_allocate);
}

template <typename E>
inline bool strip_ready(hipStream_t s, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune, bool stripe = false)
{
    if (!strip_applicable<E>(rows, nbits, tune))
        return false;
    const StripGeom c = make_strip_geom<E>(rows, cols, nbits, tune.strip_spin_limit, strip_per_die<E>(nbits, zt, stripe));
    return (uint64_t) (cols + kStripDies) * c.strips <= 0x7FFFFFFFull && c.strips <= strip_max_strips<E>(nbits, zt, stripe) &&
           strip_scratch_ready(*tune.strip, s, cols, c.strips, strip_records<E>(), tune.strip_may_allocate);
}

// A strip kernel on one matrix of either element type: the scratch buffer (grown if need be), the order against the last
// launch that used it on another stream, then `launch(geometry, scratch)`.
template <typename E, typename Launch>
inline hipError_t launch_on_strips(hipStream_t s, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune, bool stripe,
                                   Launch launch, bool passes = false)
{
    // (in passes: strips side by side in the grid whatever their number, and no pause before a first look that finds everything)
    StripGeom c = make_strip_geom<E>(rows, cols, nbits, tune.strip_spin_limit, passes ? 0u : strip_per_die<E>(nbits, zt, stripe));
    if (passes)
    {
        c.poll_first = 0;
        if (tune.strip == nullptr || nbits >= (size_t) Word<E>::kBits || c.strips < 2 || (uint64_t) (cols + kStripDies) * c.strips > 0x7FFFFFFFull)
            return hipErrorInvalidValue;
    }
    else if (!strip_applicable<E>(rows, nbits, tune) || (uint64_t) (cols + kStripDies) * c.strips > 0x7FFFFFFFull ||
             c.strips > strip_max_strips<E>(nbits, zt, stripe))
        return hipErrorInvalidValue;
    StripScratchOwner& o = *tune.strip;
    StripScratch scratch;
    hipError_t rc = strip_scratch_for(o, s, cols, c.strips, strip_records<E>(), scratch);
    if (rc != hipSuccess)
        return rc;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(s, &st) != hipSuccess || st != hipStreamCaptureStatusNone;
    if (capturing)
        o.captured = true;
    if (!capturing)
    {
        if (o.order_event == nullptr && (rc = hipEventCreateWithFlags(&o.order_event, hipEventDisableTiming)) != hipSuccess)
            return rc;
        if (o.launched && o.last_stream != s && (rc = hipStreamWaitEvent(s, o.order_event, 0)) != hipSuccess)
            return rc;
    }
    rc = launch(c, scratch);
    if (rc == hipSuccess && !capturing)
    {
        rc = hipEventRecord(o.order_event, s);
        o.last_stream = s;
        o.launched = true;
    }
    return rc;
}

template <typename E>
inline hipError_t launch_strip_quantize(hipStream_t s, LaunchEvents ev, const E* g, const E* r_in, E* r_out, char* qc, size_t rows, size_t cols,
                                        size_t nbits, bool zt, const LaunchTuning& tune)
{
    return launch_on_strips<E>(s, rows, cols, nbits, zt, tune, false, [&](const StripGeom& c, const StripScratch& scratch) {
        return family_strip_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols, c, scratch);
    });
}

// ... cut into two or three launches: for columns of more strips than the device holds at once (same bytes)
template <typename E>
inline hipError_t launch_strip_quantize_passes(hipStream_t s, LaunchEvents ev, const E* g, const E* r_in, E* r_out, char* qc, size_t rows,
                                               size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    return launch_on_strips<E>(
        s, rows, cols, nbits, zt, tune, false,
        [&](const StripGeom& c, const StripScratch& scratch) {
            return family_strip_quantize_passes(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols, c, scratch);
        },
        true);
}

// The fused stripe reduction on strips: for stripes taller than the kernels with a workgroup per column take, where a
// quantize call on (aggregate, stripe residual) takes the strip kernel too, so that both give the same bytes.
template <typename E>
inline hipError_t launch_strip_stripe(hipStream_t s, LaunchEvents ev, const StripeSources& src, E* stripe_res, char* q_out, E* agg_out, size_t rows,
                                      size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    return launch_on_strips<E>(s, rows, cols, nbits, zt, tune, true, [&](const StripGeom& c, const StripScratch& scratch) {
        return family_strip_stripe(nbits, zt, s, ev, src, stripe_res, q_out, agg_out, (uint32_t) cols, c, scratch);
    });
}

// which path launch_quantize takes for this matrix when nothing is forced
inline int quantize_auto_path(const float* g, const float* r_in, const float* r_out, const void* q, size_t rows, size_t nbits,
                              bool strip_available = false)
{
    // (2048 rows at 1 bit: the unrolled LDS kernel, where its conditions hold, is as fast)
    const bool unrolled = rows <= 2048 && col_applicable(g, r_in, r_out, q, rows, nbits) && col_unrolled(q, rows, nbits) &&
                          !quantize_line_shift(g, r_in, r_out, rows);
    if (!unrolled && reg_applicable(g, r_in, r_out, q, rows, nbits))
        return kPathReg;
    // not whole aligned pieces (odd heights, slices at a 4-byte offset): the register kernel with edge elements
    if (rows > kRegEdge256MinRows && reg_edge_applicable(g, r_in, r_out, q, rows, nbits))
        return kPathReg;
    if (rows > kTileMaxRows)
    {
        // What no workgroup's registers hold in whole aligned pieces (the three matrices at different offsets within 16
        // bytes): one element per access up to 98304 rows (as fast there as the strips, and faster below 50000 rows),
        // then strips of the column on several workgroups, then -- above what a die holds of them -- the kernel that re-reads its column.
        if (regs_applicable(rows, nbits))
            return kPathRegScalar;
        return strip_available ? kPathStrip : kPathTall;
    }
    if (col_applicable(g, r_in, r_out, q, rows, nbits))
        return kPathCol;
    return kPathTile;
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
        path = quantize_auto_path(g, r_in, r_out, q, rows, nbits, strip_applicable<float>(rows, nbits, tune));
        // (a stream under capture cannot wait for a larger scratch buffer: the kernels that need none take the matrix)
        if (path == kPathStrip && (tune.strip_never_waits || !strip_ready<float>(s, rows, cols, nbits, zt, tune)))
            path = regs_applicable(rows, nbits) ? kPathRegScalar : kPathTall;
        // columns of more strips than the device holds at once: the strips in passes, which read the matrix two or three
        // times like the kernel with one workgroup per column, but on the whole device
        if (path == kPathTall && nbits < 32 && strip_passes_ready<float>(s, rows, cols, nbits, tune))
            path = kPathStripPasses;
    }
    if (path == kPathReg)
    {
        if (!reg_applicable(g, r_in, r_out, q, rows, nbits, true))
        {
            // not whole aligned pieces: the variant with edge elements, where the three matrices allow it
            if (!reg_edge_applicable(g, r_in, r_out, q, rows, nbits))
                return hipErrorInvalidValue;
            const uint32_t threads = reg_edge_threads(rows);
            RegGeom c = make_reg_geom(rows, nbits, threads, true); // always dealt by the residual's lines
            return family_reg_edge_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols, c, threads);
        }
        const uint32_t threads = reg_threads(rows);
        // up to 14336 rows the shift is part of the summation order all column kernels share; above, it is used where
        // the registers allow
        const bool line_shift = quantize_line_shift(g, r_in, r_out, rows) && (threads == 256 || rows / 4 + 7 <= 1024 * (size_t) kRegMaxShiftPer);
        return family_reg_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols,
                                           make_reg_geom(rows, nbits, threads, line_shift), threads);
    }
    if (path == kPathStrip)
        return launch_strip_quantize<float>(s, ev, g, r_in, r_out, qc, rows, cols, nbits, zt, tune);
    if (path == kPathStripPasses)
        return launch_strip_quantize_passes<float>(s, ev, g, r_in, r_out, qc, rows, cols, nbits, zt, tune);
    if (path == kPathRegScalar)
    {
        if (!regs_applicable(rows, nbits))
            return hipErrorInvalidValue;
        RegGeom c = make_reg_geom(rows, nbits, kRegsThreads, false);
        c.step_k = kRegsThreads / c.nq; // a thread's next element lies 1024 elements further on
        c.step_w = kRegsThreads % c.nq;
        return family_regs_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols, c);
    }
    if (path == kPathCol)
    {
        if (!col_applicable(g, r_in, r_out, q, rows, nbits, true))
            return hipErrorInvalidValue;
        // (the unrolled kernels deal pieces without a shift: only for columns that start on lines)
        const bool line_shift = quantize_line_shift(g, r_in, r_out, rows);
        if (line_shift || !col_unrolled(q, rows, nbits))
            return family_col_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) cols, make_col_geom(rows, nbits, line_shift));
        const uint64_t qcol = qcol_bytes(nbits, rows);
        const uint32_t c = (uint32_t) cols;
        return family_col_quantize_unrolled(zt, rows == 1024 ? 1 : (rows == 2048 ? 2 : 4), s, ev, g, r_in, r_out, qc, c, qcol);
    }
    if (path == kPathTile)
    {
        if (rows > kTileMaxRows)
            return hipErrorInvalidValue;
        const TileGeom t = make_tile_geom(rows, cols, nbits, tune.tile_gs, tune.tile_stage, tune.tile_threads);
        return family_tile_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, t);
    }
    return family_tall_quantize(nbits, zt, s, ev, g, r_in, r_out, qc, (uint32_t) rows, (uint32_t) cols,
                                        (uint32_t) qwords_per_col(rows, nbits), (uint64_t) qcol_bytes(nbits, rows));
}

// Tallest column the fused stripe reduction takes at this bit width: up to kTileMaxRows with the LDS kernels, above it
// with the register kernel, whose LDS holds the output QWords and one worker's packed record.
inline size_t stripe_reduce_max_rows(size_t nbits)
{
    if (nbits >= 32)
        return kTileMaxRows;
    const size_t max_nq = (kRegMaxLdsBytes / 4 - kRegRedSlots - 2) / 2;
    const size_t by_lds = max_nq * (32 / nbits);
    const size_t by_regs = kRegMaxRows - 32;
    const size_t tall = by_lds < by_regs ? by_lds : by_regs;
    return tall > kTileMaxRows ? tall : kTileMaxRows;
}

// Heights at which no kernel with one workgroup per column takes a matrix whatever its alignment, so that the automatic
// choice of a quantize call is the strip kernels (or, without them, the kernel that re-reads its columns).
inline bool strip_only_height(size_t rows, size_t nbits)
{
    return nbits < 32 && rows > kTileMaxRows && (rows > kRegMaxRows || !reg_lds_fits(rows, nbits));
}

// Whether the fused stripe reduction takes a stripe taller than stripe_reduce_max_rows: on strips, where a quantize call
// on (aggregate, stripe residual) would run on strips as well (same bytes), with the scratch buffer there or obtainable.
inline bool stripe_takes_strips(hipStream_t s, size_t rows, size_t cols, size_t nbits, bool zt, const LaunchTuning& tune)
{
    zt = zt && nbits == 1;
    return !tune.strip_never_waits && strip_only_height(rows, nbits) && strip_ready<float>(s, rows, cols, nbits, zt, tune, false) &&
           strip_ready<float>(s, rows, cols, nbits, zt, tune, true);
}

// Whether a stripe whose height and alignment would let the LDS column kernels take it goes to the table-driven register
// kernel with 256 threads instead (1 bit, up to eight workers, above 2048 rows), and how many pieces a thread holds there.
inline bool stripe_looks_up(size_t rows, size_t nbits, size_t workers)
{
    return nbits == 1 && workers >= 1 && workers <= 8 && rows > 2048;
}
inline uint32_t stripe_lookup_per(size_t rows, bool line_shift)
{
    return (uint32_t) ((rows / 4 + (line_shift ? 7 : 0) + 255) / 256);
}

// Whether the fused stripe reduction runs the 1024-thread register kernel: wherever a quantize call on (aggregate, stripe
// residual) would run the register kernels with edge elements or with 1024 threads, whose summation order it shares -- above
// the LDS kernels' heights, and from kRegEdge256MinRows + 1 rows on for stripes that are not whole aligned pieces.
inline bool stripe_uses_reg(size_t rows, const void* stripe_res, size_t nbits, int forced_path = kPathAuto)
{
    if (rows > kTileMaxRows)
        return true;
    const bool whole = rows % 4 == 0 && (reinterpret_cast<uintptr_t>(stripe_res) & 15u) == 0;
    return forced_path == kPathAuto && rows > kRegEdge256MinRows && !whole && nbits < 32;
}

inline hipError_t launch_stripe_reduce(hipStream_t s, LaunchEvents ev, const StripeSources& src, float* stripe_res, void* q_out,
                                       float* agg_out, size_t rows, size_t cols, size_t nbits, bool zt,
                                       const LaunchTuning& tune)
{
    zt = zt && (nbits == 1);
    if (rows > stripe_reduce_max_rows(nbits))
    {
        if (!stripe_takes_strips(s, rows, cols, nbits, zt, tune) || (reinterpret_cast<uintptr_t>(q_out) & 3u) != 0)
            return hipErrorInvalidValue;
        return launch_strip_stripe<float>(s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, rows, cols, nbits, zt, tune);
    }
    if (stripe_uses_reg(rows, stripe_res, nbits, tune.quantize_path))
    {
        if (rows > stripe_reduce_max_rows(nbits) || (reinterpret_cast<uintptr_t>(q_out) & 3u) != 0)
            return hipErrorInvalidValue;
        // The slots are dealt as a quantize call on (aggregate, stripe residual) deals them, given the residual's address:
        // whole aligned pieces and a line shift where columns start inside a line, or the variant with edge elements
        // (always shifted); a shift that would need a 26th piece per thread is dropped there as here.
        const bool whole = rows % 4 == 0 && (reinterpret_cast<uintptr_t>(stripe_res) & 15u) == 0;
        bool line_shift = whole ? !columns_start_on_lines(stripe_res, rows) : true;
        if (whole && rows / 4 + 7 > 1024 * (size_t) kRegMaxShiftPer)
            line_shift = false;
        // (only stripes that are not whole aligned pieces get here below the LDS kernels' limit: 256 threads up to 7168 rows)
        const uint32_t threads = rows > kTileMaxRows ? 1024u : reg_edge_threads(rows);
        const RegGeom c = make_reg_geom(rows, nbits, threads, line_shift);
        return family_reg_stripe(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, (uint32_t) cols, c,
                                                 threads);
    }
    bool aligned8 = (reinterpret_cast<uintptr_t>(q_out) & 7u) == 0;
    for (uint32_t w = 0; w < src.workers; ++w)
        aligned8 = aligned8 && (reinterpret_cast<uintptr_t>(src.q[w]) & 7u) == 0;
    const bool col_forced = tune.quantize_path == kPathCol;
    // (a quantize call on a residual that is not 16-byte aligned takes the tile kernel, and so does the automatic choice here)
    const bool col = (tune.quantize_path == kPathAuto || col_forced) && rows % 4 == 0 &&
                     (col_forced || (rows >= kColMinRows && (reinterpret_cast<uintptr_t>(stripe_res) & 15u) == 0));
    // the summation order a quantize call on (aggregate, stripe residual) would use, given the residual's address
    const bool line_shift = !columns_start_on_lines(stripe_res, rows);
    if (col && (line_shift || !(aligned8 && col_unrolled(q_out, rows, nbits))))
    {
        // 1 bit, up to eight workers, above 2048 rows: the table-driven register kernel with 256 threads, which sums the
        // statistics in the LDS column kernels' order (same bytes) and is faster (6144 x 3101, K = 8: 39 against 69 us;
        // at 1152 rows there is nothing in it)
        if (tune.quantize_path == kPathAuto && stripe_looks_up(rows, nbits, src.workers))
        {
            const RegGeom c = make_reg_geom(rows, nbits, 256, line_shift);
            return family_reg_stripe(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, (uint32_t) cols, c,
                                                     256u);
        }
        return family_col_stripe(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, (uint32_t) cols,
                                                 make_col_geom(rows, nbits, line_shift));
    }
    if (col)
    {
        // same column statistics, in the same order, as quantize_col_kernel
        const uint64_t qcol = qcol_bytes(nbits, rows);
        const uint32_t c = (uint32_t) cols;
        char* qo = static_cast<char*>(q_out);
        return family_col_stripe_unrolled(zt, rows == 1024 ? 1 : (rows == 2048 ? 2 : 4), s, ev, src, stripe_res, qo, agg_out, c, qcol);
    }
    // Same tile geometry as launch_quantize would use for a matrix of this height, so that the statistics are summed in
    // the same order and the fused call gives the bytes of the reference's unquantize ... quantize call sequence.
    const TileGeom t = make_tile_geom(rows, cols, nbits, tune.tile_gs, tune.tile_stage, tune.tile_threads);
    return family_tile_stripe(nbits, zt, s, ev, src, stripe_res, static_cast<char*>(q_out), agg_out, t);
}

// ---- unquantize: which decoder, with which geometry ---------------------------------------------------

struct UnquantizePlan
{
    uint32_t kind = kUnqScalar;
    UnqGeom qw;
    UnqSegGeom seg;
    UnqRowGeom rowg;
    UnqTileGeom tile;
    UnqFlatGeom flat;
    uint32_t blocks = 0; // 256-thread blocks
    size_t lds = 0;      // dynamic LDS (kUnqRows, kUnqTile)
    bool ok = false;
};

// The geometry of the LDS-free decoder for short columns (per16 elements in 16 bytes): heights that are multiples of per16,
// per16 QWords or more, fewer than 2^32 elements. False where it cannot run.
inline bool make_unq_flat_geom(UnqFlatGeom& t, size_t rows, size_t cols, size_t nq, uint64_t qcol, size_t per16)
{
    const uint64_t elems = (uint64_t) rows * cols;
    if (rows == 0 || rows % per16 != 0 || nq < per16 || elems == 0 || elems > 0xFFFFFFFFull)
        return false;
    t.rows = (uint32_t) rows;
    t.nq = (uint32_t) nq;
    t.groups = (uint32_t) (elems / per16);
    t.blocks = (uint32_t) ((t.groups + 256 * kUnqDirectPieces - 1) / (256 * kUnqDirectPieces));
    t.inv_rows = 1.0 / (double) rows;
    t.inv_nq = 1.0 / (double) nq;
    t.qcol = qcol;
    return true;
}

constexpr size_t kUnqRowsMaxLds = 48 * 1024;
constexpr uint32_t kUnqRowsChunk = 2048;
constexpr size_t kUnqTileMaxRows = 16384; // 4 columns of that height: 65536 elements, small enough for the magic divisions
constexpr size_t kUnqTileElems = 4096;    // values per workgroup the tile decoder aims for
constexpr size_t kUnqRowsMinRows = 1664;  // from this height on a column per workgroup (row-major decoder) beats several columns per
                                          // workgroup (tile decoder): 1152 x 8192 7.5 us against 9.8 us, 1792 x 5266 8.5 us against 7.6 us

// The geometry of the row-major decoder that fetches its QWords itself: chunks of 256 threads x kUnqDirectPieces 16-byte
// stores (per16 elements each). False if the grid would not fit.
inline bool make_unq_direct_geom(UnqRowGeom& t, size_t rows, size_t cols, size_t nq, uint64_t qcol, size_t per16)
{
    const size_t chunk = 256 * kUnqDirectPieces * per16;
    const uint64_t chunks = (rows + chunk - 1) / chunk;
    const uint64_t blocks = (uint64_t) cols * chunks;
    if (blocks > 0x7FFFFFFFull)
        return false;
    t.rows = (uint32_t) rows;
    t.nq = (uint32_t) nq;
    t.chunk = (uint32_t) chunk;
    t.chunks = (uint32_t) chunks;
    t.blocks = (uint32_t) blocks;
    t.pad = 0;
    t.qcol = qcol;
    return true;
}

inline UnquantizePlan plan_unquantize(const void* q, const float* out, size_t rows, size_t cols, size_t nbits,
                                      const LaunchTuning& tune)
{
    UnquantizePlan p;
    std::memset(&p.qw, 0, sizeof p.qw);
    std::memset(&p.seg, 0, sizeof p.seg);
    std::memset(&p.rowg, 0, sizeof p.rowg);
    const size_t vpw = 32 / nbits;
    const size_t nq = qwords_per_col(rows, nbits);
    std::memset(&p.tile, 0, sizeof p.tile);
    std::memset(&p.flat, 0, sizeof p.flat);
    const int mode = tune.unq_mode;
    const bool out16 = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    const bool slots_free = tune.unq_slots == 0;
    // QWord-major decoder with 16-byte stores. It is at its best when every bit position of a column is a run of whole
    // 128-byte lines: QWords a multiple of 32, all of them full, columns starting on a line.
    const bool vec_can = (nq % 4 == 0) && (rows % 4 == 0) && out16 && (reinterpret_cast<uintptr_t>(q) & 7u) == 0;
    const bool vec_ideal = vec_can && nq % 32 == 0 && rows % 32 == 0 && rows * nbits == nq * 32;
    const bool rows_can = slots_free && rows >= 16 && nq >= 32 && nq * 4 <= kUnqRowsMaxLds; // any height, any (4-byte) alignment
    const bool tile_can = slots_free && rows <= kUnqTileMaxRows; // (any 4-byte alignment of the output)
    const bool direct_can = slots_free && rows >= 16 && nq >= 32; // any height, any (4-byte) alignment
    // Where the row-major decoder that fetches its QWords itself is the automatic choice (measured against the others):
    // from 16384 rows on; from 8192 rows at 2 bits and more where the QWord-major stores would not be whole lines, unless
    // the last chunk of a column would be mostly empty; and the 1- and 2-bit columns of exactly one to four chunks
    // (2048 ... 8192 rows), by 2 to 3 % -- in a launch of their own: as members of a gradient-set launch they measured slower.
    const size_t direct_chunk = 256 * kUnqDirectPieces * 4;
    const bool direct_full = (((rows + direct_chunk - 1) / direct_chunk) * direct_chunk - rows) * 8 <= rows;
    const bool direct_auto = direct_can && (rows >= 16384 || (!vec_ideal && nbits >= 2 && rows >= 8192 && direct_full) ||
                                            (vec_ideal && nbits <= 2 && rows % direct_chunk == 0 && rows <= 8192 && !tune.unq_member));
    bool vec = false, rowmajor = false, tile = false, seg_allowed = true, direct = false;
    // The LDS-free decoder for short columns, wherever it can run below 10000 rows: in a launch of its
    // own it measured 4 to 24 % faster than the tile, row-major and QWord-major decoders it replaces (512 x 100000: 38.3 ->
    // 33.7 us, 576 x 16384 at 2 bits 9.1 -> 7.0 us, 64 x 400000 at 8 bits 22.9 -> 19.4 us, 1536 x 12288 13.4 -> 12.1 us,
    // 1000 x 20000 at 1 / 8 bits 16.3 / 21.5 -> 12.9 / 17.1 us;
    // even at 512 x 40000 and 2304 x 4096 at 4 bits). As a member of a gradient-set launch only a large matrix (4 M elements)
    // gains (the LSTM set's decode with its 512 x 100000 and 1024 x 4096 members: 80.6 -> 69.4 us); ResNet-50's 161 members
    // and the 2048 x 1163 stripes of the all-reduce measured 5 to 7 % slower with it and keep their decoders.
    const bool flat_auto = mode == 0 && !direct_auto && rows < 10000 && // (9304 x 2048: 14.4 -> 13.7 us; even from 10000 rows on)
                           (!tune.unq_member || (uint64_t) rows * cols >= ((uint64_t) 1 << 22));
    if ((mode == 6 || flat_auto) && slots_free && out16 && make_unq_flat_geom(p.flat, rows, cols, nq, qcol_bytes(nbits, rows), 4))
    {
        p.kind = kUnqFlat;
        p.blocks = p.flat.blocks;
        p.ok = true;
        return p;
    }
    if (mode == 5 && direct_can)
        direct = true;
    else if (mode == 0 && direct_auto)
        direct = true;
    else if (mode == 1)
        seg_allowed = false; // QWord-major, 4-byte stores
    else if (mode == 2 && tile_can)
        tile = true;
    else if (mode == 4 && rows_can)
        rowmajor = true;
    else if (mode == 3 || !slots_free)
    {
        // the choice without the tile decoder
        vec = vec_can;
        rowmajor = !vec && rows_can;
    }
    else if (vec_ideal)
        vec = true;
    else if (rows_can && rows >= kUnqRowsMinRows)
        rowmajor = true; // a column fills a workgroup
    else if (tile_can)
        tile = true;
    else if (rows_can)
        rowmajor = true;
    else
        vec = vec_can;
    if (tile)
    {
        UnqTileGeom& t = p.tile;
        t.rows = (uint32_t) rows;
        t.cols = (uint32_t) cols;
        t.nq = (uint32_t) nq;
        size_t cpt = (kUnqTileElems / rows) & ~(size_t) 3;
        if (cpt < 4)
            cpt = 4;
        t.cpt = (uint32_t) cpt;
        t.rec_words = (uint32_t) nq + 2;
        t.rows_magic = rows > 1 ? (uint32_t) ((((uint64_t) 1 << 32) + rows - 1) / rows) : 0u;
        t.nq_magic = nq > 1 ? (uint32_t) ((((uint64_t) 1 << 32) + nq - 1) / nq) : 0u;
        const uint64_t blocks = (cols + cpt - 1) / cpt;
        if (blocks <= 0x7FFFFFFFull && unq_tile_lds_bytes(t) <= 64 * 1024)
        {
            t.blocks = (uint32_t) blocks;
            p.kind = kUnqTile;
            p.blocks = t.blocks;
            p.lds = unq_tile_lds_bytes(t);
            p.ok = true;
            return p;
        }
        vec = vec_can;
    }
    if (direct && make_unq_direct_geom(p.rowg, rows, cols, nq, qcol_bytes(nbits, rows), 4))
    {
        p.kind = kUnqDirect;
        p.blocks = p.rowg.blocks;
        p.ok = true;
        return p;
    }
    if (rowmajor)
    {
        UnqRowGeom& t = p.rowg;
        t.rows = (uint32_t) rows;
        t.nq = (uint32_t) nq;
        // small chunks keep many workgroups in flight; a chunk still spans several bit positions so that copying the
        // packed column into LDS stays a small part of the work
        // (columns of more than 1024 QWords did best with two bit positions, shorter ones with four)
        const size_t mult = nq > 1024 ? 2 : 4;
        size_t chunk = ((mult * nq + 1023) / 1024) * 1024;
        if (chunk < kUnqRowsChunk)
            chunk = kUnqRowsChunk;
        t.chunk = (uint32_t) chunk;
        // the last chunk is the remainder, or takes the remainder along when that is less than half a chunk
        t.chunks = rows >= chunk ? (uint32_t) ((rows + chunk / 2) / chunk) : 1u;
        const uint64_t blocks = (uint64_t) cols * t.chunks;
        if (blocks <= 0x7FFFFFFFull)
        {
            t.blocks = (uint32_t) blocks;
            t.qcol = qcol_bytes(nbits, rows);
            p.kind = kUnqRows;
            p.blocks = t.blocks;
            p.lds = nq * 4;
            p.ok = true;
            return p;
        }
    }
    // other long columns that the QWord-major decoder could only serve with 4-byte stores go to the segment decoder
    const bool seg = !vec && seg_allowed && out16 && nq >= 32;
    if (seg)
    {
        UnqSegGeom& t = p.seg;
        t.rows = (uint32_t) rows;
        t.nq = (uint32_t) nq;
        t.segs = (uint32_t) ((rows + nq - 1) / nq);
        t.gps = (uint32_t) ((nq + 3 + 3) / 4);
        const uint64_t items = (uint64_t) cols * t.segs * t.gps;
        if (items <= 0xFFFFFFFFull)
        {
            t.items = (uint32_t) items;
            t.inv_gps = 1.0 / (double) t.gps;
            t.inv_segs = 1.0 / (double) t.segs;
            t.qcol = qcol_bytes(nbits, rows);
            p.kind = kUnqSegment;
            p.blocks = (uint32_t) ((items + 255) / 256);
            p.ok = true;
            return p;
        }
    }
    const uint32_t wv = vec ? 4 : 1;
    UnqGeom& t = p.qw;
    t.rows = (uint32_t) rows;
    t.cols = (uint32_t) cols;
    t.nq = (uint32_t) nq;
    t.groups = (uint32_t) ((nq + wv - 1) / wv);
    uint32_t slots = tune.unq_slots;
    if (slots == 0)
        slots = vpw < 2 ? (uint32_t) vpw : 2;
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
            t.swz_members = (uint32_t) (per_col / 256); // every workgroup of the column spans all its QWords
        else if (t.groups % 256 == 0)
        {
            t.swz_members = t.chunks;
            t.swz_gw = t.groups / 256;
        }
    }
    t.qcol = qcol_bytes(nbits, rows);
    p.kind = vec ? kUnqVec4 : kUnqScalar;
    p.blocks = (uint32_t) ((items + 255) / 256);
    p.ok = true;
    return p;
}

inline hipError_t launch_unquantize(hipStream_t s, LaunchEvents ev, const void* q, float* out, size_t rows, size_t cols, size_t nbits,
                                    bool add, const LaunchTuning& tune)
{
    const UnquantizePlan p = plan_unquantize(q, out, rows, cols, nbits, tune);
    if (!p.ok)
        return hipErrorInvalidValue;
    return family_unquantize(nbits, s, ev, static_cast<const char*>(q), out, p, add ? 1 : 0);
}

// ---- many matrices per launch -----------------------------------------------------------------------
// The entry tables live in device memory; the caller (the C-ABI layer) owns them and keeps them alive until the
// kernel has finished.

inline hipError_t launch_quantize_batch(hipStream_t s, LaunchEvents ev, const QuantizeBatchEntry* entries, const uint32_t* begins,
                                        uint32_t count, uint32_t total_blocks, size_t lds, size_t nbits, bool zt)
{
    zt = zt && (nbits == 1);
    return family_batch_quantize(nbits, zt, s, ev, entries, begins, count, total_blocks, lds);
}

inline hipError_t launch_stripe_reduce_batch(hipStream_t s, LaunchEvents ev, const StripeBatchEntry* entries, const uint32_t* begins,
                                             uint32_t count, uint32_t total_blocks, size_t lds, size_t nbits, bool zt, bool wide)
{
    zt = zt && (nbits == 1);
    return family_batch_stripe(nbits, zt, s, ev, entries, begins, count, total_blocks, lds, wide);
}

// which kernel family launch_stripe_reduce takes by itself for a stripe of this height: columns (true) or tiles
inline bool stripe_auto_col(size_t rows, const void* stripe_res)
{
    return rows % 4 == 0 && rows >= kColMinRows && (reinterpret_cast<uintptr_t>(stripe_res) & 15u) == 0;
}

// colg_lds_bytes for a bit width known only at run time
inline size_t colg_lds_bytes_rt(const ColGeom& c, size_t nbits)
{
    return ((size_t) c.rows + (nbits <= 2 ? c.nq : 0) + kColgRedSlots) * sizeof(float);
}


} // namespace cntkq
