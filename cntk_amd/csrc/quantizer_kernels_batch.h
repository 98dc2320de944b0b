// gfx950 kernels of the per-column gradient quantizer: whole gradient sets in one launch.
#pragma once

#include "quantizer_kernels_column.h"
#include "quantizer_kernels_unquantize.h"

namespace cntkq {

// largest e with begins[e] <= b (begins ascending, begins[0] = 0); b and everything derived from it is uniform over the
// workgroup. One round trip to the table instead of log2(count) dependent ones: the 64 lanes of a wavefront test one
// entry each, and the number of entries <= b, minus one, is the answer; above 64 entries a first pass over every
// stride-th entry narrows the range to at most 64 (4096 entries: two round trips). Every wavefront of the workgroup
// does the same look-up. A workgroup of a batched launch lives a few microseconds, of which the dependent loads of a
// binary search were a noticeable part (8 stripe views of 2048 x 1163 decoded in 15.8 us against 12.2 us for the
// plain launch on the whole matrix).
__device__ __forceinline__ uint32_t batch_find(const uint32_t* __restrict__ begins, uint32_t count, uint32_t b)
{
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t first = 0, n = count;
    while (n > 64)
    {
        const uint32_t stride = (n + 63) / 64;
        const uint32_t idx = lane * stride;
        const uint32_t v = idx < n ? begins[first + idx] : 0xFFFFFFFFu;
        const uint32_t cell = (uint32_t) __popcll(__ballot(v <= b)) - 1u;
        first += cell * stride;
        n = min(stride, n - cell * stride);
    }
    const uint32_t v = lane < n ? begins[first + lane] : 0xFFFFFFFFu;
    return first + (uint32_t) __popcll(__ballot(v <= b)) - 1u;
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
    // 0: tiles (t), 1: columns (c), 2 / 3 / 4: 1-bit columns of 1024 / 2048 / 4096 rows (the unrolled body; c.qcol),
    // 5: columns staged in the residual's memory instead of LDS (c), 6 / 7: columns in registers, up to 3 / 6 pieces per
    // thread (r; below 32 bits)
    uint32_t kind;
    uint32_t pad;
    union // the geometry of the entry's kind
    {
        TileGeom t;
        ColGeom c;
        RegGeom r;
    };
    uint32_t reserved[6]; // (keeps the entry at the size the no-allocation call's fixed array is laid out for)
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
    else if (entries[e].kind == 5)
    {
        const ColGeom c = entries[e].c;
        quantize_colg_body<NBITS, ZT, true>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, c, index, smem_v4);
    }
    else if (NBITS < 32 && entries[e].kind >= 6)
    {
        // the column in registers: the bytes of the LDS column body, a fifth faster from 2304 rows up
        if constexpr (NBITS < 32)
        {
            const RegGeom c = entries[e].r;
            if (entries[e].kind == 6)
                quantize_reg_body<NBITS, ZT, kTileThreads, 3>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, c, index, smem_v4);
            else
                quantize_reg_body<NBITS, ZT, kTileThreads, 6>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, c, index, smem_v4);
        }
    }
    else if (NBITS != 1 || entries[e].kind == 1)
    {
        const ColGeom c = entries[e].c;
        quantize_colg_body<NBITS, ZT>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, c, index, smem_v4);
    }
    else if constexpr (NBITS == 1)
    {
        // the unrolled 1-bit column bodies: two thirds of the general body's instructions for the same bytes
        const uint64_t qcol = entries[e].c.qcol;
        if (entries[e].kind == 2)
            quantize_col_body<ZT, 1>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, qcol, index, smem_v4);
        else if (entries[e].kind == 3)
            quantize_col_body<ZT, 2>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, qcol, index, smem_v4);
        else
            quantize_col_body<ZT, 4>(entries[e].g, entries[e].r_in, entries[e].r_out, entries[e].q, qcol, index, smem_v4);
    }
}

// The owner's stripe reductions of a whole gradient set in one launch: same grid construction as quantize_batch_kernel.
struct StripeBatchEntry
{
    StripeSources src;
    float* stripe_res;
    char* q_out;
    float* agg_out;
    // 0: tiles (t), 1: columns (c), 2 / 3: 1-bit columns of 1024 / 2048 rows (the unrolled body; c.qcol),
    // 4 / 5: 1-bit columns of up to eight workers, sums looked up, up to 3 / 6 pieces per thread (r)
    uint32_t kind;
    uint32_t pad;
    TileGeom t;
    ColGeom c;
    RegGeom r;
};

// LOOKUP: the variant that also runs members of kinds 4 and 5 (76 registers instead of 44: a launch without such members
// takes the other one and keeps eight wavefronts per SIMD)
template <int NBITS, bool ZT, bool LOOKUP>
__device__ __forceinline__ void stripe_reduce_batch_body(const StripeBatchEntry* __restrict__ entries, const uint32_t* __restrict__ begins,
                                                         uint32_t count)
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
    else if (NBITS != 1 || en.kind == 1)
    {
        const ColGeom c = en.c;
        stripe_reduce_colg_body<NBITS, ZT>(en.src, en.stripe_res, en.q_out, en.agg_out, c, index, smem_v4);
    }
    else if (LOOKUP && NBITS == 1 && en.kind >= 4)
    {
        // the plain call's kernel for these stripes: the bytes of the general column body, up to twice as fast
        if constexpr (LOOKUP && NBITS == 1)
        {
            const RegGeom c = en.r;
            if (en.kind == 4)
                stripe_reduce_lut_body<ZT, 3, kTileThreads>(en.src, en.stripe_res, en.q_out, en.agg_out, c, index, smem_v4);
            else
                stripe_reduce_lut_body<ZT, 6, kTileThreads>(en.src, en.stripe_res, en.q_out, en.agg_out, c, index, smem_v4);
        }
    }
    else if constexpr (NBITS == 1)
    {
        const uint64_t qcol = en.c.qcol;
        // (workgroups with the same index modulo 8 run on one die wherever the member starts in the grid)
        const uint32_t column = column_of_workgroup(index, begins[e + 1] - begins[e]);
        // (4096 rows stay with the general body: unrolled they take 74 registers, which would cost every member of the
        // launch two of its eight wavefronts per SIMD)
        if (en.kind == 2)
            stripe_reduce_col_body<ZT, 1>(en.src, en.stripe_res, en.q_out, en.agg_out, qcol, column, smem_v4);
        else
            stripe_reduce_col_body<ZT, 2>(en.src, en.stripe_res, en.q_out, en.agg_out, qcol, column, smem_v4);
    }
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kTileThreads) CNTKQ_SGPRS_FOR_8_WAVES void stripe_reduce_batch_kernel(const StripeBatchEntry* __restrict__ entries,
                                                                                                   const uint32_t* __restrict__ begins, uint32_t count)
{
    stripe_reduce_batch_body<NBITS, ZT, false>(entries, begins, count);
}

// (six wavefronts per SIMD by its vector registers: as many scalar registers as the compiler likes)
template <bool ZT>
__global__ __launch_bounds__(kTileThreads) void stripe_reduce_batch_lookup_kernel(const StripeBatchEntry* __restrict__ entries,
                                                                                  const uint32_t* __restrict__ begins, uint32_t count)
{
    stripe_reduce_batch_body<1, ZT, true>(entries, begins, count);
}


// Many matrices in one launch (see quantize_batch_kernel): the 256-thread blocks of all matrices form one grid.
enum UnqKind : uint32_t
{
    kUnqVec4 = 0,    // QWord-major, 16-byte stores
    kUnqScalar = 1,  // QWord-major, 4-byte stores
    kUnqSegment = 2, // segment decoder
    kUnqRows = 3,    // row-major decoder, packed column in LDS
    kUnqTile = 4,    // several short columns per workgroup, packed records in LDS
    kUnqDirect = 5,  // row-major decoder, QWords fetched by the threads that decode them (geometry in rowg)
    kUnqFlat = 6     // the same for short columns: the matrix as one run of groups of consecutive elements
};

struct UnquantizeBatchEntry
{
    const char* q;
    float* out;
    uint32_t kind;
    uint32_t pad;
    UnqGeom qw;      // valid for kUnqVec4 / kUnqScalar
    UnqSegGeom seg;  // valid for kUnqSegment
    UnqRowGeom rowg; // valid for kUnqRows / kUnqDirect
    UnqTileGeom tile; // valid for kUnqTile
    UnqFlatGeom flat; // valid for kUnqFlat
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
        unquantize_tile_body<NBITS>(en.q, en.out, t, add, block, reinterpret_cast<uint32_t*>(smem_v4));
    }
}

} // namespace cntkq
