// gfx950 kernels of the per-column gradient quantizer: columns of any height cut into strips of QWords.
//
// A column of `rows` elements is packed into nq QWords, element i in QWord i % nq at bit position i / nq. A strip is a run
// of W consecutive QWords with ALL their bit positions: 32 / NBITS runs of W consecutive elements, nq elements apart. One
// 256-thread workgroup owns one strip: a thread holds four consecutive QWords' elements at up to eight bit positions (32
// values: eight 16-byte loads of gradient and residual, at any 4-byte alignment), builds its part of the four QWords and
// writes the residual back from registers; the parts of a QWord meet in LDS. Gradient and residual are read once whatever
// the height, which columns above 102400 rows -- more than any workgroup's registers hold -- could otherwise only have by
// reading their inputs two or three times. A strip needs 1 to 4 KB of LDS and, at 1 to 4 bits, some 100 registers (its 32
// values, their addresses, the masks of the ragged last strip), so five workgroups share a CU; it is the exchange
// described next, not memory, that bounds the kernel (3.3 to 4.4 TB/s), and below 102400 rows the kernels with one workgroup
// per column are faster.
//
// The column statistics span the strips of a column. Every workgroup publishes its partial sums in a scratch buffer, one
// 8-byte record per sum: the value and the tag of the launch, written by one atomic store, so that whoever reads the tag
// of this launch has the value with it and no second word needs ordering against the first. Then the first wavefront of
// every workgroup of the column polls the S records (a lane per record, with pauses) until all carry the tag, and adds them up, lanes
// meeting by butterfly -- one fixed order, the same bytes in every workgroup. One exchange for the sum of squares (more than 1 bit) or
// the split sums (1 bit against 0), two for 1 bit against the mean (mean, then split sums). The tag is a launch count
// kept in the scratch buffer itself: every workgroup reads it when it starts, and the last workgroup to finish (a second
// counter tells) raises it, so that replays of a recorded graph see fresh tags like any other launch. The strips of a
// column take workgroup indices 8 apart: the device's eight dies take the workgroups of a grid in turn, so a column's
// strips run on one die, next to each other in its queue, and start together (at most half of what the die holds: all must be resident
// at once; a column of more strips has them side by side in the grid instead, on all dies, up to half of what the device holds). That placement is what the hardware does, not what any specification promises, so the wait is bounded: after
// `spin_limit` polls a lane gives up. A workgroup that gave up raises the error word, marks its own records as abandoned
// (the launch's tag with the top bit set) and stores nothing: no header, no codes, no residual. A workgroup of the same
// column that finds an abandoned record abandons its strip in the same way, without waiting. A column whose strips did
// not all become resident in time is therefore left as it was -- with the residual updated in place, the error feedback
// of that column survives and the call can be repeated -- and the grid always drains. (What remains open is a strip that
// is resident, has published its first sum and then stalls for the whole bounded wait before its second exchange: its
// neighbours abandon the column while it may still complete its own part.) Strip 0 of an abandoned column counts the
// column in the scratch header.
#pragma once

#include "quantizer_kernels_common.h"

namespace cntkq {

constexpr uint32_t kStripThreads = 256;
constexpr uint32_t kStripDies = 8; // accelerator dies that take the workgroups of a grid in turn

template <int NBITS>
struct StripShape
{
    using PS = PackShape<NBITS>;
    static constexpr uint32_t SLOTS = PS::SLOTS;                  // bit positions per thread
    static constexpr uint32_t CHUNKS = PS::CHUNKS;                // threads per QWord quad
    static constexpr uint32_t QUADS = kStripThreads / CHUNKS;     // quads of four QWords per strip
    static constexpr uint32_t WORDS = 4 * QUADS;                  // QWords per strip: 256, 512, 1024, 1024, 1024 at 1, 2, 4, 8, 16 bits
    // wavefronts per SIMD the kernels are compiled for (the registers that leaves them: 96 at 5, 64 at 8); with more at 1 to 4
    // bits the ragged last strip spills, and every strip of its column waits for it
    static constexpr uint32_t WAVES = NBITS <= 4 ? 5 : 8;
};

// how many QWords a strip holds at this bit width (host side)
__host__ __device__ inline uint32_t strip_words(size_t nbits)
{
    return nbits == 1 ? StripShape<1>::WORDS : nbits == 2 ? StripShape<2>::WORDS : StripShape<4>::WORDS;
}

struct StripGeom
{
    uint32_t rows;
    uint32_t cols;
    uint32_t nq;
    uint32_t strips;     // workgroups per column: ceil(nq / WORDS)
    uint32_t spin_limit; // polls of a record before a lane gives up
    uint32_t poll_pause; // pauses of 64 cycles between two polls of a record
    uint32_t poll_first; // ... and before the first poll
    double inv_strips;   // for workgroup index -> (column, strip)
    uint32_t spread;     // non-zero: a column's strips take consecutive workgroup indices, i.e. all dies (columns of more strips than one die holds)
    uint32_t pad;
    uint64_t qcol;
};

// Scratch of one launch stream: a header, the finish counters, then four records per (column, strip): the statistic, then
// the two split sums and the count below the threshold. The buffer starts zeroed; tags start at 1.
//
// Reads of one address take their turns like atomic operations on it (a few nanoseconds each, but thousands of workgroups
// start within microseconds), so the launch count is kept in 256 copies, 256 bytes apart, and a wavefront reads the copy
// its index selects.
constexpr uint32_t kStripTagCopies = 256;
struct StripHeader
{
    struct
    {
        uint32_t launches; // strip launches completed on this buffer: the tag of a launch is this + 1
        uint32_t pad[63];
    } copy[kStripTagCopies];
    uint32_t finished; // groups of workgroups of the running launch that are done; back to zero when the last one is
    uint32_t pad[63];
    uint32_t abandoned; // columns left untouched because their strips gave up waiting for each other; only ever counted up
    uint32_t pad2[63];
};
constexpr uint32_t kStripAbandoned = 0x80000000u; // top bit of a record's tag: the strip's workgroup gave up; tags proper have 31 bits
constexpr uint32_t kStripRecords = 4;
constexpr uint32_t kStripFinishGroup = 64;
struct StripScratch
{
    uint32_t* error;      // pinned host memory
    StripHeader* header;
    uint32_t* groups;     // workgroups done per group of kStripFinishGroup; zero between launches
    uint64_t* records;    // [column][field][strip]: value in the low half, tag in the high half
};

// Bytes of finish counters and of records that a launch of this geometry uses. The two live in regions of the buffer
// that never move (counters must find zeros, not what another geometry's records left behind).
inline size_t strip_groups_bytes(size_t cols, size_t strips)
{
    const size_t grid = (cols + kStripDies - 1) / kStripDies * kStripDies * strips;
    return (grid + kStripFinishGroup - 1) / kStripFinishGroup * sizeof(uint32_t);
}
inline size_t strip_records_bytes(size_t cols, size_t strips)
{
    return cols * strips * kStripRecords * sizeof(uint64_t);
}

__device__ __forceinline__ void strip_publish(uint64_t* rec, uint32_t value_bits, uint32_t tag)
{
    __hip_atomic_store(rec, ((uint64_t) tag << 32) | value_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One wavefront collects the S records of a field: lane l polls records l, l + 64, ... until they carry the tag, adds
// their values in ascending order, and the lanes meet by butterfly. Every lane returns the same bits.
// Polls are loads at device scope, and a thousand resident workgroups polling as fast as they can took half of the L2's
// request rate from the loads and stores that the records wait for: a lane pauses poll_pause x 64 cycles between two polls
// (200000 x 256 at 1 bit over 1 / 16 / 64 / 128 / 256: 214 / 208 / 200 / 198 / 208 us), and first_pause x 64 cycles
// before the first one of an exchange, which with many strips per column practically never finds the record there
// (262144 x 200, 32 strips: 174 -> 154 us with 64; 24576 x 2048, 3 strips: 116 -> 132 us, so only from 16 strips on).
template <typename T>
__device__ __forceinline__ T strip_collect(const uint64_t* recs, uint32_t strips, uint32_t tag, const StripGeom& c, uint32_t first_pause, bool& gave_up)
{
    T t = 0;
    bool bad = false;
    for (uint32_t s = threadIdx.x & 63u; s < strips; s += 64)
    {
        uint32_t polls = 0;
        for (uint32_t z = 0; z < first_pause; ++z)
            __builtin_amdgcn_s_sleep(1);
        uint64_t x;
        for (;;)
        {
            x = __hip_atomic_load(recs + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t got = (uint32_t) (x >> 32);
            if (got == tag)
                break;
            // abandoned by its workgroup, or not there after the bounded wait
            if (got == (tag | kStripAbandoned) || polls >= c.spin_limit)
            {
                bad = true;
                break;
            }
            ++polls;
            for (uint32_t z = 0; z < c.poll_pause; ++z)
                __builtin_amdgcn_s_sleep(1);
        }
        T val;
        const uint32_t lo = (uint32_t) x;
        __builtin_memcpy(&val, &lo, 4);
        t += val;
    }
    gave_up = gave_up || __ballot(bad) != 0ull; // the same in every lane of the wavefront
    return wave_sum(t);
}

// The workgroup abandons its strip: every record of it says so (whichever exchange a neighbour is in, it meets the mark),
// the host learns of it through the error word, and strip 0 counts the column.
__device__ __forceinline__ void strip_abandon(uint64_t* recs, uint32_t strip, uint32_t tag, const StripGeom& c, const StripScratch& scratch)
{
    for (uint32_t f = 0; f < kStripRecords; ++f)
        strip_publish(recs + f * c.strips + strip, 0u, tag | kStripAbandoned);
    __hip_atomic_store(scratch.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (strip == 0)
        __hip_atomic_fetch_add(&scratch.header->abandoned, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A workgroup is done with the scratch buffer: the last one of the launch readies the header for the next launch. Atomic
// operations on one address take their turns (some 50 ns each), so the workgroups count in groups of 64 and only the last
// of a group counts at the header.
__device__ __forceinline__ void strip_finish(const StripScratch& sc, uint32_t tag)
{
    const uint32_t group = blockIdx.x / kStripFinishGroup, groups = (gridDim.x + kStripFinishGroup - 1) / kStripFinishGroup;
    const uint32_t members = min(kStripFinishGroup, gridDim.x - group * kStripFinishGroup);
    if (__hip_atomic_fetch_add(&sc.groups[group], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 != members)
        return;
    __hip_atomic_store(&sc.groups[group], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (__hip_atomic_fetch_add(&sc.header->finished, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 != groups)
        return;
    __hip_atomic_store(&sc.header->finished, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (uint32_t i = 0; i < kStripTagCopies; ++i)
        __hip_atomic_store(&sc.header->copy[i].launches, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum of a value over the workgroup in a fixed order (lanes by butterfly, then the four wavefronts in ascending order),
// the same bits in every thread. red: 4 slots; two barriers.
__device__ __forceinline__ float strip_block_sum(float v, float* red)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63u) == 0)
        red[threadIdx.x >> 6] = v;
    __syncthreads();
    const float t = ((red[0] + red[1]) + red[2]) + red[3];
    __syncthreads();
    return t;
}

__device__ __forceinline__ uint32_t strip_block_sum(uint32_t v, uint32_t* red)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63u) == 0)
        red[threadIdx.x >> 6] = v;
    __syncthreads();
    const uint32_t t = red[0] + red[1] + red[2] + red[3];
    __syncthreads();
    return t;
}

// The column's statistic from the strip's: every workgroup of the column publishes its own and adds all of them in the
// order of strip_collect. red: the workgroup's reduction slots. Every thread returns the same bits, in every workgroup of the column.
__device__ __forceinline__ float strip_exchange_stat(float stat, uint32_t column, uint32_t strip, uint32_t tag, const StripGeom& c,
                                                     const StripScratch& scratch, float* red, bool& ok)
{
    if (c.strips == 1)
        return stat;
    uint64_t* recs = scratch.records + (size_t) column * kStripRecords * c.strips; // [field][strip]
    if (threadIdx.x == 0)
        strip_publish(recs + strip, __float_as_uint(stat), tag);
    if (threadIdx.x < 64)
    {
        bool gave_up = false;
        const float t = strip_collect<float>(recs, c.strips, tag, c, c.poll_first, gave_up);
        if (threadIdx.x == 0)
        {
            red[0] = t;
            red[3] = gave_up ? 1.0f : 0.0f;
            if (gave_up)
                strip_abandon(recs, strip, tag, c, scratch);
        }
    }
    __syncthreads();
    const float total = red[0];
    ok = red[3] == 0.0f;
    __syncthreads();
    return total;
}

// the same for the sums on either side of the 1-bit threshold and the count below it
__device__ __forceinline__ void strip_exchange_split(float& s0, float& s1, uint32_t& n0, uint32_t column, uint32_t strip, uint32_t tag,
                                                     const StripGeom& c, const StripScratch& scratch, float* red, bool& ok)
{
    if (c.strips == 1)
        return;
    uint64_t* recs = scratch.records + (size_t) column * kStripRecords * c.strips;
    if (threadIdx.x == 0)
    {
        strip_publish(recs + 1 * c.strips + strip, __float_as_uint(s0), tag);
        strip_publish(recs + 2 * c.strips + strip, __float_as_uint(s1), tag);
        strip_publish(recs + 3 * c.strips + strip, n0, tag);
    }
    if (threadIdx.x < 64)
    {
        bool gave_up = false;
        const float t0 = strip_collect<float>(recs + 1 * c.strips, c.strips, tag, c, c.poll_first, gave_up);
        const float t1 = strip_collect<float>(recs + 2 * c.strips, c.strips, tag, c, 0u, gave_up);
        const uint32_t tn = strip_collect<uint32_t>(recs + 3 * c.strips, c.strips, tag, c, 0u, gave_up);
        if (threadIdx.x == 0)
        {
            red[0] = t0;
            red[1] = t1;
            red[2] = __uint_as_float(tn);
            red[3] = gave_up ? 1.0f : 0.0f;
            if (gave_up)
                strip_abandon(recs, strip, tag, c, scratch);
        }
    }
    __syncthreads();
    s0 = red[0];
    s1 = red[1];
    n0 = __float_as_uint(red[2]);
    ok = red[3] == 0.0f;
    __syncthreads();
}

// From the strip's sums to the column's header: the exchanges, the header (written by strip 0) and the release of the
// scratch buffer. `sums(mean, s0, s1, n0)` gives the strip's split sums (1 bit only), in the same bits in every thread.
// False (in every thread of the workgroup alike): the column was abandoned and nothing of it may be stored.
template <int NBITS, bool ZT, typename SplitSums>
__device__ __forceinline__ bool strip_column_range(float stat, SplitSums sums, uint32_t column, uint32_t strip, uint32_t tag, const StripGeom& c,
                                                   const StripScratch& scratch, float* red, char* qc, float& lo, float& hi)
{
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    float total = 0.0f;
    bool ok = true;
    if constexpr (need_stat)
        total = strip_exchange_stat(stat, column, strip, tag, c, scratch, red, ok);
    if constexpr (NBITS == 1)
    {
        // (an abandoned strip takes no part in the second exchange: its records already say so)
        if (ok)
        {
            const float mean = ZT ? 0.0f : total / (float) c.rows;
            float s0, s1;
            uint32_t n0;
            sums(mean, s0, s1, n0);
            strip_exchange_split(s0, s1, n0, column, strip, tag, c, scratch, red, ok);
            finish_stats_1bit<ZT>(mean, s0, s1, n0, c.rows - n0, c.rows, lo, hi);
        }
    }
    else
        finish_stats_multibit(total, c.rows, lo, hi);
    if (c.strips > 1 && threadIdx.x == 0)
        strip_finish(scratch, tag);
    if (ok && strip == 0 && threadIdx.x == 0)
    {
        float* gh = reinterpret_cast<float*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    return ok;
}

// A strip with its values in registers: v[kk] = the four values of QWords w ... w + 3 at bit position k0 + kk. FULL: every
// QWord of the strip exists and has an element at every bit position; otherwise `valid` has bit 4 * kk + e set for the
// values that exist, and the others are zero (which no sum notices; the count below the threshold is corrected, the codes
// are masked and nothing is stored for them). Statistics across the strips of the column,
// header, codes, residual and packed QWords. smem: 8 reduction slots, then WORDS partial QWords when a QWord has several
// threads. Used by the quantize and the stripe-reduction kernel, which therefore give the same bytes for the same column.
template <int NBITS, bool ZT, bool FULL>
__device__ __forceinline__ void strip_stats_pack(f32x4 (&v)[StripShape<NBITS>::SLOTS], uint32_t valid, uint32_t w, uint32_t k0, uint32_t column,
                                                 uint32_t strip, uint32_t tag, const StripGeom& c, const StripScratch& scratch, float* smem,
                                                 float* res_col, char* qc)
{
    using SS = StripShape<NBITS>;
    using PS = PackShape<NBITS>;
    const uint32_t tid = threadIdx.x;
    float* red = smem;
    uint32_t* red_u = reinterpret_cast<uint32_t*>(smem + 4);
    uint32_t* words = reinterpret_cast<uint32_t*>(smem + 8);
    if constexpr (SS::CHUNKS > 1)
    {
        for (uint32_t x = tid; x < SS::WORDS; x += kStripThreads)
            words[x] = 0u;
    }
    float stat = 0.0f;
    if constexpr ((NBITS != 1) || !ZT)
    {
#pragma unroll
        for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
            for (uint32_t e = 0; e < 4; ++e)
            {
                const float x = v[kk][e];
                stat += NBITS == 1 ? x : x * x;
            }
        stat = strip_block_sum(stat, red);
    }
    float lo = 0.0f, hi = 0.0f;
    const bool column_ok = strip_column_range<NBITS, ZT>(
        stat,
        [&](float mean, float& s0, float& s1, uint32_t& n0) {
            s0 = 0.0f, s1 = 0.0f, n0 = 0;
#pragma unroll
            for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
                for (uint32_t e = 0; e < 4; ++e)
                {
                    const float x = v[kk][e];
                    const bool below = x < mean;
                    s0 += below ? x : 0.0f;
                    s1 += below ? 0.0f : x;
                    n0 += below ? 1u : 0u;
                }
            if constexpr (!FULL)
                n0 -= 0.0f < mean ? (uint32_t) __popc(~valid) : 0u; // the zeros that stand in for elements that do not exist
            s0 = strip_block_sum(s0, red);
            s1 = strip_block_sum(s1, red);
            n0 = strip_block_sum(n0, red_u);
        },
        column, strip, tag, c, scratch, red, qc, lo, hi);
    if (!column_ok)
        return; // abandoned column: codes and residual stay as they were
    const ValueQ vq = make_vq<NBITS>(lo, hi);
    const float val0 = unquantize_value<NBITS>(vq, 0u);
    const float val1 = unquantize_value<NBITS>(vq, 1u);
    uint32_t word[4] = {0u, 0u, 0u, 0u};
    float* res = res_col + (size_t) k0 * c.nq; // k0 is the same in a wavefront: a scalar base, one offset per lane
#pragma unroll
    for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
    {
        f32x4 r;
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e)
        {
            const float x = v[kk][e];
            uint32_t code = quantize_value<NBITS, ZT>(vq, x);
            float back;
            if constexpr (NBITS == 1)
                back = code ? val1 : val0;
            else
                back = unquantize_value<NBITS>(vq, code);
            r[e] = x - back;
            if constexpr (!FULL)
                code &= 0u - ((valid >> (4 * kk + e)) & 1u);
            word[e] |= code << ((k0 + kk) * PS::SHIFT);
        }
        float* dst = res + (size_t) kk * c.nq + w;
        const uint32_t ok = FULL ? 15u : (valid >> (4 * kk)) & 15u;
        if (ok == 15u)
            __builtin_nontemporal_store(r, reinterpret_cast<f32x4_u*>(dst));
        else if (ok != 0u)
        {
#pragma unroll
            for (uint32_t e = 0; e < 4; ++e)
                if ((ok >> e) & 1u)
                    dst[e] = r[e];
        }
    }
    uint32_t* bits = reinterpret_cast<uint32_t*>(qc + 8);
    if constexpr (SS::CHUNKS == 1)
    {
        if (FULL || w + 4 <= c.nq)
            *reinterpret_cast<u32x4_u*>(bits + w) = u32x4{word[0], word[1], word[2], word[3]};
        else
        {
#pragma unroll
            for (uint32_t e = 0; e < 4; ++e)
                if (w + e < c.nq)
                    bits[w + e] = word[e];
        }
    }
    else
    {
        const uint32_t local = w - strip * SS::WORDS;
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e)
            atomicOr(&words[local + e], word[e]);
        __syncthreads();
        for (uint32_t x = tid; x < SS::WORDS; x += kStripThreads)
            if (FULL || strip * SS::WORDS + x < c.nq)
                bits[strip * SS::WORDS + x] = words[x];
    }
}

__host__ __device__ inline size_t strip_lds_bytes(size_t nbits)
{
    return (8 + (nbits <= 2 ? (size_t) strip_words(nbits) : 0)) * 4;
}

// whether every QWord of the strip exists and has an element at every bit position (only the last bit position can be
// short of elements, and only in the last QWords of the column)
template <int NBITS>
__device__ __forceinline__ bool strip_is_full(const StripGeom& c, uint32_t strip)
{
    const uint32_t end = (strip + 1) * StripShape<NBITS>::WORDS;
    return end <= c.nq && (uint64_t) (PackShape<NBITS>::VPW - 1) * c.nq + end <= c.rows;
}

// which QWords and bit positions a thread holds of a full strip: four QWords from w, SLOTS bit positions from k0 (the
// same in a wavefront, so returned as a scalar)
template <int NBITS>
__device__ __forceinline__ void strip_thread_slots(uint32_t strip, uint32_t& w, uint32_t& k0)
{
    using SS = StripShape<NBITS>;
    static_assert(SS::QUADS % kWave == 0, "a wavefront holds one range of bit positions");
    w = strip * SS::WORDS + 4 * (threadIdx.x % SS::QUADS);
    k0 = __builtin_amdgcn_readfirstlane(threadIdx.x / SS::QUADS) * SS::SLOTS;
}

// Workgroups go to the eight dies of the device in turn, each die starting its share in order. The strips of a column
// take indices 8 apart, so they land on one die, one after the other in its queue, and start together. Returns the tag of
// the launch, or false for a workgroup beyond the last column (the grid is rounded up to eight columns).
__device__ __forceinline__ bool strip_assignment(const StripGeom& c, const StripScratch& scratch, uint32_t& column, uint32_t& strip, uint32_t& tag)
{
    if (c.spread)
    {
        // a column of more strips than one die holds: its strips side by side in the grid, on all dies, which start them in
        // order like everything else (the partial sums then meet in memory instead of one die's L2)
        divmod_u32(blockIdx.x, c.strips, c.inv_strips, column, strip);
    }
    else
    {
        divmod_u32(blockIdx.x / kStripDies, c.strips, c.inv_strips, column, strip);
        column = column * kStripDies + blockIdx.x % kStripDies;
    }
    strip = c.strips - 1 - strip; // the strip at the ragged end of the column, which takes longest, starts first
    // the same tag in every workgroup: the count moves when all of them are done
    const uint32_t copy = (blockIdx.x * (kStripThreads / kWave) + threadIdx.x / kWave) % kStripTagCopies;
    tag = c.strips > 1 ? (__hip_atomic_load(&scratch.header->copy[copy].launches, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) % 0x7FFFFFFFu) + 1u : 0u;
    if (column < c.cols)
        return true;
    if (c.strips > 1 && threadIdx.x == 0)
        strip_finish(scratch, tag);
    return false;
}

// which of a thread's 4 * SLOTS values exist in a strip at the ragged end of its column
template <int NBITS>
__device__ __forceinline__ uint32_t strip_valid_mask(const StripGeom& c, uint32_t w, uint32_t k0)
{
    using SS = StripShape<NBITS>;
    uint32_t valid = ~(uint32_t) ((1ull << (4 * SS::SLOTS)) - 1ull); // bits beyond the thread's values count as present
#pragma unroll
    for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e)
        {
            const uint64_t i = (uint64_t) (w + e) + (uint64_t) (k0 + kk) * c.nq;
            valid |= (w + e < c.nq && i < c.rows) ? (1u << (4 * kk + e)) : 0u;
        }
    return valid;
}

// Four consecutive values of a column from element i on, at any 4-byte alignment. FULL: all exist. Otherwise bit e of `ok`
// says whether value e does, the others read as zero; the 16-byte load never leaves the column (it moves back to the
// column's last four elements when it would), and the few lanes with some but not all of their values fetch them one by one.
template <bool FULL>
__device__ __forceinline__ f32x4 strip_load4(const float* col, uint32_t i, uint32_t rows, uint32_t ok)
{
    if constexpr (FULL)
        return __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(col + i));
    else
    {
        const uint32_t at = (rows >= 4 && i + 4 > rows) ? rows - 4 : i;
        f32x4 x = {0.0f, 0.0f, 0.0f, 0.0f};
        if (rows >= 4)
            x = __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(col + at));
        if (ok != 15u)
        {
#pragma unroll
            for (uint32_t e = 0; e < 4; ++e)
                x[e] = ((ok >> e) & 1u) ? col[i + e] : 0.0f;
        }
        return x;
    }
}

// The gradient goes straight into the registers that will hold the sums, the residual joins it four loads at a time. Every
// value of the strip is in registers before anything is stored, so r_out may be r_in.
template <int NBITS, bool ZT, bool FULL>
__device__ __forceinline__ void quantize_strip_body(const float* g_col, const float* r_col, float* res_col, char* qc, uint32_t column, uint32_t strip,
                                                    uint32_t tag, const StripGeom& c, const StripScratch& scratch, float* smem)
{
    using SS = StripShape<NBITS>;
    uint32_t w, k0;
    strip_thread_slots<NBITS>(strip, w, k0);
    const uint32_t valid = FULL ? 0xFFFFFFFFu : strip_valid_mask<NBITS>(c, w, k0);
    const uint32_t i0 = k0 * c.nq + w;
    f32x4 v[SS::SLOTS];
#pragma unroll
    for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
        v[kk] = strip_load4<FULL>(g_col, i0 + kk * c.nq, c.rows, (valid >> (4 * kk)) & 15u);
    constexpr uint32_t BATCH = SS::SLOTS < 4 ? SS::SLOTS : 4;
#pragma unroll
    for (uint32_t k1 = 0; k1 < SS::SLOTS; k1 += BATCH)
    {
        f32x4 b[BATCH];
#pragma unroll
        for (uint32_t kk = 0; kk < BATCH; ++kk)
            b[kk] = strip_load4<FULL>(r_col, i0 + (k1 + kk) * c.nq, c.rows, (valid >> (4 * (k1 + kk))) & 15u);
#pragma unroll
        for (uint32_t kk = 0; kk < BATCH; ++kk)
            v[k1 + kk] = v[k1 + kk] + b[kk];
    }
    strip_stats_pack<NBITS, ZT, FULL>(v, valid, w, k0, column, strip, tag, c, scratch, smem, res_col, qc);
}

template <int NBITS, bool ZT>
__global__ __launch_bounds__(kStripThreads, StripShape<NBITS>::WAVES) void quantize_strip_kernel(const float* __restrict__ g, const float* r_in,
                                                                                                 float* r_out, char* __restrict__ q, StripGeom c,
                                                                                                 StripScratch scratch)
{
    static_assert(NBITS < 32, "32-bit codes are whole QWords: nothing to assemble");
    extern __shared__ f32x4 smem_v4[];
    float* smem = reinterpret_cast<float*>(smem_v4);
    uint32_t column, strip, tag;
    if (!strip_assignment(c, scratch, column, strip, tag))
        return;
    const size_t base = (size_t) column * c.rows;
    char* qc = q + (size_t) column * c.qcol;
    if (strip_is_full<NBITS>(c, strip))
        quantize_strip_body<NBITS, ZT, true>(g + base, r_in + base, r_out + base, qc, column, strip, tag, c, scratch, smem);
    else
        quantize_strip_body<NBITS, ZT, false>(g + base, r_in + base, r_out + base, qc, column, strip, tag, c, scratch, smem);
}

} // namespace cntkq
