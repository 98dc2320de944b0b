// gfx950 kernels of the per-column gradient quantizer: columns of any height cut into strips of QWords.
//
// A column of `rows` elements is packed into nq QWords, element i in QWord i % nq at bit position i / nq. A strip is a
// run of W consecutive QWords with ALL their bit positions: 32 / NBITS runs of W consecutive elements, nq elements
// apart. One 512-thread workgroup owns one strip: a thread holds the elements of 16 bytes' worth of consecutive QWords
// (four of a float column, two of a double column) at up to eight bit positions (eight 16-byte loads of gradient and
// residual, at any alignment the element type allows), builds its part of those QWords and writes the residual back
// from registers; the parts of a QWord meet in LDS. The kernels are written once over the element type. Gradient and
// residual are read once whatever the height, which columns above 102400 rows -- more than any workgroup's registers
// hold -- could otherwise only have by reading their inputs two or three times. A strip needs 2 to 8 KB of LDS and, at
// 1 to 4 bits, some 100 registers (its 32 values, their addresses, the masks of the ragged last strip), so two
// workgroups share a CU; it is the exchange described next, not memory, that bounds the kernel (4.0 to 5.0 TB/s), and
// below 102400 rows the kernels with one workgroup per column are faster. (Strips of 256 threads, five to a CU, were 7
// to 25 % slower, strips of 1024 threads about as fast as these at a few shapes and slower at most: the fewer
// workgroups a column's sums must cross, the better, until too few bytes are in flight.)
//
// The column statistics span the strips of a column. Every workgroup publishes its partial sums in a scratch buffer,
// one 8-byte record per 32 bits of a sum (a double takes two): the bits and the tag of the launch, written by one
// atomic store, so that whoever reads the tag of this launch has the bits with it and no second word needs ordering
// against the first. Then the first wavefront of every workgroup of the column polls the S records (a lane per record,
// with pauses) until all carry the tag, and adds them up, lanes meeting by butterfly -- one fixed order, the same bytes
// in every workgroup. One exchange for the sum of squares (more than 1 bit) or the split sums (1 bit against 0), two
// for 1 bit against the mean (mean, then split sums). The tag is a launch count kept in the scratch buffer itself:
// every workgroup reads it when it starts, and the last workgroup to finish (a second counter tells) raises it, so that
// replays of a recorded graph see fresh tags like any other launch. The strips of a column take workgroup indices 8
// apart: the device's eight dies take the workgroups of a grid in turn, so a column's strips run on one die, next to
// each other in its queue, and start together (at most half of what the die holds: all must be resident at once; a
// column of more strips has them side by side in the grid instead, on all dies, up to half of what the device holds).
// That placement is what the hardware does, not what any specification promises, so the wait is bounded: after
// `spin_limit` polls a lane gives up. A workgroup that gave up raises the error word, marks its own records as
// abandoned (the launch's tag with the top bit set) and stores nothing: no header, no codes, no residual. A workgroup
// of the same column that finds an abandoned record abandons its strip in the same way, without waiting. A column whose
// strips did not all become resident in time is therefore left as it was -- with the residual updated in place, the
// error feedback of that column survives and the call can be repeated -- and the grid always drains. (What remains open
// is a strip that is resident, has published its first sum and then stalls for the whole bounded wait before its second
// exchange: its neighbours abandon the column while it may still complete its own part.) Strip 0 of an abandoned column
// counts the column in the scratch header.
#pragma once

#include <type_traits>

#include "quantizer_kernels_tile.h" // StripeSources, stripe_order

namespace cntkq {

constexpr uint32_t kStripThreads = 512;
constexpr uint32_t kStripWaves = kStripThreads / 64;
constexpr uint32_t kStripDies = 8; // accelerator dies that take the workgroups of a grid in turn

typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
typedef u64x2 u64x2_u __attribute__((aligned(8)));

// The 16-byte accesses of either element type: PER consecutive elements, or QWords, at the alignment of one.
template <typename E>
struct StripElem;
template <>
struct StripElem<float>
{
    typedef f32x4 V;
    typedef f32x4_u VU;
    typedef u32x4 QV;
    typedef u32x4_u QVU;
    static constexpr uint32_t PER = 4;
    static __device__ __forceinline__ QV words(const uint32_t* w) { return QV{w[0], w[1], w[2], w[3]}; }
};
template <>
struct StripElem<double>
{
    typedef f64x2 V;
    typedef f64x2_u VU;
    typedef u64x2 QV;
    typedef u64x2_u QVU;
    static constexpr uint32_t PER = 2;
    static __device__ __forceinline__ QV words(const uint64_t* w) { return QV{w[0], w[1]}; }
};

template <typename E>
using StripVec = typename StripElem<E>::V;

template <int NBITS, typename E>
struct StripShape
{
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    static constexpr uint32_t PER = StripElem<E>::PER;            // consecutive QWords per thread
    static constexpr uint32_t SLOTS = PS::SLOTS;                  // bit positions per thread
    static constexpr uint32_t CHUNKS = PS::CHUNKS;                // threads per run of PER QWords
    static constexpr uint32_t RUNS = kStripThreads / CHUNKS;      // runs of PER QWords per strip
    // QWords per strip: float 512, 1024, 2048, 2048, 2048 at 1, 2, 4, 8, 16 bits; double 128, 256, 512, 1024, 1024, 1024 at 1 ... 32 bits
    static constexpr uint32_t WORDS = PER * RUNS;
    // wavefronts per SIMD the kernels are compiled for (the registers that leaves them: 128 at 4, 64 at 8): two workgroups of
    // eight wavefronts are what a compute unit holds where a thread has eight bit positions, and with fewer registers the
    // ragged last strip spills, and every strip of its column waits for it
    static constexpr uint32_t WAVES = SLOTS == 8 ? 4 : 8;
};

// how many QWords a strip holds at this bit width (host side; the same arithmetic as StripShape)
template <typename E>
__host__ __device__ inline uint32_t strip_words(size_t nbits)
{
    const uint32_t vpw = (uint32_t) (Word<E>::kBits / nbits);
    const uint32_t slots = vpw < 8 ? vpw : 8;
    return (uint32_t) (16 / sizeof(E)) * (kStripThreads / (vpw / slots));
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
    uint32_t whole_positions; // rows / nq: bit positions at which every QWord of a column has an element
    uint32_t last_words;      // rows % nq: QWords with an element at bit position whole_positions (none beyond it)
    uint32_t pad;
    uint64_t qcol;
};

// Scratch of one launch stream: a header, the finish counters, then the records of every (column, strip): the statistic,
// then the two split sums (each one record for floats, two for doubles) and the count below the threshold. The buffer
// starts zeroed; tags start at 1.
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
// records per (column, strip): three sums of the element type and a count (doubles: one record stays unused)
template <typename E>
constexpr uint32_t strip_records()
{
    return 4u * (uint32_t) (sizeof(E) / 4);
}
constexpr uint32_t kStripFinishGroup = 64;
struct StripScratch
{
    uint32_t* error;      // pinned host memory
    StripHeader* header;
    uint32_t* groups;     // workgroups done per group of kStripFinishGroup; zero between launches
    uint64_t* records;    // [column][record][strip]: 32 bits of a value in the low half, tag in the high half
};

// Bytes of finish counters and of records that a launch of this geometry uses. The two live in regions of the buffer
// that never move (counters must find zeros, not what another geometry's records left behind).
inline size_t strip_groups_bytes(size_t cols, size_t strips)
{
    const size_t grid = (cols + kStripDies - 1) / kStripDies * kStripDies * strips;
    return (grid + kStripFinishGroup - 1) / kStripFinishGroup * sizeof(uint32_t);
}
inline size_t strip_records_bytes(size_t cols, size_t strips, size_t records_each)
{
    return cols * strips * records_each * sizeof(uint64_t);
}

__device__ __forceinline__ void strip_publish(uint64_t* rec, uint32_t value_bits, uint32_t tag)
{
    __hip_atomic_store(rec, ((uint64_t) tag << 32) | value_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// a value of 4 or 8 bytes: records `rec`, and `rec + strips` for the upper half
template <typename T>
__device__ __forceinline__ void strip_publish_value(uint64_t* rec, uint32_t strips, T value, uint32_t tag)
{
    uint32_t w[sizeof(T) / 4];
    __builtin_memcpy(w, &value, sizeof(T));
#pragma unroll
    for (uint32_t h = 0; h < sizeof(T) / 4; ++h)
        strip_publish(rec + h * strips, w[h], tag);
}

// Waits for one record to carry the tag and returns its 32 bits. `bad`: its workgroup abandoned it, or it was not there
// after the bounded wait.
__device__ __forceinline__ uint32_t strip_poll(const uint64_t* rec, uint32_t tag, const StripGeom& c, bool& bad)
{
    uint32_t polls = 0;
    uint64_t x;
    for (;;)
    {
        x = __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t got = (uint32_t) (x >> 32);
        if (got == tag)
            break;
        if (got == (tag | kStripAbandoned) || polls >= c.spin_limit)
        {
            bad = true;
            break;
        }
        ++polls;
        for (uint32_t z = 0; z < c.poll_pause; ++z)
            __builtin_amdgcn_s_sleep(1);
    }
    return (uint32_t) x;
}

// One wavefront collects the S values of a sum: lane l polls the records of strips l, l + 64, ... until they carry the tag,
// adds their values in ascending order, and the lanes meet by butterfly. Every lane returns the same bits.
// Polls are loads at device scope, and a thousand resident workgroups polling as fast as they can took half of the L2's
// request rate from the loads and stores that the records wait for: a lane pauses poll_pause x 64 cycles between two polls
// (200000 x 256 at 1 bit over 1 / 16 / 64 / 128 / 256: 214 / 208 / 200 / 198 / 208 us), and first_pause x 64 cycles
// before the first one of an exchange, which with many strips per column practically never finds the record there
// (with strips of 256 threads: 262144 x 200, 32 strips: 174 -> 154 us with 64; 24576 x 2048, 3 strips: 116 -> 132 us; with
// strips of 512 threads: 204800 x 256, 13 strips: 140 -> 135 us; 102401 x 512, 7 strips: 173 -> 175 us: from 8 strips on).
template <typename T>
__device__ __forceinline__ T strip_collect(const uint64_t* recs, uint32_t strips, uint32_t tag, const StripGeom& c, uint32_t first_pause, bool& gave_up)
{
    T t = 0;
    bool bad = false;
    for (uint32_t s = threadIdx.x & 63u; s < strips; s += 64)
    {
        for (uint32_t z = 0; z < first_pause; ++z)
            __builtin_amdgcn_s_sleep(1);
        uint32_t w[sizeof(T) / 4];
#pragma unroll
        for (uint32_t h = 0; h < sizeof(T) / 4; ++h)
            w[h] = bad ? 0u : strip_poll(recs + h * strips + s, tag, c, bad);
        T val;
        __builtin_memcpy(&val, w, sizeof(T));
        t += val;
    }
    gave_up = gave_up || __ballot(bad) != 0ull; // the same in every lane of the wavefront
    return wave_sum(t);
}

// The workgroup abandons its strip: every record of it says so (whichever exchange a neighbour is in, it meets the mark),
// the host learns of it through the error word, and strip 0 counts the column.
__device__ __forceinline__ void strip_abandon(uint64_t* recs, uint32_t records_each, uint32_t strip, uint32_t tag, const StripGeom& c,
                                              const StripScratch& scratch)
{
    for (uint32_t f = 0; f < records_each; ++f)
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
template <typename T>
__device__ __forceinline__ T strip_block_sum(T v, T* red)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63u) == 0)
        red[threadIdx.x >> 6] = v;
    __syncthreads();
    T t = red[0];
#pragma unroll
    for (uint32_t i = 1; i < kStripWaves; ++i)
        t = t + red[i];
    __syncthreads();
    return t;
}

// The column's statistic from the strip's: every workgroup of the column publishes its own and adds all of them in the
// order of strip_collect. red, red_u: the workgroup's reduction slots (four each). Every thread returns the same bits, in
// every workgroup of the column.
//
// PASS: 0 = one kernel does everything and its workgroups wait for each other. Otherwise the work is cut where they would
// wait, into kernels that run one after the other on a stream (kStripPassStat: publish the statistic and stop;
// kStripPassSplit: collect the statistics, publish the split sums and stop; kStripPassPack: collect and go on), each
// loading the strip's values anew: nothing waits, so no workgroup need be resident beside another, and the sums are the
// same bits as the single kernel's.
constexpr int kStripPassStat = 1, kStripPassSplit = 2, kStripPassPack = 3;

template <int PASS, typename E>
__device__ __forceinline__ E strip_exchange_stat(E stat, uint32_t column, uint32_t strip, uint32_t tag, const StripGeom& c,
                                                 const StripScratch& scratch, E* red, uint32_t* red_u, bool& ok)
{
    if (PASS == 0 && c.strips == 1)
        return stat;
    constexpr uint32_t H = sizeof(E) / 4; // records per sum
    uint64_t* recs = scratch.records + (size_t) column * strip_records<E>() * c.strips; // [record][strip]
    if (threadIdx.x == 0 && PASS <= kStripPassStat)
        strip_publish_value(recs + strip, c.strips, stat, tag);
    if constexpr (PASS == kStripPassStat)
        return stat;
    if (threadIdx.x < 64)
    {
        bool gave_up = false;
        const E t = strip_collect<E>(recs, c.strips, tag, c, c.poll_first, gave_up);
        if (threadIdx.x == 0)
        {
            red[0] = t;
            red_u[3] = gave_up ? 1u : 0u;
            if (gave_up)
                strip_abandon(recs, H * 4, strip, tag, c, scratch);
        }
    }
    __syncthreads();
    const E total = red[0];
    ok = red_u[3] == 0u;
    __syncthreads();
    return total;
}

// the same for the sums on either side of the 1-bit threshold and the count below it
template <int PASS, typename E>
__device__ __forceinline__ void strip_exchange_split(E& s0, E& s1, uint32_t& n0, uint32_t column, uint32_t strip, uint32_t tag,
                                                     const StripGeom& c, const StripScratch& scratch, E* red, uint32_t* red_u, bool& ok)
{
    if (PASS == 0 && c.strips == 1)
        return;
    constexpr uint32_t H = sizeof(E) / 4;
    uint64_t* recs = scratch.records + (size_t) column * strip_records<E>() * c.strips;
    if (threadIdx.x == 0 && PASS != kStripPassPack)
    {
        strip_publish_value(recs + 1 * H * c.strips + strip, c.strips, s0, tag);
        strip_publish_value(recs + 2 * H * c.strips + strip, c.strips, s1, tag);
        strip_publish_value(recs + 3 * H * c.strips + strip, c.strips, n0, tag);
    }
    if constexpr (PASS == kStripPassSplit)
        return;
    if (threadIdx.x < 64)
    {
        bool gave_up = false;
        const E t0 = strip_collect<E>(recs + 1 * H * c.strips, c.strips, tag, c, c.poll_first, gave_up);
        const E t1 = strip_collect<E>(recs + 2 * H * c.strips, c.strips, tag, c, 0u, gave_up);
        const uint32_t tn = strip_collect<uint32_t>(recs + 3 * H * c.strips, c.strips, tag, c, 0u, gave_up);
        if (threadIdx.x == 0)
        {
            red[0] = t0;
            red[1] = t1;
            red_u[2] = tn;
            red_u[3] = gave_up ? 1u : 0u;
            if (gave_up)
                strip_abandon(recs, H * 4, strip, tag, c, scratch);
        }
    }
    __syncthreads();
    s0 = red[0];
    s1 = red[1];
    n0 = red_u[2];
    ok = red_u[3] == 0u;
    __syncthreads();
}

// From the strip's sums to the column's header: the exchanges, the header (written by strip 0) and the release of the
// scratch buffer. `sums(mean, s0, s1, n0)` gives the strip's split sums (1 bit only), in the same bits in every thread.
// False (in every thread of the workgroup alike): nothing of the column may be stored, because it was abandoned or because
// this pass ends with its sums.
template <int NBITS, bool ZT, int PASS, typename E, typename SplitSums>
__device__ __forceinline__ bool strip_column_range(E stat, SplitSums sums, uint32_t column, uint32_t strip, uint32_t tag, const StripGeom& c,
                                                   const StripScratch& scratch, E* red, uint32_t* red_u, char* qc, E& lo, E& hi)
{
    constexpr bool need_stat = (NBITS != 1) || !ZT;
    static_assert(PASS != kStripPassStat || need_stat, "no statistic before the split sums against zero");
    static_assert(PASS != kStripPassSplit || NBITS == 1, "split sums at 1 bit only");
    E total = 0;
    bool ok = true;
    if constexpr (need_stat)
        total = strip_exchange_stat<PASS>(stat, column, strip, tag, c, scratch, red, red_u, ok);
    if constexpr (PASS == kStripPassStat)
        return false;
    if constexpr (NBITS == 1)
    {
        // (an abandoned strip takes no part in the second exchange: its records already say so)
        if (ok)
        {
            const E mean = ZT ? (E) 0 : total / (E) c.rows;
            E s0 = 0, s1 = 0;
            uint32_t n0 = 0;
            if constexpr (PASS != kStripPassPack)
                sums(mean, s0, s1, n0);
            strip_exchange_split<PASS>(s0, s1, n0, column, strip, tag, c, scratch, red, red_u, ok);
            if constexpr (PASS == kStripPassSplit)
                return false;
            finish_stats_1bit<ZT>(mean, s0, s1, n0, c.rows - n0, c.rows, lo, hi);
        }
        else if (PASS == kStripPassSplit)
            return false;
    }
    else
        finish_stats_multibit(total, c.rows, lo, hi);
    if ((PASS != 0 || c.strips > 1) && threadIdx.x == 0)
        strip_finish(scratch, tag);
    if (ok && strip == 0 && threadIdx.x == 0)
    {
        E* gh = reinterpret_cast<E*>(qc);
        gh[0] = lo;
        gh[1] = hi;
    }
    return ok;
}

// A strip with its values in registers: v[kk] (kk below SLOTS) = the PER values of QWords w ... w + PER - 1 at bit position k0 + kk. FULL:
// every QWord of the strip exists and has an element at every bit position; otherwise `valid` has bit PER * kk + e set for
// the values that exist, and the others are zero (which no sum notices; the count below the threshold is corrected, the
// codes are masked and nothing is stored for them). Statistics across the strips of the column, header, codes, residual
// and packed QWords. smem: four reduction slots of the element type, four of 32 bits, then WORDS partial QWords when a QWord
// has several threads. Used by the quantize and the stripe-reduction kernel, which therefore give the same bytes for the
// same column.
template <typename E>
constexpr uint32_t kStripRedBytes = kStripWaves * sizeof(E) + 4 * kStripWaves;

template <int NBITS, bool ZT, bool FULL, typename E, int PASS = 0>
__device__ __forceinline__ void strip_stats_pack(StripVec<E>* v, uint32_t valid, uint32_t w, uint32_t k0,
                                                 uint32_t column, uint32_t strip, uint32_t tag, const StripGeom& c, const StripScratch& scratch,
                                                 char* smem, E* res_col, char* qc)
{
    using SS = StripShape<NBITS, E>;
    using PS = typename SS::PS;
    using SE = StripElem<E>;
    using Q = typename Word<E>::Q;
    constexpr uint32_t PER = SS::PER;
    const uint32_t tid = threadIdx.x;
    E* red = reinterpret_cast<E*>(smem);
    uint32_t* red_u = reinterpret_cast<uint32_t*>(smem + kStripWaves * sizeof(E));
    Q* words = reinterpret_cast<Q*>(smem + kStripRedBytes<E>);
    if constexpr (SS::CHUNKS > 1)
    {
        for (uint32_t x = tid; x < SS::WORDS; x += kStripThreads)
            words[x] = 0u;
    }
    E stat = 0;
    if constexpr (((NBITS != 1) || !ZT) && PASS <= kStripPassStat)
    {
#pragma unroll
        for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e)
            {
                const E x = v[kk][e];
                stat += NBITS == 1 ? x : x * x;
            }
        stat = strip_block_sum(stat, red);
    }
    E lo = 0, hi = 0;
    const bool column_ok = strip_column_range<NBITS, ZT, PASS, E>(
        stat,
        [&](E mean, E& s0, E& s1, uint32_t& n0) {
            s0 = 0, s1 = 0, n0 = 0;
#pragma unroll
            for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                {
                    const E x = v[kk][e];
                    const bool below = x < mean;
                    s0 += below ? x : (E) 0;
                    s1 += below ? (E) 0 : x;
                    n0 += below ? 1u : 0u;
                }
            if constexpr (!FULL)
                n0 -= (E) 0 < mean ? (uint32_t) __popc(~valid) : 0u; // the zeros that stand in for elements that do not exist
            s0 = strip_block_sum(s0, red);
            s1 = strip_block_sum(s1, red);
            n0 = strip_block_sum(n0, red_u);
        },
        column, strip, tag, c, scratch, red, red_u, qc, lo, hi);
    if (!column_ok)
        return; // abandoned column: codes and residual stay as they were (or a pass that ends with its sums)
    const ValueQOf<E> vq = make_vq<NBITS, E>(lo, hi);
    const E val0 = unquantize_value<NBITS, E>(vq, (Q) 0);
    const E val1 = unquantize_value<NBITS, E>(vq, (Q) 1);
    Q word[PER];
#pragma unroll
    for (uint32_t e = 0; e < PER; ++e)
        word[e] = 0;
    E* res = res_col + (size_t) k0 * c.nq; // (where k0 is the same in a wavefront: a scalar base, one offset per lane)
#pragma unroll
    for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
    {
        typename SE::V r;
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e)
        {
            const E x = v[kk][e];
            Q code = quantize_value<NBITS, ZT, E>(vq, x);
            E back;
            if constexpr (NBITS == 1)
                back = code ? val1 : val0;
            else
                back = unquantize_value<NBITS, E>(vq, code);
            r[e] = x - back;
            if constexpr (!FULL)
                code &= (Q) 0 - (Q) ((valid >> (PER * kk + e)) & 1u);
            word[e] |= code << ((k0 + kk) * PS::SHIFT);
        }
        E* dst = res + (size_t) kk * c.nq + w;
        constexpr uint32_t ALL = (1u << PER) - 1u;
        const uint32_t ok = FULL ? ALL : (valid >> (PER * kk)) & ALL;
        if (ok == ALL)
            __builtin_nontemporal_store(r, reinterpret_cast<typename SE::VU*>(dst));
        else if (ok != 0u)
        {
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e)
                if ((ok >> e) & 1u)
                    dst[e] = r[e];
        }
    }
    Q* bits = reinterpret_cast<Q*>(qc + 2 * sizeof(E));
    if constexpr (SS::CHUNKS == 1)
    {
        if (FULL || w + PER <= c.nq)
            *reinterpret_cast<typename SE::QVU*>(bits + w) = SE::words(word);
        else
        {
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e)
                if (w + e < c.nq)
                    bits[w + e] = word[e];
        }
    }
    else
    {
        const uint32_t local = w - strip * SS::WORDS;
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e)
        {
            if constexpr (sizeof(Q) == 8)
                atomicOr(reinterpret_cast<unsigned long long*>(&words[local + e]), (unsigned long long) word[e]);
            else
                atomicOr(&words[local + e], word[e]);
        }
        __syncthreads();
        for (uint32_t x = tid; x < SS::WORDS; x += kStripThreads)
            if (FULL || strip * SS::WORDS + x < c.nq)
                bits[strip * SS::WORDS + x] = words[x];
    }
}

template <typename E>
__host__ __device__ inline size_t strip_lds_bytes(size_t nbits)
{
    const size_t vpw = Word<E>::kBits / nbits;
    return kStripRedBytes<E> + (vpw > 8 ? (size_t) strip_words<E>(nbits) * sizeof(E) : 0);
}

// whether every QWord of the strip exists and has an element at every bit position (only the last bit position can be
// short of elements, and only in the last QWords of the column)
template <int NBITS, typename E>
__device__ __forceinline__ bool strip_is_full(const StripGeom& c, uint32_t strip)
{
    using SS = StripShape<NBITS, E>;
    const uint32_t end = (strip + 1) * SS::WORDS;
    return end <= c.nq && (uint64_t) (SS::PS::VPW - 1) * c.nq + end <= c.rows;
}

// which QWords and bit positions a thread holds of a strip: PER QWords from w, SLOTS bit positions from k0. Where a
// wavefront holds one range of bit positions k0 is a scalar.
template <int NBITS, typename E>
__device__ __forceinline__ void strip_thread_slots(uint32_t strip, uint32_t& w, uint32_t& k0)
{
    using SS = StripShape<NBITS, E>;
    w = strip * SS::WORDS + SS::PER * (threadIdx.x % SS::RUNS);
    if constexpr (SS::RUNS % kWave == 0)
        k0 = __builtin_amdgcn_readfirstlane(threadIdx.x / SS::RUNS) * SS::SLOTS;
    else
        k0 = threadIdx.x / SS::RUNS * SS::SLOTS;
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

// which of a thread's PER * SLOTS values exist in a strip at the ragged end of its column: element (QWord q, bit position
// k) is q + k * nq, so up to bit position whole_positions all of an existing QWord's do, at that one those of the first
// last_words QWords, beyond it none
template <int NBITS, typename E>
__device__ __forceinline__ uint32_t strip_valid_mask(const StripGeom& c, uint32_t w, uint32_t k0)
{
    using SS = StripShape<NBITS, E>;
    constexpr uint32_t PER = SS::PER;
    uint32_t words = 0u, last = 0u;
#pragma unroll
    for (uint32_t e = 0; e < PER; ++e)
    {
        words |= (w + e < c.nq) ? (1u << e) : 0u;
        last |= (w + e < c.last_words) ? (1u << e) : 0u;
    }
    uint32_t valid = ~(uint32_t) ((1ull << (PER * SS::SLOTS)) - 1ull); // bits beyond the thread's values count as present
#pragma unroll
    for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
    {
        const uint32_t k = k0 + kk;
        valid |= (k < c.whole_positions ? words : (k == c.whole_positions ? last : 0u)) << (PER * kk);
    }
    return valid;
}

// N pieces of a column, the PER consecutive values from element i0 + n * stride on each (16 bytes at the alignment of an
// element), all requested before any is used. FULL: all values exist. Otherwise bit PER * n + e of `valid` says whether
// value e of piece n does, and the others read as zero. Every lane loads 16 bytes from inside its column whatever it
// holds (its own piece where that ends inside the column, the column's first elements otherwise), so that no branch
// stands between the loads; what does not exist is then cleared, and the few values of a piece that runs over the
// column's end (fewer than PER per column) are fetched one by one.
template <bool FULL, uint32_t N, typename E>
__device__ __forceinline__ void strip_load_pieces(const E* col, uint32_t i0, uint32_t stride, uint32_t rows, uint32_t valid, StripVec<E>* out)
{
    using SE = StripElem<E>;
    constexpr uint32_t PER = SE::PER, ALL = (1u << PER) - 1u;
    if constexpr (FULL)
    {
#pragma unroll
        for (uint32_t n = 0; n < N; ++n)
            out[n] = __builtin_nontemporal_load(reinterpret_cast<const typename SE::VU*>(col + i0 + n * stride));
    }
    else
    {
        uint32_t over = 0; // pieces with values that run over the column's end
        if (rows >= PER)
        {
#pragma unroll
            for (uint32_t n = 0; n < N; ++n)
            {
                const uint32_t i = i0 + n * stride;
                out[n] = __builtin_nontemporal_load(reinterpret_cast<const typename SE::VU*>(col + (i + PER <= rows ? i : 0u)));
            }
#pragma unroll
            for (uint32_t n = 0; n < N; ++n)
            {
                const uint32_t i = i0 + n * stride, ok = (valid >> (PER * n)) & ALL;
                const bool inside = i + PER <= rows;
                over |= (!inside && ok != 0u) ? (1u << n) : 0u;
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                    out[n][e] = (inside && ((ok >> e) & 1u)) ? out[n][e] : (E) 0;
            }
        }
        else
        {
#pragma unroll
            for (uint32_t n = 0; n < N; ++n)
            {
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                    out[n][e] = 0;
                over |= ((valid >> (PER * n)) & ALL) != 0u ? (1u << n) : 0u;
            }
        }
        if (over != 0u)
        {
#pragma unroll
            for (uint32_t n = 0; n < N; ++n)
            {
                const uint32_t i = i0 + n * stride, ok = (valid >> (PER * n)) & ALL;
                if ((over >> n) & 1u)
                {
#pragma unroll
                    for (uint32_t e = 0; e < PER; ++e)
                        if ((ok >> e) & 1u)
                            out[n][e] = col[i + e];
                }
            }
        }
    }
}

// The gradient goes straight into the registers that will hold the sums, the residual joins it four loads at a time. Every
// value of the strip is in registers before anything is stored, so r_out may be r_in.
template <int NBITS, bool ZT, bool FULL, typename E, int PASS>
__device__ __forceinline__ void quantize_strip_body(const E* g_col, const E* r_col, E* res_col, char* qc, uint32_t column, uint32_t strip,
                                                    uint32_t tag, const StripGeom& c, const StripScratch& scratch, char* smem)
{
    using SS = StripShape<NBITS, E>;
    constexpr uint32_t PER = SS::PER;
    uint32_t w, k0;
    strip_thread_slots<NBITS, E>(strip, w, k0);
    const uint32_t valid = FULL ? 0xFFFFFFFFu : strip_valid_mask<NBITS, E>(c, w, k0);
    const uint32_t i0 = k0 * c.nq + w;
    StripVec<E> v[SS::SLOTS];
    strip_load_pieces<FULL, SS::SLOTS, E>(g_col, i0, c.nq, c.rows, valid, v);
    constexpr uint32_t BATCH = SS::SLOTS < 4 ? SS::SLOTS : 4;
#pragma unroll
    for (uint32_t k1 = 0; k1 < SS::SLOTS; k1 += BATCH)
    {
        StripVec<E> b[BATCH];
        strip_load_pieces<FULL, BATCH, E>(r_col, i0 + k1 * c.nq, c.nq, c.rows, valid >> (PER * k1), b);
#pragma unroll
        for (uint32_t kk = 0; kk < BATCH; ++kk)
            v[k1 + kk] = v[k1 + kk] + b[kk];
    }
    strip_stats_pack<NBITS, ZT, FULL, E, PASS>(v, valid, w, k0, column, strip, tag, c, scratch, smem, res_col, qc);
}

// PASS 0: the whole quantization in one launch. Otherwise one of the launches it is cut into (kStripPassStat, where the
// bit width has a statistic; kStripPassSplit, at 1 bit; kStripPassPack), issued in that order on one stream with
// geometry.spread set: for columns of more strips than the device holds at once.
template <int NBITS, bool ZT, typename E, int PASS = 0>
__global__ __launch_bounds__(kStripThreads, (StripShape<NBITS, E>::WAVES)) void quantize_strip_kernel(const E* __restrict__ g, const E* r_in, E* r_out,
                                                                                                    char* __restrict__ q, StripGeom c,
                                                                                                    StripScratch scratch)
{
    static_assert(NBITS < Word<E>::kBits, "codes as wide as a QWord are whole QWords: nothing to assemble");
    extern __shared__ f32x4 smem_v4[];
    char* smem = reinterpret_cast<char*>(smem_v4);
    uint32_t column, strip, tag;
    if (!strip_assignment(c, scratch, column, strip, tag))
        return;
    const size_t base = (size_t) column * c.rows;
    char* qc = q + (size_t) column * c.qcol;
    if (strip_is_full<NBITS, E>(c, strip))
        quantize_strip_body<NBITS, ZT, true, E, PASS>(g + base, r_in + base, r_out + base, qc, column, strip, tag, c, scratch, smem);
    else
        quantize_strip_body<NBITS, ZT, false, E, PASS>(g + base, r_in + base, r_out + base, qc, column, strip, tag, c, scratch, smem);
}

// ---- the stripe reduction of the quantized all-reduce on strips: K packed stripes -> sum -> requantize with the stripe
// residual (Source/1BitSGD/AllReduceDistGradAggregator.h:385-436: unquantize the owner's stripe, add the other workers' in
// ascending order, quantize the sum with the stripe residual). A thread decodes its QWords of every worker at its bit
// positions into the registers that strip_stats_pack then takes, so the call gives the bytes of that call sequence with the
// strip kernel as its quantize step. Every worker's column header is read before the strip publishes its first partial
// sum, and strip 0 writes the new header only after it has every strip's: q_out may be the owner's own stripe.
template <int NBITS, bool ZT, bool FULL, typename E>
__device__ __forceinline__ void stripe_reduce_strip_body(const StripeSources& src, size_t col_off, E* res_col, char* qc_out, E* agg_col,
                                                         uint32_t column, uint32_t strip, uint32_t tag, const StripGeom& c,
                                                         const StripScratch& scratch, char* smem)
{
    using SS = StripShape<NBITS, E>;
    using PS = typename SS::PS;
    using SE = StripElem<E>;
    using Q = typename Word<E>::Q;
    constexpr uint32_t PER = SS::PER, ALL = (1u << PER) - 1u;
    uint32_t w, k0;
    strip_thread_slots<NBITS, E>(strip, w, k0);
    const uint32_t valid = FULL ? 0xFFFFFFFFu : strip_valid_mask<NBITS, E>(c, w, k0);
    StripVec<E> v[SS::SLOTS];
    // The workers' QWords are requested four workers at a time, before any of them is decoded (a worker beyond the last
    // repeats the last one's addresses and is left out of the sum): one memory round trip per four workers.
    constexpr uint32_t GROUP = 4;
    auto add_group = [&](uint32_t n0, auto first_group) {
        Q word[GROUP][PER];
        E lo[GROUP], hi[GROUP];
#pragma unroll
        for (uint32_t u = 0; u < GROUP; ++u)
        {
            const uint32_t n = n0 + u < src.workers ? n0 + u : src.workers - 1;
            const char* qc = src.q[stripe_order(n, src.owner)] + col_off;
            const E* h = reinterpret_cast<const E*>(qc);
            lo[u] = h[0];
            hi[u] = h[1];
            const Q* bits = reinterpret_cast<const Q*>(qc + 2 * sizeof(E));
            if constexpr (FULL)
            {
                const typename SE::QV x = *reinterpret_cast<const typename SE::QVU*>(bits + w);
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                    word[u][e] = x[e];
            }
            else
            {
                // (QWord by QWord, from inside the column whatever the lane holds: no branch between the loads)
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                    word[u][e] = bits[w + e < c.nq ? w + e : c.nq - 1];
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < GROUP; ++u)
        {
            if (n0 + u >= src.workers)
                break;
            const ValueQOf<E> vq = make_vq<NBITS, E>(lo[u], hi[u]);
            const E val0 = unquantize_value<NBITS, E>(vq, (Q) 0);
            const E val1 = unquantize_value<NBITS, E>(vq, (Q) 1);
#pragma unroll
            for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                {
                    const Q code = (word[u][e] >> ((k0 + kk) * PS::SHIFT)) & PS::CODEMASK;
                    E x;
                    if constexpr (NBITS == 1)
                        x = code ? val1 : val0;
                    else
                        x = unquantize_value<NBITS, E>(vq, code);
                    // the first term seeds the sum; afterwards: decoded value + running sum
                    if (decltype(first_group)::value && u == 0)
                        v[kk][e] = x;
                    else
                        v[kk][e] = x + v[kk][e];
                }
        }
    };
    add_group(0u, std::true_type());
    for (uint32_t n0 = GROUP; n0 < src.workers; n0 += GROUP)
        add_group(n0, std::false_type());
    if constexpr (!FULL)
    {
        // (a QWord's bits beyond the column's last element are zero and decode to the lowest level: those values do not exist)
#pragma unroll
        for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e)
                v[kk][e] = ((valid >> (PER * kk + e)) & 1u) ? v[kk][e] : (E) 0;
    }
    const uint32_t i0 = k0 * c.nq + w;
    if (agg_col != nullptr)
    {
#pragma unroll
        for (uint32_t kk = 0; kk < SS::SLOTS; ++kk)
        {
            E* dst = agg_col + i0 + kk * c.nq;
            const uint32_t ok = FULL ? ALL : (valid >> (PER * kk)) & ALL;
            if (ok == ALL)
                __builtin_nontemporal_store(v[kk], reinterpret_cast<typename SE::VU*>(dst));
            else if (ok != 0u)
            {
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e)
                    if ((ok >> e) & 1u)
                        dst[e] = v[kk][e];
            }
        }
    }
    constexpr uint32_t BATCH = SS::SLOTS < 4 ? SS::SLOTS : 4;
#pragma unroll
    for (uint32_t k1 = 0; k1 < SS::SLOTS; k1 += BATCH)
    {
        StripVec<E> b[BATCH];
        strip_load_pieces<FULL, BATCH, E>(res_col, i0 + k1 * c.nq, c.nq, c.rows, valid >> (PER * k1), b);
#pragma unroll
        for (uint32_t kk = 0; kk < BATCH; ++kk)
            v[k1 + kk] = v[k1 + kk] + b[kk];
    }
    strip_stats_pack<NBITS, ZT, FULL, E>(v, valid, w, k0, column, strip, tag, c, scratch, smem, res_col, qc_out);
}

template <int NBITS, bool ZT, typename E>
__global__ __launch_bounds__(kStripThreads, (StripShape<NBITS, E>::WAVES)) void stripe_reduce_strip_kernel(StripeSources src, E* stripe_res, char* q_out,
                                                                                                           E* agg_out, StripGeom c, StripScratch scratch)
{
    static_assert(NBITS < Word<E>::kBits, "codes as wide as a QWord are whole QWords: nothing to assemble");
    extern __shared__ f32x4 smem_v4[];
    char* smem = reinterpret_cast<char*>(smem_v4);
    uint32_t column, strip, tag;
    if (!strip_assignment(c, scratch, column, strip, tag))
        return;
    const size_t base = (size_t) column * c.rows, col_off = (size_t) column * c.qcol;
    E* agg_col = agg_out != nullptr ? agg_out + base : nullptr;
    if (strip_is_full<NBITS, E>(c, strip))
        stripe_reduce_strip_body<NBITS, ZT, true, E>(src, col_off, stripe_res + base, q_out + col_off, agg_col, column, strip, tag, c, scratch, smem);
    else
        stripe_reduce_strip_body<NBITS, ZT, false, E>(src, col_off, stripe_res + base, q_out + col_off, agg_col, column, strip, tag, c, scratch, smem);
}

} // namespace cntkq
