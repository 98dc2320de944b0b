// gfx950 kernels of the per-column gradient quantizer: the decoders (packed codes -> values).
#pragma once

#include "quantizer_kernels_common.h"

namespace cntkq {

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

// Written over the element type: E = float with 32-bit QWords (WV = 4 QWords and rows per thread and bit position, one
// 16-byte store) or double with 64-bit QWords (WV = 2); WV = 1 stores one element at a time, whatever the alignment.
template <int NBITS, int WV, typename E>
__device__ __forceinline__ void unquantize_body(const char* __restrict__ q, E* out, const UnqGeom& t, int add, uint32_t block)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    typedef E Vec __attribute__((ext_vector_type(WV == 1 ? 2 : WV))); // (unused when WV == 1)
    static_assert(WV == 1 || WV * sizeof(E) == 16, "one 16-byte store per bit position");

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
    const E* gh = reinterpret_cast<const E*>(qc);
    ValueQOf<E> vq; // decoding needs only the code -> value factor and the lower bound
    vq.lo = gh[0];
    vq.uf = make_ufactor<NBITS>(gh[0], gh[1]);
    const E val0 = unquantize_value<NBITS>(vq, 0u);
    const E val1 = unquantize_value<NBITS>(vq, 1u);
    const QWord* bits = reinterpret_cast<const QWord*>(qc + 2 * sizeof(E));
    E* oc = out + (size_t) c * t.rows;

    QWord word[WV];
    if constexpr (WV == 4 && sizeof(QWord) == 4)
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
#pragma unroll
        for (int u = 0; u < WV; ++u)
            word[u] = bits[w0 + u]; // (double: WV == 2 only when nq is even)
    }

    const uint32_t k0 = chunk * t.slots;
    const uint32_t k1 = min(k0 + t.slots, PS::VPW);
    for (uint32_t k = k0; k < k1; ++k)
    {
        const uint32_t i = w0 + k * t.nq;
        if (i >= t.rows)
            break; // rows only grow with k
        const uint32_t sh = k * PS::SHIFT;
        if constexpr (WV > 1)
        {
            // rows, nq and i are multiples of WV: the WV rows are all inside the column and the store is 16-byte aligned
            Vec x;
#pragma unroll
            for (int u = 0; u < WV; ++u)
            {
                if constexpr (NBITS == 1)
                    x[u] = ((word[u] >> sh) & 1u) ? val1 : val0;
                else
                    x[u] = unquantize_value<NBITS>(vq, (word[u] >> sh) & PS::CODEMASK);
            }
            Vec* dst = reinterpret_cast<Vec*>(oc + i);
            if (add)
                x = x + *dst; // unquantized value + previous content
            __builtin_nontemporal_store(x, dst);
        }
        else
        {
            E x;
            if constexpr (NBITS == 1)
                x = ((word[0] >> sh) & 1u) ? val1 : val0;
            else
                x = unquantize_value<NBITS>(vq, (word[0] >> sh) & PS::CODEMASK);
            if (add)
                x = x + oc[i];
            oc[i] = x;
        }
    }
}

template <int NBITS, int WV, typename E>
__global__ __launch_bounds__(256) void unquantize_kernel(const char* __restrict__ q, E* out, UnqGeom t, int add)
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

// Written over the element type: N = 4 floats or 2 doubles per 16-byte store; `words` holds the column's QWords.
template <int NBITS, typename E>
__device__ __forceinline__ void unquantize_rows_body(const char* __restrict__ q, E* out, const UnqRowGeom& t, int add, uint32_t block,
                                                     typename Word<E>::Q* words)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    constexpr uint32_t N = 16 / sizeof(E);
    typedef E Vec __attribute__((ext_vector_type(N)));
    const uint32_t tid = threadIdx.x;
    uint32_t c, ch;
    unq_rows_block_to_chunk(block, t.chunks, t.blocks, c, ch);
    const char* qc = q + (size_t) c * t.qcol;
    const E* gh = reinterpret_cast<const E*>(qc);
    const E lo = gh[0];
    const E uf = make_ufactor<NBITS>(lo, gh[1]);
    const QWord* bits = reinterpret_cast<const QWord*>(qc + 2 * sizeof(E));
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
            QWord v[8];
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
    // The column need not start on a 16-byte boundary nor hold a multiple of N rows: `head` rows (0..N-1) lie before its
    // first aligned group of N and `tail` rows (0..N-1) after the last; chunks are counted from the first aligned row,
    // the first chunk's workgroup also writes the head rows, the last one's the tail rows, one row per thread.
    E* oc = out + (size_t) c * t.rows;
    const uint32_t head = (N - (uint32_t) ((reinterpret_cast<uintptr_t>(oc) / sizeof(E)) & (N - 1))) & (N - 1);
    const uint32_t body = (t.rows - head) & ~(N - 1); // rows in aligned groups of N
    const uint32_t tail = t.rows - head - body;
    const uint32_t r0 = ch * t.chunk;
    const uint32_t pieces = ((ch + 1 == t.chunks ? body : r0 + t.chunk) - r0) / N; // the last chunk runs to the end
    Vec* o4 = reinterpret_cast<Vec*>(oc + head + r0);
    const E val0 = unquantize_value<NBITS>(uf, lo, 0u);
    const E val1 = unquantize_value<NBITS>(uf, lo, 1u);
    {
        uint32_t row = t.rows; // none
        if (ch == 0 && tid < head)
            row = tid;
        else if (ch + 1 == t.chunks && tid >= N && tid < N + tail)
            row = head + body + (tid - N);
        if (row < t.rows)
        {
            const uint32_t k = row / t.nq;
            const QWord code = (words[row - k * t.nq] >> (k * PS::SHIFT)) & PS::CODEMASK;
            E x;
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
    // row i sits in QWord i % nq at bit position i / nq; a thread's pieces are 256 * N rows apart
    const uint32_t i0 = head + r0 + N * (vfirst - shift);
    uint32_t k0 = i0 / t.nq;
    uint32_t w0 = i0 - k0 * t.nq;
    const uint32_t dk = (256u * N) / t.nq;
    const uint32_t dw = 256u * N - dk * t.nq;
    for (uint32_t p = vfirst - shift; p < pieces; p += 256)
    {
        uint32_t k = k0, w = w0;
        Vec x;
#pragma unroll
        for (uint32_t e = 0; e < N; ++e)
        {
            const QWord code = (words[w] >> (k * PS::SHIFT)) & PS::CODEMASK;
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

template <int NBITS, typename E>
__global__ __launch_bounds__(256) void unquantize_rows_kernel(const char* __restrict__ q, E* out, UnqRowGeom t, int add)
{
    extern __shared__ f32x4 smem_v4[];
    unquantize_rows_body<NBITS>(q, out, t, add, blockIdx.x, reinterpret_cast<typename Word<E>::Q*>(smem_v4));
}

// Row-major decoder that keeps nothing in LDS: the geometry of the one above (chunks of consecutive rows of a column, its
// head and tail rows, slots dealt by 128-byte lines), but a thread fetches the QWords of its groups of N consecutive rows
// itself -- N consecutive QWords at one bit position, one 16-byte load at the alignment of a QWord -- all kUnqDirectPieces
// of them before it decodes the first. Every QWord is fetched once per bit position, from the L2 that the column's other
// chunks go through as well (their workgroups are 8 apart). No copy of the packed column per workgroup, no barrier, any
// QWord count: the choice for columns whose packed record is large against a chunk of rows.
constexpr uint32_t kUnqDirectPieces = 2;

template <int NBITS, typename E>
__device__ __forceinline__ void unquantize_direct_body(const char* __restrict__ q, E* out, const UnqRowGeom& t, int add, uint32_t block)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    constexpr uint32_t N = 16 / sizeof(E);
    constexpr uint32_t P = kUnqDirectPieces;
    typedef E Vec __attribute__((ext_vector_type(N)));
    typedef QWord QVec __attribute__((ext_vector_type(N)));
    typedef QVec QVecAtWord __attribute__((aligned(sizeof(QWord))));
    const uint32_t tid = threadIdx.x;
    uint32_t c, ch;
    unq_rows_block_to_chunk(block, t.chunks, t.blocks, c, ch);
    const char* qc = q + (size_t) c * t.qcol;
    const E* gh = reinterpret_cast<const E*>(qc);
    const E lo = gh[0];
    const E uf = make_ufactor<NBITS>(lo, gh[1]);
    const QWord* bits = reinterpret_cast<const QWord*>(qc + 2 * sizeof(E));
    // head, body and tail rows of the column as in the decoder above; here every chunk is t.chunk rows at most
    E* oc = out + (size_t) c * t.rows;
    const uint32_t head = (N - (uint32_t) ((reinterpret_cast<uintptr_t>(oc) / sizeof(E)) & (N - 1))) & (N - 1);
    const uint32_t body = (t.rows - head) & ~(N - 1);
    const uint32_t tail = t.rows - head - body;
    const uint32_t r0 = ch * t.chunk;
    const uint32_t end = body < r0 + t.chunk ? body : r0 + t.chunk;
    const uint32_t pieces = end > r0 ? (end - r0) / N : 0u;
    Vec* o4 = reinterpret_cast<Vec*>(oc + head + r0);
    const E val0 = unquantize_value<NBITS>(uf, lo, 0u);
    const E val1 = unquantize_value<NBITS>(uf, lo, 1u);
    {
        uint32_t row = t.rows; // none
        if (ch == 0 && tid < head)
            row = tid;
        else if (ch + 1 == t.chunks && tid >= N && tid < N + tail)
            row = head + body + (tid - N);
        if (row < t.rows)
        {
            const uint32_t k = row / t.nq;
            const QWord code = (bits[row - k * t.nq] >> (k * PS::SHIFT)) & PS::CODEMASK;
            E x;
            if constexpr (NBITS == 1)
                x = code ? val1 : val0;
            else
                x = unquantize_value<NBITS>(uf, lo, code);
            oc[row] = add ? x + oc[row] : x;
        }
    }
    const uint32_t shift = (uint32_t) ((reinterpret_cast<uintptr_t>(o4) >> 4) & 7u);
    const uint32_t p0 = (tid < shift ? tid + 256 : tid) - shift;
    const uint32_t i0 = head + r0 + N * p0;
    const uint32_t k0 = i0 / t.nq;
    const uint32_t w0 = i0 - k0 * t.nq;
    const uint32_t dk = (256u * N) / t.nq;
    const uint32_t dw = 256u * N - dk * t.nq;
    QVec qv[P];
    Vec prev[P];
    uint32_t ks[P], ws[P];
    {
        uint32_t k = k0, w = w0;
#pragma unroll
        for (uint32_t u = 0; u < P; ++u)
        {
            const uint32_t p = p0 + 256 * u;
            ks[u] = k;
            ws[u] = w;
            // (a group that wraps to the next bit position inside is fetched QWord by QWord below; a piece beyond the
            // chunk fetches the column's first QWords and uses nothing)
            const uint32_t from = p < pieces ? (w + N <= t.nq ? w : t.nq - N) : 0u;
            qv[u] = *reinterpret_cast<const QVecAtWord*>(bits + from);
            if (add)
                prev[u] = o4[p < pieces ? p : 0u];
            k += dk;
            w += dw;
            if (w >= t.nq)
            {
                w -= t.nq;
                ++k;
            }
        }
    }
#pragma unroll
    for (uint32_t u = 0; u < P; ++u)
    {
        const uint32_t p = p0 + 256 * u;
        if (p < pieces)
        {
            QWord wd[N];
            uint32_t sh[N];
#pragma unroll
            for (uint32_t e = 0; e < N; ++e)
            {
                wd[e] = qv[u][e];
                sh[e] = ks[u] * PS::SHIFT;
            }
            if (ws[u] + N > t.nq)
            {
#pragma unroll
                for (uint32_t e = 0; e < N; ++e)
                {
                    const bool wraps = ws[u] + e >= t.nq;
                    wd[e] = bits[wraps ? ws[u] + e - t.nq : ws[u] + e];
                    sh[e] = (wraps ? ks[u] + 1 : ks[u]) * PS::SHIFT;
                }
            }
            Vec x;
#pragma unroll
            for (uint32_t e = 0; e < N; ++e)
            {
                const QWord code = (wd[e] >> sh[e]) & PS::CODEMASK;
                if constexpr (NBITS == 1)
                    x[e] = code ? val1 : val0;
                else
                    x[e] = unquantize_value<NBITS>(uf, lo, code);
            }
            if (add)
                x = x + prev[u]; // unquantized value + previous content
            __builtin_nontemporal_store(x, o4 + p);
        }
    }
}

template <int NBITS, typename E>
__global__ __launch_bounds__(256) void unquantize_direct_kernel(const char* __restrict__ q, E* out, UnqRowGeom t, int add)
{
    unquantize_direct_body<NBITS>(q, out, t, add, blockIdx.x);
}

// The same without LDS for short columns whose heights are multiples of N (the elements of 16 bytes), with N QWords or more:
// consecutive columns are adjacent in the output, so the matrix is one run of groups of N consecutive elements, each group
// inside one column and, where the QWord count is a multiple of N too, at one bit position of N consecutive QWords. A
// thread takes kUnqDirectPieces groups, 256 groups apart, finds column, bit position and QWord of each, requests the
// column's header and the N QWords of every group and then decodes. The output is 16-byte aligned and the matrix has
// fewer than 2^32 elements (checked by the host).
struct UnqFlatGeom
{
    uint32_t rows;
    uint32_t nq;
    uint32_t groups; // rows * cols / N
    uint32_t blocks; // workgroups: 256 * kUnqDirectPieces groups each
    double inv_rows;
    double inv_nq;
    uint64_t qcol;
};

template <int NBITS, typename E>
__device__ __forceinline__ void unquantize_flat_body(const char* __restrict__ q, E* out, const UnqFlatGeom& t, int add, uint32_t block)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    constexpr uint32_t N = 16 / sizeof(E);
    constexpr uint32_t P = kUnqDirectPieces;
    typedef E Vec __attribute__((ext_vector_type(N)));
    typedef E Pair __attribute__((ext_vector_type(2)));
    typedef Pair PairAtElem __attribute__((aligned(sizeof(E))));
    typedef QWord QVec __attribute__((ext_vector_type(N)));
    typedef QVec QVecAtWord __attribute__((aligned(sizeof(QWord))));
    Vec* o4 = reinterpret_cast<Vec*>(out);
    QVec qv[P];
    Pair hd[P];
    Vec prev[P];
    uint32_t sh[P], ws[P], cs[P];
#pragma unroll
    for (uint32_t u = 0; u < P; ++u)
    {
        const uint32_t g = block * (256u * P) + 256u * u + threadIdx.x;
        const uint32_t gg = g < t.groups ? g : 0u; // a group beyond the matrix fetches the first one's and uses nothing
        uint32_t c, r, k, w;
        divmod_u32(gg * N, t.rows, t.inv_rows, c, r);
        divmod_u32(r, t.nq, t.inv_nq, k, w);
        const char* qc = q + (size_t) c * t.qcol;
        hd[u] = *reinterpret_cast<const PairAtElem*>(qc);
        // (a group that wraps to the next bit position inside -- QWord counts that are no multiple of N -- is fetched QWord by
        // QWord below)
        qv[u] = *reinterpret_cast<const QVecAtWord*>(qc + 2 * sizeof(E) + (size_t) (w + N <= t.nq ? w : t.nq - N) * sizeof(QWord));
        sh[u] = k * PS::SHIFT;
        ws[u] = w;
        cs[u] = c;
        if (add)
            prev[u] = o4[gg];
    }
#pragma unroll
    for (uint32_t u = 0; u < P; ++u)
    {
        const uint32_t g = block * (256u * P) + 256u * u + threadIdx.x;
        if (g < t.groups)
        {
            const E lo = hd[u][0];
            const E uf = make_ufactor<NBITS>(lo, hd[u][1]);
            const E val0 = unquantize_value<NBITS>(uf, lo, 0u);
            const E val1 = unquantize_value<NBITS>(uf, lo, 1u);
            QWord wd[N];
            uint32_t she[N];
#pragma unroll
            for (uint32_t e = 0; e < N; ++e)
            {
                wd[e] = qv[u][e];
                she[e] = sh[u];
            }
            if (ws[u] + N > t.nq)
            {
                const QWord* bits = reinterpret_cast<const QWord*>(q + (size_t) cs[u] * t.qcol + 2 * sizeof(E));
#pragma unroll
                for (uint32_t e = 0; e < N; ++e)
                {
                    const bool wraps = ws[u] + e >= t.nq;
                    wd[e] = bits[wraps ? ws[u] + e - t.nq : ws[u] + e];
                    she[e] = wraps ? sh[u] + PS::SHIFT : sh[u];
                }
            }
            Vec x;
#pragma unroll
            for (uint32_t e = 0; e < N; ++e)
            {
                const QWord code = (wd[e] >> she[e]) & PS::CODEMASK;
                if constexpr (NBITS == 1)
                    x[e] = code ? val1 : val0;
                else
                    x[e] = unquantize_value<NBITS>(uf, lo, code);
            }
            if (add)
                x = x + prev[u];
            __builtin_nontemporal_store(x, o4 + g);
        }
    }
}

template <int NBITS, typename E>
__global__ __launch_bounds__(256) void unquantize_flat_kernel(const char* __restrict__ q, E* out, UnqFlatGeom t, int add)
{
    unquantize_flat_body<NBITS>(q, out, t, add, blockIdx.x);
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
    uint32_t rec_words;  // nq + 2: QWords per packed record (lower, upper, bits)
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

// Written over the element type: N = 4 floats or 2 doubles per 16-byte store; a packed record is rec_words QWords
// (lower, upper, bits), and smem holds cpt records and two decode constants per column.
template <int NBITS, typename E>
__device__ __forceinline__ void unquantize_tile_body(const char* __restrict__ q, E* out, const UnqTileGeom& t, int add, uint32_t block,
                                                     typename Word<E>::Q* smem)
{
    typedef typename Word<E>::Q QWord;
    using PS = PackShapeOf<NBITS, Word<E>::kBits>;
    constexpr uint32_t N = 16 / sizeof(E);
    typedef E Vec __attribute__((ext_vector_type(N)));
    // (the output may start on any element boundary: the 16-byte accesses are then at that alignment)
    typedef Vec VecAt4 __attribute__((aligned(sizeof(E))));
    const uint32_t tid = threadIdx.x;
    const uint32_t col0 = block * t.cpt;
    const uint32_t ncols = (t.cols - col0 < t.cpt) ? t.cols - col0 : t.cpt;
    QWord* words = smem;                                        // ncols packed records
    E* dec = reinterpret_cast<E*>(smem + t.cpt * t.rec_words); // per column: the two levels (1 bit) or (ufactor, lower)
    const QWord* src = reinterpret_cast<const QWord*>(q + (size_t) col0 * t.rec_words * sizeof(QWord));
    const uint32_t total_words = ncols * t.rec_words;
    for (uint32_t x = tid; x < total_words; x += 256)
        words[x] = __builtin_nontemporal_load(src + x);
    __syncthreads();
    for (uint32_t c = tid; c < ncols; c += 256)
    {
        const E lo = Word<E>::value_of(words[c * t.rec_words]);
        const E hi = Word<E>::value_of(words[c * t.rec_words + 1]);
        const E uf = make_ufactor<NBITS>(lo, hi);
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
    E* o = out + (size_t) col0 * t.rows;
    // slots dealt by 128-byte lines: slot v = tid, tid + 256, ... holds the group of N that starts at element
    // N * (v - shift), shift = the tile's offset into its line in 16-byte pieces
    const uint32_t shift = (uint32_t) ((reinterpret_cast<uintptr_t>(o) >> 4) & 7u);
    if (t.rows % N == 0 && t.nq % N == 0)
    {
        // Heights and QWord counts that are multiples of N (64, 128, 256, 512, 576, 1152 rows at 2 to 8 bits; 512 rows at
        // 1 bit): a group of N consecutive elements lies in one column at one bit position of N consecutive QWords, so
        // column, bit position and QWord are worked out once per group and nothing wraps inside it (the general loop below
        // checks both wraps after every element: some 19 vector instructions per element against 6 here).
        for (uint32_t i = N * ((tid < shift ? tid + 256 : tid) - shift); i < elems; i += 256 * N)
        {
            const uint32_t c = small_div(i, t.rows, t.rows_magic);
            const uint32_t r = i - c * t.rows;
            const uint32_t k = small_div(r, t.nq, t.nq_magic);
            const QWord* cw = words + c * t.rec_words + 2 + (r - k * t.nq);
            const E d0 = dec[2 * c], d1 = dec[2 * c + 1];
            const uint32_t sh = k * PS::SHIFT;
            QWord packed[N];
            if constexpr (N == 4)
            {
                // (records are an even number of QWords long here and start on one: pairs of QWords are 8-byte aligned)
                typedef QWord Pair __attribute__((ext_vector_type(2)));
                const Pair a = *reinterpret_cast<const Pair*>(cw), b = *reinterpret_cast<const Pair*>(cw + 2);
                packed[0] = a.x, packed[1] = a.y, packed[2] = b.x, packed[3] = b.y;
            }
            else
            {
#pragma unroll
                for (uint32_t e = 0; e < N; ++e)
                    packed[e] = cw[e];
            }
            Vec x;
#pragma unroll
            for (uint32_t e = 0; e < N; ++e)
            {
                const QWord code = (packed[e] >> sh) & PS::CODEMASK;
                if constexpr (NBITS == 1)
                    x[e] = code ? d1 : d0;
                else
                    x[e] = unquantize_value<NBITS>(d0, d1, code);
            }
            VecAt4* o4 = reinterpret_cast<VecAt4*>(o + i);
            if (add)
                x = x + *o4; // unquantized value + previous content
            __builtin_nontemporal_store(x, o4);
        }
        return;
    }
    for (uint32_t i = N * ((tid < shift ? tid + 256 : tid) - shift); i < elems; i += 256 * N)
    {
        uint32_t c = small_div(i, t.rows, t.rows_magic);
        uint32_t r = i - c * t.rows;
        uint32_t k = small_div(r, t.nq, t.nq_magic);
        uint32_t w = r - k * t.nq;
        const QWord* cw = words + c * t.rec_words + 2;
        E d0 = dec[2 * c], d1 = dec[2 * c + 1];
        Vec x;
#pragma unroll
        for (uint32_t e = 0; e < N; ++e)
        {
            // (past the end of the matrix c == ncols: the reads stay inside the LDS block and the value is not stored)
            const QWord code = (cw[w] >> (k * PS::SHIFT)) & PS::CODEMASK;
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
        if (i + N <= elems)
        {
            VecAt4* o4 = reinterpret_cast<VecAt4*>(o + i);
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

template <int NBITS, typename E>
__global__ __launch_bounds__(256) void unquantize_tile_kernel(const char* __restrict__ q, E* out, UnqTileGeom t, int add)
{
    extern __shared__ f32x4 smem_v4[];
    unquantize_tile_body<NBITS>(q, out, t, add, blockIdx.x, reinterpret_cast<typename Word<E>::Q*>(smem_v4));
}

} // namespace cntkq
