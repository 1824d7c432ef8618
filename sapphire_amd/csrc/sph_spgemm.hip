// CSR x CSR -> CSR product on the device.
//
// The reference declares this product (Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:16-100,
// Sparse::Cuda::Gemm over arrays of SparseMatrix, one block per output row, a hash table per
// row, a bitonic sort and a load-distribution pre-pass; helper bodies in
// Sources/Sapphire/compute/cudaUtil/SparseUtil.cu) and defines no host entry for it.  The
// contract kept here is the one its dense leaf gives on the densified operands
// (Sources/Sapphire/compute/dense/naive/NaiveGemm.cpp:12-38): element (i, j) is the sum over
// A's row i, entries in storage order, of a * B[k][j], product and sum rounded separately,
// starting from +0; results that are exactly 0 are not stored (SparseUtil.cu:55-60 deletes
// them as well); a row's entries come out in ascending column order.
//
// One wavefront owns one output row.  Instead of a hash table and a sort it keeps a dense
// strip of the row in LDS (up to 4096 columns, 16 KiB; wider matrices are done strip by
// strip): A's entries are taken in order, the entries of the matching row of B are spread
// over the 64 lanes and added into the strip, and because the columns of one row of B are
// distinct no two lanes touch the same element in one step, which makes the sum order fixed
// and the result bit-identical to the CPU loop.  A bit per column records which elements were
// touched.  The strip is then swept in column order, which yields the sorted row without
// sorting: every lane owns a run of consecutive columns (its words of the bit map), counts the
// touched elements of its run that are not zero, a prefix sum over the lanes turns the counts
// into output positions, and the lane writes its entries.  Touched elements are set back to
// zero as they are read, so the strip is cleared once per workgroup and the cost of a strip
// follows the entries it produces, not its width.  The same kernel runs twice: once to count
// the entries of every row (the caller then allocates), once to write them.
//
// Matrices wider than two strips: rows with few products (A's row at most 64 entries, at most
// 256 products) go to SpgemmHashKernel, which keeps the row in a hash table instead and whose
// cost does not depend on the width; the strip kernel then takes only the remaining rows.
//
// Requirements on the operands: column indices of B below N and distinct within a row;
// column indices of A below the row count of B.
#include "sph_internal.h"

#include <algorithm>

#pragma clang fp contract(off)

namespace
{
constexpr uint32_t kStripMax = 4096;  // columns per LDS strip
constexpr uint32_t kAhead = 8;        // rows of B whose first 64 entries are in flight together
constexpr uint32_t kRowsPerTurnMax = 8;  // consecutive output rows a wavefront takes at a time
constexpr uint32_t kWordsPerLaneMax = kStripMax / 32 / 64;  // bit-map words a lane owns
// Wide matrices (more than one strip): rows with few products go through a hash table instead
constexpr uint32_t kHashSlots = 512;            // power of two
constexpr uint32_t kHashProducts = kHashSlots / 2;  // a row with at most this many products is "light"
constexpr uint32_t kEmpty = 0xffffffffu;
// two strips still cost less than the table and its sort (8192 columns, 8 entries per row on
// both sides: 82 us on strips, 96 us through the table); from three strips on the table wins
constexpr uint32_t kHashFromWidth = 2 * kStripMax;
static_assert(kHashSlots == 512, "the hash takes the top 9 bits of a product");
static_assert(kWordsPerLaneMax <= 4, "the sweep takes a lane's words as two pairs");

struct SpgemmArgs
{
    const float* VA;
    const uint32_t* COLA;
    const uint32_t* ROWA;
    const float* VB;
    const uint32_t* COLB;
    const uint32_t* ROWB;
    uint32_t M, K, N;
    uint32_t strip;  // columns per strip (multiple of 64)
    uint32_t rowsPerTurn;  // 1 .. kRowsPerTurnMax
    uint32_t heavyOnly;    // strip kernel: leave the rows SpgemmHashKernel takes alone
    // count pass: counts (M + 1 entries, counts[M] = 0).  fill pass: ROWC, VC, COLC.
    // stage pass: counts as in the count pass, and row r's entries into VC / COLC at
    // r * slot .. r * slot + slot - 1 (what does not fit is counted and dropped).
    uint32_t* counts;
    const uint32_t* ROWC;
    float* VC;
    uint32_t* COLC;
    uint32_t slot;      // stage pass: entries per staging slot
    uint32_t skipUpTo;  // fill pass: rows with at most this many entries are left alone
    uint32_t capacity;  // fill pass: nothing is stored at or past this index
    // stage pass: cleared; the move kernel sets it when a row did not fit its slot; a fill
    // pass that is given it returns at once while it is zero
    uint32_t* overflow;
};

// what a pass of the two product kernels does with a row's entries
constexpr int kCount = 0, kFill = 1, kStage = 2;

__device__ __forceinline__ uint32_t Uniform(uint32_t v, uint32_t lane)
{
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane));
}

__device__ __forceinline__ float Uniform(float v, uint32_t lane)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), static_cast<int>(lane)));
}

__device__ __forceinline__ void Touch(uint32_t* bits, uint32_t column)
{
    __hip_atomic_fetch_or(&bits[column >> 5], 1u << (column & 31), __ATOMIC_RELAXED,
                          __HIP_MEMORY_SCOPE_WORKGROUP);
}

__device__ __forceinline__ uint32_t WaveSum(uint32_t v)
{
#pragma unroll
    for (uint32_t d = 1; d < 64; d *= 2)
        v += __shfl_xor(v, d, 64);
    return v;
}

// A row is light when A's row has at most 64 entries and the rows of B they select hold at
// most kHashProducts entries together.  Both kernels decide from these two numbers.
__device__ __forceinline__ bool LightRow(uint32_t entriesOfA, uint32_t products)
{
    return entriesOfA <= 64 && products <= kHashProducts;
}

// Light rows of a wide product.  The strip kernel walks all products of a row once per strip
// of 4096 columns, which is wasted on a row whose few products fall into a matrix of, say,
// 65536 columns.  Here a wavefront keeps the row in an LDS hash table keyed by column instead
// (the design the reference sketches, SparseGemm.cuh:16-36): the products are generated in the
// same order as in the strip kernel -- A's entries in storage order, the entries of one row of
// B across the lanes, so no two lanes of a step hold the same column -- a lane finds or claims
// (compare-and-swap on the key) the slot of its column and adds into it, which keeps the sum
// order of every element fixed.  Claimed slots are listed as they are claimed; at the end of
// the row the listed (column, sum) pairs are sorted by column (bitonic, in LDS), sums that are
// exactly zero are dropped, and the table is reset through the list.  The cost of a row follows
// its products, not the width of the matrix.
template <int MODE>
__global__ __launch_bounds__(64) void SpgemmHashKernel(const SpgemmArgs args)
{
    constexpr bool FILL = MODE != kCount;    // entries are stored
    constexpr bool COUNTS = MODE != kFill;   // counts are stored
    if (MODE == kFill && args.overflow != nullptr && *args.overflow == 0)
        return;  // every row is in place already
    __shared__ uint32_t keys[kHashSlots];
    __shared__ float sums[kHashSlots];
    __shared__ uint32_t sortKey[kHashProducts];  // first the list of claimed slots, then columns
    __shared__ float sortVal[kHashProducts];
    const uint32_t lane = threadIdx.x;
    const uint64_t below = (1ull << lane) - 1ull;
    for (uint32_t t = lane; t < kHashSlots; t += 64)
    {
        keys[t] = kEmpty;
        sums[t] = 0.0f;
    }

    // A wavefront takes rows blockIdx.x, blockIdx.x + gridDim.x, ... in turns of up to 64: their
    // extents are read in one go (one row per lane), and the loads that lead to a row's
    // products form a pipeline over the rows of the turn: while row i is multiplied, the
    // entries of A's row i+2 and the extents of the rows of B that row i+1 selects are on
    // their way.
    for (uint64_t first = blockIdx.x; first < args.M; first += 64ull * gridDim.x)
    {
        const uint64_t mine = first + static_cast<uint64_t>(lane) * gridDim.x;
        const uint32_t rowsHere = static_cast<uint32_t>(
            min(static_cast<uint64_t>(64), (args.M - first + gridDim.x - 1) / gridDim.x));
        uint32_t extentBegin = 0, extentEnd = 0, outBegin = 0, outEnd = 0;
        if (mine < args.M)
        {
            extentBegin = args.ROWA[mine];
            extentEnd = args.ROWA[mine + 1];
            if (MODE == kFill)
            {
                outBegin = args.ROWC[mine];
                outEnd = args.ROWC[mine + 1];
            }
            if (MODE == kStage)
            {
                outBegin = static_cast<uint32_t>(mine) * args.slot;
                outEnd = outBegin + args.slot;
            }
        }
        if (MODE == kFill && args.skipUpTo != 0 &&
            __ballot(mine < args.M && outEnd - outBegin > args.skipUpTo) == 0)
            continue;  // all of these rows are in place already
        // stage 1: this lane's entry of A's row i (rows with more than 64 entries are not ours)
        auto loadStage1 = [&](uint32_t i, uint32_t& k, float& value) {
            k = kEmpty;
            value = 0.0f;
            if (i < rowsHere)
            {
                const uint32_t begin = Uniform(extentBegin, i), end = Uniform(extentEnd, i);
                if (end - begin <= 64 && begin + lane < end)
                {
                    k = args.COLA[begin + lane];
                    value = args.VA[begin + lane];
                }
            }
        };
        // stage 2: the extent of the row of B that entry selects
        auto loadStage2 = [&](uint32_t k, uint32_t& begin, uint32_t& end) {
            begin = 0;
            end = 0;
            if (k < args.K)
            {
                begin = args.ROWB[k];
                end = args.ROWB[k + 1];
            }
        };
        uint32_t k1, k2, nextBegin, nextEnd;
        float value1, value2;
        loadStage1(0, k2, value2);
        loadStage2(k2, nextBegin, nextEnd);
        loadStage1(1, k1, value1);

      for (uint32_t i = 0; i < rowsHere; ++i)
      {
        const uint32_t row = static_cast<uint32_t>(first + static_cast<uint64_t>(i) * gridDim.x);
        const uint32_t entriesOfA = Uniform(extentEnd, i) - Uniform(extentBegin, i);
        const uint32_t bBegin = nextBegin, bEnd = nextEnd;
        const float aValue = value2;
        k2 = k1;
        value2 = value1;
        loadStage2(k2, nextBegin, nextEnd);
        loadStage1(i + 2, k1, value1);
        if (!LightRow(entriesOfA, WaveSum(bEnd - bBegin)))
            continue;  // heavy: the strip kernel's row
        if (MODE == kFill && Uniform(outEnd, i) - Uniform(outBegin, i) <= args.skipUpTo)
            continue;  // already in place

        uint32_t listed = 0;  // claimed slots so far (uniform)
        for (uint32_t j0 = 0; j0 < entriesOfA; j0 += kAhead)
        {
            // the first 64 entries of kAhead rows of B are requested before the first is used
            uint32_t s[kAhead], e[kAhead], col[kAhead];
            float a[kAhead], b[kAhead];
#pragma unroll
            for (uint32_t u = 0; u < kAhead; ++u)
            {
                const uint32_t j = min(j0 + u, 63u);
                s[u] = Uniform(bBegin, j);
                e[u] = j0 + u < entriesOfA ? Uniform(bEnd, j) : s[u];
                a[u] = Uniform(aValue, j);
            }
#pragma unroll
            for (uint32_t u = 0; u < kAhead; ++u)
            {
                col[u] = kEmpty;
                b[u] = 0.0f;
                if (s[u] + lane < e[u])
                {
                    col[u] = args.COLB[s[u] + lane];
                    b[u] = args.VB[s[u] + lane];
                }
            }
            // one product per lane: find or claim the column's slot and add into it
            auto insert = [&](uint32_t c, float product, bool have) {
                bool claimed = false;
                uint32_t h = 0;
                if (have)
                {
                    h = (c * 2654435761u) >> 23;  // top 9 bits: kHashSlots = 512
                    for (uint32_t tries = 0; tries < kHashSlots; ++tries)
                    {
                        const uint32_t k = keys[h];
                        if (k == c)
                            break;
                        if (k == kEmpty)
                        {
                            const uint32_t old = atomicCAS(&keys[h], kEmpty, c);
                            if (old == kEmpty)
                            {
                                claimed = true;
                                break;
                            }
                            if (old == c)
                                break;
                        }
                        h = (h + 1) & (kHashSlots - 1);
                    }
                    sums[h] = sums[h] + product;
                }
                const uint64_t m = __ballot(claimed);
                if (claimed)
                    sortKey[listed + static_cast<uint32_t>(__popcll(m & below))] = h;
                listed += static_cast<uint32_t>(__popcll(m));
            };
#pragma unroll
            for (uint32_t u = 0; u < kAhead; ++u)
            {
                insert(col[u], a[u] * b[u], col[u] < args.N);
                // rows of B with more than 64 entries: the rest, 64 at a time
                for (uint32_t pb0 = s[u] + 64; pb0 < e[u]; pb0 += 64)
                {
                    const bool have = pb0 + lane < e[u];
                    const uint32_t c = have ? args.COLB[pb0 + lane] : kEmpty;
                    const float bv = have ? args.VB[pb0 + lane] : 0.0f;
                    insert(c, a[u] * bv, have && c < args.N);
                }
            }
        }

        uint32_t emitted = 0;
        const uint32_t rowBase = FILL ? Uniform(outBegin, i) : 0u;
        const uint32_t rowLimit =
            MODE == kFill ? min(Uniform(outEnd, i), args.capacity) : FILL ? Uniform(outEnd, i) : 0u;
        if (listed <= 64)
        {
            // one (column, sum) pair per lane: sorted in registers with cross-lane exchanges
            uint32_t c = kEmpty;
            float v = 0.0f;
            if (lane < listed)
            {
                const uint32_t h = sortKey[lane];
                c = keys[h];
                v = sums[h];
                keys[h] = kEmpty;
                sums[h] = 0.0f;
            }
#pragma unroll
            for (uint32_t size = 2; size <= 64; size *= 2)
#pragma unroll
                for (uint32_t stride = size / 2; stride > 0; stride /= 2)
                {
                    const uint32_t oc = __shfl_xor(c, stride, 64);
                    const float ov = __shfl_xor(v, stride, 64);
                    // in an ascending run the lower lane of a pair keeps the smaller column
                    const bool wantsSmaller = ((lane & stride) == 0) == ((lane & size) == 0);
                    const bool takeOther = wantsSmaller ? oc < c : oc > c;
                    c = takeOther ? oc : c;
                    v = takeOther ? ov : v;
                }
            const bool keep = c != kEmpty && v != 0.0f;  // exact zeros are not stored
            const uint64_t m = __ballot(keep);
            if (FILL)
            {
                const uint32_t at = rowBase + static_cast<uint32_t>(__popcll(m & below));
                if (keep && at < rowLimit)
                {
                    args.VC[at] = v;
                    args.COLC[at] = c;
                }
            }
            emitted = static_cast<uint32_t>(__popcll(m));
        }
        else
        {
            // the listed slots become (column, sum) pairs, and the table is empty again
            uint32_t padded = 64;
            while (padded < listed)
                padded *= 2;
            for (uint32_t q = lane; q < padded; q += 64)
            {
                uint32_t c = kEmpty;
                float v = 0.0f;
                if (q < listed)
                {
                    const uint32_t h = sortKey[q];
                    c = keys[h];
                    v = sums[h];
                    keys[h] = kEmpty;
                    sums[h] = 0.0f;
                }
                sortKey[q] = c;
                sortVal[q] = v;
            }
            // bitonic sort by column; the padding (kEmpty) ends up behind the entries
            for (uint32_t size = 2; size <= padded; size *= 2)
                for (uint32_t stride = size / 2; stride > 0; stride /= 2)
                    for (uint32_t t = lane; t < padded / 2; t += 64)
                    {
                        const uint32_t lo = 2 * t - (t & (stride - 1));  // lower index of pair t
                        const uint32_t hi = lo + stride;
                        const bool ascending = (lo & size) == 0;
                        const uint32_t kLo = sortKey[lo], kHi = sortKey[hi];
                        if ((kLo > kHi) == ascending)
                        {
                            const float vLo = sortVal[lo], vHi = sortVal[hi];
                            sortKey[lo] = kHi;
                            sortKey[hi] = kLo;
                            sortVal[lo] = vHi;
                            sortVal[hi] = vLo;
                        }
                    }
            // entries in column order; sums that are exactly zero are not stored
            for (uint32_t i0 = 0; i0 < listed; i0 += 64)
            {
                const uint32_t x = i0 + lane;
                const float v = x < listed ? sortVal[x] : 0.0f;
                const bool keep = v != 0.0f;
                const uint64_t m = __ballot(keep);
                if (FILL)
                {
                    const uint32_t at = rowBase + emitted + static_cast<uint32_t>(__popcll(m & below));
                    if (keep && at < rowLimit)
                    {
                        args.VC[at] = v;
                        args.COLC[at] = sortKey[x];
                    }
                }
                emitted += static_cast<uint32_t>(__popcll(m));
            }
        }
        if (COUNTS && lane == 0)
            args.counts[row] = emitted;
      }
    }
}

template <int MODE>
__global__ __launch_bounds__(64) void SpgemmRowKernel(const SpgemmArgs args)
{
    constexpr bool FILL = MODE != kCount;    // entries are stored
    constexpr bool COUNTS = MODE != kFill;   // counts are stored
    extern __shared__ float strip[];
    // one bit per column, after the strip; lane l owns words l*wordsPerLane .. +wordsPerLane-1
    uint32_t* bits = reinterpret_cast<uint32_t*>(strip + args.strip);
    const uint32_t wordsInStrip = args.strip / 32;
    const uint32_t wordsPerLane = (wordsInStrip + 63) / 64;  // at most kStripMax / 2048
    const uint32_t lane = threadIdx.x;
    if (MODE == kFill && args.overflow != nullptr && *args.overflow == 0)
        return;  // every row is in place already
    if (COUNTS && blockIdx.x == 0 && lane == 0)
        args.counts[args.M] = 0;
    if (MODE == kStage && blockIdx.x == 0 && lane == 0)
        *args.overflow = 0;
    // cleared once; every block that is touched is cleared again when it is swept
    for (uint32_t x = lane; x < args.strip; x += 64)
        strip[x] = 0.0f;
    for (uint32_t t = lane; t < wordsInStrip; t += 64)
        bits[t] = 0;

    // A wavefront takes rowsPerTurn consecutive rows per turn.  Their extents are read in one
    // go, and the loads that lead to a row's products form a pipeline over the rows of the
    // turn: while row i is multiplied, the first 64 (column, value) pairs of A's row i+2 and
    // the extents of the rows of B that row i+1 needs are already on their way.
    for (uint32_t turn = blockIdx.x * args.rowsPerTurn; turn < args.M;
         turn += gridDim.x * args.rowsPerTurn)
    {
        const uint32_t rowsHere = min(args.rowsPerTurn, args.M - turn);
        uint32_t extentA = 0, extentC = 0;
        if (lane <= rowsHere)
        {
            extentA = args.ROWA[turn + lane];
            if (MODE == kFill)
                extentC = args.ROWC[turn + lane];
            if (MODE == kStage)
                extentC = (turn + lane) * args.slot;
        }
        if (MODE == kFill && args.skipUpTo != 0)
        {
            const uint32_t nextC = __shfl_down(extentC, 1, 64);
            if (__ballot(lane < rowsHere && nextC - extentC > args.skipUpTo) == 0)
                continue;  // all rows of this turn are in place already
        }
        // stage 1 (columns and values of A's row) and stage 2 (extents in B) of the pipeline
        auto loadStage1 = [&](uint32_t i, uint32_t& k, float& value) {
            k = 0xffffffffu;
            value = 0.0f;
            if (i < rowsHere)
            {
                const uint32_t begin = Uniform(extentA, i), end = Uniform(extentA, i + 1);
                if (begin + lane < end)
                {
                    k = args.COLA[begin + lane];
                    value = args.VA[begin + lane];
                }
            }
        };
        auto loadStage2 = [&](uint32_t k, uint32_t& bBegin, uint32_t& bEnd) {
            bBegin = 0;
            bEnd = 0;
            if (k < args.K)
            {
                bBegin = args.ROWB[k];
                bEnd = args.ROWB[k + 1];
            }
        };
        uint32_t k1, k2, nextBegin, nextEnd;
        float value1, value2;
        loadStage1(0, k2, value2);
        loadStage2(k2, nextBegin, nextEnd);
        loadStage1(1, k1, value1);

      for (uint32_t i = 0; i < rowsHere; ++i)
      {
        const uint32_t aBegin = Uniform(extentA, i);
        const uint32_t aEnd = Uniform(extentA, i + 1);
        uint32_t emitted = 0;  // entries of this row found so far (all strips)
        const uint32_t rowBase = FILL ? Uniform(extentC, i) : 0u;
        const uint32_t rowEnd = FILL ? Uniform(extentC, i + 1) : 0u;
        const uint32_t rowLimit = MODE == kFill ? min(rowEnd, args.capacity) : rowEnd;
        // this row's first batch comes out of the pipeline, which then moves on
        const uint32_t firstBegin = nextBegin, firstEnd = nextEnd;
        const float firstValue = value2;
        k2 = k1;
        value2 = value1;
        loadStage2(k2, nextBegin, nextEnd);
        loadStage1(i + 2, k1, value1);
        // in a wide product the light rows belong to SpgemmHashKernel
        if (args.heavyOnly != 0 && LightRow(aEnd - aBegin, WaveSum(firstEnd - firstBegin)))
            continue;
        if (MODE == kFill && rowEnd - rowBase <= args.skipUpTo)
            continue;  // already in place

        for (uint32_t c0 = 0; c0 < args.N; c0 += args.strip)
        {
            const uint32_t width = min(args.strip, args.N - c0);

            for (uint32_t pa0 = aBegin; pa0 < aEnd; pa0 += 64)
            {
                // up to 64 entries of A's row, one per lane, with the extent of their rows of B
                const uint32_t have = min(64u, aEnd - pa0);
                uint32_t bBegin = firstBegin, bEnd = firstEnd;
                float aValue = firstValue;
                if (pa0 != aBegin)
                {
                    bBegin = 0;
                    bEnd = 0;
                    aValue = 0.0f;
                    if (lane < have)
                    {
                        const uint32_t k = args.COLA[pa0 + lane];
                        aValue = args.VA[pa0 + lane];
                        if (k < args.K)
                        {
                            bBegin = args.ROWB[k];
                            bEnd = args.ROWB[k + 1];
                        }
                    }
                }
                // the entries are applied in order; the first 64 entries of kAhead rows of B
                // are requested before the first of them is used
                for (uint32_t j0 = 0; j0 < have; j0 += kAhead)
                {
                    uint32_t s[kAhead], e[kAhead], col[kAhead];
                    float a[kAhead], b[kAhead];
#pragma unroll
                    for (uint32_t u = 0; u < kAhead; ++u)
                    {
                        const uint32_t j = min(j0 + u, 63u);
                        s[u] = Uniform(bBegin, j);
                        e[u] = j0 + u < have ? Uniform(bEnd, j) : s[u];
                        a[u] = Uniform(aValue, j);
                    }
#pragma unroll
                    for (uint32_t u = 0; u < kAhead; ++u)
                    {
                        col[u] = 0xffffffffu;
                        b[u] = 0.0f;
                        if (s[u] + lane < e[u])
                        {
                            col[u] = args.COLB[s[u] + lane];
                            b[u] = args.VB[s[u] + lane];
                        }
                    }
#pragma unroll
                    for (uint32_t u = 0; u < kAhead; ++u)
                    {
                        if (col[u] - c0 < width)  // also false for the 0xffffffff of idle lanes
                        {
                            strip[col[u] - c0] = strip[col[u] - c0] + a[u] * b[u];
                            Touch(bits, col[u] - c0);
                        }
                        // rows of B with more than 64 entries: the rest, 64 at a time
                        for (uint32_t pb = s[u] + 64 + lane; pb < e[u]; pb += 64)
                        {
                            const uint32_t c = args.COLB[pb];
                            if (c - c0 < width)
                            {
                                strip[c - c0] = strip[c - c0] + a[u] * args.VB[pb];
                                Touch(bits, c - c0);
                            }
                        }
                    }
                }
            }

            // sweep: this lane's touched columns in ascending order, as two 64-column runs
            // (a pair of bit-map words each)
            auto fetchPair = [&](uint32_t first) {
                uint32_t lo = 0, hi = 0;
                const uint32_t w = lane * wordsPerLane + first;
                if (first < wordsPerLane && w < wordsInStrip)
                {
                    lo = bits[w];
                    if (lo != 0)
                        bits[w] = 0;
                }
                if (first + 1 < wordsPerLane && w + 1 < wordsInStrip)
                {
                    hi = bits[w + 1];
                    if (hi != 0)
                        bits[w + 1] = 0;
                }
                return (static_cast<uint64_t>(hi) << 32) | lo;
            };
            const uint64_t mine0 = fetchPair(0);
            const uint64_t mine1 = fetchPair(2);
            const uint32_t base0 = lane * wordsPerLane * 32;  // first column of run 0
            const uint32_t base1 = base0 + 64;

            // next touched column of this lane's runs, removed from the set
            auto take = [&](uint64_t& set0, uint64_t& set1) {
                if (set0 != 0)
                {
                    const uint32_t b = static_cast<uint32_t>(__builtin_ctzll(set0));
                    set0 &= set0 - 1;
                    return base0 + b;
                }
                const uint32_t b = static_cast<uint32_t>(__builtin_ctzll(set1));
                set1 &= set1 - 1;
                return base1 + b;
            };
            // pass 1: how many of them hold a value that is not zero (the count pass
            // clears them here; the fill pass needs them once more)
            uint32_t kept = 0;
            {
                uint64_t set0 = mine0, set1 = mine1;
                while ((set0 | set1) != 0)
                {
                    const uint32_t x = take(set0, set1);
                    if (strip[x] != 0.0f)
                        ++kept;
                    if (!FILL)
                        strip[x] = 0.0f;  // the storing passes read it once more below
                }
            }
            // positions: exclusive prefix sum of `kept` over the lanes
            uint32_t inclusive = kept;
#pragma unroll
            for (uint32_t d = 1; d < 64; d *= 2)
            {
                const uint32_t other = __shfl_up(inclusive, d, 64);
                if (lane >= d)
                    inclusive += other;
            }
            if (FILL)
            {
                uint32_t at = rowBase + emitted + inclusive - kept;
                uint64_t set0 = mine0, set1 = mine1;
                while ((set0 | set1) != 0)
                {
                    const uint32_t x = take(set0, set1);
                    const float v = strip[x];
                    strip[x] = 0.0f;
                    if (v != 0.0f)
                    {
                        if (at < rowLimit)
                        {
                            args.VC[at] = v;
                            args.COLC[at] = c0 + x;
                        }
                        ++at;
                    }
                }
            }
            emitted += Uniform(inclusive, 63);
        }
        if (COUNTS && lane == 0)
            args.counts[turn + i] = emitted;
      }
    }
}

// Staged rows move to their place: row r's ROWC[r + 1] - ROWC[r] entries from r * slot.  Rows
// that did not fit their slot are left to a fill pass.  One wavefront per row, 4 per workgroup.
__global__ __launch_bounds__(256) void SpgemmUnstageKernel(float* __restrict__ VC,
                                                           uint32_t* __restrict__ COLC,
                                                           const uint32_t* __restrict__ ROWC,
                                                           const float* __restrict__ stageV,
                                                           const uint32_t* __restrict__ stageCol,
                                                           uint32_t M, uint32_t slot,
                                                           uint32_t capacity, uint32_t* overflow)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M)
        return;
    const uint32_t first = ROWC[row];
    const uint32_t count = ROWC[row + 1] - first;
    if (count > slot)
    {
        if (lane == 0)
            *overflow = 1;
        return;
    }
    const size_t from = static_cast<size_t>(row) * slot;
    for (uint32_t i = lane; i < count; i += 64)
        if (first + i < capacity)
        {
            VC[first + i] = stageV[from + i];
            COLC[first + i] = stageCol[from + i];
        }
}

// load[p] = entries of the row of B that entry p of A selects (the multiplications entry p
// causes); *total (when given, zero before the launch) receives their sum.
__global__ __launch_bounds__(256) void SpgemmLoadKernel(uint32_t* __restrict__ load,
                                                        const uint32_t* __restrict__ COLA,
                                                        const uint32_t* __restrict__ ROWB,
                                                        uint32_t entries, uint32_t K,
                                                        unsigned long long* total)
{
    unsigned long long sum = 0;
    for (uint64_t p = blockIdx.x * 256ull + threadIdx.x; p < entries; p += 256ull * gridDim.x)
    {
        const uint32_t k = COLA[p];
        const uint32_t n = k < K ? ROWB[k + 1] - ROWB[k] : 0u;
        if (load != nullptr)
            load[p] = n;
        sum += n;
    }
    if (total == nullptr)
        return;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1)
        sum += __shfl_xor(sum, d, 64);
    if ((threadIdx.x & 63u) == 0 && sum != 0)
        atomicAdd(total, sum);
}

__global__ void ClearTotalKernel(unsigned long long* total)
{
    *total = 0;
}

uint32_t StripFor(uint32_t N)
{
    const uint32_t padded = (N + 63u) / 64u * 64u;
    return std::max<uint32_t>(64u, std::min(padded, kStripMax));
}

// Rows per turn: long turns let the loads of consecutive rows overlap, short ones give a small
// matrix enough workgroups to fill the chip (about eight resident per compute unit).
uint32_t RowsPerTurnFor(uint32_t M)
{
    const uint32_t wanted = static_cast<uint32_t>(sph::ComputeUnits()) * 8;
    return std::max<uint32_t>(1, std::min<uint32_t>(kRowsPerTurnMax, M / std::max<uint32_t>(wanted, 1)));
}

// one wavefront per workgroup, rows dealt round robin; 6 KiB of LDS each
uint32_t HashGridFor(uint32_t M)
{
    const uint64_t cap = static_cast<uint64_t>(sph::ComputeUnits()) * 32;
    return static_cast<uint32_t>(std::max<uint64_t>(1, std::min<uint64_t>(M, cap)));
}

uint32_t GridFor(uint32_t M, uint32_t rowsPerTurn)
{
    const uint64_t cap = static_cast<uint64_t>(sph::ComputeUnits()) * 64;
    const uint64_t turns = (static_cast<uint64_t>(M) + rowsPerTurn - 1) / rowsPerTurn;
    return static_cast<uint32_t>(std::max<uint64_t>(1, std::min<uint64_t>(turns, cap)));
}
}  // namespace

extern "C" {

int sph_spgemm_row_offsets_f32(uint32_t* ROWC, const float* VA, const uint32_t* COLA,
                               const uint32_t* ROWA, const float* VB, const uint32_t* COLB,
                               const uint32_t* ROWB, uint32_t M, uint32_t K, uint32_t N,
                               uint32_t* nnzHost)
{
    SPH_REQUIRE(ROWC != nullptr && ROWA != nullptr, "null pointer");
    SPH_REQUIRE(M < 0xffffffffu, "too many rows");
    SPH_REQUIRE(K == 0 || ROWB != nullptr, "null pointer");
    if (sph::ScanWaitsOrAllocates(M + 1, nnzHost))
        SPH_REFUSE_WHILE_CAPTURING();  // before anything is enqueued into the graph
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    SpgemmArgs args{};
    args.VA = VA;
    args.COLA = COLA;
    args.ROWA = ROWA;
    args.VB = VB;
    args.COLB = COLB;
    args.ROWB = ROWB;
    args.M = M;
    args.K = K;
    args.N = N;
    args.strip = StripFor(N);
    args.rowsPerTurn = RowsPerTurnFor(M);
    args.counts = ROWC;
    args.heavyOnly = N > kHashFromWidth ? 1u : 0u;
    if (args.heavyOnly != 0 && M != 0)
        hipLaunchKernelGGL(SpgemmHashKernel<kCount>, dim3(HashGridFor(M)), dim3(64), 0, stream, args);
    hipLaunchKernelGGL(SpgemmRowKernel<kCount>, dim3(GridFor(M, args.rowsPerTurn)), dim3(64),
                       args.strip * sizeof(float) + args.strip / 8, stream, args);
    SPH_CHECK_LAUNCH();
    return sph::ExclusiveScanInPlace(ROWC, M + 1, nnzHost, stream);
}

int sph_spgemm_fill_f32(float* VC, uint32_t* COLC, const uint32_t* ROWC, const float* VA,
                        const uint32_t* COLA, const uint32_t* ROWA, const float* VB,
                        const uint32_t* COLB, const uint32_t* ROWB, uint32_t M, uint32_t K,
                        uint32_t N)
{
    if (M == 0 || N == 0)
        return SPH_OK;
    SPH_REQUIRE(ROWC != nullptr && ROWA != nullptr, "null pointer");
    SPH_REQUIRE(K == 0 || ROWB != nullptr, "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    SpgemmArgs args{};
    args.VA = VA;
    args.COLA = COLA;
    args.ROWA = ROWA;
    args.VB = VB;
    args.COLB = COLB;
    args.ROWB = ROWB;
    args.M = M;
    args.K = K;
    args.N = N;
    args.strip = StripFor(N);
    args.rowsPerTurn = RowsPerTurnFor(M);
    args.ROWC = ROWC;
    args.VC = VC;
    args.COLC = COLC;
    args.capacity = 0xffffffffu;
    args.heavyOnly = N > kHashFromWidth ? 1u : 0u;
    if (args.heavyOnly != 0)
        hipLaunchKernelGGL(SpgemmHashKernel<kFill>, dim3(HashGridFor(M)), dim3(64), 0, stream, args);
    hipLaunchKernelGGL(SpgemmRowKernel<kFill>, dim3(GridFor(M, args.rowsPerTurn)), dim3(64),
                       args.strip * sizeof(float) + args.strip / 8, stream, args);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_spgemm_load_u32(uint32_t* load, const uint32_t* COLA, const uint32_t* ROWB,
                        uint32_t entries, uint32_t K, uint64_t* productsHost)
{
    SPH_REQUIRE(entries == 0 || COLA != nullptr, "COLA is null");
    SPH_REQUIRE(entries == 0 || K == 0 || ROWB != nullptr, "ROWB is null");
    if (productsHost != nullptr)
        SPH_REFUSE_WHILE_CAPTURING();  // reads back and takes a scratch word
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    if (entries == 0)
    {
        if (productsHost != nullptr)
            *productsHost = 0;
        return SPH_OK;
    }
    unsigned long long* total = nullptr;
    if (productsHost != nullptr)
    {
        ::sph::CountAllocation();
        SPH_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&total), sizeof(*total), stream));
        hipLaunchKernelGGL(ClearTotalKernel, dim3(1), dim3(1), 0, stream, total);
    }
    const uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>(
        (static_cast<uint64_t>(entries) + 255) / 256, static_cast<uint64_t>(sph::ComputeUnits()) * 8));
    hipLaunchKernelGGL(SpgemmLoadKernel, dim3(blocks), dim3(256), 0, stream, load, COLA, ROWB,
                       entries, K, total);
    const hipError_t launched = hipGetLastError();
    hipError_t copied = hipSuccess;
    if (launched == hipSuccess && productsHost != nullptr)
    {
        static_assert(sizeof(unsigned long long) == sizeof(uint64_t), "64-bit total");
        copied = hipMemcpyAsync(productsHost, total, sizeof(uint64_t), hipMemcpyDeviceToHost, stream);
        if (copied == hipSuccess)
            copied = hipStreamSynchronize(stream);
    }
    if (total != nullptr)
        SPH_HIP_TRY(hipFreeAsync(total, stream));
    if (launched != hipSuccess)
        return sph::Fail(SPH_ERR_DEVICE, std::string("sph_spgemm_load_u32 - launch failed with ") +
                                             hipGetErrorString(launched));
    SPH_HIP_TRY(copied);
    return SPH_OK;
}

int sph_spgemm_f32(float* VC, uint32_t* COLC, uint32_t* ROWC, uint32_t capacity, const float* VA,
                   const uint32_t* COLA, const uint32_t* ROWA, const float* VB,
                   const uint32_t* COLB, const uint32_t* ROWB, uint32_t M, uint32_t K, uint32_t N,
                   uint32_t* nnzHost)
{
    SPH_REQUIRE(ROWC != nullptr && ROWA != nullptr, "null pointer");
    SPH_REQUIRE(M < 0xffffffffu, "too many rows");
    SPH_REQUIRE(K == 0 || ROWB != nullptr, "null pointer");
    SPH_REQUIRE(capacity == 0 || (VC != nullptr && COLC != nullptr), "VC or COLC is null");
    SPH_REFUSE_WHILE_CAPTURING();  // takes a scratch allocation; before anything is enqueued
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    SpgemmArgs args{};
    args.VA = VA;
    args.COLA = COLA;
    args.ROWA = ROWA;
    args.VB = VB;
    args.COLB = COLB;
    args.ROWB = ROWB;
    args.M = M;
    args.K = K;
    args.N = N;
    args.strip = StripFor(N);
    args.rowsPerTurn = RowsPerTurnFor(M);
    args.counts = ROWC;
    args.heavyOnly = N > kHashFromWidth ? 1u : 0u;
    const dim3 hashGrid(HashGridFor(M)), rowGrid(GridFor(M, args.rowsPerTurn)), wave(64);
    const size_t rowLds = args.strip * sizeof(float) + args.strip / 8;

    // staging slot per row: twice the mean the capacity allows plus 64; without room for that
    // (or without rows) the count, scan and fill passes run one after the other
    const uint64_t slot = M != 0 ? 2 * static_cast<uint64_t>(capacity / M) + 64 : 0;
    const bool staged = M != 0 && N != 0 && capacity != 0 && slot * M < (1ull << 31);
    float* stageV = nullptr;
    if (staged)
    {
        ::sph::CountAllocation();
        SPH_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&stageV), slot * M * 8 + 4, stream));
        args.VC = stageV;
        args.COLC = reinterpret_cast<uint32_t*>(stageV + slot * M);
        args.overflow = args.COLC + slot * M;
        args.slot = static_cast<uint32_t>(slot);
        if (args.heavyOnly != 0)
            hipLaunchKernelGGL(SpgemmHashKernel<kStage>, hashGrid, wave, 0, stream, args);
        hipLaunchKernelGGL(SpgemmRowKernel<kStage>, rowGrid, wave, rowLds, stream, args);
    }
    else
    {
        if (args.heavyOnly != 0 && M != 0)
            hipLaunchKernelGGL(SpgemmHashKernel<kCount>, hashGrid, wave, 0, stream, args);
        hipLaunchKernelGGL(SpgemmRowKernel<kCount>, rowGrid, wave, rowLds, stream, args);
    }
    hipError_t launched = hipGetLastError();
    int rc = SPH_OK;
    if (launched == hipSuccess)
        rc = sph::ExclusiveScanInPlace(ROWC, M + 1, nullptr, stream);
    if (launched == hipSuccess && rc == SPH_OK && M != 0 && N != 0 && capacity != 0)
    {
        if (staged)
            hipLaunchKernelGGL(SpgemmUnstageKernel, dim3((M + 3) / 4), dim3(256), 0, stream, VC,
                               COLC, ROWC, stageV, args.COLC, M, args.slot, capacity,
                               args.overflow);
        // rows that did not fit their slot (all rows, without staging) are multiplied again
        args.ROWC = ROWC;
        args.VC = VC;
        args.COLC = COLC;
        args.capacity = capacity;
        args.skipUpTo = staged ? args.slot : 0u;
        // after staging this pass usually finds nothing to do (it returns at once then), so it
        // is launched with few workgroups, which walk all rows if they must: dispatching the
        // full grid of empty workgroups alone took 15 us
        const uint32_t few = static_cast<uint32_t>(sph::ComputeUnits()) * 2;
        const dim3 fillHashGrid(staged ? std::min(hashGrid.x, few) : hashGrid.x);
        const dim3 fillRowGrid(staged ? std::min(rowGrid.x, few) : rowGrid.x);
        if (args.heavyOnly != 0)
            hipLaunchKernelGGL(SpgemmHashKernel<kFill>, fillHashGrid, wave, 0, stream, args);
        hipLaunchKernelGGL(SpgemmRowKernel<kFill>, fillRowGrid, wave, rowLds, stream, args);
        launched = hipGetLastError();
    }
    if (stageV != nullptr)
        SPH_HIP_TRY(hipFreeAsync(stageV, stream));
    if (launched != hipSuccess)
        return sph::Fail(SPH_ERR_DEVICE, std::string("sph_spgemm_f32 - launch failed with ") +
                                             hipGetErrorString(launched));
    if (rc != SPH_OK)
        return rc;
    if (nnzHost != nullptr)
    {
        SPH_HIP_TRY(hipMemcpyAsync(nnzHost, ROWC + M, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                   stream));
        SPH_HIP_TRY(hipStreamSynchronize(stream));
    }
    return SPH_OK;
}

}  // extern "C"
