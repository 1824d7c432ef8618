// Dense <-> CSR conversion on the device.
//
// The container is the reference's SparseMatrix
// (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:28-38); the reference declares the two
// conversions (Includes/Sapphire/compute/sparse/Sparse.hpp:150-160,
// CreateSparseMatrixWithDenseMatrix / ConvertSparseMatrixToDenseMatrix over matrices of m
// rows, n columns and a row pitch of paddedN floats) and defines neither.  An entry is kept
// when its value compares unequal to zero (so -0.0 is dropped and NaN is kept); entries of a
// row are stored in ascending column order.
//
// All of this is one- or two-pass integer/byte work bound by HBM:
//   row offsets   read the dense matrix once, popcount per row, exclusive scan of M+1 counts
//   fill          read it again, ballot + popcount give every kept entry its slot
//   to dense      one wavefront per row clears it and writes its entries over the zeros
// A row is handled by a group of LPR lanes (a power of two, 4..64, chosen from the row
// length) so that narrow matrices do not idle most of a wavefront; each lane takes 4
// consecutive columns (16 bytes) per step.
#include "sph_internal.h"

#include <algorithm>
#include <mutex>

namespace
{
constexpr int kThreads = 256;

// Block totals of the row-offset scan for sph_csr_row_offsets_noalloc_f32: one 32-bit total
// per 4096 counts, 4096 totals = 16 KiB per device for the life of the process.  In host code
// this name is only a handle for hipGetSymbolAddress; kernels get the resolved pointer.
constexpr uint32_t kNoAllocMaxBlocks = 4096;
static __device__ __align__(256) uint32_t scratch[kNoAllocMaxBlocks];

constexpr int kMaxScratchDevices = 16;
std::mutex gScratchMutex;
uint32_t* gScratchPtr[kMaxScratchDevices] = {};

struct DenseView
{
    const float* data;
    uint32_t M, N, ld;
};

// 4 consecutive columns of one row; columns past N read as 0
__device__ __forceinline__ float4 LoadQuad(const DenseView& d, uint32_t row, uint32_t col,
                                           bool rowOk)
{
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (rowOk && col < d.N)
    {
        const float* p = d.data + static_cast<size_t>(row) * d.ld + col;
        // four columns that all exist: one 16-byte access, which only asks for 4-byte alignment
        if (col + 4 <= d.N)
        {
            typedef float floatx4 __attribute__((ext_vector_type(4)));
            typedef floatx4 floatx4a4 __attribute__((aligned(4)));
            const floatx4 w = *reinterpret_cast<const floatx4a4*>(p);
            v = make_float4(w[0], w[1], w[2], w[3]);
        }
        else
        {
            v.x = p[0];
            if (col + 1 < d.N) v.y = p[1];
            if (col + 2 < d.N) v.z = p[2];
            if (col + 3 < d.N) v.w = p[3];
        }
    }
    return v;
}

// counts[r] = number of entries != 0 in row r; counts[M] = 0 (the slot the scan turns into nnz)
template <int LPR>
__global__ __launch_bounds__(kThreads) void CsrCountKernel(uint32_t* __restrict__ counts,
                                                           const DenseView d)
{
    constexpr uint32_t kGroups = kThreads / LPR;
    const uint32_t lane = threadIdx.x % LPR;
    const uint32_t group = threadIdx.x / LPR;
    const uint32_t rowsPerPass = gridDim.x * kGroups;
    if (blockIdx.x == 0 && threadIdx.x == 0)
        counts[d.M] = 0;
    // every group of a wavefront runs the same number of passes and steps
    const uint32_t passes = (d.M + rowsPerPass - 1) / rowsPerPass;
    for (uint32_t pass = 0; pass < passes; ++pass)
    {
        const uint32_t row = pass * rowsPerPass + blockIdx.x * kGroups + group;
        const bool rowOk = row < d.M;
        uint32_t c = 0;
        for (uint32_t col = lane * 4; col < d.N; col += LPR * 4)
        {
            const float4 v = LoadQuad(d, row, col, rowOk);
            c += (v.x != 0.f) + (v.y != 0.f) + (v.z != 0.f) + (v.w != 0.f);
        }
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1)
            c += __shfl_xor(c, off, LPR);
        if (rowOk && lane == 0)
            counts[row] = c;
    }
}

// ---- exclusive scan of n uint32 in place, 4096 per workgroup -----------------------------
constexpr int kScanThreads = 1024;
constexpr int kScanPerBlock = kScanThreads * 4;
constexpr uint32_t kScanSingleLimit = 16 * kScanPerBlock;  // scanned by one workgroup

// exclusive scan of one value per thread across the workgroup; returns the prefix and leaves
// the workgroup total in `total`
__device__ __forceinline__ uint32_t BlockExclusiveScan(uint32_t value, uint32_t& total,
                                                       uint32_t* waveSums)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    uint32_t inclusive = value;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
    {
        const uint32_t up = __shfl_up(inclusive, off, 64);
        if (lane >= static_cast<uint32_t>(off))
            inclusive += up;
    }
    if (lane == 63)
        waveSums[wave] = inclusive;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kScanThreads / 64; ++w)
    {
        const uint32_t s = waveSums[w];
        if (static_cast<uint32_t>(w) < wave)
            before += s;
        all += s;
    }
    __syncthreads();  // waveSums may be reused by the caller's next round
    total = all;
    return before + inclusive - value;
}

__global__ __launch_bounds__(kScanThreads) void ScanBlocksKernel(uint32_t* __restrict__ data,
                                                                 uint32_t* __restrict__ blockSums,
                                                                 uint32_t n)
{
    __shared__ uint32_t waveSums[kScanThreads / 64];
    const size_t base = static_cast<size_t>(blockIdx.x) * kScanPerBlock + threadIdx.x * 4;
    uint32_t v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        v[e] = base + e < n ? data[base + e] : 0u;
    uint32_t total;
    uint32_t run = BlockExclusiveScan(v[0] + v[1] + v[2] + v[3], total, waveSums);
#pragma unroll
    for (int e = 0; e < 4; ++e)
    {
        if (base + e < n)
            data[base + e] = run;
        run += v[e];
    }
    if (threadIdx.x == 0 && blockSums != nullptr)
        blockSums[blockIdx.x] = total;
}

// one workgroup: exclusive scan of the per-block totals in place
__global__ __launch_bounds__(kScanThreads) void ScanSumsKernel(uint32_t* __restrict__ sums,
                                                               uint32_t count)
{
    __shared__ uint32_t waveSums[kScanThreads / 64];
    uint32_t carry = 0;
    for (uint32_t start = 0; start < count; start += kScanThreads)
    {
        const uint32_t i = start + threadIdx.x;
        const uint32_t v = i < count ? sums[i] : 0u;
        uint32_t total;
        const uint32_t prefix = BlockExclusiveScan(v, total, waveSums);
        if (i < count)
            sums[i] = carry + prefix;
        carry += total;
    }
}

// one workgroup: exclusive scan of n values in place, 4096 per round with a running carry
__global__ __launch_bounds__(kScanThreads) void ScanSingleKernel(uint32_t* __restrict__ data,
                                                                 uint32_t n)
{
    __shared__ uint32_t waveSums[kScanThreads / 64];
    uint32_t carry = 0;
    for (size_t start = 0; start < n; start += kScanPerBlock)
    {
        const size_t base = start + threadIdx.x * 4;
        uint32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            v[e] = base + e < n ? data[base + e] : 0u;
        uint32_t total;
        uint32_t run = carry + BlockExclusiveScan(v[0] + v[1] + v[2] + v[3], total, waveSums);
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            if (base + e < n)
                data[base + e] = run;
            run += v[e];
        }
        carry += total;
    }
}

__global__ __launch_bounds__(kScanThreads) void AddBlockOffsetsKernel(
    uint32_t* __restrict__ data, const uint32_t* __restrict__ blockOffsets, uint32_t n)
{
    // block 0 needs no offset: the grid starts at block 1
    const uint32_t block = blockIdx.x + 1;
    const uint32_t add = blockOffsets[block];
    const size_t base = static_cast<size_t>(block) * kScanPerBlock + threadIdx.x * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if (base + e < n)
            data[base + e] += add;
}

// V / COL of every kept entry, rows laid out by ROW
template <int LPR>
__global__ __launch_bounds__(kThreads) void CsrFillKernel(float* __restrict__ V,
                                                          uint32_t* __restrict__ COL,
                                                          const uint32_t* __restrict__ ROW,
                                                          const DenseView d,
                                                          const uint32_t capacity)
{
    constexpr uint32_t kGroups = kThreads / LPR;
    const uint32_t lane = threadIdx.x % LPR;
    const uint32_t group = threadIdx.x / LPR;
    // position of this group inside its wavefront, as a shift for 64-bit ballots
    const uint32_t shift = (threadIdx.x & 63u) - lane;
    const uint64_t groupMask = LPR == 64 ? ~0ull : ((1ull << LPR) - 1ull);
    const uint64_t below = (1ull << lane) - 1ull;
    const uint32_t rowsPerPass = gridDim.x * kGroups;
    const uint32_t passes = (d.M + rowsPerPass - 1) / rowsPerPass;
    for (uint32_t pass = 0; pass < passes; ++pass)
    {
        const uint32_t row = pass * rowsPerPass + blockIdx.x * kGroups + group;
        const bool rowOk = row < d.M;
        uint32_t slot = rowOk ? ROW[row] : 0u;
        // a ROW that was not computed from this matrix must not make the stores run past the
        // row, and nothing is stored past the capacity of V and COL
        const uint32_t rowEnd = rowOk ? min(ROW[row + 1], capacity) : 0u;
        for (uint32_t col0 = 0; col0 < d.N; col0 += LPR * 4)
        {
            const uint32_t col = col0 + lane * 4;
            const float4 q = LoadQuad(d, row, col, rowOk);
            const float v[4] = { q.x, q.y, q.z, q.w };
            // entries are ordered by (lane, element): everything lower lanes keep comes first
            uint32_t before = 0, kept = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                const uint64_t m = (__ballot(v[e] != 0.f) >> shift) & groupMask;
                before += __popcll(m & below);
                kept += __popcll(m);
            }
            uint32_t at = slot + before;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (v[e] != 0.f && at < rowEnd)
                {
                    V[at] = v[e];
                    COL[at] = col + e;
                    ++at;
                }
            slot += kept;
        }
    }
}

// ---------------------------------------------------------------------------
// Dense -> CSR with one pass over the matrix (rows of 128 .. 8192 columns, 16-byte aligned).
//
// A row's place in V / COL depends on the counts of all rows above, which are not known while
// the row is in registers.  Waiting for them inside the kernel (a decoupled look-back over row
// tiles) was built and measured on the 8192 x 8192 matrix at 1 %: the pass alone took 42 us,
// with the look-back 95 us and with ordered tile tickets on top 134 us (8192 device-scope
// atomics on one address cost 8 ns each, and 2048 resident tiles polling each other's state
// words slow the loads they are waiting for).  So the pass does not wait: every row writes its
// entries, in order, into a staging slot of `stage` entries at row * stage, and its count into
// ROW; the counts are scanned; a second, small kernel moves the staged entries to their final
// place (8 bytes read and written per entry).  A row with more than `stage` entries (the slot is
// sized from the caller's capacity, twice the mean plus 32) is rebuilt from the dense matrix by
// the second kernel instead, so any input converts correctly.
// ---------------------------------------------------------------------------
constexpr uint32_t kStageWaves = 4;  // wavefronts per workgroup

// A workgroup holds 4 / WPR rows; WPR wavefronts share a row, each taking QUADS float4 per lane
// of a contiguous part of it.  Requires N <= WPR * QUADS * 256.  Few
// registers per wavefront on purpose: many small workgroups per compute unit, out of step with
// each other, keep loads in flight while others count and store.
template <int WPR, int QUADS>
__global__ __launch_bounds__(kStageWaves * 64) void CsrStageKernel(
    float* __restrict__ stageV, uint32_t* __restrict__ stageCol, uint32_t* __restrict__ counts,
    const uint32_t stage, const DenseView d)
{
    constexpr uint32_t kRows = kStageWaves / WPR;  // rows per workgroup
    __shared__ uint32_t sCounts[kStageWaves];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * kRows + wave / WPR;
    const uint32_t part = wave % WPR;  // which part of the row
    const bool rowOk = row < d.M;
    if (blockIdx.x == 0 && threadIdx.x == 0)
        counts[d.M] = 0;  // the slot the scan turns into the number of entries

    // quad j of lane l of part p holds columns 256 (p QUADS + j) + 4 l .. + 3
    float4 q[QUADS];
#pragma unroll
    for (int j = 0; j < QUADS; ++j)
    {
        const uint32_t col = ((part * QUADS + j) * 64 + lane) * 4;
        q[j] = LoadQuad(d, row, col, rowOk);
    }
    uint32_t total = 0;  // the same in every lane
#pragma unroll
    for (int j = 0; j < QUADS; ++j)
        total += __popcll(__ballot(q[j].x != 0.f)) + __popcll(__ballot(q[j].y != 0.f)) +
                 __popcll(__ballot(q[j].z != 0.f)) + __popcll(__ballot(q[j].w != 0.f));
    if (lane == 0)
        sCounts[wave] = total;
    __syncthreads();
    // entries of the parts before this one in the same row
    uint32_t slot = 0, rowCount = 0;
#pragma unroll
    for (uint32_t p = 0; p < WPR; ++p)
    {
        const uint32_t c = sCounts[wave - part + p];
        rowCount += c;
        if (p < part)
            slot += c;
    }
    if (rowOk && part == 0 && lane == 0)
        counts[row] = rowCount;
    if (!rowOk || rowCount > stage)
        return;  // the second kernel rebuilds an overfull row from the dense matrix

    // inside a part the entries are ordered by (quad, lane, element): ascending columns
    float* outV = stageV + static_cast<size_t>(row) * stage;
    uint32_t* outCol = stageCol + static_cast<size_t>(row) * stage;
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
    for (int j = 0; j < QUADS; ++j)
    {
        const float v[4] = { q[j].x, q[j].y, q[j].z, q[j].w };
        uint32_t before = 0, kept = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            const uint64_t m = __ballot(v[e] != 0.f);
            before += __popcll(m & below);
            kept += __popcll(m);
        }
        if (kept == 0)
            continue;
        uint32_t at = slot + before;
        const uint32_t col = ((part * QUADS + j) * 64 + lane) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (v[e] != 0.f)
            {
                outV[at] = v[e];
                outCol[at] = col + e;
                ++at;
            }
        slot += kept;
    }
}

// One wavefront per row: staged entries move to ROW[row] ..; a row that did not fit its staging
// slot is read from the dense matrix again.  Nothing is stored at or past `capacity`.
__global__ __launch_bounds__(256) void CsrUnstageKernel(float* __restrict__ V,
                                                        uint32_t* __restrict__ COL,
                                                        const uint32_t* __restrict__ ROW,
                                                        const float* __restrict__ stageV,
                                                        const uint32_t* __restrict__ stageCol,
                                                        const uint32_t stage,
                                                        const uint32_t capacity, const DenseView d)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= d.M)
        return;
    const uint32_t first = ROW[row];
    const uint32_t count = ROW[row + 1] - first;
    if (count <= stage)
    {
        const float* inV = stageV + static_cast<size_t>(row) * stage;
        const uint32_t* inCol = stageCol + static_cast<size_t>(row) * stage;
        for (uint32_t i = lane; i < count; i += 64)
            if (first + i < capacity)
            {
                V[first + i] = inV[i];
                COL[first + i] = inCol[i];
            }
        return;
    }
    const uint64_t below = (1ull << lane) - 1ull;
    uint32_t slot = first;
    for (uint32_t col0 = 0; col0 < d.N; col0 += 256)
    {
        const uint32_t col = col0 + lane * 4;
        const float4 q = LoadQuad(d, row, col, true);
        const float v[4] = { q.x, q.y, q.z, q.w };
        uint32_t before = 0, kept = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            const uint64_t m = __ballot(v[e] != 0.f);
            before += __popcll(m & below);
            kept += __popcll(m);
        }
        uint32_t at = slot + before;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (v[e] != 0.f)
            {
                if (at < capacity)
                {
                    V[at] = v[e];
                    COL[at] = col + e;
                }
                ++at;
            }
        slot += kept;
    }
}

// One wavefront per row, one pass over the dense matrix.  A row of at most 128 entries is
// merged into the zeros in registers; a longer one is cleared first, then its entries are
// written over the zeros.  Four columns that all exist are stored 16 bytes at a time, whatever
// the alignment of the row (a vector store only asks for 4-byte alignment).
__device__ __forceinline__ void StoreQuad(float* p, float4 q, uint32_t col, uint32_t N)
{
    if (col + 4 <= N)
    {
        typedef float floatx4 __attribute__((ext_vector_type(4)));
        typedef floatx4 floatx4a4 __attribute__((aligned(4)));
        *reinterpret_cast<floatx4a4*>(p) = floatx4{ q.x, q.y, q.z, q.w };
    }
    else
    {
        if (col + 0 < N) p[0] = q.x;
        if (col + 1 < N) p[1] = q.y;
        if (col + 2 < N) p[2] = q.z;
    }
}

__global__ __launch_bounds__(kThreads) void CsrToDenseRowKernel(float* __restrict__ dense,
                                                                uint32_t ld, uint32_t M,
                                                                uint32_t N,
                                                                const float* __restrict__ V,
                                                                const uint32_t* __restrict__ COL,
                                                                const uint32_t* __restrict__ ROW)
{
    constexpr uint32_t kWaves = kThreads / 64;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    for (uint32_t row = blockIdx.x * kWaves + wave; row < M; row += gridDim.x * kWaves)
    {
        float* out = dense + static_cast<size_t>(row) * ld;
        const uint32_t begin = ROW[row];
        const uint32_t end = ROW[row + 1];
        if (end - begin <= 128)
        {
            // A short row is held in registers (two entries per lane) and merged into the
            // stream of zeros: every 1 KiB piece of the row is stored once, entries included,
            // so nothing is written twice and no store waits for another.
            uint32_t c0 = 0xffffffffu, c1 = 0xffffffffu;
            float v0 = 0.f, v1 = 0.f;
            if (begin + lane < end)
            {
                c0 = COL[begin + lane];
                v0 = V[begin + lane];
            }
            if (begin + 64 + lane < end)
            {
                c1 = COL[begin + 64 + lane];
                v1 = V[begin + 64 + lane];
            }
            // an entry outside the matrix is dropped, never written
            c0 = c0 < N ? c0 : 0xffffffffu;
            c1 = c1 < N ? c1 : 0xffffffffu;
            for (uint32_t base = 0; base < N; base += 256)
            {
                float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
                auto place = [&](uint64_t hits, uint32_t cols, float vals) {
                    while (hits != 0)
                    {
                        const uint32_t e = static_cast<uint32_t>(__builtin_ctzll(hits));
                        hits &= hits - 1;
                        const uint32_t c = static_cast<uint32_t>(__builtin_amdgcn_readlane(
                                               static_cast<int>(cols), static_cast<int>(e))) - base;
                        const float v = __builtin_bit_cast(
                            float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, vals),
                                                             static_cast<int>(e)));
                        const bool mine = lane == (c >> 2);
                        switch (c & 3u)
                        {
                            case 0: q.x = mine ? v : q.x; break;
                            case 1: q.y = mine ? v : q.y; break;
                            case 2: q.z = mine ? v : q.z; break;
                            default: q.w = mine ? v : q.w; break;
                        }
                    }
                };
                // c - base < 256 in unsigned arithmetic: base <= c < base + 256
                place(__ballot(c0 - base < 256u && c0 != 0xffffffffu), c0, v0);
                place(__ballot(c1 - base < 256u && c1 != 0xffffffffu), c1, v1);
                StoreQuad(out + base + lane * 4, q, base + lane * 4, N);
            }
            continue;
        }
        for (uint32_t c = lane * 4; c < N; c += 256)
            StoreQuad(out + c, make_float4(0.f, 0.f, 0.f, 0.f), c, N);
        // An entry is written by another lane than the one that cleared its place: the zeros
        // have to be acknowledged by the cache before the entries follow them.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (uint32_t p = begin + lane; p < end; p += 64)
        {
            const uint32_t c = COL[p];
            if (c < N)  // an entry outside the matrix is dropped, never written
                out[c] = V[p];
        }
    }
}

int LanesPerRow(uint32_t N)
{
    const uint32_t quads = (N + 3) / 4;
    int lpr = 4;
    while (lpr < 64 && static_cast<uint32_t>(lpr) < quads)
        lpr *= 2;
    return lpr;
}

uint32_t RowGrid(uint32_t M, int lanesPerRow)
{
    const uint32_t groups = kThreads / static_cast<uint32_t>(lanesPerRow);
    const uint64_t blocks = (static_cast<uint64_t>(M) + groups - 1) / groups;
    const uint64_t cap = static_cast<uint64_t>(sph::ComputeUnits()) * 16;
    return static_cast<uint32_t>(std::max<uint64_t>(1, std::min(blocks, cap)));
}

DenseView MakeView(const float* dense, uint32_t M, uint32_t N, uint32_t ld)
{
    DenseView d{};
    d.data = dense;
    d.M = M;
    d.N = N;
    d.ld = ld;
    return d;
}

template <template <int> class Launcher, typename... Args>
void DispatchLanes(int lanesPerRow, Args&&... args)
{
    switch (lanesPerRow)
    {
        case 4: Launcher<4>::Run(args...); break;
        case 8: Launcher<8>::Run(args...); break;
        case 16: Launcher<16>::Run(args...); break;
        case 32: Launcher<32>::Run(args...); break;
        default: Launcher<64>::Run(args...); break;
    }
}

template <int LPR>
struct CountLauncher
{
    static void Run(uint32_t grid, hipStream_t stream, uint32_t* counts, const DenseView& d)
    {
        hipLaunchKernelGGL(CsrCountKernel<LPR>, dim3(grid), dim3(kThreads), 0, stream, counts, d);
    }
};

template <int LPR>
struct FillLauncher
{
    static void Run(uint32_t grid, hipStream_t stream, float* V, uint32_t* COL,
                    const uint32_t* ROW, const DenseView& d, uint32_t capacity)
    {
        hipLaunchKernelGGL(CsrFillKernel<LPR>, dim3(grid), dim3(kThreads), 0, stream, V, COL, ROW,
                           d, capacity);
    }
};
}  // namespace

namespace sph
{
bool ScanWaitsOrAllocates(uint32_t n, const uint32_t* lastHost)
{
    return lastHost != nullptr || n > kScanSingleLimit;
}

int ResolveCsrScratch(uint32_t** out)
{
    const int device = sph::CurrentDevice();
    if (device < 0 || device >= kMaxScratchDevices)
        return sph::Fail(SPH_ERR_INVALID, "ResolveCsrScratch - device id out of range");
    std::lock_guard<std::mutex> lock(gScratchMutex);
    if (gScratchPtr[device] == nullptr)
    {
        // every device holds its own copy of the array at its own address
        SPH_HIP_TRY(hipSetDevice(device));
        uint32_t* ptr = nullptr;
        SPH_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
        if (ptr == nullptr)
            return sph::Fail(SPH_ERR_DEVICE, "ResolveCsrScratch - null symbol address");
        gScratchPtr[device] = ptr;
    }
    if (out != nullptr)
        *out = gScratchPtr[device];
    return SPH_OK;
}

int ExclusiveScanInPlace(uint32_t* data, uint32_t n, uint32_t* lastHost, hipStream_t stream,
                         uint32_t* sums)
{
    if (lastHost != nullptr || (n > kScanSingleLimit && sums == nullptr))
        SPH_REFUSE_WHILE_CAPTURING();  // reads back, or takes a scratch allocation
    const uint32_t blocks = (n + kScanPerBlock - 1) / kScanPerBlock;
    if (n <= kScanSingleLimit)
    {
        // up to 16 rounds of one workgroup cost less than three launches
        hipLaunchKernelGGL(ScanSingleKernel, dim3(1), dim3(kScanThreads), 0, stream, data, n);
        SPH_CHECK_LAUNCH();
    }
    else
    {
        // per-block totals: the caller's workspace, or a stream-ordered scratch allocation
        const bool own = sums == nullptr;
        if (own)
            ::sph::CountAllocation();
            SPH_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&sums),
                                       blocks * sizeof(uint32_t), stream));
        hipLaunchKernelGGL(ScanBlocksKernel, dim3(blocks), dim3(kScanThreads), 0, stream, data,
                           sums, n);
        hipLaunchKernelGGL(ScanSumsKernel, dim3(1), dim3(kScanThreads), 0, stream, sums, blocks);
        hipLaunchKernelGGL(AddBlockOffsetsKernel, dim3(blocks - 1), dim3(kScanThreads), 0, stream,
                           data, sums, n);
        const hipError_t launched = hipGetLastError();
        if (own)
            SPH_HIP_TRY(hipFreeAsync(sums, stream));
        if (launched != hipSuccess)
            return sph::Fail(SPH_ERR_DEVICE, std::string("exclusive scan launch failed with ") +
                                                 hipGetErrorString(launched));
    }
    if (lastHost != nullptr && n != 0)
    {
        SPH_HIP_TRY(hipMemcpyAsync(lastHost, data + (n - 1), sizeof(uint32_t),
                                   hipMemcpyDeviceToHost, stream));
        SPH_HIP_TRY(hipStreamSynchronize(stream));
    }
    return SPH_OK;
}
}  // namespace sph

extern "C" {

int sph_csr_row_offsets_f32(uint32_t* ROW, const float* dense, uint32_t M, uint32_t N,
                            uint32_t ld, uint32_t* nnzHost)
{
    SPH_REQUIRE(ROW != nullptr, "ROW is null");
    SPH_REQUIRE(ld >= N, "row pitch is shorter than a row");
    SPH_REQUIRE(M < 0xffffffffu, "too many rows");
    SPH_REQUIRE(M == 0 || N == 0 || dense != nullptr, "dense is null");
    if (sph::ScanWaitsOrAllocates(M + 1, nnzHost))
        SPH_REFUSE_WHILE_CAPTURING();  // before anything is enqueued into the graph
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;

    const DenseView d = MakeView(dense, M, N, ld);
    const int lanes = LanesPerRow(N);
    DispatchLanes<CountLauncher>(lanes, RowGrid(M, lanes), stream, ROW, d);
    SPH_CHECK_LAUNCH();

    return sph::ExclusiveScanInPlace(ROW, M + 1, nnzHost, stream);
}

int sph_csr_row_offsets_noalloc_f32(uint32_t* ROW, const float* dense, uint32_t M, uint32_t N,
                                    uint32_t ld)
{
    SPH_REQUIRE(ROW != nullptr, "ROW is null");
    SPH_REQUIRE(ld >= N, "row pitch is shorter than a row");
    SPH_REQUIRE(M == 0 || N == 0 || dense != nullptr, "dense is null");
    SPH_REQUIRE(M < static_cast<uint64_t>(kNoAllocMaxBlocks) * kScanPerBlock,
                "more than 16777215 rows exceed the fixed scratch array");
    uint32_t* sums = nullptr;
    const int rc = sph::ResolveCsrScratch(&sums);
    if (rc != SPH_OK)
        return rc;
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;

    const DenseView d = MakeView(dense, M, N, ld);
    const int lanes = LanesPerRow(N);
    DispatchLanes<CountLauncher>(lanes, RowGrid(M, lanes), stream, ROW, d);
    SPH_CHECK_LAUNCH();

    // every total the scan reads is written by the same call first: nothing has to be cleared
    return sph::ExclusiveScanInPlace(ROW, M + 1, nullptr, stream, sums);
}

int sph_csr_from_dense_f32(float* V, uint32_t* COL, uint32_t* ROW, uint32_t capacity,
                           const float* dense, uint32_t M, uint32_t N, uint32_t ld,
                           uint32_t* nnzHost)
{
    SPH_REQUIRE(ROW != nullptr, "ROW is null");
    SPH_REQUIRE(ld >= N, "row pitch is shorter than a row");
    SPH_REQUIRE(M < 0xffffffffu, "too many rows");
    SPH_REQUIRE(M == 0 || N == 0 || dense != nullptr, "dense is null");
    SPH_REQUIRE(capacity == 0 || (V != nullptr && COL != nullptr), "V or COL is null");
    SPH_REFUSE_WHILE_CAPTURING();  // takes a scratch allocation; before anything is enqueued
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const DenseView d = MakeView(dense, M, N, ld);

    // staging slot per row of the one-pass path: twice the mean the caller's capacity allows
    // plus 32, a multiple of 4
    const uint64_t mean = M != 0 ? capacity / M : 0;
    const uint64_t stage64 = (2 * mean + 32 + 3) / 4 * 4;
    // (below 16 Mi elements the three launches of the one-pass path cost more than the second
    // pass over the matrix they save: 8192 x 1000 18 us against 26 us, equal at 8192 x 2048)
    if (!(M != 0 && N >= 128 && N <= 8192 && stage64 * 4 <= N &&
          static_cast<uint64_t>(M) * N >= (1ull << 24)))
    {
        // narrow, very wide, small or not very sparse matrices (a staging area of more
        // than a quarter of the dense matrix): count, scan and fill as separate passes
        const int lanes = LanesPerRow(N);
        DispatchLanes<CountLauncher>(lanes, RowGrid(M, lanes), stream, ROW, d);
        SPH_CHECK_LAUNCH();
        const int rc = sph::ExclusiveScanInPlace(ROW, M + 1, nullptr, stream);
        if (rc != SPH_OK)
            return rc;
        if (M != 0 && N != 0 && capacity != 0)
        {
            DispatchLanes<FillLauncher>(lanes, RowGrid(M, lanes), stream, V, COL, ROW, d, capacity);
            SPH_CHECK_LAUNCH();
        }
        if (nnzHost != nullptr)
        {
            SPH_HIP_TRY(hipMemcpyAsync(nnzHost, ROW + M, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                       stream));
            SPH_HIP_TRY(hipStreamSynchronize(stream));
        }
        return SPH_OK;
    }

    // waves per row and float4 per lane: the narrowest pair that covers a row
    uint32_t wpr = 1, quads = 1;
    while (wpr < kStageWaves && wpr * 256 < N)
        wpr *= 2;
    while (wpr * quads * 256 < N)
        quads *= 2;
    const uint32_t stage = static_cast<uint32_t>(stage64);
    const size_t stageEntries = static_cast<size_t>(M) * stage;
    float* stageV = nullptr;
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&stageV), stageEntries * 8, stream));
    uint32_t* stageCol = reinterpret_cast<uint32_t*>(stageV + stageEntries);
    const uint32_t rowsPerGroup = kStageWaves / wpr;
    const dim3 grid((M + rowsPerGroup - 1) / rowsPerGroup), block(kStageWaves * 64);
#define SPH_STAGE(W, Q)                                                                        \
    hipLaunchKernelGGL((CsrStageKernel<W, Q>), grid, block, 0, stream, stageV, stageCol, ROW,   \
                       stage, d)
    if (wpr == 1)
        SPH_STAGE(1, 1);
    else if (wpr == 2)
        SPH_STAGE(2, 1);
    else if (quads == 1)
        SPH_STAGE(4, 1);
    else if (quads == 2)
        SPH_STAGE(4, 2);
    else if (quads == 4)
        SPH_STAGE(4, 4);
    else
        SPH_STAGE(4, 8);
#undef SPH_STAGE
    hipError_t launched = hipGetLastError();
    int rc = SPH_OK;
    if (launched == hipSuccess)
        rc = sph::ExclusiveScanInPlace(ROW, M + 1, nullptr, stream);
    if (launched == hipSuccess && rc == SPH_OK && capacity != 0)
    {
        hipLaunchKernelGGL(CsrUnstageKernel, dim3((M + 3) / 4), dim3(256), 0, stream, V, COL, ROW,
                           stageV, stageCol, stage, capacity, d);
        launched = hipGetLastError();
    }
    SPH_HIP_TRY(hipFreeAsync(stageV, stream));
    if (launched != hipSuccess)
        return sph::Fail(SPH_ERR_DEVICE, std::string("sph_csr_from_dense_f32 - launch failed with ") +
                                             hipGetErrorString(launched));
    if (rc != SPH_OK)
        return rc;
    if (nnzHost != nullptr)
    {
        SPH_HIP_TRY(hipMemcpyAsync(nnzHost, ROW + M, sizeof(uint32_t), hipMemcpyDeviceToHost,
                                   stream));
        SPH_HIP_TRY(hipStreamSynchronize(stream));
    }
    return SPH_OK;
}

int sph_csr_fill_f32(float* V, uint32_t* COL, const uint32_t* ROW, const float* dense, uint32_t M,
                     uint32_t N, uint32_t ld)
{
    if (M == 0 || N == 0)
        return SPH_OK;
    SPH_REQUIRE(ROW != nullptr && dense != nullptr, "null pointer");
    SPH_REQUIRE(ld >= N, "row pitch is shorter than a row");
    // V and COL may be null only for a matrix without entries; the kernel then writes nothing
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const DenseView d = MakeView(dense, M, N, ld);
    const int lanes = LanesPerRow(N);
    DispatchLanes<FillLauncher>(lanes, RowGrid(M, lanes), stream, V, COL, ROW, d, 0xffffffffu);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_csr_to_dense_f32(float* dense, uint32_t ld, const float* V, const uint32_t* COL,
                         const uint32_t* ROW, uint32_t M, uint32_t N)
{
    if (M == 0 || N == 0)
        return SPH_OK;
    SPH_REQUIRE(dense != nullptr && ROW != nullptr, "null pointer");
    SPH_REQUIRE(ld >= N, "row pitch is shorter than a row");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const uint32_t grid = RowGrid(M, 64);
    hipLaunchKernelGGL(CsrToDenseRowKernel, dim3(grid), dim3(kThreads), 0, stream, dense, ld, M, N,
                       V, COL, ROW);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

}  // extern "C"

// ---------------------------------------------------------------------------
// Validation of a CSR record before it is handed to a kernel that trusts it.
//
// The products (sph_spmm_csr_f32, sph_spgemm_*) read B[COL[p]] and V[ROW[i] .. ROW[i + 1])
// without checking: an index past the operand is a memory fault that can take the device
// down for every process on it.  A caller that builds the arrays itself checks them here
// first; the check only reads ROW[0 .. M] and COL[0 .. nnz), so it is safe on any contents.
// ---------------------------------------------------------------------------
namespace
{
enum : uint32_t
{
    kCsrRowStart = 1u,       // ROW[0] != 0
    kCsrRowOrder = 2u,       // ROW[i] > ROW[i + 1]
    kCsrRowTotal = 4u,       // ROW[M] != nnz
    kCsrColRange = 8u,       // COL[p] >= Kdim
    kCsrColUnsorted = 16u,   // a row's columns are not strictly ascending (not an error)
};

__global__ __launch_bounds__(256) void CsrValidateKernel(const uint32_t* __restrict__ COL,
                                                         const uint32_t* __restrict__ ROW,
                                                         uint32_t M, uint32_t Kdim, uint32_t nnz,
                                                         uint32_t* __restrict__ problems)
{
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint32_t found = 0;
    if (first == 0)
    {
        if (ROW[0] != 0)
            found |= kCsrRowStart;
        if (ROW[M] != nnz)
            found |= kCsrRowTotal;
    }
    for (uint64_t i = first; i < M; i += stride)
    {
        const uint32_t begin = ROW[i], end = ROW[i + 1];
        if (begin > end)
            found |= kCsrRowOrder;
        else if (end <= nnz)
        {
            // ascending columns inside the row; every index read lies below nnz
            for (uint32_t p = begin; p + 1 < end; ++p)
                if (COL[p] >= COL[p + 1])
                {
                    found |= kCsrColUnsorted;
                    break;
                }
        }
    }
    for (uint64_t p = first; p < nnz; p += stride)
        if (COL[p] >= Kdim)
            found |= kCsrColRange;
    if (found != 0)
        atomicOr(problems, found);
}
}  // namespace

extern "C" {

int sph_csr_validate_u32(const uint32_t* COL, const uint32_t* ROW, uint32_t M, uint32_t Kdim,
                         uint32_t nnz, uint32_t* problemsHost)
{
    if (problemsHost != nullptr)
        *problemsHost = 0;
    SPH_REQUIRE(ROW != nullptr, "ROW is null");
    SPH_REQUIRE(nnz == 0 || COL != nullptr, "COL is null");
    SPH_REQUIRE(M < 0xffffffffu, "too many rows");
    SPH_REFUSE_WHILE_CAPTURING();  // reads the result back
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    uint32_t* problems = nullptr;
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&problems), sizeof(uint32_t), stream));
    SPH_HIP_TRY(hipMemsetAsync(problems, 0, sizeof(uint32_t), stream));
    const uint64_t items = std::max<uint64_t>(std::max<uint64_t>(M, nnz), 1);
    const uint32_t grid = static_cast<uint32_t>(std::min<uint64_t>((items + 255) / 256, 4096));
    hipLaunchKernelGGL(CsrValidateKernel, dim3(grid), dim3(256), 0, stream, COL, ROW, M, Kdim, nnz,
                       problems);
    const hipError_t launched = hipGetLastError();
    uint32_t found = 0;
    hipError_t copied = hipSuccess;
    if (launched == hipSuccess)
    {
        copied = hipMemcpyAsync(&found, problems, sizeof(uint32_t), hipMemcpyDeviceToHost, stream);
        if (copied == hipSuccess)
            copied = hipStreamSynchronize(stream);
    }
    SPH_HIP_TRY(hipFreeAsync(problems, stream));
    if (launched != hipSuccess)
        return sph::Fail(SPH_ERR_DEVICE, std::string("sph_csr_validate_u32 launch failed with ") +
                                             hipGetErrorString(launched));
    SPH_HIP_TRY(copied);
    if (problemsHost != nullptr)
        *problemsHost = found;
    if ((found & (kCsrRowStart | kCsrRowOrder | kCsrRowTotal | kCsrColRange)) != 0)
    {
        std::string what;
        if (found & kCsrRowStart) what += " ROW[0] is not 0;";
        if (found & kCsrRowOrder) what += " ROW is not non-decreasing;";
        if (found & kCsrRowTotal) what += " ROW[M] differs from the entry count;";
        if (found & kCsrColRange) what += " a column index is not below the column count;";
        return sph::Fail(SPH_ERR_INVALID, "sph_csr_validate_u32 -" + what);
    }
    return SPH_OK;
}

}  // extern "C"
