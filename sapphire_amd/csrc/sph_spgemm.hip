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
// strip of the row in LDS (up to 8192 columns, 32 KiB; wider matrices are done strip by
// strip): A's entries are taken in order, the entries of the matching row of B are spread
// over the 64 lanes and added into the strip, and because the columns of one row of B are
// distinct no two lanes touch the same element in one step, which makes the sum order fixed
// and the result bit-identical to the CPU loop.  The strip is then swept in column order,
// which yields the sorted row without sorting.  A byte per block of 64 columns records which
// blocks were touched; only those are swept, and they are set back to zero as they are read,
// so the strip is cleared once per workgroup and the cost of a row follows the entries it
// produces, not the width of the matrix.  The same kernel runs twice: once to count the
// entries of every row (the caller then allocates), once to write them.
//
// Requirements on the operands: column indices of B below N and distinct within a row;
// column indices of A below the row count of B.
#include "sph_internal.h"

#include <algorithm>

#pragma clang fp contract(off)

namespace
{
constexpr uint32_t kStripMax = 8192;  // columns per LDS strip
constexpr uint32_t kAhead = 8;        // rows of B whose first 64 entries are in flight together
constexpr uint32_t kRowsPerTurn = 8;  // consecutive output rows a wavefront takes at a time

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
    // count pass: counts (M + 1 entries, counts[M] = 0).  fill pass: ROWC, VC, COLC.
    uint32_t* counts;
    const uint32_t* ROWC;
    float* VC;
    uint32_t* COLC;
};

__device__ __forceinline__ uint32_t Uniform(uint32_t v, uint32_t lane)
{
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane));
}

__device__ __forceinline__ float Uniform(float v, uint32_t lane)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), static_cast<int>(lane)));
}

template <bool FILL>
__global__ __launch_bounds__(64) void SpgemmRowKernel(const SpgemmArgs args)
{
    extern __shared__ float strip[];
    // one flag per block of 64 columns, after the strip
    unsigned char* touched = reinterpret_cast<unsigned char*>(strip + args.strip);
    const uint32_t blocksInStrip = args.strip / 64;
    const uint32_t lane = threadIdx.x;
    if (!FILL && blockIdx.x == 0 && lane == 0)
        args.counts[args.M] = 0;
    // cleared once; every block that is touched is cleared again when it is swept
    for (uint32_t x = lane; x < args.strip; x += 64)
        strip[x] = 0.0f;
    for (uint32_t t = lane; t < blocksInStrip; t += 64)
        touched[t] = 0;

    // A wavefront takes kRowsPerTurn consecutive rows per turn.  Their extents are read in one
    // go, and the loads that lead to a row's products form a pipeline over the rows of the
    // turn: while row i is multiplied, the first 64 (column, value) pairs of A's row i+2 and
    // the extents of the rows of B that row i+1 needs are already on their way.
    for (uint32_t turn = blockIdx.x * kRowsPerTurn; turn < args.M; turn += gridDim.x * kRowsPerTurn)
    {
        const uint32_t rowsHere = min(kRowsPerTurn, args.M - turn);
        uint32_t extentA = 0, extentC = 0;
        if (lane <= rowsHere)
        {
            extentA = args.ROWA[turn + lane];
            if (FILL)
                extentC = args.ROWC[turn + lane];
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
        const uint32_t rowLimit = FILL ? Uniform(extentC, i + 1) : 0u;
        // this row's first batch comes out of the pipeline, which then moves on
        const uint32_t firstBegin = nextBegin, firstEnd = nextEnd;
        const float firstValue = value2;
        k2 = k1;
        value2 = value1;
        loadStage2(k2, nextBegin, nextEnd);
        loadStage1(i + 2, k1, value1);

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
                            touched[(col[u] - c0) >> 6] = 1;
                        }
                        // rows of B with more than 64 entries: the rest, 64 at a time
                        for (uint32_t pb = s[u] + 64 + lane; pb < e[u]; pb += 64)
                        {
                            const uint32_t c = args.COLB[pb];
                            if (c - c0 < width)
                            {
                                strip[c - c0] = strip[c - c0] + a[u] * args.VB[pb];
                                touched[(c - c0) >> 6] = 1;
                            }
                        }
                    }
                }
            }

            // sweep the touched blocks in column order and leave them zero again
            for (uint32_t t0 = 0; t0 < blocksInStrip; t0 += 64)
            {
                const bool mine = t0 + lane < blocksInStrip && touched[t0 + lane] != 0;
                uint64_t pending = __ballot(mine);
                if (mine)
                    touched[t0 + lane] = 0;
                while (pending != 0)
                {
                    // up to four touched blocks per round, read together so that their LDS
                    // latencies overlap, then emitted in order
                    uint32_t x[4];
                    float v[4];
                    uint32_t rounds = 0;
#pragma unroll
                    for (uint32_t u = 0; u < 4; ++u)
                    {
                        x[u] = 0;
                        v[u] = 0.0f;
                        if (pending != 0)
                        {
                            const uint32_t t =
                                t0 + static_cast<uint32_t>(__builtin_ctzll(pending));
                            pending &= pending - 1;
                            x[u] = t * 64 + lane;
                            v[u] = strip[x[u]];
                            strip[x[u]] = 0.0f;
                            rounds = u + 1;
                        }
                    }
#pragma unroll
                    for (uint32_t u = 0; u < 4; ++u)
                    {
                        if (u >= rounds)
                            break;
                        const bool keep = v[u] != 0.0f;
                        const uint64_t m = __ballot(keep);
                        if (FILL)
                        {
                            const uint32_t at =
                                rowBase + emitted + __popcll(m & ((1ull << lane) - 1ull));
                            if (keep && at < rowLimit)
                            {
                                args.VC[at] = v[u];
                                args.COLC[at] = c0 + x[u];
                            }
                        }
                        emitted += __popcll(m);
                    }
                }
            }
        }
        if (!FILL && lane == 0)
            args.counts[turn + i] = emitted;
      }
    }
}

uint32_t StripFor(uint32_t N)
{
    const uint32_t padded = (N + 63u) / 64u * 64u;
    return std::max<uint32_t>(64u, std::min(padded, kStripMax));
}

uint32_t GridFor(uint32_t M)
{
    const uint64_t cap = static_cast<uint64_t>(sph::ComputeUnits()) * 64;
    const uint64_t turns = (static_cast<uint64_t>(M) + kRowsPerTurn - 1) / kRowsPerTurn;
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
    args.counts = ROWC;
    hipLaunchKernelGGL(SpgemmRowKernel<false>, dim3(GridFor(M)), dim3(64),
                       args.strip * sizeof(float) + args.strip / 64, stream, args);
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
    args.ROWC = ROWC;
    args.VC = VC;
    args.COLC = COLC;
    hipLaunchKernelGGL(SpgemmRowKernel<true>, dim3(GridFor(M)), dim3(64),
                       args.strip * sizeof(float) + args.strip / 64, stream, args);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

}  // extern "C"
