// CSR sparse x dense product  out[m][:] (+)= sum_p V[p] * B[COL[p]][:].
//
// The container is the reference's SparseMatrix
// (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:28-38): V values, COL
// column per entry, ROW offsets (M+1 of them).  The reference has no kernel
// for this product; the arithmetic contract is the one its dense leaf
// (Sources/Sapphire/compute/dense/naive/NaiveGemm.cpp:12-38) gives on the
// densified matrix: entries in storage order, product and sum rounded
// separately, one running fp32 sum per output element started at +0, then a
// single add into out.  Each output element is owned by exactly one lane which
// walks the row front to back, so the result is bit-identical to that loop.
//
// Two mappings.
//
// SpmmSlabVec4 (dense width a multiple of 4, aligned bases): the dense columns are cut
// into slabs of 32; all workgroups that run on one XCD (ids congruent mod 8) work on the
// same slab, so the part of B an XCD gathers from (K x 32 floats, 1 MiB at K = 8192) stays
// resident in that XCD's L2 instead of being streamed through it again and again.  A
// wavefront handles 8 rows at once: 8 lanes per row, 4 columns (16 bytes) per lane.  Each
// 8-lane group fetches 8 (COL, V) pairs of its row with one coalesced load per array and
// hands them round with ds_swizzle; every entry then costs one 128-byte gather per row.
//
// SpmmRowScalar / SpmmRowVec4: one wavefront per sparse row (any width, any alignment).  The row's (COL, V) pairs are fetched
// 64 at a time with one coalesced load per array and handed round with
// v_readlane; for every entry the wavefront reads one contiguous stretch of the
// dense row B[COL[p]] -- 16 bytes per lane, 1 KiB per wavefront when N >= 256 --
// so the gather is made of full cache lines.  Several B loads are issued before
// the first is consumed to keep the memory pipe busy.
#include "sph_internal.h"

#include <cstdlib>

namespace
{
constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / 64;
constexpr int kUnroll = 8;

struct SpmmArgs
{
    float* out;
    const float* V;
    const uint32_t* COL;
    const uint32_t* ROW;
    const float* B;
    uint32_t M, N;
    int accumulate;
};

__device__ __forceinline__ float Bcast(float v, int srcLane)
{
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), srcLane));
}

__device__ __forceinline__ uint32_t Bcast(uint32_t v, int srcLane)
{
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), srcLane));
}

// 4 output columns per lane, 16-byte loads and stores (N % 4 == 0, aligned bases)
__global__ __launch_bounds__(kThreads) void SpmmRowVec4(const SpmmArgs args)
{
#pragma clang fp contract(off)
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= args.M)
        return;
    const uint32_t N = args.N;
    const uint32_t begin = args.ROW[row];
    const uint32_t end = args.ROW[row + 1];
    const float* __restrict__ B = args.B;

    for (uint32_t colBase = 0; colBase < N; colBase += 256)
    {
        const uint32_t n = colBase + lane * 4;
        const bool active = n < N;
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);

        for (uint32_t p = begin; p < end; p += 64)
        {
            const uint32_t mine = p + lane;
            uint32_t c = 0;
            float v = 0.f;
            if (mine < end)
            {
                c = args.COL[mine];
                v = args.V[mine];
            }
            const uint32_t count = min(64u, end - p);
            uint32_t j = 0;
            for (; j + kUnroll <= count; j += kUnroll)
            {
                float4 b[kUnroll];
                float vj[kUnroll];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                {
                    const uint32_t cj = Bcast(c, static_cast<int>(j) + u);
                    vj[u] = Bcast(v, static_cast<int>(j) + u);
                    b[u] = active ? *reinterpret_cast<const float4*>(
                                        B + static_cast<size_t>(cj) * N + n)
                                  : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                {
                    sum.x = sum.x + vj[u] * b[u].x;
                    sum.y = sum.y + vj[u] * b[u].y;
                    sum.z = sum.z + vj[u] * b[u].z;
                    sum.w = sum.w + vj[u] * b[u].w;
                }
            }
            for (; j < count; ++j)
            {
                const uint32_t cj = Bcast(c, static_cast<int>(j));
                const float vv = Bcast(v, static_cast<int>(j));
                if (active)
                {
                    const float4 bb =
                        *reinterpret_cast<const float4*>(B + static_cast<size_t>(cj) * N + n);
                    sum.x = sum.x + vv * bb.x;
                    sum.y = sum.y + vv * bb.y;
                    sum.z = sum.z + vv * bb.z;
                    sum.w = sum.w + vv * bb.w;
                }
            }
        }

        if (active)
        {
            float4* dst = reinterpret_cast<float4*>(args.out + static_cast<size_t>(row) * N + n);
            if (args.accumulate)
            {
                const float4 old = *dst;
                sum.x = old.x + sum.x;
                sum.y = old.y + sum.y;
                sum.z = old.z + sum.z;
                sum.w = old.w + sum.w;
            }
            *dst = sum;
        }
    }
}


// ---- slab mapping ------------------------------------------------------------------
constexpr int kSlabCols = 32;      // dense columns per slab
constexpr int kLanesPerRow = 8;    // 4 columns per lane
constexpr int kRowsPerWave = 64 / kLanesPerRow;
constexpr int kRowsPerBlock = kRowsPerWave * kWavesPerBlock;

struct SlabPlan
{
    uint32_t slabs;           // ceil(N / 32)
    uint32_t rowParts;        // row partitions per slab (spreads few slabs over all XCDs)
    uint32_t rowsPerPart;     // multiple of kRowsPerBlock
    uint32_t blocksPerColumn; // row blocks of one (slab, part) work column
    uint32_t columnsPerXcd;   // ceil(slabs * rowParts / 8)
};

// lane' = (lane & 0x18) | j inside each half of the wavefront: entry j of the lane's own
// 8-lane group
template <int J>
__device__ __forceinline__ uint32_t GroupBroadcast(uint32_t v)
{
    return static_cast<uint32_t>(
        __builtin_amdgcn_ds_swizzle(static_cast<int>(v), (J << 5) | 0x18));
}

__global__ __launch_bounds__(kThreads) void SpmmSlabVec4(const SpmmArgs args, const SlabPlan plan)
{
#pragma clang fp contract(off)
    // work column w = slab + slabs * part runs on XCD w % 8
    const uint32_t xcd = blockIdx.x % 8;
    const uint32_t local = blockIdx.x / 8;
    const uint32_t w = xcd + 8 * (local / plan.blocksPerColumn);
    if (w >= plan.slabs * plan.rowParts)
        return;
    const uint32_t slab = w % plan.slabs;
    const uint32_t part = w / plan.slabs;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t t = lane & (kLanesPerRow - 1);
    const uint32_t rowInPart = (local % plan.blocksPerColumn) * kRowsPerBlock +
                               (threadIdx.x >> 6) * kRowsPerWave + (lane >> 3);
    const uint32_t row = part * plan.rowsPerPart + rowInPart;
    const uint32_t N = args.N;
    const uint32_t col = slab * kSlabCols + t * 4;
    const bool rowOk = rowInPart < plan.rowsPerPart && row < args.M;
    const bool active = rowOk && col < N;

    uint32_t p = 0, end = 0;
    if (rowOk)
    {
        p = args.ROW[row];
        end = args.ROW[row + 1];
    }
    const float* __restrict__ Bcol = args.B + col;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);

    // all lanes of the wavefront stay in the loop until the longest of its 8 rows is done
    while (__builtin_amdgcn_ballot_w64(p < end) != 0)
    {
        uint32_t c = 0;
        float v = 0.f;
        if (p + t < end)
        {
            c = args.COL[p + t];
            v = args.V[p + t];
        }
        uint32_t cj[8];
        float vj[8];
        float4 b[8];
        cj[0] = GroupBroadcast<0>(c);
        cj[1] = GroupBroadcast<1>(c);
        cj[2] = GroupBroadcast<2>(c);
        cj[3] = GroupBroadcast<3>(c);
        cj[4] = GroupBroadcast<4>(c);
        cj[5] = GroupBroadcast<5>(c);
        cj[6] = GroupBroadcast<6>(c);
        cj[7] = GroupBroadcast<7>(c);
        const uint32_t vbits = __builtin_bit_cast(uint32_t, v);
        vj[0] = __builtin_bit_cast(float, GroupBroadcast<0>(vbits));
        vj[1] = __builtin_bit_cast(float, GroupBroadcast<1>(vbits));
        vj[2] = __builtin_bit_cast(float, GroupBroadcast<2>(vbits));
        vj[3] = __builtin_bit_cast(float, GroupBroadcast<3>(vbits));
        vj[4] = __builtin_bit_cast(float, GroupBroadcast<4>(vbits));
        vj[5] = __builtin_bit_cast(float, GroupBroadcast<5>(vbits));
        vj[6] = __builtin_bit_cast(float, GroupBroadcast<6>(vbits));
        vj[7] = __builtin_bit_cast(float, GroupBroadcast<7>(vbits));
#pragma unroll
        for (int j = 0; j < 8; ++j)
        {
            // entries past the end of the row carry c = 0, v = 0 and are not added
            const bool take = active && (p + j < end);
            b[j] = take ? *reinterpret_cast<const float4*>(Bcol + static_cast<size_t>(cj[j]) * N)
                        : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
        {
            if (p + j < end)
            {
                sum.x = sum.x + vj[j] * b[j].x;
                sum.y = sum.y + vj[j] * b[j].y;
                sum.z = sum.z + vj[j] * b[j].z;
                sum.w = sum.w + vj[j] * b[j].w;
            }
        }
        p = min(p + 8, end);
    }

    if (active)
    {
        float4* dst = reinterpret_cast<float4*>(args.out + static_cast<size_t>(row) * N + col);
        if (args.accumulate)
        {
            const float4 old = *dst;
            sum.x = old.x + sum.x;
            sum.y = old.y + sum.y;
            sum.z = old.z + sum.z;
            sum.w = old.w + sum.w;
        }
        *dst = sum;
    }
}

// one output column per lane; any N, any alignment
__global__ __launch_bounds__(kThreads) void SpmmRowScalar(const SpmmArgs args)
{
#pragma clang fp contract(off)
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= args.M)
        return;
    const uint32_t N = args.N;
    const uint32_t begin = args.ROW[row];
    const uint32_t end = args.ROW[row + 1];
    const float* __restrict__ B = args.B;

    for (uint32_t colBase = 0; colBase < N; colBase += 64)
    {
        const uint32_t n = colBase + lane;
        const bool active = n < N;
        float sum = 0.f;
        for (uint32_t p = begin; p < end; p += 64)
        {
            const uint32_t mine = p + lane;
            uint32_t c = 0;
            float v = 0.f;
            if (mine < end)
            {
                c = args.COL[mine];
                v = args.V[mine];
            }
            const uint32_t count = min(64u, end - p);
            for (uint32_t j = 0; j < count; ++j)
            {
                const uint32_t cj = Bcast(c, static_cast<int>(j));
                const float vv = Bcast(v, static_cast<int>(j));
                if (active)
                    sum = sum + vv * B[static_cast<size_t>(cj) * N + n];
            }
        }
        if (active)
        {
            float* dst = args.out + static_cast<size_t>(row) * N + n;
            *dst = args.accumulate ? (*dst + sum) : sum;
        }
    }
}
}  // namespace

extern "C" {

int sph_spmm_csr_f32(float* out, const float* V, const uint32_t* COL, const uint32_t* ROW,
                     uint32_t M, uint32_t Kdim, uint32_t N, const float* B, int accumulate)
{
    (void)Kdim;  // column indices are trusted to lie below Kdim, as in the dense leaf
    if (M == 0 || N == 0)
        return SPH_OK;
    SPH_REQUIRE(out != nullptr && ROW != nullptr && B != nullptr, "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;

    SpmmArgs args{};
    args.out = out;
    args.V = V;
    args.COL = COL;
    args.ROW = ROW;
    args.B = B;
    args.M = M;
    args.N = N;
    args.accumulate = accumulate ? 1 : 0;

    const uint32_t blocks = (M + kWavesPerBlock - 1) / kWavesPerBlock;
    const bool vec = (N % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(B)) & 15u) == 0;
    static const bool rowMapping = [] {
        const char* e = getenv("SPH_SPMM_ROW");
        return e != nullptr && e[0] == '1';
    }();
    if (vec && !rowMapping)
    {
        SlabPlan plan{};
        plan.slabs = (N + kSlabCols - 1) / kSlabCols;
        plan.rowParts = plan.slabs >= 8 ? 1u : 8u / plan.slabs;
        const uint32_t rowsPerPart = (M + plan.rowParts - 1) / plan.rowParts;
        plan.blocksPerColumn = (rowsPerPart + kRowsPerBlock - 1) / kRowsPerBlock;
        plan.rowsPerPart = plan.blocksPerColumn * kRowsPerBlock;
        plan.columnsPerXcd = (plan.slabs * plan.rowParts + 7) / 8;
        const uint64_t grid = 8ull * plan.columnsPerXcd * plan.blocksPerColumn;
        SPH_REQUIRE(grid < (1ull << 31), "too many workgroups for one launch");
        hipLaunchKernelGGL(SpmmSlabVec4, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0,
                           stream, args, plan);
    }
    else if (vec)
        hipLaunchKernelGGL(SpmmRowVec4, dim3(blocks), dim3(kThreads), 0, stream, args);
    else
        hipLaunchKernelGGL(SpmmRowScalar, dim3(blocks), dim3(kThreads), 0, stream, args);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

}  // extern "C"
