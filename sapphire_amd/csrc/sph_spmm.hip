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
// SpmmSlabVec4 (N >= 4): the dense columns are cut
// into slabs of 64 (32 for narrow operands); all workgroups that run on one XCD (ids
// congruent mod 8) work on the same slab, so the part of B an XCD gathers from (K x 64
// floats, 2 MiB at K = 8192) stays resident in that XCD's L2 instead of being streamed
// through it again and again.  A wavefront handles 4 rows at once: 16 lanes per row, 4
// columns (16 bytes) per lane.  Each 16-lane group fetches 16 (COL, V) pairs of its row with
// one coalesced load per array and hands them round with ds_swizzle; every entry then costs
// one 256-byte gather per row, eight of them in flight per lane.  The loop has no branches:
// entries past the end of a row gather row 0 of B and a select keeps them out of the sum.
//
// With N = 4 q + r the one lane per row whose four columns would reach past N takes the last
// four columns instead and stores only the r sums that are its own (a separate pass over the last
// r columns, one lane per row and column, cost as much as three quarters of a 256-column product).
//
// SpmmRowScalar: one wavefront per sparse row, one column per lane (operands whose byte
// offsets do not fit 32 bits, N < 4); the row's (COL, V) pairs are fetched 64 at a time and
// handed round with v_readlane.
#include "sph_internal.h"

#include <cstdlib>
#include <type_traits>

// Products and sums are rounded separately everywhere in this file (no fused multiply-add):
// that is what makes the result equal to the CPU loop bit for bit.
#pragma clang fp contract(off)

namespace
{
constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / 64;

struct SpmmArgs
{
    float* out;
    const float* V;
    const uint32_t* COL;
    const uint32_t* ROW;
    const float* B;
    uint32_t M, N;
    // floats between consecutive rows of B and of out: N, unless a launch covers some of the
    // columns of a wider operand
    uint32_t ldB, ldOut;
    int accumulate;
    // when set: out[row][*] = (0 + rowBias[row]) + sum, out is not read -- what accumulating into
    // an out that the K = 1 product bias x ones has filled gives
    const float* rowBias;
};

// four floats that need only be 4-byte aligned: rows of B and of out start anywhere when their
// pitch is no multiple of 4, and a 16-byte vector memory access only asks for dword alignment
typedef float floatx4v __attribute__((ext_vector_type(4)));
typedef floatx4v floatx4a4 __attribute__((aligned(4)));
__device__ __forceinline__ float4 Load4(const void* p)
{
    const floatx4v v = *reinterpret_cast<const floatx4a4*>(p);
    return make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void Store4(void* p, float4 v)
{
    *reinterpret_cast<floatx4a4*>(p) = floatx4v{ v.x, v.y, v.z, v.w };
}

__device__ __forceinline__ float Bcast(float v, int srcLane)
{
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), srcLane));
}

__device__ __forceinline__ uint32_t Bcast(uint32_t v, int srcLane)
{
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), srcLane));
}

// ---- slab mapping ------------------------------------------------------------------
// LPR lanes per row (8 or 16), 4 columns per lane: slabs of 4*LPR columns, 64/LPR rows per
// wavefront.

struct SlabPlan
{
    uint32_t slabs;           // ceil(N / slab width)
    uint32_t rowParts;        // row partitions per slab (spreads few slabs over all XCDs)
    uint32_t rowsPerPart;     // multiple of kRowsPerBlock
    uint32_t blocksPerColumn; // row blocks of one (slab, part) work column
    uint32_t columnsPerXcd;   // ceil(slabs * rowParts / 8)
};

// lane' = (lane & ~(LPR-1) & 31) | j inside each half of the wavefront: entry j of the lane's
// own LPR-lane group
template <int LPR, int J>
__device__ __forceinline__ uint32_t GroupBroadcast(uint32_t v)
{
    return static_cast<uint32_t>(
        __builtin_amdgcn_ds_swizzle(static_cast<int>(v), (J << 5) | (0x1f & ~(LPR - 1))));
}

template <int LPR>
__global__ __launch_bounds__(kThreads) void SpmmSlabVec4(const SpmmArgs args, const SlabPlan plan)
{
    constexpr int kSlabCols = 4 * LPR;
    constexpr int kLanesPerRow = LPR;
    constexpr int kRowsPerWave = 64 / LPR;
    constexpr int kRowsPerBlock = kRowsPerWave * kWavesPerBlock;
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
                               (threadIdx.x >> 6) * kRowsPerWave + lane / LPR;
    const uint32_t row = part * plan.rowsPerPart + rowInPart;
    const uint32_t N = args.N;
    // A lane whose four columns reach past N (N = 4 q + r: one lane per row, in the last slab)
    // takes columns N - 4 .. N - 1 instead and stores only the last r of its sums: the 16-byte
    // accesses need no alignment beyond 4 bytes, and the other columns are another lane's.
    const uint32_t colNatural = slab * kSlabCols + t * 4;
    const bool ragged = colNatural < N && colNatural + 4 > N;
    const uint32_t col = ragged ? N - 4 : colNatural;
    const uint32_t storeFrom = ragged ? colNatural + 4 - N : 0;  // first component to store
    const bool rowOk = rowInPart < plan.rowsPerPart && row < args.M;
    const bool active = rowOk && colNatural < N;

    uint32_t p = 0, end = 0;
    if (rowOk)
    {
        p = args.ROW[row];
        end = args.ROW[row + 1];
    }
    // Every lane gathers from a valid address on every step, so the loop has no branches:
    // lanes outside the matrix read the last four columns, entries past the end of a row
    // read row 0 of B (their COL is 0), and a select keeps such products out of the sum.
    // Byte offsets into B fit 32 bits (checked by the launcher) and are formed with a 24-bit
    // multiply-add.
    const char* __restrict__ Bbytes = reinterpret_cast<const char*>(args.B);
    const uint32_t colBytes = (colNatural < N ? col : N - 4) * 4;
    const uint32_t rowBytes = args.ldB * 4;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);

    // all lanes of the wavefront stay in the loop until the longest of its rows is done
    while (__builtin_amdgcn_ballot_w64(p < end) != 0)
    {
        uint32_t c = 0;
        float v = 0.f;
        if (p + t < end)
        {
            c = args.COL[p + t];
            v = args.V[p + t];
        }
        const uint32_t vbits = __builtin_bit_cast(uint32_t, v);
        const uint32_t left = end - p;  // entries of this lane's row still to do

        // eight entries at a time: broadcast, gather, then add in storage order
        auto eight = [&](auto baseC) {
            constexpr int base = decltype(baseC)::value;
            uint32_t cj[8];
            float vj[8];
            float4 b[8];
            cj[0] = GroupBroadcast<LPR, base + 0>(c);
            cj[1] = GroupBroadcast<LPR, base + 1>(c);
            cj[2] = GroupBroadcast<LPR, base + 2>(c);
            cj[3] = GroupBroadcast<LPR, base + 3>(c);
            cj[4] = GroupBroadcast<LPR, base + 4>(c);
            cj[5] = GroupBroadcast<LPR, base + 5>(c);
            cj[6] = GroupBroadcast<LPR, base + 6>(c);
            cj[7] = GroupBroadcast<LPR, base + 7>(c);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                b[j] = Load4(Bbytes + (__umul24(cj[j], rowBytes) + colBytes));
            vj[0] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 0>(vbits));
            vj[1] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 1>(vbits));
            vj[2] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 2>(vbits));
            vj[3] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 3>(vbits));
            vj[4] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 4>(vbits));
            vj[5] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 5>(vbits));
            vj[6] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 6>(vbits));
            vj[7] = __builtin_bit_cast(float, GroupBroadcast<LPR, base + 7>(vbits));
#pragma unroll
            for (int j = 0; j < 8; ++j)
            {
                const bool take = static_cast<uint32_t>(base + j) < left;
                const float x = sum.x + vj[j] * b[j].x;
                const float y = sum.y + vj[j] * b[j].y;
                const float z = sum.z + vj[j] * b[j].z;
                const float w = sum.w + vj[j] * b[j].w;
                sum.x = take ? x : sum.x;
                sum.y = take ? y : sum.y;
                sum.z = take ? z : sum.z;
                sum.w = take ? w : sum.w;
            }
        };
        eight(std::integral_constant<int, 0>{});
        if constexpr (LPR >= 16)
            eight(std::integral_constant<int, 8>{});
        p = min(p + LPR, end);
    }

    if (active)
    {
        float* dst = args.out + static_cast<size_t>(row) * args.ldOut + col;
        if (args.rowBias != nullptr)
        {
            const float old = 0.f + args.rowBias[row];
            sum.x = old + sum.x;
            sum.y = old + sum.y;
            sum.z = old + sum.z;
            sum.w = old + sum.w;
        }
        else if (args.accumulate)
        {
            // (the ragged lane reads values another lane is about to replace or has replaced in
            // the components it does not store; it uses only the ones it owns)
            const float4 old = Load4(dst);
            sum.x = old.x + sum.x;
            sum.y = old.y + sum.y;
            sum.z = old.z + sum.z;
            sum.w = old.w + sum.w;
        }
        if (!ragged)
            Store4(dst, sum);
        else
        {
            if (storeFrom <= 1) dst[1] = sum.y;
            if (storeFrom <= 2) dst[2] = sum.z;
            dst[3] = sum.w;
        }
    }
}

// one output column per lane; any N, any alignment
__global__ __launch_bounds__(kThreads) void SpmmRowScalar(const SpmmArgs args)
{
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
                    sum = sum + vv * B[static_cast<size_t>(cj) * args.ldB + n];
            }
        }
        if (active)
        {
            float* dst = args.out + static_cast<size_t>(row) * args.ldOut + n;
            if (args.rowBias != nullptr)
                *dst = (0.f + args.rowBias[row]) + sum;
            else
                *dst = args.accumulate ? (*dst + sum) : sum;
        }
    }
}
}  // namespace

static int LaunchSpmm(float* out, const float* V, const uint32_t* COL, const uint32_t* ROW,
                      uint32_t M, uint32_t Kdim, uint32_t N, const float* B, int accumulate,
                      const float* rowBias)
{
    // column indices are trusted to lie below Kdim, as in the dense leaf
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
    args.rowBias = rowBias;

    args.ldB = N;
    args.ldOut = N;

    // the slab kernel forms 32-bit byte offsets into B with a 24-bit multiply; larger operands
    // run on the scalar kernel, whose offsets are 64-bit.  Its 16-byte accesses need no
    // alignment beyond 4 bytes, so any N >= 4 is served by the slab kernel: every output
    // element is summed by one lane in storage order
    // (measured on the 8192 x 8192 matrix at 1 %: N = 255 134 us on the scalar kernel).
    const bool slabFits = static_cast<uint64_t>(Kdim) * N * 4 < (1ull << 32) &&
                          Kdim < (1u << 24) && N < (1u << 22);
    if (slabFits && N >= 4)
    {
        // 16 lanes per row (64-column slabs, 4 rows per wavefront) measured fastest from N = 64
        // up; narrower operands use 8 lanes per row so that fewer lanes idle
        const int lanesPerRow = N <= 32 ? 8 : 16;
        const uint32_t slabCols = 4u * static_cast<uint32_t>(lanesPerRow);
        const uint32_t rowsPerBlock = (64u / static_cast<uint32_t>(lanesPerRow)) * kWavesPerBlock;
        SlabPlan plan{};
        plan.slabs = (N + slabCols - 1) / slabCols;
        // rows are cut into parts so that the (slab, part) work columns fill the 8 XCDs evenly:
        // slabs * parts is the least common multiple of the slab count and 8
        uint32_t common = 8;  // gcd(slabs, 8)
        while (plan.slabs % common != 0)
            common /= 2;
        plan.rowParts = 8u / common;
        const uint32_t rowsPerPart = (M + plan.rowParts - 1) / plan.rowParts;
        plan.blocksPerColumn = (rowsPerPart + rowsPerBlock - 1) / rowsPerBlock;
        plan.rowsPerPart = plan.blocksPerColumn * rowsPerBlock;
        plan.columnsPerXcd = (plan.slabs * plan.rowParts + 7) / 8;
        const uint64_t grid = 8ull * plan.columnsPerXcd * plan.blocksPerColumn;
        SPH_REQUIRE(grid < (1ull << 31), "too many workgroups for one launch");
        if (lanesPerRow == 16)
            hipLaunchKernelGGL(SpmmSlabVec4<16>, dim3(static_cast<uint32_t>(grid)),
                               dim3(kThreads), 0, stream, args, plan);
        else
            hipLaunchKernelGGL(SpmmSlabVec4<8>, dim3(static_cast<uint32_t>(grid)), dim3(kThreads),
                               0, stream, args, plan);
    }
    else
    {
        const uint32_t blocks = (M + kWavesPerBlock - 1) / kWavesPerBlock;
        hipLaunchKernelGGL(SpmmRowScalar, dim3(blocks), dim3(kThreads), 0, stream, args);
    }
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

extern "C" {

int sph_spmm_csr_f32(float* out, const float* V, const uint32_t* COL, const uint32_t* ROW,
                     uint32_t M, uint32_t Kdim, uint32_t N, const float* B, int accumulate)
{
    return LaunchSpmm(out, V, COL, ROW, M, Kdim, N, B, accumulate, nullptr);
}

int sph_spmm_csr_bias_f32(float* out, const float* V, const uint32_t* COL, const uint32_t* ROW,
                          uint32_t M, uint32_t Kdim, uint32_t N, const float* B,
                          const float* rowBias)
{
    SPH_REQUIRE(M == 0 || N == 0 || rowBias != nullptr, "rowBias is null");
    return LaunchSpmm(out, V, COL, ROW, M, Kdim, N, B, 0, rowBias);
}

}  // extern "C"
