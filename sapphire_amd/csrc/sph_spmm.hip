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
// Mapping: one wavefront per sparse row.  The row's (COL, V) pairs are fetched
// 64 at a time with one coalesced load per array and handed round with
// v_readlane; for every entry the wavefront reads one contiguous stretch of the
// dense row B[COL[p]] -- 16 bytes per lane, 1 KiB per wavefront when N >= 256 --
// so the gather is made of full cache lines.  Several B loads are issued before
// the first is consumed to keep the memory pipe busy.
#include "sph_internal.h"

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
    if (vec)
        hipLaunchKernelGGL(SpmmRowVec4, dim3(blocks), dim3(kThreads), 0, stream, args);
    else
        hipLaunchKernelGGL(SpmmRowScalar, dim3(blocks), dim3(kThreads), 0, stream, args);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

}  // extern "C"
