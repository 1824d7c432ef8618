// One-pass, HBM-bound neighbours of the matrix-multiplication path: constant
// fill, ReLU, fp32 -> fp16 conversion and the batched 2-D transpose.  All of
// them move 16 bytes per lane per access where alignment allows and use
// grid-stride loops sized to a few workgroups per compute unit.
#include "sph_internal.h"

#include <hip/hip_fp16.h>

#include <algorithm>

namespace
{
constexpr int kThreads = 256;

int GridFor(size_t items)
{
    const size_t blocks = (items + kThreads - 1) / kThreads;
    const size_t cap = static_cast<size_t>(sph::ComputeUnits()) * 8;
    return static_cast<int>(std::max<size_t>(1, std::min(blocks, cap)));
}

bool Aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

__global__ __launch_bounds__(kThreads) void FillKernel(float* __restrict__ dst, float value,
                                                       size_t count, int vec)
{
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t step = static_cast<size_t>(gridDim.x) * kThreads;
    size_t done = 0;
    if (vec)
    {
        const size_t quads = count / 4;
        float4* d4 = reinterpret_cast<float4*>(dst);
        const float4 v4 = make_float4(value, value, value, value);
        for (size_t i = tid; i < quads; i += step)
            d4[i] = v4;
        done = quads * 4;
    }
    for (size_t i = done + tid; i < count; i += step)
        dst[i] = value;
}

__global__ __launch_bounds__(kThreads) void ReluKernel(float* __restrict__ out,
                                                       const float* __restrict__ in,
                                                       size_t count, int vec)
{
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t step = static_cast<size_t>(gridDim.x) * kThreads;
    size_t done = 0;
    if (vec)
    {
        const size_t quads = count / 4;
        const float4* s4 = reinterpret_cast<const float4*>(in);
        float4* d4 = reinterpret_cast<float4*>(out);
        for (size_t i = tid; i < quads; i += step)
        {
            float4 v = s4[i];
            v.x = v.x > 0 ? v.x : 0;
            v.y = v.y > 0 ? v.y : 0;
            v.z = v.z > 0 ? v.z : 0;
            v.w = v.w > 0 ? v.w : 0;
            d4[i] = v;
        }
        done = quads * 4;
    }
    for (size_t i = done + tid; i < count; i += step)
    {
        const float v = in[i];
        out[i] = v > 0 ? v : 0;
    }
}

__global__ __launch_bounds__(kThreads) void ConvertKernel(__half* __restrict__ dst,
                                                          const float* __restrict__ src,
                                                          size_t count, int vec)
{
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t step = static_cast<size_t>(gridDim.x) * kThreads;
    size_t done = 0;
    if (vec)
    {
        // 8 values per lane: two 16-byte loads, one 16-byte store
        const size_t octs = count / 8;
        const float4* s4 = reinterpret_cast<const float4*>(src);
        uint4* d4 = reinterpret_cast<uint4*>(dst);
        for (size_t i = tid; i < octs; i += step)
        {
            const float4 a = s4[2 * i];
            const float4 b = s4[2 * i + 1];
            union
            {
                __half2 h[4];
                uint4 u;
            } pack;
            pack.h[0] = __floats2half2_rn(a.x, a.y);
            pack.h[1] = __floats2half2_rn(a.z, a.w);
            pack.h[2] = __floats2half2_rn(b.x, b.y);
            pack.h[3] = __floats2half2_rn(b.z, b.w);
            d4[i] = pack.u;
        }
        done = octs * 8;
    }
    for (size_t i = done + tid; i < count; i += step)
        dst[i] = __float2half_rn(src[i]);
}

// 64 x 64 tile through LDS; the extra column keeps the column-wise read-out
// off a single bank.
constexpr int kTile = 64;

__global__ __launch_bounds__(kThreads) void TransposeKernel(float* __restrict__ out,
                                                            const float* __restrict__ in,
                                                            uint32_t rows, uint32_t cols,
                                                            uint32_t tilesC, uint32_t tilesR,
                                                            int broadcast)
{
    __shared__ float tile[kTile][kTile + 1];
    uint32_t id = blockIdx.x;
    const uint32_t tc = id % tilesC;
    id /= tilesC;
    const uint32_t tr = id % tilesR;
    const uint32_t b = id / tilesR;

    const size_t plane = static_cast<size_t>(rows) * cols;
    const float* src = in + (broadcast ? 0 : plane * b);
    float* dst = out + plane * b;

    const uint32_t lx = threadIdx.x % kTile;
    const uint32_t ly = threadIdx.x / kTile;  // 0..3
    for (uint32_t r = ly; r < kTile; r += kThreads / kTile)
    {
        const uint32_t gr = tr * kTile + r;
        const uint32_t gc = tc * kTile + lx;
        if (gr < rows && gc < cols)
            tile[r][lx] = src[static_cast<size_t>(gr) * cols + gc];
    }
    __syncthreads();
    for (uint32_t r = ly; r < kTile; r += kThreads / kTile)
    {
        // output row = input column
        const uint32_t oc = tr * kTile + lx;  // input row index -> output column
        const uint32_t orow = tc * kTile + r;
        if (orow < cols && oc < rows)
            dst[static_cast<size_t>(orow) * rows + oc] = tile[lx][r];
    }
}
}  // namespace

extern "C" {

int sph_fill_f32(float* dst, float value, size_t count)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(dst != nullptr, "dst is null");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int vec = Aligned16(dst) ? 1 : 0;
    hipLaunchKernelGGL(FillKernel, dim3(GridFor(vec ? count / 4 + 3 : count)), dim3(kThreads), 0,
                       stream, dst, value, count, vec);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_relu_f32(float* out, const float* in, size_t count)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(out != nullptr && in != nullptr, "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int vec = (Aligned16(out) && Aligned16(in)) ? 1 : 0;
    hipLaunchKernelGGL(ReluKernel, dim3(GridFor(vec ? count / 4 + 3 : count)), dim3(kThreads), 0,
                       stream, out, in, count, vec);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_convert_f32_to_f16(sph_f16* dst, const float* src, size_t count)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(dst != nullptr && src != nullptr, "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int vec = (Aligned16(dst) && Aligned16(src)) ? 1 : 0;
    hipLaunchKernelGGL(ConvertKernel, dim3(GridFor(vec ? count / 8 + 7 : count)), dim3(kThreads),
                       0, stream, reinterpret_cast<__half*>(dst), src, count, vec);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_transpose_f32(float* out, const float* in, uint32_t rows, uint32_t cols, uint32_t batch,
                      int broadcast)
{
    if (rows == 0 || cols == 0 || batch == 0)
        return SPH_OK;
    SPH_REQUIRE(out != nullptr && in != nullptr, "null pointer");
    SPH_REQUIRE(out != in, "in-place transpose is not supported");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const uint32_t tilesC = (cols + kTile - 1) / kTile;
    const uint32_t tilesR = (rows + kTile - 1) / kTile;
    const uint64_t blocks = static_cast<uint64_t>(tilesC) * tilesR * batch;
    SPH_REQUIRE(blocks < (1ull << 31), "too many tiles for one launch");
    hipLaunchKernelGGL(TransposeKernel, dim3(static_cast<uint32_t>(blocks)), dim3(kThreads), 0,
                       stream, out, in, rows, cols, tilesC, tilesR, broadcast ? 1 : 0);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

}  // extern "C"
