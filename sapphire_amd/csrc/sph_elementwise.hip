// One-pass, HBM-bound neighbours of the matrix-multiplication path: constant
// fill, ReLU and its backward, scale, subtract, the SGD update, fp32 -> fp16
// conversion and the batched 2-D transpose.  All of them move 16 bytes per lane
// per access where alignment allows and use grid-stride loops sized to a few
// workgroups per compute unit.
#include "sph_internal.h"

// Products and sums are rounded separately, as in the reference's CPU loops.
#pragma clang fp contract(off)

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

// out may alias in: every element is read before it is written, by the same lane
__global__ __launch_bounds__(kThreads) void ReluKernel(float* out, const float* in,
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

// Generic one-pass map over `count` floats: F(i) for the tail and scalar path,
// F4(i) for 4 consecutive elements starting at 4*i.
template <typename F4, typename F1>
__device__ __forceinline__ void MapRange(size_t count, int vec, F4 quad, F1 single)
{
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t step = static_cast<size_t>(gridDim.x) * kThreads;
    size_t done = 0;
    if (vec)
    {
        const size_t quads = count / 4;
        for (size_t i = tid; i < quads; i += step)
            quad(i);
        done = quads * 4;
    }
    for (size_t i = done + tid; i < count; i += step)
        single(i);
}

// out may alias in: every element is read before it is written, by the same lane
__global__ __launch_bounds__(kThreads) void ScaleKernel(float* out, const float* in, float factor,
                                                        size_t count, int vec)
{
    MapRange(
        count, vec,
        [&](size_t i) {
            float4 v = reinterpret_cast<const float4*>(in)[i];
            v.x *= factor;
            v.y *= factor;
            v.z *= factor;
            v.w *= factor;
            reinterpret_cast<float4*>(out)[i] = v;
        },
        [&](size_t i) { out[i] = in[i] * factor; });
}

__global__ __launch_bounds__(kThreads) void SubKernel(float* out, const float* a, const float* b,
                                                      size_t count, int vec)
{
    MapRange(
        count, vec,
        [&](size_t i) {
            const float4 x = reinterpret_cast<const float4*>(a)[i];
            const float4 y = reinterpret_cast<const float4*>(b)[i];
            reinterpret_cast<float4*>(out)[i] =
                make_float4(x.x - y.x, x.y - y.y, x.z - y.z, x.w - y.w);
        },
        [&](size_t i) { out[i] = a[i] - b[i]; });
}

// a and/or b repeat every `la` / `lb` elements
__global__ __launch_bounds__(kThreads) void SubWrapKernel(float* __restrict__ out,
                                                          const float* __restrict__ a,
                                                          const float* __restrict__ b,
                                                          size_t count, size_t la, size_t lb)
{
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t step = static_cast<size_t>(gridDim.x) * kThreads;
    for (size_t i = tid; i < count; i += step)
        out[i] = a[i % la] - b[i % lb];
}

__global__ __launch_bounds__(kThreads) void ReluBackwardKernel(float* __restrict__ dx,
                                                               const float* __restrict__ dy,
                                                               const float* __restrict__ x,
                                                               size_t count, int vec)
{
    MapRange(
        count, vec,
        [&](size_t i) {
            float4 d = reinterpret_cast<const float4*>(dx)[i];
            const float4 g = reinterpret_cast<const float4*>(dy)[i];
            const float4 v = reinterpret_cast<const float4*>(x)[i];
            d.x += v.x > 0.0f ? g.x : 0.0f;
            d.y += v.y > 0.0f ? g.y : 0.0f;
            d.z += v.z > 0.0f ? g.z : 0.0f;
            d.w += v.w > 0.0f ? g.w : 0.0f;
            reinterpret_cast<float4*>(dx)[i] = d;
        },
        [&](size_t i) { dx[i] += x[i] > 0.0f ? dy[i] : 0.0f; });
}

// The product is an fp32 value of its own before it is subtracted.  Written with plain
// operators under this file's contract(off): the rounded-arithmetic intrinsics of the HIP
// headers are compiled with contraction allowed and would fuse after inlining.
__device__ __forceinline__ float Rounded(float v)
{
    return v;
}

__global__ __launch_bounds__(kThreads) void SgdStepKernel(float* __restrict__ z,
                                                          const float* __restrict__ dz, float lr,
                                                          size_t count, int vec)
{
    MapRange(
        count, vec,
        [&](size_t i) {
            float4 w = reinterpret_cast<const float4*>(z)[i];
            const float4 g = reinterpret_cast<const float4*>(dz)[i];
            w.x = w.x - Rounded(g.x * lr);
            w.y = w.y - Rounded(g.y * lr);
            w.z = w.z - Rounded(g.z * lr);
            w.w = w.w - Rounded(g.w * lr);
            reinterpret_cast<float4*>(z)[i] = w;
        },
        [&](size_t i) { z[i] = z[i] - Rounded(dz[i] * lr); });
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

int sph_scale_f32(float* out, const float* in, float factor, size_t count)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(out != nullptr && in != nullptr, "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int vec = (Aligned16(out) && Aligned16(in)) ? 1 : 0;
    hipLaunchKernelGGL(ScaleKernel, dim3(GridFor(vec ? count / 4 + 3 : count)), dim3(kThreads), 0,
                       stream, out, in, factor, count, vec);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_sub_f32(float* out, const float* a, const float* b, size_t count, size_t inputStride,
                int broadcastA, int broadcastB)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(out != nullptr && a != nullptr && b != nullptr, "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    if (broadcastA || broadcastB)
    {
        SPH_REQUIRE(inputStride != 0, "inputStride must be non-zero with a broadcast operand");
        SPH_REQUIRE(out != a && out != b, "in-place subtraction with a broadcast operand");
        const size_t la = broadcastA ? inputStride : count;
        const size_t lb = broadcastB ? inputStride : count;
        hipLaunchKernelGGL(SubWrapKernel, dim3(GridFor(count)), dim3(kThreads), 0, stream, out, a,
                           b, count, la, lb);
    }
    else
    {
        const int vec = (Aligned16(out) && Aligned16(a) && Aligned16(b)) ? 1 : 0;
        hipLaunchKernelGGL(SubKernel, dim3(GridFor(vec ? count / 4 + 3 : count)), dim3(kThreads),
                           0, stream, out, a, b, count, vec);
    }
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_relu_backward_f32(float* dx, const float* dy, const float* x, size_t count)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(dx != nullptr && dy != nullptr && x != nullptr, "null pointer");
    SPH_REQUIRE(dx != dy && dx != x, "dx must not alias dy or x");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int vec = (Aligned16(dx) && Aligned16(dy) && Aligned16(x)) ? 1 : 0;
    hipLaunchKernelGGL(ReluBackwardKernel, dim3(GridFor(vec ? count / 4 + 3 : count)),
                       dim3(kThreads), 0, stream, dx, dy, x, count, vec);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int sph_sgd_step_f32(float* z, const float* dz, float learningRate, size_t count)
{
    if (count == 0)
        return SPH_OK;
    SPH_REQUIRE(z != nullptr && dz != nullptr, "null pointer");
    SPH_REQUIRE(z != dz, "z must not alias dz");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int vec = (Aligned16(z) && Aligned16(dz)) ? 1 : 0;
    hipLaunchKernelGGL(SgdStepKernel, dim3(GridFor(vec ? count / 4 + 3 : count)), dim3(kThreads),
                       0, stream, z, dz, learningRate, count, vec);
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
