// Measurement aid, not part of the product ABI: what the matrix cores of one MI355X deliver on
// given operand VALUES when the main loop of the 256 x 256-tile fp16 GEMM is stripped down to
// its parts.  Built into sapphire_amd/libsapphire_probe.so and loaded by
// `bench.py --only mfma_ceiling` alone.
//
// Every variant issues the matrix instructions of M = N = K = 4096 (256 workgroups x 8
// wavefronts x 2048 32x32x16-equivalents) and nothing of the GEMM's addressing: fragments come
// from a small LDS array, copies from a 1 MiB region that stays in L2, results go to a sink.
// The operands are N(0, sigma) halves (sigma = 0 gives all-zero operands).  Comparing a
// variant on N(0, 1/64) with the same variant on zeros separates what the instruction stream
// costs from what the operand values cost (the chip holds a power limit and lowers its clock
// when the operands toggle).
//
// Variants (per workgroup and K step of 32: 8 wavefronts, each a 128 x 64 part):
//   0  v_mfma_f32_32x32x16_f16, fragments from LDS: 12 16-byte reads per 16 instructions
//   1  v_mfma_f32_16x16x32_f16, fragments from LDS: 12 reads per 32 instructions
//   2  variant 0 + one workgroup barrier per half step
//   3  variant 0 + 32 KiB per K step copied L2 -> LDS (global_load_lds_dwordx4)
//   4  variant 0 with 8 reads per 16 instructions (the ratio of a 128 x 128 wavefront part)
//   5  variant 1 + the 32 KiB per K step of copies (the instruction and the copy volume of
//      the product kernel)
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <random>
#include <vector>

namespace
{
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* LdsPtr;

constexpr int kSrcVectors = 65536;           // halfx8 the kernels index (1 MiB)
constexpr size_t kSrcHalves = 65536u * 8 * 4;  // allocated: 4 MiB, the copies reach past 1 MiB
constexpr int kBlocks = 256;
constexpr int kThreads = 512;
constexpr int kIters = 128;                  // K steps of 32 per launch: K = 4096

#define PROBE_FENCE() __builtin_amdgcn_sched_barrier(0)

// 2 KiB per wavefront per half step = 32 KiB per workgroup per K step, from a region the 32
// workgroups of an XCD share
__device__ __forceinline__ void CopyHalfStep(const char* src, uint32_t ldsAddr, uint32_t it,
                                             uint32_t wave, uint32_t lane)
{
    const uint32_t off = ((it * 8 + wave) * 2048u) % (1u << 20) + lane * 16;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:1024"
                 :
                 : "s"(ldsAddr), "v"(off), "s"(src)
                 : "memory");
    asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
}

// LDSMODE 1: 6 reads per 8 instructions; 2: 4 reads per 8 instructions
template <int LDSMODE, int BARRIER, int DMA>
__global__ __launch_bounds__(kThreads) void Loop32(const halfx8* src, float* sink, int iters)
{
    __shared__ halfx8 lds[4096];
    __shared__ halfx8 dmaBuf[DMA ? 4096 : 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 4096; i += blockDim.x)
        lds[i] = src[(blockIdx.x * 4096 + i) & (kSrcVectors - 1)];
    __syncthreads();
    const uint32_t dmaLds = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)(dmaBuf))) + wave * 4096);
    const char* dmaSrc = reinterpret_cast<const char*>(src) + static_cast<size_t>(blockIdx.x % 32) * 32768;
    halfx8 a[2][4], b[2][2];
    for (int i = 0; i < 4; ++i)
    {
        a[0][i] = src[(blockIdx.x * 512 + threadIdx.x + i * 7919) & (kSrcVectors - 1)];
        a[1][i] = src[(blockIdx.x * 512 + threadIdx.x + i * 7919 + 3001) & (kSrcVectors - 1)];
    }
    for (int j = 0; j < 2; ++j)
    {
        b[0][j] = src[(blockIdx.x * 512 + threadIdx.x + j * 104729 + 31) & (kSrcVectors - 1)];
        b[1][j] = src[(blockIdx.x * 512 + threadIdx.x + j * 104729 + 977) & (kSrcVectors - 1)];
    }
    floatx16 acc[4][2] = {};
    const halfx8* base = &lds[wave * 512 + lane];
    for (int it = 0; it < iters * 2; it += 2)
    {
#pragma unroll
        for (int h = 0; h < 2; ++h)
        {
            // multiply buffer h, fill buffer h ^ 1
#pragma unroll
            for (int x = 0; x < 4; ++x)
#pragma unroll
                for (int y = 0; y < 2; ++y)
                {
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[h][y], a[h][x], acc[x][y], 0, 0, 0);
                    PROBE_FENCE();
                    if (LDSMODE == 1)
                    {
                        if (y == 0)
                            a[h ^ 1][x] = base[((it + h) * 6 + x) * 64 & 3583];
                        else if (x < 2)
                            b[h ^ 1][x] = base[((it + h) * 6 + 4 + x) * 64 & 3583];
                    }
                    else
                    {
                        if (y == 0 && x < 2)
                            a[h ^ 1][x] = base[((it + h) * 6 + x) * 64 & 3583];
                        else if (y == 1 && x < 1)
                            b[h ^ 1][x] = base[((it + h) * 6 + 4 + x) * 64 & 3583];
                        else if (y == 1 && x == 1)
                            a[h ^ 1][2] = base[((it + h) * 6 + 2) * 64 & 3583];
                    }
                    PROBE_FENCE();
                }
            if (BARRIER)
                __builtin_amdgcn_s_barrier();
            if (DMA)
                CopyHalfStep(dmaSrc, dmaLds, it + h, wave, lane);
            if (LDSMODE == 2)
            {
                a[h ^ 1][3] = a[h][0];
                b[h ^ 1][1] = b[h][0];
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float s = 0;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 2; ++j)
            for (int v = 0; v < 16; ++v)
                s += acc[i][j][v];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s + static_cast<float>(dmaBuf[0][0]);
}

// wavefront part 128 x 64 = 8 x 4 blocks of 16 x 16; one K step of 32 = 32 instructions and 12
// fragment reads
template <int DMA>
__global__ __launch_bounds__(kThreads) void Loop16(const halfx8* src, float* sink, int iters)
{
    __shared__ halfx8 lds[4096];
    __shared__ halfx8 dmaBuf[DMA ? 4096 : 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 4096; i += blockDim.x)
        lds[i] = src[(blockIdx.x * 4096 + i) & (kSrcVectors - 1)];
    __syncthreads();
    const uint32_t dmaLds = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)(dmaBuf))) + wave * 4096);
    const char* dmaSrc = reinterpret_cast<const char*>(src) + static_cast<size_t>(blockIdx.x % 32) * 32768;
    halfx8 a0[8], b0[4], a1[8], b1[4];
    for (int i = 0; i < 8; ++i)
    {
        a0[i] = src[(blockIdx.x * 512 + threadIdx.x + i * 7919) & (kSrcVectors - 1)];
        a1[i] = src[(blockIdx.x * 512 + threadIdx.x + i * 7919 + 3001) & (kSrcVectors - 1)];
    }
    for (int j = 0; j < 4; ++j)
    {
        b0[j] = src[(blockIdx.x * 512 + threadIdx.x + j * 104729 + 31) & (kSrcVectors - 1)];
        b1[j] = src[(blockIdx.x * 512 + threadIdx.x + j * 104729 + 977) & (kSrcVectors - 1)];
    }
    floatx4 acc[8][4] = {};
    const halfx8* base = &lds[wave * 512 + lane];
    auto step = [&](halfx8 (&A)[8], halfx8 (&B)[4], halfx8 (&AN)[8], halfx8 (&BN)[4], int it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(B[j], A[i], acc[i][j], 0, 0, 0);
                PROBE_FENCE();
                if (j == 0)
                    AN[i] = base[(it * 12 + i) * 64 & 3583];
                else if (j == 1 && i < 4)
                    BN[i] = base[(it * 12 + 8 + i) * 64 & 3583];
                PROBE_FENCE();
            }
            if (DMA && (i == 3 || i == 7))
                CopyHalfStep(dmaSrc, dmaLds, 2 * it + i / 4, wave, lane);
        }
    };
    for (int it = 0; it < iters; it += 2)
    {
        step(a0, b0, a1, b1, it);
        step(a1, b1, a0, b0, it + 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float s = 0;
    for (int i = 0; i < 8; ++i)
        for (int j = 0; j < 4; ++j)
            for (int v = 0; v < 4; ++v)
                s += acc[i][j][v];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s + static_cast<float>(dmaBuf[0][0]);
}

hipError_t LaunchVariant(int variant, const halfx8* src, float* sink, hipStream_t stream)
{
    const dim3 grid(kBlocks), block(kThreads);
    switch (variant)
    {
    case 0: hipLaunchKernelGGL((Loop32<1, 0, 0>), grid, block, 0, stream, src, sink, kIters); break;
    case 1: hipLaunchKernelGGL((Loop16<0>), grid, block, 0, stream, src, sink, kIters); break;
    case 2: hipLaunchKernelGGL((Loop32<1, 1, 0>), grid, block, 0, stream, src, sink, kIters); break;
    case 3: hipLaunchKernelGGL((Loop32<1, 0, 1>), grid, block, 0, stream, src, sink, kIters); break;
    case 4: hipLaunchKernelGGL((Loop32<2, 0, 0>), grid, block, 0, stream, src, sink, kIters); break;
    case 5: hipLaunchKernelGGL((Loop16<1>), grid, block, 0, stream, src, sink, kIters); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
}  // namespace

extern "C" {

int sph_probe_variants(void)
{
    return 6;
}

// flop of one launch of any variant: the matrix instructions of a 4096^3 product
double sph_probe_flop_per_launch(void)
{
    return 256.0 * 8 * kIters * 16 * 32768.0;
}

// Runs `variant` on N(0, sigma) operands: launches for settleMs milliseconds untimed (the clock
// needs about half a second of load to reach its working point), then `timed` launches between
// two events.  Returns 0 and the microseconds per launch, or a hipError_t.
int sph_probe_mfma_run(int variant, double sigma, double settleMs, int timed, double* usPerLaunch)
{
    if (usPerLaunch == nullptr || timed <= 0)
        return static_cast<int>(hipErrorInvalidValue);
    std::vector<_Float16> host(kSrcHalves);
    std::mt19937 gen(1234);
    std::normal_distribution<float> normal(0.f, sigma > 0 ? static_cast<float>(sigma) : 1.f);
    for (auto& x : host)
        x = sigma > 0 ? static_cast<_Float16>(normal(gen)) : static_cast<_Float16>(0.f);
    halfx8* src = nullptr;
    float* sink = nullptr;
    hipEvent_t begin = nullptr, end = nullptr;
    hipError_t rc = hipMalloc(reinterpret_cast<void**>(&src), kSrcHalves * sizeof(_Float16));
    if (rc == hipSuccess)
        rc = hipMalloc(reinterpret_cast<void**>(&sink), kBlocks * kThreads * sizeof(float));
    if (rc == hipSuccess)
        rc = hipMemcpy(src, host.data(), kSrcHalves * sizeof(_Float16), hipMemcpyHostToDevice);
    if (rc == hipSuccess)
        rc = hipEventCreate(&begin);
    if (rc == hipSuccess)
        rc = hipEventCreate(&end);
    if (rc == hipSuccess)
    {
        // settle: batches of launches until the wall clock says enough
        hipEvent_t probeBegin = begin, probeEnd = end;
        double spentMs = 0;
        while (rc == hipSuccess && spentMs < settleMs)
        {
            rc = hipEventRecord(probeBegin, nullptr);
            for (int r = 0; r < 50 && rc == hipSuccess; ++r)
                rc = LaunchVariant(variant, src, sink, nullptr);
            if (rc == hipSuccess)
                rc = hipEventRecord(probeEnd, nullptr);
            if (rc == hipSuccess)
                rc = hipEventSynchronize(probeEnd);
            float ms = 0;
            if (rc == hipSuccess)
                rc = hipEventElapsedTime(&ms, probeBegin, probeEnd);
            spentMs += ms > 0 ? ms : 1.0;
        }
    }
    if (rc == hipSuccess)
        rc = hipEventRecord(begin, nullptr);
    for (int r = 0; r < timed && rc == hipSuccess; ++r)
        rc = LaunchVariant(variant, src, sink, nullptr);
    if (rc == hipSuccess)
        rc = hipEventRecord(end, nullptr);
    if (rc == hipSuccess)
        rc = hipEventSynchronize(end);
    float ms = 0;
    if (rc == hipSuccess)
        rc = hipEventElapsedTime(&ms, begin, end);
    if (rc == hipSuccess)
        *usPerLaunch = static_cast<double>(ms) * 1e3 / timed;
    (void)hipDeviceSynchronize();
    if (begin != nullptr)
        (void)hipEventDestroy(begin);
    if (end != nullptr)
        (void)hipEventDestroy(end);
    if (src != nullptr)
        (void)hipFree(src);
    if (sink != nullptr)
        (void)hipFree(sink);
    return static_cast<int>(rc);
}

}  // extern "C"
