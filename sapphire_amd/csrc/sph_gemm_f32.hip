// fp32 GEMM  out[u] += A[u] * B[u]  on the CDNA4 matrix cores.
//
// Storage, products and accumulation are all fp32 (v_mfma_f32_32x32x2_f32), so
// the only difference from the reference's scalar CPU loop
// (Sources/Sapphire/compute/dense/naive/NaiveGemm.cpp:12-38) is the order in
// which the K products are summed.
//
// Work decomposition
//   * one workgroup (4 wavefronts of 64 lanes, arranged 2 x 2) owns a
//     BM x BN tile of one M x N unit; BM = BN = 128 when that still gives at
//     least one tile per compute unit, 64 otherwise;
//   * the K loop advances 16 columns at a time: the A slab (BM x 16) is stored
//     k-major in LDS and the B slab (16 x BN) row-major, so that both MFMA
//     operands are read with lane-consecutive addresses (no bank conflicts);
//   * the slab for step i+1 is fetched from HBM into registers while the MFMAs
//     of step i run, and written to the other LDS buffer afterwards;
//   * units come either from (batch, stride) arithmetic -- stride 0 repeats an
//     operand -- or from a table of element offsets in device memory.
//
// Loads are 16 bytes wide when K, N and every base/stride allow it; otherwise
// a scalar, fully predicated path handles arbitrary shapes such as the
// reference's random test sizes (Tests/UnitTests/Sources/FunctionTest/GemmTest.cpp:26-33).
#include "sph_internal.h"

#include <cstring>
#include <mutex>
#include <unordered_set>

namespace
{
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kBK = 16;

struct GemmF32Args
{
    float* out;
    const float* A;
    const float* B;
    const SphGemmEntry* entries;  // device table, or null for stride arithmetic
    uint32_t M, N, K;
    uint32_t tilesM, tilesN;
    uint32_t outVec;     // 16-byte accesses to out are possible
    uint32_t overwrite;  // out = A*B instead of out += A*B
    int64_t strideOut, strideA, strideB;
};

// Slab loaders.  An operand is stored either with K contiguous (A as given, B when it is
// passed transposed: `rows` indexes M or N) or with the M/N index contiguous (B as given, A
// when it is passed transposed: `rows` indexes K).  Both end up k-major in LDS, S[k][x].
template <int BX, int QUADS, bool VEC>
__device__ __forceinline__ void FetchKContig(float4 (&stage)[QUADS], const float* __restrict__ src,
                                             uint32_t tid, uint32_t xBase, uint32_t xLimit,
                                             uint32_t k0, uint32_t K)
{
#pragma unroll
    for (int i = 0; i < QUADS; ++i)
    {
        const uint32_t q = tid + i * kThreads;
        const uint32_t r = q >> 2;
        const uint32_t kq = (q & 3) * 4;
        const uint32_t gx = xBase + r;
        const uint32_t gk = k0 + kq;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (gx < xLimit)
        {
            const float* p = src + static_cast<size_t>(gx) * K + gk;
            if (VEC)
            {
                if (gk < K)
                    v = *reinterpret_cast<const float4*>(p);
            }
            else
            {
                if (gk + 0 < K) v.x = p[0];
                if (gk + 1 < K) v.y = p[1];
                if (gk + 2 < K) v.z = p[2];
                if (gk + 3 < K) v.w = p[3];
            }
        }
        stage[i] = v;
    }
}

template <int BX, int QUADS, bool VEC>
__device__ __forceinline__ void FetchXContig(float4 (&stage)[QUADS], const float* __restrict__ src,
                                             uint32_t tid, uint32_t xBase, uint32_t xLimit,
                                             uint32_t k0, uint32_t K)
{
#pragma unroll
    for (int i = 0; i < QUADS; ++i)
    {
        const uint32_t q = tid + i * kThreads;
        const uint32_t kr = q / (BX / 4);
        const uint32_t xq = (q % (BX / 4)) * 4;
        const uint32_t gk = k0 + kr;
        const uint32_t gx = xBase + xq;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (gk < K)
        {
            const float* p = src + static_cast<size_t>(gk) * xLimit + gx;
            if (VEC)
            {
                if (gx < xLimit)
                    v = *reinterpret_cast<const float4*>(p);
            }
            else
            {
                if (gx + 0 < xLimit) v.x = p[0];
                if (gx + 1 < xLimit) v.y = p[1];
                if (gx + 2 < xLimit) v.z = p[2];
                if (gx + 3 < xLimit) v.w = p[3];
            }
        }
        stage[i] = v;
    }
}

template <int BX, int LD, int QUADS>
__device__ __forceinline__ void StashKContig(float* __restrict__ slab, const float4 (&stage)[QUADS],
                                             uint32_t tid)
{
#pragma unroll
    for (int i = 0; i < QUADS; ++i)
    {
        const uint32_t q = tid + i * kThreads;
        const uint32_t r = q >> 2;
        const uint32_t kq = (q & 3) * 4;
        float* dst = slab + kq * LD + r;
        dst[0 * LD] = stage[i].x;
        dst[1 * LD] = stage[i].y;
        dst[2 * LD] = stage[i].z;
        dst[3 * LD] = stage[i].w;
    }
}

template <int BX, int LD, int QUADS>
__device__ __forceinline__ void StashXContig(float* __restrict__ slab, const float4 (&stage)[QUADS],
                                             uint32_t tid)
{
#pragma unroll
    for (int i = 0; i < QUADS; ++i)
    {
        const uint32_t q = tid + i * kThreads;
        const uint32_t kr = q / (BX / 4);
        const uint32_t xq = (q % (BX / 4)) * 4;
        *reinterpret_cast<float4*>(slab + kr * LD + xq) = stage[i];
    }
}

template <int BM, int BN, bool VEC, bool TA, bool TB>
__global__ __launch_bounds__(kThreads) void GemmF32Kernel(const GemmF32Args args)
{
    constexpr int WM = BM / 2;   // rows per wavefront
    constexpr int WN = BN / 2;   // columns per wavefront
    constexpr int TM = WM / 32;  // MFMA tiles per wavefront, vertically
    constexpr int TN = WN / 32;
    constexpr int LDA = BM + 4;  // k-major A slab: As[k][m]
    constexpr int LDB = BN + 4;  // Bs[k][n]
    constexpr int A_QUADS = BM * kBK / 4 / kThreads;  // 4-element groups per lane
    constexpr int B_QUADS = BN * kBK / 4 / kThreads;

    __shared__ float As[2][kBK * LDA];
    __shared__ float Bs[2][kBK * LDB];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t waveM = wave >> 1;
    const uint32_t waveN = wave & 1;

    uint32_t id = blockIdx.x;
    const uint32_t tn = id % args.tilesN;
    id /= args.tilesN;
    const uint32_t tm = id % args.tilesM;
    const uint32_t unit = id / args.tilesM;

    const float* __restrict__ A;
    const float* __restrict__ B;
    float* __restrict__ out;
    if (args.entries != nullptr)
    {
        const SphGemmEntry e = args.entries[unit];
        A = args.A + e.aOff;
        B = args.B + e.bOff;
        out = args.out + e.outOff;
    }
    else
    {
        A = args.A + args.strideA * static_cast<int64_t>(unit);
        B = args.B + args.strideB * static_cast<int64_t>(unit);
        out = args.out + args.strideOut * static_cast<int64_t>(unit);
    }

    const uint32_t M = args.M, N = args.N, K = args.K;
    const uint32_t rowBase = tm * BM;
    const uint32_t colBase = tn * BN;

    // ---- 4-element groups this lane moves from HBM to LDS -----------------------
    // A as given is M x K (K contiguous); with TA it is K x M.  B as given is K x N (N
    // contiguous); with TB it is N x K.
    float4 stageA[A_QUADS];
    float4 stageB[B_QUADS];

    auto fetch = [&](uint32_t k0) {
        if constexpr (TA)
            FetchXContig<BM, A_QUADS, VEC>(stageA, A, tid, rowBase, M, k0, K);
        else
            FetchKContig<BM, A_QUADS, VEC>(stageA, A, tid, rowBase, M, k0, K);
        if constexpr (TB)
            FetchKContig<BN, B_QUADS, VEC>(stageB, B, tid, colBase, N, k0, K);
        else
            FetchXContig<BN, B_QUADS, VEC>(stageB, B, tid, colBase, N, k0, K);
    };

    auto stash = [&](int buf) {
        if constexpr (TA)
            StashXContig<BM, LDA, A_QUADS>(As[buf], stageA, tid);
        else
            StashKContig<BM, LDA, A_QUADS>(As[buf], stageA, tid);
        if constexpr (TB)
            StashKContig<BN, LDB, B_QUADS>(Bs[buf], stageB, tid);
        else
            StashXContig<BN, LDB, B_QUADS>(Bs[buf], stageB, tid);
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[i][j][v] = 0.f;

    const uint32_t steps = (K + kBK - 1) / kBK;
    if (steps > 0)
    {
        fetch(0);
        stash(0);
    }
    __syncthreads();

    // MFMA 32x32x2 operand layout: lane l supplies A[l % 32][l / 32] and
    // B[l / 32][l % 32]; two k values per instruction.
    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;

    for (uint32_t s = 0; s < steps; ++s)
    {
        const int cur = s & 1;
        if (s + 1 < steps)
            fetch((s + 1) * kBK);

        const float* as = &As[cur][waveM * WM + l32];
        const float* bs = &Bs[cur][waveN * WN + l32];
        // fragments of k pair kk+2 are read while the MFMAs of pair kk run; the fences keep
        // the compiler from sinking the reads back to their first use
        float a[2][TM], b[2][TN];
        auto readPair = [&](int slot, int kk) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
                a[slot][i] = as[(kk + khalf) * LDA + i * 32];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b[slot][j] = bs[(kk + khalf) * LDB + j * 32];
        };
        readPair(0, 0);
#pragma unroll
        for (int kk = 0; kk < kBK; kk += 2)
        {
            const int slot = (kk / 2) & 1;
            if (kk + 2 < kBK)
                readPair(slot ^ 1, kk + 2);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    // operands swapped: the 32x32 result block comes out indexed
                    // [column][row], which leaves 4 consecutive columns in a lane
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[slot][j], a[slot][i],
                                                                     acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }

        if (s + 1 < steps)
            stash(cur ^ 1);
        __syncthreads();
    }

    // ---- out += acc ---------------------------------------------------------
    // With the operands swapped, register v of lane l holds row l%32 and column
    // 8*(v/4) + 4*(l/32) + v%4 of its 32x32 block: registers 4q..4q+3 are 4
    // consecutive columns.  The old values of the whole wavefront block are requested
    // in one batch, then added and stored.
    constexpr int kQuads = TM * TN * 4;
    float4 old[kQuads];
    const bool wide = args.outVec != 0;  // N % 4 == 0 and 16-byte aligned output rows
    const bool accumulate = args.overwrite == 0;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t r = rowBase + waveM * WM + i * 32 + l32;
                const uint32_t c = colBase + waveN * WN + j * 32 + 8 * q + 4 * khalf;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (accumulate && r < M && c < N)
                {
                    const float* p = out + static_cast<size_t>(r) * N + c;
                    if (wide)
                        v = *reinterpret_cast<const float4*>(p);
                    else
                    {
                        v.x = p[0];
                        if (c + 1 < N) v.y = p[1];
                        if (c + 2 < N) v.z = p[2];
                        if (c + 3 < N) v.w = p[3];
                    }
                }
                old[(i * TN + j) * 4 + q] = v;
            }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t r = rowBase + waveM * WM + i * 32 + l32;
                const uint32_t c = colBase + waveN * WN + j * 32 + 8 * q + 4 * khalf;
                if (r < M && c < N)
                {
                    float4 v = old[(i * TN + j) * 4 + q];
                    v.x += acc[i][j][4 * q + 0];
                    v.y += acc[i][j][4 * q + 1];
                    v.z += acc[i][j][4 * q + 2];
                    v.w += acc[i][j][4 * q + 3];
                    float* p = out + static_cast<size_t>(r) * N + c;
                    if (wide)
                        *reinterpret_cast<float4*>(p) = v;
                    else
                    {
                        p[0] = v.x;
                        if (c + 1 < N) p[1] = v.y;
                        if (c + 2 < N) p[2] = v.z;
                        if (c + 3 < N) p[3] = v.w;
                    }
                }
            }
}

// ---------------------------------------------------------------------------
// Few-tile shapes (small M x N, long K): 32 x 32 output tile per workgroup, K split four
// ways across its wavefronts.
//
// With few output tiles the tiled kernel above leaves most compute units idle and is bound by
// the latency of one load -> LDS -> MFMA chain per K step.  Here every wavefront reads its
// operands straight from global memory in MFMA layout (A: 16 bytes per lane along K, lines
// reused from L1 over the next steps; B: one row segment per lane half), keeps several loads
// in flight, and accumulates a private 32 x 32 partial over its quarter of K.  The four
// partials are then added in wavefront order through LDS, so the result does not depend on
// timing.  The two k values of one MFMA come from lanes 0-31 and 32-63; which k each half
// holds is free as long as A and B agree, and is chosen so that A is read with float4.
// ---------------------------------------------------------------------------
constexpr int kSkinnyThreads = 256;

template <bool VEC, bool TA, bool TB>
__global__ __launch_bounds__(kSkinnyThreads) void GemmF32SkinnyKernel(const GemmF32Args args)
{
    __shared__ float partial[3][32 * 32];

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;

    uint32_t id = blockIdx.x;
    const uint32_t tn = id % args.tilesN;
    id /= args.tilesN;
    const uint32_t tm = id % args.tilesM;
    const uint32_t unit = id / args.tilesM;

    const float* __restrict__ A;
    const float* __restrict__ B;
    float* __restrict__ out;
    if (args.entries != nullptr)
    {
        const SphGemmEntry e = args.entries[unit];
        A = args.A + e.aOff;
        B = args.B + e.bOff;
        out = args.out + e.outOff;
    }
    else
    {
        A = args.A + args.strideA * static_cast<int64_t>(unit);
        B = args.B + args.strideB * static_cast<int64_t>(unit);
        out = args.out + args.strideOut * static_cast<int64_t>(unit);
    }
    const uint32_t M = args.M, N = args.N, K = args.K;
    const uint32_t row = tm * 32 + l32;
    const uint32_t col = tn * 32 + l32;

    // this wavefront's K range, in groups of 8 (one float4 of A per lane half)
    const uint32_t groups = (K + 7) / 8;
    const uint32_t perWave = (groups + 3) / 4;
    const uint32_t gBegin = min(wave * perWave, groups);
    const uint32_t gEnd = min(gBegin + perWave, groups);

    const bool rowOk = row < M;
    const bool colOk = col < N;

    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v)
        acc[v] = 0.f;

    // Lane half h holds k = 8*g + 4*h + e for e = 0..3.  An operand stored with K contiguous
    // (A as given, B passed transposed) is read as one 16-byte segment of its row; one stored
    // k-major (B as given, A passed transposed) as 4 elements `ld` apart.
    auto loadAlongK = [&](const float* rowPtr, bool ok, uint32_t g) {
        const uint32_t k = g * 8 + khalf * 4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ok)
        {
            if (VEC)
            {
                if (k < K)
                    v = *reinterpret_cast<const float4*>(rowPtr + k);
            }
            else
            {
                if (k + 0 < K) v.x = rowPtr[k + 0];
                if (k + 1 < K) v.y = rowPtr[k + 1];
                if (k + 2 < K) v.z = rowPtr[k + 2];
                if (k + 3 < K) v.w = rowPtr[k + 3];
            }
        }
        return v;
    };
    auto loadAcrossK = [&](const float* colPtr, size_t ld, bool ok, uint32_t g) {
        const uint32_t k = g * 8 + khalf * 4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ok)
        {
            const float* p = colPtr + static_cast<size_t>(k) * ld;
            if (k + 0 < K) v.x = p[0];
            if (k + 1 < K) v.y = p[ld];
            if (k + 2 < K) v.z = p[2 * ld];
            if (k + 3 < K) v.w = p[3 * ld];
        }
        return v;
    };
    const float* aPtr = TA ? A + min(row, M - 1) : A + static_cast<size_t>(min(row, M - 1)) * K;
    const float* bPtr = TB ? B + static_cast<size_t>(min(col, N - 1)) * K : B + min(col, N - 1);
    auto loadA = [&](uint32_t g) {
        if constexpr (TA)
            return loadAcrossK(aPtr, M, rowOk, g);
        else
            return loadAlongK(aPtr, rowOk, g);
    };
    auto loadB = [&](uint32_t g) {
        if constexpr (TB)
            return loadAlongK(bPtr, colOk, g);
        else
            return loadAcrossK(bPtr, N, colOk, g);
    };

    constexpr int kDepth = 4;  // groups in flight
    float4 fa[kDepth], fb[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; ++d)
    {
        fa[d] = gBegin + d < gEnd ? loadA(gBegin + d) : make_float4(0.f, 0.f, 0.f, 0.f);
        fb[d] = gBegin + d < gEnd ? loadB(gBegin + d) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (uint32_t g = gBegin; g < gEnd; g += kDepth)
    {
#pragma unroll
        for (int d = 0; d < kDepth; ++d)
        {
            const float4 a = fa[d];
            const float4 b = fb[d];
            const uint32_t next = g + kDepth + d;
            fa[d] = next < gEnd ? loadA(next) : make_float4(0.f, 0.f, 0.f, 0.f);
            fb[d] = next < gEnd ? loadB(next) : make_float4(0.f, 0.f, 0.f, 0.f);
            // groups past gEnd carry zeros and add nothing
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.x, a.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.y, a.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.z, a.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b.w, a.w, acc, 0, 0, 0);
        }
    }

    // partial sums of wavefronts 1..3 go through LDS; wavefront 0 adds them in order
    if (wave != 0)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4*>(&partial[wave - 1][l32 * 32 + 8 * q + 4 * khalf]) =
                make_float4(acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
    }
    __syncthreads();
    if (wave != 0)
        return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const float4 p =
                *reinterpret_cast<const float4*>(&partial[w][l32 * 32 + 8 * q + 4 * khalf]);
            acc[4 * q + 0] += p.x;
            acc[4 * q + 1] += p.y;
            acc[4 * q + 2] += p.z;
            acc[4 * q + 3] += p.w;
        }
    // operands were swapped: lane l holds row l%32, columns 8q + 4*(l/32) + 0..3
    if (!rowOk)
        return;
    const bool wide = args.outVec != 0;
#pragma unroll
    for (int q = 0; q < 4; ++q)
    {
        const uint32_t c = tn * 32 + 8 * q + 4 * khalf;
        if (c >= N)
            continue;
        float* p = out + static_cast<size_t>(row) * N + c;
        if (args.overwrite)
        {
            p[0] = acc[4 * q + 0];
            if (c + 1 < N) p[1] = acc[4 * q + 1];
            if (c + 2 < N) p[2] = acc[4 * q + 2];
            if (c + 3 < N) p[3] = acc[4 * q + 3];
        }
        else if (wide)
        {
            float4 v = *reinterpret_cast<const float4*>(p);
            v.x += acc[4 * q + 0];
            v.y += acc[4 * q + 1];
            v.z += acc[4 * q + 2];
            v.w += acc[4 * q + 3];
            *reinterpret_cast<float4*>(p) = v;
        }
        else
        {
            p[0] += acc[4 * q + 0];
            if (c + 1 < N) p[1] += acc[4 * q + 1];
            if (c + 2 < N) p[2] += acc[4 * q + 2];
            if (c + 3 < N) p[3] += acc[4 * q + 3];
        }
    }
}

// Device table for grouped launches: one growing buffer per device with a
// pinned staging copy.  The table is shared by every caller, so its use is
// serialised by a mutex and, across streams, by waiting for the stream that
// used it last.
struct EntryTable
{
    SphGemmEntry* dev = nullptr;
    SphGemmEntry* staging = nullptr;  // pinned
    size_t capacity = 0;
    hipEvent_t uploaded = nullptr;    // staging may be overwritten after this
    bool uploadPending = false;
    hipStream_t lastStream = nullptr;
};
std::mutex gTableMutex;
EntryTable gTables[16];

template <bool TA, bool TB>
void LaunchSkinny(const GemmF32Args& args, dim3 grid, bool vec, hipStream_t stream)
{
    if (vec)
        hipLaunchKernelGGL((GemmF32SkinnyKernel<true, TA, TB>), grid, dim3(kSkinnyThreads), 0,
                           stream, args);
    else
        hipLaunchKernelGGL((GemmF32SkinnyKernel<false, TA, TB>), grid, dim3(kSkinnyThreads), 0,
                           stream, args);
}

template <bool TA, bool TB>
void LaunchTiled(const GemmF32Args& args, dim3 grid, bool big, bool vec, hipStream_t stream)
{
    const dim3 block(kThreads);
    if (big)
    {
        if (vec)
            hipLaunchKernelGGL((GemmF32Kernel<128, 128, true, TA, TB>), grid, block, 0, stream,
                               args);
        else
            hipLaunchKernelGGL((GemmF32Kernel<128, 128, false, TA, TB>), grid, block, 0, stream,
                               args);
    }
    else
    {
        if (vec)
            hipLaunchKernelGGL((GemmF32Kernel<64, 64, true, TA, TB>), grid, block, 0, stream,
                               args);
        else
            hipLaunchKernelGGL((GemmF32Kernel<64, 64, false, TA, TB>), grid, block, 0, stream,
                               args);
    }
}

// `transA`: A is stored K x M; `transB`: B is stored N x K.
int Launch(const GemmF32Args& base, uint32_t units, bool allowVector, bool outOffsetsAligned,
           bool transA, bool transB, hipStream_t stream)
{
    GemmF32Args args = base;
    args.outVec = (outOffsetsAligned && (args.N % 4 == 0) &&
                   (reinterpret_cast<uintptr_t>(args.out) & 15u) == 0)
                      ? 1u
                      : 0u;
    const bool basesAligned =
        ((reinterpret_cast<uintptr_t>(args.A) | reinterpret_cast<uintptr_t>(args.B)) & 15u) == 0;
    // row lengths of the two operands as stored
    const uint32_t lda = transA ? args.M : args.K;
    const uint32_t ldb = transB ? args.K : args.N;
    const bool aligned = allowVector && basesAligned && (lda % 4 == 0) && (ldb % 4 == 0);

    // few 64 x 64 tiles and a long K: split K inside the workgroup instead
    const uint64_t tiles64 =
        static_cast<uint64_t>((args.M + 63) / 64) * ((args.N + 63) / 64) * units;
    if (tiles64 * 2 <= static_cast<uint64_t>(sph::ComputeUnits()) && args.K >= 64)
    {
        args.tilesM = (args.M + 31) / 32;
        args.tilesN = (args.N + 31) / 32;
        const uint64_t blocks32 = static_cast<uint64_t>(args.tilesM) * args.tilesN * units;
        const dim3 grid32(static_cast<uint32_t>(blocks32));
        // 16-byte loads are used only for operands stored with K contiguous
        bool kVec = allowVector && (args.K % 4 == 0);
        if (!transA)
            kVec = kVec && (reinterpret_cast<uintptr_t>(args.A) & 15u) == 0;
        if (transB)
            kVec = kVec && (reinterpret_cast<uintptr_t>(args.B) & 15u) == 0;
        if (transA && transB)
            LaunchSkinny<true, true>(args, grid32, kVec, stream);
        else if (transA)
            LaunchSkinny<true, false>(args, grid32, false, stream);
        else if (transB)
            LaunchSkinny<false, true>(args, grid32, kVec, stream);
        else
            LaunchSkinny<false, false>(args, grid32, kVec, stream);
        SPH_CHECK_LAUNCH();
        return SPH_OK;
    }

    const uint64_t tiles128 =
        static_cast<uint64_t>((args.M + 127) / 128) * ((args.N + 127) / 128) * units;
    const bool big = tiles128 >= static_cast<uint64_t>(sph::ComputeUnits());
    const uint32_t bm = big ? 128 : 64;
    args.tilesM = (args.M + bm - 1) / bm;
    args.tilesN = (args.N + bm - 1) / bm;
    const uint64_t blocks = static_cast<uint64_t>(args.tilesM) * args.tilesN * units;
    if (blocks >= (1ull << 31))
        return sph::Fail(SPH_ERR_INVALID, "sph_gemm_f32 - too many tiles for one launch");

    const dim3 grid(static_cast<uint32_t>(blocks));
    if (transA && transB)
        LaunchTiled<true, true>(args, grid, big, aligned, stream);
    else if (transA)
        LaunchTiled<true, false>(args, grid, big, aligned, stream);
    else if (transB)
        LaunchTiled<false, true>(args, grid, big, aligned, stream);
    else
        LaunchTiled<false, false>(args, grid, big, aligned, stream);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int GrowTable(EntryTable& t, size_t count)
{
    if (t.capacity >= count)
        return SPH_OK;
    // nothing may still be reading the old buffers
    if (t.lastStream != nullptr)
        SPH_HIP_TRY(hipStreamSynchronize(t.lastStream));
    if (t.dev != nullptr)
        SPH_HIP_TRY(hipFree(t.dev));
    if (t.staging != nullptr)
        SPH_HIP_TRY(hipHostFree(t.staging));
    t.dev = nullptr;
    t.staging = nullptr;
    t.capacity = 0;
    t.uploadPending = false;
    size_t cap = 1024;
    while (cap < count)
        cap *= 2;
    SPH_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&t.dev), cap * sizeof(SphGemmEntry)));
    SPH_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&t.staging), cap * sizeof(SphGemmEntry),
                              hipHostMallocDefault));
    if (t.uploaded == nullptr)
        SPH_HIP_TRY(hipEventCreateWithFlags(&t.uploaded, hipEventDisableTiming));
    t.capacity = cap;
    return SPH_OK;
}
}  // namespace

extern "C" {

int sph_gemm_f32_ex(float* out, const float* A, const float* B, uint32_t M, uint32_t N,
                    uint32_t K, uint32_t batch, int64_t strideOut, int64_t strideA,
                    int64_t strideB, uint32_t flags)
{
    SPH_REQUIRE(M != 0 && N != 0 && batch != 0, "M, N and batch must be non-zero");
    SPH_REQUIRE((flags & ~(SPH_GEMM_OVERWRITE | SPH_GEMM_TRANS_A | SPH_GEMM_TRANS_B)) == 0,
                "unknown flag");
    const bool overwrite = (flags & SPH_GEMM_OVERWRITE) != 0;
    if (K == 0 && !overwrite)
        return SPH_OK;
    SPH_REQUIRE(out != nullptr, "null pointer");
    SPH_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "null pointer");
    SPH_REQUIRE(strideOut >= 0 && strideA >= 0 && strideB >= 0, "negative stride");
    SPH_REQUIRE(batch == 1 || strideOut >= static_cast<int64_t>(M) * N,
                "output matrices of a batch must not overlap");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;

    GemmF32Args args{};
    args.out = out;
    args.A = A;
    args.B = B;
    args.entries = nullptr;
    args.M = M;
    args.N = N;
    args.K = K;
    args.overwrite = overwrite ? 1u : 0u;
    args.strideOut = strideOut;
    args.strideA = strideA;
    args.strideB = strideB;
    const bool stridesAligned = (strideA % 4 == 0) && (strideB % 4 == 0);
    return Launch(args, batch, stridesAligned, strideOut % 4 == 0 || batch == 1,
                  (flags & SPH_GEMM_TRANS_A) != 0, (flags & SPH_GEMM_TRANS_B) != 0, stream);
}

int sph_gemm_f32(float* out, const float* A, const float* B, uint32_t M, uint32_t N, uint32_t K,
                 uint32_t batch, int64_t strideOut, int64_t strideA, int64_t strideB)
{
    return sph_gemm_f32_ex(out, A, B, M, N, K, batch, strideOut, strideA, strideB,
                           SPH_GEMM_ACCUMULATE);
}

int sph_gemm_f32_grouped(const SphGemmEntry* entries, uint32_t count, float* out, const float* A,
                         const float* B, uint32_t M, uint32_t N, uint32_t K)
{
    SPH_REQUIRE(M != 0 && N != 0, "M and N must be non-zero");
    if (count == 0 || K == 0)
        return SPH_OK;
    SPH_REQUIRE(entries != nullptr && out != nullptr && A != nullptr && B != nullptr,
                "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;

    bool offsetsAligned = true, outAligned = true;
    for (uint32_t i = 0; i < count; ++i)
    {
        offsetsAligned = offsetsAligned && ((entries[i].aOff | entries[i].bOff) % 4) == 0;
        outAligned = outAligned && (entries[i].outOff % 4) == 0;
    }

    std::lock_guard<std::mutex> lock(gTableMutex);
    EntryTable& t = gTables[sph::CurrentDevice()];
    {
        const int rc = GrowTable(t, count);
        if (rc != SPH_OK)
            return rc;
    }
    if (t.lastStream != nullptr && t.lastStream != stream)
        SPH_HIP_TRY(hipStreamSynchronize(t.lastStream));
    if (t.uploadPending)
        SPH_HIP_TRY(hipEventSynchronize(t.uploaded));
    std::memcpy(t.staging, entries, count * sizeof(SphGemmEntry));
    SPH_HIP_TRY(hipMemcpyAsync(t.dev, t.staging, count * sizeof(SphGemmEntry),
                               hipMemcpyHostToDevice, stream));
    SPH_HIP_TRY(hipEventRecord(t.uploaded, stream));
    t.uploadPending = true;
    t.lastStream = stream;

    // Entries that add into the same output unit must be applied in order:
    // cut the list into launches inside which every outOff is distinct.
    uint32_t begin = 0;
    std::unordered_set<uint64_t> seen;
    while (begin < count)
    {
        seen.clear();
        uint32_t end = begin;
        while (end < count && seen.insert(entries[end].outOff).second)
            ++end;

        GemmF32Args args{};
        args.out = out;
        args.A = A;
        args.B = B;
        args.entries = t.dev + begin;
        args.M = M;
        args.N = N;
        args.K = K;
        const int rc = Launch(args, end - begin, offsetsAligned, outAligned, false, false, stream);
        if (rc != SPH_OK)
            return rc;
        begin = end;
    }
    return SPH_OK;
}

}  // extern "C"
