// fp16-input / fp32-accumulate GEMM  out[u] (+)= A[u] * B[u]  on the CDNA4
// matrix cores (v_mfma_f32_32x32x16_f16).  This is the tensor-core path the
// reference only declares (WmmaGemm,
// Includes/Sapphire/compute/dense/cuda/kernels/GemmKernel.cuh:14-50): half
// inputs, fp32 accumulation, row-major operands, result added into out.
//
// Two kernels:
//
//   GemmF16Tile256  M, N multiples of 256, K a multiple of 64, 16-byte aligned
//     rows.  One workgroup of 8 wavefronts (2 x 4) owns a 256 x 256 output
//     tile; each wavefront a 128 x 64 part of it (4 x 2 MFMA tiles, 128
//     accumulator registers).  K advances 64 at a time through two LDS stages
//     of 64 KiB (A 256x64, B 64x256).  Global memory is copied straight into
//     LDS (global_load_lds, 16 bytes per lane, no VGPR staging); the copy of
//     stage i+1 is in flight while the MFMAs of stage i run.  LDS is written
//     lane-linear by those copies, so bank conflicts are removed by choosing
//     WHICH global chunk each lane fetches: A rows are XOR-swizzled in 16-byte
//     chunks (chunk ^ row%8), B rows in 32-byte chunks (chunk ^ 2*(k%4)); both
//     patterns measured conflict-free for the reads below.
//     A fragments are read with ds_read_b128 (8 consecutive k of one row); B is
//     stored k-major, so its fragments (8 consecutive k of one column) come
//     from two ds_read_b64_tr_b16 transposing reads.  The MFMA operands are
//     swapped (B fragment first) so that every lane ends up with 4 consecutive
//     columns of one output row and the epilogue moves 16 bytes per access.
//     Workgroup ids are remapped so that the 32 workgroups that land on one
//     XCD (ids congruent mod 8) cover a compact 8 x 4 block of tiles and share
//     their A and B panels through that XCD's L2.
//
//   GemmF16General  any shape.  128 x 128 tile, 4 wavefronts, K step 32, global
//     loads staged through registers with per-element predication (16-byte
//     loads when K, N and the bases allow), padded LDS rows.
#include "sph_internal.h"

namespace
{
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* LdsPtr;
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4* LdsShortx4Ptr;

struct GemmF16Args
{
    float* out;
    const _Float16* A;
    const _Float16* B;
    uint32_t M, N, K;
    uint32_t tilesM, tilesN;
    uint32_t totalTiles;  // tilesM * tilesN * batch
    int64_t strideOut, strideA, strideB;
    uint32_t overwrite;
};

// Transposing LDS read: within each group of 16 lanes, lane s supplies the
// address of 4 halves (row s/4 of a 4-row block, columns 4*(s%4)..+3) and
// receives the 4 rows' values of column s.
__device__ __forceinline__ halfx4 LdsReadTr(const _Float16* p)
{
    return __builtin_bit_cast(halfx4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsShortx4Ptr)(p)));
}

__device__ __forceinline__ halfx8 Join(halfx4 lo, halfx4 hi)
{
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Spreads consecutive workgroup ids, which the hardware deals round-robin to
// the 8 XCDs, so that each XCD works on one contiguous range of the tile
// order, and lays that order out in bands of 8 tile rows walked column by
// column.  Returns false for the padding ids of the last range.
__device__ __forceinline__ bool MapTile(uint32_t id, uint32_t tilesM, uint32_t tilesN,
                                        uint32_t totalTiles, uint32_t& unit, uint32_t& tm,
                                        uint32_t& tn)
{
    const uint32_t perXcd = (totalTiles + 7) / 8;
    const uint32_t linear = (id % 8) * perXcd + id / 8;
    if (linear >= totalTiles)
        return false;
    const uint32_t perUnit = tilesM * tilesN;
    unit = linear / perUnit;
    const uint32_t t = linear % perUnit;
    constexpr uint32_t kBand = 8;
    const uint32_t bandSize = kBand * tilesN;
    const uint32_t band = t / bandSize;
    const uint32_t inBand = t % bandSize;
    const uint32_t rowsHere = min(kBand, tilesM - band * kBand);
    tm = band * kBand + inBand % rowsHere;
    tn = inBand / rowsHere;
    return true;
}

// ---------------------------------------------------------------------------
// 256 x 256 x 64 tile kernel
// ---------------------------------------------------------------------------
constexpr int kT = 256;         // tile edge
constexpr int kTK = 64;         // K step
constexpr int kTThreads = 512;  // 8 wavefronts
constexpr int kStageHalfs = kT * kTK;  // per operand per stage (32 KiB)

__global__ __launch_bounds__(kTThreads) void GemmF16Tile256(const GemmF16Args args)
{
    __shared__ __attribute__((aligned(1024))) _Float16 As[2][kStageHalfs];  // [row][64], swizzled
    __shared__ __attribute__((aligned(1024))) _Float16 Bs[2][kStageHalfs];  // [k][256], swizzled

    uint32_t unit, tm, tn;
    if (!MapTile(blockIdx.x, args.tilesM, args.tilesN, args.totalTiles, unit, tm, tn))
        return;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t waveM = wave >> 2;  // 0..1 -> 128 rows each
    const uint32_t waveN = wave & 3;   // 0..3 -> 64 columns each

    const uint32_t K = args.K, N = args.N;
    const _Float16* __restrict__ A =
        args.A + args.strideA * static_cast<int64_t>(unit) + static_cast<size_t>(tm) * kT * K;
    const _Float16* __restrict__ B =
        args.B + args.strideB * static_cast<int64_t>(unit) + static_cast<size_t>(tn) * kT;
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit) +
                              static_cast<size_t>(tm) * kT * N + static_cast<size_t>(tn) * kT;

    // ---- global -> LDS copy plan --------------------------------------------
    // Each pass moves 8 KiB per operand: wavefront w writes the 1 KiB at
    // pass*8192 + w*1024, lane i its 16 bytes at + i*16.
    //   A stage [256 rows][128 B]: that is row pass*64 + w*8 + i/8, physical
    //     chunk i%8, which must hold logical chunk (i%8) ^ (row%8) = (i%8)^(i/8).
    //   B stage [64 k][512 B]: k = pass*16 + w*2 + i/32, physical 16-byte chunk
    //     i%32; 32-byte chunks are swizzled with 2*(k%4).
    const uint32_t aRow = wave * 8 + (lane >> 3);                  // + pass*64
    const uint32_t aChunk = (lane & 7) ^ (lane >> 3);              // logical
    const _Float16* aSrc = A + static_cast<size_t>(aRow) * K + aChunk * 8;
    const size_t aPassStride = static_cast<size_t>(64) * K;

    const uint32_t bK = wave * 2 + (lane >> 5);                    // + pass*16
    const uint32_t bPhys16 = lane & 31;
    const uint32_t bLogical16 = (((bPhys16 >> 1) ^ (2 * (bK & 3))) << 1) | (bPhys16 & 1);
    const _Float16* bSrc = B + static_cast<size_t>(bK) * N + bLogical16 * 8;
    const size_t bPassStride = static_cast<size_t>(16) * N;

    auto copyStage = [&](int stage, uint32_t kt) {
        const _Float16* a = aSrc + static_cast<size_t>(kt) * kTK;
        const _Float16* b = bSrc + static_cast<size_t>(kt) * kTK * N;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass)
        {
            __builtin_amdgcn_global_load_lds(
                a + pass * aPassStride,
                (LdsPtr)(&As[stage][pass * 4096 + wave * 512]), 16, 0, 0);
        }
#pragma unroll
        for (int pass = 0; pass < 4; ++pass)
        {
            __builtin_amdgcn_global_load_lds(
                b + pass * bPassStride,
                (LdsPtr)(&Bs[stage][pass * 4096 + wave * 512]), 16, 0, 0);
        }
    };

    // ---- LDS -> fragment read plan ------------------------------------------
    // A fragment (MFMA tile row block i, k sub-step ks): lane l reads row
    //   waveM*128 + i*32 + l%32, logical chunk ks*2 + l/32.
    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;
    const uint32_t aFragRow = waveM * 128 + l32;  // + i*32 (row%8 unchanged)
    const uint32_t aRowSwz = aFragRow & 7;
    // B fragment (tile column block j, sub-step ks): 16-lane group g = l/16,
    //   s = l%16; columns waveN*64 + j*32 + 16*(g%2) + 4*(s%4)..+3,
    //   k = ks*16 + 8*(g/2) + 4*h + s/4 for the two reads h = 0, 1.
    const uint32_t g = lane >> 4;
    const uint32_t s = lane & 15;
    const uint32_t bKLocal = 8 * (g >> 1) + (s >> 2);               // + ks*16 + 4*h
    const uint32_t bCol32 = (waveN * 64 + 16 * (g & 1)) / 16;       // + j*2, logical 32B chunk
    const uint32_t bSwz = 2 * ((s >> 2) & 3);                       // 2*(k%4)
    const uint32_t bInChunk = (s & 3) * 4;                          // halves inside the 32B chunk

    floatx16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[i][j][v] = 0.f;

    const uint32_t steps = K / kTK;
    copyStage(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (uint32_t kt = 0; kt < steps; ++kt)
    {
        const int cur = kt & 1;
        if (kt + 1 < steps)
            copyStage(cur ^ 1, kt + 1);

        const _Float16* as = As[cur];
        const _Float16* bs = Bs[cur];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
        {
            halfx8 af[4];
            halfx8 bf[2];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const uint32_t chunk = (ks * 2 + khalf) ^ aRowSwz;
                af[i] = *reinterpret_cast<const halfx8*>(as + (aFragRow + i * 32) * kTK +
                                                         chunk * 8);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j)
            {
                const uint32_t chunk32 = (bCol32 + j * 2) ^ bSwz;
                const _Float16* p = bs + (ks * 16 + bKLocal) * kT + chunk32 * 16 + bInChunk;
                const halfx4 lo = LdsReadTr(p);
                const halfx4 hi = LdsReadTr(p + 4 * kT);
                bf[j] = Join(lo, hi);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j],
                                                                       0, 0, 0);
        }

        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // ---- epilogue -------------------------------------------------------------
    // With the operands swapped the 32x32 result block is indexed [n][m]:
    // register v of lane l holds column 8*(v/4) + 4*(l/32) + v%4 of row l%32,
    // i.e. registers 4q..4q+3 are 4 consecutive columns.
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const uint32_t r = waveM * 128 + i * 32 + l32;
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t c = waveN * 64 + j * 32 + 8 * q + 4 * khalf;
                float4* p = reinterpret_cast<float4*>(out + static_cast<size_t>(r) * N + c);
                float4 v = make_float4(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1],
                                       acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
                if (!args.overwrite)
                {
                    const float4 old = *p;
                    v.x += old.x;
                    v.y += old.y;
                    v.z += old.z;
                    v.w += old.w;
                }
                *p = v;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// general kernel: 128 x 128 x 32, any shape
// ---------------------------------------------------------------------------
constexpr int kG = 128;
constexpr int kGK = 32;
constexpr int kGThreads = 256;
constexpr int kGLda = kGK + 8;   // halves per A row in LDS (80 B)
constexpr int kGLdb = kG + 32;   // halves per B row in LDS (320 B)

template <bool VEC>
__global__ __launch_bounds__(kGThreads) void GemmF16General(const GemmF16Args args)
{
    __shared__ __attribute__((aligned(16))) _Float16 As[2][kG * kGLda];
    __shared__ __attribute__((aligned(16))) _Float16 Bs[2][kGK * kGLdb];

    uint32_t unit, tm, tn;
    if (!MapTile(blockIdx.x, args.tilesM, args.tilesN, args.totalTiles, unit, tm, tn))
        return;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t waveM = wave >> 1;
    const uint32_t waveN = wave & 1;
    const uint32_t M = args.M, N = args.N, K = args.K;

    const _Float16* __restrict__ A = args.A + args.strideA * static_cast<int64_t>(unit);
    const _Float16* __restrict__ B = args.B + args.strideB * static_cast<int64_t>(unit);
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit);
    const uint32_t rowBase = tm * kG;
    const uint32_t colBase = tn * kG;

    halfx8 stageA[2], stageB[2];

    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            const uint32_t gr = rowBase + q / 4;
            const uint32_t gk = k0 + (q % 4) * 8;
            halfx8 v = { 0, 0, 0, 0, 0, 0, 0, 0 };
            if (gr < M)
            {
                const _Float16* p = A + static_cast<size_t>(gr) * K + gk;
                if (VEC)
                {
                    if (gk < K)
                        v = *reinterpret_cast<const halfx8*>(p);
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (gk + e < K)
                            v[e] = p[e];
                }
            }
            stageA[i] = v;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            const uint32_t gk = k0 + q / 16;
            const uint32_t gc = colBase + (q % 16) * 8;
            halfx8 v = { 0, 0, 0, 0, 0, 0, 0, 0 };
            if (gk < K)
            {
                const _Float16* p = B + static_cast<size_t>(gk) * N + gc;
                if (VEC)
                {
                    if (gc < N)
                        v = *reinterpret_cast<const halfx8*>(p);
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (gc + e < N)
                            v[e] = p[e];
                }
            }
            stageB[i] = v;
        }
    };

    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            *reinterpret_cast<halfx8*>(&As[buf][(q / 4) * kGLda + (q % 4) * 8]) = stageA[i];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            *reinterpret_cast<halfx8*>(&Bs[buf][(q / 16) * kGLdb + (q % 16) * 8]) = stageB[i];
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[i][j][v] = 0.f;

    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;
    const uint32_t g = lane >> 4;
    const uint32_t s = lane & 15;

    const uint32_t steps = (K + kGK - 1) / kGK;
    if (steps > 0)
    {
        fetch(0);
        stash(0);
    }
    __syncthreads();

    for (uint32_t kt = 0; kt < steps; ++kt)
    {
        const int cur = kt & 1;
        if (kt + 1 < steps)
            fetch((kt + 1) * kGK);

        const _Float16* as = As[cur];
        const _Float16* bs = Bs[cur];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
        {
            halfx8 af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[i] = *reinterpret_cast<const halfx8*>(
                    as + (waveM * 64 + i * 32 + l32) * kGLda + (ks * 2 + khalf) * 8);
#pragma unroll
            for (int j = 0; j < 2; ++j)
            {
                const _Float16* p = bs + (ks * 16 + 8 * (g >> 1) + (s >> 2)) * kGLdb +
                                    waveN * 64 + j * 32 + 16 * (g & 1) + (s & 3) * 4;
                bf[j] = Join(LdsReadTr(p), LdsReadTr(p + 4 * kGLdb));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j],
                                                                       0, 0, 0);
        }

        if (kt + 1 < steps)
            stash(cur ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
    {
        const uint32_t r = rowBase + waveM * 64 + i * 32 + l32;
        if (r >= M)
            continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t c = colBase + waveN * 64 + j * 32 + 8 * q + 4 * khalf;
                float* p = out + static_cast<size_t>(r) * N + c;
                if (VEC && (N % 4 == 0))
                {
                    if (c < N)
                    {
                        float4* p4 = reinterpret_cast<float4*>(p);
                        float4 v = make_float4(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1],
                                               acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
                        if (!args.overwrite)
                        {
                            const float4 old = *p4;
                            v.x += old.x;
                            v.y += old.y;
                            v.z += old.z;
                            v.w += old.w;
                        }
                        *p4 = v;
                    }
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (c + e < N)
                            p[e] = args.overwrite ? acc[i][j][4 * q + e]
                                                  : p[e] + acc[i][j][4 * q + e];
                }
            }
    }
}
}  // namespace

extern "C" {

int sph_gemm_f16f32(float* out, const sph_f16* A, const sph_f16* B, uint32_t M, uint32_t N,
                    uint32_t K, uint32_t batch, int64_t strideOut, int64_t strideA,
                    int64_t strideB, uint32_t flags)
{
    SPH_REQUIRE(M != 0 && N != 0 && batch != 0, "M, N and batch must be non-zero");
    SPH_REQUIRE((flags & ~SPH_GEMM_OVERWRITE) == 0, "unknown flag");
    SPH_REQUIRE(out != nullptr, "null pointer");
    SPH_REQUIRE(strideOut >= 0 && strideA >= 0 && strideB >= 0, "negative stride");
    SPH_REQUIRE(batch == 1 || strideOut >= static_cast<int64_t>(M) * N,
                "output matrices of a batch must not overlap");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    if (K == 0)
    {
        if (flags & SPH_GEMM_OVERWRITE)
        {
            // an empty sum stored over out
            for (uint32_t b = 0; b < batch; ++b)
            {
                const int rc = sph_fill_f32(out + strideOut * static_cast<int64_t>(b), 0.f,
                                            static_cast<size_t>(M) * N);
                if (rc != SPH_OK)
                    return rc;
            }
        }
        return SPH_OK;
    }
    SPH_REQUIRE(A != nullptr && B != nullptr, "null pointer");

    GemmF16Args args{};
    args.out = out;
    args.A = reinterpret_cast<const _Float16*>(A);
    args.B = reinterpret_cast<const _Float16*>(B);
    args.M = M;
    args.N = N;
    args.K = K;
    args.strideOut = strideOut;
    args.strideA = strideA;
    args.strideB = strideB;
    args.overwrite = (flags & SPH_GEMM_OVERWRITE) ? 1u : 0u;

    const bool aligned16 =
        ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) |
          reinterpret_cast<uintptr_t>(out)) & 15u) == 0 &&
        (strideA % 8 == 0) && (strideB % 8 == 0) && (strideOut % 4 == 0);

    const bool tile256 = aligned16 && (M % kT == 0) && (N % kT == 0) && (K % kTK == 0);
    const uint32_t edge = tile256 ? kT : kG;
    args.tilesM = (M + edge - 1) / edge;
    args.tilesN = (N + edge - 1) / edge;
    const uint64_t total = static_cast<uint64_t>(args.tilesM) * args.tilesN * batch;
    SPH_REQUIRE(total < (1ull << 31) - 8, "too many tiles for one launch");
    args.totalTiles = static_cast<uint32_t>(total);
    const uint32_t grid = ((args.totalTiles + 7) / 8) * 8;

    if (tile256)
    {
        hipLaunchKernelGGL(GemmF16Tile256, dim3(grid), dim3(kTThreads), 0, stream, args);
    }
    else
    {
        const bool vec = aligned16 && (K % 8 == 0) && (N % 8 == 0);
        if (vec)
            hipLaunchKernelGGL(GemmF16General<true>, dim3(grid), dim3(kGThreads), 0, stream, args);
        else
            hipLaunchKernelGGL(GemmF16General<false>, dim3(grid), dim3(kGThreads), 0, stream,
                               args);
    }
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

}  // extern "C"
