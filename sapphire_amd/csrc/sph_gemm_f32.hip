// fp32 GEMM  out[u] += A[u] * B[u]  on the CDNA4 matrix cores.
//
// Storage, products and accumulation are all fp32 (v_mfma_f32_32x32x2_f32, and
// v_mfma_f32_16x16x4_f32 in the few-tile kernel), so
// the only difference from the reference's scalar CPU loop
// (Sources/Sapphire/compute/dense/naive/NaiveGemm.cpp:12-38) is the order in
// which the K products are summed.
//
// Four kernels, chosen from the shape and the alignment of the operands:
//   GemmF32DmaKernel     16-byte aligned bases, K >= 16, an N (an M, for A stored K x M) that
//                        is a multiple of 4: slabs travel global -> LDS without staging
//                        registers, several K steps ahead (the fast path; a K that is no
//                        multiple of the step ends in a partial step);
//                        with more 64-tiles than resident workgroups each workgroup walks
//                        several tiles and the copy stream runs across the tile boundaries;
//                        with 65 to 128 tiles of 64 x 64, 64 x 32 tiles whose K steps are
//                        split over two groups of wavefronts (KSPLIT = 2: another order of
//                        the K products, chosen for the whole product at once);
//   GemmF32Kernel        any shape and alignment: register-staged double buffering, 16-byte
//                        loads when possible, scalar predicated loads otherwise (small K,
//                        misaligned bases, e.g. some of the reference's random test sizes,
//                        Tests/UnitTests/Sources/FunctionTest/GemmTest.cpp:26-33);
//   GemmF32SkinnyKernel  few output tiles: 16 x 16 or 32 x 32 tiles with K split over the
//                        wavefronts of a workgroup;
//   GemvRowKernel        a single output row.
// A product for the tiled kernels is cut by the launcher into a body and up to two thin strips:
// the last N % 4 columns, the last M % 4 rows (from 68 rows up) and up to 16 rows or columns
// just past a tile edge.  The strips are computed by the few-tile kernel's code on the last
// workgroups of the body's own launch (GemmF32Strips), or by launches of their own beside a
// register-staged body.
// The first two share one decomposition: a workgroup (4 wavefronts, 2 x 2) owns a BM x BN tile
// of one M x N unit, BM = BN = 128 or 64 (whichever loads the busiest compute unit less),
// and they add the K products of an element in the same order, so which of them
// runs never changes a bit.  Either operand may be stored transposed (template flags), the
// result may overwrite out or take a bias row and a ReLU in the epilogue, and units come from
// (batch, stride) arithmetic -- stride 0 repeats an operand -- or from a table of element
// offsets in device memory.
#include "sph_internal.h"
#include "sph_k_partition.h"

#include <algorithm>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <unordered_set>
#include <vector>

namespace
{
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
// four floats that need only be 4-byte aligned: the rows of out start anywhere when N is no
// multiple of 4, and a 16-byte vector memory access only asks for dword alignment
typedef floatx4 floatx4a4 __attribute__((aligned(4)));

constexpr int kThreads = 256;
constexpr int kBK = 16;

struct GemmF32Args
{
    float* out;
    const float* A;
    const float* B;
    const SphGemmEntry* entries;  // device table, or null for stride arithmetic
    uint32_t M, N, K;
    // floats between consecutive rows of B as stored K x N and of out: N, unless a launch covers
    // some of the columns of a wider matrix; likewise of an A stored K x M: M, unless a launch
    // covers some of the rows
    uint32_t ldb, ldc, lda;
    uint32_t split;      // launcher: 1 = a part of the columns, 2 = a part of the rows, 4 = the
                         // tiled kernels have been chosen, 8 = the K-split kernel among them,
                         // 16 = a thin strip of a wider product: the few-tile kernel, 16 x 16
                         // tiles, four wavefronts
    uint32_t basesOk;    // launcher: the caller's A and B start on 16-byte boundaries
    uint32_t tilesM, tilesN;
    uint32_t tilesTotal;  // tilesM * tilesN * units
    uint32_t perXcd;      // ceil(tilesTotal / 8): the grid has 8 * perXcd workgroups
    uint32_t band;        // tile rows per band of the in-unit ordering
    uint32_t outVec;     // 16-byte accesses to out are possible
    uint32_t overwrite;  // out = A*B instead of out += A*B
    uint32_t relu;       // out = max(., 0) applied to the value that is stored
    const float* bias;   // when set: out = (0 + bias[column]) + A*B, out is not read
    // when sgd is set: out = out - ((A*B) * sgdScale) * sgdRate, every operation rounded on its
    // own -- the update Scale + Sub apply to a gradient that was stored first
    uint32_t sgd;
    float sgdScale, sgdRate;
    int64_t strideOut, strideA, strideB;
};

// Thin strips of a product's last rows and columns that ride along with the launch of its body:
// the workgroups from `first` on (the body's own come before, so they keep their numbers and with
// them their place among the 8 XCDs) run the few-tile kernel's code on part[0] (blocks[0] of
// them) and then part[1] (blocks[1]).  A strip's workgroups are short; coming last they fill the
// places that the body's last tiles leave free, where a launch of their own would start after the
// body's last tile has finished.  (Placed first they cost a large product a round of tiles on
// some compute units: 4096 x 4095 x 4096 with B stored N x K 931 -> 1147 us.)
struct GemmF32Strips
{
    GemmF32Args part[2];
    uint32_t blocks[2];
    uint32_t first;  // launcher: the number of the body's workgroups
};

// Slab loaders.  An operand is stored either with K contiguous (A as given, B when it is
// passed transposed: `rows` indexes M or N) or with the M/N index contiguous (B as given, A
// when it is passed transposed: `rows` indexes K).  Both end up k-major in LDS, S[k][x].
template <int BX, int QUADS, bool VEC>
__device__ __forceinline__ void FetchKContig(float4 (&stage)[QUADS], const float* __restrict__ src,
                                             uint32_t tid, uint32_t xBase, uint32_t xLimit,
                                             uint32_t k0, uint32_t K)  // rows of K floats
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
                                             uint32_t k0, uint32_t K, uint32_t pitch)
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
            const float* p = src + static_cast<size_t>(gk) * pitch + gx;
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

// Workgroup -> tile.  Workgroups are handed to the 8 XCDs round robin (id % 8), and each XCD
// has its own L2.  Workgroup `id` therefore takes logical tile (id % 8) * perXcd + id / 8, so
// that an XCD owns one contiguous run of logical tiles; inside a unit the logical order walks
// bands of `band` tile rows column by column, which makes a run a compact block of the
// output whose A rows and B columns the XCD's workgroups share.  Returns false for the
// surplus workgroups of a grid rounded up to 8 * perXcd.
__device__ __forceinline__ void MapLogical(const GemmF32Args& args, uint32_t logical, uint32_t& tm,
                                           uint32_t& tn, uint32_t& unit)
{
    const uint32_t perUnit = args.tilesM * args.tilesN;
    unit = logical / perUnit;
    const uint32_t t = logical - unit * perUnit;
    const uint32_t perBand = args.band * args.tilesN;
    const uint32_t bandIdx = t / perBand;
    const uint32_t within = t - bandIdx * perBand;
    const uint32_t rows = min(args.band, args.tilesM - bandIdx * args.band);
    tm = bandIdx * args.band + within % rows;
    tn = within / rows;
}

__device__ __forceinline__ bool MapTile(const GemmF32Args& args, uint32_t& tm, uint32_t& tn,
                                        uint32_t& unit)
{
    const uint32_t id = blockIdx.x;
    const uint32_t logical = (id & 7u) * args.perXcd + (id >> 3);
    if (logical >= args.tilesTotal)
        return false;
    MapLogical(args, logical, tm, tn, unit);
    return true;
}

// What is stored for an element whose old value (or bias term) is `old` and whose product sum
// is `sum`.  Contraction is off: a fused multiply-add would round once where the separate
// Scale and Sub of the optimizer round twice.
__device__ __forceinline__ float Combine(const GemmF32Args& args, float old, float sum)
{
#pragma clang fp contract(off)
    if (args.sgd != 0)
    {
        const float scaled = sum * args.sgdScale;
        const float step = scaled * args.sgdRate;
        return old - step;
    }
    return old + sum;
}

// k index (inside a 16-wide step) that lane half `khalf` feeds to MFMA instruction t
__device__ __forceinline__ constexpr uint32_t KOfPair(uint32_t t, uint32_t khalf)
{
    return 8u * (t / 4u) + 4u * khalf + (t % 4u);
}

// out (+)= acc for the TM x TN blocks of 32 x 32 one wavefront owns; rowBase / colBase are
// the wavefront's first row and column.  Four consecutive columns that all exist are accessed
// 16 bytes at a time, whatever the alignment of the row.
template <int TM, int TN>
__device__ __forceinline__ void StoreTile(const floatx16 (&acc)[TM][TN], float* __restrict__ out,
                                          uint32_t rowBase, uint32_t colBase, uint32_t M,
                                          uint32_t N, uint32_t l32, uint32_t khalf,
                                          const GemmF32Args& args)
{
    const bool accumulate = args.overwrite == 0;
    const float* __restrict__ bias = args.bias;
    const bool relu = args.relu != 0;
    // ---- out += acc ---------------------------------------------------------
    // With the operands swapped, register v of lane l holds row l%32 and column
    // 8*(v/4) + 4*(l/32) + v%4 of its 32x32 block: registers 4q..4q+3 are 4
    // consecutive columns.  The old values of the whole wavefront block are requested
    // in one batch, then added and stored.
    constexpr int kQuads = TM * TN * 4;
    float4 old[kQuads];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t r = rowBase + i * 32 + l32;
                const uint32_t c = colBase + j * 32 + 8 * q + 4 * khalf;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (bias != nullptr)
                {
                    // what the K = 1 product ones x bias leaves in a zero-filled out
                    if (c + 0 < N) v.x = 0.f + bias[c + 0];
                    if (c + 1 < N) v.y = 0.f + bias[c + 1];
                    if (c + 2 < N) v.z = 0.f + bias[c + 2];
                    if (c + 3 < N) v.w = 0.f + bias[c + 3];
                }
                else if (accumulate && r < M && c < N)
                {
                    const float* p = out + static_cast<size_t>(r) * args.ldc + c;
                    if (c + 4 <= N)
                    {
                        const floatx4 w = *reinterpret_cast<const floatx4a4*>(p);
                        v = make_float4(w[0], w[1], w[2], w[3]);
                    }
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
                const uint32_t r = rowBase + i * 32 + l32;
                const uint32_t c = colBase + j * 32 + 8 * q + 4 * khalf;
                if (r < M && c < N)
                {
                    float4 v = old[(i * TN + j) * 4 + q];
                    v.x = Combine(args, v.x, acc[i][j][4 * q + 0]);
                    v.y = Combine(args, v.y, acc[i][j][4 * q + 1]);
                    v.z = Combine(args, v.z, acc[i][j][4 * q + 2]);
                    v.w = Combine(args, v.w, acc[i][j][4 * q + 3]);
                    if (relu)
                    {
                        v.x = v.x > 0 ? v.x : 0;
                        v.y = v.y > 0 ? v.y : 0;
                        v.z = v.z > 0 ? v.z : 0;
                        v.w = v.w > 0 ? v.w : 0;
                    }
                    float* p = out + static_cast<size_t>(r) * args.ldc + c;
                    if (c + 4 <= N)
                        *reinterpret_cast<floatx4a4*>(p) = floatx4{ v.x, v.y, v.z, v.w };
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

    uint32_t tm, tn, unit;
    if (!MapTile(args, tm, tn, unit))
        return;

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
            FetchXContig<BM, A_QUADS, VEC>(stageA, A, tid, rowBase, M, k0, K, args.lda);
        else
            FetchKContig<BM, A_QUADS, VEC>(stageA, A, tid, rowBase, M, k0, K);
        if constexpr (TB)
            FetchKContig<BN, B_QUADS, VEC>(stageB, B, tid, colBase, N, k0, K);
        else
            FetchXContig<BN, B_QUADS, VEC>(stageB, B, tid, colBase, N, k0, K, args.ldb);
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

    // MFMA 32x32x2 operand layout: lane l supplies A[l % 32][k] and B[k][l % 32] where k is
    // one value for lanes 0-31 and another for lanes 32-63.  Which two k an instruction takes
    // is free as long as A and B agree: instruction t of a step takes k = 8*(t/4) + t%4 from
    // the lower half and that + 4 from the upper half, the assignment every fp32 kernel of
    // this file uses, so that they all add the K products in the same order.
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
                a[slot][i] = as[KOfPair(kk / 2, khalf) * LDA + i * 32];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b[slot][j] = bs[KOfPair(kk / 2, khalf) * LDB + j * 32];
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

    StoreTile<TM, TN>(acc, out, rowBase + waveM * WM, colBase + waveN * WN, M, N, l32, khalf, args);
}

// ---------------------------------------------------------------------------
// Pipelined variant.
//
// The tiled kernel above holds a K step in registers between its global load and its LDS
// store, so only one step can be in flight; with one workgroup per compute unit (mid-size
// products) every step then waits out a full memory latency.  Here the slabs travel from
// global memory straight into a ring of STAGES LDS stages (global_load_lds_dwordx4, no
// registers in between), STAGES - 2 steps ahead of the one being multiplied, with one barrier
// per step.
//
// LDS layout of one stage (K step BK = 16 or 32).  An operand stored with K contiguous keeps
// its rows: X rows of BK floats in 16-byte chunks, chunk c of row x at position
// c ^ ((x >> 2) & 3) for BK = 16 and c ^ ((x >> 1) & 7) for BK = 32, so that the 16-byte
// fragment reads of 16 consecutive rows touch every bank once.  BK = 32 makes a row segment a
// whole 128-byte cache line.  A lane then
// gets k = 4h..4h+3 of its row in one read (h = lane / 32), which is why the k assignment of
// this file gives lane half h the values 8q + 4h + e.  An operand stored k-major keeps its 16
// rows of X floats, with 128 bytes of padding after every 4 rows so that the two lane halves
// of a 4-byte fragment read (rows k and k + 4) fall into different banks.
// Rows / columns past the matrix edge are clamped to the last valid ones: they only feed
// output elements that are never stored.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* LdsVoidPtr;

__device__ __forceinline__ void DmaToLds16(uint32_t laneByteOffset, const void* uniformBase,
                                           uint32_t ldsByteAddr)
{
    // lane i reads 16 bytes at uniformBase + laneByteOffset; they land at ldsByteAddr + 16*i
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(ldsByteAddr), "v"(laneByteOffset), "s"(uniformBase)
                 : "memory");
}

template <int N>
__device__ __forceinline__ void WaitVmem()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <int X, int BK>
struct DmaTile
{
    // K-contiguous slab: X rows of BK floats.  k-major slab: BK rows of X floats.
    static constexpr uint32_t kCopies = X * BK / 256;     // 1 KiB copies per operand and step
    static constexpr uint32_t kChunks = BK / 4;           // 16-byte chunks of a K-contiguous row
    static constexpr uint32_t kRowsPerCopyK = 256 / BK;   // K-contiguous rows per copy
    static constexpr uint32_t kRowsPer256 = 64 / BK;      // K-contiguous rows per 256 bytes
    static constexpr uint32_t kRowBytes = X * 4;          // k-major row
    static constexpr uint32_t kRowsPerCopyX = 1024 / kRowBytes;
    static constexpr uint32_t kBytesKContig = X * BK * 4;
    // X = 32: a copy (1 KiB, written lane-linear) holds 8 whole rows, so no padding can be put
    // between rows 3 and 4; instead the copy fetches its rows in the order 0 4 1 5 2 6 3 7, which
    // puts rows k and k + 4 (read together by the two lane halves) 128 bytes apart
    static constexpr bool kPairedRows = X == 32;
    static constexpr uint32_t kBytesXContig = kPairedRows ? X * BK * 4 : X * BK * 4 + (BK / 4) * 128;

    // position of chunk c of K-contiguous row x
    static __device__ __forceinline__ uint32_t Swizzle(uint32_t x)
    {
        return (x / kRowsPer256) & (kChunks - 1);
    }
    // LDS offset of copy j of a k-major slab (128 bytes of padding after every 4 rows)
    static __device__ __forceinline__ constexpr uint32_t CopyOffsetXContig(uint32_t j)
    {
        return kPairedRows ? j * 1024u : j * 1024u + ((j * kRowsPerCopyX) / 4u) * 128u;
    }
    static __device__ __forceinline__ constexpr uint32_t RowOffsetXContig(uint32_t k)
    {
        return kPairedRows ? ((k & ~7u) + 2u * (k & 3u) + ((k >> 2) & 1u)) * kRowBytes
                           : k * kRowBytes + (k / 4u) * 128u;
    }
    // k-major slab: the row of the slab that lies at row position p of the unpadded copy stream
    static __device__ __forceinline__ constexpr uint32_t RowAtPosition(uint32_t p)
    {
        return kPairedRows ? (p & ~7u) + ((p & 7u) >> 1) + 4u * (p & 1u) : p;
    }
};

// WALK: a workgroup walks several tiles (every 64th of its XCD's run, 64 = two resident
// workgroups on each of an XCD's 32 compute units) instead of one.  The copy pipeline runs on
// across the tile boundary - the last steps of a tile already fetch the first slabs of the
// next one - and the old values of `out` are requested at a tile's first step and added after
// its last one, so the matrix pipe does not wait for the first slabs and for `out` once per
// tile.  The launcher takes this form only for whole tiles, 16-byte output rows and a K
// that fills the LDS ring a whole number of times, which keeps the number of loads and stores
// per tile fixed.  Per element the arithmetic is the same as without WALK.
//
// TAIL: K = BK q + r with 0 < r < BK.  The last of the q + 1 steps copies only the r values of
// k that exist - a lane whose 16-byte chunk (K-contiguous operand) or row (k-major operand)
// lies past K copies the slab's first chunk or row instead, one whose chunk reaches past K the
// 4 values that end at K - and the fragments are put right where they are used (zeros for
// k >= K, for A and B alike), so the step adds what a zero-padded slab would: the same sum,
// in the same order, as the register-staged kernel.
//
// KSPLIT = 2: two groups of wavefronts share the tile; of the four 8-wide k blocks of a
// 32-wide step group 0 multiplies the first two and group 1 the last two, each into a sum of
// its own, and after the last step group 1 hands its sum to group 0 through LDS, which adds
// it to its own (one fixed order: group 0's sum + group 1's) and stores.  A compute unit then
// holds two wavefronts per SIMD with independent accumulators - one's wait for a barrier or
// a fragment is covered by the other's matrix instructions - which is what a product with at
// most one 64 x 64 tile per compute unit lacks.  With KSPLIT = 2 a 64 x 32 tile (two
// wavefronts per group) gives products with fewer 64-tiles than compute units twice as many
// workgroups.  The K products of an element are then summed in another order than with
// KSPLIT = 1 (within the fp32 tolerance, not bit-identical to it).
template <int TILE, bool TA, bool TB, int WAVES>
__device__ __forceinline__ void GemmF32SkinnyBody(const GemmF32Args& args, uint32_t block);

template <int BM, int BN, int BK, int STAGES, bool TA, bool TB, bool WALK, bool TAIL = false,
          int KSPLIT = 1>
__global__ __launch_bounds__(((BN >= 64) ? 4 : 2) * KSPLIT * 64) void GemmF32DmaKernel(
    const GemmF32Args args, const GemmF32Strips strips)
{
    static_assert(BK == 16 || BK == 32, "K step of 16 or 32");
    static_assert(!(WALK && TAIL), "a walk needs whole rings of steps");
    static_assert(KSPLIT == 1 || (KSPLIT == 2 && BK == 32 && !WALK), "K split over two groups");
    static_assert(BN >= 64 || KSPLIT == 2, "the 32-wide tile has two wavefronts per group");
    constexpr int WAVES_M = 2;
    constexpr int WAVES_N = BN >= 64 ? 2 : 1;
    constexpr int GROUP_WAVES = WAVES_M * WAVES_N;      // wavefronts that cover the tile once
    constexpr int NW = GROUP_WAVES * KSPLIT;            // wavefronts of the workgroup
    constexpr int WM = BM / WAVES_M;
    constexpr int WN = BN / WAVES_N;
    constexpr int TM = WM / 32;
    constexpr int TN = WN / 32;
    using TileA = DmaTile<BM, BK>;
    using TileB = DmaTile<BN, BK>;
    constexpr uint32_t kBytesA = TA ? TileA::kBytesXContig : TileA::kBytesKContig;
    constexpr uint32_t kBytesB = TB ? TileB::kBytesKContig : TileB::kBytesXContig;
    constexpr uint32_t kStageBytes = kBytesA + kBytesB;
    static_assert(TileA::kCopies % NW == 0 && TileB::kCopies % NW == 0,
                  "every wavefront copies the same number of pieces");
    constexpr uint32_t kCopiesPerWave = (TileA::kCopies + TileB::kCopies) / NW;  // per step
    constexpr uint32_t kCopiesA = TileA::kCopies / NW;  // per wavefront
    constexpr uint32_t kCopiesB = TileB::kCopies / NW;
    constexpr uint32_t kBlocks = BK / 8 / KSPLIT;  // 8-wide k blocks (4 MFMAs each) per step
                                                   // and wavefront
    constexpr int kQuads = TM * TN * 4;   // float4 of `out` per lane

    __shared__ __attribute__((aligned(1024))) char lds[STAGES * kStageBytes];

    // strips of the product's edge come last in the grid (a walk has none)
    const uint32_t block = blockIdx.x;
    if constexpr (!WALK)
    {
        static_assert(NW == 4, "the strips' code runs on four wavefronts");
        if (block >= strips.first)
        {
            const uint32_t local = block - strips.first;
            if (local < strips.blocks[0])
                GemmF32SkinnyBody<16, TA, TB, 4>(strips.part[0], local);
            else
                GemmF32SkinnyBody<16, TA, TB, 4>(strips.part[1], local - strips.blocks[0]);
            return;
        }
    }

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t kgroup = wave / GROUP_WAVES;  // which k blocks of a step (0 without KSPLIT)
    const uint32_t waveM = (wave % GROUP_WAVES) / WAVES_N;
    const uint32_t waveN = (wave % GROUP_WAVES) % WAVES_N;
    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;

    // ---- the tile(s) of this workgroup ------------------------------------------------------
    uint32_t logical = (block & 7u) * args.perXcd + (block >> 3);
    uint32_t logicalEnd = args.tilesTotal;
    uint32_t logicalStride = 0;
    if constexpr (WALK)
    {
        logicalEnd = min((block & 7u) * args.perXcd + args.perXcd, args.tilesTotal);
        logicalStride = gridDim.x >> 3;
    }
    if (logical >= logicalEnd)
        return;
    const uint32_t M = args.M, N = args.N, K = args.K;

    // Where a tile's operands and output start, and what this lane copies of it every step:
    // copy j of an operand is taken by wavefront j % NW; lane offsets are bytes from the
    // operand's base at step 0, the base advances by one K step per step.
    struct Place
    {
        const char* a;
        const char* b;
        float* out;
        uint32_t rowBase, colBase;
        uint32_t aLane[kCopiesA], bLane[kCopiesB];
        // TAIL: the same for the last, partial slab
        uint32_t aTail[TAIL ? kCopiesA : 1], bTail[TAIL ? kCopiesB : 1];
    };
    const uint32_t steps = TAIL ? (K + BK - 1) / BK : K / BK;
    const uint32_t lastValid = TAIL ? K - (steps - 1) * BK : BK;  // values of k in the last slab
    const uint32_t wholeSteps = TAIL ? steps - 1 : steps;          // steps of the pipelined loop
    // `valid`: values of k the slab holds
    // TAIL: operand bases are moved kTailBias bytes down and lane offsets up, because the chunk
    // that ends at K may begin before the slab does
    constexpr uint32_t kTailBias = TAIL ? 16 : 0;
    auto laneOffsetKContig = [&](uint32_t j, uint32_t xBase, uint32_t limit, uint32_t valid) {
        using T = TileA;  // chunk geometry depends on BK only
        const uint32_t x = j * T::kRowsPerCopyK + lane / T::kChunks;  // row inside the tile
        const uint32_t c = (lane % T::kChunks) ^ T::Swizzle(x);
        // float offset of the chunk inside the slab's row, + 4: a chunk that reaches past
        // `valid` copies the last 4 values of the row (its LDS slot then holds k = valid - 4
        // .. valid - 1), one that begins past it the row's first chunk
        uint32_t k4 = c * 4 + 4;
        if (k4 > valid)
            k4 = k4 - 4 < valid ? valid : 4;
        const uint32_t gx = min(xBase + x, limit - 1);
        return (gx * K + k4) * 4u - 16u + kTailBias;
    };
    auto laneOffsetXContig = [&](uint32_t j, uint32_t xBase, uint32_t limit, uint32_t pitch,
                                 uint32_t rowBytes, uint32_t valid, auto rowAtPosition) {
        const uint32_t b = j * 1024 + lane * 16;  // byte inside the unpadded slab
        uint32_t k = rowAtPosition(b / rowBytes);
        if (k >= valid)
            k = 0;
        const uint32_t col = (b % rowBytes) / 4;
        const uint32_t gx = min(xBase + col, limit - 4);
        return (k * pitch + gx) * 4u + kTailBias;
    };
    auto locate = [&](uint32_t logicalTile, Place& p) {
        uint32_t tm, tn, unit;
        MapLogical(args, logicalTile, tm, tn, unit);
        if (args.entries != nullptr)
        {
            const SphGemmEntry e = args.entries[unit];
            p.a = reinterpret_cast<const char*>(args.A + e.aOff) - kTailBias;
            p.b = reinterpret_cast<const char*>(args.B + e.bOff) - kTailBias;
            p.out = args.out + e.outOff;
        }
        else
        {
            p.a = reinterpret_cast<const char*>(args.A + args.strideA * static_cast<int64_t>(unit)) -
                  kTailBias;
            p.b = reinterpret_cast<const char*>(args.B + args.strideB * static_cast<int64_t>(unit)) -
                  kTailBias;
            p.out = args.out + args.strideOut * static_cast<int64_t>(unit);
        }
        p.rowBase = tm * BM;
        p.colBase = tn * BN;
#pragma unroll
        for (uint32_t i = 0; i < kCopiesA; ++i)
        {
            const uint32_t j = wave + NW * i;
            p.aLane[i] = TA ? laneOffsetXContig(j, p.rowBase, M, args.lda, TileA::kRowBytes, BK, TileA::RowAtPosition)
                            : laneOffsetKContig(j, p.rowBase, M, BK);
            if constexpr (TAIL)
                p.aTail[i] = TA ? laneOffsetXContig(j, p.rowBase, M, args.lda, TileA::kRowBytes,
                                                    lastValid, TileA::RowAtPosition)
                                : laneOffsetKContig(j, p.rowBase, M, lastValid);
        }
#pragma unroll
        for (uint32_t i = 0; i < kCopiesB; ++i)
        {
            const uint32_t j = wave + NW * i;
            p.bLane[i] = TB ? laneOffsetKContig(j, p.colBase, N, BK)
                            : laneOffsetXContig(j, p.colBase, N, args.ldb, TileB::kRowBytes, BK, TileB::RowAtPosition);
            if constexpr (TAIL)
                p.bTail[i] = TB ? laneOffsetKContig(j, p.colBase, N, lastValid)
                                : laneOffsetXContig(j, p.colBase, N, args.ldb, TileB::kRowBytes,
                                                    lastValid, TileB::RowAtPosition);
        }
    };
    // LDS offsets of this wavefront's copies inside a stage
    uint32_t aDst[kCopiesA], bDst[kCopiesB];
#pragma unroll
    for (uint32_t i = 0; i < kCopiesA; ++i)
        aDst[i] = TA ? TileA::CopyOffsetXContig(wave + NW * i) : (wave + NW * i) * 1024;
#pragma unroll
    for (uint32_t i = 0; i < kCopiesB; ++i)
        bDst[i] = kBytesA +
                  (TB ? (wave + NW * i) * 1024 : TileB::CopyOffsetXContig(wave + NW * i));

    Place cur, nxt;
    locate(logical, cur);

    const size_t aStepBytes = TA ? static_cast<size_t>(BK) * args.lda * 4 : BK * 4;
    const size_t bStepBytes = TB ? BK * 4 : static_cast<size_t>(BK) * args.ldb * 4;
    const uint32_t ldsBase =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsVoidPtr)(lds)));

    // ---- the copy stream ------------------------------------------------------------------
    // Copy n (0 .. kCopiesPerWave-1) of this wavefront's share of the next slab to fetch goes
    // into stage `stage`; aSrc / bSrc point at that slab.  After a tile's last slab the stream
    // moves on to the next tile of the walk; when there is none it fetches the last slab again
    // into a stage nobody reads any more, which keeps the number of outstanding copies the same
    // in every step.
    const char* aSrc = cur.a;
    const char* bSrc = cur.b;
    uint32_t aLane[kCopiesA], bLane[kCopiesB];
#pragma unroll
    for (uint32_t i = 0; i < kCopiesA; ++i)
        aLane[i] = cur.aLane[i];
#pragma unroll
    for (uint32_t i = 0; i < kCopiesB; ++i)
        bLane[i] = cur.bLane[i];
    uint32_t aLaneLast[TAIL ? kCopiesA : 1], bLaneLast[TAIL ? kCopiesB : 1];
    if constexpr (TAIL)
    {
#pragma unroll
        for (uint32_t i = 0; i < kCopiesA; ++i)
            aLaneLast[i] = cur.aTail[i];
#pragma unroll
        for (uint32_t i = 0; i < kCopiesB; ++i)
            bLaneLast[i] = cur.bTail[i];
    }
    uint32_t slabsLeft = steps;  // of the tile being fetched, the one at aSrc / bSrc included
    bool haveNext = false;       // `nxt` describes a tile the copy stream has not reached yet
    auto issueOne = [&](uint32_t stage, uint32_t n) {
        const uint32_t base = ldsBase + stage * kStageBytes;
        // TAIL: the slab at aSrc / bSrc is the tile's last one when slabsLeft is 1
        const bool partial = TAIL && slabsLeft == 1;
        if (n < kCopiesA)
            DmaToLds16(partial ? aLaneLast[TAIL ? n : 0] : aLane[n], aSrc, base + aDst[n]);
        else
            DmaToLds16(partial ? bLaneLast[TAIL ? n - kCopiesA : 0] : bLane[n - kCopiesA], bSrc,
                       base + bDst[n - kCopiesA]);
    };
    auto advance = [&]() {
        if (--slabsLeft != 0)
        {
            aSrc += aStepBytes;
            bSrc += bStepBytes;
        }
        else if (WALK && haveNext)
        {
            aSrc = nxt.a;
            bSrc = nxt.b;
#pragma unroll
            for (uint32_t i = 0; i < kCopiesA; ++i)
                aLane[i] = nxt.aLane[i];
#pragma unroll
            for (uint32_t i = 0; i < kCopiesB; ++i)
                bLane[i] = nxt.bLane[i];
            slabsLeft = steps;
            haveNext = false;
        }
        else
            slabsLeft = 1;
    };

    floatx16 acc[TM][TN];

    // ---- fragment addresses inside a stage -------------------------------------------------
    // K-contiguous operand: byte offset of this lane's row, chunk chosen per 8-wide k block.
    // k-major operand: byte offset of this lane's column; the row offset is added per k.
    uint32_t aFrag[TM], bFrag[TN];
    uint32_t aSwz[TM], bSwz[TN];
    // Group g of a K split takes k blocks kBlocks*g .. of every step: for a K-contiguous
    // operand that is chunk 2*kBlocks*g + ..., folded into the swizzle (the bits do not overlap);
    // for a k-major operand rows 8*kBlocks*g + ..., a constant added to the lane's offset.
    const uint32_t groupChunk = kgroup * (2 * kBlocks);
    const uint32_t groupRowsA = TileA::RowOffsetXContig(8 * kBlocks) * kgroup;
    const uint32_t groupRowsB = TileB::RowOffsetXContig(8 * kBlocks) * kgroup;
    static_assert(KSPLIT == 1 || (8 * kBlocks) % 4 == 0, "whole padding groups per k group");
#pragma unroll
    for (int i = 0; i < TM; ++i)
    {
        const uint32_t x = waveM * WM + i * 32 + l32;
        aFrag[i] = TA ? x * 4 + groupRowsA : x * BK * 4;
        aSwz[i] = TileA::Swizzle(x) ^ groupChunk;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j)
    {
        const uint32_t x = waveN * WN + j * 32 + l32;
        bFrag[j] = kBytesA + (TB ? x * BK * 4 : x * 4 + groupRowsB);
        bSwz[j] = TileB::Swizzle(x) ^ groupChunk;
    }

    // fragments of k block q (k = 8q + 4*khalf + e, e = 0..3)
    auto loadFragments = [&](float (&a)[TM][4], float (&b)[TN][4], const char* stage,
                             uint32_t q) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
        {
            if constexpr (TA)
            {
#pragma unroll
                for (uint32_t e = 0; e < 4; ++e)
                    a[i][e] = *reinterpret_cast<const float*>(
                        stage + aFrag[i] + TileA::RowOffsetXContig(8 * q + e) +
                        khalf * (TileA::RowOffsetXContig(4) - TileA::RowOffsetXContig(0)));
            }
            else
            {
                const float4 v = *reinterpret_cast<const float4*>(
                    stage + aFrag[i] + (((2 * q + khalf) ^ aSwz[i]) << 4));
                a[i][0] = v.x;
                a[i][1] = v.y;
                a[i][2] = v.z;
                a[i][3] = v.w;
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j)
        {
            if constexpr (TB)
            {
                const float4 v = *reinterpret_cast<const float4*>(
                    stage + bFrag[j] + (((2 * q + khalf) ^ bSwz[j]) << 4));
                b[j][0] = v.x;
                b[j][1] = v.y;
                b[j][2] = v.z;
                b[j][3] = v.w;
            }
            else
            {
#pragma unroll
                for (uint32_t e = 0; e < 4; ++e)
                    b[j][e] = *reinterpret_cast<const float*>(
                        stage + bFrag[j] + TileB::RowOffsetXContig(8 * q + e) +
                        khalf * (TileB::RowOffsetXContig(4) - TileB::RowOffsetXContig(0)));
            }
        }
    };
    // TAIL: what the fragments of block q would be if the last slab were zero-padded to a whole
    // step; `valid` values of k exist.  Put in where the fragments are used so that the reads
    // above stay in flight behind the MFMAs of the block before.
    //   k-major operand: zeros for k >= valid.
    //   K-contiguous operand: chunks that begin at or past `valid` become zeros; the chunk
    //   that reaches past it was copied from valid - 4 on, so its values are moved down by
    //   4 - valid % 4 places and followed by zeros.
    auto dropMissing = [&](float (&a)[TM][4], float (&b)[TN][4], uint32_t q, uint32_t valid) {
        if constexpr (TAIL)
        {
            // k of this lane's fragment element 0 (q counts this group's blocks)
            const uint32_t k0 = 8 * (q + kgroup * kBlocks) + 4 * khalf;
            const uint32_t shift = (4 - valid % 4) % 4;
            const bool whole = k0 + 4 <= valid;
            const bool reaches = !whole && k0 < valid;
            auto fixKContig = [&](float (&f)[4]) {
                float g[4];
#pragma unroll
                for (uint32_t e = 0; e < 4; ++e)
                {
                    // element e + shift of the copied chunk, a zero when that is past its end
                    float moved = 0.f;
                    moved = (shift == 1 && e + 1 < 4) ? f[(e + 1) & 3] : moved;
                    moved = (shift == 2 && e + 2 < 4) ? f[(e + 2) & 3] : moved;
                    moved = (shift == 3 && e + 3 < 4) ? f[(e + 3) & 3] : moved;
                    g[e] = whole ? f[e] : (reaches ? moved : 0.f);
                }
#pragma unroll
                for (uint32_t e = 0; e < 4; ++e)
                    f[e] = g[e];
            };
            auto fixKMajor = [&](float (&f)[4]) {
#pragma unroll
                for (uint32_t e = 0; e < 4; ++e)
                    f[e] = k0 + e < valid ? f[e] : 0.f;
            };
#pragma unroll
            for (int i = 0; i < TM; ++i)
            {
                if constexpr (TA)
                    fixKMajor(a[i]);
                else
                    fixKContig(a[i]);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j)
            {
                if constexpr (TB)
                    fixKContig(b[j]);
                else
                    fixKMajor(b[j]);
            }
            // all of them ahead of the block's MFMAs, which then issue back to back
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto multiply = [&](const float (&a)[TM][4], const float (&b)[TN][4]) {
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] =
                        __builtin_amdgcn_mfma_f32_32x32x2f32(b[j][e], a[i][e], acc[i][j], 0, 0, 0);
    };

    // ---- WALK: the values the tile's products are added to ----------------------------------
    // Register v of lane l holds row l%32 and column 8*(v/4) + 4*(l/32) + v%4 of its 32x32
    // block, so registers 4q..4q+3 are one float4 of `out`.
    floatx4 old[WALK ? kQuads : 1];
    // One straight run of loads per mode, so that none of them is waited for here.
    auto fetchOld = [&]() {
        auto where = [&](int idx, uint32_t& r, uint32_t& c) {
            const int q = idx & 3, j = (idx >> 2) % TN, i = (idx >> 2) / TN;
            r = cur.rowBase + waveM * WM + i * 32 + l32;
            c = cur.colBase + waveN * WN + j * 32 + 8 * q + 4 * khalf;
        };
        if (args.bias != nullptr)
        {
#pragma unroll
            for (int idx = 0; idx < kQuads; ++idx)
            {
                uint32_t r, c;
                where(idx, r, c);
                old[idx] = *reinterpret_cast<const floatx4*>(args.bias + c);
            }
        }
        else if (args.overwrite == 0)
        {
#pragma unroll
            for (int idx = 0; idx < kQuads; ++idx)
            {
                uint32_t r, c;
                where(idx, r, c);
                old[idx] = *reinterpret_cast<const floatx4a4*>(
                    cur.out + static_cast<size_t>(r) * args.ldc + c);
            }
        }
        else
        {
#pragma unroll
            for (int idx = 0; idx < kQuads; ++idx)
                old[idx] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
    };
    // Makes the compiler wait for the values here, where only the copies of one step are in
    // flight, rather than at their first use after the last step with three steps in flight.
    auto settleOld = [&]() {
#pragma unroll
        for (int i = 0; i < (WALK ? kQuads : 1); ++i)
            asm volatile("" : "+v"(old[i]));
    };
    auto addAndStore = [&]() {
        const bool relu = args.relu != 0;
        const bool hasBias = args.bias != nullptr;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                {
                    const uint32_t r = cur.rowBase + waveM * WM + i * 32 + l32;
                    const uint32_t c = cur.colBase + waveN * WN + j * 32 + 8 * q + 4 * khalf;
                    floatx4 v = old[(i * TN + j) * 4 + q];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        // 0 + bias: what the K = 1 product ones x bias leaves in a zero-filled out
                        if (hasBias)
                            v[e] = 0.f + v[e];
                        v[e] = Combine(args, v[e], acc[i][j][4 * q + e]);
                        if (relu)
                            v[e] = v[e] > 0 ? v[e] : 0;
                    }
                    *reinterpret_cast<floatx4a4*>(cur.out + static_cast<size_t>(r) * args.ldc + c) = v;
                }
    };

    // First k block of step s.  The step's housekeeping sits between its MFMAs, where the
    // matrix pipe is already busy: behind the first one the wait for step s+1's copies and the
    // barrier, behind each of the next ones one copy of step s+STAGES-1.
    static_assert(kCopiesPerWave <= 4 * TM * TN, "one copy per MFMA of the first block");
    auto multiplyAndFeed = [&](const float (&a)[TM][4], const float (&b)[TN][4],
                               uint32_t fillStage, bool tileStart, bool settle) {
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                {
                    const uint32_t n = (e * TM + i) * TN + j;
                    acc[i][j] =
                        __builtin_amdgcn_mfma_f32_32x32x2f32(b[j][e], a[i][e], acc[i][j], 0, 0, 0);
                    if (n == 0)
                    {
                        // steps up to s+1 have landed once at most the STAGES-3 later ones
                        // are pending (loads and stores complete in the order they were issued,
                        // so the stores and `out` loads of a tile boundary only make this wait
                        // stricter); behind the barrier everybody's copies are visible and
                        // everybody has read the last fragment of step s-1
                        WaitVmem<(STAGES - 3) * kCopiesPerWave>();
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                        if constexpr (WALK)
                        {
                            // both flags are constants once the ring loop is unrolled
                            if (tileStart)
                                fetchOld();
                            if (settle)
                                settleOld();
                        }
                    }
                    if (n < kCopiesPerWave)
                    {
                        issueOne(fillStage, n);
                        if (n + 1 == kCopiesPerWave)
                            advance();
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
    };

#pragma unroll
    for (uint32_t p = 0; p < STAGES - 1; ++p)
    {
#pragma unroll
        for (uint32_t n = 0; n < kCopiesPerWave; ++n)
            issueOne(p, n);
        advance();
    }

    // Fragments are read one k block (8 values) ahead of the MFMAs that use them; the first
    // block of step s+1 is read while the last block of step s is multiplied (at a tile's last
    // step that is the first block of the next tile).  Stage s+1 is known to be complete from
    // the barrier inside the first block of step s.
    float fa[2][TM][4], fb[2][TN][4];
    WaitVmem<(STAGES - 2) * kCopiesPerWave>();
    __syncthreads();
    loadFragments(fa[0], fb[0], lds, 0);

    for (;;)
    {
        if constexpr (WALK)
        {
            // describe the tile after this one before the copy stream gets there
            const uint32_t after = logical + logicalStride;
            if (after < logicalEnd)
            {
                locate(after, nxt);
                haveNext = true;
            }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    acc[i][j][v] = 0.f;

        // The loop is unrolled over the ring so that every stage offset is a constant.  With
        // WALK the step count is a positive multiple of STAGES and the first trip round the
        // ring, which fetches and settles `old`, is written out on its own: the compiler then
        // sees that no path leads round the place where `old` settles and waits for nothing
        // when `old` is used after the last step.
        auto ringCycle = [&](uint32_t s0, auto firstOfTile) {
            constexpr bool kFirst = decltype(firstOfTile)::value;
#pragma unroll
            for (uint32_t u = 0; u < STAGES; ++u)
            {
                if (!WALK && s0 + u >= wholeSteps)
                    break;
                const char* stage = lds + u * kStageBytes;
                const char* next = lds + ((u + 1) % STAGES) * kStageBytes;
#pragma unroll
                for (uint32_t q = 0; q < kBlocks; ++q)
                {
                    if (q + 1 < kBlocks)
                        loadFragments(fa[(q + 1) & 1], fb[(q + 1) & 1], stage, q + 1);
                    else
                        loadFragments(fa[(q + 1) & 1], fb[(q + 1) & 1], next, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (q == 0)
                        multiplyAndFeed(fa[0], fb[0], (u + STAGES - 1) % STAGES,
                                        kFirst && u == 0, kFirst && u == 1);
                    else
                        multiply(fa[q & 1], fb[q & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if constexpr (WALK)
        {
            ringCycle(0, std::true_type{});
            for (uint32_t s0 = STAGES; s0 < steps; s0 += STAGES)
                ringCycle(s0, std::false_type{});
        }
        else
        {
            for (uint32_t s0 = 0; s0 < wholeSteps; s0 += STAGES)
                ringCycle(s0, std::false_type{});
        }
        if constexpr (TAIL)
        {
            // The partial step on its own, so that the steps before it carry no selects.  Its
            // slab has landed (the step before waited for it, or the prologue did) and its
            // first fragments are in fa[0] / fb[0]; no copy that is still in flight targets its
            // stage.
            const char* stage = lds + ((steps - 1) % STAGES) * kStageBytes;
#pragma unroll
            for (uint32_t q = 0; q < kBlocks; ++q)
            {
                if (q + 1 < kBlocks)
                    loadFragments(fa[(q + 1) & 1], fb[(q + 1) & 1], stage, q + 1);
                __builtin_amdgcn_sched_barrier(0);
                dropMissing(fa[q & 1], fb[q & 1], q, lastValid);
                multiply(fa[q & 1], fb[q & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        if constexpr (!WALK)
            break;
        else
        {
            addAndStore();
            logical += logicalStride;
            if (logical >= logicalEnd)
                break;
            cur.out = nxt.out;
            cur.rowBase = nxt.rowBase;
            cur.colBase = nxt.colBase;
        }
    }
    WaitVmem<0>();  // the surplus copies of the last steps still target LDS

    if constexpr (KSPLIT == 2)
    {
        // group 1 hands its sums over: float4 v of block (i, j) of wavefront w of a group lies at
        // ((i*TN + j)*4 + v) * GROUP_WAVES*64 + w*64 + lane, so a wavefront access is contiguous
        static_assert(TM * TN * 16 * GROUP_WAVES * 64 * 4 <= STAGES * kStageBytes, "fits the ring");
        __syncthreads();  // every wavefront has read its last fragments
        floatx4* hand = reinterpret_cast<floatx4*>(lds) + (wave % GROUP_WAVES) * 64 + lane;
        if (kgroup == 1)
        {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        hand[((i * TN + j) * 4 + v) * (GROUP_WAVES * 64)] =
                            floatx4{ acc[i][j][4 * v], acc[i][j][4 * v + 1], acc[i][j][4 * v + 2],
                                     acc[i][j][4 * v + 3] };
        }
        __syncthreads();
        if (kgroup == 1)
            return;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                {
                    const floatx4 other = hand[((i * TN + j) * 4 + v) * (GROUP_WAVES * 64)];
                    acc[i][j][4 * v] += other[0];
                    acc[i][j][4 * v + 1] += other[1];
                    acc[i][j][4 * v + 2] += other[2];
                    acc[i][j][4 * v + 3] += other[3];
                }
    }

    if constexpr (!WALK)
        StoreTile<TM, TN>(acc, cur.out, cur.rowBase + waveM * WM, cur.colBase + waveN * WN, M, N,
                          l32, khalf, args);
}

// ---------------------------------------------------------------------------
// Few-tile shapes (small M x N, long K): a TILE x TILE output tile per workgroup (32, or 16
// when at most four of those per compute unit cover the output), K split across its WAVES
// wavefronts (4, or 16 for 16-wide tiles that fit the chip once and K >= 512).
//
// With few output tiles the tiled kernel above leaves most compute units idle and is bound by
// the latency of one load -> LDS -> MFMA chain per K step.  Here every wavefront reads its
// operands straight from global memory in MFMA layout (A: 16 bytes per lane along K, lines
// reused from L1 over the next steps; B: one row segment per group of TILE lanes), keeps
// several loads in flight, and accumulates a private TILE x TILE partial over its share of K.
// The partials are then added in wavefront order through LDS, so the result does not depend on
// timing.  One MFMA (32x32x2 or 16x16x4) takes its 64 / TILE values of k from the 64 / TILE
// groups of TILE lanes; which k each group holds is free as long as A and B agree, and is
// chosen so that A is read with float4: group h holds k = (256 / TILE) * g + 4 * h + e.
// A workgroup's matrix pipes are the bound once K is long (one tile's K runs on one compute
// unit), which is why the 16-wide tile, a quarter of the work per workgroup on four times as
// many compute units, is preferred whenever its tiles still fit the chip.
// ---------------------------------------------------------------------------
template <int TILE, bool TA, bool TB, int WAVES>
__device__ __forceinline__ void GemmF32SkinnyBody(const GemmF32Args& args, uint32_t block)
{
    static_assert(TILE == 32 || TILE == 16, "MFMA shapes 32x32x2 and 16x16x4");
    constexpr uint32_t kLaneGroups = 64 / TILE;       // values of k per MFMA
    constexpr uint32_t kGroupK = 4 * kLaneGroups;     // k per float4 round: 8 or 16
    constexpr int kAcc = TILE * TILE / 64;            // accumulator registers: 16 or 4
    constexpr int kQuads = kAcc / 4;
    using Acc = typename std::conditional<TILE == 32, floatx16, floatx4>::type;

    __shared__ float partial[WAVES - 1][TILE * TILE];

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lt = lane % TILE;   // row of A / column of B this lane feeds
    const uint32_t kh = lane / TILE;   // which k of an MFMA

    uint32_t id = block;
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
    const uint32_t row = tm * TILE + lt;
    const uint32_t col = tn * TILE + lt;

    // this wavefront's K range, in groups of kGroupK (one float4 of A per lane); groups in
    // flight: 8, or twice the wavefronts per tile, are slower: the loop is bound by what the
    // caches deliver, not by the latency of a load
    constexpr int kDepth = 4;
    const sph::KPartition part = sph::PartitionK(K, kGroupK, WAVES, wave, kDepth);

    const bool rowOk = row < M;

    Acc acc;
#pragma unroll
    for (int v = 0; v < kAcc; ++v)
        acc[v] = 0.f;

    // Lane group h holds k = kGroupK*g + 4*h + e for e = 0..3.  An operand stored with K
    // contiguous (A as given, B passed transposed) is read as one 16-byte segment of its row
    // (from any 4-byte-aligned address); one stored k-major (B as given, A passed transposed) as
    // 4 elements `ld` apart.  Rows and columns past the edge read the last valid one: what they
    // produce is never stored.
    const float* aPtr = TA ? A + min(row, M - 1) : A + static_cast<size_t>(min(row, M - 1)) * K;
    const float* bPtr = TB ? B + static_cast<size_t>(min(col, N - 1)) * K : B + min(col, N - 1);
    // whole groups (every k below K): no conditions anywhere, so the loads of several groups
    // stay in flight behind the matrix instructions (a load inside a branch makes the compiler
    // wait for all of them)
    auto loadAlongK = [&](const float* rowPtr, uint32_t g) {
        const floatx4a4 w =
            *reinterpret_cast<const floatx4a4*>(rowPtr + (g * kGroupK + kh * 4));
        return make_float4(w[0], w[1], w[2], w[3]);
    };
    auto loadAcrossK = [&](const float* colPtr, size_t ld, uint32_t g) {
        const float* p = colPtr + static_cast<size_t>(g * kGroupK + kh * 4) * ld;
        return make_float4(p[0], p[ld], p[2 * ld], p[3 * ld]);
    };
    auto loadA = [&](uint32_t g) {
        if constexpr (TA)
            return loadAcrossK(aPtr, args.lda, g);
        else
            return loadAlongK(aPtr, g);
    };
    auto loadB = [&](uint32_t g) {
        if constexpr (TB)
            return loadAlongK(bPtr, g);
        else
            return loadAcrossK(bPtr, args.ldb, g);
    };
    // the last group when K is no multiple of kGroupK: element by element, zeros past K
    auto loadPartial = [&](const float* base, size_t step, uint32_t g) {
        const uint32_t k = g * kGroupK + kh * 4;
        const float* p = base + static_cast<size_t>(k) * step;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k + 0 < K) v.x = p[0];
        if (k + 1 < K) v.y = p[step];
        if (k + 2 < K) v.z = p[2 * step];
        if (k + 3 < K) v.w = p[3 * step];
        return v;
    };
    // operands swapped: the result block comes out indexed [column][row], which leaves 4
    // consecutive columns of one row in a lane
    auto multiply = [&](float b, float a) {
        if constexpr (TILE == 32)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, acc, 0, 0, 0);
        else
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b, a, acc, 0, 0, 0);
    };
    auto multiplyGroup = [&](const float4& a, const float4& b) {
        multiply(b.x, a.x);
        multiply(b.y, a.y);
        multiply(b.z, a.z);
        multiply(b.w, a.w);
    };

    const uint32_t whole = part.whole;
    if (part.gBegin < part.wholeEnd)
    {
        const uint32_t wholeEnd = part.wholeEnd, roundsEnd = part.roundsEnd;
        float4 fa[kDepth], fb[kDepth];
#pragma unroll
        for (int d = 0; d < kDepth; ++d)
        {
            // past the last whole group: that group once more, loaded and not used
            fa[d] = loadA(sph::KPartitionFirst(part, d));
            fb[d] = loadB(sph::KPartitionFirst(part, d));
        }
        for (uint32_t g = part.gBegin; g < roundsEnd; g += kDepth)
        {
#pragma unroll
            for (int d = 0; d < kDepth; ++d)
            {
                // multiply, then load the group kDepth further on into the same registers
                // (loading first needs a second set and a copy, behind a wait for every load,
                // at the end of each round); the fences keep that order
                multiplyGroup(fa[d], fb[d]);
                __builtin_amdgcn_sched_barrier(0);
                const uint32_t next = sph::KPartitionNext(part, g, kDepth, d);
                fa[d] = loadA(next);
                fb[d] = loadB(next);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // fewer than kDepth whole groups left: already in registers
#pragma unroll
        for (int d = 0; d < kDepth - 1; ++d)
            if (roundsEnd + d < wholeEnd)
                multiplyGroup(fa[d], fb[d]);
    }
    if (part.ownsPartial)
    {
        // at most one group, and only in the wavefront that holds the end of K
        const float4 a = TA ? loadPartial(aPtr, args.lda, whole) : loadPartial(aPtr, 1, whole);
        const float4 b = TB ? loadPartial(bPtr, 1, whole) : loadPartial(bPtr, args.ldb, whole);
        multiplyGroup(a, b);
    }

    // lane l holds row l % TILE, columns 4*kLaneGroups*q + 4*(l / TILE) + 0..3 of the tile;
    // partial sums of the other wavefronts go through LDS, wavefront 0 adds them in order
    if (wave != 0)
    {
#pragma unroll
        for (int q = 0; q < kQuads; ++q)
            *reinterpret_cast<float4*>(
                &partial[wave - 1][lt * TILE + 4 * kLaneGroups * q + 4 * kh]) =
                make_float4(acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
    }
    __syncthreads();
    if (wave != 0)
        return;
#pragma unroll
    for (int w = 0; w < WAVES - 1; ++w)
#pragma unroll
        for (int q = 0; q < kQuads; ++q)
        {
            const float4 p = *reinterpret_cast<const float4*>(
                &partial[w][lt * TILE + 4 * kLaneGroups * q + 4 * kh]);
            acc[4 * q + 0] += p.x;
            acc[4 * q + 1] += p.y;
            acc[4 * q + 2] += p.z;
            acc[4 * q + 3] += p.w;
        }
    if (!rowOk)
        return;
    const bool wide = args.outVec != 0;
#pragma unroll
    for (int q = 0; q < kQuads; ++q)
    {
        const uint32_t c = tn * TILE + 4 * kLaneGroups * q + 4 * kh;
        if (c >= N)
            continue;
        float* p = out + static_cast<size_t>(row) * args.ldc + c;
        if (args.bias != nullptr || args.relu || args.sgd)
        {
            // fused epilogues: (0 + bias) + product with an optional ReLU (out not read), or the
            // optimizer step
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (c + e < N)
                {
                    float old = 0.f;
                    if (args.bias != nullptr)
                        old = 0.f + args.bias[c + e];
                    else if (!args.overwrite)
                        old = p[e];
                    float v = Combine(args, old, acc[4 * q + e]);
                    if (args.relu)
                        v = v > 0 ? v : 0;
                    p[e] = v;
                }
        }
        else if (args.overwrite)
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

template <int TILE, bool TA, bool TB, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void GemmF32SkinnyKernel(const GemmF32Args args)
{
    GemmF32SkinnyBody<TILE, TA, TB, WAVES>(args, blockIdx.x);
}

// ---------------------------------------------------------------------------
// One output row (M = 1):  out[1 x N] (+)= a[1 x K] * B[K x N], e.g. the column sums
// ones x dy of the bias gradient.  A matrix-core tile would use one of its 32 rows; this is a
// plain reduction bound by reading B once.  A workgroup owns 64 consecutive columns (one per
// lane, 256-byte row segments) and splits K over its 16 wavefronts; the 16 partial sums are
// added in wavefront order through LDS, so the result does not depend on timing.
// ---------------------------------------------------------------------------
constexpr int kGemvWaves = 16;

__global__ __launch_bounds__(kGemvWaves * 64) void GemvRowKernel(const GemmF32Args args)
{
    __shared__ float partial[kGemvWaves][64];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t unit = blockIdx.y;
    const float* __restrict__ a = args.A + args.strideA * static_cast<int64_t>(unit);
    const float* __restrict__ B = args.B + args.strideB * static_cast<int64_t>(unit);
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit);
    const uint32_t N = args.N, K = args.K;
    const uint32_t col = blockIdx.x * 64 + lane;
    const bool colOk = col < N;

    const uint32_t perWave = (K + kGemvWaves - 1) / kGemvWaves;
    const uint32_t kBegin = min(wave * perWave, K);
    const uint32_t kEnd = min(kBegin + perWave, K);
    // four independent chains keep loads in flight; they are combined in a fixed order
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (colOk)
    {
        const float* p = B + static_cast<size_t>(kBegin) * N + col;
        uint32_t k = kBegin;
#pragma unroll 4
        for (; k + 4 <= kEnd; k += 4)
        {
            s0 = fmaf(a[k + 0], p[0], s0);
            s1 = fmaf(a[k + 1], p[static_cast<size_t>(N)], s1);
            s2 = fmaf(a[k + 2], p[2 * static_cast<size_t>(N)], s2);
            s3 = fmaf(a[k + 3], p[3 * static_cast<size_t>(N)], s3);
            p += 4 * static_cast<size_t>(N);
        }
        for (; k < kEnd; ++k)
        {
            s0 = fmaf(a[k], p[0], s0);
            p += N;
        }
    }
    partial[wave][lane] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (wave != 0 || !colOk)
        return;
    float sum = partial[0][lane];
#pragma unroll
    for (int w = 1; w < kGemvWaves; ++w)
        sum += partial[w][lane];
    float old = 0.f;
    if (args.bias != nullptr)
        old = 0.f + args.bias[col];
    else if (!args.overwrite)
        old = out[col];
    float v = Combine(args, old, sum);
    if (args.relu)
        v = v > 0 ? v : 0;
    out[col] = v;
}

// Offset tables of grouped launches: a device buffer the kernels read plus a pinned staging
// copy, per host thread and device, like the thread's stream -- two threads never wait for
// each other.  A thread's launches are ordered by its stream, so the only waits are for the
// thread's own earlier upload (before the staging copy is overwritten) and, when the thread
// has moved to another stream since (sph_set_stream), an event wait of the new stream for the
// old one.  Tables of threads that have ended are kept for the next thread.
struct EntryTable
{
    SphGemmEntry* dev = nullptr;
    SphGemmEntry* staging = nullptr;  // pinned
    size_t capacity = 0;
    hipEvent_t uploaded = nullptr;    // staging may be overwritten after this
    hipEvent_t consumed = nullptr;    // the last launch that read dev has finished after this
    bool uploadPending = false;
    hipStream_t lastStream = nullptr;
};
std::mutex gIdleTableMutex;
std::vector<EntryTable> gIdleTables[16];

struct ThreadTables
{
    EntryTable table[16];
    bool have[16] = {};
    ~ThreadTables()
    {
        std::lock_guard<std::mutex> lock(gIdleTableMutex);
        for (int d = 0; d < 16; ++d)
            if (have[d])
                gIdleTables[d].push_back(table[d]);
    }
};
thread_local ThreadTables tlsTables;

EntryTable& ThreadTable(int device)
{
    if (!tlsTables.have[device])
    {
        std::lock_guard<std::mutex> lock(gIdleTableMutex);
        if (!gIdleTables[device].empty())
        {
            tlsTables.table[device] = gIdleTables[device].back();
            gIdleTables[device].pop_back();
        }
        tlsTables.have[device] = true;
    }
    return tlsTables.table[device];
}

template <int TILE, bool TA, bool TB>
void LaunchSkinnyTile(const GemmF32Args& args, dim3 grid, bool wide, hipStream_t stream)
{
    // `wide` (16 x 16 tiles only): 16 wavefronts per tile instead of 4 when K is long enough to
    // give each wavefront a few steps
    if constexpr (TILE == 16)
    {
        if (wide)
        {
            hipLaunchKernelGGL((GemmF32SkinnyKernel<16, TA, TB, 16>), grid, dim3(1024), 0, stream,
                               args);
            return;
        }
    }
    hipLaunchKernelGGL((GemmF32SkinnyKernel<TILE, TA, TB, 4>), grid, dim3(256), 0, stream, args);
}

template <bool TA, bool TB>
void LaunchSkinny(const GemmF32Args& args, dim3 grid, uint32_t tile, bool wide, hipStream_t stream)
{
    if (tile == 16)
        LaunchSkinnyTile<16, TA, TB>(args, grid, wide, stream);
    else
        LaunchSkinnyTile<32, TA, TB>(args, grid, wide, stream);
}

// `walk`: 64-tiles only, each workgroup takes several tiles
// `ksplit`: 0, or 2 = K split over two groups of wavefronts on 64 x 32 tiles
// `strips`: edge strips that ride along; only the straight-to-LDS kernels that are no walk take
// any
template <bool TA, bool TB>
void LaunchTiled(const GemmF32Args& args, const GemmF32Strips& strips, dim3 grid, bool big,
                 bool vec, bool dma, bool walk, int ksplit, hipStream_t stream)
{
    const dim3 block(kThreads);
    if (dma && ksplit != 0)
    {
        if (args.K % 32 == 0)
            hipLaunchKernelGGL((GemmF32DmaKernel<64, 32, 32, 4, TA, TB, false, false, 2>), grid,
                               dim3(256), 0, stream, args, strips);
        else
            hipLaunchKernelGGL((GemmF32DmaKernel<64, 32, 32, 4, TA, TB, false, true, 2>), grid,
                               dim3(256), 0, stream, args, strips);
        return;
    }
    if (dma)
    {
        if (big && args.K % 16 != 0)
            hipLaunchKernelGGL((GemmF32DmaKernel<128, 128, 16, 4, TA, TB, false, true>), grid,
                               block, 0, stream, args, strips);
        else if (big)
            hipLaunchKernelGGL((GemmF32DmaKernel<128, 128, 16, 4, TA, TB, false>), grid, block, 0,
                               stream, args, strips);
        else if (walk)
            hipLaunchKernelGGL((GemmF32DmaKernel<64, 64, 32, 4, TA, TB, true>), grid, block, 0,
                               stream, args, strips);
        else if (args.K % 32 == 0)
            hipLaunchKernelGGL((GemmF32DmaKernel<64, 64, 32, 4, TA, TB, false>), grid, block, 0,
                               stream, args, strips);
        else if (args.K % 16 == 0)
            hipLaunchKernelGGL((GemmF32DmaKernel<64, 64, 16, 6, TA, TB, false>), grid, block, 0,
                               stream, args, strips);
        else
            hipLaunchKernelGGL((GemmF32DmaKernel<64, 64, 32, 4, TA, TB, false, true>), grid,
                               block, 0, stream, args, strips);
        return;
    }
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

// Tile edge: the matrix pipes bound the tiled kernels, so a launch lasts as long as the compute
// unit with the most tiles needs.  A 128-tile costs four 64-tiles and moves half the operand
// bytes per flop (measured 7 % faster at equal load), but a compute unit with a single 128-tile
// has nothing to run beside that tile's first loads and epilogue, which four 64-tiles overlap
// (measured 6 % slower then).  Returns the smaller cost of the busiest compute unit and which
// edge has it.
uint64_t TileCost(uint32_t M, uint32_t N, uint32_t units, bool* big)
{
    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    const uint64_t tiles128 = static_cast<uint64_t>((M + 127) / 128) * ((N + 127) / 128) * units;
    const uint64_t tiles64 = static_cast<uint64_t>((M + 63) / 64) * ((N + 63) / 64) * units;
    const uint64_t rounds128 = (tiles128 + cus - 1) / cus;
    const uint64_t cost128 = rounds128 * 400 + (rounds128 == 1 ? 32 : 0);
    const uint64_t cost64 = ((tiles64 + cus - 1) / cus) * 107;
    *big = cost128 <= cost64;
    return std::min(cost128, cost64);
}

template <bool TA, bool TB>
void LaunchStripAlone(const GemmF32Args& strip, uint32_t blocks, hipStream_t stream)
{
    hipLaunchKernelGGL((GemmF32SkinnyKernel<16, TA, TB, 4>), dim3(blocks), dim3(256), 0, stream,
                       strip);
}

int LaunchStrip(const GemmF32Args& strip, uint32_t blocks, bool transA, bool transB,
                hipStream_t stream)
{
    if (transA && transB)
        LaunchStripAlone<true, true>(strip, blocks, stream);
    else if (transA)
        LaunchStripAlone<true, false>(strip, blocks, stream);
    else if (transB)
        LaunchStripAlone<false, true>(strip, blocks, stream);
    else
        LaunchStripAlone<false, false>(strip, blocks, stream);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

// A thin strip of a product's last rows or columns: 16 x 16 tiles of the few-tile kernel on four
// wavefronts, whether it then rides along with the body's launch (`pending` has room) or is
// launched on its own, so that its bits do not depend on which.
int AddStrip(GemmF32Args strip, uint32_t units, bool outOffsetsAligned, bool transA, bool transB,
             GemmF32Strips* pending, hipStream_t stream)
{
    strip.tilesM = (strip.M + 15) / 16;
    strip.tilesN = (strip.N + 15) / 16;
    const uint64_t blocks = static_cast<uint64_t>(strip.tilesM) * strip.tilesN * units;
    if (blocks >= (1ull << 30))
        return sph::Fail(SPH_ERR_INVALID, "sph_gemm_f32 - too many tiles for one launch");
    strip.outVec = (outOffsetsAligned && (strip.N % 4 == 0) && (strip.ldc % 4 == 0) &&
                    (reinterpret_cast<uintptr_t>(strip.out) & 15u) == 0)
                       ? 1u
                       : 0u;
    for (int i = 0; i < 2 && pending != nullptr; ++i)
        if (pending->blocks[i] == 0)
        {
            pending->part[i] = strip;
            pending->blocks[i] = static_cast<uint32_t>(blocks);
            return SPH_OK;
        }
    return LaunchStrip(strip, static_cast<uint32_t>(blocks), transA, transB, stream);
}

// `transA`: A is stored K x M; `transB`: B is stored N x K.
// `pending`: strips waiting for a launch to ride along with; a launch that takes them empties
// the list.
int LaunchPart(const GemmF32Args& base, uint32_t units, bool allowVector, bool outOffsetsAligned,
               bool transA, bool transB, GemmF32Strips* pending, hipStream_t stream)
{
    GemmF32Args args = base;
    if (args.split == 0)
    {
        args.ldb = args.N;
        args.ldc = args.N;
        args.lda = args.M;
        args.basesOk =
            ((reinterpret_cast<uintptr_t>(args.A) | reinterpret_cast<uintptr_t>(args.B)) & 15u) == 0
                ? 1u
                : 0u;
    }
    const uint64_t wholeTiles64 =
        static_cast<uint64_t>((args.M + 63) / 64) * ((args.N + 63) / 64) * units;
    // Between a quarter and a half as many 64-tiles as compute units the straight-to-LDS
    // kernel on 64 x 32 tiles (K split over two groups of wavefronts) gives every compute
    // unit a tile and beats the few-tile kernel, whose 32 x 32 tiles ask the caches for twice
    // the operand bytes per flop (512 x 1024 x 1024: 17.0 us on the few-tile kernel).
    const uint64_t cusAll = static_cast<uint64_t>(sph::ComputeUnits());
    const bool midTiled = wholeTiles64 * 4 > cusAll && wholeTiles64 * 2 <= cusAll &&
                          args.basesOk != 0 && args.K >= 64 && args.M >= 4 && args.N >= 4 &&
                          // (rows past the last multiple of 4 are cut off from 68 rows up)
                          (args.M % 4 == 0 || args.M >= 68) &&
                          static_cast<uint64_t>(args.M) * args.K < (1ull << 30) &&
                          static_cast<uint64_t>(args.K) * args.N < (1ull << 30);
    const bool wholeIsFewTiles = wholeTiles64 * 2 <= cusAll && args.K >= 64 && !midTiled;
    // decided once, on the whole product, and carried by its parts (bit 2: tiled kernels, bit 3:
    // the K-split kernel on 64 x 32 tiles), so that a product's columns and rows are all summed
    // in one order however it is cut up
    const bool whole = args.split == 0;
    if (whole && !wholeIsFewTiles)
        args.split = midTiled ? 12u : 4u;
    // A product for the tiled kernels is cut into a body and up to two thin strips of its last
    // rows and columns, which the few-tile kernel's code computes (it reads any rows and columns
    // from anywhere); every output element is still computed once.  Cut off are
    //  - the last N % 4 columns: the rows of a B stored K x N are copied 4 columns at a time
    //    (measured 4096 x 4095 x 4096: 1615 us on the register-staged kernel's 4-byte loads);
    //  - the last M % 4 rows, from 68 rows up: an A stored K x M is copied 4 rows at a time;
    //  - up to 16 rows or columns past a multiple of the tile edge, when the compute unit with
    //    the most tiles then has fewer of them (1025^3: 17 x 17 tiles of 64 are two per
    //    compute unit somewhere, 16 x 16 one everywhere; measured 44.8 -> 23.4 us).
    // The cut depends on M, N, K and the batch only, not on how the operands are stored or
    // aligned, so a product's bits do not depend on that either.
    if (whole && (args.split & 4u) != 0 && args.M > 1 && args.K >= kBK)
    {
        const uint32_t baseM = (args.M >= 68 && args.N >= 4) ? args.M % 4 : 0;
        const uint32_t baseN = args.N > 4 ? args.N % 4 : 0;
        uint32_t peelM = baseM, peelN = baseN;
        if ((args.split & 8u) == 0)
        {
            auto candidates = [](uint32_t x, uint32_t base, bool allowed, uint32_t* list) {
                int n = 0;
                list[n++] = base;
                for (uint32_t edge = 64; edge <= 128 && allowed; edge *= 2)
                {
                    const uint32_t r = x % edge;
                    if (r != 0 && r <= 16 && r > base && x - r >= edge && r != list[n - 1])
                        list[n++] = r;
                }
                return n;
            };
            uint32_t listM[3], listN[3];
            const int countM = candidates(args.M, baseM, args.N >= 4, listM);
            const int countN = candidates(args.N, baseN, true, listN);
            // a strip's 16 x 16 tile: a sixteenth of a 64-tile's flops at about a quarter of
            // its rate, beside the body's tiles
            auto stripCost = [&](uint32_t rows, uint32_t cols) {
                const uint64_t blocks =
                    static_cast<uint64_t>((rows + 15) / 16) * ((cols + 15) / 16) * units;
                return (blocks + cusAll - 1) / cusAll * 27;
            };
            uint64_t best = ~0ull;
            for (int i = 0; i < countM; ++i)
                for (int j = 0; j < countN; ++j)
                {
                    bool big;
                    uint64_t cost = TileCost(args.M - listM[i], args.N - listN[j], units, &big);
                    if (listM[i] > baseM)
                        cost += stripCost(listM[i], args.N);
                    if (listN[j] > baseN)
                        cost += stripCost(args.M - listM[i], listN[j]);
                    if (cost < best)
                    {
                        best = cost;
                        peelM = listM[i];
                        peelN = listN[j];
                    }
                }
        }
        if (peelM != 0 || peelN != 0)
        {
            GemmF32Args body = args;
            body.split |= 3u;
            body.M = args.M - peelM;
            body.N = args.N - peelN;
            if (peelM != 0)
            {
                // rows [M - peelM, M), every column
                GemmF32Args bottom = args;
                bottom.split |= 3u;
                bottom.M = peelM;
                bottom.A = args.A + (transA ? body.M : static_cast<size_t>(body.M) * args.K);
                bottom.out = args.out + static_cast<size_t>(body.M) * args.ldc;
                const int rc = AddStrip(bottom, units, outOffsetsAligned, transA, transB, pending,
                                        stream);
                if (rc != SPH_OK)
                    return rc;
            }
            if (peelN != 0)
            {
                // rows [0, M - peelM), columns [N - peelN, N)
                GemmF32Args right = args;
                right.split |= 3u;
                right.M = body.M;
                right.N = peelN;
                right.B = args.B + (transB ? static_cast<size_t>(body.N) * args.K : body.N);
                right.out = args.out + body.N;
                if (args.bias != nullptr)
                    right.bias = args.bias + body.N;
                const int rc = AddStrip(right, units, outOffsetsAligned, transA, transB, pending,
                                        stream);
                if (rc != SPH_OK)
                    return rc;
            }
            return LaunchPart(body, units, allowVector, outOffsetsAligned, transA, transB, pending,
                              stream);
        }
    }
    // few 64 x 64 tiles and a long K: the kernel that splits K inside the workgroup (decided on
    // the whole product, so that its parts run the kernels the whole would)
    const uint64_t tiles64 =
        static_cast<uint64_t>((args.M + 63) / 64) * ((args.N + 63) / 64) * units;
    const bool fewTiles = (args.split & 4u) == 0 &&
                          tiles64 * 2 <= static_cast<uint64_t>(sph::ComputeUnits()) &&
                          args.K >= 64;
    args.outVec = (outOffsetsAligned && (args.N % 4 == 0) && (args.ldc % 4 == 0) &&
                   (reinterpret_cast<uintptr_t>(args.out) & 15u) == 0)
                      ? 1u
                      : 0u;
    // (of this launch: a part of a wider product may start anywhere)
    const bool basesAligned =
        ((reinterpret_cast<uintptr_t>(args.A) | reinterpret_cast<uintptr_t>(args.B)) & 15u) == 0;
    // row lengths of the two operands as stored
    const uint32_t lda = transA ? args.lda : args.K;
    const uint32_t ldb = transB ? args.K : args.ldb;
    const bool aligned = allowVector && basesAligned && (lda % 4 == 0) && (ldb % 4 == 0);

    // a single output row is a reduction over the rows of B, not a matrix-core job
    if (args.M == 1 && !transB && args.entries == nullptr && args.K >= 64 && units <= 65535 &&
        (args.split & 3u) == 0)
    {
        hipLaunchKernelGGL(GemvRowKernel, dim3((args.N + 63) / 64, units), dim3(kGemvWaves * 64),
                           0, stream, args);
        SPH_CHECK_LAUNCH();
        return SPH_OK;
    }

    if (fewTiles)
    {
        // (a product's strips are planned by AddStrip: always 16 x 16 tiles on four wavefronts)
        // 16 x 16 tiles while there are at most two per compute unit, or for a matrix of at most
        // 16 rows or columns: a quarter of the matrix-core work per workgroup on four times as
        // many compute units and less of a tile outside a narrow matrix, but twice the operand
        // bytes per flop (measured, 16-wide against 32-wide tiles: 256^3 3.7 / 5.2 us,
        // 1024 x 10 x 1024 7.2 / 8.9, 128 x 128 x 4096 13.8 / 23.4, 128 x 1024 x 1024 8.4 / 8.8;
        // 192 x 1024 x 1024 11.0 / 9.3, 256 x 1024 x 1024 14.0 / 9.0, 512^3 9.6 / 6.6,
        // 256 x 1024 x 4096 51.5 / 25.3)
        const uint64_t blocks16 =
            static_cast<uint64_t>((args.M + 15) / 16) * ((args.N + 15) / 16) * units;
        const uint32_t tile = (blocks16 <= static_cast<uint64_t>(sph::ComputeUnits()) * 2 ||
                               std::min(args.M, args.N) <= 16)
                                  ? 16u
                                  : 32u;
        args.tilesM = (args.M + tile - 1) / tile;
        args.tilesN = (args.N + tile - 1) / tile;
        const uint64_t blocks = static_cast<uint64_t>(args.tilesM) * args.tilesN * units;
        if (blocks >= (1ull << 31))
            return sph::Fail(SPH_ERR_INVALID, "sph_gemm_f32 - too many tiles for one launch");
        const dim3 gridSkinny(static_cast<uint32_t>(blocks));
        const bool wide = tile == 16 && blocks <= static_cast<uint64_t>(sph::ComputeUnits()) &&
                          args.K >= 512;
        if (transA && transB)
            LaunchSkinny<true, true>(args, gridSkinny, tile, wide, stream);
        else if (transA)
            LaunchSkinny<true, false>(args, gridSkinny, tile, wide, stream);
        else if (transB)
            LaunchSkinny<false, true>(args, gridSkinny, tile, wide, stream);
        else
            LaunchSkinny<false, false>(args, gridSkinny, tile, wide, stream);
        SPH_CHECK_LAUNCH();
        return SPH_OK;
    }

    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    // straight-to-LDS pipeline: whole K steps, 16-byte chunks everywhere, at least one chunk
    // per clamped edge, and lane offsets that fit 32 bits
    // (a K that is no multiple of the step: a last, partial one).  The copies take 16 bytes from
    // any 4-byte-aligned address, so only an operand stored k-major, which is copied 4 rows or
    // columns of the product at a time, needs a row length that is a multiple of 4.
    // (unit strides and table offsets may be anything)
    const bool dmaLayout = args.basesOk != 0 && (!transA || args.M % 4 == 0) &&
                           (transB || args.N % 4 == 0);
    const bool dma = dmaLayout && args.K >= kBK && args.M >= 4 && args.N >= 4 &&
                     static_cast<uint64_t>(args.M) * args.K < (1ull << 30) &&
                     static_cast<uint64_t>(args.K) * args.N < (1ull << 30);
    bool big;
    (void)TileCost(args.M, args.N, units, &big);
    // 64 x 32 tiles with K split over two groups of wavefronts (see the top of Launch).  The same
    // split on 64 x 64 tiles with eight wavefronts was measured for products with one 64-tile
    // per compute unit and does not pay (1024^3: 18.8 against 18.4 us): their loop already runs
    // at the matrix pipe's rate and what is left is the fixed cost of a launch.
    const int ksplit = ((args.split & 8u) != 0 && dma && !big && args.K >= 64) ? 2 : 0;
    const uint32_t bm = big ? 128 : 64;
    const uint32_t bn = ksplit == 2 ? 32 : bm;
    args.tilesM = (args.M + bm - 1) / bm;
    args.tilesN = (args.N + bn - 1) / bn;
    const uint64_t blocks = static_cast<uint64_t>(args.tilesM) * args.tilesN * units;
    if (blocks >= (1ull << 31) - 8)
        return sph::Fail(SPH_ERR_INVALID, "sph_gemm_f32 - too many tiles for one launch");
    args.tilesTotal = static_cast<uint32_t>(blocks);
    args.perXcd = (args.tilesTotal + 7) / 8;
    // band height ~ square root of the tiles an XCD works on at once (32 compute units, up
    // to two resident workgroups each), as a power of two
    {
        const uint32_t together = std::min<uint32_t>(args.perXcd, 64);
        uint32_t band = 1;
        while (band * band * 4 <= together)
            band *= 2;
        args.band = std::min(band, args.tilesM);
    }

    // More 64-tiles than workgroups that can be resident (two per compute unit): each
    // workgroup walks several tiles with the copy pipeline running across the tile boundaries
    // (configuration 2: 37.8 -> 35.9 us).  With fewer tiles every workgroup takes one, and the
    // form still pays because the old values of out are requested at the tile's first step
    // instead of after its last (1024^3: 18.7 -> 18.3 us, 1024 x 1024 x 256: 7.9 -> 7.4 us).
    // Only for whole tiles and a K
    // that fills the 4-stage ring of 32-wide steps a whole number of times.  The 128-tile
    // kernel would need more than 256 registers for it and lose its second resident workgroup
    // (measured 4096^3: 921 -> 966 us), so it keeps one tile per workgroup.
    const uint32_t slotsPerXcd = static_cast<uint32_t>(cus / 8 * 2);
    const bool walk = dma && !big && ksplit == 0 &&
                      args.M % 64 == 0 && args.N % 64 == 0 && args.K % 128 == 0 &&
                      (reinterpret_cast<uintptr_t>(args.bias) & 15u) == 0;
    // strips that wait ride along with a straight-to-LDS launch that is no walk
    GemmF32Strips strips{};
    if (pending != nullptr && dma && !walk && pending->blocks[0] != 0 &&
        blocks + pending->blocks[0] + pending->blocks[1] < (1ull << 31) - 8)
    {
        strips = *pending;
        *pending = GemmF32Strips{};
    }
    strips.first = (walk ? std::min(slotsPerXcd, args.perXcd) : args.perXcd) * 8;
    const dim3 grid(strips.first + strips.blocks[0] + strips.blocks[1]);
    if (transA && transB)
        LaunchTiled<true, true>(args, strips, grid, big, aligned, dma, walk, ksplit, stream);
    else if (transA)
        LaunchTiled<true, false>(args, strips, grid, big, aligned, dma, walk, ksplit, stream);
    else if (transB)
        LaunchTiled<false, true>(args, strips, grid, big, aligned, dma, walk, ksplit, stream);
    else
        LaunchTiled<false, false>(args, strips, grid, big, aligned, dma, walk, ksplit, stream);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

int Launch(const GemmF32Args& base, uint32_t units, bool allowVector, bool outOffsetsAligned,
           bool transA, bool transB, hipStream_t stream)
{
    GemmF32Strips pending{};
    int rc = LaunchPart(base, units, allowVector, outOffsetsAligned, transA, transB, &pending,
                        stream);
    // strips no launch has taken along: each on its own
    for (int i = 0; i < 2 && rc == SPH_OK; ++i)
        if (pending.blocks[i] != 0)
            rc = LaunchStrip(pending.part[i], pending.blocks[i], transA, transB, stream);
    return rc;
}

int GrowTable(EntryTable& t, size_t count)
{
    if (t.capacity >= count)
        return SPH_OK;
    // nothing may still be reading the old buffers
    if (t.lastStream != nullptr)
        SPH_HIP_TRY(hipEventSynchronize(t.consumed));
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
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&t.dev), cap * sizeof(SphGemmEntry)));
    ::sph::CountAllocation();
    SPH_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&t.staging), cap * sizeof(SphGemmEntry),
                              hipHostMallocDefault));
    if (t.uploaded == nullptr)
        SPH_HIP_TRY(hipEventCreateWithFlags(&t.uploaded, hipEventDisableTiming));
    if (t.consumed == nullptr)
        SPH_HIP_TRY(hipEventCreateWithFlags(&t.consumed, hipEventDisableTiming));
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
    const bool stridesAligned = batch == 1 || ((strideA % 4 == 0) && (strideB % 4 == 0));
    return Launch(args, batch, stridesAligned, strideOut % 4 == 0 || batch == 1,
                  (flags & SPH_GEMM_TRANS_A) != 0, (flags & SPH_GEMM_TRANS_B) != 0, stream);
}

int sph_gemm_f32_sgd(float* out, const float* A, const float* B, uint32_t M, uint32_t N,
                     uint32_t K, float scale, float rate, uint32_t flags)
{
    SPH_REQUIRE(M != 0 && N != 0, "M and N must be non-zero");
    SPH_REQUIRE((flags & ~(SPH_GEMM_TRANS_A | SPH_GEMM_TRANS_B)) == 0, "unknown flag");
    SPH_REQUIRE(out != nullptr, "null pointer");
    SPH_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    if (K == 0)
        return SPH_OK;  // an empty gradient: out - 0 leaves every value as it is
    GemmF32Args args{};
    args.out = out;
    args.A = A;
    args.B = B;
    args.entries = nullptr;
    args.M = M;
    args.N = N;
    args.K = K;
    args.overwrite = 0u;  // the old value of out takes part
    args.sgd = 1u;
    args.sgdScale = scale;
    args.sgdRate = rate;
    return Launch(args, 1, true, true, (flags & SPH_GEMM_TRANS_A) != 0,
                  (flags & SPH_GEMM_TRANS_B) != 0, stream);
}

int sph_linear_forward_f32(float* y, const float* x, const float* W, const float* bias,
                           uint32_t batch, uint32_t inputs, uint32_t outputs, uint32_t flags)
{
    SPH_REQUIRE(batch != 0 && outputs != 0, "batch and outputs must be non-zero");
    SPH_REQUIRE((flags & ~SPH_LINEAR_RELU) == 0, "unknown flag");
    SPH_REQUIRE(y != nullptr && bias != nullptr, "null pointer");
    SPH_REQUIRE(inputs == 0 || (x != nullptr && W != nullptr), "null pointer");
    SPH_REQUIRE(y != x && y != W, "y must not alias an input");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;

    GemmF32Args args{};
    args.out = y;
    args.A = x;
    args.B = W;
    args.entries = nullptr;
    args.M = batch;
    args.N = outputs;
    args.K = inputs;
    args.overwrite = 1u;
    args.bias = bias;
    args.relu = (flags & SPH_LINEAR_RELU) ? 1u : 0u;
    return Launch(args, 1, true, true, false, false, stream);
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
    SPH_REFUSE_WHILE_CAPTURING();  // the offset table is uploaded from host memory
    if (count == 0 || K == 0)
        return SPH_OK;
    SPH_REQUIRE(entries != nullptr && out != nullptr && A != nullptr && B != nullptr,
                "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const int device = sph::CurrentDevice();
    SPH_REQUIRE(device >= 0 && device < 16, "device id out of range");

    bool offsetsAligned = true, outAligned = true;
    for (uint32_t i = 0; i < count; ++i)
    {
        offsetsAligned = offsetsAligned && ((entries[i].aOff | entries[i].bOff) % 4) == 0;
        outAligned = outAligned && (entries[i].outOff % 4) == 0;
    }

    EntryTable& t = ThreadTable(device);
    {
        const int rc = GrowTable(t, count);
        if (rc != SPH_OK)
            return rc;
    }
    // the thread has moved to another stream since the table was last read: order the new
    // stream behind that launch (no host wait)
    if (t.lastStream != nullptr && t.lastStream != stream)
        SPH_HIP_TRY(hipStreamWaitEvent(stream, t.consumed, 0));
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
    int rc = SPH_OK;
    while (begin < count && rc == SPH_OK)
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
        rc = Launch(args, end - begin, offsetsAligned, outAligned, false, false, stream);
        begin = end;
    }
    SPH_HIP_TRY(hipEventRecord(t.consumed, stream));
    return rc;
}

int sph_gemm_f32_grouped_device(const SphGemmEntry* deviceEntries, uint32_t count, float* out,
                                const float* A, const float* B, uint32_t M, uint32_t N,
                                uint32_t K, uint32_t flags)
{
    SPH_REQUIRE(M != 0 && N != 0, "M and N must be non-zero");
    SPH_REQUIRE((flags & ~SPH_GROUPED_OFFSETS_MULTIPLE_OF_4) == 0, "unknown flag");
    if (count == 0 || K == 0)
        return SPH_OK;
    SPH_REQUIRE(deviceEntries != nullptr && out != nullptr && A != nullptr && B != nullptr,
                "null pointer");
    hipStream_t stream = sph::CurrentStream();
    if (stream == nullptr)
        return SPH_ERR_DEVICE;
    const bool aligned = (flags & SPH_GROUPED_OFFSETS_MULTIPLE_OF_4) != 0;
    GemmF32Args args{};
    args.out = out;
    args.A = A;
    args.B = B;
    args.entries = deviceEntries;
    args.M = M;
    args.N = N;
    args.K = K;
    return Launch(args, count, aligned, aligned, false, false, stream);
}

}  // extern "C"
