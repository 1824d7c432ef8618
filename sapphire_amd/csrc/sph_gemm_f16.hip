// fp16-input / fp32-accumulate GEMM  out[u] (+)= A[u] * B[u]  on the CDNA4
// matrix cores.  This is the tensor-core path the reference only declares (WmmaGemm,
// Includes/Sapphire/compute/dense/cuda/kernels/GemmKernel.cuh:14-50): half
// inputs, fp32 accumulation, row-major operands, result added into out.
//
// Six kernels:
//
//   GemmF16Few      products with at most one 32 x 32 output tile per compute unit (or at most 16
//     rows or columns), whatever K, the storage flags and the alignment: one 32 x 32 or 16 x 16
//     tile per workgroup, K split over its wavefronts, fragments loaded straight from global
//     memory in MFMA layout.  The tiled kernels below would use a few compute units for these
//     and wait out a memory latency per K step on each.
//
//   GemmF16Tile256  K >= 32 (a multiple of 32, or any K >= 64), N a multiple of 8, at least three
//     quarters as many 256 x 256 tiles as compute units and at least three quarters of
//     the tiled area inside the matrix (a variant with clamped copies and a guarded
//     epilogue serves M, N that are not multiples of 256).  One workgroup of 8 wavefronts
//     (2 x 4) owns a 256 x 256 output tile; each wavefront a 128 x 64 part of it: 8 x 4
//     blocks of v_mfma_f32_16x16x32_f16, 128 accumulator registers.  K advances 32 at a
//     time through four LDS stages of 32 KiB (A 256x32, B 32x256).  Global memory is
//     copied straight into LDS (global_load_lds, 16 bytes per lane, no VGPR staging),
//     three to four steps ahead of the MFMAs.  LDS is written lane-linear by those
//     copies, so bank conflicts are removed by choosing WHICH global chunk each lane
//     fetches: A rows are XOR-swizzled in 16-byte chunks (chunk ^ (row/2)%8), B k-rows
//     in 32-byte chunks (chunk ^ (2*(k%4) + (k/8)%2)); both patterns measured
//     conflict-free for the reads below (4.6 and 2.6 clocks per wavefront read).
//     A fragments are read with ds_read_b128 (8 consecutive k of one row); B is stored
//     k-major, so its fragments (8 consecutive k of one column) come from two
//     ds_read_b64_tr_b16 transposing reads.  The MFMA operands are swapped (B fragment
//     first) so that every lane ends up with 4 consecutive columns of one output row
//     and the epilogue moves 16 bytes per access.  Workgroup ids are remapped so that
//     the 32 workgroups that land on one XCD (ids congruent mod 8) cover a compact
//     8 x 4 block of tiles and share their A and B panels through that XCD's L2.
//
//   GemmF16Tile256<..., NT = 128>  the same kernel on 256 x 128 tiles, taken while there are
//     between 11/16 of such a tile and one tile per compute unit.
//
//   GemmF16Dma128   the same conditions, any M: the
//     same ingredients on 128 x 128 tiles with 4 or 8 wavefronts (v_mfma_f32_32x32x16_f16), for
//     shapes with too few 256-tiles to fill the chip.
//
//   GemmF16Dma64    at most half as many 128 x 128 tiles as compute units and K >= 64: 64 x 64
//     tiles, K steps of 64, 4 wavefronts.
//
//   GemmF16General  everything else.  128 x 128 tile, 4 wavefronts, K step 32,
//     global loads staged through registers, 16 bytes at a time (aligned, from a 4-byte
//     boundary, or as aligned dwords that are shifted when a row starts at an odd half), padded
//     LDS rows.
//
// K = 32 q + r, r != 0, K >= 64 stays on the first two kernels: a last step over [K - 32, K) in
// which the fragment positions whose k was multiplied already are cleared.
//
// N = 8 q + r, r != 0: the first 8 q columns go to the tiled straight-to-LDS kernels when they
// would take that shape (the copies into LDS need no alignment, so rows of B and of out may start
// anywhere; only a copy's 8 columns have to lie inside the row) and the last r columns to the
// code of GemmF16Few, as do the last M % 8 rows of an A stored K x M and up to 16 rows or columns
// just past a tile edge: as strips on the last workgroups of the body's own launch (LaunchF16).
#include "sph_internal.h"
#include "sph_k_partition.h"

#include <algorithm>
#include <type_traits>

namespace
{
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
// eight halves that need only be 4-byte aligned: a 16-byte vector memory access asks for no more
typedef halfx8 halfx8a4 __attribute__((aligned(4)));
typedef __attribute__((address_space(3))) void* LdsPtr;
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4* LdsShortx4Ptr;

struct GemmF16Args
{
    float* out;
    const _Float16* A;
    const _Float16* B;
    uint32_t M, N, K;
    uint32_t lda;  // halves between consecutive rows of A as stored (K; M for an A stored
                   // K x M, unless a launch covers some of the rows)
    uint32_t ldb;  // halves between consecutive k-rows of a B stored K x N (N unless a launch
                   // covers some of the columns)
    uint32_t ldc;  // floats between consecutive rows of out (likewise)
    uint32_t tilesM, tilesN;
    uint32_t totalTiles;  // tilesM * tilesN * batch
    int64_t strideOut, strideA, strideB;
    uint32_t overwrite;
    uint32_t outVec;  // general kernel: out may be accessed 16 bytes at a time
};

// Eight consecutive halves from any 2-byte-aligned address, as aligned dwords: a 16-byte load from
// an address that is no multiple of 4 is several times slower than one from a multiple of 4
// (measured on the few-tile kernel, 128 x 128 x 4095 against x 4096: 24.4 / 10.5 us).  The five
// dwords that hold the halves are loaded (four as one access, the fifth on its own) and, for an
// odd half index, shifted down by 16 bits.  Every dword read holds at least one of the eight
// halves, so nothing is read that does not share an aligned dword with the operand.  The
// shift is applied by Get(), where the value is used, so that a load can stay in flight until
// then.
struct Halves8
{
    uintx4 w;
    uint32_t extra;
    __device__ __forceinline__ static Halves8 Load(const _Float16* p)
    {
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        const uint32_t odd = static_cast<uint32_t>(a >> 1) & 1u;
        const uint32_t* q = reinterpret_cast<const uint32_t*>(a - 2 * odd);
        typedef uintx4 uintx4a4 __attribute__((aligned(4)));
        Halves8 h;
        h.w = *reinterpret_cast<const uintx4a4*>(q);
        h.extra = q[3 + odd];  // even address: the fourth dword once more
        return h;
    }
    // 16 for halves loaded from an address that is no multiple of 4, else 0
    __device__ __forceinline__ static uint32_t Shift(const _Float16* p)
    {
        return (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)) & 2u) * 8u;
    }
    __device__ __forceinline__ halfx8 Get(uint32_t shift) const
    {
        uintx4 r;
        r[0] = __builtin_amdgcn_alignbit(w[1], w[0], shift);
        r[1] = __builtin_amdgcn_alignbit(w[2], w[1], shift);
        r[2] = __builtin_amdgcn_alignbit(w[3], w[2], shift);
        r[3] = __builtin_amdgcn_alignbit(extra, w[3], shift);
        return __builtin_bit_cast(halfx8, r);
    }
};

// Thin strips of a product's last rows and columns that ride along with the launch of its body:
// the workgroups from `first` on (the body's own come before, so they keep their numbers and with
// them their place among the 8 XCDs) run the few-tile kernel's code, 16 x 16 tiles, on part[0]
// (blocks[0] of them) and then part[1] (blocks[1]).  A strip's workgroups are short; coming last
// they fill the places that the body's last tiles leave free, where a launch of their own would
// start after the body's last tile has finished.
struct GemmF16Strips
{
    GemmF16Args part[2];
    uint32_t blocks[2];
    uint32_t first;  // launcher: the number of the body's workgroups
};

template <int TILE, bool TA, bool TB, int WAVES, bool ODD>
__device__ __forceinline__ void GemmF16FewBody(const GemmF16Args& args, uint32_t block,
                                               float* partial);

// Tile edge of the strips.  (A kernel of eight wavefronts keeps one or two workgroups on a compute
// unit and its strips' workgroups take such a place each; 32 x 32 tiles would halve their number
// but load twice the rows each, and measured slower: 2048 x 2052 x 2048 31.6 -> 41.2 us,
// 4096 x 4100 x 4096 129 -> 144 us.)
constexpr uint32_t kStripTile = 16;

// The strip a workgroup of a body's launch computes, if it is one of those from `first` on: true,
// and the workgroup is done.  `scratch`: (WAVES - 1) * kStripTile^2 floats of LDS.
template <bool TA, bool TB, int WAVES>
__device__ __forceinline__ bool RunStrip(const GemmF16Strips& strips, uint32_t block,
                                         float* scratch)
{
    if (block < strips.first)
        return false;
    const uint32_t local = block - strips.first;
    const uint32_t which = local < strips.blocks[0] ? 0u : 1u;
    GemmF16FewBody<static_cast<int>(kStripTile), TA, TB, WAVES, true>(
        strips.part[which], local - (which != 0 ? strips.blocks[0] : 0u), scratch);
    return true;
}

// Transposing LDS read: within each group of 16 lanes, lane s supplies the
// address of 4 halves (row s/4 of a 4-row block, columns 4*(s%4)..+3) and
// receives the 4 rows' values of column s.
__device__ __forceinline__ halfx4 LdsReadTr(const _Float16* p)
{
    return __builtin_bit_cast(halfx4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsShortx4Ptr)(p)));
}

// Asynchronous 16-byte-per-lane copy from global memory straight into LDS
// (global_load_lds_dwordx4): lane i reads 16 bytes at uniformBase + laneByteOffset +
// OFFSET and they land at ldsByteAddr + OFFSET + 16*i.  ldsByteAddr must be uniform
// across the wavefront (it travels in M0) and so must uniformBase (an SGPR pair).
// The copy is counted by vmcnt like any vector memory load; the caller waits with
// WaitVmem() before the data is read.  Issued through inline assembly so that the
// compiler does not serialise it against unrelated LDS reads.
template <int OFFSET>
__device__ __forceinline__ void DmaToLds16(uint32_t laneByteOffset, const void* uniformBase,
                                           uint32_t ldsByteAddr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
                 :
                 : "s"(ldsByteAddr), "v"(laneByteOffset), "s"(uniformBase), "n"(OFFSET)
                 : "memory");
}

template <int N>
__device__ __forceinline__ void WaitVmem()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

__device__ __forceinline__ uint32_t LdsAddress(const void* p)
{
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)(p)));
}

// 16-byte accesses to out with the streaming hint: the tile is read once and written once, so
// it should neither displace the A and B panels in the L2 nor stay there dirty until the end of
// the kernel.
typedef float floatx4 __attribute__((ext_vector_type(4)));
// Four floats that need only be 4-byte aligned: rows of out start anywhere when the row pitch is
// not a multiple of 4 floats, and a 16-byte vector memory access only asks for dword alignment.
typedef floatx4 floatx4a4 __attribute__((aligned(4)));
__device__ __forceinline__ float4 NtLoad4(const float* p)
{
    const floatx4 v = __builtin_nontemporal_load(reinterpret_cast<const floatx4a4*>(p));
    return make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ float4 Load4(const float* p)
{
    const floatx4 v = *reinterpret_cast<const floatx4a4*>(p);
    return make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void Store4(float* p, float4 v)
{
    const floatx4 w = { v.x, v.y, v.z, v.w };
    *reinterpret_cast<floatx4a4*>(p) = w;
}

__device__ __forceinline__ halfx8 Join(halfx4 lo, halfx4 hi)
{
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// K = 32 q + r, r != 0: the last K step runs over the window [K - 32, K), whose first 32 - r
// positions the step before has multiplied already.  A fragment register holds 8 consecutive
// positions (those of group `group`, 8 group .. 8 group + 7); TailMask gives the bits of the
// ones that are new, KeepNew clears the others.  Both operands are cleared, so that a value
// that lies in both windows counts once even when it is an infinity.
__device__ __forceinline__ uintx4 TailMask(uint32_t group, uint32_t repeated)
{
    uintx4 m;
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const uint32_t first = 8 * group + 2 * i;
        m[i] = (first >= repeated ? 0x0000ffffu : 0u) | (first + 1 >= repeated ? 0xffff0000u : 0u);
    }
    return m;
}
__device__ __forceinline__ halfx8 KeepNew(halfx8 f, uintx4 m)
{
    return __builtin_bit_cast(halfx8, __builtin_bit_cast(uintx4, f) & m);
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
// 256 x 256 tile: K step 32, four LDS stages
// ---------------------------------------------------------------------------
constexpr int kT = 256;         // tile edge
constexpr int kTK = 32;         // K step
constexpr int kTStages = 4;
constexpr int kStageBytes = kT * kTK * 2;  // per operand per stage (16 KiB)

// ---------------------------------------------------------------------------
// 256 x 256 tile kernel, v_mfma_f32_16x16x32_f16
// ---------------------------------------------------------------------------
// Why the 16x16x32 instruction: on real (non-zero) operands the chip holds a power limit and
// the matrix-core rate follows the energy per product, not the issue rate.  The deeper
// instruction reads and writes every accumulator once per 32 products instead of once per 16:
// matrix cores fed from LDS only, N(0, 1/64) operands, take 72.8 us for the flops of 4096^3
// with it against 80.6 us with v_mfma_f32_32x32x16_f16 (on all-zero operands, where nothing
// is limited by power, 63.6 against 61.1 us).
//
// Stage layout.  A stage: 128 LDS rows of 128 bytes; LDS row R holds A[R][k0..k0+31] in its
// first 64 bytes and A[R+128][k0..k0+31] in the last 64, 16-byte chunks XOR-swizzled with
// (R/2)%8: the LDS serves a 16-byte read to 16 lanes per clock from 64 banks, and 16
// consecutive 128-byte rows are 8 even ones on banks 0-31 and 8 odd ones on banks 32-63, so
// the 8 rows of either parity must take 8 different chunk positions.  B stage: 32 k-rows of
// 512 bytes, 32-byte chunks XOR-swizzled with 2*(k%4) + (k/8)%2, so that the two 16-lane
// groups a transposing read serves in one clock (k and k + 8) fall on different banks.
//
// Fragments.
//   A fragment i (rows 16i..16i+15 of the wavefront's 128): lane l holds row l%16, k 8*(l/16)..+7:
//     one 16-byte LDS read.
//   B fragment j (columns 16j..16j+15 of its 64): lane l holds column l%16, k 8*(l/16)..+7: two
//     transposing reads, each 16-lane group g reading the 4 x 16 block at k = 8g + 4h.
//   With the operands swapped, register v of lane l is row l%16, column 4*(l/16) + v of a block.
//
// Pipeline.  LDS holds four K steps.  While step kt is multiplied, the B copies of step kt+3
// and the A copies of step kt+4 are issued between the MFMAs; a copy has three steps to land.
// Copies complete in issue order and exactly 2*COPIES_PER_STAGE are issued between the last
// copy of step kt+1 and the synchronisation point of step kt, so vmcnt <= 2*COPIES_PER_STAGE
// there means step kt+1 is in LDS.  A step is split by rows: blocks 0-3 before the barrier, 4-7
// after it.  The A fragments of a step's second half are read during its first half; behind
// the barrier the first half's A registers take the next step's rows 0-63 and a second set of
// B registers its B fragments.  The loop body is written out for the four stages so that
// every LDS address is a register plus an immediate; sched_barrier fences pin the
// interleaving of MFMAs, LDS reads and copies written here.
//
// RAGGED: M and N need not be multiples of 256 (N still a multiple of 8).  Rows past M and
// 16-byte column chunks past N are clamped to the last valid ones when they are copied (they
// feed only outputs that are never stored) and the epilogue skips what lies outside.
//
// CSP != 0 (whole tiles, accumulating, at least CLoopSteps(CSP) K steps): the old contents of
// out are not read in the epilogue, when every workgroup would ask for them at once, but
// during the first K steps: every CSP-th step a wavefront has one of its eight 16-row blocks
// copied straight into a 4 KiB LDS mailbox in accumulator layout and, CSP steps later, adds it
// to the accumulators of that block.  The epilogue then only stores.  out + A*B is therefore
// associated as (partial sum + out) + rest of the sum, like a tensor-core kernel that loads
// the accumulator fragment from C, not as "sum, then one add".
//
// Epilogue.  One store instruction in accumulator layout would touch 16 rows with 64 bytes
// each.  To write (and, without CSP, read) whole 256-byte row segments instead, each
// wavefront turns its 128 x 64 part round through a private 16 KiB piece of LDS, 64 rows at a
// time: after that a lane holds 4 consecutive columns and 16 consecutive lanes cover one row.
constexpr int CLoopSteps(int csp, int rowBlocks = 8)
{
    return (rowBlocks * csp + 1 + 3) / 4 * 4;
}
//
// NT = 128: the tile is 256 rows by 128 columns and the eight wavefronts are arranged 4 x 2, a
// 64 x 64 part each (4 x 4 blocks, 64 accumulator registers), for products with too few
// 256 x 256 tiles to fill the chip: against 128 x 128 tiles a compute unit moves three quarters
// of the bytes per flop into LDS and a wavefront reads 8 fragments per 16 matrix instructions
// instead of 4 per 4.  The B stage then has k-rows of 256 bytes (the same chunk swizzle) and a
// wavefront makes two copies of A and one of B per step.
template <bool RAGGED, int CSP, bool TA, bool TB, bool TAIL, int NT = 256>
__global__ __launch_bounds__(512) void GemmF16Tile256(const GemmF16Args args,
                                                      const GemmF16Strips strips)
{
    static_assert(NT == 256 || NT == 128, "256 x 256 or 256 x 128 tiles");
    constexpr int WAVES = 8;
    constexpr int WN = NT / 64;               // wavefronts across the tile: 4 or 2
    constexpr int WMROWS = kT / (WAVES / WN); // rows per wavefront: 128 or 64
    constexpr int MB = WMROWS / 16;           // 16-row blocks per wavefront: 8 or 4
    constexpr int ROUNDS_A = 2;               // 1 KiB copies per wavefront and stage: A 16 KiB,
    constexpr int ROUNDS_B = NT / 128;        // B 64 * NT bytes
    constexpr int COPIES_PER_STAGE = ROUNDS_A + ROUNDS_B;
    constexpr int kBytesStageA = kStageBytes;
    constexpr int kBytesStageB = NT * kTK * 2;
    constexpr uint32_t kBias = 4096;
    constexpr bool CLOOP = CSP != 0;
    constexpr int kCLoopSteps = CLoopSteps(CSP, MB);
    static_assert(!(CLOOP && RAGGED), "old values are added in the loop for whole tiles only");

    // the ring of stages; the epilogue reuses it as eight private pieces of 16 KiB
    constexpr int kRingBytes = kTStages * (kBytesStageA + kBytesStageB);
    constexpr int kLdsBytes = kRingBytes > WAVES * 64 * 64 * 4 ? kRingBytes : WAVES * 64 * 64 * 4;
    __shared__ __attribute__((aligned(1024))) char LdsRaw[kLdsBytes];
    __shared__ __attribute__((aligned(1024))) float CMail[CLOOP ? WAVES * 1024 : 4];
    auto AStage = [&](int stage) {
        return reinterpret_cast<_Float16*>(LdsRaw + stage * kBytesStageA);
    };
    auto BStage = [&](int stage) {
        return reinterpret_cast<_Float16*>(LdsRaw + kTStages * kBytesStageA + stage * kBytesStageB);
    };

    uint32_t unit, tm, tn;
    const uint32_t block = blockIdx.x;
    if (RunStrip<TA, TB, WAVES>(strips, block, reinterpret_cast<float*>(LdsRaw)))
        return;
    if (!MapTile(block, args.tilesM, args.tilesN, args.totalTiles, unit, tm, tn))
        return;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t waveM = wave / WN;  // WMROWS rows each
    const uint32_t waveN = wave % WN;  // 64 columns each

    const uint32_t K = args.K, N = args.N;
    const uint32_t rowsLeft = RAGGED ? min(static_cast<uint32_t>(kT), args.M - tm * kT) : kT;
    const uint32_t colsLeft = RAGGED ? min(static_cast<uint32_t>(NT), N - tn * NT) : NT;
    // An operand is either K-contiguous (x-rows of K halves: A as given, B stored N x K with
    // TB) or k-major (k-rows of x halves: B as given, A stored K x M with TA); x is the row of A
    // or the column of B.  A K-contiguous operand takes the "A stage" layout and the 16-byte
    // fragment read described above, a k-major one the "B stage" layout and the transposing
    // read, whichever matrix it is, so the MFMAs and their order do not depend on the flags.
    const uint32_t pitchA = args.lda;  // halves between rows of A as stored
    const uint32_t pitchB = TB ? K : args.ldb;
    const uint32_t ldc = args.ldc;
    const _Float16* __restrict__ A = args.A + args.strideA * static_cast<int64_t>(unit) +
                                     static_cast<size_t>(tm) * kT * (TA ? 1u : pitchA);
    const _Float16* __restrict__ B = args.B + args.strideB * static_cast<int64_t>(unit) +
                                     static_cast<size_t>(tn) * NT * (TB ? pitchB : 1u);
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit) +
                              static_cast<size_t>(tm) * kT * ldc + static_cast<size_t>(tn) * NT;

    // ---- global -> LDS copy plan --------------------------------------------
    // A copy instruction moves 1 KiB per wavefront.  Wavefront w fills ROUNDS KiB at
    // w*ROUNDS*1024 of an operand's stage in ROUNDS copies (ROUNDS_A, ROUNDS_B); copy r puts lane
    // i's 16 bytes at w*ROUNDS*1024 + r*1024 + i*16.
    //   K-contiguous: that is LDS row R = w*8*ROUNDS + r*8 + i/8, physical chunk i%8, which
    //      must hold logical chunk L = (i%8) ^ ((R/2)%8): x = R (L < 4) or R+128 (L >= 4),
    //      k offset (L%4)*8.
    //   k-major (256 columns; twice the k-rows per copy for 128): k = w*2*ROUNDS + r*2 + i/32,
    //      physical 16-byte chunk i%32, 32-byte chunks
    //      swizzled as described above.
    // The global address of a copy is a uniform base that advances with the K step plus a
    // per-lane byte offset that never changes.  The instruction offset r*1024 is added to
    // both the LDS and the global address, so the lane offsets subtract it again.  K steps
    // beyond the last are clamped to it: those copies land in buffers that are no longer
    // read, which keeps the number of copies in flight constant.
    // (an operand of X rows or columns, `rounds` copies per wavefront: the rows / k-rows are
    // dealt to the wavefronts in order, X / 2 LDS rows or 32 k-rows in all)
    auto laneKContig = [&](int r, uint32_t xLeft, uint32_t pitch, uint32_t X, uint32_t rounds) {
        const uint32_t R = wave * (8 * rounds) + 8 * r + (lane >> 3);
        const uint32_t L = (lane & 7) ^ ((R >> 1) & 7);
        const uint32_t x = R + ((L & 4) ? X / 2 : 0u);
        return (min(x, xLeft - 1) * pitch + (L & 3) * 8) * 2 + kBias - r * 1024;
    };
    auto laneKMajor = [&](int r, uint32_t xLeft, uint32_t pitch, uint32_t X, uint32_t rounds) {
        const uint32_t lanesPerRow = X / 8;          // 16-byte chunks of a k-row
        const uint32_t rowsPerCopy = 64 / lanesPerRow;
        const uint32_t phys16 = lane % lanesPerRow;
        const uint32_t k = (wave * rounds + r) * rowsPerCopy + lane / lanesPerRow;
        const uint32_t swz = 2 * (k & 3) + ((k >> 3) & 1);
        const uint32_t logical16 = (((phys16 >> 1) ^ swz) << 1) | (phys16 & 1);
        return (k * pitch + min(logical16 * 8, xLeft - 8)) * 2 + kBias - r * 1024;
    };
    uint32_t aLane[ROUNDS_A], bLane[ROUNDS_B];
#pragma unroll
    for (int r = 0; r < ROUNDS_A; ++r)
        aLane[r] = TA ? laneKMajor(r, rowsLeft, pitchA, kT, ROUNDS_A)
                      : laneKContig(r, rowsLeft, pitchA, kT, ROUNDS_A);
#pragma unroll
    for (int r = 0; r < ROUNDS_B; ++r)
        bLane[r] = TB ? laneKContig(r, colsLeft, pitchB, NT, ROUNDS_B)
                      : laneKMajor(r, colsLeft, pitchB, NT, ROUNDS_B);
    const uint32_t waveU = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t aLds = LdsAddress(AStage(0)) + waveU * (ROUNDS_A * 1024);
    const uint32_t bLds = LdsAddress(BStage(0)) + waveU * (ROUNDS_B * 1024);
    const char* aGlobal = reinterpret_cast<const char*>(A) - kBias;
    const char* bGlobal = reinterpret_cast<const char*>(B) - kBias;
    const size_t aStepBytes = TA ? static_cast<size_t>(kTK) * pitchA * 2 : kTK * 2;
    const size_t bStepBytes = TB ? kTK * 2 : static_cast<size_t>(kTK) * pitchB * 2;

    // TAIL: K = 32 q + r with 0 < r < 32.  The last of the q + 1 steps takes the window
    // [K - 32, K), which lies inside the matrix and needs no other lane offsets (only its
    // start differs from a whole step's); its first 32 - r values of k were multiplied in
    // step q - 1 already, so the fragment positions that hold them (for A and B alike) are
    // cleared before that step's MFMAs.
    const uint32_t steps = TAIL ? K / kTK + 1 : K / kTK;
    const size_t aLastBytes = TAIL ? (TA ? static_cast<size_t>(K - kTK) * pitchA * 2 : (K - kTK) * 2) : 0;
    const size_t bLastBytes = TAIL ? (TB ? (K - kTK) * 2 : static_cast<size_t>(K - kTK) * pitchB * 2) : 0;
    auto copyA = [&](uint32_t kt, int stage, auto round) {
        constexpr int r = decltype(round)::value;
        const uint32_t src = min(kt, steps - 1);
        const size_t start = (TAIL && src == steps - 1) ? aLastBytes : static_cast<size_t>(src) * aStepBytes;
        DmaToLds16<r * 1024>(aLane[r], aGlobal + start, aLds + stage * kBytesStageA);
    };
    auto copyB = [&](uint32_t kt, int stage, auto round) {
        constexpr int r = decltype(round)::value;
        const uint32_t src = min(kt, steps - 1);
        const size_t start = (TAIL && src == steps - 1) ? bLastBytes : static_cast<size_t>(src) * bStepBytes;
        DmaToLds16<r * 1024>(bLane[r], bGlobal + start, bLds + stage * kBytesStageB);
    };

    // ---- LDS -> fragment read plan ---------------------------------------------------
    // Block b of an operand = x in [x0 + 16b, x0 + 16b + 16) with x0 the wavefront's first row
    // (A: waveM*128, 8 blocks) or column (B: waveN*64, 4 blocks); a lane wants x = l16 of the
    // block and k = 8g .. 8g+7.
    //   K-contiguous: x is half x/128 of LDS row x%128 = (x0%128) + 16b + l16, logical chunk
    //      4*(x/128) + g, swizzle (row/2)%8 = (l16/2)%8: one base offset plus 16b rows.
    //   k-major: k-row 8g + 4h + l16/4, 32-byte chunk x0/16 + b swizzled, halves 4*(l16%4)..+3
    //      of it: one offset per block.
    const uint32_t l16 = lane & 15;
    const uint32_t g = lane >> 4;
    // (X = extent of the operand in the tile: 256 rows of A, NT columns of B)
    auto offKContig = [&](uint32_t x0, uint32_t X) {
        const uint32_t row = (x0 & (X / 2 - 1)) + l16;
        return row * 64 + ((((x0 / (X / 2)) * 4 + g) ^ ((l16 >> 1) & 7)) * 8);  // + b*16*64
    };
    auto offKMajor = [&](uint32_t x0, int b, uint32_t X) {
        const uint32_t kRow = 8 * g + (l16 >> 2);
        const uint32_t swz = 2 * ((l16 >> 2) & 3) + (g & 1);
        return kRow * X + (((x0 / 16 + b) ^ swz) * 16) + (l16 & 3) * 4;
    };
    constexpr int kOffA = TA ? MB : 1, kOffB = TB ? 1 : 4;
    uint32_t aOff[kOffA], bOff[kOffB];
#pragma unroll
    for (int b = 0; b < kOffA; ++b)
        aOff[b] = TA ? offKMajor(waveM * WMROWS, b, kT) : offKContig(waveM * WMROWS, kT);
#pragma unroll
    for (int b = 0; b < kOffB; ++b)
        bOff[b] = TB ? offKContig(waveN * 64, NT) : offKMajor(waveN * 64, b, NT);
    auto readKContig = [&](const _Float16* p) { return *reinterpret_cast<const halfx8*>(p); };
    auto readKMajor = [&](const _Float16* p, int X) {
        return Join(LdsReadTr(p), LdsReadTr(p + 4 * X));
    };
    auto loadA = [&](int stage, int i) {
        if constexpr (TA)
            return readKMajor(AStage(stage) + aOff[i], kT);
        else
            return readKContig(AStage(stage) + aOff[0] + i * 16 * 64);
    };
    auto loadB = [&](int stage, int j) {
        if constexpr (TB)
            return readKContig(BStage(stage) + bOff[0] + j * 16 * 64);
        else
            return readKMajor(BStage(stage) + bOff[j], NT);
    };

    floatx4 acc[MB][4];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[i][j] = floatx4{ 0.f, 0.f, 0.f, 0.f };

#define SPH_FENCE() __builtin_amdgcn_sched_barrier(0)

    auto copyAllA = [&](uint32_t kt, int stage) {
        copyA(kt, stage, std::integral_constant<int, 0>{});
        copyA(kt, stage, std::integral_constant<int, 1>{});
    };
    auto copyAllB = [&](uint32_t kt, int stage) {
        copyB(kt, stage, std::integral_constant<int, 0>{});
        if constexpr (ROUNDS_B == 2)
            copyB(kt, stage, std::integral_constant<int, 1>{});
    };
#pragma unroll
    for (int st = 0; st < 3; ++st)
    {
        copyAllA(st, st);
        copyAllB(st, st);
    }
    copyAllA(3, 3);
    // stage 0 is followed by the copies of stages 1 and 2 and of A's stage 3
    WaitVmem<2 * COPIES_PER_STAGE + ROUNDS_A>();
    __syncthreads();

    halfx8 af[MB], bf0[4], bf1[4];
#pragma unroll
    for (int i = 0; i < MB / 2; ++i)
        af[i] = loadA(0, i);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        bf0[j] = loadB(0, j);

    // One K step, stage index known at compile time.  BF holds this step's B fragments, BFN
    // receives the next step's.  EXTRA = vector memory operations other than stage copies
    // issued since the first half of the step before.
    const uintx4 tailMask = TailMask(g, kTK - K % kTK);
    auto stepWith = [&](auto stageC, uint32_t kt, auto extraC, halfx8 (&BF)[4],
                        halfx8 (&BFN)[4], auto&& behindBarrier) {
        constexpr int cur = decltype(stageC)::value;
        constexpr int nxt = (cur + 1) % kTStages;
        constexpr int EXTRA = decltype(extraC)::value;
        const bool last = TAIL && kt == steps - 1;
        const uintx4 keep = last ? tailMask : uintx4{ ~0u, ~0u, ~0u, ~0u };
        auto mask = [&](halfx8& f) {
            if constexpr (TAIL)
                f = KeepNew(f, keep);
        };
#pragma unroll
        for (int j = 0; j < 4; ++j)
            mask(BF[j]);
        // first half: the upper half of the wavefront's row blocks, fetch this step's lower
        // half, request B of step kt+3
#pragma unroll
        for (int i = 0; i < MB / 2; ++i)
        {
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                if (j == 0)
                    mask(af[i]);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(BF[j], af[i], acc[i][j], 0, 0, 0);
                SPH_FENCE();
                if (i < MB / 4 && (j & 1) == 0)
                    af[MB / 2 + 2 * i + j / 2] = loadA(cur, MB / 2 + 2 * i + j / 2);
                SPH_FENCE();
            }
            if (i == 1)
                copyB(kt + 3, (cur + 3) % kTStages, std::integral_constant<int, 0>{});
            if constexpr (ROUNDS_B == 2)
            {
                if (i == 3)
                    copyB(kt + 3, (cur + 3) % kTStages, std::integral_constant<int, 1>{});
            }
            SPH_FENCE();
        }
        // step kt+1 has landed for every wavefront, and every wavefront is done reading
        // step kt, whose A buffer now takes step kt+4
        WaitVmem<2 * COPIES_PER_STAGE + EXTRA>();
        __syncthreads();
        behindBarrier();
        // second half: rows 64-127, fetch the next step's rows 0-63 and B, request A of kt+4
#pragma unroll
        for (int i = MB / 2; i < MB; ++i)
        {
            constexpr int kHalf = MB / 2;
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                if (j == 0)
                    mask(af[i]);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(BF[j], af[i], acc[i][j], 0, 0, 0);
                SPH_FENCE();
                // the next step's first MB / 2 fragments of A and its 4 of B, one per slot
                if ((j & 1) == 0)
                {
                    if (i - kHalf < MB / 4)
                        af[2 * (i - kHalf) + j / 2] = loadA(nxt, 2 * (i - kHalf) + j / 2);
                }
                else if (i - kHalf < 2)
                    BFN[2 * (i - kHalf) + j / 2] = loadB(nxt, 2 * (i - kHalf) + j / 2);
                SPH_FENCE();
            }
            if (i == (MB == 8 ? 5 : 2))
                copyA(kt + 4, cur, std::integral_constant<int, 0>{});
            if (i == (MB == 8 ? 7 : 3))
                copyA(kt + 4, cur, std::integral_constant<int, 1>{});
            SPH_FENCE();
        }
    };
    auto stepThen = [&](auto stageC, uint32_t kt, auto extraC, auto&& behindBarrier) {
        if constexpr (decltype(stageC)::value % 2 == 0)
            stepWith(stageC, kt, extraC, bf0, bf1, behindBarrier);
        else
            stepWith(stageC, kt, extraC, bf1, bf0, behindBarrier);
    };
    auto step = [&](auto stageC, uint32_t kt, auto extraC) { stepThen(stageC, kt, extraC, [] {}); };

    constexpr std::integral_constant<int, 0> kNoExtra{};
    if constexpr (CLOOP)
    {
        // Row block i of this wavefront (16 rows x 64 columns = 4 accumulator blocks): copy j
        // moves, per lane, the 4 floats of block (i, j) to mailbox + j*1024 + 16*l; the
        // instruction offset 64*j (added to both addresses) selects the block, so M0 takes it
        // off again.
        const uint32_t mail = LdsAddress(&CMail[0]) + waveU * 4096;
        const uint32_t cLane0 = ((waveM * WMROWS + l16) * ldc + waveN * 64 + 4 * g) * 4;
        const uint32_t cRowStep = 16 * ldc * 4;
        auto issueC = [&](auto bC) {
            constexpr int i = decltype(bC)::value;
            const uint32_t laneOff = cLane0 + i * cRowStep;
            DmaToLds16<0>(laneOff, out, mail);
            DmaToLds16<64>(laneOff, out, mail + 960);
            DmaToLds16<128>(laneOff, out, mail + 2 * 960);
            DmaToLds16<192>(laneOff, out, mail + 3 * 960);
        };
        auto addC = [&](auto bC) {
            constexpr int i = decltype(bC)::value;
            const float* box = &CMail[wave * 1024 + lane * 4];
            // two blocks at a time: the four reads at once would not fit the register budget
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const float4 c = *reinterpret_cast<const float4*>(box + j * 256);
                acc[i][j][0] += c.x;
                acc[i][j][1] += c.y;
                acc[i][j][2] += c.z;
                acc[i][j][3] += c.w;
                if (j == 1)
                    SPH_FENCE();
            }
        };
        // Step s = CSP*b requests row block b behind its barrier, where the copies issued
        // next are the ones needed last (three steps later); step s + CSP adds it at the same
        // place.  Vector memory operations complete in issue order, so a block that is late
        // holds back the stage copies behind it (spacing 4 measured 113.6 us on configuration
        // 3 against 115.3 us with spacing 2).  Ahead of the mid-step wait of step s lie the
        // stage copies counted there plus the 4 block copies of step s-1 or s-2, if one of them
        // requested a block; ahead of the wait for block b in step CSP*(b+1) lie the stage
        // copies of the CSP steps since its request.
        constexpr int kBlocks = MB;
        static_assert(CSP >= 2, "at most one request among two consecutive steps");
        auto requestsAt = [](int st) { return st >= 0 && st % CSP == 0 && st / CSP < kBlocks; };
        auto cStep = [&](auto stageC, auto sC) {
            constexpr int st = decltype(sC)::value;
            constexpr bool requests = st % CSP == 0 && st / CSP < kBlocks;
            constexpr bool adds = st % CSP == 0 && st >= CSP && st / CSP <= kBlocks;
            constexpr int extra = (requestsAt(st - 1) || requestsAt(st - 2)) ? 4 : 0;
            stepThen(stageC, static_cast<uint32_t>(st), std::integral_constant<int, extra>{}, [&] {
                if constexpr (adds)
                {
                    WaitVmem<CSP * COPIES_PER_STAGE>();
                    addC(std::integral_constant<int, adds ? st / CSP - 1 : 0>{});
                }
                if constexpr (requests)
                    issueC(std::integral_constant<int, requests ? st / CSP : 0>{});
            });
        };
        static_assert(CSP * COPIES_PER_STAGE <= 63, "vmcnt holds 6 bits");
        auto cRound = [&](auto rC) {
            constexpr int r = decltype(rC)::value;
            if constexpr (4 * r < kCLoopSteps)
            {
                cStep(std::integral_constant<int, 0>{}, std::integral_constant<int, 4 * r + 0>{});
                cStep(std::integral_constant<int, 1>{}, std::integral_constant<int, 4 * r + 1>{});
                cStep(std::integral_constant<int, 2>{}, std::integral_constant<int, 4 * r + 2>{});
                cStep(std::integral_constant<int, 3>{}, std::integral_constant<int, 4 * r + 3>{});
            }
        };
        static_assert(kCLoopSteps <= 4 * 9, "rounds written out below");
        cRound(std::integral_constant<int, 0>{});
        cRound(std::integral_constant<int, 1>{});
        cRound(std::integral_constant<int, 2>{});
        cRound(std::integral_constant<int, 3>{});
        cRound(std::integral_constant<int, 4>{});
        cRound(std::integral_constant<int, 5>{});
        cRound(std::integral_constant<int, 6>{});
        cRound(std::integral_constant<int, 7>{});
        cRound(std::integral_constant<int, 8>{});
    }
    auto regularSteps = [&](uint32_t first) {
        for (uint32_t kt = first;; kt += 4)
        {
            step(std::integral_constant<int, 0>{}, kt, kNoExtra);
            if (kt + 1 >= steps)
                break;
            step(std::integral_constant<int, 1>{}, kt + 1, kNoExtra);
            if (kt + 2 >= steps)
                break;
            step(std::integral_constant<int, 2>{}, kt + 2, kNoExtra);
            if (kt + 3 >= steps)
                break;
            step(std::integral_constant<int, 3>{}, kt + 3, kNoExtra);
            if (kt + 4 >= steps)
                break;
        }
    };
    if constexpr (CLOOP)
    {
        if (steps > kCLoopSteps)
            regularSteps(kCLoopSteps);
    }
    else
        regularSteps(0);
#undef SPH_FENCE

    // ---- epilogue ---------------------------------------------------------------
    WaitVmem<0>();      // clamped copies of the last steps still target LDS
    __syncthreads();    // ... and every wavefront is done with the stage buffers
    {
        // 64 rows x 64 floats per wavefront, 16-byte chunks XOR-swizzled with row % 16 so
        // that neither the column-wise writes nor the row-wise reads pile up on one bank
        float* stage = reinterpret_cast<float*>(LdsRaw) + wave * (64 * 64);
        const uint32_t rdRow = lane >> 4;        // + 4*t
        const uint32_t rdChunk = lane & 15;
        float* outBlock =
            out + static_cast<size_t>(waveM * WMROWS + rdRow) * ldc + waveN * 64 + rdChunk * 4;
        const size_t rowStep = static_cast<size_t>(4) * ldc;
        const uint32_t rowFirst = waveM * WMROWS + rdRow;
        const bool colExists = !RAGGED || waveN * 64 + rdChunk * 4 < colsLeft;
        auto exists = [&](int half, int t) {
            return !RAGGED || (colExists && rowFirst + 4 * (half * 16 + t) < rowsLeft);
        };
        auto stageHalf = [&](int half) {
#pragma unroll
            for (int ii = 0; ii < 4; ++ii)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const int i = half * 4 + ii;
                    const uint32_t row = ii * 16 + l16;
                    const uint32_t chunk = (j * 4 + g) ^ (row & 15);
                    *reinterpret_cast<float4*>(&stage[row * 64 + chunk * 4]) =
                        make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        };
        auto loadOld = [&](int half, float4 (&old)[16]) {
#pragma unroll
            for (int t = 0; t < 16; ++t)
            {
                old[t] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (exists(half, t))
                    old[t] = NtLoad4(outBlock + (half * 16 + t) * rowStep);
            }
        };
        auto storeHalf = [&](int half, const float4 (&old)[16], auto accumulate) {
#pragma unroll
            for (int t = 0; t < 16; ++t)
            {
                const uint32_t r = rdRow + 4 * t;
                float4 v = *reinterpret_cast<const float4*>(
                    &stage[r * 64 + ((rdChunk ^ (r & 15)) * 4)]);
                if constexpr (decltype(accumulate)::value)
                {
                    v.x += old[t].x;
                    v.y += old[t].y;
                    v.z += old[t].z;
                    v.w += old[t].w;
                }
                if (exists(half, t))
                    Store4(outBlock + (half * 16 + t) * rowStep, v);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        };

        float4 old[16];
        // (64 rows at a time: twice for a wavefront part of 128 rows)
        if (CLOOP || args.overwrite)
        {
            stageHalf(0);
            storeHalf(0, old, std::false_type{});
            if constexpr (MB == 8)
            {
                stageHalf(1);
                storeHalf(1, old, std::false_type{});
            }
        }
        else
        {
            loadOld(0, old);
            stageHalf(0);
            storeHalf(0, old, std::true_type{});
            if constexpr (MB == 8)
            {
                loadOld(1, old);
                stageHalf(1);
                storeHalf(1, old, std::true_type{});
            }
        }
    }
}

// ---------------------------------------------------------------------------
// 128 x 128 x 32 kernel with straight-to-LDS copies, ragged M and N
// ---------------------------------------------------------------------------
// For shapes the 256-tile kernel does not take (M or N not a multiple of 256) as long as K is a
// multiple of 32 (or any K from 64 up) and N of 8.  Four wavefronts (2 x 2, each 64 x 64 = 2 x 2 MFMA blocks) or eight (2 x 4, each
// 64 x 32), four LDS stages of 16 KiB (two workgroups per compute unit), copies issued two steps
// ahead, one barrier per step (placed, with the copies, between the MFMAs of the step's first
// half), fragments read half a step ahead.
// A stage: 128 rows of 64 bytes, 16-byte chunk c of row x at position c ^ ((x >> 2) & 3).
// B stage: 32 k-rows of 256 bytes, 32-byte chunks XOR-swizzled with 2*(k%4), read with the
// transposing LDS load like the 256-tile kernel.  Rows past M and columns past N are clamped to
// the last valid ones: they only feed outputs that are not stored.
// TA (A stored K x M) / TB (B stored N x K): an operand stored the other way round simply takes
// the other operand's stage layout and fragment read -- an A stored k-major is copied and read
// like B, a B stored with K contiguous like A -- so the MFMAs and their order do not change.
constexpr int kD = 128;
constexpr int kDStages = 4;
constexpr int kDStageBytes = 2 * kD * kTK * 2;  // A + B

// TAIL: K = 32 q + r, 0 < r < 32: a last step over the window [K - 32, K) whose slab has the
// positions of the 32 - r values of k already multiplied cleared in LDS.
template <bool TA, bool TB, bool TAIL, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void GemmF16Dma128(const GemmF16Args args,
                                                            const GemmF16Strips strips)
{
    static_assert(WAVES == 4 || WAVES == 8, "2 x 2 or 2 x 4 wavefronts");
    constexpr int WN = WAVES / 2;          // wavefronts across the tile
    constexpr int TN = 2 / (WN / 2);       // 32-column blocks per wavefront: 2 or 1
    constexpr int kCopiesPer = 8 / WAVES;  // 1 KiB copies per operand, step and wavefront
    constexpr int kDCopies = 2 * kCopiesPer;
    __shared__ __attribute__((aligned(1024))) char lds[kDStages * kDStageBytes];
    constexpr uint32_t kBytesA = kD * kTK * 2;  // 8 KiB

    uint32_t unit, tm, tn;
    const uint32_t block = blockIdx.x;
    if (RunStrip<TA, TB, WAVES>(strips, block, reinterpret_cast<float*>(lds)))
        return;
    if (!MapTile(block, args.tilesM, args.tilesN, args.totalTiles, unit, tm, tn))
        return;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t waveM = wave / WN;
    const uint32_t waveN = wave % WN;
    const uint32_t M = args.M, N = args.N, K = args.K;

    const _Float16* A = args.A + args.strideA * static_cast<int64_t>(unit);
    const _Float16* B = args.B + args.strideB * static_cast<int64_t>(unit);
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit);
    const uint32_t rowBase = tm * kD;
    const uint32_t colBase = tn * kD;

    // ---- copy plan: copy j of an operand (j = wave, wave + 4) ---------------------------
    // K-contiguous operand (x = row of A / column of a transposed B, `pitch` halves apart):
    // 16 x per copy; lane -> x = j*16 + lane/4, physical chunk lane%4.
    auto laneKContig = [&](uint32_t j, uint32_t xBase, uint32_t limit, uint32_t pitch) {
        const uint32_t x = j * 16 + (lane >> 2);
        const uint32_t c = (lane & 3) ^ ((lane >> 4) & 3);  // (x >> 2) & 3 == (lane >> 4) & 3
        const uint32_t gx = min(xBase + x, limit - 1);
        return (gx * pitch + c * 8) * 2u;
    };
    // k-major operand (x = column of B / row of a transposed A, rows `pitch` halves apart):
    // 4 k-rows per copy; lane -> k = j*4 + lane/16, physical 16-byte chunk lane%16.
    auto laneKMajor = [&](uint32_t j, uint32_t xBase, uint32_t limit, uint32_t pitch) {
        const uint32_t k = j * 4 + (lane >> 4);
        const uint32_t phys16 = lane & 15;
        const uint32_t logical16 = (((phys16 >> 1) ^ (2 * (k & 3))) << 1) | (phys16 & 1);
        const uint32_t gx = min(xBase + logical16 * 8, limit - 8);
        return (k * pitch + gx) * 2u;
    };
    uint32_t aLane[kCopiesPer], bLane[kCopiesPer], aDst[kCopiesPer], bDst[kCopiesPer];
#pragma unroll
    for (uint32_t i = 0; i < kCopiesPer; ++i)
    {
        const uint32_t j = wave + WAVES * i;
        aLane[i] = TA ? laneKMajor(j, rowBase, M, args.lda) : laneKContig(j, rowBase, M, args.lda);
        bLane[i] = TB ? laneKContig(j, colBase, N, K) : laneKMajor(j, colBase, N, args.ldb);
        aDst[i] = j * 1024;
        bDst[i] = kBytesA + j * 1024;
    }
    const size_t aStepBytes = TA ? static_cast<size_t>(kTK) * args.lda * 2 : kTK * 2;
    const size_t bStepBytes = TB ? kTK * 2 : static_cast<size_t>(kTK) * args.ldb * 2;
    const uint32_t ldsBase = LdsAddress(lds);
    const uint32_t steps = TAIL ? K / kTK + 1 : K / kTK;
    // the last window starts K % 32 values of k after the one before it
    const uint32_t kLast = K % kTK;
    const size_t aLastBytes = TA ? static_cast<size_t>(kLast) * args.lda * 2 : kLast * 2;
    const size_t bLastBytes = TB ? kLast * 2 : static_cast<size_t>(kLast) * args.ldb * 2;
    // Copy n (0..3: two of A, two of B) of the next step to fetch, into stage `stage`.  aSrc /
    // bSrc point at that step's slabs; surplus steps re-fetch the last one into a stage nobody
    // reads any more, which keeps the number of outstanding copies the same in every iteration.
    const char* aSrc = reinterpret_cast<const char*>(A);
    const char* bSrc = reinterpret_cast<const char*>(B);
    uint32_t stepsToAdvance = steps - 1;
    auto issueOne = [&](uint32_t stage, uint32_t n) {
        const uint32_t base = ldsBase + stage * kDStageBytes;
        if (n < kCopiesPer)
            DmaToLds16<0>(aLane[n], aSrc, base + aDst[n]);
        else
            DmaToLds16<0>(bLane[n - kCopiesPer], bSrc, base + bDst[n - kCopiesPer]);
    };
    auto advance = [&]() {
        if (stepsToAdvance != 0)
        {
            size_t aBytes = aStepBytes, bBytes = bStepBytes;
            if (TAIL && stepsToAdvance == 1)
            {
                aBytes = aLastBytes;
                bBytes = bLastBytes;
            }
            aSrc += aBytes;
            bSrc += bBytes;
            --stepsToAdvance;
        }
    };

    // ---- fragment plan ----------------------------------------------------------------
    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;
    const uint32_t g = lane >> 4;
    const uint32_t s = lane & 15;
    // bytes inside an operand's part of a stage, [ks][block]
    auto offKContig = [&](int ks, uint32_t x) {
        return x * 64 + (((ks * 2 + khalf) ^ ((x >> 2) & 3)) << 4);
    };
    auto offKMajor = [&](int ks, uint32_t chunkBase) {
        const uint32_t k = ks * 16 + 8 * (g >> 1) + (s >> 2);  // + 4 for the second read
        const uint32_t chunk32 = (chunkBase + (g & 1)) ^ (2 * ((s >> 2) & 3));
        return k * 256 + chunk32 * 32 + (s & 3) * 8;
    };
    // a wavefront owns rows waveM*64 .. +63 (two blocks) and columns waveN*32*TN .. (TN blocks)
    uint32_t aOff[2][2], bOff[2][TN];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
    {
#pragma unroll
        for (int b = 0; b < 2; ++b)
            aOff[ks][b] = TA ? offKMajor(ks, waveM * 4 + b * 2)
                             : offKContig(ks, waveM * 64 + b * 32 + l32);
#pragma unroll
        for (int b = 0; b < TN; ++b)
            bOff[ks][b] = kBytesA + (TB ? offKContig(ks, (waveN * TN + b) * 32 + l32)
                                        : offKMajor(ks, (waveN * TN + b) * 2));
    }
    auto readKContig = [&](const char* p) { return *reinterpret_cast<const halfx8*>(p); };
    auto readKMajor = [&](const char* p) {
        const _Float16* h = reinterpret_cast<const _Float16*>(p);
        return Join(LdsReadTr(h), LdsReadTr(h + 4 * 128));
    };
    auto loadFragments = [&](halfx8 (&af)[2], halfx8 (&bf)[TN], const char* stage, int ks) {
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
            if constexpr (TA)
                af[b] = readKMajor(stage + aOff[ks][b]);
            else
                af[b] = readKContig(stage + aOff[ks][b]);
        }
#pragma unroll
        for (int b = 0; b < TN; ++b)
        {
            if constexpr (TB)
                bf[b] = readKContig(stage + bOff[ks][b]);
            else
                bf[b] = readKMajor(stage + bOff[ks][b]);
        }
    };

    floatx16 acc[2][TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[i][j][v] = 0.f;
    // TAIL: the positions of the last slab whose k the step before has multiplied are cleared
    // in LDS, by the lane that copied them, once the copies have landed and before the barrier
    // that publishes the stage, so the steps themselves carry no masks (1024 x 1024 x 784:
    // 13.6 -> 11.4 us against masks on the fragments of every step; the 256-tile kernel keeps
    // those, it has no registers to spare for this and measured 134 -> 143 us).
    auto clearRepeated = [&](char* stage) {
        const uint32_t repeated = kTK - K % kTK;
        const uint32_t c = (lane & 3) ^ ((lane >> 4) & 3);  // chunk of a K-contiguous row
        const uintx4 contig = TailMask(c, repeated);
#pragma unroll
        for (uint32_t i = 0; i < kCopiesPer; ++i)
        {
            const uint32_t j = wave + WAVES * i;
            const uint32_t k = j * 4 + (lane >> 4);  // row of a k-major slab
            const uint32_t keepAll = k < repeated ? 0u : ~0u;
            const uintx4 major = { keepAll, keepAll, keepAll, keepAll };
            uintx4* a = reinterpret_cast<uintx4*>(stage + j * 1024 + lane * 16);
            uintx4* b = reinterpret_cast<uintx4*>(stage + kBytesA + j * 1024 + lane * 16);
            *a = *a & (TA ? major : contig);
            *b = *b & (TB ? contig : major);
        }
    };
    auto multiply = [&](const halfx8 (&af)[2], const halfx8 (&bf)[TN]) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] =
                    __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
    };

    // First half of a step.  The step's housekeeping sits between its MFMAs, where the matrix
    // pipe is already busy: behind the first one the wait for the copies of step st+1 and the
    // barrier, behind every one a copy of step st+3.
    static_assert(kDCopies == 2 * TN, "one copy behind every MFMA of the first half");
    auto multiplyAndFeed = [&](const halfx8 (&af)[2], const halfx8 (&bf)[TN], uint32_t fillStage,
                               bool nextIsLast, char* next) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
            {
                acc[i][j] =
                    __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
                if (i == 0 && j == 0)
                {
                    // steps up to st+1 have landed once at most one later step is pending;
                    // behind the barrier everybody's copies are visible and everybody has
                    // read the last fragment of step st-1
                    WaitVmem<(kDStages - 3) * kDCopies>();
                    if constexpr (TAIL)
                    {
                        if (nextIsLast)
                        {
                            clearRepeated(next);
                            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        }
                    }
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                }
                issueOne(fillStage, i * TN + j);
                if (i == 1 && j == TN - 1)
                    advance();
                __builtin_amdgcn_sched_barrier(0);
            }
    };

#pragma unroll
    for (uint32_t p = 0; p < kDStages - 1; ++p)
    {
#pragma unroll
        for (uint32_t n = 0; n < kDCopies; ++n)
            issueOne(p, n);
        advance();
    }
    halfx8 af[2][2], bf[2][TN];
    WaitVmem<(kDStages - 2) * kDCopies>();
    __syncthreads();
    loadFragments(af[0], bf[0], lds, 0);

    // Fragments are read half a step ahead of their MFMAs; stage st+1 is known to be complete
    // from the barrier inside the first half of step st.  The loop is unrolled over the ring
    // so that every stage offset is a constant.
    for (uint32_t s0 = 0; s0 < steps; s0 += kDStages)
    {
#pragma unroll
        for (uint32_t u = 0; u < kDStages; ++u)
        {
            if (s0 + u >= steps)
                break;
            const char* cur = lds + u * kDStageBytes;
            char* next = lds + ((u + 1) % kDStages) * kDStageBytes;
            loadFragments(af[1], bf[1], cur, 1);
            __builtin_amdgcn_sched_barrier(0);
            multiplyAndFeed(af[0], bf[0], (u + kDStages - 1) % kDStages,
                            TAIL && s0 + u + 2 == steps, next);
            __builtin_amdgcn_sched_barrier(0);
            loadFragments(af[0], bf[0], next, 0);
            __builtin_amdgcn_sched_barrier(0);
            multiply(af[1], bf[1]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    WaitVmem<0>();  // the surplus copies of the last steps still target LDS

    // ---- epilogue: lane holds row l%32 of a block, columns 8q + 4*(l/32) + 0..3 -----------
    const bool accumulate = args.overwrite == 0;
    float4 old[8 * TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t r = rowBase + waveM * 64 + i * 32 + l32;
                const uint32_t c = colBase + (waveN * TN + j) * 32 + 8 * q + 4 * khalf;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (accumulate && r < M && c < N)  // N % 8 == 0: whole quads only
                    v = Load4(out + static_cast<size_t>(r) * args.ldc + c);
                old[(i * TN + j) * 4 + q] = v;
            }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t r = rowBase + waveM * 64 + i * 32 + l32;
                const uint32_t c = colBase + (waveN * TN + j) * 32 + 8 * q + 4 * khalf;
                if (r < M && c < N)
                {
                    float4 v = old[(i * TN + j) * 4 + q];
                    v.x += acc[i][j][4 * q + 0];
                    v.y += acc[i][j][4 * q + 1];
                    v.z += acc[i][j][4 * q + 2];
                    v.w += acc[i][j][4 * q + 3];
                    Store4(out + static_cast<size_t>(r) * args.ldc + c, v);
                }
            }
}

// ---------------------------------------------------------------------------
// 64 x 64 x 64 kernel with straight-to-LDS copies, ragged M and N
// ---------------------------------------------------------------------------
// For products with at most half as many 128 x 128 tiles as compute units.  The tiled kernels
// are bound by what a compute unit's LDS moves per K step (the copies' writes plus the fragment
// reads), so a product that gives only a quarter of the compute units a 128-tile uses a quarter
// of the chip's LDS bandwidth; 64 x 64 tiles move half as many more bytes through LDS per flop
// but spread them over four times as many compute units (1024^3: 10.8 us on 64 tiles of 128).
// Four wavefronts (2 x 2), one 32 x 32 block of v_mfma_f32_32x32x16_f16 each; K advances 64 at
// a time, so that a row of a K-contiguous operand is one whole 128-byte line per step; four
// stages of 16 KiB, so two workgroups share a compute unit.
// K-contiguous operand (A as given, B stored N x K): 64 rows of 128 bytes, 16-byte chunk c of
// row x at position c ^ ((x >> 1) & 7): 16 consecutive rows reading one chunk touch every bank
// once.  k-major operand (B as given, A stored K x M): 64 k-rows of 128 bytes, the two 64-byte
// halves of k-row k swapped when (k >> 1) & 1, so that the four k-rows a transposing read
// serves in one clock (64 bytes each) cover the 64 banks.
// TAIL: K = 64 q + r, 0 < r < 64, K >= 64: a last step over the window [K - 64, K) whose slab has
// the positions of the 64 - r values of k already multiplied cleared in LDS.
constexpr int kS = 64;         // tile edge
constexpr int kSK = 64;        // K step
constexpr int kSStages = 4;
constexpr int kSOperandBytes = kS * kSK * 2;        // 8 KiB
constexpr int kSStageBytes = 2 * kSOperandBytes;    // A + B

template <bool TA, bool TB, bool TAIL>
__global__ __launch_bounds__(256) void GemmF16Dma64(const GemmF16Args args,
                                                    const GemmF16Strips strips)
{
    constexpr int kCopiesPer = 2;            // 1 KiB copies per operand, step and wavefront
    constexpr int kCopies = 2 * kCopiesPer;  // per step and wavefront
    __shared__ __attribute__((aligned(1024))) char lds[kSStages * kSStageBytes];

    uint32_t unit, tm, tn;
    const uint32_t block = blockIdx.x;
    if (RunStrip<TA, TB, 4>(strips, block, reinterpret_cast<float*>(lds)))
        return;
    if (!MapTile(block, args.tilesM, args.tilesN, args.totalTiles, unit, tm, tn))
        return;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t waveM = wave >> 1;
    const uint32_t waveN = wave & 1;
    const uint32_t M = args.M, N = args.N, K = args.K;

    const _Float16* A = args.A + args.strideA * static_cast<int64_t>(unit);
    const _Float16* B = args.B + args.strideB * static_cast<int64_t>(unit);
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit);
    const uint32_t rowBase = tm * kS;
    const uint32_t colBase = tn * kS;

    // ---- copy plan: copy j of an operand (j = wave, wave + 4) covers LDS bytes j*1024 .. -----
    // K-contiguous: 8 rows per copy; lane -> x = 8 j + lane / 8, physical chunk lane % 8.
    auto laneKContig = [&](uint32_t j, uint32_t xBase, uint32_t limit, uint32_t pitch) {
        const uint32_t x = j * 8 + (lane >> 3);
        const uint32_t c = (lane & 7) ^ ((x >> 1) & 7);
        const uint32_t gx = min(xBase + x, limit - 1);
        return (gx * pitch + c * 8) * 2u;
    };
    // k-major: 8 k-rows per copy; lane -> k = 8 j + lane / 8, physical 16-byte chunk lane % 8 of
    // which bit 2 (the 64-byte half) is swapped for k-rows with (k >> 1) & 1.
    auto laneKMajor = [&](uint32_t j, uint32_t xBase, uint32_t limit, uint32_t pitch) {
        const uint32_t k = j * 8 + (lane >> 3);
        const uint32_t logical16 = (lane & 7) ^ (((k >> 1) & 1) << 2);
        const uint32_t gx = min(xBase + logical16 * 8, limit - 8);
        return (k * pitch + gx) * 2u;
    };
    const uint32_t pitchB = TB ? K : args.ldb;
    uint32_t aLane[kCopiesPer], bLane[kCopiesPer], aDst[kCopiesPer], bDst[kCopiesPer];
#pragma unroll
    for (uint32_t i = 0; i < kCopiesPer; ++i)
    {
        const uint32_t j = wave + 4 * i;
        aLane[i] = TA ? laneKMajor(j, rowBase, M, args.lda) : laneKContig(j, rowBase, M, args.lda);
        bLane[i] = TB ? laneKContig(j, colBase, N, pitchB) : laneKMajor(j, colBase, N, pitchB);
        aDst[i] = j * 1024;
        bDst[i] = kSOperandBytes + j * 1024;
    }
    const size_t aStepBytes = TA ? static_cast<size_t>(kSK) * args.lda * 2 : kSK * 2;
    const size_t bStepBytes = TB ? kSK * 2 : static_cast<size_t>(kSK) * pitchB * 2;
    const uint32_t ldsBase = LdsAddress(lds);
    const uint32_t steps = TAIL ? K / kSK + 1 : K / kSK;
    // the last window starts K % 64 values of k after the one before it
    const uint32_t kLast = K % kSK;
    const size_t aLastBytes = TA ? static_cast<size_t>(kLast) * args.lda * 2 : kLast * 2;
    const size_t bLastBytes = TB ? kLast * 2 : static_cast<size_t>(kLast) * pitchB * 2;
    // Copy n (0, 1: A; 2, 3: B) of the next step to fetch, into stage `stage`.  Surplus steps
    // re-fetch the last slab into a stage nobody reads any more, which keeps the number of
    // outstanding copies the same in every step.
    const char* aSrc = reinterpret_cast<const char*>(A);
    const char* bSrc = reinterpret_cast<const char*>(B);
    uint32_t stepsToAdvance = steps - 1;
    auto issueOne = [&](uint32_t stage, uint32_t n) {
        const uint32_t base = ldsBase + stage * kSStageBytes;
        if (n < kCopiesPer)
            DmaToLds16<0>(aLane[n], aSrc, base + aDst[n]);
        else
            DmaToLds16<0>(bLane[n - kCopiesPer], bSrc, base + bDst[n - kCopiesPer]);
    };
    auto advance = [&]() {
        if (stepsToAdvance != 0)
        {
            size_t aBytes = aStepBytes, bBytes = bStepBytes;
            if (TAIL && stepsToAdvance == 1)
            {
                aBytes = aLastBytes;
                bBytes = bLastBytes;
            }
            aSrc += aBytes;
            bSrc += bBytes;
            --stepsToAdvance;
        }
    };

    // ---- fragment plan: ks = 0..3, k = 16 ks + 8 khalf .. + 7 ---------------------------------
    const uint32_t l32 = lane & 31;
    const uint32_t khalf = lane >> 5;
    const uint32_t g = lane >> 4;
    const uint32_t s = lane & 15;
    auto offKContig = [&](int ks, uint32_t x) {
        return x * 128 + (((ks * 2 + khalf) ^ ((x >> 1) & 7)) << 4);
    };
    // 32 columns (or rows of a transposed A) from `half` * 32 on: lanes of g & 1 take the
    // second 16 of them; the second read of a fragment is 4 k-rows further on
    auto offKMajor = [&](int ks, uint32_t half) {
        const uint32_t k = ks * 16 + 8 * (g >> 1) + (s >> 2);
        return k * 128 + ((half ^ ((k >> 1) & 1)) << 6) + ((g & 1) << 5) + (s & 3) * 8;
    };
    uint32_t aOff[4], bOff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
    {
        aOff[ks] = TA ? offKMajor(ks, waveM) : offKContig(ks, waveM * 32 + l32);
        bOff[ks] = kSOperandBytes + (TB ? offKContig(ks, waveN * 32 + l32) : offKMajor(ks, waveN));
    }
    auto readKContig = [&](const char* p) { return *reinterpret_cast<const halfx8*>(p); };
    auto readKMajor = [&](const char* p) {
        // the second read takes the k-rows 4 further on, whose halves are swapped alike
        const _Float16* h = reinterpret_cast<const _Float16*>(p);
        return Join(LdsReadTr(h), LdsReadTr(h + 4 * 64));
    };
    auto loadA = [&](const char* stage, int ks) {
        if constexpr (TA)
            return readKMajor(stage + aOff[ks]);
        else
            return readKContig(stage + aOff[ks]);
    };
    auto loadB = [&](const char* stage, int ks) {
        if constexpr (TB)
            return readKContig(stage + bOff[ks]);
        else
            return readKMajor(stage + bOff[ks]);
    };

    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v)
        acc[v] = 0.f;

    // TAIL: the positions of the last slab whose k the step before has multiplied are cleared
    // in LDS, by the lane that copied them, once the copies have landed and before the barrier
    // that publishes the stage.
    auto clearRepeated = [&](char* stage) {
        const uint32_t repeated = kSK - K % kSK;
#pragma unroll
        for (uint32_t i = 0; i < kCopiesPer; ++i)
        {
            const uint32_t j = wave + 4 * i;
            const uint32_t row = j * 8 + (lane >> 3);  // x of a K-contiguous slab, k of a k-major one
            const uint32_t c = (lane & 7) ^ ((row >> 1) & 7);
            const uintx4 contig = TailMask(c, repeated);
            const uint32_t keepAll = row < repeated ? 0u : ~0u;
            const uintx4 major = { keepAll, keepAll, keepAll, keepAll };
            uintx4* a = reinterpret_cast<uintx4*>(stage + j * 1024 + lane * 16);
            uintx4* b = reinterpret_cast<uintx4*>(stage + kSOperandBytes + j * 1024 + lane * 16);
            *a = *a & (TA ? major : contig);
            *b = *b & (TB ? contig : major);
        }
    };

#pragma unroll
    for (uint32_t p = 0; p < kSStages - 1; ++p)
    {
#pragma unroll
        for (uint32_t n = 0; n < kCopies; ++n)
            issueOne(p, n);
        advance();
    }
    halfx8 af[2][4], bf[2][4];
    WaitVmem<(kSStages - 2) * kCopies>();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
    {
        af[0][ks] = loadA(lds, ks);
        bf[0][ks] = loadB(lds, ks);
    }

    // One step with the stage known at compile time: the fragments of step st are in set P;
    // behind the first matrix instruction the wait for the copies of step st + 1 and the
    // barrier, behind each one a copy of step st + 3; the fragments of step st + 1 are read
    // into set Q from the stage the barrier has just published.
    auto step = [&](auto uC, uint32_t st, halfx8 (&PA)[4], halfx8 (&PB)[4], halfx8 (&QA)[4],
                    halfx8 (&QB)[4]) {
        constexpr uint32_t u = decltype(uC)::value;
        char* next = lds + ((u + 1) % kSStages) * kSStageBytes;
        const uint32_t fill = (u + kSStages - 1) % kSStages;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
        {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(PB[ks], PA[ks], acc, 0, 0, 0);
            if (ks == 0)
            {
                WaitVmem<(kSStages - 3) * kCopies>();
                if constexpr (TAIL)
                {
                    if (st + 2 == steps)
                    {
                        clearRepeated(next);
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    }
                }
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
            issueOne(fill, ks);
            if (ks == 3)
                advance();
            __builtin_amdgcn_sched_barrier(0);
            QA[ks] = loadA(next, ks);
            QB[ks] = loadB(next, ks);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (uint32_t s0 = 0; s0 < steps; s0 += kSStages)
    {
        step(std::integral_constant<uint32_t, 0>{}, s0, af[0], bf[0], af[1], bf[1]);
        if (s0 + 1 >= steps)
            break;
        step(std::integral_constant<uint32_t, 1>{}, s0 + 1, af[1], bf[1], af[0], bf[0]);
        if (s0 + 2 >= steps)
            break;
        step(std::integral_constant<uint32_t, 2>{}, s0 + 2, af[0], bf[0], af[1], bf[1]);
        if (s0 + 3 >= steps)
            break;
        step(std::integral_constant<uint32_t, 3>{}, s0 + 3, af[1], bf[1], af[0], bf[0]);
    }
    WaitVmem<0>();  // the surplus copies of the last steps still target LDS

    // ---- epilogue: lane holds row l % 32 of its block, columns 8 q + 4 (l / 32) + 0..3 ----------
    const bool accumulate = args.overwrite == 0;
    const uint32_t r = rowBase + waveM * 32 + l32;
    float4 old[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
    {
        const uint32_t c = colBase + waveN * 32 + 8 * q + 4 * khalf;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (accumulate && r < M && c < N)  // N % 8 == 0: whole quads only
            v = Load4(out + static_cast<size_t>(r) * args.ldc + c);
        old[q] = v;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
    {
        const uint32_t c = colBase + waveN * 32 + 8 * q + 4 * khalf;
        if (r < M && c < N)
        {
            float4 v = old[q];
            v.x += acc[4 * q + 0];
            v.y += acc[4 * q + 1];
            v.z += acc[4 * q + 2];
            v.w += acc[4 * q + 3];
            Store4(out + static_cast<size_t>(r) * args.ldc + c, v);
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

// VEC = 8: K, the row strides, N and the bases are all multiples of 8 halves, so every 8-half
// piece is 16-byte aligned and lies wholly inside or outside its row.  VEC = 2: multiples of 2
// halves, VEC = 1: anything; a piece that lies inside its row is still read 16 bytes at a time
// (one load from a 4-byte-aligned address, or aligned dwords that are shifted, see Halves8),
// one that straddles the row's end half by half.
// TA: A is stored K x M; TB: B is stored N x K.  A transposed operand is read along its
// contiguous dimension like the other one and turned round on its way into LDS (8 two-byte
// stores per chunk instead of one 16-byte store), so the MFMA side does not change.
template <int VEC, bool TA, bool TB>
__global__ __launch_bounds__(kGThreads) void GemmF16General(const GemmF16Args args,
                                                            const GemmF16Strips strips)
{
    __shared__ __attribute__((aligned(16))) _Float16 As[2][kG * kGLda];
    __shared__ __attribute__((aligned(16))) _Float16 Bs[2][kGK * kGLdb];

    uint32_t unit, tm, tn;
    const uint32_t block = blockIdx.x;
    if (RunStrip<TA, TB, 4>(strips, block, reinterpret_cast<float*>(&As[0][0])))
        return;
    if (!MapTile(block, args.tilesM, args.tilesN, args.totalTiles, unit, tm, tn))
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

    // 8 consecutive halves starting at p, of which those with index + first < limit exist
    auto load8 = [&](const _Float16* p, uint32_t first, uint32_t limit) {
        halfx8 v = { 0, 0, 0, 0, 0, 0, 0, 0 };
        if constexpr (VEC == 8)
        {
            if (first < limit)
                v = *reinterpret_cast<const halfx8*>(p);
        }
        else
        {
            if (first + 8 <= limit)
            {
                if constexpr (VEC >= 2)
                    v = *reinterpret_cast<const halfx8a4*>(p);
                else
                    v = Halves8::Load(p).Get(Halves8::Shift(p));
            }
            else
            {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (first + e < limit)
                        v[e] = p[e];
            }
        }
        return v;
    };
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            halfx8 v = { 0, 0, 0, 0, 0, 0, 0, 0 };
            if constexpr (TA)
            {
                // 8 consecutive rows m of one k
                const uint32_t gk = k0 + q / 16;
                const uint32_t gr = rowBase + (q % 16) * 8;
                if (gk < K)
                    v = load8(A + static_cast<size_t>(gk) * args.lda + gr, gr, M);
            }
            else
            {
                const uint32_t gr = rowBase + q / 4;
                const uint32_t gk = k0 + (q % 4) * 8;
                if (gr < M)
                    v = load8(A + static_cast<size_t>(gr) * args.lda + gk, gk, K);
            }
            stageA[i] = v;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            halfx8 v = { 0, 0, 0, 0, 0, 0, 0, 0 };
            if constexpr (TB)
            {
                // 8 consecutive k of one column n
                const uint32_t gc = colBase + q / 4;
                const uint32_t gk = k0 + (q % 4) * 8;
                if (gc < N)
                    v = load8(B + static_cast<size_t>(gc) * K + gk, gk, K);
            }
            else
            {
                const uint32_t gk = k0 + q / 16;
                const uint32_t gc = colBase + (q % 16) * 8;
                if (gk < K)
                    v = load8(B + static_cast<size_t>(gk) * args.ldb + gc, gc, N);
            }
            stageB[i] = v;
        }
    };

    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            if constexpr (TA)
            {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    As[buf][((q % 16) * 8 + e) * kGLda + q / 16] = stageA[i][e];
            }
            else
                *reinterpret_cast<halfx8*>(&As[buf][(q / 4) * kGLda + (q % 4) * 8]) = stageA[i];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
        {
            const uint32_t q = tid + i * kGThreads;
            if constexpr (TB)
            {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    Bs[buf][((q % 4) * 8 + e) * kGLdb + q / 4] = stageB[i][e];
            }
            else
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
                float* p = out + static_cast<size_t>(r) * args.ldc + c;
                if (args.outVec)
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

// variant 0: whole tiles, out read in the epilogue; 1 / 2: out added inside the loop with
// spacing 2 / 4; 3: ragged tiles
template <bool TA, bool TB, bool TAIL, int NT>
void LaunchTile256(int variant, uint32_t grid, hipStream_t stream, const GemmF16Args& args,
                   const GemmF16Strips& strips)
{
    const dim3 g(grid), b(512);
    if (variant == 2)
        hipLaunchKernelGGL((GemmF16Tile256<false, 4, TA, TB, TAIL, NT>), g, b, 0, stream, args, strips);
    else if (variant == 1)
        hipLaunchKernelGGL((GemmF16Tile256<false, 2, TA, TB, TAIL, NT>), g, b, 0, stream, args, strips);
    else if (variant == 0)
        hipLaunchKernelGGL((GemmF16Tile256<false, 0, TA, TB, TAIL, NT>), g, b, 0, stream, args, strips);
    else
        hipLaunchKernelGGL((GemmF16Tile256<true, 0, TA, TB, TAIL, NT>), g, b, 0, stream, args, strips);
}

// ---------------------------------------------------------------------------
// Few output tiles: one 32 x 32 (v_mfma_f32_32x32x16_f16) or 16 x 16 (16x16x32) tile per
// workgroup, K split across its WAVES wavefronts
// ---------------------------------------------------------------------------
// A product whose output covers only a few 128-tiles leaves most of the chip idle on the tiled
// kernels, and each of their workgroups then waits out a memory latency per K step (128 x 1024
// x 1024: 10.6 us on 8 compute units).  Here every wavefront reads its fragments straight from
// global memory in MFMA layout - lane l holds row (column) l % TILE and the 8 values
// k = kGroupK g + 8 (l / TILE) .. + 7 of group g: 16 bytes from an operand stored with K
// contiguous (any 2-byte-aligned address, see ODD below), eight 2-byte loads `ld` apart from one
// stored k-major - keeps the loads of several groups in flight, and accumulates a private TILE x TILE
// partial over its share of K.  The partials are added in wavefront order through LDS, so the
// result does not depend on timing, and the k assignment is the same for every storage order,
// so it does not depend on the flags either.  Any M, N, K, pitch and alignment.
// ODD: rows of an operand stored with K contiguous may start at an odd half (any pitch, any
// base): they are read as aligned dwords and shifted.  Otherwise they start at multiples of 4
// bytes and a lane's 8 halves are one 16-byte load: two thirds of the loads (128 x 128 x 4096:
// 10.5 us against 15.8).  A product's strips always take the first form.
// `partial`: (WAVES - 1) * TILE * TILE floats of LDS
template <int TILE, bool TA, bool TB, int WAVES, bool ODD>
__device__ __forceinline__ void GemmF16FewBody(const GemmF16Args& args, uint32_t block,
                                               float* partial)
{
    static_assert(TILE == 32 || TILE == 16, "MFMA shapes 32x32x16 and 16x16x32");
    constexpr uint32_t kLaneGroups = 64 / TILE;     // groups of TILE lanes
    constexpr uint32_t kGroupK = 8 * kLaneGroups;   // k per MFMA: 16 or 32
    constexpr int kAcc = TILE * TILE / 64;          // accumulator registers: 16 or 4
    constexpr int kQuads = kAcc / 4;
    using Acc = typename std::conditional<TILE == 32, floatx16, floatx4>::type;

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lt = lane % TILE;  // row of A / column of B this lane feeds
    const uint32_t kh = lane / TILE;  // which 8 values of k of an MFMA

    uint32_t id = block;
    const uint32_t tn = id % args.tilesN;
    id /= args.tilesN;
    const uint32_t tm = id % args.tilesM;
    const uint32_t unit = id / args.tilesM;

    const _Float16* __restrict__ A = args.A + args.strideA * static_cast<int64_t>(unit);
    const _Float16* __restrict__ B = args.B + args.strideB * static_cast<int64_t>(unit);
    float* __restrict__ out = args.out + args.strideOut * static_cast<int64_t>(unit);
    const uint32_t M = args.M, N = args.N, K = args.K;
    const uint32_t row = tm * TILE + lt;
    const uint32_t col = tn * TILE + lt;

    // this wavefront's K range, in groups of kGroupK
    constexpr int kDepth = 4;  // groups in flight
    const sph::KPartition part = sph::PartitionK(K, kGroupK, WAVES, wave, kDepth);

    Acc acc;
#pragma unroll
    for (int v = 0; v < kAcc; ++v)
        acc[v] = 0.f;

    // rows and columns past the edge read the last valid one: what they produce is never stored
    const _Float16* aPtr = TA ? A + min(row, M - 1) : A + static_cast<size_t>(min(row, M - 1)) * args.lda;
    const _Float16* bPtr = TB ? B + static_cast<size_t>(min(col, N - 1)) * K : B + min(col, N - 1);
    // whole groups (every k below K): no conditions anywhere, so that the compiler can count
    // the loads in flight instead of waiting for all of them.  The eight 2-byte values of an
    // operand stored k-major stay in a register each while they are in flight and are packed
    // where they are used: packed where they are loaded, every round would end with a wait for
    // its last load.
    struct AlongKOdd
    {
        Halves8 h;
        __device__ __forceinline__ halfx8 get(uint32_t shift) const { return h.Get(shift); }
    };
    struct AlongKEven
    {
        halfx8 v;
        __device__ __forceinline__ halfx8 get(uint32_t) const { return v; }
    };
    using AlongK = typename std::conditional<ODD, AlongKOdd, AlongKEven>::type;
    struct AcrossK
    {
        uint32_t r[8];
        __device__ __forceinline__ halfx8 get(uint32_t) const
        {
            uintx4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = r[2 * i] | (r[2 * i + 1] << 16);
            return __builtin_bit_cast(halfx8, w);
        }
    };
    // (a group is a whole number of dwords on from the operand's first one, so one shift serves
    // every group of a lane)
    const uint32_t aShift = Halves8::Shift(aPtr + kh * 8);
    const uint32_t bShift = Halves8::Shift(bPtr + kh * 8);
    using FragA = typename std::conditional<TA, AcrossK, AlongK>::type;
    using FragB = typename std::conditional<TB, AlongK, AcrossK>::type;
    auto loadAlongK = [&](const _Float16* rowPtr, uint32_t g) {
        AlongK f;
        if constexpr (ODD)
            f.h = Halves8::Load(rowPtr + (g * kGroupK + kh * 8));
        else
            f.v = *reinterpret_cast<const halfx8a4*>(rowPtr + (g * kGroupK + kh * 8));
        return f;
    };
    auto loadAcrossK = [&](const _Float16* colPtr, size_t ld, uint32_t g) {
        const uint16_t* p =
            reinterpret_cast<const uint16_t*>(colPtr + static_cast<size_t>(g * kGroupK + kh * 8) * ld);
        AcrossK f;
#pragma unroll
        for (int e = 0; e < 8; ++e)
            f.r[e] = p[e * ld];
        return f;
    };
    auto loadA = [&](uint32_t g) -> FragA {
        if constexpr (TA)
            return loadAcrossK(aPtr, args.lda, g);
        else
            return loadAlongK(aPtr, g);
    };
    auto loadB = [&](uint32_t g) -> FragB {
        if constexpr (TB)
            return loadAlongK(bPtr, g);
        else
            return loadAcrossK(bPtr, args.ldb, g);
    };
    // the last group when K is no multiple of kGroupK: element by element, zeros past K
    auto loadPartial = [&](const _Float16* base, size_t step, uint32_t g) -> halfx8 {
        const uint32_t k = g * kGroupK + kh * 8;
        const _Float16* p = base + static_cast<size_t>(k) * step;
        halfx8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e)
        {
            v[e] = static_cast<_Float16>(0.f);
            if (k + e < K)
                v[e] = p[e * step];
        }
        return v;
    };
    // operands swapped: the result block comes out indexed [column][row], which leaves 4
    // consecutive columns of one row in a lane
    auto multiply = [&](const halfx8& a, const halfx8& b) {
        if constexpr (TILE == 32)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, acc, 0, 0, 0);
        else
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(b, a, acc, 0, 0, 0);
    };

    const uint32_t whole = part.whole;
    if (part.gBegin < part.wholeEnd)
    {
        const uint32_t wholeEnd = part.wholeEnd, roundsEnd = part.roundsEnd;
        FragA fa[kDepth];
        FragB fb[kDepth];
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
                multiply(fa[d].get(aShift), fb[d].get(bShift));
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
                multiply(fa[d].get(aShift), fb[d].get(bShift));
    }
    if (part.ownsPartial)
    {
        // at most one group, and only in the wavefront that holds the end of K
        const halfx8 a = TA ? loadPartial(aPtr, args.lda, whole) : loadPartial(aPtr, 1, whole);
        const halfx8 b = TB ? loadPartial(bPtr, 1, whole) : loadPartial(bPtr, args.ldb, whole);
        multiply(a, b);
    }

    // lane l holds row l % TILE, columns 4*kLaneGroups*q + 4*(l / TILE) + 0..3 of the tile;
    // partial sums of the other wavefronts go through LDS, wavefront 0 adds them in order
    if (wave != 0)
    {
#pragma unroll
        for (int q = 0; q < kQuads; ++q)
            *reinterpret_cast<float4*>(
                &partial[(wave - 1) * TILE * TILE + lt * TILE + 4 * kLaneGroups * q + 4 * kh]) =
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
                &partial[w * TILE * TILE + lt * TILE + 4 * kLaneGroups * q + 4 * kh]);
            acc[4 * q + 0] += p.x;
            acc[4 * q + 1] += p.y;
            acc[4 * q + 2] += p.z;
            acc[4 * q + 3] += p.w;
        }
    if (row >= M)
        return;
#pragma unroll
    for (int q = 0; q < kQuads; ++q)
    {
        const uint32_t c = tn * TILE + 4 * kLaneGroups * q + 4 * kh;
        if (c >= N)
            continue;
        float* p = out + static_cast<size_t>(row) * args.ldc + c;
        if (c + 4 <= N)
        {
            floatx4 v = floatx4{acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
            if (!args.overwrite)
            {
                const floatx4 old = *reinterpret_cast<const floatx4a4*>(p);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    v[e] = old[e] + v[e];
            }
            *reinterpret_cast<floatx4a4*>(p) = v;
        }
        else
        {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (c + e < N)
                    p[e] = args.overwrite ? acc[4 * q + e] : p[e] + acc[4 * q + e];
        }
    }
}

template <int TILE, bool TA, bool TB, int WAVES, bool ODD>
__global__ __launch_bounds__(WAVES * 64) void GemmF16Few(const GemmF16Args args)
{
    static_assert(!ODD || !TA || TB, "no operand with K contiguous: one form");
    __shared__ __attribute__((aligned(16))) float partial[(WAVES - 1) * TILE * TILE];
    GemmF16FewBody<TILE, TA, TB, WAVES, ODD>(args, blockIdx.x, partial);
}

// What one launch may assume about where its operands lie.
struct F16Layout
{
    bool transA, transB;
};

enum class F16Kernel { kTile256, kTile256x128, kDma64, kDma128, kGeneral };

// The kernel that would take M x N x K with these operands.  The straight-to-LDS copies take 16
// bytes from any 2-byte-aligned address, so the rows of a K x N matrix B may start anywhere
// (any ldb, any base); N itself has to be a multiple of 8 because a copy is 8 columns wide.
// out is accessed 16 bytes at a time from 4-byte-aligned addresses.
F16Kernel PickF16(const GemmF16Args& args, uint32_t N, uint32_t batch, const F16Layout& lay)
{
    const uint32_t M = args.M, K = args.K;
    const bool transA = lay.transA, transB = lay.transB;
    // the 256-tile kernel needs about one tile per compute unit; below three quarters of that
    // the 128-tile kernel keeps more of the chip busy (measured: 2048^3 44 -> 31 us)
    const uint64_t minTiles = static_cast<uint64_t>(sph::ComputeUnits()) * 3 / 4;
    const uint64_t tiles256 =
        static_cast<uint64_t>((M + kT - 1) / kT) * ((N + kT - 1) / kT) * batch;
    // ragged shapes only while at least three quarters of the tiled area is real output
    const bool fills256 =
        static_cast<uint64_t>(M) * N * 4 >=
        static_cast<uint64_t>((M + kT - 1) / kT) * ((N + kT - 1) / kT) * kT * kT * 3;
    // lane offsets of the copies are 32-bit: 256 rows of a K-contiguous operand, 32 of a
    // k-major one (and 256 rows of out in the kernels that copy it)
    const uint64_t pitchA = args.lda, pitchB = transB ? K : args.ldb;
    const bool offsetsFit = (transA ? 32 : 256) * pitchA * 2 + 8192 < (1ull << 32) &&
                            (transB ? 256 : 32) * pitchB * 2 + 8192 < (1ull << 32) &&
                            256ull * args.ldc * 4 + 8192 < (1ull << 32);
    // K = 32 q + r, 0 < r < 32: the straight-to-LDS kernels take the r values in a last,
    // partly masked step (measured 4096 x 4096 x 4080, operands stored plainly: 229 us on the
    // general kernel, 175 us with the r values left to a second launch, 128 us this way)
    const bool tailInKernel = K % kTK != 0 && K >= 2 * kTK;
    const bool dma = K >= kTK &&
                     (K % kTK == 0 || tailInKernel) && N % 8 == 0 && N >= 8 &&
                     (!transA || (M % 8 == 0 && M >= 8));
    if (dma && tiles256 >= minTiles && fills256 && offsetsFit)
        return F16Kernel::kTile256;
    // Too few 256 x 256 tiles for the chip: 256 x 128 tiles while there are between 11/16 of a
    // tile and one tile per compute unit.  All three tiled kernels are bound by what a compute
    // unit's LDS moves per K step (fragment reads plus the copies' writes, about 128 bytes per
    // clock: 64 KiB for a 128 x 128 step of 256 matrix-core clocks, 88 KiB for a 256 x 128 step of
    // 512, 128 KiB for a 256 x 256 step of 1024), so the larger tile needs fewer LDS clocks per
    // flop but only pays once it keeps most of the chip busy (measured, accumulating, 128-tiles
    // against 256 x 128: 3072 x 2048 x 2048 42.2 / 35.3 us, 2048 x 4096 x 2048 47.3 / 42.0 us;
    // 2048^3, 128 tiles on half of the compute units, 28.2 / 32.9 us).
    const uint64_t tilesHalf =
        static_cast<uint64_t>((M + kT - 1) / kT) * ((N + 127) / 128) * batch;
    const bool fillsHalf =
        static_cast<uint64_t>(M) * N * 4 >=
        static_cast<uint64_t>((M + kT - 1) / kT) * ((N + 127) / 128) * kT * 128 * 3;
    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    if (dma && tilesHalf * 16 >= cus * 11 && tilesHalf <= cus && fillsHalf && offsetsFit)
        return F16Kernel::kTile256x128;
    const bool offsets128Fit = static_cast<uint64_t>(M) * (transA ? kTK : args.lda) < (1ull << 31) &&
                               static_cast<uint64_t>(N) * (transB ? K : kTK) < (1ull << 31) &&
                               32ull * args.ldb < (1ull << 30);
    // at most half as many 128-tiles as compute units: 64 x 64 tiles with K steps of 64
    const uint64_t tiles128 =
        static_cast<uint64_t>((M + kG - 1) / kG) * ((N + kG - 1) / kG) * batch;
    if (dma && offsets128Fit && K >= kSK && tiles128 <= cus / 2)
        return F16Kernel::kDma64;
    if (dma && offsets128Fit)
        return F16Kernel::kDma128;
    return F16Kernel::kGeneral;
}

// One launch over all of args.N columns with the kernel `kind`; the workgroups of the strips
// `ride` come last in its grid.
int LaunchF16Kernel(GemmF16Args args, uint32_t batch, F16Kernel kind, const F16Layout& lay,
                    const GemmF16Strips& ride, hipStream_t stream)
{
    const uint32_t M = args.M, N = args.N, K = args.K;
    const bool transA = lay.transA, transB = lay.transB;
    const bool plain = !transA && !transB;
    const bool half = kind == F16Kernel::kTile256x128;  // 256 x 128 tiles
    const bool tile256 = kind == F16Kernel::kTile256 || half;
    const uint32_t edge = tile256 ? kT : kG;
    const uint32_t edgeN = half ? 128u : edge;
    const bool whole256 = (M % kT == 0) && (N % edgeN == 0);
    args.tilesM = (M + edge - 1) / edge;
    args.tilesN = (N + edgeN - 1) / edgeN;
    const uint64_t total = static_cast<uint64_t>(args.tilesM) * args.tilesN * batch;
    SPH_REQUIRE(total < (1ull << 31) - 8, "too many tiles for one launch");
    args.totalTiles = static_cast<uint32_t>(total);
    GemmF16Strips strips = ride;
    strips.first = ((args.totalTiles + 7) / 8) * 8;
    const uint32_t grid = strips.first + strips.blocks[0] + strips.blocks[1];

    if (tile256)
    {
        // old contents of out added inside the loop: spacing 4 from 36 K steps, 2 from 20
        const bool cloop = whole256 && !args.overwrite;
        const uint32_t ksteps = (K + kTK - 1) / kTK;
        const int rowBlocks = half ? 4 : 8;  // per wavefront
        const int variant = !whole256 ? 3
                            : (cloop && ksteps >= static_cast<uint32_t>(CLoopSteps(4, rowBlocks))) ? 2
                            : (cloop && ksteps >= static_cast<uint32_t>(CLoopSteps(2, rowBlocks))) ? 1
                                                                                                : 0;
        const bool tail = K % kTK != 0;
#define SPH_TILE256(TA_, TB_)                                                                     \
    do                                                                                            \
    {                                                                                             \
        if (tail && half)                                                                         \
            LaunchTile256<TA_, TB_, true, 128>(variant, grid, stream, args, strips);                      \
        else if (tail)                                                                            \
            LaunchTile256<TA_, TB_, true, 256>(variant, grid, stream, args, strips);                      \
        else if (half)                                                                            \
            LaunchTile256<TA_, TB_, false, 128>(variant, grid, stream, args, strips);                     \
        else                                                                                      \
            LaunchTile256<TA_, TB_, false, 256>(variant, grid, stream, args, strips);                     \
    } while (0)
        if (transA && transB)
            SPH_TILE256(true, true);
        else if (transA)
            SPH_TILE256(true, false);
        else if (transB)
            SPH_TILE256(false, true);
        else
            SPH_TILE256(false, false);
#undef SPH_TILE256
    }
    else if (kind == F16Kernel::kDma64)
    {
        args.tilesM = (M + kS - 1) / kS;
        args.tilesN = (N + kS - 1) / kS;
        const uint64_t tiles = static_cast<uint64_t>(args.tilesM) * args.tilesN * batch;
        SPH_REQUIRE(tiles < (1ull << 31) - 8, "too many tiles for one launch");
        args.totalTiles = static_cast<uint32_t>(tiles);
        strips.first = ((args.totalTiles + 7) / 8) * 8;
        const dim3 g(strips.first + strips.blocks[0] + strips.blocks[1]), b(256);
        const bool tail = K % kSK != 0;
#define SPH_DMA64(TA_, TB_)                                                                       \
    do                                                                                            \
    {                                                                                             \
        if (tail)                                                                                 \
            hipLaunchKernelGGL((GemmF16Dma64<TA_, TB_, true>), g, b, 0, stream, args, strips);            \
        else                                                                                      \
            hipLaunchKernelGGL((GemmF16Dma64<TA_, TB_, false>), g, b, 0, stream, args, strips);           \
    } while (0)
        if (transA && transB)
            SPH_DMA64(true, true);
        else if (transA)
            SPH_DMA64(true, false);
        else if (transB)
            SPH_DMA64(false, true);
        else
            SPH_DMA64(false, false);
#undef SPH_DMA64
    }
    else if (kind == F16Kernel::kDma128)
    {
        // whole K steps and 16-byte chunks everywhere: straight-to-LDS 128-tile kernel
        // Eight wavefronts per tile (2 x 4, 64 x 32 each) while there is at most one tile per
        // compute unit: a second wavefront per SIMD covers the LDS latency and the barrier of
        // the other (1024^3 13.1 -> 10.8 us, 512 x 512 x 4096 28.8 -> 23.6 us).  With more tiles
        // two workgroups of four share a compute unit anyway and read fewer fragments per
        // flop (4096 x 2048 x 2048: 50.9 us against 52.5 us on eight).
        const bool wide = args.totalTiles <= static_cast<uint32_t>(sph::ComputeUnits());
        const dim3 g(grid);
        const bool tail = K % kTK != 0;
#define SPH_DMA128_(TA_, TB_, TAIL_)                                                              \
    do                                                                                            \
    {                                                                                             \
        if (wide)                                                                                 \
            hipLaunchKernelGGL((GemmF16Dma128<TA_, TB_, TAIL_, 8>), g, dim3(512), 0, stream,      \
                               args, strips);                                                             \
        else                                                                                      \
            hipLaunchKernelGGL((GemmF16Dma128<TA_, TB_, TAIL_, 4>), g, dim3(256), 0, stream,      \
                               args, strips);                                                             \
    } while (0)
#define SPH_DMA128(TA_, TB_)                                                                      \
    do                                                                                            \
    {                                                                                             \
        if (tail)                                                                                 \
            SPH_DMA128_(TA_, TB_, true);                                                          \
        else                                                                                      \
            SPH_DMA128_(TA_, TB_, false);                                                         \
    } while (0)
        if (transA && transB)
            SPH_DMA128(true, true);
        else if (transA)
            SPH_DMA128(true, false);
        else if (transB)
            SPH_DMA128(false, true);
        else
            SPH_DMA128(false, false);
#undef SPH_DMA128
#undef SPH_DMA128_
    }
    else
    {
        // widest load every row start, every row length and every base allows (in halves);
        // an operand is read along its contiguous dimension: K (A), N (B), M (A stored K x M)
        // or K (B stored N x K)
        const uint64_t mix = static_cast<uint64_t>(K) | (transA ? (M | args.lda) : args.lda) |
                             (transB ? K : (args.ldb | N)) |
                             static_cast<uint64_t>(args.strideA) |
                             static_cast<uint64_t>(args.strideB) |
                             (reinterpret_cast<uintptr_t>(args.A) / 2) |
                             (reinterpret_cast<uintptr_t>(args.B) / 2) | 8u;
        const uint32_t vec = static_cast<uint32_t>(mix & (~mix + 1));  // lowest set bit: 1, 2, 4, 8
        args.outVec = ((reinterpret_cast<uintptr_t>(args.out) & 15u) == 0 && args.strideOut % 4 == 0 &&
                       N % 4 == 0 && args.ldc % 4 == 0)
                          ? 1u
                          : 0u;
        const dim3 g(grid), b(kGThreads);
        if (plain)
        {
            if (vec == 8)
                hipLaunchKernelGGL((GemmF16General<8, false, false>), g, b, 0, stream, args,
                                   strips);
            else if (vec >= 2)
                hipLaunchKernelGGL((GemmF16General<2, false, false>), g, b, 0, stream, args,
                                   strips);
            else
                hipLaunchKernelGGL((GemmF16General<1, false, false>), g, b, 0, stream, args,
                                   strips);
        }
        else if (vec == 8)
        {
            if (transA && transB)
                hipLaunchKernelGGL((GemmF16General<8, true, true>), g, b, 0, stream, args, strips);
            else if (transA)
                hipLaunchKernelGGL((GemmF16General<8, true, false>), g, b, 0, stream, args, strips);
            else
                hipLaunchKernelGGL((GemmF16General<8, false, true>), g, b, 0, stream, args, strips);
        }
        else
        {
            if (transA && transB)
                hipLaunchKernelGGL((GemmF16General<1, true, true>), g, b, 0, stream, args, strips);
            else if (transA)
                hipLaunchKernelGGL((GemmF16General<1, true, false>), g, b, 0, stream, args, strips);
            else
                hipLaunchKernelGGL((GemmF16General<1, false, true>), g, b, 0, stream, args, strips);
        }
    }
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}

// Picks the kernels for one call: a body for one of the kernels above and up to two thin strips
// of the product's last rows and columns, which the few-tile kernel's code computes (it reads any
// rows and columns from anywhere) on the first workgroups of the body's launch.  Every output
// element is computed once.  Cut off are
//  - the last N % 8 columns, when a straight-to-LDS kernel then takes the rest (its copies are 8
//    columns wide; row pitches of B and out stay N; measured 4096 x 4100 x 4096: 270 us on the
//    general kernel alone, 129 us with the strip in a launch of its own);
//  - the last M % 8 rows of an A stored K x M, likewise (it is copied 8 rows of the product at a
//    time);
//  - up to 16 rows or columns past a multiple of the tile edge, when the compute unit with the
//    most tiles then has fewer of them (1025^3: 17 x 17 tiles of 64 are two per compute unit
//    somewhere, 16 x 16 one everywhere).
int LaunchFewTiles(GemmF16Args args, uint32_t batch, const F16Layout& lay, hipStream_t stream);

// Tiles of the kernel `kind` over M x N and what one costs, in hundredths of the time a 64 x 64
// tile takes on the 256-tile kernel (measured rates: the smaller the tile, the more LDS traffic
// and fixed cost per flop).
uint64_t F16Cost(F16Kernel kind, uint32_t M, uint32_t N, uint32_t batch)
{
    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    uint32_t edgeM = kG, edgeN = kG;
    uint64_t perTile = 1200;  // general kernel, 128 x 128
    switch (kind)
    {
    case F16Kernel::kTile256: edgeM = edgeN = kT; perTile = 1600; break;
    case F16Kernel::kTile256x128: edgeM = kT; edgeN = 128; perTile = 920; break;
    case F16Kernel::kDma128: perTile = 760; break;
    case F16Kernel::kDma64: edgeM = edgeN = kS; perTile = 220; break;
    case F16Kernel::kGeneral: break;
    }
    const uint64_t tiles =
        static_cast<uint64_t>((M + edgeM - 1) / edgeM) * ((N + edgeN - 1) / edgeN) * batch;
    return (tiles + cus - 1) / cus * perTile;
}

int LaunchF16(GemmF16Args args, uint32_t batch, const F16Layout& lay, hipStream_t stream)
{
    const uint32_t M = args.M, N = args.N;
    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    // candidates for the rows (columns) cut off: none, the remainder the copies cannot take, and
    // the remainders past a tile edge
    auto candidates = [](uint32_t x, uint32_t unit, bool unitAllowed, uint32_t* list) {
        int n = 0;
        list[n++] = 0;
        if (unitAllowed && x % unit != 0 && x > 2 * unit)
            list[n++] = x % unit;
        for (uint32_t edge = 64; edge <= 256; edge *= 2)
        {
            const uint32_t r = x % edge;
            bool seen = false;
            for (int i = 0; i < n; ++i)
                seen = seen || list[i] == r;
            if (r != 0 && r <= 16 && x - r >= edge && !seen)
                list[n++] = r;
        }
        return n;
    };
    uint32_t listM[5], listN[5];
    const int countM = candidates(M, 8, lay.transA, listM);
    const int countN = candidates(N, 8, true, listN);
    // a strip's 16 x 16 tile: a sixteenth of a 64-tile's flops at about a quarter of its rate
    auto stripCost = [&](uint32_t rows, uint32_t cols) {
        const uint64_t blocks =
            static_cast<uint64_t>((rows + 15) / 16) * ((cols + 15) / 16) * batch;
        return (blocks + cus - 1) / cus * 60;
    };
    uint64_t best = ~0ull;
    uint32_t peelM = 0, peelN = 0;
    F16Kernel kind = F16Kernel::kGeneral;
    for (int i = 0; i < countM; ++i)
        for (int j = 0; j < countN; ++j)
        {
            GemmF16Args body = args;
            body.M = M - listM[i];
            const uint32_t bodyN = N - listN[j];
            const F16Kernel k = PickF16(body, bodyN, batch, lay);
            uint64_t cost = F16Cost(k, body.M, bodyN, batch);
            if (listM[i] != 0)
                cost += stripCost(listM[i], N);
            if (listN[j] != 0)
                cost += stripCost(body.M, listN[j]);
            if (cost < best)
            {
                best = cost;
                peelM = listM[i];
                peelN = listN[j];
                kind = k;
            }
        }

    GemmF16Strips strips{};
    int count = 0;
    auto addStrip = [&](GemmF16Args strip) {
        strip.tilesM = (strip.M + kStripTile - 1) / kStripTile;
        strip.tilesN = (strip.N + kStripTile - 1) / kStripTile;
        const uint64_t blocks = static_cast<uint64_t>(strip.tilesM) * strip.tilesN * batch;
        if (blocks >= (1ull << 30))
            return false;
        strips.part[count] = strip;
        strips.blocks[count] = static_cast<uint32_t>(blocks);
        ++count;
        return true;
    };
    GemmF16Args body = args;
    body.M = M - peelM;
    body.N = N - peelN;
    if (peelM != 0)
    {
        // rows [M - peelM, M), every column
        GemmF16Args bottom = args;
        bottom.M = peelM;
        bottom.A = args.A + (lay.transA ? body.M : static_cast<size_t>(body.M) * args.lda);
        bottom.out = args.out + static_cast<size_t>(body.M) * args.ldc;
        SPH_REQUIRE(addStrip(bottom), "too many tiles for one launch");
    }
    if (peelN != 0)
    {
        // rows [0, M - peelM), columns [N - peelN, N)
        GemmF16Args right = args;
        right.M = body.M;
        right.N = peelN;
        right.B = args.B + (lay.transB ? static_cast<size_t>(body.N) * args.K : body.N);
        right.out = args.out + body.N;
        SPH_REQUIRE(addStrip(right), "too many tiles for one launch");
    }
    return LaunchF16Kernel(body, batch, kind, lay, strips, stream);
}

template <bool TA, bool TB, bool ODD>
void LaunchFewForm(const GemmF16Args& args, uint32_t blocks, uint32_t tile, bool wide,
                   hipStream_t stream)
{
    const dim3 g(blocks);
    if (tile == 16 && wide)
        hipLaunchKernelGGL((GemmF16Few<16, TA, TB, 16, ODD>), g, dim3(1024), 0, stream, args);
    else if (tile == 16)
        hipLaunchKernelGGL((GemmF16Few<16, TA, TB, 4, ODD>), g, dim3(256), 0, stream, args);
    else
        hipLaunchKernelGGL((GemmF16Few<32, TA, TB, 4, ODD>), g, dim3(256), 0, stream, args);
}

template <bool TA, bool TB>
void LaunchFew(const GemmF16Args& args, uint32_t blocks, uint32_t tile, bool wide,
               hipStream_t stream)
{
    // do the rows of an operand stored with K contiguous all start at multiples of 4 bytes?
    uint64_t mix = 0;
    if (!TA)
        mix |= args.lda | static_cast<uint64_t>(args.strideA) |
               (reinterpret_cast<uintptr_t>(args.A) / 2);
    if (TB)
        mix |= args.K | static_cast<uint64_t>(args.strideB) |
               (reinterpret_cast<uintptr_t>(args.B) / 2);
    if constexpr (!TA || TB)
    {
        if ((mix & 1u) != 0)
        {
            LaunchFewForm<TA, TB, true>(args, blocks, tile, wide, stream);
            return;
        }
    }
    LaunchFewForm<TA, TB, false>(args, blocks, tile, wide, stream);
}

// Products with at most one 32 x 32 output tile per compute unit, and narrow ones (16 rows or
// columns at most) with up to four 16 x 16 tiles per compute unit, run on the few-tile kernel,
// whatever their storage flags and alignment: the decision looks at M, N, K and the batch only,
// so one product always takes the same kernel and sums in the same order.  Measured against the
// 128-tile kernel (us, plain / A stored K x M / B stored N x K): 256 x 1024 x 1024 6.5 / 7.0 /
// 7.3 against 10.6 / 11.7 / 10.3, 512^3 5.2 against 8.5, 100 x 1024 x 784 5.4 against 10.4,
// 1024 x 10 x 1024 4.5 against 12.5, 16384 x 10 x 256 4.6 against 11.9; with two tiles per
// compute unit (512 x 1024 x 1024) the two are level, with four the tiled kernel wins.
// A product that the 64 x 64-tile kernel takes whole whatever its storage flags (M and N multiples
// of 8, K >= 64) goes there from half a 32-tile per compute unit up (measured, few-tile kernel
// against 64-tiles: 256 x 1024 x 1024 6.5 / 5.8 us, 256 x 512 x 2048 8.9 / 7.6, 128 x 1024 x 1024
// 6.4 / 5.7; below that the few-tile kernel wins: 256^3 3.6 / 4.2, 64 x 1024 x 1024 4.8 / 5.7,
// 256 x 256 x 4096 11.0 / 11.4).
bool TakesFewTiles(uint32_t M, uint32_t N, uint32_t K, uint32_t batch)
{
    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    const uint64_t blocks32 = static_cast<uint64_t>((M + 31) / 32) * ((N + 31) / 32) * batch;
    const uint64_t blocks16 = static_cast<uint64_t>((M + 15) / 16) * ((N + 15) / 16) * batch;
    const bool tiles64Whole = M % 8 == 0 && N % 8 == 0 && K >= 64;
    const uint64_t limit32 = tiles64Whole ? cus / 2 - 1 : cus;
    return blocks32 <= limit32 || (std::min(M, N) <= 16 && blocks16 <= 4 * cus);
}

int LaunchFewTiles(GemmF16Args args, uint32_t batch, const F16Layout& lay, hipStream_t stream)
{
    // 16 x 16 tiles while there are at most one and a half per compute unit, or for a narrow
    // matrix (less of a tile outside it): a quarter of the matrix-core work per workgroup on
    // four times as many compute units, but twice the operand bytes per flop (64 x 1024 x 1024:
    // 4.9 us against 6.3 on 32 x 32; 128 x 1024 x 1024: 6.9 against 6.4); 16 wavefronts per tile
    // when the tiles fit the chip once and K is long (128 x 128 x 4096: 10.4 us against 14.2)
    const uint64_t cus = static_cast<uint64_t>(sph::ComputeUnits());
    const uint64_t blocks16 =
        static_cast<uint64_t>((args.M + 15) / 16) * ((args.N + 15) / 16) * batch;
    const uint32_t tile =
        (2 * blocks16 <= 3 * cus || std::min(args.M, args.N) <= 16) ? 16u : 32u;
    args.tilesM = (args.M + tile - 1) / tile;
    args.tilesN = (args.N + tile - 1) / tile;
    const uint64_t blocks = static_cast<uint64_t>(args.tilesM) * args.tilesN * batch;
    SPH_REQUIRE(blocks < (1ull << 31), "too many tiles for one launch");
    const bool wide = tile == 16 && blocks <= cus && args.K >= 1024;
    if (lay.transA && lay.transB)
        LaunchFew<true, true>(args, static_cast<uint32_t>(blocks), tile, wide, stream);
    else if (lay.transA)
        LaunchFew<true, false>(args, static_cast<uint32_t>(blocks), tile, wide, stream);
    else if (lay.transB)
        LaunchFew<false, true>(args, static_cast<uint32_t>(blocks), tile, wide, stream);
    else
        LaunchFew<false, false>(args, static_cast<uint32_t>(blocks), tile, wide, stream);
    SPH_CHECK_LAUNCH();
    return SPH_OK;
}
}  // namespace

extern "C" {

int sph_gemm_f16f32(float* out, const sph_f16* A, const sph_f16* B, uint32_t M, uint32_t N,
                    uint32_t K, uint32_t batch, int64_t strideOut, int64_t strideA,
                    int64_t strideB, uint32_t flags)
{
    SPH_REQUIRE(M != 0 && N != 0 && batch != 0, "M, N and batch must be non-zero");
    SPH_REQUIRE((flags & ~(SPH_GEMM_OVERWRITE | SPH_GEMM_TRANS_A | SPH_GEMM_TRANS_B)) == 0,
                "unknown flag");
    const bool transA = (flags & SPH_GEMM_TRANS_A) != 0;
    const bool transB = (flags & SPH_GEMM_TRANS_B) != 0;
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

    F16Layout lay{};
    lay.transA = transA;
    lay.transB = transB;

    GemmF16Args args{};
    args.out = out;
    args.A = reinterpret_cast<const _Float16*>(A);
    args.B = reinterpret_cast<const _Float16*>(B);
    args.M = M;
    args.N = N;
    args.K = K;
    args.lda = transA ? M : K;
    args.ldb = N;
    args.ldc = N;
    args.strideOut = strideOut;
    args.strideA = strideA;
    args.strideB = strideB;
    args.overwrite = (flags & SPH_GEMM_OVERWRITE) ? 1u : 0u;

    if (TakesFewTiles(M, N, K, batch))
        return LaunchFewTiles(args, batch, lay, stream);
    return LaunchF16(args, batch, lay, stream);
}

}  // extern "C"
