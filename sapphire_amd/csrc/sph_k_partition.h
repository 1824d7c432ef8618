// How the few-tile GEMM kernels (fp32 GemmF32SkinnyKernel, fp16 GemmF16Few) hand the K range of a
// tile to the tile's wavefronts.  One definition for both kernels and for the host, so that the
// CPU tests exercise the arithmetic the kernels run.
//
// K is cut into groups of groupK values (what one lane-wide load covers); wavefront w of `waves`
// takes a contiguous run of groups [gBegin, gEnd).  Groups below `whole` have every k below K and
// are multiplied in a loop free of conditions that keeps `depth` groups in flight: the loads
// run `depth` groups ahead of the matrix instructions and an index past the wavefront's last
// whole group is clamped to that group (loaded once more, not used).  The loop body is written
// out `depth` times, so whole groups in [gBegin, roundsEnd) are multiplied inside full rounds
// and the up to depth - 1 that remain straight from the registers.  The one group that K may
// end in is read element by element by the wavefront that owns it.
#ifndef SPH_K_PARTITION_H
#define SPH_K_PARTITION_H

#include <cstdint>

#if defined(__HIPCC__)
#define SPH_HOST_DEVICE __host__ __device__
#else
#define SPH_HOST_DEVICE
#endif

namespace sph
{
struct KPartition
{
    uint32_t gBegin, gEnd;  // this wavefront's groups
    uint32_t whole;         // groups with every k below K
    uint32_t wholeEnd;      // this wavefront's whole groups end here
    uint32_t lastWhole;     // its last whole group (meaningful when gBegin < wholeEnd)
    uint32_t roundsEnd;     // its whole groups below this one run in full rounds of `depth`
    bool ownsPartial;       // the group that K ends in belongs to this wavefront
};

SPH_HOST_DEVICE inline uint32_t KPartitionMin(uint32_t a, uint32_t b)
{
    return a < b ? a : b;
}

SPH_HOST_DEVICE inline KPartition PartitionK(uint32_t K, uint32_t groupK, uint32_t waves,
                                             uint32_t wave, uint32_t depth)
{
    KPartition p;
    const uint32_t groups = (K + groupK - 1) / groupK;
    const uint32_t perWave = (groups + waves - 1) / waves;
    p.gBegin = KPartitionMin(wave * perWave, groups);
    p.gEnd = KPartitionMin(p.gBegin + perWave, groups);
    p.whole = K / groupK;
    p.wholeEnd = KPartitionMin(p.gEnd, p.whole);
    p.lastWhole = p.wholeEnd != 0 ? p.wholeEnd - 1 : 0;
    p.roundsEnd = p.gBegin < p.wholeEnd ? p.gBegin + (p.wholeEnd - p.gBegin) / depth * depth : p.gBegin;
    p.ownsPartial = p.gBegin <= p.whole && p.whole < p.gEnd;
    return p;
}

// the group the loop loads into slot d while it multiplies round g .. g + depth - 1
SPH_HOST_DEVICE inline uint32_t KPartitionNext(const KPartition& p, uint32_t g, uint32_t depth,
                                               uint32_t d)
{
    return KPartitionMin(g + depth + d, p.lastWhole);
}

// the group slot d holds before the first round
SPH_HOST_DEVICE inline uint32_t KPartitionFirst(const KPartition& p, uint32_t d)
{
    return KPartitionMin(p.gBegin + d, p.lastWhole);
}
}  // namespace sph

#endif
