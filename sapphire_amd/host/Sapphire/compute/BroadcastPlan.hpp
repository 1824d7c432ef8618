// The batch-broadcast walk of the operator layer, run once on the host to produce a plan
// instead of one device call per leaf.
//
// The reference's BroadcastWith2Inputs (Includes/Sapphire/compute/Broadcast.hpp:83-133) walks
// the leading dimensions of (y, a, b) and calls a functor per leaf with pointers offset by
// (chunkIdx % chunkSizeX) * strideX.  That rule is not NumPy broadcasting (a broadcast
// dimension below an equal leading one selects operand i % b, not i / M), so the offsets here
// are produced by the same walk, in the same unsigned-int arithmetic, rather than derived from
// first principles.  The result is a list of leaves; each leaf is a run of
// totalSizeOut / (M*N) back-to-back unit products.
#ifndef SAPPHIRE_AMD_COMPUTE_BROADCASTPLAN_HPP
#define SAPPHIRE_AMD_COMPUTE_BROADCASTPLAN_HPP

#include <Sapphire/util/Shape.hpp>

#include <cstdint>
#include <vector>

namespace Sapphire::Compute
{
struct BroadcastLeaf
{
    std::uint64_t outOff;   //!< element offsets from the three tensor bases
    std::uint64_t aOff;
    std::uint64_t bOff;
    unsigned int totalSizeOut;  //!< what the leaf functor would receive as totalSize
};

//! Leaves in the order the reference's recursion visits them.  The three shapes must have the
//! same Dim(); the trailing `minimumRequiredDim` dimensions belong to the leaf.
std::vector<BroadcastLeaf> PlanBroadcastWith2Inputs(const Shape& yShape, const Shape& aShape,
                                                    const Shape& bShape,
                                                    unsigned int totalSizeOut,
                                                    unsigned int totalSizeA,
                                                    unsigned int totalSizeB,
                                                    unsigned int shapeIdx,
                                                    unsigned int minimumRequiredDim);

//! Number of trailing dimensions on which every shape agrees
//! (Includes/Sapphire/util/UnitUtils.hpp:38-73).  Throws std::runtime_error for an empty list.
int GetMatchingDim(const std::vector<Shape>& shapes);

//! Shape bookkeeping of Compute::Gemm (Sources/Sapphire/compute/BasicOps.cpp:189-230).
struct GemmPlan
{
    unsigned int M = 0, N = 0, K = 0;
    int maxDim = 0;
    int sizeOut = 0, sizeA = 0, sizeB = 0;
    std::vector<BroadcastLeaf> leaves;
};

GemmPlan PlanGemm(const Shape& y, const Shape& a, const Shape& b);

//! True when the unit products of the plan, in order, are
//! (u*strideOut, u*strideA, u*strideB) for u = 0..count-1, i.e. one strided-batched launch
//! (stride 0 = operand repeated) reproduces the whole walk.
bool AsStridedBatch(const GemmPlan& plan, std::uint32_t& count, std::int64_t& strideOut,
                    std::int64_t& strideA, std::int64_t& strideB);
}  // namespace Sapphire::Compute

#endif
