#include <Sapphire/compute/BroadcastPlan.hpp>

#include <algorithm>
#include <stdexcept>

namespace Sapphire::Compute
{
namespace
{
struct Walker
{
    const Shape& y;
    const Shape& a;
    const Shape& b;
    unsigned int limit;  // first dimension that belongs to the leaf
    std::vector<BroadcastLeaf>& out;

    void Visit(unsigned int sizeOut, unsigned int sizeA, unsigned int sizeB, std::uint64_t offOut,
               std::uint64_t offA, std::uint64_t offB, unsigned int idx) const
    {
        // leading dimensions on which all three agree are folded into one run
        unsigned int folded = 1;
        while (idx < limit && y.At(static_cast<int>(idx)) == a.At(static_cast<int>(idx)) &&
               y.At(static_cast<int>(idx)) == b.At(static_cast<int>(idx)))
        {
            folded *= static_cast<unsigned int>(y.At(static_cast<int>(idx)));
            ++idx;
        }
        if (idx >= limit)
        {
            out.push_back({ offOut, offA, offB, sizeOut });
            return;
        }

        // first dimension where they differ: each tensor is cut into folded*extent chunks and
        // the longest chunk list drives the loop, the shorter ones wrap round
        const unsigned int chunksOut = folded * static_cast<unsigned int>(y.At(static_cast<int>(idx)));
        const unsigned int chunksA = folded * static_cast<unsigned int>(a.At(static_cast<int>(idx)));
        const unsigned int chunksB = folded * static_cast<unsigned int>(b.At(static_cast<int>(idx)));
        const unsigned int stepOut = sizeOut / chunksOut;
        const unsigned int stepA = sizeA / chunksA;
        const unsigned int stepB = sizeB / chunksB;
        const unsigned int rounds = std::max({ chunksOut, chunksA, chunksB });
        for (unsigned int c = 0; c < rounds; ++c)
        {
            // products are formed in unsigned int, like pointer + unsigned in the reference
            const unsigned int dOut = (c % chunksOut) * stepOut;
            const unsigned int dA = (c % chunksA) * stepA;
            const unsigned int dB = (c % chunksB) * stepB;
            Visit(stepOut, stepA, stepB, offOut + dOut, offA + dA, offB + dB, idx + 1);
        }
    }
};
}  // namespace

std::vector<BroadcastLeaf> PlanBroadcastWith2Inputs(const Shape& yShape, const Shape& aShape,
                                                    const Shape& bShape,
                                                    unsigned int totalSizeOut,
                                                    unsigned int totalSizeA,
                                                    unsigned int totalSizeB,
                                                    unsigned int shapeIdx,
                                                    unsigned int minimumRequiredDim)
{
    std::vector<BroadcastLeaf> leaves;
    const unsigned int limit = static_cast<unsigned int>(yShape.Dim()) - minimumRequiredDim;
    const Walker walker{ yShape, aShape, bShape, limit, leaves };
    walker.Visit(totalSizeOut, totalSizeA, totalSizeB, 0, 0, 0, shapeIdx);
    return leaves;
}

int GetMatchingDim(const std::vector<Shape>& shapes)
{
    if (shapes.empty())
        throw std::runtime_error("Util::GetMatchingDim - shapes is empty");
    // count trailing positions that exist in every shape and hold the same extent
    int matched = 0;
    for (;;)
    {
        const int fromLast = matched + 1;
        bool agree = true;
        for (const Shape& shape : shapes)
            if (shape.Dim() < fromLast || shape.At(-fromLast) != shapes.front().At(-fromLast))
            {
                agree = false;
                break;
            }
        if (!agree)
            return matched;
        ++matched;
    }
}

GemmPlan PlanGemm(const Shape& y, const Shape& a, const Shape& b)
{
    GemmPlan plan;
    Shape so = y, sa = a, sb = b;
    // 1-D operands are rows
    so.Expand(2);
    sa.Expand(2);
    sb.Expand(2);
    plan.M = static_cast<unsigned int>(so.Rows());
    plan.N = static_cast<unsigned int>(so.Cols());
    plan.K = static_cast<unsigned int>(sa.Cols());
    // the batch dimensions are whatever the longest of the original shapes has
    plan.maxDim = std::max({ y.Dim(), a.Dim(), b.Dim(), 2 });
    so.Expand(plan.maxDim);
    sa.Expand(plan.maxDim);
    sb.Expand(plan.maxDim);
    plan.sizeOut = so.Size();
    plan.sizeA = sa.Size();
    plan.sizeB = sb.Size();
    plan.leaves = PlanBroadcastWith2Inputs(so, sa, sb, static_cast<unsigned int>(plan.sizeOut),
                                           static_cast<unsigned int>(plan.sizeA),
                                           static_cast<unsigned int>(plan.sizeB), 0, 2);
    return plan;
}

bool AsStridedBatch(const GemmPlan& plan, std::uint32_t& count, std::int64_t& strideOut,
                    std::int64_t& strideA, std::int64_t& strideB)
{
    const std::uint64_t mn = static_cast<std::uint64_t>(plan.M) * plan.N;
    const std::uint64_t mk = static_cast<std::uint64_t>(plan.M) * plan.K;
    const std::uint64_t kn = static_cast<std::uint64_t>(plan.K) * plan.N;
    if (mn == 0 || plan.leaves.empty())
        return false;

    bool have = false;
    std::uint64_t units = 0;
    std::uint64_t firstOut = 0, firstA = 0, firstB = 0;
    auto accept = [&](std::uint64_t o, std::uint64_t a, std::uint64_t b) {
        if (units == 0)
        {
            firstOut = o;
            firstA = a;
            firstB = b;
            if (o != 0 || a != 0 || b != 0)
                return false;
        }
        else if (!have)
        {
            // the second unit fixes the strides; offsets never decrease in an affine walk
            if (o < firstOut || a < firstA || b < firstB)
                return false;
            strideOut = static_cast<std::int64_t>(o - firstOut);
            strideA = static_cast<std::int64_t>(a - firstA);
            strideB = static_cast<std::int64_t>(b - firstB);
            have = true;
        }
        else if (o != units * static_cast<std::uint64_t>(strideOut) ||
                 a != units * static_cast<std::uint64_t>(strideA) ||
                 b != units * static_cast<std::uint64_t>(strideB))
            return false;
        ++units;
        return true;
    };

    for (const BroadcastLeaf& leaf : plan.leaves)
    {
        const std::uint64_t run = leaf.totalSizeOut / mn;
        for (std::uint64_t u = 0; u < run; ++u)
            if (!accept(leaf.outOff + u * mn, leaf.aOff + u * mk, leaf.bOff + u * kn))
                return false;
    }
    if (units == 0 || units > 0xffffffffull)
        return false;
    if (!have)
    {
        strideOut = static_cast<std::int64_t>(mn);
        strideA = static_cast<std::int64_t>(mk);
        strideB = static_cast<std::int64_t>(kn);
    }
    // distinct outputs are required for one launch
    if (units > 1 && static_cast<std::uint64_t>(strideOut) < mn)
        return false;
    count = static_cast<std::uint32_t>(units);
    return true;
}
}  // namespace Sapphire::Compute
