#include <Sapphire/compute/BasicOps.hpp>

#include <Sapphire/compute/BroadcastPlan.hpp>
#include <Sapphire/compute/dense/cuda/Gemm.hpp>

#include <algorithm>
#include <stdexcept>
#include <string>

namespace Sapphire::Compute
{
namespace
{
void RequireSameMode(const TensorData& y, const TensorData& x, const char* op)
{
    if (y.Mode() != x.Mode())
        throw std::invalid_argument(std::string("Compute::") + op + " - Device mode inequality");
}

void RequireDeviceMode(const TensorData& y, const char* op)
{
    if (y.Mode() != ComputeMode::Cuda)
        throw std::runtime_error(std::string("Compute::") + op +
                                 " - Host mode is not provided by the device backend");
}
}  // namespace

void Gemm(TensorData& y, const TensorData& a, const TensorData& b)
{
    RequireSameMode(y, a, "Gemm");
    RequireSameMode(y, b, "Gemm");
    RequireDeviceMode(y, "Gemm");

    const GemmPlan plan = PlanGemm(y.GetShape(), a.GetShape(), b.GetShape());
    const int deviceId = y.GetCudaDevice().GetID();
    const float* A = a.CudaRawPtr();
    const float* B = b.CudaRawPtr();

    // the whole walk as one strided-batched launch when its offsets are affine (all the
    // common cases: no batch, equal batches, one operand shared by the batch) ...
    std::uint32_t count = 0;
    std::int64_t strideOut = 0, strideA = 0, strideB = 0;
    const bool strided = AsStridedBatch(plan, count, strideOut, strideA, strideB);
    // A fresh y whose zero fill is still deferred, written exactly once everywhere by this
    // walk: y += a*b on zeros is y = a*b, so the product is stored and neither the fill nor
    // the read of the zeros happens (same result bits: 0 + s == s for every sum the kernels
    // produce, none of which is -0).
    if (strided && strideOut == static_cast<std::int64_t>(plan.M) * plan.N &&
        static_cast<std::uint64_t>(count) * plan.M * plan.N ==
            static_cast<std::uint64_t>(y.Size()) &&
        y.TakeDeferredZero())
    {
        Dense::Cuda::GemmStrided(y.CudaOverwriteRawPtr(), A, B, plan.M, plan.N, plan.K, count,
                                 strideOut, strideA, strideB, true, deviceId);
        return;
    }
    float* out = y.CudaMutableRawPtr();
    if (strided)
    {
        if (strideOut == static_cast<std::int64_t>(plan.M) * plan.N &&
            strideA == static_cast<std::int64_t>(plan.M) * plan.K &&
            strideB == static_cast<std::int64_t>(plan.K) * plan.N)
        {
            Dense::Cuda::Gemm(count * plan.M * plan.N, out, A, B, plan.M, plan.N, plan.K, deviceId);
            return;
        }
        if ((strideA == 0 || strideA == static_cast<std::int64_t>(plan.M) * plan.K) &&
            (strideB == 0 || strideB == static_cast<std::int64_t>(plan.K) * plan.N) &&
            strideOut == static_cast<std::int64_t>(plan.M) * plan.N)
        {
            Dense::Cuda::GemmMatrixWiseBroadcast(out, A, B, plan.M, plan.N, plan.K, count,
                                                 strideA == 0, strideB == 0, deviceId);
            return;
        }
    }

    // ... otherwise as one grouped launch over the list of unit products
    const std::uint64_t mn = static_cast<std::uint64_t>(plan.M) * plan.N;
    const std::uint64_t mk = static_cast<std::uint64_t>(plan.M) * plan.K;
    const std::uint64_t kn = static_cast<std::uint64_t>(plan.K) * plan.N;
    std::vector<Dense::Cuda::GemmUnit> units;
    for (const BroadcastLeaf& leaf : plan.leaves)
    {
        const std::uint64_t run = mn ? leaf.totalSizeOut / mn : 0;
        for (std::uint64_t u = 0; u < run; ++u)
            units.push_back({ leaf.outOff + u * mn, leaf.aOff + u * mk, leaf.bOff + u * kn });
    }
    Dense::Cuda::GemmGrouped(units, out, A, B, plan.M, plan.N, plan.K, deviceId);
}

void GemmHalf(TensorData& y, const std::uint16_t* a, const std::uint16_t* b, unsigned int K)
{
    RequireDeviceMode(y, "GemmHalf");
    if (a == nullptr || b == nullptr)
        throw std::invalid_argument("Compute::GemmHalf - null operand");
    const auto M = static_cast<unsigned int>(y.Rows());
    const auto N = static_cast<unsigned int>(y.Cols());
    const auto batch = static_cast<unsigned int>(y.GetNumUnits(2));
    const int deviceId = y.GetCudaDevice().GetID();
    const std::size_t mn = static_cast<std::size_t>(M) * N;
    const bool freshZero = y.TakeDeferredZero();
    float* out = freshZero ? y.CudaOverwriteRawPtr() : y.CudaMutableRawPtr();
    Dense::Cuda::GemmHalf(out, a, b, M, N, K, batch, mn, static_cast<std::size_t>(M) * K,
                          static_cast<std::size_t>(K) * N, freshZero, deviceId);
}

void Transpose(TensorData& y, const TensorData& x)
{
    RequireSameMode(y, x, "Transpose");
    RequireDeviceMode(y, "Transpose");
    const int rows = x.Rows();
    const int cols = x.Cols();
    const bool broadcast = x.GetNumUnits(2) == 1;
    const int matrices = y.GetShape().Size() / (rows * cols);
    // writes every element of y (matrices * rows * cols of them)
    float* out = static_cast<long long>(matrices) * rows * cols == y.Size() ? y.CudaOverwriteRawPtr()
                                                                           : y.CudaMutableRawPtr();
    Dense::Cuda::Transpose(out, x.CudaRawPtr(), static_cast<unsigned int>(rows),
                           static_cast<unsigned int>(cols), static_cast<unsigned int>(matrices),
                           broadcast);
}

void ReLU(TensorData& y, const TensorData& x)
{
    RequireSameMode(y, x, "ReLU");
    RequireDeviceMode(y, "ReLU");
    Dense::Cuda::ReLU(y.CudaOverwriteRawPtr(), x.CudaRawPtr(), static_cast<unsigned int>(y.Size()));
}

void ReLUBackward(TensorData& dx, const TensorData& dy, const TensorData& x)
{
    RequireSameMode(dx, dy, "ReLUBackward");
    RequireSameMode(dx, x, "ReLUBackward");
    RequireDeviceMode(dx, "ReLUBackward");
    Dense::Cuda::ReLUBackward(dx.CudaMutableRawPtr(), dy.CudaRawPtr(), x.CudaRawPtr(),
                              static_cast<unsigned int>(dx.Size()));
}

void Scale(TensorData& y, const TensorData& x, const float factor)
{
    RequireSameMode(y, x, "Scale");
    RequireDeviceMode(y, "Scale");
    // y may be x (in place): settle x first, then y has no deferred fill left to drop
    const float* in = x.CudaRawPtr();
    Dense::Cuda::Scale(y.CudaOverwriteRawPtr(), in, factor,
                       static_cast<unsigned int>(y.GetShape().Size()));
}

void Sub(TensorData& y, const TensorData& a, const TensorData& b)
{
    RequireSameMode(y, a, "Sub");
    RequireSameMode(y, b, "Sub");
    RequireDeviceMode(y, "Sub");

    Shape shapeOut = y.GetShape(), shapeA = a.GetShape(), shapeB = b.GetShape();
    const int maxDim = std::max({ shapeOut.Dim(), shapeA.Dim(), shapeB.Dim() });
    shapeOut.Expand(maxDim);
    shapeA.Expand(maxDim);
    shapeB.Expand(maxDim);
    const int leafDim = GetMatchingDim({ shapeOut, shapeA, shapeB });

    const auto leaves = PlanBroadcastWith2Inputs(
        shapeOut, shapeA, shapeB, static_cast<unsigned int>(shapeOut.Size()),
        static_cast<unsigned int>(shapeA.Size()), static_cast<unsigned int>(shapeB.Size()), 0,
        static_cast<unsigned int>(leafDim));
    for (const BroadcastLeaf& leaf : leaves)
        Dense::Cuda::Sub(leaf.totalSizeOut, y.CudaMutableRawPtr() + leaf.outOff,
                         a.CudaRawPtr() + leaf.aOff, b.CudaRawPtr() + leaf.bOff, 0, false, false);
}
}  // namespace Sapphire::Compute
