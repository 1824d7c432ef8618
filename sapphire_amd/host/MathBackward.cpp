#include <Sapphire/operations/Backward/MathBackward.hpp>

#include <Sapphire/compute/BasicOps.hpp>
#include <Sapphire/compute/dense/cuda/Gemm.hpp>

#include <stdexcept>

namespace Sapphire::BackProp
{
using TensorUtil::TensorData;

namespace
{
// leading dimensions of the three tensors agree and all have at least two dimensions
bool PlainBatch(const TensorData& dy, const TensorData& a, const TensorData& b)
{
    const Shape sy = dy.GetShape(), sa = a.GetShape(), sb = b.GetShape();
    if (sy.Dim() < 2 || sa.Dim() != sy.Dim() || sb.Dim() != sy.Dim())
        return false;
    for (int i = 0; i < sy.Dim() - 2; ++i)
        if (sa.At(i) != sy.At(i) || sb.At(i) != sy.At(i))
            return false;
    return sa.Rows() == sy.Rows() && sb.Cols() == sy.Cols() && sa.Cols() == sb.Rows();
}
}  // namespace

void MatMulBackward(TensorData& da, TensorData& db, const TensorData& dy, const TensorData& a,
                    const TensorData& b, Sequence sequence)
{
    if (da.Mode() != dy.Mode() || db.Mode() != dy.Mode() || a.Mode() != dy.Mode() ||
        b.Mode() != dy.Mode())
        throw std::invalid_argument("BackProp::MatMul - Device mode inequality");
    if (dy.Mode() != ComputeMode::Cuda)
        throw std::runtime_error(
            "BackProp::MatMul - Host mode is not provided by the device backend");

    if (sequence == Sequence::Direct && PlainBatch(dy, a, b))
    {
        const auto m = static_cast<unsigned int>(a.Rows());
        const auto k = static_cast<unsigned int>(a.Cols());
        const auto n = static_cast<unsigned int>(b.Cols());
        const auto batch = static_cast<unsigned int>(dy.GetNumUnits(2));
        const int deviceId = dy.GetCudaDevice().GetID();
        // da [m, k] += dy [m, n] * (b [k, n])^T
        Compute::Dense::Cuda::GemmTransposed(da.CudaMutableRawPtr(), dy.CudaRawPtr(),
                                             b.CudaRawPtr(), m, k, n, batch, false, true, false,
                                             deviceId);
        // db [k, n] += (a [m, k])^T * dy [m, n]
        Compute::Dense::Cuda::GemmTransposed(db.CudaMutableRawPtr(), a.CudaRawPtr(),
                                             dy.CudaRawPtr(), k, n, m, batch, true, false, false,
                                             deviceId);
        return;
    }

    TensorData transposedA(a.GetShape().GetTranspose(), a.GetType(), a.GetCudaDevice());
    TensorData transposedB(b.GetShape().GetTranspose(), b.GetType(), b.GetCudaDevice());
    transposedA.SetMode(a.Mode());
    transposedB.SetMode(b.Mode());
    Compute::Transpose(transposedA, a);
    Compute::Transpose(transposedB, b);
    Compute::Gemm(da, dy, transposedB);
    Compute::Gemm(db, transposedA, dy);
}
}  // namespace Sapphire::BackProp
