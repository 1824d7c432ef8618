#include <Sapphire/operations/Forward/LinearForward.hpp>

#include <Sapphire/compute/BasicOps.hpp>
#include <Sapphire/compute/Initialize.hpp>
#include <Sapphire/compute/dense/cuda/Gemm.hpp>
#include <Sapphire/compute/sparse/SparseGemm.hpp>

#include <stdexcept>

namespace Sapphire::Util
{
void ChangeTensorDataDimension(int dimension, TensorUtil::TensorData& data)
{
    Shape shape = data.GetShape();
    shape.Expand(dimension);
    shape.Shrink(dimension);
    data.Reshape(shape);
}
}  // namespace Sapphire::Util

namespace Sapphire::NN
{
void LinearForward(TensorUtil::TensorData& y, const TensorUtil::TensorData& x,
                   const TensorUtil::TensorData& weight, const TensorUtil::TensorData& bias)
{
    if (x.Mode() != weight.Mode() || x.Mode() != bias.Mode() || x.Mode() != y.Mode())
        throw std::invalid_argument("NN::Linear - Device mode inequality");

    const int batchSize = x.GetShape().GetNumUnits(1);
    TensorUtil::TensorData ones(Shape({ batchSize, 1 }), Type::Dense, bias.GetCudaDevice());
    ones.SetMode(bias.Mode());
    Compute::Initialize::Ones(ones);

    // shallow views with 2-D shapes; the buffers are the caller's
    TensorUtil::TensorData x2 = x, y2 = y, bias2 = bias;
    Util::ChangeTensorDataDimension(2, x2);
    Util::ChangeTensorDataDimension(2, y2);
    Util::ChangeTensorDataDimension(2, bias2);

    Compute::Gemm(y2, ones, bias2);
    Compute::Gemm(y2, x2, weight);
}

void LinearForwardFused(TensorUtil::TensorData& y, const TensorUtil::TensorData& x,
                        const TensorUtil::TensorData& weight,
                        const TensorUtil::TensorData& bias, bool relu)
{
    if (x.Mode() != weight.Mode() || x.Mode() != bias.Mode() || x.Mode() != y.Mode())
        throw std::invalid_argument("NN::Linear - Device mode inequality");
    if (x.Mode() != ComputeMode::Cuda)
        throw std::runtime_error("NN::Linear - Host mode is not provided by the device backend");
    const int batchSize = x.GetShape().GetNumUnits(1);
    const int inputs = weight.Rows();
    const int outputs = weight.Cols();
    if (x.Size() != batchSize * inputs || y.Size() != batchSize * outputs ||
        bias.Size() != outputs)
        throw std::invalid_argument("NN::Linear - shape mismatch");
    // y is written everywhere and not read
    Compute::Dense::Cuda::LinearForward(
        y.CudaOverwriteRawPtr(), x.CudaRawPtr(), weight.CudaRawPtr(), bias.CudaRawPtr(),
        static_cast<unsigned int>(batchSize), static_cast<unsigned int>(inputs),
        static_cast<unsigned int>(outputs), relu, y.GetCudaDevice().GetID());
}

void SparseLinearForward(TensorUtil::TensorData& y, const TensorUtil::TensorData& x,
                         const SparseMatrix& weightTransposed,
                         const TensorUtil::TensorData& bias)
{
    if (x.Mode() != bias.Mode() || x.Mode() != y.Mode())
        throw std::invalid_argument("NN::Linear - Device mode inequality");
    if (x.Mode() != ComputeMode::Cuda)
        throw std::runtime_error("NN::Linear - Host mode is not provided by the device backend");

    const int batchSize = x.GetShape().GetNumUnits(1);
    const int inputs = static_cast<int>(weightTransposed.N);
    const int outputs = static_cast<int>(weightTransposed.M);
    if (x.Size() != batchSize * inputs || y.Size() != batchSize * outputs ||
        bias.Size() != outputs)
        throw std::invalid_argument("NN::Linear - sparse weight shape mismatch");
    const CudaDevice device = x.GetCudaDevice();

    TensorUtil::TensorData x2 = x, y2 = y;
    Util::ChangeTensorDataDimension(2, x2);
    Util::ChangeTensorDataDimension(2, y2);

    TensorUtil::TensorData xT(Shape({ inputs, batchSize }), Type::Dense, device);
    TensorUtil::TensorData yT(Shape({ outputs, batchSize }), Type::Dense, device);
    xT.SetMode(ComputeMode::Cuda);
    yT.SetMode(ComputeMode::Cuda);

    // yT = bias x ones + W^T_csr * xT in one launch: the bias of an output row is the value the
    // product is added to, which is what Zeros(yT); Gemm(yT, bias, ones); accumulate leaves
    Compute::Transpose(xT, x2);
    Compute::Sparse::Cuda::GemmBias(yT.CudaOverwriteRawPtr(), &weightTransposed, xT.CudaRawPtr(),
                                    static_cast<unsigned int>(batchSize), bias.CudaRawPtr(),
                                    device.GetID());
    Compute::Transpose(y2, yT);
}
}  // namespace Sapphire::NN
