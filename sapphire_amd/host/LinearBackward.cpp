#include <Sapphire/operations/Backward/LinearBackward.hpp>

#include <Sapphire/compute/BasicOps.hpp>
#include <Sapphire/compute/Initialize.hpp>
#include <Sapphire/compute/dense/cuda/Gemm.hpp>

#include <stdexcept>

namespace Sapphire::Optimizer
{
void SGD::operator()(TensorUtil::TensorData& z, const TensorUtil::TensorData& dz,
                     const std::string&) const
{
    if (z.Mode() != dz.Mode())
        throw std::invalid_argument("Optimizer::SGD - Device mode inequality");
    if (m_fused)
    {
        if (z.Mode() != ComputeMode::Cuda)
            throw std::runtime_error(
                "Optimizer::SGD - Host mode is not provided by the device backend");
        Compute::Dense::Cuda::SgdStep(z.CudaMutableRawPtr(), dz.CudaRawPtr(), m_learningRate,
                                      static_cast<unsigned int>(z.Size()));
        return;
    }
    TensorUtil::TensorData temp(dz.GetShape(), dz.GetType(), dz.GetCudaDevice());
    temp.SetMode(dz.Mode());
    Compute::Scale(temp, dz, m_learningRate);
    Compute::Sub(z, z, temp);
}
}  // namespace Sapphire::Optimizer

namespace Sapphire::BackProp
{
using TensorUtil::TensorData;

namespace
{
void RunReference(TensorData& dx, TensorData& weight, TensorData& bias, const TensorData& dy,
                  const TensorData& x, unsigned int batchSize, const Optimizer::SGD& optimizer)
{
    // dx += dy * weight^T
    TensorData weightTranspose(weight.GetShape().GetTranspose(), weight.GetType(),
                               weight.GetCudaDevice());
    weightTranspose.SetMode(weight.Mode());
    Compute::Transpose(weightTranspose, weight);
    Compute::Gemm(dx, dy, weightTranspose);

    // dw = x^T * dy, then the weight update
    TensorData xTranspose(x.GetShape().GetTranspose(), x.GetType(), x.GetCudaDevice());
    TensorData dw(weight.GetShape(), weight.GetType(), weight.GetCudaDevice());
    xTranspose.SetMode(x.Mode());
    dw.SetMode(weight.Mode());
    Compute::Transpose(xTranspose, x);
    Compute::Initialize::Zeros(dw);
    Compute::Gemm(dw, xTranspose, dy);
    optimizer(weight, dw);

    // dB = column sums of dy / batch, then the bias update
    TensorData transposedOnes(Shape({ 1, static_cast<int>(batchSize) }), dy.GetType(),
                              dy.GetCudaDevice());
    TensorData dB(bias.GetShape(), bias.GetType(), bias.GetCudaDevice());
    dB.SetMode(bias.Mode());
    transposedOnes.SetMode(bias.Mode());
    Compute::Initialize::Ones(transposedOnes);
    Compute::Initialize::Zeros(dB);
    Compute::Gemm(dB, transposedOnes, dy);
    Compute::Scale(dB, dB, 1.0f / static_cast<float>(batchSize));
    optimizer(bias, dB);
}

void RunDirect(TensorData& dx, TensorData& weight, TensorData& bias, const TensorData& dy,
               const TensorData& x, unsigned int batchSize, const Optimizer::SGD& optimizer)
{
    const int deviceId = dx.GetCudaDevice().GetID();
    const unsigned int inputs = static_cast<unsigned int>(weight.Rows());
    const unsigned int outputs = static_cast<unsigned int>(weight.Cols());
    const unsigned int rows = static_cast<unsigned int>(dy.Size()) / outputs;

    // dx [rows, in] += dy [rows, out] * (weight [in, out])^T
    // (a fresh dx is stored into instead of filled, read and added to)
    const bool dxFresh = static_cast<std::size_t>(dx.Size()) ==
                             static_cast<std::size_t>(rows) * inputs &&
                         dx.TakeDeferredZero();
    Compute::Dense::Cuda::GemmTransposed(dxFresh ? dx.CudaOverwriteRawPtr() : dx.CudaMutableRawPtr(),
                                         dy.CudaRawPtr(), weight.CudaRawPtr(), rows, inputs,
                                         outputs, 1, false, true, dxFresh, deviceId);

    // dB [1, out] = ones [1, batch] * dy, the ones that Linear's backward pass fills
    TensorData transposedOnes(Shape({ 1, static_cast<int>(batchSize) }), dy.GetType(),
                              dy.GetCudaDevice());
    transposedOnes.SetMode(bias.Mode());
    Compute::Initialize::Ones(transposedOnes);

    if (optimizer.Fused())
    {
        // neither gradient is stored: the products end in the optimizer's step
        // weight -= ((x^T * dy) * 1) * lr;  bias -= ((ones * dy) * (1 / batch)) * lr
        Compute::Dense::Cuda::GemmSgd(weight.CudaMutableRawPtr(), x.CudaRawPtr(), dy.CudaRawPtr(),
                                      inputs, outputs, rows, true, false, 1.0f,
                                      optimizer.LearningRate(), deviceId);
        Compute::Dense::Cuda::GemmSgd(bias.CudaMutableRawPtr(), transposedOnes.CudaRawPtr(),
                                      dy.CudaRawPtr(), 1, outputs, batchSize, false, false,
                                      1.0f / static_cast<float>(batchSize),
                                      optimizer.LearningRate(), deviceId);
        return;
    }

    // dw [in, out] = (x [rows, in])^T * dy [rows, out]
    TensorData dw(weight.GetShape(), weight.GetType(), weight.GetCudaDevice());
    dw.SetMode(weight.Mode());
    Compute::Dense::Cuda::GemmTransposed(dw.CudaOverwriteRawPtr(), x.CudaRawPtr(), dy.CudaRawPtr(),
                                         inputs, outputs, rows, 1, true, false, true, deviceId);
    optimizer(weight, dw);

    TensorData dB(bias.GetShape(), bias.GetType(), bias.GetCudaDevice());
    dB.SetMode(bias.Mode());
    Compute::Dense::Cuda::GemmTransposed(dB.CudaOverwriteRawPtr(), transposedOnes.CudaRawPtr(),
                                         dy.CudaRawPtr(), 1, outputs, batchSize, 1, false, false,
                                         true, deviceId);
    Compute::Scale(dB, dB, 1.0f / static_cast<float>(batchSize));
    optimizer(bias, dB);
}
}  // namespace

void LinearBackward(TensorData& dx, TensorData& weight, TensorData& bias, const TensorData& dy,
                    const TensorData& x, unsigned int batchSize, const Optimizer::SGD& optimizer,
                    Sequence sequence)
{
    if (dx.Mode() != dy.Mode() || dx.Mode() != x.Mode() || dx.Mode() != weight.Mode() ||
        dx.Mode() != bias.Mode())
        throw std::invalid_argument("BackProp::Linear - Device mode inequality");
    if (dx.Mode() != ComputeMode::Cuda)
        throw std::runtime_error(
            "BackProp::Linear - Host mode is not provided by the device backend");
    if (batchSize == 0)
        throw std::invalid_argument("BackProp::Linear - batch size is zero");
    if (sequence == Sequence::Reference)
        RunReference(dx, weight, bias, dy, x, batchSize, optimizer);
    else
        RunDirect(dx, weight, bias, dy, x, batchSize, optimizer);
}
}  // namespace Sapphire::BackProp
