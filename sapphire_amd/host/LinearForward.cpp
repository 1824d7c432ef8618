#include <Sapphire/operations/Forward/LinearForward.hpp>

#include <Sapphire/compute/BasicOps.hpp>
#include <Sapphire/compute/Initialize.hpp>

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
}  // namespace Sapphire::NN
