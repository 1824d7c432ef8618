// Constant fills.
//
//   Dense::Cuda::Scalar   raw device fill, the reference's launcher of the same name
//                         (Sources/Sapphire/compute/dense/cuda/Initialize.cu:46-59)
//   Initialize::Ones / Zeros / Scalar   TensorData-level fills in the tensor's current mode
//                         (Sources/Sapphire/compute/Initialize.cpp), used by Linear
//                         (Sources/Sapphire/operations/Forward/Linear.cpp:118,133)
#ifndef SAPPHIRE_AMD_COMPUTE_INITIALIZE_HPP
#define SAPPHIRE_AMD_COMPUTE_INITIALIZE_HPP

#include <cstddef>

namespace Sapphire::TensorUtil
{
class TensorData;
}

namespace Sapphire::Compute::Dense::Cuda
{
void Scalar(float* data, float value, std::size_t size);
}

namespace Sapphire::Compute::Initialize
{
void Scalar(TensorUtil::TensorData& data, float value);
void Ones(TensorUtil::TensorData& data);
void Zeros(TensorUtil::TensorData& data);
}  // namespace Sapphire::Compute::Initialize

#endif
