// Operator-level entry points on TensorData, with the reference's signatures
// (Includes/Sapphire/compute/BasicOps.hpp:16-31, Includes/Sapphire/compute/ActivationOps.hpp).
//
// Only the device branch lives here.  The reference's Host branch (its scalar CPU loops)
// stays where it is in the reference; calling these with tensors in ComputeMode::Host throws
// std::runtime_error, there is no CPU fallback in this library.
#ifndef SAPPHIRE_AMD_COMPUTE_BASICOPS_HPP
#define SAPPHIRE_AMD_COMPUTE_BASICOPS_HPP

#include <Sapphire/tensor/TensorData.hpp>

#include <cstdint>

namespace Sapphire::Compute
{
using TensorUtil::TensorData;

//! y += a * b over the trailing two dimensions, leading dimensions broadcast by the walk of
//! BroadcastWith2Inputs.  No shape validation, as documented for the reference
//! (Includes/Sapphire/compute/BasicOps.hpp:16-19).  All three must be in the same mode.
void Gemm(TensorData& y, const TensorData& a, const TensorData& b);

//! y += a * b with half-precision operands and fp32 accumulation, the operand form of the
//! tensor-core product the reference declares (WmmaGemm,
//! Includes/Sapphire/compute/dense/cuda/kernels/GemmKernel.cuh:14-50).  TensorData holds fp32
//! only, so a and b are device arrays of IEEE binary16 bit patterns: a is [batch, M, K], b is
//! [batch, K, N] with M, N the trailing dimensions of y and batch its leading ones, packed back
//! to back.  A fresh y (zero fill still deferred) receives the product without being read.
void GemmHalf(TensorData& y, const std::uint16_t* a, const std::uint16_t* b, unsigned int K);

//! y = transpose of the trailing two dimensions of x; a 2-D x is repeated for every matrix
//! of y (Sources/Sapphire/compute/BasicOps.cpp:269-290).
void Transpose(TensorData& y, const TensorData& x);

//! y = x > 0 ? x : 0 (Sources/Sapphire/compute/ActivationOps.cpp:52-67).
void ReLU(TensorData& y, const TensorData& x);

//! dx += x > 0 ? dy : 0 (Sources/Sapphire/compute/ActivationOps.cpp:69-85).
void ReLUBackward(TensorData& dx, const TensorData& dy, const TensorData& x);

//! y = x * factor over y's element count (Sources/Sapphire/compute/BasicOps.cpp:250-267).
void Scale(TensorData& y, const TensorData& x, float factor);

//! y = a - b.  The trailing dimensions on which the three shapes agree form one leaf; the
//! leading ones are walked by BroadcastWith2Inputs, operands offset by
//! (index % extent) * stride (Sources/Sapphire/compute/BasicOps.cpp:63-103).
void Sub(TensorData& y, const TensorData& a, const TensorData& b);
}  // namespace Sapphire::Compute

#endif
