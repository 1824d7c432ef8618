// Backward pass of the matrix product y = a * b on TensorData: the compute part of
// BackProp::MulBackProp::m_runBackProp
// (Sources/Sapphire/operations/Backward/MathBackward.cpp:35-51):
//
//     da += dy * b^T          (Transpose(transposedB, b); Gemm(da, dy, transposedB))
//     db += a^T * dy          (Transpose(transposedA, a); Gemm(db, transposedA, dy))
//
// Sequence::Reference issues those four operator calls.  Sequence::Direct reads a and b
// transposed inside the matrix kernel instead (same bits); it applies when a, b and dy have
// the same leading (batch) dimensions and falls back to the reference sequence otherwise.
#ifndef SAPPHIRE_AMD_OPERATIONS_BACKWARD_MATHBACKWARD_HPP
#define SAPPHIRE_AMD_OPERATIONS_BACKWARD_MATHBACKWARD_HPP

#include <Sapphire/operations/Backward/LinearBackward.hpp>
#include <Sapphire/tensor/TensorData.hpp>

namespace Sapphire::BackProp
{
void MatMulBackward(TensorUtil::TensorData& da, TensorUtil::TensorData& db,
                    const TensorUtil::TensorData& dy, const TensorUtil::TensorData& a,
                    const TensorUtil::TensorData& b, Sequence sequence = Sequence::Direct);
}  // namespace Sapphire::BackProp

#endif
