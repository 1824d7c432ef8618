// Backward pass and parameter update of the fully connected layer on TensorData: the compute
// part of BackProp::LinearBackProp::m_runBackProp
// (Sources/Sapphire/operations/Backward/LinearBackward.cpp:27-99) without the autograd
// bookkeeping around it.  With x [batch, in], weight [in, out], bias [out], dy [batch, out]:
//
//     dx     += dy * weight^T                                   (LinearBackward.cpp:37-51)
//     dw      = x^T * dy;           weight <- optimizer(weight, dw)   (:53-77)
//     dB      = ones[1, batch] * dy; dB *= 1 / batch;
//                                   bias   <- optimizer(bias, dB)     (:79-99)
//
// in that order, so dx is formed with the weights from before the update.
//
// Sequence::Reference issues exactly the reference's operator calls: it materialises both
// transposes, zero-fills dw and dB and accumulates into them.  Sequence::Direct reads the
// stored operands transposed inside the matrix kernel and stores dw and dB without the
// zero-fill; the K products of every element are still added in the same order, so both
// sequences give the same bits.
#ifndef SAPPHIRE_AMD_OPERATIONS_BACKWARD_LINEARBACKWARD_HPP
#define SAPPHIRE_AMD_OPERATIONS_BACKWARD_LINEARBACKWARD_HPP

#include <Sapphire/operations/optimizers/SGD.hpp>
#include <Sapphire/tensor/TensorData.hpp>

namespace Sapphire::BackProp
{
enum class Sequence
{
    Reference,
    Direct,
};

void LinearBackward(TensorUtil::TensorData& dx, TensorUtil::TensorData& weight,
                    TensorUtil::TensorData& bias, const TensorUtil::TensorData& dy,
                    const TensorUtil::TensorData& x, unsigned int batchSize,
                    const Optimizer::SGD& optimizer, Sequence sequence = Sequence::Direct);
}  // namespace Sapphire::BackProp

#endif
