// Forward pass of the fully connected layer on TensorData, i.e. the compute part of
// NN::Linear::operator() (Sources/Sapphire/operations/Forward/Linear.cpp:113-136) without the
// autograd bookkeeping around it:
//
//     ones = [batch, 1] filled with 1            (Linear.cpp:113-118)
//     x, y, bias viewed as 2-D                   (Linear.cpp:121, Util::ChangeTensorDataDimension)
//     Gemm(y, ones, bias)    K = 1, adds the bias to every row   (Linear.cpp:134)
//     Gemm(y, x, weight)     weight stored [in, out]             (Linear.cpp:136)
//
// y is expected to hold zeros on entry (a fresh TensorData does).
#ifndef SAPPHIRE_AMD_OPERATIONS_FORWARD_LINEARFORWARD_HPP
#define SAPPHIRE_AMD_OPERATIONS_FORWARD_LINEARFORWARD_HPP

#include <Sapphire/compute/sparse/SparseMatrix.hpp>
#include <Sapphire/tensor/TensorData.hpp>

namespace Sapphire::Util
{
//! Views `data` with exactly `dimension` extents: Expand then Shrink of its shape
//! (Includes/Sapphire/util/UnitUtils.hpp:18-36).
void ChangeTensorDataDimension(int dimension, TensorUtil::TensorData& data);
}  // namespace Sapphire::Util

namespace Sapphire::NN
{
void LinearForward(TensorUtil::TensorData& y, const TensorUtil::TensorData& x,
                   const TensorUtil::TensorData& weight, const TensorUtil::TensorData& bias);

//! The same layer as one launch: the bias row and, with `relu`, the activation that follows
//! the layer (Compute::ReLU) are applied where the product is stored.  y is overwritten; the
//! result has the bits of LinearForward on a zero y followed by Compute::ReLU.
void LinearForwardFused(TensorUtil::TensorData& y, const TensorUtil::TensorData& x,
                        const TensorUtil::TensorData& weight,
                        const TensorUtil::TensorData& bias, bool relu);

//! The same layer with a sparse weight, the variant NN::Linear rejects with
//! "Sparse version not implemented" (Sources/Sapphire/operations/Forward/Linear.cpp:28-30).
//! `weightTransposed` is a device record of the transposed weight, [out, in] in CSR, so that
//! the CSR x dense kernel applies:  y^T [out, batch] = bias * ones[1, batch] (K = 1 GEMM),
//! y^T += weightTransposed * x^T, y = transpose(y^T).  y is overwritten; the result equals
//! LinearForward on the densified weight with a zero y, bit for bit on the CPU contract
//! (entries in ascending input index, products and sums rounded separately).
void SparseLinearForward(TensorUtil::TensorData& y, const TensorUtil::TensorData& x,
                         const SparseMatrix& weightTransposed,
                         const TensorUtil::TensorData& bias);
}  // namespace Sapphire::NN

#endif
