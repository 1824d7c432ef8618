// Sparse (CSR) x dense product on the device.
//
// The reference declares sparse containers and a sparse x sparse product
// (Includes/Sapphire/compute/sparse/Sparse.hpp:20-162,
//  Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:16-100) but defines none of them and
// has no sparse x dense product at all.  This entry sits beside those declarations, takes the
// reference's SparseMatrix record and produces what its dense leaf would produce on the
// densified matrix, bit for bit.
#ifndef SAPPHIRE_AMD_COMPUTE_SPARSE_SPARSEGEMM_HPP
#define SAPPHIRE_AMD_COMPUTE_SPARSE_SPARSEGEMM_HPP

#include <Sapphire/compute/sparse/SparseMatrix.hpp>
#include <Sapphire/tensor/TensorData.hpp>

#include <cstddef>
#include <vector>

namespace Sapphire::Compute::Sparse::Cuda
{
//! out[a->M x denseCols] (+)= a * B[a->N x denseCols].  `a` is a host-side record whose V,
//! COL and ROW arrays are device memory; out and B are device memory.  With accumulate false
//! the product is stored (rows without entries become 0), otherwise added into out.
void Gemm(float* out, const SparseMatrix* a, const float* B, unsigned int denseCols,
          bool accumulate, int deviceId);

//! Builds a record with device arrays from host CSR arrays (rowOffsets has rows + 1
//! entries, columns ascending inside a row); memory comes from ResourceManager's
//! preserved device pool.  Release with FreeSparseMatrix.
SparseMatrix CreateSparseMatrix(const std::vector<float>& values,
                                const std::vector<uint32_t>& columns,
                                const std::vector<uint32_t>& rowOffsets, uint32_t rows,
                                uint32_t cols, int deviceId);
void FreeSparseMatrix(SparseMatrix& matrix);

//! Sparse x sparse: output i = cudaA[i] * cudaB[i] for numMatrices device records of shapes
//! m x k and k x n, with the signature the reference declares
//! (Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:38-42).  *cudaOutput receives a new
//! array of device records (release with Compute::DeepFreeSparseCuda); with copyResultToHost
//! *hostOutput receives host copies (release with Compute::DeepFreeSparseHost), otherwise
//! nullptr.  Sums that are exactly zero are not stored; columns ascend within a row.
void Gemm(SparseMatrix** hostOutput, SparseMatrix** cudaOutput, SparseMatrix* cudaA,
          SparseMatrix* cudaB, uint32_t m, uint32_t n, std::size_t numMatrices, int deviceId,
          bool copyResultToHost);
}  // namespace Sapphire::Compute::Sparse::Cuda

namespace Sapphire::Compute
{
//! y (+)= a * b where a is a Type::Sparse tensor whose SparseMatCuda record is set and y, b
//! are dense tensors in Cuda mode: the TensorData-level form of the product above.
void SparseGemm(TensorUtil::TensorData& y, const TensorUtil::TensorData& a,
                const TensorUtil::TensorData& b, bool accumulate = true);
}  // namespace Sapphire::Compute

#endif
