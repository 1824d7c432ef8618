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

//! out[a->M x denseCols] = (0 + rowBias[i]) + a * B: the product accumulated into an out that
//! holds the bias of row i in every column, without reading out (the feature-major bias step of
//! a sparse Linear layer in the same launch).  rowBias has a->M entries in device memory.
void GemmBias(float* out, const SparseMatrix* a, const float* B, unsigned int denseCols,
              const float* rowBias, int deviceId);

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
//! nullptr.  Sums that are exactly zero are not stored; columns ascend within a row.  The number
//! of products of a pair (the load-distribution pre-pass) bounds the entries of its result, so
//! V and COL are allocated for that bound and the products are computed once; a result with
//! less than half of the bound in use is moved to arrays of its own size.
void Gemm(SparseMatrix** hostOutput, SparseMatrix** cudaOutput, SparseMatrix* cudaA,
          SparseMatrix* cudaB, uint32_t m, uint32_t n, std::size_t numMatrices, int deviceId,
          bool copyResultToHost);

//! The load-distribution pre-pass of the sparse x sparse product, with the signatures the
//! reference declares (Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:16-18, 43-46).
//! CallLoadDist: a, b and loadDist are arrays of device records (loadDist[i] allocated with the
//! shape and entry count of a[i], e.g. by Compute::DeepAllocateLoadDistCuda); loadDist[i]
//! receives a[i]'s COL and ROW and, per entry, the number of entries in the row of b[i] it
//! selects -- the multiplications that entry causes.  nnzArray[i] (host, may be null) receives
//! the number of products of pair i, which bounds the entries of a[i] * b[i] from above
//! (saturated at 2^32 - 1).  M is the row count of every a[i].
void CallLoadDist(SparseMatrix* a, SparseMatrix* b, LoadDistMatrix* loadDist, uint32_t M,
                  uint32_t* nnzArray, std::size_t numMatrices, int deviceId);
//! GetLoadDist: the same into host records (allocated like cudaA, e.g. by
//! Compute::DeepAllocateLoadDistHost); the device records it needs are temporary.
void GetLoadDist(LoadDistMatrix* hostLoadDist, SparseMatrix* cudaA, SparseMatrix* cudaB,
                 uint32_t m, std::size_t numMatrices, int deviceId);
}  // namespace Sapphire::Compute::Sparse::Cuda

namespace Sapphire::Compute
{
//! y (+)= a * b where a is a Type::Sparse tensor whose SparseMatCuda record is set and y, b
//! are dense tensors in Cuda mode: the TensorData-level form of the product above.
void SparseGemm(TensorUtil::TensorData& y, const TensorUtil::TensorData& a,
                const TensorUtil::TensorData& b, bool accumulate = true);
}  // namespace Sapphire::Compute

#endif
