// Allocation, copies and dense <-> CSR conversion of SparseMatrix records, with the names the
// reference declares (Includes/Sapphire/compute/sparse/Sparse.hpp:20-162) and never defines.
//
// A "host" record has its V / COL / ROW arrays in host memory; a "device" record is the same
// 48-byte struct, kept in host memory, whose three arrays are device memory -- the form the
// kernels behind the C ABI take (they receive the arrays, not the struct).  Arrays come from
// ResourceManager's preserved pools.  The LoadDistMatrix overloads (Sparse.hpp:28, 41, 59, 75,
// 102, 118, 135, 150 of the reference) do the same for the load-distribution records of the
// sparse x sparse product.
#ifndef SAPPHIRE_AMD_COMPUTE_SPARSE_SPARSE_HPP
#define SAPPHIRE_AMD_COMPUTE_SPARSE_SPARSE_HPP

#include <Sapphire/compute/sparse/SparseMatrix.hpp>

#include <cstdint>

namespace Sapphire::Compute
{
//! numMatrices host records of m x n with nnz[i] entries each (arrays zero-filled).
void DeepAllocateSparseHost(SparseMatrix** sparseMatrixArray, uint32_t m, uint32_t n,
                            const uint32_t nnz[], uint32_t numMatrices);
void DeepFreeSparseHost(SparseMatrix* sparseMatrixArray, uint32_t numMatrices);

//! Device records with the sizes of the given host records (contents not copied).
void DeepAllocateSparseCuda(SparseMatrix** deviceSparseArray,
                            const SparseMatrix* hostSparseMatrixArray, uint32_t numMatrices,
                            int deviceId);
void DeepFreeSparseCuda(SparseMatrix* deviceSparseArray, uint32_t numMatrices, int deviceId);

//! Copies of V, COL, ROW and the three counters; destination records must have been allocated
//! with at least the source's NNZ and M.  Throws std::invalid_argument otherwise.
void DeepCopyHostToDevice(SparseMatrix* deviceDstArray, const SparseMatrix* hostSrcArray,
                          uint32_t numMatrices, int deviceId);
void DeepCopyDeviceToHost(SparseMatrix* hostDstArray, const SparseMatrix* deviceSrcArray,
                          uint32_t numMatrices, int deviceId);
void DeepCopyDeviceToDevice(SparseMatrix* deviceDstArray, const SparseMatrix* deviceSrcArray,
                            uint32_t numMatrices, int deviceId);
void DeepCopyHostToHost(SparseMatrix* hostDstArray, const SparseMatrix* hostSrcArray,
                        uint32_t numMatrices);

//! Load-distribution records with the shape and entry counts of the given sparse records
//! (arrays zero-filled on the host, not initialised on the device).
void DeepAllocateLoadDistHost(LoadDistMatrix** loadDistArray, SparseMatrix* sparseArray,
                              uint32_t numMatrices);
void DeepFreeLoadDistHost(LoadDistMatrix* loadDistArray, uint32_t numMatrices);
void DeepAllocateLoadDistCuda(LoadDistMatrix** deviceLoadDistArray,
                              LoadDistMatrix* hostLoadDistArray, uint32_t numMatrices,
                              int deviceId);
void DeepFreeLoadDistCuda(LoadDistMatrix* deviceLoadDistArray, uint32_t numMatrices,
                          int deviceId);
void DeepCopyDeviceToDevice(LoadDistMatrix* deviceDstArray, LoadDistMatrix* deviceSrcArray,
                            uint32_t numMatrices, int deviceId);
void DeepCopyHostToDevice(LoadDistMatrix* deviceDstArray, LoadDistMatrix* hostSrcArray,
                          uint32_t numMatrices, int deviceId);
void DeepCopyDeviceToHost(LoadDistMatrix* hostDstArray, LoadDistMatrix* deviceSrcArray,
                          uint32_t numMatrices, int deviceId);
void DeepCopyHostToHost(LoadDistMatrix* hostDstArray, LoadDistMatrix* hostSrcArray,
                        uint32_t numMatrices);

//! Builds numMatrices device records from dense matrices in device memory: matrix i starts at
//! src + i * m * paddedN, rows are paddedN floats apart, the first n columns count.  Entries
//! with value != 0 are kept, ascending columns.  Release with DeepFreeSparseCuda.
void CreateSparseMatrixWithDenseMatrix(SparseMatrix** dst, const float* src, uint32_t m,
                                       uint32_t n, uint32_t paddedN, uint32_t numMatrices,
                                       int deviceId);

//! The inverse, into pre-allocated device memory of numMatrices * m * paddedN floats; the
//! padding columns are left as they are.
void ConvertSparseMatrixToDenseMatrix(float* dst, const SparseMatrix* src, uint32_t m, uint32_t n,
                                      uint32_t paddedN, uint32_t numMatrices, int deviceId);
}  // namespace Sapphire::Compute

#endif
