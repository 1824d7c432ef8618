#include <Sapphire/compute/sparse/SparseGemm.hpp>

#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/util/ResourceManager.hpp>

#include <sapphire_hip.h>

#include <stdexcept>
#include <string>

namespace Sapphire::Compute::Sparse::Cuda
{
void Gemm(float* out, const SparseMatrix* a, const float* B, unsigned int denseCols,
          bool accumulate, int deviceId)
{
    if (a == nullptr)
        throw std::invalid_argument("Sparse::Cuda::Gemm - sparse operand is null");
    Compute::Cuda::CudaSetDevice(deviceId);
    if (sph_spmm_csr_f32(out, a->V, a->COL, a->ROW, a->M, a->N, denseCols, B,
                         accumulate ? 1 : 0) != SPH_OK)
        throw std::runtime_error(std::string("Sparse::Cuda::Gemm failed with ") +
                                 sph_last_error());
}

SparseMatrix CreateSparseMatrix(const std::vector<float>& values,
                                const std::vector<uint32_t>& columns,
                                const std::vector<uint32_t>& rowOffsets, uint32_t rows,
                                uint32_t cols, int deviceId)
{
    if (rowOffsets.size() != static_cast<std::size_t>(rows) + 1)
        throw std::invalid_argument("CreateSparseMatrix - rowOffsets must hold rows + 1 entries");
    if (values.size() != columns.size() || values.size() != rowOffsets.back())
        throw std::invalid_argument("CreateSparseMatrix - value / column / offset counts disagree");
    Compute::Cuda::CudaSetDevice(deviceId);
    SparseMatrix m{};
    m.NNZ = static_cast<uint32_t>(values.size());
    m.M = rows;
    m.N = cols;
    const std::size_t nnzBytes = std::max<std::size_t>(values.size(), 1) * 4;
    m.V = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(nnzBytes, true));
    m.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(nnzBytes, true));
    m.ROW = static_cast<uint32_t*>(
        Util::ResourceManager::GetMemoryCuda(rowOffsets.size() * 4, true));
    Compute::Cuda::CopyHostToDevice(m.V, values.data(), values.size() * 4);
    Compute::Cuda::CopyHostToDevice(m.COL, columns.data(), columns.size() * 4);
    Compute::Cuda::CopyHostToDevice(m.ROW, rowOffsets.data(), rowOffsets.size() * 4);
    return m;
}

void FreeSparseMatrix(SparseMatrix& matrix)
{
    Compute::Cuda::Synchronize();
    if (matrix.V != nullptr)
        Util::ResourceManager::FreePreservedCuda(matrix.V);
    if (matrix.COL != nullptr)
        Util::ResourceManager::FreePreservedCuda(matrix.COL);
    if (matrix.ROW != nullptr)
        Util::ResourceManager::FreePreservedCuda(matrix.ROW);
    matrix = SparseMatrix{};
}
}  // namespace Sapphire::Compute::Sparse::Cuda

namespace Sapphire::Compute
{
void SparseGemm(TensorUtil::TensorData& y, const TensorUtil::TensorData& a,
                const TensorUtil::TensorData& b, bool accumulate)
{
    if (y.Mode() != ComputeMode::Cuda || b.Mode() != ComputeMode::Cuda)
        throw std::runtime_error(
            "Compute::SparseGemm - Host mode is not provided by the device backend");
    if (a.SparseMatCuda == nullptr)
        throw std::invalid_argument("Compute::SparseGemm - sparse operand has no device record");
    const SparseMatrix* m = a.SparseMatCuda;
    if (static_cast<uint32_t>(b.Rows()) != m->N || static_cast<uint32_t>(y.Rows()) != m->M ||
        y.Cols() != b.Cols())
        throw std::invalid_argument("Compute::SparseGemm - shape mismatch");
    Sparse::Cuda::Gemm(y.CudaMutableRawPtr(), m, b.CudaRawPtr(),
                       static_cast<unsigned int>(b.Cols()), accumulate,
                       y.GetCudaDevice().GetID());
}
}  // namespace Sapphire::Compute
