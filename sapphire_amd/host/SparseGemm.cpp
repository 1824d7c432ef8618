#include <Sapphire/compute/sparse/SparseGemm.hpp>

#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/compute/sparse/Sparse.hpp>
#include <Sapphire/util/ResourceManager.hpp>

#include <sapphire_hip.h>

#include <algorithm>
#include <stdexcept>
#include <string>
#include <vector>

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

void GemmBias(float* out, const SparseMatrix* a, const float* B, unsigned int denseCols,
              const float* rowBias, int deviceId)
{
    if (a == nullptr)
        throw std::invalid_argument("Sparse::Cuda::GemmBias - sparse operand is null");
    Compute::Cuda::CudaSetDevice(deviceId);
    if (sph_spmm_csr_bias_f32(out, a->V, a->COL, a->ROW, a->M, a->N, denseCols, B, rowBias) !=
        SPH_OK)
        throw std::runtime_error(std::string("Sparse::Cuda::GemmBias failed with ") +
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

void CallLoadDist(SparseMatrix* a, SparseMatrix* b, LoadDistMatrix* loadDist, uint32_t M,
                  uint32_t* nnzArray, std::size_t numMatrices, int deviceId)
{
    if (a == nullptr || b == nullptr || loadDist == nullptr)
        throw std::invalid_argument("Sparse::Cuda::CallLoadDist - null array");
    Compute::Cuda::CudaSetDevice(deviceId);
    for (std::size_t i = 0; i < numMatrices; ++i)
    {
        const SparseMatrix& left = a[i];
        const SparseMatrix& right = b[i];
        LoadDistMatrix& d = loadDist[i];
        if (left.M != M || left.N != right.M)
            throw std::invalid_argument("Sparse::Cuda::CallLoadDist - shape mismatch");
        if (d.Load == nullptr || d.COL == nullptr || d.ROW == nullptr || d.NNZ < left.NNZ ||
            d.M < left.M)
            throw std::invalid_argument("Sparse::Cuda::CallLoadDist - record is too small");
        Compute::Cuda::CopyDeviceToDevice(d.COL, left.COL, static_cast<std::size_t>(left.NNZ) * 4);
        Compute::Cuda::CopyDeviceToDevice(d.ROW, left.ROW,
                                          (static_cast<std::size_t>(left.M) + 1) * 4);
        d.NNZ = left.NNZ;
        d.M = left.M;
        d.N = left.N;
        uint64_t products = 0;
        if (sph_spgemm_load_u32(d.Load, left.COL, right.ROW, left.NNZ, right.M,
                                nnzArray != nullptr ? &products : nullptr) != SPH_OK)
            throw std::runtime_error(std::string("Sparse::Cuda::CallLoadDist failed with ") +
                                     sph_last_error());
        if (nnzArray != nullptr)
            nnzArray[i] = static_cast<uint32_t>(std::min<uint64_t>(products, 0xffffffffull));
    }
}

void GetLoadDist(LoadDistMatrix* hostLoadDist, SparseMatrix* cudaA, SparseMatrix* cudaB,
                 uint32_t m, std::size_t numMatrices, int deviceId)
{
    if (hostLoadDist == nullptr)
        throw std::invalid_argument("Sparse::Cuda::GetLoadDist - null array");
    const auto count = static_cast<uint32_t>(numMatrices);
    LoadDistMatrix* device = nullptr;
    DeepAllocateLoadDistCuda(&device, hostLoadDist, count, deviceId);
    try
    {
        CallLoadDist(cudaA, cudaB, device, m, nullptr, numMatrices, deviceId);
        DeepCopyDeviceToHost(hostLoadDist, device, count, deviceId);
    }
    catch (...)
    {
        DeepFreeLoadDistCuda(device, count, deviceId);
        throw;
    }
    DeepFreeLoadDistCuda(device, count, deviceId);
}

void Gemm(SparseMatrix** hostOutput, SparseMatrix** cudaOutput, SparseMatrix* cudaA,
          SparseMatrix* cudaB, uint32_t m, uint32_t n, std::size_t numMatrices, int deviceId,
          bool copyResultToHost)
{
    if (cudaOutput == nullptr || (copyResultToHost && hostOutput == nullptr))
        throw std::invalid_argument("Sparse::Cuda::Gemm - output pointer is null");
    Compute::Cuda::CudaSetDevice(deviceId);
    const auto count = static_cast<uint32_t>(numMatrices);
    auto* result = new SparseMatrix[count]();
    auto check = [&](int status) {
        if (status != SPH_OK)
            throw std::runtime_error(std::string("Sparse::Cuda::Gemm failed with ") +
                                     sph_last_error());
    };
    try
    {
        // The number of products of a pair bounds the entries of its result; with room for that
        // many the products are computed once (the counting pass stages every row).  Reading
        // that bound back drains the stream once per matrix (a small kernel each); the products
        // themselves are all enqueued before any entry count is read back, so they cost one
        // more drain for the whole batch.  When the arrays for the bound (or the staging area
        // behind sph_spgemm_f32, 8 bytes per bounded entry and more) cannot be had, the matrix
        // falls back to the two passes: count, allocate exactly, fill.
        std::vector<uint32_t> capacity(count);
        std::vector<bool> exact(count, false);
        auto twoPasses = [&](uint32_t i) {
            const SparseMatrix& a = cudaA[i];
            const SparseMatrix& b = cudaB[i];
            SparseMatrix& c = result[i];
            uint32_t nnz = 0;
            check(sph_spgemm_row_offsets_f32(c.ROW, a.V, a.COL, a.ROW, b.V, b.COL, b.ROW, m, a.N,
                                             n, &nnz));
            const std::size_t exactBytes = std::max<std::size_t>(nnz, 1) * 4;
            c.V = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(exactBytes, true));
            c.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(exactBytes, true));
            check(sph_spgemm_fill_f32(c.V, c.COL, c.ROW, a.V, a.COL, a.ROW, b.V, b.COL, b.ROW, m,
                                      a.N, n));
            c.NNZ = nnz;
            capacity[i] = nnz;
            exact[i] = true;
        };
        for (uint32_t i = 0; i < count; ++i)
        {
            const SparseMatrix& a = cudaA[i];
            const SparseMatrix& b = cudaB[i];
            if (a.M != m || b.N != n || a.N != b.M)
                throw std::invalid_argument("Sparse::Cuda::Gemm - shape mismatch");
            uint64_t products = 0;
            check(sph_spgemm_load_u32(nullptr, a.COL, b.ROW, a.NNZ, b.M, &products));
            capacity[i] = static_cast<uint32_t>(std::min<uint64_t>(
                { products, static_cast<uint64_t>(m) * n, 0xffffffffull }));
        }
        for (uint32_t i = 0; i < count; ++i)
        {
            const SparseMatrix& a = cudaA[i];
            const SparseMatrix& b = cudaB[i];
            SparseMatrix& c = result[i];
            c.M = m;
            c.N = n;
            c.ROW = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(
                (static_cast<std::size_t>(m) + 1) * 4, true));
            const std::size_t bytes = std::max<std::size_t>(capacity[i], 1) * 4;
            bool oneCall = true;
            try
            {
                c.V = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(bytes, true));
                c.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(bytes, true));
                oneCall = sph_spgemm_f32(c.V, c.COL, c.ROW, capacity[i], a.V, a.COL, a.ROW, b.V,
                                         b.COL, b.ROW, m, a.N, n, nullptr) == SPH_OK;
            }
            catch (const std::runtime_error&)
            {
                oneCall = false;  // no memory for the bound
            }
            if (!oneCall)
            {
                if (c.V != nullptr)
                    Util::ResourceManager::FreePreservedCuda(c.V);
                if (c.COL != nullptr)
                    Util::ResourceManager::FreePreservedCuda(c.COL);
                c.V = nullptr;
                c.COL = nullptr;
                twoPasses(i);
            }
        }
        for (uint32_t i = 0; i < count; ++i)
        {
            SparseMatrix& c = result[i];
            if (exact[i])
                continue;
            uint32_t nnz = 0;
            Compute::Cuda::CopyDeviceToHost(&nnz, c.ROW + m, sizeof(nnz));
            c.NNZ = nnz;
            if (static_cast<uint64_t>(nnz) * 2 < capacity[i] && capacity[i] > 1024)
            {
                // mostly unused: move the entries to arrays of their own size
                const std::size_t bytes = std::max<std::size_t>(nnz, 1) * 4;
                auto* v = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(bytes, true));
                auto* col = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(bytes, true));
                Compute::Cuda::CopyDeviceToDevice(v, c.V, static_cast<std::size_t>(nnz) * 4);
                Compute::Cuda::CopyDeviceToDevice(col, c.COL, static_cast<std::size_t>(nnz) * 4);
                Util::ResourceManager::FreePreservedCuda(c.V);
                Util::ResourceManager::FreePreservedCuda(c.COL);
                c.V = v;
                c.COL = col;
            }
        }
        if (copyResultToHost)
        {
            std::vector<uint32_t> counts(count);
            for (uint32_t i = 0; i < count; ++i)
                counts[i] = result[i].NNZ;
            DeepAllocateSparseHost(hostOutput, m, n, counts.data(), count);
            DeepCopyDeviceToHost(*hostOutput, result, count, deviceId);
        }
        else if (hostOutput != nullptr)
            *hostOutput = nullptr;
    }
    catch (...)
    {
        DeepFreeSparseCuda(result, count, deviceId);
        throw;
    }
    *cudaOutput = result;
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
    // every element of y is written; a fresh y (zero fill deferred) is stored into, not read
    const bool whole = static_cast<std::size_t>(y.Size()) ==
                       static_cast<std::size_t>(m->M) * static_cast<std::size_t>(b.Cols());
    const bool store = whole && (!accumulate || y.TakeDeferredZero());
    Sparse::Cuda::Gemm(store ? y.CudaOverwriteRawPtr() : y.CudaMutableRawPtr(), m, b.CudaRawPtr(),
                       static_cast<unsigned int>(b.Cols()), store ? false : accumulate,
                       y.GetCudaDevice().GetID());
}
}  // namespace Sapphire::Compute
