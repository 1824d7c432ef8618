#include <Sapphire/compute/sparse/Sparse.hpp>

#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/util/ResourceManager.hpp>

#include <sapphire_hip.h>

#include <algorithm>
#include <cstring>
#include <stdexcept>
#include <string>

namespace Sapphire::Compute
{
namespace
{
std::size_t Bytes(std::size_t count)
{
    return std::max<std::size_t>(count, 1) * 4;
}

void Check(int status, const char* function)
{
    if (status != SPH_OK)
        throw std::runtime_error(std::string(function) + " failed with " + sph_last_error());
}

void RequireRoom(const SparseMatrix& dst, const SparseMatrix& src, const char* function)
{
    if (dst.V == nullptr || dst.COL == nullptr || dst.ROW == nullptr)
        throw std::invalid_argument(std::string(function) + " - destination is not allocated");
    if (dst.NNZ < src.NNZ || dst.M < src.M)
        throw std::invalid_argument(std::string(function) + " - destination is too small");
}

SparseMatrix AllocateCuda(uint32_t m, uint32_t n, uint32_t nnz)
{
    SparseMatrix r{};
    r.M = m;
    r.N = n;
    r.NNZ = nnz;
    r.V = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(Bytes(nnz), true));
    r.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(Bytes(nnz), true));
    r.ROW = static_cast<uint32_t*>(
        Util::ResourceManager::GetMemoryCuda(Bytes(static_cast<std::size_t>(m) + 1), true));
    return r;
}

void ReleaseCuda(SparseMatrix& r)
{
    if (r.V != nullptr)
        Util::ResourceManager::FreePreservedCuda(r.V);
    if (r.COL != nullptr)
        Util::ResourceManager::FreePreservedCuda(r.COL);
    if (r.ROW != nullptr)
        Util::ResourceManager::FreePreservedCuda(r.ROW);
    r = SparseMatrix{};
}
}  // namespace

void DeepAllocateSparseHost(SparseMatrix** sparseMatrixArray, uint32_t m, uint32_t n,
                            const uint32_t nnz[], uint32_t numMatrices)
{
    auto* array = new SparseMatrix[numMatrices]();
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        SparseMatrix& r = array[i];
        r.M = m;
        r.N = n;
        r.NNZ = nnz[i];
        r.V = static_cast<float*>(Util::ResourceManager::GetMemoryHost(Bytes(nnz[i]), true));
        r.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryHost(Bytes(nnz[i]), true));
        r.ROW = static_cast<uint32_t*>(
            Util::ResourceManager::GetMemoryHost(Bytes(static_cast<std::size_t>(m) + 1), true));
        std::memset(r.V, 0, Bytes(nnz[i]));
        std::memset(r.COL, 0, Bytes(nnz[i]));
        std::memset(r.ROW, 0, Bytes(static_cast<std::size_t>(m) + 1));
    }
    *sparseMatrixArray = array;
}

void DeepFreeSparseHost(SparseMatrix* sparseMatrixArray, uint32_t numMatrices)
{
    if (sparseMatrixArray == nullptr)
        return;
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        SparseMatrix& r = sparseMatrixArray[i];
        if (r.V != nullptr)
            Util::ResourceManager::FreePreservedHost(r.V);
        if (r.COL != nullptr)
            Util::ResourceManager::FreePreservedHost(r.COL);
        if (r.ROW != nullptr)
            Util::ResourceManager::FreePreservedHost(r.ROW);
    }
    delete[] sparseMatrixArray;
}

void DeepAllocateSparseCuda(SparseMatrix** deviceSparseArray,
                            const SparseMatrix* hostSparseMatrixArray, uint32_t numMatrices,
                            int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    auto* array = new SparseMatrix[numMatrices]();
    for (uint32_t i = 0; i < numMatrices; ++i)
        array[i] = AllocateCuda(hostSparseMatrixArray[i].M, hostSparseMatrixArray[i].N,
                                hostSparseMatrixArray[i].NNZ);
    *deviceSparseArray = array;
}

void DeepFreeSparseCuda(SparseMatrix* deviceSparseArray, uint32_t numMatrices, int deviceId)
{
    if (deviceSparseArray == nullptr)
        return;
    Cuda::CudaSetDevice(deviceId);
    Cuda::Synchronize();  // kernels may still be reading the arrays
    for (uint32_t i = 0; i < numMatrices; ++i)
        ReleaseCuda(deviceSparseArray[i]);
    delete[] deviceSparseArray;
}

void DeepCopyHostToDevice(SparseMatrix* deviceDstArray, const SparseMatrix* hostSrcArray,
                          uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        const SparseMatrix& s = hostSrcArray[i];
        SparseMatrix& d = deviceDstArray[i];
        RequireRoom(d, s, "DeepCopyHostToDevice");
        Cuda::CopyHostToDevice(d.V, s.V, static_cast<std::size_t>(s.NNZ) * 4);
        Cuda::CopyHostToDevice(d.COL, s.COL, static_cast<std::size_t>(s.NNZ) * 4);
        Cuda::CopyHostToDevice(d.ROW, s.ROW, (static_cast<std::size_t>(s.M) + 1) * 4);
        d.NNZ = s.NNZ;
        d.M = s.M;
        d.N = s.N;
    }
}

void DeepCopyDeviceToHost(SparseMatrix* hostDstArray, const SparseMatrix* deviceSrcArray,
                          uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        const SparseMatrix& s = deviceSrcArray[i];
        SparseMatrix& d = hostDstArray[i];
        RequireRoom(d, s, "DeepCopyDeviceToHost");
        Cuda::CopyDeviceToHost(d.V, s.V, static_cast<std::size_t>(s.NNZ) * 4);
        Cuda::CopyDeviceToHost(d.COL, s.COL, static_cast<std::size_t>(s.NNZ) * 4);
        Cuda::CopyDeviceToHost(d.ROW, s.ROW, (static_cast<std::size_t>(s.M) + 1) * 4);
        d.NNZ = s.NNZ;
        d.M = s.M;
        d.N = s.N;
    }
}

void DeepCopyDeviceToDevice(SparseMatrix* deviceDstArray, const SparseMatrix* deviceSrcArray,
                            uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        const SparseMatrix& s = deviceSrcArray[i];
        SparseMatrix& d = deviceDstArray[i];
        RequireRoom(d, s, "DeepCopyDeviceToDevice");
        Cuda::CopyDeviceToDevice(d.V, s.V, static_cast<std::size_t>(s.NNZ) * 4);
        Cuda::CopyDeviceToDevice(d.COL, s.COL, static_cast<std::size_t>(s.NNZ) * 4);
        Cuda::CopyDeviceToDevice(d.ROW, s.ROW, (static_cast<std::size_t>(s.M) + 1) * 4);
        d.NNZ = s.NNZ;
        d.M = s.M;
        d.N = s.N;
    }
}

void DeepCopyHostToHost(SparseMatrix* hostDstArray, const SparseMatrix* hostSrcArray,
                        uint32_t numMatrices)
{
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        const SparseMatrix& s = hostSrcArray[i];
        SparseMatrix& d = hostDstArray[i];
        RequireRoom(d, s, "DeepCopyHostToHost");
        std::memcpy(d.V, s.V, static_cast<std::size_t>(s.NNZ) * 4);
        std::memcpy(d.COL, s.COL, static_cast<std::size_t>(s.NNZ) * 4);
        std::memcpy(d.ROW, s.ROW, (static_cast<std::size_t>(s.M) + 1) * 4);
        d.NNZ = s.NNZ;
        d.M = s.M;
        d.N = s.N;
    }
}

void CreateSparseMatrixWithDenseMatrix(SparseMatrix** dst, const float* src, uint32_t m,
                                       uint32_t n, uint32_t paddedN, uint32_t numMatrices,
                                       int deviceId)
{
    if (paddedN < n)
        throw std::invalid_argument("CreateSparseMatrixWithDenseMatrix - paddedN is below n");
    Cuda::CudaSetDevice(deviceId);
    auto* array = new SparseMatrix[numMatrices]();
    try
    {
        // Counting passes of all matrices first, nothing read back: the stream is drained once,
        // by the first read of an entry count, instead of once per matrix.
        for (uint32_t i = 0; i < numMatrices; ++i)
        {
            const float* dense = src + static_cast<std::size_t>(i) * m * paddedN;
            SparseMatrix& r = array[i];
            r.M = m;
            r.N = n;
            r.ROW = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(
                Bytes(static_cast<std::size_t>(m) + 1), true));
            Check(sph_csr_row_offsets_f32(r.ROW, dense, m, n, paddedN, nullptr),
                  "CreateSparseMatrixWithDenseMatrix");
        }
        for (uint32_t i = 0; i < numMatrices; ++i)
        {
            uint32_t nnz = 0;
            Cuda::CopyDeviceToHost(&nnz, array[i].ROW + m, sizeof(nnz));
            array[i].NNZ = nnz;
        }
        for (uint32_t i = 0; i < numMatrices; ++i)
        {
            const float* dense = src + static_cast<std::size_t>(i) * m * paddedN;
            SparseMatrix& r = array[i];
            r.V = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(Bytes(r.NNZ), true));
            r.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(Bytes(r.NNZ), true));
            Check(sph_csr_fill_f32(r.V, r.COL, r.ROW, dense, m, n, paddedN),
                  "CreateSparseMatrixWithDenseMatrix");
        }
    }
    catch (...)
    {
        Cuda::Synchronize();
        for (uint32_t i = 0; i < numMatrices; ++i)
            ReleaseCuda(array[i]);
        delete[] array;
        throw;
    }
    *dst = array;
}

void ConvertSparseMatrixToDenseMatrix(float* dst, const SparseMatrix* src, uint32_t m, uint32_t n,
                                      uint32_t paddedN, uint32_t numMatrices, int deviceId)
{
    if (paddedN < n)
        throw std::invalid_argument("ConvertSparseMatrixToDenseMatrix - paddedN is below n");
    Cuda::CudaSetDevice(deviceId);
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        if (src[i].M != m || src[i].N != n)
            throw std::invalid_argument("ConvertSparseMatrixToDenseMatrix - record shape differs");
        Check(sph_csr_to_dense_f32(dst + static_cast<std::size_t>(i) * m * paddedN, paddedN,
                                   src[i].V, src[i].COL, src[i].ROW, m, n),
              "ConvertSparseMatrixToDenseMatrix");
    }
}
}  // namespace Sapphire::Compute
