#include <Sapphire/compute/sparse/Sparse.hpp>

#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/util/ResourceManager.hpp>

#include <sapphire_hip.h>

#include <algorithm>
#include <cstring>
#include <functional>
#include <utility>
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

// The two record types differ in the name and element type of their first array only (4-byte
// elements in both); everything below is written once over "first array, COL, ROW".
void* First(const SparseMatrix& r)
{
    return r.V;
}
void* First(const LoadDistMatrix& r)
{
    return r.Load;
}
void SetFirst(SparseMatrix& r, void* p)
{
    r.V = static_cast<float*>(p);
}
void SetFirst(LoadDistMatrix& r, void* p)
{
    r.Load = static_cast<uint32_t*>(p);
}

template <typename Record>
void RequireRoom(const Record& dst, const Record& src, const char* function)
{
    if (First(dst) == nullptr || dst.COL == nullptr || dst.ROW == nullptr)
        throw std::invalid_argument(std::string(function) + " - destination is not allocated");
    if (dst.NNZ < src.NNZ || dst.M < src.M)
        throw std::invalid_argument(std::string(function) + " - destination is too small");
}

template <typename Record>
Record AllocateCudaRecord(uint32_t m, uint32_t n, uint32_t nnz)
{
    Record r{};
    r.M = m;
    r.N = n;
    r.NNZ = nnz;
    SetFirst(r, Util::ResourceManager::GetMemoryCuda(Bytes(nnz), true));
    r.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryCuda(Bytes(nnz), true));
    r.ROW = static_cast<uint32_t*>(
        Util::ResourceManager::GetMemoryCuda(Bytes(static_cast<std::size_t>(m) + 1), true));
    return r;
}

SparseMatrix AllocateCuda(uint32_t m, uint32_t n, uint32_t nnz)
{
    return AllocateCudaRecord<SparseMatrix>(m, n, nnz);
}

template <typename Record>
void ReleaseCudaRecord(Record& r)
{
    if (First(r) != nullptr)
        Util::ResourceManager::FreePreservedCuda(First(r));
    if (r.COL != nullptr)
        Util::ResourceManager::FreePreservedCuda(r.COL);
    if (r.ROW != nullptr)
        Util::ResourceManager::FreePreservedCuda(r.ROW);
    r = Record{};
}

void ReleaseCuda(SparseMatrix& r)
{
    ReleaseCudaRecord(r);
}

template <typename Record>
Record* AllocateHostArray(uint32_t numMatrices, uint32_t m, uint32_t n,
                          const std::function<uint32_t(uint32_t)>& nnzOf,
                          const std::function<std::pair<uint32_t, uint32_t>(uint32_t)>& shapeOf)
{
    auto* array = new Record[numMatrices]();
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        Record& r = array[i];
        const auto shape = shapeOf ? shapeOf(i) : std::make_pair(m, n);
        r.M = shape.first;
        r.N = shape.second;
        r.NNZ = nnzOf(i);
        SetFirst(r, Util::ResourceManager::GetMemoryHost(Bytes(r.NNZ), true));
        r.COL = static_cast<uint32_t*>(Util::ResourceManager::GetMemoryHost(Bytes(r.NNZ), true));
        r.ROW = static_cast<uint32_t*>(
            Util::ResourceManager::GetMemoryHost(Bytes(static_cast<std::size_t>(r.M) + 1), true));
        std::memset(First(r), 0, Bytes(r.NNZ));
        std::memset(r.COL, 0, Bytes(r.NNZ));
        std::memset(r.ROW, 0, Bytes(static_cast<std::size_t>(r.M) + 1));
    }
    return array;
}

template <typename Record>
void FreeHostArray(Record* array, uint32_t numMatrices)
{
    if (array == nullptr)
        return;
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        Record& r = array[i];
        if (First(r) != nullptr)
            Util::ResourceManager::FreePreservedHost(First(r));
        if (r.COL != nullptr)
            Util::ResourceManager::FreePreservedHost(r.COL);
        if (r.ROW != nullptr)
            Util::ResourceManager::FreePreservedHost(r.ROW);
    }
    delete[] array;
}

template <typename Record, typename SizesFrom>
Record* AllocateCudaArray(const SizesFrom* like, uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    auto* array = new Record[numMatrices]();
    for (uint32_t i = 0; i < numMatrices; ++i)
        array[i] = AllocateCudaRecord<Record>(like[i].M, like[i].N, like[i].NNZ);
    return array;
}

template <typename Record>
void FreeCudaArray(Record* array, uint32_t numMatrices, int deviceId)
{
    if (array == nullptr)
        return;
    Cuda::CudaSetDevice(deviceId);
    Cuda::Synchronize();  // kernels may still be reading the arrays
    for (uint32_t i = 0; i < numMatrices; ++i)
        ReleaseCudaRecord(array[i]);
    delete[] array;
}

// `copy(dst, src, bytes)` moves one array
template <typename Record, typename Copy>
void CopyArray(Record* dstArray, const Record* srcArray, uint32_t numMatrices,
               const char* function, Copy&& copy)
{
    for (uint32_t i = 0; i < numMatrices; ++i)
    {
        const Record& s = srcArray[i];
        Record& d = dstArray[i];
        RequireRoom(d, s, function);
        copy(First(d), First(s), static_cast<std::size_t>(s.NNZ) * 4);
        copy(d.COL, s.COL, static_cast<std::size_t>(s.NNZ) * 4);
        copy(d.ROW, s.ROW, (static_cast<std::size_t>(s.M) + 1) * 4);
        d.NNZ = s.NNZ;
        d.M = s.M;
        d.N = s.N;
    }
}

const auto kHostToDevice = [](void* d, const void* s, std::size_t n) { Cuda::CopyHostToDevice(d, s, n); };
const auto kDeviceToHost = [](void* d, const void* s, std::size_t n) { Cuda::CopyDeviceToHost(d, s, n); };
const auto kDeviceToDevice = [](void* d, const void* s, std::size_t n) { Cuda::CopyDeviceToDevice(d, s, n); };
const auto kHostToHost = [](void* d, const void* s, std::size_t n) { std::memcpy(d, s, n); };
}  // namespace

void DeepAllocateSparseHost(SparseMatrix** sparseMatrixArray, uint32_t m, uint32_t n,
                            const uint32_t nnz[], uint32_t numMatrices)
{
    *sparseMatrixArray = AllocateHostArray<SparseMatrix>(
        numMatrices, m, n, [&](uint32_t i) { return nnz[i]; }, nullptr);
}

void DeepFreeSparseHost(SparseMatrix* sparseMatrixArray, uint32_t numMatrices)
{
    FreeHostArray(sparseMatrixArray, numMatrices);
}

void DeepAllocateSparseCuda(SparseMatrix** deviceSparseArray,
                            const SparseMatrix* hostSparseMatrixArray, uint32_t numMatrices,
                            int deviceId)
{
    *deviceSparseArray = AllocateCudaArray<SparseMatrix>(hostSparseMatrixArray, numMatrices, deviceId);
}

void DeepFreeSparseCuda(SparseMatrix* deviceSparseArray, uint32_t numMatrices, int deviceId)
{
    FreeCudaArray(deviceSparseArray, numMatrices, deviceId);
}

void DeepCopyHostToDevice(SparseMatrix* deviceDstArray, const SparseMatrix* hostSrcArray,
                          uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    CopyArray(deviceDstArray, hostSrcArray, numMatrices, "DeepCopyHostToDevice", kHostToDevice);
}

void DeepCopyDeviceToHost(SparseMatrix* hostDstArray, const SparseMatrix* deviceSrcArray,
                          uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    CopyArray(hostDstArray, deviceSrcArray, numMatrices, "DeepCopyDeviceToHost", kDeviceToHost);
}

void DeepCopyDeviceToDevice(SparseMatrix* deviceDstArray, const SparseMatrix* deviceSrcArray,
                            uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    CopyArray(deviceDstArray, deviceSrcArray, numMatrices, "DeepCopyDeviceToDevice",
              kDeviceToDevice);
}

void DeepCopyHostToHost(SparseMatrix* hostDstArray, const SparseMatrix* hostSrcArray,
                        uint32_t numMatrices)
{
    CopyArray(hostDstArray, hostSrcArray, numMatrices, "DeepCopyHostToHost", kHostToHost);
}

void DeepAllocateLoadDistHost(LoadDistMatrix** loadDistArray, SparseMatrix* sparseArray,
                              uint32_t numMatrices)
{
    *loadDistArray = AllocateHostArray<LoadDistMatrix>(
        numMatrices, 0, 0, [&](uint32_t i) { return sparseArray[i].NNZ; },
        [&](uint32_t i) { return std::make_pair(sparseArray[i].M, sparseArray[i].N); });
}

void DeepFreeLoadDistHost(LoadDistMatrix* loadDistArray, uint32_t numMatrices)
{
    FreeHostArray(loadDistArray, numMatrices);
}

void DeepAllocateLoadDistCuda(LoadDistMatrix** deviceLoadDistArray,
                              LoadDistMatrix* hostLoadDistArray, uint32_t numMatrices,
                              int deviceId)
{
    *deviceLoadDistArray =
        AllocateCudaArray<LoadDistMatrix>(hostLoadDistArray, numMatrices, deviceId);
}

void DeepFreeLoadDistCuda(LoadDistMatrix* deviceLoadDistArray, uint32_t numMatrices, int deviceId)
{
    FreeCudaArray(deviceLoadDistArray, numMatrices, deviceId);
}

void DeepCopyDeviceToDevice(LoadDistMatrix* deviceDstArray, LoadDistMatrix* deviceSrcArray,
                            uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    CopyArray(deviceDstArray, static_cast<const LoadDistMatrix*>(deviceSrcArray), numMatrices,
              "DeepCopyDeviceToDevice", kDeviceToDevice);
}

void DeepCopyHostToDevice(LoadDistMatrix* deviceDstArray, LoadDistMatrix* hostSrcArray,
                          uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    CopyArray(deviceDstArray, static_cast<const LoadDistMatrix*>(hostSrcArray), numMatrices,
              "DeepCopyHostToDevice", kHostToDevice);
}

void DeepCopyDeviceToHost(LoadDistMatrix* hostDstArray, LoadDistMatrix* deviceSrcArray,
                          uint32_t numMatrices, int deviceId)
{
    Cuda::CudaSetDevice(deviceId);
    CopyArray(hostDstArray, static_cast<const LoadDistMatrix*>(deviceSrcArray), numMatrices,
              "DeepCopyDeviceToHost", kDeviceToHost);
}

void DeepCopyHostToHost(LoadDistMatrix* hostDstArray, LoadDistMatrix* hostSrcArray,
                        uint32_t numMatrices)
{
    CopyArray(hostDstArray, static_cast<const LoadDistMatrix*>(hostSrcArray), numMatrices,
              "DeepCopyHostToHost", kHostToHost);
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
