#include <Sapphire/tensor/TensorData.hpp>

#include <Sapphire/compute/Initialize.hpp>
#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/util/ResourceManager.hpp>

#include <algorithm>
#include <cstring>
#include <stdexcept>
#include <string>

namespace Sapphire::TensorUtil
{
namespace
{
void RequireDense(Type type, const char* where)
{
    if (type == Type::Sparse)
        throw std::runtime_error(std::string(where) + " - Sparse not implemented");
}
}  // namespace

TensorData::TensorData(Shape shape, Type type, bool preserve)
    : m_shape(std::move(shape)), m_type(type), m_mode(ComputeMode::Host), m_preserve(preserve)
{
    AllocateHost();
}

TensorData::TensorData(Shape shape, Type type, int parentDescKey, bool preserve)
    : m_shape(std::move(shape)),
      m_parentDescKey(parentDescKey),
      m_type(type),
      m_mode(ComputeMode::Host),
      m_preserve(preserve)
{
    AllocateHost();
}

TensorData::TensorData(Shape shape, Type type, CudaDevice device, bool preserve)
    : TensorData(std::move(shape), type, std::move(device), -1, preserve)
{
}

TensorData::TensorData(Shape shape, Type type, CudaDevice device, int parentDescKey, bool preserve)
    : m_shape(std::move(shape)),
      m_parentDescKey(parentDescKey),
      m_type(type),
      m_device(std::move(device)),
      m_preserve(preserve)
{
    if (m_device.GetID() >= 0)
    {
        m_mode = ComputeMode::Cuda;
        AllocateCuda();
    }
    else
        AllocateHost();
}

void TensorData::Steal(TensorData& other) noexcept
{
    HostTotalSize = other.HostTotalSize;
    DenseTotalLengthCuda = other.DenseTotalLengthCuda;
    SparseTotalLength = other.SparseTotalLength;
    SparseMatHost = other.SparseMatHost;
    SparseMatCuda = other.SparseMatCuda;
    m_shape = std::move(other.m_shape);
    m_denseHost = other.m_denseHost;
    m_denseCuda = other.m_denseCuda;
    m_parentDescKey = other.m_parentDescKey;
    m_type = other.m_type;
    m_mode = other.m_mode;
    m_device = std::move(other.m_device);
    m_preserve = other.m_preserve;
    other.HostTotalSize = 0;
    other.DenseTotalLengthCuda = 0;
    other.SparseTotalLength = 0;
    other.m_denseHost = nullptr;
    other.m_denseCuda = nullptr;
    other.SparseMatHost = nullptr;
    other.SparseMatCuda = nullptr;
}

TensorData::TensorData(TensorData&& other) noexcept
{
    Steal(other);
}

TensorData& TensorData::operator=(TensorData&& other) noexcept
{
    if (this != &other)
        Steal(other);
    return *this;
}

const float* TensorData::CudaRawPtr() const
{
    return CudaMutableRawPtr();
}

float* TensorData::CudaMutableRawPtr() const
{
    if (m_denseCuda != nullptr && Util::ResourceManager::TakeZeroPendingCuda(m_denseCuda))
    {
        Compute::Cuda::CudaSetDevice(m_device.GetID());
        Compute::Dense::Cuda::Scalar(m_denseCuda, 0.0f, DenseTotalLengthCuda);
    }
    return m_denseCuda;
}

float* TensorData::CudaOverwriteRawPtr() const
{
    if (m_denseCuda != nullptr)
        (void)Util::ResourceManager::TakeZeroPendingCuda(m_denseCuda);
    return m_denseCuda;
}

bool TensorData::TakeDeferredZero() const
{
    return m_denseCuda != nullptr && Util::ResourceManager::TakeZeroPendingCuda(m_denseCuda);
}

void TensorData::Reshape(const Shape& shape)
{
    if (shape.Size() != m_shape.Size())
        throw std::runtime_error(
            "TensorData::Reshape - Attempt to change shape having different size");
    m_shape = shape;
}

std::vector<float> TensorData::GetDataCopy()
{
    if (m_mode == ComputeMode::Cuda)
        DownloadDense();
    std::vector<float> values(static_cast<std::size_t>(m_shape.Size()));
    std::copy_n(m_denseHost, std::min<std::size_t>(values.size(), HostTotalSize), values.begin());
    return values;
}

void TensorData::SetData(std::vector<float> data)
{
    const int expected = m_shape.Size();
    if (static_cast<int>(data.size()) != expected)
        throw std::invalid_argument("Tensor::SetForwardData - data size mismatch Given size : (" +
                                    std::to_string(data.size()) + ") expected size : (" +
                                    std::to_string(expected) + ")");
    if (m_mode == ComputeMode::Cuda)
        Compute::Cuda::CopyHostToDevice(CudaOverwriteRawPtr(), data.data(),
                                        sizeof(float) * data.size());
    else
        std::copy(data.begin(), data.end(), m_denseHost);
}

void TensorData::SetDevice(CudaDevice device)
{
    if (device != m_device)
    {
        const bool hadNone = m_device.GetID() == -1;
        m_device = std::move(device);
        if (hadNone && m_denseCuda == nullptr)
            AllocateCuda();
    }
}

TensorData TensorData::CreateCopy() const
{
    TensorData copy(m_shape, m_type, m_device, m_parentDescKey);
    copy.SetMode(m_mode);
    DeepCopy(copy, *this);
    return copy;
}

void TensorData::SetMode(ComputeMode mode)
{
    m_mode = mode;
    if (mode == ComputeMode::Host && m_denseHost == nullptr)
        AllocateHost();
    if (mode == ComputeMode::Cuda && m_denseCuda == nullptr)
    {
        if (m_device.GetID() == -1)
            throw std::runtime_error(
                "TensorData::SetMode - TensorData has not been configured to  use cuda device");
        AllocateCuda();
    }
}

void TensorData::ToCuda()
{
    if (m_denseHost == nullptr && m_mode == ComputeMode::Cuda)
        return;
    SetMode(ComputeMode::Cuda);
    UploadDense();
}

void TensorData::ToHost()
{
    if (m_denseCuda == nullptr && m_mode == ComputeMode::Host)
        return;
    SetMode(ComputeMode::Host);
    DownloadDense();
}

void TensorData::DeepCopy(TensorData& dst, const TensorData& src)
{
    if (dst.GetType() != src.GetType())
        throw std::invalid_argument("DeepCopy - matrix or device type mismatch");
    if (dst.Mode() != src.Mode())
        throw std::invalid_argument("DeepCopy - Mode mismatch");
    if (dst.Size() < src.Size())
        throw std::invalid_argument("DeepCopy - size of src cannot be larger than dst");
    if (src.Size() == 0 || dst.Size() % src.Size() != 0)
        throw std::invalid_argument("DeepCopy - size of dst must be multiple of src");
    if (dst.GetType() == Type::Sparse)
        throw std::runtime_error(dst.Mode() == ComputeMode::Cuda
                                     ? "DeepCopy - Cuda Sparse deep copy is not implemented"
                                     : "DeepCopy - Host Sparse ddp copy is not implemented");

    // one copy of src per repetition (the reference passes the whole dst length to every
    // copy, which overruns dst from the second repetition on; the intent is kept, not that)
    const std::size_t unit = static_cast<std::size_t>(src.Size());
    const std::size_t repeats = static_cast<std::size_t>(dst.Size()) / unit;
    if (dst.Mode() == ComputeMode::Cuda)
        Compute::Cuda::CopyDeviceToDeviceBroadcast(dst.CudaOverwriteRawPtr(), src.CudaRawPtr(),
                                                   repeats * unit * sizeof(float),
                                                   unit * sizeof(float));
    else
        for (std::size_t i = 0; i < repeats; ++i)
            std::memcpy(dst.m_denseHost + i * unit, src.m_denseHost, unit * sizeof(float));
}

void TensorData::UploadDense()
{
    RequireDense(m_type, "TensorData::m_toCuda");
    if (m_denseCuda == nullptr)
        AllocateCuda();
    // the whole device buffer when the two sides have the same length (they always do here)
    float* dst = HostTotalSize == DenseTotalLengthCuda ? CudaOverwriteRawPtr() : CudaMutableRawPtr();
    Compute::Cuda::CopyHostToDevice(dst, m_denseHost, HostTotalSize * sizeof(float));
}

void TensorData::DownloadDense()
{
    RequireDense(m_type, "TensorData::m_toHost");
    if (m_denseHost == nullptr)
        AllocateHost();
    Compute::Cuda::CopyDeviceToHost(m_denseHost, CudaRawPtr(), HostTotalSize * sizeof(float));
}

void TensorData::AllocateHost()
{
    RequireDense(m_type, "m_allocate");
    HostTotalSize = static_cast<unsigned long>(m_shape.Size());
    m_denseHost = static_cast<float*>(
        Util::ResourceManager::GetMemoryHost(HostTotalSize * sizeof(float), m_preserve));
    std::memset(m_denseHost, 0, HostTotalSize * sizeof(float));
}

void TensorData::AllocateCuda()
{
    RequireDense(m_type, "m_allocate");
    DenseTotalLengthCuda = static_cast<unsigned long>(m_shape.Size());
    Compute::Cuda::CudaSetDevice(m_device.GetID());
    m_denseCuda = static_cast<float*>(
        Util::ResourceManager::GetMemoryCuda(DenseTotalLengthCuda * sizeof(float), m_preserve));
    // Every fresh device buffer reads as zeros (TensorData.cpp:354 of the reference fills it
    // here).  The fill is deferred to the first use of the buffer: CudaRawPtr() /
    // CudaMutableRawPtr() enqueue it, an operator that writes the whole buffer drops it.
    Util::ResourceManager::MarkZeroPendingCuda(m_denseCuda);
}
}  // namespace Sapphire::TensorUtil
