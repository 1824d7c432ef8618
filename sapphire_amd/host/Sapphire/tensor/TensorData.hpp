// Storage behind a tensor: a shape plus one contiguous fp32 buffer on the host and/or one
// on the device, and the mode that says which of the two the operators use.
//
// Interface and behaviour follow the reference's Sapphire::TensorUtil::TensorData
// (Includes/Sapphire/tensor/TensorData.hpp:18-213, Sources/Sapphire/tensor/TensorData.cpp):
// copies are shallow views of the same buffers; buffers come from ResourceManager and are
// zero-filled when they are first allocated; ToCuda / ToHost switch the mode and copy.
// Device memory is HIP memory; the names keep the reference's "Cuda" wording.
#ifndef SAPPHIRE_AMD_TENSOR_TENSORDATA_HPP
#define SAPPHIRE_AMD_TENSOR_TENSORDATA_HPP

#include <Sapphire/compute/sparse/SparseMatrix.hpp>
#include <Sapphire/util/CudaDevice.hpp>
#include <Sapphire/util/Shape.hpp>

#include <cstddef>
#include <vector>

namespace Sapphire::TensorUtil
{
class TensorData
{
public:
    TensorData() = default;
    //! Host-only tensor.
    TensorData(Shape shape, Type type, bool preserve = false);
    TensorData(Shape shape, Type type, int parentDescKey, bool preserve = false);
    //! Device tensor when `device` is configured (id >= 0), host tensor otherwise.
    TensorData(Shape shape, Type type, CudaDevice device, bool preserve = false);
    TensorData(Shape shape, Type type, CudaDevice device, int parentDescKey,
               bool preserve = false);

    // copies alias the same buffers (TensorData.hpp:35-38 of the reference)
    TensorData(const TensorData&) = default;
    TensorData& operator=(const TensorData&) = default;
    TensorData(TensorData&& other) noexcept;
    TensorData& operator=(TensorData&& other) noexcept;

    unsigned long HostTotalSize = 0;
    unsigned long DenseTotalLengthCuda = 0;
    unsigned long SparseTotalLength = 0;

    //! Contents as a vector; in Cuda mode the device buffer is fetched first.
    [[nodiscard]] std::vector<float> GetDataCopy();
    //! Loads `data` into the buffer of the current mode; throws std::invalid_argument when the
    //! element count differs from the shape's.
    void SetData(std::vector<float> data);

    void SetDevice(CudaDevice device);
    [[nodiscard]] CudaDevice GetCudaDevice() const { return m_device; }

    //! Throws std::runtime_error when the element count would change.
    void Reshape(const Shape& shape);

    [[nodiscard]] int GetDescriptorKey() const { return m_parentDescKey; }
    [[nodiscard]] int GetNumUnits(int requiredDim) const { return m_shape.GetNumUnits(requiredDim); }
    [[nodiscard]] int GetUnitSize(int requiredDim) const { return m_shape.GetUnitSize(requiredDim); }
    [[nodiscard]] Shape GetShape() const { return m_shape; }
    [[nodiscard]] int Rows() const { return m_shape.Rows(); }
    [[nodiscard]] int Cols() const { return m_shape.Cols(); }
    [[nodiscard]] int Size() const { return m_shape.Size(); }
    [[nodiscard]] Type GetType() const { return m_type; }
    [[nodiscard]] std::size_t GetHostElementSize() const { return static_cast<std::size_t>(m_shape.Size()); }
    [[nodiscard]] std::size_t GetCudaElementSize() const { return static_cast<std::size_t>(m_shape.Size()); }

    //! A new tensor with its own buffers holding the same values.
    [[nodiscard]] TensorData CreateCopy() const;

    //! Selects the side the operators work on, allocating it when needed.  Throws
    //! std::runtime_error when Cuda is requested and no device was configured.
    void SetMode(ComputeMode mode);
    [[nodiscard]] ComputeMode Mode() const { return m_mode; }

    void ToCuda();
    void ToHost();

    //! dst receives dst.Size() / src.Size() copies of src (same type and mode required).
    static void DeepCopy(TensorData& dst, const TensorData& src);

    [[nodiscard]] const float* HostRawPtr() const { return m_denseHost; }
    [[nodiscard]] float* HostMutableRawPtr() const { return m_denseHost; }
    //! The device buffer.  A fresh device buffer reads as zeros
    //! (Sources/Sapphire/tensor/TensorData.cpp:330,354 of the reference fill it at allocation);
    //! here the fill is deferred until the buffer is first asked for through these two, which
    //! enqueue it on the calling thread's stream before they return the pointer.
    [[nodiscard]] const float* CudaRawPtr() const;
    [[nodiscard]] float* CudaMutableRawPtr() const;
    //! For an operator that is about to write every element of the device buffer without
    //! reading any: the pointer, with a deferred fill dropped instead of run.
    [[nodiscard]] float* CudaOverwriteRawPtr() const;
    //! True when the device buffer is fresh and its zero fill still deferred; the state is
    //! cleared and nothing is filled.  For an accumulating operator that covers the whole
    //! buffer: y += f(..) on known zeros is y = f(..), so it may store instead of add and
    //! must then take the pointer from CudaOverwriteRawPtr().
    [[nodiscard]] bool TakeDeferredZero() const;

    //! CSR record with host arrays / with device arrays, for Type::Sparse operands of the
    //! sparse x dense product (owned by the caller).
    SparseMatrix* SparseMatHost = nullptr;
    SparseMatrix* SparseMatCuda = nullptr;

private:
    void AllocateHost();
    void AllocateCuda();
    void UploadDense();
    void DownloadDense();
    void Steal(TensorData& other) noexcept;

    Shape m_shape;
    float* m_denseHost = nullptr;
    float* m_denseCuda = nullptr;
    int m_parentDescKey = -1;
    Type m_type = Type::Dense;
    ComputeMode m_mode = ComputeMode::Host;
    CudaDevice m_device;
    bool m_preserve = false;
};
}  // namespace Sapphire::TensorUtil

#endif
