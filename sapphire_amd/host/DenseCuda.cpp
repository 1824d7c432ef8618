#include <Sapphire/compute/Initialize.hpp>
#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/compute/dense/cuda/Gemm.hpp>
#include <Sapphire/tensor/TensorData.hpp>

#include <sapphire_hip.h>

#include <algorithm>
#include <stdexcept>
#include <string>

namespace Sapphire::Compute::Dense::Cuda
{
namespace
{
void Check(int status, const char* function)
{
    if (status != SPH_OK)
        throw std::runtime_error(std::string(function) + " failed with " + sph_last_error());
}
}  // namespace

void Scalar(float* data, float value, std::size_t size)
{
    Check(sph_fill_f32(data, value, size), "Scalar");
}

void Gemm(unsigned int totalSize, float* out, const float* A, const float* B, unsigned int M,
          unsigned int N, unsigned int K, int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    const std::uint64_t unit = static_cast<std::uint64_t>(M) * N;
    if (unit == 0 || totalSize < unit)
        throw std::runtime_error("Gemm failed with an empty output (M*N is zero or exceeds totalSize)");
    Check(sph_gemm_f32(out, A, B, M, N, K, static_cast<std::uint32_t>(totalSize / unit),
                       static_cast<std::int64_t>(unit), static_cast<std::int64_t>(M) * K,
                       static_cast<std::int64_t>(K) * N),
          "Gemm");
}

void GemmMatrixWiseBroadcast(float* out, const float* A, const float* B, unsigned int M,
                             unsigned int N, unsigned int K, unsigned int batchSize,
                             bool broadcastA, bool broadcastB, int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    Check(sph_gemm_f32(out, A, B, M, N, K, batchSize, static_cast<std::int64_t>(M) * N,
                       broadcastA ? 0 : static_cast<std::int64_t>(M) * K,
                       broadcastB ? 0 : static_cast<std::int64_t>(K) * N),
          "GemmMatrixWiseBroadcast");
}

void GemmStrided(float* out, const float* A, const float* B, unsigned int M, unsigned int N,
                 unsigned int K, unsigned int batchSize, std::int64_t strideOut,
                 std::int64_t strideA, std::int64_t strideB, bool overwrite, int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    Check(sph_gemm_f32_ex(out, A, B, M, N, K, batchSize, strideOut, strideA, strideB,
                          overwrite ? SPH_GEMM_OVERWRITE : SPH_GEMM_ACCUMULATE),
          "GemmStrided");
}

void GemmGrouped(const std::vector<GemmUnit>& units, float* out, const float* A, const float* B,
                 unsigned int M, unsigned int N, unsigned int K, int deviceId)
{
    if (units.empty())
        return;
    Compute::Cuda::CudaSetDevice(deviceId);
    static_assert(sizeof(GemmUnit) == sizeof(SphGemmEntry), "entry layouts must agree");
    Check(sph_gemm_f32_grouped(reinterpret_cast<const SphGemmEntry*>(units.data()),
                               static_cast<std::uint32_t>(units.size()), out, A, B, M, N, K),
          "GemmGrouped");
}

void GemmHalf(float* out, const std::uint16_t* A, const std::uint16_t* B, unsigned int M,
              unsigned int N, unsigned int K, unsigned int batchSize, std::size_t strideOut,
              std::size_t strideA, std::size_t strideB, bool overwrite, int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    Check(sph_gemm_f16f32(out, A, B, M, N, K, batchSize, static_cast<std::int64_t>(strideOut),
                          static_cast<std::int64_t>(strideA), static_cast<std::int64_t>(strideB),
                          overwrite ? SPH_GEMM_OVERWRITE : SPH_GEMM_ACCUMULATE),
          "GemmHalf");
}

void GemmTransposed(float* out, const float* A, const float* B, unsigned int M, unsigned int N,
                    unsigned int K, unsigned int batchSize, bool transposeA, bool transposeB,
                    bool overwrite, int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    const std::uint32_t flags = (transposeA ? SPH_GEMM_TRANS_A : 0u) |
                                (transposeB ? SPH_GEMM_TRANS_B : 0u) |
                                (overwrite ? SPH_GEMM_OVERWRITE : SPH_GEMM_ACCUMULATE);
    Check(sph_gemm_f32_ex(out, A, B, M, N, K, batchSize, static_cast<std::int64_t>(M) * N,
                          static_cast<std::int64_t>(M) * K, static_cast<std::int64_t>(K) * N,
                          flags),
          "GemmTransposed");
}

void GemmSgd(float* out, const float* A, const float* B, unsigned int M, unsigned int N,
             unsigned int K, bool transposeA, bool transposeB, float scale, float rate,
             int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    const std::uint32_t flags =
        (transposeA ? SPH_GEMM_TRANS_A : 0u) | (transposeB ? SPH_GEMM_TRANS_B : 0u);
    Check(sph_gemm_f32_sgd(out, A, B, M, N, K, scale, rate, flags), "GemmSgd");
}

void LinearForward(float* y, const float* x, const float* W, const float* bias,
                   unsigned int batch, unsigned int inputs, unsigned int outputs, bool relu,
                   int deviceId)
{
    Compute::Cuda::CudaSetDevice(deviceId);
    Check(sph_linear_forward_f32(y, x, W, bias, batch, inputs, outputs,
                                 relu ? SPH_LINEAR_RELU : 0u),
          "LinearForward");
}

void ConvertToHalf(std::uint16_t* dst, const float* src, std::size_t size)
{
    Check(sph_convert_f32_to_f16(dst, src, size), "ConvertToHalf");
}

void ReLU(float* y, const float* x, unsigned int totalSize)
{
    Check(sph_relu_f32(y, x, totalSize), "ReLU");
}

void ReLUBackward(float* dx, const float* dy, const float* x, unsigned int totalSize)
{
    Check(sph_relu_backward_f32(dx, dy, x, totalSize), "ReLUBackward");
}

void Scale(float* y, const float* x, float factor, unsigned int totalSize)
{
    Check(sph_scale_f32(y, x, factor, totalSize), "Scale");
}

void Sub(unsigned int totalSize, float* out, const float* A, const float* B,
         unsigned int inputStride, bool broadcastInputA, bool broadcastInputB)
{
    Check(sph_sub_f32(out, A, B, totalSize, inputStride, broadcastInputA ? 1 : 0,
                      broadcastInputB ? 1 : 0),
          "Sub");
}

void SgdStep(float* z, const float* dz, float learningRate, unsigned int totalSize)
{
    Check(sph_sgd_step_f32(z, dz, learningRate, totalSize), "SgdStep");
}

void Transpose(float* y, const float* x, unsigned int inputNumRows, unsigned int inputNumCols,
               unsigned int batchSize, bool broadcastInput)
{
    Check(sph_transpose_f32(y, x, inputNumRows, inputNumCols, batchSize, broadcastInput ? 1 : 0),
          "Transpose");
}
}  // namespace Sapphire::Compute::Dense::Cuda

namespace Sapphire::Compute::Initialize
{
void Scalar(TensorUtil::TensorData& data, float value)
{
    if (data.Mode() == ComputeMode::Cuda)
        Dense::Cuda::Scalar(data.CudaOverwriteRawPtr(), value, data.DenseTotalLengthCuda);
    else
        std::fill_n(data.HostMutableRawPtr(), data.HostTotalSize, value);
}

void Ones(TensorUtil::TensorData& data)
{
    Scalar(data, 1.0f);
}

void Zeros(TensorUtil::TensorData& data)
{
    Scalar(data, 0.0f);
}
}  // namespace Sapphire::Compute::Initialize
