// Device leaves of the dense matrix product, with the reference's signatures
// (Includes/Sapphire/compute/dense/cuda/Gemm.cuh:15-25).  Where the reference calls
// cublasGemmStridedBatchedEx (Sources/Sapphire/compute/dense/cuda/Gemm.cu:19-85) these
// forward to the MFMA kernels behind the C ABI.  A failing call throws std::runtime_error.
#ifndef SAPPHIRE_AMD_COMPUTE_DENSE_CUDA_GEMM_HPP
#define SAPPHIRE_AMD_COMPUTE_DENSE_CUDA_GEMM_HPP

#include <cstddef>
#include <cstdint>
#include <vector>

namespace Sapphire::Compute::Dense::Cuda
{
//! out[c] += A[c] * B[c] for c < totalSize / (M*N); matrices packed back to back.
void Gemm(unsigned int totalSize, float* out, const float* A, const float* B, unsigned int M,
          unsigned int N, unsigned int K, int deviceId);

//! Same with one shared A and/or B for the whole batch.
void GemmMatrixWiseBroadcast(float* out, const float* A, const float* B, unsigned int M,
                             unsigned int N, unsigned int K, unsigned int batchSize,
                             bool broadcastA, bool broadcastB, int deviceId);

//! out[c] (+)= A[c] * B[c] for c < batchSize with the three element strides given (0 repeats an
//! operand): the general form behind the two calls above.  `overwrite` stores the product
//! without reading out.
void GemmStrided(float* out, const float* A, const float* B, unsigned int M, unsigned int N,
                 unsigned int K, unsigned int batchSize, std::int64_t strideOut,
                 std::int64_t strideA, std::int64_t strideB, bool overwrite, int deviceId);

//! Element offsets of one M x N unit product.
struct GemmUnit
{
    std::uint64_t outOff, aOff, bOff;
};

//! All units in one launch: out[outOff] += A[aOff] * B[bOff] for every unit, units that share
//! an output applied in list order.  This is how a whole broadcast walk is issued.
void GemmGrouped(const std::vector<GemmUnit>& units, float* out, const float* A, const float* B,
                 unsigned int M, unsigned int N, unsigned int K, int deviceId);

//! Half-precision inputs, fp32 accumulation (the path the reference declares as WmmaGemm,
//! Includes/Sapphire/compute/dense/cuda/kernels/GemmKernel.cuh:14-50).  A and B hold IEEE
//! binary16 bit patterns; strides in elements, 0 repeats the operand.
void GemmHalf(float* out, const std::uint16_t* A, const std::uint16_t* B, unsigned int M,
              unsigned int N, unsigned int K, unsigned int batchSize, std::size_t strideOut,
              std::size_t strideA, std::size_t strideB, bool overwrite, int deviceId);

//! out[b] (+)= op(A[b]) * op(B[b]) with operands that may be stored transposed (A as K x M, B
//! as N x K), so that the backward products need no materialised transpose; matrices packed
//! back to back.  `overwrite` stores the product without reading out.
void GemmTransposed(float* out, const float* A, const float* B, unsigned int M, unsigned int N,
                    unsigned int K, unsigned int batchSize, bool transposeA, bool transposeB,
                    bool overwrite, int deviceId);

//! out -= ((op(A) * op(B)) * scale) * rate for one M x N matrix, every operation rounded on its
//! own: the gradient product, its optional scaling and the SGD step (Scale + Sub) in one launch,
//! with the result bits of the separate calls.
void GemmSgd(float* out, const float* A, const float* B, unsigned int M, unsigned int N,
             unsigned int K, bool transposeA, bool transposeB, float scale, float rate,
             int deviceId);

//! y = act((0 + bias) + x * W) in one launch: the two GEMMs of Linear's forward pass on a zero
//! y, optionally followed by ReLU, with the same result bits.
void LinearForward(float* y, const float* x, const float* W, const float* bias,
                   unsigned int batch, unsigned int inputs, unsigned int outputs, bool relu,
                   int deviceId);

//! dst[i] = binary16(src[i]), round to nearest even.
void ConvertToHalf(std::uint16_t* dst, const float* src, std::size_t size);

//! y = x > 0 ? x : 0 (Sources/Sapphire/compute/dense/cuda/Activation.cu, ReLU).
void ReLU(float* y, const float* x, unsigned int totalSize);

//! dx += x > 0 ? dy : 0 (Sources/Sapphire/compute/ActivationOps.cpp:69-85).
void ReLUBackward(float* dx, const float* dy, const float* x, unsigned int totalSize);

//! y = x * factor (device leaf of Compute::Scale, Sources/Sapphire/compute/BasicOps.cpp:250-267).
void Scale(float* y, const float* x, float factor, unsigned int totalSize);

//! Leaf of Compute::Sub with the reference's argument order
//! (Sources/Sapphire/compute/dense/naive/NaiveBasic.cpp:28-39).
void Sub(unsigned int totalSize, float* out, const float* A, const float* B,
         unsigned int inputStride, bool broadcastInputA, bool broadcastInputB);

//! z -= dz * learningRate in one pass, with the rounding of Scale followed by Sub.
void SgdStep(float* z, const float* dz, float learningRate, unsigned int totalSize);

//! Batched 2-D transpose (Sources/Sapphire/compute/dense/cuda/Basic.cu:85-102).
void Transpose(float* y, const float* x, unsigned int inputNumRows, unsigned int inputNumCols,
               unsigned int batchSize, bool broadcastInput);
}  // namespace Sapphire::Compute::Dense::Cuda

#endif
