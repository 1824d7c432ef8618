/*
 * sapphire_hip.h -- C ABI of the MI355X (gfx950) backend for Sapphire's
 * matrix-multiplication path.
 *
 * Everything the reference's device leaf needs is reachable through these
 * entry points: plain pointers and sizes, no C++ or framework types.  Every
 * function returns 0 on success and a non-zero SphStatus otherwise; the text
 * of the last failure on the calling thread is available from
 * sph_last_error().  Nothing throws across this boundary.
 *
 * All device work is enqueued on one HIP stream per (device, host thread),
 * the slot the reference fills with a cuBLAS handle per (device, thread)
 * (Sources/Sapphire/compute/dense/cuda/Gemm.cu:24-30,
 *  Includes/Sapphire/util/ResourceManager.hpp:152-157).  Calls from one thread
 * execute in call order; copies to the host wait for preceding work, as the
 * reference's blocking cudaMemcpy did.
 *
 * Citations are relative to the reference tree.
 */
#ifndef SAPPHIRE_HIP_H
#define SAPPHIRE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum
{
    SPH_OK = 0,
    SPH_ERR_INVALID = 1,  /* bad argument (null pointer, zero M*N, size overflow) */
    SPH_ERR_DEVICE = 2,   /* a HIP runtime call failed */
    SPH_ERR_UNSUPPORTED = 3
} SphStatus;

/* IEEE binary16 bit pattern */
typedef uint16_t sph_f16;

/* Text of the last non-zero status on this thread ("" if none). */
const char* sph_last_error(void);

/* ---- device / memory / stream ------------------------------------------- *
 * Replace Sapphire::Compute::Cuda::{CudaSetDevice,CudaMalloc,CudaFree,
 * CopyHostToDevice,CopyDeviceToHost,CopyDeviceToDevice,CopyDeviceToDeviceAsync}
 * (Includes/Sapphire/compute/cudaUtil/Memory.hpp:14-30,
 *  Sources/Sapphire/compute/cudaUtil/Memory.cpp:14-98).  Sizes are size_t: the
 * reference's unsigned-int byte counts (4 GiB cap) are not inherited. */

typedef struct
{
    char name[128];
    char arch[32];            /* e.g. "gfx950:sramecc+:xnack-" */
    int computeUnits;
    int clockMHz;             /* peak engine clock */
    int memoryClockMHz;
    int memoryBusWidthBits;
    int ldsBytesPerBlock;
    int l2Bytes;
    uint64_t totalMemoryBytes;
    int wavefrontSize;
} SphDeviceInfo;

int sph_device_count(int* count);
/* replaces CudaSetDevice (Memory.cpp:14-28); SPH_ERR_INVALID when deviceId is
 * not below the device count */
int sph_set_device(int deviceId);
int sph_get_device(int* deviceId);
int sph_device_info(int deviceId, SphDeviceInfo* info);

int sph_malloc(void** ptr, size_t bytes);              /* Memory.cpp:30-36 */
int sph_free(void* ptr);                               /* Memory.cpp:38-44 */
/* Stream-ordered allocation on the calling thread's stream (hipMallocAsync):
 * the block may be used by work enqueued after the call and is returned to
 * the device's pool, not to the driver, when it is freed, so neither call
 * waits for the device.  The pool behind the reference's ResourceManager
 * (Sources/Sapphire/util/ResourceManager.cpp:38-72 calls cudaMalloc / cudaFree,
 * both of which synchronise).  sph_mem_pool_trim hands idle pool memory back. */
int sph_malloc_async(void** ptr, size_t bytes);
int sph_free_async(void* ptr);
int sph_mem_pool_trim(void);
/* Number of device and pinned-host allocations the library has made in this
 * process so far (hipMalloc, hipMallocAsync, hipHostMalloc: the caller's own
 * sph_malloc* calls and the library's internal scratch blocks and tables).  No
 * counterpart in the reference.  For callers that must show that a call
 * allocates nothing: read it before and after. */
int sph_allocation_count(uint64_t* count);
int sph_memcpy_h2d(void* dev, const void* host, size_t bytes); /* :46-53 */
int sph_memcpy_d2h(void* host, const void* dev, size_t bytes); /* :55-63 */
int sph_memcpy_d2d(void* dst, const void* src, size_t bytes);  /* :65-72 */
/* enqueue only, no wait (Memory.cpp:74-82) */
int sph_memcpy_d2d_async(void* dst, const void* src, size_t bytes);
/* pinned host staging memory for callers that want asynchronous transfers */
int sph_host_malloc(void** ptr, size_t bytes);
int sph_host_free(void* ptr);

/* Wait for everything this thread enqueued on the current device. */
int sph_stream_sync(void);
/* Wait for everything any thread enqueued on the current device (what the
 * reference's cudaFree and cudaDeviceSynchronize did implicitly). */
int sph_device_sync(void);
/* Work this thread enqueues from now on waits for everything hipStream holds so
 * far; no host wait.  NULL or the thread's own stream is a no-op.  For memory
 * that passes from one thread's stream to another's (the buffer pool behind
 * Sources/Sapphire/util/ResourceManager.cpp:38-72 hands blocks across threads). */
int sph_stream_wait_stream(void* hipStream);
/* The hipStream_t this thread's calls run on (created on first use). */
int sph_get_stream(void** hipStream);
/* Run this thread's later calls on a caller-owned hipStream_t; NULL returns
 * to the library's own stream.  The stream must outlive every buffer that was
 * used on it and is still held by a pool above this library (the C++ layer's
 * ResourceManager remembers the stream a block was last used on and makes the
 * next user wait for it): drain the stream and release or ClearAll() such
 * pools before destroying it. */
int sph_set_stream(void* hipStream);

/* Events on this thread's stream, for timing launches from a host language
 * that has no HIP binding. */
int sph_event_create(void** event);
int sph_event_record(void* event);
int sph_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for stop */
int sph_event_destroy(void* event);

/* ---- graphs -------------------------------------------------------------- */

/* Launch-bound sequences (a layer's forward or backward pass is a handful of
 * kernels of a few microseconds each) can be recorded once and replayed as one
 * HIP graph.  Between begin and end the calling thread's entry points enqueue
 * into the graph instead of running; entry points that wait for the device,
 * allocate, free, read back or change the stream or device (copies to or from
 * the host, sph_stream_sync, sph_malloc/sph_free, sph_event_elapsed_ms,
 * sph_gemm_f32_grouped -- use sph_gemm_f32_grouped_device --,
 * sph_csr_row_offsets_f32 with a host count or more than 65535 rows) return SPH_ERR_UNSUPPORTED and leave the capture intact.
 * sph_graph_launch enqueues one replay on the thread's stream.  The recorded
 * pointers and sizes are fixed; change inputs by writing into the same
 * buffers.  No counterpart in the reference (its cuBLAS calls are issued one
 * by one). */
int sph_graph_begin_capture(void);
int sph_graph_end_capture(void** graph);
int sph_graph_launch(void* graph);
int sph_graph_destroy(void* graph);

/* ---- fills and element-wise neighbours ----------------------------------- */

/* dst[i] = value.  Replaces Dense::Cuda::Scalar
 * (Sources/Sapphire/compute/dense/cuda/Initialize.cu:46-59), which zero-fills
 * every fresh device buffer (Sources/Sapphire/tensor/TensorData.cpp:354) and
 * backs Initialize::Ones/Zeros in Linear (Linear.cpp:118,133). */
int sph_fill_f32(float* dst, float value, size_t count);

/* out[i] = in[i] > 0 ? in[i] : 0.  Replaces Dense::Cuda::ReLU
 * (Sources/Sapphire/compute/dense/cuda/kernels/ActivationKernel.cu:11-22);
 * CPU counterpart NaiveBasic.cpp:159-165.  out may alias in. */
int sph_relu_f32(float* out, const float* in, size_t count);

/* Batched 2-D transpose, out[b][j][i] = in[b][i][j]; with broadcast != 0 the
 * one input matrix is used for every batch.  Replaces Dense::Cuda::Transpose
 * (Sources/Sapphire/compute/dense/cuda/Basic.cu:85-102,
 *  kernels/BasicKernel.cu:78-113). */
int sph_transpose_f32(float* out, const float* in, uint32_t rows, uint32_t cols,
                      uint32_t batch, int broadcast);

/* dst[i] = (binary16, round-to-nearest-even) src[i] */
int sph_convert_f32_to_f16(sph_f16* dst, const float* src, size_t count);

/* out[i] = in[i] * factor.  Replaces Dense::Cuda::Scale (called from
 * Sources/Sapphire/compute/BasicOps.cpp Compute::Scale); CPU counterpart
 * NaiveBasic.cpp:54-61.  out may alias in. */
int sph_scale_f32(float* out, const float* in, float factor, size_t count);

/* out[i] = a[i % la] - b[i % lb] with la = broadcastA ? inputStride : count,
 * lb likewise: the leaf Compute::Sub hands to BroadcastWith2Inputs
 * (Sources/Sapphire/compute/BasicOps.cpp:70-103).  Replaces Dense::Cuda::Sub;
 * CPU counterpart NaiveBasic.cpp:28-39.  out may alias a or b when neither is
 * broadcast.  inputStride must be non-zero when a broadcast flag is set. */
int sph_sub_f32(float* out, const float* a, const float* b, size_t count,
                size_t inputStride, int broadcastA, int broadcastB);

/* dx[i] += x[i] > 0 ? dy[i] : 0.  Replaces Dense::Cuda::ReLUBackward
 * (Sources/Sapphire/compute/ActivationOps.cpp:69-85); CPU counterpart
 * NaiveBasic.cpp:167-174. */
int sph_relu_backward_f32(float* dx, const float* dy, const float* x, size_t count);

/* z[i] = z[i] - dz[i] * learningRate, the product rounded to fp32 before the
 * subtraction: one pass with the result of the Scale-into-temporary followed
 * by Sub that Optimizer::SGD performs (Sources/Sapphire/operations/optimizers/SGD.cpp:22-28),
 * bit for bit, without the temporary. */
int sph_sgd_step_f32(float* z, const float* dz, float learningRate, size_t count);

/* ---- dense GEMM ---------------------------------------------------------- */

/* flags of the GEMM entry points that take them */
#define SPH_GEMM_ACCUMULATE 0u /* out += A*B, like the reference            */
#define SPH_GEMM_OVERWRITE 1u  /* out  = A*B, out is not read               */
#define SPH_GEMM_TRANS_A 2u    /* A is stored K x M (the transpose of M x K) */
#define SPH_GEMM_TRANS_B 4u    /* B is stored N x K (the transpose of K x N) */

/* out[b] += A[b] * B[b] for b < batch; row-major; A is M x K, B is K x N,
 * out is M x N; fp32 storage, fp32 MFMA products and accumulation.
 * Strides are in elements between consecutive matrices; 0 repeats the
 * operand for every b (batch broadcast).
 *
 * Replaces Dense::Cuda::Gemm (Includes/Sapphire/compute/dense/cuda/Gemm.cuh:15-18,
 * Sources/Sapphire/compute/dense/cuda/Gemm.cu:19-51): batch = totalSize/(M*N),
 * strideOut = M*N, strideA = M*K, strideB = K*N; and
 * Dense::Cuda::GemmMatrixWiseBroadcast (Gemm.cuh:20-25, Gemm.cu:55-85):
 * strideA = 0 when broadcastA, strideB = 0 when broadcastB.
 * K == 0 leaves out untouched; M*N == 0 or batch == 0 is SPH_ERR_INVALID. */
int sph_gemm_f32(float* out, const float* A, const float* B, uint32_t M,
                 uint32_t N, uint32_t K, uint32_t batch, int64_t strideOut,
                 int64_t strideA, int64_t strideB);

/* sph_gemm_f32 with flags.  SPH_GEMM_TRANS_A / SPH_GEMM_TRANS_B read an
 * operand that is stored transposed, so that the products of the backward
 * pass, dx += dy * W^T and dw = x^T * dy, need no materialised transpose:
 * they replace the Compute::Transpose + Compute::Gemm pairs of
 * Sources/Sapphire/operations/Backward/LinearBackward.cpp:49-50,70-73 and
 * MathBackward.cpp:46-51.  The K products of an output element are added in
 * the same order with or without the flags, so the result is bit-identical
 * to sph_transpose_f32 followed by sph_gemm_f32 -- except for a single output
 * row (M == 1, K >= 64) with SPH_GEMM_TRANS_B: the plain call then runs a
 * row-reduction kernel that adds in another order, and the two agree within
 * the fp32 tolerance only.  SPH_GEMM_OVERWRITE stores the product without
 * reading out (K == 0 then stores zeros). */
int sph_gemm_f32_ex(float* out, const float* A, const float* B, uint32_t M,
                    uint32_t N, uint32_t K, uint32_t batch, int64_t strideOut,
                    int64_t strideA, int64_t strideB, uint32_t flags);

/* sph_gemm_f32_sgd: the weight update of Linear's backward pass in one launch,
 * out = out - ((A * B) * scale) * rate with every operation rounded on its own
 * (no fused multiply-add), for one M x N matrix.  It replaces, with the same
 * result bits, the sequence the reference runs
 * (Sources/Sapphire/operations/Backward/LinearBackward.cpp:55-76 and
 * Sources/Sapphire/optimizers/SGD.cpp:22-28): Zeros(dw); Gemm(dw, x^T, dy)
 * [; Scale(dw, dw, scale)]; Scale(temp, dw, rate); Sub(w, w, temp) -- the
 * gradient is never stored.  scale = 1 for the weights, 1 / batch for the
 * bias row (A = ones, M = 1).  flags: SPH_GEMM_TRANS_A / SPH_GEMM_TRANS_B as
 * in sph_gemm_f32_ex.  K = 0 leaves out as it is. */
int sph_gemm_f32_sgd(float* out, const float* A, const float* B, uint32_t M,
                     uint32_t N, uint32_t K, float scale, float rate,
                     uint32_t flags);

/* The forward pass of a fully connected layer in one launch:
 *   y[b][j] = act((0 + bias[j]) + sum_k x[b][k] * W[k][j])
 * x is batch x inputs, W inputs x outputs, bias has outputs entries, y is
 * batch x outputs and is not read.  This is what
 * Sources/Sapphire/operations/Forward/Linear.cpp:113-136 computes with
 * Gemm(y, ones, bias) and Gemm(y, x, W) on a zero y; with SPH_LINEAR_RELU the
 * ReLU that follows the layer (Sources/Sapphire/compute/ActivationOps.cpp:52-67)
 * is applied to the value before it is stored.  The product term and the bits
 * of the result are those of sph_fill_f32 + two sph_gemm_f32 (+ sph_relu_f32). */
#define SPH_LINEAR_RELU 1u
int sph_linear_forward_f32(float* y, const float* x, const float* W,
                           const float* bias, uint32_t batch, uint32_t inputs,
                           uint32_t outputs, uint32_t flags);

/* One M x N unit product per entry, out[outOff] += A[aOff] * B[bOff], offsets
 * in elements from the three bases.  Entries are read from host memory.  This
 * is the whole leaf list of BroadcastWith2Inputs
 * (Includes/Sapphire/compute/Broadcast.hpp:83-133) issued as one launch in
 * place of one cuBLAS call per leaf.  Entries whose outOff coincide are
 * applied in entry order.  The table travels through a staging buffer and a
 * device buffer that belong to the calling thread, so calls from different
 * threads do not wait for each other. */
typedef struct
{
    uint64_t outOff;
    uint64_t aOff;
    uint64_t bOff;
} SphGemmEntry;

int sph_gemm_f32_grouped(const SphGemmEntry* entries, uint32_t count, float* out,
                         const float* A, const float* B, uint32_t M, uint32_t N,
                         uint32_t K);

/* The same launch with the table already in device memory that the caller
 * owns (and keeps unchanged until the launch has run): nothing is uploaded, so
 * the call can be recorded into a graph and never waits.  The caller
 * guarantees that no two entries share an outOff (sph_gemm_f32_grouped cuts
 * such lists into ordered launches on the host; here one launch applies all
 * entries at once).  SPH_GROUPED_OFFSETS_MULTIPLE_OF_4 promises that every
 * offset is a multiple of 4 elements, which lets the kernels use 16-byte
 * accesses when the bases and M, N, K allow; without it they assume nothing. */
#define SPH_GROUPED_OFFSETS_MULTIPLE_OF_4 1u
int sph_gemm_f32_grouped_device(const SphGemmEntry* deviceEntries, uint32_t count,
                                float* out, const float* A, const float* B,
                                uint32_t M, uint32_t N, uint32_t K, uint32_t flags);

/* Half-precision inputs, fp32 accumulation, fp32 output: the tensor-core path
 * the reference declares as WmmaGemm
 * (Includes/Sapphire/compute/dense/cuda/kernels/GemmKernel.cuh:14-50) and
 * never defines.  Same layout, stride and += contract as sph_gemm_f32.
 * flags: SPH_GEMM_OVERWRITE stores A*B without reading out (for callers that
 * know out holds zeros); default accumulates like the reference.
 * SPH_GEMM_TRANS_A / SPH_GEMM_TRANS_B read an operand stored transposed
 * (A as K x M, B as N x K), as in sph_gemm_f32_ex.  The order in which the K
 * products of an output element are added depends on the shape and, on the
 * last M % 8 rows and N % 8 columns, on the storage order: results agree with
 * the CPU loop within the fp16 path's 1e-2 tolerance, and exactly whenever
 * every partial sum is exactly representable (the products themselves are
 * exact in fp32, subnormal inputs included). */

int sph_gemm_f16f32(float* out, const sph_f16* A, const sph_f16* B, uint32_t M,
                    uint32_t N, uint32_t K, uint32_t batch, int64_t strideOut,
                    int64_t strideA, int64_t strideB, uint32_t flags);

/* ---- CSR sparse x dense -------------------------------------------------- */

/* out[m][n] (+)= sum over p in [ROW[m], ROW[m+1]) of V[p] * B[COL[p]][n],
 * entries taken in storage order, products and sums rounded separately in
 * fp32 (no fused multiply-add), so the result equals the reference's dense
 * leaf on the densified matrix bit for bit.
 * V/COL/ROW are the device arrays of a SparseMatrix
 * (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:28-38); ROW holds M+1
 * offsets.  Kdim is the sparse matrix's column count (= rows of B); N is the
 * dense column count.  accumulate == 0 stores (rows without entries become
 * 0), otherwise adds into out.
 * The reference declares no sparse x dense product (Sparse.hpp:20-162 holds
 * sparse x sparse declarations only); this entry fills that slot.
 * The equality with the dense leaf on the densified matrix holds for finite B
 * only: the dense loop adds 0 * B[k][n] for the absent entries, which is NaN
 * where B holds Inf or NaN, while the CSR loop never touches those rows of B.
 * Inf and NaN in V or in the rows of B that are referenced propagate as in the
 * storage-order CPU loop, element by element. */
int sph_spmm_csr_f32(float* out, const float* V, const uint32_t* COL,
                     const uint32_t* ROW, uint32_t M, uint32_t Kdim, uint32_t N,
                     const float* B, int accumulate);
/* sph_spmm_csr_bias_f32: out[i][j] = (0 + rowBias[i]) + sum_p V[p] * B[COL[p]][j],
 * out is not read: the bits that sph_spmm_csr_f32 with accumulate leaves in an
 * out filled by sph_fill_f32(0) and the K = 1 product rowBias x ones -- the
 * feature-major form of Linear's bias step
 * (Sources/Sapphire/operations/Forward/Linear.cpp:113-136) for a sparse weight,
 * without the fill, the ones and the K = 1 launch. */
int sph_spmm_csr_bias_f32(float* out, const float* V, const uint32_t* COL,
                          const uint32_t* ROW, uint32_t M, uint32_t Kdim,
                          uint32_t N, const float* B, const float* rowBias);

/* ---- dense <-> CSR ------------------------------------------------------- */

/* The reference declares CreateSparseMatrixWithDenseMatrix(dst, src, m, n,
 * paddedN, numMatrices) and ConvertSparseMatrixToDenseMatrix(dst, src, m, n,
 * paddedN, numMatrices) (Includes/Sapphire/compute/sparse/Sparse.hpp:150-160)
 * and defines neither; these three calls are their device work for one matrix
 * of M rows, N columns and a row pitch of ld floats (ld = paddedN).  An entry
 * is kept when its value != 0 (-0.0 is dropped, NaN kept); a row's entries are
 * stored in ascending column order.
 *
 * sph_csr_row_offsets_f32: ROW (device, M + 1 entries) receives the offsets,
 * ROW[M] = number of kept entries.  With nnzHost != NULL that count is also
 * copied to *nnzHost and the call returns after the stream has drained, so the
 * caller can size V and COL; with NULL the call is asynchronous.
 * sph_csr_fill_f32: writes V and COL (device, ROW[M] entries each) from the
 * same dense matrix and the ROW just computed.
 * sph_csr_to_dense_f32: dense[r][c] = the stored value, 0 where none is
 * stored; columns >= N in COL are ignored; the pitch padding is not written. */
int sph_csr_row_offsets_f32(uint32_t* ROW, const float* dense, uint32_t M,
                            uint32_t N, uint32_t ld, uint32_t* nnzHost);
/* sph_csr_row_offsets_f32 for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops that must not reach the
 * allocator, harnesses that forbid it).  No counterpart in the reference.
 * Same ROW, bit for bit, for any M, including the M + 1 > 65536 case in which
 * sph_csr_row_offsets_f32 takes a stream-ordered scratch block: the per-block
 * totals of the scan live in a fixed 16 KiB array inside the library (one copy
 * per device, held until the process ends) instead.  Allocates nothing, waits
 * for nothing, copies nothing to the host (read ROW[M] yourself) and can be
 * recorded into a graph.  M above 16777215 is SPH_ERR_INVALID.  All calls on
 * one device share the array: calls that overlap in time on different streams
 * of one device race; calls on one stream are ordered and need no clearing
 * between them. */
int sph_csr_row_offsets_noalloc_f32(uint32_t* ROW, const float* dense,
                                    uint32_t M, uint32_t N, uint32_t ld);
int sph_csr_fill_f32(float* V, uint32_t* COL, const uint32_t* ROW,
                     const float* dense, uint32_t M, uint32_t N, uint32_t ld);
int sph_csr_to_dense_f32(float* dense, uint32_t ld, const float* V,
                         const uint32_t* COL, const uint32_t* ROW, uint32_t M,
                         uint32_t N);
/* sph_csr_from_dense_f32: the conversion of CreateSparseMatrixWithDenseMatrix
 * (Includes/Sapphire/compute/sparse/Sparse.hpp:153-156) for a caller that can
 * bound the number of entries beforehand: ROW, V and COL in one call.  V and
 * COL hold `capacity` entries; ROW (M + 1 entries) is always complete and
 * ROW[M] is the true count, but only entries with an index below `capacity`
 * are stored: when the count turns out larger, grow V and COL and call
 * sph_csr_fill_f32 with the ROW already there.  With nnzHost != NULL the
 * count is copied to *nnzHost and the call returns after the stream has
 * drained; with NULL it is asynchronous.
 * For rows of 128 .. 8192 columns, at least 16 Mi elements and a capacity of at
 * most about an eighth of the matrix the dense matrix is read once: every row is
 * compacted into a staging slot of 2 * capacity / M + 32 entries (a
 * stream-ordered scratch allocation of 8 bytes per slot entry), the counts
 * are scanned and a small kernel moves the staged entries into place; a row
 * with more entries than its slot is read a second time.  Other shapes run
 * the count, scan and fill passes inside the call.  Refused during graph
 * capture (scratch allocation).  Same ROW, V and COL, bit for bit, as
 * sph_csr_row_offsets_f32 followed by sph_csr_fill_f32. */
int sph_csr_from_dense_f32(float* V, uint32_t* COL, uint32_t* ROW,
                           uint32_t capacity, const float* dense, uint32_t M,
                           uint32_t N, uint32_t ld, uint32_t* nnzHost);

/* sph_csr_validate_u32: checks a CSR record before a product that trusts it.
 * The reference's SparseMatrix (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:28-38)
 * carries no invariant checks, and neither do the products here: they read
 * B[COL[p]] and the entries ROW[i] .. ROW[i + 1] as given, so an index outside
 * the operand is a device memory fault.  This call reads only ROW[0 .. M] and
 * COL[0 .. nnz) and reports, after the stream has drained (refused during
 * graph capture): ROW[0] == 0, ROW non-decreasing, ROW[M] == nnz, every
 * COL[p] < Kdim.  Any violation is SPH_ERR_INVALID with the violated rules
 * named in sph_last_error(); when problemsHost is not NULL it receives a bit
 * mask (1 ROW[0] != 0, 2 ROW decreasing, 4 ROW[M] != nnz, 8 column out of
 * range, 16 a row whose columns are not strictly ascending -- the last one is
 * reported but is no error: the products do not need sorted rows). */
int sph_csr_validate_u32(const uint32_t* COL, const uint32_t* ROW, uint32_t M,
                         uint32_t Kdim, uint32_t nnz, uint32_t* problemsHost);

/* ---- CSR x CSR ------------------------------------------------------------ */

/* C = A * B with all three in CSR (A is M x K, B is K x N).  The reference
 * declares this product (Sparse::Cuda::Gemm over arrays of SparseMatrix,
 * Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:16-42, with device
 * helpers in Sources/Sapphire/compute/cudaUtil/SparseUtil.cu) and defines no
 * host entry.  Element (i, j) is the sum over the entries of A's row i, in
 * storage order, of a * B[k][j], product and sum rounded separately in fp32
 * from +0 -- what the dense leaf gives on the densified operands; sums that
 * are exactly 0 are not stored (SparseUtil.cu:55-60 deletes them too); a
 * row's entries come out in ascending column order.  Column indices of B
 * must be distinct within a row.
 *
 * Two steps, like the dense -> CSR conversion: sph_spgemm_row_offsets_f32
 * computes ROWC (device, M + 1 entries; ROWC[M] = entries of C, copied to
 * *nnzHost when that is not NULL, after which the stream has drained), the
 * caller sizes VC / COLC, and sph_spgemm_fill_f32 writes them. */
int sph_spgemm_row_offsets_f32(uint32_t* ROWC, const float* VA,
                               const uint32_t* COLA, const uint32_t* ROWA,
                               const float* VB, const uint32_t* COLB,
                               const uint32_t* ROWB, uint32_t M, uint32_t K,
                               uint32_t N, uint32_t* nnzHost);
int sph_spgemm_fill_f32(float* VC, uint32_t* COLC, const uint32_t* ROWC,
                        const float* VA, const uint32_t* COLA,
                        const uint32_t* ROWA, const float* VB,
                        const uint32_t* COLB, const uint32_t* ROWB, uint32_t M,
                        uint32_t K, uint32_t N);
/* sph_spgemm_f32: the same product in one call for a caller that can bound
 * the number of entries of C beforehand (VC and COLC hold `capacity` entries).
 * ROWC is always complete and ROWC[M] the true count; only entries with an
 * index below `capacity` are stored: when the count turns out larger, grow VC
 * and COLC and call sph_spgemm_fill_f32 with the ROWC already there.  The
 * products are computed once instead of twice: the counting pass also writes
 * every row into a staging slot of 2 * capacity / M + 64 entries (a
 * stream-ordered scratch allocation of 8 bytes per slot entry), the counts
 * are scanned, a small kernel moves the staged rows into place and only rows
 * that did not fit their slot are multiplied again.  nnzHost as in
 * sph_spgemm_row_offsets_f32.  Refused during graph capture.  Same ROWC, VC
 * and COLC, bit for bit, as the two calls above. */
int sph_spgemm_f32(float* VC, uint32_t* COLC, uint32_t* ROWC,
                   uint32_t capacity, const float* VA, const uint32_t* COLA,
                   const uint32_t* ROWA, const float* VB, const uint32_t* COLB,
                   const uint32_t* ROWB, uint32_t M, uint32_t K, uint32_t N,
                   uint32_t* nnzHost);
/* sph_spgemm_load_u32: the load-distribution pre-pass the reference declares
 * (LoadDistKernel, "assigns number of calculation for each element",
 * Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:48-60): load[p] = the
 * number of entries in the row of B that entry p of A selects, i.e. the
 * multiplications entry p causes (0 for a column >= K).  `entries` = entries
 * of A.  With productsHost != NULL the sum of all loads -- the number of
 * products, an upper bound on the entries of A * B and so a safe `capacity`
 * for sph_spgemm_f32 -- is copied to *productsHost and the call returns after
 * the stream has drained (refused during graph capture); load may be NULL
 * when only that sum is wanted. */
int sph_spgemm_load_u32(uint32_t* load, const uint32_t* COLA,
                        const uint32_t* ROWB, uint32_t entries, uint32_t K,
                        uint64_t* productsHost);

#ifdef __cplusplus
}
#endif
#endif
