// C entry points over the C++ operator layer so that the Python parity tests can drive it the
// way the reference's own tests drive Compute::Gemm and friends: build TensorData objects,
// move them to the device, call the operator, bring the result back
// (Tests/UnitTests/Sources/FunctionTest/GemmTest.cpp:20-84, BroadcastTest.cpp:20-202).
// Every function returns 0 on success and -1 after catching an exception, whose text
// sphh_last_error() returns.
#include <Sapphire/compute/BasicOps.hpp>
#include <Sapphire/compute/BroadcastPlan.hpp>
#include <Sapphire/compute/Initialize.hpp>
#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/compute/sparse/Sparse.hpp>
#include <Sapphire/compute/sparse/SparseGemm.hpp>
#include <Sapphire/operations/Backward/LinearBackward.hpp>
#include <Sapphire/operations/Backward/MathBackward.hpp>
#include <Sapphire/operations/Forward/LinearForward.hpp>
#include <Sapphire/util/BlockPool.hpp>
#include <Sapphire/util/ResourceManager.hpp>

#include <sapphire_hip.h>
#include <sph_k_partition.h>

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <exception>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

using namespace Sapphire;
using TensorUtil::TensorData;

namespace
{
thread_local std::string lastError;

Shape MakeShape(const int* dims, int n)
{
    return Shape(std::vector<int>(dims, dims + n));
}

template <typename F>
int Guard(F&& body)
{
    try
    {
        body();
        return 0;
    }
    catch (const std::exception& e)
    {
        lastError = e.what();
        return -1;
    }
}

// A device tensor holding `values`: built in Host mode, filled, then sent with ToCuda(), the
// sequence the reference's tests use.
TensorData Upload(const Shape& shape, const float* values, const CudaDevice& device)
{
    TensorData t(shape, Type::Dense, device);
    t.SetMode(ComputeMode::Host);
    t.SetData(std::vector<float>(values, values + shape.Size()));
    t.ToCuda();
    return t;
}

void Download(TensorData& t, float* out)
{
    t.ToHost();
    std::memcpy(out, t.HostRawPtr(), t.HostTotalSize * sizeof(float));
}
}  // namespace

extern "C" {

const char* sphh_last_error()
{
    return lastError.c_str();
}

// op 0: Expand(arg), 1: Shrink(arg), 2: Squeeze(), 3: GetTranspose; returns the new Dim
int sphh_shape_op(const int* dims, int n, int op, int arg, int* outDims)
{
    int result = -1;
    Guard([&] {
        Shape s = MakeShape(dims, n);
        if (op == 0)
            s.Expand(arg);
        else if (op == 1)
            s.Shrink(arg);
        else if (op == 2)
            s.Squeeze();
        else
            s = s.GetTranspose();
        for (int i = 0; i < s.Dim(); ++i)
            outDims[i] = s.At(i);
        result = s.Dim();
    });
    return result;
}

// what 0: Rows, 1: Cols, 2: Size, 3: GetNumUnits(arg), 4: GetUnitSize(arg)
int sphh_shape_query(const int* dims, int n, int what, int arg)
{
    int result = -1;
    Guard([&] {
        const Shape s = MakeShape(dims, n);
        switch (what)
        {
            case 0: result = s.Rows(); break;
            case 1: result = s.Cols(); break;
            case 2: result = s.Size(); break;
            case 3: result = s.GetNumUnits(arg); break;
            default: result = s.GetUnitSize(arg); break;
        }
    });
    return result;
}

// The buffer pool's bookkeeping on fake memory and fake streams (no device): `ops` holds
// triples (code, stream, argument) with code 0 = volatile request of `argument` bytes,
// 1 = preserved request, 2 = Clean, 3 = FreePreserved(block `argument`), 4 = ClearFree,
// 5 = ClearVolatile, 6 = ClearPreserved; `stream` (1, 2, ...) is the stream of the thread that
// makes the call.  The log receives triples (event, a, b): event 0 = block a handed out,
// 1 = block a allocated, 2 = block a released on stream b, 3 = stream a made to wait for
// stream b.  Returns the number of log triples written, -1 on an exception.
namespace
{
struct FakeMemory
{
    long long* log = nullptr;
    int cap = 0, used = 0;
    long long nextBlock = 1;
    long long stream = 0;
    void Log(long long e, long long a, long long b)
    {
        if (used < cap)
        {
            log[3 * used] = e;
            log[3 * used + 1] = a;
            log[3 * used + 2] = b;
        }
        ++used;
    }
};
FakeMemory* gFake = nullptr;
void* FakeAllocate(std::size_t)
{
    const long long id = gFake->nextBlock++;
    gFake->Log(1, id, 0);
    return reinterpret_cast<void*>(static_cast<uintptr_t>(id));
}
void FakeRelease(void* ptr)
{
    gFake->Log(2, static_cast<long long>(reinterpret_cast<uintptr_t>(ptr)), gFake->stream);
}
void* FakeStream()
{
    return reinterpret_cast<void*>(static_cast<uintptr_t>(gFake->stream));
}
void FakeWait(void* stream)
{
    gFake->Log(3, gFake->stream, static_cast<long long>(reinterpret_cast<uintptr_t>(stream)));
}
}  // namespace

int sphh_block_pool_run(const int* ops, int count, long long* log, int logCap)
{
    int written = -1;
    Guard([&] {
        FakeMemory fake;
        fake.log = log;
        fake.cap = logCap;
        gFake = &fake;
        Util::BlockPool pool({ FakeAllocate, FakeRelease, FakeStream, FakeWait });
        for (int i = 0; i < count; ++i)
        {
            const int code = ops[3 * i], arg = ops[3 * i + 2];
            fake.stream = ops[3 * i + 1];
            void* block = reinterpret_cast<void*>(static_cast<uintptr_t>(arg));
            switch (code)
            {
                case 0:
                case 1:
                    fake.Log(0, static_cast<long long>(reinterpret_cast<uintptr_t>(
                                    pool.Get(static_cast<std::size_t>(arg), code == 1))), 0);
                    break;
                case 2: pool.Clean(); break;
                case 3: pool.FreePreserved(block, "FreePreserved"); break;
                case 4: pool.ClearFree(); break;
                case 5: pool.ClearVolatile(); break;
                default: pool.ClearPreserved(); break;
            }
        }
        gFake = nullptr;
        written = fake.used;
    });
    return written;
}

// leaves: 4 x uint64 per leaf (outOff, aOff, bOff, totalSizeOut); dims7: M N K maxDim sizes;
// strided4: [isStrided, count, strideOut, strideA, strideB]
long sphh_gemm_plan(const int* y, int yn, const int* a, int an, const int* b, int bn, int* dims7,
                    unsigned long long* leaves, long cap, long long* strided5)
{
    long count = -1;
    Guard([&] {
        const Compute::GemmPlan plan = Compute::PlanGemm(MakeShape(y, yn), MakeShape(a, an),
                                                         MakeShape(b, bn));
        dims7[0] = static_cast<int>(plan.M);
        dims7[1] = static_cast<int>(plan.N);
        dims7[2] = static_cast<int>(plan.K);
        dims7[3] = plan.maxDim;
        dims7[4] = plan.sizeOut;
        dims7[5] = plan.sizeA;
        dims7[6] = plan.sizeB;
        long i = 0;
        for (const auto& leaf : plan.leaves)
        {
            if (i < cap)
            {
                leaves[4 * i + 0] = leaf.outOff;
                leaves[4 * i + 1] = leaf.aOff;
                leaves[4 * i + 2] = leaf.bOff;
                leaves[4 * i + 3] = leaf.totalSizeOut;
            }
            ++i;
        }
        std::uint32_t n = 0;
        std::int64_t so = 0, sa = 0, sb = 0;
        strided5[0] = Compute::AsStridedBatch(plan, n, so, sa, sb) ? 1 : 0;
        strided5[1] = n;
        strided5[2] = so;
        strided5[3] = sa;
        strided5[4] = sb;
        count = i;
    });
    return count;
}

// y (holding yData on entry) += a * b through Compute::Gemm in Cuda mode
int sphh_compute_gemm(float* yData, const int* y, int yn, const float* aData, const int* a, int an,
                      const float* bData, const int* b, int bn)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData A = Upload(MakeShape(a, an), aData, cuda);
        TensorData B = Upload(MakeShape(b, bn), bData, cuda);
        TensorData Out = Upload(MakeShape(y, yn), yData, cuda);
        Compute::Gemm(Out, A, B);
        Download(Out, yData);
        Util::ResourceManager::Clean();
    });
}

// The K partition of the few-tile GEMM kernels, computed by the code the kernels use
// (sapphire_amd/csrc/sph_k_partition.h).  out: gBegin, gEnd, whole, wholeEnd, lastWhole,
// roundsEnd, ownsPartial.  No device is touched.
int sphh_k_partition(unsigned K, unsigned groupK, unsigned waves, unsigned wave, unsigned depth,
                     unsigned* out)
{
    const sph::KPartition p = sph::PartitionK(K, groupK, waves, wave, depth);
    out[0] = p.gBegin;
    out[1] = p.gEnd;
    out[2] = p.whole;
    out[3] = p.wholeEnd;
    out[4] = p.lastWhole;
    out[5] = p.roundsEnd;
    out[6] = p.ownsPartial ? 1u : 0u;
    return 0;
}

// slot d of the load pipeline: the group it holds before the first round (g == 0xffffffff) or
// the one loaded while round g .. g + depth - 1 is multiplied
unsigned sphh_k_partition_slot(unsigned K, unsigned groupK, unsigned waves, unsigned wave,
                               unsigned depth, unsigned g, unsigned d)
{
    const sph::KPartition p = sph::PartitionK(K, groupK, waves, wave, depth);
    return g == 0xffffffffu ? sph::KPartitionFirst(p, d) : sph::KPartitionNext(p, g, depth, d);
}

// Compute::Gemm into a FRESH y (never filled, never read): the operator sees the deferred zero
// state of the new buffer and stores the product.  yOut receives the result.
int sphh_compute_gemm_fresh_y(float* yOut, const int* y, int yn, const float* aData, const int* a,
                              int an, const float* bData, const int* b, int bn)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData A = Upload(MakeShape(a, an), aData, cuda);
        TensorData B = Upload(MakeShape(b, bn), bData, cuda);
        TensorData Out(MakeShape(y, yn), Type::Dense, cuda);
        Compute::Gemm(Out, A, B);
        Download(Out, yOut);
        Util::ResourceManager::Clean();
    });
}

// Compute::GemmHalf on device arrays of binary16 bit patterns.  freshY != 0: y is a new
// TensorData (deferred zero fill, the product is stored); otherwise y holds yData and the
// product is added to it.  yData receives the result.
int sphh_gemm_half(float* yData, const int* y, int yn, const std::uint16_t* aDev,
                   const std::uint16_t* bDev, unsigned int K, int freshY)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData Out = freshY ? TensorData(MakeShape(y, yn), Type::Dense, cuda)
                                : Upload(MakeShape(y, yn), yData, cuda);
        Compute::GemmHalf(Out, aDev, bDev, K);
        Download(Out, yData);
        Util::ResourceManager::Clean();
    });
}

// Times `steps` passes of: take a fresh y [n, n] from the pool, y += a * b through
// Compute::GemmHalf, hand the pass's blocks back (ResourceManager::Clean(), what a model does at
// the end of a pass).  settleMs of the same passes run untimed first.  eventMs: per pass from
// events on the thread's stream; wallMs: per pass between two stream synchronisations.
int sphh_bench_gemm_half_fresh_y(const std::uint16_t* aDev, const std::uint16_t* bDev, int n,
                                 int steps, int warmup, double settleMs, float* eventMs,
                                 double* wallMs)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        Compute::Cuda::CudaSetDevice(0);
        auto pass = [&] {
            TensorData y(Shape({ n, n }), Type::Dense, cuda);
            Compute::GemmHalf(y, aDev, bDev, static_cast<unsigned int>(n));
            Util::ResourceManager::Clean();
        };
        auto require = [](int rc, const char* what) {
            if (rc != SPH_OK)
                throw std::runtime_error(std::string(what) + " failed with " + sph_last_error());
        };
        const auto t0 = std::chrono::steady_clock::now();
        auto elapsedMs = [&](std::chrono::steady_clock::time_point from) {
            return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - from)
                .count();
        };
        while (elapsedMs(t0) < settleMs)
        {
            for (int i = 0; i < 20; ++i)
                pass();
            require(sph_stream_sync(), "sph_stream_sync");
        }
        for (int i = 0; i < warmup; ++i)
            pass();
        require(sph_stream_sync(), "sph_stream_sync");
        void *begin = nullptr, *end = nullptr;
        require(sph_event_create(&begin), "sph_event_create");
        require(sph_event_create(&end), "sph_event_create");
        const auto w0 = std::chrono::steady_clock::now();
        require(sph_event_record(begin), "sph_event_record");
        for (int i = 0; i < steps; ++i)
            pass();
        require(sph_event_record(end), "sph_event_record");
        require(sph_stream_sync(), "sph_stream_sync");
        *wallMs = elapsedMs(w0) / steps;
        float ms = 0;
        require(sph_event_elapsed_ms(begin, end, &ms), "sph_event_elapsed_ms");
        *eventMs = ms / static_cast<float>(steps);
        sph_event_destroy(begin);
        sph_event_destroy(end);
        Util::ResourceManager::ClearAll();
    });
}

// Compute::Gemm on Host-mode tensors must throw: returns 1 when it does
int sphh_gemm_in_host_mode_throws()
{
    TensorData A(Shape({ 2, 2 }), Type::Dense), B(Shape({ 2, 2 }), Type::Dense),
        Y(Shape({ 2, 2 }), Type::Dense);
    const int rc = Guard([&] { Compute::Gemm(Y, A, B); });
    Util::ResourceManager::Clean();
    return rc == -1 ? 1 : 0;
}

// layers Linear -> ReLU -> ... -> Linear (no ReLU after the last), sizes has layers + 1 entries
int sphh_mlp_forward(const float* x, int batch, const int* sizes, int layers,
                     const float* const* weights, const float* const* biases, float* out,
                     int fused)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData cur = Upload(Shape({ batch, sizes[0] }), x, cuda);
        for (int l = 0; l < layers; ++l)
        {
            TensorData W = Upload(Shape({ sizes[l], sizes[l + 1] }), weights[l], cuda);
            TensorData bias = Upload(Shape({ sizes[l + 1] }), biases[l], cuda);
            TensorData y(Shape({ batch, sizes[l + 1] }), Type::Dense, cuda);  // zero-filled
            if (fused)
            {
                // one launch per layer, activation included
                NN::LinearForwardFused(y, cur, W, bias, l + 1 < layers);
                cur = y;
                continue;
            }
            NN::LinearForward(y, cur, W, bias);
            if (l + 1 < layers)
            {
                TensorData act(y.GetShape(), Type::Dense, cuda);
                Compute::ReLU(act, y);
                cur = act;
            }
            else
                cur = y;
        }
        Download(cur, out);
        Util::ResourceManager::Clean();
    });
}

int sphh_transpose(float* yData, const int* y, int yn, const float* xData, const int* x, int xn)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData X = Upload(MakeShape(x, xn), xData, cuda);
        TensorData Y(MakeShape(y, yn), Type::Dense, cuda);
        Compute::Transpose(Y, X);
        Download(Y, yData);
        Util::ResourceManager::Clean();
    });
}

// Util::GetMatchingDim over `count` shapes stored back to back, dims[i] extents each
int sphh_matching_dim(const int* flat, const int* dims, int count)
{
    int result = -1;
    const int rc = Guard([&] {
        std::vector<Shape> shapes;
        for (int i = 0; i < count; ++i)
        {
            shapes.push_back(MakeShape(flat, dims[i]));
            flat += dims[i];
        }
        result = Compute::GetMatchingDim(shapes);
    });
    return rc == 0 ? result : -1;
}

// y = a - b through Compute::Sub in Cuda mode
int sphh_sub(float* yData, const int* y, int yn, const float* aData, const int* a, int an,
             const float* bData, const int* b, int bn)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData A = Upload(MakeShape(a, an), aData, cuda);
        TensorData B = Upload(MakeShape(b, bn), bData, cuda);
        TensorData Out = Upload(MakeShape(y, yn), yData, cuda);
        Compute::Sub(Out, A, B);
        Download(Out, yData);
        Util::ResourceManager::Clean();
    });
}

// y = x * factor through Compute::Scale; inPlace scales x itself
int sphh_scale(float* yData, const float* xData, int n, float factor, int inPlace)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData X = Upload(Shape({ n }), xData, cuda);
        if (inPlace)
        {
            Compute::Scale(X, X, factor);
            Download(X, yData);
        }
        else
        {
            TensorData Y(Shape({ n }), Type::Dense, cuda);
            Compute::Scale(Y, X, factor);
            Download(Y, yData);
        }
        Util::ResourceManager::Clean();
    });
}

// dx (holding dxData on entry) += x > 0 ? dy : 0 through Compute::ReLUBackward
int sphh_relu_backward(float* dxData, const float* dyData, const float* xData, int n)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData Dx = Upload(Shape({ n }), dxData, cuda);
        TensorData Dy = Upload(Shape({ n }), dyData, cuda);
        TensorData X = Upload(Shape({ n }), xData, cuda);
        Compute::ReLUBackward(Dx, Dy, X);
        Download(Dx, dxData);
        Util::ResourceManager::Clean();
    });
}

// BackProp::LinearBackward with an SGD optimizer.  dx, weight and bias are updated in place.
// sequence: 0 the reference's operator calls, 1 direct; fusedSgd selects the one-pass update.
int sphh_linear_backward(float* dx, float* weight, float* bias, const float* dy, const float* x,
                         int batch, int inputs, int outputs, float learningRate, int sequence,
                         int fusedSgd)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData Dx = Upload(Shape({ batch, inputs }), dx, cuda);
        TensorData W = Upload(Shape({ inputs, outputs }), weight, cuda);
        TensorData B = Upload(Shape({ outputs }), bias, cuda);
        TensorData Dy = Upload(Shape({ batch, outputs }), dy, cuda);
        TensorData X = Upload(Shape({ batch, inputs }), x, cuda);
        const Optimizer::SGD sgd(learningRate, fusedSgd != 0);
        BackProp::LinearBackward(Dx, W, B, Dy, X, static_cast<unsigned int>(batch), sgd,
                                 sequence == 0 ? BackProp::Sequence::Reference
                                               : BackProp::Sequence::Direct);
        Download(Dx, dx);
        Download(W, weight);
        Download(B, bias);
        Util::ResourceManager::Clean();
    });
}

// Dense (host, numMatrices x m x paddedN) -> device -> CreateSparseMatrixWithDenseMatrix ->
// DeepCopyDeviceToDevice into fresh records -> DeepCopyDeviceToHost -> out arrays (entries of
// all matrices back to back in V / COL, m + 1 offsets per matrix in ROW, counts in nnz), and
// ConvertSparseMatrixToDenseMatrix of the copied records into denseBack, which is pre-filled
// with `fill` so that untouched padding stays visible.  capacity bounds V / COL.
int sphh_csr_round_trip(const float* dense, unsigned m, unsigned n, unsigned paddedN,
                        unsigned numMatrices, unsigned* nnz, float* V, unsigned* COL,
                        unsigned* ROW, unsigned long capacity, float* denseBack, float fill)
{
    return Guard([&] {
        const std::size_t total = static_cast<std::size_t>(numMatrices) * m * paddedN;
        const std::size_t bytes = std::max<std::size_t>(total, 1) * sizeof(float);
        Compute::Cuda::CudaSetDevice(0);
        void* dDense = nullptr;
        void* dBack = nullptr;
        Compute::Cuda::CudaMalloc(&dDense, bytes);
        Compute::Cuda::CudaMalloc(&dBack, bytes);
        SparseMatrix* created = nullptr;
        SparseMatrix* copied = nullptr;
        SparseMatrix* host = nullptr;
        try
        {
            Compute::Cuda::CopyHostToDevice(dDense, dense, total * sizeof(float));
            Compute::CreateSparseMatrixWithDenseMatrix(&created, static_cast<const float*>(dDense),
                                                       m, n, paddedN, numMatrices, 0);
            Compute::DeepAllocateSparseCuda(&copied, created, numMatrices, 0);
            Compute::DeepCopyDeviceToDevice(copied, created, numMatrices, 0);
            std::vector<uint32_t> counts(numMatrices);
            for (unsigned i = 0; i < numMatrices; ++i)
                counts[i] = nnz[i] = copied[i].NNZ;
            Compute::DeepAllocateSparseHost(&host, m, n, counts.data(), numMatrices);
            Compute::DeepCopyDeviceToHost(host, copied, numMatrices, 0);
            std::size_t at = 0;
            for (unsigned i = 0; i < numMatrices; ++i)
            {
                if (at + host[i].NNZ > capacity)
                    throw std::runtime_error("sphh_csr_round_trip - capacity too small");
                std::memcpy(V + at, host[i].V, host[i].NNZ * sizeof(float));
                std::memcpy(COL + at, host[i].COL, host[i].NNZ * sizeof(unsigned));
                std::memcpy(ROW + static_cast<std::size_t>(i) * (m + 1), host[i].ROW,
                            (static_cast<std::size_t>(m) + 1) * sizeof(unsigned));
                at += host[i].NNZ;
            }
            Compute::Dense::Cuda::Scalar(static_cast<float*>(dBack), fill, total);
            Compute::ConvertSparseMatrixToDenseMatrix(static_cast<float*>(dBack), copied, m, n,
                                                      paddedN, numMatrices, 0);
            Compute::Cuda::CopyDeviceToHost(denseBack, dBack, total * sizeof(float));
        }
        catch (...)
        {
            Compute::DeepFreeSparseHost(host, numMatrices);
            Compute::DeepFreeSparseCuda(copied, numMatrices, 0);
            Compute::DeepFreeSparseCuda(created, numMatrices, 0);
            Compute::Cuda::CudaFree(dDense);
            Compute::Cuda::CudaFree(dBack);
            throw;
        }
        Compute::DeepFreeSparseHost(host, numMatrices);
        Compute::DeepFreeSparseCuda(copied, numMatrices, 0);
        Compute::DeepFreeSparseCuda(created, numMatrices, 0);
        Compute::Cuda::CudaFree(dDense);
        Compute::Cuda::CudaFree(dBack);
        Util::ResourceManager::Clean();
    });
}

// NN::SparseLinearForward: the weight arrives dense [inputs, outputs] on the host, is sent to
// the device, transposed there and converted to CSR there.
int sphh_sparse_linear_forward(const float* x, int batch, int inputs, int outputs,
                               const float* weight, const float* bias, float* y)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData X = Upload(Shape({ batch, inputs }), x, cuda);
        TensorData W = Upload(Shape({ inputs, outputs }), weight, cuda);
        TensorData B = Upload(Shape({ outputs }), bias, cuda);
        TensorData Wt(Shape({ outputs, inputs }), Type::Dense, cuda);
        Compute::Transpose(Wt, W);
        SparseMatrix* record = nullptr;
        Compute::CreateSparseMatrixWithDenseMatrix(&record, Wt.CudaRawPtr(),
                                                   static_cast<uint32_t>(outputs),
                                                   static_cast<uint32_t>(inputs),
                                                   static_cast<uint32_t>(inputs), 1, 0);
        TensorData Y(Shape({ batch, outputs }), Type::Dense, cuda);
        try
        {
            NN::SparseLinearForward(Y, X, record[0], B);
            Download(Y, y);
        }
        catch (...)
        {
            Compute::DeepFreeSparseCuda(record, 1, 0);
            throw;
        }
        Compute::DeepFreeSparseCuda(record, 1, 0);
        Util::ResourceManager::Clean();
    });
}

// Sparse::Cuda::Gemm on one pair of matrices given dense on the host: both are sent to the
// device and converted to CSR there; the product comes back as host CSR arrays (nnz, ROW with
// m + 1 entries, V / COL up to `capacity`).
int sphh_sparse_sparse_gemm(const float* denseA, const float* denseB, unsigned m, unsigned k,
                            unsigned n, unsigned* nnz, unsigned* ROW, float* V, unsigned* COL,
                            unsigned long capacity)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData A = Upload(Shape({ static_cast<int>(m), static_cast<int>(k) }), denseA, cuda);
        TensorData B = Upload(Shape({ static_cast<int>(k), static_cast<int>(n) }), denseB, cuda);
        SparseMatrix* a = nullptr;
        SparseMatrix* b = nullptr;
        SparseMatrix* cDevice = nullptr;
        SparseMatrix* cHost = nullptr;
        try
        {
            Compute::CreateSparseMatrixWithDenseMatrix(&a, A.CudaRawPtr(), m, k, k, 1, 0);
            Compute::CreateSparseMatrixWithDenseMatrix(&b, B.CudaRawPtr(), k, n, n, 1, 0);
            Compute::Sparse::Cuda::Gemm(&cHost, &cDevice, a, b, m, n, 1, 0, true);
            *nnz = cHost[0].NNZ;
            if (cHost[0].NNZ > capacity)
                throw std::runtime_error("sphh_sparse_sparse_gemm - capacity too small");
            std::memcpy(ROW, cHost[0].ROW, (static_cast<std::size_t>(m) + 1) * sizeof(unsigned));
            std::memcpy(V, cHost[0].V, cHost[0].NNZ * sizeof(float));
            std::memcpy(COL, cHost[0].COL, cHost[0].NNZ * sizeof(unsigned));
        }
        catch (...)
        {
            Compute::DeepFreeSparseHost(cHost, 1);
            Compute::DeepFreeSparseCuda(cDevice, 1, 0);
            Compute::DeepFreeSparseCuda(b, 1, 0);
            Compute::DeepFreeSparseCuda(a, 1, 0);
            throw;
        }
        Compute::DeepFreeSparseHost(cHost, 1);
        Compute::DeepFreeSparseCuda(cDevice, 1, 0);
        Compute::DeepFreeSparseCuda(b, 1, 0);
        Compute::DeepFreeSparseCuda(a, 1, 0);
        Util::ResourceManager::Clean();
    });
}

// The load-distribution records of the sparse x sparse product for one pair of matrices given
// dense on the host: GetLoadDist into a host record, then that record through every
// LoadDistMatrix copy overload (host -> host, host -> device, device -> device, device -> host),
// and CallLoadDist for the number of products.  load / col hold `capacity` entries, row m + 1.
int sphh_load_dist(const float* denseA, const float* denseB, unsigned m, unsigned k, unsigned n,
                   unsigned* nnzA, unsigned* load, unsigned* col, unsigned* row,
                   unsigned* products, unsigned long capacity)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData A = Upload(Shape({ static_cast<int>(m), static_cast<int>(k) }), denseA, cuda);
        TensorData B = Upload(Shape({ static_cast<int>(k), static_cast<int>(n) }), denseB, cuda);
        SparseMatrix* a = nullptr;
        SparseMatrix* b = nullptr;
        LoadDistMatrix* host = nullptr;
        LoadDistMatrix* hostCopy = nullptr;
        LoadDistMatrix* device = nullptr;
        LoadDistMatrix* deviceCopy = nullptr;
        auto release = [&] {
            Compute::DeepFreeLoadDistCuda(deviceCopy, 1, 0);
            Compute::DeepFreeLoadDistCuda(device, 1, 0);
            Compute::DeepFreeLoadDistHost(hostCopy, 1);
            Compute::DeepFreeLoadDistHost(host, 1);
            Compute::DeepFreeSparseCuda(b, 1, 0);
            Compute::DeepFreeSparseCuda(a, 1, 0);
        };
        try
        {
            Compute::CreateSparseMatrixWithDenseMatrix(&a, A.CudaRawPtr(), m, k, k, 1, 0);
            Compute::CreateSparseMatrixWithDenseMatrix(&b, B.CudaRawPtr(), k, n, n, 1, 0);
            *nnzA = a[0].NNZ;
            if (a[0].NNZ > capacity)
                throw std::runtime_error("sphh_load_dist - capacity too small");
            Compute::DeepAllocateLoadDistHost(&host, a, 1);
            Compute::Sparse::Cuda::GetLoadDist(host, a, b, m, 1, 0);
            Compute::DeepAllocateLoadDistHost(&hostCopy, a, 1);
            Compute::DeepCopyHostToHost(hostCopy, host, 1);
            Compute::DeepAllocateLoadDistCuda(&device, hostCopy, 1, 0);
            Compute::DeepCopyHostToDevice(device, hostCopy, 1, 0);
            Compute::DeepAllocateLoadDistCuda(&deviceCopy, hostCopy, 1, 0);
            Compute::DeepCopyDeviceToDevice(deviceCopy, device, 1, 0);
            std::memset(hostCopy[0].Load, 0xff, static_cast<std::size_t>(a[0].NNZ) * 4);
            Compute::DeepCopyDeviceToHost(hostCopy, deviceCopy, 1, 0);
            std::memcpy(load, hostCopy[0].Load, static_cast<std::size_t>(a[0].NNZ) * 4);
            std::memcpy(col, hostCopy[0].COL, static_cast<std::size_t>(a[0].NNZ) * 4);
            std::memcpy(row, hostCopy[0].ROW, (static_cast<std::size_t>(m) + 1) * 4);
            if (hostCopy[0].M != m || hostCopy[0].N != k || hostCopy[0].NNZ != a[0].NNZ)
                throw std::runtime_error("sphh_load_dist - record counters were not carried over");
            Compute::Sparse::Cuda::CallLoadDist(a, b, device, m, products, 1, 0);
        }
        catch (...)
        {
            release();
            throw;
        }
        release();
        Util::ResourceManager::Clean();
    });
}

// BackProp::MatMulBackward: da and db hold values on entry and are accumulated into.
int sphh_matmul_backward(float* da, float* db, const float* dy, const float* a, const float* b,
                         const int* aShape, int an, const int* bShape, int bn, const int* yShape,
                         int yn, int sequence)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        TensorData A = Upload(MakeShape(aShape, an), a, cuda);
        TensorData B = Upload(MakeShape(bShape, bn), b, cuda);
        TensorData Dy = Upload(MakeShape(yShape, yn), dy, cuda);
        TensorData Da = Upload(MakeShape(aShape, an), da, cuda);
        TensorData Db = Upload(MakeShape(bShape, bn), db, cuda);
        BackProp::MatMulBackward(Da, Db, Dy, A, B,
                                 sequence == 0 ? BackProp::Sequence::Reference
                                               : BackProp::Sequence::Direct);
        Download(Da, da);
        Download(Db, db);
        Util::ResourceManager::Clean();
    });
}

int sphh_sparse_gemm(float* yData, int M, int K, int N, const float* V, const unsigned* COL,
                     const unsigned* ROW, const float* bData, int accumulate)
{
    return Guard([&] {
        const CudaDevice cuda(0, "device0");
        const unsigned nnz = ROW[M];
        SparseMatrix m = Compute::Sparse::Cuda::CreateSparseMatrix(
            std::vector<float>(V, V + nnz), std::vector<uint32_t>(COL, COL + nnz),
            std::vector<uint32_t>(ROW, ROW + M + 1), static_cast<uint32_t>(M),
            static_cast<uint32_t>(K), 0);
        TensorData A;
        A.SparseMatCuda = &m;
        TensorData B = Upload(Shape({ K, N }), bData, cuda);
        TensorData Y = Upload(Shape({ M, N }), yData, cuda);
        Compute::SparseGemm(Y, A, B, accumulate != 0);
        Download(Y, yData);
        Compute::Sparse::Cuda::FreeSparseMatrix(m);
        Util::ResourceManager::Clean();
    });
}

// Life cycle checks of TensorData / ResourceManager on the device; returns 0 when all hold,
// otherwise the number of the first failed check (text in sphh_last_error()).
int sphh_tensor_lifecycle()
{
    int failed = 0;
    const int rc = Guard([&] {
        auto check = [&](bool ok, int id, const char* what) {
            if (!ok && failed == 0)
            {
                failed = id;
                lastError = what;
            }
        };
        Util::ResourceManager::ClearAll();
        const CudaDevice cuda(0, "device0");
        {
            TensorData t(Shape({ 3, 5 }), Type::Dense, cuda);
            check(t.Mode() == ComputeMode::Cuda, 1, "device tensor starts in Cuda mode");
            std::vector<float> v = t.GetDataCopy();
            bool zero = true;
            for (float f : v)
                zero = zero && f == 0.0f;
            check(v.size() == 15 && zero, 2, "fresh device buffer is zero");
            std::vector<float> data(15);
            for (int i = 0; i < 15; ++i)
                data[i] = static_cast<float>(i) - 7.f;
            t.SetData(data);
            TensorData view = t;  // shallow
            check(view.CudaRawPtr() == t.CudaRawPtr(), 3, "copies alias the buffer");
            view.Reshape(Shape({ 15 }));
            check(view.GetDataCopy() == data, 4, "reshaped view sees the same values");
            t.ToHost();
            check(t.Mode() == ComputeMode::Host && t.HostRawPtr()[14] == 7.f, 5, "ToHost copies");
            t.HostMutableRawPtr()[0] = 42.f;
            t.ToCuda();
            check(t.GetDataCopy()[0] == 42.f, 6, "ToCuda copies");
            TensorData copy = t.CreateCopy();
            check(copy.CudaRawPtr() != t.CudaRawPtr() && copy.GetDataCopy() == t.GetDataCopy(), 7,
                  "CreateCopy is deep");
            bool threw = false;
            try
            {
                t.SetData(std::vector<float>(3));
            }
            catch (const std::invalid_argument&)
            {
                threw = true;
            }
            check(threw, 8, "SetData with a wrong size throws");
            threw = false;
            try
            {
                t.Reshape(Shape({ 4, 4 }));
            }
            catch (const std::runtime_error&)
            {
                threw = true;
            }
            check(threw, 9, "Reshape to another size throws");
        }
        const auto before = Util::ResourceManager::Statistics();
        check(before.cudaVolatile >= 2 && before.cudaFree == 0, 10, "blocks are volatile while in use");
        Util::ResourceManager::Clean();
        const auto cleaned = Util::ResourceManager::Statistics();
        check(cleaned.cudaVolatile == 0 && cleaned.cudaFree == before.cudaVolatile, 11,
              "Clean moves volatile blocks to the free pool");
        {
            TensorData again(Shape({ 3, 5 }), Type::Dense, cuda);
            const auto reused = Util::ResourceManager::Statistics();
            check(reused.cudaFree == cleaned.cudaFree - 1, 12, "an equal-size request reuses a free block");
            std::vector<float> v = again.GetDataCopy();
            bool zero = true;
            for (float f : v)
                zero = zero && f == 0.0f;
            check(zero, 13, "a reused block is zero-filled again");
        }
        {
            TensorData hostOnly(Shape({ 4 }), Type::Dense);
            bool threw = false;
            try
            {
                hostOnly.SetMode(ComputeMode::Cuda);
            }
            catch (const std::runtime_error&)
            {
                threw = true;
            }
            check(threw, 14, "SetMode(Cuda) without a device throws");
        }
        {
            bool threw = false;
            try
            {
                Compute::Cuda::CudaSetDevice(99);
            }
            catch (const std::runtime_error& e)
            {
                threw = std::string(e.what()).find("exceeds number of available devices") !=
                        std::string::npos;
            }
            check(threw, 15, "CudaSetDevice out of range throws");
        }
        Util::ResourceManager::ClearAll();
        const auto end = Util::ResourceManager::Statistics();
        check(end.cudaVolatile + end.cudaFree + end.cudaPreserved == 0, 16, "ClearAll releases everything");
    });
    if (rc != 0)
        return -1;
    return failed;
}

// Host-only checks (no device): pools, TensorData in Host mode, error paths.
// A device block that passes from one thread's stream to another's through the pool: the
// first thread keeps its stream busy writing 1 into the block, returns the block with Clean()
// without waiting, and a second thread takes the block of that size, writes 2 and reads it
// back.  Every element must read 2: the second stream has to wait for the first one's writes.
// Returns 0 when that holds, 1 when the block was not reused, 2 when stale values were seen.
int sphh_pool_handover()
{
    int result = -1;
    Guard([&] {
        Util::ResourceManager::ClearAll();
        Compute::Cuda::CudaSetDevice(0);
        const std::size_t count = std::size_t(16) << 20;  // 64 MiB of floats
        float* first = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(count * 4));
        for (int i = 0; i < 40; ++i)
            Compute::Dense::Cuda::Scalar(first, 1.0f, count);
        Util::ResourceManager::Clean();  // no wait: the writes above are still in flight
        int outcome = 0;
        std::thread second([&] {
            try
            {
                Compute::Cuda::CudaSetDevice(0);
                float* block = static_cast<float*>(Util::ResourceManager::GetMemoryCuda(count * 4));
                if (block != first)
                    outcome = 1;
                Compute::Dense::Cuda::Scalar(block, 2.0f, count);
                std::vector<float> host(count);
                Compute::Cuda::CopyDeviceToHost(host.data(), block, count * 4);
                Compute::Cuda::Synchronize();
                // give the first stream time to finish what it still had queued
                Compute::Cuda::SynchronizeDevice();
                Compute::Cuda::CopyDeviceToHost(host.data(), block, count * 4);
                for (float v : host)
                    if (v != 2.0f && outcome == 0)
                        outcome = 2;
            }
            catch (const std::exception& e)
            {
                lastError = e.what();
                outcome = 3;
            }
        });
        second.join();
        Compute::Cuda::SynchronizeDevice();
        Util::ResourceManager::ClearAll();
        result = outcome;
    });
    return result;
}

int sphh_host_only_lifecycle()
{
    int failed = 0;
    const int rc = Guard([&] {
        auto check = [&](bool ok, int id, const char* what) {
            if (!ok && failed == 0)
            {
                failed = id;
                lastError = what;
            }
        };
        {
            TensorData t(Shape({ 2, 3 }), Type::Dense);
            check(t.Mode() == ComputeMode::Host && t.HostTotalSize == 6, 1, "host tensor");
            check(t.GetDataCopy() == std::vector<float>(6, 0.f), 2, "host buffer zeroed");
            t.SetData({ 1, 2, 3, 4, 5, 6 });
            TensorData wide(Shape({ 2, 2, 3 }), Type::Dense);
            TensorData::DeepCopy(wide, t);
            const std::vector<float> twice = { 1, 2, 3, 4, 5, 6, 1, 2, 3, 4, 5, 6 };
            check(wide.GetDataCopy() == twice, 3, "DeepCopy repeats src");
            Compute::Initialize::Ones(t);
            check(t.GetDataCopy() == std::vector<float>(6, 1.f), 4, "Ones on host");
            bool threw = false;
            try
            {
                TensorData sparse(Shape({ 2, 2 }), Type::Sparse);
            }
            catch (const std::runtime_error&)
            {
                threw = true;
            }
            check(threw, 5, "sparse storage is not implemented, as in the reference");
        }
        const auto s = Util::ResourceManager::Statistics();
        check(s.hostVolatile == 2, 6, "two volatile host blocks");
        Util::ResourceManager::Clean();
        check(Util::ResourceManager::Statistics().hostFree == 2, 7, "Clean keeps them for reuse");
        void* p = Util::ResourceManager::GetMemoryHost(100, true);
        Util::ResourceManager::MoveToVolatileHost(p);
        Util::ResourceManager::MoveToPreservedHost(p);
        Util::ResourceManager::FreePreservedHost(p);
        bool threw = false;
        try
        {
            Util::ResourceManager::FreePreservedHost(p);
        }
        catch (const std::runtime_error&)
        {
            threw = true;
        }
        check(threw, 8, "freeing an unknown pointer throws");
        Util::ResourceManager::ClearFreePool();
        check(Util::ResourceManager::Statistics().hostFree == 0, 9, "ClearFreePool");
    });
    if (rc != 0)
        return -1;
    return failed;
}

}  // extern "C"
