// C entry points over the reference's own objects -- TEST INFRASTRUCTURE ONLY.
//
// This file is compiled together with the reference's sources where they lie
// (NaiveGemm.cpp, NaiveBasic.cpp, shape.cpp, Broadcast.hpp; see the Makefile)
// into oracle/_ref/libsapphire_ref.so.  It contains no arithmetic of its own:
// every function forwards to a reference function or class.  The only logic
// restated here is the host branch of Compute::Gemm
// (Sources/Sapphire/compute/BasicOps.cpp:183-248), whose translation unit
// cannot be built without CUDA headers; it is re-expressed with the
// reference's Shape class and BroadcastWith2Inputs template so that the walk
// and the leaf are still the reference's code.
#include <Sapphire/compute/Broadcast.hpp>
#include <Sapphire/compute/dense/naive/NaiveBasic.hpp>
#include <Sapphire/compute/dense/naive/NaiveGemm.hpp>
#include <Sapphire/util/Shape.hpp>

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <vector>

namespace
{
Sapphire::Shape MakeShape(const int* v, int dim)
{
    return Sapphire::Shape(std::vector<int>(v, v + dim));
}

struct Leaf
{
    uint64_t outOff, aOff, bOff;
    uint32_t totalSizeOut;
};

struct Recorder
{
    const float* outBase;
    const float* aBase;
    const float* bBase;
    Leaf* leaves;
    size_t cap;
    size_t* count;

    void operator()(unsigned int totalSize, float* out, const float* A,
                    const float* B, unsigned int, unsigned int,
                    unsigned int) const
    {
        if (*count < cap)
        {
            leaves[*count] = { static_cast<uint64_t>(out - outBase),
                               static_cast<uint64_t>(A - aBase),
                               static_cast<uint64_t>(B - bBase), totalSize };
        }
        *count += 1;
    }
};

struct GemmShapes
{
    Sapphire::Shape out, a, b;
    int M, N, K;
    int maxDim;
};

// BasicOps.cpp:189-226
GemmShapes Prepare(const int* yShape, int yDim, const int* aShape, int aDim,
                   const int* bShape, int bDim)
{
    GemmShapes g{ MakeShape(yShape, yDim), MakeShape(aShape, aDim),
                  MakeShape(bShape, bDim), 0, 0, 0, 0 };
    g.out.Expand(2);
    g.a.Expand(2);
    g.b.Expand(2);
    g.M = g.out.Rows();
    g.N = g.out.Cols();
    g.K = g.a.Cols();
    g.maxDim = std::max({ yDim, aDim, bDim });
    g.out.Expand(g.maxDim);
    g.a.Expand(g.maxDim);
    g.b.Expand(g.maxDim);
    return g;
}
}  // namespace

extern "C" {

void ref_naive_gemm(unsigned int totalSize, float* out, const float* A,
                    const float* B, unsigned int M, unsigned int N,
                    unsigned int K)
{
    Sapphire::Compute::Dense::Naive::Gemm(totalSize, out, A, B, M, N, K);
}

void ref_relu(float* out, const float* in, unsigned int totalSize)
{
    Sapphire::Compute::Dense::Naive::ReLU(out, in, totalSize);
}

void ref_transpose(float* out, const float* in, unsigned int rows,
                   unsigned int cols, unsigned int batch, int broadcast)
{
    Sapphire::Compute::Dense::Naive::Transpose(out, in, rows, cols, batch,
                                               broadcast != 0);
}

void ref_scale(float* out, const float* in, float factor, unsigned int totalSize)
{
    Sapphire::Compute::Dense::Naive::Scale(out, in, factor, totalSize);
}

void ref_sub(unsigned int totalSize, float* out, const float* A, const float* B,
             unsigned int inputStride, int broadcastA, int broadcastB)
{
    Sapphire::Compute::Dense::Naive::Sub(totalSize, out, A, B, inputStride,
                                         broadcastA != 0, broadcastB != 0);
}

void ref_relu_backward(float* dx, const float* dy, const float* x,
                       unsigned int totalSize)
{
    Sapphire::Compute::Dense::Naive::ReLUBackward(dx, dy, x, totalSize);
}

// Host branch of Compute::Sub, BasicOps.cpp:70-103, with the matching
// dimension passed in (Util::GetMatchingDim lives in a header that pulls in
// the model classes and cannot be compiled here).
void ref_compute_sub(float* y, const int* yShape, int yDim, const float* a,
                     const int* aShape, int aDim, const float* b,
                     const int* bShape, int bDim, int minRequiredDim)
{
    auto so = MakeShape(yShape, yDim);
    auto sa = MakeShape(aShape, aDim);
    auto sb = MakeShape(bShape, bDim);
    const int maxDim = std::max({ yDim, aDim, bDim });
    so.Expand(maxDim);
    sa.Expand(maxDim);
    sb.Expand(maxDim);
    Sapphire::Compute::BroadcastWith2Inputs(
        so, sa, sb, so.Size(), sa.Size(), sb.Size(), y, a, b, 0, minRequiredDim,
        Sapphire::Compute::Dense::Naive::Sub, 0, false, false);
}

// op: 0 Expand(arg), 1 Shrink(arg); writes the resulting dims, returns Dim
int ref_shape_op(const int* v, int dim, int op, int arg, int* outDims)
{
    auto s = MakeShape(v, dim);
    if (op == 0)
        s.Expand(arg);
    else
        s.Shrink(arg);
    for (int i = 0; i < s.Dim(); ++i)
        outDims[i] = s.At(i);
    return s.Dim();
}

// what: 0 Rows, 1 Cols, 2 Size, 3 GetNumUnits(arg)
int ref_shape_query(const int* v, int dim, int what, int arg)
{
    const auto s = MakeShape(v, dim);
    switch (what)
    {
        case 0: return s.Rows();
        case 1: return s.Cols();
        case 2: return s.Size();
        default: return s.GetNumUnits(arg);
    }
}

// Leaves of the reference walk for Compute::Gemm on these shapes.
// dims receives M, N, K, maxDim, sizeOut, sizeA, sizeB.
size_t ref_gemm_plan(const int* yShape, int yDim, const int* aShape, int aDim,
                     const int* bShape, int bDim, int* dims, void* leaves,
                     size_t cap)
{
    auto g = Prepare(yShape, yDim, aShape, aDim, bShape, bDim);
    dims[0] = g.M;
    dims[1] = g.N;
    dims[2] = g.K;
    dims[3] = g.maxDim;
    dims[4] = g.out.Size();
    dims[5] = g.a.Size();
    dims[6] = g.b.Size();
    // Offsets are recovered from pointer differences against a base that is
    // never dereferenced by the recorder.
    static float anchor[1];
    float* base = anchor;
    size_t count = 0;
    Recorder rec{ base, base, base, static_cast<Leaf*>(leaves), cap, &count };
    Sapphire::Compute::BroadcastWith2Inputs(
        g.out, g.a, g.b, g.out.Size(), g.a.Size(), g.b.Size(), base, base,
        base, 0, 2, rec, g.M, g.N, g.K);
    return count;
}

// Host branch of Compute::Gemm, BasicOps.cpp:240-247
void ref_compute_gemm(float* y, const int* yShape, int yDim, const float* a,
                      const int* aShape, int aDim, const float* b,
                      const int* bShape, int bDim)
{
    auto g = Prepare(yShape, yDim, aShape, aDim, bShape, bDim);
    Sapphire::Compute::BroadcastWith2Inputs(
        g.out, g.a, g.b, g.out.Size(), g.a.Size(), g.b.Size(), y, a, b, 0, 2,
        Sapphire::Compute::Dense::Naive::Gemm, g.M, g.N, g.K);
}

}  // extern "C"
