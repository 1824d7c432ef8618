/*
 * CPU oracle for the Sapphire matrix-multiplication path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * host arithmetic; it exists so that tests, the smoke check and the bench's
 * cpu_baseline leg have a checker.  Nothing in the product library links it,
 * loads it or falls back to it.
 *
 * Every function names the reference file:line it follows.  How each one is
 * pinned (against the reference's own objects built into oracle/_ref, closed
 * forms and brute force) is listed next to the function.
 */
#ifndef SAPPHIRE_ORACLE_H
#define SAPPHIRE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_MAX_DIM 16

/* ---- Shape arithmetic (Sources/Sapphire/util/shape.cpp) ------------------ */

typedef struct
{
    int dim;
    int d[ORC_MAX_DIM];
} orc_shape;

/* shape.cpp:138-158  left-pad with 1s up to `dim`; no-op if already >= dim.
 * returns -1 for dim < 0 or dim > ORC_MAX_DIM.
 * pinned: oracle/_ref (reference Shape class), hand table in tests. */
int orc_shape_expand(orc_shape* s, int dim);

/* shape.cpp:205-229  fold leading dims into the first of the kept `dim` dims.
 * pinned: oracle/_ref, hand table. */
int orc_shape_shrink(orc_shape* s, int dim);

/* Shape.hpp:58-63  second-to-last dim, 1 if fewer than two dims. */
int orc_shape_rows(const orc_shape* s);
/* Shape.hpp:65-70  last dim, 0 if empty. */
int orc_shape_cols(const orc_shape* s);
/* shape.cpp:99-110 product of dims in int arithmetic, 0 if empty. */
int orc_shape_size(const orc_shape* s);
/* shape.cpp:231-247 product of the leading (Dim - requiredDim) dims, else 1. */
int orc_shape_num_units(const orc_shape* s, int requiredDim);

/* ---- Dense leaf (Sources/Sapphire/compute/dense/naive/NaiveGemm.cpp) ----- */

/* NaiveGemm.cpp:12-38.  For chunk < totalSize/(M*N):
 *   out[c][m][n] += sum_{k ascending} A[c][m][k]*B[c][k][n]
 * with a local float sum started at 0, product and add rounded separately.
 * Strides M*K, K*N, M*N are computed in unsigned int like the reference.
 * pinned: bit-exact against the reference object in oracle/_ref; identity,
 * ones and K=1 closed forms; float64 brute force bound. */
void orc_naive_gemm(unsigned int totalSize, float* out, const float* A,
                    const float* B, unsigned int M, unsigned int N,
                    unsigned int K);

/* Same arithmetic per output element as orc_naive_gemm (k ascending, separate
 * multiply and add, one final add into out) but walks m,k,n with a row of
 * running sums so that B is read with unit stride, and splits the M rows of
 * every chunk across `threads` workers.  Results are bit-identical to
 * orc_naive_gemm; that identity is asserted by the tests.
 * batch strides are explicit (elements; 0 repeats the operand).
 * pinned: bit-exact against orc_naive_gemm and oracle/_ref. */
void orc_gemm_rows(float* out, const float* A, const float* B, unsigned int M,
                   unsigned int N, unsigned int K, unsigned int batch,
                   size_t strideOut, size_t strideA, size_t strideB,
                   int threads);

/* ---- Batch broadcast (Includes/Sapphire/compute/Broadcast.hpp) ----------- */

typedef struct
{
    uint64_t outOff; /* element offsets from the tensor bases */
    uint64_t aOff;
    uint64_t bOff;
    uint32_t totalSizeOut; /* what the leaf functor receives as totalSize */
} orc_leaf;

/* Broadcast.hpp:83-133 with the functor replaced by "append a leaf".
 * Shapes must already be expanded to the same Dim.  Offsets follow the
 * reference rule  base + (chunkIdx % chunkSizeX) * strideX  in unsigned int.
 * Returns the number of leaves the recursion produces; writes at most `cap`.
 * pinned: oracle/_ref running the reference template with a recording
 * functor; the six-leaf fixture for {2,1,3,2}x{2,3,2,2}. */
size_t orc_broadcast_with_2_inputs(const orc_shape* y, const orc_shape* a,
                                   const orc_shape* b, unsigned int totalSizeOut,
                                   unsigned int totalSizeA,
                                   unsigned int totalSizeB, unsigned int shapeIdx,
                                   unsigned int minimumRequiredDim,
                                   orc_leaf* leaves, size_t cap);

/* ---- Operator (Sources/Sapphire/compute/BasicOps.cpp:183-248) ------------ */

typedef struct
{
    unsigned int M, N, K;
    int maxDim;
    int sizeOut, sizeA, sizeB;
} orc_gemm_dims;

/* BasicOps.cpp:189-230: Expand(2), M = out.Rows, N = out.Cols, K = a.Cols,
 * Expand(maxDim), sizes.  Then the broadcast walk from shapeIdx 0 with
 * minimumRequiredDim 2.  Returns leaf count (writes at most cap).
 * pinned: oracle/_ref; table of shape cases incl. 1-D operands. */
size_t orc_gemm_plan(const int* yShape, int yDim, const int* aShape, int aDim,
                     const int* bShape, int bDim, orc_gemm_dims* dims,
                     orc_leaf* leaves, size_t cap);

/* BasicOps.cpp:183-248 host branch: plan + orc_naive_gemm per leaf.
 * `threads` > 1 runs each leaf through orc_gemm_rows instead (bit-identical).
 * Returns 0, or -1 when the plan does not fit the internal leaf buffer. */
int orc_compute_gemm(float* y, const int* yShape, int yDim, const float* a,
                     const int* aShape, int aDim, const float* b,
                     const int* bShape, int bDim, int threads);

/* ---- Neighbours used by the Linear / backward callers -------------------- */

/* NaiveBasic.cpp:159-165  out = in > 0 ? in : 0. */
void orc_relu(float* out, const float* in, unsigned int totalSize);

/* NaiveBasic.cpp:63-84  batched 2-D transpose; with `broadcast` the source
 * index wraps modulo rows*cols while the source base still advances by one
 * matrix per batch (restated as written). */
void orc_transpose(float* out, const float* in, unsigned int inputRows,
                   unsigned int inputCols, unsigned int batchSize,
                   int broadcast);

/* NaiveBasic.cpp:54-61  out = in * factor.
 * pinned: oracle/_ref bit-exact. */
void orc_scale(float* out, const float* in, float factor,
               unsigned int totalSize);

/* NaiveBasic.cpp:28-39  out[i] = A[i % la] - B[i % lb], la = broadcastA ?
 * inputStride : totalSize (lb likewise).
 * pinned: oracle/_ref bit-exact, with and without the broadcast flags. */
void orc_sub(unsigned int totalSize, float* out, const float* A, const float* B,
             unsigned int inputStride, int broadcastA, int broadcastB);

/* NaiveBasic.cpp:167-174  dx += x > 0 ? dy : 0.
 * pinned: oracle/_ref bit-exact. */
void orc_relu_backward(float* dx, const float* dy, const float* x,
                       unsigned int totalSize);

/* Includes/Sapphire/util/UnitUtils.hpp:38-73: number of trailing dimensions on
 * which all `count` shapes agree (a shape that runs out stops the count).
 * -1 when count == 0 (the reference throws).
 * The header cannot be compiled here (it includes the model classes), so this
 * is pinned by a hand-derived table: equal shapes, differing last dimension,
 * shorter shapes, single shape. */
int orc_get_matching_dim(const orc_shape* shapes, int count);

/* Sources/Sapphire/compute/BasicOps.cpp:63-103 host branch: shapes expanded to
 * the longest, leaf dims = orc_get_matching_dim, walk from shapeIdx 0, each
 * leaf orc_sub(totalSizeOut, ..., 0, false, false).
 * pinned: oracle/_ref running the reference walk with the reference leaf (the
 * matching dimension supplied by orc_get_matching_dim); y = a - b closed form
 * for equal shapes. */
int orc_compute_sub(float* y, const int* yShape, int yDim, const float* a,
                    const int* aShape, int aDim, const float* b,
                    const int* bShape, int bDim);

/* Sources/Sapphire/operations/optimizers/SGD.cpp:22-28: temp = dz * lr
 * (orc_scale), z = z - temp (orc_sub through the operator; equal shapes, one
 * leaf).  pinned: composition of pinned parts. */
void orc_sgd(float* z, const float* dz, float learningRate, unsigned int size);

/* Sources/Sapphire/operations/Backward/LinearBackward.cpp:27-99 with the SGD
 * optimizer, as the sequence of operator calls written there:
 *   Wt = transpose(W); dx += dy*Wt;
 *   xt = transpose(x); dw = 0; dw += xt*dy; sgd(W, dw);
 *   ones[1,batch]; dB = 0; dB += ones*dy; dB *= 1/batch; sgd(bias, dB).
 * x [batch,in], W [in,out], bias [out], dy [batch,out], dx [batch,in].
 * dx, W and bias are updated in place.
 * pinned: composition of pinned parts; closed form with one-hot x and dy. */
void orc_linear_backward(float* dx, float* W, float* bias, const float* dy,
                         const float* x, unsigned int batch, unsigned int in,
                         unsigned int outF, float learningRate, int threads);

/* Sources/Sapphire/operations/Forward/Linear.cpp:113-136: y (zero on entry,
 * [batch,out]) receives ones[batch,1]*bias[1,out] through the K=1 GEMM and
 * then x[batch,in]*W[in,out] through a second GEMM, both via the operator.
 * pinned: composition of pinned parts; closed form with identity weights. */
void orc_linear_forward(float* y, const float* x, const float* W,
                        const float* bias, unsigned int batch, unsigned int in,
                        unsigned int outF, int threads);

/* ---- CSR x dense --------------------------------------------------------- */

/* The reference declares the CSR container only
 * (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:28-38) and no sparse x
 * dense product.  This is the product the dense leaf would give on the
 * densified matrix:  out[m][n] += sum over the row's entries in storage
 * order (columns ascending) of V[p]*B[COL[p]][n], local float sum from 0.
 * ROW has M+1 offsets.
 * pinned: bit-exact against densify + orc_naive_gemm / oracle/_ref (adding
 * the 0*b terms of the dense loop leaves a float running sum unchanged for
 * finite b); brute force on tiny matrices. */
void orc_spmm_csr(float* out, const float* V, const uint32_t* COL,
                  const uint32_t* ROW, uint32_t M, uint32_t N,
                  const float* B, int threads);

/* ---- dense <-> CSR ------------------------------------------------------- */

/* The reference declares the conversions only
 * (Includes/Sapphire/compute/sparse/Sparse.hpp:150-160:
 * CreateSparseMatrixWithDenseMatrix / ConvertSparseMatrixToDenseMatrix with m,
 * n, paddedN) and its tests fill pitched dense matrices the same way
 * (Tests/UnitTests/Sources/TestUtil.cpp:17-60: element (row, col) of matrix i
 * at i*m*paddedN + row*paddedN + col).  Restated contract: an entry is kept
 * when value != 0; row-major, ascending columns; ROW has M + 1 offsets.
 * Returns nnz.  V and COL may be NULL to count only.
 * pinned: scipy.sparse.csr_matrix on the same matrices (values, indices,
 * indptr), count_nonzero, dense -> CSR -> dense round trip, hand example with
 * -0.0 and NaN. */
uint32_t orc_csr_from_dense(float* V, uint32_t* COL, uint32_t* ROW,
                            const float* dense, uint32_t M, uint32_t N,
                            uint32_t ld);

/* dense[r*ld + COL[p]] = V[p], other columns < N zero; padding untouched.
 * pinned: scipy toarray(), round trip. */
void orc_csr_to_dense(float* dense, uint32_t ld, const float* V,
                      const uint32_t* COL, const uint32_t* ROW, uint32_t M,
                      uint32_t N);

/* ---- CSR x CSR ----------------------------------------------------------- */

/* The reference declares the product only
 * (Includes/Sapphire/compute/sparse/cuda/SparseGemm.cuh:16-42; its device
 * helper deletes sums that reach 0, Sources/Sapphire/compute/cudaUtil/SparseUtil.cu:55-60).
 * Restated contract: for each row of A, a dense running row started at +0,
 * A's entries in storage order, acc[col] = acc[col] + a*b for the entries of
 * B's row k (unfused); then the non-zero elements in ascending column order.
 * Returns nnz; VC / COLC may be NULL to count only.  ROWC has M + 1 entries.
 * pinned: bit-exact against densify + orc_naive_gemm + orc_csr_from_dense;
 * scipy.sparse product (values to rounding, structure where nothing
 * cancels); hand example with a cancelling pair. */
uint32_t orc_spgemm_csr(float* VC, uint32_t* COLC, uint32_t* ROWC, const float* VA,
                        const uint32_t* COLA, const uint32_t* ROWA,
                        const float* VB, const uint32_t* COLB,
                        const uint32_t* ROWB, uint32_t M, uint32_t K,
                        uint32_t N);

#ifdef __cplusplus
}
#endif
#endif
