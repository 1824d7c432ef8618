/*
 * CPU oracle for the Sapphire matrix-multiplication path -- TEST
 * INFRASTRUCTURE ONLY (see sapphire_oracle.h).  Plain C restatement of the
 * reference's host arithmetic; build with
 *   gcc -O3 -mavx -mavx2 -ffp-contract=off
 * i.e. the reference's own flags (CMake/CompileOptions.cmake:147,203) plus an
 * explicit ban on fused multiply-add so that the rounding order cannot drift.
 */
#include "sapphire_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ shapes */

int orc_shape_expand(orc_shape* s, int dim)
{
    /* shape.cpp:138-158 */
    if (dim < 0 || dim > ORC_MAX_DIM)
        return -1;
    if (dim <= s->dim)
        return 0;
    const int pad = dim - s->dim;
    for (int i = s->dim - 1; i >= 0; --i)
        s->d[i + pad] = s->d[i];
    for (int i = 0; i < pad; ++i)
        s->d[i] = 1;
    s->dim = dim;
    return 0;
}

int orc_shape_shrink(orc_shape* s, int dim)
{
    /* shape.cpp:205-229: keep the trailing `dim` dims, multiply every dropped
     * leading dim into the first kept one.  dim == 0 on a non-empty shape
     * writes through an empty vector in the reference; not reachable from the
     * path (callers pass 2) and rejected here. */
    if (dim < 0)
        return -1;
    if (dim >= s->dim)
        return 0;
    if (dim == 0)
        return -1;
    const int drop = s->dim - dim;
    int lead = s->d[drop];
    for (int i = drop - 1; i >= 0; --i)
        lead *= s->d[i];
    s->d[0] = lead;
    for (int i = 1; i < dim; ++i)
        s->d[i] = s->d[drop + i];
    s->dim = dim;
    return 0;
}

int orc_shape_rows(const orc_shape* s)
{
    return s->dim > 1 ? s->d[s->dim - 2] : 1;
}

int orc_shape_cols(const orc_shape* s)
{
    return s->dim > 0 ? s->d[s->dim - 1] : 0;
}

int orc_shape_size(const orc_shape* s)
{
    if (s->dim == 0)
        return 0;
    int size = 1;
    for (int i = 0; i < s->dim; ++i)
        size *= s->d[i];
    return size;
}

int orc_shape_num_units(const orc_shape* s, int requiredDim)
{
    if (requiredDim < 0)
        return -1;
    int units = 1;
    for (int i = 0; i < s->dim - requiredDim; ++i)
        units *= s->d[i];
    return units;
}

/* -------------------------------------------------------------- dense leaf */

void orc_naive_gemm(unsigned int totalSize, float* out, const float* A,
                    const float* B, unsigned int M, unsigned int N,
                    unsigned int K)
{
    /* NaiveGemm.cpp:12-38 */
    const unsigned int strideA = M * K;
    const unsigned int strideB = K * N;
    const unsigned int strideOut = M * N;
    const long chunks = (long)(totalSize / strideOut);

    for (long c = 0; c < chunks; ++c)
    {
        const float* a = A + (size_t)strideA * (size_t)c;
        const float* b = B + (size_t)strideB * (size_t)c;
        float* o = out + (size_t)strideOut * (size_t)c;
        for (size_t m = 0; m < M; ++m)
            for (size_t n = 0; n < N; ++n)
            {
                float sum = 0.0f;
                for (size_t k = 0; k < K; ++k)
                    sum += a[(size_t)K * m + k] * b[(size_t)N * k + n];
                o[(size_t)N * m + n] += sum;
            }
    }
}

typedef struct
{
    float* out;
    const float* A;
    const float* B;
    unsigned int N, K;
    size_t rowBegin, rowEnd;
} rows_job;

/* One slice of rows of one matrix: for every row keep N running sums, add the
 * products k ascending (the same sequence of float operations each output
 * element sees in orc_naive_gemm), then add the sums into out. */
static void* rows_worker(void* p)
{
    const rows_job* j = (const rows_job*)p;
    const size_t N = j->N, K = j->K;
    float* sum = (float*)malloc((N ? N : 1) * sizeof(float));
    for (size_t m = j->rowBegin; m < j->rowEnd; ++m)
    {
        for (size_t n = 0; n < N; ++n)
            sum[n] = 0.0f;
        const float* arow = j->A + K * m;
        for (size_t k = 0; k < K; ++k)
        {
            const float av = arow[k];
            const float* brow = j->B + N * k;
            for (size_t n = 0; n < N; ++n)
                sum[n] += av * brow[n];
        }
        float* orow = j->out + N * m;
        for (size_t n = 0; n < N; ++n)
            orow[n] += sum[n];
    }
    free(sum);
    return NULL;
}

static void run_jobs(void* (*fn)(void*), void* jobs, size_t stride, int count)
{
    if (count <= 1)
    {
        if (count == 1)
            fn(jobs);
        return;
    }
    pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)count);
    for (int t = 0; t < count; ++t)
        pthread_create(&tid[t], NULL, fn, (char*)jobs + stride * (size_t)t);
    for (int t = 0; t < count; ++t)
        pthread_join(tid[t], NULL);
    free(tid);
}

void orc_gemm_rows(float* out, const float* A, const float* B, unsigned int M,
                   unsigned int N, unsigned int K, unsigned int batch,
                   size_t strideOut, size_t strideA, size_t strideB,
                   int threads)
{
    if (threads < 1)
        threads = 1;
    if ((unsigned int)threads > M)
        threads = (int)(M ? M : 1);
    rows_job* jobs = (rows_job*)malloc(sizeof(rows_job) * (size_t)threads);
    for (unsigned int c = 0; c < batch; ++c)
    {
        for (int t = 0; t < threads; ++t)
        {
            jobs[t].out = out + strideOut * c;
            jobs[t].A = A + strideA * c;
            jobs[t].B = B + strideB * c;
            jobs[t].N = N;
            jobs[t].K = K;
            jobs[t].rowBegin = (size_t)M * (size_t)t / (size_t)threads;
            jobs[t].rowEnd = (size_t)M * (size_t)(t + 1) / (size_t)threads;
        }
        run_jobs(rows_worker, jobs, sizeof(rows_job), threads);
    }
    free(jobs);
}

/* --------------------------------------------------------------- broadcast */

typedef struct
{
    orc_leaf* leaves;
    size_t cap;
    size_t count;
} leaf_sink;

static void emit_leaf(leaf_sink* s, unsigned int totalSizeOut, uint64_t outOff,
                      uint64_t aOff, uint64_t bOff)
{
    if (s->count < s->cap)
    {
        orc_leaf* l = &s->leaves[s->count];
        l->outOff = outOff;
        l->aOff = aOff;
        l->bOff = bOff;
        l->totalSizeOut = totalSizeOut;
    }
    s->count += 1;
}

static void walk2(const orc_shape* y, const orc_shape* a, const orc_shape* b,
                  unsigned int totalSizeOut, unsigned int totalSizeA,
                  unsigned int totalSizeB, uint64_t outOff, uint64_t aOff,
                  uint64_t bOff, unsigned int shapeIdx, unsigned int minDim,
                  leaf_sink* sink)
{
    /* Broadcast.hpp:83-133.  `limit` is yShape.Dim() - minimumRequiredDim in
     * unsigned arithmetic, as the reference's int/unsigned mix evaluates. */
    const unsigned int limit = (unsigned int)y->dim - minDim;
    if (shapeIdx >= limit)
    {
        emit_leaf(sink, totalSizeOut, outOff, aOff, bOff);
        return;
    }

    unsigned int chunkSize = 1;
    while (shapeIdx < limit && y->d[shapeIdx] == a->d[shapeIdx] &&
           y->d[shapeIdx] == b->d[shapeIdx])
    {
        chunkSize *= (unsigned int)y->d[shapeIdx];
        shapeIdx += 1;
    }

    if (shapeIdx >= limit)
    {
        emit_leaf(sink, totalSizeOut, outOff, aOff, bOff);
        return;
    }

    const unsigned int chunkSizeA = chunkSize * (unsigned int)a->d[shapeIdx];
    const unsigned int chunkSizeB = chunkSize * (unsigned int)b->d[shapeIdx];
    const unsigned int chunkSizeOut = chunkSize * (unsigned int)y->d[shapeIdx];

    const unsigned int strideA = totalSizeA / chunkSizeA;
    const unsigned int strideB = totalSizeB / chunkSizeB;
    const unsigned int strideOut = totalSizeOut / chunkSizeOut;

    unsigned int maxChunk = chunkSizeOut;
    if (chunkSizeA > maxChunk)
        maxChunk = chunkSizeA;
    if (chunkSizeB > maxChunk)
        maxChunk = chunkSizeB;

    for (unsigned int chunkIdx = 0; chunkIdx < maxChunk; ++chunkIdx)
    {
        /* pointer + unsigned: the product is formed in unsigned int first */
        const unsigned int dOut = (chunkIdx % chunkSizeOut) * strideOut;
        const unsigned int dA = (chunkIdx % chunkSizeA) * strideA;
        const unsigned int dB = (chunkIdx % chunkSizeB) * strideB;
        walk2(y, a, b, strideOut, strideA, strideB, outOff + dOut, aOff + dA,
              bOff + dB, shapeIdx + 1, minDim, sink);
    }
}

size_t orc_broadcast_with_2_inputs(const orc_shape* y, const orc_shape* a,
                                   const orc_shape* b, unsigned int totalSizeOut,
                                   unsigned int totalSizeA,
                                   unsigned int totalSizeB, unsigned int shapeIdx,
                                   unsigned int minimumRequiredDim,
                                   orc_leaf* leaves, size_t cap)
{
    leaf_sink sink = { leaves, cap, 0 };
    walk2(y, a, b, totalSizeOut, totalSizeA, totalSizeB, 0, 0, 0, shapeIdx,
          minimumRequiredDim, &sink);
    return sink.count;
}

/* ---------------------------------------------------------------- operator */

static void load_shape(orc_shape* s, const int* v, int dim)
{
    s->dim = dim;
    for (int i = 0; i < dim; ++i)
        s->d[i] = v[i];
}

size_t orc_gemm_plan(const int* yShape, int yDim, const int* aShape, int aDim,
                     const int* bShape, int bDim, orc_gemm_dims* dims,
                     orc_leaf* leaves, size_t cap)
{
    /* BasicOps.cpp:189-230 */
    orc_shape so, sa, sb;
    load_shape(&so, yShape, yDim);
    load_shape(&sa, aShape, aDim);
    load_shape(&sb, bShape, bDim);

    orc_shape_expand(&so, 2);
    orc_shape_expand(&sa, 2);
    orc_shape_expand(&sb, 2);

    dims->M = (unsigned int)orc_shape_rows(&so);
    dims->N = (unsigned int)orc_shape_cols(&so);
    dims->K = (unsigned int)orc_shape_cols(&sa);

    /* BasicOps.cpp:204-218 is unreachable: it needs Dim()==2 for all three
     * tensors and GetNumUnits(2) > 1, which is 1 for any 2-D shape. */

    int maxDim = yDim;
    if (aDim > maxDim)
        maxDim = aDim;
    if (bDim > maxDim)
        maxDim = bDim;
    /* the original (unexpanded) dims decide maxDim; 1-D inputs were already
     * lifted to 2-D above, so the walk never sees fewer than two dims */
    if (maxDim < 2)
        maxDim = 2;
    dims->maxDim = maxDim;

    orc_shape_expand(&so, maxDim);
    orc_shape_expand(&sa, maxDim);
    orc_shape_expand(&sb, maxDim);

    dims->sizeOut = orc_shape_size(&so);
    dims->sizeA = orc_shape_size(&sa);
    dims->sizeB = orc_shape_size(&sb);

    return orc_broadcast_with_2_inputs(
        &so, &sa, &sb, (unsigned int)dims->sizeOut, (unsigned int)dims->sizeA,
        (unsigned int)dims->sizeB, 0, 2, leaves, cap);
}

int orc_compute_gemm(float* y, const int* yShape, int yDim, const float* a,
                     const int* aShape, int aDim, const float* b,
                     const int* bShape, int bDim, int threads)
{
    orc_gemm_dims dims;
    size_t cap = 1024;
    orc_leaf* leaves = (orc_leaf*)malloc(cap * sizeof(orc_leaf));
    size_t n = orc_gemm_plan(yShape, yDim, aShape, aDim, bShape, bDim, &dims,
                             leaves, cap);
    if (n > cap)
    {
        free(leaves);
        cap = n;
        leaves = (orc_leaf*)malloc(cap * sizeof(orc_leaf));
        if (!leaves)
            return -1;
        n = orc_gemm_plan(yShape, yDim, aShape, aDim, bShape, bDim, &dims,
                          leaves, cap);
    }
    for (size_t i = 0; i < n; ++i)
    {
        const orc_leaf* l = &leaves[i];
        if (threads > 1)
        {
            const unsigned int mn = dims.M * dims.N;
            const unsigned int batch = mn ? l->totalSizeOut / mn : 0;
            orc_gemm_rows(y + l->outOff, a + l->aOff, b + l->bOff, dims.M,
                          dims.N, dims.K, batch, (size_t)mn,
                          (size_t)(dims.M * dims.K), (size_t)(dims.K * dims.N),
                          threads);
        }
        else
            orc_naive_gemm(l->totalSizeOut, y + l->outOff, a + l->aOff,
                           b + l->bOff, dims.M, dims.N, dims.K);
    }
    free(leaves);
    return 0;
}

/* -------------------------------------------------------------- neighbours */

void orc_relu(float* out, const float* in, unsigned int totalSize)
{
    /* NaiveBasic.cpp:159-165 */
    for (unsigned int i = 0; i < totalSize; ++i)
        out[i] = in[i] > 0 ? in[i] : 0;
}

void orc_transpose(float* out, const float* in, unsigned int inputRows,
                   unsigned int inputCols, unsigned int batchSize,
                   int broadcast)
{
    /* NaiveBasic.cpp:63-84 */
    const unsigned int leftOver =
        broadcast ? inputRows * inputCols : batchSize * inputRows * inputCols;
    for (unsigned int bi = 0; bi < batchSize; ++bi)
    {
        float* o = out + (size_t)bi * inputCols * inputRows;
        const float* s = in + (size_t)bi * inputRows * inputCols;
        for (unsigned int i = 0; i < inputRows; ++i)
            for (unsigned int j = 0; j < inputCols; ++j)
                o[j * inputRows + i] = s[(i * inputCols + j) % leftOver];
    }
}

void orc_scale(float* out, const float* in, float factor,
               unsigned int totalSize)
{
    /* NaiveBasic.cpp:54-61 */
    for (unsigned int i = 0; i < totalSize; i++)
        out[i] = in[i] * factor;
}

void orc_sub(unsigned int totalSize, float* out, const float* A, const float* B,
             unsigned int inputStride, int broadcastA, int broadcastB)
{
    /* NaiveBasic.cpp:28-39 */
    const unsigned int leftOverA = broadcastA ? inputStride : totalSize;
    const unsigned int leftOverB = broadcastB ? inputStride : totalSize;
    for (unsigned int i = 0; i < totalSize; i++)
        out[i] = A[i % leftOverA] - B[i % leftOverB];
}

void orc_relu_backward(float* dx, const float* dy, const float* x,
                       unsigned int totalSize)
{
    /* NaiveBasic.cpp:167-174 */
    for (unsigned int i = 0; i < totalSize; ++i)
        dx[i] += x[i] > 0.0f ? dy[i] : 0.0f;
}

int orc_get_matching_dim(const orc_shape* shapes, int count)
{
    /* UnitUtils.hpp:38-73: curDimFromLast runs -1, -2, ... while every shape
     * still has that position and holds shapes[0]'s extent there. */
    if (count <= 0)
        return -1;
    int curDimFromLast = -1;
    for (;;)
    {
        if (shapes[0].dim + curDimFromLast < 0)
            break;
        const int want = shapes[0].d[shapes[0].dim + curDimFromLast];
        int match = 1;
        for (int s = 0; s < count; ++s)
        {
            if (shapes[s].dim + curDimFromLast < 0 ||
                shapes[s].d[shapes[s].dim + curDimFromLast] != want)
            {
                match = 0;
                break;
            }
        }
        if (!match)
            break;
        curDimFromLast -= 1;
    }
    return -(curDimFromLast + 1);
}

static void fill_shape(orc_shape* s, const int* v, int dim)
{
    s->dim = dim;
    for (int i = 0; i < dim; ++i)
        s->d[i] = v[i];
}

int orc_compute_sub(float* y, const int* yShape, int yDim, const float* a,
                    const int* aShape, int aDim, const float* b,
                    const int* bShape, int bDim)
{
    /* BasicOps.cpp:63-103 */
    orc_shape sh[3];
    fill_shape(&sh[0], yShape, yDim);
    fill_shape(&sh[1], aShape, aDim);
    fill_shape(&sh[2], bShape, bDim);
    int maxDim = yDim;
    if (aDim > maxDim) maxDim = aDim;
    if (bDim > maxDim) maxDim = bDim;
    for (int i = 0; i < 3; ++i)
        if (orc_shape_expand(&sh[i], maxDim) != 0)
            return -1;
    const int minRequiredDim = orc_get_matching_dim(sh, 3);
    size_t cap = 1024;
    orc_leaf* leaves = (orc_leaf*)malloc(cap * sizeof(orc_leaf));
    size_t n = orc_broadcast_with_2_inputs(
        &sh[0], &sh[1], &sh[2], (unsigned int)orc_shape_size(&sh[0]),
        (unsigned int)orc_shape_size(&sh[1]), (unsigned int)orc_shape_size(&sh[2]),
        0, (unsigned int)minRequiredDim, leaves, cap);
    if (n > cap)
    {
        free(leaves);
        cap = n;
        leaves = (orc_leaf*)malloc(cap * sizeof(orc_leaf));
        if (!leaves)
            return -1;
        n = orc_broadcast_with_2_inputs(
            &sh[0], &sh[1], &sh[2], (unsigned int)orc_shape_size(&sh[0]),
            (unsigned int)orc_shape_size(&sh[1]),
            (unsigned int)orc_shape_size(&sh[2]), 0,
            (unsigned int)minRequiredDim, leaves, cap);
    }
    for (size_t i = 0; i < n; ++i)
        orc_sub(leaves[i].totalSizeOut, y + leaves[i].outOff,
                a + leaves[i].aOff, b + leaves[i].bOff, 0, 0, 0);
    free(leaves);
    return 0;
}

void orc_sgd(float* z, const float* dz, float learningRate, unsigned int size)
{
    /* SGD.cpp:22-28 */
    float* temp = (float*)malloc((size ? size : 1) * sizeof(float));
    const int shape[1] = { (int)size };
    orc_scale(temp, dz, learningRate, size);
    orc_compute_sub(z, shape, 1, z, shape, 1, temp, shape, 1);
    free(temp);
}

void orc_linear_backward(float* dx, float* W, float* bias, const float* dy,
                         const float* x, unsigned int batch, unsigned int in,
                         unsigned int outF, float learningRate, int threads)
{
    const int dxs[2] = { (int)batch, (int)in };
    const int dys[2] = { (int)batch, (int)outF };
    const int ws[2] = { (int)in, (int)outF };
    const int wts[2] = { (int)outF, (int)in };
    const int xts[2] = { (int)in, (int)batch };
    const int os[2] = { 1, (int)batch };
    const int bs[1] = { (int)outF };

    /* LinearBackward.cpp:37-51 */
    float* wt = (float*)calloc((size_t)in * outF + 1, sizeof(float));
    orc_transpose(wt, W, in, outF, 1, 1);
    orc_compute_gemm(dx, dxs, 2, dy, dys, 2, wt, wts, 2, threads);
    free(wt);

    /* LinearBackward.cpp:53-77 */
    float* xt = (float*)calloc((size_t)batch * in + 1, sizeof(float));
    float* dw = (float*)calloc((size_t)in * outF + 1, sizeof(float));
    orc_transpose(xt, x, batch, in, 1, 1);
    orc_compute_gemm(dw, ws, 2, xt, xts, 2, dy, dys, 2, threads);
    orc_sgd(W, dw, learningRate, in * outF);
    free(xt);
    free(dw);

    /* LinearBackward.cpp:79-99 */
    float* ones = (float*)malloc((batch ? batch : 1) * sizeof(float));
    float* dB = (float*)calloc(outF + 1, sizeof(float));
    for (unsigned int i = 0; i < batch; ++i)
        ones[i] = 1.0f;
    orc_compute_gemm(dB, bs, 1, ones, os, 2, dy, dys, 2, 1);
    orc_scale(dB, dB, 1.0f / (float)batch, outF);
    orc_sgd(bias, dB, learningRate, outF);
    free(ones);
    free(dB);
}

void orc_linear_forward(float* y, const float* x, const float* W,
                        const float* bias, unsigned int batch, unsigned int in,
                        unsigned int outF, int threads)
{
    /* Linear.cpp:113-118 ones[batch,1]; :121 everything viewed 2-D;
     * :134-136 Gemm(y, ones, bias) then Gemm(y, x, W). */
    float* ones = (float*)malloc((batch ? batch : 1) * sizeof(float));
    for (unsigned int i = 0; i < batch; ++i)
        ones[i] = 1.0f;
    const int ys[2] = { (int)batch, (int)outF };
    const int os[2] = { (int)batch, 1 };
    const int bs[2] = { 1, (int)outF }; /* bias [out] viewed as [1,out] */
    const int xs[2] = { (int)batch, (int)in };
    const int ws[2] = { (int)in, (int)outF };
    orc_compute_gemm(y, ys, 2, ones, os, 2, bias, bs, 2, 1);
    orc_compute_gemm(y, ys, 2, x, xs, 2, W, ws, 2, threads);
    free(ones);
}

/* --------------------------------------------------------------- CSR x dense */

typedef struct
{
    float* out;
    const float* V;
    const uint32_t* COL;
    const uint32_t* ROW;
    const float* B;
    uint32_t N;
    uint32_t rowBegin, rowEnd;
} spmm_job;

static void* spmm_worker(void* p)
{
    const spmm_job* j = (const spmm_job*)p;
    const size_t N = j->N;
    float* sum = (float*)malloc((N ? N : 1) * sizeof(float));
    for (uint32_t m = j->rowBegin; m < j->rowEnd; ++m)
    {
        for (size_t n = 0; n < N; ++n)
            sum[n] = 0.0f;
        for (uint32_t p2 = j->ROW[m]; p2 < j->ROW[m + 1]; ++p2)
        {
            const float v = j->V[p2];
            const float* brow = j->B + (size_t)j->COL[p2] * N;
            for (size_t n = 0; n < N; ++n)
                sum[n] += v * brow[n];
        }
        float* orow = j->out + (size_t)m * N;
        for (size_t n = 0; n < N; ++n)
            orow[n] += sum[n];
    }
    free(sum);
    return NULL;
}

void orc_spmm_csr(float* out, const float* V, const uint32_t* COL,
                  const uint32_t* ROW, uint32_t M, uint32_t N,
                  const float* B, int threads)
{
    if (threads < 1)
        threads = 1;
    if ((uint32_t)threads > M)
        threads = (int)(M ? M : 1);
    spmm_job* jobs = (spmm_job*)malloc(sizeof(spmm_job) * (size_t)threads);
    for (int t = 0; t < threads; ++t)
    {
        jobs[t].out = out;
        jobs[t].V = V;
        jobs[t].COL = COL;
        jobs[t].ROW = ROW;
        jobs[t].B = B;
        jobs[t].N = N;
        jobs[t].rowBegin = (uint32_t)((uint64_t)M * (uint64_t)t / (uint64_t)threads);
        jobs[t].rowEnd = (uint32_t)((uint64_t)M * (uint64_t)(t + 1) / (uint64_t)threads);
    }
    run_jobs(spmm_worker, jobs, sizeof(spmm_job), threads);
    free(jobs);
}

/* -------------------------------------------------------------- dense <-> CSR */

uint32_t orc_csr_from_dense(float* V, uint32_t* COL, uint32_t* ROW,
                            const float* dense, uint32_t M, uint32_t N,
                            uint32_t ld)
{
    uint32_t nnz = 0;
    for (uint32_t r = 0; r < M; ++r)
    {
        ROW[r] = nnz;
        for (uint32_t c = 0; c < N; ++c)
        {
            const float v = dense[(size_t)r * ld + c];
            if (v != 0.0f)
            {
                if (V)
                    V[nnz] = v;
                if (COL)
                    COL[nnz] = c;
                ++nnz;
            }
        }
    }
    ROW[M] = nnz;
    return nnz;
}

void orc_csr_to_dense(float* dense, uint32_t ld, const float* V,
                      const uint32_t* COL, const uint32_t* ROW, uint32_t M,
                      uint32_t N)
{
    for (uint32_t r = 0; r < M; ++r)
    {
        float* row = dense + (size_t)r * ld;
        for (uint32_t c = 0; c < N; ++c)
            row[c] = 0.0f;
        for (uint32_t p = ROW[r]; p < ROW[r + 1]; ++p)
            if (COL[p] < N)
                row[COL[p]] = V[p];
    }
}

/* ------------------------------------------------------------------ CSR x CSR */

uint32_t orc_spgemm_csr(float* VC, uint32_t* COLC, uint32_t* ROWC, const float* VA,
                        const uint32_t* COLA, const uint32_t* ROWA,
                        const float* VB, const uint32_t* COLB,
                        const uint32_t* ROWB, uint32_t M, uint32_t K,
                        uint32_t N)
{
    float* acc = (float*)malloc(((size_t)N + 1) * sizeof(float));
    uint32_t nnz = 0;
    for (uint32_t i = 0; i < M; ++i)
    {
        ROWC[i] = nnz;
        for (uint32_t j = 0; j < N; ++j)
            acc[j] = 0.0f;
        for (uint32_t pa = ROWA[i]; pa < ROWA[i + 1]; ++pa)
        {
            const uint32_t k = COLA[pa];
            const float a = VA[pa];
            if (k >= K)
                continue;
            for (uint32_t pb = ROWB[k]; pb < ROWB[k + 1]; ++pb)
            {
                const float prod = a * VB[pb];
                acc[COLB[pb]] = acc[COLB[pb]] + prod;
            }
        }
        for (uint32_t j = 0; j < N; ++j)
            if (acc[j] != 0.0f)
            {
                if (VC)
                    VC[nnz] = acc[j];
                if (COLC)
                    COLC[nnz] = j;
                ++nnz;
            }
    }
    ROWC[M] = nnz;
    free(acc);
    return nnz;
}
