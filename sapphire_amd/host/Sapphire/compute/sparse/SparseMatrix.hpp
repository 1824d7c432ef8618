// CSR container shared with the reference
// (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:20-38): a 48-byte, 16-byte aligned
// record whose arrays live on the host or on the device depending on where the record is
// used.  ROW holds M + 1 offsets (the reference never states the length; this is the
// standard CSR convention and the one every kernel here assumes).
#ifndef SAPPHIRE_AMD_COMPUTE_SPARSE_SPARSEMATRIX_HPP
#define SAPPHIRE_AMD_COMPUTE_SPARSE_SPARSEMATRIX_HPP

#include <cstdint>

#define MAX_NNZ_PER_ROW (1 << 10)
#define MAX_NNZ_PER_ROW_HOST (1 << 10)

struct alignas(16) SparseMatrix
{
    float* V;        //!< NNZ values, row by row
    uint32_t* COL;   //!< column of each value, ascending inside a row
    uint32_t* ROW;   //!< M + 1 offsets into V / COL
    uint32_t NNZ;
    uint32_t M;      //!< rows
    uint32_t N;      //!< columns
    uint32_t Padding[3];
};

static_assert(sizeof(SparseMatrix) == 48, "SparseMatrix must stay 48 bytes");

// The companion record of the reference's sparse x sparse product
// (Includes/Sapphire/compute/sparse/SparseMatrix.hpp:40-50): the shape of a SparseMatrix with,
// in place of each value, the number of multiplications that entry causes in a product.
struct alignas(16) LoadDistMatrix
{
    uint32_t* Load;  //!< per entry: entries in the row of the right operand it selects
    uint32_t* COL;
    uint32_t* ROW;   //!< M + 1 offsets
    uint32_t NNZ;
    uint32_t M;
    uint32_t N;
    uint32_t Padding[3];
};

static_assert(sizeof(LoadDistMatrix) == 48, "LoadDistMatrix must stay 48 bytes");

#endif
