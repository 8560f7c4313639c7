// Benchmark helpers of the harness: error checking and operand generation.
// Counterpart of the helpers of GEMM/include/bm_test_utils.h: the two that the
// reference's FP8 GEMM path uses (checkCuda :12-19, MakeDenseMatrix :131-143) and the
// generators of its sparse operand formats (blocked-ELL :48-68, compressed sparse rows
// :71-128, row orders :197-216), which feed fp8gemm_spmm_* / fp8gemm_spmv_*.
#ifndef BM_TEST_UTILS_H
#define BM_TEST_UTILS_H

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <numeric>
#include <random>
#include <vector>

#include "fp8.h"
#include "synth.h"

// Prints the error and stops: a failed allocation or copy leaves nothing to
// benchmark.  (The reference asserts, which vanishes under NDEBUG.)
inline void checkHip(hipError_t result)
{
    if (result != hipSuccess) {
        std::fprintf(stderr, "HIP Runtime Error: %s\n", hipGetErrorString(result));
        std::exit(EXIT_FAILURE);
    }
}

// The reference's generator: uniform(-1, 1) floats converted to the fp8 type.
// The engine is taken by value, so two calls with the same engine object see
// the same random stream (A and B start with identical values), as there.
template <typename ValueType>
void MakeDenseMatrix(int rows, int columns, ValueType *matrix, std::default_random_engine generator)
{
    std::uniform_real_distribution<float> distribution(-1.0f, 1.0f);
    const int64_t count = static_cast<int64_t>(rows) * columns;
    for (int64_t i = 0; i < count; ++i) matrix[i] = ValueType(distribution(generator));
}

// Seeded, platform-independent generators for the benchmark configurations.
//   "uniform"    U(-1, 1)                     "normal"  N(0, 1)
//   "normal4"    4 * N(0, 1)                  "weights" N(0, 0.02) scaled to the format's max
//   "loguniform" +-2^u over the whole finite exponent range
// Returns false for an unknown name.
template <typename ValueType>
bool MakeDenseMatrixSeeded(int rows, int columns, ValueType *matrix, const char *dist, uint64_t seed)
{
    uint8_t *dst = reinterpret_cast<uint8_t *>(matrix);
    const size_t count = static_cast<size_t>(rows) * columns;
    const int fmt = ValueType::format;
    if (!std::strcmp(dist, "uniform")) synth::fill_uniform(dst, count, fmt, seed, -1.0f, 1.0f);
    else if (!std::strcmp(dist, "normal")) synth::fill_normal(dst, count, fmt, seed, 0.0f, 1.0f);
    else if (!std::strcmp(dist, "normal4")) synth::fill_normal(dst, count, fmt, seed, 0.0f, 4.0f);
    else if (!std::strcmp(dist, "weights")) synth::fill_weights(dst, count, fmt, seed, 0.02f);
    else if (!std::strcmp(dist, "loguniform")) synth::fill_loguniform(dst, count, fmt, seed);
    else return false;
    return true;
}

// ---- sparse operands ------------------------------------------------------------------
// Block column numbers of a blocked-ELL matrix: every one of num_block_row block rows stores
// num_block_nnz_col blocks at distinct block columns drawn uniformly from num_block_col, in
// rising order; ellColInd is num_block_row x num_block_nnz_col.  The engine is taken by value,
// as everywhere in this header.
inline void GenerateUniformBlockedELLIndex(int num_block_col, int num_block_nnz_col, int num_block_row, int *ellColInd,
                                           std::default_random_engine generator)
{
    std::vector<int> pick(num_block_col);
    for (int r = 0; r < num_block_row; ++r) {
        std::iota(pick.begin(), pick.end(), 0);
        // the first num_block_nnz_col places of a shuffle are a uniform draw without replacement
        for (int j = 0; j < num_block_nnz_col; ++j) {
            std::uniform_int_distribution<int> rest(j, num_block_col - 1);
            std::swap(pick[j], pick[rest(generator)]);
        }
        std::sort(pick.begin(), pick.begin() + num_block_nnz_col);
        std::copy(pick.begin(), pick.begin() + num_block_nnz_col, ellColInd + static_cast<int64_t>(r) * num_block_nnz_col);
    }
}

// rows x columns matrix with exactly `nonzeros` stored entries at uniformly drawn places, values
// uniform(-1, 1) converted to ValueType, in compressed sparse rows (row_offsets of rows + 1
// entries, rising columns inside a row).  row_padding > 0 pads every row to a multiple of it
// with zero-valued entries that repeat the row's last column, so that they index no place
// outside the dense operand.  Returns the number of stored entries, padding included; the
// arrays must hold nonzeros + rows * (row_padding - 1) entries in the worst case.
template <typename ValueType, typename IndexType>
int64_t MakeSparseMatrixRandomUniform(int rows, int columns, int nonzeros, ValueType *values, IndexType *row_offsets,
                                      IndexType *column_indices, std::default_random_engine generator, int row_padding)
{
    const int64_t places = static_cast<int64_t>(rows) * columns;
    if (nonzeros <= 0 || nonzeros > places || row_padding < 0) return -1;
    std::uniform_real_distribution<float> distribution(-1.0f, 1.0f);
    // choose the places: a shuffled numbering, the places numbered below `nonzeros` are kept
    std::vector<int64_t> number(places);
    std::iota(number.begin(), number.end(), 0);
    std::shuffle(number.begin(), number.end(), generator);
    int64_t at = 0;
    row_offsets[0] = 0;
    for (int64_t i = 0; i < rows; ++i) {
        const int64_t first = at;
        for (int64_t j = 0; j < columns; ++j)
            if (number[i * columns + j] < nonzeros) {
                values[at] = ValueType(distribution(generator));
                column_indices[at] = static_cast<IndexType>(j);
                ++at;
            }
        if (row_padding > 0 && at > first)
            while ((at - first) % row_padding != 0) {
                values[at] = ValueType(0.0f);
                column_indices[at] = column_indices[at - 1];
                ++at;
            }
        row_offsets[i + 1] = static_cast<IndexType>(at);
    }
    return at;
}

inline void IdentityRowSwizzle(int rows, int *row_indices) { std::iota(row_indices, row_indices + rows, 0); }

// rows by falling number of stored entries: the long rows start first
inline void SortedRowSwizzle(int rows, const int *row_offsets, int *row_indices)
{
    std::iota(row_indices, row_indices + rows, 0);
    std::stable_sort(row_indices, row_indices + rows, [row_offsets](int a, int b) {
        return row_offsets[a + 1] - row_offsets[a] > row_offsets[b + 1] - row_offsets[b];
    });
}

// Host loop of the sampled dense-dense product (the reference's Host_sddmm,
// GEMM/include/bm_test_utils.h:172-194): the output pattern has m_vec rows of column vectors of
// VecLength; stored vector j of row i receives, for v < VecLength, the running fp32 sum along K of
// lhs_matrix[i * VecLength + v][:] * rhs_matrix[col_indices[j]][:], both operands row-major with k
// columns.  output_values: row_offsets[m_vec] x VecLength.
template <typename ValueType, typename OutType>
void Host_sddmm(int m_vec, int k, int VecLength, const int *row_offsets, const int *col_indices, const ValueType *lhs_matrix,
                const ValueType *rhs_matrix, OutType *output_values)
{
    for (int i = 0; i < m_vec; ++i)
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            const ValueType *right = rhs_matrix + static_cast<size_t>(col_indices[j]) * k;
            for (int v = 0; v < VecLength; ++v) {
                const ValueType *left = lhs_matrix + (static_cast<size_t>(i) * VecLength + v) * k;
                float sum = 0.0f;
                for (int l = 0; l < k; ++l) sum += static_cast<float>(left[l]) * static_cast<float>(right[l]);
                output_values[static_cast<size_t>(j) * VecLength + v] = static_cast<OutType>(sum);
            }
        }
}

#endif  // BM_TEST_UTILS_H
