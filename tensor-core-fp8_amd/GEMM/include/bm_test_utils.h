// Benchmark helpers of the harness: error checking and operand generation.
// Counterpart of the two helpers of GEMM/include/bm_test_utils.h that the
// reference's FP8 GEMM path uses (checkCuda :12-19, MakeDenseMatrix :131-143).
#ifndef BM_TEST_UTILS_H
#define BM_TEST_UTILS_H

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>

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

#endif  // BM_TEST_UTILS_H
