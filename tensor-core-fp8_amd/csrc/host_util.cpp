// Host-side helpers exported through the C ABI: the bit-exact fp8 codec in bulk
// form, the seeded synthetic matrix generators and the row order of the sparse kernels.  They play the role of the
// fp8 converting constructors and MakeDenseMatrix in the reference's harness
// (GEMM/include/bm_test_utils.h:131-143) with explicit seeds and distributions.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <numeric>

#include "fp8.h"
#include "fp8gemm.h"
#include "synth.h"

extern "C" {

uint8_t fp8gemm_encode_one(float x, int fmt) { return fp8::encode(x, fmt ? fp8::E5M2 : fp8::E4M3); }

float fp8gemm_decode_one(uint8_t code, int fmt) { return fp8::decode(code, fmt ? fp8::E5M2 : fp8::E4M3); }

void fp8gemm_encode(const float *src, uint8_t *dst, size_t count, int fmt)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; ++i) dst[i] = fp8::encode(src[i], fmt);
}

void fp8gemm_decode(const uint8_t *src, float *dst, size_t count, int fmt)
{
    float lut[256];
    for (int c = 0; c < 256; ++c) lut[c] = fp8::decode((uint8_t)c, fmt);
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; ++i) dst[i] = lut[src[i]];
}

void fp8gemm_fill_uniform(uint8_t *dst, size_t count, int fmt, uint64_t seed, float lo, float hi)
{
    synth::fill_uniform(dst, count, fmt, seed, lo, hi);
}

void fp8gemm_fill_normal(uint8_t *dst, size_t count, int fmt, uint64_t seed, float mean, float sigma)
{
    synth::fill_normal(dst, count, fmt, seed, mean, sigma);
}

void fp8gemm_fill_weights(uint8_t *dst, size_t count, int fmt, uint64_t seed, float sigma)
{
    synth::fill_weights(dst, count, fmt, seed, sigma);
}

void fp8gemm_fill_loguniform(uint8_t *dst, size_t count, int fmt, uint64_t seed)
{
    synth::fill_loguniform(dst, count, fmt, seed);
}

void fp8gemm_sorted_row_swizzle(int m, const int *row_offsets, int *row_indices)
{
    std::iota(row_indices, row_indices + m, 0);
    std::stable_sort(row_indices, row_indices + m, [row_offsets](int a, int b) {
        return row_offsets[a + 1] - row_offsets[a] > row_offsets[b + 1] - row_offsets[b];
    });
}

}  // extern "C"
