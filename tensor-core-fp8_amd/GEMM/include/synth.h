// Seeded synthetic fp8 matrices for the harness and the benchmarks.
//
// The reference fills its operands with MakeDenseMatrix
// (GEMM/include/bm_test_utils.h:131-143): uniform(-1,1) floats from a
// default-seeded std::default_random_engine passed by value, so A and B get the
// same stream.  Here every generator is counter-based -- element i is a pure
// function of (seed, i) through SplitMix64 -- which makes the data independent
// of thread count and platform, and lets A and B use different seeds.
#ifndef FP8GEMM_SYNTH_H
#define FP8GEMM_SYNTH_H

#include <cmath>
#include <cstddef>
#include <cstdint>

#include "fp8.h"

namespace synth {

inline uint64_t splitmix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// two independent 64-bit words for element i of stream `seed`
inline uint64_t word(uint64_t seed, uint64_t i, uint64_t lane)
{
    return splitmix64(splitmix64(seed) ^ splitmix64(2 * i + lane));
}

// uniform in (0, 1): 53 random bits, never exactly 0
inline double unit(uint64_t w) { return ((double)(w >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

inline double std_normal(uint64_t seed, uint64_t i)
{
    const double u1 = unit(word(seed, i, 0));
    const double u2 = unit(word(seed, i, 1));
    return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
}

inline void fill_uniform(uint8_t *dst, size_t count, int fmt, uint64_t seed, float lo, float hi)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; ++i) {
        const double u = unit(word(seed, (uint64_t)i, 0));
        dst[i] = fp8::encode((float)(lo + (hi - lo) * u), fmt);
    }
}

inline void fill_normal(uint8_t *dst, size_t count, int fmt, uint64_t seed, float mean, float sigma)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; ++i)
        dst[i] = fp8::encode((float)(mean + sigma * std_normal(seed, (uint64_t)i)), fmt);
}

// N(0, sigma) scaled per tensor so that max|w| lands on the largest finite code
inline void fill_weights(uint8_t *dst, size_t count, int fmt, uint64_t seed, float sigma)
{
    double amax = 0.0;
#pragma omp parallel for schedule(static) reduction(max : amax)
    for (long long i = 0; i < (long long)count; ++i) {
        const double v = std::fabs(sigma * std_normal(seed, (uint64_t)i));
        if (v > amax) amax = v;
    }
    const double top = (fmt == fp8::E4M3) ? 448.0 : 57344.0;
    const double scale = amax > 0.0 ? top / amax : 1.0;
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; ++i)
        dst[i] = fp8::encode((float)(scale * sigma * std_normal(seed, (uint64_t)i)), fmt);
}

// +-2^u with u uniform over the format's finite exponent range, subnormals
// included; saturating encode keeps every code finite
inline void fill_loguniform(uint8_t *dst, size_t count, int fmt, uint64_t seed)
{
    const double lo = (fmt == fp8::E4M3) ? -9.0 : -16.0;
    const double hi = (fmt == fp8::E4M3) ? std::log2(448.0) : std::log2(57344.0);
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; ++i) {
        const double u = lo + (hi - lo) * unit(word(seed, (uint64_t)i, 0));
        const double sgn = (word(seed, (uint64_t)i, 1) >> 63) ? -1.0 : 1.0;
        uint8_t c = fp8::encode((float)(sgn * std::exp2(u)), fmt);
        dst[i] = c;
    }
}

}  // namespace synth

#endif  // FP8GEMM_SYNTH_H
