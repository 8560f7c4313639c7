// Host-side code under AddressSanitizer and UndefinedBehaviorSanitizer: the product codec and
// seeded generators (csrc/host_util.cpp, GEMM/include/fp8.h, synth.h) and the CPU oracle
// (oracle/fp8_oracle.c), driven over edge inputs: every code, special floats, empty and odd
// sizes, ragged GEMM shapes.  Exit status 0 = no sanitizer report and every check held.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <vector>

#include "fp8gemm.h"

extern "C" {
float oracle_fp8_decode(uint8_t code, int fmt);
uint8_t oracle_fp8_encode(float x, int fmt);
void oracle_gemm_verbatim(int M, int K, int N, const uint8_t *A, int afmt, const uint8_t *B, int bfmt, float *C);
void oracle_gemm_fast(int M, int K, int N, const uint8_t *A, int afmt, const uint8_t *B, int bfmt, const int *rows, int R,
                      float *C, double *S);
}

static int failures = 0;
#define EXPECT(c) do { if (!(c)) { std::printf("line %d: %s\n", __LINE__, #c); ++failures; } } while (0)

int main()
{
    // every code, both formats: product decode == oracle decode (NaN by class), round trip of finite codes
    for (int fmt = 0; fmt < 2; ++fmt)
        for (int c = 0; c < 256; ++c) {
            const float p = fp8gemm_decode_one((uint8_t)c, fmt), o = oracle_fp8_decode((uint8_t)c, fmt);
            EXPECT((std::isnan(p) && std::isnan(o)) || std::memcmp(&p, &o, 4) == 0);
            if (std::isfinite(p)) EXPECT(fp8gemm_encode_one(p, fmt) == (uint8_t)c);
        }
    // special floats and a sweep of bit patterns: product encode == oracle encode
    const float inf = std::numeric_limits<float>::infinity();
    const float specials[] = {0.0f, -0.0f, inf, -inf, std::numeric_limits<float>::quiet_NaN(), std::numeric_limits<float>::denorm_min(),
                              -std::numeric_limits<float>::denorm_min(), std::numeric_limits<float>::max(), std::numeric_limits<float>::lowest(),
                              448.0f, 464.0f, 465.0f, 57344.0f, 61440.0f, 0.0009765625f, 7.62939453125e-06f};
    for (int fmt = 0; fmt < 2; ++fmt) {
        for (float v : specials) EXPECT(fp8gemm_encode_one(v, fmt) == oracle_fp8_encode(v, fmt));
        for (uint64_t bits = 0; bits < (1ull << 32); bits += 65521) {      // a prime stride over all 2^32 patterns
            const uint32_t b32 = (uint32_t)bits;
            float v;
            std::memcpy(&v, &b32, 4);
            EXPECT(fp8gemm_encode_one(v, fmt) == oracle_fp8_encode(v, fmt));
        }
    }
    // bulk entry points on empty and odd sizes (buffers sized exactly: an overrun is a report)
    for (size_t count : {(size_t)0, (size_t)1, (size_t)7, (size_t)1023, (size_t)4099}) {
        std::vector<float> src(count), back(count);
        std::vector<uint8_t> codes(count);
        for (size_t i = 0; i < count; ++i) src[i] = (float)((int)(i % 97) - 48) * 0.37f;
        for (int fmt = 0; fmt < 2; ++fmt) {
            fp8gemm_encode(src.data(), codes.data(), count, fmt);
            fp8gemm_decode(codes.data(), back.data(), count, fmt);
            for (size_t i = 0; i < count; ++i) EXPECT(codes[i] == oracle_fp8_encode(src[i], fmt));
            fp8gemm_fill_uniform(codes.data(), count, fmt, 1, -1.0f, 1.0f);
            fp8gemm_fill_normal(codes.data(), count, fmt, 2, 0.0f, 4.0f);
            fp8gemm_fill_weights(codes.data(), count, fmt, 3, 0.02f);
            fp8gemm_fill_loguniform(codes.data(), count, fmt, 4);
            for (size_t i = 0; i < count; ++i) EXPECT(std::isfinite(fp8gemm_decode_one(codes[i], fmt)));
        }
    }
    // oracle GEMM on ragged shapes: fast == verbatim bit for bit, row subsets, S >= |C|
    const int shapes[][3] = {{1, 1, 1}, {3, 17, 5}, {33, 130, 19}, {64, 256, 48}, {7, 1000, 9}};
    for (auto &sh : shapes) {
        const int M = sh[0], K = sh[1], N = sh[2];
        std::vector<uint8_t> A((size_t)M * K), B((size_t)N * K);
        fp8gemm_fill_normal(A.data(), A.size(), 0, 11, 0.0f, 2.0f);
        fp8gemm_fill_loguniform(B.data(), B.size(), 1, 12);
        for (auto &b : B) if (((b >> 2) & 0x1F) > 24) b = (uint8_t)((b & 0x83) | 0x3C);     // keep sums finite
        std::vector<float> C1((size_t)M * N), C2((size_t)M * N);
        std::vector<double> S((size_t)M * N);
        oracle_gemm_verbatim(M, K, N, A.data(), 0, B.data(), 1, C1.data());
        oracle_gemm_fast(M, K, N, A.data(), 0, B.data(), 1, nullptr, M, C2.data(), S.data());
        EXPECT(std::memcmp(C1.data(), C2.data(), C1.size() * 4) == 0);
        for (size_t i = 0; i < C1.size(); ++i) EXPECT(S[i] * (1.0 + 1e-6) + 1e-30 >= std::fabs((double)C1[i]));
        const int rows[2] = {M - 1, 0};
        std::vector<float> Cr((size_t)2 * N);
        oracle_gemm_fast(M, K, N, A.data(), 0, B.data(), 1, rows, 2, Cr.data(), nullptr);
        EXPECT(std::memcmp(Cr.data(), C1.data() + (size_t)(M - 1) * N, (size_t)N * 4) == 0);
        EXPECT(std::memcmp(Cr.data() + N, C1.data(), (size_t)N * 4) == 0);
    }
    if (!failures) std::printf("sanitize check: all checks passed\n");
    return failures ? 1 : 0;
}
