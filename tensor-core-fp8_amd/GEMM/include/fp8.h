// OCP FP8 storage types for the host side of the GEMM library.
//
// Takes the place of the two typedefs at GEMM/include/gemm.cuh:6-7 of the
// reference (e4m3 / e5m2 = NVIDIA's __nv_fp8_e4m3 / __nv_fp8_e5m2): one byte of
// storage, an explicit converting constructor from float (round to nearest
// even, saturate to the largest finite value) and an explicit conversion back
// to float.  gfx950 consumes the OCP encodings natively, so the bytes are fed
// to the MFMA units unchanged.
#ifndef FP8GEMM_FP8_H
#define FP8GEMM_FP8_H

#include <cstdint>
#include <cstring>

namespace fp8 {

enum Format : int { E4M3 = 0, E5M2 = 1 };

// Round-to-nearest-even, saturate-to-finite conversion working on the float's
// bit pattern.  MBITS = stored mantissa bits, BIAS = exponent bias, MAXNORM =
// code of the largest finite magnitude.
template <int MBITS, int BIAS, uint8_t MAXNORM>
inline uint8_t encode_bits(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint8_t sign = static_cast<uint8_t>((u >> 31) << 7);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x7F;                       // NaN (sign dropped)
    // float bit pattern of the largest finite fp8 magnitude
    constexpr int EMAX = (MBITS == 3) ? 8 : 15;
    constexpr uint32_t MAXBITS =
        (static_cast<uint32_t>(EMAX + 127) << 23) |
        (static_cast<uint32_t>(MAXNORM & ((1u << MBITS) - 1u)) << (23 - MBITS));
    if (a >= MAXBITS) return static_cast<uint8_t>(sign | MAXNORM);   // saturate (Inf too)
    constexpr int EMIN = 1 - BIAS;                          // exponent of the least normal
    const int e = static_cast<int>(a >> 23) - 127;
    if (e < EMIN - MBITS - 1) return sign;                  // below half the least subnormal
    const uint32_t mant = (a & 0x007FFFFFu) | 0x00800000u;  // 1.m as a 24-bit integer
    const int ebin = e < EMIN ? EMIN : e;                   // binade the result lives in
    const int shift = (23 - MBITS) + (ebin - e);            // bits dropped, <= 25 here
    uint32_t n = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (n & 1u))) ++n;       // ties to even
    // normals carry their implicit bit in n, so adding n to the binade's base
    // code minus one binade lands on the right code, carries included
    uint32_t code = (static_cast<uint32_t>(ebin - EMIN) << MBITS) + n;
    if (code > MAXNORM) code = MAXNORM;
    return static_cast<uint8_t>(sign | code);
}

inline float decode_e4m3_bits(uint8_t c)
{
    const uint32_t sign = static_cast<uint32_t>(c & 0x80u) << 24;
    const uint32_t E = (c >> 3) & 0xFu;
    const uint32_t Mn = c & 0x7u;
    uint32_t u;
    if ((c & 0x7Fu) == 0x7Fu) {
        u = 0x7FC00000u;                                    // NaN
    } else if (E == 0) {
        const float v = static_cast<float>(Mn) * 0x1p-9f;   // subnormal: M * 2^-9
        std::memcpy(&u, &v, 4);
        u |= sign;
    } else {
        u = sign | ((E - 7 + 127) << 23) | (Mn << 20);
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

inline float decode_e5m2_bits(uint8_t c)
{
    // e5m2 is the upper byte of an IEEE binary16
    const uint32_t sign = static_cast<uint32_t>(c & 0x80u) << 24;
    const uint32_t E = (c >> 2) & 0x1Fu;
    const uint32_t Mn = c & 0x3u;
    uint32_t u;
    if (E == 31) {
        u = Mn ? 0x7FC00000u : (sign | 0x7F800000u);        // NaN / Inf
    } else if (E == 0) {
        const float v = static_cast<float>(Mn) * 0x1p-16f;  // subnormal: M * 2^-16
        std::memcpy(&u, &v, 4);
        u |= sign;
    } else {
        u = sign | ((E - 15 + 127) << 23) | (Mn << 21);
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

inline uint8_t encode(float f, int fmt)
{
    return fmt == E4M3 ? encode_bits<3, 7, 0x7E>(f) : encode_bits<2, 15, 0x7B>(f);
}

inline float decode(uint8_t c, int fmt)
{
    return fmt == E4M3 ? decode_e4m3_bits(c) : decode_e5m2_bits(c);
}

}  // namespace fp8

struct e4m3 {
    uint8_t x;
    static constexpr int format = fp8::E4M3;
    e4m3() = default;
    explicit e4m3(float f) : x(fp8::encode_bits<3, 7, 0x7E>(f)) {}
    explicit operator float() const { return fp8::decode_e4m3_bits(x); }
};

struct e5m2 {
    uint8_t x;
    static constexpr int format = fp8::E5M2;
    e5m2() = default;
    explicit e5m2(float f) : x(fp8::encode_bits<2, 15, 0x7B>(f)) {}
    explicit operator float() const { return fp8::decode_e5m2_bits(x); }
};

static_assert(sizeof(e4m3) == 1 && sizeof(e5m2) == 1, "fp8 types are one byte");

#endif  // FP8GEMM_FP8_H
