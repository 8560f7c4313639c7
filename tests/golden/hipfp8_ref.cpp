// Independent library cross-check for the fp8 codec tests: the host-side OCP FP8
// conversions that ship with ROCm (hip/hip_fp8.h), exported with a C ABI.
// Built by tests/golden/make_codec_vectors.py; not part of the library.
#include <hip/hip_fp8.h>
#include <cstddef>
#include <cstdint>

extern "C" void hipfp8_encode(const float *src, uint8_t *dst, size_t n, int fmt)
{
    for (size_t i = 0; i < n; ++i)
        dst[i] = __hip_cvt_float_to_fp8(src[i], __HIP_SATFINITE, fmt == 0 ? __HIP_E4M3 : __HIP_E5M2);
}

extern "C" void hipfp8_decode(const uint8_t *src, float *dst, size_t n, int fmt)
{
    for (size_t i = 0; i < n; ++i) {
        const __half_raw h = __hip_cvt_fp8_to_halfraw(src[i], fmt == 0 ? __HIP_E4M3 : __HIP_E5M2);
        dst[i] = __half2float(__half(h));
    }
}
