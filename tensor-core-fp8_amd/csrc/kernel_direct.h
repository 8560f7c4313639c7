// General-shape kernel: one wave per 32x32 tile of C, operands straight from
// global memory into MFMA registers.  Slow (no reuse through LDS) but accepts
// any m, k, n >= 1 and any pointer alignment; the tiled and skinny kernels take
// over wherever their shape rules hold.
#ifndef FP8GEMM_KERNEL_DIRECT_H
#define FP8GEMM_KERNEL_DIRECT_H

#include "device_common.h"

// 32 bytes of `row` starting at byte column kk; bytes outside the matrix read
// as fp8 code 0x00 (+0.0), which adds exactly nothing to a dot product.
__device__ __forceinline__ v8i direct_load32(const uint8_t *__restrict__ base, int row, int rows,
                                             int kk, int K, bool vec_ok)
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row >= rows || kk >= K) return r;
    const uint8_t *p = base + (size_t)row * K + kk;
    if (vec_ok && kk + 32 <= K) {
        const v4i lo = *reinterpret_cast<const v4i *>(p);
        const v4i hi = *reinterpret_cast<const v4i *>(p + 16);
        return pack8(lo, hi);
    }
    const int nb = (K - kk < 32) ? K - kk : 32;
    for (int w = 0; w < 8; ++w) {
        uint32_t word = 0;
        for (int b = 0; b < 4; ++b) {
            const int idx = w * 4 + b;
            if (idx < nb) word |= (uint32_t)p[idx] << (8 * b);
        }
        r[w] = (int)word;
    }
    return r;
}

template <int AF, int BF>
__global__ __launch_bounds__(64) void gemm_direct_kernel(int M, int K, int N,
                                                         const uint8_t *__restrict__ A,
                                                         const uint8_t *__restrict__ B,
                                                         void *__restrict__ C, int tiles_n, int vec_ok, OutSpec spec)
{
    const int lane = threadIdx.x;
    const int i = lane & 31;
    const int g = lane >> 5;
    // a one-dimensional grid (row-major over the tiles of C): neither dimension is capped at 65535 tiles
    const int m0 = (int)(blockIdx.x / (unsigned)tiles_n) * 32;
    const int n0 = (int)(blockIdx.x % (unsigned)tiles_n) * 32;
    v16f acc;
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    for (int k0 = 0; k0 < K; k0 += 64) {
        const int kk = k0 + g * 32;
        const v8i a = direct_load32(A, m0 + i, M, kk, K, vec_ok != 0);
        const v8i b = direct_load32(B, n0 + i, N, kk, K, vec_ok != 0);
        acc = mfma_32x32x64<AF, BF>(a, b, acc);
    }

    const int col = n0 + i;
    const OutFactors ofac = out_factors(spec);
    float amax_local = 0.0f;
    if (col < N) {
        for (int r = 0; r < 16; ++r) {
            const int row = m0 + 8 * (r >> 2) + 4 * g + (r & 3);
            if (row < M) {
                const size_t index = (size_t)row * N + col;
                store_out(C, index, finish_one(spec, ofac, index, acc[r], amax_local), spec.type);
            }
        }
    }
    amax_commit(spec, amax_local);
}

#endif  // FP8GEMM_KERNEL_DIRECT_H
