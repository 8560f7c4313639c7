// Sum of split-K partial results: C[i] = ws[0][i] + ws[1][i] + ... in ascending
// slice order, so the result does not depend on how the slices were scheduled.
// HBM-bound: (nsplit + 1) * count * 4 bytes; 128-bit accesses when count and the
// pointers allow.
#ifndef FP8GEMM_KERNEL_REDUCE_H
#define FP8GEMM_KERNEL_REDUCE_H

#include "device_common.h"

__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float *__restrict__ ws,
                                                                 float *__restrict__ C,
                                                                 size_t count, int nsplit)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float s = ws[i];
    for (int p = 1; p < nsplit; ++p) s += ws[(size_t)p * count + i];
    C[i] = s;
}

// count4 = count / 4; requires count % 4 == 0 and 16-byte aligned ws and C
__global__ __launch_bounds__(256) void gemm_splitk_reduce4_kernel(const v4f *__restrict__ ws,
                                                                  v4f *__restrict__ C,
                                                                  size_t count4, int nsplit)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count4) return;
    v4f s = ws[i];
    for (int p = 1; p < nsplit; ++p) {
        const v4f v = ws[(size_t)p * count4 + i];
        s[0] += v[0];
        s[1] += v[1];
        s[2] += v[2];
        s[3] += v[3];
    }
    C[i] = s;
}

#endif  // FP8GEMM_KERNEL_REDUCE_H
