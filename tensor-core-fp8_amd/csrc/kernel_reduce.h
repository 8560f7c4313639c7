// Sum of split-K partial results: C[i] = ws[0][i] + ws[1][i] + ... in ascending
// slice order, so the result does not depend on how the slices were scheduled.
// HBM-bound: (nsplit + 1) * count * 4 bytes; 128-bit accesses when count and the
// pointers allow.
#ifndef FP8GEMM_KERNEL_REDUCE_H
#define FP8GEMM_KERNEL_REDUCE_H

#include "device_common.h"

__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float *__restrict__ ws,
                                                                 void *__restrict__ C,
                                                                 size_t count, int nsplit, OutSpec spec)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    float amax_local = 0.0f;
    if (i < count) {
        float s = ws[i];
        for (int p = 1; p < nsplit; ++p) s += ws[(size_t)p * count + i];
        store_out(C, i, finish_one(spec, out_factors(spec), i, s, amax_local), spec.type);
    }
    amax_commit(spec, amax_local);
}

// count4 = count / 4; requires count % 4 == 0 and 16-byte aligned ws and C
__global__ __launch_bounds__(256) void gemm_splitk_reduce4_kernel(const v4f *__restrict__ ws,
                                                                  void *__restrict__ C,
                                                                  size_t count4, int nsplit, OutSpec spec)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    float amax_local = 0.0f;
    if (i < count4) {
        v4f s = ws[i];
        for (int p = 1; p < nsplit; ++p) {
            const v4f v = ws[(size_t)p * count4 + i];
            s[0] += v[0];
            s[1] += v[1];
            s[2] += v[2];
            s[3] += v[3];
        }
        store_out4(C, i * 4, finish_four(spec, out_factors(spec), i * 4, s, amax_local), spec.type);
    }
    amax_commit(spec, amax_local);
}

// Partial sums of the persistent tiled kernel: scratch slot s*tail + u holds slice s of
// tail tile u as BM x BN floats (row stride BN).  One thread per 4 consecutive columns
// of a tile adds the slices in ascending order and writes the part that lies inside C.
// The tile numbering is the kernel's: strips of GM tile rows, down a column first.
__global__ __launch_bounds__(256) void gemm_tile_slices_reduce_kernel(const float *__restrict__ ws,
                                                                      void *__restrict__ C, int M, int N,
                                                                      int BM, int BN, int tiles_m, int tiles_n,
                                                                      int GM, int CB, int bulk, int tail, int nsplit,
                                                                      OutSpec spec)
{
    const int quads_per_tile = BM * BN / 4;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int u = (int)(id / quads_per_tile);
    float amax_local = 0.0f;
    if (u < tail) {
        const int q = (int)(id - (size_t)u * quads_per_tile);
        const int row = q / (BN / 4);
        const int col = (q - row * (BN / 4)) * 4;
        const int g = bulk + u;
        int tm, tn;
        tile_of_number(g, tiles_m, tiles_n, GM, CB, tm, tn);
        const int grow = tm * BM + row;
        const int gcol = tn * BN + col;
        if (grow < M && gcol < N) {
            const size_t tile_floats = (size_t)BM * BN;
            const float *src = ws + (size_t)u * tile_floats + (size_t)row * BN + col;
            v4f s = *reinterpret_cast<const v4f *>(src);
            for (int p = 1; p < nsplit; ++p) {
                const v4f v = *reinterpret_cast<const v4f *>(src + (size_t)p * tail * tile_floats);
                s[0] += v[0];
                s[1] += v[1];
                s[2] += v[2];
                s[3] += v[3];
            }
            const OutFactors ofac = out_factors(spec);
            const size_t index = (size_t)grow * N + gcol;
            const bool aligned = reinterpret_cast<uintptr_t>(C) % 16 == 0 && (!spec.c || reinterpret_cast<uintptr_t>(spec.c) % 16 == 0);
            if (gcol + 3 < N && N % 4 == 0 && aligned) {
                store_out4(C, index, finish_four(spec, ofac, index, s, amax_local), spec.type);
            } else {
                for (int e = 0; e < 4; ++e)
                    if (gcol + e < N) store_out(C, index + e, finish_one(spec, ofac, index + e, s[e], amax_local), spec.type);
            }
        }
    }
    amax_commit(spec, amax_local);
}

#endif  // FP8GEMM_KERNEL_REDUCE_H
