// Launch API of the FP8 GEMM library, as C++ overloads.
//
// Same names, overload set and argument order as the reference's
// GEMM/include/gemm.cuh:11-55: gemm::GEMM and gemm::GEMM4, overloaded on the
// operand types (e4m3 / e5m2 for A and for B), arguments (m, k, n, a, b, out),
// returning the launch status.  Each overload forwards to one extern "C" entry
// point of include/fp8gemm.h; the kernels run asynchronously on the default
// stream, as the reference's launchers do (GEMM/src/gemm.cu:263-285).
//
//   out[i*n + j] = sum_t float(a[i*k + t]) * float(b[j*k + t])
//
// A row-major m x k, B stored n x k ("row-col"), C row-major m x n fp32.
#ifndef GEMM_H
#define GEMM_H

#include <hip/hip_runtime.h>

#include "fp8.h"
#include "fp8gemm.h"

namespace gemm {

// kernel 1 (gemm.cuh:12-15)
inline hipError_t GEMM(int m, int k, int n, const e4m3 *__restrict__ a_matrix,
                       const e4m3 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e4m3_e4m3_stage2(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 2 (gemm.cuh:18-21)
inline hipError_t GEMM4(int m, int k, int n, const e4m3 *__restrict__ a_matrix,
                        const e4m3 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e4m3_e4m3_stage4(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 3 (gemm.cuh:24-27)
inline hipError_t GEMM(int m, int k, int n, const e5m2 *__restrict__ a_matrix,
                       const e5m2 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e5m2_e5m2_stage2(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 4 (gemm.cuh:30-33)
inline hipError_t GEMM4(int m, int k, int n, const e5m2 *__restrict__ a_matrix,
                        const e5m2 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e5m2_e5m2_stage4(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 5 (gemm.cuh:36-39)
inline hipError_t GEMM(int m, int k, int n, const e4m3 *__restrict__ a_matrix,
                       const e5m2 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e4m3_e5m2_stage2(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 6 (gemm.cuh:41-44)
inline hipError_t GEMM4(int m, int k, int n, const e4m3 *__restrict__ a_matrix,
                        const e5m2 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e4m3_e5m2_stage4(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 7 (gemm.cuh:47-50)
inline hipError_t GEMM(int m, int k, int n, const e5m2 *__restrict__ a_matrix,
                       const e4m3 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e5m2_e4m3_stage2(m, k, n, a_matrix, b_matrix, output_matrix));
}

// kernel 8 (gemm.cuh:52-55)
inline hipError_t GEMM4(int m, int k, int n, const e5m2 *__restrict__ a_matrix,
                        const e4m3 *__restrict__ b_matrix, float *__restrict__ output_matrix)
{
    return static_cast<hipError_t>(fp8gemm_e5m2_e4m3_stage4(m, k, n, a_matrix, b_matrix, output_matrix));
}

}  // namespace gemm

#endif  // GEMM_H
