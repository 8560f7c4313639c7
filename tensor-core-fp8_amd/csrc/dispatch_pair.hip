// One operand pairing of the launch code (dispatch.h).  Compiled four times, with
// -DFP8GEMM_PAIR_A=<0|1> -DFP8GEMM_PAIR_B=<0|1> (0 = E4M3, 1 = E5M2).
#include "dispatch.h"

#if !defined(FP8GEMM_PAIR_A) || !defined(FP8GEMM_PAIR_B)
#error "compile with -DFP8GEMM_PAIR_A=<0|1> -DFP8GEMM_PAIR_B=<0|1>"
#endif

namespace fp8gemm_detail {
template hipError_t dispatch<FP8GEMM_PAIR_A, FP8GEMM_PAIR_B>(int, int, int, const uint8_t *, const uint8_t *, void *, int, int, int,
                                                             const OutSpec &, Workspace &, hipStream_t);
template hipError_t dispatch_bell<FP8GEMM_PAIR_A, FP8GEMM_PAIR_B>(int, int, int, const uint8_t *, const uint8_t *, float *, const BellSpec &,
                                                                  Workspace &, hipStream_t);
}  // namespace fp8gemm_detail
