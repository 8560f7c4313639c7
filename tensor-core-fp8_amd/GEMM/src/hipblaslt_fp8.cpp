// Vendor-library comparator: e4m3 x e4m3 -> fp32 GEMM through hipBLASLt, swept
// over square sizes, with this library's own launch timed on the same operands
// next to it.
//
// Stands where the reference's cuBLASLt sample stands (GEMM/src/cublas.cu with
// the TestBench of GEMM/include/helper.h): same problem set-up (op(A) = T with
// lda = k, op(B) = N with ldb = k, i.e. A row-major m x k and B stored n x k, the
// operand layout of gemm::GEMM), per-tensor scale pointers for A and B (and, in `sample`
// mode, for C and D and the pointer that receives the largest |D|, as cublas.cu:41-46 hands
// them over; dropped again, with a note, if the library offers no algorithm with them for an
// fp32 D), a 32 MiB workspace, the first heuristic result, `repeat` launches timed one by
// one with events and averaged (cublas.cu:66-94; here after a warm-up and in blocks that
// alternate between the two libraries, so that both see the same clocks), and a sweep over
// 256, 512, .. 16384 (cublas.cu:123-130).
//
// Differences, on purpose:
//  * operands are N(0,1) values rounded to e4m3 (the sample fills them with
//    InType(i), which saturates almost everywhere); on this chip the speed of
//    the matrix pipe depends on the data;
//  * alpha = 1, beta = 0 and unit scales by default, so that the call computes
//    what gemm::GEMM computes and the two results can be compared; the
//    sample's alpha = 2, beta = 1, scales 2 / 0.5 / 1 / 1 are available as `sample`, where
//    this library's side is fp8gemm_launch_epilogue with the same scalars and pointers and the
//    two results (and largest magnitudes) are compared as well;
//  * the rate is printed in true GFLOP/s (2mnk / seconds / 1e9); the sample
//    divides by 1024 * 1024 and milliseconds (cublas.cu:101).
//
// usage: hipblaslt_fp8 <repeat> [first last step] [sample]
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <stdexcept>
#include <vector>

#include "fp8gemm.h"

namespace {

void check_hip(hipError_t status, const char *what)
{
    if (status != hipSuccess) {
        printf("HIP call failed (%s): %d %s\n", what, (int)status, hipGetErrorString(status));
        throw std::runtime_error("HIP call failed");
    }
}

void check_lt(hipblasStatus_t status, const char *what)
{
    if (status != HIPBLAS_STATUS_SUCCESS) {
        printf("hipBLASLt call failed (%s): status %d\n", what, (int)status);
        throw std::runtime_error("hipBLASLt call failed");
    }
}

// Device buffers and scalars of one problem size (the role of helper.h's TestBench).
struct Problem {
    int m, n, k;
    float alpha, beta;
    size_t workspace_bytes;
    void *a = nullptr, *b = nullptr, *workspace = nullptr;
    float *c = nullptr, *d = nullptr, *ours = nullptr;
    float *scales = nullptr;   // device: a_scale, b_scale, c_scale, d_scale, amax of the vendor's D, amax of ours

    Problem(int m_, int n_, int k_, float alpha_, float beta_, float a_scale, float b_scale, size_t ws)
        : m(m_), n(n_), k(k_), alpha(alpha_), beta(beta_), workspace_bytes(ws)
    {
        std::vector<unsigned char> ha((size_t)m * k), hb((size_t)n * k);
        fp8gemm_fill_normal(ha.data(), ha.size(), FP8GEMM_E4M3, 0xA11CEull + (unsigned)m, 0.0f, 1.0f);
        fp8gemm_fill_normal(hb.data(), hb.size(), FP8GEMM_E4M3, 0xB0Bull + (unsigned)n, 0.0f, 1.0f);
        check_hip(hipMalloc(&a, ha.size()), "hipMalloc A");
        check_hip(hipMalloc(&b, hb.size()), "hipMalloc B");
        check_hip(hipMalloc(&c, (size_t)m * n * sizeof(float)), "hipMalloc C");
        check_hip(hipMalloc(&d, (size_t)m * n * sizeof(float)), "hipMalloc D");
        check_hip(hipMalloc(&ours, (size_t)m * n * sizeof(float)), "hipMalloc ours");
        check_hip(hipMalloc(&workspace, workspace_bytes), "hipMalloc workspace");
        check_hip(hipMalloc(&scales, 6 * sizeof(float)), "hipMalloc scales");
        check_hip(hipMemcpy(a, ha.data(), ha.size(), hipMemcpyHostToDevice), "copy A");
        check_hip(hipMemcpy(b, hb.data(), hb.size(), hipMemcpyHostToDevice), "copy B");
        check_hip(hipMemset(c, 0, (size_t)m * n * sizeof(float)), "clear C");
        const float hs[6] = {a_scale, b_scale, 1.0f, 1.0f, -1.0f, -1.0f};      // C and D scales as in the sample (helper.h:62)
        check_hip(hipMemcpy(scales, hs, sizeof(hs), hipMemcpyHostToDevice), "copy scales");
    }
    ~Problem()
    {
        (void)hipFree(a);
        (void)hipFree(b);
        (void)hipFree(c);
        (void)hipFree(d);
        (void)hipFree(ours);
        (void)hipFree(workspace);
        (void)hipFree(scales);
    }
    Problem(const Problem &) = delete;
    Problem &operator=(const Problem &) = delete;
};

// Sum of the per-launch times of `count` launches, each bracketed by its own event pair
// and a synchronisation (the sample's way of timing, cublas.cu:66-94).
float timed_launches_ms(int count, const std::function<void()> &launch)
{
    hipEvent_t start, stop;
    check_hip(hipEventCreate(&start), "event");
    check_hip(hipEventCreate(&stop), "event");
    float total = 0.0f;
    for (int i = 0; i < count; ++i) {
        check_hip(hipEventRecord(start, nullptr), "record");
        launch();
        check_hip(hipEventRecord(stop, nullptr), "record");
        check_hip(hipEventSynchronize(stop), "sync");
        float ms = 0.0f;
        check_hip(hipEventElapsedTime(&ms, start, stop), "elapsed");
        total += ms;
    }
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return total;
}

// Times two launchers under the same conditions: the chip's clocks depend on what ran in
// the last few milliseconds, so both are warmed up first and then timed in alternating
// blocks instead of one after the other.
void average_ms_pair(int repeat, const std::function<void()> &first, const std::function<void()> &second,
                     float &ms_first, float &ms_second)
{
    const int warm = repeat < 10 ? repeat : 10;
    (void)timed_launches_ms(warm, first);
    (void)timed_launches_ms(warm, second);
    const int blocks = repeat >= 8 ? 4 : 1;
    float total_first = 0.0f, total_second = 0.0f;
    int done = 0;
    for (int blk = 0; blk < blocks; ++blk) {
        const int count = (blk == blocks - 1) ? repeat - done : repeat / blocks;
        total_first += timed_launches_ms(count, first);
        total_second += timed_launches_ms(count, second);
        done += count;
    }
    ms_first = total_first / (float)repeat;
    ms_second = total_second / (float)repeat;
}

// Returns false when the library offers no algorithm for the problem.
bool run_size(hipblasLtHandle_t handle, Problem &p, int repeat, bool comparable)
{
    hipblasLtMatmulDesc_t op = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr, ld = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    check_lt(hipblasLtMatmulDescCreate(&op, HIPBLAS_COMPUTE_32F, HIP_R_32F), "desc create");
    check_lt(hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "transa");
    check_lt(hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "transb");
    const float *sa = p.scales, *sb = p.scales + 1;
    check_lt(hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_A_SCALE_POINTER, &sa, sizeof(sa)), "a scale");
    check_lt(hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_B_SCALE_POINTER, &sb, sizeof(sb)), "b scale");
    // column-major views: A is k x m (leading dimension k), B is k x n, C and D are m x n
    check_lt(hipblasLtMatrixLayoutCreate(&la, HIP_R_8F_E4M3, p.k, p.m, p.k), "layout A");
    check_lt(hipblasLtMatrixLayoutCreate(&lb, HIP_R_8F_E4M3, p.k, p.n, p.k), "layout B");
    check_lt(hipblasLtMatrixLayoutCreate(&lc, HIP_R_32F, p.m, p.n, p.m), "layout C");
    check_lt(hipblasLtMatrixLayoutCreate(&ld, HIP_R_32F, p.m, p.n, p.m), "layout D");
    check_lt(hipblasLtMatmulPreferenceCreate(&pref), "pref create");
    check_lt(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES,
                                                   &p.workspace_bytes, sizeof(p.workspace_bytes)),
             "workspace");
    hipblasLtMatmulHeuristicResult_t heur = {};
    int found = 0;
    bool vendor_amax = false;
    if (!comparable) {
        // the sample also hands over scale pointers for C and D and a pointer for the largest |D|
        const float *sc = p.scales + 2, *sd = p.scales + 3;
        float *amax = p.scales + 4;
        const bool set = hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_C_SCALE_POINTER, &sc, sizeof(sc)) == HIPBLAS_STATUS_SUCCESS &&
                         hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_D_SCALE_POINTER, &sd, sizeof(sd)) == HIPBLAS_STATUS_SUCCESS &&
                         hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_AMAX_D_POINTER, &amax, sizeof(amax)) == HIPBLAS_STATUS_SUCCESS;
        if (set && hipblasLtMatmulAlgoGetHeuristic(handle, op, la, lb, lc, ld, pref, 1, &heur, &found) == HIPBLAS_STATUS_SUCCESS && found > 0) {
            vendor_amax = true;
        } else {
            printf("(no hipBLASLt algorithm takes C / D scale and amax pointers for an fp32 D: A and B scales only)\n");
            const void *none = nullptr;
            (void)hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_C_SCALE_POINTER, &none, sizeof(none));
            (void)hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_D_SCALE_POINTER, &none, sizeof(none));
            (void)hipblasLtMatmulDescSetAttribute(op, HIPBLASLT_MATMUL_DESC_AMAX_D_POINTER, &none, sizeof(none));
            found = 0;
        }
    }
    if (found == 0) check_lt(hipblasLtMatmulAlgoGetHeuristic(handle, op, la, lb, lc, ld, pref, 1, &heur, &found), "heuristic");
    bool ok = found > 0;
    if (!ok) {
        printf("no heuristic function available for current configuration\n");
    } else {
        auto vendor = [&] {
            check_lt(hipblasLtMatmul(handle, op, &p.alpha, p.a, la, p.b, lb, &p.beta, p.c, lc, p.d, ld,
                                     &heur.algo, p.workspace, p.workspace_bytes, nullptr),
                     "matmul");
        };
        auto own = [&] {
            // the plain launch, or (sample mode) the epilogue entry point with the sample's scalars and pointers;
            // C holds zeros, so its layout (column-major there, row-major here) does not matter
            const int e = comparable
                              ? fp8gemm_launch(p.m, p.k, p.n, p.a, FP8GEMM_E4M3, p.b, FP8GEMM_E4M3, p.ours, 2, nullptr)
                              : fp8gemm_launch_epilogue(p.m, p.k, p.n, p.a, FP8GEMM_E4M3, p.b, FP8GEMM_E4M3, p.ours, FP8GEMM_OUT_F32, p.alpha,
                                                        p.beta, p.c, FP8GEMM_OUT_F32, p.scales, p.scales + 1, p.scales + 2, p.scales + 3,
                                                        p.scales + 5, nullptr);
            if (e != 0) {
                printf("fp8gemm launch failed: %d %s\n", e, fp8gemm_error_string(e));
                throw std::runtime_error("fp8gemm launch failed");
            }
        };
        vendor();
        own();
        check_hip(hipDeviceSynchronize(), "sync");
        float ms_vendor = 0.0f, ms_own = 0.0f;
        average_ms_pair(repeat, vendor, own, ms_vendor, ms_own);
        const double flop = 2.0 * p.m * (double)p.n * p.k;
        printf("Average hipblasLtMatmul execution time %f (ms)\n", ms_vendor);
        printf("GEMM-hipblaslt-fp8: M[%d] x N[%d] x K[%d], performance = %lfGFLOPS.\n", p.m, p.n, p.k,
               flop / (ms_vendor * 1e-3) / 1e9);
        printf("GEMM-fp8gemm-fp8:   M[%d] x N[%d] x K[%d], performance = %lfGFLOPS (%f ms).\n", p.m, p.n, p.k,
               flop / (ms_own * 1e-3) / 1e9, ms_own);
        {
            // D is column-major m x n, ours row-major m x n: D[i + j*m] against ours[i*n + j]
            // on a strided sample; both are fp32 sums of the same products in different orders
            std::vector<float> hd((size_t)p.m * p.n), ho((size_t)p.m * p.n);
            check_hip(hipMemcpy(hd.data(), p.d, hd.size() * sizeof(float), hipMemcpyDeviceToHost), "copy D");
            check_hip(hipMemcpy(ho.data(), p.ours, ho.size() * sizeof(float), hipMemcpyDeviceToHost), "copy ours");
            double worst = 0.0, scale = 0.0;
            const size_t stride = hd.size() > (1u << 22) ? 61 : 1;
            for (size_t idx = 0; idx < hd.size(); idx += stride) {
                const size_t i = idx / p.n, j = idx % p.n;
                const double diff = std::fabs((double)hd[i + j * (size_t)p.m] - (double)ho[idx]);
                if (diff > worst) worst = diff;
                if (std::fabs((double)ho[idx]) > scale) scale = std::fabs((double)ho[idx]);
            }
            printf("max |hipblaslt - fp8gemm| = %g (largest |C| = %g, sqrt(K) * 2^-24 * that = %g)\n", worst, scale,
                   std::sqrt((double)p.k) * std::ldexp(1.0, -24) * scale);
            if (!comparable) {
                float amax[2] = {0.0f, 0.0f};
                check_hip(hipMemcpy(amax, p.scales + 4, sizeof(amax), hipMemcpyDeviceToHost), "copy amax");
                if (vendor_amax)
                    printf("largest |D|: hipblaslt %g, fp8gemm %g\n", amax[0], amax[1]);
                else
                    printf("largest |D|: fp8gemm %g (hipblaslt took no amax pointer)\n", amax[1]);
            }
        }
    }
    if (pref) check_lt(hipblasLtMatmulPreferenceDestroy(pref), "destroy");
    if (ld) check_lt(hipblasLtMatrixLayoutDestroy(ld), "destroy");
    if (lc) check_lt(hipblasLtMatrixLayoutDestroy(lc), "destroy");
    if (lb) check_lt(hipblasLtMatrixLayoutDestroy(lb), "destroy");
    if (la) check_lt(hipblasLtMatrixLayoutDestroy(la), "destroy");
    if (op) check_lt(hipblasLtMatmulDescDestroy(op), "destroy");
    return ok;
}

}  // namespace

int main(int argc, char *argv[])
{
    if (argc < 2) {
        printf("Usage: %s <repeat> [first last step] [sample]\n       %s <repeat> shape M K N\n", argv[0], argv[0]);
        return 1;
    }
    const int repeat = atoi(argv[1]);
    if (argc == 6 && strcmp(argv[2], "shape") == 0) {
        // one shape that need not be square (same weight buffer for every launch)
        const int m = atoi(argv[3]), k = atoi(argv[4]), n = atoi(argv[5]);
        if (repeat < 1 || m < 1 || k < 1 || n < 1) {
            printf("bad arguments\n");
            return 1;
        }
        try {
            hipblasLtHandle_t handle = nullptr;
            check_lt(hipblasLtCreate(&handle), "create");
            Problem p(m, n, k, 1.0f, 0.0f, 1.0f, 1.0f, 32ull * 1024 * 1024);
            run_size(handle, p, repeat, true);
            check_lt(hipblasLtDestroy(handle), "destroy");
        } catch (const std::exception &e) {
            printf("aborted: %s\n", e.what());
            return 2;
        }
        return 0;
    }
    int first = 256, last = 16384, step = 256;
    bool sample = false;
    int pos = 2;
    if (argc >= 5 && strcmp(argv[2], "sample") != 0) {
        first = atoi(argv[2]);
        last = atoi(argv[3]);
        step = atoi(argv[4]);
        pos = 5;
    }
    if (argc > pos && strcmp(argv[pos], "sample") == 0) sample = true;
    if (repeat < 1 || first < 1 || last < first || step < 1) {
        printf("bad arguments\n");
        return 1;
    }
    try {
        hipblasLtHandle_t handle = nullptr;
        check_lt(hipblasLtCreate(&handle), "create");
        for (int size = first; size <= last; size += step) {
            // the sample's scalars (cublas.cu:131-134, helper.h:60-62), or the ones that make
            // the call compute exactly what gemm::GEMM computes
            Problem p(size, size, size, sample ? 2.0f : 1.0f, sample ? 1.0f : 0.0f, sample ? 2.0f : 1.0f,
                      sample ? 0.5f : 1.0f, 32ull * 1024 * 1024);
            run_size(handle, p, repeat, !sample);
            fflush(stdout);
        }
        check_lt(hipblasLtDestroy(handle), "destroy");
    } catch (const std::exception &e) {
        printf("aborted: %s\n", e.what());
        return 2;
    }
    return 0;
}
