// Benchmark-and-verify harness of the FP8 GEMM library.
//
// Same command line and flow as the reference's GEMM/gemm_main.cpp:
//   ./out/gemm dimM dimK dimN kernel verify record testbench [dist [seed]]
// random fp8 operands -> optional CPU fp32 reference GEMM -> 20 warm-up + 100
// timed launches, one event pair per launch (gemm_main.cpp:25-26, 69-83) ->
// GFLOPS print (:84-86) -> optional CSV row M,K,N,GFLOPS appended to
// ./data/fp8_gemm_v<kernel>.csv (:87-110) -> optional verification (:159-184).
//
// kernel: 1/2 e4m3 x e4m3, 3/4 e5m2 x e5m2, 5/6 e4m3 x e5m2, 7/8 e5m2 x e4m3;
// odd ids call gemm::GEMM, even ids gemm::GEMM4 (gemm_main.cpp:223-255).  All
// eight ids run here (the reference leaves 4, 6 and 8 commented out).  Kernel 0
// is an addition: it runs and times only the CPU reference path, without
// touching the GPU.
//
// Kernels 10 to 13 are additions for the sparse kernels the reference's README plans (SpMM, SpMV;
// README.md:7): 10 SpMM and 11 SpMV with S (dimM x dimK) in blocked-ELL form, 12 SpMM and 13 SpMV
// with S in compressed sparse rows, e4m3 x e4m3, operands from the generators of
// include/bm_test_utils.h (GenerateUniformBlockedELLIndex, MakeSparseMatrixRandomUniform,
// SortedRowSwizzle).  GEMM_SPARSE_BLOCK (default 128) and GEMM_SPARSE_KEEP (share of blocks or
// elements kept, default 0.25 / 0.1) shape the operand; dimN is the number of dense columns (SpMV: 1).
//
// Differences kept on purpose: verification counts its errors (the reference's
// `if(num_errors = 0)` assigns) and uses the bound
// |C_gpu - C_ref| <= 2*K*2^-24 * sum_k |a*b| next to the reference's absolute
// 0.25; operands may come from seeded generators (dist/seed arguments) besides
// the reference's default-seeded uniform(-1,1) stream.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <random>
#include <string>
#include <vector>

#include <sys/stat.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#include "./include/bm_test_utils.h"
#include "./include/gemm.h"

#define repeat 100
#define warmup 20

// MI355X peaks the reported fractions refer to: dense FP8 MFMA 5.0 PFLOP/s, HBM3E 8 TB/s
static const double kPeakFp8Tflops = 5000.0;
static const double kPeakHbmGBs = 8000.0;

struct Options {
    const char *dist = "reference";   // "reference" = MakeDenseMatrix as in the reference
    uint64_t seed = 0;
};

template <typename T>
static const char *type_name() { return T::format == fp8::E4M3 ? "e4m3" : "e5m2"; }

// CPU fp32 reference GEMM: for m, n, k:  C[m*N+n] += (float)A[m*K+k] * (float)B[n*K+k]
// (gemm_main.cpp:39-53 of the reference).  Every output is a running fp32 sum in
// ascending k; rows of C are independent, so they are spread over threads, and
// decoding goes through a 256-entry table instead of once per multiply.  S, when
// given, receives sum_k |a*b| per output (the scale of the verification bound) and W the
// sum over groups of 8 consecutive K bytes of (8 x largest |a*b| of the group): the MFMA adds
// the products of such a group aligned to the largest of them and keeps 13 binary places
// below its leading bit, so W * 2^-13 bounds what the groups can lose.
static const int kWindowBlock = 8;
template <typename AType, typename BType>
static void cpu_reference_gemm(int M, int K, int N, const AType *A, const BType *B, float *C, double *S, double *W,
                               int threads)
{
    float lutA[256], lutB[256];
    for (int c = 0; c < 256; ++c) {
        lutA[c] = fp8::decode((uint8_t)c, AType::format);
        lutB[c] = fp8::decode((uint8_t)c, BType::format);
    }
    (void)threads;
#pragma omp parallel num_threads(threads)
    {
        std::vector<float> arow(K);
#pragma omp for schedule(dynamic, 4)
        for (int m = 0; m < M; ++m) {
            for (int k = 0; k < K; ++k) arow[k] = lutA[A[(size_t)m * K + k].x];
            for (int n = 0; n < N; ++n) {
                const BType *brow = B + (size_t)n * K;
                float acc = 0.0f;
                if (S) {
                    double sabs = 0.0, window = 0.0;
                    for (int k0 = 0; k0 < K; k0 += kWindowBlock) {
                        const int k1 = std::min(K, k0 + kWindowBlock);
                        double largest = 0.0;
                        for (int k = k0; k < k1; ++k) {
                            const float p = arow[k] * lutB[brow[k].x];   // exact: 8 significant bits at most
                            acc += p;
                            sabs += std::fabs((double)p);
                            largest = std::max(largest, std::fabs((double)p));
                        }
                        window += largest * (k1 - k0);
                    }
                    S[(size_t)m * N + n] = sabs;
                    if (W) W[(size_t)m * N + n] = window;
                } else {
                    for (int k = 0; k < K; ++k) acc += arow[k] * lutB[brow[k].x];
                }
                C[(size_t)m * N + n] = acc;
            }
        }
    }
}

static int host_threads()
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static double seconds_since(std::chrono::steady_clock::time_point t0)
{
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

template <typename AType, typename BType>
static void fill_operands(int M, int K, int N, AType *A, BType *B, const Options &opt)
{
    if (!std::strcmp(opt.dist, "reference")) {
        std::default_random_engine generator;
        MakeDenseMatrix<AType>(M, K, A, generator);
        MakeDenseMatrix<BType>(N, K, B, generator);
        return;
    }
    const uint64_t seedA = 0xA11CEull + opt.seed, seedB = 0xB0Bull + opt.seed;
    // activations use the named distribution; "weights" applies to B only, as in an LLM linear layer
    const char *distA = std::strcmp(opt.dist, "weights") ? opt.dist : "normal";
    if (!MakeDenseMatrixSeeded<AType>(M, K, A, distA, seedA) || !MakeDenseMatrixSeeded<BType>(N, K, B, opt.dist, seedB)) {
        std::fprintf(stderr, "unknown distribution '%s'\n", opt.dist);
        std::exit(EXIT_FAILURE);
    }
}

static void record_csv(int kernel, int M, int K, int N, double gflops, double usec, double gbs)
{
    mkdir("./data", 0755);
    const std::string base = "./data/fp8_gemm_v" + std::to_string(kernel);
    std::ofstream f(base + ".csv", std::ios::app);           // the reference's columns
    f << M << ',' << K << ',' << N << ',' << gflops << std::endl;
    std::ofstream g(base + "_ext.csv", std::ios::app);       // M,K,N,GFLOPS,TFLOPS,latency_us,GB/s,frac_mfma_peak,frac_hbm_peak
    g << M << ',' << K << ',' << N << ',' << gflops << ',' << gflops / 1e3 << ',' << usec << ',' << gbs << ','
      << gflops / 1e3 / kPeakFp8Tflops << ',' << gbs / kPeakHbmGBs << std::endl;
}

// CPU-only mode (kernel 0): times the reference CPU path, single thread and all threads.
template <typename AType, typename BType>
static void BmCPU(int M, int K, int N, const Options &opt)
{
    std::vector<AType> A((size_t)M * K);
    std::vector<BType> B((size_t)N * K);
    fill_operands(M, K, N, A.data(), B.data(), opt);
    std::vector<float> C1((size_t)M * N), Cn((size_t)M * N);
    const double flop = 2.0 * M * K * N;
    auto t0 = std::chrono::steady_clock::now();
    cpu_reference_gemm(M, K, N, A.data(), B.data(), C1.data(), nullptr, nullptr, 1);
    const double s1 = seconds_since(t0);
    t0 = std::chrono::steady_clock::now();
    cpu_reference_gemm(M, K, N, A.data(), B.data(), Cn.data(), nullptr, nullptr, host_threads());
    const double sn = seconds_since(t0);
    const bool same = std::memcmp(C1.data(), Cn.data(), C1.size() * sizeof(float)) == 0;
    std::printf("CPU reference GEMM %s x %s: M = %d, K = %d, N = %d\n", type_name<AType>(), type_name<BType>(), M, K, N);
    std::printf("  1 thread : %.3f s  %.3f GFlops\n", s1, flop / s1 / 1e9);
    std::printf("  %d threads: %.3f s  %.3f GFlops  (bit-identical to 1 thread: %s)\n", host_threads(), sn,
                flop / sn / 1e9, same ? "yes" : "NO");
    double checksum = 0.0;
    for (float v : C1) checksum += v;
    std::printf("  checksum %.9g\n", checksum);
}

template <typename AType, typename BType, typename CType>
void BmFN(int M, int K, int N, int kernel, bool func, bool record, const Options &opt)
{
    // operands and reference output in host memory
    std::vector<AType> h_A((size_t)M * K);   // row major
    std::vector<BType> h_B((size_t)N * K);   // col major: stored N x K
    fill_operands(M, K, N, h_A.data(), h_B.data(), opt);
    std::vector<float> h_ref;
    std::vector<double> h_scale, h_window;
    if (func) {
        h_ref.assign((size_t)M * N, 0.0f);
        h_scale.assign((size_t)M * N, 0.0);
        h_window.assign((size_t)M * N, 0.0);
        const auto t0 = std::chrono::steady_clock::now();
        cpu_reference_gemm(M, K, N, h_A.data(), h_B.data(), h_ref.data(), h_scale.data(), h_window.data(), host_threads());
        std::printf("CPU reference: %.3f s on %d threads\n", seconds_since(t0), host_threads());
    }

    AType *d_A;
    BType *d_B;
    CType *d_C;
    checkHip(hipMalloc(&d_A, h_A.size() * sizeof(AType)));
    checkHip(hipMalloc(&d_B, h_B.size() * sizeof(BType)));
    checkHip(hipMalloc(&d_C, (size_t)M * N * sizeof(CType)));
    checkHip(hipMemcpy(d_A, h_A.data(), h_A.size() * sizeof(AType), hipMemcpyHostToDevice));
    checkHip(hipMemcpy(d_B, h_B.data(), h_B.size() * sizeof(BType), hipMemcpyHostToDevice));

    const bool four = (kernel % 2 == 0);
    auto launch = [&]() -> hipError_t {
        return four ? gemm::GEMM4(M, K, N, d_A, d_B, d_C) : gemm::GEMM(M, K, N, d_A, d_B, d_C);
    };

    // one event pair per launch, as the reference times it
    hipEvent_t start, end;
    checkHip(hipEventCreate(&start));
    checkHip(hipEventCreate(&end));
    float total_msec = 0.0f;
    for (int i = 0; i < repeat + warmup; ++i) {
        float msec = 0.0f;
        checkHip(hipEventRecord(start));
        checkHip(launch());
        checkHip(hipEventRecord(end));
        checkHip(hipEventSynchronize(end));
        checkHip(hipEventElapsedTime(&msec, start, end));
        if (i >= warmup) total_msec += msec;
    }
    // and one pair around the whole batch, which leaves out the per-launch synchronisation gaps
    float batch_msec = 0.0f;
    checkHip(hipEventRecord(start));
    for (int i = 0; i < repeat; ++i) checkHip(launch());
    checkHip(hipEventRecord(end));
    checkHip(hipEventSynchronize(end));
    checkHip(hipEventElapsedTime(&batch_msec, start, end));

    const double flop = 2.0 * (double)M * K * N;
    const double bytes = (double)M * K + (double)N * K + 4.0 * (double)M * N;
    const double Gperf = flop / 1000 / 1000 / total_msec * repeat;
    const double Gbatch = flop / 1000 / 1000 / batch_msec * repeat;
    const double usec = batch_msec / repeat * 1e3;
    const double gbs = bytes / (batch_msec / repeat) / 1e6;
    std::printf("GEMM-stage%d:  M = %d, K = %d, N = %d\n", four ? 4 : 2, M, K, N);
    std::printf("\033[33mFP8-TC Avager Performance = \033[35m%lf\033[0m \033[33mGFlops\033[0m\n", Gperf);
    std::printf("batch of %d launches: %.3f us per launch, %.1f TFlops (%.1f%% of %.0f dense FP8 peak), %.1f GB/s (%.1f%% of %.0f)\n",
                repeat, usec, Gbatch / 1e3, Gbatch / 1e3 / kPeakFp8Tflops * 100.0, kPeakFp8Tflops, gbs, gbs / kPeakHbmGBs * 100.0,
                kPeakHbmGBs);
    if (record) record_csv(kernel, M, K, N, Gperf, usec, gbs);

    if (func) {
        std::vector<CType> h_C((size_t)M * N);
        checkHip(hipMemcpy(h_C.data(), d_C, h_C.size() * sizeof(CType), hipMemcpyDeviceToHost));
        size_t num_errors = 0, num_abs = 0;
        double max_error = 0.0, worst_ratio = 0.0;
        for (size_t i = 0; i < h_C.size(); ++i) {
            const double err = std::fabs((double)h_C[i] - (double)h_ref[i]);
            // fp32 reordering bound; for a short K (few products per output) what the MFMA's
            // groups of 8 products drop below 2^-13 of their largest product shows next to it
            double tol = 2.0 * K * std::ldexp(1.0, -24) * h_scale[i];
            if (K < 1024) tol += std::ldexp(1.0, -13) * h_window[i];
            if (!(err <= tol)) ++num_errors;                    // also catches NaN
            if (err > 0.25) ++num_abs;                          // the reference's criterion
            if (err > max_error) max_error = err;
            if (tol > 0 && err / tol > worst_ratio) worst_ratio = err / tol;
        }
        if (num_errors == 0)
            std::printf("Result Verified!\n");
        else
            std::cout << "There are " << num_errors << " errors." << std::endl;
        std::printf("MAx Error is %f\n", max_error);
        std::printf("worst |err| / (2*K*2^-24*sum|a*b|) = %.4g; outputs off by more than 0.25: %zu\n", worst_ratio, num_abs);
    }
    checkHip(hipEventDestroy(start));
    checkHip(hipEventDestroy(end));
    checkHip(hipFree(d_A));
    checkHip(hipFree(d_B));
    checkHip(hipFree(d_C));
    std::printf("end BmFN\n");
}

// ---- sparse kernels ------------------------------------------------------------------
// CPU reference: out[i][j] = sum over the stored entries of row i, in storage order, of
// float(value) * float(B[j][column]) -- the loop of cpu_reference_gemm with the zeros left out.
// S receives sum |a*b| per output.
template <typename SType, typename BType>
static void cpu_reference_spmm(int M, int K, int N, const SType *values, const int *row_offsets, const int *col, const BType *B,
                               float *out, double *S)
{
    float lutS[256], lutB[256];
    for (int c = 0; c < 256; ++c) {
        lutS[c] = fp8::decode((uint8_t)c, SType::format);
        lutB[c] = fp8::decode((uint8_t)c, BType::format);
    }
#pragma omp parallel for schedule(dynamic, 4)
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            const BType *brow = B + (size_t)j * K;
            float acc = 0.0f;
            double sabs = 0.0;
            for (int e = row_offsets[i]; e < row_offsets[i + 1]; ++e) {
                const float p = lutS[values[e].x] * lutB[brow[col[e]].x];
                acc += p;
                sabs += std::fabs((double)p);
            }
            out[(size_t)i * N + j] = acc;
            S[(size_t)i * N + j] = sabs;
        }
}

static double env_number(const char *name, double fallback)
{
    const char *v = std::getenv(name);
    return v ? std::atof(v) : fallback;
}

// kernel 10: SpMM blocked-ELL, 11: SpMV blocked-ELL, 12: SpMM CSR, 13: SpMV CSR (rows longest first)
template <typename SType, typename BType>
static void BmSparse(int M, int K, int N, int kernel, bool func, bool record)
{
    const bool bell = kernel == 10 || kernel == 11, vec = kernel == 11 || kernel == 13;
    if (vec) N = 1;
    std::default_random_engine generator;
    std::vector<SType> h_val;
    std::vector<int> h_off, h_col, h_bcols, h_order;
    int block = 0, ell = 0;
    if (bell) {
        block = (int)env_number("GEMM_SPARSE_BLOCK", 128);
        if (block <= 0 || block % 16 != 0 || M % block != 0 || K % block != 0) {
            std::printf("blocked-ELL needs dimM and dimK to be multiples of the block (%d), a multiple of 16\n", block);
            return;
        }
        const int nbr = M / block, nbc = K / block;
        ell = std::max(1, std::min(nbc, (int)std::lround(nbc * env_number("GEMM_SPARSE_KEEP", 0.25))));
        h_bcols.resize((size_t)nbr * ell);
        GenerateUniformBlockedELLIndex(nbc, ell, nbr, h_bcols.data(), generator);
        h_val.resize((size_t)M * ell * block);
        MakeDenseMatrix<SType>(M, ell * block, h_val.data(), generator);
        // the same operand as rows of entries, for the CPU loop
        h_off.resize(M + 1);
        h_col.resize(h_val.size());
        for (int i = 0; i <= M; ++i) h_off[i] = i * ell * block;
        for (int i = 0; i < M; ++i)
            for (int t = 0; t < ell * block; ++t) h_col[(size_t)i * ell * block + t] = h_bcols[(size_t)(i / block) * ell + t / block] * block + t % block;
    } else {
        const double keep = env_number("GEMM_SPARSE_KEEP", 0.1);
        const int nonzeros = (int)std::max(1.0, std::min((double)M * K, keep * (double)M * K));
        const int padding = 4;
        h_val.resize((size_t)nonzeros + (size_t)M * (padding - 1));
        h_col.resize(h_val.size());
        h_off.resize(M + 1);
        const int64_t stored = MakeSparseMatrixRandomUniform<SType, int>(M, K, nonzeros, h_val.data(), h_off.data(), h_col.data(), generator, padding);
        h_val.resize(stored);
        h_col.resize(stored);
        h_order.resize(M);
        SortedRowSwizzle(M, h_off.data(), h_order.data());
    }
    std::vector<BType> h_B((size_t)N * K);
    MakeDenseMatrix<BType>(N, K, h_B.data(), generator);
    const size_t stored = h_val.size();
    std::printf("%s %s: S %d x %d with %zu stored entries (%.1f %%)%s, %d dense column%s\n", bell ? "blocked-ELL" : "CSR", vec ? "SpMV" : "SpMM", M, K,
                stored, 100.0 * stored / ((double)M * K), bell ? (" in blocks of " + std::to_string(block)).c_str() : "", N, N == 1 ? "" : "s");

    std::vector<float> h_ref;
    std::vector<double> h_scale;
    if (func) {
        h_ref.assign((size_t)M * N, 0.0f);
        h_scale.assign((size_t)M * N, 0.0);
        cpu_reference_spmm(M, K, N, h_val.data(), h_off.data(), h_col.data(), h_B.data(), h_ref.data(), h_scale.data());
    }
    SType *d_val;
    BType *d_B;
    float *d_C;
    int *d_off = nullptr, *d_col = nullptr, *d_bcols = nullptr, *d_order = nullptr;
    checkHip(hipMalloc(&d_val, stored * sizeof(SType)));
    checkHip(hipMalloc(&d_B, h_B.size() * sizeof(BType)));
    checkHip(hipMalloc(&d_C, (size_t)M * N * sizeof(float)));
    checkHip(hipMemcpy(d_val, h_val.data(), stored * sizeof(SType), hipMemcpyHostToDevice));
    checkHip(hipMemcpy(d_B, h_B.data(), h_B.size() * sizeof(BType), hipMemcpyHostToDevice));
    auto upload = [](const std::vector<int> &h, int **d) {
        checkHip(hipMalloc(d, h.size() * sizeof(int)));
        checkHip(hipMemcpy(*d, h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice));
    };
    if (bell) {
        upload(h_bcols, &d_bcols);
    } else {
        upload(h_off, &d_off);
        upload(h_col, &d_col);
        upload(h_order, &d_order);
    }
    const int fs = SType::format, fb = BType::format;
    auto launch = [&]() -> hipError_t {
        int code;
        if (kernel == 10) code = fp8gemm_spmm_bell(M, K, N, block, ell, d_val, fs, d_bcols, d_B, fb, d_C, nullptr);
        else if (kernel == 11) code = fp8gemm_spmv_bell(M, K, block, ell, d_val, fs, d_bcols, d_B, fb, d_C, nullptr);
        else if (kernel == 12) code = fp8gemm_spmm_csr(M, K, N, d_val, fs, d_off, d_col, d_B, fb, d_C, nullptr);
        else code = fp8gemm_spmv_csr(M, K, d_val, fs, d_off, d_col, d_order, d_B, fb, d_C, nullptr);
        return static_cast<hipError_t>(code);
    };
    hipEvent_t start, end;
    checkHip(hipEventCreate(&start));
    checkHip(hipEventCreate(&end));
    for (int i = 0; i < warmup; ++i) checkHip(launch());
    float batch_msec = 0.0f;
    checkHip(hipEventRecord(start));
    for (int i = 0; i < repeat; ++i) checkHip(launch());
    checkHip(hipEventRecord(end));
    checkHip(hipEventSynchronize(end));
    checkHip(hipEventElapsedTime(&batch_msec, start, end));
    const double usec = batch_msec / repeat * 1e3;
    const double flop = 2.0 * (double)stored * N;
    const double bytes = (double)stored * (bell ? 1.0 : 5.0) + (double)N * K + 4.0 * (double)M * N;
    const double gflops = flop / usec / 1e3, gbs = bytes / usec / 1e3;
    std::printf("batch of %d launches: %.3f us per launch, %.1f GFlops on the stored entries, %.1f GB/s (%.1f%% of %.0f)\n", repeat, usec,
                gflops, gbs, gbs / kPeakHbmGBs * 100.0, kPeakHbmGBs);
    if (record) record_csv(kernel, M, K, N, gflops, usec, gbs);
    if (func) {
        std::vector<float> h_C((size_t)M * N);
        checkHip(hipMemcpy(h_C.data(), d_C, h_C.size() * sizeof(float), hipMemcpyDeviceToHost));
        size_t num_errors = 0;
        double max_error = 0.0, worst_ratio = 0.0;
        for (size_t i = 0; i < h_C.size(); ++i) {
            const double err = std::fabs((double)h_C[i] - (double)h_ref[i]);
            // reordered fp32 sums over at most K terms, plus what the MFMA's groups of 8 products can drop (2^-13 of
            // eight times the largest product of a group, bounded by 2^-10 of the sum of magnitudes)
            const double tol = (2.0 * K * std::ldexp(1.0, -24) + std::ldexp(1.0, -10)) * h_scale[i];
            if (!(err <= tol)) ++num_errors;
            if (err > max_error) max_error = err;
            if (tol > 0 && err / tol > worst_ratio) worst_ratio = err / tol;
        }
        if (num_errors == 0)
            std::printf("Result Verified!\n");
        else
            std::cout << "There are " << num_errors << " errors." << std::endl;
        std::printf("MAx Error is %f\n", max_error);
        std::printf("worst |err| / tolerance = %.4g\n", worst_ratio);
    }
    checkHip(hipEventDestroy(start));
    checkHip(hipEventDestroy(end));
    checkHip(hipFree(d_val));
    checkHip(hipFree(d_B));
    checkHip(hipFree(d_C));
    for (int *p : {d_off, d_col, d_bcols, d_order})
        if (p) checkHip(hipFree(p));
    std::printf("end BmSparse\n");
}

// kernel 14: sampled dense-dense product, dimM x dimN outputs in column vectors of GEMM_SDDMM_VEC (8) rows, the
// fraction GEMM_SPARSE_KEEP (0.1) of the vectors stored, at uniformly drawn places
template <typename LType, typename RType>
static void BmSddmm(int M, int K, int N, bool func, bool record)
{
    const int vec = (int)env_number("GEMM_SDDMM_VEC", 8);
    if (vec <= 0 || M % vec != 0) {
        std::printf("SDDMM needs dimM to be a multiple of the vector length (%d)\n", vec);
        return;
    }
    const int m_vec = M / vec;
    std::default_random_engine generator;
    const double keep = env_number("GEMM_SPARSE_KEEP", 0.1);
    const int vectors = (int)std::max(1.0, std::min((double)m_vec * N, keep * (double)m_vec * N));
    std::vector<LType> unused(vectors);
    std::vector<int> h_off(m_vec + 1), h_col(vectors);
    const int64_t stored = MakeSparseMatrixRandomUniform<LType, int>(m_vec, N, vectors, unused.data(), h_off.data(), h_col.data(), generator, 0);
    std::vector<LType> h_L((size_t)M * K);
    std::vector<RType> h_R((size_t)N * K);
    MakeDenseMatrix<LType>(M, K, h_L.data(), generator);
    MakeDenseMatrix<RType>(N, K, h_R.data(), generator);
    std::printf("SDDMM: %d x %d outputs in vectors of %d, %lld vectors stored (%.1f %%), K = %d\n", M, N, vec, (long long)stored,
                100.0 * stored / ((double)m_vec * N), K);
    LType *d_L;
    RType *d_R;
    float *d_out;
    int *d_off, *d_col;
    checkHip(hipMalloc(&d_L, h_L.size()));
    checkHip(hipMalloc(&d_R, h_R.size()));
    checkHip(hipMalloc(&d_out, (size_t)stored * vec * sizeof(float)));
    checkHip(hipMalloc(&d_off, h_off.size() * sizeof(int)));
    checkHip(hipMalloc(&d_col, h_col.size() * sizeof(int)));
    checkHip(hipMemcpy(d_L, h_L.data(), h_L.size(), hipMemcpyHostToDevice));
    checkHip(hipMemcpy(d_R, h_R.data(), h_R.size(), hipMemcpyHostToDevice));
    checkHip(hipMemcpy(d_off, h_off.data(), h_off.size() * sizeof(int), hipMemcpyHostToDevice));
    checkHip(hipMemcpy(d_col, h_col.data(), h_col.size() * sizeof(int), hipMemcpyHostToDevice));
    auto launch = [&]() -> hipError_t {
        return static_cast<hipError_t>(fp8gemm_sddmm(m_vec, K, vec, d_off, d_col, d_L, LType::format, d_R, RType::format, d_out, nullptr));
    };
    hipEvent_t start, end;
    checkHip(hipEventCreate(&start));
    checkHip(hipEventCreate(&end));
    for (int i = 0; i < warmup; ++i) checkHip(launch());
    float batch_msec = 0.0f;
    checkHip(hipEventRecord(start));
    for (int i = 0; i < repeat; ++i) checkHip(launch());
    checkHip(hipEventRecord(end));
    checkHip(hipEventSynchronize(end));
    checkHip(hipEventElapsedTime(&batch_msec, start, end));
    const double usec = batch_msec / repeat * 1e3;
    const double gflops = 2.0 * (double)stored * vec * K / usec / 1e3;
    const double gbs = ((double)stored * K + (double)M * K + 4.0 * (double)stored * (vec + 1)) / usec / 1e3;
    std::printf("batch of %d launches: %.3f us per launch, %.1f GFlops on the stored outputs, %.1f GB/s of gathered rows and results\n", repeat,
                usec, gflops, gbs);
    if (record) record_csv(14, M, K, N, gflops, usec, gbs);
    if (func) {
        std::vector<float> h_out((size_t)stored * vec), h_ref((size_t)stored * vec);
        checkHip(hipMemcpy(h_out.data(), d_out, h_out.size() * sizeof(float), hipMemcpyDeviceToHost));
        Host_sddmm<LType, float>(m_vec, K, vec, h_off.data(), h_col.data(), h_L.data(), h_R.data(), h_ref.data());
        size_t num_errors = 0;
        double max_error = 0.0, worst_ratio = 0.0;
        for (int i = 0; i < m_vec; ++i)
            for (int j = h_off[i]; j < h_off[i + 1]; ++j)
                for (int v = 0; v < vec; ++v) {
                    double sabs = 0.0;
                    const LType *l = h_L.data() + ((size_t)i * vec + v) * K;
                    const RType *r = h_R.data() + (size_t)h_col[j] * K;
                    for (int t = 0; t < K; ++t) sabs += std::fabs((double)float(l[t]) * (double)float(r[t]));
                    const size_t at = (size_t)j * vec + v;
                    const double err = std::fabs((double)h_out[at] - (double)h_ref[at]);
                    const double tol = (2.0 * K * std::ldexp(1.0, -24) + std::ldexp(1.0, -10)) * sabs;
                    if (!(err <= tol)) ++num_errors;
                    if (err > max_error) max_error = err;
                    if (tol > 0 && err / tol > worst_ratio) worst_ratio = err / tol;
                }
        if (num_errors == 0)
            std::printf("Result Verified!\n");
        else
            std::cout << "There are " << num_errors << " errors." << std::endl;
        std::printf("MAx Error is %f\n", max_error);
        std::printf("worst |err| / tolerance = %.4g\n", worst_ratio);
    }
    checkHip(hipEventDestroy(start));
    checkHip(hipEventDestroy(end));
    checkHip(hipFree(d_L));
    checkHip(hipFree(d_R));
    checkHip(hipFree(d_out));
    checkHip(hipFree(d_off));
    checkHip(hipFree(d_col));
    std::printf("end BmSddmm\n");
}

static void usage(void)
{
    std::printf("!!!!!!!\n");
    std::printf("Input Help!\n");
    std::printf("Input Format is  ./gemm_main [dimM] [dimK] [dimN] [kernel] [verify] [reocrd] [testbench] [dist [seed]]\n");
    std::printf("dim: M-K-N in GEMM\n");
    std::printf("kernel: {1,2: e4m3*e4m3  3,4: e5m2*e5m2  5,6: e4m3*e5m2  7,8: e5m2*e4m3; odd = 2-stage, even = 4-stage; 0: CPU path only;\n");
    std::printf("         10: SpMM blocked-ELL  11: SpMV blocked-ELL  12: SpMM CSR  13: SpMV CSR  14: SDDMM}\n");
    std::printf("verify: {0 not verify result with cpu, 1: verify result}\n");
    std::printf("record: {record in csv files}\n");
    std::printf("testbench: {1: sweep square sizes 256..16384}\n");
    std::printf("dist: {reference, uniform, normal, normal4, weights, loguniform}  seed: integer\n");
    std::printf("!!!!!!!\n");
    std::exit(1);
}

static bool run_kernel(int kernel, int M, int K, int N, bool verify, bool record, const Options &opt)
{
    switch (kernel) {
    case 0:
        BmCPU<e4m3, e4m3>(M, K, N, opt);
        return true;
    case 1: case 2:
        std::printf("e4m3 * e4m3 = fp32\n");
        BmFN<e4m3, e4m3, float>(M, K, N, kernel, verify, record, opt);
        return true;
    case 3: case 4:
        std::printf("e5m2 * e5m2 = fp32\n");
        BmFN<e5m2, e5m2, float>(M, K, N, kernel, verify, record, opt);
        return true;
    case 5: case 6:
        std::printf("e4m3 * e5m2 = fp32\n");
        BmFN<e4m3, e5m2, float>(M, K, N, kernel, verify, record, opt);
        return true;
    case 7: case 8:
        std::printf("e5m2 * e4m3 = fp32\n");
        BmFN<e5m2, e4m3, float>(M, K, N, kernel, verify, record, opt);
        return true;
    case 10: case 11: case 12: case 13:
        std::printf("sparse e4m3 * e4m3 = fp32\n");
        BmSparse<e4m3, e4m3>(M, K, N, kernel, verify, record);
        return true;
    case 14:
        std::printf("sampled e4m3 * e4m3 = fp32\n");
        BmSddmm<e4m3, e4m3>(M, K, N, verify, record);
        return true;
    default:
        std::printf("unsupported kernel\n");
        return false;
    }
}

int main(int argc, char **argv)
{
    if (argc < 8 || argc > 10 || std::strcmp(argv[1], "-h") == 0 || std::strcmp(argv[1], "--help") == 0) usage();
    int dimM = std::atoi(argv[1]);   // A_rows_num
    int dimK = std::atoi(argv[2]);   // A_cols_num = B_cols_num (B is stored N x K)
    int dimN = std::atoi(argv[3]);   // B_rows_num
    const int kernel = std::atoi(argv[4]);
    const int verify = std::atoi(argv[5]);
    const int record = std::atoi(argv[6]);
    const int testbench = std::atoi(argv[7]);
    Options opt;
    if (argc > 8) opt.dist = argv[8];
    if (argc > 9) opt.seed = std::strtoull(argv[9], nullptr, 0);
    if (dimM <= 0 || dimK <= 0 || dimN <= 0) usage();

    if (testbench == 0) {
        run_kernel(kernel, dimM, dimK, dimN, verify, record, opt);
    } else {
        // the reference walks 64 sizes; GEMM_TESTBENCH_SIZES shortens the walk (for tests)
        int test_num = 64;
        if (const char *env = std::getenv("GEMM_TESTBENCH_SIZES")) test_num = std::max(1, std::min(64, std::atoi(env)));
        for (int i = 0; i < test_num; ++i) {
            const int dim = 256 * (i + 1);
            if (!run_kernel(kernel, dim, dim, dim, verify, record, opt)) break;
        }
    }
    return 0;
}
