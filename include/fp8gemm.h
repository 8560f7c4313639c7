/*
 * fp8gemm.h -- C ABI of the MI355X (gfx950) FP8 GEMM library.
 *
 * Every entry point computes, on the current HIP device,
 *
 *     out[i*n + j] = sum_{t<k} float(a[i*k + t]) * float(b[j*k + t])
 *
 * with A row-major m x k, B stored n x k ("row-col"), C row-major m x n fp32,
 * fp32 accumulation, pure overwrite (C is never read; no alpha/beta/scales).
 * a, b, out are caller-owned DEVICE pointers that must not alias.  Launches
 * are asynchronous on the given HIP stream (NULL = the default stream).
 * Return value: a hipError_t as int, 0 (hipSuccess) on success,
 * 1 (hipErrorInvalidValue) for null pointers, non-positive dimensions, bad
 * format / stage / algorithm codes.  Any m, k, n >= 1 is computed in full
 * (the reference silently leaves tiles past the last multiple of 128 unwritten,
 * GEMM/src/gemm.cu:45-47; this library does not).
 *
 * Format codes: 0 = OCP E4M3 (bias 7, max 448, no Inf), 1 = OCP E5M2.
 */
#ifndef FP8GEMM_H
#define FP8GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FP8GEMM_E4M3 0
#define FP8GEMM_E5M2 1

/* Kernel families, for fp8gemm_launch_algo (testing / tuning hook). */
#define FP8GEMM_ALGO_AUTO 0    /* shape-based choice, what every other entry uses */
#define FP8GEMM_ALGO_DIRECT 1  /* one wave per 32x32 tile, global->register, any shape */
#define FP8GEMM_ALGO_TILE 2    /* LDS-tiled MFMA kernel for compute-bound shapes */
#define FP8GEMM_ALGO_SKINNY 3  /* B-streaming kernel for small m (HBM-bound) */

/*
 * The eight per-precision launch entry points.  Each replaces one C++ overload
 * of the reference's launch API (GEMM/include/gemm.cuh), argument order
 * (m, k, n, a, b, out) as there, default stream as there
 * (GEMM/src/gemm.cu:263-285).  "stage2" backs gemm::GEMM, "stage4" backs
 * gemm::GEMM4.  Both run the same plan and the same kernels, as the reference's
 * GEMM4 runs the kernel of GEMM (GEMM/src/gemm.cu:687-694): the depth of the LDS
 * ring (2 to 5 slots) belongs to the tile shape that the planner picks for the
 * problem, not to the entry point.
 */
int fp8gemm_e4m3_e4m3_stage2(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:12-15 */
int fp8gemm_e4m3_e4m3_stage4(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:18-21 */
int fp8gemm_e5m2_e5m2_stage2(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:24-27 */
int fp8gemm_e5m2_e5m2_stage4(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:30-33 */
int fp8gemm_e4m3_e5m2_stage2(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:36-39 */
int fp8gemm_e4m3_e5m2_stage4(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:41-44 */
int fp8gemm_e5m2_e4m3_stage2(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:47-50 */
int fp8gemm_e5m2_e4m3_stage4(int m, int k, int n, const void *a, const void *b, float *out); /* gemm.cuh:52-55 */

/*
 * Generic form of the above (the launchers GEMMex / GEMMex4 of
 * GEMM/src/gemm.cu:263-277, 670-686 folded into one): formats and stage count
 * as arguments, explicit stream (a hipStream_t passed as void*).
 * stages must be 2 or 4.
 */
int fp8gemm_launch(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                   float *out, int stages, void *stream);

/*
 * Matrix-vector product y = W x: W stored n x k row-major (the layout of B above), x of k
 * codes, y of n floats.  The GEMV that the reference's roadmap names next to GEMM
 * (README.md:7 there; it holds no GEMV code to match).  It is fp8gemm_launch with m = 1:
 * the single-wave streaming kernel reads every byte of W once (k % 128 == 0 and n % 16 == 0;
 * any other shape runs on the tiled or the general kernel).
 */
int fp8gemm_gemv(int n, int k, const void *w, int w_fmt, const void *x, int x_fmt, float *y, void *stream);

/*
 * ---- Sparse operands: SpMM, SpMV and SDDMM ---------------------------------------------
 * out = S * B^T with S (m x k) sparse and B dense, stored n x k like the B of the GEMM; out is
 * m x n fp32 row-major, overwritten; n = 1 with a vector x of k codes is the SpMV.  The
 * reference names SpMM and SpMV as planned kernels (README.md:7) and holds none; what it holds
 * are the host helpers that generate the two operand formats taken here
 * (GEMM/include/bm_test_utils.h:48-68 blocked-ELL column lists, :71-128 compressed sparse rows
 * with optional row padding, :197-216 row orders).  Every stored entry contributes
 * float(value) * float(b[j][column]) to out[i][j], fp32 accumulation; all pointers are device
 * pointers; formats as for the GEMM; launches are asynchronous on `stream`.  The matrix-vector
 * products and fp8gemm_sddmm allocate nothing; fp8gemm_spmm_bell and fp8gemm_spmm_csr take scratch
 * from the stream's pool like fp8gemm_launch (so a call that is captured into a HIP graph must have
 * been made once on that stream before).
 *
 * Blocked-ELL: square blocks of `block` x `block` elements (block % 16 == 0, m % block == 0,
 * k % block == 0); every block row stores ell_cols blocks.  values: m x (ell_cols * block)
 * codes row-major, 16-byte aligned (stored block t of a row's block row occupies bytes
 * t * block .. of the row); block_cols: (m / block) x ell_cols ints, the block column of each
 * stored block, or -1 for a padding block that contributes nothing.  The kernels feed the MFMA
 * from the stored blocks directly; blocks that are not stored cost nothing.  Blocks of 32 rows and
 * multiples run on the LDS-tiled kernel of the GEMM (n >= 64), other sizes on a kernel without
 * LDS.  b 16-byte aligned.
 */
int fp8gemm_spmm_bell(int m, int k, int n, int block, int ell_cols, const void *values, int s_fmt, const int *block_cols,
                      const void *b, int b_fmt, float *out, void *stream);
int fp8gemm_spmv_bell(int m, int k, int block, int ell_cols, const void *values, int s_fmt, const int *block_cols,
                      const void *x, int x_fmt, float *y, void *stream);
/*
 * Compressed sparse rows: values (codes), row_offsets (m + 1 ints, ascending from 0), col_idx
 * (ints in [0, k)).  fp8gemm_spmv_csr streams values and indices once, one wave per row, rows
 * taken in the order row_order gives (m ints, a permutation of 0 .. m-1, e.g. longest rows
 * first, see fp8gemm_sorted_row_swizzle; NULL = 0, 1, 2, ..); entries of a row that name the same
 * column are added.  fp8gemm_spmm_csr writes S out as a dense m x k fp8 matrix in the stream's
 * scratch (fp8gemm_spmm_csr_scratch_bytes tells how much it takes from the per-stream pool
 * described under "Device scratch") and runs the dense GEMM on it: no matrix instruction takes
 * single elements, and with B stored n x k an element-wise kernel would gather single bytes.
 * For this one the columns of a row must be distinct, except that entries whose value is +-0
 * may repeat a column (the zero padding of the reference's generator does) and are skipped.
 */
int fp8gemm_spmv_csr(int m, int k, const void *values, int s_fmt, const int *row_offsets, const int *col_idx,
                     const int *row_order, const void *x, int x_fmt, float *y, void *stream);
int fp8gemm_spmm_csr(int m, int k, int n, const void *values, int s_fmt, const int *row_offsets, const int *col_idx,
                     const void *b, int b_fmt, float *out, void *stream);
size_t fp8gemm_spmm_csr_scratch_bytes(int m, int k, int n);
/*
 * Sampled dense-dense product with a vector-sparse output pattern, the loop of the reference's host
 * helper Host_sddmm (GEMM/include/bm_test_utils.h:172-194):
 *     out[j * vec_length + v] = sum_l float(lhs[(i * vec_length + v) * k + l]) * float(rhs[col_idx[j] * k + l])
 * for every vector row i < m_vec, every stored entry j in [row_offsets[i], row_offsets[i+1]) and every
 * v < vec_length.  lhs: (m_vec * vec_length) x k, rhs: n x k, both row-major codes (col_idx < n); out:
 * row_offsets[m_vec] x vec_length floats.  All device pointers.  vec_length <= 16 with k % 16 == 0 and
 * 16-byte aligned operands runs on the MFMA; anything else one thread per output.
 */
int fp8gemm_sddmm(int m_vec, int k, int vec_length, const int *row_offsets, const int *col_idx, const void *lhs, int l_fmt,
                  const void *rhs, int r_fmt, float *out, void *stream);
/*
 * Host helper: rows ordered by falling number of stored entries (ties in rising row number),
 * the order of the reference's SortedRowSwizzle (GEMM/include/bm_test_utils.h:202-216).
 * row_offsets and row_indices are HOST arrays of m + 1 and m ints.
 */
void fp8gemm_sorted_row_swizzle(int m, const int *row_offsets, int *row_indices);

/*
 * Extended epilogue, with no counterpart in the reference's gemm:: API; it covers what the
 * reference's vendor-library sample hands to cuBLASLt next to the operands
 * (GEMM/src/cublas.cu:9-23, 41-46; GEMM/include/helper.h:84, 125, 159-160: host alpha and
 * beta, device pointers to per-tensor scales of A, B, C and D, a device pointer that receives
 * the largest magnitude of the output) and 16-bit matrices:
 *
 *     y[i*n+j] = alpha * a_scale * b_scale * sum_t a[i*k+t] * b[j*k+t]  +  beta * c_scale * c[i*n+j]
 *     *amax_d  = max_ij |y[i*n+j]|                      (before d_scale; NaNs do not enter)
 *     d[i*n+j] = cast_d_type( d_scale * y[i*n+j] )      (one rounding to nearest even)
 *
 * The sum is accumulated in fp32 as in fp8gemm_launch and all epilogue arithmetic is fp32.
 * d_type / c_type: FP8GEMM_OUT_F32 (float), FP8GEMM_OUT_BF16, FP8GEMM_OUT_F16 (2-byte
 * elements).  a_scale, b_scale, c_scale, d_scale: device pointers to one float each, read by
 * the kernel when it runs, or NULL for 1.  c: device matrix m x n row-major of c_type, or NULL
 * (then beta and c_scale are ignored and nothing is read); c may be d itself when both have
 * the same type (in place).  amax_d: device pointer to one float that the call overwrites, or
 * NULL.  fp8gemm_launch_ex is the subset without c, d_scale and amax_d.
 */
#define FP8GEMM_OUT_F32 0
#define FP8GEMM_OUT_BF16 1
#define FP8GEMM_OUT_F16 2
int fp8gemm_launch_epilogue(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                            void *d, int d_type, float alpha, float beta, const void *c, int c_type,
                            const float *a_scale, const float *b_scale, const float *c_scale, const float *d_scale,
                            float *amax_d, void *stream);
int fp8gemm_launch_ex(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                      void *out, int out_type, float alpha, const float *a_scale, const float *b_scale,
                      void *stream);

/*
 * fp8gemm_launch for callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
 * (whose kernels need no scratch).  The partial sums of K slices go to a static device
 * array of FP8GEMM_NOALLOC_SCRATCH_BYTES bytes that is part of the library's code object
 * (every GPU the library runs on holds its own copy until the process ends); the call
 * allocates and frees nothing.  A shape whose plan needs more scratch than the array holds
 * (see fp8gemm_scratch_bytes) is refused with hipErrorOutOfMemory (2) before anything is
 * launched.  All calls on one GPU share that GPU's array: calls on one stream are ordered by
 * the stream, calls that overlap on different streams of one GPU race on it and must be
 * ordered by the caller.  The first 16 KiB of the array are the arrival counters of the K
 * slices: they must be zero when a kernel starts, they are (static storage starts as zeros),
 * and the slice that arrives last puts its tile's counter back to zero, so every kernel
 * leaves them as it found them; nothing else in the array has to start at any value
 * (every slot a call reads has been written by that call).
 */
#define FP8GEMM_NOALLOC_SCRATCH_BYTES ((size_t)64 << 20)
int fp8gemm_launch_noalloc(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                           float *out, int stages, void *stream);

/*
 * ---- Internal: testing and tuning hooks --------------------------------------------
 * fp8gemm_launch_algo, fp8gemm_launch_tuned, fp8gemm_num_variants, fp8gemm_plan and
 * fp8gemm_tile_order expose the kernel families, their compiled variants and the planner
 * to the test suite and the tuning sweeps.  They are not part of the drop-in surface:
 * variant numbers, plan encodings and the set of variants change between versions.
 */
/* As fp8gemm_launch, but forces one kernel family (FP8GEMM_ALGO_*).  Returns
 * hipErrorInvalidValue when the family cannot run the shape. */
int fp8gemm_launch_algo(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                        float *out, int stages, int algo, void *stream);

/*
 * Internal tuning hook with no counterpart in the reference: forces a kernel family
 * and one of its compiled shape variants (0 .. fp8gemm_num_variants(algo)-1,
 * -1 = the default for the shape).  For FP8GEMM_ALGO_SKINNY, variant may add
 * 16 * columns-per-wave/16 to override the planned column count per wave; for
 * FP8GEMM_ALGO_TILE it may add 32 * (1 + r) to force the K-walk rotation mode
 * r (0 none, 1 per tile column, 2 per XCD and round).  split_k > 0 overrides
 * the planned number of K slices (skinny kernel and persistent tiled kernels);
 * split_k < 0 (tiled kernels only) cuts only the tiles that do not fill a
 * round of 256 into -split_k slices; a forced tile variant runs unsplit unless
 * split_k says otherwise.
 */
int fp8gemm_launch_tuned(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                         float *out, int algo, int variant, int split_k, void *stream);
int fp8gemm_num_variants(int algo);

/* Which family FP8GEMM_ALGO_AUTO picks for a shape (pure host logic). */
int fp8gemm_select_algo(int m, int k, int n);

/* What fp8gemm_launch would run for a shape with 16-byte aligned operands (pure
 * host logic): plan[0] = family (FP8GEMM_ALGO_*), plan[1] = compiled shape variant
 * of that family, plan[2] = number of K slices (1 = none, no scratch), plan[3] =
 * columns of C per wave (skinny family) or, for the tiled family, the K-walk
 * rotation mode, plus 16 when only the tiles that do not fill a round are cut.
 * Returns 0, or hipErrorInvalidValue for bad arguments. */
int fp8gemm_plan(int m, int k, int n, int stages, int plan[4]);

/*
 * Order in which the persistent tiled kernel walks the bm x bn tiles of C for a
 * shape (pure host logic, for tests): tile number `index` (0 .. tiles-1) ->
 * its tile row and tile column.  256 consecutive numbers run at the same time,
 * 32 consecutive ones on one XCD.  No counterpart in the reference, whose
 * kernels take the tile from blockIdx (GEMM/src/gemm.cu:39-44).
 */
int fp8gemm_tile_order(int m, int k, int n, int bm, int bn, int index, int *tile_row, int *tile_col);

/*
 * Device scratch.  A shape whose plan cuts K into slices needs device memory for the
 * slices' partial sums; fp8gemm_scratch_bytes tells how much (0 when the shape needs
 * none: 8192^3, M=16 N=28672 K=8192, ...; the same for both stage counts, which run the same
 * plan; it includes 16 KiB of arrival counters ahead of the sums).
 * With the library's own scratch the slices of tiles up to 128 x 128 are added up inside the
 * GEMM kernel, by the slice of a tile that arrives last (the counters start at zero and
 * every kernel leaves them at zero); larger tiles, and every shape run on a caller's
 * workspace, whose contents the library cannot vouch for, are added up by a second kernel.
 * Both add in slice order: the results are the same bit for bit.  The scratch is the only
 * device memory the library ever allocates.  The reference's launchers are stateless and re-entrant
 * (GEMM/src/gemm.cu:263-277); to keep that contract the scratch is held per (device,
 * stream): calls on one stream are ordered by the stream, calls on different streams
 * never share a buffer and may overlap freely, from one host thread or several.  A
 * stream's buffer is allocated on its first K-sliced call (hipMalloc), reused by later
 * calls, and replaced by a larger one when a shape needs more; the smaller buffer is kept
 * and handed to another stream once the work queued on it has finished.  No call waits
 * for the device and none frees memory.  fp8gemm_release_scratch synchronises the current
 * device and frees everything held for it; fp8gemm_scratch_held_bytes reports what is held.
 * hipMalloc is illegal while a stream is being captured into a graph: capture only shapes
 * that need no scratch or whose stream already owns a large enough buffer, or call
 * fp8gemm_launch_ws.
 */
size_t fp8gemm_scratch_bytes(int m, int k, int n);
int fp8gemm_release_scratch(void);
size_t fp8gemm_scratch_held_bytes(void);

/*
 * fp8gemm_launch with the scratch supplied by the caller: `workspace` is device memory of
 * `workspace_bytes` bytes, 16-byte aligned, that the call's kernels may overwrite and that
 * must stay untouched until they have run (NULL / 0 for shapes that need none).  Returns
 * hipErrorOutOfMemory (2) without launching anything when the shape needs more than
 * workspace_bytes (see fp8gemm_scratch_bytes).  The library allocates nothing in this call.
 * No counterpart in the reference, whose kernels need no workspace.
 */
int fp8gemm_launch_ws(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                      float *out, int stages, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The current device against what the plans are laid out for (MI355X as one partition: 256 CUs
 * in 8 XCDs): info[0] = CUs of the device, info[1] = CUs the plans assume, info[2] = 1 on gfx950,
 * info[3] = 1 when both match.  On any other layout the results are unchanged, only the plans
 * are not tuned for it.  Returns 0 or a HIP error.
 */
int fp8gemm_device_info(int info[4]);

/* Text for a return code (hipGetErrorString). */
const char *fp8gemm_error_string(int code);

/* Library version, major*100 + minor. */
int fp8gemm_version(void);

/*
 * Host-side fp8 codec (bit-exact OCP conversions; the arithmetic the
 * reference gets from the converting constructor / operator float of its fp8
 * types, GEMM/include/bm_test_utils.h:139 and GEMM/gemm_main.cpp:48).
 */
uint8_t fp8gemm_encode_one(float x, int fmt);
float fp8gemm_decode_one(uint8_t code, int fmt);
void fp8gemm_encode(const float *src, uint8_t *dst, size_t count, int fmt);
void fp8gemm_decode(const uint8_t *src, float *dst, size_t count, int fmt);

/*
 * Seeded synthetic matrices written straight to fp8 codes in HOST memory (the
 * role of MakeDenseMatrix, GEMM/include/bm_test_utils.h:131-143).  All are
 * counter-based (element i depends only on seed and i), so results do not
 * depend on thread count.
 *   uniform    : U(lo, hi)
 *   normal     : mean + sigma * N(0,1)
 *   weights    : sigma * N(0,1), then scaled so the largest magnitude maps to
 *                the format's largest finite value (per-tensor scaling)
 *   loguniform : +-2^u, u uniform over the format's whole finite exponent
 *                range (subnormals included), never NaN/Inf
 */
void fp8gemm_fill_uniform(uint8_t *dst, size_t count, int fmt, uint64_t seed, float lo, float hi);
void fp8gemm_fill_normal(uint8_t *dst, size_t count, int fmt, uint64_t seed, float mean, float sigma);
void fp8gemm_fill_weights(uint8_t *dst, size_t count, int fmt, uint64_t seed, float sigma);
void fp8gemm_fill_loguniform(uint8_t *dst, size_t count, int fmt, uint64_t seed);

#ifdef __cplusplus
}
#endif

#endif /* FP8GEMM_H */
