// Sparse-times-dense kernels: out = S * B^T with S (m x k) sparse and B dense, stored n x k
// like the B of the GEMM; n = 1 is the sparse matrix-vector product.
//
// Two operand formats, the two that the reference's host helpers generate:
//   * blocked-ELL (GEMM/include/bm_test_utils.h:48-68): square blocks of `block` x `block`,
//     every block row stores ell_cols blocks; values m x (ell_cols * block) fp8 row-major,
//     block_cols (m / block) x ell_cols block column numbers, -1 = padding.  Seen from a row of
//     S this is a dense row of K_ell = ell_cols * block bytes whose 16-byte pieces pair with
//     16-byte pieces of B's rows at gathered positions: exactly what an MFMA wants, because a
//     dot product does not care where in K its bytes come from as long as both operands agree.
//     spmm_bell_kernel feeds v_mfma_f32_16x16x128_f8f6f4 straight from global memory.
//   * compressed sparse rows (bm_test_utils.h:71-128): single elements.  No matrix instruction
//     takes those; the matrix-vector product streams values and indices once (spmv_csr_kernel,
//     HBM-bound), the matrix-matrix product scatters S into a dense fp8 matrix
//     (csr_densify_kernel) that the dense GEMM then multiplies: with B stored n x k, an
//     element-wise kernel would gather single bytes of B at stride k, m * n * nnz_row of them.
#ifndef FP8GEMM_KERNEL_SPARSE_H
#define FP8GEMM_KERNEL_SPARSE_H

#include "device_common.h"

// fp8 code -> float, by the bits (exact; subnormals, infinities and NaNs included)
template <int F>
__device__ __forceinline__ float fp8_to_float(uint32_t code)
{
    if (F == 1) {      // E5M2 is the upper byte of an IEEE half
        return (float)__builtin_bit_cast(_Float16, (unsigned short)(code << 8));
    }
    const uint32_t sign = (code & 0x80u) << 24;
    const uint32_t e = (code >> 3) & 0xFu, mant = code & 7u;
    if ((code & 0x7Fu) == 0x7Fu) return __builtin_bit_cast(float, sign | 0x7FC00000u);
    if (e == 0) return __builtin_bit_cast(float, sign | __builtin_bit_cast(uint32_t, (float)mant * 0.001953125f));   // mant * 2^-9
    return __builtin_bit_cast(float, sign | ((e + 120u) << 23) | (mant << 20));
}

__device__ __forceinline__ v4i load_piece(const uint8_t *p)
{
    return *reinterpret_cast<const v4i *>(p);
}

// One wave per 16 rows of S and 16 * TN columns of out.  A K step is 128 bytes of the rows'
// stored values = 8 pieces of 16 bytes; lane (i = lane % 16, q = lane / 16) supplies pieces
// 2q and 2q + 1 of row i of S, and of rows i, 16 + i, .. of B the 16 bytes at the positions
// those pieces stand for: piece at byte p of the stored row lies in stored block p / block,
// whose block column c puts it at byte c * block + p % block of a row of B.  A padding block
// (c < 0) and pieces past the end of the stored row count as zeros.  The loads of the next K
// step are issued before the MFMAs of the current one.
// Requirements checked by the host: block % 16 == 0, m % block == 0, k % block == 0,
// 16-byte aligned values and b.
template <int SF, int BF, int TN>
__global__ __launch_bounds__(64) void spmm_bell_kernel(int m, int k, int n, int block, int ell_cols,
                                                       const uint8_t *__restrict__ values,
                                                       const int *__restrict__ block_cols,
                                                       const uint8_t *__restrict__ B,
                                                       float *__restrict__ out, int groups_n)
{
    const int lane = threadIdx.x;
    const int i = lane & 15, q = lane >> 4;
    const int gm = blockIdx.x / groups_n, gn = blockIdx.x - gm * groups_n;
    const int row0 = gm * 16, n0 = gn * 16 * TN;
    const int kell = ell_cols * block;
    const int steps = (kell + 127) / 128;
    const int *cols = block_cols + (size_t)(row0 / block) * ell_cols;
    const uint8_t *srow = values + (size_t)(row0 + i) * kell;
    const uint8_t *brow[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        int r = n0 + j * 16 + i;
        r = r < n ? r : n - 1;
        brow[j] = B + (size_t)r * k;
    }

    struct Step {
        v4i a[2], b[TN][2];
    };
    auto fetch = [&](int s, Step &f) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int p = s * 128 + (2 * q + h) * 16;
            int pos = -1;
            if (p < kell) {
                const int blk = p / block;
                const int c = cols[blk];
                if (c >= 0) pos = c * block + (p - blk * block);
            }
            const v4i zero = {0, 0, 0, 0};
            f.a[h] = pos >= 0 ? load_piece(srow + p) : zero;
            const int bp = pos >= 0 ? pos : 0;
#pragma unroll
            for (int j = 0; j < TN; ++j) f.b[j][h] = load_piece(brow[j] + bp);
        }
    };

    v4f acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    Step cur, nxt;
    fetch(0, cur);
    for (int s = 0; s < steps; ++s) {
        if (s + 1 < steps) fetch(s + 1, nxt);
        const v8i a8 = pack8(cur.a[0], cur.a[1]);
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[j] = mfma_16x16x128<SF, BF>(a8, pack8(cur.b[j][0], cur.b[j][1]), acc[j]);
        cur = nxt;
    }
    // register r of lane (i, q) holds out[row0 + 4q + r][n0 + 16j + i]
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = n0 + j * 16 + i;
        if (col < n) {
#pragma unroll
            for (int r = 0; r < 4; ++r) out[(size_t)(row0 + 4 * q + r) * n + col] = acc[j][r];
        }
    }
}

// y[row] = sum over the stored entries of the row of float(values[e]) * float(x[col[e]]):
// one wave per row, in the order row_order gives (null: 0, 1, 2, ..; the reference's
// SortedRowSwizzle, bm_test_utils.h:202-216, puts the longest rows first so that they start
// first).  Lane l takes entries l, l + 64, .. of the row; the 64 running sums are folded by a
// butterfly.  Values and indices are read once, coalesced; x is gathered through the caches.
template <int SF, int XF>
__global__ __launch_bounds__(256) void spmv_csr_kernel(int m, const uint8_t *__restrict__ values,
                                                        const int *__restrict__ row_offsets,
                                                        const int *__restrict__ col,
                                                        const int *__restrict__ row_order,
                                                        const uint8_t *__restrict__ x, float *__restrict__ y)
{
    const int lane = threadIdx.x & 63;
    const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (w >= m) return;
    const int row = row_order ? row_order[w] : w;
    const int e0 = row_offsets[row], e1 = row_offsets[row + 1];
    float acc = 0.0f;
    for (int e = e0 + lane; e < e1; e += 64) acc += fp8_to_float<SF>(values[e]) * fp8_to_float<XF>(x[col[e]]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) y[row] = acc;
}

// dense[0 .. count16) = 0, 16 bytes per thread
__global__ __launch_bounds__(256) void zero_bytes16_kernel(v4i *__restrict__ dense, size_t count16)
{
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t < count16) dense[t] = v4i{0, 0, 0, 0};
}

// dense[row][col[e]] = values[e] for the stored entries of S, one wave per row; `dense` (m x ld
// bytes, ld >= k) holds zeros.  Entries whose value is +-0 are left out: they change no sum, and
// the zero-valued padding entries that the reference's generator appends to a row repeat the
// column of the row's last real entry (bm_test_utils.h:106-118), which they must not overwrite.
__global__ __launch_bounds__(256) void csr_densify_kernel(int m, size_t ld, const uint8_t *__restrict__ values,
                                                           const int *__restrict__ row_offsets,
                                                           const int *__restrict__ col, uint8_t *__restrict__ dense)
{
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= m) return;
    const int e1 = row_offsets[row + 1];
    for (int e = row_offsets[row] + lane; e < e1; e += 64) {
        const uint8_t v = values[e];
        if ((v & 0x7F) != 0) dense[(size_t)row * ld + col[e]] = v;
    }
}

#endif  // FP8GEMM_KERNEL_SPARSE_H
