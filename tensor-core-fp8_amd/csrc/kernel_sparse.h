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
// Also here: the sampled dense-dense product (sddmm_kernel), whose output is sparse instead.
#ifndef FP8GEMM_KERNEL_SPARSE_H
#define FP8GEMM_KERNEL_SPARSE_H

#include "device_common.h"

// fp8 code (the lowest byte of `code`) -> float through the conversion instructions, which on gfx950
// take the OCP formats: exact for every code, subnormals, infinities and NaNs included (held to that by
// the one-hot tests: a row with a single 1.0 must return the other operand's decoded value bit for bit).
template <int F>
__device__ __forceinline__ float fp8_to_float(uint32_t code)
{
    return F == 1 ? __builtin_amdgcn_cvt_f32_bf8((int)code, 0) : __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
}

// the four codes of a 32-bit word
template <int F>
__device__ __forceinline__ void fp8x4_to_float(uint32_t w, float out[4])
{
    if (F == 1) {
        out[0] = __builtin_amdgcn_cvt_f32_bf8((int)w, 0);
        out[1] = __builtin_amdgcn_cvt_f32_bf8((int)w, 1);
        out[2] = __builtin_amdgcn_cvt_f32_bf8((int)w, 2);
        out[3] = __builtin_amdgcn_cvt_f32_bf8((int)w, 3);
    } else {
        out[0] = __builtin_amdgcn_cvt_f32_fp8((int)w, 0);
        out[1] = __builtin_amdgcn_cvt_f32_fp8((int)w, 1);
        out[2] = __builtin_amdgcn_cvt_f32_fp8((int)w, 2);
        out[3] = __builtin_amdgcn_cvt_f32_fp8((int)w, 3);
    }
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

// Matrix-vector product with S in blocked-ELL form, x (k codes, k <= kSpmvLdsBytes) held in LDS.
// Bound by reading the stored values once, so the loads take whole lines: one load instruction of a wave
// takes 1024 contiguous bytes of stored rows (a "slot"), 16 bytes a lane.  (A lane layout that gives each of
// the MFMA's 16 rows to another row of S, as spmm_bell_kernel has it, loads a quarter of a 128-byte line of
// each of 16 rows per instruction, and the memory pipeline then carries every line in two requests:
// measured 24 us against 13.5 us for 59 MB.)  Piece number 4i + q of the slot goes to lane
// (i = lane % 16, q = lane / 16), so the four lanes that make up row i of the MFMA's first operand hold 64
// consecutive bytes, and R lanes (a power of two, 4..64; 64 for stored rows of 1024 bytes and more) cover
// one stored row.  The second operand is, lane for lane, the 16 bytes of x that the lane's piece of S
// multiplies (from LDS).  The MFMA then computes a 16 x 16 matrix of which only the diagonal is wanted:
// element (i, i) is the dot product of the 64-byte run i of the slot with its x, and the other 240 are cross
// terms nobody reads (the matrix unit has the time).  Two slots of the same row feed one MFMA; rows shorter
// than a slot leave the second half zero.  At a row's end the diagonal is taken out (register i % 4 of lane
// (i, i / 4)), added over q and over the R / 4 runs of a row, and stored.
// Two ways of handing out the work, chosen by the host (`ksplit`):
//   1: a wave handles the 64 / R rows of a "row item" at a time (wave w of all takes items w, w + waves, ..)
//      and keeps the loads of two MFMA steps in flight across row boundaries (deeper rings measured no
//      faster: what counts is how many waves are resident, so the host launches as many workgroups as the
//      chip holds at once);
//   2 or 4: few rows -- that many waves of a workgroup share an item, wave u of them taking MFMA steps u,
//      u + ksplit, ..; their sums meet in LDS and are added in the order of u.  One pass: the grid covers
//      every item.
constexpr int kSpmvLdsBytes = 60 * 1024;       // with the room for the sums: the 64 KiB of LDS a kernel gets without asking
constexpr int kSpmvSumBytes = 4 * 16 * 4;      // 16 sums per wave

template <int SF, int XF, int ksplit>
__global__ __launch_bounds__(256) void spmv_bell_kernel(int m, int k, int block, int block_shift, int ell_cols, int lanes_per_row,
                                                         const uint8_t *__restrict__ values,
                                                         const int *__restrict__ block_cols,
                                                         const uint8_t *__restrict__ x, float *__restrict__ y)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_x[];      // x, then kSpmvSumBytes for the waves' sums
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const int lp = 4 * i + q;                                            // the lane's piece of a slot
    const int R = lanes_per_row, rows_per_item = 64 / R, G = R / 4;      // G: 64-byte runs per row and slot
    const int kell = ell_cols * block;
    const int U = (kell + 16 * R - 1) / (16 * R);                        // slots per row (1 when R < 64)
    const int NM = (U + 1) / 2;                                          // MFMA steps per row item
    const int items = (m + rows_per_item - 1) / rows_per_item;
    const int sub = wave % ksplit;                                       // which share of an item's MFMA steps
    const int per_wg = 4 / ksplit;                                       // items a workgroup has at a time
    const int waves = gridDim.x * per_wg, w = blockIdx.x * per_wg + wave / ksplit;
    const int mine = w < items ? (items - w + waves - 1) / waves : 0;    // row items of this wave (ksplit > 1: at most 1)
    const int share = NM > sub ? (NM - sub + ksplit - 1) / ksplit : 0;   // MFMA steps sub, sub + ksplit, .. of an item
    const int total = mine * share;                                      // MFMA steps of this wave
    const int per_item = share > 0 ? share : 1;
    const int sub_row = lp / R, in_row = lp - sub_row * R;
    const v4i zero = {0, 0, 0, 0};

    struct Step {
        v4i s[2];
        int at[2];      // where in x the piece lies; -1: nowhere (padding block, past the stored row or the last row)
    };
    // step t of this wave: row item w + (t / share) * waves, MFMA step sub + (t % share) * ksplit of it,
    // which takes slots 2 * step and the one after
    auto fetch = [&](int t, Step &f) __attribute__((always_inline)) {
        const int it = t / per_item, ms = sub + (t - it * per_item) * ksplit;
        const int row = (w + it * waves) * rows_per_item + sub_row;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int u = 2 * ms + h;
            const int p = (u * R + in_row) * 16;
            f.s[h] = zero;
            f.at[h] = -1;
            if (t < total && u < U && row < m && p < kell) {
                const int blk = block_shift >= 0 ? p >> block_shift : p / block;
                const int c = block_cols[(size_t)(row / block) * ell_cols + blk];
                f.s[h] = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(values + (size_t)row * kell + p));
                f.at[h] = c < 0 ? -1 : c * block + (p - blk * block);
            }
        }
    };
    Step ring[2];
    fetch(0, ring[0]);
    // (x is staged after the first loads of S have been issued, so that their latencies overlap)
    for (int t = threadIdx.x * 16; t < k; t += 256 * 16) *reinterpret_cast<v4i *>(lds_x + t) = load_piece(x + t);
    __syncthreads();

    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    float part = 0.0f;                                                   // ksplit > 1: this wave's share of its item's sums
    auto consume = [&](int t, const Step &f) __attribute__((always_inline)) {
        if (t >= total) return;                                          // (uniform)
        v4i xs[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) xs[h] = f.at[h] >= 0 ? *reinterpret_cast<const v4i *>(lds_x + f.at[h]) : zero;
        acc = mfma_16x16x128<SF, XF>(pack8(f.s[0], f.s[1]), pack8(xs[0], xs[1]), acc);
        const int it = t / per_item;
        if (t - it * per_item == share - 1) {                            // (uniform) this wave's part of the item is complete
            const int r = i & 3;
            float v = r == 0 ? acc[0] : (r == 1 ? acc[1] : (r == 2 ? acc[2] : acc[3]));
            v = (i >> 2) == q ? v : 0.0f;
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            for (int off = 1; off < G; off <<= 1) v += __shfl_xor(v, off, 64);
            const int row = (w + it * waves) * rows_per_item + i / G;
            if (ksplit == 1) {
                if (q == 0 && i % G == 0 && row < m) y[row] = v;
            } else {
                part = v;
            }
            acc = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
    };
    for (int t0 = 0; t0 < total; t0 += 2) {
        fetch(t0 + 1, ring[1]);
        consume(t0, ring[0]);
        fetch(t0 + 2, ring[0]);
        consume(t0 + 1, ring[1]);
    }
    if (ksplit > 1) {                                                    // (uniform over the grid)
        float *sums = reinterpret_cast<float *>(lds_x + ((k + 15) & ~15));
        if (q == 0) sums[wave * 16 + i] = part;
        __syncthreads();
        const int row = w * rows_per_item + i / G;
        if (sub == 0 && q == 0 && i % G == 0 && w < items && row < m) {
            float v = part;
            for (int u = 1; u < ksplit; ++u) v += sums[(wave + u) * 16 + i];
            y[row] = v;
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

// The same with 16-byte loads of the indices and 4-byte loads of the values (four entries per lane
// and pass, four passes in flight), waves that walk a few rows each (row w, w + waves, ..), and x in LDS
// (XLDS: k <= kSpmvLdsBytes; otherwise x is gathered through the caches).  A row's entries are taken in
// aligned groups of four starting at the group that holds its first entry; entries of the neighbouring
// rows in the first and last group are masked out, and the last groups of the arrays are read
// element by element, so nothing past the arrays' ends is touched.
// Requirements checked by the host: col 16-byte aligned, values 4-byte aligned.
template <int SF, int XF, bool XLDS>
__global__ __launch_bounds__(256) void spmv_csr_vec_kernel(int m, int k, const uint8_t *__restrict__ values,
                                                            const int *__restrict__ row_offsets,
                                                            const int *__restrict__ col,
                                                            const int *__restrict__ row_order,
                                                            const uint8_t *__restrict__ x, float *__restrict__ y)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_x[];
    const int lane = threadIdx.x & 63;
    const int waves = gridDim.x * 4;
    const int nnz = row_offsets[m];
    const int vec_end = nnz & ~3;                 // groups of four that lie wholly inside the arrays
    int w = blockIdx.x * 4 + (threadIdx.x >> 6);
    int row = 0, e0 = 0, e1 = 0;
    if (w < m) {
        row = row_order ? row_order[w] : w;
        e0 = row_offsets[row];
        e1 = row_offsets[row + 1];
    }
    if (XLDS) {
        // (k need not be a multiple of 16: the tail goes byte by byte)
        const int k16 = k & ~15;
        const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0;
        if (aligned)
            for (int t = threadIdx.x * 16; t < k16; t += 256 * 16) *reinterpret_cast<v4i *>(lds_x + t) = load_piece(x + t);
        for (int t = (aligned ? k16 : 0) + threadIdx.x; t < k; t += 256) lds_x[t] = x[t];
        __syncthreads();
    }
    const uint8_t *xs = XLDS ? lds_x : x;
    while (w < m) {
        // the next row's bounds are on their way while this row is added up
        const int wn = w + waves;
        int rown = 0, e0n = 0, e1n = 0;
        if (wn < m) {
            rown = row_order ? row_order[wn] : wn;
            e0n = row_offsets[rown];
            e1n = row_offsets[rown + 1];
        }
        float acc = 0.0f;
        auto one = [&](int e) __attribute__((always_inline)) {
            if (e >= e0 && e < e1) acc += fp8_to_float<SF>(values[e]) * fp8_to_float<XF>(xs[col[e]]);
        };
        auto four = [&](int e) __attribute__((always_inline)) {
            if (e + 4 <= vec_end) {
                const v4i c4 = *reinterpret_cast<const v4i *>(col + e);
                const uint32_t v4 = *reinterpret_cast<const uint32_t *>(values + e);
                float v[4];
                fp8x4_to_float<SF>(v4, v);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (e + t >= e0 && e + t < e1) acc += v[t] * fp8_to_float<XF>(xs[c4[t]]);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (e + t < nnz) one(e + t);
            }
        };
        for (int e = (e0 & ~3) + lane * 4; e < e1; e += 1024) {
            // four passes of 256 entries in flight: the loads first, then the arithmetic
            v4i c4[4];
            uint32_t v4[4];
            bool vec[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int eu = e + 256 * u;
                vec[u] = eu < e1 && eu + 4 <= vec_end;
                if (vec[u]) {
                    c4[u] = *reinterpret_cast<const v4i *>(col + eu);
                    v4[u] = *reinterpret_cast<const uint32_t *>(values + eu);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int eu = e + 256 * u;
                if (vec[u]) {
                    float v[4];
                    fp8x4_to_float<SF>(v4[u], v);
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (eu + t >= e0 && eu + t < e1) acc += v[t] * fp8_to_float<XF>(xs[c4[u][t]]);
                } else if (eu < e1) {
                    four(eu);                      // the last groups of the arrays, element by element
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (lane == 0) y[row] = acc;
        w = wn;
        row = rown;
        e0 = e0n;
        e1 = e1n;
    }
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

// The same in one pass for rows of up to kSpmvLdsBytes bytes (k % 16 == 0): a workgroup builds a
// row of the dense matrix in LDS -- zeros, then the row's stored entries -- and writes it out in
// whole 16-byte pieces; `dense` need not hold zeros.
__global__ __launch_bounds__(256) void csr_densify_rows_kernel(int m, int k, const uint8_t *__restrict__ values,
                                                                const int *__restrict__ row_offsets,
                                                                const int *__restrict__ col, uint8_t *__restrict__ dense)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_row[];
    const v4i zero = {0, 0, 0, 0};
    for (int row = blockIdx.x; row < m; row += gridDim.x) {
        for (int t = threadIdx.x * 16; t < k; t += 256 * 16) *reinterpret_cast<v4i *>(lds_row + t) = zero;
        __syncthreads();
        const int e1 = row_offsets[row + 1];
        for (int e = row_offsets[row] + threadIdx.x; e < e1; e += 256) {
            const uint8_t v = values[e];
            if ((v & 0x7F) != 0) lds_row[col[e]] = v;
        }
        __syncthreads();
        for (int t = threadIdx.x * 16; t < k; t += 256 * 16)
            *reinterpret_cast<v4i *>(dense + (size_t)row * k + t) = *reinterpret_cast<const v4i *>(lds_row + t);
        __syncthreads();
    }
}

// Sampled dense-dense product with a vector-sparse output pattern (the reference's Host_sddmm,
// GEMM/include/bm_test_utils.h:172-194): out[j * vec + v] = lhs[i * vec + v] . rhs[col[j]] for every
// stored entry j of vector row i; lhs (m_vec * vec) x k and rhs n x k, both row-major: every dot
// product runs along K on both sides, which is the MFMA's operand layout.  One workgroup of eight waves per
// vector row; a wave takes 16 stored entries at a time (chunks wave, wave + 8, ..): the up to 16 rows of lhs
// are the MFMA's A, the 16 gathered rows of rhs its B, and out[j][v] is element (v, j) of the 16 x 16 result.
// Lane (i = lane % 16, q = lane / 16) supplies 32 bytes of row i per K step.  What bounds the kernel is the
// latency of the gather -- the column index first, then the row of rhs it names -- so both run ahead of the
// MFMA across chunk boundaries: the column indices two chunks ahead, the rows of rhs one K step ahead (the
// last K step of a chunk fetches the first of the next), and eight waves to a row keep 32 waves on a CU.
// (With everything fetched inside the chunk that used it: 24.4 us for 840 k stored vectors at K = 128; now 11.)
// The rows of lhs, which every chunk of the vector row needs again, are taken from LDS when they fit (ALDS:
// rows kSddmmLdsPad bytes apart from a multiple of 128, so that the 16 lanes of a quarter read 16 different
// bank groups); otherwise they are loaded next to the rows of rhs.  WIDE: vec % 4 == 0 and out 16-byte
// aligned, a lane's four results leave in one store.
// Requirements checked by the host: vec <= 16, k % 16 == 0, 16-byte aligned lhs and rhs; ALDS:
// vec * (k + kSddmmLdsPad) bytes of dynamic LDS.
constexpr int kSddmmLdsPad = 16;
constexpr int kSddmmLdsBytes = 64 * 1024;
constexpr int kSddmmWaves = 8;

template <int LF, int RF, bool ALDS, bool WIDE>
__global__ __launch_bounds__(64 * kSddmmWaves) void sddmm_kernel(int k, int vec, const int *__restrict__ row_offsets,
                                                                  const int *__restrict__ col, const uint8_t *__restrict__ lhs,
                                                                  const uint8_t *__restrict__ rhs, float *__restrict__ out)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t sddmm_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const int vrow = blockIdx.x;
    const int e0 = row_offsets[vrow], e1 = row_offsets[vrow + 1];
    if (e0 >= e1) return;                                     // (the whole workgroup)
    const int steps = (k + 127) / 128;
    const v4i zero = {0, 0, 0, 0};
    // rows of lhs past vec re-read the last one; their results are never stored
    const int ai = i < vec ? i : vec - 1;
    const uint8_t *arow = lhs + (size_t)(vrow * vec + ai) * k;
    const int lds_stride = k + kSddmmLdsPad;
    // the entry this lane gathers for chunk number c of this wave (past the row's end: its last entry again)
    auto entry_of = [&](int c) __attribute__((always_inline)) {
        const long j = (long)e0 + ((long)wave + (long)kSddmmWaves * c) * 16 + i;
        return j < e1 ? (int)j : e1 - 1;
    };
    const int chunks = (e1 - e0 + 15) / 16;
    const int mine = chunks > wave ? (chunks - wave + kSddmmWaves - 1) / kSddmmWaves : 0;      // chunks of this wave
    int col_next = 0, col_after = 0;
    const uint8_t *brow = rhs;
    if (mine > 0) {
        brow = rhs + (size_t)col[entry_of(0)] * k;
        col_next = col[entry_of(1)];
    }
    struct Step {
        v4i a[2], b[2];
    };
    auto fetch = [&](const uint8_t *b_row, int s, Step &f) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int p = s * 128 + (2 * q + h) * 16;
            if constexpr (!ALDS) f.a[h] = p < k ? load_piece(arow + p) : zero;
            f.b[h] = p < k ? load_piece(b_row + p) : zero;
        }
    };
    Step cur, nxt;
    if (mine > 0) fetch(brow, 0, cur);
    if constexpr (ALDS) {
        const int per_row = k / 16;
        for (int t = threadIdx.x; t < vec * per_row; t += 64 * kSddmmWaves) {
            const int r = t / per_row, c = t - r * per_row;
            *reinterpret_cast<v4i *>(sddmm_lds + r * lds_stride + c * 16) = load_piece(lhs + (size_t)(vrow * vec + r) * k + c * 16);
        }
        __syncthreads();
    }
    const uint8_t *alds = sddmm_lds + ai * lds_stride;
    for (int c = 0; c < mine; ++c) {
        col_after = col[entry_of(c + 2)];
        const uint8_t *brow_next = rhs + (size_t)col_next * k;
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int s = 0; s < steps; ++s) {
            if (s + 1 < steps)
                fetch(brow, s + 1, nxt);
            else
                fetch(brow_next, 0, nxt);                     // (after the last chunk: the last entry's row once more)
            if constexpr (ALDS) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int p = s * 128 + (2 * q + h) * 16;
                    cur.a[h] = p < k ? *reinterpret_cast<const v4i *>(alds + p) : zero;
                }
            }
            acc = mfma_16x16x128<LF, RF>(pack8(cur.a[0], cur.a[1]), pack8(cur.b[0], cur.b[1]), acc);
            cur = nxt;
        }
        // register r of lane (i, q) holds lhs row 4q + r times rhs row col[j]
        const long j = (long)e0 + ((long)wave + (long)kSddmmWaves * c) * 16 + i;
        if (j < e1) {
            if constexpr (WIDE) {
                if (4 * q < vec) *reinterpret_cast<v4f *>(out + (size_t)j * vec + 4 * q) = acc;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (4 * q + r < vec) out[(size_t)j * vec + 4 * q + r] = acc[r];
            }
        }
        brow = brow_next;
        col_next = col_after;
    }
}

// The same for any k, vec and alignment: one thread per output, a running fp32 sum along K.
template <int LF, int RF>
__global__ __launch_bounds__(256) void sddmm_general_kernel(int m_vec, int k, int vec, const int *__restrict__ row_offsets,
                                                             const int *__restrict__ col, const uint8_t *__restrict__ lhs,
                                                             const uint8_t *__restrict__ rhs, float *__restrict__ out)
{
    const int vrow = blockIdx.x;
    if (vrow >= m_vec) return;
    const int e0 = row_offsets[vrow], e1 = row_offsets[vrow + 1];
    for (long t = threadIdx.x; t < (long)(e1 - e0) * vec; t += 256) {
        const int j = e0 + (int)(t / vec), v = (int)(t % vec);
        const uint8_t *a = lhs + (size_t)(vrow * vec + v) * k, *b = rhs + (size_t)col[j] * k;
        float acc = 0.0f;
        for (int l = 0; l < k; ++l) acc += fp8_to_float<LF>(a[l]) * fp8_to_float<RF>(b[l]);
        out[(size_t)j * vec + v] = acc;
    }
}

#endif  // FP8GEMM_KERNEL_SPARSE_H
