// Shared device-side vocabulary for the gfx950 FP8 GEMM kernels.
#ifndef FP8GEMM_DEVICE_COMMON_H
#define FP8GEMM_DEVICE_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define FP8GEMM_WAVE 64

// v_mfma_f32_32x32x64_f8f6f4: D(32x32 fp32) += A(32x64 fp8) * B(64x32 fp8).
// AF / BF: 0 = E4M3, 1 = E5M2 (the instruction's cbsz / blgp fields).  Both
// block-scale operands are literal zero, which selects the unscaled opcode.
//
// Operand layout: lane l supplies 32 bytes of row (l % 32) of A, respectively
// of column (l % 32) of B, covering one K half chosen by (l / 32).  A and B use
// the same lane->K map, so any K bytes may be given to a lane as long as the
// A lane and the B lane of equal (l / 32) are given the same ones.
// Result layout: register r of lane l holds D[8*(r/4) + 4*(l/32) + r%4][l%32].
template <int AF, int BF>
__device__ __forceinline__ v16f mfma_32x32x64(v8i a, v8i b, v16f c)
{
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, AF, BF, 0, 0, 0, 0);
}

// v_mfma_f32_16x16x128_f8f6f4: D(16x16) += A(16x128) * B(128x16).  Lane l
// supplies 32 bytes of row / column (l % 16), K quarter (l / 16); register r of
// lane l holds D[4*(l/16) + r][l%16].
template <int AF, int BF>
__device__ __forceinline__ v4f mfma_16x16x128(v8i a, v8i b, v4f c)
{
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, AF, BF, 0, 0, 0, 0);
}

__device__ __forceinline__ v8i pack8(v4i lo, v4i hi)
{
    v8i r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
}

// Numbering of the tiles of C, shared by the persistent kernel and the reduction of its K
// slices: column blocks of CB tile columns (CB >= tiles_n: a single block), inside a block
// strips of GM tile rows, inside a strip down a column first.  256 consecutive numbers are
// then a compact window of (256 / CB) x CB tiles where the matrix is large enough, and 32
// consecutive ones a window of GM x (32 / GM).
__host__ __device__ __forceinline__ void tile_of_number(int g, int tiles_m, int tiles_n, int GM, int CB, int &tm, int &tn)
{
    const int block_tiles = tiles_m * CB;
    const int cb = g / block_tiles;
    const int gb = g - cb * block_tiles;
    int w = tiles_n - cb * CB;
    w = w > CB ? CB : w;
    const int per_strip = GM * w;
    const int strip = gb / per_strip;
    const int rem = gb - strip * per_strip;
    int h = tiles_m - strip * GM;
    h = h > GM ? GM : h;
    const int col = rem / h;
    tn = cb * CB + col;
    tm = strip * GM + rem - col * h;
}

// What a kernel does with a finished fp32 sum s of element i:
//     y = alpha * a_scale * b_scale * s  +  beta * c_scale * C[i]        (C read only when given)
//     amax = max(amax, |y|)                                              (only when given)
//     D[i] = cast_type(d_scale * y)                                      (round to nearest even)
// -- what the reference's vendor-library sample hands to cuBLASLt next to the operands
// (GEMM/src/cublas.cu:9-23, 41-46: host alpha and beta, device pointers to per-tensor scales
// of A, B, C and D, a device pointer for the largest magnitude of the output).  The scale
// pointers point to one float each, or are null for 1; c is a device matrix laid out like D
// (m x n row-major) of type c_type, or null (then beta is not used and C is never read); c may
// be D itself.  The plain entry points use {1, null, null, fp32, ...nothing else}: the
// multiplication by 1.0f is exact, results are the bare sums.
#define FP8GEMM_DEV_OUT_F32 0
#define FP8GEMM_DEV_OUT_BF16 1
#define FP8GEMM_DEV_OUT_F16 2
struct OutSpec {
    float alpha;
    const float *a_scale;
    const float *b_scale;
    int type;
    float beta;
    const void *c;
    int c_type;
    const float *c_scale;
    const float *d_scale;
    float *amax;
};

// A sparse A in blocked-ELL form for the tiled kernel (kernel_sparse.h describes the format): A
// is then the m x K matrix of stored values (K = ell_cols * block bytes per row), and K tile g of a
// tile row pairs with the bytes of B's rows at block column cols[tile row's block row][g * BK / block].
// block % BM == 0, so all rows of a tile share one list; with block % BK == 0 a K tile lies inside
// one stored block, with smaller blocks it spans several (`sub`).
struct BellSpec {
    const int *cols;      // (m / block) x ell_cols block column numbers, -1 = padding (counts as zeros)
    int ell_cols, block;
    int kb;               // row stride of B in bytes (the k of the sparse matrix)
    int sub;              // blocks smaller than a K tile: gcd(block, 128), the bytes of a K tile that share a stored block
};

__device__ __forceinline__ float out_scale(const OutSpec &o)
{
    float s = o.alpha;
    if (o.a_scale) s *= *o.a_scale;
    if (o.b_scale) s *= *o.b_scale;
    return s;
}

// the three factors of the epilogue, read once per kernel
struct OutFactors {
    float ab, c, d;
};

__device__ __forceinline__ OutFactors out_factors(const OutSpec &o)
{
    // (the same in every lane: pinned to scalar registers, the kernels are short of vector ones)
    const auto uniform = [](float v) { return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v))); };
    OutFactors f;
    f.ab = uniform(out_scale(o));
    f.c = uniform(o.c ? (o.c_scale ? o.beta * *o.c_scale : o.beta) : 0.0f);
    f.d = uniform(o.d_scale ? *o.d_scale : 1.0f);
    return f;
}

__device__ __forceinline__ uint32_t out_bits16(float v, int type)
{
    if (type == FP8GEMM_DEV_OUT_BF16) {
        const __bf16 h = (__bf16)v;
        return (uint32_t)__builtin_bit_cast(unsigned short, h);
    }
    const _Float16 h = (_Float16)v;
    return (uint32_t)__builtin_bit_cast(unsigned short, h);
}

// Output pointers arrive as generic pointers (a choice between C and the scratch buffer, a
// void pointer for the three output types); they always point to global memory, and saying
// so keeps the stores from being issued as flat instructions, which also count as LDS
// traffic in the wave's counters.
#define FP8GEMM_GLOBAL __attribute__((address_space(1)))

// element `index` of an output matrix of the given type
__device__ __forceinline__ void store_out(void *base, size_t index, float v, int type)
{
    if (type == FP8GEMM_DEV_OUT_F32)
        ((FP8GEMM_GLOBAL float *)base)[index] = v;
    else
        ((FP8GEMM_GLOBAL unsigned short *)base)[index] = (unsigned short)out_bits16(v, type);
}

typedef unsigned int v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ v2u out_pack4(v4f v, int type)
{
    v2u w;
    w[0] = out_bits16(v[0], type) | (out_bits16(v[1], type) << 16);
    w[1] = out_bits16(v[2], type) | (out_bits16(v[3], type) << 16);
    return w;
}

// four consecutive elements starting at `index` (index % 4 == 0, 16-byte aligned base)
__device__ __forceinline__ void store_out4(void *base, size_t index, v4f v, int type)
{
    if (type == FP8GEMM_DEV_OUT_F32)
        *(FP8GEMM_GLOBAL v4f *)((FP8GEMM_GLOBAL float *)base + index) = v;
    else
        *(FP8GEMM_GLOBAL v2u *)((FP8GEMM_GLOBAL unsigned short *)base + index) = out_pack4(v, type);
}

// element `index` of an input matrix of the given type (the C operand of the epilogue)
__device__ __forceinline__ float load_in(const void *base, size_t index, int type)
{
    if (type == FP8GEMM_DEV_OUT_F32) return ((const FP8GEMM_GLOBAL float *)base)[index];
    const unsigned short h = ((const FP8GEMM_GLOBAL unsigned short *)base)[index];
    if (type == FP8GEMM_DEV_OUT_BF16) return __builtin_bit_cast(float, (uint32_t)h << 16);
    return (float)__builtin_bit_cast(_Float16, h);
}

// four consecutive elements starting at `index` (index % 4 == 0, 16-byte aligned base)
__device__ __forceinline__ v4f load_in4(const void *base, size_t index, int type)
{
    if (type == FP8GEMM_DEV_OUT_F32) return *(const FP8GEMM_GLOBAL v4f *)((const FP8GEMM_GLOBAL float *)base + index);
    const v2u w = *(const FP8GEMM_GLOBAL v2u *)((const FP8GEMM_GLOBAL unsigned short *)base + index);
    v4f r;
    if (type == FP8GEMM_DEV_OUT_BF16) {
        r[0] = __builtin_bit_cast(float, w[0] << 16);
        r[1] = __builtin_bit_cast(float, w[0] & 0xFFFF0000u);
        r[2] = __builtin_bit_cast(float, w[1] << 16);
        r[3] = __builtin_bit_cast(float, w[1] & 0xFFFF0000u);
    } else {
        r[0] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[0] & 0xFFFFu));
        r[1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[0] >> 16));
        r[2] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[1] & 0xFFFFu));
        r[3] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[1] >> 16));
    }
    return r;
}

// The epilogue of one element / of four consecutive ones: fp32 sum -> value to store, and the
// thread's running largest |y| (NaNs do not enter it).
__device__ __forceinline__ float finish_one(const OutSpec &o, const OutFactors &f, size_t index, float sum, float &amax)
{
    float y = sum * f.ab;
    if (o.c) y += f.c * load_in(o.c, index, o.c_type);
    amax = fmaxf(amax, fabsf(y));
    return y * f.d;
}

__device__ __forceinline__ v4f finish_four(const OutSpec &o, const OutFactors &f, size_t index, v4f sum, float &amax)
{
    v4f y = {sum[0] * f.ab, sum[1] * f.ab, sum[2] * f.ab, sum[3] * f.ab};
    if (o.c) {
        const v4f c = load_in4(o.c, index, o.c_type);
        y[0] += f.c * c[0];
        y[1] += f.c * c[1];
        y[2] += f.c * c[2];
        y[3] += f.c * c[3];
    }
    amax = fmaxf(fmaxf(amax, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
    y[0] *= f.d;
    y[1] *= f.d;
    y[2] *= f.d;
    y[3] *= f.d;
    return y;
}

// Folds the threads' largest magnitudes into *o.amax (which the host has set to zero on the
// stream before the kernel): one atomic per wave.  Non-negative floats order like their bit
// patterns, so an integer maximum does it.
__device__ __forceinline__ void amax_commit(const OutSpec &o, float amax)
{
    if (!o.amax) return;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((threadIdx.x & 63) == 0 && amax > 0.0f) atomicMax(reinterpret_cast<int *>(o.amax), __builtin_bit_cast(int, amax));
}

// The same with the streaming (non-temporal) hint, for results that no kernel reads again:
// a finished tile of C leaves through the L2 without pushing the operand panels out of it.
// Written as assembly: where a branch chooses between a plain and a non-temporal store of
// the same value, the optimizer merges the two into one plain store and the hint is lost.
__device__ __forceinline__ void store_out4_stream(void *base, size_t index, v4f v, int type)
{
    if (type == FP8GEMM_DEV_OUT_F32) {
        FP8GEMM_GLOBAL v4f *p = (FP8GEMM_GLOBAL v4f *)((FP8GEMM_GLOBAL float *)base + index);
        asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(p), "v"(v) : "memory");
    } else {
        FP8GEMM_GLOBAL v2u *p = (FP8GEMM_GLOBAL v2u *)((FP8GEMM_GLOBAL unsigned short *)base + index);
        const v2u w = out_pack4(v, type);
        asm volatile("global_store_dwordx2 %0, %1, off nt" : : "v"(p), "v"(w) : "memory");
    }
}

// ---- device-scope accesses ---------------------------------------------------------------
// The eight XCDs each have an L2 of their own, and a plain store may sit in the writer's L2
// where a workgroup on another XCD does not see it.  Accesses with the sc1 bit act at device
// scope: such a store is written through to memory before it counts as done (vmcnt), such a
// load does not take a line that another XCD may have changed from its own L2.  Data handed
// from one workgroup to another inside a launch goes through these, with the writer's
// s_waitcnt vmcnt(0) and a device-scope atomic in between; no whole-cache write-back or
// invalidate is needed.  (Buffer instructions, because their cache bits can be set from C++.)
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
constexpr int kDeviceScope = 16;      // the sc1 bit of a buffer instruction's cache policy

__device__ __forceinline__ __amdgpu_buffer_rsrc_t device_scope_window(void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)bytes, 0x00020000);      // raw 32-bit data format
}

__device__ __forceinline__ void store_f32x4_device_scope(__amdgpu_buffer_rsrc_t window, uint32_t byte_offset, v4f v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), window, (int)byte_offset, 0, kDeviceScope);
}

__device__ __forceinline__ v4f load_f32x4_device_scope(__amdgpu_buffer_rsrc_t window, uint32_t byte_offset)
{
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(window, (int)byte_offset, 0, kDeviceScope));
}

#endif  // FP8GEMM_DEVICE_COMMON_H
