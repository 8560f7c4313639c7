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

// What a kernel does with a finished fp32 sum: multiply by alpha * a_scale * b_scale and
// store as fp32, bf16 or fp16 (round to nearest even).  The scale pointers are device
// pointers to one float each, or null for 1.  The plain entry points use {1, null, null,
// fp32}: the multiplication by 1.0f is exact, results are the bare sums.
#define FP8GEMM_DEV_OUT_F32 0
#define FP8GEMM_DEV_OUT_BF16 1
#define FP8GEMM_DEV_OUT_F16 2
struct OutSpec {
    float alpha;
    const float *a_scale;
    const float *b_scale;
    int type;
};

__device__ __forceinline__ float out_scale(const OutSpec &o)
{
    float s = o.alpha;
    if (o.a_scale) s *= *o.a_scale;
    if (o.b_scale) s *= *o.b_scale;
    return s;
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

#endif  // FP8GEMM_DEVICE_COMMON_H
