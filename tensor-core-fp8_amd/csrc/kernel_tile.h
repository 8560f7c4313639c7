// Vocabulary of the LDS-tiled MFMA kernels: tile shapes, the LDS swizzle, the wait on the
// vector-memory counter.
//
// A workgroup of WM x WN waves computes a BM x BN tile of C.  Per K tile of BK bytes, A and
// B rows are streamed with 128-bit global->LDS direct loads into a STAGES-deep ring of LDS
// buffers; every wave then reads its operand fragments with ds_read_b128 and issues MFMAs.
//
// LDS layout of one ring slot: BM rows of A then BN rows of B, each row BK bytes, the
// 16-byte chunks of a row permuted by XOR with a function of the row index (swizzle) so
// that fragment reads of 32 consecutive rows spread over all banks.  A direct load writes
// LDS at wave_base + lane*16, so the permutation is applied by choosing which global chunk
// each lane fetches.  A dot product does not change when the same permutation of K is
// applied to both operands, so lanes own whichever 16-byte K chunks load best.
#ifndef FP8GEMM_KERNEL_TILE_H
#define FP8GEMM_KERNEL_TILE_H

#include "device_common.h"

#define GLOBAL_AS __attribute__((address_space(1)))
#define LDS_AS __attribute__((address_space(3)))

// s_waitcnt that only constrains the vector-memory counter (gfx9 encoding:
// vmcnt = imm[15:14]:imm[3:0], expcnt = imm[6:4], lgkmcnt = imm[11:8]).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

template <int BK, int SWZ>
__device__ __forceinline__ int tile_swizzle(int row)
{
    constexpr int CH = BK / 16;
    if (SWZ == 0) return 0;
    if (SWZ == 1) return row % CH;
    if (SWZ == 2) return (row / (256 / BK)) % CH;
    return ((row % CH) ^ ((row / CH) & 1)) % CH;
}

// MF16_: the persistent kernel computes with v_mfma_f32_16x16x128_f8f6f4 (64 blocks of
// 16 x 16 per wave) instead of v_mfma_f32_32x32x64_f8f6f4 (16 blocks of 32 x 32)
template <int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, int SWZ_, bool MF16_ = false>
struct TileShape {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int STAGES = STAGES_, SWZ = SWZ_;
    static constexpr bool MF16 = MF16_;
    static constexpr int NW = WM * WN;
    static constexpr int THREADS = NW * 64;
    static constexpr int CH = BK / 16;            // 16-byte chunks per row
    static constexpr int RPI = 64 / CH;           // rows covered by one wave-wide load
    static constexpr int A_LOADS = BM / RPI / NW; // direct loads per thread per K tile
    static constexpr int B_LOADS = BN / RPI / NW;
    static constexpr int LOADS = A_LOADS + B_LOADS;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int LDS_BYTES = STAGE_BYTES * STAGES;
    static constexpr int TM = BM / WM / 32;       // 32x32 MFMA tiles per wave, M direction
    static constexpr int TN = BN / WN / 32;
    static constexpr int KSTEPS = BK / 64;
    // epilogue staging of the persistent kernel: LDS not used by the next tile's first
    // STAGES-1 K tiles (the last ring slot and whatever lies between the ring and 160 KiB)
    static constexpr int LDS_MAX = 160 * 1024;
    static constexpr int EP_OFFSET = STAGE_BYTES * (STAGES - 1);
    static constexpr int EP_WIDE = BN / WN;                                       // all columns of a wave at once
    static constexpr int EP_COLS = (NW * 32 * (EP_WIDE * 4 + 16) <= LDS_MAX - EP_OFFSET) ? EP_WIDE : EP_WIDE / 2;
    static constexpr int EP_BYTES = NW * 32 * (EP_COLS * 4 + 16);
    static constexpr int PTILE_LDS_BYTES = (EP_OFFSET + EP_BYTES > LDS_BYTES) ? EP_OFFSET + EP_BYTES : LDS_BYTES;
    static_assert(EP_OFFSET + EP_BYTES <= LDS_MAX, "epilogue staging does not fit");
    static_assert(BM % (RPI * NW) == 0 && BN % (RPI * NW) == 0, "tile rows must split over waves");
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be whole MFMA tiles");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt cannot count that many loads");
};

#endif  // FP8GEMM_KERNEL_TILE_H
