// LDS-tiled MFMA kernel for compute-bound shapes.
//
// One workgroup of WM x WN waves computes a BM x BN tile of C.  Per K tile of
// BK bytes, A and B rows are streamed with 128-bit global->LDS direct loads
// into a STAGES-deep ring of LDS buffers; every wave then reads its operand
// fragments with ds_read_b128 and issues v_mfma_f32_32x32x64_f8f6f4.
//
// LDS layout of one stage: BM rows of A then BN rows of B, each row BK bytes,
// the 16-byte chunks of a row permuted by XOR with a function of the row index
// (swizzle) so that fragment reads of 32 consecutive rows spread over all
// banks.  A direct load writes LDS at wave_base + lane*16, so the permutation
// is applied by choosing which global chunk each lane fetches.
//
// Requirements checked by the host: K % BK == 0, 16-byte aligned a and b.
// M and N are arbitrary: loads clamp the row index, stores are predicated.
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

// Maps the linear workgroup id to a tile so that the workgroups resident on one
// XCD (ids congruent mod 8 are dispatched to the same XCD and share its L2)
// cover compact GM x GN blocks of tiles.  Returns false for padding ids.
__device__ __forceinline__ bool tile_of_workgroup(int pid, int tiles_m, int tiles_n, int GM, int GN,
                                                  int &tm, int &tn)
{
    const int xcd = pid & 7;
    const int slot = pid >> 3;
    const int per_block = GM * GN;
    const int nb_n = (tiles_n + GN - 1) / GN;
    const int nb_m = (tiles_m + GM - 1) / GM;
    const int blk = (slot / per_block) * 8 + xcd;
    if (blk >= nb_m * nb_n) return false;
    const int within = slot % per_block;
    tm = (blk / nb_n) * GM + within / GN;
    tn = (blk % nb_n) * GN + within % GN;
    return tm < tiles_m && tn < tiles_n;
}

template <class S, int AF, int BF>
__global__ __launch_bounds__(S::THREADS) void gemm_tile_kernel(int M, int K, int N,
                                                                const uint8_t *__restrict__ A,
                                                                const uint8_t *__restrict__ B,
                                                                float *__restrict__ C,
                                                                int tiles_m, int tiles_n, int GM, int GN)
{
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, CH = S::CH, RPI = S::RPI;
    constexpr int STAGES = S::STAGES, TM = S::TM, TN = S::TN;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    int tile_m, tile_n;
    if (!tile_of_workgroup(blockIdx.x, tiles_m, tiles_n, GM, GN, tile_m, tile_n)) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / S::WN;
    const int wn = wave % S::WN;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    // ---- global->LDS load plan (constant over the K loop) -------------------
    // load j of this wave covers tile rows (wave*LOADS_x + j)*RPI .. +RPI-1; lane
    // handles row lane/CH of those and LDS chunk slot lane%CH.
    const int lrow = lane / CH;
    const int lslot = lane % CH;
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int row = (wave * S::A_LOADS + j) * RPI + lrow;
        const int chunk = lslot ^ tile_swizzle<BK, S::SWZ>(row);
        int grow = m0 + row;
        grow = grow < M ? grow : M - 1;
        a_off[j] = (uint32_t)(grow - m0) * (uint32_t)K + chunk * 16;
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int row = (wave * S::B_LOADS + j) * RPI + lrow;
        const int chunk = lslot ^ tile_swizzle<BK, S::SWZ>(row);
        int grow = n0 + row;
        grow = grow < N ? grow : N - 1;
        b_off[j] = (uint32_t)(grow - n0) * (uint32_t)K + chunk * 16;
    }
    const uint8_t *gA = A + (size_t)m0 * K;
    const uint8_t *gB = B + (size_t)n0 * K;

    auto issue_loads = [&](int ktile, int stage) {
        uint8_t *sA = lds + stage * S::STAGE_BYTES + (wave * S::A_LOADS) * RPI * BK;
        uint8_t *sB = lds + stage * S::STAGE_BYTES + BM * BK + (wave * S::B_LOADS) * RPI * BK;
        const uint8_t *pa = gA + (size_t)ktile * BK;
        const uint8_t *pb = gB + (size_t)ktile * BK;
#pragma unroll
        for (int j = 0; j < S::A_LOADS; ++j)
            __builtin_amdgcn_global_load_lds((const GLOBAL_AS void *)(pa + a_off[j]),
                                             (LDS_AS void *)(sA + j * RPI * BK), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < S::B_LOADS; ++j)
            __builtin_amdgcn_global_load_lds((const GLOBAL_AS void *)(pb + b_off[j]),
                                             (LDS_AS void *)(sB + j * RPI * BK), 16, 0, 0);
    };

    // ---- fragment read plan --------------------------------------------------
    // lane (i = lane%32, g = lane/32) feeds row i of each 32-row block; in K step
    // s it owns logical chunks  s*4 + 2g + {0,1}  (BK=128)  or  2g + {0,1} (BK=64).
    const int fi = lane & 31;
    const int fg = lane >> 5;
    const int a_row0 = wm * (BM / S::WM) + fi;
    const int b_row0 = wn * (BN / S::WN) + fi;
    // the swizzle only sees row bits below 32 where both bases are multiples of 32
    const int sw = tile_swizzle<BK, S::SWZ>(fi);
    uint32_t frag_off[S::KSTEPS][2];
#pragma unroll
    for (int s = 0; s < S::KSTEPS; ++s)
#pragma unroll
        for (int j = 0; j < 2; ++j) frag_off[s][j] = (uint32_t)(((s * 4 + 2 * fg + j) ^ sw) * 16);
    const uint32_t a_base = (uint32_t)a_row0 * BK;
    const uint32_t b_base = (uint32_t)(BM * BK) + (uint32_t)b_row0 * BK;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int T = K / BK;
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
        if (t < T) issue_loads(t, t);

    for (int t = 0; t < T; ++t) {
        // tile t has landed once at most the (STAGES-2) younger tiles are in flight
        if (t + STAGES - 2 < T)
            wait_vmcnt<S::LOADS *(STAGES - 2)>();
        else
            wait_vmcnt<0>();
        __syncthreads();
        // every wave is past tile t-1, whose stage is the one refilled now
        if (t + STAGES - 1 < T) issue_loads(t + STAGES - 1, (t + STAGES - 1) % STAGES);

        const uint8_t *st = lds + (t % STAGES) * S::STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < S::KSTEPS; ++s) {
            v8i af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const uint8_t *p = st + a_base + i * 32 * BK;
                af[i] = pack8(*reinterpret_cast<const v4i *>(p + frag_off[s][0]),
                              *reinterpret_cast<const v4i *>(p + frag_off[s][1]));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const uint8_t *p = st + b_base + j * 32 * BK;
                bf[j] = pack8(*reinterpret_cast<const v4i *>(p + frag_off[s][0]),
                              *reinterpret_cast<const v4i *>(p + frag_off[s][1]));
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma_32x32x64<AF, BF>(af[i], bf[j], acc[i][j]);
        }
    }

    // ---- epilogue: registers -> C ---------------------------------------------
    const int crow0 = m0 + wm * (BM / S::WM) + 4 * fg;
    const int ccol0 = n0 + wn * (BN / S::WN) + fi;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = ccol0 + j * 32;
            if (col < N) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = crow0 + i * 32 + 8 * (r >> 2) + (r & 3);
                    if (row < M) C[(size_t)row * N + col] = acc[i][j][r];
                }
            }
        }
}

#endif  // FP8GEMM_KERNEL_TILE_H
