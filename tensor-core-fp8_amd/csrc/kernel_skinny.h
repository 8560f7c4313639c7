// B-streaming kernel for small m (1..64 rows of A): the shape is bound by
// reading B (n x k fp8) from HBM exactly once, so the kernel is organised as a
// set of independent single-wave streams with as many bytes in flight as LDS
// can hold and no workgroup barriers at all.
//
// One wave (= one workgroup of 64 threads) owns 16*TN consecutive columns of C
// (rows of B) and one K range [split*kchunk, (split+1)*kchunk).  Per K step of
// BK bytes it brings its 16*TN rows of B and the MT*16 rows of A into a private
// ring of STAGES LDS buffers with 128-bit global->LDS direct loads (coalesced
// along K), reads operand fragments back with ds_read_b128 and issues
// v_mfma_f32_16x16x128_f8f6f4.  Rows of A past m re-read row m-1; their results
// are never stored.
//
// With nsplit == 1 results go straight to C; otherwise fp32 partials go to a
// scratch buffer ws[split][m][n] and the reduction kernel (kernel_reduce.h) adds them
// in ascending split order (deterministic).
//
// Requirements checked by the host: kchunk % BK == 0, n % (16*TN) == 0,
// m <= 16*MT, 16-byte aligned a and b.
#ifndef FP8GEMM_KERNEL_SKINNY_H
#define FP8GEMM_KERNEL_SKINNY_H

#include "kernel_tile.h"

constexpr int skinny_min3(int a, int b, int c) { return a < b ? (a < c ? a : c) : (b < c ? b : c); }

// Largest K step <= bk (halving) for which two ring slots of (mt+tn)*16 rows fit in
// `cap` bytes of LDS and one slot's loads stay countable by vmcnt.
constexpr int skinny_fit_bk(int mt, int tn, int bk, int cap)
{
    while (bk > 128 && ((mt + tn) * 16 * bk * 2 > cap || (mt + tn) * 16 * bk / 1024 > 31)) bk /= 2;
    return bk;
}

// BK_ is the wanted K step and STAGES_ the wanted ring depth; both are cut back so
// that the ring stays within LDS_CAP_ bytes and the loads in flight stay countable
// by vmcnt (6 bits).
template <int MT_, int TN_, int BK_, int STAGES_, int LDS_CAP_ = 64 * 1024>
struct SkinnyShape {
    static constexpr int MT = MT_, TN = TN_;
    static constexpr int BK = skinny_fit_bk(MT_, TN_, BK_, LDS_CAP_);
    static constexpr int STAGES = skinny_min3(STAGES_, 63 / ((MT_ + TN_) * 16 * BK / 1024) + 1,
                                              LDS_CAP_ / ((MT_ + TN_) * 16 * BK));
    static constexpr int MP = MT * 16;            // padded rows of A
    static constexpr int NP = TN * 16;            // columns of C per wave
    static constexpr int CH = BK / 16;            // 16-byte chunks per row
    static constexpr int RPI = 64 / CH > 0 ? 64 / CH : 1;   // rows per wave-wide load
    static constexpr int LPR = CH / 64 > 0 ? CH / 64 : 1;   // wave-wide loads per row (BK = 1024: 1)
    static constexpr int ROWS = MP + NP;
    static constexpr int LOADS = ROWS * BK / 1024;          // direct loads per K step
    static constexpr int A_LOADS = MP * BK / 1024;
    static constexpr int STAGE_BYTES = ROWS * BK;
    static constexpr int LDS_BYTES = STAGE_BYTES * STAGES;
    static constexpr int KSTEPS = BK / 128;       // MFMA K steps per stage
    static_assert(BK % 128 == 0 && BK <= 1024, "BK must be a multiple of the MFMA K and at most one wave-wide load per row");
    static_assert(MP % RPI == 0 && NP % RPI == 0, "row counts must split into whole loads");
    static_assert(STAGES >= 2, "ring needs at least two stages");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt cannot count that many loads");
};

// chunk permutation: conflict-free for 16 consecutive rows read at one logical
// chunk, for row strides of 128 bytes and up
template <int BK>
__device__ __forceinline__ int skinny_swizzle(int row)
{
    constexpr int CH = BK / 16;
    if (CH >= 16) return row & 15;
    return ((row & 7) ^ ((row >> 3) & 1));
}

template <class S, int AF, int BF>
__global__ __launch_bounds__(64) void gemm_skinny_kernel(int M, int K, int N,
                                                         const uint8_t *__restrict__ A,
                                                         const uint8_t *__restrict__ B,
                                                         void *__restrict__ out,
                                                         int ngroups, int kchunk, int nsplit, OutSpec spec)
{
    constexpr int BK = S::BK, CH = S::CH, RPI = S::RPI, STAGES = S::STAGES;
    constexpr int MT = S::MT, TN = S::TN, MP = S::MP;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int lane = threadIdx.x;
    const int group = blockIdx.x % ngroups;
    const int split = blockIdx.x / ngroups;
    const int n0 = group * S::NP;
    const int kbeg = split * kchunk;

    // ---- load plan: stage rows 0..MP-1 hold A, rows MP.. hold B ---------------
    const int lrow = lane / CH;
    const int lslot = lane % CH;
    const uint8_t *src[S::LOADS];
#pragma unroll
    for (int j = 0; j < S::LOADS; ++j) {
        const int row = j * RPI + lrow;
        const int chunk = lslot ^ (skinny_swizzle<BK>(row) % CH);
        if (j < S::A_LOADS) {
            const int grow = row < M ? row : M - 1;
            src[j] = A + (size_t)grow * K + kbeg + chunk * 16;
        } else {
            src[j] = B + (size_t)(n0 + row - MP) * K + kbeg + chunk * 16;
        }
    }
    // Every stream starts its K walk at a different K step (and wraps around): streams
    // that start together would otherwise sweep the same address bits -- the same HBM
    // channels -- at the same time.  The rotation only reorders the fp32 sum.
    const int T = kchunk / BK;
    const int t0 = (int)(((unsigned)group * 2654435761u >> 8) % (unsigned)T);
    auto issue_loads = [&](int tt, int stage) {
        int t = tt + t0;
        t = t >= T ? t - T : t;
#pragma unroll
        for (int j = 0; j < S::LOADS; ++j)
            // B is read exactly once: the non-temporal hint (cache-policy bit 1) lets it stream
            // through the caches without displacing A, which every stream re-reads
            if (j < S::A_LOADS)
                __builtin_amdgcn_global_load_lds((const GLOBAL_AS void *)(src[j] + (size_t)t * BK),
                                                 (LDS_AS void *)(lds + stage * S::STAGE_BYTES + j * RPI * BK),
                                                 16, 0, 0);
            else
                __builtin_amdgcn_global_load_lds((const GLOBAL_AS void *)(src[j] + (size_t)t * BK),
                                                 (LDS_AS void *)(lds + stage * S::STAGE_BYTES + j * RPI * BK),
                                                 16, 0, 2);
    };

    // ---- fragment plan: lane (i = lane%16, q = lane/16) feeds row i of a 16-row
    // block and owns logical chunks s*8 + 2q + {0,1} of K step s ----------------
    const int fi = lane & 15;
    const int fq = lane >> 4;
    const int sw = skinny_swizzle<BK>(fi) % CH;
    uint32_t frag_off[S::KSTEPS][2];
#pragma unroll
    for (int s = 0; s < S::KSTEPS; ++s)
#pragma unroll
        for (int j = 0; j < 2; ++j) frag_off[s][j] = (uint32_t)(fi * BK + (((s * 8 + 2 * fq + j) ^ sw) * 16));

    v4f acc[MT][TN];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
        if (t < T) issue_loads(t, t);

    for (int t = 0; t < T; ++t) {
        // refill the stage consumed one step ago, then wait for stage t
        if (t + STAGES - 1 < T) {
            issue_loads(t + STAGES - 1, (t + STAGES - 1) % STAGES);
            wait_vmcnt<S::LOADS *(STAGES - 1)>();
        } else {
            wait_vmcnt<0>();
        }
        const uint8_t *st = lds + (t % STAGES) * S::STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < S::KSTEPS; ++s) {
            v8i af[MT], bf[TN];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const uint8_t *p = st + i * 16 * BK;
                af[i] = pack8(*reinterpret_cast<const v4i *>(p + frag_off[s][0]),
                              *reinterpret_cast<const v4i *>(p + frag_off[s][1]));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const uint8_t *p = st + (MP + j * 16) * BK;
                bf[j] = pack8(*reinterpret_cast<const v4i *>(p + frag_off[s][0]),
                              *reinterpret_cast<const v4i *>(p + frag_off[s][1]));
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma_16x16x128<AF, BF>(af[i], bf[j], acc[i][j]);
        }
        // all fragment reads of this stage have returned before it is refilled
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0) only
        __builtin_amdgcn_sched_barrier(0);
    }

    // with K slices `out` is the fp32 scratch (plane `split`, bare sums; the reduction
    // applies scale and output type), otherwise the output matrix itself
    const bool partial = nsplit > 1;
    const int type = partial ? FP8GEMM_DEV_OUT_F32 : spec.type;
    const size_t plane = partial ? (size_t)split * M * N : 0;
    OutFactors ofac = {1.0f, 0.0f, 1.0f};
    if (!partial) ofac = out_factors(spec);
    float amax_local = 0.0f;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = i * 16 + 4 * fq + r;
                if (row < M) {
                    const size_t index = plane + (size_t)row * N + n0 + j * 16 + fi;
                    const float y = partial ? acc[i][j][r] : finish_one(spec, ofac, index, acc[i][j][r], amax_local);
                    store_out(out, index, y, type);
                }
            }
    if (!partial) amax_commit(spec, amax_local);
}

#endif  // FP8GEMM_KERNEL_SKINNY_H
