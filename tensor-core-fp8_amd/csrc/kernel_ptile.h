// Persistent LDS-tiled MFMA kernel for compute-bound shapes.
//
// The grid is one workgroup per CU; every workgroup walks a list of work items,
// each a BM x BN tile of C over all of K or over one slice of K.  Inside an item
// the K loop is a software pipeline with three levels, all of them explicit:
//   * global -> LDS: 128-bit buffer loads that write LDS directly
//     (buffer_load_dwordx4 ... lds) into a ring of STAGES buffers, issued
//     STAGES-1 K tiles ahead of their use; no registers involved;
//   * LDS -> registers: the operand fragments of K step u+1 are read while the
//     MFMAs of K step u issue (two fragment sets, ping-pong);
//   * registers -> C of tile i overlaps the first global loads of tile i+1.
// One workgroup barrier per K tile, placed after the last fragment read of the
// tile so that the MFMAs already issued keep the matrix pipe busy across it.
//
// The instruction order of a K step is fixed by hand: after every MFMA come at
// most one global->LDS load and one or two fragment reads, so that the single
// wave of a SIMD never makes the matrix pipe wait behind a block of memory
// instructions and the texture-address unit sees an even stream (four waves x
// one 1 KiB load per MFMA slot is its full rate of 64 B/clk).
//
// Two forms of the K loop, chosen by the tile shape type: v_mfma_f32_32x32x64_f8f6f4 with
// ping-pong fragment sets (above), and v_mfma_f32_16x16x128_f8f6f4 (S::MF16) with the B
// fragments of a K tile resident and the A fragments streamed; the second needs less
// energy per flop, which is what limits the large shapes on a power-capped board.  Loads,
// ring, work list and epilogue are shared.
//
// MFMA operand roles are swapped (src0 = B rows, src1 = A rows): the result
// registers of a lane are then 4 consecutive columns of one row of C, which
// turns the epilogue into 128-bit stores.
//
// LDS layout, swizzle and the K-permutation freedom are described in kernel_tile.h.
// Requirements checked by the host: K % 16 == 0 (rows start 16-byte aligned and a
// 16-byte chunk never straddles the end of a row), K < 2^23, 16-byte aligned a and b.
#ifndef FP8GEMM_KERNEL_PTILE_H
#define FP8GEMM_KERNEL_PTILE_H

#include <type_traits>

#include "kernel_tile.h"

// s_waitcnt on the LDS/scalar counter only
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

// One wave-wide 16-byte-per-lane load from a buffer straight into LDS at
// lds_addr + lane*16.  rsrc: buffer resource (SGPRs), voff: per-lane byte offset,
// soff: uniform byte offset.  Bytes outside the buffer's extent read as zero.
// Written as inline assembly so that the compiler does not order it against the
// fragment reads (they never touch the ring slot being filled; the barrier
// protocol guarantees it).  Completion is tracked with wait_vmcnt by hand.
// M0 (the LDS base of the load) is named as clobbered so that the compiler keeps nothing
// in it across the statement; it warns that M0 is a reserved register, which is the point.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// (lds_addr is the same in every lane; where the compiler has let it drift into a vector
// register, v_readfirstlane_b32 brings it back -- otherwise the call is folded away)
__device__ __forceinline__ void buffer_load_lds_b128(v4i rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff)
{
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "m0");
}
// the same with the non-temporal hint, for an operand that no other workgroup reads
__device__ __forceinline__ void buffer_load_lds_b128_stream(v4i rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff)
{
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "m0");
}
// One 4-byte-per-lane load from per-lane addresses straight into LDS at lds_addr + lane*4.
__device__ __forceinline__ void global_load_lds_b32(const uint8_t *ptr, uint32_t lds_addr)
{
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :
                 : "s"(lds_addr), "v"(ptr)
                 : "m0", "memory");
}
#pragma clang diagnostic pop

// f(integral_constant<int, I>) for I = FIRST .. LAST-1, unrolled at compile time
template <int FIRST, int LAST, class F>
__device__ __forceinline__ void static_for(F &f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>{});
        static_for<FIRST + 1, LAST>(f);
    }
}

// 16-byte-per-lane LDS store whose data operand stays in accumulation registers
// (the MFMA results live there; copying all of them to ordinary vector registers
// first would need 256 more registers per lane).
__device__ __forceinline__ void lds_store_b128_acc(uint32_t lds_addr, v4f data)
{
    asm volatile("ds_write_b128 %0, %1" : : "v"(lds_addr), "a"(data) : "memory");
}

__device__ __forceinline__ v4i make_buffer_resource(const void *base, unsigned long long bytes)
{
    const unsigned long long a = reinterpret_cast<unsigned long long>(base);
    const uint32_t extent = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)bytes;
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xFFFFu));   // stride 0
    r[2] = __builtin_amdgcn_readfirstlane((int)extent);
    r[3] = 0x00020000;                                                             // raw 32-bit data format
    return r;
}

// Whether the kernel for tile shape S can add up the K slices of a tile itself (the slice that
// arrives last does it).  One CU then reads every slice of the tile, which pays up to 128 x 128.
template <class S>
constexpr bool ptile_sums_slices_in_kernel = S::BM * S::BN <= 128 * 128;

// KOVER: the last K tile may overhang K (K % BK != 0); compiled separately so that the
// common case carries no test for it.  EX: the output goes through `spec` (scale, fp32 /
// bf16 / fp16); without it C receives the bare fp32 sums and `spec` is ignored.  BSTREAM: B is
// loaded with the non-temporal hint (for a C with a single row of tiles, where every byte of B
// is read by exactly one workgroup).  BELL: A is sparse in blocked-ELL form (`bell`).  NOPF: without
// the L2 prefetch (see NPF below).
template <class S, int AF, int BF, bool KOVER, bool EX, bool BSTREAM, bool BELL, bool NOPF>
__device__ __forceinline__ void gemm_ptile_body(int M, int K, int N,
                                                const uint8_t *__restrict__ A,
                                                const uint8_t *__restrict__ B,
                                                void *__restrict__ C,
                                                float *__restrict__ ws,
                                                int *__restrict__ counters,
                                                int tiles_m, int tiles_n, int GM, int CB,
                                                int bulk, int tail, int nsplit,
                                                int rounds, int rotate_and_skew, OutSpec spec, BellSpec bell)
{
    static_assert(!BELL || !BSTREAM, "the blocked-ELL form shares B between tile rows");
    // Small blocks (tiles of fewer than 128 rows): a 128-byte K tile spans several stored blocks, so
    // where a chunk of B lies depends on which `bell.sub` bytes of the K tile (one stored block, or the
    // part of one) it belongs to; the offsets then ride in the loads' per-lane offsets.
    constexpr bool BELL_SMALL = BELL && S::BM < 128;
    constexpr int BELL_SUBS = BELL_SMALL ? 4 : 1;  // sub-blocks of a K tile at most (bell.sub >= 32)
    const int KB = BELL ? bell.kb : K;             // row stride of B
    const int rotate = rotate_and_skew & 0xFF;
    const int skew = rotate_and_skew >> 8;
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, CH = S::CH, RPI = S::RPI;
    constexpr int STAGES = S::STAGES, TM = S::TM, TN = S::TN, KSTEPS = S::KSTEPS;
    constexpr int NMFMA = TM * TN;
    constexpr bool SUM_HERE = ptile_sums_slices_in_kernel<S>;
    constexpr int NREADS = 2 * (TM + TN);          // ds_read_b128 per K step
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(LDS_AS uint8_t *)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / S::WN;
    const int wn = wave % S::WN;

    // lane constants of the load plan and the fragment plan
    const int lrow = lane / CH;
    const int lslot = lane % CH;
    const int fi = lane & 31;
    const int fg = lane >> 5;
    const int sw = tile_swizzle<BK, S::SWZ>(fi);
    uint32_t frag_off[KSTEPS][2];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int j = 0; j < 2; ++j) frag_off[s][j] = (uint32_t)(((s * 4 + 2 * fg + j) ^ sw) * 16);
    const uint32_t a_base = (uint32_t)(wm * (BM / S::WM) + fi) * BK;
    const uint32_t b_base = (uint32_t)(BM * BK) + (uint32_t)(wn * (BN / S::WN) + fi) * BK;
    const int KT = (K + BK - 1) / BK;              // K tiles of the whole problem; the last may overhang K
    // the partial sums of the K slices, as a window for device-scope accesses (used with counters)
    const __amdgpu_buffer_rsrc_t ws_window =
        device_scope_window(ws, counters ? (uint32_t)nsplit * (uint32_t)tail * (uint32_t)(BM * BN * 4) : 0u);

    // Work items.  The tiles of C are numbered along strips of GM tile rows (down a
    // column of the strip first, then on to the next column), so that consecutive tile
    // numbers form compact GM-row windows; where B is too large for the last-level cache
    // the strips are cut into blocks of CB columns, so that a round of 256 tiles covers a
    // square window and reads far fewer rows of B.  The first `bulk` tiles (a multiple of 256)
    // are items of their own, 256 per round: XCD x takes 32 consecutive ones, one per
    // CU, and shares their operand panels in its L2 (workgroups with equal id mod 8 sit
    // on one XCD).  The last `tail` tiles, too few to fill a round, are cut into nsplit
    // K slices each (slice-major item order: neighbours are still neighbouring tiles);
    // every round of such items is spread evenly over the eight XCDs.  Slice s of tail
    // tile u writes its partial sums to slot s*tail + u of the scratch `ws` (BM x BN
    // floats, row stride BN; the slices are added up by the one that arrives last, see the end of
    // the item, or by a reduction kernel that the host launches afterwards); unsplit items
    // write C directly.
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int bulk_rounds = bulk >> 8;
    const int tail_items = tail * nsplit;

    // item of round r: tile, slice, K-tile range [kt0, kt0 + T), scratch slot (-1: writes C);
    // false when this workgroup has none
    int items_in_xcd = 32;             // work items of this round on this workgroup's XCD
    auto tile_of_round = [&](int r, int &tm, int &tn, int &kt0, int &T, int &ws_slot) -> bool {
        if (r >= rounds) return false;
        int g, slice = 0;
        ws_slot = -1;
        if (r < bulk_rounds) {
            if (slot >= 32) return false;
            items_in_xcd = 32;
            g = r * 256 + xcd * 32 + slot;
        } else {
            const int first = (r - bulk_rounds) * 256;
            int count = tail_items - first;
            count = count > 256 ? 256 : count;
            if (count <= 0) return false;
            const int per_xcd = (count + 7) >> 3;
            items_in_xcd = per_xcd;
            const int local = xcd * per_xcd + slot;
            if (slot >= per_xcd || local >= count) return false;
            const int u = first + local;
            slice = u / tail;
            const int t = u - slice * tail;
            g = bulk + t;
            if (nsplit > 1) ws_slot = slice * tail + t;
        }
        int row, col;
        tile_of_number(g, tiles_m, tiles_n, GM, CB, row, col);
        // (the divisions may run on the vector unit; every lane holds the same values)
        tn = __builtin_amdgcn_readfirstlane(col);
        tm = __builtin_amdgcn_readfirstlane(row);
        const int split = r < bulk_rounds ? 1 : nsplit;
        const int k0 = (int)((long)KT * slice / split);
        kt0 = __builtin_amdgcn_readfirstlane(k0);
        T = __builtin_amdgcn_readfirstlane((int)((long)KT * (slice + 1) / split) - k0);
        ws_slot = __builtin_amdgcn_readfirstlane(ws_slot);
        return true;
    };

    // Global -> LDS load plan: one buffer resource per operand and tile (base =
    // first row of the tile, extent = the tile's rows that exist), a loop-invariant
    // 32-bit offset per load (row * K + chunk * 16) and a uniform offset that walks K.
    // Rows past the end of the matrix fall outside the extent and read as zero bytes
    // (fp8 +0.0), which is how tiles that overhang m or n are handled; in the K tile
    // that overhangs K, the chunks past the end of a row are sent outside the extent
    // on purpose (they would otherwise read the next row).
    uint32_t ld_off[S::LOADS];
#pragma unroll
    for (int j = 0; j < S::LOADS; ++j) {
        const int jj = j < S::A_LOADS ? j : j - S::A_LOADS;
        const int per = j < S::A_LOADS ? S::A_LOADS : S::B_LOADS;
        const int row = (wave * per + jj) * RPI + lrow;
        ld_off[j] = (uint32_t)row * (uint32_t)(j < S::A_LOADS ? K : KB) + (uint32_t)((lslot ^ tile_swizzle<BK, S::SWZ>(row)) * 16);
        // (small blocks: B's chunk counts from the start of its sub-block, whose place the block list gives)
        if (BELL_SMALL && j >= S::A_LOADS) ld_off[j] -= (uint32_t)((((lslot ^ tile_swizzle<BK, S::SWZ>(row)) * 16) / bell.sub) * bell.sub);
    }
    // which sub-block of a K tile this lane's chunks of B lie in: the swizzle only ever changes the
    // lowest bit of the chunk number between a lane's loads, and a sub-block holds two chunks or more
    const int bell_sb = BELL_SMALL ? ((lslot ^ tile_swizzle<BK, S::SWZ>(lrow)) * 16) / bell.sub : 0;
    const uint32_t ldsA = lds_base + (uint32_t)(wave * S::A_LOADS * RPI * BK);
    const uint32_t ldsB = lds_base + (uint32_t)(BM * BK + wave * S::B_LOADS * RPI * BK);
    v4i rsA = {0, 0, 0, 0}, rsB = {0, 0, 0, 0};
    // L2 prefetch: after the loads of a K tile each wave touches, with one 4-byte load per lane
    // whose data nobody uses, one 128-byte line per lane of the K tile pf_dist further on, so
    // that the line is on its way from HBM or the last-level cache into this XCD's L2 a K tile
    // and more before the loads that need it (whose own latency budget is about one K tile).
    // The workgroups of an XCD that share a panel split its rows among them, so that every line
    // is asked for once per XCD: with strips of GM tile rows, GM workgroups share a panel of B
    // and up to 8 share a panel of A.  B comes first (where C has one row of tiles it is
    // the operand that streams from HBM), A takes the lanes that are left.
    const uint8_t *pf_ptr = A;
    auto plan_prefetch = [&](int tile_m_, int tile_n_, int items_in_xcd) __attribute__((always_inline)) {
        const int q = wave * 64 + lane;                      // 0 .. 255: line number inside this workgroup's share
        int a_parts = items_in_xcd / GM;
        a_parts = a_parts > 8 ? 8 : (a_parts < 1 ? 1 : a_parts);
        const int nb = (BN + GM - 1) / GM, na = (BM + a_parts - 1) / a_parts;
        const int bpart = slot % GM, apart = (slot / GM) % a_parts;
        const uint8_t *p = A + (size_t)(tile_m_ * BM) * K;   // lanes without a line of their own: one valid address
        if (q < nb) {
            int row = tile_n_ * BN + bpart * nb + q;
            row = row < N ? row : N - 1;
            p = B + (size_t)row * KB;
        } else if (q - nb < na) {
            int row = tile_m_ * BM + apart * na + (q - nb);
            row = row < M ? row : M - 1;
            p = A + (size_t)row * K;
        }
        pf_ptr = p;
    };
    // K walk of the planned item: K tiles kt_base + ((t + kt_rot) mod kt_count), t = 0, 1, ..
    // The rotation kt_rot only reorders the fp32 sum.  Workgroups that walk K in step read,
    // at any moment, addresses that agree in the bits below the row stride; with a
    // power-of-two K those are the bits that select the HBM channel, so the whole chip
    // would queue on a few channels at a time.  rotate == 1 starts every tile column at
    // its own K tile (the workgroups of a column still share their B rows through L2; A
    // must then be small enough to stay in L2), rotate == 2 every XCD in every round (all
    // sharing inside an XCD is kept), 0 leaves the walk alone.
    int kt_base = 0, kt_rot = 0, kt_count = 1;
    // Blocked-ELL A: where in B's rows each K tile of the planned item's walk lies.  Lane l of bell_at
    // holds that byte offset for walk step 64 * bell_chunk + l (-1: a padding block), so the K loop
    // gets it with v_readlane_b32 and no memory access; a fresh set of 64 is fetched when the walk
    // crosses into the next chunk (a vector load whose wait drains the ring once per 64 K tiles).
    // Small blocks: one such register per sub-block of a K tile, and bell_vat = the offset of this
    // lane's sub-block in the K tile being loaded.
    const int *bell_row = nullptr;                 // block column list of the planned item's block row
    int bell_at[BELL_SUBS], bell_chunk = -1;
#pragma unroll
    for (int u = 0; u < BELL_SUBS; ++u) bell_at[u] = -1;
    uint32_t bell_koff = 0;                        // ... of the K tile being loaded
    bool bell_pad = false;                         // ... or that it is a padding block
    int bell_vat = -1;
    auto bell_fetch = [&](int chunk) __attribute__((always_inline)) {
        const int tt = chunk * 64 + lane;
#pragma unroll
        for (int u = 0; u < BELL_SUBS; ++u) {
            int v = -1;
            if (tt < kt_count && (!BELL_SMALL || u * bell.sub < BK)) {
                int kk = tt + kt_rot;
                kk = kk >= kt_count ? kk - kt_count : kk;
                const int pos = (kt_base + kk) * BK + (BELL_SMALL ? u * bell.sub : 0);   // byte position in the stored row
                if (pos < K) {                                          // (small blocks: the last K tile may overhang the stored row)
                    const int blk = pos / bell.block;
                    const int c = bell_row[blk];
                    v = c < 0 ? -1 : c * bell.block + (pos - blk * bell.block);
                }
            }
            bell_at[u] = v;
        }
        bell_chunk = chunk;
    };
    auto plan_loads = [&](int tile_m, int tile_n, int kt0, int count, int item) __attribute__((always_inline)) {
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        const int rows_a = M - m0 < BM ? M - m0 : BM;
        const int rows_b = N - n0 < BN ? N - n0 : BN;
        rsA = make_buffer_resource(A + (size_t)m0 * K, (unsigned long long)rows_a * (unsigned long long)K);
        rsB = make_buffer_resource(B + (size_t)n0 * KB, (unsigned long long)rows_b * (unsigned long long)KB);
        if constexpr (BELL) bell_row = bell.cols + (size_t)(m0 / bell.block) * bell.ell_cols;
        kt_base = kt0;
        kt_count = count;
        const unsigned key = rotate == 1 ? (unsigned)tile_n : (unsigned)item;   // item: (round, XCD)
        // (the division runs on the vector unit; the result is the same in every lane)
        kt_rot = rotate == 0 ? 0 : __builtin_amdgcn_readfirstlane((int)(((key * 2654435761u) >> 8) % (unsigned)count));
        plan_prefetch(tile_m, tile_n, items_in_xcd);
        if constexpr (BELL) bell_fetch(0);
    };
    // load number j (0 .. LOADS-1) of step `ktile` of the planned item's K walk into ring slot `stage`
    // (the lambdas around the loads are forced inline: a closure left in memory would turn the
    // scalar operands of the load instruction into per-lane values)
    auto issue_load = [&](int j, int ktile, int stage) __attribute__((always_inline)) {
        int kk = ktile + kt_rot;
        kk = kk >= kt_count ? kk - kt_count : kk;
        // (pinned to a scalar register: it is an SGPR operand of the load and also feeds per-lane arithmetic)
        const uint32_t koff = (uint32_t)__builtin_amdgcn_readfirstlane((kt_base + kk) * BK);
        const uint32_t sbase = (uint32_t)(stage * S::STAGE_BYTES);
        // the K tile that overhangs K: chunks past the end of the row go outside the extent
        uint32_t voff = ld_off[j];
        if (KOVER && kt_base + kk == KT - 1) {                      // uniform, rarely taken
            const int jj = j < S::A_LOADS ? j : j - S::A_LOADS;
            const int per = j < S::A_LOADS ? S::A_LOADS : S::B_LOADS;
            const int row = (wave * per + jj) * RPI + lrow;
            const uint32_t kpos = koff + (uint32_t)((lslot ^ tile_swizzle<BK, S::SWZ>(row)) * 16);
            voff = kpos >= (uint32_t)K ? 0xFFFFFFF0u : voff;
        }
        if constexpr (BELL) {
            if (j == S::A_LOADS) {                 // first load of B of this K tile: where its block lies
                if ((ktile >> 6) != bell_chunk) bell_fetch(ktile >> 6);               // (uniform, once per 64 K tiles)
                if constexpr (BELL_SMALL) {
                    int mine = __builtin_amdgcn_readlane(bell_at[0], ktile & 63);
#pragma unroll
                    for (int u = 1; u < BELL_SUBS; ++u) {
                        const int at = __builtin_amdgcn_readlane(bell_at[u], ktile & 63);
                        mine = bell_sb == u ? at : mine;
                    }
                    bell_vat = mine;
                } else {
                    const int at = __builtin_amdgcn_readlane(bell_at[0], ktile & 63);
                    bell_pad = at < 0;
                    bell_koff = (uint32_t)at;
                }
            }
            if (BELL_SMALL && j >= S::A_LOADS) {
                // (a padding block, or past the end of the stored row: outside the extent, reads zeros)
                buffer_load_lds_b128(rsB, ldsB + sbase + (uint32_t)((j - S::A_LOADS) * RPI * BK),
                                     bell_vat < 0 ? 0xFFFFFFF0u : ld_off[j] + (uint32_t)bell_vat, 0u);
                return;
            }
            if (j >= S::A_LOADS) {
                // a padding block: every lane's address goes outside the extent and reads zeros
                buffer_load_lds_b128(rsB, ldsB + sbase + (uint32_t)((j - S::A_LOADS) * RPI * BK), bell_pad ? 0xFFFFFFF0u : voff,
                                     bell_pad ? 0u : bell_koff);
                return;
            }
        }
        if (j < S::A_LOADS)
            buffer_load_lds_b128(rsA, ldsA + sbase + (uint32_t)(j * RPI * BK), voff, koff);
        else if (BSTREAM)
            buffer_load_lds_b128_stream(rsB, ldsB + sbase + (uint32_t)((j - S::A_LOADS) * RPI * BK), voff, koff);
        else
            buffer_load_lds_b128(rsB, ldsB + sbase + (uint32_t)((j - S::A_LOADS) * RPI * BK), voff, koff);
    };
    auto issue_all_loads = [&](int ktile, int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < S::LOADS; ++j) issue_load(j, ktile, stage);
    };

    // (a load that writes LDS, into 256 bytes past everything else that nobody reads: a load
    // into a register would write that register whenever it returns, behind the compiler's back)
    auto issue_prefetch = [&](int ktile) __attribute__((always_inline)) {
        if constexpr (BSTREAM || BELL || NOPF) return;
        int kk = ktile < kt_count ? ktile : kt_count - 1;
        kk += kt_rot;
        kk = kk >= kt_count ? kk - kt_count : kk;
        // (K is a multiple of 16: the last, overhanging K tile still starts inside the row)
        const uint32_t koff = (uint32_t)__builtin_amdgcn_readfirstlane((kt_base + kk) * BK);
        global_load_lds_b32(pf_ptr + koff, lds_base + (uint32_t)S::PTILE_LDS_BYTES);
    };
    // Prefetch instructions that close a batch of loads, and how many K tiles they run ahead of
    // the batch.  One K tile ahead is best (MI355X, 16384^3: 56.4 % of the FP8 peak without, 60.9 %
    // one K tile ahead, 60.7 / 60.3 / 59.6 % two / three / four ahead; 3072^3 ... 6144^3 gain 1-3 %,
    // shapes whose operands stay in the caches are unchanged).  Not where B streams past with the
    // non-temporal hint (one row of tiles: M=256 N=28672 K=8192 76 -> 84 us with the prefetch):
    // there every line is used once, by one workgroup, and asking for it twice only adds requests.
    // Nor (NOPF) where both operands stay in the 256 MB last-level cache and the launch runs at the
    // board's power limit: the extra requests then cost more than the latency they hide
    // (8192^3: 368.2 -> 364.8 us without, 4096^3: 54.9 -> 53.9 us).
    constexpr int NPF = (BSTREAM || BELL || NOPF) ? 0 : 1;
    constexpr int pf_dist = 1;

    // Start skew: the workgroups of an XCD that work on tile row i of its window start i * skew
    // ticks (10 ns each) late and stay that far apart for the rest of the launch, so that
    // their epilogues -- which share the XCD's write path -- do not all come at once.
    if (skew > 0 && bulk > 0) {
        const unsigned long long ticks = (unsigned long long)((slot % GM) * skew);
        const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
        while (__builtin_amdgcn_s_memrealtime() - t0 < ticks) __builtin_amdgcn_s_sleep(8);
    }

    int tile_m = 0, tile_n = 0, kt0 = 0, T = 0, ws_slot = -1;
    bool have = tile_of_round(0, tile_m, tile_n, kt0, T, ws_slot);
    if (have) {
        plan_loads(tile_m, tile_n, kt0, T, xcd);
#pragma unroll
        for (int t = 0; t < STAGES - 1; ++t)
            if (t < T) issue_all_loads(t, t);
    }

    for (int r = 0; r < rounds; ++r) {
        if (!have) {
            // nothing here this round; still look at the next one
            have = tile_of_round(r + 1, tile_m, tile_n, kt0, T, ws_slot);
            if (have) {
                plan_loads(tile_m, tile_n, kt0, T, (r + 1) * 8 + xcd);
#pragma unroll
                for (int t = 0; t < STAGES - 1; ++t)
                    if (t < T) issue_all_loads(t, t);
            }
            continue;
        }
        const int m0 = tile_m * BM, n0 = tile_n * BN;

        // accumulators: TM x TN blocks of 32 x 32 (16 registers each), or twice as many
        // blocks of 16 x 16 each way (4 registers each); 256 registers per lane either way
        using AccT = std::conditional_t<S::MF16, v4f, v16f>;
        constexpr int AM = S::MF16 ? 2 * TM : TM, AN = S::MF16 ? 2 * TN : TN;
        AccT acc[AM][AN];
#pragma unroll
        for (int i = 0; i < AM; ++i)
#pragma unroll
            for (int j = 0; j < AN; ++j)
#pragma unroll
                for (int q = 0; q < (S::MF16 ? 4 : 16); ++q) acc[i][j][q] = 0.0f;

        if constexpr (!S::MF16) {
            // fragment sets: frag[p][0..TM-1] = A blocks, frag[p][TM..TM+TN-1] = B blocks
            v4i frag[2][TM + TN][2];
            // read number q (0 .. NREADS-1) of K step ks of ring slot `stage` into set p.
            // Order: B0, A0, B1 .. B(TN-1), A1 .. A(TM-1), the order the MFMAs need them.
            auto issue_read = [&](auto pc, int q, int stage, int ks) {
                constexpr int P = decltype(pc)::value;
                const int f = q >> 1, h = q & 1;
                int idx;           // index into frag[P]
                if (f == 0) idx = TM;
                else if (f == 1) idx = 0;
                else if (f <= TN) idx = TM + f - 1;
                else idx = f - TN;
                const uint32_t rowbase = idx < TM ? a_base + (uint32_t)(idx * 32 * BK) : b_base + (uint32_t)((idx - TM) * 32 * BK);
                const uint8_t *p = lds + stage * S::STAGE_BYTES + rowbase + frag_off[ks][h];
                frag[P][idx][h] = *reinterpret_cast<const v4i *>(p);
            };

            // K tile 0 must have landed before the first fragment read.  The stores of
            // the previous tile's epilogue are still in flight and share the counter
            // with the loads (and may retire out of order with them), so wait for all.
            wait_vmcnt<0>();
            __syncthreads();
            if (STAGES - 1 < T) {
                issue_all_loads(STAGES - 1, STAGES - 1);
                issue_prefetch(STAGES - 1 + pf_dist);
            }
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
#pragma unroll
            for (int q = 0; q < NREADS; ++q) issue_read(I0{}, q, 0, 0);

            // One K step.  P = parity of the global step (which fragment set feeds the
            // MFMAs), KS = K step inside the K tile, next = a further K tile follows,
            // load = a K tile STAGES ahead exists and is fetched now (both uniform; the
            // steady-state loop passes constants so that no branch is left in it).
            auto kstep = [&](auto pc, auto sc, const bool next, const bool load, int t) {
                constexpr int P = decltype(pc)::value;
                constexpr int KS = decltype(sc)::value;
                using PN = std::integral_constant<int, P ^ 1>;
                const int stage = t % STAGES;
                constexpr bool last_ks = (KS + 1 == KSTEPS);
                int rstage = stage, rks = KS + 1;
                bool reads = true;
                if (last_ks) {
                    rstage = (t + 1) % STAGES;
                    rks = 0;
                    reads = next;
                    if (next) {
                        // every fragment read of K tile t has been issued; once they have
                        // returned this wave no longer needs the ring slot
                        // K tile t + 1 has landed once only the younger batches of loads (each
                        // closed by its prefetch) and the prefetch that closed its own are left
                        wait_lgkmcnt0();
                        if (load)
                            wait_vmcnt<(S::LOADS + NPF) * (STAGES - 2) + NPF>();
                        else
                            wait_vmcnt<0>();
                        __syncthreads();
                    }
                }
                // reads per MFMA slot and loads per MFMA slot, rounded up
                constexpr int RD_PER = (NREADS + NMFMA - 1) / NMFMA;
                constexpr int LD_PER = (S::LOADS + NMFMA - 1) / NMFMA;
#pragma unroll
                for (int m = 0; m < NMFMA; ++m) {
                    const int i = m / TN, j = m % TN;
                    acc[i][j] = mfma_32x32x64<BF, AF>(pack8(frag[P][TM + j][0], frag[P][TM + j][1]),
                                                      pack8(frag[P][i][0], frag[P][i][1]), acc[i][j]);
                    if (last_ks && load) {
#pragma unroll
                        for (int u = 0; u < LD_PER; ++u)
                            if (m * LD_PER + u < S::LOADS) issue_load(m * LD_PER + u, t + STAGES, stage);
                        if (m == NMFMA - 1) issue_prefetch(t + STAGES + pf_dist);
                    }
                    if (reads) {
#pragma unroll
                        for (int u = 0; u < RD_PER; ++u)
                            if (m * RD_PER + u < NREADS) issue_read(PN{}, m * RD_PER + u, rstage, rks % KSTEPS);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            // K tiles [0, T-STAGES) fetch ahead, [T-STAGES, T-1) only consume, T-1 is last
            const int t_load_end = T - STAGES > 0 ? T - STAGES : 0;
            if (KSTEPS == 2) {
                int t = 0;
                for (; t < t_load_end; ++t) {
                    kstep(I0{}, I0{}, true, true, t);
                    kstep(I1{}, I1{}, true, true, t);
                }
                for (; t < T; ++t) {
                    kstep(I0{}, I0{}, t + 1 < T, false, t);
                    kstep(I1{}, I1{}, t + 1 < T, false, t);
                }
            } else {
                // one K step per K tile: the fragment sets alternate from K tile to K tile, so
                // K tiles go in pairs (an odd count ends on a single one)
                const int t_pair_end = t_load_end & ~1;
                int t = 0;
                for (; t < t_pair_end; t += 2) {
                    kstep(I0{}, I0{}, true, true, t);
                    kstep(I1{}, I0{}, true, true, t + 1);
                }
                for (; t < T; t += 2) {
                    kstep(I0{}, I0{}, t + 1 < T, t < t_load_end, t);
                    if (t + 1 < T) kstep(I1{}, I0{}, t + 2 < T, t + 1 < t_load_end, t + 1);
                }
            }

        } else {
            // ---- v_mfma_f32_16x16x128_f8f6f4: one MFMA K step per K tile -------------
            // Lane (hi = lane % 16, hq = lane / 16) feeds row hi of a 16-row block with K
            // quarter hq (chunks 2*hq, 2*hq + 1 of the row).  The B fragments of a K tile
            // (8 blocks, 64 registers) stay resident for all its MFMAs and are double
            // buffered across K tiles; the A fragments (8 blocks for 128 rows per wave, 6 for
            // 96) stream through: all but the first are read during the first FIRST MFMAs, so
            // that every read of the ring slot has been issued when the one barrier of the K
            // tile comes, 32 MFMAs before its end.  By then the next K tile has landed (its B
            // fragments and first A fragment are read during those last 32 MFMAs) and the slot
            // just read is free for the K tile after that.
            static_assert(STAGES == 2 && KSTEPS == 2 && (TM == 4 || TM == 3) && TN == 4,
                          "the 16x16x128 schedule is written for 128 or 96 x 128 per wave, 128-byte K tiles, two ring slots");
            constexpr int ABLK = 2 * TM;                  // A blocks of 16 rows per wave
            constexpr int FIRST = 8 * ABLK - 32;          // MFMAs before the barrier
            constexpr int ASTEP = FIRST / (ABLK - 1);     // A block b is read beside MFMAs ASTEP*(b-1), +1
            const int hi = lane & 15, hq = lane >> 4;
            const int hsw = tile_swizzle<BK, S::SWZ>(hi);             // same for rows hi + 16 * block
            const uint32_t hoff0 = (uint32_t)(((2 * hq) ^ hsw) * 16), hoff1 = (uint32_t)(((2 * hq + 1) ^ hsw) * 16);
            const uint32_t ha_base = (uint32_t)(wm * (BM / S::WM) + hi) * BK;
            const uint32_t hb_base = (uint32_t)(BM * BK) + (uint32_t)(wn * (BN / S::WN) + hi) * BK;
            v4i fb[2][8][2], fa[6][2];       // A block 0 lives in fa[5], block i > 0 in fa[(i - 1) % 5]
            auto read_a = [&](int blk, int h, int stage) __attribute__((always_inline)) {
                fa[blk == 0 ? 5 : (blk - 1) % 5][h] = *reinterpret_cast<const v4i *>(lds + stage * S::STAGE_BYTES + ha_base + (uint32_t)(blk * 16 * BK) + (h ? hoff1 : hoff0));
            };
            auto read_b = [&](auto pc, int blk, int h, int stage) __attribute__((always_inline)) {
                constexpr int P = decltype(pc)::value;
                fb[P][blk][h] = *reinterpret_cast<const v4i *>(lds + stage * S::STAGE_BYTES + hb_base + (uint32_t)(blk * 16 * BK) + (h ? hoff1 : hoff0));
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            wait_vmcnt<0>();
            __syncthreads();
            if (1 < T) issue_all_loads(1, 1);
            issue_prefetch(1 + pf_dist);
            read_a(0, 0, 0);
            read_a(0, 1, 0);

            // K tile t with B fragment set P; next: a further K tile follows; load: the K tile
            // after that exists and is fetched now (both uniform)
            auto ktile = [&](auto pc, const bool next, const bool load, int t) __attribute__((always_inline)) {
                constexpr int P = decltype(pc)::value;
                using PN = std::integral_constant<int, P ^ 1>;
                const int stage = t & 1, nstage = stage ^ 1;
#pragma unroll
                for (int m = 0; m < FIRST; ++m) {
                    const int i = m >> 3, j = m & 7;
                    acc[i][j] = mfma_16x16x128<BF, AF>(pack8(fb[P][j][0], fb[P][j][1]), pack8(fa[i == 0 ? 5 : (i - 1) % 5][0], fa[i == 0 ? 5 : (i - 1) % 5][1]), acc[i][j]);
                    // block b > 5 goes to the place of block b - 5, whose block row is over by then
                    if (1 + m / ASTEP < ABLK && m % ASTEP < 2) read_a(1 + m / ASTEP, m % ASTEP, stage);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (next) {
                    // every load but the youngest has landed: the youngest is the prefetch that
                    // closed the previous batch of loads, whose data nobody waits for
                    wait_lgkmcnt0();
                    wait_vmcnt<NPF>();
                    __syncthreads();
                }
#pragma unroll
                for (int m = 0; m < 32; ++m) {
                    const int i = FIRST / 8 + (m >> 3), j = m & 7;
                    acc[i][j] = mfma_16x16x128<BF, AF>(pack8(fb[P][j][0], fb[P][j][1]), pack8(fa[(i - 1) % 5][0], fa[(i - 1) % 5][1]), acc[i][j]);
                    // a 16x16x128 MFMA lasts 32 clocks: room for about one memory instruction
                    // beside it.  Even slots take the loads (16 or 14) of the K tile after next, odd
                    // slots the 16 reads of the next B fragments, slots 0 and 2 also the two
                    // reads of the next first A fragment (its own registers: free since block row 0).
                    if ((m & 1) == 0) {
                        if (load && (m >> 1) < S::LOADS) issue_load(m >> 1, t + 2, stage);
                        if (next && m < 4) read_a(0, (m >> 1) & 1, nstage);
                    } else if (next) {
                        read_b(PN{}, m >> 2, (m >> 1) & 1, nstage);
                    }
                    if (m == 31 && load) issue_prefetch(t + 2 + pf_dist);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            static_assert(S::LOADS <= 16, "the loads of a K tile are issued beside every other one of the last 32 MFMAs");
            // K tiles go in pairs, one per B fragment set; an odd count starts with a single K
            // tile on set 1.  T >= 2 (the host sends shorter K walks to the 32x32x64 kernel),
            // so the last pair is written out and no branch surrounds a K tile inside the
            // loop: all 256 accumulation registers are taken, and a copy of an accumulator
            // at a join would have nowhere to go.
            int t = 0;
            if (T & 1) {
#pragma unroll
                for (int q = 0; q < 16; ++q) read_b(I1{}, q >> 1, q & 1, 0);
                ktile(I1{}, true, true, 0);
                t = 1;
            } else {
#pragma unroll
                for (int q = 0; q < 16; ++q) read_b(I0{}, q >> 1, q & 1, 0);
            }
            for (; t < T - 2; t += 2) {
                ktile(I0{}, true, true, t);
                ktile(I1{}, true, true, t + 1);
            }
            ktile(I0{}, true, false, t);
            ktile(I1{}, false, false, t + 1);
        }

        // all waves are done reading LDS for this tile before the ring is reused
        wait_lgkmcnt0();
        __syncthreads();
        int next_m = 0, next_n = 0, next_kt0 = 0, next_T = 0, next_ws_slot = -1;
        have = tile_of_round(r + 1, next_m, next_n, next_kt0, next_T, next_ws_slot);
        if (have) {
            plan_loads(next_m, next_n, next_kt0, next_T, (r + 1) * 8 + xcd);
#pragma unroll
            for (int t = 0; t < STAGES - 1; ++t)
                if (t < next_T) issue_all_loads(t, t);
        }
        // ---- epilogue: registers -> C -------------------------------------------
        // register q of lane (fi, fg) holds C[row0 + fi][col0 + 8*(q/4) + 4*fg + q%4]
        const int wrow0 = m0 + wm * (BM / S::WM);
        const int wcol0 = n0 + wn * (BN / S::WN);
        // destination of this item: its tile of C (row stride N), or a whole BM x BN slot of
        // the scratch (row stride BN; rows and columns past the matrix hold zeros)
        // (the scratch takes bare fp32 sums; scale and output type are applied where C is written)
        const bool to_ws = ws_slot >= 0;
        void *__restrict__ tile_base = to_ws ? static_cast<void *>(ws) : C;
        const size_t tile_origin = to_ws ? (size_t)ws_slot * (size_t)(BM * BN) : (size_t)m0 * (size_t)N + n0;
        const size_t ldo = to_ws ? (size_t)BN : (size_t)N;
        // (the epilogue arithmetic -- scales, beta * C, largest magnitude -- only where C itself is
        // written, and only in the kernels compiled for it)
        const bool finish = EX && !to_ws;
        const int otype = finish ? spec.type : FP8GEMM_DEV_OUT_F32;
        OutFactors ofac = {1.0f, 0.0f, 1.0f};
        if (finish) ofac = out_factors(spec);
        float amax_local = 0.0f;
        const bool full = to_ws || ((m0 + BM <= M) && (n0 + BN <= N) && (N % 4 == 0) &&
                                    (reinterpret_cast<uintptr_t>(C) % 16 == 0) &&
                                    (!EX || !spec.c || reinterpret_cast<uintptr_t>(spec.c) % 16 == 0));
        {
            // Each wave transposes its results through a private strip of LDS (the part of
            // the ring the next tile's first loads do not use, plus the LDS above the ring)
            // so that every store instruction writes whole contiguous row segments of C:
            // a CU drains full-line stores about three times faster than 32-byte pieces.
            // Tiles that overhang C take the same route with every element store guarded.
            constexpr int EP = S::EP_COLS;                       // columns staged at a time
            constexpr int ROWB = EP * 4 + 16;                    // padded row: conflict-free both ways
            constexpr int LPR = EP / 4;                          // lanes per row when reading back
            constexpr int RPI_ST = 64 / LPR;                     // rows per store instruction
            uint8_t *stg = lds + S::EP_OFFSET + wave * (32 * ROWB);
            const uint32_t stg_addr = lds_base + (uint32_t)(S::EP_OFFSET + wave * (32 * ROWB));
            const int rl = lane / LPR, cl = lane % LPR;
            constexpr int CHUNKS = TN * 32 / EP;                 // column chunks of a 32-row block
            constexpr int NSTEP = TM * CHUNKS;                   // strips to stage
            constexpr int NR = 32 / RPI_ST;                      // store instructions per strip
            // strip st = rows 32*(st / CHUNKS) .., columns EP*(st % CHUNKS) .. of the wave's part
            auto stage_strip = [&](auto stc) __attribute__((always_inline)) {
                constexpr int ST = decltype(stc)::value;
                constexpr int i = ST / CHUNKS, c0 = (ST % CHUNKS) * EP;
                if constexpr (!S::MF16) {
#pragma unroll
                    for (int j = c0 / 32; j < (c0 + EP) / 32; ++j)
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            v4f v = {acc[i][j][4 * q4], acc[i][j][4 * q4 + 1], acc[i][j][4 * q4 + 2], acc[i][j][4 * q4 + 3]};
                            lds_store_b128_acc(stg_addr + (uint32_t)(fi * ROWB + (j * 32 - c0 + 8 * q4 + 4 * fg) * 4), v);
                        }
                } else {
                    // lane (lane % 16, lane / 16) of block (ib, jb) holds C[16*ib + lane%16][16*jb + 4*(lane/16) .. +3]
#pragma unroll
                    for (int ib = 2 * i; ib < 2 * i + 2; ++ib)
#pragma unroll
                        for (int jb = c0 / 16; jb < (c0 + EP) / 16; ++jb)
                            lds_store_b128_acc(stg_addr + (uint32_t)((16 * (ib & 1) + (lane & 15)) * ROWB + (16 * jb - c0 + 4 * (lane >> 4)) * 4), acc[ib][jb]);
                }
            };
            auto drain_strip = [&](auto stc) __attribute__((always_inline)) {
                constexpr int ST = decltype(stc)::value;
                constexpr int i = ST / CHUNKS, c0 = (ST % CHUNKS) * EP;
                const int lrow0 = wrow0 - m0 + i * 32 + rl;          // inside the tile
                const int lcol_ = wcol0 - n0 + c0 + cl * 4;
                const size_t first = tile_origin + (size_t)lrow0 * ldo + lcol_;
                if (full) {
                    // All reads of the strip go out back to back, then the next strip is staged
                    // (the LDS serves one wave's instructions in order, so those writes land after
                    // these reads), then the stores follow as the data arrive: one LDS round trip
                    // per strip instead of one per store.
                    v4f buf[NR];
#pragma unroll
                    for (int u = 0; u < NR; ++u)
                        buf[u] = *reinterpret_cast<const v4f *>(stg + (u * RPI_ST + rl) * ROWB + cl * 16);
                    if constexpr (ST + 1 < NSTEP) stage_strip(std::integral_constant<int, ST + 1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    if (EX) {
                        if (finish) {
                            // (four rows at a time: all the reads of C at once would need a second
                            // set of registers as large as buf)
#pragma unroll
                            for (int u = 0; u < NR; ++u) {
                                buf[u] = finish_four(spec, ofac, first + (size_t)(u * RPI_ST) * ldo, buf[u], amax_local);
                                if ((u & 3) == 3) __builtin_amdgcn_sched_barrier(0);
                            }
                        }
                    }
                    // partial sums in the scratch are read back soon (keep them cached);
                    // C itself is not (streaming stores)
                    if (SUM_HERE && to_ws && counters) {
                        // (read back by a workgroup that may sit on another XCD)
#pragma unroll
                        for (int u = 0; u < NR; ++u)
                            store_f32x4_device_scope(ws_window, (uint32_t)(first + (size_t)(u * RPI_ST) * ldo) * 4u, buf[u]);
                    } else if (to_ws) {
#pragma unroll
                        for (int u = 0; u < NR; ++u) store_out4(tile_base, first + (size_t)(u * RPI_ST) * ldo, buf[u], otype);
                    } else {
#pragma unroll
                        for (int u = 0; u < NR; ++u) store_out4_stream(tile_base, first + (size_t)(u * RPI_ST) * ldo, buf[u], otype);
                    }
                } else {
                    // a tile that overhangs C: every element store guarded, a few rows at a time
#pragma unroll 2
                    for (int r0 = 0; r0 < 32; r0 += RPI_ST) {
                        v4f v = *reinterpret_cast<const v4f *>(stg + (r0 + rl) * ROWB + cl * 16);
                        const size_t index = first + (size_t)r0 * ldo;
                        if (m0 + lrow0 + r0 < M) {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (n0 + lcol_ + e < N) {
                                    const float y = (EX && finish) ? finish_one(spec, ofac, index + e, v[e], amax_local) : v[e];
                                    store_out(tile_base, index + e, y, otype);
                                }
                        }
                    }
                    if constexpr (ST + 1 < NSTEP) stage_strip(std::integral_constant<int, ST + 1>{});
                }
            };
            stage_strip(std::integral_constant<int, 0>{});
            static_for<0, NSTEP>(drain_strip);
            if (EX && finish) amax_commit(spec, amax_local);
        }
        // ---- K slices: the slice that arrives last adds them up ---------------------
        // Hand-over of the partial sums between workgroups that may sit on different XCDs, in
        // three steps:
        //   1. every thread writes its partial sums with device-scope (sc1) stores and waits for
        //      them itself (s_waitcnt vmcnt(0)): such a store counts as done only once it is
        //      written through.  A workgroup barrier does not wait for outstanding stores;
        //   2. after the barrier (all threads' stores are done) one thread counts the slice on the
        //      tile's arrival counter with a device-scope atomic;
        //   3. the slice that finds all the others there reads the slots back with device-scope
        //      (sc1) loads, issued only after the counter's value is known (they depend on it
        //      through the flag in LDS and a barrier), in slice order -- the order the reduction
        //      kernel uses, so the bits are the same -- and writes the tile of C.
        // Nobody waits for anybody.  The counter is left at zero for the next launch.
        if (SUM_HERE && to_ws && counters) {                       // (uniform)
            const int t_cut = ws_slot % tail;                      // number of the cut tile
            LDS_AS int *flag = (LDS_AS int *)(lds + S::PTILE_LDS_BYTES + 256);
            wait_vmcnt<0>();                                       // step 1: this thread's stores are written through
            __syncthreads();
            if (tid == 0) {
                const int before = __hip_atomic_fetch_add(counters + t_cut, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const int last = before == nsplit - 1;
                if (last) __hip_atomic_store(counters + t_cut, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *flag = last;
            }
            __syncthreads();
            if (*flag) {
                const uint32_t slot0 = (uint32_t)t_cut * (uint32_t)(BM * BN * 4);      // bytes
                const uint32_t plane = (uint32_t)tail * (uint32_t)(BM * BN * 4);
                OutFactors rfac = {1.0f, 0.0f, 1.0f};
                if (EX) rfac = out_factors(spec);
                float ramax = 0.0f;
                const bool aligned = N % 4 == 0 && reinterpret_cast<uintptr_t>(C) % 16 == 0 &&
                                     (!EX || !spec.c || reinterpret_cast<uintptr_t>(spec.c) % 16 == 0);
                const int rtype = EX ? spec.type : FP8GEMM_DEV_OUT_F32;
                constexpr int QUADS = BM * BN / 4;                 // groups of four columns in a tile
                constexpr int QB = 4;                              // groups a thread has in flight
                static_assert(QUADS % (S::THREADS * QB) == 0, "tile does not divide among the threads");
                for (int q0 = tid; q0 < QUADS; q0 += S::THREADS * QB) {
                    v4f sum[QB];
#pragma unroll
                    for (int u = 0; u < QB; ++u) sum[u] = load_f32x4_device_scope(ws_window, slot0 + (uint32_t)(q0 + u * S::THREADS) * 16u);
                    for (int p = 1; p < nsplit; p += 2) {          // two more slices at a time
                        const bool two = p + 1 < nsplit;
                        v4f v0[QB], v1[QB];
#pragma unroll
                        for (int u = 0; u < QB; ++u) {
                            const uint32_t at = slot0 + (uint32_t)(q0 + u * S::THREADS) * 16u + (uint32_t)p * plane;
                            v0[u] = load_f32x4_device_scope(ws_window, at);
                            if (two) v1[u] = load_f32x4_device_scope(ws_window, at + plane);
                        }
#pragma unroll
                        for (int u = 0; u < QB; ++u) {
                            sum[u] += v0[u];
                            if (two) sum[u] += v1[u];
                        }
                    }
#pragma unroll
                    for (int u = 0; u < QB; ++u) {
                        const int q = q0 + u * S::THREADS;
                        const int row = q / (BN / 4), col = (q - row * (BN / 4)) * 4;
                        const int grow = m0 + row, gcol = n0 + col;
                        if (grow < M && gcol < N) {
                            const size_t index = (size_t)grow * N + gcol;
                            if (gcol + 3 < N && aligned) {
                                store_out4_stream(C, index, EX ? finish_four(spec, rfac, index, sum[u], ramax) : sum[u], rtype);
                            } else {
                                for (int e = 0; e < 4; ++e)
                                    if (gcol + e < N)
                                        store_out(C, index + e, EX ? finish_one(spec, rfac, index + e, sum[u][e], ramax) : sum[u][e], rtype);
                            }
                        }
                    }
                }
                if (EX) amax_commit(spec, ramax);
            }
        }
        tile_m = next_m;
        tile_n = next_n;
        kt0 = next_kt0;
        T = next_T;
        ws_slot = next_ws_slot;
    }
}

template <class S, int AF, int BF, bool KOVER, bool EX, bool BSTREAM, bool NOPF = false>
__global__ __launch_bounds__(S::THREADS) void gemm_ptile_kernel(int M, int K, int N,
                                                                 const uint8_t *__restrict__ A,
                                                                 const uint8_t *__restrict__ B,
                                                                 void *__restrict__ C,
                                                                 float *__restrict__ ws,
                                                                 int *__restrict__ counters,
                                                                 int tiles_m, int tiles_n, int GM, int CB,
                                                                 int bulk, int tail, int nsplit,
                                                                 int rounds, int rotate_and_skew, OutSpec spec)
{
    gemm_ptile_body<S, AF, BF, KOVER, EX, BSTREAM, false, NOPF>(M, K, N, A, B, C, ws, counters, tiles_m, tiles_n, GM, CB, bulk, tail,
                                                          nsplit, rounds, rotate_and_skew, spec, BellSpec{nullptr, 0, 0, 0, 0});
}

// The same kernel with A in blocked-ELL form: out = S * B^T, S stored as `A` (M x K values) and `bell`.
template <class S, int AF, int BF>
__global__ __launch_bounds__(S::THREADS) void gemm_ptile_bell_kernel(int M, int K, int N,
                                                                      const uint8_t *__restrict__ A,
                                                                      const uint8_t *__restrict__ B,
                                                                      void *__restrict__ C,
                                                                      float *__restrict__ ws,
                                                                      int *__restrict__ counters,
                                                                      int tiles_m, int tiles_n, int GM, int CB,
                                                                      int bulk, int tail, int nsplit,
                                                                      int rounds, int rotate_and_skew, BellSpec bell)
{
    const OutSpec plain = {1.0f, nullptr, nullptr, FP8GEMM_DEV_OUT_F32, 0.0f, nullptr, FP8GEMM_DEV_OUT_F32, nullptr, nullptr, nullptr};
    // (tiles of fewer than 128 rows serve small blocks, whose stored rows need not be whole K tiles)
    gemm_ptile_body<S, AF, BF, (S::BM < 128), false, false, true, false>(M, K, N, A, B, C, ws, counters, tiles_m, tiles_n, GM, CB, bulk, tail,
                                                          nsplit, rounds, rotate_and_skew, plain, bell);
}

#endif  // FP8GEMM_KERNEL_PTILE_H
