// Kernel choice and launch for one operand pairing: everything between the validated
// arguments of the C ABI and hipLaunchKernelGGL.  Included by dispatch_pair.hip, which is
// compiled once per pairing so that the four pairings build in parallel.
#ifndef FP8GEMM_DISPATCH_H
#define FP8GEMM_DISPATCH_H

#include <atomic>

#include "kernel_direct.h"
#include "kernel_ptile.h"
#include "kernel_skinny.h"
#include "kernel_tile.h"
#include "plan.h"

namespace fp8gemm_detail {

// ------------------------------------------------------------------ variants
// Tiled kernel shapes: <BM, BN, BK, waves_m, waves_n, stages, swizzle>.
using TileP2 = TileShape<256, 256, 128, 2, 2, 2, 3>;  // 2 x 64 KiB ring, 128x128 per wave
using TileP2h = TileShape<256, 256, 128, 2, 2, 2, 3, true>;   // the same on v_mfma_f32_16x16x128_f8f6f4
using TileT2h = TileShape<192, 256, 128, 2, 2, 2, 3, true>;   // 192 x 256 on that MFMA
using TileH3 = TileShape<128, 256, 128, 2, 2, 3, 3>;  // half-height tile, 3 x 48 KiB ring
using TileQ2 = TileShape<128, 128, 128, 2, 2, 2, 3>;  // quarter tile
using TileW3 = TileShape<256, 128, 128, 2, 2, 3, 3>;  // half-width tile, 3 x 48 KiB ring
using TileT2 = TileShape<192, 256, 128, 2, 2, 2, 3>;  // three-quarter-height tile: other tile counts
// weight streaming through the tiled kernel (one row of tiles, B read once with the non-temporal hint):
// deep rings, so that many bytes of B are in flight per CU
// (M=64 N=28672 K=8192, weights cold: 39.3 us against 50.0 us of the single-wave streaming kernel; rings of 4, 5
// and 6 slots run alike, 64-byte K tiles in an 8-deep ring 57 us, a 64 x 256 tile 54 us)
using TileE5 = TileShape<64, 128, 128, 1, 4, 5, 3>;    // up to 64 rows of A: four waves of 64 x 32, 5 x 24 KiB ring
using TileQ4s = TileShape<128, 128, 128, 2, 2, 4, 3>;  // up to 128 rows: the quarter tile with a 4 x 32 KiB ring

// blocked-ELL operands with blocks of 64 and 32 rows: tiles as tall as a block, four waves side by side
using TileB64 = TileShape<64, 256, 128, 1, 4, 3, 3>;   // 64 x 64 per wave, 3 x 40 KiB ring
using TileB32 = TileShape<32, 256, 128, 1, 4, 4, 3>;   // 32 x 64 per wave, 4 x 36 KiB ring

// Skinny kernel shapes: <MT, TN, BK, stages>.
template <int MT, int TN>
using SkinnyV0 = SkinnyShape<MT, TN, 128, 5>;
template <int MT, int TN>
using SkinnyV1 = SkinnyShape<MT, TN, 256, 4>;
template <int MT, int TN>
using SkinnyV4 = SkinnyShape<MT, TN, 512, 4, 80 * 1024>;
template <int MT, int TN>
using SkinnyV5 = SkinnyShape<MT, TN, 1024, 3, 80 * 1024>;

// Raises a kernel's dynamic LDS limit above the 64 KiB default.  Done once per kernel
// and device (the attribute call costs host time on every launch otherwise); KernelTag
// is a type unique to the kernel instantiation, it only keys the bookkeeping.
template <class KernelTag, class Kernel>
hipError_t allow_lds(Kernel kernel, int bytes)
{
    if (bytes <= 64 * 1024) return hipSuccess;
    static std::atomic<unsigned long long> done{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < 64;
    if (tracked && ((done.load(std::memory_order_acquire) >> dev) & 1ull)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && tracked) done.fetch_or(1ull << dev, std::memory_order_release);
    return e;
}

template <class S, int AF, int BF, bool KOVER, bool EX, bool BSTREAM, bool NOPF = false>
struct PtileKernelTag {};
template <class S, int AF, int BF>
struct SkinnyKernelTag {};
// ------------------------------------------------------------------ direct
template <int AF, int BF>
hipError_t launch_direct(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                         const OutSpec &spec, hipStream_t stream)
{
    const long gy = (m + 31) / 32, gx = (n + 31) / 32;
    if (gx * gy > 0x7FFFFFFFL) return hipErrorInvalidValue;       // 2^41 elements of C and more
    const bool vec_ok = (k % 16 == 0) && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) % 16 == 0);
    hipLaunchKernelGGL((gemm_direct_kernel<AF, BF>), dim3((unsigned)(gx * gy)), dim3(64), 0, stream,
                       m, k, n, a, b, out, (int)gx, vec_ok ? 1 : 0, spec);
    return hipGetLastError();
}

// ------------------------------------------------------------------ tiled
// Start skew between the tile rows of an XCD's window, in ticks of 10 ns (see the kernel).  It
// costs three times the skew once and shortens every epilogue (8192^3: 368 -> 365 us with 1.5 to
// 2.5 us, 375 us with 4 us), so it is used from four rounds of whole tiles on.
inline int start_skew(const PtileWork &w)
{
    return w.bulk / 256 >= 4 ? 200 : 0;
}

// persistent form: one workgroup per CU walks its share of the work list; the K slices'
// partial sums go through the scratch buffer and a reduction pass
template <class S, int AF, int BF, bool KOVER, bool EX, bool BSTREAM, bool NOPF = false>
hipError_t launch_ptile_work(const PtileWork &w, int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                             float *ws, int *counters, int rotate, const OutSpec &spec, hipStream_t stream)
{
    auto kernel = gemm_ptile_kernel<S, AF, BF, KOVER, EX, BSTREAM, NOPF>;
    constexpr int kLdsBytes = S::PTILE_LDS_BYTES + 256 + 16;      // + the landing place of the L2 prefetches + a flag
    hipError_t e = allow_lds<PtileKernelTag<S, AF, BF, KOVER, EX, BSTREAM, NOPF>>(kernel, kLdsBytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(8 * w.slots)), dim3(S::THREADS), kLdsBytes, stream,
                       m, k, n, a, b, out, ws, counters, w.tiles_m, w.tiles_n, w.GM, tile_column_block(w.tiles_n, m, n, k), w.bulk, w.tail,
                       w.nsplit, w.rounds, rotate | (start_skew(w) << 8), spec);
    return hipGetLastError();
}

// STREAM_TOO: this shape is also compiled with non-temporal loads of B, used when C has a
// single row of tiles (every byte of B is then read by exactly one workgroup)
template <class S, int AF, int BF, bool KOVER, bool EX, bool STREAM_TOO>
hipError_t launch_ptile_shape_k(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                                int nsplit, bool split_all, int rotate, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
    if (k % 16 != 0 || k > (1 << 23) || nsplit < 1 || nsplit > (k + S::BK - 1) / S::BK) return hipErrorInvalidValue;
    const PtileWork w = ptile_work(m, n, S::BM, S::BN, nsplit, split_all);
    if (!w.ok) return hipErrorInvalidValue;
    // Scratch of a K-sliced launch: arrival counters, then the partial sums.  For tiles up to
    // 128 x 128, where the counters can be relied on (see Workspace), the slice of a tile that
    // arrives last adds the slices up inside the kernel; otherwise a reduction kernel follows.
    // (One CU adding up the slices of a larger tile is slower than the reduction kernel, which
    // spreads that over the chip.  MI355X, M=256, weights cold, sum in the kernel / by the reduction
    // kernel: 128 x 256 tiles in 3 slices at N=10240 K=8192 41.3 / 38.2 us, 256 x 128 in 4 slices at
    // N=8192 K=28672 75.1 / 69.8 us, 256 x 256 in 2 slices at N=28672 K=8192 76.2 / 73.0 us;
    // for a 64 x 128 tile it is 128 KiB per tile and 1 to 2 us faster than a second launch.)
    constexpr bool kSumInKernel = ptile_sums_slices_in_kernel<S>;
    float *base = nullptr, *ws = nullptr;
    int *counters = nullptr;
    if (w.nsplit > 1) {
        void *p = nullptr;
        hipError_t e = wsp.get(ptile_scratch_bytes(w, S::BM, S::BN), &p);
        if (e != hipSuccess) return e;
        base = static_cast<float *>(p);
        ws = base + kSliceCounterBytes / sizeof(float);
        // (the kernel addresses the partial sums through a buffer window with 32-bit offsets)
        const bool window_fits = ptile_scratch_bytes(w, S::BM, S::BN) <= 0xFFFFFFFFull;
        if (kSumInKernel && wsp.counters_zero() && w.tail <= kMaxSliceCounters && window_fits) counters = static_cast<int *>(p);
    }
    hipError_t e;
    // the compute-bound tiles on operands that both stay in the last-level cache: no L2 prefetch (see the kernel)
    const bool cached = (size_t)m * k + (size_t)n * k <= ((size_t)192 << 20);
    if constexpr (S::MF16 && !KOVER && !EX) {
        if (cached) {
            e = launch_ptile_work<S, AF, BF, false, false, false, true>(w, m, k, n, a, b, out, ws, counters, rotate, spec, stream);
            if (e != hipSuccess || w.nsplit == 1 || counters) return e;
            return launch_tile_slices_reduce(base, out, m, n, k, S::BM, S::BN, w, spec, stream);
        }
    }
    if constexpr (STREAM_TOO && !KOVER) {
        e = w.tiles_m == 1 ? launch_ptile_work<S, AF, BF, KOVER, EX, true>(w, m, k, n, a, b, out, ws, counters, rotate, spec, stream)
                           : launch_ptile_work<S, AF, BF, KOVER, EX, false>(w, m, k, n, a, b, out, ws, counters, rotate, spec, stream);
    } else {
        e = launch_ptile_work<S, AF, BF, KOVER, EX, false>(w, m, k, n, a, b, out, ws, counters, rotate, spec, stream);
    }
    if (e != hipSuccess || w.nsplit == 1 || counters) return e;
    return launch_tile_slices_reduce(base, out, m, n, k, S::BM, S::BN, w, spec, stream);
}

// OVERHANG_TOO: this shape is also compiled for a K that is not a multiple of its K tile.
// EX_TOO: ... and for the extended epilogue (scale, 16-bit output).
template <class S, int AF, int BF, bool OVERHANG_TOO, bool EX_TOO, bool STREAM_TOO = false>
hipError_t launch_ptile_shape(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                              int nsplit, bool split_all, int rotate, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
    const bool over = k % S::BK != 0;
    if (plain_output(spec)) {
        if (!over)
            return launch_ptile_shape_k<S, AF, BF, false, false, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
        if constexpr (OVERHANG_TOO)
            return launch_ptile_shape_k<S, AF, BF, true, false, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
        return hipErrorInvalidValue;
    }
    if constexpr (EX_TOO) {
        if (!over)
            return launch_ptile_shape_k<S, AF, BF, false, true, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
        if constexpr (OVERHANG_TOO)
            return launch_ptile_shape_k<S, AF, BF, true, true, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    }
    return hipErrorInvalidValue;
}

template <int AF, int BF>
hipError_t launch_tile(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                       int variant, int nsplit, bool split_all, int rotate, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
    switch (variant) {
    case 0: return launch_ptile_shape<TileP2, AF, BF, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 5: return launch_ptile_shape<TileH3, AF, BF, true, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 6: return launch_ptile_shape<TileQ2, AF, BF, true, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 8: return launch_ptile_shape<TileW3, AF, BF, false, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 9: return launch_ptile_shape<TileT2, AF, BF, false, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 13:
        if (!p2h_ok(k, nsplit)) return hipErrorInvalidValue;
        return launch_ptile_shape<TileP2h, AF, BF, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 14:
        if (!p2h_ok(k, nsplit)) return hipErrorInvalidValue;
        return launch_ptile_shape<TileT2h, AF, BF, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 15: return launch_ptile_shape<TileE5, AF, BF, false, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    case 16: return launch_ptile_shape<TileQ4s, AF, BF, false, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, wsp, stream);
    default: return hipErrorInvalidValue;
    }
}

// ------------------------------------------------------------------ blocked-ELL A through the tiled kernel
template <class S, int AF, int BF>
struct PtileBellKernelTag {};

template <class S, int AF, int BF>
hipError_t launch_ptile_bell(int m, int kell, int n, const uint8_t *values, const uint8_t *b, float *out, const BellSpec &bell,
                             int nsplit, bool split_all, int rotate, Workspace &wsp, hipStream_t stream)
{
    const bool small = S::BM < 128;              // blocks below a K tile: any stored row length, sub-blocks of 32 bytes or more
    if (bell.block % S::BM != 0 || (small ? bell.sub < 32 : (bell.block % S::BK != 0 || kell % S::BK != 0)) || kell % 16 != 0 ||
        kell > (1 << 23) || bell.kb > (1 << 23) || nsplit < 1 || nsplit > (kell + S::BK - 1) / S::BK)
        return hipErrorInvalidValue;
    const PtileWork w = ptile_work(m, n, S::BM, S::BN, nsplit, split_all);
    if (!w.ok) return hipErrorInvalidValue;
    float *base = nullptr, *ws = nullptr;
    int *counters = nullptr;
    if (w.nsplit > 1) {
        void *p = nullptr;
        hipError_t e = wsp.get(ptile_scratch_bytes(w, S::BM, S::BN), &p);
        if (e != hipSuccess) return e;
        base = static_cast<float *>(p);
        ws = base + kSliceCounterBytes / sizeof(float);
        const bool window_fits = ptile_scratch_bytes(w, S::BM, S::BN) <= 0xFFFFFFFFull;
        if (ptile_sums_slices_in_kernel<S> && wsp.counters_zero() && w.tail <= kMaxSliceCounters && window_fits)
            counters = static_cast<int *>(p);
    }
    auto kernel = gemm_ptile_bell_kernel<S, AF, BF>;
    constexpr int kLdsBytes = S::PTILE_LDS_BYTES + 256 + 16;
    hipError_t e = allow_lds<PtileBellKernelTag<S, AF, BF>>(kernel, kLdsBytes);
    if (e != hipSuccess) return e;
    const int cb = tile_column_block(w.tiles_n, m, n, kell);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(8 * w.slots)), dim3(S::THREADS), kLdsBytes, stream, m, kell, n, values, b,
                       static_cast<void *>(out), ws, counters, w.tiles_m, w.tiles_n, w.GM, cb, w.bulk, w.tail, w.nsplit, w.rounds,
                       rotate | (start_skew(w) << 8), bell);
    e = hipGetLastError();
    if (e != hipSuccess || w.nsplit == 1 || counters) return e;
    const OutSpec plain = {1.0f, nullptr, nullptr, FP8GEMM_DEV_OUT_F32, 0.0f, nullptr, FP8GEMM_DEV_OUT_F32, nullptr, nullptr, nullptr};
    return launch_tile_slices_reduce(base, out, m, n, kell, S::BM, S::BN, w, plain, stream);
}

template <int AF, int BF>
hipError_t dispatch_bell(int m, int kell, int n, const uint8_t *values, const uint8_t *b, float *out, const BellSpec &bell,
                         Workspace &wsp, hipStream_t stream)
{
    if (bell.block % 128 != 0) {
        // small blocks: tiles as tall as a block; too few tiles for the chip are cut into K slices
        const int bm = bell.block % 64 == 0 ? 64 : 32;
        const long tiles = (long)(m / bm) * ((n + 255) / 256);
        const int kt = (kell + 127) / 128;
        int nsplit = 1;
        if (tiles < 256) {
            nsplit = (int)((256 + tiles - 1) / tiles);
            if (nsplit > kt / 8) nsplit = kt / 8;
            if (nsplit < 1) nsplit = 1;
        }
        if (bm == 64) return launch_ptile_bell<TileB64, AF, BF>(m, kell, n, values, b, out, bell, nsplit, nsplit > 1, 2, wsp, stream);
        return launch_ptile_bell<TileB32, AF, BF>(m, kell, n, values, b, out, bell, nsplit, nsplit > 1, 2, wsp, stream);
    }
    // tile shapes whose rows share one block row: 128-row tiles, and 256-row ones where the blocks are that tall
    unsigned allowed = (1u << 5) | (1u << 6);
    if (bell.block % 256 == 0) allowed |= (1u << 0) | (1u << 13);
    const TilePlan p = plan_tile(m, kell, n, allowed);
    switch (p.variant) {
    case 0: return launch_ptile_bell<TileP2, AF, BF>(m, kell, n, values, b, out, bell, p.nsplit, p.split_all, p.rotate, wsp, stream);
    case 5: return launch_ptile_bell<TileH3, AF, BF>(m, kell, n, values, b, out, bell, p.nsplit, p.split_all, p.rotate, wsp, stream);
    case 6: return launch_ptile_bell<TileQ2, AF, BF>(m, kell, n, values, b, out, bell, p.nsplit, p.split_all, p.rotate, wsp, stream);
    case 13:
        if (!p2h_ok(kell, p.nsplit)) return hipErrorInvalidValue;
        return launch_ptile_bell<TileP2h, AF, BF>(m, kell, n, values, b, out, bell, p.nsplit, p.split_all, p.rotate, wsp, stream);
    default: return hipErrorInvalidValue;
    }
}

// ------------------------------------------------------------------ skinny
template <class S, int AF, int BF>
hipError_t launch_skinny_shape(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                               int nsplit, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
    if (m > S::MP || n % S::NP != 0 || nsplit < 1 || k % nsplit != 0 || (k / nsplit) % S::BK != 0)
        return hipErrorInvalidValue;
    const int ngroups = n / S::NP;
    const int kchunk = k / nsplit;
    void *dst = out;
    if (nsplit > 1) {
        void *ws = nullptr;
        // (the start of every scratch buffer belongs to the tiled kernel's arrival counters)
        hipError_t e = wsp.get(kSliceCounterBytes + (size_t)nsplit * m * n * sizeof(float), &ws);
        if (e != hipSuccess) return e;
        dst = static_cast<unsigned char *>(ws) + kSliceCounterBytes;
    }
    auto kernel = gemm_skinny_kernel<S, AF, BF>;
    hipError_t e = allow_lds<SkinnyKernelTag<S, AF, BF>>(kernel, S::LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(ngroups * nsplit)), dim3(64), S::LDS_BYTES, stream,
                       m, k, n, a, b, dst, ngroups, kchunk, nsplit, spec);
    e = hipGetLastError();
    if (e != hipSuccess || nsplit == 1) return e;
    return launch_reduce(static_cast<const float *>(dst), out, (size_t)m * n, nsplit, spec, stream);
}

template <template <int, int> class V, int AF, int BF>
hipError_t launch_skinny_mt(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                            const SkinnyPlan &p, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
#define SK(MT, TN) \
    if (p.mt == MT && p.tn == TN) return launch_skinny_shape<V<MT, TN>, AF, BF>(m, k, n, a, b, out, p.nsplit, spec, wsp, stream);
    SK(1, 1) SK(1, 2) SK(1, 4)
#undef SK
    return hipErrorInvalidValue;
}

template <int AF, int BF>
hipError_t launch_skinny(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                         const SkinnyPlan &p, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
    switch (p.variant) {
    case 0: return launch_skinny_mt<SkinnyV0, AF, BF>(m, k, n, a, b, out, p, spec, wsp, stream);
    case 1: return launch_skinny_mt<SkinnyV1, AF, BF>(m, k, n, a, b, out, p, spec, wsp, stream);
    case 4: return launch_skinny_mt<SkinnyV4, AF, BF>(m, k, n, a, b, out, p, spec, wsp, stream);
    case 5: return launch_skinny_mt<SkinnyV5, AF, BF>(m, k, n, a, b, out, p, spec, wsp, stream);
    default: return hipErrorInvalidValue;
    }
}

template <int AF, int BF>
hipError_t dispatch(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                    int algo, int variant, int nsplit, const OutSpec &spec, Workspace &wsp, hipStream_t stream)
{
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) % 16) == 0;
    if (algo == FP8GEMM_ALGO_AUTO) {
        algo = select_algo(m, k, n);
        if (!aligned) algo = FP8GEMM_ALGO_DIRECT;
    }
    switch (algo) {
    case FP8GEMM_ALGO_DIRECT:
        return launch_direct<AF, BF>(m, k, n, a, b, out, spec, stream);
    case FP8GEMM_ALGO_TILE: {
        if (!aligned || k % 16 != 0 || k > (1 << 23)) return hipErrorInvalidValue;
        TilePlan p = plan_tile(m, k, n);
        if (variant >= 0) {
            // tuning hook: variant = shape index + 16 * (1 + K-walk rotation mode); a bare
            // shape index keeps the plan's rotation and runs unsplit unless split_k says otherwise
            if (variant >= 32) {
                p.rotate = variant / 32 - 1;
                if (p.rotate > 2) return hipErrorInvalidValue;
            }
            p.variant = variant % 32;
            p.nsplit = 1;
            p.split_all = false;
        }
        if (nsplit > 0) {          // forced: K slices for every tile
            p.nsplit = nsplit;
            p.split_all = true;
        } else if (nsplit < 0) {   // forced: K slices for the tiles that do not fill a round
            p.nsplit = -nsplit;
            p.split_all = false;
        }
        return launch_tile<AF, BF>(m, k, n, a, b, out, p.variant, p.nsplit, p.split_all, p.rotate, spec, wsp, stream);
    }
    case FP8GEMM_ALGO_SKINNY: {
        if (!aligned || !skinny_ok(m, k, n)) return hipErrorInvalidValue;
        SkinnyPlan p = plan_skinny(m, k, n);
        if (variant >= 0) {
            // tuning hook: variant = shape_index + 16 * columns-per-wave/16 (0 keeps the plan's)
            p.variant = variant % 16;
            if (variant / 16 > 0) p.tn = variant / 16;
        }
        if (nsplit > 0) p.nsplit = nsplit;
        if (nsplit < 0) return hipErrorInvalidValue;
        return launch_skinny<AF, BF>(m, k, n, a, b, out, p, spec, wsp, stream);
    }
    default:
        return hipErrorInvalidValue;
    }
}

}  // namespace fp8gemm_detail

#endif  // FP8GEMM_DISPATCH_H
