// C ABI, argument validation and kernel selection of the gfx950 FP8 GEMM
// library.  The entry points are declared in include/fp8gemm.h; together they
// stand where the launch functions of the reference stand
// (GEMM/include/gemm.cuh:11-55, defined at GEMM/src/gemm.cu:263-285 and
// siblings): validate, pick a kernel, launch asynchronously, return the launch
// status.
#include "fp8gemm.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

#include "kernel_direct.h"
#include "kernel_ptile.h"
#include "kernel_reduce.h"
#include "kernel_skinny.h"
#include "kernel_tile.h"

namespace {

constexpr int kVersion = 100;
constexpr int kMaxDevices = 64;

// ------------------------------------------------------------------ variants
// Tiled kernel shapes: <BM, BN, BK, waves_m, waves_n, stages, swizzle>.
using TileP2 = TileShape<256, 256, 128, 2, 2, 2, 3>;  // persistent, 2 x 64 KiB ring, 128x128 per wave
using TileP2h = TileShape<256, 256, 128, 2, 2, 2, 3, true>;   // the same on v_mfma_f32_16x16x128_f8f6f4
using TileT2h = TileShape<192, 256, 128, 2, 2, 2, 3, true>;   // 192 x 256 on that MFMA
using TileP4 = TileShape<256, 256, 64, 2, 2, 4, 2>;   // persistent, 4 x 32 KiB ring
using TileP8 = TileShape<256, 256, 128, 2, 4, 2, 3>;  // persistent, 8 waves, 128x64 per wave
using TileS2 = TileShape<128, 128, 128, 2, 2, 2, 3>;  // one tile per workgroup, for small problems
using TileS4 = TileShape<128, 128, 128, 2, 2, 4, 3>;
using TileH3 = TileShape<128, 256, 128, 2, 2, 3, 3>;  // persistent, half-height tile, 3 x 48 KiB ring
using TileQ2 = TileShape<128, 128, 128, 2, 2, 2, 3>;  // persistent, quarter tile
using TileS64 = TileShape<128, 128, 64, 2, 2, 4, 2>;  // one tile per workgroup, 64-byte K tiles
using TileW3 = TileShape<256, 128, 128, 2, 2, 3, 3>;  // persistent, half-width tile, 3 x 48 KiB ring
using TileT2 = TileShape<192, 256, 128, 2, 2, 2, 3>;  // persistent, three-quarter-height tile: other tile counts
// the 4-deep rings of 64-byte K tiles behind the stage-4 entry points, same tile shapes
using TileT4 = TileShape<192, 256, 64, 2, 2, 4, 2>;
using TileH4 = TileShape<128, 256, 64, 2, 2, 4, 2>;
using TileQ4 = TileShape<128, 128, 64, 2, 2, 4, 2>;
constexpr int kNumTileVariants = 15;              // 0 P2, 1 P4, 2 P8, 3 S2, 4 S4, 5 H3, 6 Q2, 7 S64, 8 W3, 9 T2, 10 T4, 11 H4, 12 Q4, 13 P2h, 14 T2h

// Skinny kernel shapes: <MT, TN, BK, stages>.
template <int MT, int TN>
using SkinnyV0 = SkinnyShape<MT, TN, 128, 5>;
template <int MT, int TN>
using SkinnyV1 = SkinnyShape<MT, TN, 256, 4>;
template <int MT, int TN>
using SkinnyV2 = SkinnyShape<MT, TN, 128, 8>;
template <int MT, int TN>
using SkinnyV3 = SkinnyShape<MT, TN, 256, 6>;
template <int MT, int TN>
using SkinnyV4 = SkinnyShape<MT, TN, 512, 4, 80 * 1024>;
template <int MT, int TN>
using SkinnyV5 = SkinnyShape<MT, TN, 1024, 3, 80 * 1024>;
constexpr int kNumSkinnyVariants = 6;

struct Scratch {
    void *ptr = nullptr;
    size_t bytes = 0;
};
Scratch g_scratch[kMaxDevices];
std::mutex g_scratch_mutex;

hipError_t scratch_get(size_t bytes, void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    Scratch &s = g_scratch[dev];
    if (s.bytes < bytes) {
        if (s.ptr) {
            // earlier launches may still be reading the old buffer
            e = hipDeviceSynchronize();
            if (e != hipSuccess) return e;
            (void)hipFree(s.ptr);
            s.ptr = nullptr;
            s.bytes = 0;
        }
        e = hipMalloc(&s.ptr, bytes);
        if (e != hipSuccess) {
            s.ptr = nullptr;
            return e;
        }
        s.bytes = bytes;
    }
    *out = s.ptr;
    return hipSuccess;
}

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

template <class S, int AF, int BF>
struct TileKernelTag {};
template <class S, int AF, int BF, bool KOVER, bool EX, bool BSTREAM>
struct PtileKernelTag {};
template <class S, int AF, int BF>
struct SkinnyKernelTag {};

// out[i] = sum over the nsplit planes of ws, on `stream`
hipError_t launch_reduce(const float *ws, void *out, size_t count, int nsplit, const OutSpec &spec, hipStream_t stream)
{
    const bool vec = count % 4 == 0 &&
                     ((reinterpret_cast<uintptr_t>(ws) | reinterpret_cast<uintptr_t>(out)) % 16) == 0;
    if (vec) {
        const size_t count4 = count / 4;
        hipLaunchKernelGGL(gemm_splitk_reduce4_kernel, dim3((unsigned)((count4 + 255) / 256)), dim3(256), 0, stream,
                           reinterpret_cast<const v4f *>(ws), out, count4, nsplit, spec);
    } else {
        hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream,
                           ws, out, count, nsplit, spec);
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------ direct
template <int AF, int BF>
hipError_t launch_direct(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                         const OutSpec &spec, hipStream_t stream)
{
    const long gy = (m + 31) / 32, gx = (n + 31) / 32;
    if (gy > 65535) return hipErrorInvalidValue;
    const bool vec_ok = (k % 16 == 0) && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) % 16 == 0);
    hipLaunchKernelGGL((gemm_direct_kernel<AF, BF>), dim3((unsigned)gx, (unsigned)gy), dim3(64), 0, stream,
                       m, k, n, a, b, out, vec_ok ? 1 : 0, spec);
    return hipGetLastError();
}

// ------------------------------------------------------------------ tiled
template <class S, int AF, int BF>
hipError_t launch_tile_shape(int m, int k, int n, const uint8_t *a, const uint8_t *b, float *out,
                             hipStream_t stream)
{
    if (k % S::BK != 0) return hipErrorInvalidValue;
    const int tiles_m = (m + S::BM - 1) / S::BM;
    const int tiles_n = (n + S::BN - 1) / S::BN;
    // XCD-local super-blocks of tiles: 32 CUs per XCD -> blocks of up to 32 tiles,
    // shaped to balance A-panel and B-panel reuse.
    int GM = 4, GN = 8;
    if (tiles_m < GM) { GM = tiles_m; }
    if (tiles_n < GN) { GN = tiles_n; }
    const int nb = ((tiles_m + GM - 1) / GM) * ((tiles_n + GN - 1) / GN);
    const long grid = (long)((nb + 7) / 8) * 8 * GM * GN;
    auto kernel = gemm_tile_kernel<S, AF, BF>;
    hipError_t e = allow_lds<TileKernelTag<S, AF, BF>>(kernel, S::LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(S::THREADS), S::LDS_BYTES, stream,
                       m, k, n, a, b, out, tiles_m, tiles_n, GM, GN);
    return hipGetLastError();
}

// Work list of the persistent kernel for a tile shape: `bulk` tiles (a multiple of 256)
// run as whole items, 256 per round; the remaining `tail` tiles are cut into nsplit K
// slices each.  split_all cuts every tile (bulk = 0); otherwise only the tiles that do
// not fill a round are cut.
struct PtileWork {
    int tiles_m, tiles_n, GM, bulk, tail, nsplit, rounds, slots;
    bool ok;
};
PtileWork ptile_work(int m, int n, int bm, int bn, int nsplit, bool split_all)
{
    PtileWork w = {};
    w.tiles_m = (m + bm - 1) / bm;
    w.tiles_n = (n + bn - 1) / bn;
    const long nt = (long)w.tiles_m * w.tiles_n;
    w.ok = nt <= (1L << 30) / 16;
    if (!w.ok) return w;
    w.GM = w.tiles_m < 4 ? w.tiles_m : 4;
    w.bulk = (split_all && nsplit > 1) ? 0 : (int)(nt / 256) * 256;
    w.tail = (int)nt - w.bulk;
    w.nsplit = w.tail > 0 ? nsplit : 1;
    const long tail_items = (long)w.tail * w.nsplit;
    w.rounds = w.bulk / 256 + (int)((tail_items + 255) / 256);
    const long first_tail_round = tail_items < 256 ? tail_items : 256;
    w.slots = w.bulk > 0 ? 32 : (int)((first_tail_round + 7) / 8);
    return w;
}

// Column blocking of the tile numbering.  A round of 256 tiles in strips of 4 tile rows spans
// 64 tile columns: where B (n x k bytes) no longer fits the 256 MB last-level cache, every
// round streams all of it from HBM.  Blocks of 16 tile columns make a round a 16 x 16 window
// instead (16 + 16 operand panels instead of 4 + 64) -- at the price of walking all of A once
// per column block, so only where A is small enough to stay in that cache meanwhile
// (M=8192, N=K=16384: 2.87 -> 3.2 PFLOP/s; with A as large as B it gains nothing, and where
// B still fits the cache it costs 3-5 %).
int tile_column_block(int tiles_n, int m, int n, int k)
{
    const bool b_is_large = (size_t)n * (size_t)k >= ((size_t)192 << 20);
    const bool a_is_small = (size_t)m * (size_t)k <= ((size_t)160 << 20);
    return (b_is_large && a_is_small && tiles_n > 16) ? 16 : tiles_n;
}

size_t ptile_scratch_bytes(const PtileWork &w, int bm, int bn)
{
    return w.nsplit > 1 ? (size_t)w.nsplit * w.tail * bm * bn * sizeof(float) : 0;
}

// persistent form: one workgroup per CU walks its share of the work list; the K slices'
// partial sums go through the scratch buffer and a reduction pass
template <class S, int AF, int BF, bool KOVER, bool EX, bool BSTREAM>
hipError_t launch_ptile_work(const PtileWork &w, int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                             float *ws, int rotate, const OutSpec &spec, hipStream_t stream)
{
    auto kernel = gemm_ptile_kernel<S, AF, BF, KOVER, EX, BSTREAM>;
    hipError_t e = allow_lds<PtileKernelTag<S, AF, BF, KOVER, EX, BSTREAM>>(kernel, S::PTILE_LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(8 * w.slots)), dim3(S::THREADS), S::PTILE_LDS_BYTES, stream,
                       m, k, n, a, b, out, ws, w.tiles_m, w.tiles_n, w.GM, tile_column_block(w.tiles_n, m, n, k), w.bulk, w.tail,
                       w.nsplit, w.rounds, rotate, spec);
    return hipGetLastError();
}

// STREAM_TOO: this shape is also compiled with non-temporal loads of B, used when C has a
// single row of tiles (every byte of B is then read by exactly one workgroup)
template <class S, int AF, int BF, bool KOVER, bool EX, bool STREAM_TOO>
hipError_t launch_ptile_shape_k(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                                int nsplit, bool split_all, int rotate, const OutSpec &spec, hipStream_t stream)
{
    if (k % 16 != 0 || k > (1 << 23) || nsplit < 1 || nsplit > (k + S::BK - 1) / S::BK) return hipErrorInvalidValue;
    const PtileWork w = ptile_work(m, n, S::BM, S::BN, nsplit, split_all);
    if (!w.ok) return hipErrorInvalidValue;
    float *ws = nullptr;
    if (w.nsplit > 1) {
        void *p = nullptr;
        hipError_t e = scratch_get(ptile_scratch_bytes(w, S::BM, S::BN), &p);
        if (e != hipSuccess) return e;
        ws = static_cast<float *>(p);
    }
    hipError_t e;
    if constexpr (STREAM_TOO && !KOVER) {
        e = w.tiles_m == 1 ? launch_ptile_work<S, AF, BF, KOVER, EX, true>(w, m, k, n, a, b, out, ws, rotate, spec, stream)
                           : launch_ptile_work<S, AF, BF, KOVER, EX, false>(w, m, k, n, a, b, out, ws, rotate, spec, stream);
    } else {
        e = launch_ptile_work<S, AF, BF, KOVER, EX, false>(w, m, k, n, a, b, out, ws, rotate, spec, stream);
    }
    if (e != hipSuccess || w.nsplit == 1) return e;
    const size_t threads = (size_t)w.tail * (S::BM * S::BN / 4);
    hipLaunchKernelGGL(gemm_tile_slices_reduce_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                       ws, out, m, n, S::BM, S::BN, w.tiles_m, w.tiles_n, w.GM, tile_column_block(w.tiles_n, m, n, k), w.bulk, w.tail,
                       w.nsplit, spec);
    return hipGetLastError();
}

bool plain_output(const OutSpec &spec)
{
    return spec.type == FP8GEMM_DEV_OUT_F32 && spec.alpha == 1.0f && !spec.a_scale && !spec.b_scale;
}

// OVERHANG_TOO: this shape is also compiled for a K that is not a multiple of its K tile.
// EX_TOO: ... and for the extended epilogue (scale, 16-bit output).
template <class S, int AF, int BF, bool OVERHANG_TOO, bool EX_TOO, bool STREAM_TOO = false>
hipError_t launch_ptile_shape(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                              int nsplit, bool split_all, int rotate, const OutSpec &spec, hipStream_t stream)
{
    const bool over = k % S::BK != 0;
    if (plain_output(spec)) {
        if (!over)
            return launch_ptile_shape_k<S, AF, BF, false, false, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
        if constexpr (OVERHANG_TOO)
            return launch_ptile_shape_k<S, AF, BF, true, false, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
        return hipErrorInvalidValue;
    }
    if constexpr (EX_TOO) {
        if (!over)
            return launch_ptile_shape_k<S, AF, BF, false, true, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
        if constexpr (OVERHANG_TOO)
            return launch_ptile_shape_k<S, AF, BF, true, true, STREAM_TOO>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    }
    return hipErrorInvalidValue;
}

// The 16x16x128 forms of the 256 x 256 and 192 x 256 tiles need whole 128-byte K tiles, at least two per
// work item (a tile, or one of its nsplit K slices).
bool p2h_ok(int k, int nsplit)
{
    return k % 128 == 0 && (k / 128) / nsplit >= 2;
}

template <int AF, int BF>
hipError_t launch_tile(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                       int variant, int nsplit, bool split_all, int rotate, const OutSpec &spec, hipStream_t stream)
{
    const bool persistent = !(variant == 3 || variant == 4 || variant == 7);
    if (!persistent && nsplit != 1) return hipErrorInvalidValue;   // K slices only in the persistent kernels
    // the one-tile-per-workgroup kernels write bare fp32 sums only
    if (!persistent && !plain_output(spec)) return hipErrorInvalidValue;
    switch (variant) {
    case 0: return launch_ptile_shape<TileP2, AF, BF, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 1: return launch_ptile_shape<TileP4, AF, BF, true, false>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 2: return launch_ptile_shape<TileP8, AF, BF, false, false>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 3: return launch_tile_shape<TileS2, AF, BF>(m, k, n, a, b, static_cast<float *>(out), stream);
    case 4: return launch_tile_shape<TileS4, AF, BF>(m, k, n, a, b, static_cast<float *>(out), stream);
    case 5: return launch_ptile_shape<TileH3, AF, BF, true, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 6: return launch_ptile_shape<TileQ2, AF, BF, true, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 7: return launch_tile_shape<TileS64, AF, BF>(m, k, n, a, b, static_cast<float *>(out), stream);
    case 8: return launch_ptile_shape<TileW3, AF, BF, false, true, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 9: return launch_ptile_shape<TileT2, AF, BF, false, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 10: return launch_ptile_shape<TileT4, AF, BF, false, false>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 11: return launch_ptile_shape<TileH4, AF, BF, false, false>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 12: return launch_ptile_shape<TileQ4, AF, BF, false, false>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 13:
        if (!p2h_ok(k, nsplit)) return hipErrorInvalidValue;
        return launch_ptile_shape<TileP2h, AF, BF, false, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    case 14:
        if (!p2h_ok(k, nsplit)) return hipErrorInvalidValue;
        return launch_ptile_shape<TileT2h, AF, BF, false, true>(m, k, n, a, b, out, nsplit, split_all, rotate, spec, stream);
    default: return hipErrorInvalidValue;
    }
}

// ------------------------------------------------------------------ skinny
struct SkinnyPlan {
    int mt, tn, variant, nsplit;
};

template <class S, int AF, int BF>
hipError_t launch_skinny_shape(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                               int nsplit, const OutSpec &spec, hipStream_t stream)
{
    if (m > S::MP || n % S::NP != 0 || nsplit < 1 || k % nsplit != 0 || (k / nsplit) % S::BK != 0)
        return hipErrorInvalidValue;
    const int ngroups = n / S::NP;
    const int kchunk = k / nsplit;
    void *dst = out;
    if (nsplit > 1) {
        void *ws = nullptr;
        hipError_t e = scratch_get((size_t)nsplit * m * n * sizeof(float), &ws);
        if (e != hipSuccess) return e;
        dst = ws;
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
                            const SkinnyPlan &p, const OutSpec &spec, hipStream_t stream)
{
#define SK(MT, TN) \
    if (p.mt == MT && p.tn == TN) return launch_skinny_shape<V<MT, TN>, AF, BF>(m, k, n, a, b, out, p.nsplit, spec, stream);
    SK(1, 1) SK(1, 2) SK(1, 4)
    SK(2, 1) SK(2, 2) SK(2, 4)
    SK(3, 1) SK(3, 2) SK(3, 4)
    SK(4, 1) SK(4, 2) SK(4, 4)
#undef SK
    return hipErrorInvalidValue;
}

template <int AF, int BF>
hipError_t launch_skinny(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                         const SkinnyPlan &p, const OutSpec &spec, hipStream_t stream)
{
    switch (p.variant) {
    case 0: return launch_skinny_mt<SkinnyV0, AF, BF>(m, k, n, a, b, out, p, spec, stream);
    case 1: return launch_skinny_mt<SkinnyV1, AF, BF>(m, k, n, a, b, out, p, spec, stream);
    case 2: return launch_skinny_mt<SkinnyV2, AF, BF>(m, k, n, a, b, out, p, spec, stream);
    case 3: return launch_skinny_mt<SkinnyV3, AF, BF>(m, k, n, a, b, out, p, spec, stream);
    case 4: return launch_skinny_mt<SkinnyV4, AF, BF>(m, k, n, a, b, out, p, spec, stream);
    case 5: return launch_skinny_mt<SkinnyV5, AF, BF>(m, k, n, a, b, out, p, spec, stream);
    default: return hipErrorInvalidValue;
    }
}

bool skinny_ok(int m, int k, int n)
{
    return m <= 64 && n % 16 == 0 && k % 128 == 0;
}

// Picks columns per wave, LDS shape and split-K factor.  Measured on MI355X with
// operands that are cold in every cache.  Up to 32 rows of A the HBM pipe is fullest
// with one to two fat streams per CU (256..512 streams, each with a deep LDS ring)
// rather than many thin ones, and a split-K pass costs 10 % and more, so K is cut only
// when the columns alone give too few streams.  From 33 rows on a stream spends most
// of its LDS ring on A: the widest column group (64 columns) keeps the share of B up,
// and about two streams per CU hide the longer MFMA phases, even at the price of K
// slices.  Long K steps (512 bytes per row and load group) help a little.
SkinnyPlan plan_skinny(int m, int k, int n)
{
    SkinnyPlan p;
    p.mt = (m + 15) / 16;
    const int ksteps = k / 128;
    int tn = 4, split = 1;
    if (p.mt >= 3) {
        while (n % (16 * tn) != 0) tn /= 2;       // n % 16 == 0 is guaranteed by the caller
        // slices shorter than 4 KiB of K lose more to their ramp than the extra streams gain
        while ((long)(n / (16 * tn)) * split < 448 && split < 16 && ksteps % (2 * split) == 0 && ksteps / (2 * split) >= 32)
            split *= 2;
    } else {
        while (tn > 1 && (n % (16 * tn) != 0 || n / (16 * tn) < 256)) tn /= 2;
        while (n % (16 * tn) != 0) tn /= 2;
        while ((long)(n / (16 * tn)) * split < 192 && split < 16 && ksteps % (2 * split) == 0 && ksteps / (2 * split) >= 8)
            split *= 2;
    }
    p.tn = tn;
    p.nsplit = split;
    const int kchunk = k / split;
    // fat streams (64 columns) run best on 128-byte K steps in a deep ring; thinner ones want
    // longer K steps, so that a ring stage still holds 16 KiB or more
    p.variant = (tn == 4 && p.mt <= 3) ? 0 : (kchunk % 512 == 0) ? 4 : (kchunk % 256 == 0) ? 1 : 0;
    return p;
}

int select_algo(int m, int k, int n)
{
    if (skinny_ok(m, k, n)) return FP8GEMM_ALGO_SKINNY;
    if (k % 16 == 0 && k <= (1 << 23)) return FP8GEMM_ALGO_TILE;
    return FP8GEMM_ALGO_DIRECT;
}

// Which tiled kernel, how many K slices, which K-walk rotation.
struct TilePlan {
    int variant, nsplit, rotate;
    bool split_all;      // K slices for every tile (else only for the tiles that do not fill a round)
};

// Cost model behind the choice, in microseconds, fitted to MI355X timings of the
// persistent kernels (128-byte K tiles; 45 shapes x 7 tile kernels x 12 ways of cutting K;
// the pick is within 1 % of the best measured candidate on average):
//   a round of 256 whole tiles     = k_tiles * per_k_tile + per_item
//   a round of tail items          = k_tiles_per_slice * per_k_tile * load + per_item
//   load                           = 0.6 + 0.4 * (share of the 256 CUs with an item): a chip
//                                    that is partly idle clocks higher and contends less
//   main kernel                    = max(sum of rounds, input_bytes / stream_rate)
//   K slices add one reduction pass over (nsplit + 1) x the cut tiles.
// The model only has to rank the candidates, not to predict the time.
struct PtileCost {
    int variant, variant4, bm, bn;              // variant4: the same tile with a 4-deep ring of 64-byte K tiles (-1: none)
    double per_k_tile, per_item, stream_rate;   // us, us, bytes per us
};
constexpr PtileCost kPtileCosts[] = {
    {0, 1, 256, 256, 1.30, 13.0, 4.0e6},
    {13, 13, 256, 256, 1.25, 13.0, 4.0e6},     // the same tile on the 16x16x128 MFMA: less energy per flop, and
                                               // the compute-bound shapes run at the board's power limit.  One MFMA
                                               // step takes 128 bytes of K, so a 4-deep ring of 64-byte K tiles and
                                               // a 2-deep ring of 128-byte ones are the same pipeline: the 4-stage
                                               // entry points share this kernel with the 2-stage ones
    {9, 10, 192, 256, 1.15, 9.0, 4.6e6},
    {14, 14, 192, 256, 1.10, 9.0, 4.0e6},
    {5, 11, 128, 256, 1.00, 6.0, 6.5e6},
    {6, 12, 128, 128, 0.75, 2.5, 4.0e6},
    {8, -1, 256, 128, 0.90, 10.0, 4.6e6},
};
constexpr double kIdleChipFactor = 0.6;
constexpr int kSplitChoices[] = {1, 2, 3, 4, 6, 8, 12, 16};
constexpr int kMinKTilesPerSlice = 12;
constexpr size_t kMaxSplitScratch = (size_t)1 << 30;

TilePlan plan_tile(int m, int k, int n, int stages)
{
    TilePlan best = {0, 1, 2, false};
    const int kt = (k + 127) / 128;
    double best_cost = 1e30;
    for (const PtileCost &c : kPtileCosts) {
        // the 256 x 128 tile pays off where it holds all rows of A at once (no second
        // row of tiles re-reading the same B rows) and is at least half full
        if (c.variant == 8 && (m <= 128 || m > 256)) continue;
        if (stages == 4) {
            // the 4-deep rings rank like their 2- and 3-deep twins (same tiles, same work list);
            // only the 256 x 256 one is compiled for a K that is not a multiple of its K tile
            if (c.variant4 < 0 || (k % 64 != 0 && c.variant4 != 1)) continue;
        } else if (k % 128 != 0 && !(c.variant == 0 || c.variant == 5 || c.variant == 6)) {
            continue;      // overhanging K tile: only the shapes compiled for it
        }
        for (int mode = 0; mode < 2; ++mode)          // 0: slices for the tail tiles only, 1: for all
            for (int split : kSplitChoices) {
                if (mode == 1 && split == 1) continue;      // same as mode 0
                const PtileWork w = ptile_work(m, n, c.bm, c.bn, split, mode == 1);
                if (!w.ok) continue;
                if (split > 1 && (w.nsplit == 1 || kt / split < kMinKTilesPerSlice ||
                                  ptile_scratch_bytes(w, c.bm, c.bn) > kMaxSplitScratch))
                    continue;
                if ((c.variant == 13 || c.variant == 14) && !p2h_ok(k, w.nsplit)) continue;
                // whole-tile rounds run with every CU busy; the rounds of tail items with
                // whatever share of the CUs they fill
                double cost = (w.bulk / 256) * (kt * c.per_k_tile + c.per_item);
                const long tail_items = (long)w.tail * w.nsplit;
                if (tail_items > 0) {
                    const int tail_rounds = (int)((tail_items + 255) / 256);
                    const double busy = (double)tail_items / (256.0 * tail_rounds);
                    const int kt_item = (kt + w.nsplit - 1) / w.nsplit;
                    cost += tail_rounds * (kt_item * c.per_k_tile * (kIdleChipFactor + (1.0 - kIdleChipFactor) * busy) + c.per_item);
                }
                const double stream = ((double)m * k + (double)n * k) / c.stream_rate;
                if (stream > cost) cost = stream;
                if (w.nsplit > 1) cost += 6.0 + (w.nsplit + 1) * (double)w.tail * c.bm * c.bn * 4.0 / 6.0e6;
                if (cost < best_cost) {
                    best_cost = cost;
                    best.variant = stages == 4 ? c.variant4 : c.variant;
                    best.nsplit = w.nsplit;
                    best.split_all = mode == 1;
                }
            }
    }
    // K-walk rotation: per tile column while A is small enough to stay in an XCD's L2
    // next to the B rows in flight, else per XCD and round
    best.rotate = ((size_t)m * k <= ((size_t)2 << 20)) ? 1 : 2;
    return best;
}

size_t tile_plan_scratch_bytes(int m, int n, const TilePlan &p)
{
    if (p.nsplit <= 1) return 0;
    for (const PtileCost &c : kPtileCosts)
        if (c.variant == p.variant || c.variant4 == p.variant) {
            const PtileWork w = ptile_work(m, n, c.bm, c.bn, p.nsplit, p.split_all);
            return w.ok ? ptile_scratch_bytes(w, c.bm, c.bn) : 0;
        }
    return 0;
}

template <int AF, int BF>
hipError_t dispatch(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out, int stages,
                    int algo, int variant, int nsplit, const OutSpec &spec, hipStream_t stream)
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
        TilePlan p = plan_tile(m, k, n, stages);
        if (variant >= 0) {
            // tuning hook: variant = shape index + 16 * (1 + K-walk rotation mode); a bare
            // shape index keeps the plan's rotation and runs unsplit unless split_k says otherwise
            if (variant >= 16) {
                p.rotate = variant / 16 - 1;
                if (p.rotate > 2) return hipErrorInvalidValue;
            }
            p.variant = variant % 16;
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
        return launch_tile<AF, BF>(m, k, n, a, b, out, p.variant, p.nsplit, p.split_all, p.rotate, spec, stream);
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
        return launch_skinny<AF, BF>(m, k, n, a, b, out, p, spec, stream);
    }
    default:
        return hipErrorInvalidValue;
    }
}

const OutSpec kPlainOut = {1.0f, nullptr, nullptr, FP8GEMM_DEV_OUT_F32};

int launch_checked(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt, void *out,
                   int stages, int algo, int variant, int nsplit, void *stream, const OutSpec &spec = kPlainOut)
{
    if (m <= 0 || k <= 0 || n <= 0 || !a || !b || !out) return (int)hipErrorInvalidValue;
    if ((a_fmt != FP8GEMM_E4M3 && a_fmt != FP8GEMM_E5M2) || (b_fmt != FP8GEMM_E4M3 && b_fmt != FP8GEMM_E5M2))
        return (int)hipErrorInvalidValue;
    if (stages != 2 && stages != 4) return (int)hipErrorInvalidValue;
    if (algo < FP8GEMM_ALGO_AUTO || algo > FP8GEMM_ALGO_SKINNY) return (int)hipErrorInvalidValue;
    const uint8_t *pa = static_cast<const uint8_t *>(a);
    const uint8_t *pb = static_cast<const uint8_t *>(b);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the launch status is read back with hipGetLastError(); drop whatever an earlier,
    // unrelated runtime call of this thread may have left there
    (void)hipGetLastError();
    hipError_t e;
    if (a_fmt == FP8GEMM_E4M3 && b_fmt == FP8GEMM_E4M3)
        e = dispatch<0, 0>(m, k, n, pa, pb, out, stages, algo, variant, nsplit, spec, s);
    else if (a_fmt == FP8GEMM_E5M2 && b_fmt == FP8GEMM_E5M2)
        e = dispatch<1, 1>(m, k, n, pa, pb, out, stages, algo, variant, nsplit, spec, s);
    else if (a_fmt == FP8GEMM_E4M3)
        e = dispatch<0, 1>(m, k, n, pa, pb, out, stages, algo, variant, nsplit, spec, s);
    else
        e = dispatch<1, 0>(m, k, n, pa, pb, out, stages, algo, variant, nsplit, spec, s);
    return (int)e;
}

}  // namespace

extern "C" {

int fp8gemm_launch(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                   float *out, int stages, void *stream)
{
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, stages, FP8GEMM_ALGO_AUTO, -1, 0, stream);
}

int fp8gemm_launch_algo(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                        float *out, int stages, int algo, void *stream)
{
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, stages, algo, -1, 0, stream);
}

int fp8gemm_launch_tuned(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                         float *out, int algo, int variant, int split_k, void *stream)
{
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, 2, algo, variant, split_k, stream);
}

int fp8gemm_launch_ex(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                      void *out, int out_type, float alpha, const float *a_scale, const float *b_scale,
                      void *stream)
{
    if (out_type != FP8GEMM_OUT_F32 && out_type != FP8GEMM_OUT_BF16 && out_type != FP8GEMM_OUT_F16)
        return (int)hipErrorInvalidValue;
    if (!(alpha == alpha)) return (int)hipErrorInvalidValue;      // NaN
    const OutSpec spec = {alpha, a_scale, b_scale, out_type};
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, 2, FP8GEMM_ALGO_AUTO, -1, 0, stream, spec);
}

int fp8gemm_num_variants(int algo)
{
    if (algo == FP8GEMM_ALGO_TILE) return kNumTileVariants;
    if (algo == FP8GEMM_ALGO_SKINNY) return kNumSkinnyVariants;
    return algo == FP8GEMM_ALGO_DIRECT ? 1 : 0;
}

int fp8gemm_select_algo(int m, int k, int n)
{
    if (m <= 0 || k <= 0 || n <= 0) return -1;
    return select_algo(m, k, n);
}

int fp8gemm_plan(int m, int k, int n, int stages, int plan[4])
{
    if (m <= 0 || k <= 0 || n <= 0 || !plan || (stages != 2 && stages != 4)) return (int)hipErrorInvalidValue;
    const int algo = select_algo(m, k, n);
    plan[0] = algo;
    plan[1] = 0;
    plan[2] = 1;
    plan[3] = 0;
    if (algo == FP8GEMM_ALGO_SKINNY) {
        const SkinnyPlan p = plan_skinny(m, k, n);
        plan[1] = p.variant;
        plan[2] = p.nsplit;
        plan[3] = 16 * p.tn;
    } else if (algo == FP8GEMM_ALGO_TILE) {
        const TilePlan p = plan_tile(m, k, n, stages);
        plan[1] = p.variant;
        plan[2] = p.nsplit;
        plan[3] = p.rotate + ((p.nsplit > 1 && !p.split_all) ? 16 : 0);
    }
    return 0;
}

int fp8gemm_tile_order(int m, int k, int n, int bm, int bn, int index, int *tile_row, int *tile_col)
{
    if (m <= 0 || k <= 0 || n <= 0 || bm <= 0 || bn <= 0 || !tile_row || !tile_col) return (int)hipErrorInvalidValue;
    const PtileWork w = ptile_work(m, n, bm, bn, 1, false);
    if (!w.ok || index < 0 || index >= w.tiles_m * w.tiles_n) return (int)hipErrorInvalidValue;
    tile_of_number(index, w.tiles_m, w.tiles_n, w.GM, tile_column_block(w.tiles_n, m, n, k), *tile_row, *tile_col);
    return 0;
}

size_t fp8gemm_scratch_bytes(int m, int k, int n)
{
    if (m <= 0 || k <= 0 || n <= 0) return 0;
    int nsplit = 1;
    const int algo = select_algo(m, k, n);
    if (algo == FP8GEMM_ALGO_SKINNY) nsplit = plan_skinny(m, k, n).nsplit;
    if (algo == FP8GEMM_ALGO_TILE) return tile_plan_scratch_bytes(m, n, plan_tile(m, k, n, 2));
    return nsplit > 1 ? (size_t)nsplit * m * n * sizeof(float) : 0;
}

const char *fp8gemm_error_string(int code)
{
    return hipGetErrorString(static_cast<hipError_t>(code));
}

int fp8gemm_version(void) { return kVersion; }

#define FP8GEMM_ENTRY(NAME, AFMT, BFMT, STAGES)                                              \
    int NAME(int m, int k, int n, const void *a, const void *b, float *out)                  \
    {                                                                                        \
        return launch_checked(m, k, n, a, AFMT, b, BFMT, out, STAGES, FP8GEMM_ALGO_AUTO, -1, \
                              0, nullptr);                                                   \
    }

FP8GEMM_ENTRY(fp8gemm_e4m3_e4m3_stage2, FP8GEMM_E4M3, FP8GEMM_E4M3, 2)
FP8GEMM_ENTRY(fp8gemm_e4m3_e4m3_stage4, FP8GEMM_E4M3, FP8GEMM_E4M3, 4)
FP8GEMM_ENTRY(fp8gemm_e5m2_e5m2_stage2, FP8GEMM_E5M2, FP8GEMM_E5M2, 2)
FP8GEMM_ENTRY(fp8gemm_e5m2_e5m2_stage4, FP8GEMM_E5M2, FP8GEMM_E5M2, 4)
FP8GEMM_ENTRY(fp8gemm_e4m3_e5m2_stage2, FP8GEMM_E4M3, FP8GEMM_E5M2, 2)
FP8GEMM_ENTRY(fp8gemm_e4m3_e5m2_stage4, FP8GEMM_E4M3, FP8GEMM_E5M2, 4)
FP8GEMM_ENTRY(fp8gemm_e5m2_e4m3_stage2, FP8GEMM_E5M2, FP8GEMM_E4M3, 2)
FP8GEMM_ENTRY(fp8gemm_e5m2_e4m3_stage4, FP8GEMM_E5M2, FP8GEMM_E4M3, 4)

}  // extern "C"
