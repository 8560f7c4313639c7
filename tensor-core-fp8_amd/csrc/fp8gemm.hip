// C ABI, argument validation, planning and scratch of the gfx950 FP8 GEMM library.
// The entry points are declared in include/fp8gemm.h; together they
// stand where the launch functions of the reference stand
// (GEMM/include/gemm.cuh:11-55, defined at GEMM/src/gemm.cu:263-285 and
// siblings): validate, pick a kernel, launch asynchronously, return the launch
// status.  The kernels and their launch code are compiled per operand pairing
// (dispatch.h, dispatch_pair.hip).
#include "fp8gemm.h"

#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>
#include <utility>

#include "kernel_reduce.h"
#include "kernel_sparse.h"
#include "plan.h"
#include "scratch_pool.h"

namespace fp8gemm_detail {

extern template hipError_t dispatch<0, 0>(int, int, int, const uint8_t *, const uint8_t *, void *, int, int, int,
                                          const OutSpec &, Workspace &, hipStream_t);
extern template hipError_t dispatch<0, 1>(int, int, int, const uint8_t *, const uint8_t *, void *, int, int, int,
                                          const OutSpec &, Workspace &, hipStream_t);
extern template hipError_t dispatch<1, 0>(int, int, int, const uint8_t *, const uint8_t *, void *, int, int, int,
                                          const OutSpec &, Workspace &, hipStream_t);
extern template hipError_t dispatch<1, 1>(int, int, int, const uint8_t *, const uint8_t *, void *, int, int, int,
                                          const OutSpec &, Workspace &, hipStream_t);

extern template hipError_t dispatch_bell<0, 0>(int, int, int, const uint8_t *, const uint8_t *, float *, const BellSpec &, Workspace &, hipStream_t);
extern template hipError_t dispatch_bell<0, 1>(int, int, int, const uint8_t *, const uint8_t *, float *, const BellSpec &, Workspace &, hipStream_t);
extern template hipError_t dispatch_bell<1, 0>(int, int, int, const uint8_t *, const uint8_t *, float *, const BellSpec &, Workspace &, hipStream_t);
extern template hipError_t dispatch_bell<1, 1>(int, int, int, const uint8_t *, const uint8_t *, float *, const BellSpec &, Workspace &, hipStream_t);

namespace {
constexpr int kVersion = 103;
// What the work lists and the planner's constants are laid out for: MI355X as one partition,
// 256 CUs in 8 XCDs of 32, workgroups handed to the XCDs round robin (id mod 8).  On another
// partition mode every result is still right (the work list only decides who computes what);
// the plans are then merely not the best ones.  fp8gemm_device_info tells a caller which it is.
constexpr int kPlannedCus = 256;
constexpr int kMaxDevices = 64;

// ------------------------------------------------------------------ scratch
__global__ void zero_ints_kernel(int *p, int count)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = 0;
}

// Device runtime behind the scratch bookkeeping (scratch_pool.h).
struct HipScratchBackend {
    using Event = hipEvent_t;
    // A new buffer starts with zeroed arrival counters (the kernels leave them at zero).  They
    // are cleared by a kernel on the stream that asked for the buffer: ordered before that
    // stream's GEMM, without the host or any other stream waiting (a hipMemset would run on the
    // null stream, which a non-blocking stream is not ordered against).
    int alloc(size_t bytes, void *stream, void **ptr)
    {
        hipError_t e = hipMalloc(ptr, bytes);
        if (e != hipSuccess) return (int)e;
        const size_t ints = (bytes < kSliceCounterBytes ? bytes : kSliceCounterBytes) / sizeof(int);
        (void)hipGetLastError();
        hipLaunchKernelGGL(zero_ints_kernel, dim3((unsigned)((ints + 255) / 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<int *>(*ptr), (int)ints);
        e = hipGetLastError();
        if (e != hipSuccess) (void)hipFree(*ptr);
        return (int)e;
    }
    void free(void *ptr) { (void)hipFree(ptr); }
    int record(void *stream, Event *ev)
    {
        hipError_t e = hipEventCreateWithFlags(ev, hipEventDisableTiming);
        if (e != hipSuccess) return (int)e;
        e = hipEventRecord(*ev, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) (void)hipEventDestroy(*ev);
        return (int)e;
    }
    bool passed(Event ev) { return hipEventQuery(ev) == hipSuccess; }
    void drop(Event ev) { (void)hipEventDestroy(ev); }
};
ScratchPool<HipScratchBackend> g_pool;

// The scratch array of the entry point that allocates nothing: part of the code object,
// so every device the library runs on holds its own copy from the moment the code is loaded.
constexpr size_t kStaticScratchBytes = FP8GEMM_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
void *g_static_scratch[kMaxDevices];       // device address of `scratch`, per device
std::mutex g_static_scratch_mutex;

// Device address of this device's copy of `scratch` (the array's name is only a host-side
// handle; kernels and runtime calls take the address looked up here).
hipError_t static_scratch_address(void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (!g_static_scratch[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_static_scratch[dev] = p;
    }
    *out = g_static_scratch[dev];
    return hipSuccess;
}

}  // namespace

__global__ void fill_float_kernel(float *p, float v) { *p = v; }

hipError_t Workspace::get(size_t need, void **out)
{
    if (!pooled_) {
        // too small a workspace is the caller's to fix: nothing is allocated in its place
        if (need > bytes_ || !ptr_) return hipErrorOutOfMemory;
        *out = ptr_;
        return hipSuccess;
    }
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (!lock_.owns_lock()) lock_ = std::unique_lock<std::mutex>(g_pool.mutex());
    e = static_cast<hipError_t>(g_pool.get(dev, stream_, need, out));
    // (an event that is still pending is reported as "not ready"; that is no launch error)
    (void)hipGetLastError();
    return e;
}

// out[i] = sum over the nsplit planes of ws, on `stream`
hipError_t launch_reduce(const float *ws, void *out, size_t count, int nsplit, const OutSpec &spec, hipStream_t stream)
{
    const bool vec = count % 4 == 0 &&
                     ((reinterpret_cast<uintptr_t>(ws) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(spec.c)) % 16) == 0;
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

hipError_t launch_tile_slices_reduce(const float *ws, void *out, int m, int n, int k, int bm, int bn, const PtileWork &w,
                                     const OutSpec &spec, hipStream_t stream)
{
    ws += kSliceCounterBytes / sizeof(float);      // the partial sums follow the arrival counters
    const size_t threads = (size_t)w.tail * ((size_t)bm * bn / 4);
    hipLaunchKernelGGL(gemm_tile_slices_reduce_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                       ws, out, m, n, bm, bn, w.tiles_m, w.tiles_n, w.GM, tile_column_block(w.tiles_n, m, n, k), w.bulk, w.tail,
                       w.nsplit, spec);
    return hipGetLastError();
}

// ------------------------------------------------------------------ planning
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
    return w.nsplit > 1 ? kSliceCounterBytes + (size_t)w.nsplit * w.tail * bm * bn * sizeof(float) : 0;
}

bool plain_output(const OutSpec &spec)
{
    return spec.type == FP8GEMM_DEV_OUT_F32 && spec.alpha == 1.0f && !spec.a_scale && !spec.b_scale && !spec.c &&
           !spec.d_scale && !spec.amax;
}

bool p2h_ok(int k, int nsplit)
{
    return k % 16 == 0 && ((k + 127) / 128) / nsplit >= 2;
}

// the single-wave streams: up to 16 rows of A (one 16-row MFMA block)
bool skinny_ok(int m, int k, int n)
{
    return m <= 16 && n % 16 == 0 && k % 128 == 0;
}

// Picks columns per wave, LDS shape and split-K factor.  Measured on MI355X with
// operands that are cold in every cache.  The HBM pipe is fullest with one to two fat
// streams per CU (256..512 streams, each with a deep LDS ring) rather than many thin
// ones, and a split-K pass costs 10 % and more, so K is cut only when the columns alone
// give too few streams.
SkinnyPlan plan_skinny(int m, int k, int n)
{
    SkinnyPlan p;
    p.mt = 1;
    const int ksteps = k / 128;
    int tn = 4, split = 1;
    {
        // Streams of 64, 32 or 16 columns: the widest that still gives 400 streams or more (every
        // stream re-reads A, and a wide stream's ring holds more of B per load instruction); with
        // more than a few rows of A, a count that fills the 256 CUs evenly (a multiple of 256) is
        // taken before that; failing both, the count that loads the CUs most evenly, the wider
        // streams on a tie.  Measured (cold, us) for 64 / 32 / 16 columns: M=1 N=10240 K=8192
        // 16.9 / 17.6 / 15.6, M=16 18.4 / 19.4 / 17.5; M=1 N=8192 K=28672 37.4 / 37.5 / 35.6,
        // M=16 38.8 / 37.5 / 38.1; M=16 N=6144 K=8192 - / 11.3 / 12.6; N=28672 is best at 64.
        int pick = 0;
        for (int t = 4; t >= 1 && !pick; t /= 2) {
            if (n % (16 * t) != 0) continue;
            const int streams = n / (16 * t);
            if (streams >= 400 || (m > 4 && streams >= 256 && streams % 256 == 0)) pick = t;
        }
        if (!pick) {
            double best = -1.0;
            for (int t = 4; t >= 1; t /= 2) {
                if (n % (16 * t) != 0) continue;
                const int streams = n / (16 * t);
                const double even = (double)streams / (256.0 * ((streams + 255) / 256));
                if (even > best + 1e-9) {
                    best = even;
                    pick = t;
                }
            }
        }
        tn = pick;
        // (K slices cost a second launch, about 2.5 us: only while there are fewer streams than CUs
        // and a slice keeps 4 KiB of K or more)
        while ((long)(n / (16 * tn)) * split < 256 && split < 16 && ksteps % (2 * split) == 0 && ksteps / (2 * split) >= 32)
            split *= 2;
    }
    p.tn = tn;
    p.nsplit = split;
    const int kchunk = k / split;
    const long waves = (long)(n / (16 * tn)) * split;
    // Fat streams (64 columns) run best on 128-byte K steps in a deep ring; thinner ones want
    // longer K steps, so that a ring stage still holds 16 KiB or more: the thinnest, on a long K
    // and with two waves or more per CU, whole 1 KiB rows.  Three waves or more per CU on a
    // short K: a ring small enough for all of them to be resident at once.
    if (tn == 4)
        p.variant = 0;
    else if (tn == 1 && kchunk % 1024 == 0 && kchunk >= 8192 && waves >= 512)
        p.variant = 5;
    else if (waves > 512 && kchunk < 8192)
        p.variant = kchunk % 256 == 0 ? 1 : 0;
    else
        p.variant = (kchunk % 512 == 0) ? 4 : (kchunk % 256 == 0) ? 1 : 0;
    return p;
}

// Up to 16 rows of A the single-wave streams are the fastest form (M=16 N=28672 K=8192: 37.0 us
// against 38.0 us of the 64 x 128 tile); from 17 rows on the tiled kernel's deep shared ring
// wins (M=32 38.5 against 40.5 us, M=64 39.3 against 50.0 us): a stream of its own per wave
// re-reads all of A for every 64 columns.
int select_algo(int m, int k, int n)
{
    if (skinny_ok(m, k, n)) return FP8GEMM_ALGO_SKINNY;
    if (k % 16 == 0 && k <= (1 << 23)) return FP8GEMM_ALGO_TILE;
    return FP8GEMM_ALGO_DIRECT;
}

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
    int variant, bm, bn;
    double per_k_tile, per_item, stream_rate;   // us, us, bytes per us
};
constexpr PtileCost kPtileCosts[] = {
    {0, 256, 256, 1.30, 13.0, 4.0e6},
    {13, 256, 256, 1.25, 13.0, 4.0e6},         // the same tile on the 16x16x128 MFMA: less energy per flop, and
                                               // the compute-bound shapes run at the board's power limit
    {9, 192, 256, 1.15, 9.0, 4.6e6},
    {14, 192, 256, 1.10, 9.0, 4.0e6},
    {5, 128, 256, 1.00, 6.0, 6.5e6},
    {6, 128, 128, 0.75, 2.5, 4.0e6},
    {8, 256, 128, 0.90, 10.0, 4.6e6},
    // weight streaming (one row of tiles, B loaded once with the non-temporal hint, rings 5 and 4 slots deep)
    {15, 64, 128, 0.586, 5.5, 6.4e6},
    {16, 128, 128, 0.70, 5.5, 6.0e6},
};
constexpr double kIdleChipFactor = 0.6;
constexpr int kSplitChoices[] = {1, 2, 3, 4, 6, 8, 12, 16};
constexpr int kMinKTilesPerSlice = 12;
constexpr size_t kMaxSplitScratch = (size_t)1 << 30;

// The plan does not depend on the stage count of the entry point: the depth of the LDS ring (2 to
// 5 slots) belongs to the tile shape, and the 2- and 4-stage entry points run the same kernels --
// as the reference's GEMM4 runs the kernel of GEMM (GEMM/src/gemm.cu:687-694).  On the 16x16x128
// MFMA, whose one step takes 128 bytes of K, a 4-deep ring of 64-byte K tiles and a 2-deep ring of
// 128-byte ones are the same pipeline; 4-deep rings of 64-byte K tiles under the 32x32x64 MFMA
// measured 5 to 11 % slower than the 2- and 3-deep rings of 128-byte K tiles on every shape class.
TilePlan plan_tile(int m, int k, int n, unsigned allowed)
{
    TilePlan best = {0, 1, 2, false};
    const int kt = (k + 127) / 128;
    double best_cost = 1e30;
    for (const PtileCost &c : kPtileCosts) {
        if (!((allowed >> c.variant) & 1u)) continue;
        // the 256 x 128 tile pays off where it holds all rows of A at once (no second
        // row of tiles re-reading the same B rows) and is at least half full
        if (c.variant == 8 && (m <= 128 || m > 256)) continue;
        // the weight-streaming tiles: one row of tiles, whole 128-byte K tiles
        if ((c.variant == 15 || c.variant == 16) && (m > c.bm || k % 128 != 0)) continue;
        // ... and up to 64 rows nothing else comes close to them
        if (m <= 64 && k % 128 == 0 && c.variant != 15 && ((allowed >> 15) & 1u)) continue;
        // overhanging K tile: only the shapes compiled for it
        if (k % 128 != 0 && !(c.variant == 0 || c.variant == 5 || c.variant == 6 || c.variant == 13 || c.variant == 14)) continue;
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
                    best.variant = c.variant;
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
        if (c.variant == p.variant) {
            const PtileWork w = ptile_work(m, n, c.bm, c.bn, p.nsplit, p.split_all);
            return w.ok ? ptile_scratch_bytes(w, c.bm, c.bn) : 0;
        }
    return 0;
}

namespace {

const OutSpec kPlainOut = {1.0f, nullptr, nullptr, FP8GEMM_DEV_OUT_F32, 0.0f, nullptr, FP8GEMM_DEV_OUT_F32, nullptr, nullptr, nullptr};

int launch_checked(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt, void *out,
                   int stages, int algo, int variant, int nsplit, void *stream, const OutSpec &spec,
                   Workspace &wsp)
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
        e = dispatch<0, 0>(m, k, n, pa, pb, out, algo, variant, nsplit, spec, wsp, s);
    else if (a_fmt == FP8GEMM_E5M2 && b_fmt == FP8GEMM_E5M2)
        e = dispatch<1, 1>(m, k, n, pa, pb, out, algo, variant, nsplit, spec, wsp, s);
    else if (a_fmt == FP8GEMM_E4M3)
        e = dispatch<0, 1>(m, k, n, pa, pb, out, algo, variant, nsplit, spec, wsp, s);
    else
        e = dispatch<1, 0>(m, k, n, pa, pb, out, algo, variant, nsplit, spec, wsp, s);
    return (int)e;
}

// the library's own scratch: one buffer per (device, stream)
int launch_pooled(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt, void *out,
                  int stages, int algo, int variant, int nsplit, void *stream, const OutSpec &spec = kPlainOut)
{
    Workspace wsp = Workspace::pooled(static_cast<hipStream_t>(stream));
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, stages, algo, variant, nsplit, stream, spec, wsp);
}

}  // namespace

}  // namespace fp8gemm_detail

using namespace fp8gemm_detail;

// ------------------------------------------------------------------ sparse operands
namespace {

template <int SF, int BF>
hipError_t launch_spmm_bell(int m, int k, int n, int block, int ell_cols, const uint8_t *values, const int *block_cols,
                            const uint8_t *b, float *out, hipStream_t stream)
{
    // columns of out per wave: as many as n fills, up to 64
    const int tn = n <= 16 ? 1 : (n <= 32 ? 2 : 4);
    const long groups_n = (n + 16 * tn - 1) / (16 * tn);
    const long grid = (long)(m / 16) * groups_n;
    if (grid > 0x7FFFFFFFL) return hipErrorInvalidValue;
    if (tn == 1)
        hipLaunchKernelGGL((spmm_bell_kernel<SF, BF, 1>), dim3((unsigned)grid), dim3(64), 0, stream, m, k, n, block, ell_cols,
                           values, block_cols, b, out, (int)groups_n);
    else if (tn == 2)
        hipLaunchKernelGGL((spmm_bell_kernel<SF, BF, 2>), dim3((unsigned)grid), dim3(64), 0, stream, m, k, n, block, ell_cols,
                           values, block_cols, b, out, (int)groups_n);
    else
        hipLaunchKernelGGL((spmm_bell_kernel<SF, BF, 4>), dim3((unsigned)grid), dim3(64), 0, stream, m, k, n, block, ell_cols,
                           values, block_cols, b, out, (int)groups_n);
    return hipGetLastError();
}

template <int SF, int XF>
hipError_t launch_spmv_csr(int m, int k, const uint8_t *values, const int *row_offsets, const int *col, const int *row_order,
                           const uint8_t *x, float *y, hipStream_t stream)
{
    // 16-byte loads of the indices need the arrays aligned; up to 2048 waves walk the rows
    const bool vec = reinterpret_cast<uintptr_t>(col) % 16 == 0 && reinterpret_cast<uintptr_t>(values) % 4 == 0;
    if (!vec) {
        hipLaunchKernelGGL((spmv_csr_kernel<SF, XF>), dim3((unsigned)((m + 3) / 4)), dim3(256), 0, stream, m, values, row_offsets,
                           col, row_order, x, y);
        return hipGetLastError();
    }
    // (workgroups of four waves; a wave walks a few rows, and some thirty waves per CU keep enough loads in flight)
    const int groups = (m + 7) / 8 < 2048 ? (m + 7) / 8 : 2048;
    if (k <= kSpmvLdsBytes) {
        const int lds = (k + 15) / 16 * 16;
        hipLaunchKernelGGL((spmv_csr_vec_kernel<SF, XF, true>), dim3((unsigned)groups), dim3(256), lds, stream, m, k, values,
                           row_offsets, col, row_order, x, y);
    } else {
        hipLaunchKernelGGL((spmv_csr_vec_kernel<SF, XF, false>), dim3((unsigned)groups), dim3(256), 0, stream, m, k, values,
                           row_offsets, col, row_order, x, y);
    }
    return hipGetLastError();
}

constexpr int kLdsBytesPerCu = 160 * 1024;

template <int SF, int XF>
hipError_t launch_spmv_bell(int m, int k, int block, int ell_cols, const uint8_t *values, const int *block_cols,
                            const uint8_t *x, float *y, hipStream_t stream)
{
    int shift = -1;
    for (int b = 4; b < 31; ++b)
        if (block == (1 << b)) shift = b;
    const int kell = ell_cols * block;
    const int lds = (k + 15) / 16 * 16 + kSpmvSumBytes;
    // R lanes per stored row; a row item = the 64 / R rows a wave has at a time
    int lanes_per_row = 4;
    while (lanes_per_row < 64 && lanes_per_row * 16 < kell) lanes_per_row *= 2;
    const int rows_per_item = 64 / lanes_per_row, items = (m + rows_per_item - 1) / rows_per_item;
    const int mfma_steps = ((kell + 16 * lanes_per_row - 1) / (16 * lanes_per_row) + 1) / 2;
    // few items: two or four waves share the MFMA steps of an item, so that about 2048 waves and more run
    int ksplit = items >= 1024 ? 1 : (items >= 512 ? 2 : 4);
    while (ksplit > 1 && mfma_steps < 2 * ksplit) ksplit /= 2;
    const int per_wg = 4 / ksplit;
    int grid = (items + per_wg - 1) / per_wg;
    // (ksplit 1: no more workgroups than the chip holds at once, eight per CU, fewer where x takes more of the LDS)
    if (ksplit == 1) grid = std::min(grid, kPlannedCus * std::max(1, std::min(8, kLdsBytesPerCu / lds)));
    auto kernel = ksplit == 1 ? spmv_bell_kernel<SF, XF, 1> : (ksplit == 2 ? spmv_bell_kernel<SF, XF, 2> : spmv_bell_kernel<SF, XF, 4>);
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), lds, stream, m, k, block, shift, ell_cols, lanes_per_row, values,
                       block_cols, x, y);
    return hipGetLastError();
}

template <int LF, int RF>
hipError_t launch_sddmm(int m_vec, int k, int vec, const int *row_offsets, const int *col, const uint8_t *lhs, const uint8_t *rhs,
                        float *out, hipStream_t stream)
{
    const bool fast = vec <= 16 && k % 16 == 0 && (reinterpret_cast<uintptr_t>(lhs) | reinterpret_cast<uintptr_t>(rhs)) % 16 == 0;
    const size_t lds = (size_t)vec * (k + kSddmmLdsPad);
    const bool alds = lds <= (size_t)kSddmmLdsBytes;
    const bool wide = vec % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (fast) {
        auto kernel = alds ? (wide ? sddmm_kernel<LF, RF, true, true> : sddmm_kernel<LF, RF, true, false>)
                           : (wide ? sddmm_kernel<LF, RF, false, true> : sddmm_kernel<LF, RF, false, false>);
        hipLaunchKernelGGL(kernel, dim3((unsigned)m_vec), dim3(64 * kSddmmWaves), alds ? lds : 0, stream, k, vec, row_offsets, col, lhs,
                           rhs, out);
    } else {
        hipLaunchKernelGGL((sddmm_general_kernel<LF, RF>), dim3((unsigned)m_vec), dim3(256), 0, stream, m_vec, k, vec, row_offsets, col,
                           lhs, rhs, out);
    }
    return hipGetLastError();
}

bool fmt_ok(int f) { return f == FP8GEMM_E4M3 || f == FP8GEMM_E5M2; }

// The tiled kernel takes blocks whose rows fill whole tiles (32, 64, 128 or 256 rows: block % 32 == 0)
// and whose bytes inside a 128-byte K tile come in runs of 32 or more (the same condition); below 64
// columns of output its tiles are mostly empty.
bool bell_tiled(int block, int n) { return block % 32 == 0 && n >= 64; }

}  // namespace

extern "C" {

int fp8gemm_launch(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                   float *out, int stages, void *stream)
{
    return launch_pooled(m, k, n, a, a_fmt, b, b_fmt, out, stages, FP8GEMM_ALGO_AUTO, -1, 0, stream);
}

int fp8gemm_gemv(int n, int k, const void *w, int w_fmt, const void *x, int x_fmt, float *y, void *stream)
{
    return launch_pooled(1, k, n, x, x_fmt, w, w_fmt, y, 2, FP8GEMM_ALGO_AUTO, -1, 0, stream);
}

// ------------------------------------------------------------------ sparse operands
int fp8gemm_spmm_bell(int m, int k, int n, int block, int ell_cols, const void *values, int s_fmt, const int *block_cols,
                      const void *b, int b_fmt, float *out, void *stream)
{
    if (m <= 0 || k <= 0 || n <= 0 || block <= 0 || ell_cols <= 0 || !values || !block_cols || !b || !out)
        return (int)hipErrorInvalidValue;
    if (!fmt_ok(s_fmt) || !fmt_ok(b_fmt)) return (int)hipErrorInvalidValue;
    if (block % 16 != 0 || m % block != 0 || k % block != 0) return (int)hipErrorInvalidValue;
    if ((long)ell_cols * block > (1L << 30)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(values) | reinterpret_cast<uintptr_t>(b)) % 16 != 0) return (int)hipErrorInvalidValue;
    const uint8_t *pv = static_cast<const uint8_t *>(values), *pb = static_cast<const uint8_t *>(b);
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    hipError_t e;
    // Blocks of 32 rows and multiples go through the LDS-tiled persistent kernel (the stored values
    // are its A, the block list steers where the K tiles of B, or with blocks below 128 the parts of
    // a K tile, come from); other block sizes, and outputs of a few columns, through the direct kernel.
    if (bell_tiled(block, n)) {
        int sub = 128;                                  // gcd(block, 128)
        while (block % sub != 0) sub /= 2;
        const BellSpec bell = {block_cols, ell_cols, block, k, sub};
        const int kell = ell_cols * block;
        Workspace wsp = Workspace::pooled(s);
        if (s_fmt == FP8GEMM_E4M3 && b_fmt == FP8GEMM_E4M3)
            e = dispatch_bell<0, 0>(m, kell, n, pv, pb, out, bell, wsp, s);
        else if (s_fmt == FP8GEMM_E5M2 && b_fmt == FP8GEMM_E5M2)
            e = dispatch_bell<1, 1>(m, kell, n, pv, pb, out, bell, wsp, s);
        else if (s_fmt == FP8GEMM_E4M3)
            e = dispatch_bell<0, 1>(m, kell, n, pv, pb, out, bell, wsp, s);
        else
            e = dispatch_bell<1, 0>(m, kell, n, pv, pb, out, bell, wsp, s);
        return (int)e;
    }
    if (n == 1 && k <= kSpmvLdsBytes) {
        // matrix-vector: x fits LDS
        if (s_fmt == FP8GEMM_E4M3 && b_fmt == FP8GEMM_E4M3)
            e = launch_spmv_bell<0, 0>(m, k, block, ell_cols, pv, block_cols, pb, out, s);
        else if (s_fmt == FP8GEMM_E5M2 && b_fmt == FP8GEMM_E5M2)
            e = launch_spmv_bell<1, 1>(m, k, block, ell_cols, pv, block_cols, pb, out, s);
        else if (s_fmt == FP8GEMM_E4M3)
            e = launch_spmv_bell<0, 1>(m, k, block, ell_cols, pv, block_cols, pb, out, s);
        else
            e = launch_spmv_bell<1, 0>(m, k, block, ell_cols, pv, block_cols, pb, out, s);
        return (int)e;
    }
    if (s_fmt == FP8GEMM_E4M3 && b_fmt == FP8GEMM_E4M3)
        e = launch_spmm_bell<0, 0>(m, k, n, block, ell_cols, pv, block_cols, pb, out, s);
    else if (s_fmt == FP8GEMM_E5M2 && b_fmt == FP8GEMM_E5M2)
        e = launch_spmm_bell<1, 1>(m, k, n, block, ell_cols, pv, block_cols, pb, out, s);
    else if (s_fmt == FP8GEMM_E4M3)
        e = launch_spmm_bell<0, 1>(m, k, n, block, ell_cols, pv, block_cols, pb, out, s);
    else
        e = launch_spmm_bell<1, 0>(m, k, n, block, ell_cols, pv, block_cols, pb, out, s);
    return (int)e;
}

int fp8gemm_spmv_bell(int m, int k, int block, int ell_cols, const void *values, int s_fmt, const int *block_cols,
                      const void *x, int x_fmt, float *y, void *stream)
{
    return fp8gemm_spmm_bell(m, k, 1, block, ell_cols, values, s_fmt, block_cols, x, x_fmt, y, stream);
}

int fp8gemm_spmv_csr(int m, int k, const void *values, int s_fmt, const int *row_offsets, const int *col_idx,
                     const int *row_order, const void *x, int x_fmt, float *y, void *stream)
{
    if (m <= 0 || k <= 0 || !values || !row_offsets || !col_idx || !x || !y) return (int)hipErrorInvalidValue;
    if (!fmt_ok(s_fmt) || !fmt_ok(x_fmt)) return (int)hipErrorInvalidValue;
    const uint8_t *pv = static_cast<const uint8_t *>(values), *px = static_cast<const uint8_t *>(x);
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    hipError_t e;
    if (s_fmt == FP8GEMM_E4M3 && x_fmt == FP8GEMM_E4M3)
        e = launch_spmv_csr<0, 0>(m, k, pv, row_offsets, col_idx, row_order, px, y, s);
    else if (s_fmt == FP8GEMM_E5M2 && x_fmt == FP8GEMM_E5M2)
        e = launch_spmv_csr<1, 1>(m, k, pv, row_offsets, col_idx, row_order, px, y, s);
    else if (s_fmt == FP8GEMM_E4M3)
        e = launch_spmv_csr<0, 1>(m, k, pv, row_offsets, col_idx, row_order, px, y, s);
    else
        e = launch_spmv_csr<1, 0>(m, k, pv, row_offsets, col_idx, row_order, px, y, s);
    return (int)e;
}

int fp8gemm_sddmm(int m_vec, int k, int vec_length, const int *row_offsets, const int *col_idx, const void *lhs, int l_fmt,
                  const void *rhs, int r_fmt, float *out, void *stream)
{
    if (m_vec <= 0 || k <= 0 || vec_length <= 0 || !row_offsets || !col_idx || !lhs || !rhs || !out) return (int)hipErrorInvalidValue;
    if (!fmt_ok(l_fmt) || !fmt_ok(r_fmt)) return (int)hipErrorInvalidValue;
    const uint8_t *pl = static_cast<const uint8_t *>(lhs), *pr = static_cast<const uint8_t *>(rhs);
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    hipError_t e;
    if (l_fmt == FP8GEMM_E4M3 && r_fmt == FP8GEMM_E4M3)
        e = launch_sddmm<0, 0>(m_vec, k, vec_length, row_offsets, col_idx, pl, pr, out, s);
    else if (l_fmt == FP8GEMM_E5M2 && r_fmt == FP8GEMM_E5M2)
        e = launch_sddmm<1, 1>(m_vec, k, vec_length, row_offsets, col_idx, pl, pr, out, s);
    else if (l_fmt == FP8GEMM_E4M3)
        e = launch_sddmm<0, 1>(m_vec, k, vec_length, row_offsets, col_idx, pl, pr, out, s);
    else
        e = launch_sddmm<1, 0>(m_vec, k, vec_length, row_offsets, col_idx, pl, pr, out, s);
    return (int)e;
}

size_t fp8gemm_spmm_csr_scratch_bytes(int m, int k, int n)
{
    if (m <= 0 || k <= 0 || n <= 0) return 0;
    const size_t dense = ((size_t)m * k + 255) / 256 * 256;
    return kSliceCounterBytes + dense + fp8gemm_scratch_bytes(m, k, n);
}

int fp8gemm_spmm_csr(int m, int k, int n, const void *values, int s_fmt, const int *row_offsets, const int *col_idx,
                     const void *b, int b_fmt, float *out, void *stream)
{
    if (m <= 0 || k <= 0 || n <= 0 || !values || !row_offsets || !col_idx || !b || !out) return (int)hipErrorInvalidValue;
    if (!fmt_ok(s_fmt) || !fmt_ok(b_fmt)) return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // scratch of this stream: [arrival counters of the pool's buffer, left alone | S as a dense m x k
    // fp8 matrix | the workspace of the dense GEMM]
    const size_t dense_bytes = ((size_t)m * k + 255) / 256 * 256;
    const size_t gemm_bytes = fp8gemm_scratch_bytes(m, k, n);
    Workspace pool = Workspace::pooled(s);
    void *p = nullptr;
    hipError_t e = pool.get(kSliceCounterBytes + dense_bytes + gemm_bytes, &p);
    if (e != hipSuccess) return (int)e;
    uint8_t *dense = static_cast<uint8_t *>(p) + kSliceCounterBytes;
    (void)hipGetLastError();
    if (k % 16 == 0 && k <= kSpmvLdsBytes) {
        // a row at a time through LDS: one pass, whole 16-byte pieces out
        hipLaunchKernelGGL(csr_densify_rows_kernel, dim3((unsigned)(m < 4096 ? m : 4096)), dim3(256), k, s, m, k,
                           static_cast<const uint8_t *>(values), row_offsets, col_idx, dense);
    } else {
        const size_t count16 = dense_bytes / 16;
        hipLaunchKernelGGL(zero_bytes16_kernel, dim3((unsigned)((count16 + 255) / 256)), dim3(256), 0, s,
                           reinterpret_cast<v4i *>(dense), count16);
        hipLaunchKernelGGL(csr_densify_kernel, dim3((unsigned)((m + 3) / 4)), dim3(256), 0, s, m, (size_t)k,
                           static_cast<const uint8_t *>(values), row_offsets, col_idx, dense);
    }
    e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    Workspace gemm_ws = Workspace::fixed(gemm_bytes ? dense + dense_bytes : nullptr, gemm_bytes, false);
    return launch_checked(m, k, n, dense, s_fmt, b, b_fmt, out, 2, FP8GEMM_ALGO_AUTO, -1, 0, stream, kPlainOut, gemm_ws);
}

int fp8gemm_launch_ws(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                      float *out, int stages, void *workspace, size_t workspace_bytes, void *stream)
{
    if (workspace && reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return (int)hipErrorInvalidValue;
    Workspace wsp = Workspace::fixed(workspace, workspace ? workspace_bytes : 0, false);
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, stages, FP8GEMM_ALGO_AUTO, -1, 0, stream, kPlainOut, wsp);
}

int fp8gemm_launch_noalloc(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                           float *out, int stages, void *stream)
{
    void *ptr = nullptr;
    const hipError_t e = static_scratch_address(&ptr);
    if (e != hipSuccess) return (int)e;
    Workspace wsp = Workspace::fixed(ptr, kStaticScratchBytes, true);      // static storage starts as zeros
    return launch_checked(m, k, n, a, a_fmt, b, b_fmt, out, stages, FP8GEMM_ALGO_AUTO, -1, 0, stream, kPlainOut, wsp);
}

int fp8gemm_device_info(int info[4])
{
    if (!info) return (int)hipErrorInvalidValue;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    const bool gfx950 = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    info[0] = prop.multiProcessorCount;
    info[1] = kPlannedCus;
    info[2] = gfx950 ? 1 : 0;
    info[3] = (gfx950 && prop.multiProcessorCount == kPlannedCus) ? 1 : 0;
    return 0;
}

int fp8gemm_release_scratch(void)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    std::lock_guard<std::mutex> lock(g_pool.mutex());
    e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    g_pool.release(dev);
    return 0;
}

size_t fp8gemm_scratch_held_bytes(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(g_pool.mutex());
    return g_pool.held_bytes(dev);
}

int fp8gemm_launch_algo(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                        float *out, int stages, int algo, void *stream)
{
    return launch_pooled(m, k, n, a, a_fmt, b, b_fmt, out, stages, algo, -1, 0, stream);
}

int fp8gemm_launch_tuned(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                         float *out, int algo, int variant, int split_k, void *stream)
{
    return launch_pooled(m, k, n, a, a_fmt, b, b_fmt, out, 2, algo, variant, split_k, stream);
}

int fp8gemm_launch_epilogue(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                            void *d, int d_type, float alpha, float beta, const void *c, int c_type,
                            const float *a_scale, const float *b_scale, const float *c_scale, const float *d_scale,
                            float *amax_d, void *stream)
{
    const auto type_ok = [](int t) { return t == FP8GEMM_OUT_F32 || t == FP8GEMM_OUT_BF16 || t == FP8GEMM_OUT_F16; };
    if (!type_ok(d_type) || (c && !type_ok(c_type))) return (int)hipErrorInvalidValue;
    if (!(alpha == alpha) || !(beta == beta)) return (int)hipErrorInvalidValue;      // NaN
    // in place (c == d) only with one element type: a thread then reads exactly the bytes it overwrites
    if (c && c == d && c_type != d_type) return (int)hipErrorInvalidValue;
    if (m <= 0 || k <= 0 || n <= 0 || !a || !b || !d) return (int)hipErrorInvalidValue;
    if (amax_d) {
        // the kernels fold |y| into *amax_d with an atomic maximum, starting from zero
        (void)hipGetLastError();
        hipLaunchKernelGGL(fill_float_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), amax_d, 0.0f);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    const OutSpec spec = {alpha, a_scale, b_scale, d_type, beta, c, c ? c_type : FP8GEMM_OUT_F32, c_scale, d_scale, amax_d};
    return launch_pooled(m, k, n, a, a_fmt, b, b_fmt, d, 2, FP8GEMM_ALGO_AUTO, -1, 0, stream, spec);
}

int fp8gemm_launch_ex(int m, int k, int n, const void *a, int a_fmt, const void *b, int b_fmt,
                      void *out, int out_type, float alpha, const float *a_scale, const float *b_scale,
                      void *stream)
{
    return fp8gemm_launch_epilogue(m, k, n, a, a_fmt, b, b_fmt, out, out_type, alpha, 0.0f, nullptr, FP8GEMM_OUT_F32,
                                   a_scale, b_scale, nullptr, nullptr, nullptr, stream);
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
        const TilePlan p = plan_tile(m, k, n);
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
    if (algo == FP8GEMM_ALGO_TILE) return tile_plan_scratch_bytes(m, n, plan_tile(m, k, n));
    return nsplit > 1 ? kSliceCounterBytes + (size_t)nsplit * m * n * sizeof(float) : 0;
}

const char *fp8gemm_error_string(int code)
{
    return hipGetErrorString(static_cast<hipError_t>(code));
}

int fp8gemm_version(void) { return kVersion; }

#define FP8GEMM_ENTRY(NAME, AFMT, BFMT, STAGES)                                              \
    int NAME(int m, int k, int n, const void *a, const void *b, float *out)                  \
    {                                                                                        \
        return launch_pooled(m, k, n, a, AFMT, b, BFMT, out, STAGES, FP8GEMM_ALGO_AUTO, -1,  \
                             0, nullptr);                                                    \
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
