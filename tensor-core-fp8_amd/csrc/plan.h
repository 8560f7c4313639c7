// Host-side vocabulary shared by the C ABI (fp8gemm.hip) and the per-pairing launch code
// (dispatch.h): work lists, plans, the workspace of a call.
#ifndef FP8GEMM_PLAN_H
#define FP8GEMM_PLAN_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <mutex>

#include "device_common.h"
#include "fp8gemm.h"

namespace fp8gemm_detail {

// Tiled kernel shapes by number (the tuning hook's `variant`): 0 P2 (256 x 256), 5 H3 (128 x 256), 6 Q2 (128 x 128),
// 8 W3 (256 x 128), 9 T2 (192 x 256), 13 P2h and 14 T2h (256 x 256 and 192 x 256 on the 16x16x128 MFMA), 15 E5 (64 x 128,
// weight streaming), 16 Q4s (128 x 128, weight streaming).  Streaming (single-wave) ring shapes: 0, 1, 4, 5.  A number
// below the count that is not listed names no compiled kernel and is refused.
constexpr int kNumTileVariants = 17;
constexpr int kNumSkinnyVariants = 6;

// Work list of the persistent kernel for a tile shape: `bulk` tiles (a multiple of 256)
// run as whole items, 256 per round; the remaining `tail` tiles are cut into nsplit K
// slices each.  split_all cuts every tile (bulk = 0); otherwise only the tiles that do
// not fill a round are cut.
struct PtileWork {
    int tiles_m, tiles_n, GM, bulk, tail, nsplit, rounds, slots;
    bool ok;
};
PtileWork ptile_work(int m, int n, int bm, int bn, int nsplit, bool split_all);
// The scratch of a K-sliced launch starts with one arrival counter per cut tile (the slice that
// arrives last adds the slices up), then the slices' partial sums follow.
constexpr size_t kSliceCounterBytes = 16 * 1024;
constexpr int kMaxSliceCounters = (int)(kSliceCounterBytes / sizeof(int));
int tile_column_block(int tiles_n, int m, int n, int k);
size_t ptile_scratch_bytes(const PtileWork &w, int bm, int bn);

// the plain entry points: bare fp32 sums, no scaling
bool plain_output(const OutSpec &spec);
// The 16x16x128 forms of the 256 x 256 and 192 x 256 tiles need at least two 128-byte K tiles per work
// item (a tile, or one of its nsplit K slices); the last K tile may overhang a K that is a multiple of 16.
bool p2h_ok(int k, int nsplit);

struct SkinnyPlan {
    int mt, tn, variant, nsplit;
};
bool skinny_ok(int m, int k, int n);
SkinnyPlan plan_skinny(int m, int k, int n);
int select_algo(int m, int k, int n);

// Which tiled kernel, how many K slices, which K-walk rotation.
struct TilePlan {
    int variant, nsplit, rotate;
    bool split_all;      // K slices for every tile (else only for the tiles that do not fill a round)
};
// allowed: bit v set = tile shape number v may be picked
TilePlan plan_tile(int m, int k, int n, unsigned allowed = ~0u);
size_t tile_plan_scratch_bytes(int m, int n, const TilePlan &p);

// Where the partial sums of one call's K slices go: a buffer of the per-(device, stream)
// pool, or a fixed buffer (the caller's workspace, or the static array).  A pooled
// workspace keeps the pool locked from its first lookup until it goes out of scope, i.e.
// until the call's kernels are enqueued.
class Workspace {
public:
    static Workspace pooled(hipStream_t stream) { return Workspace(stream, nullptr, 0, true, true); }
    // counters_zero: the first kSliceCounterBytes of the buffer are known to hold zeros
    static Workspace fixed(void *ptr, size_t bytes, bool counters_zero) { return Workspace(nullptr, ptr, bytes, false, counters_zero); }
    hipError_t get(size_t need, void **out);
    // whether the arrival counters at the start of the buffer can be relied on (they start at
    // zero and every kernel leaves them at zero): the pool's buffers and the static array, not a
    // caller's workspace
    bool counters_zero() const { return counters_zero_; }

private:
    Workspace(hipStream_t stream, void *ptr, size_t bytes, bool pooled, bool counters_zero)
        : stream_(stream), ptr_(ptr), bytes_(bytes), pooled_(pooled), counters_zero_(counters_zero) {}
    hipStream_t stream_;
    void *ptr_;
    size_t bytes_;
    bool pooled_;
    bool counters_zero_;
    std::unique_lock<std::mutex> lock_;
};

// out[i] = sum over the nsplit planes of ws, on `stream`
hipError_t launch_reduce(const float *ws, void *out, size_t count, int nsplit, const OutSpec &spec, hipStream_t stream);
// sum of the K slices of the persistent kernel's tail tiles (scratch slots of bm x bn floats) into C
hipError_t launch_tile_slices_reduce(const float *ws, void *out, int m, int n, int k, int bm, int bn, const PtileWork &w,
                                     const OutSpec &spec, hipStream_t stream);

// Validated operands -> kernel choice and launch for one operand pairing (AF, BF: 0 = E4M3,
// 1 = E5M2).  Each pairing is compiled in a translation unit of its own (dispatch_pair.hip).
template <int AF, int BF>
hipError_t dispatch(int m, int k, int n, const uint8_t *a, const uint8_t *b, void *out,
                    int algo, int variant, int nsplit, const OutSpec &spec, Workspace &wsp, hipStream_t stream);

// The same for a sparse A in blocked-ELL form whose blocks hold whole tiles (block % 128 == 0):
// `values` is the m x kell matrix of stored values, `bell` the block list and B's row stride.
template <int AF, int BF>
hipError_t dispatch_bell(int m, int kell, int n, const uint8_t *values, const uint8_t *b, float *out, const BellSpec &bell,
                         Workspace &wsp, hipStream_t stream);

}  // namespace fp8gemm_detail

#endif  // FP8GEMM_PLAN_H
