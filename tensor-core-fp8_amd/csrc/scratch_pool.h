// Bookkeeping of the device scratch that holds the partial sums of K slices.
//
// The launch functions this library stands in for are stateless and re-entrant
// (GEMM/src/gemm.cu:263-277 of the reference): two calls on different streams may
// overlap freely.  A K-sliced launch needs device memory of its own between its two
// kernels, so the scratch is kept per (device, stream): work queued on one stream is
// ordered, work on different streams never shares a buffer.
//
// Rules:
//   * get() is called with the pool's mutex held, and the caller keeps holding it until
//     the kernels that use the buffer have been enqueued (see Lease): a buffer cannot be
//     handed on between another thread's lookup and its launch.
//   * a stream whose buffer is too small receives another one; the old one is retired
//     behind an event recorded on that stream and becomes reusable (by any stream of the
//     device) once the event has passed.  Nothing is freed and nothing waits inside a
//     launch; release() frees what a device holds, after the caller has synchronised it.
//
// The device runtime is reached through a Backend type, so the bookkeeping can be
// exercised on the host with a fake one:
//   int  alloc(size_t bytes, void *stream, void **ptr)   a new buffer, made ready for use by work queued on
//                                               `stream` from now on; 0 on success, else an error code
//   void free(void *ptr)
//   int  record(void *stream, Event *ev)        marks what `stream` has queued so far
//   bool passed(Event ev)                       true once that work is done
//   void drop(Event ev)
#ifndef FP8GEMM_SCRATCH_POOL_H
#define FP8GEMM_SCRATCH_POOL_H

#include <cstddef>
#include <mutex>
#include <vector>

template <class Backend>
class ScratchPool {
public:
    using Event = typename Backend::Event;

    explicit ScratchPool(Backend backend = Backend()) : backend_(backend) {}

    std::mutex &mutex() { return mutex_; }

    // Buffer of at least `bytes` for (dev, stream).  Mutex held by the caller.
    int get(int dev, void *stream, size_t bytes, void **out)
    {
        Slot *slot = nullptr;
        for (Slot &s : slots_)
            if (s.dev == dev && s.stream == stream) slot = &s;
        if (!slot) {
            slots_.push_back(Slot{dev, stream, nullptr, 0});
            slot = &slots_.back();
        }
        if (slot->bytes >= bytes && slot->ptr) {
            *out = slot->ptr;
            return 0;
        }
        // the stream's earlier launches may still use its present buffer
        if (slot->ptr) {
            Event ev;
            const int e = backend_.record(stream, &ev);
            if (e != 0) return e;
            retired_.push_back(Retired{dev, slot->ptr, slot->bytes, ev});
            slot->ptr = nullptr;
            slot->bytes = 0;
        }
        // smallest retired buffer of the device that is large enough and no longer in use
        int pick = -1;
        for (int i = 0; i < (int)retired_.size(); ++i) {
            const Retired &r = retired_[i];
            if (r.dev != dev || r.bytes < bytes) continue;
            if (pick >= 0 && retired_[pick].bytes <= r.bytes) continue;
            if (backend_.passed(r.done)) pick = i;
        }
        if (pick >= 0) {
            backend_.drop(retired_[pick].done);
            slot->ptr = retired_[pick].ptr;
            slot->bytes = retired_[pick].bytes;
            retired_.erase(retired_.begin() + pick);
        } else {
            const size_t granule = (size_t)2 << 20;
            const size_t want = (bytes + granule - 1) / granule * granule;
            void *p = nullptr;
            const int e = backend_.alloc(want, stream, &p);
            if (e != 0) return e;
            slot->ptr = p;
            slot->bytes = want;
        }
        *out = slot->ptr;
        return 0;
    }

    // Bytes the pool holds on a device (buffers in use and retired ones).
    size_t held_bytes(int dev)
    {
        size_t total = 0;
        for (const Slot &s : slots_)
            if (s.dev == dev) total += s.bytes;
        for (const Retired &r : retired_)
            if (r.dev == dev) total += r.bytes;
        return total;
    }

    // Frees everything held on a device.  The caller has synchronised the device, so no
    // kernel uses any of it; mutex held by the caller.
    void release(int dev)
    {
        for (size_t i = 0; i < slots_.size();) {
            if (slots_[i].dev == dev) {
                if (slots_[i].ptr) backend_.free(slots_[i].ptr);
                slots_.erase(slots_.begin() + i);
            } else {
                ++i;
            }
        }
        for (size_t i = 0; i < retired_.size();) {
            if (retired_[i].dev == dev) {
                backend_.drop(retired_[i].done);
                backend_.free(retired_[i].ptr);
                retired_.erase(retired_.begin() + i);
            } else {
                ++i;
            }
        }
    }

    Backend &backend() { return backend_; }

private:
    struct Slot {
        int dev;
        void *stream;
        void *ptr;
        size_t bytes;
    };
    struct Retired {
        int dev;
        void *ptr;
        size_t bytes;
        Event done;
    };
    Backend backend_;
    std::mutex mutex_;
    std::vector<Slot> slots_;
    std::vector<Retired> retired_;
};

#endif  // FP8GEMM_SCRATCH_POOL_H
