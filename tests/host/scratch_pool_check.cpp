// Host check of the scratch bookkeeping (tensor-core-fp8_amd/csrc/scratch_pool.h) with a
// fake device runtime: "events" pass when the test says so, "allocations" are counted.
// Exit status 0 = every expectation held; each failure prints its line.
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <thread>

#include "scratch_pool.h"

static int g_failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("line %d: expectation failed: %s\n", __LINE__, #cond); \
            ++g_failures;                                                   \
        }                                                                   \
    } while (0)

struct FakeState {
    int allocs = 0, frees = 0, next_event = 1;
    size_t live_bytes = 0;
    std::map<void *, size_t> buffers;
    std::map<int, void *> event_stream;      // event -> stream it was recorded on
    std::set<int> passed;
    bool fail_alloc = false;
};

struct FakeBackend {
    using Event = int;
    FakeState *st;
    int alloc(size_t bytes, void *, void **ptr)
    {
        if (st->fail_alloc) return 2;
        *ptr = std::malloc(16);
        st->buffers[*ptr] = bytes;
        st->live_bytes += bytes;
        ++st->allocs;
        return 0;
    }
    void free(void *ptr)
    {
        st->live_bytes -= st->buffers.at(ptr);
        st->buffers.erase(ptr);
        std::free(ptr);
        ++st->frees;
    }
    int record(void *stream, Event *ev)
    {
        *ev = st->next_event++;
        st->event_stream[*ev] = stream;
        return 0;
    }
    bool passed(Event ev) { return st->passed.count(ev) != 0; }
    void drop(Event ev) { st->event_stream.erase(ev); }
};

int main()
{
    FakeState st;
    ScratchPool<FakeBackend> pool(FakeBackend{&st});
    void *s1 = (void *)0x10, *s2 = (void *)0x20;
    void *a = nullptr, *b = nullptr, *c = nullptr;

    // two streams never share a buffer; a second call on a stream reuses its buffer
    EXPECT(pool.get(0, s1, 1000, &a) == 0);
    EXPECT(pool.get(0, s2, 1000, &b) == 0);
    EXPECT(a && b && a != b);
    EXPECT(pool.get(0, s1, 500, &c) == 0 && c == a);
    EXPECT(st.allocs == 2 && st.frees == 0);
    // sizes are rounded up to whole 2 MiB granules
    EXPECT(pool.held_bytes(0) == 2 * ((size_t)2 << 20));
    EXPECT(pool.get(0, s1, (size_t)2 << 20, &c) == 0 && c == a);

    // growth: the stream gets a new buffer, the old one is retired behind an event recorded
    // on that stream, nothing is freed
    void *big = nullptr;
    EXPECT(pool.get(0, s1, (size_t)5 << 20, &big) == 0);
    EXPECT(big != a && big != b);
    EXPECT(st.allocs == 3 && st.frees == 0);
    EXPECT(st.event_stream.size() == 1 && st.event_stream.begin()->second == s1);
    const int ev_a = st.event_stream.begin()->first;

    // while that event is pending the retired buffer is not handed out: stream 2 growing to a
    // size the retired buffer could not hold anyway allocates; a new stream asking for little
    // allocates as well (buffer `a` may still be read by stream 1's earlier kernels)
    void *s3 = (void *)0x30, *d = nullptr;
    EXPECT(pool.get(0, s3, 100, &d) == 0);
    EXPECT(d != a && st.allocs == 4);
    // once the event has passed, the retired buffer serves the next request that fits
    st.passed.insert(ev_a);
    void *s4 = (void *)0x40, *e = nullptr;
    EXPECT(pool.get(0, s4, 100, &e) == 0);
    EXPECT(e == a && st.allocs == 4);
    EXPECT(st.event_stream.empty());                 // its event was dropped

    // another device has its own buffers, also for the same stream handle
    void *f = nullptr;
    EXPECT(pool.get(1, s1, 100, &f) == 0);
    EXPECT(f != big && st.allocs == 5);

    // the smallest fitting retired buffer is preferred
    void *g1 = nullptr, *g2 = nullptr;
    EXPECT(pool.get(0, s2, (size_t)3 << 20, &g1) == 0);        // retires b (2 MiB)
    EXPECT(pool.get(0, s3, (size_t)7 << 20, &g2) == 0);        // retires d (2 MiB)
    for (auto &kv : st.event_stream) st.passed.insert(kv.first);
    void *s5 = (void *)0x50, *h = nullptr;
    EXPECT(pool.get(0, s5, 10, &h) == 0);
    EXPECT((h == b || h == d) && st.allocs == 7);

    // an allocation failure is reported and leaves the stream without a buffer, not with a stale one
    st.fail_alloc = true;
    void *s6 = (void *)0x60, *z = nullptr;
    EXPECT(pool.get(0, s6, (size_t)64 << 20, &z) == 2);
    st.fail_alloc = false;
    EXPECT(pool.get(0, s6, (size_t)64 << 20, &z) == 0 && z);

    // release frees everything of one device and nothing of another
    const int allocs = st.allocs;
    pool.release(0);
    EXPECT(pool.held_bytes(0) == 0);
    EXPECT(pool.held_bytes(1) == ((size_t)2 << 20));
    EXPECT(st.frees == allocs - 1);
    pool.release(1);
    EXPECT(st.live_bytes == 0 && st.buffers.empty());

    // many threads, each holding the mutex from lookup to "enqueue": a stream's buffer is
    // stable while the lock is held, and streams never collide
    {
        FakeState st2;
        ScratchPool<FakeBackend> pool2(FakeBackend{&st2});
        std::set<void *> seen[4];
        std::thread th[4];
        bool clash = false;
        for (int t = 0; t < 4; ++t)
            th[t] = std::thread([&, t] {
                for (int i = 0; i < 2000; ++i) {
                    std::lock_guard<std::mutex> lock(pool2.mutex());
                    void *p = nullptr;
                    if (pool2.get(0, (void *)(uintptr_t)(0x100 + t), 1000 + (size_t)(i % 7) * ((size_t)1 << 20), &p) != 0) clash = true;
                    seen[t].insert(p);
                }
            });
        for (auto &x : th) x.join();
        for (int t = 0; t < 4; ++t)
            for (int u = t + 1; u < 4; ++u)
                for (void *p : seen[t])
                    if (seen[u].count(p)) clash = true;     // no event ever passes here, so no buffer may move
        EXPECT(!clash);
        pool2.release(0);
    }

    if (g_failures == 0) std::printf("scratch pool: all checks passed\n");
    return g_failures == 0 ? 0 : 1;
}
