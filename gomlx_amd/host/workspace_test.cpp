// Host-only test of the scratch-memory bookkeeping (gomlx_amd/csrc/workspace.hpp) against fake
// device hooks: growth, retirement, graph pinning, stream destruction, and the sequence lock that
// keeps two host threads on one stream from interleaving their launches.  No GPU, no HIP.
#include "../csrc/workspace.hpp"

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <set>
#include <thread>

using namespace gq;

namespace {

std::mutex g_mu;
std::set<void *> g_live;          // what the fake allocator has handed out and not taken back
std::set<const void *> g_capturing;
int g_syncs = 0, g_allocs = 0, g_frees = 0, g_double_free = 0;

int fake_alloc(void **p, size_t bytes) {
    std::lock_guard<std::mutex> l(g_mu);
    *p = std::malloc(bytes > 64 ? 64 : bytes);  // the test never touches the memory
    g_live.insert(*p);
    g_allocs++;
    return 0;
}
void fake_release(void *p) {
    std::lock_guard<std::mutex> l(g_mu);
    if (!g_live.erase(p)) g_double_free++;
    else std::free(p);
    g_frees++;
}
void fake_sync(const void *) { std::lock_guard<std::mutex> l(g_mu); g_syncs++; }
bool fake_capturing(const void *s) { std::lock_guard<std::mutex> l(g_mu); return g_capturing.count(s) != 0; }
void set_capturing(const void *s, bool on) {
    std::lock_guard<std::mutex> l(g_mu);
    if (on) g_capturing.insert(s); else g_capturing.erase(s);
}

int failures = 0;
#define CHECK(cond)                                                            \
    do {                                                                       \
        if (!(cond)) { std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); failures++; } \
    } while (0)

void *get(WorkspacePool &pool, const void *s, int slot, size_t bytes, int *rc_out = nullptr) {
    WsStreamRef st = pool.stream(s);
    SeqLock lock;
    lock.lock(st);
    void *p = nullptr;
    const int rc = pool.acquire(*st, s, slot, bytes, &p);
    if (rc_out) *rc_out = rc;
    return rc == kWsOk ? p : nullptr;
}

}  // namespace

int main() {
    const WsHooks hooks{fake_alloc, fake_release, fake_sync, fake_capturing};
    const void *s1 = reinterpret_cast<const void *>(0x1000), *s2 = reinterpret_cast<const void *>(0x2000);

    {   // reuse, growth, separate streams and slots
        WorkspacePool pool(hooks);
        void *a = get(pool, s1, 0, 1000);
        CHECK(a && pool.live_blocks() == 1 && pool.live_bytes() == kWsMinBytes);
        CHECK(get(pool, s1, 0, 2000) == a);                        // fits: same buffer
        void *b = get(pool, s1, 1, 10);
        CHECK(b && b != a && pool.live_blocks() == 2);             // other slot: other buffer
        void *c = get(pool, s2, 0, 10);
        CHECK(c && c != a && c != b && pool.live_blocks() == 3);   // other stream: other buffer
        const int syncs = g_syncs;
        void *d = get(pool, s1, 0, kWsMinBytes + 1);               // outgrown: drained, freed, replaced
        CHECK(d && pool.live_blocks() == 3 && pool.live_bytes() == 2 * kWsMinBytes + 2 * kWsMinBytes);
        CHECK(g_syncs == syncs + 1);
        CHECK(g_live.count(a) == 0);
        pool.destroy_stream(s1);
        CHECK(pool.live_blocks() == 1 && pool.stream_count() == 1);
        pool.destroy_stream(s2);
        CHECK(pool.live_blocks() == 0 && pool.live_bytes() == 0 && pool.stream_count() == 0);
        pool.destroy_stream(s2);                                   // unknown stream: nothing happens
    }
    CHECK(g_live.empty() && g_double_free == 0);

    {   // a recording may not allocate, pins what it uses, and the pin outlives growth and the stream
        WorkspacePool pool(hooks);
        int rc = 0;
        pool.begin_recording(s1);
        set_capturing(s1, true);
        CHECK(get(pool, s1, 0, 100, &rc) == nullptr && rc == kWsWouldAllocateInRecording);
        set_capturing(s1, false);
        (void)pool.end_recording(s1);
        void *a = get(pool, s1, 0, 100);
        pool.begin_recording(s1);
        set_capturing(s1, true);
        CHECK(get(pool, s1, 0, 100) == a);
        CHECK(get(pool, s1, 0, 50) == a);                          // pinned once however often it is used
        CHECK(get(pool, s1, 0, 2 * kWsMinBytes, &rc) == nullptr && rc == kWsWouldAllocateInRecording);
        set_capturing(s1, false);
        std::vector<WsBlockRef> graph = pool.end_recording(s1);
        CHECK(graph.size() == 1 && graph[0]->ptr == a && graph[0]->graph_refs == 1);
        void *b = get(pool, s1, 0, 2 * kWsMinBytes);               // outgrown while a graph points at it: kept
        CHECK(b && b != a && g_live.count(a) == 1 && pool.live_blocks() == 2);
        pool.begin_recording(s1);                                  // second graph on the new buffer
        set_capturing(s1, true);
        CHECK(get(pool, s1, 0, 10) == b);
        set_capturing(s1, false);
        std::vector<WsBlockRef> graph2 = pool.end_recording(s1);
        pool.destroy_stream(s1);                                   // the stream goes, both graphs still hold their buffers
        CHECK(g_live.count(a) == 1 && g_live.count(b) == 1 && pool.live_blocks() == 2);
        pool.unpin(graph);
        CHECK(g_live.count(a) == 0 && g_live.count(b) == 1 && pool.live_blocks() == 1);
        pool.unpin(graph2);
        CHECK(pool.live_blocks() == 0 && pool.live_bytes() == 0);
        // an abandoned recording's pins are dropped by the next begin
        void *c = get(pool, s2, 0, 10);
        pool.begin_recording(s2);
        set_capturing(s2, true);
        CHECK(get(pool, s2, 0, 10) == c);
        set_capturing(s2, false);
        pool.begin_recording(s2);
        CHECK(pool.stream(s2)->cur[0]->graph_refs == 0);
        pool.destroy_stream(s2);
        CHECK(pool.live_blocks() == 0);
    }
    CHECK(g_live.empty() && g_double_free == 0);

    {   // two host threads on one stream: their sequences (acquire ... last launch) never interleave
        WorkspacePool pool(hooks);
        std::atomic<int> inside{0}, overlaps{0}, done{0};
        auto worker = [&](const void *s) {
            for (int i = 0; i < 200; i++) {
                WsStreamRef st = pool.stream(s);
                SeqLock lock;
                lock.lock(st);
                lock.lock(st);  // nested request of the same call: no second lock
                void *p = nullptr;
                if (pool.acquire(*st, s, 0, 64, &p) != kWsOk) overlaps += 1000;
                if (inside.fetch_add(1) != 0) overlaps++;
                std::this_thread::sleep_for(std::chrono::microseconds(20));  // "enqueue three kernels"
                inside.fetch_sub(1);
                done++;
            }
        };
        std::thread t1(worker, s1), t2(worker, s1);
        t1.join();
        t2.join();
        CHECK(overlaps == 0 && done == 400);
        // different streams do not wait for each other: both can be inside at once
        std::atomic<int> both{0}, a_in{0}, b_in{0};
        auto hold = [&](const void *s, std::atomic<int> &mine, std::atomic<int> &other) {
            WsStreamRef st = pool.stream(s);
            SeqLock lock;
            lock.lock(st);
            mine = 1;
            for (int i = 0; i < 2000 && !other; i++) std::this_thread::sleep_for(std::chrono::microseconds(100));
            if (other) both++;
        };
        std::thread t3(hold, s1, std::ref(a_in), std::ref(b_in)), t4(hold, s2, std::ref(b_in), std::ref(a_in));
        t3.join();
        t4.join();
        CHECK(both == 2);
        pool.destroy_stream(s1);
        pool.destroy_stream(s2);
        CHECK(pool.live_blocks() == 0);
    }
    CHECK(g_live.empty() && g_double_free == 0 && g_allocs == g_frees);

    std::printf("workspace bookkeeping: %d failed\n", failures);
    return failures ? 1 : 0;
}
