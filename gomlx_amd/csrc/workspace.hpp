// Scratch memory of the paths that need more than their inputs and outputs (split-K partial sums and
// activation images, the 16-bit weight image of the two-pass GEMM, the temporaries of composed calls).
//
// Rules the pool keeps:
//   * One buffer per (stream, slot); it grows geometrically and is reused by every later call on
//     the stream.  Work on one stream executes in order, so reuse is safe as long as the launches of
//     two calls are not interleaved: a caller holds the stream's sequence lock from its first request
//     until its last launch has been enqueued (SeqLock below; the lock is recursive because composed
//     entry points call the plain ones).  Two host threads that share a stream therefore enqueue
//     their sequences one after the other; threads on different streams never meet.
//   * A recording (stream capture) pins the buffers it points at: they stay allocated until the
//     recorded graph is destroyed, also when the stream outgrows or loses them in the meantime.
//   * Destroying a stream releases its buffers (those pinned by a graph: when the graph goes).
//
// The pool only does bookkeeping; device memory comes from hooks, so the same code runs against HIP
// in the library and against counters in the host-side test.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

namespace gq {

struct WsHooks {
    int (*alloc)(void **p, size_t bytes);     // 0 on success, a gq_status otherwise
    void (*release)(void *p);
    void (*sync)(const void *stream);         // returns when the work enqueued on the stream so far is done
    bool (*capturing)(const void *stream);    // a graph is being recorded on the stream
};

// 0: the dense kernels, 1: operations composed of several dense calls, 2: bf16 activations widened to fp32 for the
// entry points that take the callers around a projection in bf16
constexpr int kWsSlots = 3, kWsWidenSlot = 2;
constexpr size_t kWsMinBytes = (size_t)4 << 20;

struct WsBlock {
    void *ptr = nullptr;
    size_t bytes = 0;
    int graph_refs = 0;     // recorded graphs (and recordings in progress) that point at this block
    bool dropped = false;   // no stream owns it any more: released when graph_refs reaches zero
};
typedef std::shared_ptr<WsBlock> WsBlockRef;

struct WsStream {
    std::recursive_mutex seq;          // one enqueue sequence at a time
    WsBlockRef cur[kWsSlots];
    std::vector<WsBlockRef> recorded;  // blocks the recording in progress on this stream points at
};
typedef std::shared_ptr<WsStream> WsStreamRef;

enum { kWsOk = 0, kWsWouldAllocateInRecording = -1 };

class WorkspacePool {
 public:
    explicit WorkspacePool(const WsHooks &hooks) : hooks_(hooks) {}

    WsStreamRef stream(const void *s) {
        std::lock_guard<std::mutex> lock(mu_);
        WsStreamRef &st = streams_[s];
        if (!st) st = std::make_shared<WsStream>();
        return st;
    }

    // The caller holds st.seq.  Returns kWsOk, kWsWouldAllocateInRecording, or the allocator's status.
    int acquire(WsStream &st, const void *s, int slot, size_t bytes, void **out) {
        const bool rec = hooks_.capturing(s);
        WsBlockRef &cur = st.cur[slot];
        if (!cur || cur->bytes < bytes) {
            if (rec) return kWsWouldAllocateInRecording;
            size_t want = bytes < kWsMinBytes ? kWsMinBytes : bytes;
            if (cur && want < 2 * cur->bytes) want = 2 * cur->bytes;
            void *p = nullptr;
            if (int rc = hooks_.alloc(&p, want)) return rc;
            if (cur) retire(cur, s);
            cur = std::make_shared<WsBlock>();
            cur->ptr = p;
            cur->bytes = want;
            add_live(want);
        }
        if (rec) {
            bool seen = false;
            for (const WsBlockRef &b : st.recorded) seen |= b == cur;
            if (!seen) {
                std::lock_guard<std::mutex> lock(mu_);
                cur->graph_refs++;
                st.recorded.push_back(cur);
            }
        }
        *out = cur->ptr;
        return kWsOk;
    }

    // A recording on `s` starts: whatever an abandoned earlier recording pinned is let go.
    void begin_recording(const void *s) {
        WsStreamRef st = stream(s);
        std::lock_guard<std::recursive_mutex> seq(st->seq);
        std::vector<WsBlockRef> stale;
        stale.swap(st->recorded);
        unpin(stale);
    }
    // The recording on `s` ended: the blocks it points at now belong to the graph (give them back with unpin()).
    std::vector<WsBlockRef> end_recording(const void *s) {
        WsStreamRef st = stream(s);
        std::lock_guard<std::recursive_mutex> seq(st->seq);
        std::vector<WsBlockRef> out;
        out.swap(st->recorded);
        return out;
    }
    void unpin(std::vector<WsBlockRef> &blocks) {
        for (WsBlockRef &b : blocks) {
            bool free_now = false;
            {
                std::lock_guard<std::mutex> lock(mu_);
                if (--b->graph_refs == 0 && b->dropped) free_now = true;
            }
            if (free_now) free_block(*b);
        }
        blocks.clear();
    }

    // The stream is about to be destroyed: wait for it, then release what no graph pins.
    void destroy_stream(const void *s) {
        WsStreamRef st;
        {
            std::lock_guard<std::mutex> lock(mu_);
            auto it = streams_.find(s);
            if (it == streams_.end()) return;
            st = it->second;
            streams_.erase(it);
        }
        std::lock_guard<std::recursive_mutex> seq(st->seq);
        hooks_.sync(s);
        unpin(st->recorded);
        for (WsBlockRef &b : st->cur)
            if (b) { drop(b); b.reset(); }
    }

    size_t live_bytes() { std::lock_guard<std::mutex> lock(mu_); return live_bytes_; }
    size_t live_blocks() { std::lock_guard<std::mutex> lock(mu_); return live_blocks_; }
    size_t stream_count() { std::lock_guard<std::mutex> lock(mu_); return streams_.size(); }

 private:
    // An outgrown block: kernels enqueued earlier may still use it, so the stream is drained first;
    // a block that a graph points at outlives this and goes when the graph does.
    void retire(WsBlockRef &b, const void *s) {
        bool pinned;
        {
            std::lock_guard<std::mutex> lock(mu_);
            pinned = b->graph_refs > 0;
            if (pinned) b->dropped = true;
        }
        if (!pinned) {
            hooks_.sync(s);
            free_block(*b);
        }
    }
    void drop(WsBlockRef &b) {
        bool pinned;
        {
            std::lock_guard<std::mutex> lock(mu_);
            pinned = b->graph_refs > 0;
            if (pinned) b->dropped = true;
        }
        if (!pinned) free_block(*b);
    }
    void free_block(WsBlock &b) {
        if (!b.ptr) return;
        hooks_.release(b.ptr);
        b.ptr = nullptr;
        std::lock_guard<std::mutex> lock(mu_);
        live_bytes_ -= b.bytes;
        live_blocks_--;
    }
    void add_live(size_t bytes) {
        std::lock_guard<std::mutex> lock(mu_);
        live_bytes_ += bytes;
        live_blocks_++;
    }

    WsHooks hooks_;
    std::mutex mu_;                                  // the maps and counters below, and every graph_refs / dropped
    std::map<const void *, WsStreamRef> streams_;
    size_t live_bytes_ = 0, live_blocks_ = 0;
};

// Held by an ABI call for as long as it enqueues launches that share the stream's workspace.
class SeqLock {
 public:
    SeqLock() = default;
    SeqLock(const SeqLock &) = delete;
    SeqLock &operator=(const SeqLock &) = delete;
    ~SeqLock() { unlock(); }
    void lock(const WsStreamRef &st) {
        if (held_) return;
        st->seq.lock();
        held_ = st;
    }
    void unlock() {
        if (held_) { held_->seq.unlock(); held_.reset(); }
    }
    WsStream *held() const { return held_.get(); }
 private:
    WsStreamRef held_;
};

}  // namespace gq
