// allocator.hpp -- stream-ordered caching device allocator.
//
// Replaces ZeNu's host-side memory pool (zenu-matrix/src/memory_pool/mod.rs:79-145: three size
// classes, bump pointers inside slabs, not stream aware) together with cuda_malloc_bytes /
// cuda_free (zenu-cuda/src/runtime/mod.rs:30-60), which synchronise the stream on every call.
//
// Design
//   * Two pools.  Requests <= 1 MiB are carved out of 2 MiB segments; larger requests come from
//     segments of 20 MiB (requests < 10 MiB) or of the request rounded up to 2 MiB.  The
//     segment sizes are the reference's slab sizes (memory_pool/mod.rs:70-84); unlike its
//     bump-pointer slabs, blocks are split on allocation and merged with free neighbours on
//     release, so holes in the middle of a segment are reusable.
//   * Stream ordered.  Every free block belongs to the stream it was freed on.  An allocation
//     on the same stream reuses it immediately: the kernels already queued on that stream run
//     before anything the new owner enqueues.  An allocation on another stream may take the
//     block only through an event: record on the owner stream, make the new stream wait.  No
//     host synchronisation on any hit.
//   * Out of memory: wait for the device, release every completely free segment, retry once
//     (the flow memory_pool/mod.rs:9-20 describes), then report ZENU_ERR_OOM.
//   * free() of a pointer the pool does not know returns ZENU_ERR_NOT_OWNED so the caller can
//     fall back to a raw free (device/mod.rs:34-45).
//   * Stream capture.  A kernel recorded into a graph keeps the addresses it was recorded with
//     and writes them again on every replay, long after the capture's own frees.  A block that a
//     capturing stream takes from the pool is therefore marked; whenever it is freed (during
//     the capture or later) it goes to a list that only later captures on the same stream may
//     draw from (inside one capture the recorded order makes reuse safe), never to an ordinary
//     request.  release_captured(stream) -- or retiring the stream -- returns those blocks to
//     the ordinary lists once the caller has destroyed the graphs.
//
// The device is reached only through `Backend`, so the bookkeeping is testable on the host
// with a fake backend (as memory_pool/test.rs:18-49 does with MockDeviceBase).
#pragma once

#include <stdint.h>

#include <map>
#include <mutex>
#include <set>
#include <unordered_map>
#include <vector>

namespace zenu {

struct AllocBackend {
    virtual ~AllocBackend() {}
    virtual int raw_alloc(void **p, size_t bytes) = 0;  // 0 = ok, else out of memory / error
    virtual int raw_free(void *p) = 0;
    // order `waiter` after everything queued on `owner` so far; 0 = ok
    virtual int order_after(void *owner_stream, void *waiter_stream) = 0;
    virtual int device_synchronize() = 0;
};

struct AllocStats {
    uint64_t bytes_in_use = 0, bytes_cached = 0, bytes_reserved = 0;
    uint64_t n_alloc_calls = 0, n_cache_hits = 0, n_driver_allocs = 0, n_driver_frees = 0,
             n_oom_retries = 0;
};

class CachingAllocator {
public:
    static constexpr size_t kMinBlock = 512;               // rounding of every request
    static constexpr size_t kSmallLimit = 1u << 20;        // <= 1 MiB -> small pool
    static constexpr size_t kSmallSegment = 2u << 20;      // 2 MiB
    static constexpr size_t kLargeSegment = 20u << 20;     // 20 MiB
    static constexpr size_t kLargeSplitLimit = 10u << 20;  // < 10 MiB share a 20 MiB segment
    static constexpr size_t kRoundLarge = 2u << 20;

    // status codes mirror zenu_status_t: 0 ok, 4 arg, 6 oom, 8 not owned, 5 backend failure
    enum { kOk = 0, kErrArg = 4, kErrBackend = 5, kErrOom = 6, kErrNotOwned = 8 };

    explicit CachingAllocator(AllocBackend *backend) : be_(backend) {}
    ~CachingAllocator() { release_all(); }

    // `capturing`: `stream` is recording a graph (the caller asks the runtime)
    int malloc(void **out, size_t bytes, void *stream, bool capturing = false)
    {
        if (!out) return kErrArg;
        *out = nullptr;
        std::lock_guard<std::mutex> g(mu_);
        stats_.n_alloc_calls++;
        if (bytes == 0) bytes = 1;
        const size_t size = round_size(bytes);
        const bool small = size <= kSmallLimit;

        Block *b = nullptr;
        if (capturing) b = take_free_block(size, small, stream, /*other_streams=*/false, /*captured=*/true);
        if (!b) b = take_free_block(size, small, stream, /*other_streams=*/false);
        // a block of another stream comes with an event wait, which a capture would record: not then
        if (!b && !capturing) b = take_free_block(size, small, stream, /*other_streams=*/true);
        if (b) {
            stats_.n_cache_hits++;
        } else {
            size_t seg = segment_size(size);
            void *p = nullptr;
            int rc = be_->raw_alloc(&p, seg);
            if (rc != 0 || !p) {
                // out of memory: drop the cache and retry once
                stats_.n_oom_retries++;
                be_->device_synchronize();
                release_free_segments();
                rc = be_->raw_alloc(&p, seg);
                if (rc != 0 || !p) return kErrOom;
            }
            stats_.n_driver_allocs++;
            stats_.bytes_reserved += seg;
            b = new Block();
            b->ptr = static_cast<char *>(p);
            b->size = seg;
            b->small = small;
            b->stream = stream;
            b->segment_head = true;
        }
        // split when the remainder is worth keeping
        const size_t min_rem = small ? kMinBlock : kSmallLimit + kMinBlock;
        if (b->size - size >= min_rem) {
            Block *r = new Block();
            r->ptr = b->ptr + size;
            r->size = b->size - size;
            r->small = b->small;
            r->stream = stream;
            r->captured = b->captured;
            r->capture_stream = b->capture_stream;
            r->prev = b;
            r->next = b->next;
            if (b->next) b->next->prev = r;
            b->next = r;
            b->size = size;
            insert_free(r);
        }
        b->allocated = true;
        b->stream = stream;
        if (capturing) {
            b->captured = true;
            b->capture_stream = stream;
        }
        live_[b->ptr] = b;
        stats_.bytes_in_use += b->size;
        *out = b->ptr;
        return kOk;
    }

    int free(void *p, void *stream)
    {
        if (!p) return kOk;
        std::lock_guard<std::mutex> g(mu_);
        auto it = live_.find(static_cast<char *>(p));
        if (it == live_.end()) return kErrNotOwned;
        Block *b = it->second;
        live_.erase(it);
        stats_.bytes_in_use -= b->size;
        b->allocated = false;
        if (b->captured) stream = b->capture_stream;   // stays with the graphs of the stream that recorded it
        if (retired_.count(stream)) stream = nullptr;  // freed after its stream was destroyed (and synchronised)
        b->stream = stream;  // the last stream to use the block: stream-ordered free
        // merge with free neighbours that belong to the same stream
        b = try_merge(b, b->prev);
        b = try_merge(b, b->next);
        insert_free(b);
        return kOk;
    }

    // hand every completely free segment back to the driver
    int trim()
    {
        std::lock_guard<std::mutex> g(mu_);
        be_->device_synchronize();
        release_free_segments();
        return kOk;
    }

    // The graphs recorded on `stream` are gone: the blocks their captures took from the pool become
    // ordinary blocks again (free ones now, live ones when they are freed).
    void release_captured(void *stream)
    {
        std::lock_guard<std::mutex> g(mu_);
        release_captured_locked(stream);
    }

    // bytes held back for the graphs of all streams (free blocks only)
    uint64_t bytes_captured()
    {
        std::lock_guard<std::mutex> g(mu_);
        uint64_t n = 0;
        for (auto &kv : free_)
            if (kv.first.captured)
                for (Block *b : kv.second) n += b->size;
        return n;
    }

    // `stream` is about to be destroyed and has been synchronised: its cached blocks are idle,
    // so they move to the null stream's lists (nobody may order work after a dead stream).
    void retire_stream(void *stream)
    {
        if (!stream) return;
        std::lock_guard<std::mutex> g(mu_);
        release_captured_locked(stream);
        retired_.insert(stream);
        for (int small = 0; small < 2; small++) {
            auto it = free_.find(PoolKey{stream, small != 0, false});
            if (it == free_.end()) continue;
            std::vector<Block *> blocks(it->second.begin(), it->second.end());
            free_.erase(it);
            for (Block *b : blocks) {
                stats_.bytes_cached -= b->size;
                b->stream = nullptr;
                insert_free(b);
            }
        }
    }

    // a new stream may get the handle value of a destroyed one
    void adopt_stream(void *stream)
    {
        std::lock_guard<std::mutex> g(mu_);
        retired_.erase(stream);
    }

    AllocStats stats()
    {
        std::lock_guard<std::mutex> g(mu_);
        return stats_;
    }

    bool owns(void *p)
    {
        std::lock_guard<std::mutex> g(mu_);
        return live_.count(static_cast<char *>(p)) != 0;
    }

    static size_t round_size(size_t bytes)
    {
        if (bytes <= kSmallLimit) return (bytes + kMinBlock - 1) / kMinBlock * kMinBlock;
        return (bytes + kRoundLarge - 1) / kRoundLarge * kRoundLarge;
    }

    static size_t segment_size(size_t rounded)
    {
        if (rounded <= kSmallLimit) return kSmallSegment;
        if (rounded < kLargeSplitLimit) return kLargeSegment;
        return rounded;
    }

private:
    struct Block {
        char *ptr = nullptr;
        size_t size = 0;
        bool small = false;
        bool allocated = false;
        bool segment_head = false;  // first block of a driver allocation
        bool captured = false;      // taken from the pool by a capturing stream: recorded kernels hold its address
        void *capture_stream = nullptr;
        void *stream = nullptr;
        Block *prev = nullptr, *next = nullptr;  // neighbours inside the segment
    };
    struct BlockLess {
        bool operator()(const Block *a, const Block *b) const
        {
            if (a->size != b->size) return a->size < b->size;
            return a->ptr < b->ptr;
        }
    };
    typedef std::set<Block *, BlockLess> FreeSet;
    struct PoolKey {
        void *stream;
        bool small;
        bool captured;
        bool operator<(const PoolKey &o) const
        {
            if (stream != o.stream) return stream < o.stream;
            if (small != o.small) return small < o.small;
            return captured < o.captured;
        }
    };

    void insert_free(Block *b)
    {
        free_[PoolKey{b->stream, b->small, b->captured}].insert(b);
        stats_.bytes_cached += b->size;
    }
    void erase_free(Block *b)
    {
        auto it = free_.find(PoolKey{b->stream, b->small, b->captured});
        if (it != free_.end()) it->second.erase(b);
        stats_.bytes_cached -= b->size;
    }

    // best fit in one stream's list (other_streams=false) or any other stream's (true); `captured`
    // selects the blocks held back for the stream's graphs instead of the ordinary ones
    Block *take_free_block(size_t size, bool small, void *stream, bool other_streams, bool captured = false)
    {
        Block key;
        key.size = size;
        key.ptr = nullptr;
        for (auto &kv : free_) {
            if (kv.first.small != small || kv.first.captured != captured) continue;
            if ((kv.first.stream == stream) == other_streams) continue;
            FreeSet &fs = kv.second;
            auto it = fs.lower_bound(&key);
            if (it == fs.end()) continue;
            Block *b = *it;
            // do not burn a huge block on a much smaller large-pool request
            if (!small && size >= kLargeSplitLimit && b->size >= size + kLargeSegment) continue;
            if (other_streams) {
                if (be_->order_after(b->stream, stream) != 0) continue;
            }
            fs.erase(it);
            stats_.bytes_cached -= b->size;
            return b;
        }
        return nullptr;
    }

    Block *try_merge(Block *b, Block *nb)
    {
        if (!nb || nb->allocated || nb->stream != b->stream || nb->captured != b->captured) return b;
        erase_free(nb);
        if (nb == b->prev) {
            nb->size += b->size;
            nb->next = b->next;
            if (b->next) b->next->prev = nb;
            delete b;
            return nb;
        }
        b->size += nb->size;
        b->next = nb->next;
        if (nb->next) nb->next->prev = b;
        delete nb;
        return b;
    }

    void release_captured_locked(void *stream)
    {
        for (int small = 0; small < 2; small++) {
            auto it = free_.find(PoolKey{stream, small != 0, true});
            if (it == free_.end()) continue;
            std::vector<Block *> blocks(it->second.begin(), it->second.end());
            free_.erase(it);
            for (Block *b : blocks) {
                stats_.bytes_cached -= b->size;
                b->captured = false;
                b->capture_stream = nullptr;
                b = try_merge(b, b->prev);
                b = try_merge(b, b->next);
                insert_free(b);
            }
        }
        for (auto &kv : live_)
            if (kv.second->captured && kv.second->capture_stream == stream) {
                kv.second->captured = false;
                kv.second->capture_stream = nullptr;
            }
    }

    // Only after device_synchronize(): nothing is in flight, so free neighbours can be joined
    // whatever stream they were freed on.  Blocks held back for graphs stay as they are.
    void coalesce_across_streams()
    {
        std::vector<Block *> all;
        for (auto it = free_.begin(); it != free_.end();) {
            if (it->first.captured) {
                ++it;
                continue;
            }
            for (Block *b : it->second) {
                all.push_back(b);
                stats_.bytes_cached -= b->size;
            }
            it = free_.erase(it);
        }
        std::set<Block *> dead;
        for (Block *b : all) {
            if (dead.count(b)) continue;
            if (b->prev && !b->prev->allocated && !b->prev->captured) continue;  // not the head of its free run
            while (b->next && !b->next->allocated && !b->next->captured) {
                Block *n = b->next;
                b->size += n->size;
                b->next = n->next;
                if (n->next) n->next->prev = b;
                dead.insert(n);
            }
        }
        for (Block *b : all) {
            if (dead.count(b)) delete b;
            else insert_free(b);
        }
    }

    void release_free_segments()
    {
        coalesce_across_streams();
        for (auto &kv : free_) {
            if (kv.first.captured) continue;   // recorded kernels still hold these addresses
            FreeSet &fs = kv.second;
            for (auto it = fs.begin(); it != fs.end();) {
                Block *b = *it;
                if (b->segment_head && !b->prev && !b->next) {
                    it = fs.erase(it);
                    stats_.bytes_cached -= b->size;
                    stats_.bytes_reserved -= b->size;
                    stats_.n_driver_frees++;
                    be_->raw_free(b->ptr);
                    delete b;
                } else {
                    ++it;
                }
            }
        }
    }

    void release_all()
    {
        std::lock_guard<std::mutex> g(mu_);
        release_free_segments();
        // blocks still live or fragmented at shutdown: free their segments through the heads
        std::vector<Block *> rest;
        for (auto &kv : free_)
            for (Block *b : kv.second) rest.push_back(b);
        for (auto &kv : live_) rest.push_back(kv.second);
        free_.clear();
        live_.clear();
        for (Block *b : rest)
            if (b->segment_head) {
                be_->raw_free(b->ptr);
                stats_.n_driver_frees++;
            }
        for (Block *b : rest) delete b;
        stats_.bytes_cached = stats_.bytes_in_use = stats_.bytes_reserved = 0;
    }

    AllocBackend *be_;
    std::mutex mu_;
    std::map<PoolKey, FreeSet> free_;
    std::unordered_map<char *, Block *> live_;
    std::set<void *> retired_;   // destroyed streams: blocks freed in their name go to the null stream
    AllocStats stats_;
};

}  // namespace zenu
