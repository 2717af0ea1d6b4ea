// Host-only test driver for zenu_amd/csrc/allocator.hpp with a fake device backend (the role
// MockDeviceBase plays in zenu-matrix/src/memory_pool/test.rs:18-49): bookkeeping, stream
// ordering, out-of-memory handling and foreign pointers, without a GPU.
// Prints one "ok <name>" line per check; exits non-zero on the first failure.
#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>

#include "../../zenu_amd/csrc/allocator.hpp"

using namespace zenu;

struct FakeBackend : AllocBackend {
    size_t capacity = 1ull << 40, used = 0;
    uintptr_t next = 0x10000000;
    std::set<void *> live;
    std::vector<std::pair<void *, void *>> orderings;  // (owner stream, waiter stream)
    int syncs = 0, fail_next = 0;
    int raw_alloc(void **p, size_t bytes) override
    {
        if (fail_next > 0) { fail_next--; *p = nullptr; return 1; }
        if (used + bytes > capacity) { *p = nullptr; return 1; }
        *p = reinterpret_cast<void *>(next);
        next += (bytes + 0xfffff) & ~0xfffffull;
        used += bytes;
        live.insert(*p);
        sizes[*p] = bytes;
        return 0;
    }
    int raw_free(void *p) override
    {
        if (!live.count(p)) return 1;
        live.erase(p);
        used -= sizes[p];
        return 0;
    }
    int order_after(void *owner, void *waiter) override { orderings.push_back({owner, waiter}); return 0; }
    int device_synchronize() override { syncs++; return 0; }
    std::map<void *, size_t> sizes;
};

#define CHECK(cond, name)                                             \
    do {                                                              \
        if (!(cond)) { printf("FAIL %s (line %d)\n", name, __LINE__); return 1; } \
    } while (0)

int main()
{
    void *S1 = reinterpret_cast<void *>(0x1), *S2 = reinterpret_cast<void *>(0x2);
    {   // size classes: small requests share a 2 MiB segment, large ones get their own
        FakeBackend be; CachingAllocator a(&be);
        void *p1, *p2, *p3;
        CHECK(a.malloc(&p1, 1000, S1) == 0 && a.malloc(&p2, 5000, S1) == 0, "small alloc");
        CHECK(be.live.size() == 1 && a.stats().bytes_reserved == CachingAllocator::kSmallSegment, "one small segment");
        CHECK((char *)p2 - (char *)p1 == 1024, "512-byte rounding, adjacent blocks");
        CHECK(a.malloc(&p3, 100u << 20, S1) == 0 && be.live.size() == 2, "large alloc own segment");
        CHECK(a.stats().bytes_in_use == 1024 + 5120 + (100u << 20), "bytes_in_use");
        CHECK(a.free(p1, S1) == 0 && a.free(p2, S1) == 0 && a.free(p3, S1) == 0, "free");
        CHECK(a.stats().bytes_in_use == 0 && a.stats().bytes_cached == a.stats().bytes_reserved, "all cached");
        printf("ok size_classes\n");
    }
    {   // reuse on the same stream: immediate, no driver call, no ordering needed
        FakeBackend be; CachingAllocator a(&be);
        void *p, *q;
        a.malloc(&p, 64u << 20, S1); a.free(p, S1);
        a.malloc(&q, 64u << 20, S1);
        CHECK(q == p && a.stats().n_driver_allocs == 1 && a.stats().n_cache_hits == 1, "same-stream reuse");
        CHECK(be.orderings.empty() && be.syncs == 0, "no synchronisation on a hit");
        a.free(q, S1);
        printf("ok same_stream_reuse\n");
    }
    {   // reuse across streams goes through an event: owner stream -> waiter stream
        FakeBackend be; CachingAllocator a(&be);
        void *p, *q;
        a.malloc(&p, 64u << 20, S1); a.free(p, S1);
        a.malloc(&q, 64u << 20, S2);
        CHECK(q == p && a.stats().n_driver_allocs == 1, "cross-stream reuse");
        CHECK(be.orderings.size() == 1 && be.orderings[0].first == S1 && be.orderings[0].second == S2, "event ordering");
        a.free(q, S2);
        void *r; a.malloc(&r, 64u << 20, S2);
        CHECK(r == p && be.orderings.size() == 1, "block now belongs to the second stream");
        a.free(r, S2);
        printf("ok cross_stream_reuse\n");
    }
    {   // a stream that is destroyed hands its cached blocks to the null stream: nothing is ever
        // ordered after the dead stream again
        FakeBackend be; CachingAllocator a(&be);
        void *p, *s, *q, *t;
        a.malloc(&p, 64u << 20, S1); a.malloc(&s, 4096, S1);
        a.free(p, S1); a.free(s, S1);
        const uint64_t cached = a.stats().bytes_cached;
        a.retire_stream(S1);
        CHECK(a.stats().bytes_cached == cached, "retiring keeps the cache");
        a.malloc(&q, 64u << 20, S2); a.malloc(&t, 4096, S2);
        CHECK(q == p && t == s && a.stats().n_driver_allocs == 2, "blocks of the retired stream are reused");
        for (auto &o : be.orderings) CHECK(o.first != S1, "no ordering after the retired stream");
        CHECK(be.orderings.size() == 2 && be.orderings[0].first == nullptr, "ordered after the null stream instead");
        a.free(q, S2); a.free(t, S2);
        // a block still live when its stream died is freed in the dead stream's name: null stream too
        void *u, *w;
        a.malloc(&u, 32u << 20, S1);          // S1 is retired: a caller's stale handle
        a.free(u, S1);
        const size_t before = be.orderings.size();
        a.malloc(&w, 32u << 20, S2);
        CHECK(w == u && be.orderings.size() == before + 1 && be.orderings.back().first == nullptr, "stale handle mapped to the null stream");
        a.free(w, S2);
        a.adopt_stream(S1);                   // the handle value comes back as a new stream
        a.malloc(&u, 48u << 20, S1); a.free(u, S1); a.malloc(&w, 48u << 20, S2);
        CHECK(w == u && be.orderings.back().first == S1, "an adopted stream is a stream again");
        a.free(w, S2);
        printf("ok retire_stream\n");
    }
    {   // holes in the middle of a segment are reusable; neighbours merge on free
        FakeBackend be; CachingAllocator a(&be);
        void *p[4];
        for (int i = 0; i < 4; i++) a.malloc(&p[i], 256 << 10, S1);
        a.free(p[1], S1);
        void *h; a.malloc(&h, 200 << 10, S1);
        CHECK(h == p[1], "hole reused (the reference's bump allocator cannot)");
        a.free(h, S1); a.free(p[2], S1);
        void *m; a.malloc(&m, 512 << 10, S1);
        CHECK(m == p[1], "freed neighbours merged");
        a.free(m, S1); a.free(p[0], S1); a.free(p[3], S1);
        CHECK(a.trim() == 0 && be.live.empty() && a.stats().bytes_reserved == 0, "trim returns whole segments");
        printf("ok split_merge_trim\n");
    }
    {   // out of memory: synchronise, drop the cache, retry once; then a clean error
        FakeBackend be; be.capacity = 300u << 20; CachingAllocator a(&be);
        void *p, *q, *r;
        CHECK(a.malloc(&p, 200u << 20, S1) == 0, "first");
        a.free(p, S1);
        CHECK(a.malloc(&q, 250u << 20, S1) == 0, "retry after trimming the cache");
        CHECK(a.stats().n_oom_retries == 1 && be.syncs == 1 && a.stats().n_driver_frees == 1, "oom path taken");
        CHECK(a.malloc(&r, 200u << 20, S1) == CachingAllocator::kErrOom && r == nullptr, "clean OOM error");
        a.free(q, S1);
        printf("ok oom_retry\n");
    }
    {   // a failing driver call (injected) also takes the retry path
        FakeBackend be; CachingAllocator a(&be);
        be.fail_next = 1;
        void *p;
        CHECK(a.malloc(&p, 4u << 20, S1) == 0 && a.stats().n_oom_retries == 1, "transient failure retried");
        be.fail_next = 2;
        void *q;
        CHECK(a.malloc(&q, 40u << 20, S1) == CachingAllocator::kErrOom, "persistent failure reported");
        a.free(p, S1);
        printf("ok injected_failure\n");
    }
    {   // foreign pointer / double free -> not owned (the caller falls back to a raw free)
        FakeBackend be; CachingAllocator a(&be);
        void *p; a.malloc(&p, 4096, S1);
        CHECK(a.free(reinterpret_cast<void *>(0xdeadbeef), S1) == CachingAllocator::kErrNotOwned, "foreign pointer");
        CHECK(a.free(p, S1) == 0 && a.free(p, S1) == CachingAllocator::kErrNotOwned, "double free");
        CHECK(a.free(nullptr, S1) == 0, "null is a no-op");
        printf("ok not_owned\n");
    }
    {   // blocks a capturing stream took from the pool stay with that stream's graphs
        FakeBackend be; CachingAllocator a(&be);
        void *w, *t1, *t2, *e, *out;
        a.malloc(&w, 64u << 20, S1); a.free(w, S1);                  // rehearsal: the pool holds the block
        CHECK(a.malloc(&t1, 64u << 20, S1, true) == 0 && t1 == w, "capture takes the cached block");
        CHECK(a.free(t1, S1) == 0, "free during capture");
        CHECK(a.bytes_captured() == (64u << 20), "held back for the graph");
        CHECK(a.malloc(&t2, 64u << 20, S1, true) == 0 && t2 == w, "reused inside the capture (recorded order)");
        a.free(t2, S1);
        CHECK(a.malloc(&out, 4096, S1, true) == 0, "an output allocated during the capture");
        // capture over: an ordinary request must not get the block the recorded kernels write
        CHECK(a.malloc(&e, 64u << 20, S1) == 0 && e != w, "eager request gets other memory");
        CHECK(a.stats().n_driver_allocs == 3, "a new segment for the eager tensor");
        void *e2; CHECK(a.malloc(&e2, 64u << 20, S2) == 0 && e2 != w, "other streams neither");
        a.free(e2, S2);
        a.free(out, S2);                                             // freed eagerly, on another stream: still the graph's
        void *o2; CHECK(a.malloc(&o2, 4096, S1) == 0 && o2 != out, "captured output not handed out eagerly");
        a.free(o2, S1);
        a.trim();
        CHECK(a.bytes_captured() >= (64u << 20), "trim leaves the graph's blocks alone");
        AllocStats st = a.stats();
        CHECK(st.bytes_reserved == st.bytes_in_use + st.bytes_cached, "accounting with captured blocks");
        a.release_captured(S1);                                      // graphs destroyed
        CHECK(a.bytes_captured() == 0, "released");
        void *r; CHECK(a.malloc(&r, 64u << 20, S1) == 0 && r == w, "ordinary again after release");
        a.free(r, S1); a.free(e, S1);
        a.trim();
        CHECK(be.live.empty(), "everything returns to the driver");
        // a live captured block at release time becomes ordinary when it is freed later
        void *l; a.malloc(&l, 8192, S1, true);
        a.release_captured(S1);
        a.free(l, S1);
        CHECK(a.bytes_captured() == 0, "live block released with its stream");
        // retiring the stream releases too
        void *m; a.malloc(&m, 8192, S2, true); a.free(m, S2);
        CHECK(a.bytes_captured() > 0, "held");
        a.retire_stream(S2);
        CHECK(a.bytes_captured() == 0, "retire releases");
        printf("ok capture_blocks\n");
    }
    {   // randomized stress against a shadow model: no overlap, accounting consistent
        FakeBackend be; CachingAllocator a(&be);
        struct L { char *p; size_t n; void *s; };
        std::vector<L> live;
        unsigned x = 1;
        auto rnd = [&]() { x = x * 1664525u + 1013904223u; return x >> 8; };
        for (int it = 0; it < 20000; it++) {
            if (live.empty() || rnd() % 3) {
                size_t n = (rnd() % 4 == 0) ? (size_t)(rnd() % (32u << 20)) + 1 : (size_t)(rnd() % 70000) + 1;
                void *s = (rnd() & 1) ? S1 : S2, *p;
                CHECK(a.malloc(&p, n, s, rnd() % 5 == 0) == 0, "stress alloc");
                for (auto &l : live) CHECK((char *)p + n <= l.p || l.p + l.n <= (char *)p, "no overlap");
                live.push_back({(char *)p, n, s});
            } else {
                size_t i = rnd() % live.size();
                CHECK(a.free(live[i].p, live[i].s) == 0, "stress free");
                live[i] = live.back(); live.pop_back();
            }
            if (it % 997 == 0) a.release_captured((rnd() & 1) ? S1 : S2);
            if (it % 4001 == 0) a.trim();
            AllocStats st = a.stats();
            CHECK(st.bytes_reserved == st.bytes_in_use + st.bytes_cached, "reserved = in use + cached");
        }
        for (auto &l : live) a.free(l.p, l.s);
        CHECK(a.stats().bytes_in_use == 0, "all returned");
        a.release_captured(S1); a.release_captured(S2);
        a.trim();
        CHECK(be.live.empty(), "trim frees everything when nothing is live");
        printf("ok stress\n");
    }
    return 0;
}
