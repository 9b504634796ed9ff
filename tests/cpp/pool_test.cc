// Host-only test of hipcx::MemoryPool with a fake allocator (no GPU, no HIP): the behaviours the backend's Device layer relies
// on.  Built and run by tests/test_memory_pool.py, once plainly and once under ThreadSanitizer.
//   retry path            the reference's MemoryPool::Malloc frees unused blocks and tries again before OutOfMemoryError
//                         (CX/cuda/memory_pool.cc:236-243; its own test: CX/cuda/memory_pool_test.cc MallocFreeUnusedBlocks..)
//   deleter after pool    Device::Allocate results may outlive the pool (CX/cuda/cuda_device/memory.cc:19-24)
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <set>
#include <thread>
#include <vector>

#include "memory_pool.h"

using namespace hipcx;

static int g_failures = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);    \
            ++g_failures;                                                    \
        }                                                                    \
    } while (0)

// Hands out fake addresses; fails while more than `capacity` bytes would be outstanding.
struct FakeState {
    std::mutex mu;
    size_t capacity = ~size_t{0};
    size_t outstanding = 0;
    size_t mallocs = 0, frees = 0, refusals = 0;
    uintptr_t next = 0x10000;
    std::map<void*, size_t> live;
};
class FakeAllocator : public Allocator {
public:
    explicit FakeAllocator(std::shared_ptr<FakeState> s) : s_(std::move(s)) {}
    bool Malloc(void** ptr, size_t bytes) override {
        std::lock_guard<std::mutex> lock(s_->mu);
        if (s_->outstanding + bytes > s_->capacity) {
            ++s_->refusals;
            return false;
        }
        *ptr = reinterpret_cast<void*>(s_->next);
        s_->next += bytes + 4096;
        s_->live[*ptr] = bytes;
        s_->outstanding += bytes;
        ++s_->mallocs;
        return true;
    }
    void Free(void* ptr) noexcept override {
        std::lock_guard<std::mutex> lock(s_->mu);
        auto it = s_->live.find(ptr);
        if (it == s_->live.end()) {
            std::printf("FAILED: allocator asked to free an unknown pointer\n");
            ++g_failures;
            return;
        }
        s_->outstanding -= it->second;
        s_->live.erase(it);
        ++s_->frees;
    }

    // a fake stream is a pointer to a bool that says whether the stream has caught up
    std::function<bool()> Fence(void* stream) override {
        const bool* idle = static_cast<const bool*>(stream);
        ++fences_;
        return [idle] { return *idle; };
    }
    int fences_ = 0;

private:
    std::shared_ptr<FakeState> s_;
};

static void TestRounding() {
    CHECK(MemoryPool::RoundSize(1) == 512);
    CHECK(MemoryPool::RoundSize(512) == 512);
    CHECK(MemoryPool::RoundSize(513) == 1024);
    CHECK(MemoryPool::RoundSize(4096) == 4096);
    for (size_t n : {size_t{4097}, size_t{70000}, size_t{1} << 20, (size_t{1} << 20) + 1, size_t{15} << 20, size_t{16} << 20, (size_t{100} << 20) + 5}) {
        size_t r = MemoryPool::RoundSize(n);
        CHECK(r >= n && r % kAllocationUnit == 0);
        CHECK(r - n <= n / 8 + (2u << 20));  // bounded slack
        CHECK(MemoryPool::RoundSize(r) == r);  // classes are fixed points
    }
}

static void TestReuseAndZero() {
    auto fs = std::make_shared<FakeState>();
    MemoryPool pool(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    CHECK(pool.Malloc(0) == nullptr);
    void* a = pool.Malloc(1000);
    pool.Free(a);
    void* b = pool.Malloc(900);  // same class (1024): the cached block comes back
    CHECK(a == b);
    CHECK(fs->mallocs == 1);
    PoolStats st = pool.stats();
    CHECK(st.in_use_bytes == 1024 && st.cached_bytes == 0 && st.in_use_blocks == 1);
    pool.Free(b);
    st = pool.stats();
    CHECK(st.in_use_bytes == 0 && st.cached_bytes == 1024 && st.cached_blocks == 1);
    bool threw = false;
    try {
        pool.Free(reinterpret_cast<void*>(0x1234));
    } catch (const std::runtime_error&) {
        threw = true;
    }
    CHECK(threw);                                   // out-of-pool pointer
    pool.FreeNoExcept(reinterpret_cast<void*>(0x1234));  // must not throw
    pool.Free(nullptr);
    pool.FreeUnusedBlocks();
    CHECK(fs->frees == 1 && fs->outstanding == 0);
    CHECK(pool.stats().cached_bytes == 0);
}

static void TestRetryThenOutOfMemory() {
    auto fs = std::make_shared<FakeState>();
    fs->capacity = 10 * 1024;
    MemoryPool pool(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    void* a = pool.Malloc(4096);
    void* b = pool.Malloc(4096);
    pool.Free(a);
    pool.Free(b);  // 8 KiB cached, 2 KiB of capacity left
    // another class: the allocator refuses, the pool releases its cache and the second try succeeds
    void* c = pool.Malloc(6000);
    CHECK(c != nullptr);
    CHECK(fs->refusals == 1 && fs->frees == 2);
    CHECK(pool.stats().retries == 1 && pool.stats().cached_bytes == 0);
    // now nothing is cached: the next refusal is final
    bool oom = false;
    try {
        pool.Malloc(8000);
    } catch (const OutOfMemoryError& e) {
        oom = std::string(e.what()).find("8000") != std::string::npos;
    }
    CHECK(oom);
    CHECK(pool.stats().in_use_blocks == 1);  // the failed call left no trace
    pool.Free(c);
}

static void TestDeleterOutlivesPool() {
    auto fs = std::make_shared<FakeState>();
    std::shared_ptr<void> survivor;
    {
        auto pool = std::make_shared<MemoryPool>(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
        survivor = MemoryPool::MakeShared(pool, 2048);
        std::shared_ptr<void> returned = MemoryPool::MakeShared(pool, 2048);
        void* p = returned.get();
        returned.reset();  // back to the pool
        CHECK(pool->stats().cached_blocks == 1);
        CHECK(pool->Malloc(2048) == p);
    }
    // the pool is gone and gave everything back, the block `survivor` points at included
    CHECK(fs->outstanding == 0 && fs->live.empty());
    survivor.reset();  // must neither crash nor touch the allocator again
    CHECK(fs->frees == fs->mallocs);
}

static void TestArenas() {
    auto fs = std::make_shared<FakeState>();
    fs->capacity = 64 * 1024;
    MemoryPool pool(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    pool.SetArena(7);
    void* g1 = pool.Malloc(4096);
    void* g2 = pool.Malloc(4096);
    pool.Free(g1);
    pool.SetArena(0);
    void* n1 = pool.Malloc(4096);
    CHECK(n1 != g1);  // the general arena does not get the graph arena's cached block
    pool.SetArena(7);
    CHECK(pool.Malloc(4096) == g1);  // the arena itself does
    pool.SetArena(0);
    pool.Free(g1);
    pool.Free(g2);  // freed outside the scope: still returns to arena 7
    void* n2 = pool.Malloc(4096);
    CHECK(n2 != g1 && n2 != g2);
    // running out of memory releases the general cache only
    pool.Free(n1);
    pool.Free(n2);
    void* big = pool.Malloc(52 * 1024);  // 16 KiB outstanding of 64: refused once, general cache (8 KiB) released
    CHECK(big != nullptr && pool.stats().retries == 1);
    CHECK(pool.stats().cached_blocks == 2);  // arena 7's two blocks survived
    pool.Free(big);
    pool.ReleaseArena(7);
    void* r = pool.Malloc(4096);
    CHECK(r == g1 || r == g2);  // now anybody may have them
    pool.Free(r);
}

static void TestPartitions() {
    auto fs = std::make_shared<FakeState>();
    fs->capacity = 64 * 1024;
    MemoryPool pool(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    void* a = pool.Malloc(4096, 1u);  // "stream 1"
    pool.Free(a);
    void* b = pool.Malloc(4096, 2u);  // "stream 2" must not get stream 1's block
    CHECK(b != a);
    void* c = pool.Malloc(4096, 1u);  // stream 1 does
    CHECK(c == a);
    pool.Free(b);
    pool.Free(c);
    // arenas and partitions combine: a graph arena's block stays in its partition when the arena is released
    pool.SetArena(3);
    void* g = pool.Malloc(8192, 2u);
    pool.Free(g);
    pool.SetArena(0);
    CHECK(pool.Malloc(8192, 2u) != g);
    pool.ReleaseArena(3);
    void* h1 = pool.Malloc(8192, 1u);
    CHECK(h1 != g);
    void* h2 = pool.Malloc(8192, 2u);
    CHECK(h2 == g);
    // out of memory releases every partition of the general arena
    size_t cached_before = pool.stats().cached_blocks;
    CHECK(cached_before >= 2);
    void* big = pool.Malloc(40 * 1024, 5u);
    CHECK(big != nullptr);
    CHECK(pool.stats().cached_blocks == 0);
}

static void TestThreads() {
    auto fs = std::make_shared<FakeState>();
    fs->capacity = size_t{1} << 26;
    auto pool = std::make_shared<MemoryPool>(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    std::vector<std::thread> threads;
    for (int t = 0; t < 4; ++t) {
        threads.emplace_back([pool, t] {
            std::vector<std::shared_ptr<void>> mine;
            unsigned x = 12345u + t;
            for (int i = 0; i < 4000; ++i) {
                x = x * 1664525u + 1013904223u;
                size_t bytes = 1 + (x >> 8) % 200000;
                mine.push_back(MemoryPool::MakeShared(pool, bytes));
                if (mine.size() > 16) mine.erase(mine.begin() + (x % mine.size()));
                if (i % 500 == 499) pool->FreeUnusedBlocks();
            }
        });
    }
    for (auto& th : threads) th.join();
    CHECK(pool->stats().in_use_blocks == 0);
    pool.reset();
    CHECK(fs->outstanding == 0);
}

// A block used on a stream other than its own: after RecordStream its Free holds it back until that stream has caught up; without
// the announcement it is handed out again at once (the documented rule: the owner waits before freeing).
static void TestRecordStream() {
    auto fs = std::make_shared<FakeState>();
    MemoryPool pool(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    bool stream_b_idle = false, stream_c_idle = false;
    void* a = pool.Malloc(1000, 1);
    pool.RecordStream(a, &stream_b_idle);
    pool.RecordStream(a, &stream_b_idle);  // recorded once
    pool.RecordStream(a, &stream_c_idle);
    pool.Free(a);
    CHECK(pool.pending_blocks() == 1);
    CHECK(pool.stats().in_use_blocks == 1 && pool.stats().cached_blocks == 0);  // held back: still counted as in use
    void* b = pool.Malloc(1000, 1);
    CHECK(b != a);  // a new block: the kernel on the other stream may still read a
    bool threw = false;
    try {
        pool.Free(a);  // freed twice
    } catch (const std::runtime_error&) {
        threw = true;
    }
    CHECK(threw);
    threw = false;
    try {
        pool.RecordStream(a, &stream_b_idle);  // no longer the caller's
    } catch (const std::runtime_error&) {
        threw = true;
    }
    CHECK(threw);
    stream_b_idle = true;
    void* c = pool.Malloc(1000, 1);
    CHECK(c != a);  // one of the two streams is still busy
    stream_c_idle = true;
    void* d = pool.Malloc(1000, 1);
    CHECK(d == a && pool.pending_blocks() == 0);
    CHECK(pool.InUsePointers().size() == 3);
    pool.Free(b), pool.Free(c), pool.Free(d);
    // the same sequence without the announcement: immediate reuse
    void* e = pool.Malloc(5000, 1);
    pool.Free(e);
    CHECK(pool.Malloc(5000, 1) == e);
    // a held-back block is not among the pointers whose frees are still to come, and goes back to the allocator with the pool
    bool never = false;
    void* f = pool.Malloc(70000, 2);
    pool.RecordStream(f, &never);
    pool.Free(f);
    for (void* p : pool.InUsePointers()) CHECK(p != f);
    pool.FreeUnusedBlocks();
    CHECK(pool.pending_blocks() == 1);
}

// hipcx_pool_destroy, then a new pool on the device, then the stale frees of the first pool's blocks: swallowed, whatever address
// the new pool hands out.
static void TestOrphans() {
    auto fs = std::make_shared<FakeState>();
    OrphanSet orphans;
    void* stale = nullptr;
    {
        MemoryPool first(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
        stale = first.Malloc(3000);
        void* freed = first.Malloc(3000);
        first.Free(freed);
        std::vector<void*> in_use = first.InUsePointers();
        CHECK(in_use.size() == 1 && in_use[0] == stale);
        orphans.Add(in_use);
    }  // the pool takes its memory with it
    CHECK(fs->outstanding == 0);
    fs->next = reinterpret_cast<uintptr_t>(stale);  // the driver hands the same address out again
    MemoryPool second(std::unique_ptr<Allocator>(new FakeAllocator(fs)));
    void* fresh = second.Malloc(3000);
    CHECK(fresh == stale);
    auto free_like_the_entry_point = [&](void* p) {
        if (orphans.Take(p)) return;
        second.Free(p);
    };
    free_like_the_entry_point(stale);  // the first pool's owner lets go: must not free the second pool's live block
    CHECK(second.stats().in_use_blocks == 1 && orphans.size() == 0);
    free_like_the_entry_point(fresh);  // the real free
    CHECK(second.stats().in_use_blocks == 0 && second.stats().cached_blocks == 1);
    CHECK(!orphans.Take(fresh));
}

int main() {
    TestRecordStream();
    TestOrphans();
    TestRounding();
    TestReuseAndZero();
    TestRetryThenOutOfMemory();
    TestDeleterOutlivesPool();
    TestArenas();
    TestPartitions();
    TestThreads();
    if (g_failures != 0) {
        std::printf("%d check(s) failed\n", g_failures);
        return 1;
    }
    std::printf("memory pool: all checks passed\n");
    return 0;
}
