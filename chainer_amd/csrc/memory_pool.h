// Device / pinned-host memory pool of the hip backend (host code only: no HIP headers, so that the class can be
// built and exercised with a fake allocator on a machine without a GPU).
//
// Role in the reference: chainerx::cuda::MemoryPool (CX/cuda/memory_pool.{h,cc}) behind CudaDevice::Allocate
// (CX/cuda/cuda_device/memory.cc:17-26).  Kept from it: the 512-byte allocation unit (memory_pool.h:29), Malloc(0) ==
// nullptr (memory_pool.cc:209-211), "release every cached block and try once more" before an allocation is reported as
// out of memory (memory_pool.cc:236-243), Free of a pointer the pool does not know is an error (memory_pool.cc:262-264),
// a noexcept free for deleters (memory_pool.cc:296-302) and deleters that outlive the pool (weak_ptr,
// cuda_device/memory.cc:19-24).
//
// Different by design (sized for one process owning a 288 GB device, launches on HIP streams and graphs):
//  * no splitting and merging of chunks: requests are rounded to size classes (512-byte units up to 4 KiB, then steps of
//    1/8 of the size, then whole 2 MiB pages from 16 MiB on) and a freed block serves later requests of its class only --
//    O(log classes) per call, no neighbour bookkeeping, at most 12.5 % of slack per block;
//  * arenas: a block remembers the arena it was allocated in and returns to that arena's free lists.  A HIP graph is
//    captured inside an arena of its own, so the addresses baked into the graph are never handed to anybody else
//    until the arena is released (the graph destroyed);
//  * partitions: inside an arena, a freed block is only reused by allocations of the same partition.  The device layer
//    uses one partition per HIP stream: work queued on a stream runs in order, so a block freed and reallocated on one
//    stream needs no synchronisation, while another stream never gets it (the reference launches everything on one
//    stream and has no such problem).  That covers a block used on the stream it was allocated for.  A block that is also
//    used on another stream is announced with RecordStream; its Free then holds it back until that stream has caught up.
//    Without the announcement the owner must not free the block before the foreign stream's work on it was waited for;
//  * when the device allocator reports failure only the general arena's cache is released: the blocks of a graph's
//    arena stay where the graph expects them.
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <utility>
#include <vector>

namespace hipcx {

constexpr size_t kAllocationUnit = 512;  // CX/cuda/memory_pool.h:29 kAllocationUnitSize

// What the pool allocates from (CX/cuda/memory_pool.h:48-78: Allocator, DeviceMemoryAllocator, PinnedMemoryAllocator).
class Allocator {
public:
    virtual ~Allocator() = default;
    virtual bool Malloc(void** ptr, size_t bytes) = 0;  // false: out of memory (any other failure throws)
    virtual void Free(void* ptr) noexcept = 0;
    // A predicate that turns true once the work queued on `stream` up to now has run (device memory: an event recorded on the
    // stream).  An empty function: nothing to wait for.  Used for blocks that were announced with MemoryPool::RecordStream.
    virtual std::function<bool()> Fence(void* stream) {
        (void)stream;
        return {};
    }
};

class OutOfMemoryError : public std::runtime_error {  // CX/cuda/memory_pool.h:34-37
public:
    explicit OutOfMemoryError(size_t bytes) : std::runtime_error("Out of memory allocating " + std::to_string(bytes) + " bytes.") {}
};

struct PoolStats {
    size_t in_use_bytes = 0;     // handed out and not yet freed (rounded sizes)
    size_t cached_bytes = 0;     // free blocks held for reuse, all arenas
    size_t in_use_blocks = 0;
    size_t cached_blocks = 0;
    size_t allocator_calls = 0;  // successful Allocator::Malloc calls so far
    size_t retries = 0;          // allocations that only succeeded after the cache was released
};

class MemoryPool {
public:
    explicit MemoryPool(std::unique_ptr<Allocator> allocator) : allocator_(std::move(allocator)) {}
    // Gives everything back to the allocator, blocks still in use included (CX/cuda/memory_pool.cc:160-170): once the pool
    // is gone the memory is gone; deleters made by MakeShared notice and do nothing.
    ~MemoryPool() {
        for (auto& kv : in_use_) allocator_->Free(kv.first);
        for (auto& arena : free_) {
            for (auto& bin : arena.second) {
                for (void* p : bin.second) allocator_->Free(p);
            }
        }
    }
    MemoryPool(const MemoryPool&) = delete;
    MemoryPool& operator=(const MemoryPool&) = delete;

    static size_t RoundSize(size_t bytes) {
        size_t units = (bytes + kAllocationUnit - 1) / kAllocationUnit;
        if (bytes >= (16u << 20)) {  // whole 2 MiB pages
            constexpr size_t kPage = 2u << 20;
            return (bytes + kPage - 1) / kPage * kPage;
        }
        if (units <= 8) return units * kAllocationUnit;
        // steps of 1/8 of the power of two below: 8, 9, ..., 16, 18, ..., 32, 36, ...
        size_t p = 8;
        while (p * 2 <= units) p *= 2;
        size_t step = p / 8;
        return (units + step - 1) / step * step * kAllocationUnit;
    }

    // nullptr for 0 bytes; throws OutOfMemoryError when the allocator fails twice.  `arena`: see SetArena().
    void* Malloc(size_t bytes, uint32_t partition = 0) { return Malloc(bytes, current_arena_.load(), partition); }
    void* Malloc(size_t bytes, int arena_number, uint32_t partition) {
        if (bytes == 0) return nullptr;
        const size_t size = RoundSize(bytes);
        const uint64_t arena = Key(arena_number, partition);
        std::lock_guard<std::mutex> lock(mutex_);
        CollectPendingLocked();
        void* ptr = nullptr;
        auto a = free_.find(arena);
        if (a != free_.end()) {
            auto bin = a->second.find(size);
            if (bin != a->second.end() && !bin->second.empty()) {
                ptr = bin->second.back();
                bin->second.pop_back();
                stats_.cached_bytes -= size;
                --stats_.cached_blocks;
            }
        }
        if (ptr == nullptr) {
            if (!allocator_->Malloc(&ptr, size)) {
                ReleaseCachedLocked();
                ++stats_.retries;
                if (!allocator_->Malloc(&ptr, size)) {
                    --stats_.retries;
                    throw OutOfMemoryError(bytes);
                }
            }
            ++stats_.allocator_calls;
        }
        in_use_.emplace(ptr, Block{size, arena, {}});
        stats_.in_use_bytes += size;
        ++stats_.in_use_blocks;
        return ptr;
    }

    // Returns the block to the free lists of the arena it came from.  Throws for a pointer that is not in use.
    // A block with recorded streams (RecordStream) is held back -- still counted as in use -- until the work those streams had
    // queued at this moment has run; Malloc and FreeUnusedBlocks move such blocks on.
    void Free(void* ptr) {
        if (ptr == nullptr) return;
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = in_use_.find(ptr);
        if (it == in_use_.end()) throw std::runtime_error("Cannot free out-of-pool memory");
        if (pending_.count(ptr) != 0) throw std::runtime_error("Cannot free out-of-pool memory");  // freed twice
        if (!it->second.streams.empty()) {
            std::vector<std::function<bool()>> fences;
            for (void* stream : it->second.streams) {
                std::function<bool()> f = allocator_->Fence(stream);
                if (f) fences.push_back(std::move(f));
            }
            it->second.streams.clear();
            if (!fences.empty()) {
                pending_.emplace(ptr, std::move(fences));
                return;
            }
        }
        ReleaseLocked(it);
    }
    // `ptr` (in use) has work queued on `stream`, which is not the stream it was allocated for: its Free must not hand the block
    // to a new owner before that work has run.  The caller filters out the block's own stream (BlockPartition).
    void RecordStream(void* ptr, void* stream) {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = in_use_.find(ptr);
        if (it == in_use_.end() || pending_.count(ptr) != 0) throw std::runtime_error("record_stream: not a block in use");
        for (void* s : it->second.streams) {
            if (s == stream) return;
        }
        it->second.streams.push_back(stream);
    }
    // The partition (stream) the block was allocated for; false if `ptr` is not in use.
    bool BlockPartition(void* ptr, uint32_t* partition) const {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = in_use_.find(ptr);
        if (it == in_use_.end()) return false;
        *partition = PartitionOf(it->second.arena);
        return true;
    }
    // Pointers handed out and not yet freed (blocks held back by Free included).
    std::vector<void*> InUsePointers() const {
        std::lock_guard<std::mutex> lock(mutex_);
        std::vector<void*> v;
        v.reserve(in_use_.size());
        for (auto& kv : in_use_) {
            if (pending_.count(kv.first) == 0) v.push_back(kv.first);
        }
        return v;
    }
    size_t pending_blocks() const {
        std::lock_guard<std::mutex> lock(mutex_);
        return pending_.size();
    }
    void FreeNoExcept(void* ptr) noexcept {
        try {
            Free(ptr);
        } catch (...) {
        }
    }

    // Gives the cached blocks of the general arena back to the allocator (MemoryPool::FreeUnusedBlocks, memory_pool.cc:172-203).
    void FreeUnusedBlocks() {
        std::lock_guard<std::mutex> lock(mutex_);
        CollectPendingLocked();
        ReleaseCachedLocked();
    }

    // Allocations made through Malloc(bytes) from now on belong to `arena` (0 is the general arena).  One setting for the
    // pool, not per thread: a HIP graph is captured by one thread while the others are idle.
    void SetArena(int arena) { current_arena_.store(arena); }
    int arena() const { return current_arena_.load(); }
    // The cached blocks of `arena` join the general arena (each in its partition); blocks of it still in use will follow
    // when they are freed.
    void ReleaseArena(int arena) {
        if (arena == 0) return;
        std::lock_guard<std::mutex> lock(mutex_);
        for (auto a = free_.begin(); a != free_.end();) {
            if (ArenaOf(a->first) != arena) {
                ++a;
                continue;
            }
            auto& general = free_[Key(0, PartitionOf(a->first))];
            for (auto& bin : a->second) {
                auto& dst = general[bin.first];
                dst.insert(dst.end(), bin.second.begin(), bin.second.end());
            }
            a = free_.erase(a);
        }
        for (auto& kv : in_use_) {
            if (ArenaOf(kv.second.arena) == arena) kv.second.arena = Key(0, PartitionOf(kv.second.arena));
        }
        int expected = arena;
        current_arena_.compare_exchange_strong(expected, 0);
    }

    PoolStats stats() const {
        std::lock_guard<std::mutex> lock(mutex_);
        return stats_;
    }

    // shared_ptr whose deleter returns the block if the pool is still alive and does nothing otherwise
    // (the ownership rule of Device::Allocate results, CX/cuda/cuda_device/memory.cc:17-26).
    static std::shared_ptr<void> MakeShared(const std::shared_ptr<MemoryPool>& pool, size_t bytes, uint32_t partition = 0) {
        std::weak_ptr<MemoryPool> weak = pool;
        return std::shared_ptr<void>(pool->Malloc(bytes, partition), [weak](void* p) noexcept {
            if (std::shared_ptr<MemoryPool> alive = weak.lock()) alive->FreeNoExcept(p);
        });
    }

private:
    struct Block {
        size_t size;
        uint64_t arena;  // Key(arena, partition)
        std::vector<void*> streams;  // RecordStream
    };
    void ReleaseLocked(std::unordered_map<void*, Block>::iterator it) {
        void* ptr = it->first;
        const size_t size = it->second.size;
        const uint64_t arena = it->second.arena;
        in_use_.erase(it);
        stats_.in_use_bytes -= size;
        --stats_.in_use_blocks;
        free_[arena][size].push_back(ptr);
        stats_.cached_bytes += size;
        ++stats_.cached_blocks;
    }
    void CollectPendingLocked() {
        for (auto p = pending_.begin(); p != pending_.end();) {
            bool done = true;
            for (auto& fence : p->second) done = done && fence();
            if (!done) {
                ++p;
                continue;
            }
            ReleaseLocked(in_use_.find(p->first));
            p = pending_.erase(p);
        }
    }
    static uint64_t Key(int arena, uint32_t partition) { return (static_cast<uint64_t>(static_cast<uint32_t>(arena)) << 32) | partition; }
    static int ArenaOf(uint64_t key) { return static_cast<int>(key >> 32); }
    static uint32_t PartitionOf(uint64_t key) { return static_cast<uint32_t>(key & 0xffffffffu); }
    void ReleaseCachedLocked() {  // every partition of the general arena
        for (auto a = free_.begin(); a != free_.end();) {
            if (ArenaOf(a->first) != 0) {
                ++a;
                continue;
            }
            for (auto& bin : a->second) {
                for (void* p : bin.second) {
                    allocator_->Free(p);
                    stats_.cached_bytes -= bin.first;
                    --stats_.cached_blocks;
                }
            }
            a = free_.erase(a);
        }
    }

    std::unique_ptr<Allocator> allocator_;
    mutable std::mutex mutex_;
    std::unordered_map<void*, Block> in_use_;
    std::unordered_map<void*, std::vector<std::function<bool()>>> pending_;  // freed, waiting for foreign streams (still in in_use_)
    std::map<uint64_t, std::map<size_t, std::vector<void*>>> free_;  // (arena, partition) -> rounded size -> blocks
    std::atomic<int> current_arena_{0};
    PoolStats stats_;
};

// Pointers that were still in use when a device's pool was destroyed (the pool takes their memory with it).  Their owners'
// deleters run later, perhaps after a new pool exists on the device -- which may even have been given the same address again.
// Such a free must not reach the new pool: the first Free of an orphaned address is swallowed here.  (If the new pool did hand
// the address out again and its new owner frees first, that free is the one swallowed and the block stays allocated until the
// stale free arrives: late, never wrong.)  The reference ties each deleter to its pool object with a weak_ptr instead
// (CX/cuda/cuda_device/memory.cc:19-24); a C ABI that frees by (device, pointer) needs the bookkeeping on this side.
class OrphanSet {
public:
    void Add(const std::vector<void*>& ptrs) {
        std::lock_guard<std::mutex> lock(mutex_);
        for (void* p : ptrs) orphans_.insert(p);
    }
    bool Take(void* ptr) {  // true: ptr was an orphan and is now forgotten
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = orphans_.find(ptr);
        if (it == orphans_.end()) return false;
        orphans_.erase(it);
        return true;
    }
    size_t size() const {
        std::lock_guard<std::mutex> lock(mutex_);
        return orphans_.size();
    }

private:
    mutable std::mutex mutex_;
    std::unordered_multiset<void*> orphans_;
};

}  // namespace hipcx
