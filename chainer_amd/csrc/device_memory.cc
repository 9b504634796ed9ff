// Device side of the backend behind the C ABI: pooled allocation, host <-> device and device <-> device copies
// (chainerx::Device::Allocate / MemoryCopyFrom / MemoryCopyTo / TransferData* / FromHostMemory / MakeDataFromForeignPointer,
// CX/device.h:24-71; the CUDA backend's versions are CX/cuda/cuda_device/memory.cc:17-157).
#include <array>
#include <cstring>
#include <deque>
#include <map>

#include "common.h"
#include "memory_pool.h"

namespace hipcx {
namespace {

constexpr int kMaxDevices = 64;

class SetDeviceScope {  // CX/cuda/cuda_set_device_scope.h
public:
    explicit SetDeviceScope(int device) {
        HIPCX_CHECK_HIP(hipGetDevice(&prev_));
        if (prev_ != device) {
            HIPCX_CHECK_HIP(hipSetDevice(device));
            changed_ = true;
        }
    }
    ~SetDeviceScope() {
        if (changed_) (void)hipSetDevice(prev_);
    }

private:
    int prev_ = 0;
    bool changed_ = false;
};

class DeviceAllocator : public Allocator {  // CX/cuda/memory_pool.cc DeviceMemoryAllocator::Malloc
public:
    explicit DeviceAllocator(int device) : device_(device) {}
    bool Malloc(void** ptr, size_t bytes) override {
        SetDeviceScope scope(device_);
        hipError_t e = hipMalloc(ptr, bytes);
        if (e == hipErrorOutOfMemory) {
            (void)hipGetLastError();  // clear the sticky error: the pool retries
            return false;
        }
        HIPCX_CHECK_HIP(e);
        return true;
    }
    void Free(void* ptr) noexcept override { (void)hipFree(ptr); }
    // An event recorded behind the work `stream` holds now; the predicate polls it.  The event lives as long as the predicate.
    std::function<bool()> Fence(void* stream) override {
        SetDeviceScope scope(device_);
        hipEvent_t ev = nullptr;
        HIPCX_CHECK_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        std::shared_ptr<void> holder(ev, [](void* e) { (void)hipEventDestroy(static_cast<hipEvent_t>(e)); });
        HIPCX_CHECK_HIP(hipEventRecord(ev, static_cast<hipStream_t>(stream)));
        return [holder] { return hipEventQuery(static_cast<hipEvent_t>(holder.get())) == hipSuccess; };
    }

private:
    int device_;
};

// Page-locked host memory.  It is allocated as such (hipHostMalloc): registering existing memory is not an option here.
class PinnedAllocator : public Allocator {
public:
    explicit PinnedAllocator(int device) : device_(device) {}
    bool Malloc(void** ptr, size_t bytes) override {
        SetDeviceScope scope(device_);
        hipError_t e = hipHostMalloc(ptr, bytes, hipHostMallocDefault);
        if (e == hipErrorOutOfMemory) {
            (void)hipGetLastError();
            return false;
        }
        HIPCX_CHECK_HIP(e);
        return true;
    }
    void Free(void* ptr) noexcept override { (void)hipHostFree(ptr); }

private:
    int device_;
};

// Keeps the pinned staging buffer of an asynchronous upload alive until the copy has run (MemoryKeeper,
// CX/cuda/cuda_device/memory_keeper.*): an event recorded behind the copy; finished entries are collected on the next call.
struct DeviceState {
    std::shared_ptr<MemoryPool> device_pool;
    std::shared_ptr<MemoryPool> pinned_pool;
    std::mutex keeper_mutex;
    std::deque<std::pair<hipEvent_t, std::shared_ptr<void>>> keeper;
    std::mutex partition_mutex;
    std::map<hipStream_t, uint32_t> partitions;  // stream -> partition of the device pool (the null stream is partition 0)

    uint32_t PartitionOf(hipStream_t stream) {
        if (stream == nullptr) return 0;
        std::lock_guard<std::mutex> lock(partition_mutex);
        auto it = partitions.find(stream);
        if (it == partitions.end()) it = partitions.emplace(stream, static_cast<uint32_t>(partitions.size() + 1)).first;
        return it->second;
    }

    void Collect() {
        std::lock_guard<std::mutex> lock(keeper_mutex);
        while (!keeper.empty() && hipEventQuery(keeper.front().first) == hipSuccess) {
            (void)hipEventDestroy(keeper.front().first);
            keeper.pop_front();
        }
    }
    void Keep(hipStream_t stream, std::shared_ptr<void> memory) {
        hipEvent_t ev = nullptr;
        HIPCX_CHECK_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        hipError_t e = hipEventRecord(ev, stream);
        if (e != hipSuccess) {
            (void)hipEventDestroy(ev);
            HIPCX_CHECK_HIP(e);
        }
        std::lock_guard<std::mutex> lock(keeper_mutex);
        keeper.emplace_back(ev, std::move(memory));
    }
    void DrainKeeper() {  // waits for every pending upload
        std::lock_guard<std::mutex> lock(keeper_mutex);
        for (auto& k : keeper) {
            (void)hipEventSynchronize(k.first);
            (void)hipEventDestroy(k.first);
        }
        keeper.clear();
    }
};

// Never destroyed: at process exit the HIP runtime may already be gone when static destructors run, and the driver reclaims
// the memory anyway.  hipcx_pool_destroy is the orderly way down.
std::mutex& StatesMutex() {
    static std::mutex* m = new std::mutex;
    return *m;
}
std::array<std::shared_ptr<DeviceState>, kMaxDevices>& States() {
    static auto* states = new std::array<std::shared_ptr<DeviceState>, kMaxDevices>();
    return *states;
}

// Blocks that were in use when hipcx_pool_destroy took their pool away: see OrphanSet.
OrphanSet& OrphansOf(int device) {
    static auto* sets = new std::array<OrphanSet, kMaxDevices>();
    return (*sets)[device];
}

std::shared_ptr<DeviceState> StateOf(int device, bool create = true) {
    HIPCX_REQUIRE(device >= 0 && device < kMaxDevices, HIPCX_DEVICE_ERROR, "invalid device index " + std::to_string(device));
    std::lock_guard<std::mutex> lock(StatesMutex());
    auto& g_states = States();
    if (g_states[device] == nullptr && create) {
        int count = 0;
        HIPCX_CHECK_HIP(hipGetDeviceCount(&count));
        HIPCX_REQUIRE(device < count, HIPCX_DEVICE_ERROR, "device index " + std::to_string(device) + " out of range: " + std::to_string(count) + " devices");
        auto st = std::make_shared<DeviceState>();
        st->device_pool = std::make_shared<MemoryPool>(std::unique_ptr<Allocator>(new DeviceAllocator(device)));
        st->pinned_pool = std::make_shared<MemoryPool>(std::unique_ptr<Allocator>(new PinnedAllocator(device)));
        g_states[device] = st;
    }
    return g_states[device];
}

int GuardMemory(const std::function<void()>& f) noexcept {
    try {
        f();
        return HIPCX_OK;
    } catch (const OutOfMemoryError& e) {
        SetLastError(e.what());
        return HIPCX_OUT_OF_MEMORY_ERROR;
    } catch (const Error& e) {
        SetLastError(e.what());
        return e.status;
    } catch (const std::exception& e) {
        SetLastError(e.what());
        return HIPCX_CHAINERX_ERROR;
    } catch (...) {
        SetLastError("unknown error");
        return HIPCX_CHAINERX_ERROR;
    }
}

void UploadAsync(DeviceState& st, int device, void* dst, const void* src, size_t bytes, hipStream_t stream) {
    // CudaDevice::MemoryCopyFromHostAsync (CX/cuda/cuda_device/memory.cc:37-51): stage in pinned memory, copy asynchronously,
    // keep the staging buffer until the copy has run
    SetDeviceScope scope(device);
    st.Collect();
    std::shared_ptr<void> staging = MemoryPool::MakeShared(st.pinned_pool, bytes);
    std::memcpy(staging.get(), src, bytes);
    HIPCX_CHECK_HIP(hipMemcpyAsync(dst, staging.get(), bytes, hipMemcpyHostToDevice, stream));
    st.Keep(stream, std::move(staging));
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_malloc_on_stream(int device, size_t bytes, void* stream, void** ptr) {
    return GuardMemory([&] {
        HIPCX_REQUIRE(ptr != nullptr, HIPCX_CHAINERX_ERROR, "ptr is null");
        *ptr = nullptr;
        if (bytes == 0) return;  // Allocate(0) is a null pointer (CX/native/native_device/memory.cc:14-19)
        std::shared_ptr<DeviceState> st = StateOf(device);
        *ptr = st->device_pool->Malloc(bytes, st->PartitionOf(AsStream(stream)));
    });
}

int hipcx_malloc(int device, size_t bytes, void** ptr) { return hipcx_malloc_on_stream(device, bytes, nullptr, ptr); }

int hipcx_free(int device, void* ptr) {
    return GuardMemory([&] {
        if (ptr == nullptr) return;
        HIPCX_REQUIRE(device >= 0 && device < kMaxDevices, HIPCX_DEVICE_ERROR, "invalid device index " + std::to_string(device));
        // a block of a pool that hipcx_pool_destroy took away: its memory went with the pool (deleters outlive the pool), and the
        // pool that may exist by now must not see this pointer
        if (OrphansOf(device).Take(ptr)) return;
        std::shared_ptr<DeviceState> st = StateOf(device, false);
        if (st == nullptr) return;
        st->device_pool->Free(ptr);
    });
}

int hipcx_record_stream(int device, void* ptr, void* stream) {
    return GuardMemory([&] {
        if (ptr == nullptr) return;
        std::shared_ptr<DeviceState> st = StateOf(device, false);
        HIPCX_REQUIRE(st != nullptr, HIPCX_CHAINERX_ERROR, "record_stream: the device has no pool");
        uint32_t partition = 0;
        HIPCX_REQUIRE(st->device_pool->BlockPartition(ptr, &partition), HIPCX_CHAINERX_ERROR, "record_stream: not a block in use");
        if (st->PartitionOf(AsStream(stream)) == partition) return;  // its own stream: ordered anyway
        st->device_pool->RecordStream(ptr, stream);
    });
}

int hipcx_pool_free_unused(int device) {
    return GuardMemory([&] {
        std::shared_ptr<DeviceState> st = StateOf(device, false);
        if (st == nullptr) return;
        st->Collect();
        st->device_pool->FreeUnusedBlocks();
        st->pinned_pool->FreeUnusedBlocks();
    });
}

int hipcx_pool_stats(int device, hipcx_pool_stats_t* stats) {
    return GuardMemory([&] {
        HIPCX_REQUIRE(stats != nullptr, HIPCX_CHAINERX_ERROR, "stats is null");
        std::memset(stats, 0, sizeof(*stats));
        std::shared_ptr<DeviceState> st = StateOf(device, false);
        if (st == nullptr) return;
        PoolStats s = st->device_pool->stats();
        stats->in_use_bytes = s.in_use_bytes;
        stats->cached_bytes = s.cached_bytes;
        stats->in_use_blocks = s.in_use_blocks;
        stats->cached_blocks = s.cached_blocks;
        stats->device_allocations = s.allocator_calls;
        stats->retries = s.retries;
    });
}

int hipcx_pool_set_arena(int device, int arena) {
    return GuardMemory([&] {
        HIPCX_REQUIRE(arena >= 0, HIPCX_CHAINERX_ERROR, "arena must not be negative");
        StateOf(device)->device_pool->SetArena(arena);
    });
}

int hipcx_pool_release_arena(int device, int arena) {
    return GuardMemory([&] {
        std::shared_ptr<DeviceState> st = StateOf(device, false);
        if (st != nullptr) st->device_pool->ReleaseArena(arena);
    });
}

int hipcx_pool_destroy(int device) {
    return GuardMemory([&] {
        HIPCX_REQUIRE(device >= 0 && device < kMaxDevices, HIPCX_DEVICE_ERROR, "invalid device index");
        std::shared_ptr<DeviceState> st;
        {
            std::lock_guard<std::mutex> lock(StatesMutex());
            st.swap(States()[device]);
        }
        if (st == nullptr) return;
        SetDeviceScope scope(device);
        (void)hipDeviceSynchronize();  // nothing may still run on memory that is about to go back to the driver
        st->DrainKeeper();
        OrphansOf(device).Add(st->device_pool->InUsePointers());  // their frees are still to come: see hipcx_free
    });
}

int hipcx_memcpy_from_host(int device, void* dst, const void* src, size_t bytes, void* stream) {
    return GuardMemory([&] {
        if (bytes == 0) return;
        HIPCX_REQUIRE(dst != nullptr && src != nullptr, HIPCX_CHAINERX_ERROR, "memcpy_from_host: null pointer");
        std::shared_ptr<DeviceState> st = StateOf(device);
        UploadAsync(*st, device, dst, src, bytes, AsStream(stream));
    });
}

int hipcx_memcpy_to_host(int device, void* dst, const void* src, size_t bytes, void* stream) {
    return GuardMemory([&] {
        if (bytes == 0) return;
        HIPCX_REQUIRE(dst != nullptr && src != nullptr, HIPCX_CHAINERX_ERROR, "memcpy_to_host: null pointer");
        SetDeviceScope scope(device);
        // blocking, like CudaDevice::MemoryCopyTo towards the native device (CX/cuda/cuda_device/memory.cc:118-121): ordered
        // behind the work already queued on `stream`, and complete when the call returns
        hipStream_t s = AsStream(stream);
        HIPCX_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s));
        HIPCX_CHECK_HIP(hipStreamSynchronize(s));
        CheckDeferredIndexError(device);  // the bytes may come from a Take whose indices were out of range
    });
}

int hipcx_memcpy_device(int dst_device, void* dst, int src_device, const void* src, size_t bytes, void* stream) {
    return GuardMemory([&] {
        if (bytes == 0) return;
        HIPCX_REQUIRE(dst != nullptr && src != nullptr, HIPCX_CHAINERX_ERROR, "memcpy_device: null pointer");
        SetDeviceScope scope(dst_device);
        if (dst_device == src_device) {
            HIPCX_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, AsStream(stream)));
        } else {
            HIPCX_CHECK_HIP(hipMemcpyPeerAsync(dst, dst_device, src, src_device, bytes, AsStream(stream)));
        }
    });
}

int hipcx_from_host_memory(int device, const void* src, size_t bytes, void** out, void* stream) {
    return GuardMemory([&] {
        HIPCX_REQUIRE(out != nullptr, HIPCX_CHAINERX_ERROR, "out is null");
        *out = nullptr;
        if (bytes == 0) return;
        HIPCX_REQUIRE(src != nullptr, HIPCX_CHAINERX_ERROR, "from_host_memory: src is null");
        std::shared_ptr<DeviceState> st = StateOf(device);
        void* dst = st->device_pool->Malloc(bytes, st->PartitionOf(AsStream(stream)));
        try {
            UploadAsync(*st, device, dst, src, bytes, AsStream(stream));
        } catch (...) {
            st->device_pool->FreeNoExcept(dst);
            throw;
        }
        *out = dst;
    });
}

int hipcx_check_device_pointer(int device, const void* ptr) {
    return GuardMemory([&] {
        if (ptr == nullptr) return;
        hipPointerAttribute_t attr{};
        hipError_t e = hipPointerGetAttributes(&attr, ptr);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            throw Error(HIPCX_CHAINERX_ERROR, "Memory is not a HIP allocation");
        }
        HIPCX_REQUIRE(attr.type == hipMemoryTypeDevice && attr.device == device, HIPCX_CHAINERX_ERROR,
                      "HIP memory must reside on the device: " + std::to_string(device));
    });
}

}  // extern "C"
