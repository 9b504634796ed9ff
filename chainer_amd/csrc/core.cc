// Library-wide state: last-error string, device queries.
#include <cstdlib>
#include <cstdint>
#include <mutex>
#include "common.h"

namespace hipcx {

namespace {
thread_local std::string g_last_error;
}

void SetLastError(const std::string& msg) { g_last_error = msg; }

int64_t StreamingThresholdBytes() {
    static const int64_t bytes = [] {
        const char* e = getenv("HIPCX_STREAM_MB");
        int64_t mb = e != nullptr ? atoll(e) : 75;
        return mb <= 0 ? INT64_MAX : mb * 1000000;
    }();
    return bytes;
}

namespace {
constexpr int kMaxRecordDevices = 64;
std::mutex g_record_mu;
volatile int64_t* g_record_host[kMaxRecordDevices] = {};  // page-locked, four int64 per device
int64_t* g_record_dev[kMaxRecordDevices] = {};            // the same memory as the device addresses it
}  // namespace

int64_t* DeferredIndexErrorRecord() {
    int dev = 0;
    HIPCX_CHECK_HIP(hipGetDevice(&dev));
    HIPCX_REQUIRE(dev >= 0 && dev < kMaxRecordDevices, HIPCX_DEVICE_ERROR, "device index out of range");
    std::lock_guard<std::mutex> lock(g_record_mu);
    if (g_record_dev[dev] == nullptr) {
        void* host = nullptr;
        HIPCX_CHECK_HIP(hipHostMalloc(&host, 4 * sizeof(int64_t), hipHostMallocMapped | hipHostMallocCoherent));
        for (int i = 0; i < 4; ++i) static_cast<volatile int64_t*>(host)[i] = 0;
        void* devptr = nullptr;
        HIPCX_CHECK_HIP(hipHostGetDevicePointer(&devptr, host, 0));
        g_record_host[dev] = static_cast<volatile int64_t*>(host);
        g_record_dev[dev] = static_cast<int64_t*>(devptr);
    }
    return g_record_dev[dev];
}

void CheckDeferredIndexError(int device) {
    if (device < 0 || device >= kMaxRecordDevices) return;
    int64_t index = 0, dim = 0, axis = 0;
    {
        std::lock_guard<std::mutex> lock(g_record_mu);
        volatile int64_t* rec = g_record_host[device];
        if (rec == nullptr || rec[0] == 0) return;
        index = rec[1], dim = rec[2], axis = rec[3];
        rec[0] = 0;
    }
    throw Error(HIPCX_INDEX_ERROR, "Index " + std::to_string(index) + " is out of bounds for axis " + std::to_string(axis) + " with size " +
                                           std::to_string(dim) + " (an earlier take / add_at in the default bounds mode)");
}

int NumCUs() {
    static thread_local int cached_dev = -1;
    static thread_local int cached = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached = n;
        cached_dev = dev;
    }
    return cached;
}

}  // namespace hipcx

using namespace hipcx;

extern "C" {

const char* hipcx_last_error(void) { return g_last_error.c_str(); }

int hipcx_version(void) { return 1; }

int hipcx_device_count(int* count) {
    return Guard([&] {
        HIPCX_REQUIRE(count != nullptr, HIPCX_CHAINERX_ERROR, "count is null");
        int n = 0;
        hipError_t e = hipGetDeviceCount(&n);
        if (e == hipErrorNoDevice) {
            n = 0;
        } else {
            HIPCX_CHECK_HIP(e);
        }
        *count = n;
    });
}

int hipcx_synchronize(int device_index) {
    return Guard([&] {
        int prev = 0;
        HIPCX_CHECK_HIP(hipGetDevice(&prev));
        HIPCX_CHECK_HIP(hipSetDevice(device_index));
        hipError_t e = hipDeviceSynchronize();
        (void)hipSetDevice(prev);
        HIPCX_CHECK_HIP(e);
        CheckDeferredIndexError(device_index);
    });
}

int hipcx_device_name(int device_index, char* buf, size_t buf_len) {
    return Guard([&] {
        HIPCX_REQUIRE(buf != nullptr && buf_len > 0, HIPCX_CHAINERX_ERROR, "buffer is null");
        hipDeviceProp_t prop;
        HIPCX_CHECK_HIP(hipGetDeviceProperties(&prop, device_index));
        std::snprintf(buf, buf_len, "%s (%s)", prop.name, prop.gcnArchName);
    });
}

int64_t hipcx_conv_out_dim(int64_t in_dim, int64_t kernel_size, int64_t stride, int64_t pad, int cover_all) {
    if (stride <= 0) return -1;
    int64_t numerator = in_dim + pad * 2 - kernel_size + (cover_all ? stride - 1 : 0);
    if (numerator < 0) return -1;
    return numerator / stride + 1;
}
}
