// Library-wide state: last-error string, device queries.
#include <cstdlib>
#include <cstdint>
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
