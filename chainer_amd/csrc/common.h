// Shared host/device helpers for the gfx950 kernel library.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "hipcx.h"

namespace hipcx {

// ---------------------------------------------------------------------------------------------
// Errors.  Entry points are `extern "C"`; inside them errors travel as exceptions and are turned
// into a status code + thread-local message at the boundary.
// ---------------------------------------------------------------------------------------------
struct Error : std::runtime_error {
    int status;
    Error(int st, const std::string& msg) : std::runtime_error(msg), status(st) {}
};

void SetLastError(const std::string& msg);

// Out-of-range indices of Take / AddAt in the default bounds mode, reported late: the native backend throws IndexError from
// inside the kernel call (CX/native/native_device/indexing.cc:68-74), which on a device would cost a read-back and a host wait
// per call.  Instead each device has one sticky record of four int64 {set, index, extent, axis} in page-locked host memory that
// kernels write through its device address, and the calls at which the host waits for the device anyway -- hipcx_synchronize and
// hipcx_memcpy_to_host, the only points where results become visible (CX/cuda/cuda_device/memory.cc:94-122) -- look at it after
// their wait: a set record is cleared and becomes their HIPCX_INDEX_ERROR.
// DeferredIndexErrorRecord: the current device's record as a kernel argument (allocated on first use).
// CheckDeferredIndexError: throws Error(HIPCX_INDEX_ERROR) if `device`'s record is set; the caller has just waited for the work.
int64_t* DeferredIndexErrorRecord();
void CheckDeferredIndexError(int device);

#define HIPCX_CHECK_HIP(expr)                                                                           \
    do {                                                                                                \
        hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess) {                                                                         \
            throw ::hipcx::Error(HIPCX_BACKEND_ERROR, std::string(#expr) + ": " + hipGetErrorString(e_)); \
        }                                                                                               \
    } while (0)

#define HIPCX_REQUIRE(cond, status, msg)              \
    do {                                              \
        if (!(cond)) throw ::hipcx::Error(status, msg); \
    } while (0)

// Wraps the body of an entry point.
template <typename F>
inline int Guard(F&& f) noexcept {
    try {
        f();
        return HIPCX_OK;
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

inline void CheckLaunch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        throw Error(HIPCX_BACKEND_ERROR, std::string(what) + " launch failed: " + hipGetErrorString(e));
    }
}

// ---------------------------------------------------------------------------------------------
// dtypes
// ---------------------------------------------------------------------------------------------
using half_t = _Float16;

inline int64_t ItemSize(int dtype) {
    switch (dtype) {
        case HIPCX_BOOL:
        case HIPCX_INT8:
        case HIPCX_UINT8:
            return 1;
        case HIPCX_INT16:
        case HIPCX_FLOAT16:
            return 2;
        case HIPCX_INT32:
        case HIPCX_FLOAT32:
            return 4;
        case HIPCX_INT64:
        case HIPCX_FLOAT64:
            return 8;
        default:
            throw Error(HIPCX_DTYPE_ERROR, "invalid dtype code " + std::to_string(dtype));
    }
}

inline bool IsFloatDtype(int dtype) { return dtype == HIPCX_FLOAT16 || dtype == HIPCX_FLOAT32 || dtype == HIPCX_FLOAT64; }

inline const char* DtypeName(int dtype) {
    static const char* names[] = {"?", "bool", "int8", "int16", "int32", "int64", "uint8", "float16", "float32", "float64"};
    return (dtype >= 1 && dtype <= 9) ? names[dtype] : "?";
}

template <typename T>
struct DtypeOf;
template <> struct DtypeOf<bool> { static constexpr int value = HIPCX_BOOL; };
template <> struct DtypeOf<int8_t> { static constexpr int value = HIPCX_INT8; };
template <> struct DtypeOf<int16_t> { static constexpr int value = HIPCX_INT16; };
template <> struct DtypeOf<int32_t> { static constexpr int value = HIPCX_INT32; };
template <> struct DtypeOf<int64_t> { static constexpr int value = HIPCX_INT64; };
template <> struct DtypeOf<uint8_t> { static constexpr int value = HIPCX_UINT8; };
template <> struct DtypeOf<half_t> { static constexpr int value = HIPCX_FLOAT16; };
template <> struct DtypeOf<float> { static constexpr int value = HIPCX_FLOAT32; };
template <> struct DtypeOf<double> { static constexpr int value = HIPCX_FLOAT64; };

template <typename T>
struct Tag {
    using type = T;
};

// Calls f(Tag<T>{}) with the C++ type of `dtype` (all nine dtypes).
template <typename F>
inline void VisitDtype(int dtype, F&& f) {
    switch (dtype) {
        case HIPCX_BOOL: f(Tag<bool>{}); break;
        case HIPCX_INT8: f(Tag<int8_t>{}); break;
        case HIPCX_INT16: f(Tag<int16_t>{}); break;
        case HIPCX_INT32: f(Tag<int32_t>{}); break;
        case HIPCX_INT64: f(Tag<int64_t>{}); break;
        case HIPCX_UINT8: f(Tag<uint8_t>{}); break;
        case HIPCX_FLOAT16: f(Tag<half_t>{}); break;
        case HIPCX_FLOAT32: f(Tag<float>{}); break;
        case HIPCX_FLOAT64: f(Tag<double>{}); break;
        default: throw Error(HIPCX_DTYPE_ERROR, "invalid dtype code " + std::to_string(dtype));
    }
}

template <typename F>
inline void VisitNumericDtype(int dtype, F&& f) {
    HIPCX_REQUIRE(dtype != HIPCX_BOOL, HIPCX_DTYPE_ERROR, "bool dtype is not supported by this kernel");
    VisitDtype(dtype, std::forward<F>(f));
}

template <typename F>
inline void VisitFloatDtype(int dtype, F&& f) {
    switch (dtype) {
        case HIPCX_FLOAT16: f(Tag<half_t>{}); break;
        case HIPCX_FLOAT32: f(Tag<float>{}); break;
        case HIPCX_FLOAT64: f(Tag<double>{}); break;
        default: throw Error(HIPCX_DTYPE_ERROR, std::string("floating point dtype required, got ") + DtypeName(dtype));
    }
}

// Arithmetic type: float16 values are widened to float for every operation and rounded back
// (round-to-nearest-even) on store, as chainerx::Float16 does.
template <typename T>
struct ComputeType {
    using type = T;
};
template <>
struct ComputeType<half_t> {
    using type = float;
};
template <typename T>
using compute_t = typename ComputeType<T>::type;

// Scalar -> T with the semantics of static_cast<T>(chainerx::Scalar).
template <typename T>
inline T ScalarTo(const hipcx_scalar& s) {
    switch (s.kind) {
        case HIPCX_KIND_BOOL: return static_cast<T>(s.i != 0);
        case HIPCX_KIND_INT: return static_cast<T>(s.i);
        case HIPCX_KIND_FLOAT: return static_cast<T>(s.f);
        default: throw Error(HIPCX_CHAINERX_ERROR, "invalid scalar kind");
    }
}
template <>
inline half_t ScalarTo<half_t>(const hipcx_scalar& s) {
    switch (s.kind) {
        case HIPCX_KIND_BOOL: return static_cast<half_t>(static_cast<float>(s.i != 0));
        case HIPCX_KIND_INT: return static_cast<half_t>(static_cast<float>(s.i));
        case HIPCX_KIND_FLOAT: return static_cast<half_t>(s.f);
        default: throw Error(HIPCX_CHAINERX_ERROR, "invalid scalar kind");
    }
}

// ---------------------------------------------------------------------------------------------
// Array helpers (host)
// ---------------------------------------------------------------------------------------------
inline void ValidateArray(const hipcx_array* a, const char* name) {
    HIPCX_REQUIRE(a != nullptr, HIPCX_CHAINERX_ERROR, std::string(name) + " is null");
    HIPCX_REQUIRE(a->ndim >= 0 && a->ndim <= HIPCX_MAX_NDIM, HIPCX_DIMENSION_ERROR, std::string(name) + ": ndim out of range");
    (void)ItemSize(a->dtype);
    for (int i = 0; i < a->ndim; ++i) {
        HIPCX_REQUIRE(a->shape[i] >= 0, HIPCX_DIMENSION_ERROR, std::string(name) + ": negative extent");
    }
}

inline int64_t TotalSize(const hipcx_array* a) {
    int64_t n = 1;
    for (int i = 0; i < a->ndim; ++i) n *= a->shape[i];
    return n;
}

inline bool SameShape(const hipcx_array* a, const hipcx_array* b) {
    if (a->ndim != b->ndim) return false;
    for (int i = 0; i < a->ndim; ++i) {
        if (a->shape[i] != b->shape[i]) return false;
    }
    return true;
}

inline std::string ShapeStr(const hipcx_array* a) {
    std::string s = "(";
    for (int i = 0; i < a->ndim; ++i) {
        s += std::to_string(a->shape[i]);
        if (i + 1 < a->ndim || a->ndim == 1) s += ",";
    }
    return s + ")";
}

// C-contiguous ignoring unit-length axes (CX/shape.cc:15-32).
inline bool IsContiguous(const hipcx_array* a) {
    int64_t expect = ItemSize(a->dtype);
    for (int i = a->ndim - 1; i >= 0; --i) {
        if (a->shape[i] == 0) return true;
        if (a->shape[i] != 1 && a->strides[i] != expect) return false;
        expect *= a->shape[i];
    }
    return true;
}

inline hipStream_t AsStream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline int DivUp(int64_t a, int64_t b) { return static_cast<int>((a + b - 1) / b); }

// Number of compute units of the current device (cached); used to size grid-stride launches.
int NumCUs();

// Input size beyond which a streaming kernel loads without allocating in the caches.  A large tensor read front to back with
// allocating loads pushes out what the memory-side cache (256 MB on this part) still holds of it and of its neighbours in the
// network; the threshold (75 MB) is the measured optimum over a ResNet-50 forward pass.  HIPCX_STREAM_MB overrides (0 = never).
int64_t StreamingThresholdBytes();

}  // namespace hipcx
