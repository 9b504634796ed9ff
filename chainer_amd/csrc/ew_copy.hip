// Creation kernels: dtype-casting strided Copy (every In x Out pair, CX/native/native_device/copy.cc:21-35),
// Fill (CX/native/native_device/fill.cc:156-170) and Arange (fill.cc:33-48).
#include "elementwise.h"

namespace hipcx {
namespace {

// static_cast<Out>(In) with float16 widened through float first, as chainerx::Float16's
// conversion operators do (CX/float16.h).  float -> integer conversions of out-of-range values
// are undefined in C++; they saturate here.
template <typename TIn, typename TOut>
struct CastOp {
    using In = TIn;
    using Out = TOut;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    static constexpr bool kNarrowVectors = std::is_same<TIn, TOut>::value && sizeof(TIn) <= 4;  // plain copies
    __device__ __forceinline__ compute_t<TOut> operator()(compute_t<TIn> a, compute_t<TIn>, compute_t<TIn>, compute_t<TIn>, int64_t) const {
        if constexpr (std::is_same<TOut, bool>::value) {
            return a != compute_t<TIn>{};
        } else {
            return static_cast<compute_t<TOut>>(a);
        }
    }
};

template <typename T>
struct FillOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 0;
    static constexpr bool kNeedsIndex = false;
    T value;
    __device__ __forceinline__ T operator()(compute_t<T>, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const { return value; }
};

// out[i] = start + step * i evaluated in T (float16: in float, then rounded).
template <typename T>
struct ArangeOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 0;
    static constexpr bool kNeedsIndex = true;
    compute_t<T> start, step;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T>, compute_t<T>, compute_t<T>, compute_t<T>, int64_t i) const {
        return start + step * static_cast<compute_t<T>>(i);
    }
};

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_copy(const hipcx_array* a, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, a});
        VisitDtype(a->dtype, [&](auto in_tag) {
            using TIn = typename decltype(in_tag)::type;
            VisitDtype(out->dtype, [&](auto out_tag) {
                using TOut = typename decltype(out_tag)::type;
                LaunchElementwise(p, CastOp<TIn, TOut>{}, AsStream(stream));
            });
        });
    });
}

int hipcx_fill(const hipcx_array* out, hipcx_scalar value, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out});
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            FillOp<T> op;
            op.value = ScalarTo<T>(value);
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

int hipcx_arange(hipcx_scalar start, hipcx_scalar step, const hipcx_array* out, void* stream) {
    return Guard([&] {
        HIPCX_REQUIRE(out->ndim == 1, HIPCX_DIMENSION_ERROR, "arange output must be 1-dimensional");
        EwPlan p = MakeEwPlan({out});
        VisitNumericDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            ArangeOp<T> op;
            op.start = static_cast<compute_t<T>>(ScalarTo<T>(start));
            op.step = static_cast<compute_t<T>>(ScalarTo<T>(step));
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}
}
