// Arithmetic kernels: Add / Subtract / Multiply / Divide in array-array, array-scalar and
// scalar-array forms.  Semantics follow chainerx::ArithmeticOps (CX/arithmetic_ops.h:7-25: bool
// Add is OR, bool Multiply/Divide is AND) applied in the output dtype, float16 through float
// (CX/native/native_device/arithmetic.cc:44-219).
#include "elementwise.h"

namespace hipcx {
namespace {

enum class Arith { kAdd, kSub, kMul, kDiv };

template <Arith A, typename C>
__device__ __forceinline__ C Apply(C a, C b) {
    if constexpr (std::is_same<C, bool>::value) {
        if constexpr (A == Arith::kAdd) return a || b;
        return a && b;
    } else {
        if constexpr (A == Arith::kAdd) return a + b;
        if constexpr (A == Arith::kSub) return a - b;
        if constexpr (A == Arith::kMul) return a * b;
        if constexpr (A == Arith::kDiv) return a / b;
    }
}

template <typename T, Arith A>
struct BinaryAA {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 2;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        return Apply<A, compute_t<T>>(a, b);
    }
};

// SCALAR_LEFT: out = s op x, otherwise out = x op s.  The scalar has already been converted to T
// (static_cast<T>(Scalar), CX/native/native_device/arithmetic.cc:58).
template <typename T, Arith A, bool SCALAR_LEFT>
struct BinaryAS {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    compute_t<T> s;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        return SCALAR_LEFT ? Apply<A, compute_t<T>>(s, a) : Apply<A, compute_t<T>>(a, s);
    }
};

void RequireSameDtype(const hipcx_array* x, const hipcx_array* out, const char* what) {
    HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                  std::string(what) + ": operand dtype " + DtypeName(x->dtype) + " differs from out dtype " + DtypeName(out->dtype) +
                          " (cast with hipcx_copy first)");
}

template <Arith A>
void RunAA(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream, bool allow_bool) {
    EwPlan p = MakeEwPlan({out, x1, x2});
    RequireSameDtype(x1, out, "x1");
    RequireSameDtype(x2, out, "x2");
    HIPCX_REQUIRE(allow_bool || out->dtype != HIPCX_BOOL, HIPCX_DTYPE_ERROR, "bool dtype is not supported by this kernel");
    VisitDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        LaunchElementwise(p, BinaryAA<T, A>{}, AsStream(stream));
    });
}

template <Arith A, bool SCALAR_LEFT>
void RunAS(const hipcx_array* x, hipcx_scalar s, const hipcx_array* out, void* stream, bool allow_bool) {
    EwPlan p = MakeEwPlan({out, x});
    RequireSameDtype(x, out, "x");
    HIPCX_REQUIRE(allow_bool || out->dtype != HIPCX_BOOL, HIPCX_DTYPE_ERROR, "bool dtype is not supported by this kernel");
    VisitDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        BinaryAS<T, A, SCALAR_LEFT> op;
        op.s = static_cast<compute_t<T>>(ScalarTo<T>(s));
        LaunchElementwise(p, op, AsStream(stream));
    });
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {
int hipcx_add(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAA<Arith::kAdd>(x1, x2, out, stream, true); });
}
int hipcx_subtract(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAA<Arith::kSub>(x1, x2, out, stream, false); });
}
int hipcx_multiply(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAA<Arith::kMul>(x1, x2, out, stream, true); });
}
int hipcx_divide(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAA<Arith::kDiv>(x1, x2, out, stream, true); });
}
int hipcx_add_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAS<Arith::kAdd, false>(x1, x2, out, stream, true); });
}
int hipcx_subtract_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAS<Arith::kSub, false>(x1, x2, out, stream, false); });
}
int hipcx_multiply_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAS<Arith::kMul, false>(x1, x2, out, stream, true); });
}
int hipcx_divide_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAS<Arith::kDiv, false>(x1, x2, out, stream, true); });
}
int hipcx_divide_sa(hipcx_scalar x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunAS<Arith::kDiv, true>(x2, x1, out, stream, true); });
}
}
