// Unary float math (Exp, Log, Tanh, Sqrt), the select kernels behind ReLU / Maximum / Minimum and
// the comparison kernels.  float16 is evaluated as Float16(f(float(x))) like the native backend
// (CX/numeric.h:55-87, CX/native/native_device/{exp_log,hyperbolic,misc,logic}.cc).
#include "elementwise.h"

namespace hipcx {
namespace {

enum class Unary { kExp, kLog, kTanh, kSqrt };

template <typename T, Unary U>
struct UnaryOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        using C = compute_t<T>;
        if constexpr (std::is_same<C, float>::value) {
            if constexpr (U == Unary::kExp) return expf(a);
            if constexpr (U == Unary::kLog) return logf(a);
            if constexpr (U == Unary::kTanh) return tanhf(a);
            if constexpr (U == Unary::kSqrt) return sqrtf(a);
        } else {
            if constexpr (U == Unary::kExp) return exp(a);
            if constexpr (U == Unary::kLog) return log(a);
            if constexpr (U == Unary::kTanh) return tanh(a);
            if constexpr (U == Unary::kSqrt) return sqrt(a);
        }
    }
};

template <Unary U>
void RunUnary(const hipcx_array* x, const hipcx_array* out, void* stream) {
    EwPlan p = MakeEwPlan({out, x});
    HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x dtype differs from out dtype (cast with hipcx_copy first)");
    VisitFloatDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        LaunchElementwise(p, UnaryOp<T, U>{}, AsStream(stream));
    });
}

// out = (x1 < x2) ? pos : neg  (LESS) or (x1 > x2) ? pos : neg, x2/pos scalars.
// Inputs: a = x1, b = neg.  A NaN x1 fails both comparisons and passes `neg` through.
template <typename T, bool LESS>
struct SelectASSA {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 2;
    static constexpr bool kNeedsIndex = false;
    compute_t<T> x2, pos;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        bool c = LESS ? (a < x2) : (a > x2);
        return c ? pos : b;
    }
};

// The same with neg == x1 (one array passed twice, as Relu does: IfLessElse(x, 0, 0, x), CX/routines/activation.cc): one load per
// element instead of two of the same address; the result is the same bit for bit.
template <typename T, bool LESS>
struct SelectSelfASS {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    compute_t<T> x2, pos;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        bool c = LESS ? (a < x2) : (a > x2);
        return c ? pos : a;
    }
};

// One array described twice: same memory, dtype, shape and strides.
inline bool SameArray(const hipcx_array* a, const hipcx_array* b) {
    if (a->data != b->data || a->dtype != b->dtype || !SameShape(a, b)) return false;
    for (int i = 0; i < a->ndim; ++i) {
        if (a->shape[i] > 1 && a->strides[i] != b->strides[i]) return false;
    }
    return true;
}

template <typename T>
struct SelectGreaterAAAA {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 4;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> x1, compute_t<T> x2, compute_t<T> pos, compute_t<T> neg,
                                                       int64_t) const {
        return x1 > x2 ? pos : neg;
    }
};

template <bool LESS>
void RunSelectASSA(const hipcx_array* x1, hipcx_scalar x2, hipcx_scalar pos, const hipcx_array* neg, const hipcx_array* out,
                   void* stream) {
    ValidateArray(x1, "x1");
    ValidateArray(neg, "neg");
    HIPCX_REQUIRE(x1->dtype == out->dtype && neg->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                  "x1/neg dtype differs from out dtype (cast with hipcx_copy first)");
    if (SameArray(x1, neg)) {
        EwPlan p = MakeEwPlan({out, x1});
        VisitNumericDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            SelectSelfASS<T, LESS> op;
            op.x2 = static_cast<compute_t<T>>(ScalarTo<T>(x2));
            op.pos = static_cast<compute_t<T>>(ScalarTo<T>(pos));
            LaunchElementwise(p, op, AsStream(stream));
        });
        return;
    }
    EwPlan p = MakeEwPlan({out, x1, neg});
    VisitNumericDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        SelectASSA<T, LESS> op;
        op.x2 = static_cast<compute_t<T>>(ScalarTo<T>(x2));
        op.pos = static_cast<compute_t<T>>(ScalarTo<T>(pos));
        LaunchElementwise(p, op, AsStream(stream));
    });
}

enum class Cmp { kEq, kNe, kGt, kGe };

template <typename T, Cmp C>
struct CompareOp {
    using In = T;
    using Out = bool;
    static constexpr int kNumIn = 2;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ bool operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        if constexpr (C == Cmp::kEq) return a == b;
        if constexpr (C == Cmp::kNe) return a != b;
        if constexpr (C == Cmp::kGt) return a > b;
        if constexpr (C == Cmp::kGe) return a >= b;
    }
};

template <Cmp C>
void RunCompare(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    EwPlan p = MakeEwPlan({out, x1, x2});
    HIPCX_REQUIRE(out->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "comparison output must be bool");
    HIPCX_REQUIRE(x1->dtype == x2->dtype, HIPCX_DTYPE_ERROR, "comparison operands must share a dtype (cast with hipcx_copy first)");
    VisitDtype(x1->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        LaunchElementwise(p, CompareOp<T, C>{}, AsStream(stream));
    });
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {
int hipcx_exp(const hipcx_array* x, const hipcx_array* out, void* stream) {
    return Guard([&] { RunUnary<Unary::kExp>(x, out, stream); });
}
int hipcx_log(const hipcx_array* x, const hipcx_array* out, void* stream) {
    return Guard([&] { RunUnary<Unary::kLog>(x, out, stream); });
}
int hipcx_tanh(const hipcx_array* x, const hipcx_array* out, void* stream) {
    return Guard([&] { RunUnary<Unary::kTanh>(x, out, stream); });
}
int hipcx_sqrt(const hipcx_array* x, const hipcx_array* out, void* stream) {
    return Guard([&] { RunUnary<Unary::kSqrt>(x, out, stream); });
}
int hipcx_if_less_else_assa(const hipcx_array* x1, hipcx_scalar x2, hipcx_scalar pos, const hipcx_array* neg, const hipcx_array* out,
                            void* stream) {
    return Guard([&] { RunSelectASSA<true>(x1, x2, pos, neg, out, stream); });
}
int hipcx_if_greater_else_assa(const hipcx_array* x1, hipcx_scalar x2, hipcx_scalar pos, const hipcx_array* neg,
                               const hipcx_array* out, void* stream) {
    return Guard([&] { RunSelectASSA<false>(x1, x2, pos, neg, out, stream); });
}
int hipcx_if_greater_else_aaaa(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* pos, const hipcx_array* neg,
                               const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1, x2, pos, neg});
        HIPCX_REQUIRE(x1->dtype == out->dtype && x2->dtype == out->dtype && pos->dtype == out->dtype && neg->dtype == out->dtype,
                      HIPCX_DTYPE_ERROR, "operand dtype differs from out dtype (cast with hipcx_copy first)");
        VisitNumericDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            LaunchElementwise(p, SelectGreaterAAAA<T>{}, AsStream(stream));
        });
    });
}
int hipcx_equal(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunCompare<Cmp::kEq>(x1, x2, out, stream); });
}
int hipcx_not_equal(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunCompare<Cmp::kNe>(x1, x2, out, stream); });
}
int hipcx_greater(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunCompare<Cmp::kGt>(x1, x2, out, stream); });
}
int hipcx_greater_equal(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] { RunCompare<Cmp::kGe>(x1, x2, out, stream); });
}
}
