// Further elementwise kernels of the ChainerX kernel set: the remaining unary float math, Square / Abs / Sign, the
// IsNan / IsInf / IsFinite / LogicalNot predicates, LogicalAnd / Or / Xor, Power (three operand forms), Fmod, Arctan2 and
// Where (four operand forms).  float16 is evaluated as Float16(f(float(x))) like the native backend (CX/numeric.h:55-135).
#include "elementwise.h"

namespace hipcx {
namespace {

#define HIPCX_UNARY_CASES(SUF)                        \
    switch (OP) {                                     \
        case HIPCX_UNARY_ERF: return erf##SUF(a);     \
        case HIPCX_UNARY_EXPM1: return expm1##SUF(a); \
        case HIPCX_UNARY_EXP2: return exp2##SUF(a);   \
        case HIPCX_UNARY_LOG10: return log10##SUF(a); \
        case HIPCX_UNARY_LOG2: return log2##SUF(a);   \
        case HIPCX_UNARY_LOG1P: return log1p##SUF(a); \
        case HIPCX_UNARY_SINH: return sinh##SUF(a);   \
        case HIPCX_UNARY_COSH: return cosh##SUF(a);   \
        case HIPCX_UNARY_ARCSINH: return asinh##SUF(a); \
        case HIPCX_UNARY_ARCCOSH: return acosh##SUF(a); \
        case HIPCX_UNARY_SIN: return sin##SUF(a);     \
        case HIPCX_UNARY_COS: return cos##SUF(a);     \
        case HIPCX_UNARY_TAN: return tan##SUF(a);     \
        case HIPCX_UNARY_ARCSIN: return asin##SUF(a); \
        case HIPCX_UNARY_ARCCOS: return acos##SUF(a); \
        case HIPCX_UNARY_ARCTAN: return atan##SUF(a); \
        case HIPCX_UNARY_CEIL: return ceil##SUF(a);   \
        case HIPCX_UNARY_FLOOR: return floor##SUF(a); \
        default: return a;                            \
    }

template <typename T, int OP>
struct FloatUnaryOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        if constexpr (std::is_same<compute_t<T>, float>::value) {
            HIPCX_UNARY_CASES(f)
        } else {
            HIPCX_UNARY_CASES()
        }
    }
};

// Square: x * x; Abs: std::abs (identity for uint8); Sign: NaN passes, else (0 < x) - (x < 0)  (CX/numeric.h:33-57).
template <typename T, int OP>
struct NumericUnaryOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        using C = compute_t<T>;
        if constexpr (OP == HIPCX_UNARY_SQUARE) {
            if constexpr (std::is_integral<C>::value && std::is_signed<C>::value) {
                // wraps like the two's-complement multiplication of the narrow type, without signed-overflow undefinedness
                using U = std::make_unsigned_t<C>;
                return static_cast<C>(static_cast<U>(static_cast<U>(a) * static_cast<U>(a)));
            } else {
                return a * a;
            }
        } else if constexpr (OP == HIPCX_UNARY_ABS) {
            if constexpr (std::is_unsigned<C>::value) {
                return a;
            } else if constexpr (std::is_integral<C>::value) {
                using U = std::make_unsigned_t<C>;
                return a < 0 ? static_cast<C>(U(0) - static_cast<U>(a)) : a;  // abs(lowest) wraps to lowest
            } else if constexpr (std::is_same<C, float>::value) {
                return fabsf(a);
            } else {
                return fabs(a);
            }
        } else {
            if (a != a) return a;
            return static_cast<C>(static_cast<int>(C(0) < a) - static_cast<int>(a < C(0)));
        }
    }
};

template <typename T, int OP>
struct PredicateOp {
    using In = T;
    using Out = bool;
    static constexpr int kNumIn = 1;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ bool operator()(compute_t<T> a, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        using C = compute_t<T>;
        constexpr bool kFloat = std::is_floating_point<C>::value;
        if constexpr (OP == HIPCX_PRED_LOGICAL_NOT) return !static_cast<bool>(a);
        if constexpr (OP == HIPCX_PRED_ISNAN) return kFloat ? a != a : false;
        if constexpr (OP == HIPCX_PRED_ISINF) {
            if constexpr (kFloat) return a == __builtin_huge_val() || a == -__builtin_huge_val();
            else return false;
        }
        if constexpr (OP == HIPCX_PRED_ISFINITE) {
            if constexpr (kFloat) return a == a && a != __builtin_huge_val() && a != -__builtin_huge_val();
            else return true;
        }
    }
};

template <typename T, int OP>
struct LogicalOp {
    using In = T;
    using Out = bool;
    static constexpr int kNumIn = 2;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ bool operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        const bool x = static_cast<bool>(a), y = static_cast<bool>(b);
        if constexpr (OP == HIPCX_LOGICAL_AND) return x && y;
        if constexpr (OP == HIPCX_LOGICAL_OR) return x || y;
        if constexpr (OP == HIPCX_LOGICAL_XOR) return x != y;
    }
};

// Power (CX/numeric.h:85-135): integers by repeated squaring (wrapping), a negative exponent gives 1 / -1 for bases 1 / -1
// and 0 otherwise; floats through pow.
template <typename C>
__device__ __forceinline__ C PowerOf(C x1, C x2) {
    if constexpr (std::is_same<C, bool>::value) {
        return x1;  // never launched: bool is rejected on the host
    } else if constexpr (std::is_integral<C>::value) {
        using U = std::make_unsigned_t<C>;
        if constexpr (std::is_signed<C>::value) {
            if (x2 < 0) {
                if (x1 == C(-1)) return (x2 & 1) ? C(-1) : C(1);
                return x1 == C(1) ? C(1) : C(0);
            }
        }
        U out = 1, base = static_cast<U>(x1);
        U e = static_cast<U>(x2);
        while (e > 0) {
            if (e & 1) out *= base;
            base *= base;
            e >>= 1;
        }
        return static_cast<C>(out);
    } else if constexpr (std::is_same<C, float>::value) {
        return powf(x1, x2);
    } else {
        return pow(x1, x2);
    }
}

// kind 0: array ** array; 1: array ** scalar; 2: scalar ** array
template <typename T, int KIND>
struct PowerOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = KIND == 0 ? 2 : 1;
    static constexpr bool kNeedsIndex = false;
    compute_t<T> scalar;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        using C = compute_t<T>;
        // narrow integers are computed in their own width, as the reference's template does
        auto narrow = [](C v) { return static_cast<C>(static_cast<T>(v)); };
        if constexpr (KIND == 0) return narrow(PowerOf<C>(a, b));
        if constexpr (KIND == 1) return narrow(PowerOf<C>(a, scalar));
        if constexpr (KIND == 2) return narrow(PowerOf<C>(scalar, a));
    }
};

template <typename T, bool ATAN2>
struct FloatBinaryOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 2;
    static constexpr bool kNeedsIndex = false;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        if constexpr (std::is_same<compute_t<T>, float>::value) {
            return ATAN2 ? atan2f(a, b) : fmodf(a, b);
        } else {
            return ATAN2 ? atan2(a, b) : fmod(a, b);
        }
    }
};

// FloorDivide / Mod (native/native_device/arithmetic.cc:107-139, 260-295): integers floor towards -inf and give 0 for a zero
// divisor (Mod also for a zero dividend); floats follow fmod with the sign fixed up (Mod by zero is NaN).
template <typename C>
__device__ __forceinline__ C FloorDivideOf(C x, C y) {
    if constexpr (std::is_same<C, bool>::value) {
        return x;  // never launched
    } else if constexpr (std::is_integral<C>::value) {
        if (y == 0) return 0;
        if constexpr (std::is_unsigned<C>::value) {
            return x / y;
        } else {
            using W = std::conditional_t<sizeof(C) == 8, int64_t, int32_t>;
            if (y == C(-1)) return static_cast<C>(W(0) - static_cast<W>(x));  // avoids the trapping lowest / -1
            W q = static_cast<W>(x) / static_cast<W>(y), r = static_cast<W>(x) % static_cast<W>(y);
            return static_cast<C>(q - ((y >= 0 ? r : -r) < 0 ? 1 : 0));
        }
    } else {
        C rem = std::is_same<C, float>::value ? fmodf(x, y) : fmod(x, y);
        return (x - rem) / y - (((rem < 0 && y > 0) || (rem > 0 && y < 0)) ? C(1) : C(0));
    }
}

template <typename C>
__device__ __forceinline__ C ModOf(C x, C y) {
    if constexpr (std::is_same<C, bool>::value) {
        return x;  // never launched
    } else if constexpr (std::is_integral<C>::value) {
        if (x == 0 || y == 0) return 0;
        if constexpr (std::is_unsigned<C>::value) {
            return x % y;
        } else {
            if (y == C(-1)) return 0;
            int64_t r = static_cast<int64_t>(x) % static_cast<int64_t>(y);
            if ((r > 0 && y < 0) || (r < 0 && y > 0)) r += y;
            return static_cast<C>(r);
        }
    } else {
        if (y == C(0)) return static_cast<C>(__builtin_nanf(""));
        C r = std::is_same<C, float>::value ? fmodf(x, y) : fmod(x, y);
        if ((r > 0 && y < 0) || (r < 0 && y > 0)) return y + r;
        return r;
    }
}

// op: hipcx_binary_op; kind 0: array op array, 1: array op scalar, 2: scalar op array
template <typename T, int OP, int KIND>
struct BinaryCodeOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = KIND == 0 ? 2 : 1;
    static constexpr bool kNeedsIndex = false;
    compute_t<T> scalar;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> a, compute_t<T> b, compute_t<T>, compute_t<T>, int64_t) const {
        using C = compute_t<T>;
        const C x = KIND == 2 ? scalar : a;
        const C y = KIND == 0 ? b : (KIND == 1 ? scalar : a);
        if constexpr (OP == HIPCX_BINARY_FLOOR_DIVIDE) {
            return FloorDivideOf<C>(x, y);
        } else if constexpr (OP == HIPCX_BINARY_MOD) {
            return ModOf<C>(x, y);
        } else if constexpr (std::is_integral<C>::value) {
            if constexpr (OP == HIPCX_BINARY_BITWISE_AND) return static_cast<C>(x & y);
            if constexpr (OP == HIPCX_BINARY_BITWISE_OR) return static_cast<C>(x | y);
            if constexpr (OP == HIPCX_BINARY_BITWISE_XOR) return static_cast<C>(x ^ y);
            // shifts run in the promoted type (int for the narrow types), as `x1 << x2` does in C++; counts outside
            // [0, width) are undefined there and masked here
            using W = std::conditional_t<sizeof(C) == 8, int64_t, int32_t>;
            using UW = std::make_unsigned_t<W>;
            const int cnt = static_cast<int>(y) & (sizeof(W) * 8 - 1);
            if constexpr (OP == HIPCX_BINARY_LEFT_SHIFT) return static_cast<C>(static_cast<UW>(static_cast<W>(x)) << cnt);
            if constexpr (OP == HIPCX_BINARY_RIGHT_SHIFT) return static_cast<C>(static_cast<W>(x) >> cnt);
        } else {
            return x;  // bitwise ops and shifts on floats are rejected on the host
        }
    }
};

// Where: out = condition ? x : y (CX/native/native_device/indexing.cc:173-236); x and/or y may be scalars.
// kind 0: AAA, 1: AAS (y scalar), 2: ASA (x scalar), 3: ASS.
template <typename T, int KIND>
struct WhereOp {
    using In0 = bool;
    using In = T;
    using Out = T;
    static constexpr int kNumIn = KIND == 0 ? 3 : (KIND == 3 ? 1 : 2);
    static constexpr bool kNeedsIndex = false;
    compute_t<T> xs, ys;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T> c, compute_t<T> p, compute_t<T> q, compute_t<T>, int64_t) const {
        const bool cond = c != compute_t<T>(0);
        if constexpr (KIND == 0) return cond ? p : q;
        if constexpr (KIND == 1) return cond ? p : ys;
        if constexpr (KIND == 2) return cond ? xs : p;
        if constexpr (KIND == 3) return cond ? xs : ys;
    }
};

template <template <typename, int> class OpT, int OP, typename Visit>
void RunUnaryOp(const hipcx_array* x, const hipcx_array* out, void* stream, Visit visit) {
    EwPlan p = MakeEwPlan({out, x});
    visit(x->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        LaunchElementwise(p, OpT<T, OP>{}, AsStream(stream));
    });
}

}  // namespace
}  // namespace hipcx

namespace hipcx {
namespace {
void CheckBinaryDtype(int op, int dtype) {
    switch (op) {
        case HIPCX_BINARY_FLOOR_DIVIDE:
        case HIPCX_BINARY_MOD:
            HIPCX_REQUIRE(dtype != HIPCX_BOOL, HIPCX_DTYPE_ERROR, "bool dtype is not supported by this kernel");
            break;
        case HIPCX_BINARY_BITWISE_AND:
        case HIPCX_BINARY_BITWISE_OR:
        case HIPCX_BINARY_BITWISE_XOR:
            HIPCX_REQUIRE(!IsFloatDtype(dtype), HIPCX_DTYPE_ERROR, "Bitwise operations don't support Float types");
            break;
        case HIPCX_BINARY_LEFT_SHIFT:
        case HIPCX_BINARY_RIGHT_SHIFT:
            HIPCX_REQUIRE(!IsFloatDtype(dtype) && dtype != HIPCX_BOOL, HIPCX_DTYPE_ERROR, "Shift operations don't support Float or Bool types");
            break;
        default: throw Error(HIPCX_CHAINERX_ERROR, "unknown binary op code " + std::to_string(op));
    }
}

template <int KIND>
void RunBinaryCode(int op, const EwPlan& p, int dtype, const hipcx_scalar* scalar, hipStream_t stream) {
    CheckBinaryDtype(op, dtype);
    VisitDtype(dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        auto launch = [&](auto opc) {
            BinaryCodeOp<T, decltype(opc)::value, KIND> f;
            f.scalar = scalar != nullptr ? static_cast<compute_t<T>>(ScalarTo<T>(*scalar)) : compute_t<T>{};
            LaunchElementwise(p, f, stream);
        };
        switch (op) {
            case HIPCX_BINARY_FLOOR_DIVIDE: launch(std::integral_constant<int, HIPCX_BINARY_FLOOR_DIVIDE>{}); break;
            case HIPCX_BINARY_MOD: launch(std::integral_constant<int, HIPCX_BINARY_MOD>{}); break;
            case HIPCX_BINARY_BITWISE_AND: launch(std::integral_constant<int, HIPCX_BINARY_BITWISE_AND>{}); break;
            case HIPCX_BINARY_BITWISE_OR: launch(std::integral_constant<int, HIPCX_BINARY_BITWISE_OR>{}); break;
            case HIPCX_BINARY_BITWISE_XOR: launch(std::integral_constant<int, HIPCX_BINARY_BITWISE_XOR>{}); break;
            case HIPCX_BINARY_LEFT_SHIFT: launch(std::integral_constant<int, HIPCX_BINARY_LEFT_SHIFT>{}); break;
            default: launch(std::integral_constant<int, HIPCX_BINARY_RIGHT_SHIFT>{}); break;
        }
    });
}
}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_unary(int op, const hipcx_array* x, const hipcx_array* out, void* stream) {
    return Guard([&] {
        ValidateArray(x, "x");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x dtype differs from out dtype (cast with hipcx_copy first)");
        auto vf = [](int dt, auto&& f) { VisitFloatDtype(dt, f); };
        auto vn = [](int dt, auto&& f) { VisitNumericDtype(dt, f); };
#define HIPCX_FLOAT_CASE(code) \
    case code: RunUnaryOp<FloatUnaryOp, code>(x, out, stream, vf); break;
#define HIPCX_NUMERIC_CASE(code) \
    case code: RunUnaryOp<NumericUnaryOp, code>(x, out, stream, vn); break;
        switch (op) {
            HIPCX_FLOAT_CASE(HIPCX_UNARY_ERF)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_EXPM1)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_EXP2)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_LOG10)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_LOG2)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_LOG1P)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_SINH)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_COSH)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_ARCSINH)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_ARCCOSH)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_SIN)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_COS)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_TAN)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_ARCSIN)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_ARCCOS)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_ARCTAN)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_CEIL)
            HIPCX_FLOAT_CASE(HIPCX_UNARY_FLOOR)
            HIPCX_NUMERIC_CASE(HIPCX_UNARY_SQUARE)
            HIPCX_NUMERIC_CASE(HIPCX_UNARY_ABS)
            HIPCX_NUMERIC_CASE(HIPCX_UNARY_SIGN)
            default: throw Error(HIPCX_CHAINERX_ERROR, "hipcx_unary: unknown op code " + std::to_string(op));
        }
#undef HIPCX_FLOAT_CASE
#undef HIPCX_NUMERIC_CASE
    });
}

int hipcx_predicate(int op, const hipcx_array* x, const hipcx_array* out, void* stream) {
    return Guard([&] {
        ValidateArray(x, "x");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(out->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "predicate output must be bool");
        auto va = [](int dt, auto&& f) { VisitDtype(dt, f); };
        switch (op) {
            case HIPCX_PRED_LOGICAL_NOT: RunUnaryOp<PredicateOp, HIPCX_PRED_LOGICAL_NOT>(x, out, stream, va); break;
            case HIPCX_PRED_ISNAN: RunUnaryOp<PredicateOp, HIPCX_PRED_ISNAN>(x, out, stream, va); break;
            case HIPCX_PRED_ISINF: RunUnaryOp<PredicateOp, HIPCX_PRED_ISINF>(x, out, stream, va); break;
            case HIPCX_PRED_ISFINITE: RunUnaryOp<PredicateOp, HIPCX_PRED_ISFINITE>(x, out, stream, va); break;
            default: throw Error(HIPCX_CHAINERX_ERROR, "hipcx_predicate: unknown op code " + std::to_string(op));
        }
    });
}

int hipcx_logical(int op, const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1, x2});
        HIPCX_REQUIRE(out->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "logical output must be bool");
        HIPCX_REQUIRE(x1->dtype == x2->dtype, HIPCX_DTYPE_ERROR, "logical operands must share a dtype (cast with hipcx_copy first)");
        VisitDtype(x1->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            switch (op) {
                case HIPCX_LOGICAL_AND: LaunchElementwise(p, LogicalOp<T, HIPCX_LOGICAL_AND>{}, AsStream(stream)); break;
                case HIPCX_LOGICAL_OR: LaunchElementwise(p, LogicalOp<T, HIPCX_LOGICAL_OR>{}, AsStream(stream)); break;
                case HIPCX_LOGICAL_XOR: LaunchElementwise(p, LogicalOp<T, HIPCX_LOGICAL_XOR>{}, AsStream(stream)); break;
                default: throw Error(HIPCX_CHAINERX_ERROR, "hipcx_logical: unknown op code " + std::to_string(op));
            }
        });
    });
}

int hipcx_power(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1, x2});
        HIPCX_REQUIRE(x1->dtype == out->dtype && x2->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                      "operand dtype differs from out dtype (cast with hipcx_copy first)");
        VisitNumericDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            LaunchElementwise(p, PowerOp<T, 0>{}, AsStream(stream));
        });
    });
}

int hipcx_power_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1});
        HIPCX_REQUIRE(x1->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x1 dtype differs from out dtype (cast with hipcx_copy first)");
        VisitNumericDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            PowerOp<T, 1> op;
            op.scalar = static_cast<compute_t<T>>(ScalarTo<T>(x2));
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

int hipcx_power_sa(hipcx_scalar x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x2});
        HIPCX_REQUIRE(x2->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x2 dtype differs from out dtype (cast with hipcx_copy first)");
        VisitNumericDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            PowerOp<T, 2> op;
            op.scalar = static_cast<compute_t<T>>(ScalarTo<T>(x1));
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

int hipcx_binary(int op, const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1, x2});
        HIPCX_REQUIRE(x1->dtype == out->dtype && x2->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                      "operand dtype differs from out dtype (cast with hipcx_copy first)");
        RunBinaryCode<0>(op, p, out->dtype, nullptr, AsStream(stream));
    });
}

int hipcx_binary_as(int op, const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1});
        HIPCX_REQUIRE(x1->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x1 dtype differs from out dtype (cast with hipcx_copy first)");
        RunBinaryCode<1>(op, p, out->dtype, &x2, AsStream(stream));
    });
}

int hipcx_binary_sa(int op, hipcx_scalar x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x2});
        HIPCX_REQUIRE(x2->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x2 dtype differs from out dtype (cast with hipcx_copy first)");
        RunBinaryCode<2>(op, p, out->dtype, &x1, AsStream(stream));
    });
}

int hipcx_fmod(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1, x2});
        HIPCX_REQUIRE(x1->dtype == out->dtype && x2->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                      "operand dtype differs from out dtype (cast with hipcx_copy first)");
        VisitFloatDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            LaunchElementwise(p, FloatBinaryOp<T, false>{}, AsStream(stream));
        });
    });
}

int hipcx_arctan2(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, x1, x2});
        HIPCX_REQUIRE(x1->dtype == out->dtype && x2->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                      "operand dtype differs from out dtype (cast with hipcx_copy first)");
        VisitFloatDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            LaunchElementwise(p, FloatBinaryOp<T, true>{}, AsStream(stream));
        });
    });
}

int hipcx_where(const hipcx_array* condition, const hipcx_array* x, const hipcx_array* y, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, condition, x, y});
        HIPCX_REQUIRE(condition->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "where: condition must be bool");
        HIPCX_REQUIRE(x->dtype == out->dtype && y->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                      "operand dtype differs from out dtype (cast with hipcx_copy first)");
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            LaunchElementwise(p, WhereOp<T, 0>{}, AsStream(stream));
        });
    });
}

int hipcx_where_aas(const hipcx_array* condition, const hipcx_array* x, hipcx_scalar y, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, condition, x});
        HIPCX_REQUIRE(condition->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "where: condition must be bool");
        HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR, "x dtype differs from out dtype (cast with hipcx_copy first)");
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            WhereOp<T, 1> op;
            op.xs = compute_t<T>{};
            op.ys = static_cast<compute_t<T>>(ScalarTo<T>(y));
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

int hipcx_where_asa(const hipcx_array* condition, hipcx_scalar x, const hipcx_array* y, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, condition, y});
        HIPCX_REQUIRE(condition->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "where: condition must be bool");
        HIPCX_REQUIRE(y->dtype == out->dtype, HIPCX_DTYPE_ERROR, "y dtype differs from out dtype (cast with hipcx_copy first)");
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            WhereOp<T, 2> op;
            op.xs = static_cast<compute_t<T>>(ScalarTo<T>(x));
            op.ys = compute_t<T>{};
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

int hipcx_where_ass(const hipcx_array* condition, hipcx_scalar x, hipcx_scalar y, const hipcx_array* out, void* stream) {
    return Guard([&] {
        EwPlan p = MakeEwPlan({out, condition});
        HIPCX_REQUIRE(condition->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "where: condition must be bool");
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            WhereOp<T, 3> op;
            op.xs = static_cast<compute_t<T>>(ScalarTo<T>(x));
            op.ys = static_cast<compute_t<T>>(ScalarTo<T>(y));
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

}  // extern "C"
