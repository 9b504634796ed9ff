// Creation kernels Identity / Eye / Tri / Linspace / Diagflat (CX/native/native_device/fill.cc) and Cumsum
// (CX/native/native_device/reduction.cc:121-144 over native::Scan, CX/native/reduce.h:98-113).
#include "elementwise.h"

namespace hipcx {
namespace {

// out[i] over the C-order index i of a dense [n, m] output.
//   Identity: i % (n + 1) == 0                                 (fill.cc NativeIdentityKernel)
//   Eye:      start <= i < stop && (i - start) % (m + 1) == 0   with start = k < 0 ? -k*m : k, stop = m*(m - k)
//   Tri:      col <= row + k
template <typename T, int KIND>
struct PatternOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 0;
    static constexpr bool kNeedsIndex = true;
    int64_t m, start, stop, step, k;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T>, compute_t<T>, compute_t<T>, compute_t<T>, int64_t i) const {
        bool one;
        if constexpr (KIND == 0) {
            one = i % step == 0;
        } else if constexpr (KIND == 1) {
            one = start <= i && i < stop && (i - start) % step == 0;
        } else {
            one = (i % m) <= (i / m) + k;
        }
        return one ? compute_t<T>(1) : compute_t<T>(0);
    }
};

// Linspace: value = n == 1 ? start : (start*(n-1-i) + stop*i) / (n-1) in double, then cast (fill.cc NativeLinspaceKernel).
template <typename T>
struct LinspaceOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 0;
    static constexpr bool kNeedsIndex = true;
    int64_t n;
    double start, stop;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T>, compute_t<T>, compute_t<T>, compute_t<T>, int64_t i) const {
        double value = n == 1 ? start : (start * static_cast<double>(n - 1 - i) + stop * static_cast<double>(i)) / static_cast<double>(n - 1);
        if constexpr (std::is_same<T, bool>::value) {
            return value != 0.0;
        } else {
            return static_cast<compute_t<T>>(value);
        }
    }
};

template <typename T>
__global__ __launch_bounds__(256) void DiagflatKernel(const char* v, int64_t v_stride, int64_t nv, T* out, int64_t n, int64_t row_start,
                                                      int64_t col_start) {
    int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n * n) return;
    int64_t row = i / n, col = i - row * n;
    int64_t j = row - row_start;
    T val = T(0);
    if (j >= 0 && j < nv && col - col_start == j) val = *reinterpret_cast<const T*>(v + j * v_stride);
    out[i] = val;
}

// Cumsum: one thread per line walks the scanned axis serially -- the reference's own order, so float results are
// bit-identical to the native backend.  Consecutive threads take consecutive positions of the innermost remaining axis.
struct ScanArgs {
    const char* in;
    char* out;
    int n_outer;
    int64_t shape[HIPCX_MAX_NDIM];
    int64_t in_strides[HIPCX_MAX_NDIM];
    int64_t out_strides[HIPCX_MAX_NDIM];
    int64_t lines;
    int64_t len, in_axis_stride, out_axis_stride;
};

template <typename In, typename Out>
__global__ __launch_bounds__(256) void CumsumKernel(ScanArgs s) {
    using Acc = std::conditional_t<std::is_same<Out, half_t>::value, float, Out>;
    int64_t line = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (line >= s.lines) return;
    int64_t in_off = 0, out_off = 0, r = line;
    for (int d = s.n_outer - 1; d >= 0; --d) {
        int64_t q = r / s.shape[d];
        int64_t c = r - q * s.shape[d];
        r = q;
        in_off += c * s.in_strides[d];
        out_off += c * s.out_strides[d];
    }
    Acc acc = Acc(0);
    for (int64_t j = 0; j < s.len; ++j) {
        In v = *reinterpret_cast<const In*>(s.in + in_off + j * s.in_axis_stride);
        if constexpr (std::is_same<In, half_t>::value) {
            acc += static_cast<Acc>(static_cast<float>(v));
        } else {
            acc += static_cast<Acc>(v);
        }
        *reinterpret_cast<Out*>(s.out + out_off + j * s.out_axis_stride) = static_cast<Out>(acc);
    }
}

void RequireDense2D(const hipcx_array* out, const char* what) {
    ValidateArray(out, "out");
    HIPCX_REQUIRE(out->ndim == 2, HIPCX_DIMENSION_ERROR, std::string(what) + ": out must be 2-dimensional");
    HIPCX_REQUIRE(IsContiguous(out), HIPCX_NOT_IMPLEMENTED_ERROR, std::string(what) + ": out must be C-contiguous");
}

template <int KIND>
void RunPattern(const hipcx_array* out, int64_t m, int64_t start, int64_t stop, int64_t step, int64_t k, void* stream) {
    EwPlan p = MakeEwPlan({out});
    VisitDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        PatternOp<T, KIND> op;
        op.m = m, op.start = start, op.stop = stop, op.step = step, op.k = k;
        LaunchElementwise(p, op, AsStream(stream));
    });
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_identity(const hipcx_array* out, void* stream) {
    return Guard([&] {
        RequireDense2D(out, "identity");
        HIPCX_REQUIRE(out->shape[0] == out->shape[1], HIPCX_DIMENSION_ERROR, "identity: out must be square");
        RunPattern<0>(out, out->shape[1], 0, 0, out->shape[0] + 1, 0, stream);
    });
}

int hipcx_eye(int64_t k, const hipcx_array* out, void* stream) {
    return Guard([&] {
        RequireDense2D(out, "eye");
        const int64_t m = out->shape[1];
        RunPattern<1>(out, m, k < 0 ? -k * m : k, m * (m - k), m + 1, k, stream);
    });
}

int hipcx_tri(int64_t k, const hipcx_array* out, void* stream) {
    return Guard([&] {
        RequireDense2D(out, "tri");
        if (TotalSize(out) == 0) return;
        RunPattern<2>(out, out->shape[1], 0, 0, 1, k, stream);
    });
}

int hipcx_linspace(double start, double stop, const hipcx_array* out, void* stream) {
    return Guard([&] {
        ValidateArray(out, "out");
        HIPCX_REQUIRE(out->ndim == 1 && out->shape[0] > 0, HIPCX_DIMENSION_ERROR, "linspace: out must be 1-dimensional and non-empty");
        EwPlan p = MakeEwPlan({out});
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            LinspaceOp<T> op;
            op.n = out->shape[0], op.start = start, op.stop = stop;
            LaunchElementwise(p, op, AsStream(stream));
        });
    });
}

int hipcx_diagflat(const hipcx_array* v, int64_t k, const hipcx_array* out, void* stream) {
    return Guard([&] {
        ValidateArray(v, "v");
        RequireDense2D(out, "diagflat");
        HIPCX_REQUIRE(v->ndim == 1, HIPCX_DIMENSION_ERROR, "diagflat: v must be 1-dimensional");
        HIPCX_REQUIRE(v->dtype == out->dtype, HIPCX_DTYPE_ERROR, "diagflat: v and out must share a dtype");
        const int64_t n = out->shape[0];
        const int64_t absk = k < 0 ? -k : k;
        HIPCX_REQUIRE(out->shape[1] == n && n == v->shape[0] + absk, HIPCX_DIMENSION_ERROR, "diagflat: out must be [len(v) + |k|]^2");
        if (n == 0) return;
        HIPCX_REQUIRE((n * n + 255) / 256 < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "diagflat: output too large for one launch");
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL(DiagflatKernel<T>, dim3(static_cast<unsigned>((n * n + 255) / 256)), dim3(256), 0, AsStream(stream),
                               static_cast<const char*>(v->data), v->strides[0], v->shape[0], static_cast<T*>(out->data), n, k >= 0 ? 0 : -k,
                               k >= 0 ? k : 0);
        });
        CheckLaunch("diagflat");
    });
}

int hipcx_cumsum(const hipcx_array* a, int8_t axis, const hipcx_array* out, void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(SameShape(a, out), HIPCX_DIMENSION_ERROR, "cumsum: out must have a's shape");
        HIPCX_REQUIRE(axis >= 0 && axis < a->ndim, HIPCX_DIMENSION_ERROR, "cumsum: axis out of range");
        if (TotalSize(out) == 0) return;
        ScanArgs s{};
        s.in = static_cast<const char*>(a->data);
        s.out = static_cast<char*>(out->data);
        s.lines = 1;
        for (int d = 0; d < a->ndim; ++d) {
            if (d == axis) continue;
            s.shape[s.n_outer] = a->shape[d];
            s.in_strides[s.n_outer] = a->strides[d];
            s.out_strides[s.n_outer] = out->strides[d];
            s.lines *= a->shape[d];
            ++s.n_outer;
        }
        s.len = a->shape[axis];
        s.in_axis_stride = a->strides[axis];
        s.out_axis_stride = out->strides[axis];
        HIPCX_REQUIRE((s.lines + 255) / 256 < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "cumsum: too many lines for one launch");
        dim3 grid(static_cast<unsigned>((s.lines + 255) / 256)), block(256);
        hipStream_t st = AsStream(stream);
        // Out dtypes the routine produces: the input's float dtype, int64 for bool / integer inputs (CX/routines/reduction.cc:115-127)
        VisitDtype(a->dtype, [&](auto in_tag) {
            using In = typename decltype(in_tag)::type;
            switch (out->dtype) {
                case HIPCX_INT64: hipLaunchKernelGGL((CumsumKernel<In, int64_t>), grid, block, 0, st, s); break;
                case HIPCX_FLOAT16: hipLaunchKernelGGL((CumsumKernel<In, half_t>), grid, block, 0, st, s); break;
                case HIPCX_FLOAT32: hipLaunchKernelGGL((CumsumKernel<In, float>), grid, block, 0, st, s); break;
                case HIPCX_FLOAT64: hipLaunchKernelGGL((CumsumKernel<In, double>), grid, block, 0, st, s); break;
                default: throw Error(HIPCX_NOT_IMPLEMENTED_ERROR, std::string("hip cumsum: unsupported output dtype ") + DtypeName(out->dtype));
            }
        });
        CheckLaunch("cumsum");
    });
}

}  // extern "C"
