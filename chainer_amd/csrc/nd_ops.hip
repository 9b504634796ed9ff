// Convolution and pooling over any number of spatial axes (ConvKernel CX/kernels/connection.h:14-32, MaxPoolKernel / AveragePoolKernel
// CX/kernels/pooling.h:20-64): the correctness path for what is not 2-D.  The native backend handles every rank with one algorithm,
// Im2Col over n axes followed by TensorDot (conv.cc:52-89) or by a reduction over the kernel axes (pool.cc:68-95, 191-250); the
// dedicated kernels of this library are 2-D and floating point.  Here
//   * 0 and 1 spatial axes are 2-D problems with extents of one and run through the 2-D entry points (same kernels, same results);
//   * 3 and more spatial axes, and convolutions of the integer dtypes and bool over any number of axes (the native backend
//     multiplies those like any other dtype, in the array dtype: arithmetic modulo 2^bits, which no order changes), run the plain
//     kernels below: one thread per output element, a loop over the window (and the input
//     channels).  They follow the reference's arithmetic -- float accumulation for float16, the bias added after the sum was rounded
//     to the array dtype, max pooling that keeps a NaN once it met one and pads with the lowest value, average pooling that rounds
//     the window sum to the array dtype before the division -- and make no attempt at speed.
#include "common.h"

extern "C" {
size_t hipcx_conv_workspace_size(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out);
int hipcx_conv(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad, int cover_all,
               const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream);
int hipcx_max_pool(const hipcx_array* x, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int cover_all,
                   const hipcx_array* out, void* stream);
int hipcx_average_pool(const hipcx_array* x, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int pad_mode,
                       const hipcx_array* out, void* stream);
}

namespace hipcx {

constexpr int kMaxSpatial = HIPCX_MAX_NDIM - 2;

struct NdArgs {
    const void* x;
    const void* w;  // convolution
    const void* b;  // convolution, may be null
    void* out;
    int n;           // spatial axes
    int64_t N, C, K;  // batch, input channels, output channels (pooling: K == C)
    int64_t in[kMaxSpatial], od[kMaxSpatial], k[kMaxSpatial], s[kMaxSpatial], p[kMaxSpatial];
    int64_t xs[kMaxSpatial + 2], ws[kMaxSpatial + 2], os[kMaxSpatial + 2];  // element strides: batch, channel, spatial...
    int64_t b_stride;
    int64_t window;  // product of k
    int pad_mode;
};

namespace {

template <typename T>
__device__ __forceinline__ T LowestNd() {
    if constexpr (std::is_same<T, half_t>::value) {
        return static_cast<half_t>(-__builtin_huge_valf());
    } else if constexpr (std::is_floating_point<T>::value) {
        return -__builtin_huge_val();
    } else if constexpr (std::is_same<T, bool>::value) {
        return false;
    } else {
        return std::numeric_limits<T>::lowest();
    }
}

// Splits a flat output index into (batch, channel, o[]) and returns the output's element offset.
__device__ __forceinline__ int64_t DecodeOutput(const NdArgs& p, int64_t idx, int64_t& n, int64_t& c, int64_t* o) {
    int64_t off = 0;
    for (int d = p.n - 1; d >= 0; --d) {
        o[d] = idx % p.od[d];
        idx /= p.od[d];
        off += o[d] * p.os[d + 2];
    }
    c = idx % p.K;
    n = idx / p.K;
    return off + n * p.os[0] + c * p.os[1];
}

// Accumulator of the convolution: float for float16, an unsigned type at least as wide for integers (sums modulo 2^bits without
// signed overflow, truncated on store), 32 bits for bool (a count of products that cannot wrap, stored as "any").
template <typename T>
struct NdAcc {
    using type = compute_t<T>;
};
template <> struct NdAcc<bool> { using type = uint32_t; };
template <> struct NdAcc<int8_t> { using type = uint32_t; };
template <> struct NdAcc<uint8_t> { using type = uint32_t; };
template <> struct NdAcc<int16_t> { using type = uint32_t; };
template <> struct NdAcc<int32_t> { using type = uint32_t; };
template <> struct NdAcc<int64_t> { using type = uint64_t; };

template <typename T>
__global__ __launch_bounds__(256) void ConvNdKernel(NdArgs p, int64_t total) {
    using A = typename NdAcc<T>::type;
    const T* x = static_cast<const T*>(p.x);
    const T* w = static_cast<const T*>(p.w);
    T* out = static_cast<T*>(p.out);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t n, kch, o[kMaxSpatial];
        const int64_t ooff = DecodeOutput(p, idx, n, kch, o);
        A acc = A(0);
        for (int64_t c = 0; c < p.C; ++c) {
            const T* xc = x + n * p.xs[0] + c * p.xs[1];
            const T* wc = w + kch * p.ws[0] + c * p.ws[1];
            for (int64_t j = 0; j < p.window; ++j) {  // kernel positions in C order
                int64_t rest = j, xoff = 0, woff = 0;
                bool inside = true;
                for (int d = p.n - 1; d >= 0; --d) {
                    const int64_t kd = rest % p.k[d];
                    rest /= p.k[d];
                    const int64_t i = o[d] * p.s[d] - p.p[d] + kd;
                    inside = inside && i >= 0 && i < p.in[d];
                    xoff += i * p.xs[d + 2];
                    woff += kd * p.ws[d + 2];
                }
                if (inside) acc += static_cast<A>(xc[xoff]) * static_cast<A>(wc[woff]);
            }
        }
        T y = static_cast<T>(acc);  // TensorDot hands out the array dtype ...
        if (p.b != nullptr) y = static_cast<T>(static_cast<A>(y) + static_cast<A>(static_cast<const T*>(p.b)[kch * p.b_stride]));  // ... then the bias is added
        out[ooff] = y;
    }
}

template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void PoolNdKernel(NdArgs p, int64_t total) {
    using A = compute_t<T>;
    const T* x = static_cast<const T*>(p.x);
    T* out = static_cast<T*>(p.out);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t n, c, o[kMaxSpatial];
        const int64_t ooff = DecodeOutput(p, idx, n, c, o);
        const T* xc = x + n * p.xs[0] + c * p.xs[1];
        T best = LowestNd<T>();
        A sum = A(0);
        // the divisor of the 'ignore' mode: the product of the per-axis overlaps min(start + k, extent) - max(start, 0), not clamped
        // at zero (a window wholly outside an axis contributes a negative factor, CX/native/native_device/pool.cc:197-225)
        int64_t valid = 1;
        for (int d = 0; d < p.n; ++d) {
            const int64_t lo = o[d] * p.s[d] - p.p[d];
            const int64_t a = lo < 0 ? 0 : lo, e = lo + p.k[d] < p.in[d] ? lo + p.k[d] : p.in[d];
            valid *= e - a;
        }
        for (int64_t j = 0; j < p.window; ++j) {
            int64_t rest = j, xoff = 0;
            bool inside = true;
            for (int d = p.n - 1; d >= 0; --d) {
                const int64_t kd = rest % p.k[d];
                rest /= p.k[d];
                const int64_t i = o[d] * p.s[d] - p.p[d] + kd;
                inside = inside && i >= 0 && i < p.in[d];
                xoff += i * p.xs[d + 2];
            }
            if (!inside) continue;  // padding: the lowest value for max, zero for the sum
            const T v = xc[xoff];
            if constexpr (IS_MAX) {
                if (v != v || best < v) best = v;  // a NaN is taken and then kept (comparisons with it are false)
            } else {
                sum += static_cast<A>(v);
            }
        }
        if constexpr (IS_MAX) {
            out[ooff] = best;
        } else {
            // the window sum is an array of the input dtype before it is divided (CX/native/native_device/pool.cc:191-250)
            const T s = static_cast<T>(sum);
            const A div = static_cast<A>(static_cast<T>(static_cast<A>(p.pad_mode == HIPCX_PAD_ZERO ? p.window : valid)));
            out[ooff] = static_cast<T>(static_cast<A>(s) / div);
        }
    }
}

int64_t ElemStrideNd(const hipcx_array* a, int axis) {
    const int64_t it = ItemSize(a->dtype);
    HIPCX_REQUIRE(a->strides[axis] % it == 0, HIPCX_NOT_IMPLEMENTED_ERROR, "byte strides must be multiples of the item size");
    return a->strides[axis] / it;
}

// Validates shapes as the routine does (CX/routines/connection.cc:140-208, pooling.cc:52-169) and fills the geometry.
NdArgs MakeNdArgs(const hipcx_array* x, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all, const hipcx_array* out,
                  int64_t out_channels, const char* what) {
    ValidateArray(x, "x");
    ValidateArray(out, "out");
    HIPCX_REQUIRE(x->ndim >= 2 && out->ndim == x->ndim, HIPCX_DIMENSION_ERROR, std::string(what) + ": x and out need a batch axis, a channel axis and the same rank");
    HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR, std::string(what) + ": out must have x's dtype");
    const int n = x->ndim - 2;
    HIPCX_REQUIRE(n == 0 || (ksize && stride && pad), HIPCX_CHAINERX_ERROR, "null window parameters");
    NdArgs p{};
    p.x = x->data, p.out = out->data;
    p.n = n;
    p.N = x->shape[0], p.C = x->shape[1], p.K = out_channels;
    HIPCX_REQUIRE(out->shape[0] == p.N && out->shape[1] == p.K, HIPCX_DIMENSION_ERROR, std::string(what) + ": out has the wrong shape " + ShapeStr(out));
    p.window = 1;
    for (int d = 0; d < n; ++d) {
        HIPCX_REQUIRE(ksize[d] > 0 && stride[d] > 0 && pad[d] >= 0, HIPCX_DIMENSION_ERROR, "invalid kernel size, stride or pad");
        p.in[d] = x->shape[d + 2], p.k[d] = ksize[d], p.s[d] = stride[d], p.p[d] = pad[d];
        p.od[d] = hipcx_conv_out_dim(p.in[d], p.k[d], p.s[d], p.p[d], cover_all);
        HIPCX_REQUIRE(p.od[d] > 0, HIPCX_DIMENSION_ERROR, "Output size should be positive.");
        HIPCX_REQUIRE(out->shape[d + 2] == p.od[d], HIPCX_DIMENSION_ERROR, std::string(what) + ": out has the wrong shape " + ShapeStr(out));
        p.window *= p.k[d];
    }
    for (int d = 0; d < x->ndim; ++d) {
        p.xs[d] = ElemStrideNd(x, d);
        p.os[d] = ElemStrideNd(out, d);
    }
    p.pad_mode = HIPCX_PAD_ZERO;
    return p;
}

unsigned NdBlocks(int64_t total) {
    int64_t b = (total + 255) / 256;
    const int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
    return static_cast<unsigned>(b > cap ? cap : (b < 1 ? 1 : b));
}

// x [N, C, (W)] as [N, C, 1, W or 1]: an axis of extent one gets the stride a dense array would give it.
hipcx_array AsFourAxes(const hipcx_array* a) {
    hipcx_array r = *a;
    const int64_t it = ItemSize(a->dtype);
    r.ndim = 4;
    if (a->ndim == 2) {
        r.shape[2] = r.shape[3] = 1;
        r.strides[2] = r.strides[3] = it;
    } else {  // 3 axes
        r.shape[3] = a->shape[2], r.strides[3] = a->strides[2];
        r.shape[2] = 1, r.strides[2] = a->strides[2] * a->shape[2];
    }
    return r;
}

void FourAxisWindow(int n, const int64_t* v, int64_t fill, int64_t* out) {
    out[0] = fill;
    out[1] = n == 1 ? v[0] : fill;
}

}  // namespace

// ---- what conv.hip and pool.hip call for arrays that do not have two spatial axes ----
size_t ConvNdWorkspaceSize(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out) {
    if (x->ndim > 3 || w->ndim != x->ndim || out == nullptr || out->ndim != x->ndim) return 0;
    hipcx_array x4 = AsFourAxes(x), w4 = AsFourAxes(w), o4 = AsFourAxes(out);
    return hipcx_conv_workspace_size(&x4, &w4, &o4);
}

void ConvNd(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad, int cover_all,
            const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream) {
    ValidateArray(x, "x");
    ValidateArray(w, "w");
    ValidateArray(out, "out");
    HIPCX_REQUIRE(x->ndim >= 2 && w->ndim == x->ndim && out->ndim == x->ndim, HIPCX_DIMENSION_ERROR,
                  "conv: x, w and out need the same rank, at least 2 (batch / output channels and input channels)");
    HIPCX_REQUIRE(x->dtype == out->dtype && w->dtype == out->dtype && (b == nullptr || b->dtype == out->dtype), HIPCX_DTYPE_ERROR,
                  "conv: x, w and b must have out's dtype (cast with hipcx_copy first)");
    HIPCX_REQUIRE(w->shape[1] == x->shape[1], HIPCX_DIMENSION_ERROR, "Mismatched number of input channels in input and weights.");
    if (b != nullptr) {
        ValidateArray(b, "b");
        HIPCX_REQUIRE(b->ndim == 1 && b->shape[0] == w->shape[0], HIPCX_DIMENSION_ERROR, "Mismatched bias shape for weights.");
    }
    const int n = x->ndim - 2;
    if (n <= 1 && IsFloatDtype(out->dtype)) {
        hipcx_array x4 = AsFourAxes(x), w4 = AsFourAxes(w), o4 = AsFourAxes(out);
        int64_t s4[2], p4[2];
        FourAxisWindow(n, stride, 1, s4);
        FourAxisWindow(n, pad, 0, p4);
        int rc = hipcx_conv(&x4, &w4, b, s4, p4, cover_all, &o4, workspace, workspace_bytes, stream);
        HIPCX_REQUIRE(rc == HIPCX_OK, rc, hipcx_last_error());
        return;
    }
    int64_t ksize[kMaxSpatial];
    for (int d = 0; d < n; ++d) ksize[d] = w->shape[d + 2];
    NdArgs p = MakeNdArgs(x, ksize, stride, pad, cover_all, out, w->shape[0], "conv");
    p.w = w->data;
    for (int d = 0; d < w->ndim; ++d) p.ws[d] = ElemStrideNd(w, d);
    if (b != nullptr) {
        p.b = b->data;
        p.b_stride = ElemStrideNd(b, 0);
    }
    const int64_t total = TotalSize(out);
    if (total == 0) return;
    VisitDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        hipLaunchKernelGGL((ConvNdKernel<T>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
    });
    CheckLaunch("conv over n axes");
}

void PoolNd(bool is_max, const hipcx_array* x, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all, int pad_mode,
            const hipcx_array* out, void* stream) {
    ValidateArray(x, "x");
    HIPCX_REQUIRE(x->ndim >= 3, HIPCX_DIMENSION_ERROR, "pooling needs at least one spatial axis");
    const int n = x->ndim - 2;
    if (n == 1) {
        ValidateArray(out, "out");
        HIPCX_REQUIRE(out->ndim == 3, HIPCX_DIMENSION_ERROR, "out has the wrong rank");
        hipcx_array x4 = AsFourAxes(x), o4 = AsFourAxes(out);
        int64_t k4[2], s4[2], p4[2];
        FourAxisWindow(n, ksize, 1, k4);
        FourAxisWindow(n, stride, 1, s4);
        FourAxisWindow(n, pad, 0, p4);
        int rc = is_max ? hipcx_max_pool(&x4, k4, s4, p4, cover_all, &o4, stream) : hipcx_average_pool(&x4, k4, s4, p4, pad_mode, &o4, stream);
        HIPCX_REQUIRE(rc == HIPCX_OK, rc, hipcx_last_error());
        return;
    }
    NdArgs p = MakeNdArgs(x, ksize, stride, pad, cover_all, out, x->shape[1], is_max ? "max_pool" : "average_pool");
    p.pad_mode = pad_mode;
    const int64_t total = TotalSize(out);
    if (total == 0) return;
    if (is_max) {
        VisitDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL((PoolNdKernel<T, true>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
        });
    } else {
        VisitFloatDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL((PoolNdKernel<T, false>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
        });
    }
    CheckLaunch("pooling over n axes");
}

}  // namespace hipcx
