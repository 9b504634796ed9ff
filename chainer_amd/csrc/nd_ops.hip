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
#include "window_argmax.h"

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

// ---- gradients over n spatial axes ----
// Plain kernels again, one thread per result element, written so that the results carry the bits of the native backend's compositions:
// a product over the input channels or over the output positions is one fused-multiply-add chain in the order of the native Dot's
// loop (CX/native/native_device/dot.cc:200-214; float accumulation for float16, rounded once), and what Col2Im adds up
// (CX/native/col2im.cc:76-122: one in-place Add per kernel offset, in C order, on a zeroed array) is added in that order with one
// rounding to the array dtype per addition.

template <typename A>
__device__ __forceinline__ A FusedMulAdd(A a, A b, A c) {
    if constexpr (std::is_same<A, float>::value) {
        return __builtin_fmaf(a, b, c);
    } else {
        return __builtin_fma(a, b, c);
    }
}

// Splits a flat index over [N][channels][dims...] (C order) and returns the element offset for strides st.
__device__ __forceinline__ int64_t DecodeNd(int n_axes, const int64_t* dims, int64_t channels, const int64_t* st, int64_t idx, int64_t& n,
                                            int64_t& c, int64_t* pos) {
    int64_t off = 0;
    for (int d = n_axes - 1; d >= 0; --d) {
        pos[d] = idx % dims[d];
        idx /= dims[d];
        off += pos[d] * st[d + 2];
    }
    c = idx % channels;
    n = idx / channels;
    return off + n * st[0] + c * st[1];
}

// The window position o (per axis) that covers input position i at kernel offset kd, or false: o * s - p + kd == i, 0 <= o < od.
__device__ __forceinline__ bool CoveringWindow(const NdArgs& p, const int64_t* i, int64_t j, int64_t* o) {
    bool ok = true;
    int64_t rest = j;
    for (int d = p.n - 1; d >= 0; --d) {
        const int64_t kd = rest % p.k[d];
        rest /= p.k[d];
        const int64_t t = i[d] + p.p[d] - kd;
        const int64_t q = t / p.s[d];
        ok = ok && t >= 0 && q * p.s[d] == t && q < p.od[d];
        o[d] = q;
    }
    return ok;
}

// ConvTranspose (CX/native/native_device/conv.cc:126-160): out [N, K, od...] from x [N, C, in...] and w [C, K, k...]; out position y
// receives, per kernel offset in C order, the product over the input channels at the input position i with i * s - p + kd == y.
template <typename T>
__global__ __launch_bounds__(256) void ConvTransposeNdKernel(NdArgs p, int64_t total) {
    using A = compute_t<T>;
    const T* x = static_cast<const T*>(p.x);
    const T* w = static_cast<const T*>(p.w);
    T* out = static_cast<T*>(p.out);
    NdArgs q = p;  // CoveringWindow speaks of windows over an image: here the image is `out` and the windows are x's positions
    for (int d = 0; d < p.n; ++d) q.od[d] = p.in[d];
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t n, kch, y[kMaxSpatial], i[kMaxSpatial];
        const int64_t ooff = DecodeNd(p.n, p.od, p.K, p.os, idx, n, kch, y);
        T acc = T(0);
        for (int64_t j = 0; j < p.window; ++j) {
            if (!CoveringWindow(q, y, j, i)) continue;
            int64_t xoff = n * p.xs[0], woff = kch * p.ws[1], rest = j;
            for (int d = p.n - 1; d >= 0; --d) {
                xoff += i[d] * p.xs[d + 2];
                woff += (rest % p.k[d]) * p.ws[d + 2];
                rest /= p.k[d];
            }
            A dot = A(0);
            for (int64_t c = 0; c < p.C; ++c) dot = FusedMulAdd(static_cast<A>(w[woff + c * p.ws[0]]), static_cast<A>(x[xoff + c * p.xs[1]]), dot);
            acc = static_cast<T>(static_cast<A>(acc) + static_cast<A>(static_cast<T>(dot)));
        }
        if (p.b != nullptr) acc = static_cast<T>(static_cast<A>(acc) + static_cast<A>(static_cast<const T*>(p.b)[kch * p.b_stride]));
        out[ooff] = acc;
    }
}

// ConvGradWeight (conv.cc:91-124): gw [K, C, k...] = sum over the batch and the output positions, in C order, of
// gy[n, k, o] * x[n, c, o * s - p + kd]; positions in the padding hold zeros that are multiplied like any other value.
// Here p.x = x, p.w = gy (strides ws, [N, K, od...]), p.out = gw (strides os, [K, C, k...]).
template <typename T>
__global__ __launch_bounds__(256) void ConvGradWeightNdKernel(NdArgs p, int64_t total, int64_t positions) {
    using A = compute_t<T>;
    const T* x = static_cast<const T*>(p.x);
    const T* gy = static_cast<const T*>(p.w);
    T* gw = static_cast<T*>(p.out);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t kd[kMaxSpatial];
        int64_t rest = idx, goff = 0;
        for (int d = p.n - 1; d >= 0; --d) {
            kd[d] = rest % p.k[d];
            rest /= p.k[d];
            goff += kd[d] * p.os[d + 2];
        }
        const int64_t c = rest % p.C, kch = rest / p.C;
        goff += kch * p.os[0] + c * p.os[1];
        A acc = A(0);
        for (int64_t n = 0; n < p.N; ++n) {
            for (int64_t e = 0; e < positions; ++e) {
                int64_t r2 = e, xoff = n * p.xs[0] + c * p.xs[1], yoff = n * p.ws[0] + kch * p.ws[1];
                bool inside = true;
                for (int d = p.n - 1; d >= 0; --d) {
                    const int64_t o = r2 % p.od[d];
                    r2 /= p.od[d];
                    const int64_t i = o * p.s[d] - p.p[d] + kd[d];
                    inside = inside && i >= 0 && i < p.in[d];
                    xoff += i * p.xs[d + 2];
                    yoff += o * p.ws[d + 2];
                }
                const A xv = inside ? static_cast<A>(x[xoff]) : A(0);
                acc = FusedMulAdd(static_cast<A>(gy[yoff]), xv, acc);
            }
        }
        gw[goff] = static_cast<T>(acc);
    }
}

// ArgMax of window o of plane xc in the native reduction order; positions in the padding hold the lowest value.
template <typename T>
__device__ int WindowArgMaxNd(const NdArgs& p, const T* xc, const int64_t* o) {
    using V = win_value_t<T>;
    return NativeOrderArgMax<V>(static_cast<int>(p.window), [&](int j) -> V {
        int64_t rest = j, xoff = 0;
        bool inside = true;
        for (int d = p.n - 1; d >= 0; --d) {
            const int64_t i = o[d] * p.s[d] - p.p[d] + rest % p.k[d];
            rest /= p.k[d];
            inside = inside && i >= 0 && i < p.in[d];
            xoff += i * p.xs[d + 2];
        }
        return static_cast<V>(inside ? xc[xoff] : LowestNd<T>());
    });
}

// MaxPoolGrad / AveragePoolGrad (CX/native/native_device/pool.cc:97-143, 304-346): gx [N, C, in...] gathers, per kernel offset in C
// order, the gradient of the window that covers it there -- for max pooling only when that offset is the window's ArgMax.
// p.x = x (max only), p.w = gout (strides ws, [N, C, od...]), p.out = gx (strides os).
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void PoolGradNdKernel(NdArgs p, int64_t total) {
    using A = compute_t<T>;
    const T* x = static_cast<const T*>(p.x);
    const T* gout = static_cast<const T*>(p.w);
    T* gx = static_cast<T*>(p.out);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t n, c, i[kMaxSpatial], o[kMaxSpatial];
        const int64_t doff = DecodeNd(p.n, p.in, p.C, p.os, idx, n, c, i);
        T acc = T(0);
        for (int64_t j = 0; j < p.window; ++j) {
            if (!CoveringWindow(p, i, j, o)) continue;
            int64_t goff = n * p.ws[0] + c * p.ws[1];
            for (int d = 0; d < p.n; ++d) goff += o[d] * p.ws[d + 2];
            if constexpr (IS_MAX) {
                if (WindowArgMaxNd<T>(p, x + n * p.xs[0] + c * p.xs[1], o) != j) continue;
                acc = static_cast<T>(static_cast<A>(acc) + static_cast<A>(gout[goff]));
            } else {
                T g = gout[goff];
                if (p.pad_mode == HIPCX_PAD_IGNORE) {  // divided by the window's width before it is spread (pool.cc:333-338)
                    int64_t valid = 1;
                    for (int d = 0; d < p.n; ++d) {
                        const int64_t lo = o[d] * p.s[d] - p.p[d];
                        const int64_t a = lo < 0 ? 0 : lo, e = lo + p.k[d] < p.in[d] ? lo + p.k[d] : p.in[d];
                        valid *= e - a;
                    }
                    g = static_cast<T>(static_cast<A>(g) / static_cast<A>(static_cast<T>(static_cast<A>(valid))));
                }
                acc = static_cast<T>(static_cast<A>(acc) + static_cast<A>(g));
            }
        }
        if constexpr (!IS_MAX) {
            if (p.pad_mode == HIPCX_PAD_ZERO) acc = static_cast<T>(static_cast<A>(acc) / static_cast<A>(static_cast<T>(static_cast<A>(p.window))));
        }
        gx[doff] = acc;
    }
}

// MaxPoolGradGrad (pool.cc:147-177): ggout [N, C, od...] = ggx at the ArgMax position of x's window; the lowest value when that
// position lies in the padding.  p.x = x, p.w = ggx (strides ws, [N, C, in...]), p.out = ggout (strides os).
template <typename T>
__global__ __launch_bounds__(256) void MaxPoolGradGradNdKernel(NdArgs p, int64_t total) {
    const T* x = static_cast<const T*>(p.x);
    const T* ggx = static_cast<const T*>(p.w);
    T* ggout = static_cast<T*>(p.out);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t n, c, o[kMaxSpatial];
        const int64_t ooff = DecodeNd(p.n, p.od, p.C, p.os, idx, n, c, o);
        int64_t rest = WindowArgMaxNd<T>(p, x + n * p.xs[0] + c * p.xs[1], o);
        int64_t goff = n * p.ws[0] + c * p.ws[1];
        bool inside = true;
        for (int d = p.n - 1; d >= 0; --d) {
            const int64_t i = o[d] * p.s[d] - p.p[d] + rest % p.k[d];
            rest /= p.k[d];
            inside = inside && i >= 0 && i < p.in[d];
            goff += i * p.ws[d + 2];
        }
        ggout[ooff] = inside ? ggx[goff] : LowestNd<T>();
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

// ---- gradients: what im2col.hip, conv_grad.hip and pool.hip call for arrays that do not have two spatial axes ----
namespace {

// Geometry shared by the gradient kernels: `image` [N, C, in...] is the array at the input end of the forward operation, `windows`
// [N, K, od...] the one at its output end; od must be what the forward operation gives for (in, k, s, p, cover_all) unless
// `free_extent` (ConvTranspose, whose caller chooses the image size among those consistent with the windows).
NdArgs MakeGradArgs(const hipcx_array* image, const hipcx_array* windows, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all,
                    bool free_extent, const char* what) {
    ValidateArray(image, "image-side array");
    ValidateArray(windows, "window-side array");
    HIPCX_REQUIRE(image->ndim >= 2 && windows->ndim == image->ndim, HIPCX_DIMENSION_ERROR, std::string(what) + ": arrays need a batch axis, a channel axis and the same rank");
    HIPCX_REQUIRE(image->dtype == windows->dtype, HIPCX_DTYPE_ERROR, std::string(what) + ": arrays must share one dtype");
    HIPCX_REQUIRE(image->shape[0] == windows->shape[0], HIPCX_DIMENSION_ERROR, std::string(what) + ": batch sizes differ");
    const int n = image->ndim - 2;
    HIPCX_REQUIRE(n == 0 || (ksize && stride && pad), HIPCX_CHAINERX_ERROR, "null window parameters");
    NdArgs p{};
    p.n = n;
    p.N = image->shape[0], p.C = image->shape[1], p.K = windows->shape[1];
    p.window = 1;
    for (int d = 0; d < n; ++d) {
        HIPCX_REQUIRE(ksize[d] > 0 && stride[d] > 0 && pad[d] >= 0, HIPCX_DIMENSION_ERROR, "invalid kernel size, stride or pad");
        p.in[d] = image->shape[d + 2], p.od[d] = windows->shape[d + 2], p.k[d] = ksize[d], p.s[d] = stride[d], p.p[d] = pad[d];
        if (free_extent) {
            // every window must land inside the padded image: (od - 1) * s + k <= in + 2 p + s - 1 (CX/native/col2im.cc:76-122)
            HIPCX_REQUIRE((p.od[d] - 1) * p.s[d] + p.k[d] <= p.in[d] + 2 * p.p[d] + p.s[d] - 1, HIPCX_DIMENSION_ERROR,
                          std::string(what) + ": output size is not consistent with the input size");
        } else {
            HIPCX_REQUIRE(hipcx_conv_out_dim(p.in[d], p.k[d], p.s[d], p.p[d], cover_all) == p.od[d], HIPCX_DIMENSION_ERROR,
                          std::string(what) + ": the window-side array has the wrong shape " + ShapeStr(windows));
        }
        p.window *= p.k[d];
    }
    HIPCX_REQUIRE(p.window < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "window too large");
    return p;
}

void CopyStrides(const hipcx_array* a, int64_t* st) {
    for (int d = 0; d < a->ndim; ++d) st[d] = ElemStrideNd(a, d);
}

}  // namespace

void ConvTransposeNd(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                     const hipcx_array* out, void* stream) {
    ValidateArray(w, "w");
    HIPCX_REQUIRE(x != nullptr && out != nullptr && w->ndim == x->ndim, HIPCX_DIMENSION_ERROR, "conv_transpose: x, w and out need the same rank");
    HIPCX_REQUIRE(IsFloatDtype(out->dtype) && w->dtype == out->dtype && (b == nullptr || b->dtype == out->dtype), HIPCX_DTYPE_ERROR,
                  "conv_transpose: x, w and b must have out's floating point dtype (cast with hipcx_copy first)");
    // the image is `out`, the windows are x's positions; the kernel wants in = x's extents and od = out's
    NdArgs g = MakeGradArgs(out, x, w->shape + 2, stride, pad, 0, true, "conv_transpose");
    HIPCX_REQUIRE(w->shape[0] == x->shape[1] && w->shape[1] == out->shape[1], HIPCX_DIMENSION_ERROR, "conv_transpose: w must be [C_in, C_out, k...]");
    NdArgs p = g;
    p.C = x->shape[1], p.K = out->shape[1];
    for (int d = 0; d < p.n; ++d) p.in[d] = g.od[d], p.od[d] = g.in[d];
    p.x = x->data, p.w = w->data, p.out = out->data;
    CopyStrides(x, p.xs), CopyStrides(w, p.ws), CopyStrides(out, p.os);
    if (b != nullptr) {
        ValidateArray(b, "b");
        HIPCX_REQUIRE(b->ndim == 1 && b->shape[0] == p.K, HIPCX_DIMENSION_ERROR, "Mismatched bias shape for weights.");
        p.b = b->data;
        p.b_stride = ElemStrideNd(b, 0);
    }
    const int64_t total = TotalSize(out);
    if (total == 0) return;
    VisitFloatDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        hipLaunchKernelGGL((ConvTransposeNdKernel<T>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
    });
    CheckLaunch("conv_transpose over n axes");
}

void ConvGradWeightNd(const hipcx_array* x, const hipcx_array* gy, const int64_t* stride, const int64_t* pad, int cover_all, const hipcx_array* gw,
                      void* stream) {
    ValidateArray(gw, "gw");
    HIPCX_REQUIRE(x != nullptr && gy != nullptr && gw->ndim == x->ndim, HIPCX_DIMENSION_ERROR, "conv_grad_weight: x, gy and gw need the same rank");
    HIPCX_REQUIRE(IsFloatDtype(gw->dtype) && x->dtype == gw->dtype, HIPCX_DTYPE_ERROR,
                  "conv_grad_weight: x and gy must have gw's floating point dtype (cast with hipcx_copy first)");
    NdArgs p = MakeGradArgs(x, gy, gw->shape + 2, stride, pad, cover_all, false, "conv_grad_weight");
    HIPCX_REQUIRE(gw->shape[0] == gy->shape[1] && gw->shape[1] == x->shape[1], HIPCX_DIMENSION_ERROR, "conv_grad_weight: gw must be [K, C, k...]");
    p.x = x->data, p.w = gy->data, p.out = gw->data;
    CopyStrides(x, p.xs), CopyStrides(gy, p.ws), CopyStrides(gw, p.os);
    const int64_t total = TotalSize(gw);
    if (total == 0) return;
    int64_t positions = 1;
    for (int d = 0; d < p.n; ++d) positions *= p.od[d];
    VisitFloatDtype(gw->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        hipLaunchKernelGGL((ConvGradWeightNdKernel<T>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total, positions);
    });
    CheckLaunch("conv_grad_weight over n axes");
}

void PoolGradNd(bool is_max, const hipcx_array* x, const hipcx_array* gout, const int64_t* ksize, const int64_t* stride, const int64_t* pad,
                int cover_all, int pad_mode, const hipcx_array* gx, void* stream) {
    NdArgs p = MakeGradArgs(gx, gout, ksize, stride, pad, cover_all, false, is_max ? "max_pool_grad" : "average_pool_grad");
    HIPCX_REQUIRE(gout->shape[1] == gx->shape[1], HIPCX_DIMENSION_ERROR, "pooling gradient: channel counts differ");
    p.w = gout->data, p.out = gx->data;
    CopyStrides(gout, p.ws), CopyStrides(gx, p.os);
    p.pad_mode = pad_mode;
    if (is_max) {
        ValidateArray(x, "x");
        HIPCX_REQUIRE(x->dtype == gx->dtype && SameShape(x, gx), HIPCX_DIMENSION_ERROR, "max_pool_grad: gx must have x's shape and dtype");
        p.x = x->data;
        CopyStrides(x, p.xs);
    }
    const int64_t total = TotalSize(gx);
    if (total == 0) return;
    if (is_max) {
        VisitNumericDtype(gx->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL((PoolGradNdKernel<T, true>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
        });
    } else {
        VisitFloatDtype(gx->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL((PoolGradNdKernel<T, false>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
        });
    }
    CheckLaunch("pooling gradient over n axes");
}

void MaxPoolGradGradNd(const hipcx_array* x, const hipcx_array* ggx, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all,
                       const hipcx_array* ggout, void* stream) {
    NdArgs p = MakeGradArgs(x, ggout, ksize, stride, pad, cover_all, false, "max_pool_grad_grad");
    ValidateArray(ggx, "ggx");
    HIPCX_REQUIRE(ggx->dtype == x->dtype && SameShape(x, ggx) && ggout->shape[1] == x->shape[1], HIPCX_DIMENSION_ERROR,
                  "max_pool_grad_grad: ggx must have x's shape and dtype");
    p.x = x->data, p.w = ggx->data, p.out = ggout->data;
    CopyStrides(x, p.xs), CopyStrides(ggx, p.ws), CopyStrides(ggout, p.os);
    const int64_t total = TotalSize(ggout);
    if (total == 0) return;
    VisitNumericDtype(x->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        hipLaunchKernelGGL((MaxPoolGradGradNdKernel<T>), dim3(NdBlocks(total)), dim3(256), 0, AsStream(stream), p, total);
    });
    CheckLaunch("max_pool_grad_grad over n axes");
}

}  // namespace hipcx
