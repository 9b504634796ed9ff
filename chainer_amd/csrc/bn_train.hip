// BatchNorm in training mode and its gradient (BatchNormKernel / BatchNormGradKernel, CX/kernels/normalization.h:32-61) for the
// layout every ChainerX routine hands over: x dense [N, C, L] (L = product of the spatial extents) normalised over every axis but
// the channel axis, all arrays of one float dtype.
//
// The reference's generic kernels are routine compositions (CX/routines/normalization.cc:155-250): Mean, Var = Mean((x - mean)^2),
// 1 / sqrt(var + eps), five elementwise passes, four in-place updates of the running statistics -- about twenty launches that read
// or write the tensor a dozen times.  Here: two statistics passes (sum, then centred sum of squares: the two-pass variance of the
// reference, not E[x^2] - mean^2), one per-channel finish, one normalising pass.  Arithmetic runs in float (double for float64).
// float16 values are rounded to float16 at every point where the composition holds an array (see Rnd), so the special values of the
// reference's float16 arithmetic come out the same -- a sum past 65504 is inf, the statistics and the output that follow from it
// are inf / NaN -- and finite results differ from the composition's only by the order of the float additions inside a sum.
//
// Statistics: grid (C, S).  Block (c, s) walks images s, s + S, ... of channel c with 16-byte loads, reduces over the block and
// stores one partial; the finish kernel adds a channel's S partials in order (deterministic).
#include "elementwise.h"

namespace hipcx {
namespace {

constexpr int kBnTrainThreads = 256;

inline size_t RoundUpTo(size_t v, size_t a) { return (v + a - 1) / a * a; }

template <typename C>
__device__ __forceinline__ C BlockSum(C v, C* lds) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();  // lds may still be read by a previous call
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    C r = C(0);
    if (threadIdx.x == 0) {
        for (int w = 0; w < kBnTrainThreads / 64; ++w) r += lds[w];
    }
    return r;  // valid in thread 0
}

// float16 arrays: the reference composes BatchNorm from routines that each round their result to float16 (and its float16 Sum
// accumulates in float but hands out a float16, CX/native/native_device/reduction.cc:105-110), so a sum past 65504 is inf there,
// (x - mean)^2 past 65504 is inf, 1 / count is a float16 subnormal, and so on.  Rnd applies that rounding wherever the composition
// has an array in between; arithmetic between two roundings runs in float as the reference's Float16 operators do.  For float32
// and float64 it is the identity.
template <typename P, typename C>
__device__ __forceinline__ C Rnd(C v) {
    if constexpr (sizeof(P) == 2) {
        return static_cast<C>(static_cast<P>(v));
    } else {
        return v;
    }
}

// The per-channel state (mean, 1 / std): compute-type vectors in the workspace (forward), or the caller's arrays in the array dtype
// with an element stride (gradient: the state BatchNorm handed out) -- read in place, so the gradient needs no widening copies.
template <typename T, typename P>
__device__ __forceinline__ compute_t<T> LoadState(const void* ptr, int c, int in_array_dtype, int64_t stride) {
    using C = compute_t<T>;
    return in_array_dtype ? static_cast<C>(static_cast<const P*>(ptr)[c * stride]) : static_cast<const C*>(ptr)[c];
}

struct BnStatArgs {
    const void* x;
    const void* g;        // gradient pass only
    const void* mean;     // compute-type vector [C] (workspace)
    const void* inv_std;  // compute-type vector [C] (gradient pass)
    void* partial;        // compute-type [C][S][2]
    int N, C;
    int64_t L;
    int S;
    int state_in_array_dtype;  // see LoadState
    int64_t mean_stride, inv_stride;
};

// MODE 0: sum x.  MODE 1: sum (x - mean)^2.  MODE 2: sum g and sum g * (x - mean) * inv_std.
template <typename T, typename P, int MODE, int VEC>
__global__ __launch_bounds__(kBnTrainThreads) void BnStatKernel(BnStatArgs p) {
    using C = compute_t<T>;
    __shared__ C lds[kBnTrainThreads / 64];
    const int c = blockIdx.x, s = blockIdx.y;
    const T* x = static_cast<const T*>(p.x);
    const T* g = static_cast<const T*>(p.g);
    C m = C(0), is = C(1);
    if (MODE >= 1) m = LoadState<T, P>(p.mean, c, p.state_in_array_dtype, p.mean_stride);
    if (MODE == 2) is = LoadState<T, P>(p.inv_std, c, p.state_in_array_dtype, p.inv_stride);
    C a0 = C(0), a1 = C(0);
    // The slice's images n = s, s + S, ... times the plane's vectors form one index space shared out over the threads, so that
    // planes shorter than the workgroup (14x14, 7x7) keep every lane busy.  32-bit index arithmetic: the host checks N * L < 2^31.
    const uint32_t lv = static_cast<uint32_t>(p.L / VEC);
    const uint32_t images = static_cast<uint32_t>((p.N - s + p.S - 1) / p.S);
    const uint32_t items = images * lv;
    for (uint32_t idx = threadIdx.x; idx < items; idx += kBnTrainThreads) {
        const uint32_t j = idx / lv, v = idx - j * lv;
        const int64_t base = (static_cast<int64_t>(s + j * p.S) * p.C + c) * p.L + static_cast<int64_t>(v) * VEC;
        Vec<T, VEC> xv = *reinterpret_cast<const Vec<T, VEC>*>(x + base);
        Vec<T, VEC> gv;
        if (MODE == 2) gv = *reinterpret_cast<const Vec<T, VEC>*>(g + base);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            C xe = static_cast<C>(xv.v[e]);
            if (MODE == 0) {
                a0 += xe;
            } else if (MODE == 1) {
                C d = Rnd<P>(xe - m);
                a0 += Rnd<P>(d * d);
            } else {
                C ge = static_cast<C>(gv.v[e]);
                a0 += ge;
                a1 += Rnd<P>(ge * Rnd<P>(Rnd<P>(xe - m) * is));
            }
        }
    }
    C r0 = BlockSum<C>(a0, lds);
    C r1 = MODE == 2 ? BlockSum<C>(a1, lds) : C(0);
    if (threadIdx.x == 0) {
        C* out = static_cast<C*>(p.partial) + (static_cast<int64_t>(c) * p.S + s) * 2;
        out[0] = r0;
        out[1] = r1;
    }
}

struct BnFinishArgs {
    const void* partial;
    void* mean;     // compute-type [C]
    void* inv_std;  // compute-type [C]
    void* mean_out;     // T, stride in elements
    void* inv_std_out;  // T
    void* running_mean;
    void* running_var;
    int64_t mo_stride, io_stride, rm_stride, rv_stride;
    int C, S;
    double count;  // N * L
    double eps, decay;
};

// STEP 0: mean from the sums.  STEP 1: variance -> inv_std, state outputs, running statistics (CX/routines/normalization.cc:176-191).
template <typename T, typename P, int STEP>
__global__ __launch_bounds__(256) void BnFinishKernel(BnFinishArgs p) {
    using C = compute_t<T>;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= p.C) return;
    const C* part = static_cast<const C*>(p.partial) + static_cast<int64_t>(c) * p.S * 2;
    C sum = C(0);
    for (int s = 0; s < p.S; ++s) sum += part[s * 2];
    const C n = static_cast<C>(p.count);
    // Mean = Sum (handed out in the array dtype) / count (CX/routines/statistics.cc:113-123)
    if (STEP == 0) {
        static_cast<C*>(p.mean)[c] = Rnd<P>(Rnd<P>(sum) / n);
        return;
    }
    const C mean = static_cast<const C*>(p.mean)[c];
    const C var = Rnd<P>(Rnd<P>(sum) / n);
    // Reciprocal(Sqrt(var + eps)) with eps as a scalar of the array dtype (CX/routines/normalization.cc:141)
    C inv_std;
    if constexpr (std::is_same<C, float>::value) {
        inv_std = Rnd<P>(1.0f / Rnd<P>(sqrtf(Rnd<P>(var + Rnd<P>(static_cast<float>(p.eps))))));
    } else {
        inv_std = 1.0 / sqrt(var + p.eps);
    }
    static_cast<C*>(p.inv_std)[c] = inv_std;
    static_cast<P*>(p.mean_out)[c * p.mo_stride] = static_cast<P>(mean);
    static_cast<P*>(p.inv_std_out)[c * p.io_stride] = static_cast<P>(inv_std);
    // running *= decay; running += (inv_decay [* count / (count - 1)]) * statistic, scalars in the array dtype (CX/routines/normalization.cc:185-190)
    const C decay = Rnd<P>(static_cast<C>(p.decay));
    const C inv_decay = Rnd<P>(static_cast<C>(1.0 - p.decay));
    const C inv_decay_adjusted = Rnd<P>(static_cast<C>((1.0 - p.decay) * (p.count / (p.count - 1.0 > 1.0 ? p.count - 1.0 : 1.0))));
    P* rm = static_cast<P*>(p.running_mean) + c * p.rm_stride;
    P* rv = static_cast<P*>(p.running_var) + c * p.rv_stride;
    *rm = static_cast<P>(Rnd<P>(static_cast<C>(*rm) * decay) + Rnd<P>(inv_decay * mean));
    *rv = static_cast<P>(Rnd<P>(static_cast<C>(*rv) * decay) + Rnd<P>(inv_decay_adjusted * var));
}

struct BnApplyArgs {
    const void* x;
    const void* g;  // gradient only
    void* out;
    const void* mean;     // compute-type [C]
    const void* inv_std;  // compute-type [C]
    const void* gamma;    // T
    const void* beta;     // T (forward only)
    const void* partial;  // gradient: [C][S][2]
    void* ggamma;         // gradient outputs, T
    void* gbeta;
    int64_t gamma_stride, beta_stride, gg_stride, gb_stride;
    int C, S;
    int64_t L, total;
    double count;
    int state_in_array_dtype;  // see LoadState
    int64_t mean_stride, inv_stride;
};

// Gradient finish: ggamma = sum g * x_hat, gbeta = sum g, one thread per channel; leaves both as compute-type values at partial[c][0].
template <typename T, typename P>
__global__ __launch_bounds__(256) void BnGradFinishKernel(BnApplyArgs p) {
    using C = compute_t<T>;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= p.C) return;
    C* part = const_cast<C*>(static_cast<const C*>(p.partial)) + static_cast<int64_t>(c) * p.S * 2;
    C sg = C(0), sgx = C(0);
    for (int s = 0; s < p.S; ++s) {
        sg += part[s * 2];
        sgx += part[s * 2 + 1];
    }
    part[0] = Rnd<P>(sg);  // what the gradient pass reads back is the array-dtype sum, as in the reference
    part[1] = Rnd<P>(sgx);
    static_cast<P*>(p.gbeta)[c * p.gb_stride] = static_cast<P>(sg);
    static_cast<P*>(p.ggamma)[c * p.gg_stride] = static_cast<P>(sgx);
}

// GRAD false: out = ((x - mean) * inv_std) * gamma + beta.
// GRAD true:  gx = (gamma * inv_std) * (g - (x_hat * ggamma + gbeta) / count)   (CX/routines/normalization.cc:232-246).
template <typename T, typename P, bool GRAD, int VEC>
__global__ __launch_bounds__(256) void BnApplyKernel(BnApplyArgs p) {
    using C = compute_t<T>;
    const T* x = static_cast<const T*>(p.x);
    const T* g = static_cast<const T*>(p.g);
    T* out = static_cast<T*>(p.out);
    const int64_t nvec = p.total / VEC;
    const C inv_n = Rnd<P>(static_cast<C>(1.0 / p.count));  // a scalar of the array dtype
    // The array is one contiguous run of [N][C] planes of L elements, cut into vectors without regard to the planes: when VEC does
    // not divide L a vector can hold the end of one plane and the start of the next (never more: the host keeps VEC <= L), and
    // its elements pick the constants of their own channel.  32-bit index arithmetic: the host checks total < 2^31.
    const uint32_t L = static_cast<uint32_t>(p.L);
    const bool planes_split = (L % VEC) != 0;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < nvec; v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const uint32_t first = static_cast<uint32_t>(v) * VEC;
        const uint32_t plane = first / L;
        const uint32_t within = first - plane * L;
        const int c = static_cast<int>(plane % static_cast<uint32_t>(p.C));
        const int c2 = c + 1 == p.C ? 0 : c + 1;
        const bool split = planes_split && within + VEC > L;
        const int split_at = split ? static_cast<int>(L - within) : VEC;  // elements from split_at on belong to channel c2
        const C m = LoadState<T, P>(p.mean, c, p.state_in_array_dtype, p.mean_stride);
        const C is = LoadState<T, P>(p.inv_std, c, p.state_in_array_dtype, p.inv_stride);
        const C ga = static_cast<C>(static_cast<const P*>(p.gamma)[c * p.gamma_stride]);
        C m2 = m, is2 = is, ga2 = ga;
        if (split) {
            m2 = LoadState<T, P>(p.mean, c2, p.state_in_array_dtype, p.mean_stride);
            is2 = LoadState<T, P>(p.inv_std, c2, p.state_in_array_dtype, p.inv_stride);
            ga2 = static_cast<C>(static_cast<const P*>(p.gamma)[c2 * p.gamma_stride]);
        }
        Vec<T, VEC> xv = *reinterpret_cast<const Vec<T, VEC>*>(x + v * VEC);
        Vec<T, VEC> o;
        if constexpr (GRAD) {
            const C* part = static_cast<const C*>(p.partial) + static_cast<int64_t>(c) * p.S * 2;
            const C gbeta = part[0], ggamma = part[1];
            C gbeta2 = gbeta, ggamma2 = ggamma;
            if (split) {
                const C* part2 = static_cast<const C*>(p.partial) + static_cast<int64_t>(c2) * p.S * 2;
                gbeta2 = part2[0], ggamma2 = part2[1];
            }
            Vec<T, VEC> gv = *reinterpret_cast<const Vec<T, VEC>*>(g + v * VEC);
            const C scale = Rnd<P>(ga * is), scale2 = Rnd<P>(ga2 * is2);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const bool second = e >= split_at;
                C x_hat = Rnd<P>(Rnd<P>(static_cast<C>(xv.v[e]) - (second ? m2 : m)) * (second ? is2 : is));
                C t = Rnd<P>(Rnd<P>(Rnd<P>(x_hat * (second ? ggamma2 : ggamma)) + (second ? gbeta2 : gbeta)) * inv_n);
                o.v[e] = static_cast<T>((second ? scale2 : scale) * Rnd<P>(static_cast<C>(gv.v[e]) - t));
            }
        } else {
            const C be = static_cast<C>(static_cast<const P*>(p.beta)[c * p.beta_stride]);
            const C be2 = split ? static_cast<C>(static_cast<const P*>(p.beta)[c2 * p.beta_stride]) : be;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const bool second = e >= split_at;
                C t = Rnd<P>(Rnd<P>(static_cast<C>(xv.v[e]) - (second ? m2 : m)) * (second ? is2 : is));
                o.v[e] = static_cast<T>(Rnd<P>(t * (second ? ga2 : ga)) + (second ? be2 : be));
            }
        }
        *reinterpret_cast<Vec<T, VEC>*>(out + v * VEC) = o;
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
struct BnTrainGeom {
    int N = 0, C = 0, S = 1;
    int64_t L = 1;
    size_t csize = 4;  // bytes of the compute type
};

// x must be dense C-order with ndim >= 2 and the reduction must run over every axis but 1.
BnTrainGeom MakeGeom(const hipcx_array* x, const int8_t* axis, int naxis) {
    ValidateArray(x, "x");
    HIPCX_REQUIRE(IsFloatDtype(x->dtype), HIPCX_DTYPE_ERROR, "BatchNorm only supports floating kind inputs.");
    HIPCX_REQUIRE(x->ndim >= 2 && IsContiguous(x), HIPCX_NOT_IMPLEMENTED_ERROR, "hip batch_norm: x must be C-contiguous with at least 2 axes");
    HIPCX_REQUIRE(naxis == x->ndim - 1, HIPCX_NOT_IMPLEMENTED_ERROR, "hip batch_norm: the statistics must run over every axis but axis 1");
    for (int i = 0; i < naxis; ++i) {
        int want = i == 0 ? 0 : i + 1;
        HIPCX_REQUIRE(axis[i] == want, HIPCX_NOT_IMPLEMENTED_ERROR, "hip batch_norm: the statistics must run over every axis but axis 1");
    }
    BnTrainGeom g;
    HIPCX_REQUIRE(x->shape[0] < (1LL << 31) && x->shape[1] < (1LL << 16) * 32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip batch_norm: extent too large");
    g.N = static_cast<int>(x->shape[0]);
    g.C = static_cast<int>(x->shape[1]);
    for (int d = 2; d < x->ndim; ++d) g.L *= x->shape[d];
    g.csize = x->dtype == HIPCX_FLOAT64 ? 8 : 4;
    int want = (4 * NumCUs() + g.C - 1) / (g.C > 0 ? g.C : 1);
    g.S = want < 1 ? 1 : (want > g.N ? (g.N > 0 ? g.N : 1) : want);
    if (g.S > 65535) g.S = 65535;
    return g;
}

size_t TrainWorkspace(const BnTrainGeom& g) {
    // mean [C], inv_std [C], partials [C][S][2]
    return RoundUpTo(static_cast<size_t>(g.C) * g.csize, 16) * 2 + static_cast<size_t>(g.C) * g.S * 2 * g.csize;
}

// A per-channel vector: shape [C] or the keep-dims shape of x; returns its element stride along the channel axis.
// `param_dtype`: the dtype the per-channel arrays of the call share (see ParamDtype).
int64_t ChannelStride(const hipcx_array* a, const hipcx_array* x, const char* name, int param_dtype) {
    ValidateArray(a, name);
    HIPCX_REQUIRE(a->dtype == param_dtype, HIPCX_NOT_IMPLEMENTED_ERROR,
                  std::string(name) + ": the per-channel arrays must share one dtype, x's or (for float16 x) float32, on the hip backend");
    const int64_t it = ItemSize(a->dtype);
    if (a->ndim == 1) {
        HIPCX_REQUIRE(a->shape[0] == x->shape[1], HIPCX_DIMENSION_ERROR, std::string(name) + " must have one value per channel");
        return a->strides[0] / it;
    }
    HIPCX_REQUIRE(a->ndim == x->ndim, HIPCX_DIMENSION_ERROR, std::string(name) + " must have the keep-dims reduced shape of x");
    for (int d = 0; d < x->ndim; ++d) {
        HIPCX_REQUIRE(a->shape[d] == (d == 1 ? x->shape[1] : 1), HIPCX_DIMENSION_ERROR, std::string(name) + " must have the keep-dims reduced shape of x");
    }
    return a->strides[1] / it;
}

// The dtype of the per-channel arrays, taken from `first` (gamma): x's dtype, or float32 with a float16 x -- the mixed-precision
// call of a float16 network whose normalisation parameters stay in float32.  The reference computes in ResultType(x, gamma, beta)
// (CX/routines/normalization.cc:176-180): float32 then, with one rounding of the output to float16 and none of the float16
// overflow of an all-float16 call.
int ParamDtype(const hipcx_array* x, const hipcx_array* first) {
    ValidateArray(first, "gamma");
    HIPCX_REQUIRE(first->dtype == x->dtype || (x->dtype == HIPCX_FLOAT16 && first->dtype == HIPCX_FLOAT32), HIPCX_NOT_IMPLEMENTED_ERROR,
                  "hip batch_norm: the per-channel arrays must have x's dtype, or float32 for a float16 x");
    return first->dtype;
}

// Calls f with (tag of x's type, tag of the per-channel arrays' type).
template <typename F>
void VisitBnDtypes(int x_dtype, int param_dtype, F&& f) {
    if (x_dtype == HIPCX_FLOAT16 && param_dtype == HIPCX_FLOAT32) {
        f(Tag<half_t>{}, Tag<float>{});
        return;
    }
    VisitFloatDtype(x_dtype, [&](auto tag) { f(tag, tag); });
}

// Widths of the two kernel families.  The statistics kernels read whole planes of one channel, so their vectors must divide the
// plane (16, 8 or one element's bytes); the element-wise kernels cut the contiguous array into 16-byte vectors wherever the planes
// fall, as long as a vector is not longer than a plane.
struct BnWidths {
    int stat;    // elements per vector in the statistics kernels: full, half or 1
    bool apply;  // full vectors in the element-wise kernels
};

BnWidths PickWidths(int64_t L, int64_t total, int64_t item, std::initializer_list<const void*> pointers) {
    const int64_t full = 16 / item;
    auto aligned = [&](int64_t bytes) {
        for (const void* ptr : pointers) {
            if (ptr != nullptr && reinterpret_cast<uintptr_t>(ptr) % bytes != 0) return false;
        }
        return true;
    };
    BnWidths w{1, false};
    if (L % full == 0 && aligned(16)) w.stat = static_cast<int>(full);
    else if (full >= 4 && L % (full / 2) == 0 && aligned(8)) w.stat = static_cast<int>(full / 2);
    w.apply = total % full == 0 && L >= full && aligned(16);
    return w;
}

template <typename T, typename P, int MODE>
void LaunchStat(const BnStatArgs& a, int width, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    dim3 grid(static_cast<unsigned>(a.C), static_cast<unsigned>(a.S));
    if (width == VEC) {
        hipLaunchKernelGGL((BnStatKernel<T, P, MODE, VEC>), grid, dim3(kBnTrainThreads), 0, stream, a);
    } else if (VEC >= 4 && width == VEC / 2) {
        hipLaunchKernelGGL((BnStatKernel<T, P, MODE, (VEC >= 4 ? VEC / 2 : 1)>), grid, dim3(kBnTrainThreads), 0, stream, a);
    } else {
        hipLaunchKernelGGL((BnStatKernel<T, P, MODE, 1>), grid, dim3(kBnTrainThreads), 0, stream, a);
    }
    CheckLaunch("batch_norm statistics");
}

template <typename T, typename P, bool GRAD>
void LaunchApply(const BnApplyArgs& a, bool vec, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    int64_t nvec = a.total / (vec ? VEC : 1);
    int64_t blocks = (nvec + 255) / 256;
    int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    if (vec) {
        hipLaunchKernelGGL((BnApplyKernel<T, P, GRAD, VEC>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
    } else {
        hipLaunchKernelGGL((BnApplyKernel<T, P, GRAD, 1>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
    }
    CheckLaunch("batch_norm apply");
}

void CheckWorkspace(void* workspace, size_t workspace_bytes, size_t need) {
    HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR,
                  "batch_norm workspace too small: need " + std::to_string(need) + " bytes");
    HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_batch_norm_supported(const hipcx_array* x, const int8_t* axis, int naxis, const hipcx_array* const* params, int nparams) {
    try {
        if (x == nullptr || (nparams > 0 && params == nullptr)) return 0;
        const BnTrainGeom g = MakeGeom(x, axis, naxis);
        const int64_t total = static_cast<int64_t>(g.N) * g.C * g.L;
        if (total == 0 || total >= (int64_t{1} << 31)) return 0;
        for (int i = 0; i < nparams; ++i) {
            if (params[i] == nullptr) return 0;
            (void)ChannelStride(params[i], x, "parameter", ParamDtype(x, params[0]));
        }
        return 1;
    } catch (...) {
        return 0;
    }
}

size_t hipcx_batch_norm_workspace_size(const hipcx_array* x, const int8_t* axis, int naxis) {
    try {
        if (x == nullptr) return 0;
        return TrainWorkspace(MakeGeom(x, axis, naxis));
    } catch (...) {
        return 0;
    }
}

int hipcx_batch_norm(const hipcx_array* x, const hipcx_array* gamma, const hipcx_array* beta, const hipcx_array* running_mean,
                     const hipcx_array* running_var, hipcx_scalar eps, hipcx_scalar decay, const int8_t* axis, int naxis,
                     const hipcx_array* out, const hipcx_array* mean_out, const hipcx_array* inv_std_out, void* workspace,
                     size_t workspace_bytes, void* stream) {
    return Guard([&] {
        BnTrainGeom g = MakeGeom(x, axis, naxis);
        ValidateArray(out, "out");
        HIPCX_REQUIRE(out->dtype == x->dtype && SameShape(x, out) && IsContiguous(out), HIPCX_NOT_IMPLEMENTED_ERROR,
                      "hip batch_norm: out must be C-contiguous with x's shape and dtype");
        BnFinishArgs f{};
        BnApplyArgs a{};
        const int pd = ParamDtype(x, gamma);
        a.gamma_stride = ChannelStride(gamma, x, "gamma", pd);
        a.beta_stride = ChannelStride(beta, x, "beta", pd);
        f.rm_stride = ChannelStride(running_mean, x, "running_mean", pd);
        f.rv_stride = ChannelStride(running_var, x, "running_var", pd);
        f.mo_stride = ChannelStride(mean_out, x, "mean_out", pd);
        f.io_stride = ChannelStride(inv_std_out, x, "inv_std_out", pd);
        const int64_t total = static_cast<int64_t>(g.N) * g.C * g.L;
        if (total == 0) return;
        CheckWorkspace(workspace, workspace_bytes, TrainWorkspace(g));
        char* ws = static_cast<char*>(workspace);
        const size_t vec_bytes = RoundUpTo(static_cast<size_t>(g.C) * g.csize, 16);
        void* mean_c = ws;
        void* inv_c = ws + vec_bytes;
        void* partial = ws + 2 * vec_bytes;
        hipStream_t st = AsStream(stream);
        HIPCX_REQUIRE(total < (int64_t{1} << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "hip batch_norm: array too large for the dedicated kernels");
        const BnWidths widths = PickWidths(g.L, total, ItemSize(x->dtype), {x->data, out->data});
        BnStatArgs s{};
        s.x = x->data;
        s.mean = mean_c;
        s.inv_std = inv_c;
        s.partial = partial;
        s.N = g.N, s.C = g.C, s.L = g.L, s.S = g.S;
        f.partial = partial;
        f.mean = mean_c;
        f.inv_std = inv_c;
        f.mean_out = mean_out->data;
        f.inv_std_out = inv_std_out->data;
        f.running_mean = running_mean->data;
        f.running_var = running_var->data;
        f.C = g.C, f.S = g.S;
        f.count = static_cast<double>(g.N) * static_cast<double>(g.L);
        f.eps = ScalarTo<double>(eps);
        f.decay = ScalarTo<double>(decay);
        a.x = x->data;
        a.out = out->data;
        a.mean = mean_c;
        a.inv_std = inv_c;
        a.gamma = gamma->data;
        a.beta = beta->data;
        a.C = g.C, a.S = g.S, a.L = g.L, a.total = total;
        a.count = f.count;
        const unsigned cblocks = static_cast<unsigned>((g.C + 255) / 256);
        VisitBnDtypes(x->dtype, pd, [&](auto tag, auto ptag) {
            using T = typename decltype(tag)::type;
            using P = typename decltype(ptag)::type;
            LaunchStat<T, P, 0>(s, widths.stat, st);
            hipLaunchKernelGGL((BnFinishKernel<T, P, 0>), dim3(cblocks), dim3(256), 0, st, f);
            LaunchStat<T, P, 1>(s, widths.stat, st);
            hipLaunchKernelGGL((BnFinishKernel<T, P, 1>), dim3(cblocks), dim3(256), 0, st, f);
            CheckLaunch("batch_norm finish");
            LaunchApply<T, P, false>(a, widths.apply, st);
        });
    });
}

int hipcx_batch_norm_grad(const hipcx_array* x, const hipcx_array* gamma, const hipcx_array* gout, const hipcx_array* mean,
                          const hipcx_array* inv_std, const int8_t* axis, int naxis, const hipcx_array* gx, const hipcx_array* ggamma,
                          const hipcx_array* gbeta, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        BnTrainGeom g = MakeGeom(x, axis, naxis);
        ValidateArray(gout, "gout");
        ValidateArray(gx, "gx");
        HIPCX_REQUIRE(gout->dtype == x->dtype && SameShape(x, gout) && IsContiguous(gout), HIPCX_NOT_IMPLEMENTED_ERROR,
                      "hip batch_norm_grad: gout must be C-contiguous with x's shape and dtype");
        HIPCX_REQUIRE(gx->dtype == x->dtype && SameShape(x, gx) && IsContiguous(gx), HIPCX_NOT_IMPLEMENTED_ERROR,
                      "hip batch_norm_grad: gx must be C-contiguous with x's shape and dtype");
        BnApplyArgs a{};
        const int pd = ParamDtype(x, gamma);
        a.gamma_stride = ChannelStride(gamma, x, "gamma", pd);
        a.gg_stride = ChannelStride(ggamma, x, "ggamma", pd);
        a.gb_stride = ChannelStride(gbeta, x, "gbeta", pd);
        const int64_t mean_stride = ChannelStride(mean, x, "mean", pd);
        const int64_t inv_stride = ChannelStride(inv_std, x, "inv_std", pd);
        const int64_t total = static_cast<int64_t>(g.N) * g.C * g.L;
        if (total == 0) return;
        CheckWorkspace(workspace, workspace_bytes, TrainWorkspace(g));
        char* ws = static_cast<char*>(workspace);
        const size_t vec_bytes = RoundUpTo(static_cast<size_t>(g.C) * g.csize, 16);
        void* partial = ws + 2 * vec_bytes;  // the same layout as the forward's workspace; the state vectors before it stay unused here
        hipStream_t st = AsStream(stream);
        HIPCX_REQUIRE(total < (int64_t{1} << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "hip batch_norm_grad: array too large for the dedicated kernels");
        const BnWidths widths = PickWidths(g.L, total, ItemSize(x->dtype), {x->data, gout->data, gx->data});
        BnStatArgs s{};
        s.x = x->data;
        s.g = gout->data;
        s.mean = mean->data;  // the state as BatchNorm handed it out, read in place
        s.inv_std = inv_std->data;
        s.state_in_array_dtype = 1;
        s.mean_stride = mean_stride, s.inv_stride = inv_stride;
        s.partial = partial;
        s.N = g.N, s.C = g.C, s.L = g.L, s.S = g.S;
        a.x = x->data;
        a.g = gout->data;
        a.out = gx->data;
        a.mean = mean->data;
        a.inv_std = inv_std->data;
        a.state_in_array_dtype = 1;
        a.mean_stride = mean_stride, a.inv_stride = inv_stride;
        a.gamma = gamma->data;
        a.partial = partial;
        a.ggamma = ggamma->data;
        a.gbeta = gbeta->data;
        a.C = g.C, a.S = g.S, a.L = g.L, a.total = total;
        a.count = static_cast<double>(g.N) * static_cast<double>(g.L);
        const unsigned cblocks = static_cast<unsigned>((g.C + 255) / 256);
        VisitBnDtypes(x->dtype, pd, [&](auto tag, auto ptag) {
            using T = typename decltype(tag)::type;
            using P = typename decltype(ptag)::type;
            LaunchStat<T, P, 2>(s, widths.stat, st);
            hipLaunchKernelGGL((BnGradFinishKernel<T, P>), dim3(cblocks), dim3(256), 0, st, a);
            CheckLaunch("batch_norm_grad finish");
            LaunchApply<T, P, true>(a, widths.apply, st);
        });
    });
}

}  // extern "C"
