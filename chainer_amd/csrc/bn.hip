// FixedBatchNorm (inference batch normalisation), CX/kernels/normalization.h:107.
//
// The reference's generic kernel is six elementwise passes (CX/routines/normalization.cc:138-147):
//     inv_std = 1 / sqrt(var + eps);   out = ((x - mean) * inv_std) * gamma + beta
// Here it is one pass, evaluated in that same association order so that float32/float64 results
// carry the same roundings.  float16 data is widened to float, evaluated in float and rounded
// once (the native backend rounds every intermediate to float16; this is strictly more accurate).
//
// Two layouts get dedicated kernels -- per-channel statistics applied to channels-last memory
// ([pixels, C], parameters vary along the fast axis) and to channels-first memory ([N*C, HW],
// one parameter set per row); everything else goes through the generic strided elementwise engine.
#include "elementwise.h"

namespace hipcx {
namespace {

template <typename C>
__device__ __forceinline__ C InvStd(C var, C eps) {
    if constexpr (std::is_same<C, float>::value) {
        return 1.0f / sqrtf(var + eps);
    } else {
        return 1.0 / sqrt(var + eps);
    }
}

// ---- channels-last: x, out = [P, C] (row stride in elements), params contiguous [C] ----
template <typename T, int VEC>
__global__ __launch_bounds__(256) void BnChannelsLastKernel(const T* __restrict__ x, T* __restrict__ out, const T* __restrict__ gamma,
                                                            const T* __restrict__ beta, const T* __restrict__ mean,
                                                            const T* __restrict__ var, compute_t<T> eps, int64_t P, int cvecs,
                                                            int64_t x_row, int64_t o_row, int tpb_c, int tpb_p) {
    using C = compute_t<T>;
    const int tid = threadIdx.x;
    const int cv = blockIdx.y * tpb_c + tid % tpb_c;
    if (cv >= cvecs) return;
    const int c0 = cv * VEC;
    C m[VEC], is[VEC], g[VEC], b[VEC];
    {
        Vec<T, VEC> vm = *reinterpret_cast<const Vec<T, VEC>*>(mean + c0);
        Vec<T, VEC> vv = *reinterpret_cast<const Vec<T, VEC>*>(var + c0);
        Vec<T, VEC> vg = *reinterpret_cast<const Vec<T, VEC>*>(gamma + c0);
        Vec<T, VEC> vb = *reinterpret_cast<const Vec<T, VEC>*>(beta + c0);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            m[e] = static_cast<C>(vm.v[e]);
            is[e] = InvStd<C>(static_cast<C>(vv.v[e]), eps);
            g[e] = static_cast<C>(vg.v[e]);
            b[e] = static_cast<C>(vb.v[e]);
        }
    }
    const int64_t pstep = static_cast<int64_t>(gridDim.x) * tpb_p;
    int64_t p = static_cast<int64_t>(blockIdx.x) * tpb_p + tid / tpb_c;
    constexpr int kU = 4;
    for (; p < P; p += pstep * kU) {
        Vec<T, VEC> in[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            int64_t pu = p + u * pstep;
            if (pu < P) in[u] = *reinterpret_cast<const Vec<T, VEC>*>(x + pu * x_row + c0);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            int64_t pu = p + u * pstep;
            if (pu >= P) continue;
            Vec<T, VEC> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                C t = static_cast<C>(in[u].v[e]) - m[e];
                t = t * is[e];
                t = t * g[e];
                t = t + b[e];
                o.v[e] = static_cast<T>(t);
            }
            *reinterpret_cast<Vec<T, VEC>*>(out + pu * o_row + c0) = o;
        }
    }
}

// ---- channels-first: x, out dense [N*C rows, L]; row r uses channel r % C ----
// The array is walked as one flat run of 16-byte vectors, whatever L is.  A block covers kSpan
// consecutive elements, i.e. a handful of rows: it first derives (mean, inv_std, gamma, beta) for
// those rows into LDS, one row per thread, then every element looks its row's parameters up there.
constexpr int kBnFlatThreads = 256;
constexpr int kBnFlatUnroll = 4;

template <typename T, int VEC>
__global__ __launch_bounds__(kBnFlatThreads) void BnChannelsFirstKernel(const T* __restrict__ x, T* __restrict__ out,
                                                                        const T* __restrict__ gamma, const T* __restrict__ beta,
                                                                        const T* __restrict__ mean, const T* __restrict__ var,
                                                                        compute_t<T> eps, int C_, int64_t L, int64_t pstride,
                                                                        int64_t total, int max_rows, int stream_in) {
    using C = compute_t<T>;
    constexpr int64_t kSpan = static_cast<int64_t>(kBnFlatThreads) * kBnFlatUnroll * VEC;
    extern __shared__ __align__(16) char bn_lds[];
    C* prm = reinterpret_cast<C*>(bn_lds);  // [max_rows][4]
    const int64_t e0 = static_cast<int64_t>(blockIdx.x) * kSpan;
    const int64_t row_first = e0 / L;
    // the elements first: their loads are in flight while the parameters are fetched and staged
    const bool rows_hold_whole_vectors = L % VEC == 0;
    Vec<T, VEC> in[kBnFlatUnroll];
    int64_t idx[kBnFlatUnroll];
#pragma unroll
    for (int u = 0; u < kBnFlatUnroll; ++u) {
        idx[u] = e0 + (static_cast<int64_t>(u) * kBnFlatThreads + threadIdx.x) * VEC;
        if (idx[u] < total) {
            const char* src = reinterpret_cast<const char*>(x + idx[u]);
            in[u] = stream_in ? LoadStreaming<Vec<T, VEC>>(src) : *reinterpret_cast<const Vec<T, VEC>*>(src);
        }
    }
    for (int r = threadIdx.x; r < max_rows; r += kBnFlatThreads) {
        int ch = static_cast<int>((row_first + r) % C_);
        prm[r * 4 + 0] = static_cast<C>(mean[ch * pstride]);
        prm[r * 4 + 1] = InvStd<C>(static_cast<C>(var[ch * pstride]), eps);
        prm[r * 4 + 2] = static_cast<C>(gamma[ch * pstride]);
        prm[r * 4 + 3] = static_cast<C>(beta[ch * pstride]);
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kBnFlatUnroll; ++u) {
        if (idx[u] >= total) continue;
        int64_t row = idx[u] / L;
        int col = static_cast<int>(idx[u] - row * L);
        int r = static_cast<int>(row - row_first);
        Vec<T, VEC> o;
        if (rows_hold_whole_vectors) {  // L % VEC == 0: one parameter set per vector
            const C q0 = prm[r * 4 + 0], q1 = prm[r * 4 + 1], q2 = prm[r * 4 + 2], q3 = prm[r * 4 + 3];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                C t = static_cast<C>(in[u].v[e]) - q0;
                t = t * q1;
                t = t * q2;
                t = t + q3;
                o.v[e] = static_cast<T>(t);
            }
        } else if (L >= VEC) {  // the vector lies in one row or crosses into the next one: two parameter sets, chosen per element
            const int here = static_cast<int>(L) - col;  // elements of this vector that belong to row r
            const int r2 = r + 1 < max_rows ? r + 1 : r;
            const C p0 = prm[r * 4 + 0], p1 = prm[r * 4 + 1], p2 = prm[r * 4 + 2], p3 = prm[r * 4 + 3];
            const C n0 = prm[r2 * 4 + 0], n1 = prm[r2 * 4 + 1], n2 = prm[r2 * 4 + 2], n3 = prm[r2 * 4 + 3];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const bool first = e < here;
                C t = static_cast<C>(in[u].v[e]) - (first ? p0 : n0);
                t = t * (first ? p1 : n1);
                t = t * (first ? p2 : n2);
                t = t + (first ? p3 : n3);
                o.v[e] = static_cast<T>(t);
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if (col >= L) {  // the vector crosses into the next row(s)
                    col -= static_cast<int>(L);
                    ++r;
                }
                const C* q = prm + r * 4;
                C t = static_cast<C>(in[u].v[e]) - q[0];
                t = t * q[1];
                t = t * q[2];
                t = t + q[3];
                o.v[e] = static_cast<T>(t);
                ++col;
            }
        }
        *reinterpret_cast<Vec<T, VEC>*>(out + idx[u]) = o;
    }
}

// ---- generic: any strides, through the elementwise engine ----
template <typename T>
struct BnOp {
    using In = T;
    using Out = T;
    static constexpr int kNumIn = 5;
    static constexpr bool kNeedsIndex = false;
    compute_t<T> eps;
    __device__ __forceinline__ compute_t<T> operator()(compute_t<T>, compute_t<T>, compute_t<T>, compute_t<T>, int64_t) const {
        return compute_t<T>{};
    }
    // inputs: x, gamma, beta, mean, var
    __device__ __forceinline__ compute_t<T> Apply5(compute_t<T> x, compute_t<T> g, compute_t<T> b, compute_t<T> m, compute_t<T> v) const {
        using C = compute_t<T>;
        C t = x - m;
        t = t * InvStd<C>(v, eps);
        t = t * g;
        t = t + b;
        return t;
    }
};

bool Aligned(const void* p, int64_t bytes) { return reinterpret_cast<uintptr_t>(p) % bytes == 0; }

template <typename T>
void RunBn(const hipcx_array* x, const hipcx_array* const params[4], hipcx_scalar eps_s, const hipcx_array* out, hipStream_t stream) {
    using C = compute_t<T>;
    // eps is added in the intermediate dtype (AddAS casts the scalar to it, CX/native/native_device/arithmetic.cc:58)
    const C eps = static_cast<C>(ScalarTo<T>(eps_s));
    // broadcast views of the parameters over x's shape
    hipcx_array pb[4];
    for (int i = 0; i < 4; ++i) {
        pb[i] = *params[i];
        pb[i].ndim = x->ndim;
        for (int d = 0; d < x->ndim; ++d) {
            pb[i].shape[d] = x->shape[d];
            pb[i].strides[d] = params[i]->shape[d] == 1 ? 0 : params[i]->strides[d];
        }
    }
    EwPlan p = MakeEwPlan({out, x, &pb[0], &pb[1], &pb[2], &pb[3]});
    if (p.total == 0) return;
    constexpr int64_t it = sizeof(T);
    constexpr int VEC = 16 / sizeof(T);
    const T* xp = reinterpret_cast<const T*>(p.ptr[1]);
    T* op = reinterpret_cast<T*>(p.ptr[0]);
    const T* g = reinterpret_cast<const T*>(p.ptr[2]);
    const T* b = reinterpret_cast<const T*>(p.ptr[3]);
    const T* m = reinterpret_cast<const T*>(p.ptr[4]);
    const T* v_ = reinterpret_cast<const T*>(p.ptr[5]);

    // channels-last: [P, C] with parameters (0, it); a single pixel row gives ndim == 1.
    if (p.ndim <= 2 && p.ndim >= 1) {
        int ci = p.ndim - 1;
        bool params_ok = true;
        for (int i = 2; i < 6; ++i) {
            params_ok = params_ok && p.strides[i][ci] == it && (p.ndim == 1 || p.strides[i][0] == 0) && Aligned(p.ptr[i], 16);
        }
        int64_t Cn = p.shape[ci];
        int64_t P = p.ndim == 2 ? p.shape[0] : 1;
        bool data_ok = p.strides[0][ci] == it && p.strides[1][ci] == it && Cn % VEC == 0 && Aligned(xp, 16) && Aligned(op, 16);
        int64_t x_row = 0, o_row = 0;
        if (p.ndim == 2) {
            data_ok = data_ok && p.strides[0][0] % 16 == 0 && p.strides[1][0] % 16 == 0;
            x_row = p.strides[1][0] / it;
            o_row = p.strides[0][0] / it;
        }
        if (params_ok && data_ok && Cn / VEC < (1 << 24)) {
            int cvecs = static_cast<int>(Cn / VEC);
            int tpb_c = cvecs < 256 ? cvecs : 256;
            int tpb_p = 256 / tpb_c;
            if (tpb_p < 1) tpb_p = 1;
            int threads = tpb_c * tpb_p;
            int gy = (cvecs + tpb_c - 1) / tpb_c;
            int64_t want = (P + static_cast<int64_t>(tpb_p) * 4 - 1) / (static_cast<int64_t>(tpb_p) * 4);
            int64_t cap = static_cast<int64_t>(NumCUs()) * 16 / gy + 1;
            int gx = static_cast<int>(want < cap ? want : cap);
            if (gx < 1) gx = 1;
            hipLaunchKernelGGL((BnChannelsLastKernel<T, VEC>), dim3(gx, gy), dim3(threads), 0, stream, xp, op, g, b, m, v_, eps, P, cvecs,
                               x_row, o_row, tpb_c, tpb_p);
            CheckLaunch("fixed_batch_norm(channels-last)");
            return;
        }
    }
    // channels-first: [N, C, L] (or [C, L]) dense, parameters (0, s, 0)
    if (p.ndim == 3 || p.ndim == 2) {
        int li = p.ndim - 1, ci = p.ndim - 2;
        int64_t L = p.shape[li], Cn = p.shape[ci], Nn = p.ndim == 3 ? p.shape[0] : 1;
        bool ok = p.strides[0][li] == it && p.strides[1][li] == it && p.strides[0][ci] == L * it && p.strides[1][ci] == L * it;
        if (p.ndim == 3) ok = ok && p.strides[0][0] == Cn * L * it && p.strides[1][0] == Cn * L * it;
        int64_t ps = p.strides[2][ci];
        for (int i = 2; i < 6; ++i) {
            ok = ok && p.strides[i][li] == 0 && p.strides[i][ci] == ps && (p.ndim == 2 || p.strides[i][0] == 0);
        }
        ok = ok && ps % it == 0 && Cn < (1LL << 31);
        if (ok) {
            int64_t total = Nn * Cn * L;
            bool vec_ok = total % VEC == 0 && Aligned(xp, 16) && Aligned(op, 16);
            int v = vec_ok ? VEC : 1;
            int64_t span = static_cast<int64_t>(kBnFlatThreads) * kBnFlatUnroll * v;
            int64_t max_rows = span / L + 2;  // rows a span can touch
            int64_t lds = max_rows * 4 * static_cast<int64_t>(sizeof(C));
            int64_t blocks = (total + span - 1) / span;
            const int stream_in = vec_ok && total * it > StreamingThresholdBytes() ? 1 : 0;
            if (lds <= 48 * 1024 && blocks < (1LL << 31)) {
                if (vec_ok) {
                    hipLaunchKernelGGL((BnChannelsFirstKernel<T, VEC>), dim3(static_cast<unsigned>(blocks)), dim3(kBnFlatThreads),
                                       static_cast<size_t>(lds), stream, xp, op, g, b, m, v_, eps, static_cast<int>(Cn), L, ps / it, total,
                                       static_cast<int>(max_rows), stream_in);
                } else {
                    hipLaunchKernelGGL((BnChannelsFirstKernel<T, 1>), dim3(static_cast<unsigned>(blocks)), dim3(kBnFlatThreads),
                                       static_cast<size_t>(lds), stream, xp, op, g, b, m, v_, eps, static_cast<int>(Cn), L, ps / it, total,
                                       static_cast<int>(max_rows), stream_in);
                }
                CheckLaunch("fixed_batch_norm(channels-first)");
                return;
            }
        }
    }
    BnOp<T> bn;
    bn.eps = eps;
    LaunchElementwise(p, bn, stream);
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" int hipcx_fixed_batch_norm(const hipcx_array* x, const hipcx_array* gamma, const hipcx_array* beta, const hipcx_array* mean,
                                      const hipcx_array* var, hipcx_scalar eps, const int8_t* axis, int naxis, const hipcx_array* out,
                                      void* stream) {
    return Guard([&] {
        ValidateArray(x, "x");
        ValidateArray(out, "out");
        const hipcx_array* params[4] = {gamma, beta, mean, var};
        const char* names[4] = {"gamma", "beta", "mean", "var"};
        HIPCX_REQUIRE(IsFloatDtype(x->dtype), HIPCX_DTYPE_ERROR, "BatchNorm only supports floating kind inputs.");
        HIPCX_REQUIRE(out->dtype == x->dtype && SameShape(x, out), HIPCX_DIMENSION_ERROR, "out must have x's shape and dtype");
        bool reduced[HIPCX_MAX_NDIM] = {};
        for (int i = 0; i < naxis; ++i) {
            HIPCX_REQUIRE(axis[i] >= 0 && axis[i] < x->ndim, HIPCX_DIMENSION_ERROR, "axis out of range");
            reduced[axis[i]] = true;
        }
        for (int i = 0; i < 4; ++i) {
            ValidateArray(params[i], names[i]);
            HIPCX_REQUIRE(params[i]->dtype == x->dtype, HIPCX_NOT_IMPLEMENTED_ERROR,
                          std::string(names[i]) + ": parameters must have x's dtype on the hip backend (cast with hipcx_copy first)");
            HIPCX_REQUIRE(params[i]->ndim == x->ndim, HIPCX_DIMENSION_ERROR,
                          std::string(names[i]) + " must have the keep-dims reduced shape of x");
            for (int d = 0; d < x->ndim; ++d) {
                int64_t expect = reduced[d] ? 1 : x->shape[d];
                HIPCX_REQUIRE(params[i]->shape[d] == expect, HIPCX_DIMENSION_ERROR,
                              std::string(names[i]) + " must have the keep-dims reduced shape of x");
            }
        }
        VisitFloatDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            RunBn<T>(x, params, eps, out, AsStream(stream));
        });
    });
}
