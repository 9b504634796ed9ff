// 2-D MaxPool / AveragePool forward (CX/kernels/pooling.h:29,83) on an NCHW-shaped array with
// arbitrary strides.  The native backend materialises the windows (Im2Col) and reduces them
// (CX/native/native_device/pool.cc:69-94, 252-302); here every output is computed directly.
//
//  - max: identity is lowest / -inf, padding never wins, NaN propagates (AMax rule,
//    CX/native/native_device/statistics.cc:38-42).
//  - average: float16 sums accumulate in float, are rounded to float16 and then divided in
//    float16 arithmetic, as Sum followed by Divide does; the divisor is the window size ('zero')
//    or the number of in-image taps ('ignore').
//
// Channels-last data is processed VEC channels per thread with 16-byte accesses; any other
// layout one element per thread, with the thread order following the output's fastest axis.
#include "common.h"
#include "window_argmax.h"

namespace hipcx {
namespace {

struct PoolArgs {
    const void* x;
    void* out;
    int N, C, H, W, OH, OW;
    int kh, kw, sh, sw, ph, pw;
    int64_t xsN, xsC, xsH, xsW;  // elements
    int64_t osN, osC, osH, osW;
    int pad_mode;  // average only
    int w_fastest;  // thread order: 1 = ow fastest (channels-first memory), 0 = channel fastest
};

template <typename T, int N>
struct alignas(sizeof(T) * N) PVec {
    T v[N];
};

template <typename T>
__device__ __forceinline__ T Lowest() {
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

template <typename T>
__device__ __forceinline__ bool IsNanT(T v) {
    if constexpr (std::is_same<T, half_t>::value || std::is_floating_point<T>::value) {
        return v != v;
    } else {
        return false;
    }
}

template <typename T, int VEC, bool IS_MAX>
__global__ __launch_bounds__(256) void PoolKernel(PoolArgs p, int64_t total) {
    using C = compute_t<T>;
    const T* x = static_cast<const T*>(p.x);
    T* out = static_cast<T*>(p.out);
    const int cvecs = p.C / VEC;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        int cv, ow, oh;
        int64_t n;
        int64_t t = idx;
        if (p.w_fastest) {
            ow = static_cast<int>(t % p.OW);
            t /= p.OW;
            oh = static_cast<int>(t % p.OH);
            t /= p.OH;
            cv = static_cast<int>(t % cvecs);
            n = t / cvecs;
        } else {
            cv = static_cast<int>(t % cvecs);
            t /= cvecs;
            ow = static_cast<int>(t % p.OW);
            t /= p.OW;
            oh = static_cast<int>(t % p.OH);
            n = t / p.OH;
        }
        const int c0 = cv * VEC;
        const int h0 = oh * p.sh - p.ph;
        const int w0 = ow * p.sw - p.pw;
        const int hs = h0 < 0 ? 0 : h0;
        const int ws = w0 < 0 ? 0 : w0;
        const int he = h0 + p.kh < p.H ? h0 + p.kh : p.H;
        const int we = w0 + p.kw < p.W ? w0 + p.kw : p.W;
        const T* xb = x + n * p.xsN + static_cast<int64_t>(c0) * p.xsC;
        PVec<T, VEC> res;
        if constexpr (IS_MAX) {
            T acc[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] = Lowest<T>();
            for (int ih = hs; ih < he; ++ih) {
                for (int iw = ws; iw < we; ++iw) {
                    const T* q = xb + ih * p.xsH + iw * p.xsW;
                    PVec<T, VEC> v;
                    if constexpr (VEC > 1) {
                        v = *reinterpret_cast<const PVec<T, VEC>*>(q);
                    } else {
                        v.v[0] = *q;
                    }
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if (IsNanT(v.v[e]) || acc[e] < v.v[e]) acc[e] = v.v[e];
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) res.v[e] = acc[e];
        } else {
            C acc[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] = C(0);
            for (int ih = hs; ih < he; ++ih) {
                for (int iw = ws; iw < we; ++iw) {
                    const T* q = xb + ih * p.xsH + iw * p.xsW;
                    PVec<T, VEC> v;
                    if constexpr (VEC > 1) {
                        v = *reinterpret_cast<const PVec<T, VEC>*>(q);
                    } else {
                        v.v[0] = *q;
                    }
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[e] += static_cast<C>(v.v[e]);
                }
            }
            // divisor in T arithmetic (CX/native/native_device/pool.cc:191-250)
            C div;
            if (p.pad_mode == HIPCX_PAD_ZERO) {
                div = static_cast<C>(static_cast<T>(static_cast<C>(p.kh * p.kw)));
            } else {
                int hcnt = (h0 + p.kh < p.H ? h0 + p.kh : p.H) - hs;
                int wcnt = (w0 + p.kw < p.W ? w0 + p.kw : p.W) - ws;
                div = static_cast<C>(static_cast<T>(static_cast<C>(hcnt) * static_cast<C>(wcnt)));
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                T s = static_cast<T>(acc[e]);  // Sum rounds to the array dtype first
                res.v[e] = static_cast<T>(static_cast<C>(s) / div);
            }
        }
        T* o = out + n * p.osN + static_cast<int64_t>(c0) * p.osC + oh * p.osH + ow * p.osW;
        if constexpr (VEC > 1) {
            *reinterpret_cast<PVec<T, VEC>*>(o) = res;
        } else {
            *o = res.v[0];
        }
    }
}


// Max pooling with horizontal stride 2 over dense NCHW rows: a thread produces EPV/2 adjacent outputs of one row from
// two aligned 16-byte loads per input row (columns [2*ow0 - EPV, 2*ow0 + EPV)), instead of kh*kw scalar loads per
// output.  Requires W % EPV == 0, OW % (EPV/2) == 0, pw <= EPV and kw <= pw + 2 (then every tap falls inside the two
// chunks), which covers the 3x3/2 pad 1 and 2x2/2 pad 0 windows.
template <typename T, int KW, int PW>
__global__ __launch_bounds__(256) void MaxPoolRowsS2Kernel(PoolArgs p, int64_t total) {
    constexpr int EPV = 16 / sizeof(T);
    constexpr int VO = EPV / 2;
    const T* x = static_cast<const T*>(p.x);
    T* out = static_cast<T*>(p.out);
    const int ovecs = p.OW / VO;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        int ov, oh;
        int64_t plane;  // n * C + c
        if (total < (int64_t{1} << 31)) {  // 32-bit index arithmetic (uniform branch)
            const uint32_t i = static_cast<uint32_t>(idx), t = i / static_cast<uint32_t>(ovecs), pl = t / static_cast<uint32_t>(p.OH);
            ov = static_cast<int>(i - t * static_cast<uint32_t>(ovecs));
            oh = static_cast<int>(t - pl * static_cast<uint32_t>(p.OH));
            plane = pl;
        } else {
            ov = static_cast<int>(idx % ovecs);
            const int64_t t = idx / ovecs;
            oh = static_cast<int>(t % p.OH);
            plane = t / p.OH;
        }
        const T* xp = x + plane * p.H * p.W;
        const int ow0 = ov * VO;
        const int col0 = 2 * ow0 - EPV;  // first column of the left chunk
        T acc[VO];
#pragma unroll
        for (int e = 0; e < VO; ++e) acc[e] = Lowest<T>();
        const int h0 = oh * p.sh - p.ph;
        for (int r = 0; r < p.kh; ++r) {
            int ih = h0 + r;
            if (ih < 0 || ih >= p.H) continue;
            const T* row = xp + static_cast<int64_t>(ih) * p.W;
            T win[2 * EPV];
            PVec<T, EPV> lo, hi;
#pragma unroll
            for (int e = 0; e < EPV; ++e) lo.v[e] = hi.v[e] = Lowest<T>();
            if (col0 >= 0) lo = *reinterpret_cast<const PVec<T, EPV>*>(row + col0);
            if (col0 + EPV < p.W) hi = *reinterpret_cast<const PVec<T, EPV>*>(row + col0 + EPV);
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                win[e] = lo.v[e];
                win[EPV + e] = hi.v[e];
            }
#pragma unroll
            for (int e = 0; e < VO; ++e) {
#pragma unroll
                for (int t = 0; t < KW; ++t) {  // taps of output e: window columns EPV + 2e - PW + [0, KW)
                    T v = win[EPV + 2 * e - PW + t];
                    if (IsNanT(v) || acc[e] < v) acc[e] = v;
                }
            }
        }
        PVec<T, VO> res;
#pragma unroll
        for (int e = 0; e < VO; ++e) res.v[e] = acc[e];
        *reinterpret_cast<PVec<T, VO>*>(out + (plane * p.OH + oh) * p.OW + ow0) = res;
    }
}

// Global average pooling over dense NCHW planes (window = whole plane, no padding): a workgroup copies 256 consecutive
// planes (one contiguous run) into LDS with 16-byte loads -- eight per thread in flight at a time --, then each thread
// sums one plane in order.  Sum in the compute type, rounded to T, then divided in T arithmetic, like Sum followed by
// Divide.  Two-byte elements are read back from LDS as dwords (a plane may start in the upper half of one).
template <typename T>
__global__ __launch_bounds__(256) void GlobalAvgPoolKernel(const T* x, T* out, int64_t planes, int hw) {
    using C = compute_t<T>;
    extern __shared__ __align__(16) char lds[];
    constexpr int kBatch = 8;
    constexpr int kStep = 256 * 16;  // bytes the workgroup moves per load instruction
    const int tid = threadIdx.x;
    const int64_t p0 = static_cast<int64_t>(blockIdx.x) * 256;
    const int np = static_cast<int>(planes - p0 < 256 ? planes - p0 : 256);
    const int bytes = np * hw * static_cast<int>(sizeof(T));  // at most 64 KiB
    const char* src = reinterpret_cast<const char*>(x + p0 * hw);
    if (bytes >= 16) {
        const int last = (bytes - 16) & ~15;  // offset of the last whole 16 bytes
        for (int base = tid * 16; base < bytes; base += kBatch * kStep) {
            PVec<unsigned, 4> v[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {  // loads past the end are redirected, not skipped: no branch between the loads
                const int off = base + u * kStep;
                v[u] = *reinterpret_cast<const PVec<unsigned, 4>*>(src + (off < last ? off : last));
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int off = base + u * kStep;
                if (off + 16 <= bytes) *reinterpret_cast<PVec<unsigned, 4>*>(lds + off) = v[u];
            }
        }
    }
    for (int b = (bytes & ~15) + tid; b < bytes; b += 256) lds[b] = src[b];  // the last few bytes of the run
    __syncthreads();
    if (tid < np) {
        C acc = C(0);
        if constexpr (sizeof(T) == 2) {
            const unsigned* w = reinterpret_cast<const unsigned*>(lds);
            auto lower = [](unsigned u) { return static_cast<C>(__builtin_bit_cast(T, static_cast<unsigned short>(u & 0xffffu))); };
            auto upper = [](unsigned u) { return static_cast<C>(__builtin_bit_cast(T, static_cast<unsigned short>(u >> 16))); };
            const int first = tid * hw;  // index of the plane's first element among the workgroup's two-byte elements
            const int odd = first & 1;
            const unsigned* pw = w + (first >> 1);
            const int nwords = (hw + 2) / 2;  // the same trip count for every lane; halves outside the plane are skipped
#pragma unroll 8
            for (int j = 0; j < nwords; ++j) {
                const int e = 2 * j - odd;  // element held by the lower half
                const unsigned u = e < hw ? pw[j] : 0u;  // the last trip of a plane that starts on a word boundary holds nothing of it: no read
                                                         // (for the workgroup's last plane that word would lie past the end of the LDS)
                if (e >= 0 && e < hw) acc += lower(u);
                if (e + 1 < hw) acc += upper(u);
            }
        } else {
            const T* pl = reinterpret_cast<const T*>(lds) + tid * hw;
            for (int i = 0; i < hw; ++i) acc += static_cast<C>(pl[i]);
        }
        T s = static_cast<T>(acc);
        C div = static_cast<C>(static_cast<T>(static_cast<C>(hw)));
        out[p0 + tid] = static_cast<T>(static_cast<C>(s) / div);
    }
}

int64_t ElemStride(const hipcx_array* a, int axis) {
    int64_t it = ItemSize(a->dtype);
    HIPCX_REQUIRE(a->strides[axis] % it == 0, HIPCX_NOT_IMPLEMENTED_ERROR, "byte strides must be multiples of the item size");
    return a->strides[axis] / it;
}

bool Aligned(const void* p, int64_t bytes) { return reinterpret_cast<uintptr_t>(p) % bytes == 0; }

template <typename T, bool IS_MAX>
void RunPool(PoolArgs p, hipStream_t stream) {
    if constexpr (IS_MAX && sizeof(T) <= 8) {
        constexpr int EPV = 16 / sizeof(T);
        constexpr int VO = EPV / 2;
        bool dense_in = p.xsW == 1 && p.xsH == p.W && p.xsC == static_cast<int64_t>(p.H) * p.W && p.xsN == p.xsC * p.C;
        bool dense_out = p.osW == 1 && p.osH == p.OW && p.osC == static_cast<int64_t>(p.OH) * p.OW && p.osN == p.osC * p.C;
        if (VO >= 1 && dense_in && dense_out && p.sw == 2 && p.W % EPV == 0 && p.OW % VO == 0 && p.pw <= EPV && p.kw <= p.pw + 2 &&
            Aligned(p.x, 16) && Aligned(p.out, sizeof(T) * VO) && 2 * (p.OW - 1) - p.pw + p.kw <= p.W + p.pw) {
            int64_t total = static_cast<int64_t>(p.N) * p.C * p.OH * (p.OW / VO);
            if (total == 0) return;
            int64_t blocks = (total + 255) / 256;
            int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
            if (blocks > cap) blocks = cap;
            if (p.kw == 3 && p.pw == 1) {
                hipLaunchKernelGGL((MaxPoolRowsS2Kernel<T, 3, 1>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p, total);
                CheckLaunch("max_pool_rows");
                return;
            }
            if (p.kw == 2 && p.pw == 0) {
                hipLaunchKernelGGL((MaxPoolRowsS2Kernel<T, 2, 0>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p, total);
                CheckLaunch("max_pool_rows");
                return;
            }
        }
    }
    if constexpr (!IS_MAX) {
        bool dense_in = p.xsW == 1 && p.xsH == p.W && p.xsC == static_cast<int64_t>(p.H) * p.W && p.xsN == p.xsC * p.C;
        bool dense_out = p.osC == 1 && p.osN == p.C;  // [N, C, 1, 1]
        int hw = p.H * p.W;
        if (dense_in && dense_out && p.kh == p.H && p.kw == p.W && p.ph == 0 && p.pw == 0 && p.OH == 1 && p.OW == 1 &&
            256 * hw * static_cast<int>(sizeof(T)) <= 64 * 1024 && Aligned(p.x, 16)) {
            int64_t planes = static_cast<int64_t>(p.N) * p.C;
            if (planes == 0) return;
            int lds_bytes = 256 * hw * static_cast<int>(sizeof(T));
            hipLaunchKernelGGL((GlobalAvgPoolKernel<T>), dim3(static_cast<unsigned>((planes + 255) / 256)), dim3(256), lds_bytes, stream,
                               static_cast<const T*>(p.x), static_cast<T*>(p.out), planes, hw);
            CheckLaunch("global_avg_pool");
            return;
        }
    }
    constexpr int VEC = 16 / sizeof(T);
    bool vec_ok = p.xsC == 1 && p.osC == 1 && p.C % VEC == 0 && Aligned(p.x, 16) && Aligned(p.out, 16) && p.xsN % VEC == 0 &&
                  p.xsH % VEC == 0 && p.xsW % VEC == 0 && p.osN % VEC == 0 && p.osH % VEC == 0 && p.osW % VEC == 0;
    int64_t total = static_cast<int64_t>(p.N) * p.OH * p.OW * (vec_ok ? p.C / VEC : p.C);
    if (total == 0) return;
    // thread order follows the output's fastest axis
    int64_t a_c = p.osC < 0 ? -p.osC : p.osC, a_w = p.osW < 0 ? -p.osW : p.osW;
    p.w_fastest = (!vec_ok && a_w < a_c) ? 1 : 0;
    int64_t blocks = (total + 255) / 256;
    int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
    if (blocks > cap) blocks = cap;
    if (vec_ok) {
        hipLaunchKernelGGL((PoolKernel<T, VEC, IS_MAX>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p, total);
    } else {
        hipLaunchKernelGGL((PoolKernel<T, 1, IS_MAX>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p, total);
    }
    CheckLaunch("pool");
}

PoolArgs MakeArgs(const hipcx_array* x, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all,
                  const hipcx_array* out) {
    ValidateArray(x, "x");
    ValidateArray(out, "out");
    HIPCX_REQUIRE(x->ndim == 4 && out->ndim == 4, HIPCX_NOT_IMPLEMENTED_ERROR, "hip pooling supports 2 spatial dimensions");
    HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR, "out must have x's dtype");
    HIPCX_REQUIRE(ksize && stride && pad, HIPCX_CHAINERX_ERROR, "null window parameters");
    HIPCX_REQUIRE(ksize[0] > 0 && ksize[1] > 0 && stride[0] > 0 && stride[1] > 0 && pad[0] >= 0 && pad[1] >= 0, HIPCX_DIMENSION_ERROR,
                  "invalid kernel size, stride or pad");
    int64_t oh = hipcx_conv_out_dim(x->shape[2], ksize[0], stride[0], pad[0], cover_all);
    int64_t ow = hipcx_conv_out_dim(x->shape[3], ksize[1], stride[1], pad[1], cover_all);
    HIPCX_REQUIRE(oh > 0 && ow > 0, HIPCX_DIMENSION_ERROR, "Output size should be positive.");
    HIPCX_REQUIRE(out->shape[0] == x->shape[0] && out->shape[1] == x->shape[1] && out->shape[2] == oh && out->shape[3] == ow,
                  HIPCX_DIMENSION_ERROR, "out has the wrong shape " + ShapeStr(out));
    for (int i = 0; i < 4; ++i) HIPCX_REQUIRE(x->shape[i] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
    PoolArgs p{};
    p.x = x->data;
    p.out = out->data;
    p.N = static_cast<int>(x->shape[0]);
    p.C = static_cast<int>(x->shape[1]);
    p.H = static_cast<int>(x->shape[2]);
    p.W = static_cast<int>(x->shape[3]);
    p.OH = static_cast<int>(oh);
    p.OW = static_cast<int>(ow);
    p.kh = static_cast<int>(ksize[0]);
    p.kw = static_cast<int>(ksize[1]);
    p.sh = static_cast<int>(stride[0]);
    p.sw = static_cast<int>(stride[1]);
    p.ph = static_cast<int>(pad[0]);
    p.pw = static_cast<int>(pad[1]);
    p.xsN = ElemStride(x, 0);
    p.xsC = ElemStride(x, 1);
    p.xsH = ElemStride(x, 2);
    p.xsW = ElemStride(x, 3);
    p.osN = ElemStride(out, 0);
    p.osC = ElemStride(out, 1);
    p.osH = ElemStride(out, 2);
    p.osW = ElemStride(out, 3);
    p.pad_mode = HIPCX_PAD_ZERO;
    return p;
}

// ---------------------------------------------------------------------------------------------
// Gradients (CX/kernels/pooling.h:47-107).  The native backend scatters through Col2Im: a zeroed padded image receives, for
// every kernel offset in (r, s) order, one strided in-place Add (CX/native/col2im.cc:76-122).  Here every input position
// gathers its contributions in that same (r, s) order with the same rounding after every addition, so the result has the bits
// of the composition.
// ---------------------------------------------------------------------------------------------
struct PoolGradArgs {
    const void* x;     // max only
    const void* gout;
    void* gx;
    int N, C, H, W, OH, OW;
    int kh, kw, sh, sw, ph, pw;
    int64_t xsN, xsC, xsH, xsW;  // elements
    int64_t gsN, gsC, gsH, gsW;  // gout
    int64_t dsN, dsC, dsH, dsW;  // gx
    int pad_mode;
    int w_fastest;
    int* win_index;  // max only: ArgMax of every window, dense [N, C, OH, OW]
};

// ArgMax over the kh x kw window of output (oh, ow) as the native backend computes it: the reduction order of window_argmax.h over the
// Im2Col'ed window, whose out-of-image taps hold the lowest value (CX/native/native_device/pool.cc:97-113).
template <typename T>
__device__ int WindowArgMax(const PoolGradArgs& p, const T* xb, int oh, int ow) {
    using V = win_value_t<T>;
    const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
    int r = 0, q = 0;
    return NativeOrderArgMax<V>(p.kh * p.kw, [&](int) -> V {
        const int ih = h0 + r, iw = w0 + q;
        const T v = (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) ? xb[ih * p.xsH + iw * p.xsW] : Lowest<T>();
        if (++q == p.kw) q = 0, ++r;
        return static_cast<V>(v);
    });
}

template <typename T, typename IdxT>
__global__ __launch_bounds__(256) void WindowArgMaxKernel(PoolGradArgs p, IdxT total) {
    const T* x = static_cast<const T*>(p.x);
    for (IdxT idx = static_cast<IdxT>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total; idx += static_cast<IdxT>(gridDim.x) * blockDim.x) {
        IdxT t = idx;
        const int ow = static_cast<int>(t % p.OW);
        t /= p.OW;
        const int oh = static_cast<int>(t % p.OH);
        t /= p.OH;
        const int c = static_cast<int>(t % p.C);
        const int64_t n = static_cast<int64_t>(t / p.C);
        p.win_index[idx] = WindowArgMax<T>(p, x + n * p.xsN + static_cast<int64_t>(c) * p.xsC, oh, ow);
    }
}

// MaxPoolGradGrad (CX/native/native_device/pool.cc:147-177): the element of every window of ggx at the position where x has its
// ArgMax; a position in the padding reads the lowest value, as the Im2Col of the native kernel fills it.  gout/gs* describe ggx here
// and gx/ds* the output [N, C, OH, OW].
template <typename T, typename IdxT>
__global__ __launch_bounds__(256) void MaxPoolGradGradKernel(PoolGradArgs p, IdxT total) {
    const T* x = static_cast<const T*>(p.x);
    const T* ggx = static_cast<const T*>(p.gout);
    T* ggout = static_cast<T*>(p.gx);
    for (IdxT idx = static_cast<IdxT>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total; idx += static_cast<IdxT>(gridDim.x) * blockDim.x) {
        IdxT t = idx;
        const int ow = static_cast<int>(t % p.OW);
        t /= p.OW;
        const int oh = static_cast<int>(t % p.OH);
        t /= p.OH;
        const int c = static_cast<int>(t % p.C);
        const int64_t n = static_cast<int64_t>(t / p.C);
        const int best = WindowArgMax<T>(p, x + n * p.xsN + static_cast<int64_t>(c) * p.xsC, oh, ow);
        const int r = best / p.kw, q = best - r * p.kw;
        const int ih = oh * p.sh - p.ph + r, iw = ow * p.sw - p.pw + q;
        T v = Lowest<T>();
        if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) v = ggx[n * p.gsN + static_cast<int64_t>(c) * p.gsC + ih * p.gsH + iw * p.gsW];
        ggout[n * p.dsN + static_cast<int64_t>(c) * p.dsC + oh * p.dsH + ow * p.dsW] = v;
    }
}

// SMALL: the window is at most twice the stride along both axes, so a position is covered by at most 2 x 2 windows; their gradients
// and indices are then loaded up front, independent of each other, and accumulated in the same order as the general loop visits them.
template <typename T, bool IS_MAX, typename IdxT, bool SMALL = false>
__global__ __launch_bounds__(256) void PoolGradKernel(PoolGradArgs p, IdxT total) {
    using C = compute_t<T>;
    const T* gout = static_cast<const T*>(p.gout);
    T* gx = static_cast<T*>(p.gx);
    // strides that are powers of two (the usual 1 and 2) divide by a shift; -1: a real division
    const int sh_shift = (p.sh & (p.sh - 1)) == 0 ? __builtin_ctz(p.sh) : -1;
    const int sw_shift = (p.sw & (p.sw - 1)) == 0 ? __builtin_ctz(p.sw) : -1;
    auto pixel = [&](int64_t n, int c, int h, int w) {
        const int* wb = IS_MAX ? p.win_index + (n * p.C + c) * (static_cast<int64_t>(p.OH) * p.OW) : nullptr;
        const T* gb = gout + n * p.gsN + static_cast<int64_t>(c) * p.gsC;
        const int y = h + p.ph, xq = w + p.pw;
        T acc = T(0);
        // windows (i, j) that cover this position, walked with the kernel offset r = y - i * sh (and q) ascending
        int i_hi = sh_shift >= 0 ? y >> sh_shift : y / p.sh, j_hi = sw_shift >= 0 ? xq >> sw_shift : xq / p.sw;
        if (i_hi > p.OH - 1) i_hi = p.OH - 1;
        if (j_hi > p.OW - 1) j_hi = p.OW - 1;
        if constexpr (SMALL) {
            T g4[4];
            bool ok4[4];
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    const int i = i_hi - a, j = j_hi - b;
                    const int r = y - i * p.sh, q = xq - j * p.sw;
                    bool ok = i >= 0 && j >= 0 && r < p.kh && q < p.kw;
                    const int ic = ok ? i : 0, jc = ok ? j : 0;
                    T g = gb[ic * p.gsH + jc * p.gsW];
                    if constexpr (IS_MAX) {
                        ok = ok && wb[ic * p.OW + jc] == r * p.kw + q;
                    } else if (p.pad_mode == HIPCX_PAD_IGNORE) {
                        const int h0 = ic * p.sh - p.ph, w0 = jc * p.sw - p.pw;
                        const int hcnt = (h0 + p.kh < p.H ? h0 + p.kh : p.H) - (h0 < 0 ? 0 : h0);
                        const int wcnt = (w0 + p.kw < p.W ? w0 + p.kw : p.W) - (w0 < 0 ? 0 : w0);
                        const T width = static_cast<T>(static_cast<C>(static_cast<T>(static_cast<C>(hcnt))) * static_cast<C>(static_cast<T>(static_cast<C>(wcnt))));
                        g = static_cast<T>(static_cast<C>(g) / static_cast<C>(width));
                    }
                    g4[a * 2 + b] = g;
                    ok4[a * 2 + b] = ok;
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (ok4[e]) acc = static_cast<T>(static_cast<C>(acc) + static_cast<C>(g4[e]));
            }
        } else
        for (int i = i_hi; i >= 0; --i) {
            const int r = y - i * p.sh;
            if (r >= p.kh) break;
            for (int j = j_hi; j >= 0; --j) {
                const int q = xq - j * p.sw;
                if (q >= p.kw) break;
                T g = gb[i * p.gsH + j * p.gsW];
                if constexpr (IS_MAX) {
                    if (wb[i * p.OW + j] != r * p.kw + q) continue;
                } else if (p.pad_mode == HIPCX_PAD_IGNORE) {  // gout / width first, in T arithmetic (pool.cc:197-250, 304-346)
                    const int h0 = i * p.sh - p.ph, w0 = j * p.sw - p.pw;
                    const int hcnt = (h0 + p.kh < p.H ? h0 + p.kh : p.H) - (h0 < 0 ? 0 : h0);
                    const int wcnt = (w0 + p.kw < p.W ? w0 + p.kw : p.W) - (w0 < 0 ? 0 : w0);
                    const T width = static_cast<T>(static_cast<C>(static_cast<T>(static_cast<C>(hcnt))) * static_cast<C>(static_cast<T>(static_cast<C>(wcnt))));
                    g = static_cast<T>(static_cast<C>(g) / static_cast<C>(width));
                }
                acc = static_cast<T>(static_cast<C>(acc) + static_cast<C>(g));
            }
        }
        if (!IS_MAX && p.pad_mode == HIPCX_PAD_ZERO) {
            acc = static_cast<T>(static_cast<C>(acc) / static_cast<C>(static_cast<T>(static_cast<C>(p.kh * p.kw))));
        }
        gx[n * p.dsN + static_cast<int64_t>(c) * p.dsC + h * p.dsH + w * p.dsW] = acc;
    };
    for (IdxT idx = static_cast<IdxT>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total; idx += static_cast<IdxT>(gridDim.x) * blockDim.x) {
        int c, w, h;
        int64_t n;
        IdxT t = idx;
        if (p.w_fastest) {
            w = static_cast<int>(t % p.W);
            t /= p.W;
            h = static_cast<int>(t % p.H);
            t /= p.H;
            c = static_cast<int>(t % p.C);
            n = static_cast<int64_t>(t / p.C);
        } else {
            c = static_cast<int>(t % p.C);
            t /= p.C;
            w = static_cast<int>(t % p.W);
            t /= p.W;
            h = static_cast<int>(t % p.H);
            n = static_cast<int64_t>(t / p.H);
        }
        pixel(n, c, h, w);
    }
}

PoolGradArgs MakeGradArgs(const hipcx_array* x, const hipcx_array* gout, const int64_t* ksize, const int64_t* stride, const int64_t* pad,
                          int cover_all, const hipcx_array* gx) {
    ValidateArray(gout, "gout");
    ValidateArray(gx, "gx");
    if (x != nullptr) ValidateArray(x, "x");
    HIPCX_REQUIRE(gx->ndim == 4 && gout->ndim == 4 && (x == nullptr || x->ndim == 4), HIPCX_NOT_IMPLEMENTED_ERROR,
                  "hip pooling supports 2 spatial dimensions");
    HIPCX_REQUIRE(gout->dtype == gx->dtype && (x == nullptr || x->dtype == gx->dtype), HIPCX_DTYPE_ERROR, "x, gout and gx must share a dtype");
    HIPCX_REQUIRE(x == nullptr || SameShape(x, gx), HIPCX_DIMENSION_ERROR, "gx must have x's shape");
    HIPCX_REQUIRE(ksize && stride && pad, HIPCX_CHAINERX_ERROR, "null window parameters");
    HIPCX_REQUIRE(ksize[0] > 0 && ksize[1] > 0 && stride[0] > 0 && stride[1] > 0 && pad[0] >= 0 && pad[1] >= 0, HIPCX_DIMENSION_ERROR,
                  "invalid kernel size, stride or pad");
    int64_t oh = hipcx_conv_out_dim(gx->shape[2], ksize[0], stride[0], pad[0], cover_all);
    int64_t ow = hipcx_conv_out_dim(gx->shape[3], ksize[1], stride[1], pad[1], cover_all);
    HIPCX_REQUIRE(gout->shape[0] == gx->shape[0] && gout->shape[1] == gx->shape[1] && gout->shape[2] == oh && gout->shape[3] == ow,
                  HIPCX_DIMENSION_ERROR, "gout has the wrong shape " + ShapeStr(gout));
    for (int i = 0; i < 4; ++i) HIPCX_REQUIRE(gx->shape[i] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
    HIPCX_REQUIRE(ksize[0] * ksize[1] < (1LL << 24) && ksize[0] < (1 << 20) && ksize[1] < (1 << 20), HIPCX_NOT_IMPLEMENTED_ERROR, "window too large");
    PoolGradArgs p{};
    p.x = x ? x->data : nullptr;
    p.gout = gout->data;
    p.gx = gx->data;
    p.N = static_cast<int>(gx->shape[0]);
    p.C = static_cast<int>(gx->shape[1]);
    p.H = static_cast<int>(gx->shape[2]);
    p.W = static_cast<int>(gx->shape[3]);
    p.OH = static_cast<int>(oh);
    p.OW = static_cast<int>(ow);
    p.kh = static_cast<int>(ksize[0]);
    p.kw = static_cast<int>(ksize[1]);
    p.sh = static_cast<int>(stride[0]);
    p.sw = static_cast<int>(stride[1]);
    p.ph = static_cast<int>(pad[0]);
    p.pw = static_cast<int>(pad[1]);
    if (x != nullptr) p.xsN = ElemStride(x, 0), p.xsC = ElemStride(x, 1), p.xsH = ElemStride(x, 2), p.xsW = ElemStride(x, 3);
    p.gsN = ElemStride(gout, 0), p.gsC = ElemStride(gout, 1), p.gsH = ElemStride(gout, 2), p.gsW = ElemStride(gout, 3);
    p.dsN = ElemStride(gx, 0), p.dsC = ElemStride(gx, 1), p.dsH = ElemStride(gx, 2), p.dsW = ElemStride(gx, 3);
    p.pad_mode = HIPCX_PAD_ZERO;
    int64_t a_c = p.dsC < 0 ? -p.dsC : p.dsC, a_w = p.dsW < 0 ? -p.dsW : p.dsW;
    p.w_fastest = a_w < a_c ? 1 : 0;
    return p;
}

// ---- MaxPoolGrad of K x K windows (K = 2 or 3) at horizontal stride 2 with padding PW = 0 or 1 over dense NCHW planes whose
// width W is a multiple of 8, OW = W / 2: the usual down-sampling pooling.  Two passes like the general path (the ArgMax of every
// window, then a gather per input position), but a thread takes four neighbouring windows / eight neighbouring positions, so
// that every input row is one aligned vector load plus at most one extra element instead of a load per tap. ----

// ArgMax of N <= 32 values in the order of the native reduction loop (CX/native/reduce.h:46-83): groups of four, then the tail.
template <int N, typename V>
__device__ __forceinline__ int TreeArgMax(const V (&e)[N]) {
    using B = WinBest<V>;
    static_assert(N <= 32, "one block of the reduction tree");
    B accum{V(0), -1};
    constexpr int kMain = N - N % 4;
#pragma unroll
    for (int i = 0; i < kMain; i += 4) {
        B p0{e[i], i};
        WinReduce(B{e[i + 1], i + 1}, p0);
        B p1{e[i + 2], i + 2};
        WinReduce(B{e[i + 3], i + 3}, p1);
        WinReduce(p1, p0);
        WinReduce(p0, accum);
    }
#pragma unroll
    for (int i = kMain; i < N; ++i) WinReduce(B{e[i], i}, accum);
    return accum.i;
}

// win[((n * C + c) * OH + oh) * OW + ow] = ArgMax of the window, one byte each; a thread writes the four windows ow = 4 kk .. 4 kk + 3.
template <typename T, int K, int PW>
__global__ __launch_bounds__(256) void WindowArgMaxStride2Kernel(PoolGradArgs p, uint32_t* win, unsigned total) {
    using V = std::conditional_t<std::is_same<T, half_t>::value, float, std::conditional_t<std::is_same<T, bool>::value, int, T>>;
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const unsigned quads = static_cast<unsigned>(p.OW) / 4;
    unsigned t = idx;
    const int kk = static_cast<int>(t % quads);
    t /= quads;
    const int oh = static_cast<int>(t % p.OH);
    t /= p.OH;
    const int c = static_cast<int>(t % p.C);
    const int64_t n = t / p.C;
    const T* xb = static_cast<const T*>(p.x) + n * p.xsN + static_cast<int64_t>(c) * p.xsC;
    V e[4][K * K];
#pragma unroll
    for (int r = 0; r < K; ++r) {
        const int ih = oh * p.sh - p.ph + r;
        const bool row_ok = ih >= 0 && ih < p.H;
        const T* row = xb + static_cast<int64_t>(row_ok ? ih : 0) * p.W + 8 * kk;
        PVec<T, 8> vec = *reinterpret_cast<const PVec<T, 8>*>(row);
        T left = Lowest<T>(), right = Lowest<T>();
        if (PW == 1 && row_ok && kk > 0) left = row[-1];
        if (PW == 0 && K == 3 && row_ok && 8 * kk + 8 < p.W) right = row[8];
#pragma unroll
        for (int w4 = 0; w4 < 4; ++w4) {
#pragma unroll
            for (int q = 0; q < K; ++q) {
                const int col = 2 * w4 - PW + q;  // a constant after unrolling: -1 .. 8
                T v = col < 0 ? left : (col > 7 ? right : vec.v[col < 0 ? 0 : (col > 7 ? 7 : col)]);
                if (!row_ok) v = Lowest<T>();
                e[w4][r * K + q] = static_cast<V>(v);
            }
        }
    }
    uint32_t packed = 0;
#pragma unroll
    for (int w4 = 0; w4 < 4; ++w4) packed |= static_cast<uint32_t>(TreeArgMax(e[w4])) << (8 * w4);
    win[idx] = packed;
}

// gx over eight neighbouring positions w = 8 kk .. 8 kk + 7 of a row: the windows that cover them are two window rows at most
// (K <= 2 * sh) times the five windows j = 4 kk - 1 + PW .. 4 kk + 3 + PW; their ArgMax bytes and gradients are loaded up front (an
// aligned group of four plus one), and every position adds the gradients of the windows whose ArgMax it is, in the order of the
// general kernel (window row descending, then window column descending).
template <typename T, int K, int PW>
__global__ __launch_bounds__(256) void MaxPoolGradStride2Kernel(PoolGradArgs p, const uint8_t* win, unsigned total) {
    using C = compute_t<T>;
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const unsigned octets = static_cast<unsigned>(p.W) / 8;
    unsigned t = idx;
    const int kk = static_cast<int>(t % octets);
    t /= octets;
    const int h = static_cast<int>(t % p.H);
    t /= p.H;
    const int c = static_cast<int>(t % p.C);
    const int64_t n = t / p.C;
    const T* gb = static_cast<const T*>(p.gout) + n * p.gsN + static_cast<int64_t>(c) * p.gsC;
    const uint8_t* wb = win + (n * p.C + c) * (static_cast<int64_t>(p.OH) * p.OW);
    const int y = h + p.ph;
    int i_hi = y / p.sh;
    if (i_hi > p.OH - 1) i_hi = p.OH - 1;
    // slot s of a window row holds window j = 4 kk - 1 + s, s = 0 .. 5
    T g[2][6];
    int ix[2][6];
    bool row_ok[2];
    int row_r[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int i = i_hi - a;
        const int r = y - i * p.sh;
        row_ok[a] = i >= 0 && r < K;
        row_r[a] = r;
        const int ic = row_ok[a] ? i : 0;
        const T* grow = gb + static_cast<int64_t>(ic) * p.OW + 4 * kk;
        const uint8_t* wrow = wb + static_cast<int64_t>(ic) * p.OW + 4 * kk;
        const PVec<T, 4> g4 = *reinterpret_cast<const PVec<T, 4>*>(grow);
        const uint32_t w4 = *reinterpret_cast<const uint32_t*>(wrow);
#pragma unroll
        for (int s = 0; s < 6; ++s) g[a][s] = T(0), ix[a][s] = -1;
#pragma unroll
        for (int s = 0; s < 4; ++s) g[a][1 + s] = g4.v[s], ix[a][1 + s] = row_ok[a] ? static_cast<int>((w4 >> (8 * s)) & 0xffu) : -1;
        if (PW == 0 && K == 3 && row_ok[a] && kk > 0) g[a][0] = grow[-1], ix[a][0] = wrow[-1];
        if (PW == 1 && row_ok[a] && 4 * kk + 4 < p.OW) g[a][5] = grow[4], ix[a][5] = wrow[4];
    }
    PVec<T, 8> out;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int q_hi = (PW + k) & 1;
        const int slot = ((PW + k) >> 1) + 1;  // of window j_hi = (8 kk + PW + k) / 2
        T acc = T(0);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            if (ix[a][slot] == row_r[a] * K + q_hi) acc = static_cast<T>(static_cast<C>(acc) + static_cast<C>(g[a][slot]));
            if (K == 3 && q_hi == 0 && ix[a][slot - 1] == row_r[a] * K + 2) acc = static_cast<T>(static_cast<C>(acc) + static_cast<C>(g[a][slot - 1]));
        }
        out.v[k] = acc;
    }
    T* dst = static_cast<T*>(p.gx) + n * p.dsN + static_cast<int64_t>(c) * p.dsC + static_cast<int64_t>(h) * p.W + 8 * kk;
    *reinterpret_cast<PVec<T, 8>*>(dst) = out;
}

// Whether the two kernels above take this MaxPoolGrad.
inline bool Stride2MaxPoolGradApplies(const PoolGradArgs& p, size_t item) {
    // (2 x 2 windows with padding never give OW = W / 2)
    const bool window = p.kh == p.kw && ((p.kh == 2 && p.pw == 0) || (p.kh == 3 && (p.pw == 0 || p.pw == 1))) && p.sw == 2 && p.kh <= 2 * p.sh;
    const bool planes = p.W % 8 == 0 && p.OW * 2 == p.W && p.OH > 0;
    const bool dense = p.xsW == 1 && p.xsH == p.W && p.dsW == 1 && p.dsH == p.W && p.gsW == 1 && p.gsH == p.OW && p.xsC % 8 == 0 &&
                       p.xsN % 8 == 0 && p.dsC % 8 == 0 && p.dsN % 8 == 0 && p.gsC % 4 == 0 && p.gsN % 4 == 0;
    const bool aligned = reinterpret_cast<uintptr_t>(p.x) % (8 * item) == 0 && reinterpret_cast<uintptr_t>(p.gx) % (8 * item) == 0 &&
                         reinterpret_cast<uintptr_t>(p.gout) % (4 * item) == 0 && reinterpret_cast<uintptr_t>(p.win_index) % 4 == 0;
    return window && planes && dense && aligned;
}

template <typename T, int K, int PW>
void LaunchStride2MaxPoolGrad(const PoolGradArgs& p, hipStream_t stream) {
    const unsigned quads = static_cast<unsigned>(static_cast<int64_t>(p.N) * p.C * p.OH * (p.OW / 4));
    const unsigned octets = static_cast<unsigned>(static_cast<int64_t>(p.N) * p.C * p.H * (p.W / 8));
    hipLaunchKernelGGL((WindowArgMaxStride2Kernel<T, K, PW>), dim3((quads + 255) / 256), dim3(256), 0, stream, p,
                       reinterpret_cast<uint32_t*>(p.win_index), quads);
    CheckLaunch("window_argmax");
    hipLaunchKernelGGL((MaxPoolGradStride2Kernel<T, K, PW>), dim3((octets + 255) / 256), dim3(256), 0, stream, p,
                       reinterpret_cast<const uint8_t*>(p.win_index), octets);
    CheckLaunch("pool_grad");
}

// AveragePoolGrad of a window that is the whole, unpadded plane: every position of plane (n, c) receives the one gradient of that
// plane divided by the window size, with PoolGradKernel's roundings (the quotient in T, added to a zero of T).  gx is dense NCHW;
// a thread writes 16 bytes, which may run over into the following planes.
template <typename T, typename IdxT>
__global__ __launch_bounds__(256) void GlobalAvgPoolGradKernel(PoolGradArgs p, IdxT total) {
    using C = compute_t<T>;
    constexpr int V = 16 / sizeof(T);
    const T* gout = static_cast<const T*>(p.gout);
    T* gx = static_cast<T*>(p.gx);
    const IdxT hw = static_cast<IdxT>(p.H * p.W);
    const bool dense_gout = p.gsC == 1 && p.gsN == p.C;  // one gradient per plane, in plane order
    auto plane_value = [&](IdxT plane) {
        int64_t at = static_cast<int64_t>(plane);
        if (!dense_gout) {
            const IdxT n = plane / static_cast<IdxT>(p.C);
            at = static_cast<int64_t>(n) * p.gsN + static_cast<int64_t>(plane - n * static_cast<IdxT>(p.C)) * p.gsC;
        }
        T g = gout[at];
        if (p.pad_mode == HIPCX_PAD_IGNORE) {
            const T width = static_cast<T>(static_cast<C>(static_cast<T>(static_cast<C>(p.H))) * static_cast<C>(static_cast<T>(static_cast<C>(p.W))));
            g = static_cast<T>(static_cast<C>(g) / static_cast<C>(width));
        }
        T acc = static_cast<T>(static_cast<C>(T(0)) + static_cast<C>(g));
        if (p.pad_mode == HIPCX_PAD_ZERO) acc = static_cast<T>(static_cast<C>(acc) / static_cast<C>(static_cast<T>(static_cast<C>(p.kh * p.kw))));
        return acc;
    };
    const IdxT e0 = (static_cast<IdxT>(blockIdx.x) * 256 + threadIdx.x) * V;
    if (e0 >= total) return;
    IdxT plane = e0 / hw;
    IdxT rem = e0 - plane * hw;
    T value = plane_value(plane);
    if (hw >= static_cast<IdxT>(V) && e0 + V <= total) {
        // at most one plane boundary inside the 16 bytes: both values are fetched up front, and the vector is put together in
        // registers (sizeof(T)-sized lanes of four dwords)
        const bool crosses = rem + V > hw;
        const T later = crosses ? plane_value(plane + 1) : value;
        using Bits = std::conditional_t<sizeof(T) == 2, uint16_t, std::conditional_t<sizeof(T) == 4, uint32_t, uint64_t>>;
        const uint64_t first = __builtin_bit_cast(Bits, value), second = __builtin_bit_cast(Bits, later);
        PVec<unsigned, 4> out;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint64_t word = 0;  // the elements that overlap dword d (for 8-byte elements: one half of an element)
            if constexpr (sizeof(T) == 8) {
                const uint64_t e = rem + d / 2 < hw ? first : second;
                word = (d & 1) ? e >> 32 : e & 0xffffffffu;
            } else {
                constexpr int per = 4 / sizeof(T);
#pragma unroll
                for (int k = 0; k < per; ++k) word |= (rem + d * per + k < hw ? first : second) << (8 * sizeof(T) * k);
            }
            out.v[d] = static_cast<unsigned>(word);
        }
        *reinterpret_cast<PVec<unsigned, 4>*>(gx + e0) = out;
        return;
    }
    for (int k = 0; k < V && e0 + k < total; ++k) {
        if (rem == hw) {
            rem = 0;
            value = plane_value(++plane);
        }
        gx[e0 + k] = value;
        ++rem;
    }
}

template <typename T, bool IS_MAX>
void RunPoolGrad(const PoolGradArgs& p, hipStream_t stream) {
    const int64_t total = static_cast<int64_t>(p.N) * p.C * p.H * p.W;
    const int64_t windows = static_cast<int64_t>(p.N) * p.C * p.OH * p.OW;
    if (total == 0) return;
    const int64_t cap = static_cast<int64_t>(NumCUs()) * 64;
    auto grid_for = [&](int64_t n) { int64_t b = (n + 255) / 256; return dim3(static_cast<unsigned>(b > cap ? cap : (b < 1 ? 1 : b))); };
    const bool narrow = total + cap * 256 < (1LL << 31) && windows + cap * 256 < (1LL << 31);  // 32-bit index arithmetic
    if constexpr (IS_MAX && !std::is_same<T, bool>::value) {
        if (narrow && windows > 0 && Stride2MaxPoolGradApplies(p, sizeof(T))) {
            if (p.kh == 2) LaunchStride2MaxPoolGrad<T, 2, 0>(p, stream);
            else if (p.pw == 0) LaunchStride2MaxPoolGrad<T, 3, 0>(p, stream);
            else LaunchStride2MaxPoolGrad<T, 3, 1>(p, stream);
            return;
        }
    }
    if constexpr (IS_MAX) {
        if (windows > 0) {
            if (narrow) {
                hipLaunchKernelGGL((WindowArgMaxKernel<T, unsigned>), grid_for(windows), dim3(256), 0, stream, p, static_cast<unsigned>(windows));
            } else {
                hipLaunchKernelGGL((WindowArgMaxKernel<T, int64_t>), grid_for(windows), dim3(256), 0, stream, p, windows);
            }
            CheckLaunch("window_argmax");
        }
    }
    if constexpr (!IS_MAX) {
        const bool whole_plane = p.OH == 1 && p.OW == 1 && p.kh == p.H && p.kw == p.W && p.ph == 0 && p.pw == 0;
        const bool dense = p.dsW == 1 && p.dsH == p.W && p.dsC == static_cast<int64_t>(p.H) * p.W && p.dsN == p.dsC * p.C;
        if (whole_plane && dense && reinterpret_cast<uintptr_t>(p.gx) % 16 == 0) {
            constexpr int V = 16 / sizeof(T);
            const int64_t threads = (total + V - 1) / V;
            const dim3 blocks(static_cast<unsigned>((threads + 255) / 256));
            if (total + 16 < (1LL << 31)) {
                hipLaunchKernelGGL((GlobalAvgPoolGradKernel<T, unsigned>), blocks, dim3(256), 0, stream, p, static_cast<unsigned>(total));
            } else {
                hipLaunchKernelGGL((GlobalAvgPoolGradKernel<T, int64_t>), blocks, dim3(256), 0, stream, p, total);
            }
            CheckLaunch("pool_grad");
            return;
        }
    }
    const bool small = p.kh <= 2 * p.sh && p.kw <= 2 * p.sw && p.OH > 0 && p.OW > 0;
    const dim3 grid = grid_for(total);
    if (narrow && small) {
        hipLaunchKernelGGL((PoolGradKernel<T, IS_MAX, unsigned, true>), grid, dim3(256), 0, stream, p, static_cast<unsigned>(total));
    } else if (narrow) {
        hipLaunchKernelGGL((PoolGradKernel<T, IS_MAX, unsigned>), grid, dim3(256), 0, stream, p, static_cast<unsigned>(total));
    } else {
        hipLaunchKernelGGL((PoolGradKernel<T, IS_MAX, int64_t>), grid, dim3(256), 0, stream, p, total);
    }
    CheckLaunch("pool_grad");
}

}  // namespace
}  // namespace hipcx

namespace hipcx {
// nd_ops.hip: arrays without exactly two spatial axes
void PoolGradNd(bool is_max, const hipcx_array* x, const hipcx_array* gout, const int64_t* ksize, const int64_t* stride, const int64_t* pad,
                int cover_all, int pad_mode, const hipcx_array* gx, void* stream);
void MaxPoolGradGradNd(const hipcx_array* x, const hipcx_array* ggx, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all,
                       const hipcx_array* ggout, void* stream);
void PoolNd(bool is_max, const hipcx_array* x, const int64_t* ksize, const int64_t* stride, const int64_t* pad, int cover_all, int pad_mode,
            const hipcx_array* out, void* stream);
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_max_pool(const hipcx_array* x, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int cover_all,
                   const hipcx_array* out, void* stream) {
    return Guard([&] {
        if (x != nullptr && x->ndim != 4) {
            PoolNd(true, x, kernel_size, stride, pad, cover_all, HIPCX_PAD_ZERO, out, stream);
            return;
        }
        PoolArgs p = MakeArgs(x, kernel_size, stride, pad, cover_all, out);
        VisitDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            RunPool<T, true>(p, AsStream(stream));
        });
    });
}

int hipcx_average_pool(const hipcx_array* x, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int pad_mode,
                       const hipcx_array* out, void* stream) {
    return Guard([&] {
        HIPCX_REQUIRE(pad_mode == HIPCX_PAD_ZERO || pad_mode == HIPCX_PAD_IGNORE, HIPCX_CHAINERX_ERROR, "invalid pad mode");
        HIPCX_REQUIRE(x != nullptr && IsFloatDtype(x->dtype), HIPCX_DTYPE_ERROR, "cannot apply average pooling to non-float arrays");
        if (x->ndim != 4) {
            PoolNd(false, x, kernel_size, stride, pad, 0, pad_mode, out, stream);
            return;
        }
        PoolArgs p = MakeArgs(x, kernel_size, stride, pad, 0, out);
        p.pad_mode = pad_mode;
        VisitFloatDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            RunPool<T, false>(p, AsStream(stream));
        });
    });
}

size_t hipcx_max_pool_grad_workspace_size(const hipcx_array* gout) {
    if (gout == nullptr || gout->ndim != 4) return 0;
    int64_t n = 1;
    for (int i = 0; i < 4; ++i) n *= gout->shape[i] > 0 ? gout->shape[i] : 0;
    return static_cast<size_t>(n) * sizeof(int);
}

int hipcx_max_pool_grad(const hipcx_array* x, const hipcx_array* gout, const int64_t* kernel_size, const int64_t* stride,
                        const int64_t* pad, int cover_all, const hipcx_array* gx, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        HIPCX_REQUIRE(x != nullptr && gx != nullptr, HIPCX_CHAINERX_ERROR, "null array");
        if (x->ndim != 4) {  // not two spatial axes: nd_ops.hip
            PoolGradNd(true, x, gout, kernel_size, stride, pad, cover_all, HIPCX_PAD_ZERO, gx, stream);
            return;
        }
        PoolGradArgs p = MakeGradArgs(x, gout, kernel_size, stride, pad, cover_all, gx);
        const size_t need = hipcx_max_pool_grad_workspace_size(gout);
        HIPCX_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need), HIPCX_CHAINERX_ERROR,
                      "max_pool_grad workspace too small: need " + std::to_string(need) + " bytes");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 4 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 4-byte aligned");
        p.win_index = static_cast<int*>(workspace);
        VisitDtype(gx->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            if constexpr (std::is_same<T, bool>::value) {
                throw Error(HIPCX_DTYPE_ERROR, "max_pool_grad: bool arrays are not supported");
            } else {
                RunPoolGrad<T, true>(p, AsStream(stream));
            }
        });
    });
}

int hipcx_average_pool_grad(const hipcx_array* gout, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int pad_mode,
                            const hipcx_array* gx, void* stream) {
    return Guard([&] {
        HIPCX_REQUIRE(pad_mode == HIPCX_PAD_ZERO || pad_mode == HIPCX_PAD_IGNORE, HIPCX_CHAINERX_ERROR, "invalid pad mode");
        HIPCX_REQUIRE(gx != nullptr && IsFloatDtype(gx->dtype), HIPCX_DTYPE_ERROR, "cannot apply average pooling to non-float arrays");
        if (gx->ndim != 4) {  // not two spatial axes: nd_ops.hip
            PoolGradNd(false, nullptr, gout, kernel_size, stride, pad, 0, pad_mode, gx, stream);
            return;
        }
        PoolGradArgs p = MakeGradArgs(nullptr, gout, kernel_size, stride, pad, 0, gx);
        p.pad_mode = pad_mode;
        VisitFloatDtype(gx->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            RunPoolGrad<T, false>(p, AsStream(stream));
        });
    });
}

int hipcx_max_pool_grad_grad(const hipcx_array* x, const hipcx_array* ggx, const int64_t* kernel_size, const int64_t* stride,
                             const int64_t* pad, int cover_all, const hipcx_array* ggout, void* stream) {
    return Guard([&] {
        HIPCX_REQUIRE(x != nullptr && ggx != nullptr, HIPCX_CHAINERX_ERROR, "null array");
        if (x->ndim != 4) {  // not two spatial axes: nd_ops.hip
            MaxPoolGradGradNd(x, ggx, kernel_size, stride, pad, cover_all, ggout, stream);
            return;
        }
        // the geometry helper wants (x, window-shaped array, image-shaped array): here the image-shaped one is ggx
        PoolGradArgs p = MakeGradArgs(x, ggout, kernel_size, stride, pad, cover_all, ggx);
        // swap roles: gout/gs* <- ggx (image), gx/ds* <- ggout (windows)
        std::swap(p.gsN, p.dsN);
        std::swap(p.gsC, p.dsC);
        std::swap(p.gsH, p.dsH);
        std::swap(p.gsW, p.dsW);
        p.gout = ggx->data;
        p.gx = ggout->data;
        const int64_t windows = static_cast<int64_t>(p.N) * p.C * p.OH * p.OW;
        if (windows == 0) return;
        const int64_t cap = static_cast<int64_t>(NumCUs()) * 64;
        int64_t blocks = (windows + 255) / 256;
        if (blocks > cap) blocks = cap;
        VisitDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            if constexpr (std::is_same<T, bool>::value) {
                throw Error(HIPCX_DTYPE_ERROR, "max_pool_grad_grad: bool arrays are not supported");
            } else if (windows + cap * 256 < (1LL << 31)) {
                hipLaunchKernelGGL((MaxPoolGradGradKernel<T, unsigned>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, AsStream(stream), p,
                                   static_cast<unsigned>(windows));
            } else {
                hipLaunchKernelGGL((MaxPoolGradGradKernel<T, int64_t>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, AsStream(stream), p,
                                   windows);
            }
        });
        CheckLaunch("max_pool_grad_grad");
    });
}
}
