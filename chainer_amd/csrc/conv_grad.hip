// ConvGradWeightKernel (CX/kernels/connection.h:34-49) for dense NCHW float16 / float32 / float64 arrays.
//
// The native backend computes gw = TensorDot(gy, Im2Col(x)) over the batch and the output positions
// (CX/native/native_device/conv.cc:91-124).  Same product here, with both operands written once in the layout the MFMA matrix
// kernel reads -- the reduction index (n, oh, ow) as the unit-stride axis:
//     gy_t[k][n][oh][ow]            (one transposing copy of gy)
//     col_t[c][r][s][n][oh][ow]     (Im2Col in one launch instead of kh*kw strided copies of a padded image)
// and then gw[k][(c, r, s)] = Dot(gy_t, col_t^T), which for these shapes (few output tiles, long reduction) runs with the
// reduction split over workgroups.
//
// Filters larger than 1x1 at stride 1 (float16 / float32) avoid the kh*kw-fold Im2Col: x is written kw times as zero-padded planes
// whose rows are Wp = W + 2*pw rounded up to a 16-byte granule, copy s shifted left by s elements, and gy once with its rows
// padded to Wp with zeros.  On that common grid tap (r, s) of channel c is the window of copy s that starts r rows down, so
//     gw[k][c][r][s] = sum_n sum_q gy_p[n][k][q] * x_s[s][n][c][q + r*Wp],   q over OH*Wp
// is one accumulated matrix product per image whose right-hand rows alias windows of the copies; the zero columns of gy_p cancel
// the products that wrap around a row end.  A non-finite x value would meet a zero of gy_p in windows the reference never
// multiplies it into (0 * inf = NaN in filter taps that stay finite there), so the copy kernel flags every input channel that holds
// an inf or NaN and, after the product, GradWeightChannelFixupKernel computes the flagged channels' filter taps again the
// reference's way (the sum over the Im2Col windows, padding multiplied as zeros).  With finite data that kernel's workgroups read
// one flag each and exit.
#include "common.h"

namespace hipcx {
namespace {

struct GradWeightArgs {
    const void* x;
    const void* gy;
    void* col_t;
    void* gy_t;
    int N, C, H, W, K, kh, kw, OH, OW, sh, sw, ph, pw;
};

template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) GVec {
    T v[VEC];
};

// One thread: VEC consecutive ow of one (c, r, s, n, oh).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void Im2ColTKernel(GradWeightArgs p, int64_t total) {
    const T* x = static_cast<const T*>(p.x);
    T* col = static_cast<T*>(p.col_t);
    const int owv = p.OW / VEC;
    auto emit = [&](int64_t idx, int wv, int oh, int n, int s, int r, int c) {
        const int ih = oh * p.sh - p.ph + r;
        GVec<T, VEC> out;
        const T* row = x + ((static_cast<int64_t>(n) * p.C + c) * p.H + ih) * p.W;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const int iw = (wv * VEC + e) * p.sw - p.pw + s;
            out.v[e] = (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) ? row[iw] : T(0);
        }
        *reinterpret_cast<GVec<T, VEC>*>(col + idx * VEC) = out;  // idx enumerates the vectors of col_t in memory order
    };
    if (total < (int64_t{1} << 31)) {  // the usual case: five 32-bit divisions per vector instead of five 64-bit ones
        const uint32_t n_total = static_cast<uint32_t>(total), step = gridDim.x * 256u;
        for (uint32_t idx = blockIdx.x * 256u + threadIdx.x; idx < n_total; idx += step) {
            uint32_t t = idx;
            const uint32_t wv = t % static_cast<uint32_t>(owv);
            t /= static_cast<uint32_t>(owv);
            const uint32_t oh = t % static_cast<uint32_t>(p.OH);
            t /= static_cast<uint32_t>(p.OH);
            const uint32_t n = t % static_cast<uint32_t>(p.N);
            t /= static_cast<uint32_t>(p.N);
            const uint32_t s2 = t % static_cast<uint32_t>(p.kw);
            t /= static_cast<uint32_t>(p.kw);
            const uint32_t r = t % static_cast<uint32_t>(p.kh);
            emit(idx, static_cast<int>(wv), static_cast<int>(oh), static_cast<int>(n), static_cast<int>(s2), static_cast<int>(r),
                 static_cast<int>(t / static_cast<uint32_t>(p.kh)));
            if (idx + step < idx) break;  // the next index would wrap
        }
        return;
    }
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t t = idx;
        const int wv = static_cast<int>(t % owv);
        t /= owv;
        const int oh = static_cast<int>(t % p.OH);
        t /= p.OH;
        const int n = static_cast<int>(t % p.N);
        t /= p.N;
        const int s2 = static_cast<int>(t % p.kw);
        t /= p.kw;
        const int r = static_cast<int>(t % p.kh);
        emit(idx, wv, oh, n, s2, r, static_cast<int>(t / p.kh));
    }
}

// gy_t[k][n][p] = gy[n][k][p], VEC consecutive p per thread.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void TransposeNKKernel(GradWeightArgs p, int64_t total) {
    const T* gy = static_cast<const T*>(p.gy);
    T* gt = static_cast<T*>(p.gy_t);
    const int64_t pv = static_cast<int64_t>(p.OH) * p.OW / VEC;
    if (total < (int64_t{1} << 31)) {  // 32-bit index arithmetic
        const uint32_t n_total = static_cast<uint32_t>(total), step = gridDim.x * 256u, pv32 = static_cast<uint32_t>(pv);
        for (uint32_t idx = blockIdx.x * 256u + threadIdx.x; idx < n_total; idx += step) {
            uint32_t t = idx / pv32;
            const uint32_t v = idx - t * pv32;
            const uint32_t k = t / static_cast<uint32_t>(p.N);
            const uint32_t n = t - k * static_cast<uint32_t>(p.N);
            *reinterpret_cast<GVec<T, VEC>*>(gt + static_cast<int64_t>(idx) * VEC) =
                    *reinterpret_cast<const GVec<T, VEC>*>(gy + ((static_cast<int64_t>(n) * p.K + k) * pv + v) * VEC);
            if (idx + step < idx) break;  // the next index would wrap
        }
        return;
    }
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t t = idx;
        const int64_t v = t % pv;
        t /= pv;
        const int n = static_cast<int>(t % p.N);
        const int k = static_cast<int>(t / p.N);
        *reinterpret_cast<GVec<T, VEC>*>(gt + idx * VEC) =
                *reinterpret_cast<const GVec<T, VEC>*>(gy + ((static_cast<int64_t>(n) * p.K + k) * pv + v) * VEC);
    }
}

struct ShiftedArgs {
    const void* x;
    const void* gy;
    void* xs;   // [kw][N*C][Hp*Wp]
    void* gyp;  // [N*K][OH*Wp]
    int* nonfinite;  // [C]: set to 1 for channels of x that hold an inf or NaN (cleared by PaddedRowsKernel, which runs first)
    int planes_x, planes_gy;  // N*C, N*K
    int C;
    int H, W, OH, OW, Hp, Wp, ph, pw, kw;
};

template <typename T>
__device__ __forceinline__ bool NonFinite(T v) {
    if constexpr (sizeof(T) == 2) {
        return (__builtin_bit_cast(unsigned short, v) & 0x7c00u) == 0x7c00u;
    } else {
        return (__builtin_bit_cast(unsigned, v) & 0x7f800000u) == 0x7f800000u;
    }
}

// xs[s][plane][q] = padded x[plane][q + s]; one thread writes VEC consecutive q.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void ShiftedPlanesKernel(ShiftedArgs p, unsigned total) {
    const T* x = static_cast<const T*>(p.x);
    T* xs = static_cast<T*>(p.xs);
    const unsigned per_plane = static_cast<unsigned>(p.Hp * p.Wp / VEC);
    for (unsigned idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += gridDim.x * 256u) {
        unsigned t = idx / per_plane;
        const unsigned qv = idx - t * per_plane;
        const unsigned s = t / static_cast<unsigned>(p.planes_x);
        const unsigned plane = t - s * static_cast<unsigned>(p.planes_x);
        const T* src = x + static_cast<int64_t>(plane) * p.H * p.W;
        GVec<T, VEC> out;
        int q = static_cast<int>(qv) * VEC + static_cast<int>(s);
        int hp = q / p.Wp, wp = q - hp * p.Wp;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const int ih = hp - p.ph, iw = wp - p.pw;
            out.v[e] = (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) ? src[ih * p.W + iw] : T(0);  // rows past Hp fail ih < H
            if (++wp == p.Wp) wp = 0, ++hp;
        }
        *reinterpret_cast<GVec<T, VEC>*>(xs + static_cast<int64_t>(idx) * VEC) = out;
        if (s == 0) {  // copy 0 holds every element of x
            bool bad = false;
#pragma unroll
            for (int e = 0; e < VEC; ++e) bad |= NonFinite<T>(out.v[e]);
            if (bad) p.nonfinite[plane % static_cast<unsigned>(p.C)] = 1;
        }
        if (idx + gridDim.x * 256u < idx) break;  // the next index would wrap
    }
}

// gyp[plane][oh][w] = gy[plane][oh][w] for w < OW, 0 up to Wp.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void PaddedRowsKernel(ShiftedArgs p, unsigned total) {
    const T* gy = static_cast<const T*>(p.gy);
    T* gyp = static_cast<T*>(p.gyp);
    const unsigned per_row = static_cast<unsigned>(p.Wp / VEC);
    if (blockIdx.x == 0) {
        for (int c = threadIdx.x; c < p.C; c += 256) p.nonfinite[c] = 0;
    }
    for (unsigned idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += gridDim.x * 256u) {
        const unsigned row = idx / per_row;  // plane * OH + oh: rows of gy are OW apart
        const int w0 = static_cast<int>(idx - row * per_row) * VEC;
        const T* src = gy + static_cast<int64_t>(row) * p.OW;
        GVec<T, VEC> out;
#pragma unroll
        for (int e = 0; e < VEC; ++e) out.v[e] = w0 + e < p.OW ? src[w0 + e] : T(0);
        *reinterpret_cast<GVec<T, VEC>*>(gyp + static_cast<int64_t>(idx) * VEC) = out;
        if (idx + gridDim.x * 256u < idx) break;
    }
}

// Filter taps of the input channels flagged in `nonfinite`, summed the reference's way: gw[k][c][r][s] = sum over (n, oh, ow) of
// gy[n][k][oh][ow] * col, col = x[n][c][oh*sh - ph + r][ow*sw - pw + s] or the padding's zero (still multiplied, as TensorDot
// multiplies Im2Col's zeros: CX/native/native_device/conv.cc:91-124).  Grid (C, slices); a wave per output, lanes over the sum.
template <typename T>
__global__ __launch_bounds__(256) void GradWeightChannelFixupKernel(GradWeightArgs p, const int* nonfinite, T* gw) {
    const int c = blockIdx.x;
    if (nonfinite[c] == 0) return;
    const T* x = static_cast<const T*>(p.x);
    const T* gy = static_cast<const T*>(p.gy);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int taps = p.kh * p.kw, outputs = p.K * taps;
    const int64_t plane = static_cast<int64_t>(p.OH) * p.OW, total = plane * p.N;
    for (int o = blockIdx.y * 4 + wave; o < outputs; o += gridDim.y * 4) {
        const int k = o / taps, r = (o - k * taps) / p.kw, s = o % p.kw;
        float acc = 0.0f;
        for (int64_t i = lane; i < total; i += 64) {
            const int n = static_cast<int>(i / plane);
            const int pix = static_cast<int>(i - n * plane);
            const int oh = pix / p.OW, ow = pix - oh * p.OW;
            const int ih = oh * p.sh - p.ph + r, iw = ow * p.sw - p.pw + s;
            const float xv = (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W)
                                     ? static_cast<float>(x[((static_cast<int64_t>(n) * p.C + c) * p.H + ih) * p.W + iw]) : 0.0f;
            acc += static_cast<float>(gy[(static_cast<int64_t>(n) * p.K + k) * plane + pix]) * xv;
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) acc += __shfl_down(acc, d);
        if (lane == 0) gw[(static_cast<int64_t>(k) * p.C + c) * taps + (o - k * taps)] = static_cast<T>(acc);
    }
}

int WidestVec(int64_t extent, int64_t item, const void* a, const void* b) {
    int v = static_cast<int>(16 / item);
    while (v > 1 && (extent % v != 0 || reinterpret_cast<uintptr_t>(a) % (v * item) != 0 || reinterpret_cast<uintptr_t>(b) % (v * item) != 0)) v /= 2;
    return v;
}

struct GradWeightPlan {
    GradWeightArgs a{};
    size_t col_bytes = 0, gyt_bytes = 0;
    hipcx_array gy_t{}, col_view{};  // Dot operands: [K, NP] and the [NP, C*kh*kw] view of col_t
};

size_t RoundUp256(size_t v) { return (v + 255) / 256 * 256; }

GradWeightPlan PlanGradWeight(const hipcx_array* x, const hipcx_array* gy, const hipcx_array* gw, const int64_t* stride, const int64_t* pad,
                              int cover_all) {
    ValidateArray(x, "x");
    ValidateArray(gy, "gy");
    ValidateArray(gw, "gw");
    HIPCX_REQUIRE(x->ndim == 4 && gy->ndim == 4 && gw->ndim == 4, HIPCX_NOT_IMPLEMENTED_ERROR, "hip convolution supports 2 spatial dimensions");
    HIPCX_REQUIRE(IsFloatDtype(gw->dtype) && x->dtype == gw->dtype && gy->dtype == gw->dtype, HIPCX_DTYPE_ERROR,
                  "conv_grad_weight: x and gy must have gw's floating point dtype (cast with hipcx_copy first)");
    HIPCX_REQUIRE(IsContiguous(x) && IsContiguous(gy) && IsContiguous(gw), HIPCX_NOT_IMPLEMENTED_ERROR,
                  "hip conv_grad_weight: x, gy and gw must be C-contiguous");
    HIPCX_REQUIRE(stride && pad && stride[0] > 0 && stride[1] > 0 && pad[0] >= 0 && pad[1] >= 0, HIPCX_DIMENSION_ERROR, "invalid stride or pad");
    HIPCX_REQUIRE(gw->shape[1] == x->shape[1], HIPCX_DIMENSION_ERROR, "conv_grad_weight: gw and x disagree on the input channels");
    const int64_t oh = hipcx_conv_out_dim(x->shape[2], gw->shape[2], stride[0], pad[0], cover_all);
    const int64_t ow = hipcx_conv_out_dim(x->shape[3], gw->shape[3], stride[1], pad[1], cover_all);
    HIPCX_REQUIRE(gy->shape[0] == x->shape[0] && gy->shape[1] == gw->shape[0] && gy->shape[2] == oh && gy->shape[3] == ow, HIPCX_DIMENSION_ERROR,
                  "gy has the wrong shape " + ShapeStr(gy));
    for (int i = 0; i < 4; ++i) {
        HIPCX_REQUIRE(x->shape[i] < (1LL << 31) && gw->shape[i] < (1LL << 31) && gy->shape[i] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
    }
    GradWeightPlan pl;
    GradWeightArgs& a = pl.a;
    a.x = x->data;
    a.gy = gy->data;
    a.N = static_cast<int>(x->shape[0]), a.C = static_cast<int>(x->shape[1]), a.H = static_cast<int>(x->shape[2]), a.W = static_cast<int>(x->shape[3]);
    a.K = static_cast<int>(gw->shape[0]), a.kh = static_cast<int>(gw->shape[2]), a.kw = static_cast<int>(gw->shape[3]);
    a.OH = static_cast<int>(oh), a.OW = static_cast<int>(ow);
    a.sh = static_cast<int>(stride[0]), a.sw = static_cast<int>(stride[1]), a.ph = static_cast<int>(pad[0]), a.pw = static_cast<int>(pad[1]);
    const int64_t it = ItemSize(gw->dtype);
    const int64_t np = static_cast<int64_t>(a.N) * a.OH * a.OW;
    const int64_t ckk = static_cast<int64_t>(a.C) * a.kh * a.kw;
    pl.col_bytes = RoundUp256(static_cast<size_t>(ckk * np * it));
    pl.gyt_bytes = RoundUp256(static_cast<size_t>(a.K * np * it));
    pl.gy_t.dtype = gw->dtype, pl.gy_t.ndim = 2;
    pl.gy_t.shape[0] = a.K, pl.gy_t.shape[1] = np;
    pl.gy_t.strides[0] = np * it, pl.gy_t.strides[1] = it;
    pl.col_view.dtype = gw->dtype, pl.col_view.ndim = 2;
    pl.col_view.shape[0] = np, pl.col_view.shape[1] = ckk;
    pl.col_view.strides[0] = it, pl.col_view.strides[1] = np * it;
    return pl;
}

hipcx_array GwAsMatrix(const hipcx_array* gw) {
    hipcx_array m{};
    m.data = gw->data, m.dtype = gw->dtype, m.ndim = 2;
    m.shape[0] = gw->shape[0];
    m.shape[1] = gw->shape[1] * gw->shape[2] * gw->shape[3];
    m.strides[1] = ItemSize(gw->dtype);
    m.strides[0] = m.shape[1] * m.strides[1];
    return m;
}

template <typename T>
void RunLayouts(const GradWeightArgs& a, hipStream_t stream) {
    const int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
    auto grid = [&](int64_t n) { int64_t b = (n + 255) / 256; return dim3(static_cast<unsigned>(b > cap ? cap : (b < 1 ? 1 : b))); };
    {
        const int v = WidestVec(a.OW, sizeof(T), a.col_t, a.col_t);
        const int64_t total = static_cast<int64_t>(a.C) * a.kh * a.kw * a.N * a.OH * (a.OW / v);
        switch (v) {
            case 8: hipLaunchKernelGGL((Im2ColTKernel<T, (sizeof(T) <= 2 ? 8 : 1)>), grid(total), dim3(256), 0, stream, a, total); break;
            case 4: hipLaunchKernelGGL((Im2ColTKernel<T, (sizeof(T) <= 4 ? 4 : 1)>), grid(total), dim3(256), 0, stream, a, total); break;
            case 2: hipLaunchKernelGGL((Im2ColTKernel<T, 2>), grid(total), dim3(256), 0, stream, a, total); break;
            default: hipLaunchKernelGGL((Im2ColTKernel<T, 1>), grid(total), dim3(256), 0, stream, a, total); break;
        }
        CheckLaunch("im2col (weight gradient)");
    }
    {
        const int64_t plane = static_cast<int64_t>(a.OH) * a.OW;
        const int v = WidestVec(plane, sizeof(T), a.gy, a.gy_t);
        const int64_t total = static_cast<int64_t>(a.K) * a.N * (plane / v);
        switch (v) {
            case 8: hipLaunchKernelGGL((TransposeNKKernel<T, (sizeof(T) <= 2 ? 8 : 1)>), grid(total), dim3(256), 0, stream, a, total); break;
            case 4: hipLaunchKernelGGL((TransposeNKKernel<T, (sizeof(T) <= 4 ? 4 : 1)>), grid(total), dim3(256), 0, stream, a, total); break;
            case 2: hipLaunchKernelGGL((TransposeNKKernel<T, 2>), grid(total), dim3(256), 0, stream, a, total); break;
            default: hipLaunchKernelGGL((TransposeNKKernel<T, 1>), grid(total), dim3(256), 0, stream, a, total); break;
        }
        CheckLaunch("gy transpose (weight gradient)");
    }
}

}  // namespace
}  // namespace hipcx

namespace hipcx {
// nd_ops.hip: arrays without exactly two spatial axes
void ConvGradWeightNd(const hipcx_array* x, const hipcx_array* gy, const int64_t* stride, const int64_t* pad, int cover_all, const hipcx_array* gw,
                      void* stream);
}  // namespace hipcx

using namespace hipcx;

// conv.hip: accumulated batch of matrix products on the MFMA kernel
int BatchedProductSlices(int64_t m, int64_t n, int64_t depth, int batch, int dtype);
size_t BatchedProductPartialBytes(int64_t m, int64_t n, int64_t depth, int batch, int dtype);
bool BatchedProductApplies(const void* a, int64_t a_row, int64_t a_slice, const void* bt, int64_t bt_row, int64_t bt_slice, int64_t depth,
                           const void* out, int dtype);
void LaunchBatchedProduct(int dtype, const void* a, int64_t a_row, int64_t a_slice, const void* bt, int64_t bt_row, int64_t bt_slice, int64_t m,
                          int64_t n, int64_t depth, int batch, void* out, float* partial, hipStream_t stream, int taps_r = 0, int taps_s = 0,
                          int64_t r_stride = 0, int64_t s_stride = 0);

namespace {
// A 1x1 filter at stride 1 without padding: gw[k][c] = sum over images of gy_n [K, pixels] @ x_n [C, pixels]^T, which the MFMA kernel
// reads from gy and x where they lie (rows along the pixels, one matrix per image) -- no Im2Col, no transposed copy of gy.
// Taken when the planes are whole 16-byte granules and long enough to fill reduction steps (14x14 planes in float16 are 8-byte
// granules and 3 1/16 steps long: measured no faster than the Im2Col route).
bool DirectPointwise(const GradWeightPlan& pl, const hipcx_array* x, const hipcx_array* gy, const hipcx_array* gw) {
    static const bool enabled = [] { const char* e = getenv("HIPCX_GRAD_WEIGHT_DIRECT"); return e == nullptr || e[0] != '0'; }();
    const GradWeightArgs& a = pl.a;
    if (!enabled || a.kh != 1 || a.kw != 1 || a.sh != 1 || a.sw != 1 || a.ph != 0 || a.pw != 0 || a.OH != a.H || a.OW != a.W) return false;
    const int64_t pixels = static_cast<int64_t>(a.H) * a.W;
    if (pixels < 256 || a.N < 1) return false;
    return BatchedProductApplies(gy->data, pixels, static_cast<int64_t>(a.K) * pixels, x->data, pixels, static_cast<int64_t>(a.C) * pixels, pixels,
                                 gw->data, gw->dtype);
}

// Filters larger than 1x1 at stride 1: shifted zero-padded copies of x instead of Im2Col (see the top of the file).
struct ShiftedPlan {
    bool ok = false;
    ShiftedArgs a{};
    int64_t depth = 0, plane = 0;  // OH*Wp; Hp*Wp
    size_t xs_bytes = 0, gyp_bytes = 0, partial_bytes = 0, flag_bytes = 0;
};

ShiftedPlan PlanShifted(const GradWeightPlan& pl, int dtype) {
    ShiftedPlan sp;
    static const bool enabled = [] { const char* e = getenv("HIPCX_GRAD_WEIGHT_SHIFTED"); return e == nullptr || e[0] != '0'; }();
    const GradWeightArgs& g = pl.a;
    if (!enabled || (dtype != HIPCX_FLOAT16 && dtype != HIPCX_FLOAT32)) return sp;
    if (g.sh != 1 || g.sw != 1 || g.kh * g.kw == 1) return sp;
    if (g.OH != g.H + 2 * g.ph - g.kh + 1 || g.OW != g.W + 2 * g.pw - g.kw + 1) return sp;  // cover_all adds nothing at stride 1
    const int64_t it = ItemSize(dtype), epc = 16 / it;
    const int64_t Wp = (g.W + 2 * g.pw + epc - 1) / epc * epc, Hp = g.H + 2 * g.ph;
    // worth it when the kw copies are smaller than the kh*kw-fold Im2Col
    if (g.kw * Hp * Wp * g.C >= static_cast<int64_t>(g.kh) * g.kw * g.OH * g.OW * g.C) return sp;
    const int64_t xs_elems = static_cast<int64_t>(g.kw) * g.N * g.C * Hp * Wp, gyp_elems = static_cast<int64_t>(g.N) * g.K * g.OH * Wp;
    if (xs_elems / epc >= (1LL << 32) || gyp_elems / epc >= (1LL << 32)) return sp;  // 32-bit vector indices in the copy kernels
    sp.a.planes_x = g.N * g.C, sp.a.planes_gy = g.N * g.K;
    sp.a.H = g.H, sp.a.W = g.W, sp.a.OH = g.OH, sp.a.OW = g.OW, sp.a.Hp = static_cast<int>(Hp), sp.a.Wp = static_cast<int>(Wp);
    sp.a.ph = g.ph, sp.a.pw = g.pw, sp.a.kw = g.kw, sp.a.C = g.C;
    sp.flag_bytes = RoundUp256(static_cast<size_t>(g.C) * sizeof(int));
    sp.depth = g.OH * Wp;
    sp.plane = Hp * Wp;
    sp.xs_bytes = RoundUp256(static_cast<size_t>(xs_elems * it));
    sp.gyp_bytes = RoundUp256(static_cast<size_t>(gyp_elems * it));
    sp.partial_bytes = BatchedProductPartialBytes(g.K, static_cast<int64_t>(g.C) * g.kh * g.kw, sp.depth, g.N, dtype);
    sp.ok = true;
    return sp;
}

template <typename T>
void RunShiftedCopies(const ShiftedArgs& a, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    const int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
    auto grid = [&](int64_t n) { int64_t b = (n + 255) / 256; return dim3(static_cast<unsigned>(b > cap ? cap : (b < 1 ? 1 : b))); };
    const int64_t total_gy = static_cast<int64_t>(a.planes_gy) * a.OH * (a.Wp / VEC);
    hipLaunchKernelGGL((PaddedRowsKernel<T, VEC>), grid(total_gy), dim3(256), 0, stream, a, static_cast<unsigned>(total_gy));  // clears the flags
    CheckLaunch("padded rows (weight gradient)");
    const int64_t total_x = static_cast<int64_t>(a.kw) * a.planes_x * (a.Hp * a.Wp / VEC);
    hipLaunchKernelGGL((ShiftedPlanesKernel<T, VEC>), grid(total_x), dim3(256), 0, stream, a, static_cast<unsigned>(total_x));  // sets them
    CheckLaunch("shifted planes (weight gradient)");
}

template <typename T>
void RunChannelFixup(const GradWeightArgs& g, const int* nonfinite, void* gw, hipStream_t stream) {
    const int outputs = g.K * g.kh * g.kw;
    const int slices = std::max(1, std::min(outputs / 4, 16));
    hipLaunchKernelGGL((GradWeightChannelFixupKernel<T>), dim3(static_cast<unsigned>(g.C), static_cast<unsigned>(slices)), dim3(256), 0, stream, g,
                       nonfinite, static_cast<T*>(gw));
    CheckLaunch("non-finite channels (weight gradient)");
}
}  // namespace

extern "C" {

size_t hipcx_conv_grad_weight_workspace_size(const hipcx_array* x, const hipcx_array* gy, const hipcx_array* gw, const int64_t* stride,
                                             const int64_t* pad, int cover_all) {
    try {
        if (x == nullptr || gy == nullptr || gw == nullptr) return 0;
        if (x->ndim != 4) return 0;  // the n-axis kernel needs none
        GradWeightPlan pl = PlanGradWeight(x, gy, gw, stride, pad, cover_all);
        hipcx_array out = GwAsMatrix(gw);
        // Which path the call takes depends on the alignment of the data pointers, which a caller sizing its workspace from
        // descriptors alone may not have yet: the answer covers both.
        const size_t direct = BatchedProductPartialBytes(pl.a.K, pl.a.C, static_cast<int64_t>(pl.a.H) * pl.a.W, pl.a.N, gw->dtype) + 256;
        const size_t staged = pl.col_bytes + pl.gyt_bytes + hipcx_dot_workspace_size(&pl.gy_t, &pl.col_view, &out);
        const ShiftedPlan sp = PlanShifted(pl, gw->dtype);
        const size_t shifted = sp.ok ? sp.xs_bytes + sp.gyp_bytes + sp.partial_bytes + sp.flag_bytes + 256 : 0;
        return std::max(std::max(direct, staged), shifted);
    } catch (...) {
        return 0;
    }
}

int hipcx_conv_grad_weight(const hipcx_array* x, const hipcx_array* gy, const int64_t* stride, const int64_t* pad, int cover_all,
                           const hipcx_array* gw, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        if (x != nullptr && x->ndim != 4) {  // not two spatial axes: nd_ops.hip
            ConvGradWeightNd(x, gy, stride, pad, cover_all, gw, stream);
            return;
        }
        GradWeightPlan pl = PlanGradWeight(x, gy, gw, stride, pad, cover_all);
        hipcx_array out = GwAsMatrix(gw);
        if (out.shape[0] == 0 || out.shape[1] == 0) return;
        if (pl.gy_t.shape[1] == 0) {  // an empty batch or plane: the sum over nothing
            hipcx_scalar zero{HIPCX_KIND_INT, 0, 0, 0.0};
            int rc = hipcx_fill(gw, zero, stream);
            HIPCX_REQUIRE(rc == HIPCX_OK, rc, hipcx_last_error());
            return;
        }
        if (DirectPointwise(pl, x, gy, gw)) {
            const int64_t pixels = static_cast<int64_t>(pl.a.H) * pl.a.W;
            const size_t partial_bytes = BatchedProductPartialBytes(pl.a.K, pl.a.C, pixels, pl.a.N, gw->dtype);
            HIPCX_REQUIRE(partial_bytes == 0 || (workspace != nullptr && workspace_bytes >= partial_bytes), HIPCX_CHAINERX_ERROR,
                          "conv_grad_weight workspace too small: need " + std::to_string(partial_bytes) + " bytes");
            HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
            LaunchBatchedProduct(gw->dtype, gy->data, pixels, static_cast<int64_t>(pl.a.K) * pixels, x->data, pixels,
                                 static_cast<int64_t>(pl.a.C) * pixels, pl.a.K, pl.a.C, pixels, pl.a.N, gw->data,
                                 partial_bytes ? static_cast<float*>(workspace) : nullptr, AsStream(stream));
            return;
        }
        ShiftedPlan sp = PlanShifted(pl, gw->dtype);
        if (sp.ok && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && reinterpret_cast<uintptr_t>(gw->data) % 16 == 0) {
            const size_t need = sp.xs_bytes + sp.gyp_bytes + sp.partial_bytes + sp.flag_bytes;
            HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR,
                          "conv_grad_weight workspace too small: need " + std::to_string(need) + " bytes");
            char* ws = static_cast<char*>(workspace);
            sp.a.x = x->data, sp.a.gy = gy->data;
            sp.a.xs = ws, sp.a.gyp = ws + sp.xs_bytes;
            sp.a.nonfinite = reinterpret_cast<int*>(ws + sp.xs_bytes + sp.gyp_bytes + sp.partial_bytes);
            hipStream_t st = AsStream(stream);
            if (gw->dtype == HIPCX_FLOAT16) RunShiftedCopies<half_t>(sp.a, st);
            else RunShiftedCopies<float>(sp.a, st);
            const GradWeightArgs& g = pl.a;
            LaunchBatchedProduct(gw->dtype, sp.a.gyp, sp.depth, static_cast<int64_t>(g.K) * sp.depth, sp.a.xs, sp.plane,
                                 static_cast<int64_t>(g.C) * sp.plane, g.K, static_cast<int64_t>(g.C) * g.kh * g.kw, sp.depth, g.N, gw->data,
                                 sp.partial_bytes ? reinterpret_cast<float*>(ws + sp.xs_bytes + sp.gyp_bytes) : nullptr, st, g.kh, g.kw, sp.a.Wp,
                                 static_cast<int64_t>(g.N) * g.C * sp.plane);
            if (gw->dtype == HIPCX_FLOAT16) RunChannelFixup<half_t>(g, sp.a.nonfinite, gw->data, st);
            else RunChannelFixup<float>(g, sp.a.nonfinite, gw->data, st);
            return;
        }
        const size_t dot_bytes = hipcx_dot_workspace_size(&pl.gy_t, &pl.col_view, &out);
        const size_t need = pl.col_bytes + pl.gyt_bytes + dot_bytes;
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR,
                      "conv_grad_weight workspace too small: need " + std::to_string(need) + " bytes");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        char* ws = static_cast<char*>(workspace);
        pl.a.col_t = ws;
        pl.a.gy_t = ws + pl.col_bytes;
        pl.col_view.data = pl.a.col_t;
        pl.gy_t.data = pl.a.gy_t;
        hipStream_t st = AsStream(stream);
        VisitFloatDtype(gw->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            RunLayouts<T>(pl.a, st);
        });
        int rc = hipcx_dot(&pl.gy_t, &pl.col_view, &out, ws + pl.col_bytes + pl.gyt_bytes, dot_bytes, stream);
        HIPCX_REQUIRE(rc == HIPCX_OK, rc, hipcx_last_error());
    });
}

}  // extern "C"
