// Im2Col, Col2Im and ConvTransposeKernel for arrays with two spatial axes.
//
// Im2Col (CX/native/im2col.cc:82-149) fills a padded copy of x and gathers col[N, C, kh, kw, oh, ow] from it with one strided
// Copy per kernel offset; Col2Im (CX/native/col2im.cc:76-122) adds the planes of a col back into a zero-filled padded image,
// one strided in-place Add per kernel offset in (r, s) order, and returns the view without the padding.  Here each is one
// launch that computes every destination element directly:
//   * im2col: the element of x the window position maps to, or the padding value;
//   * col2im: the contributions of an image position summed in ascending (r, s) order, starting from zero, with one rounding
//     to the array dtype per addition -- the value the chain of in-place Add kernels leaves there, bit for bit.
//
// ConvTransposeKernel (CX/kernels/connection.h:51-66) after the native kernel (CX/native/native_device/conv.cc:126-160:
// TensorDot(w, x) over the input channels, Col2Im, bias), with two shorter routes for the shapes a backward pass meets:
//   * stride 1: a forward convolution with the filters flipped in both spatial axes, their channel axes swapped and the padding
//     k - 1 - p (one MFMA convolution; the sums run in another order than the composition's, equal to tolerance);
//   * a 1x1 filter without padding at any stride: a 1x1 forward convolution scattered to every stride-th pixel of zeros;
//   * otherwise the native composition: matrix product, then col2im.
#include "common.h"

namespace hipcx {
namespace {

struct ColArgs {
    const void* src;
    void* dst;
    int N, C, H, W;      // image extents (im2col: of x; col2im: of the result)
    int kh, kw, OH, OW;  // kernel extents and window positions (col.shape[2:6])
    int sh, sw, ph, pw;
    int64_t is[4];  // image strides, elements
    int64_t cs[6];  // col strides, elements
};

// One thread per element of col, ow fastest.
template <typename T>
__global__ __launch_bounds__(256) void Im2ColKernel(ColArgs p, T pad_value, int64_t total) {
    const T* x = static_cast<const T*>(p.src);
    T* col = static_cast<T*>(p.dst);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t t = idx;
        const int ow = static_cast<int>(t % p.OW);
        t /= p.OW;
        const int oh = static_cast<int>(t % p.OH);
        t /= p.OH;
        const int q = static_cast<int>(t % p.kw);
        t /= p.kw;
        const int r = static_cast<int>(t % p.kh);
        t /= p.kh;
        const int c = static_cast<int>(t % p.C);
        const int64_t n = t / p.C;
        const int ih = oh * p.sh - p.ph + r, iw = ow * p.sw - p.pw + q;
        T v = pad_value;
        if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) v = x[n * p.is[0] + c * p.is[1] + ih * p.is[2] + iw * p.is[3]];
        col[n * p.cs[0] + c * p.cs[1] + r * p.cs[2] + q * p.cs[3] + oh * p.cs[4] + ow * p.cs[5]] = v;
    }
}

// One thread per element of the image, w fastest.
template <typename T>
__global__ __launch_bounds__(256) void Col2ImKernel(ColArgs p, int64_t total) {
    using C = compute_t<T>;
    const T* col = static_cast<const T*>(p.src);
    T* out = static_cast<T*>(p.dst);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        int64_t t = idx;
        const int w = static_cast<int>(t % p.W);
        t /= p.W;
        const int h = static_cast<int>(t % p.H);
        t /= p.H;
        const int c = static_cast<int>(t % p.C);
        const int64_t n = t / p.C;
        const T* cb = col + n * p.cs[0] + c * p.cs[1];
        const int y = h + p.ph, xq = w + p.pw;  // position in the padded image
        T acc = T(0);
        for (int r = 0; r < p.kh; ++r) {
            const int yr = y - r;
            if (yr < 0) break;
            const int i = yr / p.sh;
            if (i * p.sh != yr || i >= p.OH) continue;
            for (int q = 0; q < p.kw; ++q) {
                const int xr = xq - q;
                if (xr < 0) break;
                const int j = xr / p.sw;
                if (j * p.sw != xr || j >= p.OW) continue;
                acc = static_cast<T>(static_cast<C>(acc) + static_cast<C>(cb[r * p.cs[2] + q * p.cs[3] + i * p.cs[4] + j * p.cs[5]]));
            }
        }
        out[n * p.is[0] + c * p.is[1] + h * p.is[2] + w * p.is[3]] = acc;
    }
}

int64_t ElemStrideOf(const hipcx_array* a, int axis, const char* name) {
    const int64_t it = ItemSize(a->dtype);
    HIPCX_REQUIRE(a->strides[axis] % it == 0, HIPCX_NOT_IMPLEMENTED_ERROR, std::string(name) + ": byte strides must be multiples of the item size");
    return a->strides[axis] / it;
}

dim3 GridFor(int64_t total) {
    int64_t blocks = (total + 255) / 256;
    const int64_t cap = static_cast<int64_t>(NumCUs()) * 32;
    return dim3(static_cast<unsigned>(blocks > cap ? cap : blocks));
}

ColArgs MakeColArgs(const hipcx_array* image, const hipcx_array* col, const int64_t* stride, const int64_t* pad) {
    ValidateArray(image, "image");
    ValidateArray(col, "col");
    HIPCX_REQUIRE(image->ndim == 4 && col->ndim == 6, HIPCX_NOT_IMPLEMENTED_ERROR, "im2col / col2im support 2 spatial dimensions");
    HIPCX_REQUIRE(image->dtype == col->dtype, HIPCX_DTYPE_ERROR, "im2col / col2im: the image and the col must have the same dtype");
    HIPCX_REQUIRE(stride && pad && stride[0] > 0 && stride[1] > 0 && pad[0] >= 0 && pad[1] >= 0, HIPCX_DIMENSION_ERROR, "invalid stride or pad");
    HIPCX_REQUIRE(col->shape[0] == image->shape[0] && col->shape[1] == image->shape[1], HIPCX_DIMENSION_ERROR,
                  "the col " + ShapeStr(col) + " and the image " + ShapeStr(image) + " disagree on batch size or channels");
    ColArgs p{};
    for (int i = 0; i < 4; ++i) HIPCX_REQUIRE(image->shape[i] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
    for (int i = 0; i < 6; ++i) HIPCX_REQUIRE(col->shape[i] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
    HIPCX_REQUIRE(stride[0] < (1LL << 31) && stride[1] < (1LL << 31) && pad[0] < (1LL << 31) && pad[1] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR,
                  "stride or pad too large");
    p.N = static_cast<int>(image->shape[0]);
    p.C = static_cast<int>(image->shape[1]);
    p.H = static_cast<int>(image->shape[2]);
    p.W = static_cast<int>(image->shape[3]);
    p.kh = static_cast<int>(col->shape[2]);
    p.kw = static_cast<int>(col->shape[3]);
    p.OH = static_cast<int>(col->shape[4]);
    p.OW = static_cast<int>(col->shape[5]);
    p.sh = static_cast<int>(stride[0]);
    p.sw = static_cast<int>(stride[1]);
    p.ph = static_cast<int>(pad[0]);
    p.pw = static_cast<int>(pad[1]);
    for (int i = 0; i < 4; ++i) p.is[i] = ElemStrideOf(image, i, "image");
    for (int i = 0; i < 6; ++i) p.cs[i] = ElemStrideOf(col, i, "col");
    return p;
}

void Check(int status) {
    if (status != HIPCX_OK) throw Error(status, hipcx_last_error());
}

hipcx_array Dense(void* data, int dtype, std::initializer_list<int64_t> shape) {
    hipcx_array a{};
    a.data = data;
    a.dtype = dtype;
    a.ndim = static_cast<int32_t>(shape.size());
    int i = 0;
    for (int64_t s : shape) a.shape[i++] = s;
    int64_t st = ItemSize(dtype);
    for (int d = a.ndim - 1; d >= 0; --d) {
        a.strides[d] = st;
        st *= a.shape[d];
    }
    return a;
}

// `a` with its axes in the order `axes` (a view).
hipcx_array Permuted(const hipcx_array& a, std::initializer_list<int> axes) {
    hipcx_array v = a;
    int i = 0;
    for (int ax : axes) {
        v.shape[i] = a.shape[ax];
        v.strides[i] = a.strides[ax];
        ++i;
    }
    return v;
}

size_t RoundUp(size_t v) { return (v + 255) / 256 * 256; }

enum Route { kFlippedConv, kPointwiseScatter, kProductCol2Im };

// w[ci, co, kh - 1 - r, kw - 1 - q] read as [co, ci, r, q]: a view (swapped channel axes, negative spatial strides)
hipcx_array FlippedFilters(const hipcx_array& w) {
    hipcx_array wv = Permuted(w, {1, 0, 2, 3});
    wv.data = static_cast<char*>(w.data) + (w.shape[2] - 1) * w.strides[2] + (w.shape[3] - 1) * w.strides[3];
    wv.strides[2] = -w.strides[2];
    wv.strides[3] = -w.strides[3];
    return wv;
}

struct TransposePlan {
    Route route;
    int64_t N, Ci, Co, H, W, kh, kw, OH, OW;
    // workspace layout (offsets in bytes, each a multiple of 256)
    size_t w_off = 0, x_off = 0, mid_off = 0, inner_off = 0, inner_bytes = 0, total = 0;
    hipcx_array w_copy{}, x_copy{}, mid{};  // descriptors over the workspace, data pointers relative to a base of 0
};

// Everything but the data pointers of the workspace pieces; `base` is added to them by the caller (any 256-byte aligned
// address gives the same sizes).
TransposePlan PlanTranspose(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                            const hipcx_array* out, char* base) {
    ValidateArray(x, "x");
    ValidateArray(w, "w");
    ValidateArray(out, "out");
    HIPCX_REQUIRE(x->ndim == 4 && w->ndim == 4 && out->ndim == 4, HIPCX_NOT_IMPLEMENTED_ERROR, "hip convolution supports 2 spatial dimensions");
    HIPCX_REQUIRE(stride && pad && stride[0] > 0 && stride[1] > 0 && pad[0] >= 0 && pad[1] >= 0, HIPCX_DIMENSION_ERROR, "invalid stride or pad");
    HIPCX_REQUIRE(IsFloatDtype(out->dtype) && x->dtype == out->dtype && w->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                  "conv_transpose: x and w must have out's floating point dtype (cast with hipcx_copy first)");
    HIPCX_REQUIRE(w->shape[0] == x->shape[1], HIPCX_DIMENSION_ERROR,
                  "Mismatched number of input channels in input of shape " + ShapeStr(x) + " and filter of shape " + ShapeStr(w));
    TransposePlan pl{};
    pl.N = x->shape[0];
    pl.Ci = x->shape[1];
    pl.H = x->shape[2];
    pl.W = x->shape[3];
    pl.Co = w->shape[1];
    pl.kh = w->shape[2];
    pl.kw = w->shape[3];
    pl.OH = out->shape[2];
    pl.OW = out->shape[3];
    HIPCX_REQUIRE(out->shape[0] == pl.N && out->shape[1] == pl.Co, HIPCX_DIMENSION_ERROR, "conv_transpose: out has the wrong shape " + ShapeStr(out));
    const int64_t in_dims[2] = {pl.H, pl.W}, out_dims[2] = {pl.OH, pl.OW}, k[2] = {pl.kh, pl.kw};
    for (int d = 0; d < 2; ++d) {  // CX/routines/connection.cc:268-279
        HIPCX_REQUIRE(in_dims[d] == hipcx_conv_out_dim(out_dims[d], k[d], stride[d], pad[d], 0) ||
                              in_dims[d] == hipcx_conv_out_dim(out_dims[d], k[d], stride[d], pad[d], 1),
                      HIPCX_DIMENSION_ERROR, "Output dims " + ShapeStr(out) + " is incosistent.");
    }
    if (b != nullptr) {
        ValidateArray(b, "b");
        HIPCX_REQUIRE(b->dtype == out->dtype, HIPCX_DTYPE_ERROR, "conv_transpose: b must have out's dtype");
        HIPCX_REQUIRE(b->ndim == 1 && b->shape[0] == pl.Co, HIPCX_DIMENSION_ERROR, "conv_transpose: b must hold one value per output channel");
    }
    const int dt = out->dtype;
    const size_t it = static_cast<size_t>(ItemSize(dt));
    if (stride[0] == 1 && stride[1] == 1 && pad[0] <= pl.kh - 1 && pad[1] <= pl.kw - 1 && pl.OH == pl.H - 1 + pl.kh - 2 * pad[0] &&
        pl.OW == pl.W - 1 + pl.kw - 2 * pad[1]) {
        pl.route = kFlippedConv;  // on a view of w: the convolution reads its filters through their strides, no copy
        pl.x_off = pl.mid_off = pl.inner_off = 0;
        const hipcx_array wv = FlippedFilters(*w);
        pl.inner_bytes = hipcx_conv_workspace_size(x, &wv, out);
    } else if (pl.kh == 1 && pl.kw == 1 && pad[0] == 0 && pad[1] == 0 && TotalSize(x) > 0) {
        pl.route = kPointwiseScatter;
        pl.w_copy = Dense(nullptr, dt, {pl.Co, pl.Ci, 1, 1});
        pl.mid = Dense(nullptr, dt, {pl.N, pl.Co, pl.H, pl.W});
        pl.x_off = pl.mid_off = RoundUp(static_cast<size_t>(TotalSize(&pl.w_copy)) * it);
        pl.inner_off = pl.mid_off + RoundUp(static_cast<size_t>(TotalSize(&pl.mid)) * it);
        hipcx_array wc = pl.w_copy, mc = pl.mid;
        wc.data = base + pl.w_off;
        mc.data = base + pl.mid_off;
        pl.inner_bytes = hipcx_conv_workspace_size(x, &wc, &mc);
    } else {
        pl.route = kProductCol2Im;
        pl.w_copy = Dense(nullptr, dt, {pl.Co * pl.kh * pl.kw, pl.Ci});                // w with its input channels last
        pl.x_copy = Dense(nullptr, dt, {pl.N * pl.H * pl.W, pl.Ci});                   // x channels-last
        pl.mid = Dense(nullptr, dt, {pl.Co * pl.kh * pl.kw, pl.N * pl.H * pl.W});      // the col: [C_out, kh, kw, N, H, W]
        pl.x_off = RoundUp(static_cast<size_t>(TotalSize(&pl.w_copy)) * it);
        pl.mid_off = pl.x_off + RoundUp(static_cast<size_t>(TotalSize(&pl.x_copy)) * it);
        pl.inner_off = pl.mid_off + RoundUp(static_cast<size_t>(TotalSize(&pl.mid)) * it);
        hipcx_array wc = pl.w_copy, xt = Permuted(pl.x_copy, {1, 0}), mc = pl.mid;
        wc.data = base + pl.w_off;
        xt.data = base + pl.x_off;
        mc.data = base + pl.mid_off;
        pl.inner_bytes = hipcx_dot_workspace_size(&wc, &xt, &mc);
    }
    pl.total = pl.inner_off + RoundUp(pl.inner_bytes);
    return pl;
}

void AddBias(const hipcx_array* b, const hipcx_array* out, void* stream) {
    if (b == nullptr) return;
    hipcx_array bb = *out;  // b as [1, C_out, 1, 1] broadcast to out's shape
    bb.data = b->data;
    bb.strides[0] = bb.strides[2] = bb.strides[3] = 0;
    bb.strides[1] = b->strides[0];
    Check(hipcx_add(out, &bb, out, stream));
}

}  // namespace
}  // namespace hipcx

namespace hipcx {
// nd_ops.hip: arrays without exactly two spatial axes
void ConvTransposeNd(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                     const hipcx_array* out, void* stream);
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_im2col(const hipcx_array* x, const int64_t* stride, const int64_t* pad, int cover_all, hipcx_scalar pad_value,
                 const hipcx_array* col, void* stream) {
    return Guard([&] {
        ColArgs p = MakeColArgs(x, col, stride, pad);
        HIPCX_REQUIRE(p.kh > 0 && p.kw > 0, HIPCX_DIMENSION_ERROR, "im2col: empty kernel");
        HIPCX_REQUIRE(hipcx_conv_out_dim(p.H, p.kh, p.sh, p.ph, cover_all) == p.OH && hipcx_conv_out_dim(p.W, p.kw, p.sw, p.pw, cover_all) == p.OW,
                      HIPCX_DIMENSION_ERROR, "im2col: col has the wrong shape " + ShapeStr(col));
        p.src = x->data;
        p.dst = col->data;
        const int64_t total = TotalSize(col);
        if (total == 0) return;
        VisitDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL((Im2ColKernel<T>), GridFor(total), dim3(256), 0, AsStream(stream), p, ScalarTo<T>(pad_value), total);
        });
        CheckLaunch("im2col");
    });
}

int hipcx_col2im(const hipcx_array* col, const int64_t* stride, const int64_t* pad, const hipcx_array* out, void* stream) {
    return Guard([&] {
        ColArgs p = MakeColArgs(out, col, stride, pad);
        HIPCX_REQUIRE(col->dtype != HIPCX_BOOL, HIPCX_DTYPE_ERROR, "col2im: bool arrays cannot be added");
        p.src = col->data;
        p.dst = out->data;
        const int64_t total = TotalSize(out);
        if (total == 0) return;
        VisitNumericDtype(col->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL((Col2ImKernel<T>), GridFor(total), dim3(256), 0, AsStream(stream), p, total);
        });
        CheckLaunch("col2im");
    });
}

size_t hipcx_conv_transpose_workspace_size(const hipcx_array* x, const hipcx_array* w, const int64_t* stride, const int64_t* pad,
                                           const hipcx_array* out) {
    if (x != nullptr && x->ndim != 4) return 0;  // the n-axis kernel needs none
    try {
        return PlanTranspose(x, w, nullptr, stride, pad, out, reinterpret_cast<char*>(uintptr_t{1} << 20)).total;
    } catch (...) {
        return 0;
    }
}

int hipcx_conv_transpose(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                         const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        if (x != nullptr && x->ndim != 4) {  // not two spatial axes: nd_ops.hip
            ConvTransposeNd(x, w, b, stride, pad, out, stream);
            return;
        }
        char* base = static_cast<char*>(workspace);
        TransposePlan pl = PlanTranspose(x, w, b, stride, pad, out, base != nullptr ? base : reinterpret_cast<char*>(uintptr_t{1} << 20));
        if (TotalSize(out) == 0) return;
        HIPCX_REQUIRE(pl.total == 0 || (workspace != nullptr && workspace_bytes >= pl.total), HIPCX_CHAINERX_ERROR,
                      "conv_transpose workspace too small: need " + std::to_string(pl.total) + " bytes");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 256-byte aligned");
        pl.w_copy.data = base + pl.w_off;
        pl.x_copy.data = base + pl.x_off;
        pl.mid.data = base + pl.mid_off;
        void* inner = base + pl.inner_off;
        const int64_t one[2] = {1, 1}, zero[2] = {0, 0};
        const int64_t it = ItemSize(out->dtype);
        if (pl.route == kFlippedConv) {
            const hipcx_array wv = FlippedFilters(*w);
            const int64_t fpad[2] = {pl.kh - 1 - pad[0], pl.kw - 1 - pad[1]};
            Check(hipcx_conv(x, &wv, b, one, fpad, 0, out, inner, pl.inner_bytes, stream));
            return;
        }
        if (pl.route == kPointwiseScatter) {
            const hipcx_array wv = Permuted(*w, {1, 0, 2, 3});
            Check(hipcx_copy(&wv, &pl.w_copy, stream));
            Check(hipcx_conv(x, &pl.w_copy, nullptr, one, zero, 0, &pl.mid, inner, pl.inner_bytes, stream));
            hipcx_scalar z{};
            z.kind = HIPCX_KIND_INT;
            Check(hipcx_fill(out, z, stream));
            // with cover_all output sizes the last input row / column may fall outside the output
            const int64_t hh = std::min<int64_t>(pl.H, (pl.OH + stride[0] - 1) / stride[0]);
            const int64_t ww = std::min<int64_t>(pl.W, (pl.OW + stride[1] - 1) / stride[1]);
            hipcx_array src = pl.mid, dst = *out;
            src.shape[2] = dst.shape[2] = hh;
            src.shape[3] = dst.shape[3] = ww;
            dst.strides[2] = out->strides[2] * stride[0];
            dst.strides[3] = out->strides[3] * stride[1];
            if (hh > 0 && ww > 0) Check(hipcx_copy(&src, &dst, stream));
            AddBias(b, out, stream);
            return;
        }
        // col = TensorDot(w, x) over the input channels (CX/native/native_device/conv.cc:139-141)
        hipcx_array wv = Permuted(*w, {1, 2, 3, 0});  // [C_out, kh, kw, C_in]
        hipcx_array w4 = Dense(pl.w_copy.data, out->dtype, {pl.Co, pl.kh, pl.kw, pl.Ci});
        Check(hipcx_copy(&wv, &w4, stream));
        hipcx_array xv = Permuted(*x, {0, 2, 3, 1});  // [N, H, W, C_in]
        hipcx_array x4 = Dense(pl.x_copy.data, out->dtype, {pl.N, pl.H, pl.W, pl.Ci});
        Check(hipcx_copy(&xv, &x4, stream));
        const hipcx_array xt = Permuted(pl.x_copy, {1, 0});  // [C_in, N*H*W], unit stride along the reduction
        Check(hipcx_dot(&pl.w_copy, &xt, &pl.mid, inner, pl.inner_bytes, stream));
        hipcx_array col{};  // [N, C_out, kh, kw, H, W] view of [C_out, kh, kw, N, H, W]
        col.data = pl.mid.data;
        col.dtype = out->dtype;
        col.ndim = 6;
        const int64_t shape6[6] = {pl.N, pl.Co, pl.kh, pl.kw, pl.H, pl.W};
        const int64_t plane = pl.H * pl.W * it;
        const int64_t strides6[6] = {plane, pl.kh * pl.kw * pl.N * plane, pl.kw * pl.N * plane, pl.N * plane, pl.W * it, it};
        for (int i = 0; i < 6; ++i) {
            col.shape[i] = shape6[i];
            col.strides[i] = strides6[i];
        }
        Check(hipcx_col2im(&col, stride, pad, out, stream));
        AddBias(b, out, stream);
    });
}

}  // extern "C"
