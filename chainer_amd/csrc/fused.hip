// Opt-in fused entries for two routine chains that the reference runs as many small kernels:
//   * LogSoftmax (CX/routines/reduction.cc:78-92): AMax, Subtract, Exp, Sum, Log, Add, Subtract -- 5 reads and 3 writes of
//     the array -- as one read + one write when a row fits in a workgroup's registers, two reads + one write otherwise;
//   * the Lstm cell (CX/routines/connection.cc:396-446): ~25 strided elementwise kernels as one.
// Both evaluate the same float operations in the same order as the chain (Exp/Tanh/Log are the same device functions the
// separate kernels call; no contraction), so for float32/float64 the Lstm cell is bit-identical to the chain and LogSoftmax
// differs only through the order of the row sum.  float16 computes in float and rounds once.
#include "common.h"

namespace hipcx {
namespace {

template <typename C>
__device__ __forceinline__ C ExpOf(C v) {
    if constexpr (std::is_same_v<C, float>) return expf(v);
    else return exp(v);
}
template <typename C>
__device__ __forceinline__ C LogOf(C v) {
    if constexpr (std::is_same_v<C, float>) return logf(v);
    else return log(v);
}
template <typename C>
__device__ __forceinline__ C TanhOf(C v) {
    if constexpr (std::is_same_v<C, float>) return tanhf(v);
    else return tanh(v);
}

// AMax's update (native/native_device/statistics.cc:27-48): NaN wins, otherwise strictly greater.
template <typename C>
__device__ __forceinline__ C MaxNan(C acc, C v) {
    return (v != v || acc < v) ? v : acc;
}

template <typename C>
__device__ __forceinline__ C ShflDown(C v, int d) {
    if constexpr (sizeof(C) == 4) {
        return __shfl_down(v, d, 64);
    } else {
        long long b = __builtin_bit_cast(long long, v);
        int lo = __shfl_down(static_cast<int>(b & 0xffffffffLL), d, 64);
        int hi = __shfl_down(static_cast<int>(b >> 32), d, 64);
        return __builtin_bit_cast(C, (static_cast<long long>(hi) << 32) | (static_cast<long long>(lo) & 0xffffffffLL));
    }
}

// Block-wide reductions for NT threads (result valid in every thread).
template <typename C, int NT, bool IS_MAX>
__device__ __forceinline__ C BlockReduce(C v, C* scratch) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        C o = ShflDown(v, d);
        v = IS_MAX ? MaxNan(v, o) : v + o;
    }
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // scratch may still be read from a previous reduction
    if ((threadIdx.x & 63) == 0) scratch[wave] = v;
    __syncthreads();
    C r = scratch[0];
#pragma unroll
    for (int w = 1; w < NT / 64; ++w) r = IS_MAX ? MaxNan(r, scratch[w]) : r + scratch[w];
    return r;
}

template <typename T, int V>
struct alignas(sizeof(T) * V) Pack {
    T e[V];
};

// ---- LogSoftmax, rows that fit in registers: one workgroup per row, VPT packs of V elements per thread ----
template <typename T, int NT, int VPT>
__global__ __launch_bounds__(NT) void LogSoftmaxRowKernel(const T* x, T* out, int64_t n, int64_t x_row, int64_t o_row, int vec_ok) {
    using C = compute_t<T>;
    constexpr int V = 16 / sizeof(T);
    __shared__ C scratch[NT / 64];
    const T* xr = x + static_cast<int64_t>(blockIdx.x) * x_row;
    T* orow = out + static_cast<int64_t>(blockIdx.x) * o_row;
    C v[VPT][V];
    const C lowest = -INFINITY;
    C m = lowest;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int64_t e0 = (static_cast<int64_t>(i) * NT + threadIdx.x) * V;
        if (vec_ok && e0 + V <= n) {
            Pack<T, V> p = *reinterpret_cast<const Pack<T, V>*>(xr + e0);
#pragma unroll
            for (int j = 0; j < V; ++j) v[i][j] = static_cast<C>(p.e[j]);
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) v[i][j] = e0 + j < n ? static_cast<C>(xr[e0 + j]) : lowest;
        }
#pragma unroll
        for (int j = 0; j < V; ++j) {
            if (e0 + j < n) m = MaxNan(m, v[i][j]);
        }
    }
    m = BlockReduce<C, NT, true>(m, scratch);
    C s = 0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int64_t e0 = (static_cast<int64_t>(i) * NT + threadIdx.x) * V;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            if (e0 + j < n) s += ExpOf<C>(v[i][j] - m);
        }
    }
    s = BlockReduce<C, NT, false>(s, scratch);
    const C lse = m + LogOf<C>(s);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int64_t e0 = (static_cast<int64_t>(i) * NT + threadIdx.x) * V;
        if (vec_ok && e0 + V <= n) {
            Pack<T, V> p;
#pragma unroll
            for (int j = 0; j < V; ++j) p.e[j] = static_cast<T>(v[i][j] - lse);
            *reinterpret_cast<Pack<T, V>*>(orow + e0) = p;
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                if (e0 + j < n) orow[e0 + j] = static_cast<T>(v[i][j] - lse);
            }
        }
    }
}

// ---- LogSoftmax, long rows: pass 1 leaves (max, sum of exp(x - max)) per (row, segment); pass 2 merges a row's
// segments, then rewrites its own segment ----
constexpr int kSegThreads = 256;

// A segment is walked in packs of 16 bytes when rows start on 16-byte boundaries (seg_len is a multiple of the pack size).
template <typename T, typename F>
__device__ __forceinline__ void ForSegment(const T* xr, int64_t lo, int64_t hi, int vec_ok, F&& f) {
    constexpr int V = 16 / sizeof(T);
    if (vec_ok) {
        const int64_t full = lo + (hi - lo) / V * V;
        for (int64_t e = lo + static_cast<int64_t>(threadIdx.x) * V; e < full; e += kSegThreads * V) {
            Pack<T, V> p = *reinterpret_cast<const Pack<T, V>*>(xr + e);
#pragma unroll
            for (int j = 0; j < V; ++j) f(e + j, p.e[j]);
        }
        for (int64_t e = full + threadIdx.x; e < hi; e += kSegThreads) f(e, xr[e]);
    } else {
        for (int64_t e = lo + threadIdx.x; e < hi; e += kSegThreads) f(e, xr[e]);
    }
}

template <typename T>
__global__ __launch_bounds__(kSegThreads) void LogSoftmaxPartialKernel(const T* x, compute_t<T>* part, int64_t n, int64_t x_row, int64_t seg_len,
                                                                       int nseg, int vec_ok) {
    using C = compute_t<T>;
    __shared__ C scratch[kSegThreads / 64];
    const int row = blockIdx.x / nseg, seg = blockIdx.x - row * nseg;
    const T* xr = x + static_cast<int64_t>(row) * x_row;
    const int64_t lo = seg * seg_len, hi = min(n, lo + seg_len);
    C m = -INFINITY;
    ForSegment<T>(xr, lo, hi, vec_ok, [&](int64_t, T v) { m = MaxNan(m, static_cast<C>(v)); });
    m = BlockReduce<C, kSegThreads, true>(m, scratch);
    C s = 0;
    ForSegment<T>(xr, lo, hi, vec_ok, [&](int64_t, T v) { s += ExpOf<C>(static_cast<C>(v) - m); });  // second walk hits L2
    s = BlockReduce<C, kSegThreads, false>(s, scratch);
    // a segment of -inf only: its terms are exp(-inf - rowmax) = 0 unless the whole row is -inf (then 0 * exp(NaN) = NaN below,
    // which is what the chain gives for such a row)
    if (m == static_cast<C>(-INFINITY)) s = 0;
    if (threadIdx.x == 0) {
        part[2 * static_cast<int64_t>(blockIdx.x)] = m;
        part[2 * static_cast<int64_t>(blockIdx.x) + 1] = s;
    }
}

template <typename T>
__global__ __launch_bounds__(kSegThreads) void LogSoftmaxApplyKernel(const T* x, T* out, const compute_t<T>* part, int64_t n, int64_t x_row,
                                                                     int64_t o_row, int64_t seg_len, int nseg, int vec_ok) {
    using C = compute_t<T>;
    constexpr int V = 16 / sizeof(T);
    __shared__ C scratch[kSegThreads / 64];
    const int row = blockIdx.x / nseg, seg = blockIdx.x - row * nseg;
    const C* pr = part + 2 * static_cast<int64_t>(row) * nseg;
    C m = -INFINITY;
    for (int i = threadIdx.x; i < nseg; i += kSegThreads) m = MaxNan(m, pr[2 * i]);
    m = BlockReduce<C, kSegThreads, true>(m, scratch);
    C s = 0;
    for (int i = threadIdx.x; i < nseg; i += kSegThreads) {
        C mi = pr[2 * i], si = pr[2 * i + 1];
        s += si * ExpOf<C>(mi - m);
    }
    s = BlockReduce<C, kSegThreads, false>(s, scratch);
    const C lse = m + LogOf<C>(s);
    const T* xr = x + static_cast<int64_t>(row) * x_row;
    T* orow = out + static_cast<int64_t>(row) * o_row;
    const int64_t lo = seg * seg_len, hi = min(n, lo + seg_len);
    if (vec_ok) {
        const int64_t full = lo + (hi - lo) / V * V;
        for (int64_t e = lo + static_cast<int64_t>(threadIdx.x) * V; e < full; e += kSegThreads * V) {
            Pack<T, V> p = *reinterpret_cast<const Pack<T, V>*>(xr + e);
#pragma unroll
            for (int j = 0; j < V; ++j) p.e[j] = static_cast<T>(static_cast<C>(p.e[j]) - lse);
            *reinterpret_cast<Pack<T, V>*>(orow + e) = p;
        }
        for (int64_t e = full + threadIdx.x; e < hi; e += kSegThreads) orow[e] = static_cast<T>(static_cast<C>(xr[e]) - lse);
    } else {
        for (int64_t e = lo + threadIdx.x; e < hi; e += kSegThreads) orow[e] = static_cast<T>(static_cast<C>(xr[e]) - lse);
    }
}

constexpr int64_t kRowInRegisters = 16384 * 4;  // bytes of a row the register kernel holds (256 threads x 16 packs x 16 bytes)
constexpr int64_t kSegmentBytes = 64 * 1024;

struct LsmShape {
    int64_t rows, n;
    int64_t x_row, o_row;  // element strides
};

LsmShape CheckLogSoftmax(const hipcx_array* x, const hipcx_array* out) {
    ValidateArray(x, "x");
    ValidateArray(out, "out");
    HIPCX_REQUIRE(IsFloatDtype(x->dtype), HIPCX_DTYPE_ERROR, std::string("log_softmax: floating point dtype required, got ") + DtypeName(x->dtype));
    HIPCX_REQUIRE(x->dtype == out->dtype, HIPCX_DTYPE_ERROR, "log_softmax: out must have x's dtype");
    HIPCX_REQUIRE(x->ndim == 2 && SameShape(x, out), HIPCX_DIMENSION_ERROR, "log_softmax: x and out must be 2-D of one shape (softmax axis 1)");
    const int64_t it = ItemSize(x->dtype);
    HIPCX_REQUIRE((x->shape[1] <= 1 || (x->strides[1] == it && out->strides[1] == it)) && x->strides[0] % it == 0 && out->strides[0] % it == 0 &&
                          x->strides[0] >= 0 && out->strides[0] >= 0,
                  HIPCX_NOT_IMPLEMENTED_ERROR, "log_softmax: rows must be dense along axis 1");
    HIPCX_REQUIRE(x->shape[0] < (1LL << 31) / 1024, HIPCX_NOT_IMPLEMENTED_ERROR, "log_softmax: too many rows for one launch");
    return LsmShape{x->shape[0], x->shape[1], x->strides[0] / it, out->strides[0] / it};
}

template <typename T>
void RunLogSoftmax(const hipcx_array* x, const hipcx_array* out, const LsmShape& sh, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    const T* xp = static_cast<const T*>(x->data);
    T* op = static_cast<T*>(out->data);
    constexpr int V = 16 / sizeof(T);
    const int vec_ok = reinterpret_cast<uintptr_t>(xp) % 16 == 0 && reinterpret_cast<uintptr_t>(op) % 16 == 0 && sh.x_row % V == 0 && sh.o_row % V == 0;
    const int64_t packs = (sh.n + V - 1) / V;
    const unsigned rows = static_cast<unsigned>(sh.rows);
    if (packs <= 64) {
        hipLaunchKernelGGL((LogSoftmaxRowKernel<T, 64, 1>), dim3(rows), dim3(64), 0, stream, xp, op, sh.n, sh.x_row, sh.o_row, vec_ok);
    } else if (packs <= 256) {
        hipLaunchKernelGGL((LogSoftmaxRowKernel<T, 256, 1>), dim3(rows), dim3(256), 0, stream, xp, op, sh.n, sh.x_row, sh.o_row, vec_ok);
    } else if (packs <= 256 * 4) {
        hipLaunchKernelGGL((LogSoftmaxRowKernel<T, 256, 4>), dim3(rows), dim3(256), 0, stream, xp, op, sh.n, sh.x_row, sh.o_row, vec_ok);
    } else if (packs <= 256 * 10) {
        hipLaunchKernelGGL((LogSoftmaxRowKernel<T, 256, 10>), dim3(rows), dim3(256), 0, stream, xp, op, sh.n, sh.x_row, sh.o_row, vec_ok);
    } else if (packs <= 256 * 16) {
        hipLaunchKernelGGL((LogSoftmaxRowKernel<T, 256, 16>), dim3(rows), dim3(256), 0, stream, xp, op, sh.n, sh.x_row, sh.o_row, vec_ok);
    } else {
        const int64_t seg_len = kSegmentBytes / static_cast<int64_t>(sizeof(T));
        const int64_t nseg = (sh.n + seg_len - 1) / seg_len;
        HIPCX_REQUIRE(sh.rows * nseg < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "log_softmax: problem too large for one launch");
        const size_t need = static_cast<size_t>(sh.rows * nseg) * 2 * sizeof(compute_t<T>);
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR,
                      "log_softmax: workspace of " + std::to_string(need) + " bytes required");
        auto* part = static_cast<compute_t<T>*>(workspace);
        const unsigned blocks = static_cast<unsigned>(sh.rows * nseg);
        hipLaunchKernelGGL(LogSoftmaxPartialKernel<T>, dim3(blocks), dim3(kSegThreads), 0, stream, xp, part, sh.n, sh.x_row, seg_len,
                           static_cast<int>(nseg), vec_ok);
        CheckLaunch("log_softmax_partial");
        hipLaunchKernelGGL(LogSoftmaxApplyKernel<T>, dim3(blocks), dim3(kSegThreads), 0, stream, xp, op, part, sh.n, sh.x_row, sh.o_row, seg_len,
                           static_cast<int>(nseg), vec_ok);
    }
    CheckLaunch("log_softmax");
}

// ---- Lstm cell ----
template <typename T>
__global__ __launch_bounds__(256) void LstmCellKernel(const T* c, const T* x, T* h_out, T* c_out, int64_t total, int H, int64_t c_row, int64_t x_row,
                                                      int64_t h_row, int64_t co_row, int vec_ok) {
    using C = compute_t<T>;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t b = idx / H;
    const int j = static_cast<int>(idx - b * H);
    const T* xg = x + b * x_row + 4 * static_cast<int64_t>(j);
    C g[4];
    if (vec_ok) {
        Pack<T, 4> p = *reinterpret_cast<const Pack<T, 4>*>(xg);
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = static_cast<C>(p.e[k]);
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = static_cast<C>(xg[k]);
    }
    // Sigmoid as the routine composes it (CX/routines/activation.cc:74-78): Reciprocal(1 + Exp(-x)) with Reciprocal = 1 / x
    auto sigmoid = [](C v) { return C(1) / (C(1) + ExpOf<C>(-v)); };
    // (the float16 chain rounds after every kernel; here the values stay in float until the two stores)
    const C a = TanhOf<C>(g[0]);
    const C i = sigmoid(g[1]);
    const C f = sigmoid(g[2]);
    const C o = sigmoid(g[3]);
    const C cprev = static_cast<C>(c[b * c_row + j]);
    const C cn = a * i + f * cprev;
    const C h = o * TanhOf<C>(cn);
    c_out[b * co_row + j] = static_cast<T>(cn);
    h_out[b * h_row + j] = static_cast<T>(h);
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

size_t hipcx_log_softmax_workspace_size(const hipcx_array* x) {
    if (x == nullptr || x->ndim != 2 || !IsFloatDtype(x->dtype)) return 0;
    const int64_t it = ItemSize(x->dtype);
    if (x->shape[1] * it <= kRowInRegisters) return 0;
    const int64_t seg_len = kSegmentBytes / it;
    const int64_t nseg = (x->shape[1] + seg_len - 1) / seg_len;
    return static_cast<size_t>(x->shape[0] * nseg) * 2 * (x->dtype == HIPCX_FLOAT64 ? 8 : 4);
}

int hipcx_log_softmax(const hipcx_array* x, const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        LsmShape sh = CheckLogSoftmax(x, out);
        if (sh.rows == 0 || sh.n == 0) return;
        VisitFloatDtype(x->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            RunLogSoftmax<T>(x, out, sh, workspace, workspace_bytes, AsStream(stream));
        });
    });
}

int hipcx_lstm_cell(const hipcx_array* c, const hipcx_array* x, const hipcx_array* h_out, const hipcx_array* c_out, void* stream) {
    return Guard([&] {
        ValidateArray(c, "c");
        ValidateArray(x, "x");
        ValidateArray(h_out, "h_out");
        ValidateArray(c_out, "c_out");
        HIPCX_REQUIRE(IsFloatDtype(c->dtype), HIPCX_DTYPE_ERROR, "Expected data type float");
        HIPCX_REQUIRE(c->dtype == x->dtype, HIPCX_DTYPE_ERROR, "Datatypes of c and x should be equal");
        HIPCX_REQUIRE(h_out->dtype == c->dtype && c_out->dtype == c->dtype, HIPCX_DTYPE_ERROR, "lstm_cell: outputs must have c's dtype");
        HIPCX_REQUIRE(c->ndim == 2 && x->ndim == 2, HIPCX_NOT_IMPLEMENTED_ERROR, "lstm_cell: 2-D c and x only");
        HIPCX_REQUIRE(x->shape[0] <= c->shape[0], HIPCX_DIMENSION_ERROR, "The batch size of x must be equal to or less than the size of c");
        HIPCX_REQUIRE(x->shape[1] == 4 * c->shape[1], HIPCX_DIMENSION_ERROR,
                      "Expected dimension at axis 1 of x to be equal 4 times dimension at axis 1 of c.");
        HIPCX_REQUIRE(x->shape[0] == c->shape[0], HIPCX_NOT_IMPLEMENTED_ERROR, "lstm_cell: ragged batches are not on the supported path");
        HIPCX_REQUIRE(SameShape(h_out, c) && SameShape(c_out, c), HIPCX_DIMENSION_ERROR, "lstm_cell: outputs must have c's shape");
        const int64_t it = ItemSize(c->dtype);
        auto dense_rows = [&](const hipcx_array* a) {
            return (a->shape[1] <= 1 || a->strides[1] == it) && a->strides[0] % it == 0 && a->strides[0] >= 0;
        };
        HIPCX_REQUIRE(dense_rows(c) && dense_rows(x) && dense_rows(h_out) && dense_rows(c_out), HIPCX_NOT_IMPLEMENTED_ERROR,
                      "lstm_cell: rows must be dense along axis 1");
        const int64_t B = c->shape[0], H = c->shape[1];
        const int64_t total = B * H;
        if (total == 0) return;
        HIPCX_REQUIRE(H < (1LL << 31) && (total + 255) / 256 < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "lstm_cell: problem too large for one launch");
        const int vec_ok = reinterpret_cast<uintptr_t>(x->data) % (4 * it) == 0 && x->strides[0] % (4 * it) == 0;
        VisitFloatDtype(c->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL(LstmCellKernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, AsStream(stream),
                               static_cast<const T*>(c->data), static_cast<const T*>(x->data), static_cast<T*>(h_out->data),
                               static_cast<T*>(c_out->data), total, static_cast<int>(H), c->strides[0] / it, x->strides[0] / it,
                               h_out->strides[0] / it, c_out->strides[0] / it, vec_ok);
        });
        CheckLaunch("lstm_cell");
    });
}

}  // extern "C"
