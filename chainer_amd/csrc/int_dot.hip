// Dot for the integer dtypes and bool (DotKernel, CX/kernels/linalg.h:13-20).  The native backend multiplies every dtype: operands
// cast to the output dtype, one accumulator of that dtype per output element, acc = a*b + acc in (i, l, j) order, and for bool
// acc = (a && b) || acc (CX/native/native_device/dot.cc:130-134, 177-227).  Integer sums do not depend on the order (arithmetic
// modulo 2^bits), so a tiled kernel reproduces them bit for bit; the cuda backend raises NotImplementedError here
// (CX/cuda/cuda_device/dot.cu:74-76).  Not an MFMA path: one 64 x 64 output tile per workgroup, 16-deep slices staged in LDS,
// 4 x 4 outputs per thread, accumulation in the unsigned type of the same width (32 bits for the narrow ones).
#include "common.h"

namespace hipcx {

namespace {

struct IntDotArgs {
    const void* a;
    const void* b;
    void* out;
    int64_t m, n, k;
    int64_t a_row, a_col, b_row, b_col, o_row, o_col;  // element strides
};

template <typename T>
struct IntAcc {
    using type = std::conditional_t<sizeof(T) == 8, uint64_t, uint32_t>;
};

constexpr int kTile = 64;
constexpr int kDepth = 16;

template <typename T>
__global__ __launch_bounds__(256) void IntDotKernel(IntDotArgs p) {
    using U = typename IntAcc<T>::type;
    __shared__ U sa[kDepth][kTile + 1];  // sa[l][i]
    __shared__ U sb[kDepth][kTile + 1];  // sb[l][j]
    const T* a = static_cast<const T*>(p.a);
    const T* b = static_cast<const T*>(p.b);
    T* out = static_cast<T*>(p.out);
    const int tid = threadIdx.x;
    const int ti = tid / 16, tj = tid % 16;  // this thread's outputs: rows ti + 16*r, columns tj + 16*c
    const int64_t i0 = static_cast<int64_t>(blockIdx.y) * kTile;
    const int64_t j0 = static_cast<int64_t>(blockIdx.x) * kTile;
    U acc[4][4] = {};
    for (int64_t l0 = 0; l0 < p.k; l0 += kDepth) {
        for (int e = tid; e < kTile * kDepth; e += 256) {
            {  // a: consecutive threads along the reduction axis
                const int l = e % kDepth, i = e / kDepth;
                const int64_t gi = i0 + i, gl = l0 + l;
                U v = 0;
                if (gi < p.m && gl < p.k) v = static_cast<U>(a[gi * p.a_row + gl * p.a_col]);
                sa[l][i] = v;
            }
            {  // b: consecutive threads along the output columns
                const int j = e % kTile, l = e / kTile;
                const int64_t gj = j0 + j, gl = l0 + l;
                U v = 0;
                if (gj < p.n && gl < p.k) v = static_cast<U>(b[gl * p.b_row + gj * p.b_col]);
                sb[l][j] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int l = 0; l < kDepth; ++l) {
            U av[4], bv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) av[r] = sa[l][ti + 16 * r];
#pragma unroll
            for (int c = 0; c < 4; ++c) bv[c] = sb[l][tj + 16 * c];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] += av[r] * bv[c];
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int64_t gi = i0 + ti + 16 * r;
        if (gi >= p.m) continue;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int64_t gj = j0 + tj + 16 * c;
            if (gj >= p.n) continue;
            if constexpr (std::is_same<T, bool>::value) {
                out[gi * p.o_row + gj * p.o_col] = acc[r][c] != 0;  // sums of at most 2^31 ones cannot wrap to zero
            } else {
                out[gi * p.o_row + gj * p.o_col] = static_cast<T>(acc[r][c]);
            }
        }
    }
}

int64_t ElemStride(const hipcx_array* a, int axis) {
    const int64_t it = ItemSize(a->dtype);
    HIPCX_REQUIRE(a->strides[axis] % it == 0, HIPCX_CHAINERX_ERROR, "dot: strides must be multiples of the item size");
    return a->strides[axis] / it;
}

}  // namespace

// a [m, k], b [k, n] and out [m, n] of one non-floating dtype, any strides; m, n, k >= 1 (the caller has handled empty extents).
void IntDot(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, hipStream_t stream) {
    IntDotArgs p;
    p.a = a->data;
    p.b = b->data;
    p.out = out->data;
    p.m = a->shape[0];
    p.k = a->shape[1];
    p.n = b->shape[1];
    p.a_row = ElemStride(a, 0), p.a_col = ElemStride(a, 1);
    p.b_row = ElemStride(b, 0), p.b_col = ElemStride(b, 1);
    p.o_row = ElemStride(out, 0), p.o_col = ElemStride(out, 1);
    const int64_t tiles_n = (p.n + kTile - 1) / kTile, tiles_m = (p.m + kTile - 1) / kTile;
    HIPCX_REQUIRE(tiles_m <= 65535, HIPCX_NOT_IMPLEMENTED_ERROR, "integer dot: more than 4194240 rows");
    VisitDtype(out->dtype, [&](auto tag) {
        using T = typename decltype(tag)::type;
        if constexpr (!std::is_floating_point<T>::value && !std::is_same<T, half_t>::value) {
            hipLaunchKernelGGL((IntDotKernel<T>), dim3(static_cast<unsigned>(tiles_n), static_cast<unsigned>(tiles_m)), dim3(256), 0, stream, p);
        } else {
            throw Error(HIPCX_DTYPE_ERROR, "IntDot: integer or bool dtype required");
        }
    });
    CheckLaunch("integer dot");
}

}  // namespace hipcx
