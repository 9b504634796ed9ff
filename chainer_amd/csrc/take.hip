// Take (gather along one axis), CX/kernels/indexing.h:17.
//
//   out[l..., i..., r...] = a[l..., index[i...], r...]          (CX/native/native_device/indexing.cc:31-103)
//
// A pure copy, so results are bit-exact for every dtype; the kernel is instantiated per element
// size, not per dtype.  Index handling follows the native backend: negative indices count from
// the end; RAISE / DEFAULT flag an out-of-range index through `error_flag` (the caller turns it
// into IndexError), WRAP is Python's modulo, CLIP clamps to [0, dim).  When rows of `a` and
// `out` are dense and 16-byte aligned (the embedding case), a thread moves 16 bytes.
#include "common.h"

namespace hipcx {
namespace {

struct DimGroup {
    int n;
    int64_t shape[HIPCX_MAX_NDIM];
    int64_t stride_a[HIPCX_MAX_NDIM];  // bytes in the source (a or indices)
    int64_t stride_o[HIPCX_MAX_NDIM];  // bytes in out
    int64_t total;
};

struct TakeArgs {
    const char* a;
    const char* idx;
    char* out;
    DimGroup left, index, right;  // index.stride_a are the strides of the indices array
    int64_t axis_dim;
    int64_t axis_stride;  // bytes
    int idx_dtype;
    int mode;
    int axis;
    int32_t* error_flag;
    int64_t* deferred;  // used when error_flag is null (DEFAULT mode)
    int64_t total;  // work items: elements, or 16-byte vectors on the row path
    int64_t right_vecs;  // row path: 16-byte vectors per row
};

__device__ __forceinline__ void Decompose(const DimGroup& g, int64_t i, int64_t& off_a, int64_t& off_o) {
    for (int d = g.n - 1; d >= 0; --d) {
        int64_t q = i / g.shape[d];
        int64_t r = i - q * g.shape[d];
        i = q;
        off_a += r * g.stride_a[d];
        off_o += r * g.stride_o[d];
    }
}

__device__ __forceinline__ int64_t LoadIndex(const char* p, int dtype) {
    switch (dtype) {
        case HIPCX_INT8: return *reinterpret_cast<const int8_t*>(p);
        case HIPCX_INT16: return *reinterpret_cast<const int16_t*>(p);
        case HIPCX_INT32: return *reinterpret_cast<const int32_t*>(p);
        case HIPCX_UINT8: return *reinterpret_cast<const uint8_t*>(p);
        default: return *reinterpret_cast<const int64_t*>(p);
    }
}

// An out-of-range index in the DEFAULT / RAISE modes is reported and replaced by 0 (the access stays in bounds; the caller discards
// the result).  Reported where: the caller's flag, or -- deferred -- the device's sticky record {set, index, extent, axis} in
// page-locked host memory, which the next synchronising call turns into the IndexError (see DeferredIndexErrorRecord).
__device__ __forceinline__ int64_t ResolveIndex(int64_t index, int64_t dim, int mode, int32_t* error_flag, int64_t* deferred, int axis) {
    if (mode == HIPCX_BOUNDS_CLIP) {
        return index < 0 ? 0 : (index >= dim ? dim - 1 : index);
    }
    if (mode == HIPCX_BOUNDS_WRAP) {
        if (index < 0) return dim - ((-index + dim - 1) % dim + 1);
        return index % dim;
    }
    if (index < -dim || index >= dim) {
        if (error_flag != nullptr) {
            *error_flag = 1;
        } else {
            deferred[1] = index, deferred[2] = dim, deferred[3] = axis;
            deferred[0] = 1;
        }
        return 0;
    }
    return index < 0 ? index + dim : index;
}

// ROWS: dense right part moved as 16-byte vectors, no left axes, out rows dense.
template <int BYTES, bool ROWS>
__global__ __launch_bounds__(256) void TakeKernel(TakeArgs t) {
    struct alignas(BYTES) Elem {
        char b[BYTES];
    };
    for (int64_t w = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; w < t.total;
         w += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        if (ROWS) {
            int64_t i = w / t.right_vecs;
            int64_t v = w - i * t.right_vecs;
            int64_t ioff = 0, unused = 0;
            Decompose(t.index, i, ioff, unused);
            int64_t index = ResolveIndex(LoadIndex(t.idx + ioff, t.idx_dtype), t.axis_dim, t.mode, t.error_flag, t.deferred, t.axis);
            *reinterpret_cast<Elem*>(t.out + w * BYTES) = *reinterpret_cast<const Elem*>(t.a + index * t.axis_stride + v * BYTES);
        } else {
            int64_t r = w % t.right.total;
            int64_t rest = w / t.right.total;
            int64_t i = rest % t.index.total;
            int64_t l = rest / t.index.total;
            int64_t a_off = 0, o_off = 0, ioff = 0;
            Decompose(t.left, l, a_off, o_off);
            Decompose(t.right, r, a_off, o_off);
            Decompose(t.index, i, ioff, o_off);
            int64_t index = ResolveIndex(LoadIndex(t.idx + ioff, t.idx_dtype), t.axis_dim, t.mode, t.error_flag, t.deferred, t.axis);
            *reinterpret_cast<Elem*>(t.out + o_off) = *reinterpret_cast<const Elem*>(t.a + a_off + index * t.axis_stride);
        }
    }
}

// Embedding-style rows (no left axes, the right part dense on both sides): a wavefront per index, which it resolves once; its lanes
// then stream the row in BYTES-sized pieces.
template <int BYTES>
__global__ __launch_bounds__(256) void TakeRowsKernel(TakeArgs t) {
    struct alignas(BYTES) Elem {
        char b[BYTES];
    };
    const int lane = threadIdx.x & 63;
    const int64_t waves = static_cast<int64_t>(gridDim.x) * (blockDim.x >> 6);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6); i < t.index.total; i += waves) {
        int64_t ioff = 0, unused = 0;
        Decompose(t.index, i, ioff, unused);
        const int64_t index = ResolveIndex(LoadIndex(t.idx + ioff, t.idx_dtype), t.axis_dim, t.mode, t.error_flag, t.deferred, t.axis);
        const Elem* src = reinterpret_cast<const Elem*>(t.a + index * t.axis_stride);
        Elem* dst = reinterpret_cast<Elem*>(t.out + i * t.right_vecs * BYTES);
#pragma unroll 4
        for (int64_t v = lane; v < t.right_vecs; v += 64) dst[v] = src[v];
    }
}

// AddAt: out[l..., index[i...], r...] += b[l..., i..., r...] on top of a copy of `a` (indexing.cc:107-190).  One thread
// owns one (l, r) position and walks the indices in C order, so contributions to the same element are added in the
// reference's order (float results are bit-identical; float16 rounds after every addition, as Float16::operator+= does).
// In TakeArgs terms: `a` is the accumulated array (with the axis), `out` is b (with the index axes).
template <typename T>
__global__ __launch_bounds__(256) void AddAtKernel(TakeArgs t) {
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (w >= t.total) return;
    const int64_t r = w % t.right.total;
    const int64_t l = w / t.right.total;
    int64_t acc_off = 0, b_off = 0;
    Decompose(t.left, l, acc_off, b_off);
    Decompose(t.right, r, acc_off, b_off);
    char* acc_base = const_cast<char*>(t.a) + acc_off;
    for (int64_t i = 0; i < t.index.total; ++i) {
        int64_t ioff = 0, bo = b_off;
        Decompose(t.index, i, ioff, bo);
        const int64_t index = ResolveIndex(LoadIndex(t.idx + ioff, t.idx_dtype), t.axis_dim, t.mode, t.error_flag, t.deferred, t.axis);
        T* dst = reinterpret_cast<T*>(acc_base + index * t.axis_stride);
        const T bv = *reinterpret_cast<const T*>(t.out + bo);
        if constexpr (std::is_same<T, bool>::value) {
            *dst = *dst || bv;
        } else if constexpr (std::is_same<T, half_t>::value) {
            *dst = static_cast<half_t>(static_cast<float>(*dst) + static_cast<float>(bv));
        } else if constexpr (std::is_integral<T>::value) {
            using U = std::make_unsigned_t<T>;
            *dst = static_cast<T>(static_cast<U>(static_cast<U>(*dst) + static_cast<U>(bv)));
        } else {
            *dst = *dst + bv;
        }
    }
}

bool DenseGroup(const DimGroup& g, const int64_t* strides, int64_t itemsize) {
    int64_t expect = itemsize;
    for (int d = g.n - 1; d >= 0; --d) {
        if (g.shape[d] != 1 && strides[d] != expect) return false;
        expect *= g.shape[d];
    }
    return true;
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" int hipcx_take(const hipcx_array* a, const hipcx_array* indices, int8_t axis, const hipcx_array* out, int mode,
                          int32_t* error_flag, void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(indices, "indices");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(axis >= 0 && axis < a->ndim, HIPCX_DIMENSION_ERROR, "take: axis out of range");
        HIPCX_REQUIRE(indices->dtype == HIPCX_INT8 || indices->dtype == HIPCX_INT16 || indices->dtype == HIPCX_INT32 ||
                              indices->dtype == HIPCX_INT64 || indices->dtype == HIPCX_UINT8,
                      HIPCX_DTYPE_ERROR, "Only arrays of integer dtype can be used as indices.");
        HIPCX_REQUIRE(out->dtype == a->dtype, HIPCX_DTYPE_ERROR, "take: out must have a's dtype");
        HIPCX_REQUIRE(mode >= HIPCX_BOUNDS_DEFAULT && mode <= HIPCX_BOUNDS_CLIP, HIPCX_CHAINERX_ERROR, "take: invalid bounds mode");
        HIPCX_REQUIRE(error_flag != nullptr || mode != HIPCX_BOUNDS_RAISE, HIPCX_CHAINERX_ERROR,
                      "take: the raise bounds mode reports out-of-range indices through error_flag, which is null");
        HIPCX_REQUIRE(out->ndim == a->ndim - 1 + indices->ndim, HIPCX_DIMENSION_ERROR, "take: out has the wrong number of dimensions");
        TakeArgs t{};
        t.a = static_cast<const char*>(a->data);
        t.idx = static_cast<const char*>(indices->data);
        t.out = static_cast<char*>(out->data);
        t.axis_dim = a->shape[axis];
        t.axis_stride = a->strides[axis];
        t.idx_dtype = indices->dtype;
        t.mode = mode;
        t.axis = axis;
        t.error_flag = error_flag;
        if (error_flag == nullptr && mode == HIPCX_BOUNDS_DEFAULT) t.deferred = DeferredIndexErrorRecord();
        t.left.total = t.index.total = t.right.total = 1;
        int o = 0;
        for (int d = 0; d < axis; ++d, ++o) {
            HIPCX_REQUIRE(out->shape[o] == a->shape[d], HIPCX_DIMENSION_ERROR, "take: out has the wrong shape");
            t.left.shape[t.left.n] = a->shape[d];
            t.left.stride_a[t.left.n] = a->strides[d];
            t.left.stride_o[t.left.n] = out->strides[o];
            t.left.total *= a->shape[d];
            ++t.left.n;
        }
        for (int d = 0; d < indices->ndim; ++d, ++o) {
            HIPCX_REQUIRE(out->shape[o] == indices->shape[d], HIPCX_DIMENSION_ERROR, "take: out has the wrong shape");
            t.index.shape[t.index.n] = indices->shape[d];
            t.index.stride_a[t.index.n] = indices->strides[d];
            t.index.stride_o[t.index.n] = out->strides[o];
            t.index.total *= indices->shape[d];
            ++t.index.n;
        }
        for (int d = axis + 1; d < a->ndim; ++d, ++o) {
            HIPCX_REQUIRE(out->shape[o] == a->shape[d], HIPCX_DIMENSION_ERROR, "take: out has the wrong shape");
            t.right.shape[t.right.n] = a->shape[d];
            t.right.stride_a[t.right.n] = a->strides[d];
            t.right.stride_o[t.right.n] = out->strides[o];
            t.right.total *= a->shape[d];
            ++t.right.n;
        }
        int64_t total = t.left.total * t.index.total * t.right.total;
        if (total == 0) return;
        HIPCX_REQUIRE(t.axis_dim > 0, HIPCX_INDEX_ERROR, "take: cannot take from an axis of extent 0");
        const int64_t it = ItemSize(a->dtype);
        hipStream_t st = AsStream(stream);
        int64_t cap = static_cast<int64_t>(NumCUs()) * 32;

        // embedding-style rows, in the widest pieces their size and alignment allow
        const int64_t row_bytes = t.right.total * it;
        const uintptr_t misalign = static_cast<uintptr_t>(row_bytes) | static_cast<uintptr_t>(t.axis_stride < 0 ? -t.axis_stride : t.axis_stride) |
                                   reinterpret_cast<uintptr_t>(t.a) | reinterpret_cast<uintptr_t>(t.out);
        const int piece = misalign % 16 == 0 ? 16 : (misalign % 8 == 0 ? 8 : (misalign % 4 == 0 ? 4 : 0));
        const bool rows = t.left.total == 1 && piece != 0 && row_bytes > 0 && DenseGroup(t.right, t.right.stride_a, it) &&
                          DenseGroup(t.right, t.right.stride_o, it) && IsContiguous(out);
        if (rows && row_bytes / piece >= 16) {
            t.right_vecs = row_bytes / piece;
            t.total = t.index.total * t.right_vecs;
            int64_t blocks = (t.index.total + 3) / 4;
            if (blocks > cap * 4) blocks = cap * 4;
            const dim3 grid(static_cast<unsigned>(blocks)), block(256);
            if (piece == 16) hipLaunchKernelGGL(TakeRowsKernel<16>, grid, block, 0, st, t);
            else if (piece == 8) hipLaunchKernelGGL(TakeRowsKernel<8>, grid, block, 0, st, t);
            else hipLaunchKernelGGL(TakeRowsKernel<4>, grid, block, 0, st, t);
            CheckLaunch("take(rows)");
            return;
        }
        if (rows && piece == 16) {  // short rows: a thread per 16-byte piece
            t.right_vecs = row_bytes / 16;
            t.total = t.index.total * t.right_vecs;
            int64_t blocks = (t.total + 255) / 256;
            if (blocks > cap) blocks = cap;
            hipLaunchKernelGGL((TakeKernel<16, true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, t);
            CheckLaunch("take(rows)");
            return;
        }
        t.total = total;
        int64_t blocks = (total + 255) / 256;
        if (blocks > cap) blocks = cap;
        dim3 grid(static_cast<unsigned>(blocks)), block(256);
        switch (it) {
            case 1: hipLaunchKernelGGL((TakeKernel<1, false>), grid, block, 0, st, t); break;
            case 2: hipLaunchKernelGGL((TakeKernel<2, false>), grid, block, 0, st, t); break;
            case 4: hipLaunchKernelGGL((TakeKernel<4, false>), grid, block, 0, st, t); break;
            default: hipLaunchKernelGGL((TakeKernel<8, false>), grid, block, 0, st, t); break;
        }
        CheckLaunch("take");
    });
}


extern "C" int hipcx_copy(const hipcx_array* a, const hipcx_array* out, void* stream);

extern "C" int hipcx_add_at(const hipcx_array* a, const hipcx_array* indices, int8_t axis, const hipcx_array* b, const hipcx_array* out, int mode,
                            int32_t* error_flag, void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        ValidateArray(indices, "indices");
        ValidateArray(b, "b");
        HIPCX_REQUIRE(axis >= 0 && axis < a->ndim, HIPCX_DIMENSION_ERROR, "add_at: axis out of range");
        HIPCX_REQUIRE(indices->dtype == HIPCX_INT8 || indices->dtype == HIPCX_INT16 || indices->dtype == HIPCX_INT32 ||
                              indices->dtype == HIPCX_INT64 || indices->dtype == HIPCX_UINT8,
                      HIPCX_DTYPE_ERROR, "Only arrays of integer dtype can be used as indices.");
        HIPCX_REQUIRE(out->dtype == a->dtype && b->dtype == a->dtype, HIPCX_DTYPE_ERROR, "add_at: a, b and out must share a dtype");
        HIPCX_REQUIRE(mode >= HIPCX_BOUNDS_DEFAULT && mode <= HIPCX_BOUNDS_CLIP, HIPCX_CHAINERX_ERROR, "add_at: invalid bounds mode");
        HIPCX_REQUIRE(error_flag != nullptr || mode != HIPCX_BOUNDS_RAISE, HIPCX_CHAINERX_ERROR,
                      "add_at: the raise bounds mode reports out-of-range indices through error_flag, which is null");
        HIPCX_REQUIRE(SameShape(a, out), HIPCX_DIMENSION_ERROR, "add_at: out must have a's shape");
        HIPCX_REQUIRE(b->ndim == a->ndim - 1 + indices->ndim, HIPCX_DIMENSION_ERROR, "add_at: b has the wrong number of dimensions");
        TakeArgs t{};
        t.a = static_cast<const char*>(out->data);
        t.idx = static_cast<const char*>(indices->data);
        t.out = static_cast<char*>(b->data);
        t.axis_dim = out->shape[axis];
        t.axis_stride = out->strides[axis];
        t.idx_dtype = indices->dtype;
        t.mode = mode;
        t.axis = axis;
        t.error_flag = error_flag;
        if (error_flag == nullptr && mode == HIPCX_BOUNDS_DEFAULT) t.deferred = DeferredIndexErrorRecord();
        t.left.total = t.index.total = t.right.total = 1;
        int o = 0;
        for (int d = 0; d < axis; ++d, ++o) {
            HIPCX_REQUIRE(b->shape[o] == out->shape[d], HIPCX_DIMENSION_ERROR, "add_at: b has the wrong shape");
            t.left.shape[t.left.n] = out->shape[d];
            t.left.stride_a[t.left.n] = out->strides[d];
            t.left.stride_o[t.left.n] = b->strides[o];
            t.left.total *= out->shape[d];
            ++t.left.n;
        }
        for (int d = 0; d < indices->ndim; ++d, ++o) {
            HIPCX_REQUIRE(b->shape[o] == indices->shape[d], HIPCX_DIMENSION_ERROR, "add_at: b has the wrong shape");
            t.index.shape[t.index.n] = indices->shape[d];
            t.index.stride_a[t.index.n] = indices->strides[d];
            t.index.stride_o[t.index.n] = b->strides[o];
            t.index.total *= indices->shape[d];
            ++t.index.n;
        }
        for (int d = axis + 1; d < out->ndim; ++d, ++o) {
            HIPCX_REQUIRE(b->shape[o] == out->shape[d], HIPCX_DIMENSION_ERROR, "add_at: b has the wrong shape");
            t.right.shape[t.right.n] = out->shape[d];
            t.right.stride_a[t.right.n] = out->strides[d];
            t.right.stride_o[t.right.n] = b->strides[o];
            t.right.total *= out->shape[d];
            ++t.right.n;
        }
        t.total = t.left.total * t.right.total;
        const bool nothing_to_add = t.total == 0 || t.index.total == 0;
        HIPCX_REQUIRE(nothing_to_add || t.axis_dim > 0, HIPCX_INDEX_ERROR, "add_at: cannot index an axis of extent 0");
        HIPCX_REQUIRE((t.total + 255) / 256 < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "add_at: problem too large for one launch");
        // every argument is accepted: only now is out written, first as a copy of a
        int copied = hipcx_copy(a, out, stream);
        HIPCX_REQUIRE(copied == HIPCX_OK, copied, hipcx_last_error());
        if (nothing_to_add) return;
        dim3 grid(static_cast<unsigned>((t.total + 255) / 256)), block(256);
        VisitDtype(out->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            hipLaunchKernelGGL(AddAtKernel<T>, grid, block, 0, AsStream(stream), t);
        });
        CheckLaunch("add_at");
    });
}
