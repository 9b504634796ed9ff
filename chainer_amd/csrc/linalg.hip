// Solve, Inverse and Cholesky (SolveKernel / InverseKernel / CholeskyKernel, CX/kernels/linalg.h:20-43) for float32 / float64
// matrices.  The native backend hands these to LAPACK (gesv, getrf + getri, potrf: CX/native/native_device/linalg.cc:280-347,
// 560-600); here each is one workgroup that factorises a dense row-major copy in place:
//   * LU with partial pivoting (the first row of largest magnitude, as idamax picks it), the row operations applied to the right-hand
//     sides as they happen, then back substitution -- Inverse is the same kernel on the identity;
//   * right-looking Cholesky on the lower triangle, the strict upper triangle of the result zeroed.
// Results agree with LAPACK's to rounding (the operation order differs), not to the bit.  A zero pivot / a non-positive diagonal
// stores its 1-based position in the caller's flag, LAPACK's `info`, for the caller to raise on.
// Functional kernels: one workgroup walks the whole matrix, which is adequate for the few-hundred-row systems these routines see
// in the reference's callers (Gaussian-process and whitening layers), not for large factorizations.
#include "common.h"

namespace hipcx {
namespace {

constexpr int kLinalgThreads = 1024;

template <typename T>
__device__ __forceinline__ T AbsT(T v) {
    return v < T(0) ? -v : v;
}

// a: [n, n] row-major, destroyed.  b: [n, m] row-major, overwritten with the solution.
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void LuSolveKernel(T* a, T* b, int n, int m, int* info) {
    __shared__ T best_val[kLinalgThreads / 64];
    __shared__ int best_row[kLinalgThreads / 64];
    __shared__ int pivot_row;
    __shared__ int singular;
    const int tid = threadIdx.x;
    if (tid == 0) singular = 0;
    __syncthreads();
    for (int k = 0; k < n; ++k) {
        // pivot: first row i >= k with the largest |a[i][k]|
        T v = T(-1);
        int r = n;
        for (int i = k + tid; i < n; i += kLinalgThreads) {
            T c = AbsT(a[static_cast<int64_t>(i) * n + k]);
            if (c > v) v = c, r = i;  // rows visited in increasing order: the first maximum stays
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            T ov = __shfl_down(v, o);
            int orow = __shfl_down(r, o);
            if (ov > v || (ov == v && orow < r)) v = ov, r = orow;
        }
        if ((tid & 63) == 0) best_val[tid >> 6] = v, best_row[tid >> 6] = r;
        __syncthreads();
        if (tid == 0) {
            T bv = best_val[0];
            int br = best_row[0];
            for (int w = 1; w < kLinalgThreads / 64; ++w) {
                if (best_val[w] > bv || (best_val[w] == bv && best_row[w] < br)) bv = best_val[w], br = best_row[w];
            }
            pivot_row = br;
            if (!(bv > T(0)) && singular == 0) singular = k + 1;  // zero (or NaN) column: LAPACK's info = k + 1
        }
        __syncthreads();
        const int p = pivot_row;
        if (p != k && p < n) {
            for (int j = tid; j < n + m; j += kLinalgThreads) {
                T* row_k = j < n ? a + static_cast<int64_t>(k) * n + j : b + static_cast<int64_t>(k) * m + (j - n);
                T* row_p = j < n ? a + static_cast<int64_t>(p) * n + j : b + static_cast<int64_t>(p) * m + (j - n);
                T t = *row_k;
                *row_k = *row_p;
                *row_p = t;
            }
        }
        __syncthreads();
        const T diag = a[static_cast<int64_t>(k) * n + k];
        if (diag != T(0)) {
            // eliminate column k below the diagonal: rows i > k, columns j > k of a and all of b
            const int rows = n - k - 1;
            const int cols = n - k - 1 + m;
            const int64_t work = static_cast<int64_t>(rows) * cols;
            for (int64_t e = tid; e < work; e += kLinalgThreads) {
                const int i = k + 1 + static_cast<int>(e / cols);
                const int jj = static_cast<int>(e % cols);
                const T l = a[static_cast<int64_t>(i) * n + k] / diag;
                if (jj < n - k - 1) {
                    const int j = k + 1 + jj;
                    a[static_cast<int64_t>(i) * n + j] -= l * a[static_cast<int64_t>(k) * n + j];
                } else {
                    const int j = jj - (n - k - 1);
                    b[static_cast<int64_t>(i) * m + j] -= l * b[static_cast<int64_t>(k) * m + j];
                }
            }
        }
        __syncthreads();
    }
    if (singular != 0) {
        if (tid == 0 && info != nullptr) *info = singular;
        return;
    }
    // back substitution with the upper triangle
    for (int k = n - 1; k >= 0; --k) {
        const T diag = a[static_cast<int64_t>(k) * n + k];
        for (int j = tid; j < m; j += kLinalgThreads) b[static_cast<int64_t>(k) * m + j] /= diag;
        __syncthreads();
        const int64_t work = static_cast<int64_t>(k) * m;
        for (int64_t e = tid; e < work; e += kLinalgThreads) {
            const int i = static_cast<int>(e / m);
            const int j = static_cast<int>(e % m);
            b[static_cast<int64_t>(i) * m + j] -= a[static_cast<int64_t>(i) * n + k] * b[static_cast<int64_t>(k) * m + j];
        }
        __syncthreads();
    }
}

// l: [n, n] row-major; on entry its lower triangle holds the matrix, on exit the factor with a zero strict upper triangle.
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void CholeskyKernel(T* l, int n, int* info) {
    const int tid = threadIdx.x;
    for (int j = 0; j < n; ++j) {
        const T d = l[static_cast<int64_t>(j) * n + j];
        if (!(d > T(0))) {  // the same value for every thread: a uniform exit
            if (tid == 0 && info != nullptr) *info = j + 1;
            return;
        }
        T root;
        if constexpr (std::is_same<T, float>::value) {
            root = sqrtf(d);
        } else {
            root = sqrt(d);
        }
        __syncthreads();  // every thread has read the diagonal before it is overwritten
        if (tid == 0) l[static_cast<int64_t>(j) * n + j] = root;
        for (int i = j + 1 + tid; i < n; i += kLinalgThreads) l[static_cast<int64_t>(i) * n + j] /= root;
        __syncthreads();
        // trailing update of the lower triangle: l[i][k] -= l[i][j] * l[k][j] for j < k <= i
        const int rows = n - j - 1;
        const int64_t work = static_cast<int64_t>(rows) * rows;
        for (int64_t e = tid; e < work; e += kLinalgThreads) {
            const int i = j + 1 + static_cast<int>(e / rows);
            const int k = j + 1 + static_cast<int>(e % rows);
            if (k <= i) l[static_cast<int64_t>(i) * n + k] -= l[static_cast<int64_t>(i) * n + j] * l[static_cast<int64_t>(k) * n + j];
        }
        __syncthreads();
    }
    for (int64_t e = tid; e < static_cast<int64_t>(n) * n; e += kLinalgThreads) {
        const int i = static_cast<int>(e / n), k = static_cast<int>(e % n);
        if (k > i) l[e] = T(0);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void IdentityFillKernel(T* out, int n) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= static_cast<int64_t>(n) * n) return;
    out[e] = (e / n == e % n) ? T(1) : T(0);
}

void CheckSquare(const hipcx_array* a, const char* name) {
    ValidateArray(a, name);
    HIPCX_REQUIRE(a->ndim == 2, HIPCX_DIMENSION_ERROR, "ChainerX linear algebra routines only support 2-dimensional arrays.");
    HIPCX_REQUIRE(a->shape[0] == a->shape[1], HIPCX_DIMENSION_ERROR, "Matrix is not square.");
    HIPCX_REQUIRE(a->shape[0] < (1LL << 15), HIPCX_NOT_IMPLEMENTED_ERROR, "hip linear algebra: matrix too large");
}

void CheckLinalgDtype(int dtype, const char* what) {
    HIPCX_REQUIRE(dtype != HIPCX_FLOAT16, HIPCX_DTYPE_ERROR, std::string("Half-precision (float16) is not supported by ") + what);
    HIPCX_REQUIRE(dtype == HIPCX_FLOAT32 || dtype == HIPCX_FLOAT64, HIPCX_DTYPE_ERROR, std::string(what) + " needs floating point arrays");
}

// dense row-major [rows, cols] descriptor over `data`
hipcx_array Dense2D(void* data, int dtype, int64_t rows, int64_t cols) {
    hipcx_array d{};
    d.data = data;
    d.dtype = dtype;
    d.ndim = 2;
    d.shape[0] = rows;
    d.shape[1] = cols;
    d.strides[1] = ItemSize(dtype);
    d.strides[0] = cols * ItemSize(dtype);
    return d;
}

void CopyInto(const hipcx_array* src, const hipcx_array* dst, void* stream, const char* what) {
    int rc = hipcx_copy(src, dst, stream);
    HIPCX_REQUIRE(rc == HIPCX_OK, HIPCX_CHAINERX_ERROR, std::string(what) + ": " + hipcx_last_error());
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

size_t hipcx_solve_workspace_size(const hipcx_array* a) {
    if (a == nullptr || a->ndim != 2 || a->shape[0] < 0) return 0;
    return static_cast<size_t>(a->shape[0]) * static_cast<size_t>(a->shape[0]) * 8;
}

int hipcx_solve(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, void* workspace, size_t workspace_bytes,
                int32_t* error_flag, void* stream) {
    return Guard([&] {
        CheckSquare(a, "a");
        ValidateArray(b, "b");
        ValidateArray(out, "out");
        CheckLinalgDtype(out->dtype, "solve");
        HIPCX_REQUIRE(b->ndim == 1 || b->ndim == 2, HIPCX_DIMENSION_ERROR, "solve: b must have 1 or 2 dimensions");
        HIPCX_REQUIRE(b->shape[0] == a->shape[0], HIPCX_DIMENSION_ERROR, "solve: a and b have mismatched leading dimensions");
        HIPCX_REQUIRE(SameShape(b, out) && IsContiguous(out), HIPCX_DIMENSION_ERROR, "solve: out must be C-contiguous with b's shape");
        const int64_t n = a->shape[0], m = b->ndim == 2 ? b->shape[1] : 1;
        if (n == 0 || m == 0) return;
        HIPCX_REQUIRE(m < (1LL << 20), HIPCX_NOT_IMPLEMENTED_ERROR, "solve: too many right-hand sides");
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= static_cast<size_t>(n * n * ItemSize(out->dtype)), HIPCX_CHAINERX_ERROR,
                      "solve workspace too small");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        hipcx_array lu = Dense2D(workspace, out->dtype, n, n);
        CopyInto(a, &lu, stream, "solve: copying a");
        CopyInto(b, out, stream, "solve: copying b");
        if (out->dtype == HIPCX_FLOAT32) {
            hipLaunchKernelGGL(LuSolveKernel<float>, dim3(1), dim3(kLinalgThreads), 0, AsStream(stream), static_cast<float*>(workspace),
                               static_cast<float*>(out->data), static_cast<int>(n), static_cast<int>(m), error_flag);
        } else {
            hipLaunchKernelGGL(LuSolveKernel<double>, dim3(1), dim3(kLinalgThreads), 0, AsStream(stream), static_cast<double*>(workspace),
                               static_cast<double*>(out->data), static_cast<int>(n), static_cast<int>(m), error_flag);
        }
        CheckLaunch("solve");
    });
}

int hipcx_inverse(const hipcx_array* a, const hipcx_array* out, void* workspace, size_t workspace_bytes, int32_t* error_flag, void* stream) {
    return Guard([&] {
        CheckSquare(a, "a");
        ValidateArray(out, "out");
        CheckLinalgDtype(out->dtype, "inverse");
        HIPCX_REQUIRE(SameShape(a, out) && IsContiguous(out), HIPCX_DIMENSION_ERROR, "inverse: out must be C-contiguous with a's shape");
        const int64_t n = a->shape[0];
        if (n == 0) return;
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= static_cast<size_t>(n * n * ItemSize(out->dtype)), HIPCX_CHAINERX_ERROR,
                      "inverse workspace too small");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        hipcx_array lu = Dense2D(workspace, out->dtype, n, n);
        CopyInto(a, &lu, stream, "inverse: copying a");
        const unsigned blocks = static_cast<unsigned>((n * n + 255) / 256);
        if (out->dtype == HIPCX_FLOAT32) {
            hipLaunchKernelGGL(IdentityFillKernel<float>, dim3(blocks), dim3(256), 0, AsStream(stream), static_cast<float*>(out->data), static_cast<int>(n));
            hipLaunchKernelGGL(LuSolveKernel<float>, dim3(1), dim3(kLinalgThreads), 0, AsStream(stream), static_cast<float*>(workspace),
                               static_cast<float*>(out->data), static_cast<int>(n), static_cast<int>(n), error_flag);
        } else {
            hipLaunchKernelGGL(IdentityFillKernel<double>, dim3(blocks), dim3(256), 0, AsStream(stream), static_cast<double*>(out->data), static_cast<int>(n));
            hipLaunchKernelGGL(LuSolveKernel<double>, dim3(1), dim3(kLinalgThreads), 0, AsStream(stream), static_cast<double*>(workspace),
                               static_cast<double*>(out->data), static_cast<int>(n), static_cast<int>(n), error_flag);
        }
        CheckLaunch("inverse");
    });
}

int hipcx_cholesky(const hipcx_array* a, const hipcx_array* out, int32_t* error_flag, void* stream) {
    return Guard([&] {
        CheckSquare(a, "a");
        ValidateArray(out, "out");
        CheckLinalgDtype(out->dtype, "cholesky");
        HIPCX_REQUIRE(SameShape(a, out) && IsContiguous(out), HIPCX_DIMENSION_ERROR, "cholesky: out must be C-contiguous with a's shape");
        const int64_t n = a->shape[0];
        if (n == 0) return;
        CopyInto(a, out, stream, "cholesky: copying a");
        if (out->dtype == HIPCX_FLOAT32) {
            hipLaunchKernelGGL(CholeskyKernel<float>, dim3(1), dim3(kLinalgThreads), 0, AsStream(stream), static_cast<float*>(out->data),
                               static_cast<int>(n), error_flag);
        } else {
            hipLaunchKernelGGL(CholeskyKernel<double>, dim3(1), dim3(kLinalgThreads), 0, AsStream(stream), static_cast<double*>(out->data),
                               static_cast<int>(n), error_flag);
        }
        CheckLaunch("cholesky");
    });
}

}  // extern "C"
