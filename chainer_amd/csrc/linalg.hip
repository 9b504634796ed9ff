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

// Symmetric eigendecomposition by cyclic Jacobi rotations, one workgroup.  s: [n, n] row-major, symmetric on entry, destroyed
// (its diagonal converges to the eigenvalues); v: [n, n] accumulates the rotations (eigenvectors as columns); w: the eigenvalues in
// ascending order, with the columns of v permuted to match (LAPACK syevd's order, CX/native/native_device/linalg.cc:602-660).
// A sweep visits all pairs in n - 1 rounds of n / 2 disjoint pairs (round-robin pairing), so the rotations of a round apply in
// parallel: first to the columns of s and v, then to the rows of s.
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void JacobiEighKernel(T* s, T* v, T* w, int n, int compute_v, int64_t v_row, int64_t v_col,
                                                                   int64_t w_stride, T* v_scratch) {
    extern __shared__ __align__(16) char eigh_lds[];
    T* cs = reinterpret_cast<T*>(eigh_lds);             // [half][2]: cosine, sine of the round's rotations
    int* pq = reinterpret_cast<int*>(cs + 2 * ((n + 1) / 2));  // [half][2]: the pairs
    __shared__ T red[kLinalgThreads / 64];
    __shared__ T off_norm, total_norm;
    const int tid = threadIdx.x;
    const int np = n + (n & 1);  // players of the round-robin schedule (one dummy when n is odd)
    const int half = np / 2;
    const int m = np - 1;
    for (int64_t e = tid; e < static_cast<int64_t>(n) * n; e += kLinalgThreads) v_scratch[e] = (e / n == e % n) ? T(1) : T(0);
    __syncthreads();
    auto block_sum = [&](T x) -> T {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) x += __shfl_down(x, o);
        __syncthreads();
        if ((tid & 63) == 0) red[tid >> 6] = x;
        __syncthreads();
        T r = T(0);
        for (int k = 0; k < kLinalgThreads / 64; ++k) r += red[k];
        return r;  // every thread adds the same partials
    };
    {
        T acc = T(0);
        for (int64_t e = tid; e < static_cast<int64_t>(n) * n; e += kLinalgThreads) acc += s[e] * s[e];
        T t = block_sum(acc);
        if (tid == 0) total_norm = t;
        __syncthreads();
    }
    const T eps = std::is_same<T, float>::value ? T(4e-7) : T(1e-15);  // relative off-diagonal norm at which rounding dominates
    for (int sweep = 0; sweep < 60; ++sweep) {
        T acc = T(0);
        for (int64_t e = tid; e < static_cast<int64_t>(n) * n; e += kLinalgThreads) {
            if (e / n != e % n) acc += s[e] * s[e];
        }
        T t = block_sum(acc);
        if (tid == 0) off_norm = t;
        __syncthreads();
        if (!(off_norm > eps * eps * total_norm)) break;  // uniform: every thread reads the same value
        for (int round = 0; round < m; ++round) {
            // the round's rotations
            for (int i = tid; i < half; i += kLinalgThreads) {
                int p = i == 0 ? m : (round + i) % m;
                int q = i == 0 ? round % m : (round - i + m) % m;
                if (p > q) { int t2 = p; p = q; q = t2; }
                T c = T(1), sn = T(0);
                if (q < n) {
                    const T apq = s[static_cast<int64_t>(p) * n + q];
                    if (apq != T(0)) {
                        const T app = s[static_cast<int64_t>(p) * n + p], aqq = s[static_cast<int64_t>(q) * n + q];
                        const T tau = (aqq - app) / (T(2) * apq);
                        const T root = std::is_same<T, float>::value ? T(sqrtf(static_cast<float>(T(1) + tau * tau))) : T(sqrt(static_cast<double>(T(1) + tau * tau)));
                        const T tt = (tau >= T(0) ? T(1) : T(-1)) / ((tau >= T(0) ? tau : -tau) + root);
                        c = T(1) / (std::is_same<T, float>::value ? T(sqrtf(static_cast<float>(T(1) + tt * tt))) : T(sqrt(static_cast<double>(T(1) + tt * tt))));
                        sn = tt * c;
                    }
                } else {
                    q = -1;  // the dummy player: no rotation
                }
                cs[2 * i] = c, cs[2 * i + 1] = sn;
                pq[2 * i] = p, pq[2 * i + 1] = q;
            }
            __syncthreads();
            // columns of s and of v: x[:, p], x[:, q] <- c x[:, p] - s x[:, q], s x[:, p] + c x[:, q]
            for (int64_t e = tid; e < static_cast<int64_t>(half) * n; e += kLinalgThreads) {
                const int r = static_cast<int>(e / half), i = static_cast<int>(e % half);  // neighbours share a row of s
                const int p = pq[2 * i], q = pq[2 * i + 1];
                if (q < 0) continue;
                const T c = cs[2 * i], sn = cs[2 * i + 1];
                T* sp = s + static_cast<int64_t>(r) * n;
                const T a = sp[p], b = sp[q];
                sp[p] = c * a - sn * b;
                sp[q] = sn * a + c * b;
                T* vp = v_scratch + static_cast<int64_t>(r) * n;
                const T va = vp[p], vb = vp[q];
                vp[p] = c * va - sn * vb;
                vp[q] = sn * va + c * vb;
            }
            __syncthreads();
            // rows of s
            for (int64_t e = tid; e < static_cast<int64_t>(half) * n; e += kLinalgThreads) {
                const int i = static_cast<int>(e / n), r = static_cast<int>(e % n);
                const int p = pq[2 * i], q = pq[2 * i + 1];
                if (q < 0) continue;
                const T c = cs[2 * i], sn = cs[2 * i + 1];
                const T a = s[static_cast<int64_t>(p) * n + r], b = s[static_cast<int64_t>(q) * n + r];
                // the rotated pair's own off-diagonal entry is zero by construction: storing the exact zero keeps rounding noise of the
                // size of the eigenvalues out of the off-diagonal part, which is what lets the sweeps converge to the threshold
                s[static_cast<int64_t>(p) * n + r] = r == q ? T(0) : c * a - sn * b;
                s[static_cast<int64_t>(q) * n + r] = r == p ? T(0) : sn * a + c * b;
            }
            __syncthreads();
        }
    }
    // ascending order: rank of every diagonal entry (ties by index), then scatter
    for (int i = tid; i < n; i += kLinalgThreads) {
        const T wi = s[static_cast<int64_t>(i) * n + i];
        int rank = 0;
        for (int j = 0; j < n; ++j) {
            const T wj = s[static_cast<int64_t>(j) * n + j];
            if (wj < wi || (wj == wi && j < i)) ++rank;
        }
        w[rank * w_stride] = wi;
        if (compute_v) {
            for (int r = 0; r < n; ++r) v[r * v_row + rank * v_col] = v_scratch[static_cast<int64_t>(r) * n + i];
        }
    }
}

// s[i][j] <- a read from the chosen triangle (upper: a[min][max], lower: a[max][min]), cast is the caller's.
template <typename T>
__global__ __launch_bounds__(256) void SymmetrizeKernel(const T* a, int64_t a_row, int64_t a_col, T* s, int n, int upper) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= static_cast<int64_t>(n) * n) return;
    const int i = static_cast<int>(e / n), j = static_cast<int>(e % n);
    const int lo = i < j ? i : j, hi = i < j ? j : i;
    s[e] = upper ? a[lo * a_row + hi * a_col] : a[hi * a_row + lo * a_col];
}

// y[i][c] -= tau * v[i] * (sum over i of v[i] * y[i][c]) for rows i in [j, m) and columns c in [c_begin, c_end): the Householder
// reflector H = I - tau v v^T with v[j] = 1 and v[i > j] = w[i][j] (LAPACK's storage), applied from the left.  Whole workgroup,
// 64 columns at a time with 16 row groups whose partial sums meet in LDS.
template <typename T>
__device__ void ApplyReflector(const T* w, int n, int j, int m, T tau, T* y, int64_t y_row, int64_t y_col, int c_begin, int c_end, T* part) {
    const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
    constexpr int kGroups = kLinalgThreads / 64;
    for (int c0 = c_begin; c0 < c_end; c0 += 64) {  // uniform bounds: every thread reaches every barrier
        const int c = c0 + tx;
        T acc = T(0);
        if (c < c_end) {
            for (int i = j + ty; i < m; i += kGroups) {
                const T vi = i == j ? T(1) : w[static_cast<int64_t>(i) * n + j];
                acc += vi * y[i * y_row + c * y_col];
            }
        }
        part[ty * 64 + tx] = acc;
        __syncthreads();
        T total = T(0);
#pragma unroll
        for (int g = 0; g < kGroups; ++g) total += part[g * 64 + tx];
        total *= tau;
        if (c < c_end) {
            for (int i = j + ty; i < m; i += kGroups) {
                const T vi = i == j ? T(1) : w[static_cast<int64_t>(i) * n + j];
                y[i * y_row + c * y_col] -= vi * total;
            }
        }
        __syncthreads();
    }
}

template <typename T>
__device__ inline T SqrtT(T x) {
    return std::is_same<T, float>::value ? T(sqrtf(static_cast<float>(x))) : T(sqrt(static_cast<double>(x)));
}

// Householder QR in place, LAPACK geqrf's result: R on and above the diagonal of w ([m, n] row-major), the reflector vectors below
// it (v[j] = 1 implied), tau[j] their scalars; reflector j is larfg's: beta = -sign(alpha) * norm(column), tau = (beta - alpha) /
// beta, v = x / (alpha - beta), tau = 0 where the column is already zero below the diagonal.
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void HouseholderQrKernel(T* w, int m, int n, T* tau, int64_t tau_stride) {
    __shared__ T part[kLinalgThreads];
    __shared__ T red[kLinalgThreads / 64];
    __shared__ T sh_tau, sh_scale, sh_beta;
    const int tid = threadIdx.x;
    const int k = m < n ? m : n;
    for (int j = 0; j < k; ++j) {
        T acc = T(0);
        for (int i = j + 1 + tid; i < m; i += kLinalgThreads) {
            const T x = w[static_cast<int64_t>(i) * n + j];
            acc += x * x;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o);
        if ((tid & 63) == 0) red[tid >> 6] = acc;
        __syncthreads();
        if (tid == 0) {
            T xnorm2 = T(0);
            for (int g = 0; g < kLinalgThreads / 64; ++g) xnorm2 += red[g];
            const T alpha = w[static_cast<int64_t>(j) * n + j];
            if (xnorm2 == T(0)) {
                sh_tau = T(0), sh_scale = T(0), sh_beta = alpha;
            } else {
                const T norm = SqrtT(alpha * alpha + xnorm2);
                const T beta = alpha >= T(0) ? -norm : norm;
                sh_tau = (beta - alpha) / beta;
                sh_scale = T(1) / (alpha - beta);
                sh_beta = beta;
            }
            tau[j * tau_stride] = sh_tau;
        }
        __syncthreads();
        const T t = sh_tau;
        if (t != T(0)) {  // uniform
            const T scale = sh_scale;
            for (int i = j + 1 + tid; i < m; i += kLinalgThreads) w[static_cast<int64_t>(i) * n + j] *= scale;
            if (tid == 0) w[static_cast<int64_t>(j) * n + j] = sh_beta;
            __syncthreads();
            ApplyReflector(w, n, j, m, t, w, static_cast<int64_t>(n), int64_t{1}, j + 1, n, part);
        }
        __syncthreads();
    }
}

// q[m, mc] = H_0 H_1 ... H_{k-1} applied to the first mc columns of the identity (LAPACK orgqr), reflectors read from w / tau.
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void FormQKernel(const T* w, int m, int n, const T* tau, int64_t tau_stride, T* q, int64_t q_row,
                                                              int64_t q_col, int mc) {
    __shared__ T part[kLinalgThreads];
    const int tid = threadIdx.x;
    const int k = m < n ? m : n;
    for (int64_t e = tid; e < static_cast<int64_t>(m) * mc; e += kLinalgThreads) {
        const int64_t i = e / mc, c = e % mc;
        q[i * q_row + c * q_col] = i == c ? T(1) : T(0);
    }
    __syncthreads();
    for (int j = k - 1; j >= 0; --j) {
        const T t = tau[j * tau_stride];
        if (t != T(0)) ApplyReflector(w, n, j, m, t, q, q_row, q_col, j, mc, part);  // columns before j are still the identity's
    }
}

// r[i][c] = w[i][c] on and above the diagonal, 0 below (rows i < r_rows); or, raw, r[c][i] = w[i][c] (the column-major factored matrix)
template <typename T>
__global__ __launch_bounds__(256) void ExtractRKernel(const T* w, int m, int n, T* r, int64_t r_row, int64_t r_col, int r_rows, int raw) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t rows = raw ? m : r_rows;
    if (e >= rows * n) return;
    const int64_t i = e / n, c = e % n;
    if (raw) r[c * r_row + i * r_col] = w[e];
    else r[i * r_row + c * r_col] = (c >= i && i < m) ? w[i * n + c] : T(0);
}

// Singular value decomposition by one-sided Jacobi rotations (Hestenes), one workgroup.  g: [M, N] row-major with M >= N, destroyed:
// its columns are rotated in pairs until they are mutually orthogonal, then their norms are the singular values and the normalised
// columns the left vectors; v: [N, N] accumulates the rotations (right vectors as columns).  Results leave in descending order of
// the singular value: s[rank], tall(i, rank) = g[i][j] / sigma_j, sq(i, rank) = v[i][j], both addressed through (row, col)
// element strides so that the caller decides which of u / vt each one is and how it is transposed.  Columns whose singular value
// is zero are left for the completion kernel; *first_fill receives the number of columns that are final.
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void JacobiSvdKernel(T* g, int M, int N, T* v, T* sigma, int* rank, T* s_out, int64_t s_stride,
                                                                  T* tall, int64_t tall_row, int64_t tall_col, T* sq, int64_t sq_row,
                                                                  int64_t sq_col, int compute_uv, int* first_fill) {
    constexpr int kGroups = kLinalgThreads / 64;
    __shared__ T part[3 * kLinalgThreads];
    __shared__ T cs[2 * 64];
    __shared__ int rotated, zeros;
    const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
    const int np = N + (N & 1), half = np / 2, rounds = np - 1;
    if (compute_uv) {
        for (int64_t e = tid; e < static_cast<int64_t>(N) * N; e += kLinalgThreads) v[e] = (e / N == e % N) ? T(1) : T(0);
    }
    const T tol = SqrtT(static_cast<T>(M)) * (std::is_same<T, float>::value ? T(1.2e-7) : T(2.3e-16));
    __syncthreads();
    for (int sweep = 0; sweep < 60; ++sweep) {
        if (tid == 0) rotated = 0;
        __syncthreads();
        for (int round = 0; round < rounds; ++round) {
            for (int c0 = 0; c0 < half; c0 += 64) {  // uniform bounds
                const int idx = c0 + tx;
                int p = 0, q = -1;
                if (idx < half) {
                    p = idx == 0 ? rounds : (round + idx) % rounds;
                    q = idx == 0 ? round % rounds : (round - idx + rounds) % rounds;
                    if (p > q) { const int t2 = p; p = q; q = t2; }
                    if (q >= N) q = -1;  // the dummy player of an odd N
                }
                T alpha = T(0), beta = T(0), gamma = T(0);
                if (q >= 0) {
                    for (int i = ty; i < M; i += kGroups) {
                        const T a = g[static_cast<int64_t>(i) * N + p], b = g[static_cast<int64_t>(i) * N + q];
                        alpha += a * a, beta += b * b, gamma += a * b;
                    }
                }
                part[ty * 64 + tx] = alpha;
                part[kLinalgThreads + ty * 64 + tx] = beta;
                part[2 * kLinalgThreads + ty * 64 + tx] = gamma;
                __syncthreads();
                if (ty == 0) {
                    alpha = beta = gamma = T(0);
#pragma unroll
                    for (int k2 = 0; k2 < kGroups; ++k2) {
                        alpha += part[k2 * 64 + tx];
                        beta += part[kLinalgThreads + k2 * 64 + tx];
                        gamma += part[2 * kLinalgThreads + k2 * 64 + tx];
                    }
                    T c = T(1), sn = T(0);
                    const T abs_gamma = gamma >= T(0) ? gamma : -gamma;
                    if (q >= 0 && abs_gamma > tol * SqrtT(alpha * beta) && abs_gamma > T(0)) {
                        const T zeta = (beta - alpha) / (T(2) * gamma);
                        const T tt = (zeta >= T(0) ? T(1) : T(-1)) / ((zeta >= T(0) ? zeta : -zeta) + SqrtT(T(1) + zeta * zeta));
                        c = T(1) / SqrtT(T(1) + tt * tt);
                        sn = c * tt;
                        rotated = 1;  // every writer stores the same value
                    }
                    cs[2 * tx] = c, cs[2 * tx + 1] = sn;
                }
                __syncthreads();
                const T c = cs[2 * tx], sn = cs[2 * tx + 1];
                if (q >= 0 && sn != T(0)) {
                    for (int i = ty; i < M; i += kGroups) {
                        T* row = g + static_cast<int64_t>(i) * N;
                        const T a = row[p], b = row[q];
                        row[p] = c * a - sn * b;
                        row[q] = sn * a + c * b;
                    }
                    if (compute_uv) {
                        for (int i = ty; i < N; i += kGroups) {
                            T* row = v + static_cast<int64_t>(i) * N;
                            const T a = row[p], b = row[q];
                            row[p] = c * a - sn * b;
                            row[q] = sn * a + c * b;
                        }
                    }
                }
                __syncthreads();
            }
        }
        const int any = rotated;
        __syncthreads();
        if (!any) break;
    }
    // singular values: the column norms
    for (int j = tid; j < N; j += kLinalgThreads) {
        T acc = T(0);
        for (int i = 0; i < M; ++i) {
            const T x = g[static_cast<int64_t>(i) * N + j];
            acc += x * x;
        }
        sigma[j] = SqrtT(acc);
    }
    if (tid == 0) zeros = 0;
    __syncthreads();
    T sigma_max = T(0);
    for (int j = 0; j < N; ++j) sigma_max = sigma[j] > sigma_max ? sigma[j] : sigma_max;
    const T floor_value = sigma_max * T(1e-30);
    for (int j = tid; j < N; j += kLinalgThreads) {
        const T sj = sigma[j];
        int r = 0;
        for (int l = 0; l < N; ++l) {
            const T sl = sigma[l];
            if (sl > sj || (sl == sj && l < j)) ++r;
        }
        rank[j] = r;
        s_out[r * s_stride] = sj;
        if (!(sj > floor_value)) atomicAdd(&zeros, 1);
    }
    __syncthreads();
    if (tid == 0) *first_fill = N - zeros;
    if (!compute_uv) return;
    for (int64_t e = tid; e < static_cast<int64_t>(M) * N; e += kLinalgThreads) {
        const int64_t i = e / N, j = e % N;
        const T sj = sigma[j];
        tall[i * tall_row + rank[j] * tall_col] = sj > floor_value ? g[e] / sj : T(0);
    }
    for (int64_t e = tid; e < static_cast<int64_t>(N) * N; e += kLinalgThreads) {
        const int64_t i = e / N, j = e % N;
        sq[i * sq_row + rank[j] * sq_col] = v[e];
    }
}

// Columns [*first_fill, cols) of tall ([M, cols], (row, col) element strides) become an orthonormal completion of the columns
// before them: unit vectors e_0, e_1, ... are orthogonalised against everything present (classical Gram-Schmidt, twice) and kept
// when enough of them is left; each candidate is tried once, which always suffices (the squared residuals of all candidates add
// up to the number of missing columns).
template <typename T>
__global__ __launch_bounds__(kLinalgThreads) void CompleteBasisKernel(T* tall, int64_t tall_row, int64_t tall_col, int M, int cols,
                                                                      const int* first_fill, T* dots) {
    __shared__ T red[kLinalgThreads / 64];
    __shared__ T sh_norm2;
    const int tid = threadIdx.x;
    int cand = 0;
    const T keep = T(1) / (T(4) * static_cast<T>(M));
    for (int col = *first_fill; col < cols; ++col) {
        bool done = false;
        while (!done && cand < M) {  // uniform: cand, col and the norm are the same in every thread
            for (int i = tid; i < M; i += kLinalgThreads) tall[i * tall_row + col * tall_col] = i == cand ? T(1) : T(0);
            __syncthreads();
            for (int pass = 0; pass < 2; ++pass) {
                for (int e = tid; e < col; e += kLinalgThreads) {
                    T acc = T(0);
                    for (int i = 0; i < M; ++i) acc += tall[i * tall_row + e * tall_col] * tall[i * tall_row + col * tall_col];
                    dots[e] = acc;
                }
                __syncthreads();
                for (int i = tid; i < M; i += kLinalgThreads) {
                    T acc = T(0);
                    for (int e = 0; e < col; ++e) acc += tall[i * tall_row + e * tall_col] * dots[e];
                    tall[i * tall_row + col * tall_col] -= acc;
                }
                __syncthreads();
            }
            T acc = T(0);
            for (int i = tid; i < M; i += kLinalgThreads) {
                const T x = tall[i * tall_row + col * tall_col];
                acc += x * x;
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o);
            if ((tid & 63) == 0) red[tid >> 6] = acc;
            __syncthreads();
            if (tid == 0) {
                T t = T(0);
                for (int k2 = 0; k2 < kLinalgThreads / 64; ++k2) t += red[k2];
                sh_norm2 = t;
            }
            __syncthreads();
            const T norm2 = sh_norm2;
            if (norm2 >= keep) {
                const T inv = T(1) / SqrtT(norm2);
                for (int i = tid; i < M; i += kLinalgThreads) tall[i * tall_row + col * tall_col] *= inv;
                done = true;
            }
            ++cand;
            __syncthreads();
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void StridedIdentityKernel(T* out, int64_t row, int64_t col, int n) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= static_cast<int64_t>(n) * n) return;
    out[(e / n) * row + (e % n) * col] = (e / n == e % n) ? T(1) : T(0);
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

size_t hipcx_syevd_workspace_size(const hipcx_array* a) {
    if (a == nullptr || a->ndim != 2 || a->shape[0] < 0) return 0;
    return static_cast<size_t>(a->shape[0]) * static_cast<size_t>(a->shape[0]) * 8 * 2;  // the working copy and the rotations
}

int hipcx_syevd(const hipcx_array* a, const hipcx_array* w, const hipcx_array* v, char uplo, int compute_v, void* workspace,
                size_t workspace_bytes, void* stream) {
    return Guard([&] {
        CheckSquare(a, "a");
        ValidateArray(w, "w");
        ValidateArray(v, "v");
        CheckLinalgDtype(a->dtype, "eigh");
        HIPCX_REQUIRE(uplo == 'U' || uplo == 'u' || uplo == 'L' || uplo == 'l', HIPCX_CHAINERX_ERROR, "eigh: uplo must be 'U' or 'L'");
        HIPCX_REQUIRE(w->dtype == a->dtype && v->dtype == a->dtype, HIPCX_DTYPE_ERROR, "eigh: w and v must have a's dtype");
        const int64_t n = a->shape[0];
        HIPCX_REQUIRE(w->ndim == 1 && w->shape[0] == n, HIPCX_DIMENSION_ERROR, "eigh: w must have one entry per row of a");
        HIPCX_REQUIRE(!compute_v || (v->ndim == 2 && v->shape[0] == n && v->shape[1] == n), HIPCX_DIMENSION_ERROR, "eigh: v must have a's shape");
        if (n == 0) return;
        HIPCX_REQUIRE(n <= 4096, HIPCX_NOT_IMPLEMENTED_ERROR, "hip eigh: matrix too large for the one-workgroup Jacobi kernel");
        const int64_t it = ItemSize(a->dtype);
        const size_t need = static_cast<size_t>(n * n * it) * 2;
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR, "eigh workspace too small");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        const int upper = (uplo == 'U' || uplo == 'u') ? 1 : 0;
        const unsigned blocks = static_cast<unsigned>((n * n + 255) / 256);
        const size_t lds = static_cast<size_t>((n + 1) / 2) * (2 * it + 2 * sizeof(int)) + 16;
        hipStream_t st = AsStream(stream);
        char* ws = static_cast<char*>(workspace);
        auto run = [&](auto tag) {
            using T = decltype(tag);
            T* s = reinterpret_cast<T*>(ws);
            T* vs = reinterpret_cast<T*>(ws + n * n * it);
            hipLaunchKernelGGL(SymmetrizeKernel<T>, dim3(blocks), dim3(256), 0, st, static_cast<const T*>(a->data), a->strides[0] / it,
                               a->strides[1] / it, s, static_cast<int>(n), upper);
            hipLaunchKernelGGL(JacobiEighKernel<T>, dim3(1), dim3(kLinalgThreads), lds, st, s, static_cast<T*>(v->data),
                               static_cast<T*>(w->data), static_cast<int>(n), compute_v ? 1 : 0, compute_v ? v->strides[0] / it : 0,
                               compute_v ? v->strides[1] / it : 0, w->strides[0] / it, vs);
        };
        if (a->dtype == HIPCX_FLOAT32) run(float{});
        else run(double{});
        CheckLaunch("eigh");
    });
}

size_t hipcx_qr_workspace_size(const hipcx_array* a) {
    if (a == nullptr || a->ndim != 2 || a->shape[0] < 0 || a->shape[1] < 0) return 0;
    return static_cast<size_t>(a->shape[0]) * static_cast<size_t>(a->shape[1]) * 8 + 256;  // the factored copy
}

int hipcx_qr(const hipcx_array* a, const hipcx_array* q, const hipcx_array* r, const hipcx_array* tau, int mode, void* workspace,
             size_t workspace_bytes, void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(r, "r");
        ValidateArray(tau, "tau");
        HIPCX_REQUIRE(a->ndim == 2, HIPCX_DIMENSION_ERROR, "ChainerX linear algebra routines only support 2-dimensional arrays.");
        HIPCX_REQUIRE(mode >= HIPCX_QR_REDUCED && mode <= HIPCX_QR_RAW, HIPCX_CHAINERX_ERROR, "Invalid QR mode");
        const int dtype = r->dtype;
        CheckLinalgDtype(dtype, "QR decomposition");
        const int64_t m = a->shape[0], n = a->shape[1], k = std::min(m, n);
        HIPCX_REQUIRE(m < (1LL << 15) && n < (1LL << 15), HIPCX_NOT_IMPLEMENTED_ERROR, "hip linear algebra: matrix too large");
        HIPCX_REQUIRE(tau->dtype == dtype && tau->ndim == 1 && tau->shape[0] == k, HIPCX_DIMENSION_ERROR, "qr: tau must hold min(m, n) values of r's dtype");
        const bool want_q = mode == HIPCX_QR_REDUCED || mode == HIPCX_QR_COMPLETE;
        const int64_t mc = (mode == HIPCX_QR_COMPLETE && m > n) ? m : k;
        const int64_t r_rows = mode == HIPCX_QR_RAW ? n : (want_q ? mc : k), r_cols = mode == HIPCX_QR_RAW ? m : n;
        HIPCX_REQUIRE(r->ndim == 2 && r->shape[0] == r_rows && r->shape[1] == r_cols, HIPCX_DIMENSION_ERROR, "qr: r has the wrong shape for this mode");
        if (want_q) {
            ValidateArray(q, "q");
            HIPCX_REQUIRE(q->dtype == dtype && q->ndim == 2 && q->shape[0] == m && q->shape[1] == mc, HIPCX_DIMENSION_ERROR,
                          "qr: q has the wrong shape or dtype for this mode");
        }
        const int64_t it = ItemSize(dtype);
        hipStream_t st = AsStream(stream);
        if (m == 0 || n == 0) {
            // nothing to factor; a complete q of an [m, 0] matrix is the identity
            if (want_q && m > 0 && mc > 0) {
                auto fill = [&](auto tag) {
                    using T = decltype(tag);
                    hipLaunchKernelGGL(FormQKernel<T>, dim3(1), dim3(kLinalgThreads), 0, st, static_cast<const T*>(nullptr), static_cast<int>(m), 0,
                                       static_cast<const T*>(nullptr), int64_t{1}, static_cast<T*>(q->data), q->strides[0] / it, q->strides[1] / it,
                                       static_cast<int>(mc));
                };
                if (dtype == HIPCX_FLOAT32) fill(float{});
                else fill(double{});
                CheckLaunch("qr");
            }
            return;
        }
        const size_t need = static_cast<size_t>(m * n * it);
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR, "qr workspace too small");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        hipcx_array w_desc = Dense2D(workspace, dtype, m, n);
        CopyInto(a, &w_desc, stream, "qr");  // cast + gather into the dense working copy
        auto run = [&](auto tag) {
            using T = decltype(tag);
            T* w = static_cast<T*>(workspace);
            T* tau_p = static_cast<T*>(tau->data);
            const int64_t tau_stride = k > 1 ? tau->strides[0] / it : 1;
            hipLaunchKernelGGL(HouseholderQrKernel<T>, dim3(1), dim3(kLinalgThreads), 0, st, w, static_cast<int>(m), static_cast<int>(n), tau_p, tau_stride);
            if (want_q) {
                hipLaunchKernelGGL(FormQKernel<T>, dim3(1), dim3(kLinalgThreads), 0, st, w, static_cast<int>(m), static_cast<int>(n), tau_p, tau_stride,
                                   static_cast<T*>(q->data), q->strides[0] / it, q->strides[1] / it, static_cast<int>(mc));
            }
            const int raw = mode == HIPCX_QR_RAW ? 1 : 0;
            const int64_t total = (raw ? m : r_rows) * n;
            hipLaunchKernelGGL(ExtractRKernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st, w, static_cast<int>(m),
                               static_cast<int>(n), static_cast<T*>(r->data), r->strides[0] / it, r->strides[1] / it, static_cast<int>(r_rows), raw);
        };
        if (dtype == HIPCX_FLOAT32) run(float{});
        else run(double{});
        CheckLaunch("qr");
    });
}

size_t hipcx_svd_workspace_size(const hipcx_array* a) {
    if (a == nullptr || a->ndim != 2 || a->shape[0] < 0 || a->shape[1] < 0) return 0;
    const size_t big = static_cast<size_t>(std::max(a->shape[0], a->shape[1])), small = static_cast<size_t>(std::min(a->shape[0], a->shape[1]));
    // the working copy, the accumulated rotations, singular values + ranks + projections, the count of final columns
    return (big * small + small * small + 2 * small + big) * 8 + 8 * 256;
}

int hipcx_svd(const hipcx_array* a, const hipcx_array* u, const hipcx_array* s, const hipcx_array* vt, int full_matrices, int compute_uv,
              void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(s, "s");
        HIPCX_REQUIRE(a->ndim == 2, HIPCX_DIMENSION_ERROR, "ChainerX linear algebra routines only support 2-dimensional arrays.");
        const int dtype = a->dtype;
        CheckLinalgDtype(dtype, "SVD");
        const int64_t m = a->shape[0], n = a->shape[1], k = std::min(m, n);
        HIPCX_REQUIRE(s->dtype == dtype && s->ndim == 1 && s->shape[0] == k, HIPCX_DIMENSION_ERROR, "svd: s must hold min(m, n) values of a's dtype");
        if (compute_uv) {
            ValidateArray(u, "u");
            ValidateArray(vt, "vt");
            HIPCX_REQUIRE(u->dtype == dtype && u->ndim == 2 && u->shape[0] == m && u->shape[1] == (full_matrices ? m : k), HIPCX_DIMENSION_ERROR,
                          "svd: u has the wrong shape or dtype");
            HIPCX_REQUIRE(vt->dtype == dtype && vt->ndim == 2 && vt->shape[1] == n && vt->shape[0] == (full_matrices ? n : k), HIPCX_DIMENSION_ERROR,
                          "svd: vt has the wrong shape or dtype");
        }
        const int64_t it = ItemSize(dtype);
        hipStream_t st = AsStream(stream);
        if (m == 0 || n == 0) {
            // the native backend's rule (CX/native/native_device/linalg.cc:445-452): full u and vt of an empty matrix are identities
            if (compute_uv && full_matrices) {
                auto fill = [&](auto tag) {
                    using T = decltype(tag);
                    for (const hipcx_array* o : {u, vt}) {
                        const int64_t side = o->shape[0];
                        if (side == 0) continue;
                        hipLaunchKernelGGL(StridedIdentityKernel<T>, dim3(static_cast<unsigned>((side * side + 255) / 256)), dim3(256), 0, st,
                                           static_cast<T*>(o->data), o->strides[0] / it, o->strides[1] / it, static_cast<int>(side));
                    }
                };
                if (dtype == HIPCX_FLOAT32) fill(float{});
                else fill(double{});
                CheckLaunch("svd");
            }
            return;
        }
        const bool transposed = m < n;
        const int64_t M = std::max(m, n), N = k;
        HIPCX_REQUIRE(M <= 4096, HIPCX_NOT_IMPLEMENTED_ERROR, "hip svd: matrix too large for the one-workgroup Jacobi kernel");
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= hipcx_svd_workspace_size(a), HIPCX_CHAINERX_ERROR, "svd workspace too small");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        char* ws = static_cast<char*>(workspace);
        size_t off = 0;
        auto take = [&](size_t bytes) { char* p = ws + off; off += (bytes + 255) / 256 * 256; return p; };
        // the size above counts 8 bytes per element for either dtype; its 8 * 256 bytes of slack cover the 256-alignment of each block
        char* g_mem = take(static_cast<size_t>(M * N) * it);
        char* v_mem = take(static_cast<size_t>(N * N) * it);
        char* sigma_mem = take(static_cast<size_t>(N) * it);
        char* dots_mem = take(static_cast<size_t>(M) * it);
        char* rank_mem = take(static_cast<size_t>(N) * sizeof(int) + sizeof(int));
        HIPCX_REQUIRE(off <= workspace_bytes, HIPCX_CHAINERX_ERROR, "svd workspace too small");
        hipcx_array g_desc = Dense2D(g_mem, dtype, M, N);
        hipcx_array src = *a;
        if (transposed) {
            std::swap(src.shape[0], src.shape[1]);
            std::swap(src.strides[0], src.strides[1]);
        }
        CopyInto(&src, &g_desc, stream, "svd");
        auto run = [&](auto tag) {
            using T = decltype(tag);
            T* tall = nullptr;
            T* sq = nullptr;
            int64_t tall_row = 0, tall_col = 0, sq_row = 0, sq_col = 0, tall_cols = N;
            if (compute_uv) {
                if (!transposed) {
                    tall = static_cast<T*>(u->data), tall_row = u->strides[0] / it, tall_col = u->strides[1] / it, tall_cols = u->shape[1];
                    sq = static_cast<T*>(vt->data), sq_row = vt->strides[1] / it, sq_col = vt->strides[0] / it;
                } else {
                    tall = static_cast<T*>(vt->data), tall_row = vt->strides[1] / it, tall_col = vt->strides[0] / it, tall_cols = vt->shape[0];
                    sq = static_cast<T*>(u->data), sq_row = u->strides[0] / it, sq_col = u->strides[1] / it;
                }
            }
            int* rank = reinterpret_cast<int*>(rank_mem);
            int* first_fill = rank + N;
            hipLaunchKernelGGL(JacobiSvdKernel<T>, dim3(1), dim3(kLinalgThreads), 0, st, reinterpret_cast<T*>(g_mem), static_cast<int>(M),
                               static_cast<int>(N), reinterpret_cast<T*>(v_mem), reinterpret_cast<T*>(sigma_mem), rank, static_cast<T*>(s->data),
                               k > 1 ? s->strides[0] / it : 1, tall, tall_row, tall_col, sq, sq_row, sq_col, compute_uv ? 1 : 0, first_fill);
            if (compute_uv) {
                hipLaunchKernelGGL(CompleteBasisKernel<T>, dim3(1), dim3(kLinalgThreads), 0, st, tall, tall_row, tall_col, static_cast<int>(M),
                                   static_cast<int>(tall_cols), first_fill, reinterpret_cast<T*>(dots_mem));
            }
        };
        if (dtype == HIPCX_FLOAT32) run(float{});
        else run(double{});
        CheckLaunch("svd");
    });
}

}  // extern "C"
