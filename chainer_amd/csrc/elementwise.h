// Elementwise engine: one launcher for every map-style kernel (arithmetic, math, select, compare,
// cast-copy, fill).
//
// Host side: the operands' (shape, byte-strides) are normalised -- unit axes dropped, axes ordered
// by decreasing output stride (any common permutation is legal for a map), mergeable neighbours
// fused -- so that an NCHW view of channels-last memory, a broadcast row vector, or a transposed
// matrix all collapse to a "rows x cols" problem whenever their memory allows it.
//
// Device side: a thread handles kUnroll vectors of VEC elements (16 bytes of the widest operand
// when alignment allows).  Operands whose inner stride is 0 are read once per vector as a scalar.
// With VEC == 1 any inner stride is accepted.  More than two remaining axes are decomposed with
// div/mod per vector (not per element).
#pragma once

#include <algorithm>
#include <cstdlib>
#include <initializer_list>

#include "common.h"

namespace hipcx {

constexpr int kEwMaxOperands = 6;  // out + up to 5 inputs
constexpr int kEwThreads = 256;
constexpr int kEwUnroll = 4;

struct EwPlan {
    int nops = 0;  // operand 0 is the output
    int ndim = 0;  // after normalisation; 0 means a single element
    int64_t total = 0;
    int64_t shape[HIPCX_MAX_NDIM];
    int64_t strides[kEwMaxOperands][HIPCX_MAX_NDIM];  // bytes
    char* ptr[kEwMaxOperands];
    int64_t itemsize[kEwMaxOperands];
};

// Builds the normalised iteration plan.  All operands must have the same shape.
inline EwPlan MakeEwPlan(std::initializer_list<const hipcx_array*> ops) {
    EwPlan p;
    p.nops = static_cast<int>(ops.size());
    HIPCX_REQUIRE(p.nops >= 1 && p.nops <= kEwMaxOperands, HIPCX_CHAINERX_ERROR, "bad operand count");
    const hipcx_array* arr[kEwMaxOperands];
    int k = 0;
    for (const hipcx_array* a : ops) {
        ValidateArray(a, "operand");
        arr[k++] = a;
    }
    const hipcx_array* out = arr[0];
    for (int i = 1; i < p.nops; ++i) {
        HIPCX_REQUIRE(SameShape(out, arr[i]), HIPCX_DIMENSION_ERROR,
                      "operand shapes differ: " + ShapeStr(out) + " vs " + ShapeStr(arr[i]));
    }
    p.total = TotalSize(out);
    for (int i = 0; i < p.nops; ++i) {
        p.ptr[i] = static_cast<char*>(arr[i]->data);
        p.itemsize[i] = ItemSize(arr[i]->dtype);
    }
    // 1. drop unit axes
    int dims[HIPCX_MAX_NDIM];
    int nd = 0;
    for (int d = 0; d < out->ndim; ++d) {
        if (out->shape[d] != 1) dims[nd++] = d;
    }
    // 2. order by decreasing |out stride| (stable, so equal strides keep their logical order)
    std::stable_sort(dims, dims + nd, [&](int a, int b) { return std::llabs(out->strides[a]) > std::llabs(out->strides[b]); });
    // 3. merge neighbours that every operand walks as one run
    int m = 0;
    for (int j = 0; j < nd; ++j) {
        int d = dims[j];
        bool merged = false;
        if (m > 0) {
            merged = true;
            for (int i = 0; i < p.nops; ++i) {
                if (p.strides[i][m - 1] != out->shape[d] * arr[i]->strides[d]) {
                    merged = false;
                    break;
                }
            }
        }
        if (merged) {
            p.shape[m - 1] *= out->shape[d];
            for (int i = 0; i < p.nops; ++i) p.strides[i][m - 1] = arr[i]->strides[d];
        } else {
            p.shape[m] = out->shape[d];
            for (int i = 0; i < p.nops; ++i) p.strides[i][m] = arr[i]->strides[d];
            ++m;
        }
    }
    p.ndim = m;
    return p;
}

// Device-side view of the plan: `cols` is the innermost axis, the others are "outer" axes.
template <int NOPS>
struct EwArgs {
    char* ptr[NOPS];
    int64_t col_stride[NOPS];  // bytes between consecutive elements of the inner axis (0 = broadcast)
    int64_t outer_stride[NOPS][HIPCX_MAX_NDIM - 1];
    int64_t outer_shape[HIPCX_MAX_NDIM - 1];
    int n_outer;
    int64_t cols;   // elements
    int64_t cvecs;  // cols / VEC
    int64_t nvec;   // rows * cvecs
    int stream_in;  // bit i + 1: input i is too large to stay in the last-level cache and is loaded without allocating there
};

// A 16-byte vector load that does not allocate in the caches (other sizes: a plain load).  A tensor larger than the memory-side
// cache that is read front to back with allocating loads evicts its own tail -- the part the producer left there -- before reaching it.
template <typename V>
__device__ __forceinline__ V LoadStreaming(const char* p) {
    if constexpr (sizeof(V) == 16) {
        typedef unsigned Raw16 __attribute__((ext_vector_type(4)));
        Raw16 r = __builtin_nontemporal_load(reinterpret_cast<const Raw16*>(p));
        return __builtin_bit_cast(V, r);
    } else {
        return *reinterpret_cast<const V*>(p);
    }
}

template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
    T v[N];
};

template <typename T>
__device__ __forceinline__ compute_t<T> LoadAs(const char* p) {
    return static_cast<compute_t<T>>(*reinterpret_cast<const T*>(p));
}

// Type of the first input: Op::In0 when the op declares one (a bool condition in front of numeric operands), else Op::In.
template <typename Op, typename = void>
struct FirstInOf {
    using type = typename Op::In;
};
template <typename Op>
struct FirstInOf<Op, std::void_t<typename Op::In0>> {
    using type = typename Op::In0;
};

// Ops that set `static constexpr bool kNarrowVectors = true` are also instantiated for 8- and 4-byte vectors.
template <typename Op, typename = void>
struct HasNarrowVectors : std::false_type {};
template <typename Op>
struct HasNarrowVectors<Op, std::enable_if_t<Op::kNarrowVectors>> : std::true_type {};

// Op interface:
//   using In = ...; using Out = ...; static constexpr int kNumIn = n;  (optionally using In0 = ... for the first input)
//   __device__ compute_t<Out> operator()(compute_t<In> a, compute_t<In> b, compute_t<In> c, compute_t<In> d, int64_t index) const
// `index` is the C-order position in the *normalised* iteration space; only ops that ask for it
// (kNeedsIndex) get a meaningful value, and those are launched on contiguous outputs.
template <typename Op, int VEC, typename IdxT>
__global__ __launch_bounds__(kEwThreads) void EwKernel(EwArgs<Op::kNumIn + 1> args, Op op) {
    using In = typename Op::In;
    using In0 = typename FirstInOf<Op>::type;
    using Out = typename Op::Out;
    using CIn = compute_t<In>;
    constexpr int NIN = Op::kNumIn;
    constexpr int NOPS = NIN + 1;

    const IdxT nvec = static_cast<IdxT>(args.nvec);
    const IdxT cvecs = static_cast<IdxT>(args.cvecs);
    IdxT base = static_cast<IdxT>(blockIdx.x) * (kEwThreads * kEwUnroll) + threadIdx.x;

    int64_t off[kEwUnroll][NOPS];
    bool live[kEwUnroll];
    IdxT colv[kEwUnroll];
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) {
        IdxT v = base + static_cast<IdxT>(u) * kEwThreads;
        live[u] = v < nvec;
        IdxT row = live[u] ? v / cvecs : 0;
        IdxT cv = live[u] ? v - row * cvecs : 0;
        colv[u] = cv;
#pragma unroll
        for (int i = 0; i < NOPS; ++i) off[u][i] = static_cast<int64_t>(cv) * VEC * args.col_stride[i];
        if (args.n_outer > 1) {
            IdxT r = row;
            for (int d = args.n_outer - 1; d >= 0; --d) {
                IdxT q = r / static_cast<IdxT>(args.outer_shape[d]);
                IdxT rem = r - q * static_cast<IdxT>(args.outer_shape[d]);
                r = q;
#pragma unroll
                for (int i = 0; i < NOPS; ++i) off[u][i] += static_cast<int64_t>(rem) * args.outer_stride[i][d];
            }
        } else {
#pragma unroll
            for (int i = 0; i < NOPS; ++i) off[u][i] += static_cast<int64_t>(row) * args.outer_stride[i][0];
        }
    }

    // loads first (all unrolled iterations in flight), then compute + store
    Vec<In, VEC> in[kEwUnroll][NIN > 0 ? NIN : 1];
    Vec<In0, VEC> in0[kEwUnroll];
    auto load_all = [&](auto stream_tag) {
        constexpr bool STREAM = decltype(stream_tag)::value;
#pragma unroll
        for (int u = 0; u < kEwUnroll; ++u) {
            if (!live[u]) continue;
#pragma unroll
            for (int i = 0; i < NIN; ++i) {
                const char* p = args.ptr[i + 1] + off[u][i + 1];
                const bool streamed = STREAM && ((args.stream_in >> (i + 1)) & 1);  // (uniform) a broadcast operand stays cached
                if (i == 0) {
                    if (VEC > 1 && args.col_stride[NOPS > 1 ? 1 : 0] != 0) {
                        in0[u] = streamed ? LoadStreaming<Vec<In0, VEC>>(p) : *reinterpret_cast<const Vec<In0, VEC>*>(p);
                    } else {
                        In0 s = *reinterpret_cast<const In0*>(p);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) in0[u].v[e] = s;
                    }
                } else if (VEC > 1) {
                    if (args.col_stride[i + 1] != 0) {
                        in[u][i] = streamed ? LoadStreaming<Vec<In, VEC>>(p) : *reinterpret_cast<const Vec<In, VEC>*>(p);
                    } else {
                        In s = *reinterpret_cast<const In*>(p);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) in[u][i].v[e] = s;
                    }
                } else {
                    in[u][i].v[0] = *reinterpret_cast<const In*>(p);
                }
            }
        }
    };
    if (VEC > 1 && args.stream_in) {
        load_all(std::integral_constant<bool, true>{});
    } else {
        load_all(std::integral_constant<bool, false>{});
    }
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) {
        if (!live[u]) continue;
        Vec<Out, VEC> o;
        int64_t index0 = 0;
        if (Op::kNeedsIndex) {
            IdxT v = base + static_cast<IdxT>(u) * kEwThreads;
            index0 = static_cast<int64_t>(v) * VEC;
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            CIn a = NIN > 0 ? static_cast<CIn>(in0[u].v[e]) : CIn{};
            CIn b = NIN > 1 ? static_cast<CIn>(in[u][NIN > 1 ? 1 : 0].v[e]) : CIn{};
            CIn c = NIN > 2 ? static_cast<CIn>(in[u][NIN > 2 ? 2 : 0].v[e]) : CIn{};
            CIn d = NIN > 3 ? static_cast<CIn>(in[u][NIN > 3 ? 3 : 0].v[e]) : CIn{};
            if constexpr (NIN > 4) {
                CIn f = static_cast<CIn>(in[u][4].v[e]);
                o.v[e] = static_cast<Out>(op.Apply5(a, b, c, d, f));
            } else {
                o.v[e] = static_cast<Out>(op(a, b, c, d, index0 + e));
            }
        }
        char* q = args.ptr[0] + off[u][0];
        if (VEC > 1) {
            *reinterpret_cast<Vec<Out, VEC>*>(q) = o;
        } else {
            *reinterpret_cast<Out*>(q) = o.v[0];
        }
    }
    (void)colv;
}

template <typename Op, int VEC>
inline void LaunchEwVec(const EwPlan& p, const Op& op, hipStream_t stream) {
    constexpr int NOPS = Op::kNumIn + 1;
    EwArgs<NOPS> a;
    std::memset(&a, 0, sizeof(a));
    int nd = p.ndim;
    int64_t cols = nd > 0 ? p.shape[nd - 1] : 1;
    for (int i = 0; i < NOPS; ++i) {
        a.ptr[i] = p.ptr[i];
        a.col_stride[i] = nd > 0 ? p.strides[i][nd - 1] : 0;
    }
    a.n_outer = nd > 1 ? nd - 1 : 1;
    int64_t rows = 1;
    if (nd > 1) {
        for (int d = 0; d < nd - 1; ++d) {
            a.outer_shape[d] = p.shape[d];
            rows *= p.shape[d];
            for (int i = 0; i < NOPS; ++i) a.outer_stride[i][d] = p.strides[i][d];
        }
    } else {
        a.outer_shape[0] = 1;
    }
    a.cols = cols;
    a.cvecs = cols / VEC;
    a.nvec = rows * a.cvecs;
    // an input streams when its own footprint (the axes it is not broadcast along) exceeds the threshold: a bias row added to a
    // large matrix is read once per matrix row and has to stay in the cache
    a.stream_in = 0;
    for (int i = 1; i < NOPS; ++i) {
        int64_t footprint = static_cast<int64_t>(sizeof(typename Op::In));
        for (int d = 0; d < nd; ++d) {
            if (p.strides[i][d] != 0) footprint *= p.shape[d];
        }
        if (footprint > StreamingThresholdBytes()) a.stream_in |= 1 << i;
    }
    int64_t per_block = static_cast<int64_t>(kEwThreads) * kEwUnroll;
    int64_t blocks = (a.nvec + per_block - 1) / per_block;
    HIPCX_REQUIRE(blocks <= 0x7fffffffLL, HIPCX_NOT_IMPLEMENTED_ERROR, "array too large for one launch");
    bool wide = a.nvec + per_block >= 0x7fffffffLL;
    dim3 grid(static_cast<unsigned>(blocks)), block(kEwThreads);
    if (!wide) {
        hipLaunchKernelGGL((EwKernel<Op, VEC, uint32_t>), grid, block, 0, stream, a, op);
    } else {
        hipLaunchKernelGGL((EwKernel<Op, VEC, int64_t>), grid, block, 0, stream, a, op);
    }
    CheckLaunch("elementwise");
}

// Picks the widest vector the operands' addresses allow and launches.
template <typename Op>
inline void LaunchElementwise(const EwPlan& p, const Op& op, hipStream_t stream) {
    using In = typename Op::In;
    using Out = typename Op::Out;
    constexpr int NOPS = Op::kNumIn + 1;
    if (p.total == 0) return;
    constexpr int kWidest = sizeof(In) > sizeof(Out) ? sizeof(In) : sizeof(Out);
    constexpr int kMaxVec = 16 / kWidest >= 1 ? 16 / kWidest : 1;  // 16-byte accesses on the widest operand

    int nd = p.ndim;
    int64_t cols = nd > 0 ? p.shape[nd - 1] : 1;
    auto fits = [&](int vec) {
        if (vec == 1) return true;
        if (cols % vec != 0) return false;
        for (int i = 0; i < NOPS; ++i) {
            int64_t cs = nd > 0 ? p.strides[i][nd - 1] : 0;
            if (cs == 0) continue;                   // scalar broadcast along the inner axis
            if (cs != p.itemsize[i]) return false;   // not unit-stride: only VEC == 1 can walk it
            int64_t bytes = p.itemsize[i] * vec;
            if (reinterpret_cast<uintptr_t>(p.ptr[i]) % bytes != 0) return false;
            for (int d = 0; d + 1 < nd; ++d) {
                if (p.strides[i][d] % bytes != 0) return false;
            }
        }
        return true;
    };
    // Two instantiations per op keep the code object small: full 16-byte vectors, or scalars.  Ops that declare
    // kNarrowVectors (plain copies: the strided copies of Im2Col, transposes and staging) also get 8- and 4-byte vectors, for
    // rows that are not whole 16-byte multiples (14x14 and 7x7 planes of float16).
    if (kMaxVec > 1 && fits(kMaxVec)) return LaunchEwVec<Op, kMaxVec>(p, op, stream);
    if constexpr (HasNarrowVectors<Op>::value) {
        if constexpr (kMaxVec >= 4) {
            if (fits(kMaxVec / 2)) return LaunchEwVec<Op, kMaxVec / 2>(p, op, stream);
        }
        if constexpr (kMaxVec >= 8) {
            if (fits(kMaxVec / 4)) return LaunchEwVec<Op, kMaxVec / 4>(p, op, stream);
        }
    }
    return LaunchEwVec<Op, 1>(p, op, stream);
}

}  // namespace hipcx
