// Reductions: Sum (CX/kernels/reduction.h:18), AMax (statistics.h:13), ArgMax (sorting.h:9).
//
// Order of operations.  The native backend reduces every output element with one fixed tree
// (CX/native/reduce.h:46-83): elements are taken in groups of four, (e0.e1).(e2.e3); eight groups
// are folded serially into a 32-element chunk; chunks are merged by a binary counter, which is a
// balanced binary tree over aligned runs of chunks, the later operand being the accumulator; the
// last chunk also takes the up-to-3 leftover elements and any groups short of a full chunk.
// Both kernels below evaluate exactly that tree, so
//   * ArgMax returns the native backend's index for every input, ties and NaNs included
//     (earlier index wins inside a chunk, later chunk wins between chunks, a NaN never replaces
//     and a leading NaN is never replaced: CX/native/native_device/reduction.cc:34-61);
//   * Sum carries the native backend's rounding sequence (float16 accumulates in float,
//     reduction.cc:105), so float results agree bit for bit;
//   * AMax propagates NaN (statistics.cc:38-42).
//
// RowReduceKernel: the reduced axes form one contiguous run (a "row").  Lane <-> group of four
// (one 16-byte load), 8 lanes <-> chunk, 16 lanes <-> two chunks merged (one LDS node), then a tree
// over the block's nodes and, for rows split over several blocks, a second pass over per-block
// partials in the workspace.
// GenericReduceKernel: any strides; one thread per output element runs the reference loop
// literally.  Consecutive threads take consecutive outputs, so reducing over outer axes of a
// dense array (a "column" reduction) is coalesced.
#include <mutex>

#include "common.h"

// Device memory for the partial results of hipcx_sum_static_scratch: part of the code object, so every device the library
// runs on holds its own copy (at its own address) from the moment the module is loaded until the process ends.
static __device__ __align__(256) unsigned char scratch[HIPCX_STATIC_SCRATCH_BYTES];

namespace hipcx {
namespace {

constexpr int kMaxDims = HIPCX_MAX_NDIM;
constexpr int kRowThreads = 256;
constexpr int kElemsPerIter = kRowThreads * 4;  // 1024 elements = 32 chunks = 4 nodes (one per wave)
constexpr int kMaxIters = 64;                   // iterations per block -> span <= 65536 elements
constexpr int kMaxNodes = kMaxIters * 16;       // LDS nodes per block: one per row of 16 lanes (two chunks) and iteration
constexpr int kMaxPartials = 1024;              // blocks per row handled by the finalize pass

// ---------------------------------------------------------------------------------------------
// Reduction functors.  Acc is what travels through the tree.
//   Identity()            impl.Identity() of the reference
//   Map(in, index)        impl.MapIn
//   Reduce(next, acc)     impl.Reduce(next, accum), additionally a no-op when `next` is the padding value Empty()
//   kSerialFold           whether the 8 groups of a chunk must be folded strictly in order (floating point addition)
//   kFast, ReduceFast     a shorter Reduce for operands known to be neither padding (kFast >= 1) nor NaN (kFast == 2);
//                         Probe(in) is a float that is NaN when `in` is
// ---------------------------------------------------------------------------------------------
template <typename In_, typename Out_>
struct SumImpl {
    using In = In_;
    using Out = Out_;
    using Acc = std::conditional_t<std::is_same<Out_, half_t>::value, float, Out_>;
    using Row = SumImpl;
    __device__ static Acc FromRow(Acc a, int64_t) { return a; }
    static constexpr bool kSerialFold = true;
    static constexpr bool kHasIndex = false;
    static constexpr int kFast = 0;
    __device__ static void ReduceFast(Acc next, Acc& acc) { Reduce(next, acc); }
    __device__ static float Probe(In) { return 0.f; }
    __device__ static Acc Identity() { return Acc(0); }
    __device__ static Acc Empty() { return Acc(0); }  // x + 0 == x for every x a chunk can produce (never -0)
    __device__ static Acc Map(In v, int64_t) {
        if constexpr (std::is_same<In, half_t>::value) {
            return static_cast<Acc>(static_cast<float>(v));
        } else {
            return static_cast<Acc>(v);
        }
    }
    __device__ static void Reduce(Acc next, Acc& acc) { acc += next; }
    __device__ static void MaskLaterNan(Acc&, bool) {}
    __device__ static Out MapOut(Acc a) {
        if constexpr (std::is_same<Out, half_t>::value) {
            return static_cast<half_t>(a);
        } else {
            return static_cast<Out>(a);
        }
    }
    __device__ static Acc Shfl(Acc a, int src) { return __shfl(a, src); }
};

template <typename T>
__device__ __forceinline__ T LowestOrInf() {
    if constexpr (std::is_same<T, half_t>::value) {
        return static_cast<half_t>(-__builtin_huge_valf());
    } else if constexpr (std::is_same<T, float>::value) {
        return -__builtin_huge_valf();
    } else if constexpr (std::is_same<T, double>::value) {
        return -__builtin_huge_val();
    } else if constexpr (std::is_same<T, bool>::value) {
        return false;
    } else {
        return std::numeric_limits<T>::lowest();
    }
}

template <typename T>
__device__ __forceinline__ T MaxOrInf() {
    if constexpr (std::is_same<T, half_t>::value) {
        return static_cast<half_t>(__builtin_huge_valf());
    } else if constexpr (std::is_same<T, float>::value) {
        return __builtin_huge_valf();
    } else if constexpr (std::is_same<T, double>::value) {
        return __builtin_huge_val();
    } else if constexpr (std::is_same<T, bool>::value) {
        return true;
    } else {
        return std::numeric_limits<T>::max();
    }
}

template <typename T>
__device__ __forceinline__ bool IsNanV(T v) {
    if constexpr (std::is_same<T, half_t>::value || std::is_floating_point<T>::value) {
        return v != v;
    } else {
        return false;
    }
}

// MIN: AMin (identity MaxOrInf, `accum > next`), the mirror image of AMax (native/native_device/statistics.cc:27-73).
template <typename T, bool MIN = false>
struct AMaxImpl {
    using In = T;
    using Out = T;
    // half values are compared as floats (exact and order preserving); bool as int
    using Acc = std::conditional_t<std::is_same<T, half_t>::value, float, std::conditional_t<std::is_same<T, bool>::value, int, T>>;
    using Row = AMaxImpl;
    __device__ static Acc FromRow(Acc a, int64_t) { return a; }
    static constexpr bool kSerialFold = false;
    static constexpr bool kHasIndex = false;
    static constexpr int kFast = (std::is_same<T, half_t>::value || std::is_floating_point<T>::value) ? 2 : 0;
    __device__ static void ReduceFast(Acc next, Acc& acc) {
        if (MIN ? acc > next : acc < next) acc = next;
    }
    __device__ static float Probe(In v) { return static_cast<float>(v); }
    __device__ static Acc Identity() { return static_cast<Acc>(MIN ? MaxOrInf<T>() : LowestOrInf<T>()); }
    __device__ static Acc Empty() { return Identity(); }
    __device__ static Acc Map(In v, int64_t) { return static_cast<Acc>(v); }
    __device__ static void Reduce(Acc next, Acc& acc) {
        if (IsNanV(next) || (MIN ? acc > next : acc < next)) acc = next;
    }
    __device__ static void MaskLaterNan(Acc&, bool) {}
    __device__ static Out MapOut(Acc a) { return static_cast<Out>(a); }
    __device__ static Acc Shfl(Acc a, int src) { return __shfl(a, src); }
};

template <typename V, typename I = int64_t>
struct MaxIdx {
    V v;
    I i;  // < 0: empty / identity
};

// MIN: ArgMin (`accum.min > next.min`), the mirror image of ArgMax (native/native_device/reduction.cc:34-92).
// I: type of the index that travels with the value.  The row kernel counts from the first element of its block (at most
// 65536 + 3 elements, Row below) and widens when it hands the result on (FromRow); every other kernel uses int64_t.
template <typename T, bool MIN = false, typename I = int64_t>
struct ArgMaxImpl {
    using In = T;
    using Out = int64_t;
    using V = std::conditional_t<std::is_same<T, half_t>::value, float, std::conditional_t<std::is_same<T, bool>::value, int, T>>;
    using Acc = MaxIdx<V, I>;
    using Row = ArgMaxImpl<T, MIN, int32_t>;
    __device__ static Acc FromRow(typename Row::Acc a, int64_t base) { return Acc{a.v, a.i < 0 ? I(-1) : static_cast<I>(base + a.i)}; }
    static constexpr bool kSerialFold = false;
    static constexpr bool kHasIndex = true;
    static constexpr int kFast = (std::is_same<T, half_t>::value || std::is_floating_point<T>::value) ? 2 : 1;
    __device__ static void ReduceFast(Acc next, Acc& acc) {
        if (MIN ? acc.v > next.v : acc.v < next.v) acc = next;
    }
    __device__ static float Probe(In v) { return static_cast<float>(v); }
    __device__ static Acc Identity() { return Acc{V(0), -1}; }
    __device__ static Acc Empty() { return Acc{V(0), -1}; }
    __device__ static Acc Map(In v, int64_t index) { return Acc{static_cast<V>(v), static_cast<I>(index)}; }
    __device__ static void Reduce(Acc next, Acc& acc) {
        if (next.i < 0) return;
        if (acc.i < 0 || (MIN ? acc.v > next.v : acc.v < next.v)) acc = next;
    }
    // Inside a chunk a NaN operand other than the very first never replaces the accumulator; turning
    // it into padding makes the in-chunk fold associative, so it can run as a shuffle tree.
    __device__ static void MaskLaterNan(Acc& a, bool is_first) {
        if (!is_first && IsNanV(a.v)) a.i = -1;
    }
    __device__ static Out MapOut(Acc a) { return a.i; }
    __device__ static Acc Shfl(Acc a, int src) {
        Acc r;
        r.v = __shfl(a.v, src);
        r.i = __shfl(a.i, src);
        return r;
    }
};

// All / Any over bool inputs (native/native_device/logic.cc: the routine casts the input to bool first).
template <bool ALL>
struct AllAnyImpl {
    using In = bool;
    using Out = bool;
    using Acc = int;
    using Row = AllAnyImpl;
    __device__ static Acc FromRow(Acc a, int64_t) { return a; }
    static constexpr bool kSerialFold = false;
    static constexpr bool kHasIndex = false;
    static constexpr int kFast = 0;
    __device__ static void ReduceFast(Acc next, Acc& acc) { Reduce(next, acc); }
    __device__ static float Probe(In) { return 0.f; }
    __device__ static Acc Identity() { return ALL ? 1 : 0; }
    __device__ static Acc Empty() { return Identity(); }
    __device__ static Acc Map(In v, int64_t) { return v ? 1 : 0; }
    __device__ static void Reduce(Acc next, Acc& acc) { acc = ALL ? (acc & next) : (acc | next); }
    __device__ static void MaskLaterNan(Acc&, bool) {}
    __device__ static Out MapOut(Acc a) { return a != 0; }
    __device__ static Acc Shfl(Acc a, int src) { return __shfl(a, src); }
};

// ---------------------------------------------------------------------------------------------
// Geometry shared by both kernels
// ---------------------------------------------------------------------------------------------
struct ReduceGeom {
    const char* in;
    char* out;
    int n_keep;   // kept (output) axes after squashing
    int n_red;    // reduced axes after squashing
    int64_t keep_shape[kMaxDims];
    int64_t keep_in_stride[kMaxDims];   // bytes
    int64_t keep_out_stride[kMaxDims];  // bytes
    int64_t red_shape[kMaxDims];
    int64_t red_stride[kMaxDims];  // bytes
    int64_t n_out;                 // product of keep_shape
    int64_t red_len;               // product of red_shape
    // Row kernel: the reduced sequence is red_len / seg_len dense runs of seg_len elements, seg_stride bytes apart
    // (one run: seg_len == red_len).  Reducing N and H*W of an NCHW array for each channel is the two-level case.
    int64_t seg_len;
    int64_t seg_stride;
};

__device__ __forceinline__ void OutOffsets(const ReduceGeom& g, int64_t o, int64_t& in_off, int64_t& out_off) {
    in_off = 0;
    out_off = 0;
    for (int d = g.n_keep - 1; d >= 1; --d) {
        int64_t q = o / g.keep_shape[d];
        int64_t r = o - q * g.keep_shape[d];
        o = q;
        in_off += r * g.keep_in_stride[d];
        out_off += r * g.keep_out_stride[d];
    }
    if (g.n_keep > 0) {  // what is left of `o` is the coordinate on the outermost kept axis: no division
        in_off += o * g.keep_in_stride[0];
        out_off += o * g.keep_out_stride[0];
    }
}

// ---------------------------------------------------------------------------------------------
// Row kernel
// ---------------------------------------------------------------------------------------------
// The value that lane + N of the same row of 16 lanes holds (N < 16; a data-parallel-primitive move: no trip through the
// LDS crossbar).  Lanes whose partner would lie in another row get zero bits (and nobody reads their results); written this
// way the compiler can fold the move into the instruction that consumes it.
template <int N, typename T>
__device__ __forceinline__ T FromLaneAbove(T v) {
    constexpr int kWords = (sizeof(T) + 3) / 4;
    int w[kWords] = {};
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (int i = 0; i < kWords; ++i) w[i] = __builtin_amdgcn_update_dpp(0, w[i], 0x100 + N /* row_shl:N */, 0xf, 0xf, true);
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

template <typename In>
struct alignas(sizeof(In) * 4) Group4 {
    In v[4];
};

template <bool ALIGNED, typename In>
__device__ __forceinline__ Group4<In> LoadGroup(const In* p) {
    if (ALIGNED) return *reinterpret_cast<const Group4<In>*>(p);
    Group4<In> q;
#pragma unroll
    for (int j = 0; j < 4; ++j) q.v[j] = p[j];
    return q;
}

// Reduce of R, or its shorter form for operands known to be neither padding nor NaN.
template <typename R, bool FAST>
struct ReduceOp {
    using Acc = typename R::Acc;
    __device__ static __forceinline__ void Reduce(Acc next, Acc& acc) {
        if constexpr (FAST) {
            R::ReduceFast(next, acc);
        } else {
            R::Reduce(next, acc);
        }
    }
};

// One step of the balanced tree over values held by lanes S apart (S < 16): the lane takes the value of lane + S as the
// later operand (the accumulator of the merge) and its own as the earlier one.  Valid in the lanes that are multiples of
// 2 * S.
template <typename Op, int S>
__device__ __forceinline__ void MergeLaneAbove(typename Op::Acc& acc) {
    typename Op::Acc later = FromLaneAbove<S>(acc);
    Op::Reduce(acc, later);
    acc = later;
}

template <int LANE, typename T>
__device__ __forceinline__ T ReadLane(T v) {  // the value held by lane LANE, in every lane (through scalar registers)
    constexpr int kWords = (sizeof(T) + 3) / 4;
    int w[kWords] = {};
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (int i = 0; i < kWords; ++i) w[i] = __builtin_amdgcn_readlane(w[i], LANE);
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

// The last two levels of the tree over a wave: the values of lanes 0, 16, 32 and 48 (the first lane of each row of 16)
// merged as (l0 . l16) . (l32 . l48), the later operand being the accumulator.  Every lane gets the result.
template <typename Op>
__device__ __forceinline__ typename Op::Acc MergeRows(typename Op::Acc acc) {
    typename Op::Acc a = ReadLane<0>(acc);
    typename Op::Acc b = ReadLane<16>(acc);
    typename Op::Acc c = ReadLane<32>(acc);
    typename Op::Acc d = ReadLane<48>(acc);
    Op::Reduce(a, b);
    Op::Reduce(c, d);
    Op::Reduce(b, d);
    return d;
}

template <typename Impl, bool ALIGNED>
__global__ __launch_bounds__(kRowThreads) void RowReduceKernel(ReduceGeom g, int64_t span, int blocks_per_row, void* partials) {
    using R = typename Impl::Row;  // the same reduction with indices counted from the block's first element
    using In = typename R::In;
    using Acc = typename R::Acc;
    __shared__ Acc nodes[kMaxNodes];
    __shared__ Acc wave_nodes[kMaxNodes / 64];

    int64_t row = blockIdx.x;
    int blk = 0;
    if (blocks_per_row != 1) {
        row = blockIdx.x / static_cast<unsigned>(blocks_per_row);
        blk = static_cast<int>(blockIdx.x - static_cast<unsigned>(row) * static_cast<unsigned>(blocks_per_row));
    }
    int64_t in_off, out_off;
    OutOffsets(g, row, in_off, out_off);
    const char* xbase = g.in + in_off;
    // address of element i of the reduced sequence; groups of four never straddle a run (seg_len % 4 == 0 when there are several)
    auto at = [&](int64_t i) -> const In* {
        if (g.seg_stride == 0) return reinterpret_cast<const In*>(xbase) + i;  // one run (uniform branch): no division
        const int64_t sidx = i / g.seg_len;
        return reinterpret_cast<const In*>(xbase + sidx * g.seg_stride) + (i - sidx * g.seg_len);
    };

    const int64_t L = g.red_len;
    const int64_t G = L / 4;                          // full groups
    const int64_t k_last = G > 0 ? (G - 1) / 8 : 0;   // chunk that also takes the tail
    const int64_t e_begin = static_cast<int64_t>(blk) * span;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int seg_lane = lane & 7;
    const int iters = static_cast<int>(span / kElemsPerIter);

    // The iterations of a block that lie wholly before the chunk with the leftover elements (all of them when the row is a
    // whole number of groups) need no bounds checks; with one dense run they need no address arithmetic either.
    const int64_t plain_len = L % 4 == 0 ? L : k_last * 32;
    int plain_iters = 0;
    if (g.seg_stride == 0 && plain_len > e_begin) {
        const int64_t n = (plain_len - e_begin) / kElemsPerIter;
        plain_iters = n < iters ? static_cast<int>(n) : iters;
    }

    // ---- N plain iterations, stage by stage so that their instructions interleave: group of four -> chunk (8 lanes) ->
    // node (wave).  FAST: no operand is padding or NaN, so the shorter Reduce applies and gives the same result. ----
    auto plain_stages = [&](int it0, const Group4<In>* q, auto count, auto fast) {
        constexpr int N = decltype(count)::value;
        constexpr bool FAST = decltype(fast)::value;
        using Op = ReduceOp<R, FAST>;
        Acc acc[N];
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int local = (it0 + u) * kElemsPerIter + tid * 4;  // index of the group's first element, counted from e_begin
            // (e0 . e1) . (e2 . e3): the later element is `next`
            Acc gv = R::Map(q[u].v[0], local);
            Op::Reduce(R::Map(q[u].v[1], local + 1), gv);
            Acc p1 = R::Map(q[u].v[2], local + 2);
            Op::Reduce(R::Map(q[u].v[3], local + 3), p1);
            Op::Reduce(p1, gv);
            acc[u] = gv;
        }
        if (R::kSerialFold) {  // Identity . g0 . g1 ... g7, strictly in order; only the chunk's first lane needs it
            Acc gv[N];
#pragma unroll
            for (int u = 0; u < N; ++u) {
                gv[u] = acc[u];
                acc[u] = R::Identity();
                Op::Reduce(gv[u], acc[u]);
            }
            auto step = [&](auto j) {
#pragma unroll
                for (int u = 0; u < N; ++u) Op::Reduce(FromLaneAbove<decltype(j)::value>(gv[u]), acc[u]);
            };
            step(std::integral_constant<int, 1>());
            step(std::integral_constant<int, 2>());
            step(std::integral_constant<int, 3>());
            step(std::integral_constant<int, 4>());
            step(std::integral_constant<int, 5>());
            step(std::integral_constant<int, 6>());
            step(std::integral_constant<int, 7>());
        } else {
            if (!FAST) {  // (with FAST, Identity . group == group and there is no NaN to mask)
#pragma unroll
                for (int u = 0; u < N; ++u) {
                    Acc m = acc[u];
                    R::MaskLaterNan(m, seg_lane == 0);
                    acc[u] = R::Identity();
                    R::Reduce(m, acc[u]);  // lane-local start: Identity . group
                }
            }
            auto step = [&](auto s) {  // the later operand is `next`
#pragma unroll
                for (int u = 0; u < N; ++u) Op::Reduce(FromLaneAbove<decltype(s)::value>(acc[u]), acc[u]);
            };
            step(std::integral_constant<int, 1>());
            step(std::integral_constant<int, 2>());
            step(std::integral_constant<int, 4>());
        }
        // the two chunks of a row of 16 lanes -> one node (the later operand is the accumulator); the tree above that level
        // runs once per block, over the nodes
#pragma unroll
        for (int u = 0; u < N; ++u) MergeLaneAbove<Op, 8>(acc[u]);
        if ((lane & 15) == 0) {
#pragma unroll
            for (int u = 0; u < N; ++u) nodes[((it0 + u) * 4 + wave) * 4 + (lane >> 4)] = acc[u];
        }
    };
    auto plain = [&](int it0, const Group4<In>* q, auto count) {
        constexpr int N = decltype(count)::value;
        if constexpr (R::kFast == 0) {
            plain_stages(it0, q, count, std::false_type());
        } else if constexpr (R::kFast == 1) {
            plain_stages(it0, q, count, std::true_type());
        } else {
            // Is a NaN among the wave's N * 256 elements?  A sum is NaN when an addend is (inf - inf also is: that only
            // costs the longer path).
            float t[N];
#pragma unroll
            for (int u = 0; u < N; ++u) t[u] = (R::Probe(q[u].v[0]) + R::Probe(q[u].v[1])) + (R::Probe(q[u].v[2]) + R::Probe(q[u].v[3]));
#pragma unroll
            for (int u = 1; u < N; ++u) t[0] += t[u];
            if (__ballot(t[0] != t[0]) == 0) {
                plain_stages(it0, q, count, std::true_type());
            } else {
                plain_stages(it0, q, count, std::false_type());
            }
        }
    };

    // ---- an iteration that may hold the end of the row: every step checked ----
    auto guarded = [&](int it) {
        const int64_t grp = e_begin / 4 + static_cast<int64_t>(it) * kRowThreads + tid;
        const int64_t chunk = grp >> 3;
        const int local = it * kElemsPerIter + tid * 4;
        Acc gv = R::Empty();
        if (grp < G) {
            const Group4<In> q = LoadGroup<ALIGNED>(at(grp * 4));
            Acc p0 = R::Map(q.v[0], local);
            R::Reduce(R::Map(q.v[1], local + 1), p0);
            Acc p1 = R::Map(q.v[2], local + 2);
            R::Reduce(R::Map(q.v[3], local + 3), p1);
            R::Reduce(p1, p0);
            gv = p0;
        }
        // ---- fold the 8 groups of a chunk into the segment leader ----
        Acc acc;
        if (R::kSerialFold) {
            acc = R::Identity();
            R::Reduce(gv, acc);
#pragma unroll
            for (int j = 1; j < 8; ++j) {
                Acc o = R::Shfl(gv, (lane & ~7) + j);
                R::Reduce(o, acc);
            }
        } else {
            R::MaskLaterNan(gv, seg_lane == 0);
            acc = R::Identity();
            R::Reduce(gv, acc);  // lane-local start: Identity . group
#pragma unroll
            for (int s = 1; s < 8; s <<= 1) {
                Acc o = R::Shfl(acc, lane + s);  // the later operand
                R::Reduce(o, acc);
            }
        }
        // ---- the last chunk also folds the leftover elements, in order ----
        if (seg_lane == 0 && chunk == k_last) {
            for (int64_t i = G * 4; i < L; ++i) R::Reduce(R::Map(*at(i), i - e_begin), acc);
        }
        if (chunk > k_last) acc = R::Empty();
        // ---- the two chunks of a row of 16 lanes -> one node, the later operand is the accumulator ----
        Acc later = R::Shfl(acc, lane + 8);
        R::Reduce(acc, later);
        if ((lane & 15) == 0) nodes[(it * 4 + wave) * 4 + (lane >> 4)] = later;
    };

    // The loads of kLoadBatch plain iterations are issued together, ahead of the arithmetic of the first of them.
    constexpr int kLoadBatch = 4;
    const In* xrow = reinterpret_cast<const In*>(xbase) + e_begin + tid * 4;
    int it = 0;
    for (; it + kLoadBatch <= plain_iters; it += kLoadBatch) {
        Group4<In> q[kLoadBatch];
#pragma unroll
        for (int u = 0; u < kLoadBatch; ++u) q[u] = LoadGroup<ALIGNED>(xrow + static_cast<int64_t>(it + u) * kElemsPerIter);
        __builtin_amdgcn_sched_barrier(0);  // all loads in flight before anything waits for the first
        plain(it, q, std::integral_constant<int, kLoadBatch>());
    }
    for (; it < plain_iters; ++it) {
        const Group4<In> q = LoadGroup<ALIGNED>(xrow + static_cast<int64_t>(it) * kElemsPerIter);
        plain(it, &q, std::integral_constant<int, 1>());
    }
    for (; it < iters; ++it) guarded(it);
    __syncthreads();

    // ---- tree over the block's nodes (a power of two, 16 to 1024): a wave folds 64 consecutive ones at a time, wave 0 then
    // folds those results (at most 16) ----
    using Op = ReduceOp<R, false>;
    const int n_nodes = iters * 16;
    Acc acc = R::Empty();
    for (int base = wave * 64; base < n_nodes; base += kRowThreads) {
        acc = base + lane < n_nodes ? nodes[base + lane] : R::Empty();  // lanes past the end hold padding
        MergeLaneAbove<Op, 1>(acc);
        MergeLaneAbove<Op, 2>(acc);
        MergeLaneAbove<Op, 4>(acc);
        MergeLaneAbove<Op, 8>(acc);
        acc = MergeRows<Op>(acc);
        if (lane == 0) wave_nodes[base >> 6] = acc;
    }
    if (n_nodes > 64) {
        __syncthreads();
        if (wave == 0) {
            acc = lane < (n_nodes >> 6) ? wave_nodes[lane] : R::Empty();
            MergeLaneAbove<Op, 1>(acc);
            MergeLaneAbove<Op, 2>(acc);
            MergeLaneAbove<Op, 4>(acc);
            MergeLaneAbove<Op, 8>(acc);
        }
    }
    if (tid == 0) {
        const typename Impl::Acc result = Impl::FromRow(acc, e_begin);
        if (blocks_per_row == 1) {
            *reinterpret_cast<typename Impl::Out*>(g.out + out_off) = Impl::MapOut(result);
        } else {
            reinterpret_cast<typename Impl::Acc*>(partials)[row * blocks_per_row + blk] = result;
        }
    }
}

// second pass: tree over the per-block partials of each row (blocks_per_row <= kMaxPartials)
template <typename Impl>
__global__ __launch_bounds__(kRowThreads) void RowFinalizeKernel(ReduceGeom g, int blocks_per_row, const void* partials) {
    using Acc = typename Impl::Acc;
    __shared__ Acc nodes[kMaxPartials];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    int n = 1;
    while (n < blocks_per_row) n <<= 1;
    const Acc* src = reinterpret_cast<const Acc*>(partials) + row * blocks_per_row;
    for (int i = tid; i < n; i += kRowThreads) nodes[i] = i < blocks_per_row ? src[i] : Impl::Empty();
    __syncthreads();
    for (int s = 1; s < n; s <<= 1) {
        for (int i = tid; (2 * i + 1) * s < n; i += kRowThreads) {
            Acc earlier = nodes[2 * i * s];
            Acc later = nodes[2 * i * s + s];
            Impl::Reduce(earlier, later);
            nodes[2 * i * s] = later;
        }
        __syncthreads();
    }
    if (tid == 0) {
        int64_t in_off, out_off;
        OutOffsets(g, row, in_off, out_off);
        *reinterpret_cast<typename Impl::Out*>(g.out + out_off) = Impl::MapOut(nodes[0]);
    }
}

// ---------------------------------------------------------------------------------------------
// Generic kernel: the reference loop, one output per thread
// ---------------------------------------------------------------------------------------------
template <typename Impl>
__global__ __launch_bounds__(256) void GenericReduceKernel(ReduceGeom g) {
    using In = typename Impl::In;
    using Acc = typename Impl::Acc;
    const int64_t o = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (o >= g.n_out) return;
    int64_t in_off, out_off;
    OutOffsets(g, o, in_off, out_off);
    const char* base = g.in + in_off;

    // odometer over the reduced axes (C order)
    int64_t cnt[kMaxDims];
    for (int d = 0; d < g.n_red; ++d) cnt[d] = 0;
    int64_t off = 0;
    int64_t i = 0;
    auto next_elem = [&]() -> Acc {
        Acc a = Impl::Map(*reinterpret_cast<const In*>(base + off), i);
        ++i;
        for (int d = g.n_red - 1; d >= 0; --d) {
            off += g.red_stride[d];
            if (++cnt[d] < g.red_shape[d]) break;
            off -= g.red_stride[d] * g.red_shape[d];
            cnt[d] = 0;
        }
        return a;
    };

    const int64_t len = g.red_len;
    const int64_t main_len = len - (len % 4);
    Acc accum = Impl::Identity();
    Acc tree[48];
    while (i < main_len) {
        if (i != 0 && i % 32 == 0) {
            int lvl = 0;
            for (int64_t k = i >> 1; k % 32 == 0; k >>= 1, ++lvl) Impl::Reduce(tree[lvl], accum);
            tree[lvl] = accum;
            accum = Impl::Identity();
        }
        Acc p0 = next_elem();
        Impl::Reduce(next_elem(), p0);
        Acc p1 = next_elem();
        Impl::Reduce(next_elem(), p1);
        Impl::Reduce(p1, p0);
        Impl::Reduce(p0, accum);
    }
    while (i < len) Impl::Reduce(next_elem(), accum);
    {
        int lvl = 0;
        for (int64_t k = (len / 4 - 1) / 8; k > 0; k >>= 1, ++lvl) {
            if (k & 1) Impl::Reduce(tree[lvl], accum);
        }
    }
    *reinterpret_cast<typename Impl::Out*>(g.out + out_off) = Impl::MapOut(accum);
}

// ---------------------------------------------------------------------------------------------
// Column kernels: one strided reduced axis, few outputs against its length (sums over the batch axis, bias gradients).
// The reduced sequence is cut into `nslices` aligned slices of 2^level 32-element blocks.  Pass 1: one thread per
// (slice, output), outputs fastest (coalesced for an inner kept axis), runs the reference loop over its slice -- whose
// result is exactly the node the sequential binary counter would hold for those blocks.  Pass 2: one thread per output
// pushes the slice nodes through the counter, then walks on through the blocks after the last slice (at least one is
// always left, so the tail and the final fold happen exactly where the reference has them).
// ---------------------------------------------------------------------------------------------
template <typename Impl>
__global__ __launch_bounds__(256) void ColumnSliceKernel(ReduceGeom g, int level, int nslices, void* partials) {
    using In = typename Impl::In;
    using Acc = typename Impl::Acc;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= g.n_out * nslices) return;
    const int64_t slice = t / g.n_out;
    const int64_t o = t - slice * g.n_out;
    int64_t in_off, out_off;
    OutOffsets(g, o, in_off, out_off);
    const int64_t stride = g.red_stride[0];
    const int64_t count = static_cast<int64_t>(32) << level;
    const int64_t i_begin = slice * count;
    const char* ptr = g.in + in_off + i_begin * stride;
    Acc accum = Impl::Identity();
    Acc tree[32];
    for (int64_t r = 0; r < count; r += 4) {
        if (r != 0 && r % 32 == 0) {
            int lvl = 0;
            for (int64_t k = r >> 1; k % 32 == 0; k >>= 1, ++lvl) Impl::Reduce(tree[lvl], accum);
            tree[lvl] = accum;
            accum = Impl::Identity();
        }
        const int64_t i = i_begin + r;
        Acc p0 = Impl::Map(*reinterpret_cast<const In*>(ptr), i);
        Impl::Reduce(Impl::Map(*reinterpret_cast<const In*>(ptr + stride), i + 1), p0);
        Acc p1 = Impl::Map(*reinterpret_cast<const In*>(ptr + 2 * stride), i + 2);
        Impl::Reduce(Impl::Map(*reinterpret_cast<const In*>(ptr + 3 * stride), i + 3), p1);
        Impl::Reduce(p1, p0);
        Impl::Reduce(p0, accum);
        ptr += 4 * stride;
    }
    for (int lvl = 0; lvl < level; ++lvl) Impl::Reduce(tree[lvl], accum);  // 2^level blocks: every lower level is pending
    reinterpret_cast<Acc*>(partials)[slice * g.n_out + o] = accum;
}

template <typename Impl>
__global__ __launch_bounds__(256) void ColumnFinishKernel(ReduceGeom g, int level, int nslices, const void* partials) {
    using In = typename Impl::In;
    using Acc = typename Impl::Acc;
    const int64_t o = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (o >= g.n_out) return;
    int64_t in_off, out_off;
    OutOffsets(g, o, in_off, out_off);
    const int64_t stride = g.red_stride[0];
    const Acc* part = reinterpret_cast<const Acc*>(partials);
    Acc tree[48];
    Acc accum;
    for (int s = 0; s < nslices; ++s) {  // the boundary merges of the reference at the end of every slice
        accum = part[static_cast<int64_t>(s) * g.n_out + o];
        int lvl = level;
        for (int t = s; t & 1; t >>= 1, ++lvl) Impl::Reduce(tree[lvl], accum);
        tree[lvl] = accum;
    }
    const int64_t len = g.red_len;
    const int64_t main_len = len - (len % 4);
    const int64_t i0 = static_cast<int64_t>(nslices) * (static_cast<int64_t>(32) << level);
    const char* ptr = g.in + in_off + i0 * stride;
    int64_t i = i0;
    accum = Impl::Identity();
    while (i < main_len) {
        if (i != i0 && i % 32 == 0) {
            int lvl = 0;
            for (int64_t k = i >> 1; k % 32 == 0; k >>= 1, ++lvl) Impl::Reduce(tree[lvl], accum);
            tree[lvl] = accum;
            accum = Impl::Identity();
        }
        Acc p0 = Impl::Map(*reinterpret_cast<const In*>(ptr), i);
        Impl::Reduce(Impl::Map(*reinterpret_cast<const In*>(ptr + stride), i + 1), p0);
        Acc p1 = Impl::Map(*reinterpret_cast<const In*>(ptr + 2 * stride), i + 2);
        Impl::Reduce(Impl::Map(*reinterpret_cast<const In*>(ptr + 3 * stride), i + 3), p1);
        Impl::Reduce(p1, p0);
        Impl::Reduce(p0, accum);
        ptr += 4 * stride;
        i += 4;
    }
    for (; i < len; ++i, ptr += stride) Impl::Reduce(Impl::Map(*reinterpret_cast<const In*>(ptr), i), accum);
    {
        int lvl = 0;
        for (int64_t k = (len / 4 - 1) / 8; k > 0; k >>= 1, ++lvl) {
            if (k & 1) Impl::Reduce(tree[lvl], accum);
        }
    }
    *reinterpret_cast<typename Impl::Out*>(g.out + out_off) = Impl::MapOut(accum);
}

// ---------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------
struct ReducePlan {
    ReduceGeom g;
    bool row_path = false;
    bool aligned = false;
    int64_t span = 0;
    int blocks_per_row = 1;
    size_t acc_size = 0;
    bool column_path = false;
    int col_level = 0;    // a slice is 2^col_level blocks of 32 elements
    int col_slices = 0;
};

ReduceGeom MakeGeom(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out) {
    ValidateArray(a, "a");
    ValidateArray(out, "out");
    bool red[kMaxDims] = {};
    int prev = -1;
    for (int i = 0; i < naxis; ++i) {
        HIPCX_REQUIRE(axis[i] >= 0 && axis[i] < a->ndim, HIPCX_DIMENSION_ERROR, "reduction axis out of range");
        HIPCX_REQUIRE(axis[i] > prev, HIPCX_DIMENSION_ERROR, "reduction axes must be sorted and unique");
        prev = axis[i];
        red[axis[i]] = true;
    }
    // out either keeps the reduced axes with extent 1 or drops them (CX/shape.cc:34-37)
    bool keepdims = out->ndim == a->ndim && naxis > 0;
    if (keepdims) {
        for (int d = 0; d < a->ndim; ++d) {
            int64_t expect = red[d] ? 1 : a->shape[d];
            if (out->shape[d] != expect) {
                keepdims = false;
                break;
            }
        }
    }
    if (!keepdims) {
        HIPCX_REQUIRE(out->ndim == a->ndim - naxis, HIPCX_DIMENSION_ERROR, "out has the wrong number of dimensions for this reduction");
        int j = 0;
        for (int d = 0; d < a->ndim; ++d) {
            if (red[d]) continue;
            HIPCX_REQUIRE(out->shape[j] == a->shape[d], HIPCX_DIMENSION_ERROR, "out has the wrong shape for this reduction");
            ++j;
        }
    }
    ReduceGeom g{};
    g.in = static_cast<const char*>(a->data);
    g.out = static_cast<char*>(out->data);
    g.n_out = 1;
    g.red_len = 1;
    int j = 0;
    for (int d = 0; d < a->ndim; ++d) {
        if (red[d]) {
            g.red_len *= a->shape[d];
            if (a->shape[d] == 1) continue;
            int n = g.n_red;
            if (n > 0 && g.red_stride[n - 1] == a->shape[d] * a->strides[d]) {  // walks on as one run
                g.red_shape[n - 1] *= a->shape[d];
                g.red_stride[n - 1] = a->strides[d];
            } else {
                g.red_shape[n] = a->shape[d];
                g.red_stride[n] = a->strides[d];
                ++g.n_red;
            }
        } else {
            int64_t ostride = keepdims ? out->strides[d] : out->strides[j];
            ++j;
            g.n_out *= a->shape[d];
            if (a->shape[d] == 1) continue;
            int n = g.n_keep;
            if (n > 0 && g.keep_in_stride[n - 1] == a->shape[d] * a->strides[d] && g.keep_out_stride[n - 1] == a->shape[d] * ostride) {
                g.keep_shape[n - 1] *= a->shape[d];
                g.keep_in_stride[n - 1] = a->strides[d];
                g.keep_out_stride[n - 1] = ostride;
            } else {
                g.keep_shape[n] = a->shape[d];
                g.keep_in_stride[n] = a->strides[d];
                g.keep_out_stride[n] = ostride;
                ++g.n_keep;
            }
        }
    }
    return g;
}

ReducePlan MakePlan(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, size_t acc_size) {
    ReducePlan pl;
    pl.g = MakeGeom(a, axis, naxis, out);
    pl.acc_size = acc_size;
    const ReduceGeom& g = pl.g;
    const int64_t it = ItemSize(a->dtype);
    // Row path: one contiguous run of at least 256 elements -- or several such runs of a multiple of four elements at a
    // constant pitch (e.g. the (0, 2, 3) axes of an NCHW array) -- short enough for 32-bit-safe bookkeeping.
    const bool one_run = g.n_red == 1 && g.red_stride[0] == it;
    const bool runs = g.n_red == 2 && g.red_stride[1] == it && g.red_shape[1] % 4 == 0 && g.red_stride[0] > 0;
    pl.g.seg_len = runs ? g.red_shape[1] : g.red_len;
    pl.g.seg_stride = runs ? g.red_stride[0] : 0;
    if ((one_run || runs) && g.red_len >= 256 && g.red_len < (1LL << 40) && g.n_out < (1LL << 31)) {
        pl.row_path = true;
        int64_t L = g.red_len;
        int64_t span = kElemsPerIter;
        while (span < L && span < static_cast<int64_t>(kMaxIters) * kElemsPerIter) span <<= 1;
        // few long rows: split rows over more blocks so that the whole chip is busy
        int64_t target_blocks = static_cast<int64_t>(NumCUs()) * 8;
        while (span > 4 * kElemsPerIter && g.n_out * ((L + span - 1) / span) < target_blocks && (L + span / 2 - 1) / (span / 2) <= kMaxPartials) {
            span >>= 1;
        }
        int64_t bpr = (L + span - 1) / span;
        if (bpr > kMaxPartials || g.n_out * bpr >= (1LL << 31)) {
            pl.row_path = false;
        } else {
            pl.span = span;
            pl.blocks_per_row = static_cast<int>(bpr);
            bool al = reinterpret_cast<uintptr_t>(g.in) % (4 * it) == 0;
            for (int d = 0; d < g.n_keep; ++d) al = al && g.keep_in_stride[d] % (4 * it) == 0;
            al = al && g.seg_stride % (4 * it) == 0;
            pl.aligned = al;
        }
    }
    // Column path: one strided reduced axis that is long against the number of outputs (one thread per output would walk it alone).
    if (!pl.row_path && g.n_red == 1 && g.red_len >= 512 && g.n_out > 0 && g.n_out < (1LL << 28)) {
        const int64_t main_len = g.red_len - g.red_len % 4;
        const int64_t nblocks = (main_len + 31) / 32;
        // Serial work of the longest thread: a slice in pass 1 (times the rounds the chip needs for all slice threads), then
        // in pass 2 the slice nodes plus the blocks behind the last slice.  Take the slice size that minimises it.
        const int64_t resident = static_cast<int64_t>(NumCUs()) * 2048;
        int best_level = -1;
        int64_t best_cost = g.red_len;  // the generic kernel's: one thread walks everything
        for (int level = 0; level < 24; ++level) {
            const int64_t slices = (nblocks - 1) >> level;  // at least one block stays behind the last slice
            if (slices < 2) break;
            if (slices > (1 << 20) || g.n_out * slices >= (1LL << 36)) continue;
            const int64_t slice_len = static_cast<int64_t>(32) << level;
            const int64_t rounds = (g.n_out * slices + resident - 1) / resident;
            const int64_t left = g.red_len - slices * slice_len;
            const int64_t cost = slice_len * rounds + slices + left;
            if (cost < best_cost) best_cost = cost, best_level = level;
        }
        if (best_level >= 0 && 2 * best_cost <= g.red_len) {
            pl.column_path = true;
            pl.col_level = best_level;
            pl.col_slices = static_cast<int>((nblocks - 1) >> best_level);
        }
    }
    return pl;
}

size_t WorkspaceBytes(const ReducePlan& pl) {
    if (pl.column_path) return static_cast<size_t>(pl.g.n_out) * pl.col_slices * pl.acc_size;
    if (!pl.row_path || pl.blocks_per_row == 1) return 0;
    return static_cast<size_t>(pl.g.n_out) * pl.blocks_per_row * pl.acc_size;
}

template <typename Impl>
void Run(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
         hipStream_t stream) {
    ReducePlan pl = MakePlan(a, axis, naxis, out, sizeof(typename Impl::Acc));
    const ReduceGeom& g = pl.g;
    if (g.n_out == 0) return;
    if (pl.row_path) {
        size_t need = WorkspaceBytes(pl);
        HIPCX_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need), HIPCX_CHAINERX_ERROR,
                      "reduction workspace too small: need " + std::to_string(need) + " bytes");
        HIPCX_REQUIRE(need == 0 || reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR,
                      "workspace must be 16-byte aligned");
        dim3 grid(static_cast<unsigned>(g.n_out * pl.blocks_per_row)), block(kRowThreads);
        if (pl.aligned) {
            hipLaunchKernelGGL((RowReduceKernel<Impl, true>), grid, block, 0, stream, g, pl.span, pl.blocks_per_row, workspace);
        } else {
            hipLaunchKernelGGL((RowReduceKernel<Impl, false>), grid, block, 0, stream, g, pl.span, pl.blocks_per_row, workspace);
        }
        CheckLaunch("row_reduce");
        if (pl.blocks_per_row > 1) {
            hipLaunchKernelGGL((RowFinalizeKernel<Impl>), dim3(static_cast<unsigned>(g.n_out)), block, 0, stream, g, pl.blocks_per_row,
                               workspace);
            CheckLaunch("row_reduce_finalize");
        }
        return;
    }
    if (pl.column_path) {
        size_t need = WorkspaceBytes(pl);
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR,
                      "reduction workspace too small: need " + std::to_string(need) + " bytes");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        const int64_t threads = g.n_out * pl.col_slices;
        hipLaunchKernelGGL((ColumnSliceKernel<Impl>), dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream, g, pl.col_level,
                           pl.col_slices, workspace);
        CheckLaunch("column_reduce_slices");
        hipLaunchKernelGGL((ColumnFinishKernel<Impl>), dim3(static_cast<unsigned>((g.n_out + 255) / 256)), dim3(256), 0, stream, g, pl.col_level,
                           pl.col_slices, workspace);
        CheckLaunch("column_reduce_finish");
        return;
    }
    int64_t blocks = (g.n_out + 255) / 256;
    HIPCX_REQUIRE(blocks < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "too many outputs for one launch");
    hipLaunchKernelGGL((GenericReduceKernel<Impl>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, g);
    CheckLaunch("generic_reduce");
}

// What a device needs for hipcx_sum_static_scratch, set up on the first call there with that device current:
//   address   the device address of `scratch`.  In host code the array's name is only a handle for this lookup, never an address a
//             kernel may be given.
//   done      an event recorded behind each call's kernels.  The array is one per device, so a call on another stream than the
//             previous one first makes its stream wait for that event: calls from different streams or host threads take turns on
//             the array instead of racing.  (Calls issued into a stream that is being captured are not chained: a graph replays at
//             times of its owner's choosing, who then orders it against other users of the array.)
struct StaticScratchSlot {
    std::mutex mu;  // host threads issue their calls one at a time
    void* address = nullptr;
    hipEvent_t done = nullptr;
    hipStream_t last = nullptr;
    bool pending = false;
};

StaticScratchSlot& StaticScratchOfCurrentDevice() {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static StaticScratchSlot slots[kMaxDevices];
    int dev = 0;
    HIPCX_CHECK_HIP(hipGetDevice(&dev));
    HIPCX_REQUIRE(dev >= 0 && dev < kMaxDevices, HIPCX_DEVICE_ERROR, "device index beyond the static scratch table");
    std::lock_guard<std::mutex> lock(mu);
    StaticScratchSlot& slot = slots[dev];
    if (slot.address == nullptr) {
        void* ptr = nullptr;
        HIPCX_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        HIPCX_REQUIRE(ptr != nullptr, HIPCX_BACKEND_ERROR, "hipGetSymbolAddress returned a null address for the static scratch");
        HIPCX_CHECK_HIP(hipEventCreateWithFlags(&slot.done, hipEventDisableTiming));
        slot.address = ptr;
    }
    return slot;
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

// Upper bound over the three reductions (they share one query): partials are at most 16 bytes each.
size_t hipcx_reduce_workspace_size(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out) {
    try {
        if (a == nullptr || out == nullptr) return 0;
        ReducePlan pl = MakePlan(a, axis, naxis, out, 16);
        return WorkspaceBytes(pl);
    } catch (...) {
        return 0;
    }
}

int hipcx_sum(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        hipStream_t st = AsStream(stream);
        const int in = a->dtype, od = out->dtype;
        // Out dtypes the routines produce: the input's float dtype, int64 for bool/int/uint inputs,
        // float32/float64 for Mean of integers (CX/routines/reduction.cc:34-49, statistics.cc:111-116).
        auto for_out = [&](auto in_tag) {
            using In = typename decltype(in_tag)::type;
            switch (od) {
                case HIPCX_INT64: Run<SumImpl<In, int64_t>>(a, axis, naxis, out, workspace, workspace_bytes, st); break;
                case HIPCX_FLOAT16: Run<SumImpl<In, half_t>>(a, axis, naxis, out, workspace, workspace_bytes, st); break;
                case HIPCX_FLOAT32: Run<SumImpl<In, float>>(a, axis, naxis, out, workspace, workspace_bytes, st); break;
                case HIPCX_FLOAT64: Run<SumImpl<In, double>>(a, axis, naxis, out, workspace, workspace_bytes, st); break;
                default:
                    throw Error(HIPCX_NOT_IMPLEMENTED_ERROR, std::string("hip sum: unsupported output dtype ") + DtypeName(od));
            }
        };
        VisitDtype(in, for_out);
    });
}

// hipcx_sum for callers that can neither allocate a workspace nor have one allocated for them: the per-block / per-slice
// partial results go to the library's own static device array.  Same kernels and launch plan as hipcx_sum, hence the same bits.
// Every partial is written before it is read, so nothing has to be cleared between calls; calls from different streams or host
// threads on one device share the array and are chained through an event (see StaticScratchSlot) -- except under stream capture.
int hipcx_sum_static_scratch(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* stream) {
    int status = Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        const size_t need = hipcx_reduce_workspace_size(a, axis, naxis, out);
        HIPCX_REQUIRE(need <= HIPCX_STATIC_SCRATCH_BYTES, HIPCX_CHAINERX_ERROR,
                      "sum_static_scratch: this reduction needs " + std::to_string(need) + " bytes of partial results, the static scratch holds " +
                              std::to_string(static_cast<size_t>(HIPCX_STATIC_SCRATCH_BYTES)) + "; use hipcx_sum with a workspace");
    });
    if (status != HIPCX_OK) return status;
    StaticScratchSlot* slot = nullptr;
    status = Guard([&] { slot = &StaticScratchOfCurrentDevice(); });
    if (status != HIPCX_OK) return status;
    std::lock_guard<std::mutex> lock(slot->mu);
    hipStream_t s = AsStream(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capture) != hipSuccess) {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusActive;  // cannot tell: leave the stream alone
    }
    const bool chained = capture == hipStreamCaptureStatusNone;
    if (chained && slot->pending && slot->last != s) {
        status = Guard([&] { HIPCX_CHECK_HIP(hipStreamWaitEvent(s, slot->done, 0)); });
        if (status != HIPCX_OK) return status;
    }
    status = hipcx_sum(a, axis, naxis, out, slot->address, HIPCX_STATIC_SCRATCH_BYTES, stream);
    if (chained) {
        int recorded = Guard([&] { HIPCX_CHECK_HIP(hipEventRecord(slot->done, s)); });
        if (recorded == HIPCX_OK) {
            slot->last = s;
            slot->pending = true;
        } else if (status == HIPCX_OK) {
            status = recorded;
        }
    }
    return status;
}

int hipcx_amax(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
               void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(a->dtype == out->dtype, HIPCX_DTYPE_ERROR, "amax: out must have a's dtype");
        for (int i = 0; i < naxis; ++i) {
            HIPCX_REQUIRE(axis[i] >= 0 && axis[i] < a->ndim && a->shape[axis[i]] > 0, HIPCX_DIMENSION_ERROR,
                          "cannot compute the maximum along zero-sized axis");
        }
        VisitDtype(a->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            Run<AMaxImpl<T>>(a, axis, naxis, out, workspace, workspace_bytes, AsStream(stream));
        });
    });
}

int hipcx_argmax(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
                 void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(out->dtype == HIPCX_INT64, HIPCX_DTYPE_ERROR, "argmax: out must be int64");
        for (int i = 0; i < naxis; ++i) {
            HIPCX_REQUIRE(axis[i] >= 0 && axis[i] < a->ndim && a->shape[axis[i]] > 0, HIPCX_DIMENSION_ERROR,
                          "cannot compute ArgMax for an empty array");
        }
        VisitDtype(a->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            Run<ArgMaxImpl<T>>(a, axis, naxis, out, workspace, workspace_bytes, AsStream(stream));
        });
    });
}

int hipcx_amin(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
               void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(a->dtype == out->dtype, HIPCX_DTYPE_ERROR, "amin: out must have a's dtype");
        for (int i = 0; i < naxis; ++i) {
            HIPCX_REQUIRE(axis[i] >= 0 && axis[i] < a->ndim && a->shape[axis[i]] > 0, HIPCX_DIMENSION_ERROR,
                          "cannot compute the minimum along zero-sized axis");
        }
        VisitDtype(a->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            Run<AMaxImpl<T, true>>(a, axis, naxis, out, workspace, workspace_bytes, AsStream(stream));
        });
    });
}

int hipcx_argmin(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
                 void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(out->dtype == HIPCX_INT64, HIPCX_DTYPE_ERROR, "argmin: out must be int64");
        for (int i = 0; i < naxis; ++i) {
            HIPCX_REQUIRE(axis[i] >= 0 && axis[i] < a->ndim && a->shape[axis[i]] > 0, HIPCX_DIMENSION_ERROR,
                          "cannot compute ArgMin for an empty array");
        }
        VisitDtype(a->dtype, [&](auto tag) {
            using T = typename decltype(tag)::type;
            Run<ArgMaxImpl<T, true>>(a, axis, naxis, out, workspace, workspace_bytes, AsStream(stream));
        });
    });
}

int hipcx_all(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(a->dtype == HIPCX_BOOL && out->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "all: a and out must be bool (cast with hipcx_copy first)");
        Run<AllAnyImpl<true>>(a, axis, naxis, out, workspace, workspace_bytes, AsStream(stream));
    });
}

int hipcx_any(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(a->dtype == HIPCX_BOOL && out->dtype == HIPCX_BOOL, HIPCX_DTYPE_ERROR, "any: a and out must be bool (cast with hipcx_copy first)");
        Run<AllAnyImpl<false>>(a, axis, naxis, out, workspace, workspace_bytes, AsStream(stream));
    });
}
}
