// Dot (CX/kernels/linalg.h:15) and Conv forward (CX/kernels/connection.h:21) on the MFMA
// implicit-GEMM core.  The arithmetic contract is the native backend's: products of the stored
// values accumulated in fp32 (fp64 for float64) and rounded once to the output dtype
// (CX/native/native_device/dot.cc:181-227, conv.cc:41-89).
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <utility>
#include <vector>

#include "gemm_pp.h"
#include "igemm.h"
#include "igemm_pipe.h"
#include "layout_kernels.h"
#include "nchw_conv.h"
#include "pw_conv.h"
#include "stem_conv.h"
#include "small_dot.h"

namespace hipcx {
namespace {

// Optional event bracketing of every implicit-GEMM launch (hipcx_profile_start/stop): the events are
// recorded on the launch stream right before and after the kernel, so their elapsed time is the
// kernel's own duration and excludes the filter repack and any host work.
struct ProfileRecord {  // one bracketed launch
    double ms, flops, bytes;
};
struct ProfileState {
    bool on = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> events;
    std::vector<ProfileRecord> records;  // flops and bytes at launch; ms filled in by stop
    double flops = 0.0;
    double bytes = 0.0;
};
ProfileState g_profile;
std::mutex g_profile_mutex;  // launches from several host threads may record into one profiling window

struct ProfileScope {
    hipStream_t stream;
    hipEvent_t stop = nullptr;
    ProfileScope(hipStream_t s, double flops, double bytes) : stream(s) {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        if (!g_profile.on) return;
        hipEvent_t start = nullptr;
        HIPCX_CHECK_HIP(hipEventCreate(&start));
        HIPCX_CHECK_HIP(hipEventCreate(&stop));
        g_profile.events.emplace_back(start, stop);
        g_profile.records.push_back(ProfileRecord{0.0, flops, bytes});
        g_profile.flops += flops;
        g_profile.bytes += bytes;
        HIPCX_CHECK_HIP(hipEventRecord(start, stream));
    }
    ~ProfileScope() {
        if (stop != nullptr) (void)hipEventRecord(stop, stream);
    }
};

// Raises a kernel's dynamic LDS limit when a launch needs more than it has been given so far.  The limit is a property of the
// function on one device; several host threads may launch the same kernel, so the bookkeeping is per kernel instantiation
// (the Tag type), per device, and serialised (the reference serialises its launchers on a mutex too, CX/cuda/elementwise.cuh:38).
template <typename Tag>
void EnsureDynamicLds(const void* kernel, int lds_bytes) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static int configured[kMaxDevices] = {};
    int dev = 0;
    HIPCX_CHECK_HIP(hipGetDevice(&dev));
    HIPCX_REQUIRE(dev >= 0 && dev < kMaxDevices, HIPCX_DEVICE_ERROR, "device index out of range");
    std::lock_guard<std::mutex> lock(mu);
    if (lds_bytes > configured[dev]) {
        HIPCX_CHECK_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
        configured[dev] = lds_bytes;
    }
}

template <typename T, int WM, int WN, bool PM>
void LaunchShape(IGemmArgs<T> p, bool fast16, bool fast8, hipStream_t stream) {
    constexpr int BM = 64 * WM, BN = 64 * WN;
    p.tiles_m = static_cast<int>((p.M + BM - 1) / BM);
    p.tiles_n = (p.K + BN - 1) / BN;
    int64_t total = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    HIPCX_REQUIRE(total < (1LL << 30), HIPCX_NOT_IMPLEMENTED_ERROR, "problem too large for one launch");
    int per = static_cast<int>((total + 7) / 8);
    // wide products: a row of concurrent tiles would read more second-operand panels than an XCD's L2 holds
    static const int band_env = [] { const char* e = getenv("HIPCX_IGEMM_BAND"); return e != nullptr ? atoi(e) : 8; }();
    p.band = p.tiles_n > 16 ? band_env : 0;
    static const bool pipe_env = [] { const char* e = getenv("HIPCX_IGEMM_PIPE"); return e != nullptr && e[0] == '1'; }();
    if (PM || pipe_env || !(fast16 || fast8) || p.partial == nullptr) p.ksplit = 1;  // only the simple fast kernel splits the reduction
    dim3 grid(per * 8, 1), block(64 * WM * WN);
    if (p.ksplit > 1 && total > 65535) p.ksplit = 1;  // never planned for that many tiles; the grid's y extent could not hold them
    if (p.ksplit > 1) grid = dim3(p.ksplit, static_cast<unsigned>(total));  // slices along x: see IGemmFastKernel
    // algorithmic work of this launch: 2 flops per multiply-add; every operand byte moved once
    double flops = 2.0 * static_cast<double>(p.M) * p.K * p.R * p.S * p.C_logical;
    double bytes = sizeof(T) * (static_cast<double>(p.N) * p.C_logical * p.H_logical * p.W_logical +
                                static_cast<double>(p.K) * p.R * p.S * p.C_logical + static_cast<double>(p.M) * p.K);
    ProfileScope prof(stream, flops, bytes);
    // the pipelined kernel indexes x and w with 32-bit element offsets
    double x_elems = static_cast<double>(p.N) * (p.xsN > 0 ? p.xsN : 1);
    bool fits32 = x_elems < 2147483647.0 && static_cast<double>(p.K) * p.wsK < 2147483647.0;
    static const bool use_pipe = [] { const char* e = getenv("HIPCX_IGEMM_PIPE"); return e != nullptr && e[0] == '1'; }();
    HIPCX_REQUIRE(p.batch == 0 || ((fast16 || fast8) && !PM), HIPCX_NOT_IMPLEMENTED_ERROR, "batched products need operands in the MFMA layout");
    if ((fast16 || fast8) && fits32 && use_pipe && p.batch == 0) {
        constexpr int lds_bytes = PipeLdsBytes<T, WM, WN, PM>();
        if (fast16) {
            auto kern = IGemmPipeKernel<T, WM, WN, 16, PM>;
            struct Tag16 {};
            EnsureDynamicLds<Tag16>(reinterpret_cast<const void*>(kern), lds_bytes);
            hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, p);
        } else {
            auto kern = IGemmPipeKernel<T, WM, WN, 8, PM>;
            struct Tag8 {};
            EnsureDynamicLds<Tag8>(reinterpret_cast<const void*>(kern), lds_bytes);
            hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, p);
        }
    } else if (fast16) {
        hipLaunchKernelGGL((IGemmFastKernel<T, WM, WN, 16, PM>), grid, block, 0, stream, p);
    } else if (fast8) {
        hipLaunchKernelGGL((IGemmFastKernel<T, WM, WN, 8, PM>), grid, block, 0, stream, p);
    } else {
        int x_row_fast = p.xsC != 1;
        int w_row_fast = p.wsK == 1;
        hipLaunchKernelGGL((IGemmGenericKernel<T, WM, WN, PM>), grid, block, 0, stream, p, x_row_fast, w_row_fast);
    }
    CheckLaunch("igemm");
    if (p.ksplit > 1) {
        int64_t blocks = (p.M * p.K + 63) / 64;  // 64 outputs per workgroup
        int64_t cap = static_cast<int64_t>(NumCUs()) * 16;
        hipLaunchKernelGGL((SplitKReduceKernel<T>), dim3(static_cast<unsigned>(blocks > cap ? cap : blocks)), dim3(256), 0, stream, p);
        CheckLaunch("igemm split reduction");
    }
}

size_t RoundUpTo(size_t v, size_t a) { return (v + a - 1) / a * a; }

bool Aligned(const void* ptr, int64_t bytes) { return reinterpret_cast<uintptr_t>(ptr) % bytes == 0; }

template <typename T>
bool FastOk(const IGemmArgs<T>& p, int lb) {
    const int epc = lb / static_cast<int>(sizeof(T));
    if (p.xsC != 1 || p.wsC != 1) return false;
    if (p.wsS != p.C || p.wsR != static_cast<int64_t>(p.S) * p.C) return false;  // rows dense in (r,s,c)
    if (p.C % epc != 0) return false;
    if (!Aligned(p.x, lb) || !Aligned(p.w, lb)) return false;
    if (p.xsN % epc || p.xsH % epc || p.xsW % epc || p.wsK % epc) return false;
    return true;
}

template <typename T>
void LaunchIGemmImpl(IGemmArgs<T> p, hipStream_t stream) {
    if (p.M == 0 || p.K == 0) return;
    if (p.C_logical == 0) {
        p.C_logical = p.C;
        p.H_logical = p.H;
        p.W_logical = p.W;
    }
    // accumulator orientation follows the output's fastest axis
    int64_t a_c = p.osC < 0 ? -p.osC : p.osC, a_w = p.osW < 0 ? -p.osW : p.osW;
    bool pm = !(a_c == 1) && (p.OH * p.OW > 1) && a_w <= a_c;
    if (pm) {
        int64_t ohw = static_cast<int64_t>(p.OH) * p.OW;
        p.out_vec = (p.osW == 1 && (p.OH == 1 || p.osH == p.OW) && ohw % 4 == 0 && Aligned(p.out, sizeof(T) * 4) && p.osN % 4 == 0 &&
                     p.osC % 4 == 0) ? 1 : 0;
    } else {
        p.out_vec = (p.osC == 1 && p.K % 4 == 0 && Aligned(p.out, sizeof(T) * 4) && p.osN % 4 == 0 && p.osH % 4 == 0 &&
                     p.osW % 4 == 0) ? 1 : 0;
    }
    {
        const int epv = 16 / static_cast<int>(sizeof(T));
        int64_t ohw = static_cast<int64_t>(p.OH) * p.OW;
        if (pm) {
            p.out_wide = (p.osW == 1 && (p.OH == 1 || p.osH == p.OW) && ohw % epv == 0 && Aligned(p.out, 16) && p.osN % epv == 0 &&
                          p.osC % epv == 0) ? 1 : 0;
        } else {
            p.out_wide = (p.osC == 1 && p.K % epv == 0 && Aligned(p.out, 16) && p.osN % epv == 0 && p.osH % epv == 0 &&
                          p.osW % epv == 0) ? 1 : 0;
        }
    }
    bool fast16 = FastOk(p, 16);
    bool fast8 = !fast16 && FastOk(p, 8);
    // Small problems (batch-sized matrix products such as Linear on 100-128 rows): at 128x128 the grid would leave most of
    // the 256 CUs idle, so they run as one-wave 64x64 tiles instead.
    const int64_t big_tiles = ((p.M + 127) / 128) * ((p.K + 127) / 128);
    if (p.ksplit > 1 && !pm && (fast16 || fast8)) {
        LaunchShape<T, 2, 2, false>(p, fast16, fast8, stream);
    } else if (big_tiles < 128 && p.M * static_cast<int64_t>(p.K) >= 64 * 64) {
        if (pm) LaunchShape<T, 1, 1, true>(p, fast16, fast8, stream);
        else LaunchShape<T, 1, 1, false>(p, fast16, fast8, stream);
    } else if (p.K <= 64) {
        if (pm) LaunchShape<T, 4, 1, true>(p, fast16, fast8, stream);
        else LaunchShape<T, 4, 1, false>(p, fast16, fast8, stream);
    } else {
        if (pm) LaunchShape<T, 2, 2, true>(p, fast16, fast8, stream);
        else LaunchShape<T, 2, 2, false>(p, fast16, fast8, stream);
    }
}


// Large float16 products with both operands' reduction index at unit stride (gemm_pp.h).  Returns false when the problem does
// not qualify: the 128 x 128 kernels below then take it.
bool TryGemmPp(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, hipStream_t stream) {
    static const bool enabled = [] { const char* e = getenv("HIPCX_DOT_PP"); return e == nullptr || e[0] != '0'; }();
    static const int band = [] { const char* e = getenv("HIPCX_DOT_PP_BAND"); return e != nullptr && atoi(e) > 0 ? atoi(e) : 8; }();
    if (!enabled) return false;
    const int64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    if (K % 32 != 0 || K < gemm_pp::kMinK || N % 4 != 0) return false;
    // a: rows of K contiguous halves; b: columns of K contiguous halves (the view Linear hands over, or a staged copy)
    if (a->strides[1] != 2 || b->strides[0] != 2 || out->strides[1] != 2) return false;
    const int64_t lda = a->strides[0] / 2, ldb = b->strides[1] / 2, ldc = out->strides[0] / 2;
    if (a->strides[0] % 16 != 0 || b->strides[1] % 16 != 0 || out->strides[0] % 8 != 0 || lda < K || ldb < K || ldc < N) return false;
    if (reinterpret_cast<uintptr_t>(a->data) % 16 != 0 || reinterpret_cast<uintptr_t>(b->data) % 16 != 0 || reinterpret_cast<uintptr_t>(out->data) % 8 != 0) return false;
    if (256 * lda * 2 >= (1LL << 31) || 256 * ldb * 2 >= (1LL << 31)) return false;  // 32-bit offsets inside a tile's rows
    const int64_t tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
    // enough 256 x 256 tiles to occupy most of the chip; smaller products fill it better with 128 x 128 tiles
    if (tiles_m * tiles_n < (NumCUs() * 3) / 4 || tiles_m * tiles_n >= (1LL << 24)) return false;
    gemm_pp::GemmArgs p{};
    p.a = static_cast<const half_t*>(a->data);
    p.b = static_cast<const half_t*>(b->data);
    p.c = static_cast<half_t*>(out->data);
    p.M = static_cast<int>(M);
    p.N = static_cast<int>(N);
    p.K = static_cast<int>(K);
    p.lda = static_cast<int>(lda);
    p.ldb = static_cast<int>(ldb);
    p.ldc = static_cast<int>(ldc);
    p.tiles_m = static_cast<int>(tiles_m);
    p.tiles_n = static_cast<int>(tiles_n);
    p.band = band;
    ProfileScope prof(stream, 2.0 * static_cast<double>(M) * N * K, 2.0 * (static_cast<double>(M) * K + static_cast<double>(N) * K + static_cast<double>(M) * N));
    struct GemmPpTag {};
    EnsureDynamicLds<GemmPpTag>(reinterpret_cast<const void*>(gemm_pp::GemmPpKernel), gemm_pp::kLdsBytes);
    const unsigned grid = static_cast<unsigned>((tiles_m * tiles_n + 7) / 8 * 8);
    hipLaunchKernelGGL(gemm_pp::GemmPpKernel, dim3(grid), dim3(512), gemm_pp::kLdsBytes, stream, p);
    CheckLaunch("gemm_pp");
    return true;
}

// Small-output matrix products (small_dot.h).  Returns false when the problem does not qualify.
template <typename T>
bool TrySmallDot(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, hipStream_t stream) {
    static const bool enabled = [] { const char* e = getenv("HIPCX_SMALL_DOT"); return e == nullptr || e[0] != '0'; }();
    if (!enabled) return false;
    const int64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    const int64_t it = sizeof(T);
    if (((M + 127) / 128) * ((N + 127) / 128) >= 128 || K < 64) return false;
    for (const hipcx_array* x : {a, b, out}) {
        if (x->strides[0] < 0 || x->strides[1] < 0 || x->strides[0] % it || x->strides[1] % it) return false;
    }
    SmallDotArgs p{};
    p.a = a->data;
    p.b = b->data;
    p.out = out->data;
    p.M = static_cast<int>(M);
    p.N = static_cast<int>(N);
    p.K = static_cast<int>(K);
    p.a_row = a->strides[0] / it;
    p.a_k = a->strides[1] / it;
    p.b_k = b->strides[0] / it;
    p.b_col = b->strides[1] / it;
    p.o_row = out->strides[0] / it;
    p.o_col = out->strides[1] / it;
    int64_t a_span = ((M - 1) * p.a_row + (K - 1) * p.a_k + 1) * it, b_span = ((K - 1) * p.b_k + (N - 1) * p.b_col + 1) * it;
    if (a_span >= (1LL << 31) || b_span >= (1LL << 31)) return false;
    p.a_bytes = static_cast<unsigned>(a_span);
    p.b_bytes = static_cast<unsigned>(b_span);
    auto dword_ok = [&](const void* ptr, int64_t line_stride) { return reinterpret_cast<uintptr_t>(ptr) % 4 == 0 && (line_stride * it) % 4 == 0; };
    p.a_vec = (p.a_k == 1 && dword_ok(a->data, p.a_row)) ? 1 : 0;
    p.b_vec = (p.b_k == 1 && dword_ok(b->data, p.b_col)) ? 1 : 0;
    p.tiles_n = static_cast<int>((N + 31) / 32);
    int64_t blocks = ((M + 31) / 32) * p.tiles_n;
    ProfileScope prof(stream, 2.0 * M * N * K, static_cast<double>(it) * (M * K + K * N + M * N));
    static const bool rows_ok = [] { const char* e = getenv("HIPCX_SMALL_DOT_ROWS"); return e == nullptr || e[0] != '0'; }();
    // whole-line loads regrouped through LDS pay off once the product is large enough to be bandwidth-bound (measured: the
    // 10000-column projection of the language model gains 15 %, the 2600- and 1000-column layers lose 10 %)
    if (rows_ok && p.a_vec && p.b_vec && 2.0 * M * N * K >= 1e9) {
        // Waves per workgroup = ways K is split: the choice that leaves the busiest SIMD the least matrix work
        // (wave-tiles are dealt over 4 SIMDs per CU; a wave's share is whole 128-byte steps).
        const int64_t steps = (K * it + 127) / 128;
        const int64_t simds = static_cast<int64_t>(NumCUs()) * 4;
        int best_nw = 1;
        int64_t best_cost = -1;
        for (int nw : {1, 2, 3, 4, 6, 8}) {
            if (nw > steps) break;
            int64_t rounds = (blocks * nw + simds - 1) / simds;
            int64_t cost = rounds * ((steps + nw - 1) / nw) * 8 + nw;  // + the partial-sum pass
            if (best_cost < 0 || cost < best_cost) best_cost = cost, best_nw = nw;
        }
        p.nw = best_nw;
        const int lds_bytes = best_nw * 2 * 32 * 144;
        struct RowsTag {};
        EnsureDynamicLds<RowsTag>(reinterpret_cast<const void*>(SmallDotRowsKernel<T>), 8 * 2 * 32 * 144);
        hipLaunchKernelGGL((SmallDotRowsKernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(64 * best_nw), lds_bytes, stream, p);
        CheckLaunch("small_dot_rows");
        return true;
    }
    hipLaunchKernelGGL((SmallDotKernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(512), 0, stream, p);
    CheckLaunch("small_dot");
    return true;
}

// float64 (no MFMA path yet): one thread per output element, fma in reduction order.
__global__ void ConvNaiveF64Kernel(IGemmArgs<double> p) {
    int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    int64_t total = p.M * p.K;
    if (idx >= total) return;
    int n = static_cast<int>(idx % p.K);
    int64_t m = idx / p.K;
    int ow = static_cast<int>(m % p.OW);
    int64_t t = m / p.OW;
    int oh = static_cast<int>(t % p.OH);
    int64_t img = t / p.OH;
    double acc = 0.0;
    for (int c = 0; c < p.C; ++c) {
        for (int r = 0; r < p.R; ++r) {
            int ih = oh * p.stride_h - p.pad_h + r;
            if (ih < 0 || ih >= p.H) continue;
            for (int s = 0; s < p.S; ++s) {
                int iw = ow * p.stride_w - p.pad_w + s;
                if (iw < 0 || iw >= p.W) continue;
                acc = fma(p.x[img * p.xsN + c * p.xsC + ih * p.xsH + iw * p.xsW],
                          p.w[static_cast<int64_t>(n) * p.wsK + c * p.wsC + r * p.wsR + s * p.wsS], acc);
            }
        }
    }
    if (p.bias != nullptr) acc += p.bias[n * p.bias_stride];
    p.out[img * p.osN + n * p.osC + oh * p.osH + ow * p.osW] = acc;
}

// float64 on the matrix cores: implicit GEMM with v_mfma_f64_16x16x4f64, any strides (operands are gathered).
// A workgroup (4 waves, 2 x 2) computes a 64 (output positions) x 64 (filters) tile; the reduction index k = (c, r, s) advances
// in chunks of 16 that are gathered into registers one chunk ahead and staged through LDS (two buffers, one barrier per chunk):
//   As[k][m]  k-major, written with consecutive lanes along m (consecutive pixels: contiguous for NCHW at stride 1)
//   Bs[n][k]  n-major, written with consecutive lanes along k (contiguous for dense filters)
// MFMA operands: A lane l <-> (m = l % 16, k = l / 16), B lane l <-> (k = l / 16, n = l % 16); the accumulator register i of lane l
// is D[m = 4 * i + l / 16][n = l % 16].  Products are summed in k order chunk by chunk, in double: equal to the sequential
// loop to rounding (tests: 1e-12).
constexpr int kF64TileM = 64, kF64TileN = 64, kF64Chunk = 16;
using double4_t = __attribute__((ext_vector_type(4))) double;

__global__ __launch_bounds__(256) void ConvMfmaF64Kernel(IGemmArgs<double> p) {
    __shared__ double As[2][kF64Chunk][kF64TileM + 2];
    __shared__ double Bs[2][kF64TileN][kF64Chunk + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave & 1) * 32, wn = (wave >> 1) * 32;
    const int64_t bm = static_cast<int64_t>(blockIdx.x % p.tiles_m) * kF64TileM;
    const int bn = static_cast<int>(blockIdx.x / p.tiles_m) * kF64TileN;
    const int RS = p.R * p.S;

    // ---- A gather: this thread's output position, and k = k0 + a_kk + 4 * i ----
    const int a_m = tid & 63, a_kk = tid >> 6;
    const int64_t m = bm + a_m;
    const bool m_ok = m < p.M;
    int ih0 = 0, iw0 = 0;
    const double* xb = p.x;
    if (m_ok) {
        const int ow = static_cast<int>(m % p.OW);
        const int64_t t = m / p.OW;
        const int oh = static_cast<int>(t % p.OH);
        const int64_t img = t / p.OH;
        ih0 = oh * p.stride_h - p.pad_h;
        iw0 = ow * p.stride_w - p.pad_w;
        xb = p.x + img * p.xsN + ih0 * p.xsH + iw0 * p.xsW;
    }
    // ---- B gather: k = k0 + b_kk, filters n = bn + b_n + 16 * i ----
    const int b_kk = tid & 15, b_n = tid >> 4;
    double ra[4], rb[4];
    auto gather = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + a_kk + 4 * i;
            double v = 0.0;
            if (m_ok && k < p.Kg) {
                int c = k, r = 0, s2 = 0;
                if (RS != 1) {  // (uniform) a matrix product or a 1x1 filter needs no division
                    c = k / RS;
                    const int rs = k - c * RS;
                    r = rs / p.S;
                    s2 = rs - r * p.S;
                }
                const int ih = ih0 + r, iw = iw0 + s2;
                if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) v = xb[c * p.xsC + r * p.xsH + s2 * p.xsW];
            }
            ra[i] = v;
        }
        const int k = k0 + b_kk;
        int64_t woff = 0;
        if (k < p.Kg) {
            int c = k, r = 0, s2 = 0;
            if (RS != 1) {
                c = k / RS;
                const int rs = k - c * RS;
                r = rs / p.S;
                s2 = rs - r * p.S;
            }
            woff = c * p.wsC + r * p.wsR + s2 * p.wsS;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = bn + b_n + 16 * i;
            rb[i] = (k < p.Kg && n < p.K) ? p.w[static_cast<int64_t>(n) * p.wsK + woff] : 0.0;
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            As[buf][a_kk + 4 * i][a_m] = ra[i];
            Bs[buf][b_n + 16 * i][b_kk] = rb[i];
        }
    };

    double4_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};
    }
    const int nchunks = (p.Kg + kF64Chunk - 1) / kF64Chunk;
    gather(0);
    stage(0);
    __syncthreads();
    for (int ch = 0; ch < nchunks; ++ch) {
        const int cur = ch & 1;
        if (ch + 1 < nchunks) gather((ch + 1) * kF64Chunk);
#pragma unroll
        for (int ks = 0; ks < kF64Chunk / 4; ++ks) {
            double a[2], b[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                a[t] = As[cur][ks * 4 + (lane >> 4)][wm + t * 16 + (lane & 15)];
                b[t] = Bs[cur][wn + t * 16 + (lane & 15)][ks * 4 + (lane >> 4)];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        }
        if (ch + 1 < nchunks) stage(cur ^ 1);  // the other buffer: its readers passed the barrier of the previous chunk
        __syncthreads();
    }

    // ---- epilogue: bias, scatter through out's strides ----
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t mo = bm + wm + i * 16 + 4 * e + (lane >> 4);
            if (mo >= p.M) continue;
            const int ow = static_cast<int>(mo % p.OW);
            const int64_t t = mo / p.OW;
            const int oh = static_cast<int>(t % p.OH);
            const int64_t img = t / p.OH;
            double* ob = p.out + img * p.osN + oh * p.osH + ow * p.osW;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int n = bn + wn + j * 16 + (lane & 15);
                if (n >= p.K) continue;
                double v = acc[i][j][e];
                if (p.bias != nullptr) v += p.bias[n * p.bias_stride];
                ob[n * p.osC] = v;
            }
        }
    }
}

void LaunchF64(IGemmArgs<double> p, hipStream_t stream) {
    int64_t total = p.M * p.K;
    if (total == 0) return;
    if (total * p.Kg < (1 << 16) || p.Kg == 0) {  // a few thousand multiply-adds: not worth mostly empty tiles
        int64_t blocks = (total + 255) / 256;
        hipLaunchKernelGGL(ConvNaiveF64Kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p);
        CheckLaunch("conv_f64");
        return;
    }
    const int64_t tiles_m = (p.M + kF64TileM - 1) / kF64TileM, tiles_n = (p.K + kF64TileN - 1) / kF64TileN;
    HIPCX_REQUIRE(tiles_m * tiles_n < (1LL << 31) && tiles_m < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "problem too large for one launch");
    p.tiles_m = static_cast<int>(tiles_m);
    p.tiles_n = static_cast<int>(tiles_n);
    ProfileScope prof(stream, 2.0 * static_cast<double>(p.M) * p.K * p.Kg,
                      8.0 * (static_cast<double>(p.N) * p.C * p.H * p.W + static_cast<double>(p.K) * p.Kg + static_cast<double>(p.M) * p.K));
    hipLaunchKernelGGL(ConvMfmaF64Kernel, dim3(static_cast<unsigned>(tiles_m * tiles_n)), dim3(256), 0, stream, p);
    CheckLaunch("conv_mfma_f64");
}

int64_t ElemStride(const hipcx_array* a, int axis, const char* name) {
    int64_t it = ItemSize(a->dtype);
    HIPCX_REQUIRE(a->strides[axis] % it == 0, HIPCX_NOT_IMPLEMENTED_ERROR,
                  std::string(name) + ": byte strides must be multiples of the item size");
    return a->strides[axis] / it;
}


// ---- float16 NCHW-native path (nchw_conv.h) ----
struct NchwPlan {
    bool ok = false;
    int taps = 1, npx = 1, ck = 32, wpx = 4, wch = 1, maxi = 1, ksplit = 1;
    int nrow = 0, nslot = 0;
    size_t wp_bytes = 0;
    int lds_bytes = 0;
};

NchwPlan PlanNchw(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out, const int64_t* stride, const int64_t* pad) {
    NchwPlan pl;
    static const bool enabled = [] { const char* e = getenv("HIPCX_CONV_NCHW"); return e == nullptr || e[0] != '0'; }();
    if (!enabled || x->dtype != HIPCX_FLOAT16) return pl;
    if (!IsContiguous(x) || !IsContiguous(out)) return pl;
    const int64_t N = x->shape[0], C = x->shape[1], H = x->shape[2], W = x->shape[3];
    const int64_t K = w->shape[0], R = w->shape[2], S = w->shape[3];
    const int64_t OH = out->shape[2], OW = out->shape[3];
    if (N * C * H * W * 2 >= (1LL << 31) || N * K * OH * OW * 2 >= (1LL << 31) || K * C * R * S * 2 >= (1LL << 31)) return pl;
    if (reinterpret_cast<uintptr_t>(x->data) % 16 != 0 || reinterpret_cast<uintptr_t>(out->data) % 16 != 0) return pl;
    const bool is1 = R == 1 && S == 1 && pad[0] == 0 && pad[1] == 0 && stride[0] == stride[1];
    const bool is3 = R == 3 && S == 3 && pad[0] == 1 && pad[1] == 1 && stride[0] == 1 && stride[1] == 1;
    if (!is1 && !is3) return pl;
    const int64_t P = OH * OW;
    // Pixels per activation load.  Wider loads would be fewer, but a thread's transposed 16-byte groups go to LDS
    // NPX slots apart from its neighbour's, and beyond a 32-byte lane stride those writes serialise on LDS banks
    // (measured: 16 clk per wave instruction at 32 bytes, 32 at 64, 64 at 128).
    auto pick = [](int64_t n) { return n % 2 == 0 ? 2 : 1; };
    if (is1) {
        if (C % 32 != 0) return pl;
        pl.taps = 1;
        pl.ck = 32;
        pl.npx = stride[0] == 1 ? pick(P) : 1;
        if (K <= 64) {
            pl.wpx = 4, pl.wch = 1;
        } else if (K >= 256 && pl.npx == 1) {
            // single-pixel gathers (strided or odd-sized planes) are the expensive part of a tile: 128 pixels x 256 channels with
            // 8 waves gathers and transposes each activation tile once for 256 output channels instead of 128
            pl.wpx = 2, pl.wch = 4;
            // too few such tiles to occupy the chip (deep layers at small batch x plane): halve the pixel extent
            if (((N * P + 127) / 128) * ((K + 255) / 256) < 128) pl.wpx = 1;
        } else {
            pl.wpx = 2, pl.wch = 2;
        }
        pl.maxi = std::max(1, pl.ck / 8 / (pl.npx * pl.wch));  // 64*wpx/npx pixel runs x ck/8 channel groups over 64*wpx*wch threads
        pl.nslot = 64 * pl.wpx;
    } else {
        if (C % 16 != 0) return pl;
        pl.taps = 9;
        pl.ck = 16;
        pl.npx = pick(W);
        pl.wpx = 4, pl.wch = 1;
        const int64_t BM = 64 * pl.wpx;
        int64_t rows = (BM + W - 2) / W + 1;
        int64_t cross = (BM + P - 2) / P;
        pl.nrow = static_cast<int>(rows + 2 * cross + 2);
        pl.nslot = pl.nrow * static_cast<int>(W + 2);
        int64_t items = static_cast<int64_t>(pl.nrow) * (W / pl.npx) * (pl.ck / 8);
        const int64_t nt = 64 * pl.wpx;
        pl.maxi = items <= 2 * nt ? 2 : 4;
        if (items > pl.maxi * nt) return pl;
    }
    const int cg = pl.ck / 8;
    const int bn = 64 * pl.wch;
    const int stage_bytes = cg * pl.nslot * 16 + cg * (pl.taps * bn * 16 + (pl.taps == 1 ? 64 : 0));
    // At most one tile per compute unit: a second group of waves takes every other channel chunk (twice the loads in flight).
    static const bool ksplit_ok = [] { const char* e = getenv("HIPCX_CONV_KSPLIT"); return e == nullptr || e[0] != '0'; }();
    const int64_t tiles = ((N * P + 64 * pl.wpx - 1) / (64 * pl.wpx)) * ((K + bn - 1) / bn);
    const int64_t nchunks = C / pl.ck;
    const bool ksplit_built = (pl.taps == 9 && pl.wpx == 4) || (pl.taps == 1 && pl.wpx * pl.wch <= 4 && pl.wch > 1);
    if (ksplit_ok && ksplit_built && tiles <= NumCUs() && nchunks >= 4 && nchunks % 2 == 0 && 4 * stage_bytes + pl.npx * 16 <= 160 * 1024) {
        pl.ksplit = 2;
    }
    pl.lds_bytes = pl.ksplit * 2 * stage_bytes + pl.npx * 16;
    pl.lds_bytes = std::max(pl.lds_bytes, bn * (64 * pl.wpx * 2 + 16));  // the epilogue's [channel][pixel] staging tile
    if (pl.ksplit > 1) pl.lds_bytes = std::max(pl.lds_bytes, 64 * pl.wpx * pl.wch * 64 * 4);  // the second group's accumulators
    if (pl.lds_bytes > 160 * 1024) return pl;
    pl.wp_bytes = RoundUpTo(static_cast<size_t>(K) * C * R * S * 2, 256);
    pl.ok = true;
    return pl;
}

// How many workgroups of `kernel` the device holds at once (for the launch shape given); asked once per kernel instantiation (the
// Tag type), device and LDS size, from any thread.
template <typename Tag>
int ResidentWorkgroups(const void* kernel, int block_threads, int lds_bytes) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static int resident[kMaxDevices] = {};
    static int asked_lds[kMaxDevices] = {};
    int dev = 0;
    HIPCX_CHECK_HIP(hipGetDevice(&dev));
    HIPCX_REQUIRE(dev >= 0 && dev < kMaxDevices, HIPCX_DEVICE_ERROR, "device index out of range");
    std::lock_guard<std::mutex> lock(mu);
    if (resident[dev] == 0 || asked_lds[dev] != lds_bytes) {
        int per_cu = 0;
        HIPCX_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block_threads, static_cast<size_t>(lds_bytes)));
        resident[dev] = std::max(1, per_cu) * NumCUs();
        asked_lds[dev] = lds_bytes;
    }
    return resident[dev];
}

template <int TAPS, int WPX, int WCH, int CK, int NPX, int MAXI, int KSPLIT = 1, bool PAIR = false>
void LaunchNchwKernel(const NchwConvArgs& a, int lds_bytes, hipStream_t stream) {
    auto kern = NchwConvKernel<TAPS, WPX, WCH, CK, NPX, MAXI, KSPLIT, PAIR>;
    struct Tag {};  // a type of its own for every instantiation of this launcher
    EnsureDynamicLds<Tag>(reinterpret_cast<const void*>(kern), lds_bytes);
    int64_t total = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
    dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8)), block(64 * WPX * WCH * KSPLIT);
    if constexpr (NchwWalksTiles(TAPS, WPX * WCH, NPX, KSPLIT)) {
        // these kernels walk tiles: no more workgroups than the chip holds at once (a multiple of 8, one share per XCD)
        static const bool walk = [] { const char* e = getenv("HIPCX_CONV_WALK"); return e == nullptr || e[0] != '0'; }();
        if (walk) {
            const int resident = ResidentWorkgroups<Tag>(reinterpret_cast<const void*>(kern), static_cast<int>(block.x), lds_bytes);
            grid.x = std::min(grid.x, static_cast<unsigned>(std::max(8, resident / 8 * 8)));
        }
    }
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, a);
    CheckLaunch("nchw_conv");
}

// Fused tail of hipcx_conv_bn_act as the kernel wants it.
struct FusedTail {
    const half_t* gamma = nullptr;
    const half_t* beta = nullptr;
    const half_t* mean = nullptr;
    const half_t* var = nullptr;
    int64_t stride = 0;
    float eps = 0.f;
    const half_t* residual = nullptr;
    int relu = 0;
};

void RunNchw(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const NchwPlan& pl, const int64_t* stride,
             const hipcx_array* out, char* workspace, hipStream_t stream, const FusedTail& tail = FusedTail{}) {
    NchwConvArgs a{};
    a.bn_gamma = tail.gamma;
    a.bn_beta = tail.beta;
    a.bn_mean = tail.mean;
    a.bn_var = tail.var;
    a.bn_stride = tail.stride;
    a.bn_eps = tail.eps;
    a.residual = tail.residual;
    a.relu = tail.relu;
    a.x = static_cast<const half_t*>(x->data);
    a.wp = reinterpret_cast<const half_t*>(workspace);
    a.bias = b ? static_cast<const half_t*>(b->data) : nullptr;
    a.bias_stride = b ? b->strides[0] / 2 : 0;
    a.out = static_cast<half_t*>(out->data);
    a.N = static_cast<int>(x->shape[0]);
    a.C = static_cast<int>(x->shape[1]);
    a.H = static_cast<int>(x->shape[2]);
    a.W = static_cast<int>(x->shape[3]);
    a.K = static_cast<int>(w->shape[0]);
    a.OH = static_cast<int>(out->shape[2]);
    a.OW = static_cast<int>(out->shape[3]);
    a.stride = static_cast<int>(stride[0]);
    a.P = a.OH * a.OW;
    a.M = a.N * a.P;
    const int BM = 64 * pl.wpx, BN = 64 * pl.wch;
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.K + BN - 1) / BN;
    a.nrow = pl.nrow;
    a.nslot = pl.nslot;
    a.x_bytes = static_cast<unsigned>(static_cast<int64_t>(a.N) * a.C * a.H * a.W * 2);
    const int RS = static_cast<int>(w->shape[2] * w->shape[3]);
    a.wp_bytes = static_cast<unsigned>(static_cast<int64_t>(a.K) * a.C * RS * 2);
    a.div_P = FastDiv(a.P);
    a.div_W = FastDiv(a.W);
    a.div_OW = FastDiv(a.OW);
    a.div_H2 = FastDiv(a.H + 2);
    if (pl.taps == 9) {
        a.div_wchunks = FastDiv(a.W / pl.npx);
        a.div_percg = FastDiv(pl.nrow * (a.W / pl.npx));
    }
    // single-pixel loads of a stride-2 layer over an even width fetch whole dwords (the wanted pixel and its odd neighbour)
    const bool pair_load = pl.taps == 1 && pl.npx == 1 && a.stride == 2 && a.W % 2 == 0;
    a.out_ev = a.P % 8 == 0 ? 8 : a.P % 4 == 0 ? 4 : a.P % 2 == 0 ? 2 : 1;
    const bool w_dense = w->strides[1] == 2 && w->strides[0] == static_cast<int64_t>(a.C) * 2 && reinterpret_cast<uintptr_t>(w->data) % 16 == 0;
    static const bool direct_ok = [] { const char* e = getenv("HIPCX_W_DIRECT"); return e == nullptr || e[0] != '0'; }();
    // in-place rows are read in 64-byte pieces a whole row apart; beyond 1024 input channels the packed copy is cheaper
    if (RS == 1 && w_dense && direct_ok && a.C <= 1024) {
        a.w_direct = 1;
        a.wp = static_cast<const half_t*>(w->data);
    } else {
        int64_t groups = static_cast<int64_t>(a.C / 8) * RS * a.K;
        hipLaunchKernelGGL(NchwRepackFiltersKernel, dim3(static_cast<unsigned>((groups + 255) / 256)), dim3(256), 0, stream,
                           static_cast<const half_t*>(w->data), reinterpret_cast<half_t*>(workspace), a.K, a.C, RS,
                           static_cast<int>(w->shape[3]), w->strides[0] / 2, w->strides[1] / 2, w->strides[2] / 2, w->strides[3] / 2);
        CheckLaunch("nchw_repack_filters");
    }
    double flops = 2.0 * a.M * a.K * RS * a.C;
    double bytes = 2.0 * (static_cast<double>(a.N) * a.C * a.H * a.W + static_cast<double>(a.K) * RS * a.C + static_cast<double>(a.M) * a.K);
    ProfileScope prof(stream, flops, bytes);
    const int key = (pl.ksplit - 1) * 1000000 + (pl.ck / 16) * 100000 + pl.taps * 10000 + pl.wpx * 1000 + pl.wch * 100 + pl.npx * 10 + pl.maxi;
    // single-pixel 1x1 kernels exist with and without dword loads
#define HIPCX_NCHW_LAUNCH(TAPS, WPX, WCH, CK, NPX, MAXI, KSPLIT)                                          \
    if constexpr (TAPS == 1 && NPX == 1) {                                                                \
        if (pair_load) LaunchNchwKernel<TAPS, WPX, WCH, CK, NPX, MAXI, KSPLIT, true>(a, pl.lds_bytes, stream); \
        else LaunchNchwKernel<TAPS, WPX, WCH, CK, NPX, MAXI, KSPLIT, false>(a, pl.lds_bytes, stream);     \
    } else {                                                                                              \
        LaunchNchwKernel<TAPS, WPX, WCH, CK, NPX, MAXI, KSPLIT>(a, pl.lds_bytes, stream);                 \
    }
#define HIPCX_NCHW_CASE(TAPS, WPX, WCH, CK, NPX, MAXI) \
    case (CK / 16) * 100000 + TAPS * 10000 + WPX * 1000 + WCH * 100 + NPX * 10 + MAXI: { HIPCX_NCHW_LAUNCH(TAPS, WPX, WCH, CK, NPX, MAXI, 1) } break;
    switch (key) {
        HIPCX_NCHW_CASE(1, 4, 1, 32, 2, 2)
        HIPCX_NCHW_CASE(1, 4, 1, 32, 1, 4)
        HIPCX_NCHW_CASE(1, 2, 2, 32, 2, 1)
        HIPCX_NCHW_CASE(1, 2, 2, 32, 1, 2)
        HIPCX_NCHW_CASE(1, 2, 4, 32, 1, 1)
        HIPCX_NCHW_CASE(1, 1, 4, 32, 1, 1)
        HIPCX_NCHW_CASE(9, 4, 1, 16, 2, 2)
        HIPCX_NCHW_CASE(9, 4, 1, 16, 2, 4)
        HIPCX_NCHW_CASE(9, 4, 1, 16, 1, 2)
        HIPCX_NCHW_CASE(9, 4, 1, 16, 1, 4)
#define HIPCX_NCHW_SPLIT_CASE(TAPS, WPX, WCH, CK, NPX, MAXI) \
    case 1000000 + (CK / 16) * 100000 + TAPS * 10000 + WPX * 1000 + WCH * 100 + NPX * 10 + MAXI: { HIPCX_NCHW_LAUNCH(TAPS, WPX, WCH, CK, NPX, MAXI, 2) } break;
        HIPCX_NCHW_SPLIT_CASE(1, 2, 2, 32, 2, 1)
        HIPCX_NCHW_SPLIT_CASE(1, 2, 2, 32, 1, 2)
        HIPCX_NCHW_SPLIT_CASE(1, 1, 4, 32, 1, 1)
        HIPCX_NCHW_SPLIT_CASE(9, 4, 1, 16, 2, 2)
        HIPCX_NCHW_SPLIT_CASE(9, 4, 1, 16, 2, 4)
        HIPCX_NCHW_SPLIT_CASE(9, 4, 1, 16, 1, 2)
        HIPCX_NCHW_SPLIT_CASE(9, 4, 1, 16, 1, 4)
#undef HIPCX_NCHW_SPLIT_CASE
        default: throw Error(HIPCX_CHAINERX_ERROR, "nchw conv: no kernel for plan " + std::to_string(key));
    }
#undef HIPCX_NCHW_CASE
#undef HIPCX_NCHW_LAUNCH
}


// ---- float16 1x1 / stride 1 layers on the LDS-direct ring (pw_conv.h) ----
struct PwPlan {
    bool ok = false;
    int wm = 2, wn = 2;  // wave grid of the workgroup: 256 pixels x 128 channels
};

PwPlan PlanPw(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const hipcx_array* out, const int64_t* stride, const int64_t* pad) {
    PwPlan pl;
    static const bool enabled = [] { const char* e = getenv("HIPCX_CONV_PW"); return e == nullptr || e[0] != '0'; }();
    if (!enabled || x->dtype != HIPCX_FLOAT16 || !IsContiguous(x) || !IsContiguous(out)) return pl;
    const int64_t N = x->shape[0], C = x->shape[1], P = x->shape[2] * x->shape[3], K = w->shape[0];
    if (w->shape[2] != 1 || w->shape[3] != 1 || stride[0] != 1 || stride[1] != 1 || pad[0] != 0 || pad[1] != 0) return pl;
    if (C % 32 != 0 || P % 4 != 0 || K > kPwMaxBiasK) return pl;
    if (w->strides[1] != 2 || w->strides[0] != C * 2 || reinterpret_cast<uintptr_t>(w->data) % 16 != 0) return pl;  // dense [K][C] rows
    if (reinterpret_cast<uintptr_t>(x->data) % 16 != 0 || reinterpret_cast<uintptr_t>(out->data) % 16 != 0) return pl;
    if (b != nullptr && b->strides[0] % 2 != 0) return pl;
    if (N * C * P * 2 >= (1LL << 31) || N * K * P * 2 >= (1LL << 31) || K * C * 2 >= (1LL << 31)) return pl;
    const int64_t PS = (P + 7) / 8 * 8;
    // Where these kernels measured faster than the 128 x 128 tiles on ResNet-50's layers at batch 128 (microseconds, the 128 x 128
    // kernels first): 256 -> 1024 at 14x14 29.6 / 26.0, 128 -> 512 at 28x28 33.5 / 26.8, 512 -> 128 at 28x28 29.8 / 22.4,
    // 64 -> 256 at 56x56 45.3 / 40.6, 512 -> 2048 at 7x7 29.9 / 25.1 -- all with four-wave workgroups on 256-pixel x 128-channel
    // tiles, two to a compute unit, which overlap each other's load, multiply and store phases.  Deep reductions into few
    // channels (1024 -> 256: 26.5 either way; 2048 -> 512 and 256 -> 64: slower) stay with the 128 x 128 tiles and their split
    // reduction.  The eight-wave variants (one workgroup per unit, 256 x 256 or 512 x 128 tiles) measured between the two.
    if (!((K >= 256 && C <= 512) || (K > 64 && K <= 128))) return pl;
    pl.wm = 2, pl.wn = 2;
    const int64_t tiles = ((N * PS + 128 * pl.wm - 1) / (128 * pl.wm)) * ((K + 64 * pl.wn - 1) / (64 * pl.wn));
    const int64_t slots = pl.wm * pl.wn == 4 ? 2 * NumCUs() : NumCUs();  // workgroups resident at a time
    if (tiles < (slots * 3) / 4 || tiles >= (1LL << 24)) return pl;
    pl.ok = true;
    return pl;
}

template <int WM, int WN>
void LaunchPw(PwConvArgs a, hipStream_t stream) {
    constexpr int BM = 128 * WM, BN = 64 * WN;
    a.tiles_m = (a.MS + BM - 1) / BM;
    a.tiles_n = (a.K + BN - 1) / BN;
    a.total_tiles = a.tiles_m * a.tiles_n;
    constexpr int lds_bytes = PwLdsBytes<WM, WN>();
    constexpr int kPerUnit = WM * WN == 4 ? 2 : 1;  // four-wave workgroups run two to a compute unit
    // workgroups walk tiles: as many as the device holds at a time (a multiple of 8, one share per XCD)
    const unsigned grid = static_cast<unsigned>(std::min((a.total_tiles + 7) / 8 * 8, std::max(8, kPerUnit * NumCUs() / 8 * 8)));
    if (a.P % 8 != 0) {
        auto kern = PwConvKernel<WM, WN, true>;
        struct Tag {};
        EnsureDynamicLds<Tag>(reinterpret_cast<const void*>(kern), lds_bytes);
        hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WM * WN), lds_bytes, stream, a);
    } else {
        auto kern = PwConvKernel<WM, WN, false>;
        struct Tag {};
        EnsureDynamicLds<Tag>(reinterpret_cast<const void*>(kern), lds_bytes);
        hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WM * WN), lds_bytes, stream, a);
    }
    CheckLaunch("pw_conv");
}

void RunPw(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const PwPlan& pl, const hipcx_array* out, hipStream_t stream) {
    PwConvArgs a{};
    a.x = static_cast<const half_t*>(x->data);
    a.w = static_cast<const half_t*>(w->data);
    a.bias = b ? static_cast<const half_t*>(b->data) : nullptr;
    a.bias_stride = b ? b->strides[0] / 2 : 0;
    a.out = static_cast<half_t*>(out->data);
    a.N = static_cast<int>(x->shape[0]);
    a.C = static_cast<int>(x->shape[1]);
    a.K = static_cast<int>(w->shape[0]);
    a.P = static_cast<int>(x->shape[2] * x->shape[3]);
    a.PS = (a.P + 7) / 8 * 8;
    a.MS = a.N * a.PS;
    a.div_PS = FastDiv(a.PS);
    a.x_bytes = static_cast<unsigned>(static_cast<int64_t>(a.N) * a.C * a.P * 2);
    a.w_bytes = static_cast<unsigned>(static_cast<int64_t>(a.K) * a.C * 2);
    a.out_bytes = static_cast<unsigned>(static_cast<int64_t>(a.N) * a.K * a.P * 2);
    const double M = static_cast<double>(a.N) * a.P;
    ProfileScope prof(stream, 2.0 * M * a.K * a.C, 2.0 * (M * a.C + static_cast<double>(a.K) * a.C + M * a.K));
    LaunchPw<2, 2>(a, stream);
}

// ---- float16 7x7/2 stem path (stem_conv.h) ----
struct StemPlan {
    bool ok = false;
    int rowp = 0, copyb = 0, lds_bytes = 0, ksteps = 0;
    size_t wp_bytes = 0;
};

StemPlan PlanStem(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out, const int64_t* stride, const int64_t* pad) {
    StemPlan pl;
    static const bool enabled = [] { const char* e = getenv("HIPCX_CONV_STEM"); return e == nullptr || e[0] != '0'; }();
    if (!enabled || x->dtype != HIPCX_FLOAT16 || !IsContiguous(x) || !IsContiguous(out)) return pl;
    const int64_t N = x->shape[0], C = x->shape[1], H = x->shape[2], W = x->shape[3];
    const int64_t K = w->shape[0], OH = out->shape[2], OW = out->shape[3];
    if (C != 3 || K != 64 || w->shape[2] != 7 || w->shape[3] != 7) return pl;
    if (stride[0] != 2 || stride[1] != 2 || pad[0] != 3 || pad[1] != 3) return pl;
    if (W % 8 != 0 || OW * 2 != W || OW % 8 != 0 || 2 * OW > 256 || OH != (H - 1) / 2 + 1) return pl;
    if (N * C * H * W * 2 >= (1LL << 31) || N * K * OH * OW * 2 >= (1LL << 31)) return pl;
    if (reinterpret_cast<uintptr_t>(x->data) % 16 != 0 || reinterpret_cast<uintptr_t>(out->data) % 16 != 0) return pl;
    pl.ksteps = static_cast<int>((C * 7 + 1) / 2);
    pl.rowp = static_cast<int>(W / 8 * 16);
    int need = static_cast<int>(C * 9 + 3) * pl.rowp;
    pl.copyb = need + ((64 - need % 256) + 256) % 256;  // copies 64 bytes apart modulo 256: neighbouring lanes hit different banks
    pl.lds_bytes = std::max(4 * pl.copyb, 64 * (static_cast<int>(OW) * 4 + 16));
    if (pl.lds_bytes > 160 * 1024) return pl;
    pl.wp_bytes = static_cast<size_t>(pl.ksteps) * 2 * 64 * 16;
    pl.ok = true;
    return pl;
}

void RunStem(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const StemPlan& pl, const hipcx_array* out, char* workspace,
             hipStream_t stream, const FusedTail& tail = FusedTail{}) {
    StemConvArgs a{};
    a.x = static_cast<const half_t*>(x->data);
    a.wp = reinterpret_cast<const half_t*>(workspace);
    a.bias = b ? static_cast<const half_t*>(b->data) : nullptr;
    a.bias_stride = b ? b->strides[0] / 2 : 0;
    a.out = static_cast<half_t*>(out->data);
    a.N = static_cast<int>(x->shape[0]);
    a.H = static_cast<int>(x->shape[2]);
    a.W = static_cast<int>(x->shape[3]);
    a.OH = static_cast<int>(out->shape[2]);
    a.OW = static_cast<int>(out->shape[3]);
    a.x_bytes = static_cast<unsigned>(static_cast<int64_t>(a.N) * 3 * a.H * a.W * 2);
    a.wp_bytes = static_cast<unsigned>(pl.wp_bytes);
    a.rowp = pl.rowp;
    a.copyb = pl.copyb;
    a.bn_gamma = tail.gamma;
    a.bn_beta = tail.beta;
    a.bn_mean = tail.mean;
    a.bn_var = tail.var;
    a.bn_stride = tail.stride;
    a.bn_eps = tail.eps;
    a.relu = tail.relu;
    int groups = pl.ksteps * 2 * 64;
    hipLaunchKernelGGL(StemRepackFiltersKernel, dim3((groups + 255) / 256), dim3(256), 0, stream, static_cast<const half_t*>(w->data),
                       reinterpret_cast<half_t*>(workspace), 3, pl.ksteps, w->strides[0] / 2, w->strides[1] / 2, w->strides[2] / 2,
                       w->strides[3] / 2);
    CheckLaunch("stem_repack_filters");
    const double M = static_cast<double>(a.N) * a.OH * a.OW;
    ProfileScope prof(stream, 2.0 * M * 64 * 3 * 49,
                      2.0 * (static_cast<double>(a.N) * 3 * a.H * a.W + 64.0 * 3 * 49 + M * 64));
    auto kern = StemConv7x7s2Kernel<3>;
    struct StemTag {};
    EnsureDynamicLds<StemTag>(reinterpret_cast<const void*>(kern), pl.lds_bytes);
    // workgroups walk tiles (two output rows of one image each): as many as the device holds at a time, two per compute unit
    static const int per_unit = [] { const char* e = getenv("HIPCX_STEM_PER_UNIT"); return e != nullptr && atoi(e) > 0 ? atoi(e) : 2; }();
    const int blocks = std::min(a.N * ((a.OH + 1) / 2), per_unit * NumCUs());
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), pl.lds_bytes, stream, a);
    CheckLaunch("stem_conv");
}

// How a convolution is staged.  The MFMA kernel wants the reduction axis (r, s, c) contiguous in
// both operands, i.e. channels-last activations and [K][R][S][C] filters.  Activations that are not
// channels-last (the C-contiguous NCHW arrays ChainerX routines allocate) are gathered into a
// channels-last staging buffer first; a strided 1x1 convolution gathers only the pixels it reads
// and then runs with stride 1; the channel axis is zero-padded to a 16-byte multiple so that
// e.g. a 3-channel image still takes the vector path.
struct ConvPlan {
    bool stage_x = false;   // gather x into the workspace
    bool repack_w = false;  // repack filters into the workspace
    int Cpad = 0;
    int Hs = 0, Ws = 0;     // staged plane extents
    int step_h = 1, step_w = 1;
    int conv_stride_h = 1, conv_stride_w = 1, conv_pad_h = 0, conv_pad_w = 0;  // geometry the MFMA kernel runs with
    size_t x_bytes = 0, w_bytes = 0;
};

size_t RoundUp(size_t v, size_t a) { return (v + a - 1) / a * a; }

ConvPlan PlanConv(const hipcx_array* x, const hipcx_array* w, const int64_t* stride, const int64_t* pad) {
    ConvPlan pl;
    const int64_t it = ItemSize(x->dtype);
    const int64_t C = x->shape[1], H = x->shape[2], W = x->shape[3];
    const int64_t K = w->shape[0], R = w->shape[2], S = w->shape[3];
    pl.conv_stride_h = static_cast<int>(stride[0]);
    pl.conv_stride_w = static_cast<int>(stride[1]);
    pl.conv_pad_h = static_cast<int>(pad[0]);
    pl.conv_pad_w = static_cast<int>(pad[1]);
    pl.Cpad = static_cast<int>(C);
    pl.Hs = static_cast<int>(H);
    pl.Ws = static_cast<int>(W);
    if (x->dtype == HIPCX_FLOAT64) return pl;  // scalar kernel, any layout
    const int64_t epv = 16 / it;
    bool x_cl = x->strides[1] == it && C % epv == 0 && reinterpret_cast<uintptr_t>(x->data) % 16 == 0 && x->strides[0] % 16 == 0 &&
                x->strides[2] % 16 == 0 && x->strides[3] % 16 == 0;
    if (!x_cl) {
        pl.stage_x = true;
        pl.Cpad = static_cast<int>((C + epv - 1) / epv * epv);
        if (R == 1 && S == 1 && pad[0] == 0 && pad[1] == 0 && (stride[0] > 1 || stride[1] > 1)) {
            pl.step_h = static_cast<int>(stride[0]);
            pl.step_w = static_cast<int>(stride[1]);
            pl.Hs = static_cast<int>((H - 1) / stride[0] + 1);
            pl.Ws = static_cast<int>((W - 1) / stride[1] + 1);
            pl.conv_stride_h = pl.conv_stride_w = 1;
        }
        pl.x_bytes = RoundUp(static_cast<size_t>(x->shape[0]) * pl.Hs * pl.Ws * pl.Cpad * it, 256);
    }
    bool w_dense = w->strides[1] == it && w->strides[3] == C * it && w->strides[2] == S * C * it && w->strides[0] % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(w->data) % 16 == 0;
    if (R == 1 && S == 1) w_dense = w->strides[1] == it && w->strides[0] % 16 == 0 && reinterpret_cast<uintptr_t>(w->data) % 16 == 0;
    if (pl.Cpad != C || !w_dense) {
        pl.repack_w = true;
        pl.w_bytes = RoundUp(static_cast<size_t>(K) * R * S * pl.Cpad * it, 256);
    }
    return pl;
}

// Repacks w[K,C,R,S] (any strides) into dense [K][R][S][Cpad] (zero-filled padding) with strided Copy launches.
void RepackFilters(const hipcx_array* w, int Cpad, void* dst, hipStream_t stream) {
    int64_t it = ItemSize(w->dtype);
    int64_t K = w->shape[0], C = w->shape[1], R = w->shape[2], S = w->shape[3];
    if (Cpad != C) {
        hipcx_array flat{};
        flat.data = dst;
        flat.dtype = w->dtype;
        flat.ndim = 1;
        flat.shape[0] = K * R * S * Cpad;
        flat.strides[0] = it;
        hipcx_scalar zero{HIPCX_KIND_INT, 0, 0, 0.0};
        int st = hipcx_fill(&flat, zero, stream);
        if (st != HIPCX_OK) throw Error(st, hipcx_last_error());
    }
    hipcx_array view = *w;
    view.data = dst;
    view.strides[0] = R * S * Cpad * it;
    view.strides[1] = it;
    view.strides[2] = S * Cpad * it;
    view.strides[3] = Cpad * it;
    int st = hipcx_copy(w, &view, stream);
    if (st != HIPCX_OK) throw Error(st, hipcx_last_error());
}

template <typename T>
void RunConv(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const ConvPlan& pl, const hipcx_array* out,
             char* workspace, hipStream_t stream) {
    IGemmArgs<T> p{};
    const int64_t it = sizeof(T);
    p.N = static_cast<int>(x->shape[0]);
    p.C_logical = static_cast<int>(x->shape[1]);
    p.H_logical = static_cast<int>(x->shape[2]);
    p.W_logical = static_cast<int>(x->shape[3]);
    p.C = pl.Cpad;
    p.H = pl.Hs;
    p.W = pl.Ws;
    p.K = static_cast<int>(w->shape[0]);
    p.R = static_cast<int>(w->shape[2]);
    p.S = static_cast<int>(w->shape[3]);
    p.OH = static_cast<int>(out->shape[2]);
    p.OW = static_cast<int>(out->shape[3]);
    p.stride_h = pl.conv_stride_h;
    p.stride_w = pl.conv_stride_w;
    p.pad_h = pl.conv_pad_h;
    p.pad_w = pl.conv_pad_w;
    char* ws = workspace;
    if (pl.stage_x) {
        ToChannelsLastArgs a{};
        a.x = x->data;
        a.out = ws;
        a.N = p.N;
        a.C = p.C_logical;
        a.Cpad = pl.Cpad;
        a.Ho = pl.Hs;
        a.Wo = pl.Ws;
        a.step_h = pl.step_h;
        a.step_w = pl.step_w;
        a.xsN = ElemStride(x, 0, "x");
        a.xsC = ElemStride(x, 1, "x");
        a.xsH = ElemStride(x, 2, "x");
        a.xsW = ElemStride(x, 3, "x");
        int64_t plane = static_cast<int64_t>(pl.Hs) * pl.Ws;
        a.vec_in = (pl.step_h == 1 && pl.step_w == 1 && a.xsW == 1 && a.xsH == pl.Ws && plane % (16 / it) == 0 &&
                    reinterpret_cast<uintptr_t>(x->data) % 16 == 0 && a.xsC % (16 / it) == 0 && a.xsN % (16 / it) == 0) ? 1 : 0;
        LaunchToChannelsLast<T>(a, stream);
        p.x = reinterpret_cast<const T*>(ws);
        p.xsC = 1;
        p.xsW = pl.Cpad;
        p.xsH = static_cast<int64_t>(pl.Ws) * pl.Cpad;
        p.xsN = static_cast<int64_t>(pl.Hs) * pl.Ws * pl.Cpad;
        ws += pl.x_bytes;
    } else {
        p.x = static_cast<const T*>(x->data);
        p.xsN = ElemStride(x, 0, "x");
        p.xsC = ElemStride(x, 1, "x");
        p.xsH = ElemStride(x, 2, "x");
        p.xsW = ElemStride(x, 3, "x");
    }
    if (pl.repack_w) {
        RepackFilters(w, pl.Cpad, ws, stream);
        p.w = reinterpret_cast<const T*>(ws);
        p.wsK = static_cast<int64_t>(p.R) * p.S * p.C;
        p.wsC = 1;
        p.wsR = static_cast<int64_t>(p.S) * p.C;
        p.wsS = p.C;
    } else {
        p.w = static_cast<const T*>(w->data);
        p.wsK = ElemStride(w, 0, "w");
        p.wsC = ElemStride(w, 1, "w");
        p.wsR = ElemStride(w, 2, "w");
        p.wsS = ElemStride(w, 3, "w");
        if (p.R == 1 && p.S == 1) {  // unit axes: any stride describes them; use the dense ones
            p.wsR = static_cast<int64_t>(p.S) * p.C;
            p.wsS = p.C;
        }
    }
    p.bias = b ? static_cast<const T*>(b->data) : nullptr;
    p.bias_stride = b ? ElemStride(b, 0, "b") : 0;
    p.out = static_cast<T*>(out->data);
    p.osN = ElemStride(out, 0, "out");
    p.osC = ElemStride(out, 1, "out");
    p.osH = ElemStride(out, 2, "out");
    p.osW = ElemStride(out, 3, "out");
    p.M = static_cast<int64_t>(p.N) * p.OH * p.OW;
    p.Kg = p.R * p.S * p.C;
    if constexpr (std::is_same<T, double>::value) {
        LaunchF64(p, stream);
    } else {
        LaunchIGemmImpl(p, stream);
    }
}

void CheckConv(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
               int cover_all, const hipcx_array* out) {
    ValidateArray(x, "x");
    ValidateArray(w, "w");
    ValidateArray(out, "out");
    HIPCX_REQUIRE(x->ndim == 4 && w->ndim == 4 && out->ndim == 4, HIPCX_NOT_IMPLEMENTED_ERROR,
                  "hip conv supports 2 spatial dimensions (4-dimensional x, w, out)");
    HIPCX_REQUIRE(IsFloatDtype(out->dtype), HIPCX_DTYPE_ERROR, "hip conv supports floating point dtypes only");
    HIPCX_REQUIRE(x->dtype == out->dtype && w->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                  "x and w must have out's dtype (cast with hipcx_copy first)");
    HIPCX_REQUIRE(w->shape[1] == x->shape[1], HIPCX_DIMENSION_ERROR, "Mismatched number of input channels in input and weights.");
    HIPCX_REQUIRE(stride && pad && stride[0] > 0 && stride[1] > 0 && pad[0] >= 0 && pad[1] >= 0, HIPCX_DIMENSION_ERROR,
                  "invalid stride or pad");
    if (b != nullptr) {
        ValidateArray(b, "b");
        HIPCX_REQUIRE(b->ndim == 1 && b->shape[0] == w->shape[0], HIPCX_DIMENSION_ERROR, "Mismatched bias shape for weights.");
        HIPCX_REQUIRE(b->dtype == out->dtype, HIPCX_DTYPE_ERROR, "b must have out's dtype");
    }
    int64_t oh = hipcx_conv_out_dim(x->shape[2], w->shape[2], stride[0], pad[0], cover_all);
    int64_t ow = hipcx_conv_out_dim(x->shape[3], w->shape[3], stride[1], pad[1], cover_all);
    HIPCX_REQUIRE(oh > 0 && ow > 0, HIPCX_DIMENSION_ERROR, "Output size should be positive.");
    HIPCX_REQUIRE(out->shape[0] == x->shape[0] && out->shape[1] == w->shape[0] && out->shape[2] == oh && out->shape[3] == ow,
                  HIPCX_DIMENSION_ERROR, "out has the wrong shape " + ShapeStr(out));
    for (int i = 0; i < 4; ++i) {
        HIPCX_REQUIRE(x->shape[i] < (1LL << 31) && w->shape[i] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
    }
    HIPCX_REQUIRE(w->shape[1] * w->shape[2] * w->shape[3] < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "reduction too long");
}

}  // namespace
}  // namespace hipcx

namespace hipcx {
// int_dot.hip: Dot for the integer dtypes and bool
void IntDot(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, hipStream_t stream);
// nd_ops.hip: arrays without exactly two spatial axes, and the integer dtypes
size_t ConvNdWorkspaceSize(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out);
void ConvNd(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad, int cover_all,
            const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream);
}  // namespace hipcx

using namespace hipcx;

extern "C" {

int hipcx_profile_start(void) {
    return Guard([&] {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        HIPCX_REQUIRE(!g_profile.on, HIPCX_CHAINERX_ERROR, "profiling is already on");
        g_profile = ProfileState{};
        g_profile.on = true;
    });
}

int hipcx_profile_stop(int64_t* launches, double* total_ms, double* flops, double* bytes) {
    return Guard([&] {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        HIPCX_REQUIRE(g_profile.on, HIPCX_CHAINERX_ERROR, "profiling is not on");
        g_profile.on = false;
        double ms = 0.0;
        for (size_t i = 0; i < g_profile.events.size(); ++i) {
            auto& ev = g_profile.events[i];
            HIPCX_CHECK_HIP(hipEventSynchronize(ev.second));
            float t = 0.f;
            HIPCX_CHECK_HIP(hipEventElapsedTime(&t, ev.first, ev.second));
            ms += t;
            g_profile.records[i].ms = t;
            (void)hipEventDestroy(ev.first);
            (void)hipEventDestroy(ev.second);
        }
        if (launches) *launches = static_cast<int64_t>(g_profile.events.size());
        if (total_ms) *total_ms = ms;
        if (flops) *flops = g_profile.flops;
        if (bytes) *bytes = g_profile.bytes;
        g_profile.events.clear();
    });
}

int hipcx_profile_records(int64_t capacity, double* ms, double* flops, double* bytes, int64_t* count) {
    return Guard([&] {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        HIPCX_REQUIRE(!g_profile.on, HIPCX_CHAINERX_ERROR, "profiling is still on: call hipcx_profile_stop first");
        const int64_t n = static_cast<int64_t>(g_profile.records.size());
        if (count) *count = n;
        for (int64_t i = 0; i < n && i < capacity; ++i) {
            if (ms) ms[i] = g_profile.records[i].ms;
            if (flops) flops[i] = g_profile.records[i].flops;
            if (bytes) bytes[i] = g_profile.records[i].bytes;
        }
    });
}

size_t hipcx_conv_workspace_size(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out) {
    if (x == nullptr || w == nullptr) return 0;
    if (!IsFloatDtype(x->dtype)) return 0;
    if (x->ndim != 4 || w->ndim != 4) {
        try {
            return x->ndim >= 2 ? ConvNdWorkspaceSize(x, w, out) : 0;
        } catch (...) {
            return 0;
        }
    }
    try {
        // the staging decision does not depend on stride/pad except for the sub-sampled 1x1 case, which needs less;
        // report the full-plane size
        int64_t one[2] = {1, 1}, zero[2] = {0, 0};
        ConvPlan pl = PlanConv(x, w, one, zero);
        size_t need = pl.x_bytes + pl.w_bytes;
        // the NCHW-native float16 path needs room for the packed filters only; report the larger of the two
        if (x->dtype == HIPCX_FLOAT16) need = std::max(need, RoundUpTo(static_cast<size_t>(TotalSize(w)) * 2, 256) + 8192);  // packed filters, padded taps
        return need;
    } catch (...) {
        return 0;
    }
}

int hipcx_conv_route(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                     const hipcx_array* out) {
    try {
        if (x == nullptr || w == nullptr || out == nullptr || stride == nullptr || pad == nullptr) return -1;
        if (x->ndim != 4 || w->ndim != 4 || out->ndim != 4) return -1;
        if (PlanPw(x, w, b, out, stride, pad).ok) return 3;
        if (PlanNchw(x, w, out, stride, pad).ok) return 1;
        if (PlanStem(x, w, out, stride, pad).ok) return 2;
        return 0;
    } catch (...) {
        return -1;
    }
}

int hipcx_conv(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
               int cover_all, const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        if (x != nullptr && out != nullptr && (x->ndim != 4 || !IsFloatDtype(out->dtype))) {  // not two spatial axes, or integers: nd_ops.hip
            ConvNd(x, w, b, stride, pad, cover_all, out, workspace, workspace_bytes, stream);
            return;
        }
        CheckConv(x, w, b, stride, pad, cover_all, out);
        if (TotalSize(out) == 0) return;
        hipStream_t st = AsStream(stream);
        PwPlan ppl = PlanPw(x, w, b, out, stride, pad);
        if (ppl.ok) {
            RunPw(x, w, b, ppl, out, st);
            return;
        }
        NchwPlan npl = PlanNchw(x, w, out, stride, pad);
        if (npl.ok) {
            HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= npl.wp_bytes, HIPCX_CHAINERX_ERROR,
                          "conv workspace too small: need " + std::to_string(npl.wp_bytes) + " bytes");
            HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
            RunNchw(x, w, b, npl, stride, out, static_cast<char*>(workspace), st);
            return;
        }
        StemPlan spl = PlanStem(x, w, out, stride, pad);
        if (spl.ok && workspace != nullptr && workspace_bytes >= spl.wp_bytes && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
            RunStem(x, w, b, spl, out, static_cast<char*>(workspace), st);
            return;
        }
        ConvPlan pl = PlanConv(x, w, stride, pad);
        size_t need = pl.x_bytes + pl.w_bytes;
        if (need > 0) {
            HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= need, HIPCX_CHAINERX_ERROR,
                          "conv workspace too small: need " + std::to_string(need) + " bytes");
            HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
        }
        char* ws = static_cast<char*>(workspace);
        if (out->dtype == HIPCX_FLOAT16) {
            RunConv<half_t>(x, w, b, pl, out, ws, st);
        } else if (out->dtype == HIPCX_FLOAT32) {
            RunConv<float>(x, w, b, pl, out, ws, st);
        } else {
            RunConv<double>(x, w, b, pl, out, ws, st);
        }
    });
}

// Channel stride (elements) of a batch-norm parameter holding one value per output channel: a vector [K] or the
// keep-dims shape [1, K, 1, 1].  Returns false for anything else.
static bool BnParamStride(const hipcx_array* a, int64_t K, int dtype, int64_t* stride) {
    if (a == nullptr || a->dtype != dtype) return false;
    int64_t it = ItemSize(dtype);
    if (a->ndim == 1 && a->shape[0] == K && a->strides[0] % it == 0) {
        *stride = a->strides[0] / it;
        return true;
    }
    if (a->ndim == 4 && a->shape[0] == 1 && a->shape[1] == K && a->shape[2] == 1 && a->shape[3] == 1 && a->strides[1] % it == 0) {
        *stride = a->strides[1] / it;
        return true;
    }
    return false;
}

int hipcx_conv_bn_act(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                      int cover_all, const hipcx_array* gamma, const hipcx_array* beta, const hipcx_array* mean, const hipcx_array* var,
                      hipcx_scalar eps, const hipcx_array* residual, int relu, const hipcx_array* out, void* workspace,
                      size_t workspace_bytes, void* stream) {
    return Guard([&] {
        CheckConv(x, w, b, stride, pad, cover_all, out);
        const bool has_bn = gamma != nullptr || beta != nullptr || mean != nullptr || var != nullptr;
        const int64_t K = w->shape[0];
        int64_t sg = 0, sb = 0, sm = 0, sv = 0;
        if (has_bn) {
            HIPCX_REQUIRE(BnParamStride(gamma, K, out->dtype, &sg) && BnParamStride(beta, K, out->dtype, &sb) &&
                              BnParamStride(mean, K, out->dtype, &sm) && BnParamStride(var, K, out->dtype, &sv),
                          HIPCX_DIMENSION_ERROR, "batch-norm parameters must have one value of out's dtype per output channel ([K] or [1,K,1,1])");
        }
        if (residual != nullptr) {
            ValidateArray(residual, "residual");
            HIPCX_REQUIRE(SameShape(residual, out) && residual->dtype == out->dtype, HIPCX_DIMENSION_ERROR,
                          "residual must have out's shape and dtype");
        }
        if (TotalSize(out) == 0) return;
        hipStream_t st = AsStream(stream);
        NchwPlan npl = PlanNchw(x, w, out, stride, pad);
        const bool same_stride = !has_bn || (sg == sb && sg == sm && sg == sv);
        const bool res_ok = residual == nullptr || (IsContiguous(residual) && reinterpret_cast<uintptr_t>(residual->data) % 16 == 0);
        FusedTail tail;
        if (has_bn) {
            tail.gamma = static_cast<const half_t*>(gamma->data);
            tail.beta = static_cast<const half_t*>(beta->data);
            tail.mean = static_cast<const half_t*>(mean->data);
            tail.var = static_cast<const half_t*>(var->data);
            tail.stride = sg;
            tail.eps = static_cast<float>(eps.kind == HIPCX_KIND_FLOAT ? eps.f : static_cast<double>(eps.i));
        }
        tail.residual = residual ? static_cast<const half_t*>(residual->data) : nullptr;
        tail.relu = relu ? 1 : 0;
        const bool ws_aligned = reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
        if (npl.ok && same_stride && res_ok) {
            HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= npl.wp_bytes, HIPCX_CHAINERX_ERROR,
                          "conv workspace too small: need " + std::to_string(npl.wp_bytes) + " bytes");
            HIPCX_REQUIRE(ws_aligned, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
            RunNchw(x, w, b, npl, stride, out, static_cast<char*>(workspace), st, tail);
            return;
        }
        StemPlan spl = PlanStem(x, w, out, stride, pad);
        if (spl.ok && same_stride && residual == nullptr && workspace != nullptr && workspace_bytes >= spl.wp_bytes && ws_aligned) {
            RunStem(x, w, b, spl, out, static_cast<char*>(workspace), st, tail);
            return;
        }
        // Any other dtype / layout / geometry: the same result from the separate kernels, in place on `out`.
        auto check = [](int status) {
            if (status != HIPCX_OK) throw Error(status, hipcx_last_error());
        };
        check(hipcx_conv(x, w, b, stride, pad, cover_all, out, workspace, workspace_bytes, stream));
        if (has_bn) {
            auto keepdims = [&](const hipcx_array* a, int64_t stride_elems) {
                hipcx_array v{};
                v.data = a->data;
                v.dtype = a->dtype;
                v.ndim = 4;
                v.shape[0] = 1, v.shape[1] = K, v.shape[2] = 1, v.shape[3] = 1;
                v.strides[1] = stride_elems * ItemSize(a->dtype);
                return v;
            };
            hipcx_array g4 = keepdims(gamma, sg), b4 = keepdims(beta, sb), m4 = keepdims(mean, sm), v4 = keepdims(var, sv);
            const int8_t axis[3] = {0, 2, 3};
            check(hipcx_fixed_batch_norm(out, &g4, &b4, &m4, &v4, eps, axis, 3, out, stream));
        }
        if (residual != nullptr) check(hipcx_add(out, residual, out, stream));
        if (relu) {
            hipcx_scalar zero{HIPCX_KIND_INT, 0, 0, 0.0};
            check(hipcx_if_less_else_assa(out, zero, zero, out, out, stream));
        }
    });
}

}  // extern "C"

namespace {
// The MFMA kernels read both operands with the reduction index k as the unit-stride axis, rows 16-byte aligned.  An operand
// laid out otherwise (a plain row-major b, a transposed a, odd pitches) is first copied into that layout -- one pass over
// the operand instead of an element-gather kernel for the whole product.
struct DotStaging {
    bool a = false, b = false;
    int64_t kpad = 0;       // staged row pitch, elements (k rounded up to 16 bytes)
    size_t a_bytes = 0, b_bytes = 0;
};

bool OperandIsFast(const void* ptr, int64_t line_stride_bytes, int64_t k_stride_bytes, int64_t k, int64_t it) {
    // 8-byte granules are enough for the fast kernel (its 16-byte variant is picked when everything is 16-byte aligned)
    return k_stride_bytes == it && reinterpret_cast<uintptr_t>(ptr) % 8 == 0 && line_stride_bytes % 8 == 0 && line_stride_bytes >= 0 &&
           (k * it) % 8 == 0;
}

DotStaging PlanDotStaging(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out) {
    DotStaging st;
    if (a == nullptr || b == nullptr || out == nullptr || a->ndim != 2 || b->ndim != 2) return st;
    if (out->dtype != HIPCX_FLOAT16 && out->dtype != HIPCX_FLOAT32) return st;
    static const bool enabled = [] { const char* e = getenv("HIPCX_DOT_STAGE"); return e == nullptr || e[0] != '0'; }();
    const int64_t it = ItemSize(out->dtype);
    const int64_t m = a->shape[0], k = a->shape[1], n = b->shape[1];
    if (!enabled || m == 0 || n == 0 || k == 0) return st;
    const bool a_fast = OperandIsFast(a->data, a->strides[0], a->strides[1], k, it);
    const bool b_fast = OperandIsFast(b->data, b->strides[1], b->strides[0], k, it);
    if (a_fast && b_fast) return st;
    // worth it only when the product is large against the copies; small outputs have their own kernel (any layout)
    if (2.0 * m * n * k < 2e8) return st;
    if (((m + 127) / 128) * ((n + 127) / 128) < 128 && k >= 64) return st;
    const int64_t epv = 16 / it;
    st.kpad = (k + epv - 1) / epv * epv;
    // a changed pitch on one side needs the same (zero-padded) k extent on the other
    st.a = !a_fast || st.kpad != k;
    st.b = !b_fast || st.kpad != k;
    st.a_bytes = st.a ? RoundUpTo(static_cast<size_t>(m * st.kpad * it), 256) : 0;
    st.b_bytes = st.b ? RoundUpTo(static_cast<size_t>(n * st.kpad * it), 256) : 0;
    return st;
}
}  // namespace

namespace {
// Matrix products with few 128x128 output tiles and a long reduction axis (weight gradients: M x N = filters, reduction = batch x
// pixels): slices of the reduction run as separate workgroups.  Returns the number of slices (1: no split).
int PlanSplitK(int64_t m, int64_t n, int64_t k, int dtype) {
    static const bool enabled = [] { const char* e = getenv("HIPCX_DOT_SPLITK"); return e == nullptr || e[0] != '0'; }();
    if (!enabled || (dtype != HIPCX_FLOAT16 && dtype != HIPCX_FLOAT32)) return 1;
    const int64_t tiles = ((m + 127) / 128) * ((n + 127) / 128);
    const int64_t steps = k * ItemSize(dtype) / 128;  // reduction steps of 128 bytes per row
    if (k < 4096 || tiles > NumCUs() || m * n < 64 * 64 || steps < 16) return 1;  // up to one tile per compute unit: a second workgroup per unit still hides latency
    int64_t s = (2 * NumCUs() + tiles - 1) / tiles;
    static const int64_t min_steps = [] { const char* e = getenv("HIPCX_DOT_SPLITK_MINSTEPS"); int v = e ? atoi(e) : 0; return v >= 1 && v <= 4096 ? v : 8; }();
    if (s > steps / min_steps) s = steps / min_steps;  // a slice of fewer steps costs more in partial sums than it gains
    static const int64_t max_slices = [] { const char* e = getenv("HIPCX_DOT_SPLITK_MAX"); int v = e ? atoi(e) : 0; return v >= 2 && v <= 1024 ? v : 256; }();
    if (s > max_slices) s = max_slices;
    return s < 2 ? 1 : static_cast<int>(s);
}
size_t SplitKBytes(int64_t m, int64_t n, int slices) { return slices > 1 ? static_cast<size_t>(slices) * m * n * sizeof(float) : 0; }
}  // namespace

// out[m][n] = sum over b < batch, k < depth of a[b][m][k] * bt[b][n][k]: one matrix product per batch entry, accumulated.  Rows of a_b
// and bt_b are dense along k; a_row / bt_row are their row strides and a_slice / bt_slice the distances between batch entries, in
// elements.  out is row-major [m][n].  Float partial sums go to `partial` when BatchedProductSlices(...) > 1
// (BatchedProductPartialBytes bytes).  float16 / float32; the operands must satisfy the MFMA kernel's 8-byte granularity.
int BatchedProductSlices(int64_t m, int64_t n, int64_t depth, int batch, int dtype) {
    const int64_t it = ItemSize(dtype);
    const int64_t steps_per = (depth * it + 127) / 128;
    const int planned = PlanSplitK(m, n, depth * batch, dtype);
    const int64_t steps = steps_per * batch;
    return planned > steps ? static_cast<int>(steps) : planned;
}

size_t BatchedProductPartialBytes(int64_t m, int64_t n, int64_t depth, int batch, int dtype) {
    return SplitKBytes(m, n, BatchedProductSlices(m, n, depth, batch, dtype));
}

bool BatchedProductApplies(const void* a, int64_t a_row, int64_t a_slice, const void* bt, int64_t bt_row, int64_t bt_slice, int64_t depth,
                           const void* out, int dtype) {
    if (dtype != HIPCX_FLOAT16 && dtype != HIPCX_FLOAT32) return false;
    const int64_t epc = 16 / ItemSize(dtype);  // 16-byte granules throughout
    return depth % epc == 0 && a_row % epc == 0 && a_slice % epc == 0 && bt_row % epc == 0 && bt_slice % epc == 0 && Aligned(a, 16) &&
           Aligned(bt, 16) && Aligned(out, 16);
}

// With taps_s > 0 row j of bt_b is a window of a larger array: j = (c, r, s) with c = j / (taps_r * taps_s) starts at
// bt_b + c * bt_row + r * r_stride + s * s_stride (elements; 16-byte granules like the other strides).
void LaunchBatchedProduct(int dtype, const void* a, int64_t a_row, int64_t a_slice, const void* bt, int64_t bt_row, int64_t bt_slice, int64_t m,
                          int64_t n, int64_t depth, int batch, void* out, float* partial, hipStream_t stream, int taps_r, int taps_s,
                          int64_t r_stride, int64_t s_stride) {
    auto run = [&](auto tag) {
        using T = decltype(tag);
        IGemmArgs<T> p{};
        p.x = static_cast<const T*>(a);
        p.w = static_cast<const T*>(bt);
        p.out = static_cast<T*>(out);
        p.N = static_cast<int>(m);
        p.C = static_cast<int>(depth);
        p.H = p.W = 1;
        p.K = static_cast<int>(n);
        p.R = p.S = 1;
        p.OH = p.OW = 1;
        p.stride_h = p.stride_w = 1;
        p.xsN = a_row, p.xsC = 1;
        p.wsK = bt_row, p.wsC = 1;
        p.wsR = p.wsS = depth;
        p.osN = n, p.osC = 1;
        p.M = m;
        p.Kg = static_cast<int>(depth);
        p.batch = batch;
        p.x_slice = a_slice, p.w_slice = bt_slice;
        p.w_taps_r = taps_r, p.w_taps_s = taps_s;
        p.w_r_stride = r_stride, p.w_s_stride = s_stride;
        p.ksplit = partial != nullptr ? BatchedProductSlices(m, n, depth, batch, dtype) : 1;
        p.partial = p.ksplit > 1 ? partial : nullptr;
        // the work accounting of the launch sees the whole reduction
        p.C_logical = static_cast<int>(std::min<int64_t>(depth * batch, 0x7fffffff));
        p.H_logical = p.W_logical = 1;
        LaunchIGemmImpl(p, stream);
    };
    if (dtype == HIPCX_FLOAT16) run(half_t{});
    else run(float{});
}

extern "C" {

size_t hipcx_dot_workspace_size(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out) {
    try {
        if (out != nullptr && !IsFloatDtype(out->dtype)) return 0;
        DotStaging st = PlanDotStaging(a, b, out);
        size_t split = 0;
        if (a != nullptr && b != nullptr && out != nullptr && a->ndim == 2 && b->ndim == 2) {
            split = SplitKBytes(a->shape[0], b->shape[1], PlanSplitK(a->shape[0], b->shape[1], a->shape[1], out->dtype));
        }
        return RoundUpTo(st.a_bytes + st.b_bytes, 256) + split;
    } catch (...) {
        return 0;
    }
}

int hipcx_dot(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream) {
    return Guard([&] {
        ValidateArray(a, "a");
        ValidateArray(b, "b");
        ValidateArray(out, "out");
        HIPCX_REQUIRE(a->ndim == 2 && b->ndim == 2 && out->ndim == 2, HIPCX_DIMENSION_ERROR,
                      "ChainerX dot supports only 2-dimensional arrays.");
        int64_t m = a->shape[0], k = a->shape[1], n = b->shape[1];
        HIPCX_REQUIRE(b->shape[0] == k && out->shape[0] == m && out->shape[1] == n, HIPCX_DIMENSION_ERROR, "dot: shape mismatch");
        HIPCX_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype, HIPCX_DTYPE_ERROR,
                      "a and b must have out's dtype (cast with hipcx_copy first)");
        HIPCX_REQUIRE(m < (1LL << 31) && n < (1LL << 31) && k < (1LL << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "extent too large");
        if (m == 0 || n == 0) return;
        hipStream_t st = AsStream(stream);
        if (k == 0) {  // the routine normally short-circuits this (CX/routines/linalg.cc:59-61)
            hipcx_scalar zero{HIPCX_KIND_INT, 0, 0, 0.0};
            int s = hipcx_fill(out, zero, stream);
            if (s != HIPCX_OK) throw Error(s, hipcx_last_error());
            return;
        }
        if (!IsFloatDtype(out->dtype)) {  // integers and bool: int_dot.hip
            IntDot(a, b, out, st);
            return;
        }
        auto fill = [&](auto& p) {
            using T = std::remove_cv_t<std::remove_pointer_t<decltype(p.out)>>;
            p.x = static_cast<const T*>(a->data);
            p.w = static_cast<const T*>(b->data);
            p.bias = nullptr;
            p.bias_stride = 0;
            p.out = static_cast<T*>(out->data);
            p.N = static_cast<int>(m);
            p.C = static_cast<int>(k);
            p.H = p.W = 1;
            p.K = static_cast<int>(n);
            p.R = p.S = 1;
            p.OH = p.OW = 1;
            p.stride_h = p.stride_w = 1;
            p.pad_h = p.pad_w = 0;
            p.xsN = ElemStride(a, 0, "a");
            p.xsC = ElemStride(a, 1, "a");
            p.xsH = p.xsW = 0;
            p.wsK = ElemStride(b, 1, "b");  // filter n is column n of b
            p.wsC = ElemStride(b, 0, "b");
            p.wsR = p.wsS = k;
            p.osN = ElemStride(out, 0, "out");
            p.osC = ElemStride(out, 1, "out");
            p.osH = p.osW = 0;
            p.M = m;
            p.Kg = static_cast<int>(k);
        };
        // operands in another layout than the MFMA kernels read are staged in the workspace first
        hipcx_array a_st = *a, b_st = *b;
        const int64_t k_given = k;  // the reduction extent the workspace query saw (staging may pad it)
        size_t staged_bytes = 0;    // the front of the workspace that holds staged operands
        if (out->dtype == a->dtype && out->dtype == b->dtype) {
            DotStaging plan = PlanDotStaging(a, b, out);
            if (plan.a || plan.b) {
                staged_bytes = plan.a_bytes + plan.b_bytes;
                HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= plan.a_bytes + plan.b_bytes, HIPCX_CHAINERX_ERROR,
                              "dot: workspace of " + std::to_string(plan.a_bytes + plan.b_bytes) + " bytes required (hipcx_dot_workspace_size)");
                HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 16-byte aligned");
                const int64_t it = ItemSize(out->dtype);
                char* ws = static_cast<char*>(workspace);
                auto stage = [&](const hipcx_array* src, bool transposed, int64_t lines, char* dst, hipcx_array& view) {
                    // lines = rows of a, or columns of b; the staged matrix is [lines][kpad]
                    const int64_t sl = src->strides[transposed ? 1 : 0] / it, sk = src->strides[transposed ? 0 : 1] / it;
                    HIPCX_REQUIRE(src->strides[0] % it == 0 && src->strides[1] % it == 0, HIPCX_NOT_IMPLEMENTED_ERROR,
                                  "dot: byte strides must be multiples of the item size");
                    if (out->dtype == HIPCX_FLOAT16) {
                        StageMatrix<half_t>(static_cast<const half_t*>(src->data), sl, sk, reinterpret_cast<half_t*>(dst), plan.kpad, lines, k, st);
                    } else {
                        StageMatrix<float>(static_cast<const float*>(src->data), sl, sk, reinterpret_cast<float*>(dst), plan.kpad, lines, k, st);
                    }
                    view.data = dst;
                    view.shape[transposed ? 1 : 0] = lines;
                    view.shape[transposed ? 0 : 1] = plan.kpad;
                    view.strides[transposed ? 1 : 0] = plan.kpad * it;
                    view.strides[transposed ? 0 : 1] = it;
                };
                if (plan.a) stage(a, false, m, ws, a_st);
                if (plan.b) stage(b, true, n, ws + plan.a_bytes, b_st);
                k = plan.kpad;
            }
        }
        a = &a_st;
        b = &b_st;
        // few output tiles over a long reduction axis, both operands laid out for the MFMA kernel: split the reduction
        int slices = 1;
        float* partial = nullptr;
        {
            const int64_t it = ItemSize(out->dtype);
            // slices from the extent the workspace query planned with; the partial sums lie behind the staged operands
            const int planned = PlanSplitK(m, n, k_given, out->dtype);
            if (planned > 1 && OperandIsFast(a->data, a->strides[0], a->strides[1], k, it) &&
                OperandIsFast(b->data, b->strides[1], b->strides[0], k, it) && out->strides[0] >= 0 && out->strides[1] >= 0) {
                const size_t offset = RoundUpTo(staged_bytes, 256);
                const size_t need = offset + SplitKBytes(m, n, planned);
                if (workspace != nullptr && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
                    slices = planned;
                    partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + offset);
                }
            }
        }
        if (out->dtype == HIPCX_FLOAT16) {
            if (slices == 1 && TryGemmPp(a, b, out, st)) return;
            if (slices == 1 && TrySmallDot<half_t>(a, b, out, st)) return;
            IGemmArgs<half_t> p{};
            fill(p);
            p.ksplit = slices;
            p.partial = partial;
            LaunchIGemmImpl(p, st);
        } else if (out->dtype == HIPCX_FLOAT32) {
            if (slices == 1 && TrySmallDot<float>(a, b, out, st)) return;
            IGemmArgs<float> p{};
            fill(p);
            p.ksplit = slices;
            p.partial = partial;
            LaunchIGemmImpl(p, st);
        } else {
            IGemmArgs<double> p{};
            fill(p);
            LaunchF64(p, st);
        }
    });
}
}
