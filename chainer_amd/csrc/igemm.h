// Implicit-GEMM core shared by Dot and Conv forward.
//
//   out[pixel m, channel n] = bias[n] + sum_{r,s,c} x[img(m), c, ih(m,r), iw(m,s)] * w[n, c, r, s]
//
// A "pixel" is one (image, oh, ow) output position; Dot is the 1x1 case with one pixel per row of
// `a`.  The reduction index runs over (r, s, c) with c fastest, which is the memory order of a
// channels-last activation and of a [K][R][S][C] filter bank.
//
// MFMA orientation: the filter tile is the A operand (rows = output channels) and the pixel tile
// the B operand (columns = pixels), so that after v_mfma_f32_32x32x{16 f16, 2 f32} a lane holds
// 4 consecutive output channels of one pixel -- an 8/16-byte store into channels-last memory.
//
// Block tile = (64*WM pixels) x (64*WN channels), 64 threads per 64x64 wave tile, K step = 128
// bytes per row.  Global -> register -> LDS software pipeline with one LDS buffer; LDS rows are
// padded by 16 bytes so that the 16-byte fragment reads of 16 consecutive rows hit distinct banks.
#pragma once

#include "common.h"

namespace hipcx {

template <typename T>
struct IGemmArgs {
    const T* x;
    const T* w;
    const T* bias;  // may be null
    int64_t bias_stride;  // elements
    T* out;
    int N, C, H, W;  // input extents (as the kernel sees them: after channel padding / sub-sampling)
    int C_logical, H_logical, W_logical;  // the caller's extents, for work accounting only
    int K, R, S;     // filters
    int OH, OW;
    int stride_h, stride_w, pad_h, pad_w;
    int64_t xsN, xsC, xsH, xsW;  // element strides of x
    int64_t wsK, wsC, wsR, wsS;  // element strides of w (fast path: wsK only, rows are [R][S][C] dense)
    int64_t osN, osC, osH, osW;  // element strides of out
    int64_t M;                   // N*OH*OW
    int Kg;                      // R*S*C
    int tiles_m, tiles_n;
    int band;                    // fast kernel: tile columns per band of the tile order (0: columns fast over the whole row)
    int out_vec;                 // 1 if the 4 accumulators a lane holds per group can be stored as one vector
    int out_wide;                // 1 if 16-byte runs along the output's contiguous axis can be stored (pipelined kernel)
    // Split reduction (matrix products with few output tiles and a long reduction axis, e.g. weight gradients): grid.x slices of
    // the reduction steps, each storing float partial sums [ksplit][M][K]; SplitKReduceKernel adds them up.  0 or 1: off.
    int ksplit;
    float* partial;
    // Batched reduction (fast kernel only): out = sum over b < batch of x_b @ w_b^T with x_b = x + b * x_slice and
    // w_b = w + b * w_slice (elements).  The reduction steps of all batches form one sequence, which is what ksplit slices.
    // 0: off.  Weight gradients of 1x1 convolutions read gy and x in place this way (one [channels, pixels] matrix per image).
    int batch;
    int64_t x_slice, w_slice;
    // Filter rows that alias shifted windows of one array (fast kernel; weight gradients of filters larger than 1x1 at stride 1):
    // row n = (c, r, s), c = n / (w_taps_r * w_taps_s), starts at w + c * wsK + r * w_r_stride + s * w_s_stride.  w_taps_s == 0: off.
    int w_taps_r, w_taps_s;
    int64_t w_r_stride, w_s_stride;
};

constexpr int kRowBytes = 128;           // bytes of the reduction axis per tile row
constexpr int kLdsRow = kRowBytes + 16;  // padded LDS row

using half8_t = __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16;
using float4_t = __attribute__((__vector_size__(4 * sizeof(float)))) float;
using float16_t = __attribute__((__vector_size__(16 * sizeof(float)))) float;

// 16- and 8-byte chunks as native vector types, so that arrays of them are promoted to registers
using Bytes16 = __attribute__((ext_vector_type(4))) unsigned int;
using Bytes8 = __attribute__((ext_vector_type(2))) unsigned int;
template <int LB>
struct BytesOf;
template <>
struct BytesOf<16> {
    using type = Bytes16;
};
template <>
struct BytesOf<8> {
    using type = Bytes8;
};

// XCD-aware tile order: hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each
// with its own L2.  Remap so that every XCD walks a contiguous range of tiles; with the channel
// tile as the fast index, blocks that share an activation tile then share an L2.
__device__ __forceinline__ bool TileOf(int tiles_m, int tiles_n, int b, int& tile_m, int& tile_n) {
    int total = tiles_m * tiles_n;
    int per = (total + 7) / 8;
    if (b >= per * 8) return false;
    int logical = (b % 8) * per + b / 8;
    if (logical >= total) return false;
    tile_n = logical % tiles_n;
    tile_m = logical / tiles_n;
    return true;
}
__device__ __forceinline__ bool TileOf(int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
    return TileOf(tiles_m, tiles_n, static_cast<int>(blockIdx.x), tile_m, tile_n);
}
// The same with the tile columns cut into bands of `band`: inside a band the column is still the fast index, and the rows are
// walked before the next band starts.  The 32 tiles an XCD runs at a time then cover band columns x 32 / band rows and read
// band + 32 / band operand panels instead of 33, and a band's filter panels stay in that XCD's L2 while its rows go by: for
// products with many tile columns (wide matrix products) this is what keeps the second operand from being fetched once per tile row.
__device__ __forceinline__ bool TileOfBanded(int tiles_m, int tiles_n, int band, int& tile_m, int& tile_n) {
    if (band <= 0) return TileOf(tiles_m, tiles_n, tile_m, tile_n);
    int total = tiles_m * tiles_n;
    int per = (total + 7) / 8;
    int b = static_cast<int>(blockIdx.x);
    if (b >= per * 8) return false;
    int logical = (b % 8) * per + b / 8;
    if (logical >= total) return false;
    int band_tiles = band * tiles_m;
    int bi = logical / band_tiles;
    int rem = logical - bi * band_tiles;
    int cols = min(band, tiles_n - bi * band);
    tile_n = bi * band + rem % cols;
    tile_m = rem / cols;
    return true;
}

template <typename T>
__device__ __forceinline__ void MfmaTile(const Bytes16& a, const Bytes16& b, float16_t& acc);

template <>
__device__ __forceinline__ void MfmaTile<half_t>(const Bytes16& a, const Bytes16& b, float16_t& acc) {
    half8_t av = __builtin_bit_cast(half8_t, a);
    half8_t bv = __builtin_bit_cast(half8_t, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
}

template <>
__device__ __forceinline__ void MfmaTile<float>(const Bytes16& a, const Bytes16& b, float16_t& acc) {
    float4_t af = __builtin_bit_cast(float4_t, a);
    float4_t bf = __builtin_bit_cast(float4_t, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[0], bf[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[1], bf[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[2], bf[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[3], bf[3], acc, 0, 0, 0);
}

// One K step over the LDS tile: every wave multiplies its 64 channels x 64 pixels.
// PM (pixel-major accumulators): the pixel tile is the A operand instead, so a lane ends up with 4
// consecutive pixels of one channel -- the vector store of channels-first (NCHW) memory.
template <typename T, bool PM>
__device__ __forceinline__ void ComputeTile(const char* ldsX, const char* ldsW, int wm, int wn, int lane, float16_t (&acc)[2][2]) {
    const int lr = lane & 31;
    const int g = lane >> 5;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        Bytes16 wf[2], xf[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            wf[t] = *reinterpret_cast<const Bytes16*>(ldsW + (wn * 64 + t * 32 + lr) * kLdsRow + (2 * q + g) * 16);
            xf[t] = *reinterpret_cast<const Bytes16*>(ldsX + (wm * 64 + t * 32 + lr) * kLdsRow + (2 * q + g) * 16);
        }
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
            for (int tj = 0; tj < 2; ++tj) {
                if (PM) {
                    MfmaTile<T>(xf[ti], wf[tj], acc[ti][tj]);
                } else {
                    MfmaTile<T>(wf[ti], xf[tj], acc[ti][tj]);
                }
            }
        }
    }
}

// Writes the wave's accumulators: lane holds, for pixel column (lane % 32) of each 32-wide pixel
// sub-tile, channel rows 8*(v/4) + 4*(lane/32) + v%4.
template <typename T>
__device__ __forceinline__ void StoreTile(const IGemmArgs<T>& p, int m0, int n0, int wm, int wn, int lane, float16_t (&acc)[2][2]) {
    const int lr = lane & 31;
    const int g = lane >> 5;
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        int64_t m = static_cast<int64_t>(m0) + wm * 64 + tj * 32 + lr;
        if (m >= p.M) continue;
        int ow = static_cast<int>(m % p.OW);
        int64_t t = m / p.OW;
        int oh = static_cast<int>(t % p.OH);
        int64_t img = t / p.OH;
        T* o = p.out + img * p.osN + oh * p.osH + ow * p.osW;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                int n = n0 + wn * 64 + ti * 32 + vq * 8 + g * 4;
                if (n >= p.K) continue;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[ti][tj][vq * 4 + e];
                if (p.bias != nullptr) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e < p.K) v[e] += static_cast<float>(p.bias[(n + e) * p.bias_stride]);
                    }
                }
                if (p.out_vec) {  // n + 3 < K is implied: K % 4 == 0
                    struct alignas(sizeof(T) * 4) Out4 {
                        T e[4];
                    } pack;
#pragma unroll
                    for (int e = 0; e < 4; ++e) pack.e[e] = static_cast<T>(v[e]);
                    *reinterpret_cast<Out4*>(o + n) = pack;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e < p.K) o[static_cast<int64_t>(n + e) * p.osC] = static_cast<T>(v[e]);
                    }
                }
            }
        }
    }
}

// Split reduction: the accumulators go out as floats, partial[slice][m][n], in StoreTile's orientation.
template <typename T>
__device__ __forceinline__ void StorePartial(const IGemmArgs<T>& p, int m0, int n0, int wm, int wn, int lane, float16_t (&acc)[2][2], int slice) {
    const int lr = lane & 31;
    const int g = lane >> 5;
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        int64_t m = static_cast<int64_t>(m0) + wm * 64 + tj * 32 + lr;
        if (m >= p.M) continue;
        float* o = p.partial + (static_cast<int64_t>(slice) * p.M + m) * p.K;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                int n = n0 + wn * 64 + ti * 32 + vq * 8 + g * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (n + e < p.K) o[n + e] = acc[ti][tj][vq * 4 + e];
                }
            }
        }
    }
}

// out[m][n] = sum over slices of partial[slice][m][n] (+ bias), for outputs addressed as out + m * osN + n * osC (matrix products).
template <typename T>
__global__ __launch_bounds__(256) void SplitKReduceKernel(IGemmArgs<T> p) {
    // 64 outputs per workgroup, the slices dealt out over its four waves (four independent loads in flight per lane), the four
    // partial sums joined through LDS: the loop over the slices is a chain of memory latencies otherwise.
    __shared__ float part[4][64];
    const int64_t total = p.M * p.K;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * 64; base < total; base += static_cast<int64_t>(gridDim.x) * 64) {
        const int64_t i = base + tx;
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        if (i < total) {
            int sl = ty;
            for (; sl + 12 < p.ksplit; sl += 16) {
                s0 += p.partial[static_cast<int64_t>(sl) * total + i];
                s1 += p.partial[static_cast<int64_t>(sl + 4) * total + i];
                s2 += p.partial[static_cast<int64_t>(sl + 8) * total + i];
                s3 += p.partial[static_cast<int64_t>(sl + 12) * total + i];
            }
            for (; sl < p.ksplit; sl += 4) s0 += p.partial[static_cast<int64_t>(sl) * total + i];
        }
        part[ty][tx] = (s0 + s1) + (s2 + s3);
        __syncthreads();
        if (ty == 0 && i < total) {
            float sum = (part[0][tx] + part[1][tx]) + (part[2][tx] + part[3][tx]);
            const int64_t m = i / p.K;
            const int n = static_cast<int>(i - m * p.K);
            if (p.bias != nullptr) sum += static_cast<float>(p.bias[n * p.bias_stride]);
            p.out[m * p.osN + static_cast<int64_t>(n) * p.osC] = static_cast<T>(sum);
        }
        __syncthreads();
    }
}

// Pixel-major variant: lane holds, for channel column (lane % 32) of each 32-wide channel sub-tile,
// pixel rows 8*(v/4) + 4*(lane/32) + v%4.  `out_vec` here means: 4 consecutive pixels of a channel
// are 4 consecutive elements (dense OH*OW planes, OH*OW % 4 == 0, aligned).
template <typename T>
__device__ __forceinline__ void StoreTilePM(const IGemmArgs<T>& p, int m0, int n0, int wm, int wn, int lane, float16_t (&acc)[2][2]) {
    const int lr = lane & 31;
    const int g = lane >> 5;
    const int64_t ohw = static_cast<int64_t>(p.OH) * p.OW;
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        int n = n0 + wn * 64 + tj * 32 + lr;
        if (n >= p.K) continue;
        float bias = p.bias != nullptr ? static_cast<float>(p.bias[n * p.bias_stride]) : 0.f;
        T* oc = p.out + static_cast<int64_t>(n) * p.osC;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                int64_t m = static_cast<int64_t>(m0) + wm * 64 + ti * 32 + vq * 8 + g * 4;
                if (m >= p.M) continue;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[ti][tj][vq * 4 + e] + bias;
                if (p.out_vec) {  // m % 4 == 0 and OH*OW % 4 == 0: the four pixels share an image and are adjacent
                    int64_t img = m / ohw;
                    int64_t pix = m - img * ohw;
                    struct alignas(sizeof(T) * 4) Out4 {
                        T e[4];
                    } pack;
#pragma unroll
                    for (int e = 0; e < 4; ++e) pack.e[e] = static_cast<T>(v[e]);
                    *reinterpret_cast<Out4*>(oc + img * p.osN + pix) = pack;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        int64_t me = m + e;
                        if (me >= p.M) continue;
                        int ow = static_cast<int>(me % p.OW);
                        int64_t t = me / p.OW;
                        int oh = static_cast<int>(t % p.OH);
                        int64_t img = t / p.OH;
                        oc[img * p.osN + oh * p.osH + ow * p.osW] = static_cast<T>(v[e]);
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Fast path: x is channels-last (xsC == 1), filter rows are dense [R][S][C]; LB-byte global loads.
// ---------------------------------------------------------------------------------------------
template <typename T, int WM, int WN, int LB, bool PM>
__global__ __launch_bounds__(64 * WM * WN) void IGemmFastKernel(IGemmArgs<T> p) {
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 64 * WM;
    constexpr int BN = 64 * WN;
    constexpr int BKE = kRowBytes / sizeof(T);  // elements of K per step
    constexpr int CPR = kRowBytes / LB;         // chunks per row
    constexpr int EPC = LB / sizeof(T);         // elements per chunk
    constexpr int XCH = BM * CPR / NT;          // chunks per thread
    constexpr int WCH = BN * CPR / NT;
    using Chunk = typename BytesOf<LB>::type;
    static_assert(NT % CPR == 0, "row index must advance uniformly");

    __shared__ __align__(16) char lds[(BM + BN) * kLdsRow];
    char* ldsX = lds;
    char* ldsW = lds + BM * kLdsRow;

    int tile_m, tile_n;
    unsigned slice = 0;
    if (p.ksplit > 1) {
        // Split reduction: grid (slices, tiles).  Workgroup ids go round-robin to the 8 XCDs with x as the fast index, so the
        // slices of one tile spread over all of them -- with the tiles along x, a product of one or two tiles would keep one
        // or two XCDs (a quarter of the chip) busy however many slices it has.
        slice = blockIdx.x;
        tile_n = static_cast<int>(blockIdx.y) % p.tiles_n;
        tile_m = static_cast<int>(blockIdx.y) / p.tiles_n;
    } else if (!TileOfBanded(p.tiles_m, p.tiles_n, p.band, tile_m, tile_n)) {
        return;
    }
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM;
    const int wn = wave / WM;
    const int kc = tid % CPR;    // chunk column of this thread (same for all its chunks)
    const int row0 = tid / CPR;  // first row; further rows are NT/CPR apart

    // per-thread pixel rows
    int64_t xbase[XCH];
    int ih0[XCH], iw0[XCH];
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
        int64_t m = static_cast<int64_t>(m0) + row0 + i * (NT / CPR);
        if (m < p.M) {
            int ow = static_cast<int>(m % p.OW);
            int64_t t = m / p.OW;
            int oh = static_cast<int>(t % p.OH);
            int64_t img = t / p.OH;
            xbase[i] = img * p.xsN;
            ih0[i] = oh * p.stride_h - p.pad_h;
            iw0[i] = ow * p.stride_w - p.pad_w;
        } else {
            xbase[i] = 0;
            ih0[i] = -0x40000000;  // fails every bounds check
            iw0[i] = 0;
        }
    }
    const T* wrow[WCH];
    bool wvalid[WCH];
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
        int n = n0 + row0 + i * (NT / CPR);
        wvalid[i] = n < p.K;
        if (!wvalid[i]) n = 0;
        if (p.w_taps_s > 0) {
            const int taps = p.w_taps_r * p.w_taps_s;
            const int c = n / taps, t = n - c * taps;
            const int r = t / p.w_taps_s, s = t - r * p.w_taps_s;
            wrow[i] = p.w + static_cast<int64_t>(c) * p.wsK + r * p.w_r_stride + s * p.w_s_stride;
        } else {
            wrow[i] = p.w + static_cast<int64_t>(n) * p.wsK;
        }
    }

    const bool uniform_rs = (p.C % BKE) == 0;
    const bool is_1x1 = (p.R == 1 && p.S == 1);
    const int nk = (p.Kg + BKE - 1) / BKE;

    Chunk xreg[XCH], wreg[WCH];
    auto load_tile = [&](int kt) {
        int64_t x_off = 0, w_off = 0;
        if (p.batch > 0) {
            const int b = kt / nk;
            kt -= b * nk;
            x_off = b * p.x_slice;
            w_off = b * p.w_slice;
        }
        const int kbase = kt * BKE;
        const int kk = kbase + kc * EPC;
        const bool kvalid = kk < p.Kg;
        int r, s, c;
        if (is_1x1) {
            r = 0;
            s = 0;
            c = kk;
        } else if (uniform_rs) {
            int rs = kbase / p.C;
            c = kbase - rs * p.C + kc * EPC;
            r = rs / p.S;
            s = rs - r * p.S;
        } else {
            int rs = kk / p.C;
            c = kk - rs * p.C;
            r = rs / p.S;
            s = rs - r * p.S;
        }
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            int ih = ih0[i] + r;
            int iw = iw0[i] + s;
            bool ok = kvalid && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            Chunk v = Chunk(0);
            if (ok) v = *reinterpret_cast<const Chunk*>(p.x + x_off + xbase[i] + ih * p.xsH + iw * p.xsW + c);
            xreg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            Chunk v = Chunk(0);
            if (kvalid && wvalid[i]) v = *reinterpret_cast<const Chunk*>(wrow[i] + w_off + kk);
            wreg[i] = v;
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            *reinterpret_cast<Chunk*>(ldsX + (row0 + i * (NT / CPR)) * kLdsRow + kc * LB) = xreg[i];
        }
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            *reinterpret_cast<Chunk*>(ldsW + (row0 + i * (NT / CPR)) * kLdsRow + kc * LB) = wreg[i];
        }
    };

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        }
    }

    const int steps = p.batch > 0 ? nk * p.batch : nk;
    int kt_begin = 0, kt_end = steps;
    if (p.ksplit > 1) {
        kt_begin = static_cast<int>(static_cast<int64_t>(steps) * slice / p.ksplit);
        kt_end = static_cast<int>(static_cast<int64_t>(steps) * (slice + 1) / p.ksplit);
    }
    if (kt_begin < kt_end) load_tile(kt_begin);
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        store_tile();
        __syncthreads();
        if (kt + 1 < kt_end) load_tile(kt + 1);
        ComputeTile<T, PM>(ldsX, ldsW, wm, wn, lane, acc);
        __syncthreads();
    }
    if (p.ksplit > 1) {
        if constexpr (!PM) StorePartial<T>(p, m0, n0, wm, wn, lane, acc, slice);
        return;
    }
    if (PM) {
        StoreTilePM<T>(p, m0, n0, wm, wn, lane, acc);
    } else {
        StoreTile<T>(p, m0, n0, wm, wn, lane, acc);
    }
}

// ---------------------------------------------------------------------------------------------
// Generic path: any strides on x and w, any C; element-wise gathers.  Per-row pixel data lives in
// LDS.  `X_ROW_FAST` / `W_ROW_FAST` choose which tile index consecutive threads walk, so that the
// memory-contiguous one is the coalesced one.
// ---------------------------------------------------------------------------------------------
template <typename T, int WM, int WN, bool PM>
__global__ __launch_bounds__(64 * WM * WN) void IGemmGenericKernel(IGemmArgs<T> p, int x_row_fast, int w_row_fast) {
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 64 * WM;
    constexpr int BN = 64 * WN;
    constexpr int BKE = kRowBytes / sizeof(T);

    __shared__ __align__(16) char lds[(BM + BN) * kLdsRow];
    __shared__ int64_t row_base[BM];
    __shared__ int row_ih0[BM];
    __shared__ int row_iw0[BM];
    char* ldsX = lds;
    char* ldsW = lds + BM * kLdsRow;

    int tile_m, tile_n;
    if (!TileOf(p.tiles_m, p.tiles_n, tile_m, tile_n)) return;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM;
    const int wn = wave / WM;

    for (int row = tid; row < BM; row += NT) {
        int64_t m = static_cast<int64_t>(m0) + row;
        if (m < p.M) {
            int ow = static_cast<int>(m % p.OW);
            int64_t t = m / p.OW;
            int oh = static_cast<int>(t % p.OH);
            int64_t img = t / p.OH;
            row_base[row] = img * p.xsN;
            row_ih0[row] = oh * p.stride_h - p.pad_h;
            row_iw0[row] = ow * p.stride_w - p.pad_w;
        } else {
            row_base[row] = 0;
            row_ih0[row] = -0x40000000;
            row_iw0[row] = 0;
        }
    }
    __syncthreads();

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        }
    }

    const int nk = (p.Kg + BKE - 1) / BKE;
    for (int kt = 0; kt < nk; ++kt) {
        const int kbase = kt * BKE;
        // activations
        for (int e = tid; e < BM * BKE; e += NT) {
            int row, kl;
            if (x_row_fast) {
                row = e % BM;
                kl = e / BM;
            } else {
                kl = e % BKE;
                row = e / BKE;
            }
            int kk = kbase + kl;
            T v = T(0);
            if (kk < p.Kg) {
                int rs = kk / p.C;
                int c = kk - rs * p.C;
                int r = rs / p.S;
                int s = rs - r * p.S;
                int ih = row_ih0[row] + r;
                int iw = row_iw0[row] + s;
                if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.W) {
                    v = p.x[row_base[row] + c * p.xsC + ih * p.xsH + iw * p.xsW];
                }
            }
            *reinterpret_cast<T*>(ldsX + row * kLdsRow + kl * sizeof(T)) = v;
        }
        // filters
        for (int e = tid; e < BN * BKE; e += NT) {
            int row, kl;
            if (w_row_fast) {
                row = e % BN;
                kl = e / BN;
            } else {
                kl = e % BKE;
                row = e / BKE;
            }
            int kk = kbase + kl;
            int n = n0 + row;
            T v = T(0);
            if (kk < p.Kg && n < p.K) {
                int rs = kk / p.C;
                int c = kk - rs * p.C;
                int r = rs / p.S;
                int s = rs - r * p.S;
                v = p.w[static_cast<int64_t>(n) * p.wsK + c * p.wsC + r * p.wsR + s * p.wsS];
            }
            *reinterpret_cast<T*>(ldsW + row * kLdsRow + kl * sizeof(T)) = v;
        }
        __syncthreads();
        ComputeTile<T, PM>(ldsX, ldsW, wm, wn, lane, acc);
        __syncthreads();
    }
    if (PM) {
        StoreTilePM<T>(p, m0, n0, wm, wn, lane, acc);
    } else {
        StoreTile<T>(p, m0, n0, wm, wn, lane, acc);
    }
}

// Host-side launcher: picks tile shape and path.  `w_dense_rsc` says that w rows are laid out as
// [R][S][C] with unit element stride (i.e. wsC == 1, wsS == C, wsR == S*C).
template <typename T>
void LaunchIGemm(IGemmArgs<T> p, hipStream_t stream);

}  // namespace hipcx
