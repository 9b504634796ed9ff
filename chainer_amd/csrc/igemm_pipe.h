// Pipelined implicit-GEMM kernel (the production path for channels-last activations).
//
// Same math and tile shape as igemm.h; what differs is how the operands travel:
//   * two register sets prefetch the tiles of K-steps kt+1 and kt+2 while step kt is multiplied,
//     so every global load has two full MFMA phases to land;
//   * two LDS buffers, rows of exactly 128 bytes, 16-byte slots XOR-swizzled with (row >> 1) & 7:
//     the 16-byte fragment reads of 16 consecutive rows then cover 16 distinct bank groups, and
//     no padding is needed (64 KiB for the 128x128 tile -> two blocks per CU);
//   * the accumulators leave through LDS: they are regrouped into 16-byte runs along the output's
//     contiguous axis (pixels for channels-first results, channels for channels-last ones) so that
//     a wave's store instruction writes whole cache lines.
#pragma once

#include "igemm.h"

namespace hipcx {

__device__ __forceinline__ int SwzSlot(int row, int slot) { return slot ^ ((row >> 1) & 7); }

// One K step out of a swizzled stage buffer.  Fragments are double-buffered by hand (the reads of
// sub-step q+1 are issued before the MFMAs of sub-step q) and scheduling barriers keep the compiler
// from hoisting all 16 fragment reads to the top, which would cost 64 registers.
template <typename T, bool PM>
__device__ __forceinline__ void ComputeTileSwz(const char* ldsX, const char* ldsW, int wm, int wn, int lane, float16_t (&acc)[2][2]) {
    const int lr = lane & 31;
    const int g = lane >> 5;
    const char* xp[2];
    const char* wp[2];
    int xs[2], ws[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        int xr = wm * 64 + t * 32 + lr;
        int wr = wn * 64 + t * 32 + lr;
        xp[t] = ldsX + xr * kRowBytes;
        wp[t] = ldsW + wr * kRowBytes;
        xs[t] = (xr >> 1) & 7;
        ws[t] = (wr >> 1) & 7;
    }
    Bytes16 wf[2][2], xf[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        wf[0][t] = *reinterpret_cast<const Bytes16*>(wp[t] + ((g ^ ws[t]) << 4));
        xf[0][t] = *reinterpret_cast<const Bytes16*>(xp[t] + ((g ^ xs[t]) << 4));
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int cur = q & 1, nxt = cur ^ 1;
        if (q < 3) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                wf[nxt][t] = *reinterpret_cast<const Bytes16*>(wp[t] + (((2 * (q + 1) + g) ^ ws[t]) << 4));
                xf[nxt][t] = *reinterpret_cast<const Bytes16*>(xp[t] + (((2 * (q + 1) + g) ^ xs[t]) << 4));
            }
        }
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
            for (int tj = 0; tj < 2; ++tj) {
                if (PM) {
                    MfmaTile<T>(xf[cur][ti], wf[cur][tj], acc[ti][tj]);
                } else {
                    MfmaTile<T>(wf[cur][ti], xf[cur][tj], acc[ti][tj]);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <typename T, int WM, int WN, int LB, bool PM>
__global__ __launch_bounds__(64 * WM * WN, 2) void IGemmPipeKernel(IGemmArgs<T> p) {
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 64 * WM;
    constexpr int BN = 64 * WN;
    constexpr int BKE = kRowBytes / sizeof(T);  // elements of K per step
    constexpr int CPR = kRowBytes / LB;         // chunks per row
    constexpr int EPC = LB / sizeof(T);         // elements per chunk
    constexpr int RS_ = NT / CPR;               // rows covered per pass
    constexpr int XCH = BM / RS_;               // chunks per thread
    constexpr int WCH = BN / RS_;
    constexpr int STAGE = (BM + BN) * kRowBytes;
    using Chunk = typename BytesOf<LB>::type;
    static_assert(NT % CPR == 0 && BM % RS_ == 0 && BN % RS_ == 0, "tile does not divide among threads");

    extern __shared__ __align__(16) char lds[];  // PipeLdsBytes(): two stages, or the epilogue's staging tile if larger

    int tile_m, tile_n;
    if (!TileOf(p.tiles_m, p.tiles_n, tile_m, tile_n)) return;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM;
    const int wn = wave / WM;
    const int kc = tid % CPR;    // chunk column of this thread (same for all its chunks)
    const int row0 = tid / CPR;  // first row; further rows are RS_ apart

    // ---- per-thread row bookkeeping (32-bit element offsets; the host checks they fit) ----
    int xoff[XCH];  // element offset of (image, ih0, iw0, c = 0); for invalid rows ih0 is far negative
    int ih0[XCH], iw0[XCH];
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
        int64_t m = static_cast<int64_t>(m0) + row0 + i * RS_;
        if (m < p.M) {
            int ow = static_cast<int>(m % p.OW);
            int64_t t = m / p.OW;
            int oh = static_cast<int>(t % p.OH);
            int img = static_cast<int>(t / p.OH);
            ih0[i] = oh * p.stride_h - p.pad_h;
            iw0[i] = ow * p.stride_w - p.pad_w;
            xoff[i] = static_cast<int>(img * p.xsN + ih0[i] * p.xsH + iw0[i] * p.xsW);
        } else {
            xoff[i] = 0;
            ih0[i] = -0x40000000;  // fails every bounds check
            iw0[i] = 0;
        }
    }
    int woff[WCH];
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
        int n = n0 + row0 + i * RS_;
        woff[i] = n < p.K ? static_cast<int>(n * p.wsK) : -1;
    }
    // LDS byte offsets of this thread's chunks inside a stage (swizzled)
    int xlds[XCH], wlds[WCH];
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
        int r = row0 + i * RS_;
        int slot16 = (kc * LB) / 16, sub = (kc * LB) % 16;
        xlds[i] = r * kRowBytes + SwzSlot(r, slot16) * 16 + sub;
    }
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
        int r = row0 + i * RS_;
        int slot16 = (kc * LB) / 16, sub = (kc * LB) % 16;
        wlds[i] = BM * kRowBytes + r * kRowBytes + SwzSlot(r, slot16) * 16 + sub;
    }

    const bool is_1x1 = (p.R == 1 && p.S == 1 && p.pad_h == 0 && p.pad_w == 0);
    const bool uniform_rs = (p.C % BKE) == 0;
    const int nk = (p.Kg + BKE - 1) / BKE;
    const int xsH = static_cast<int>(p.xsH), xsW = static_cast<int>(p.xsW);

    Chunk xreg[2][XCH], wreg[2][WCH];

    auto load_tile = [&](int kt, Chunk(&xr)[XCH], Chunk(&wr)[WCH]) {
        const int kk = kt * BKE + kc * EPC;
        const bool kvalid = kt < nk && kk < p.Kg;
        if (is_1x1) {
#pragma unroll
            for (int i = 0; i < XCH; ++i) {
                Chunk v = Chunk(0);
                if (kvalid && ih0[i] >= 0) v = *reinterpret_cast<const Chunk*>(p.x + xoff[i] + kk);
                xr[i] = v;
            }
        } else {
            int rs, c;
            if (uniform_rs) {
                int kbase = kt * BKE;
                rs = kbase / p.C;  // wave-uniform
                c = kbase - rs * p.C + kc * EPC;
            } else {
                rs = kk / p.C;
                c = kk - rs * p.C;
            }
            int r = rs / p.S;
            int s = rs - r * p.S;
            int delta = r * xsH + s * xsW + c;
#pragma unroll
            for (int i = 0; i < XCH; ++i) {
                int ih = ih0[i] + r;
                int iw = iw0[i] + s;
                bool ok = kvalid && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
                Chunk v = Chunk(0);
                if (ok) v = *reinterpret_cast<const Chunk*>(p.x + xoff[i] + delta);
                xr[i] = v;
            }
        }
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            Chunk v = Chunk(0);
            if (kvalid && woff[i] >= 0) v = *reinterpret_cast<const Chunk*>(p.w + woff[i] + kk);
            wr[i] = v;
        }
    };
    auto store_tile = [&](char* stage, const Chunk(&xr)[XCH], const Chunk(&wr)[WCH]) {
#pragma unroll
        for (int i = 0; i < XCH; ++i) *reinterpret_cast<Chunk*>(stage + xlds[i]) = xr[i];
#pragma unroll
        for (int i = 0; i < WCH; ++i) *reinterpret_cast<Chunk*>(stage + wlds[i]) = wr[i];
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

    // prologue: tile 0 -> regs[0] -> LDS[0]; tile 1 -> regs[1]
    load_tile(0, xreg[0], wreg[0]);
    load_tile(1, xreg[1], wreg[1]);
    store_tile(lds, xreg[0], wreg[0]);
    __syncthreads();

    // steady state, two K steps per trip so that the register set index is a compile-time constant
    for (int kt = 0; kt < nk; kt += 2) {
        // step kt: multiply LDS[0]; regs[0] <- tile kt+2; LDS[1] <- regs[1] (tile kt+1)
        load_tile(kt + 2, xreg[0], wreg[0]);
        ComputeTileSwz<T, PM>(lds, lds + BM * kRowBytes, wm, wn, lane, acc);
        store_tile(lds + STAGE, xreg[1], wreg[1]);
        __syncthreads();
        if (kt + 1 >= nk) break;
        // step kt+1: multiply LDS[1]; regs[1] <- tile kt+3; LDS[0] <- regs[0] (tile kt+2)
        load_tile(kt + 3, xreg[1], wreg[1]);
        ComputeTileSwz<T, PM>(lds + STAGE, lds + STAGE + BM * kRowBytes, wm, wn, lane, acc);
        store_tile(lds, xreg[0], wreg[0]);
        __syncthreads();
    }

    // ---- epilogue ----
    if (!p.out_wide) {
        if (PM) {
            StoreTilePM<T>(p, m0, n0, wm, wn, lane, acc);
        } else {
            StoreTile<T>(p, m0, n0, wm, wn, lane, acc);
        }
        return;
    }
    // Regroup through LDS.  Staging tile: PM -> [BN channels][BM pixels], else [BM pixels][BN channels]; rows padded by 16 bytes.
    constexpr int OUT_COLS = PM ? BM : BN;
    constexpr int OUT_ROWS = PM ? BN : BM;
    constexpr int OROW = OUT_COLS * static_cast<int>(sizeof(T)) + 16;
    const int lr = lane & 31;
    const int g = lane >> 5;
    struct alignas(sizeof(T) * 4) Out4 {
        T e[4];
    };
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            // PM: ti = pixel sub-tile, tj = channel sub-tile; lane column = channel, rows = pixels
            // else: ti = channel sub-tile, tj = pixel sub-tile; lane column = pixel, rows = channels
            int col_major_index = (PM ? wn : wm) * 64 + tj * 32 + lr;  // the index a lane owns alone
            float bias = 0.f;
            if (PM && p.bias != nullptr) {
                int n = n0 + col_major_index;
                if (n < p.K) bias = static_cast<float>(p.bias[n * p.bias_stride]);
            }
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                int run0 = (PM ? wm : wn) * 64 + ti * 32 + vq * 8 + g * 4;  // first of the 4 consecutive indices
                Out4 pack;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = acc[ti][tj][vq * 4 + e];
                    if (PM) {
                        v += bias;
                    } else if (p.bias != nullptr) {
                        int n = n0 + run0 + e;
                        if (n < p.K) v += static_cast<float>(p.bias[n * p.bias_stride]);
                    }
                    pack.e[e] = static_cast<T>(v);
                }
                *reinterpret_cast<Out4*>(lds + col_major_index * OROW + run0 * sizeof(T)) = pack;
            }
        }
    }
    __syncthreads();
    constexpr int EPV = 16 / sizeof(T);
    constexpr int CHUNKS_PER_ROW = OUT_COLS / EPV;
    constexpr int TOTAL_CHUNKS = OUT_ROWS * CHUNKS_PER_ROW;
    const int64_t ohw = static_cast<int64_t>(p.OH) * p.OW;
    for (int id = tid; id < TOTAL_CHUNKS; id += NT) {
        int row = id / CHUNKS_PER_ROW;
        int cc = id - row * CHUNKS_PER_ROW;
        Bytes16 v = *reinterpret_cast<const Bytes16*>(lds + row * OROW + cc * 16);
        if (PM) {
            int n = n0 + row;
            int64_t m = static_cast<int64_t>(m0) + cc * EPV;
            if (n < p.K && m < p.M) {  // M % EPV == 0 and OH*OW % EPV == 0: the run stays inside one image
                int64_t img = m / ohw;
                int64_t pix = m - img * ohw;
                *reinterpret_cast<Bytes16*>(p.out + img * p.osN + static_cast<int64_t>(n) * p.osC + pix) = v;
            }
        } else {
            int64_t m = static_cast<int64_t>(m0) + row;
            int n = n0 + cc * EPV;
            if (m < p.M && n < p.K) {  // K % EPV == 0
                int ow = static_cast<int>(m % p.OW);
                int64_t t = m / p.OW;
                int oh = static_cast<int>(t % p.OH);
                int64_t img = t / p.OH;
                *reinterpret_cast<Bytes16*>(p.out + img * p.osN + oh * p.osH + ow * p.osW + n) = v;
            }
        }
    }
}

// Dynamic LDS the kernel needs.
template <typename T, int WM, int WN, bool PM>
constexpr int PipeLdsBytes() {
    constexpr int BM = 64 * WM, BN = 64 * WN;
    constexpr int stage2 = 2 * (BM + BN) * kRowBytes;
    constexpr int out_cols = PM ? BM : BN;
    constexpr int out_rows = PM ? BN : BM;
    constexpr int staging = out_rows * (out_cols * static_cast<int>(sizeof(T)) + 16);
    return stage2 > staging ? stage2 : staging;
}

}  // namespace hipcx
