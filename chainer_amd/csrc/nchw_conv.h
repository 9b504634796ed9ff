// Convolution forward for float16 activations that are C-contiguous NCHW on both sides -- the layout every
// ChainerX routine allocates -- without a layout-conversion pass.
//
//   out[n, k, oh, ow] = bias[k] + sum_{c, r, s} x[n, c, oh*stride - pad + r, ow*stride - pad + s] * w[k, c, r, s]
//
// Supported geometries: 1x1 (any stride, no padding) and 3x3 (stride 1, padding 1).
//
// Work decomposition.  Output pixels are flattened to m = (n*OH + oh)*OW + ow; a workgroup owns BM consecutive
// pixels x BN output channels and loops over the input channels in chunks of CK.  For every chunk
//   * the activations the tile needs (for 3x3: its rows plus one halo row above and below, all columns) are
//     loaded with buffer loads of NPX consecutive pixels from 8 channel planes, transposed in registers and written
//     to LDS as 16-byte groups of 8 channels per pixel: patch[channel group][slot] (slot = pixel position in a
//     zero-bordered patch whose rows are W+2 slots wide, with an all-zero row between images);
//   * the filters of the chunk arrive pre-packed ([C/8][R*S][K][8], see NchwRepackFilters) and are copied to LDS as
//     weights[channel group][tap][BN] 16-byte groups.
// Both LDS arrays are exactly the operand layout of v_mfma_f32_32x32x16_f16 (lane = row/column, 8 consecutive
// reduction indices per lane), so a fragment is one conflict-free ds_read_b128 of consecutive 16-byte groups, and
// a 3x3 tap is a constant slot offset into the same patch: the patch is written once and read nine times.
// Two LDS stages and a software pipeline laid out by hand: while chunk i is multiplied out of one stage, the registers that
// hold chunk i+1 are transposed and written to the other stage and refilled with chunk i+2, one such operation after each
// MFMA, and the operand fragments of the step after the next are read (three rotating fragment sets); one barrier per chunk.
// All addresses are computed once per workgroup; inside the channel loop only a scalar offset advances, and
// out-of-range loads are served as zeros by the buffer bounds check instead of branches.
//
// Accumulator orientation: pixels are MFMA rows, output channels MFMA columns, so a lane ends up with 4
// consecutive pixels of one channel -- an 8-byte store into NCHW memory.
#pragma once

#include "common.h"
#include "igemm.h"

namespace hipcx {

// Division of a non-negative int below 2^31 by a positive constant chosen on the host: q = (mulhi(n, mul) + n) >> shift.
struct FastDiv {
    unsigned mul = 1, shift = 0;
    FastDiv() = default;
    explicit FastDiv(int d) {
        unsigned l = 0;
        while ((1ull << l) < static_cast<unsigned long long>(d)) ++l;
        mul = static_cast<unsigned>(((1ull << 32) * ((1ull << l) - static_cast<unsigned long long>(d))) / static_cast<unsigned long long>(d)) + 1u;
        shift = l;
    }
    __device__ __forceinline__ int operator()(int n) const {
        return static_cast<int>((__umulhi(static_cast<unsigned>(n), mul) + static_cast<unsigned>(n)) >> shift);
    }
};

struct NchwConvArgs {
    const half_t* x;
    const half_t* wp;    // packed filters [C/8][taps][K][8]; or, with w_direct, the caller's dense [K][C] 1x1 filters
    const half_t* bias;  // may be null
    half_t* out;
    int N, C, H, W;  // input
    int K;           // output channels
    int OH, OW;      // output plane
    int stride;      // spatial stride (1x1 only; 3x3 runs with 1)
    int M;           // N*OH*OW
    int P;           // OH*OW
    int tiles_m, tiles_n;
    int nrow;   // 3x3: rows of the LDS patch (upper bound over tiles)
    int nslot;  // slots per channel group in the LDS patch
    int64_t bias_stride;
    unsigned x_bytes, wp_bytes;
    int w_direct;  // 1x1 only: read the filter bank in place (a row's 8 consecutive channels are one 16-byte group already)
    // Optional fused tail (all null / 0 for a plain convolution): fixed batch normalisation over the output channels,
    // a residual addend of out's shape (dense NCHW) and ReLU.
    const half_t* bn_gamma;
    const half_t* bn_beta;
    const half_t* bn_mean;
    const half_t* bn_var;
    int64_t bn_stride;  // element stride of the four parameter vectors
    float bn_eps;
    const half_t* residual;
    int relu;
    FastDiv div_P, div_W, div_OW, div_H2, div_wchunks, div_percg;  // by P, W, OW, H + 2, W / NPX, nrow * (W / NPX)
    int out_ev;   // pixels per output store: the largest of 8, 4, 2, 1 that divides P (a run then stays inside one image)
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t MakeRsrc(const void* ptr, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(ptr), 0, static_cast<int>(bytes), 0x00020000);
}

template <int N>
struct alignas(2 * N) PVecH {
    half_t e[N];
};
template <int N>
struct RawVec;
template <>
struct RawVec<8> {
    using type = Bytes16;
};
template <>
struct RawVec<4> {
    using type = Bytes8;
};
template <>
struct RawVec<2> {
    using type = unsigned;
};
template <>
struct RawVec<1> {
    using type = unsigned short;
};

// NPX pixels (NPX * 2 bytes) of one channel plane as dwords.
template <int NPX>
struct PixVec {
    static constexpr int DW = NPX >= 2 ? NPX / 2 : 1;
    unsigned d[DW];
};

template <int NPX>
__device__ __forceinline__ PixVec<NPX> BufLoad(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    PixVec<NPX> v;
    if constexpr (NPX == 8) {
        Bytes16 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
        v.d[0] = t.x;
        v.d[1] = t.y;
        v.d[2] = t.z;
        v.d[3] = t.w;
    } else if constexpr (NPX == 4) {
        Bytes8 t = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
        v.d[0] = t.x;
        v.d[1] = t.y;
    } else if constexpr (NPX == 2) {
        v.d[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
    } else {
        v.d[0] = __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0);  // zero-extended
    }
    return v;
}

// 8 channel planes x NPX pixels -> NPX groups of 8 channels (16 bytes each).
template <int NPX>
__device__ __forceinline__ void Transpose8(const PixVec<NPX> (&in)[8], Bytes16 (&out)[NPX]) {
#pragma unroll
    for (int e = 0; e < NPX; ++e) {
        unsigned dw[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            if constexpr (NPX == 1) {
                dw[d] = __builtin_amdgcn_perm(in[2 * d + 1].d[0], in[2 * d].d[0], 0x05040100u);  // low halves (the high ones may hold a neighbour)
            } else {
                unsigned a = in[2 * d].d[e / 2], b = in[2 * d + 1].d[e / 2];
                dw[d] = (e & 1) ? __builtin_amdgcn_perm(b, a, 0x07060302u) : __builtin_amdgcn_perm(b, a, 0x05040100u);
            }
        }
        out[e] = Bytes16{dw[0], dw[1], dw[2], dw[3]};
    }
}

template <int I, int N, typename F>
__device__ __forceinline__ void StaticFor(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        StaticFor<I + 1, N>(f);
    }
}

// Which instantiations walk several tiles per workgroup: the four-wave 1x1 kernels with two-pixel loads.  (The single-pixel and
// eight-wave variants have no registers to spare for the next tile's loads during the epilogue and measured slower.)
constexpr bool NchwWalksTiles(int taps, int waves, int npx, int ksplit) { return taps == 1 && ksplit == 1 && npx == 2 && waves == 4; }

// KSPLIT = 2: a second set of WPX * WCH waves works on the same tile and takes every other channel chunk through LDS stages of
// its own; the two accumulator sets are added through LDS before the epilogue.  For grids with at most one tile per compute unit
// (7x7 planes, small batches) this doubles the waves and the loads in flight per unit, which is what bounds those layers.
// PAIR (single-pixel loads only): every wanted pixel sits at an even element offset with a readable odd neighbour (stride 2, even
// width), so a pixel is fetched as a whole dword; a template parameter because a run-time choice would put a branch after every
// load of the hand-scheduled loop.
template <int TAPS, int WPX, int WCH, int CK, int NPX, int MAXI, int KSPLIT = 1, bool PAIR = false>
// Eight-wave workgroups that do not split the reduction are meant to run two to a compute unit (four waves per SIMD): they
// are kept within 128 registers.
__global__ __launch_bounds__(64 * WPX * WCH * KSPLIT) __attribute__((amdgpu_waves_per_eu(WPX * WCH >= 8 && KSPLIT == 1 ? 4 : (NchwWalksTiles(TAPS, WPX * WCH, NPX, KSPLIT) ? 3 : 1), 8)))
void NchwConvKernel(NchwConvArgs p) {
    constexpr int PW = 2, CW = 2;  // wave tile: 64 pixels x 64 channels
    constexpr int NT = 64 * WPX * WCH;       // threads of one reduction group
    constexpr int NT_ALL = NT * KSPLIT;
    constexpr int BM = 32 * PW * WPX;
    constexpr int BN = 32 * CW * WCH;
    constexpr int CG = CK / 8;    // 16-byte channel groups per chunk
    constexpr int KS = CK / 16;   // MFMA reduction steps per chunk and tap
    constexpr int WITEMS = TAPS * CG * BN;
    constexpr int WPT = (WITEMS + NT - 1) / NT;
    // bytes of one channel group's filters in LDS; the 1x1 layout is padded by 64 bytes so that lanes that differ in the
    // channel group (the order in which filters read in place are loaded) fall on different banks
    constexpr int WCGP = TAPS * BN * 16 + (TAPS == 1 ? 64 : 0);

    extern __shared__ __align__(16) char lds[];
    const int patch_bytes = CG * p.nslot * 16;
    const int stage_bytes = patch_bytes + CG * WCGP;
    const int dump_off = KSPLIT * 2 * stage_bytes;  // NPX * 16 bytes that absorb the writes of idle load slots

    // Some 1x1 kernels (NchwWalksTiles) walk several tiles per workgroup when the grid is smaller than the tile count (the
    // host launches as many workgroups as fit on the chip at once): the first loads of the next tile are issued before the
    // current tile is written out, so that their latency and the tile's set-up hide behind the epilogue.
    constexpr bool kWalk = NchwWalksTiles(TAPS, WPX * WCH, NPX, KSPLIT);
    int vblock = blockIdx.x;  // the virtual workgroup index of the current tile
    int tile_m, tile_n;
    if (!TileOf(p.tiles_m, p.tiles_n, vblock, tile_m, tile_n)) return;
    int m0 = tile_m * BM;
    int n0 = tile_n * BN;
    const int tid_all = threadIdx.x;
    const int kg = KSPLIT > 1 ? __builtin_amdgcn_readfirstlane(tid_all / NT) : 0;  // reduction group of this wave
    const int tid = tid_all - kg * NT;                                             // thread index inside the group
    char* const glds = lds + kg * 2 * stage_bytes;                                 // the group's two stages
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wpx = wave % WPX;
    const int wch = wave / WPX;
    const int lr = lane & 31;
    const int g = lane >> 5;
    const int HW = p.H * p.W;
    const int W2 = p.W + 2;

    // ---- patch geometry (3x3): first patch row of this tile in "padded row" coordinates n*(H+2) + h + 1 ----
    int base_row = 0, last_row = 0;
    if constexpr (TAPS == 9) {
        int m_last = min(m0 + BM, p.M) - 1;
        int nf = p.div_P(m0), hf = p.div_W(m0 - nf * p.P);
        int nl = p.div_P(m_last), hl = p.div_W(m_last - nl * p.P);
        base_row = nf * (p.H + 2) + hf;          // one above the first output row
        last_row = nl * (p.H + 2) + hl + 2;      // one below the last output row
    }

    // ---- activation load slots of this thread ----
    int xvoff[MAXI];  // byte offset of (n, channel group base, first pixel) in x; out of range for idle slots
    int xlds[MAXI];   // byte offset of the first pixel's group inside a stage
    // Two-pixel loads of the 1x1 kernels: a lane's two 16-byte groups are neighbours, so the lanes of a wave write with a stride
    // of 32 bytes and would use only half of the LDS banks.  Every other run of 8 lanes therefore stores its two groups in
    // swapped order (slot s lives at s ^ ((s >> 4) & 1)); the fragment reads below apply the same exchange.
    constexpr bool kSwapPairs = TAPS == 1 && NPX == 2;
    int xflip[MAXI];  // 16 where the two groups are swapped, else 0
    auto place_x_slots = [&](int m_first) {
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
        int it = tid + i * NT;
        bool valid;
        int voff = 0, loff = 0;
        if constexpr (TAPS == 9) {
            const int wchunks = p.W / NPX;
            const int per_cg = p.nrow * wchunks;
            int cg = p.div_percg(it);
            int q = it - cg * per_cg;
            int pr = p.div_wchunks(q);
            int wc = q - pr * wchunks;
            int grow = base_row + pr;
            int n = p.div_H2(grow);
            int hh = grow - n * (p.H + 2) - 1;
            valid = cg < CG && grow <= last_row && n < p.N && hh >= 0 && hh < p.H;
            voff = (((n * p.C + cg * 8) * p.H + hh) * p.W + wc * NPX) * 2;
            loff = (cg * p.nslot + pr * W2 + wc * NPX + 1) * 16;
            xflip[i] = 0;
        } else {
            constexpr int per_cg = BM / NPX;
            int cg = it / per_cg;
            int q = it - cg * per_cg;
            int m = m_first + q * NPX;
            valid = cg < CG && m < p.M;
            int n = p.div_P(m);
            int pix = m - n * p.P;
            int oh = p.div_OW(pix);
            int ow = pix - oh * p.OW;
            voff = (((n * p.C + cg * 8) * p.H + oh * p.stride) * p.W + ow * p.stride) * 2;
            loff = (cg * p.nslot + q * NPX) * 16;
            xflip[i] = kSwapPairs ? ((q >> 3) & 1) * 16 : 0;
        }
        xvoff[i] = valid ? voff : 0x7fffffff;  // beyond the buffer: the load returns zeros
        xlds[i] = valid ? loff : -1;           // idle slots write into the dump area
    }
    };
    place_x_slots(m0);
    // ---- filter load slots ----
    int wvoff[WPT];
    int wlds[WPT];
    auto place_w_slots = [&](int n_first) {
#pragma unroll
    for (int i = 0; i < WPT; ++i) {
        int wi = tid + i * NT;
        int cg, tap, kl;
        if (TAPS == 1 && p.w_direct) {  // consecutive lanes walk a filter row: 64 contiguous bytes per row and chunk
            kl = wi / CG;
            cg = wi - kl * CG;
            tap = 0;
        } else {  // packed filters: consecutive lanes walk the output channels of one (group, tap)
            cg = wi / (TAPS * BN);
            int rest = wi - cg * (TAPS * BN);
            tap = rest / BN;
            kl = rest - tap * BN;
        }
        bool valid = wi < WITEMS && n_first + kl < p.K;
        if (TAPS == 1 && p.w_direct) {
            wvoff[i] = valid ? ((n_first + kl) * p.C + cg * 8) * 2 : 0x7fffffff;
        } else {
            wvoff[i] = valid ? ((cg * TAPS + tap) * p.K + n_first + kl) * 16 : 0x7fffffff;
        }
        wlds[i] = wi < WITEMS ? patch_bytes + cg * WCGP + (tap * BN + kl) * 16 : -1;
    }
    };
    place_w_slots(n0);

    const __amdgpu_buffer_rsrc_t xr = MakeRsrc(p.x, p.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = MakeRsrc(p.wp, p.wp_bytes);

    PixVec<NPX> xreg[MAXI][8];
    Bytes16 wreg[WPT];
    // Side work of one loop iteration, cut into single operations that the loop deals out between its MFMAs:
    //   activation slot i: one operation that transposes the registers loaded an iteration ago and writes them to LDS,
    //                      then eight operations that each load one channel plane of the chunk after the next;
    //   filter slot i:     one LDS write, one load.
    constexpr int XOPS = MAXI * 9;
    constexpr int NOPS = XOPS + WPT * 2;
    int xs_next = 0, ws_next = 0;  // scalar offsets of the chunk being loaded
    auto side = [&](auto op_tag, char* stage) {
        constexpr int op = decltype(op_tag)::value;
        if constexpr (op < XOPS) {
            constexpr int i = op / 9, r = op % 9;
            if constexpr (r == 0) {
                Bytes16 t[NPX];
                Transpose8<NPX>(xreg[i], t);
                char* dst = xlds[i] >= 0 ? stage + xlds[i] : lds + dump_off;
#pragma unroll
                for (int e = 0; e < NPX; ++e) *reinterpret_cast<Bytes16*>(dst + (kSwapPairs ? (e * 16) ^ xflip[i] : e * 16)) = t[e];
            } else {
                constexpr int j = r - 1;
                if constexpr (NPX == 1 && PAIR) {
                    xreg[i][j].d[0] = __builtin_amdgcn_raw_buffer_load_b32(xr, xvoff[i], xs_next + j * HW * 2, 0);
                } else {
                    xreg[i][j] = BufLoad<NPX>(xr, xvoff[i], xs_next + j * HW * 2);
                }
            }
        } else {
            constexpr int q = op - XOPS, i = q / 2;
            if constexpr (q % 2 == 0) {
                char* dst = wlds[i] >= 0 ? stage + wlds[i] : lds + dump_off;
                *reinterpret_cast<Bytes16*>(dst) = wreg[i];
            } else {
                wreg[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, wvoff[i], ws_next, 0);
            }
        }
    };
    auto set_chunk = [&](int gi) {  // gi: chunk number inside this group; the groups interleave chunks
        const int ci = gi * KSPLIT + kg;
        xs_next = ci * CK * HW * 2;
        ws_next = (TAPS == 1 && p.w_direct) ? ci * CK * 2 : ci * (CG * TAPS) * p.K * 16;
    };
    auto load_all = [&]() {
        StaticFor<0, NOPS>([&](auto t) {
            constexpr int op = decltype(t)::value;
            if constexpr ((op < XOPS && op % 9 != 0) || (op >= XOPS && (op - XOPS) % 2 == 1)) side(t, lds);
        });
    };
    auto store_all = [&](char* stage) {
        StaticFor<0, NOPS>([&](auto t) {
            constexpr int op = decltype(t)::value;
            if constexpr ((op < XOPS && op % 9 == 0) || (op >= XOPS && (op - XOPS) % 2 == 0)) side(t, stage);
        });
    };

    // ---- fragment addresses ----
    int aoff[PW];  // byte offset of this lane's pixel group (channel group g) inside a stage, tap (0,0) of a 3x3 = slot - W2 - 1
#pragma unroll
    for (int a = 0; a < PW; ++a) {
        int m = m0 + (wpx * PW + a) * 32 + lr;
        int slot;
        if constexpr (TAPS == 9) {
            int mm = m < p.M ? m : p.M - 1;
            int n = p.div_P(mm);
            int pix = mm - n * p.P;
            int h = p.div_W(pix);
            int w = pix - h * p.W;
            slot = (n * (p.H + 2) + h + 1 - base_row) * W2 + w + 1;
            slot -= W2 + 1;  // tap (r, s) adds r * W2 + s
        } else {
            slot = (wpx * PW + a) * 32 + lr;
            if constexpr (kSwapPairs) slot ^= (slot >> 4) & 1;
        }
        aoff[a] = (g * p.nslot + slot) * 16;
    }
    const int boff = patch_bytes + g * WCGP + (wch * CW * 32 + lr) * 16;
    const int a_ks = 2 * p.nslot * 16;  // advance of one 16-channel reduction step in the patch

    float16_t acc[PW][CW];
#pragma unroll
    for (int a = 0; a < PW; ++a) {
#pragma unroll
        for (int b = 0; b < CW; ++b) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
        }
    }

    // One loop iteration: chunk ci is multiplied out of `cur` while the registers that hold chunk ci+1 go to `nxt` and are
    // refilled with chunk ci+2.  The instruction stream is laid out by hand (every sched_barrier pins what precedes it):
    // after each MFMA one fragment read of the step after the next (fragments live in three rotating register sets, so a
    // read has two steps = 8 MFMAs to land) and this slot's share of the side operations.  The matrix pipe never waits for
    // the load path: LDS writes and buffer loads issue in the shadow of the MFMAs.
    constexpr int NSTEP = TAPS * KS;
    constexpr int NSLOT = NSTEP * PW * CW;
    Bytes16 af[3][PW], bf[3][CW];
    auto read_frag = [&](const char* stage, auto st_tag, auto q_tag) {
        constexpr int st = decltype(st_tag)::value, q = decltype(q_tag)::value;
        constexpr int tap = st / KS, ks = st % KS;
        const int toff = TAPS == 9 ? ((tap / 3) * W2 + (tap % 3)) * 16 : 0;
        if constexpr (q < PW) {
            af[st % 3][q] = *reinterpret_cast<const Bytes16*>(stage + aoff[q] + toff + ks * a_ks);
        } else {
            constexpr int b = q - PW;
            bf[st % 3][b] = *reinterpret_cast<const Bytes16*>(stage + boff + ks * 2 * WCGP + (tap * BN + b * 32) * 16);
        }
    };
    auto iteration = [&](const char* cur, char* nxt, auto stores_tag, auto loads_tag) {
        constexpr bool STORES = decltype(stores_tag)::value, LOADS = decltype(loads_tag)::value;
        StaticFor<0, (NSTEP < 2 ? NSTEP : 2)>([&](auto st) { StaticFor<0, PW + CW>([&](auto q) { read_frag(cur, st, q); }); });
        __builtin_amdgcn_sched_barrier(0);
        StaticFor<0, NSTEP>([&](auto st_tag) {
            constexpr int st = decltype(st_tag)::value;
            StaticFor<0, PW * CW>([&](auto q_tag) {
                constexpr int q = decltype(q_tag)::value;
                constexpr int a = q / CW, b = q % CW;
                constexpr int slot = st * PW * CW + q;
                MfmaTile<half_t>(af[st % 3][a], bf[st % 3][b], acc[a][b]);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (st + 2 < NSTEP) {  // PW + CW reads over PW * CW slots
                    StaticFor<q * (PW + CW) / (PW * CW), (q + 1) * (PW + CW) / (PW * CW)>(
                            [&](auto f) { read_frag(cur, std::integral_constant<int, st + 2>{}, f); });
                }
                StaticFor<slot * NOPS / NSLOT, (slot + 1) * NOPS / NSLOT>([&](auto op_tag) {
                    constexpr int op = decltype(op_tag)::value;
                    constexpr bool is_load = (op < XOPS && op % 9 != 0) || (op >= XOPS && (op - XOPS) % 2 == 1);
                    if constexpr (is_load ? LOADS : STORES) side(op_tag, nxt);
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };

    // ---- pipeline ----
    // Stage (ci & 1) holds chunk ci.  Loads run two chunks ahead of the multiplication, through registers.  The last two
    // iterations are compiled without the loads (and the last one without the LDS writes) they would have no use for.
    const int nchunks = p.C / CK / KSPLIT;  // per group; the host only picks KSPLIT when it divides the chunk count
    using True = std::integral_constant<bool, true>;
    using False = std::integral_constant<bool, false>;
    set_chunk(0);
    load_all();
    if constexpr (TAPS == 9) {  // borders of all patches must read as zero; nothing ever writes them
        for (int off = tid_all * 16; off < KSPLIT * 2 * stage_bytes; off += NT_ALL * 16) *reinterpret_cast<Bytes16*>(lds + off) = Bytes16(0);
        __syncthreads();
    }
    for (;;) {  // one pass per tile; a single pass unless this workgroup walks several tiles
    store_all(glds);
    if (nchunks > 1) {
        set_chunk(1);
        load_all();
    }
    __syncthreads();
    int ci = 0;
    for (; ci + 2 < nchunks; ++ci) {
        set_chunk(ci + 2);
        iteration(glds + (ci & 1) * stage_bytes, glds + ((ci + 1) & 1) * stage_bytes, True{}, True{});
        __syncthreads();
    }
    if (ci + 1 < nchunks) {
        iteration(glds + (ci & 1) * stage_bytes, glds + ((ci + 1) & 1) * stage_bytes, True{}, False{});
        __syncthreads();
        ++ci;
    }
    iteration(glds + (ci & 1) * stage_bytes, glds + ((ci + 1) & 1) * stage_bytes, False{}, False{});
    __syncthreads();

    // ---- the second group hands its sums over (the loop's last barrier has retired every stage read) ----
    if constexpr (KSPLIT > 1) {
        float* red = reinterpret_cast<float*>(lds);  // [PW * CW * 16][NT]: consecutive lanes, consecutive words
        if (kg == 1) {
#pragma unroll
            for (int a = 0; a < PW; ++a) {
#pragma unroll
                for (int b = 0; b < CW; ++b) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) red[((a * CW + b) * 16 + v) * NT + tid] = acc[a][b][v];
                }
            }
        }
        __syncthreads();
        if (kg == 0) {
#pragma unroll
            for (int a = 0; a < PW; ++a) {
#pragma unroll
                for (int b = 0; b < CW; ++b) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[a][b][v] += red[((a * CW + b) * 16 + v) * NT + tid];
                }
            }
        }
        __syncthreads();  // the staging tile below reuses this memory
    }

    // ---- the next tile of this workgroup: its load slots, and its first chunk on the way before this tile is written out ----
    bool more = false;
    int m0_next = 0, n0_next = 0;
    if constexpr (kWalk) {
        vblock += static_cast<int>(gridDim.x);
        int tm, tn;
        more = TileOf(p.tiles_m, p.tiles_n, vblock, tm, tn);
        if (more) {
            m0_next = tm * BM;
            n0_next = tn * BN;
            place_x_slots(m0_next);
            place_w_slots(n0_next);
            set_chunk(0);
            load_all();
        }
    }

    // ---- epilogue ----
    // A lane holds channel column lr of each 32-wide sub-tile and pixel rows 8*(v/4) + 4*g + v%4.  The tile is
    // regrouped through LDS as [channel][pixel] (the last barrier of the loop has retired every stage read), so that
    // consecutive lanes store consecutive pixel runs of one channel plane: whole cache lines per instruction.
    constexpr int OPITCH = BM * 2 + 16;  // bytes per channel row
    // The fused tail is compiled as separate straight-line variants (no per-element branches in the plain convolution).
    auto stage_tile = [&](auto bn_tag, auto relu_tag) {
        constexpr bool BN = decltype(bn_tag)::value;
        constexpr bool RELU = decltype(relu_tag)::value;
#pragma unroll
        for (int b = 0; b < CW; ++b) {
            const int row = (wch * CW + b) * 32 + lr;
            const int n = n0 + row;
            float bias = (p.bias != nullptr && n < p.K) ? static_cast<float>(p.bias[n * p.bias_stride]) : 0.f;
            // batch norm in the reference's association order, ((v - mean) * inv_std) * gamma + beta, evaluated in float
            float bn_mean = 0.f, bn_inv = 1.f, bn_gamma = 1.f, bn_beta = 0.f;
            if (BN && n < p.K) {
                bn_mean = static_cast<float>(p.bn_mean[n * p.bn_stride]);
                bn_inv = 1.0f / sqrtf(static_cast<float>(p.bn_var[n * p.bn_stride]) + p.bn_eps);
                bn_gamma = static_cast<float>(p.bn_gamma[n * p.bn_stride]);
                bn_beta = static_cast<float>(p.bn_beta[n * p.bn_stride]);
            }
#pragma unroll
            for (int a = 0; a < PW; ++a) {
#pragma unroll
                for (int vq = 0; vq < 4; ++vq) {
                    const int col = (wpx * PW + a) * 32 + vq * 8 + g * 4;
                    PVecH<4> pack;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = acc[a][b][vq * 4 + e] + bias;
                        if (BN) v = ((v - bn_mean) * bn_inv) * bn_gamma + bn_beta;
                        if (RELU) v = v < 0.f ? 0.f : v;  // NaN < 0 is false: NaN passes, like IfLessElse(x, 0, 0, x)
                        pack.e[e] = static_cast<half_t>(v);
                    }
                    *reinterpret_cast<PVecH<4>*>(lds + row * OPITCH + col * 2) = pack;
                }
            }
        }
    };
    const bool has_bn = p.bn_gamma != nullptr;
    const bool relu_here = p.relu && p.residual == nullptr;  // with a residual, ReLU follows the addition
    if (kg == 0) {
        if (has_bn) {
            if (relu_here) stage_tile(True{}, True{});
            else stage_tile(True{}, False{});
        } else {
            if (relu_here) stage_tile(False{}, True{});
            else stage_tile(False{}, False{});
        }
    }
    __syncthreads();
    auto store_rows = [&](auto ev_tag, auto res_tag) {
        constexpr int EV = decltype(ev_tag)::value;  // pixels per store
        constexpr bool RES = decltype(res_tag)::value;
        constexpr int CPR = BM / EV;                 // chunks per channel row
        static_assert(NT_ALL % CPR == 0 || CPR % NT_ALL == 0, "a thread keeps one pixel column");
        constexpr int COLS_PER_THREAD = CPR > NT_ALL ? CPR / NT_ALL : 1;
        constexpr int ROW_STEP = CPR > NT_ALL ? 1 : NT_ALL / CPR;
        using Raw = typename RawVec<EV>::type;  // one LDS read and one global store of EV * 2 bytes
#pragma unroll
        for (int cj = 0; cj < COLS_PER_THREAD; ++cj) {
            const int cc = (tid_all % (CPR > NT_ALL ? NT_ALL : CPR)) + cj * NT_ALL;
            const int m = m0 + cc * EV;
            if (m >= p.M) continue;
            const int img = p.div_P(m);
            const int pix = m - img * p.P;
            const int64_t obase = static_cast<int64_t>(img) * p.K * p.P + pix;
            for (int row = (CPR > NT_ALL ? 0 : tid_all / CPR); row < BN; row += ROW_STEP) {
                const int n = n0 + row;
                if (n >= p.K) break;
                const int64_t o = obase + static_cast<int64_t>(n) * p.P;
                Raw raw = *reinterpret_cast<const Raw*>(lds + row * OPITCH + cc * EV * 2);
                if constexpr (RES) {  // y = relu(bn(conv) + residual): the addend is read with the same coalesced runs
                    PVecH<EV> v = __builtin_bit_cast(PVecH<EV>, raw);
                    PVecH<EV> r = __builtin_bit_cast(PVecH<EV>, *reinterpret_cast<const Raw*>(p.residual + o));
#pragma unroll
                    for (int e = 0; e < EV; ++e) {
                        float t = static_cast<float>(v.e[e]) + static_cast<float>(r.e[e]);
                        if (p.relu) t = t < 0.f ? 0.f : t;
                        v.e[e] = static_cast<half_t>(t);
                    }
                    raw = __builtin_bit_cast(Raw, v);
                }
                *reinterpret_cast<Raw*>(p.out + o) = raw;
            }
        }
    };
    // EV consecutive pixels never straddle an image and are EV*2-byte aligned when P % EV == 0 (m0 % EV == 0 always)
    auto store_ev = [&](auto ev_tag) {
        if (p.residual != nullptr) store_rows(ev_tag, True{});
        else store_rows(ev_tag, False{});
    };
    switch (p.out_ev) {
        case 8: store_ev(std::integral_constant<int, 8>{}); break;
        case 4: store_ev(std::integral_constant<int, 4>{}); break;
        case 2: store_ev(std::integral_constant<int, 2>{}); break;
        default: store_ev(std::integral_constant<int, 1>{}); break;
    }
    if (!more) break;  // the same for every thread of the workgroup
    __syncthreads();   // the output tile has left LDS before the next tile's operands are written there
    m0 = m0_next;
    n0 = n0_next;
#pragma unroll
    for (int a = 0; a < PW; ++a) {
#pragma unroll
        for (int b = 0; b < CW; ++b) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
        }
    }
    }
}

// w[K][C][R][S] (element strides wsK, wsC, wsR, wsS) -> wp[C/8][R*S][K][8].
__global__ __launch_bounds__(256) void NchwRepackFiltersKernel(const half_t* w, half_t* wp, int K, int C, int RS, int S, int64_t wsK,
                                                               int64_t wsC, int64_t wsR, int64_t wsS) {
    int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;  // one 16-byte group each
    int64_t total = static_cast<int64_t>(C / 8) * RS * K;
    if (idx >= total) return;
    int k = static_cast<int>(idx % K);
    int64_t t = idx / K;
    int tap = static_cast<int>(t % RS);
    int cg = static_cast<int>(t / RS);
    int r = tap / S, s = tap - r * S;
    struct alignas(16) G {
        half_t e[8];
    } grp;
#pragma unroll
    for (int j = 0; j < 8; ++j) grp.e[j] = w[k * wsK + (cg * 8 + j) * wsC + r * wsR + s * wsS];
    *reinterpret_cast<G*>(wp + idx * 8) = grp;
}

}  // namespace hipcx
