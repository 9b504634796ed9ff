// 1x1 convolution at stride 1 without padding for float16 activations that are C-contiguous NCHW on both sides:
//
//   out[n, k, p] = bias[k] + sum_c x[n, c, p] * w[k, c]          (p = pixel of the plane, P = H * W pixels per plane)
//
// i.e. per image the matrix product out_n [K, P] = w [K, C] . x_n [C, P] with the pixels contiguous in x and out.
//
// Work decomposition.  Pixels are numbered in "slots": image n owns slots [n * PS, n * PS + P) with PS = P rounded up to a
// multiple of 8, so that a 16-byte piece of 8 consecutive slots never straddles two images.  A workgroup of four wavefronts
// owns a tile of BM = 128 * WM slots x BN = 64 * WN output channels (WM * WN = 4; a wave multiplies 128 slots x 64 channels
// = 4 x 2 MFMA 32x32x16 blocks, 128 accumulator registers) and walks the input channels in chunks of 32.  Two workgroups run
// on a compute unit, each on tiles of its own: while one writes a tile out, the other one loads and multiplies.
//
// Operands reach LDS without passing through registers: buffer loads with the LDS modifier write 16 bytes per lane,
// 1 KiB per instruction, into a ring of two stages.
//   * activations stay as they lie in memory -- rows of pixels, one row per channel: stage[c][slot].  The MFMA operand (8
//     consecutive channels of one pixel per lane) is gathered by transposing LDS reads (ds_read_b64_tr_b16: sixteen lanes read
//     a 4-channel x 16-pixel block and each receives the four channels of its pixel).  16-byte piece i of channel row c is
//     stored at piece position i ^ (4 * (c & 3)): the four channel rows of such a block then fall into four different
//     64-byte bank groups (the loading lane picks the global piece that belongs at its LDS position).
//   * filters are read in place from the dense [K][C] bank: stage[k][4 pieces of 8 channels], piece g of row k at position
//     g ^ ((k >> 2) & 3), read as whole MFMA operands with ds_read_b128.
// Per chunk a wave issues its share of the loads of the next chunk, reads the fragments of the current chunk into
// registers, multiplies (16 MFMAs), waits for the loads of the next chunk and meets the others at one barrier.
// A workgroup walks several tiles (the host launches no more workgroups than the device holds): the chunk ring runs across
// tile boundaries, so the first chunks of the next tile are on their way while the current tile is written out.
// (An eight-wave variant -- one workgroup per compute unit on 256 x 256 or 512 x 128 tiles, its two groups of four waves
// alternating between a memory and an MFMA phase half a period apart -- measured 2 to 7 microseconds slower per layer: all of
// a tile's phases then run inside one workgroup.)
//
// Epilogue: accumulators (a lane holds 4 consecutive pixels of one channel) are rounded to float16 and regrouped through a
// wave-private LDS area into 16-byte pieces of 8 pixels, stored with buffer stores whose out-of-range offsets drop the
// pieces that do not exist (tile tails, padding slots): the number of store instructions is then the same for every wave and
// tile, which the in-order memory counter needs to tell loads that have landed from stores still in flight.
#pragma once

#include "common.h"
#include "igemm.h"
#include "nchw_conv.h"

namespace hipcx {

struct PwConvArgs {
    const half_t* x;
    const half_t* w;     // dense [K][C]
    const half_t* bias;  // may be null
    half_t* out;
    int N, C, K, P;
    int PS;  // slots per image
    int MS;  // N * PS
    int tiles_m, tiles_n, total_tiles;
    int64_t bias_stride;
    unsigned x_bytes, w_bytes, out_bytes;
    FastDiv div_PS;
};

typedef int pw_int4_t __attribute__((ext_vector_type(4)));

// Raw buffer descriptor (base, no stride, size in bytes, 32-bit untyped data) as four scalars.
__device__ __forceinline__ pw_int4_t PwRsrc(const void* ptr, unsigned bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(ptr);
    return pw_int4_t{__builtin_amdgcn_readfirstlane(static_cast<int>(a & 0xffffffffu)), __builtin_amdgcn_readfirstlane(static_cast<int>((a >> 32) & 0xffffu)),
                     __builtin_amdgcn_readfirstlane(static_cast<int>(bytes)), 0x00020000};
}
// 16 bytes per lane from global memory straight into LDS at lds_addr + lane * 16 (lds_addr wave-uniform).  Written as
// assembly on purpose: the compiler orders every later LDS read behind an LDS-writing load it knows of with a wait for all
// outstanding loads, which would serialise the ring; the kernel waits for exactly the loads it needs.
__device__ __forceinline__ void PwLdsLoad16(pw_int4_t rsrc, unsigned lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc),
                 "s"(__builtin_amdgcn_readfirstlane(soff))
                 : "memory", "m0");
}
// vmcnt <= N, nothing else waited for (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
template <int N>
__device__ __forceinline__ void PwWaitVmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

constexpr int kPwStagePitch = 136;                // bytes per channel row of the epilogue's staging area (64 pixels + 8)
constexpr int kPwStageBytes = 32 * kPwStagePitch;  // per wave: 32 channels x 64 pixels
constexpr int kPwStages = 2;  // a ring of three measured 1 us slower per layer: two workgroups per unit already keep loads in flight

constexpr int kPwMaxBiasK = 2048;                 // output channels whose bias values fit the LDS copy

// The ring, the epilogue's staging areas of the four waves and the bias copy: 69 KiB for 256 x 128 tiles, two workgroups to a unit.
template <int WM, int WN>
constexpr int PwLdsBytes() {
    return kPwStages * (32 * 128 * WM * 2 + 64 * WN * 64) + 4 * kPwStageBytes + kPwMaxBiasK * 2;
}

// PART: P is not a multiple of 8 (the last piece of a plane is incomplete and goes out as one 8-byte store; P % 4 == 0).
template <int WM, int WN, bool PART>
__global__ __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(2, 2)))
void PwConvKernel(PwConvArgs p) {
    constexpr int NW = WM * WN;
    static_assert(NW == 4, "four wavefronts");
    constexpr int BM = 128 * WM, BN = 64 * WN;
    constexpr int NSTAGE = kPwStages, AHEAD = NSTAGE - 1;
    static_assert(AHEAD == 1, "the wait below counts no younger chunk in flight");
    constexpr int ROWX = BM * 2;          // bytes per channel row of the activation tile
    constexpr int XT_B = 32 * ROWX;       // activation tile of one chunk
    constexpr int WT_B = BN * 64;         // filter tile of one chunk
    constexpr int STAGE_B = XT_B + WT_B;
    constexpr int LX = BM / (16 * NW), LW = BN / (16 * NW);  // load instructions per wave and chunk (1 KiB each)
    constexpr int LPC = LX + LW;
    constexpr int RING_B = NSTAGE * STAGE_B;
    constexpr int NST = PART ? 32 : 16;  // store instructions per wave and tile
    static_assert(NST < 64, "vmcnt range");
    extern __shared__ __align__(16) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int nc = p.C / 32;

    // ---- the tiles of this workgroup: XCD x (workgroup ids go round-robin to the 8 XCDs) walks a contiguous range of the tile
    // order, output channel tile fastest, so that the workgroups that share an activation tile run side by side on one L2 ----
    const int per_xcd = (p.total_tiles + 7) / 8;
    const int xcd = blockIdx.x & 7, bx = blockIdx.x >> 3, gx = gridDim.x >> 3;
    auto tile_at = [&](int i, int& tm, int& tn) -> bool {
        const int idx = bx + i * gx;
        if (idx >= per_xcd) return false;
        const int logical = xcd * per_xcd + idx;
        if (logical >= p.total_tiles) return false;
        tn = logical % p.tiles_n;
        tm = logical / p.tiles_n;
        return true;
    };

    // The bias vector goes to LDS once, before the first operand load is issued: a global load in the epilogue would make the
    // compiler wait for every outstanding memory operation, the next tile's operand loads and this tile's stores included.
    half_t* const bias_lds = reinterpret_cast<half_t*>(lds + RING_B + NW * kPwStageBytes);
    if (p.bias != nullptr) {
        for (int k = tid; k < p.K; k += 64 * NW) bias_lds[k] = p.bias[k * p.bias_stride];
    }

    const pw_int4_t xr = PwRsrc(p.x, p.x_bytes);
    const pw_int4_t wr = PwRsrc(p.w, p.w_bytes);
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));

    // ---- load cursor ----
    int l_i = 0, l_cb = 0;
    int l_tm = 0, l_tn = 0;
    bool l_valid = tile_at(0, l_tm, l_tn);
    int vox[LX], vow[LW];
    auto place_loads = [&]() {
#pragma unroll
        for (int i = 0; i < LX; ++i) {
            const int byte = (wave * LX + i) * 1024 + lane * 16;  // position inside the activation tile
            const int c = byte / ROWX;
            const int pl = (byte % ROWX) >> 4;
            const int pg = pl ^ (4 * (c & 3));
            const int slot = l_tm * BM + 8 * pg;
            const int n = p.div_PS(slot);
            const int q = slot - n * p.PS;
            vox[i] = (slot < p.MS && q < p.P) ? ((n * p.C + c) * p.P + q) * 2 : 0x7fffffff;
        }
#pragma unroll
        for (int i = 0; i < LW; ++i) {
            const int row = (wave * LW + i) * 16 + (lane >> 2);
            const int kg = (lane & 3) ^ ((lane >> 4) & 3);
            const int k = l_tn * BN + row;
            vow[i] = k < p.K ? k * p.C * 2 + kg * 16 : 0x7fffffff;
        }
    };
    if (l_valid) place_loads();
    int g_issue = 0;  // chunks issued so far
    auto issue_next = [&]() -> bool {  // issues the next chunk of the stream, if any
        if (!l_valid) return false;
        const unsigned st = lds_base + (g_issue % NSTAGE) * STAGE_B;
        const int xs = l_cb * 32 * p.P * 2;
#pragma unroll
        for (int i = 0; i < LX; ++i) PwLdsLoad16(xr, st + (wave * LX + i) * 1024, vox[i], xs);
#pragma unroll
        for (int i = 0; i < LW; ++i) PwLdsLoad16(wr, st + XT_B + (wave * LW + i) * 1024, vow[i], l_cb * 64);
        ++g_issue;
        if (++l_cb == nc) {
            l_cb = 0;
            ++l_i;
            l_valid = tile_at(l_i, l_tm, l_tn);
            if (l_valid) place_loads();
        }
        return true;
    };

    // ---- fragment addresses ----
    // activations: lane = 16 g + 4 q + s reads channel row 8 (g >> 1) + q (+ 4 for the second half, + 16 per reduction step),
    // pixels 16 (g & 1) + 4 s .. + 3 of a 32-pixel block, and receives pixel 16 (g & 1) + 4 q + s, channels 8 (g >> 1) ..
    const int fg = lane >> 4, fq = (lane >> 2) & 3, fs = lane & 3;
    unsigned xa[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int piece = 16 * wm + 4 * (i ^ fq) + 2 * (fg & 1) + (fs >> 1);
        xa[i] = lds_base + (8 * (fg >> 1) + fq) * ROWX + piece * 16 + (fs & 1) * 8;
    }
    const int fr = lane & 31, fh = lane >> 5;
    const unsigned wb0 = lds_base + XT_B + (wn * 64 + fr) * 64 + ((fh ^ ((fr >> 2) & 3)) * 16);

    float16_t acc[4][2];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    };
    zero_acc();

    Bytes8 xlo[2][4], xhi[2][4];
    Bytes16 wf[2][2];
    auto read_frags = [&](int stage) {
        const unsigned so = stage * STAGE_B;
        const unsigned a0 = xa[0] + so, a1 = xa[1] + so, a2 = xa[2] + so, a3 = xa[3] + so;
        const unsigned b0 = wb0 + so, b1 = b0 ^ 32;
        // immediates: + 4 rows for the upper channel half, + 16 rows for the second reduction step
        constexpr int HI = 4 * ROWX, T1 = 16 * ROWX;
        asm volatile(
            "ds_read_b64_tr_b16 %0, %20\n\t"
            "ds_read_b64_tr_b16 %1, %20 offset:%26\n\t"
            "ds_read_b64_tr_b16 %2, %21\n\t"
            "ds_read_b64_tr_b16 %3, %21 offset:%26\n\t"
            "ds_read_b64_tr_b16 %4, %22\n\t"
            "ds_read_b64_tr_b16 %5, %22 offset:%26\n\t"
            "ds_read_b64_tr_b16 %6, %23\n\t"
            "ds_read_b64_tr_b16 %7, %23 offset:%26\n\t"
            "ds_read_b128 %16, %24\n\t"
            "ds_read_b128 %17, %24 offset:2048\n\t"
            "ds_read_b64_tr_b16 %8, %20 offset:%27\n\t"
            "ds_read_b64_tr_b16 %9, %20 offset:%28\n\t"
            "ds_read_b64_tr_b16 %10, %21 offset:%27\n\t"
            "ds_read_b64_tr_b16 %11, %21 offset:%28\n\t"
            "ds_read_b64_tr_b16 %12, %22 offset:%27\n\t"
            "ds_read_b64_tr_b16 %13, %22 offset:%28\n\t"
            "ds_read_b64_tr_b16 %14, %23 offset:%27\n\t"
            "ds_read_b64_tr_b16 %15, %23 offset:%28\n\t"
            "ds_read_b128 %18, %25\n\t"
            "ds_read_b128 %19, %25 offset:2048\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(xlo[0][0]), "=&v"(xhi[0][0]), "=&v"(xlo[0][1]), "=&v"(xhi[0][1]), "=&v"(xlo[0][2]), "=&v"(xhi[0][2]), "=&v"(xlo[0][3]), "=&v"(xhi[0][3]),
              "=&v"(xlo[1][0]), "=&v"(xhi[1][0]), "=&v"(xlo[1][1]), "=&v"(xhi[1][1]), "=&v"(xlo[1][2]), "=&v"(xhi[1][2]), "=&v"(xlo[1][3]), "=&v"(xhi[1][3]),
              "=&v"(wf[0][0]), "=&v"(wf[0][1]), "=&v"(wf[1][0]), "=&v"(wf[1][1])
            : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1), "n"(HI), "n"(T1), "n"(T1 + HI)
            : "memory");
    };
    auto compute = [&]() {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const Bytes16 xf{xlo[t][i].x, xlo[t][i].y, xhi[t][i].x, xhi[t][i].y};
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, xf), __builtin_bit_cast(half8_t, wf[t][j]), acc[i][j], 0, 0, 0);
                }
    };

    // ---- epilogue of the tile (tm, tn) ----
    const __amdgpu_buffer_rsrc_t orsrc = MakeRsrc(p.out, p.out_bytes);
    char* const stg = lds + RING_B + wave * kPwStageBytes;
    auto epilogue = [&](int tm, int tn) {
        const int k0 = tn * BN + wn * 64;
        // output offsets of this lane's pieces: piece lane & 7 of the 64-pixel half ip
        int obase[2], nvalid[2];
#pragma unroll
        for (int ip = 0; ip < 2; ++ip) {
            const int slot = tm * BM + wm * 128 + ip * 64 + (lane & 7) * 8;
            const int n = p.div_PS(slot);
            const int q = slot - n * p.PS;
            nvalid[ip] = slot < p.MS ? p.P - q : 0;  // pixels of the piece that exist (>= 8: all)
            obase[ip] = ((n * p.K + k0 + (lane >> 3)) * p.P + q) * 2;
        }
        auto passes = [&](auto bias_tag) {
            constexpr bool BIAS = decltype(bias_tag)::value;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int kch = k0 + j * 32 + fr;
                float bias = 0.f;
                if constexpr (BIAS) bias = kch < p.K ? static_cast<float>(bias_lds[kch]) : 0.f;
#pragma unroll
                for (int ip = 0; ip < 2; ++ip) {
#pragma unroll
                    for (int ii = 0; ii < 2; ++ii) {
#pragma unroll
                        for (int qv = 0; qv < 4; ++qv) {
                            PVecH<4> pack;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                float v = acc[2 * ip + ii][j][4 * qv + e];
                                if constexpr (BIAS) v += bias;
                                pack.e[e] = static_cast<half_t>(v);
                            }
                            *reinterpret_cast<PVecH<4>*>(stg + fr * kPwStagePitch + (ii * 32 + 8 * qv + 4 * fh) * 2) = pack;
                        }
                    }
                    // the wave reads what its own lanes wrote: no barrier, the compiler's wait for the LDS writes suffices
#pragma unroll
                    for (int it = 0; it < 4; ++it) {
                        const int row = it * 8 + (lane >> 3);
                        const Bytes8 lo = *reinterpret_cast<const Bytes8*>(stg + row * kPwStagePitch + (lane & 7) * 16);
                        const Bytes8 hi = *reinterpret_cast<const Bytes8*>(stg + row * kPwStagePitch + (lane & 7) * 16 + 8);
                        const bool kok = k0 + j * 32 + row < p.K;
                        const int off = obase[ip] + (j * 32 + it * 8) * p.P * 2;
                        __builtin_amdgcn_raw_buffer_store_b128(Bytes16{lo.x, lo.y, hi.x, hi.y}, orsrc, (kok && nvalid[ip] >= 8) ? off : 0x7fffffff, 0, 0);
                        if constexpr (PART) {
                            __builtin_amdgcn_raw_buffer_store_b64(lo, orsrc, (kok && nvalid[ip] >= 4 && nvalid[ip] < 8) ? off : 0x7fffffff, 0, 0);
                        }
                    }
                }
            }
        };
        if (p.bias != nullptr) passes(std::true_type{}); else passes(std::false_type{});
    };

    // ---- the chunk stream ----
    int c_i = 0, c_cb = 0, c_tm = 0, c_tn = 0;
    bool c_valid = tile_at(0, c_tm, c_tn);
    if (!c_valid) return;  // the same for every wave of the workgroup
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) issue_next();
    // the first chunk has landed
    PwWaitVmcnt<0>();
    __builtin_amdgcn_s_barrier();
    int g = 0;
    // Per chunk: load the next chunk, read and multiply the current one, then wait for the next chunk and meet at one barrier.
    // The latency this leaves exposed is covered by the second workgroup on the compute unit.
    while (c_valid) {
        __builtin_amdgcn_sched_barrier(0);
        issue_next();  // chunk g + 1 into the stage chunk g - 1 was read from (everybody passed the barrier)
        read_frags(g % NSTAGE);
        compute();
        ++g;
        bool stored = false;
        if (++c_cb == nc) {
            c_cb = 0;
            ++c_i;
            const int e_tm = c_tm, e_tn = c_tn;
            c_valid = tile_at(c_i, c_tm, c_tn);
            epilogue(e_tm, e_tn);
            zero_acc();
            stored = true;
        }
        // the chunk issued above must have landed; the tile's stores, if any, were issued after it
        __builtin_amdgcn_sched_barrier(0);
        if (stored) PwWaitVmcnt<NST>(); else PwWaitVmcnt<0>();
        __builtin_amdgcn_s_barrier();
    }
}

}  // namespace hipcx
