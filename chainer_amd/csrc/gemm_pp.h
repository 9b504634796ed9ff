// float16 matrix product on the matrix pipes of gfx950 for large problems whose operands both have the reduction index as
// their unit-stride axis:
//
//   c[m][n] = sum_k a[m][k] * b[n][k]          (float accumulation, one rounding to float16)
//
// A workgroup of eight wavefronts owns a 256 x 256 tile of c and walks k in chunks of 32.  Operands reach LDS without passing
// through registers (buffer loads with the LDS modifier: 16 bytes per lane, 1 KiB per instruction) into a ring of three
// stages: stage[row][4 pieces of 8 halves], piece g of row r at position g ^ ((r >> 2) & 3) (the loading lane picks the
// global piece that belongs at its LDS position), so that the 16-byte fragment reads of consecutive rows use all banks.
// A wave multiplies 128 rows of a by 64 rows of b (4 x 2 MFMA 32x32x16 blocks, 128 accumulator registers).  The waves form
// two groups of four (one of each on every SIMD) that alternate between a memory phase (issue the loads of the chunk two
// ahead, read the 12 fragments of the current chunk) and an MFMA phase (16 MFMAs on registers), half a period apart and
// separated by workgroup barriers: while one wave of a SIMD multiplies, the other one feeds.
// Tiles are ordered so that the 32 workgroups an XCD runs at a time cover `band` tile rows x 32 / band tile columns: they
// share operand rows in that XCD's L2.
#pragma once

#include "common.h"
#include "igemm.h"
#include "nchw_conv.h"

namespace hipcx {
namespace gemm_pp {

typedef int int4_t __attribute__((ext_vector_type(4)));

struct GemmArgs {
    const half_t* a;
    const half_t* b;
    half_t* c;
    int M, N, K;
    int lda, ldb, ldc;  // elements
    int tiles_m, tiles_n;
    int band;  // tile rows per band of the tile order
};

// Raw buffer descriptor (base, no stride, size in bytes, 32-bit untyped data) as four scalars.
__device__ __forceinline__ int4_t RawRsrc(const void* ptr, unsigned bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(ptr);
    return int4_t{__builtin_amdgcn_readfirstlane(static_cast<int>(a & 0xffffffffu)), __builtin_amdgcn_readfirstlane(static_cast<int>((a >> 32) & 0xffffu)),
                  __builtin_amdgcn_readfirstlane(static_cast<int>(bytes)), 0x00020000};
}
// 16 bytes per lane from global memory straight into LDS at lds_addr + lane * 16 (lds_addr wave-uniform).  Written as
// assembly on purpose: the compiler orders every later LDS read behind an LDS-writing load it knows of with a wait for all
// outstanding loads, which would serialise the ring; the kernel waits for exactly the loads it needs.
__device__ __forceinline__ void LdsLoad16(int4_t rsrc, unsigned lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc),
                 "s"(__builtin_amdgcn_readfirstlane(soff))
                 : "memory", "m0");
}
// vmcnt <= N, nothing else waited for (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
template <int N>
__device__ __forceinline__ void WaitVmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

constexpr int kStages = 3;
constexpr int kLdsBytes = kStages * 2 * 256 * 64;
constexpr int kMinK = 32 * (kStages - 1);  // the pipeline's prologue issues kStages - 1 chunks

__global__ __launch_bounds__(512) void GemmPpKernel(GemmArgs p) {
    constexpr int NSTAGE = kStages, AHEAD = NSTAGE - 1;
    constexpr int TILE_B = 256 * 64;  // bytes of one operand tile in a stage
    constexpr int STAGE_B = 2 * TILE_B;
    constexpr int LPO = 2;            // load instructions per operand, wave and chunk
    constexpr int LPC = 2 * LPO;
    extern __shared__ __align__(16) char lds[];

    // ---- tile of this workgroup: XCD x (workgroup ids go round-robin to the 8 XCDs) walks a contiguous range of the tile
    // order; inside it bands of `band` tile rows are walked column by column ----
    const int total = p.tiles_m * p.tiles_n;
    const int per = (total + 7) / 8;
    const int logical = (static_cast<int>(blockIdx.x) % 8) * per + static_cast<int>(blockIdx.x) / 8;
    if (logical >= total) return;
    int tile_m, tile_n;
    {
        const int band_tiles = p.band * p.tiles_n;
        const int bi = logical / band_tiles;
        const int rem = logical - bi * band_tiles;
        const int rows = min(p.band, p.tiles_m - bi * p.band);
        tile_m = bi * p.band + rem % rows;
        tile_n = rem / rows;
    }
    const int m0 = tile_m * 256, n0 = tile_n * 256;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;
    const int wm = wave & 1, wn = wave >> 1;
    const int r = lane & 31, h = lane >> 5;

    // ---- global -> LDS loads: a wave instruction covers 16 rows x 64 bytes; lane = 4 * row + position ----
    const int4_t ra = RawRsrc(p.a + static_cast<int64_t>(m0) * p.lda, static_cast<unsigned>(min(p.M - m0, 256)) * static_cast<unsigned>(p.lda) * 2u);
    const int4_t rb = RawRsrc(p.b + static_cast<int64_t>(n0) * p.ldb, static_cast<unsigned>(min(p.N - n0, 256)) * static_cast<unsigned>(p.ldb) * 2u);
    int voa[LPO], vob[LPO];
#pragma unroll
    for (int i = 0; i < LPO; ++i) {
        const int row = (wave * LPO + i) * 16 + (lane >> 2);
        const int piece = (lane & 3) ^ ((lane >> 4) & 3);  // (row >> 2) & 3 = (lane >> 4) & 3
        voa[i] = (m0 + row < p.M) ? row * p.lda * 2 + piece * 16 : 0x7fffffff;  // beyond the buffer: zeros
        vob[i] = (n0 + row < p.N) ? row * p.ldb * 2 + piece * 16 : 0x7fffffff;
    }
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));
    auto issue = [&](int c) {
        const unsigned st = lds_base + (c % NSTAGE) * STAGE_B + wave * LPO * 1024;
        const int so = c * 64;
#pragma unroll
        for (int i = 0; i < LPO; ++i) LdsLoad16(ra, st + i * 1024, voa[i], so);
#pragma unroll
        for (int i = 0; i < LPO; ++i) LdsLoad16(rb, st + TILE_B + i * 1024, vob[i], so);
    };

    // ---- fragment addresses: rows of a are the MFMA column operand, rows of b the row operand, so that a lane ends up with
    // 4 consecutive n of one m: an 8-byte store into row-major c ----
    const int pos0 = h ^ ((r >> 2) & 3), pos1 = (2 + h) ^ ((r >> 2) & 3);
    const unsigned fa0 = lds_base + (wm * 128 + r) * 64 + pos0 * 16, fa1 = lds_base + (wm * 128 + r) * 64 + pos1 * 16;
    const unsigned fb0 = lds_base + TILE_B + (wn * 64 + r) * 64 + pos0 * 16, fb1 = lds_base + TILE_B + (wn * 64 + r) * 64 + pos1 * 16;

    float16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    Bytes16 fm[2][4], fn[2][2];
    // All twelve fragment reads of a chunk and the wait for them in one statement: nothing touches the registers before the
    // data has landed.
    auto read_frags = [&](int c) {
        const unsigned so = (c % NSTAGE) * STAGE_B;
        const unsigned a0 = fa0 + so, a1 = fa1 + so, b0 = fb0 + so, b1 = fb1 + so;
        asm volatile(
            "ds_read_b128 %0, %12\n\t"
            "ds_read_b128 %1, %12 offset:2048\n\t"
            "ds_read_b128 %2, %12 offset:4096\n\t"
            "ds_read_b128 %3, %12 offset:6144\n\t"
            "ds_read_b128 %4, %14\n\t"
            "ds_read_b128 %5, %14 offset:2048\n\t"
            "ds_read_b128 %6, %13\n\t"
            "ds_read_b128 %7, %13 offset:2048\n\t"
            "ds_read_b128 %8, %13 offset:4096\n\t"
            "ds_read_b128 %9, %13 offset:6144\n\t"
            "ds_read_b128 %10, %15\n\t"
            "ds_read_b128 %11, %15 offset:2048\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(fm[0][0]), "=&v"(fm[0][1]), "=&v"(fm[0][2]), "=&v"(fm[0][3]), "=&v"(fn[0][0]), "=&v"(fn[0][1]), "=&v"(fm[1][0]), "=&v"(fm[1][1]),
              "=&v"(fm[1][2]), "=&v"(fm[1][3]), "=&v"(fn[1][0]), "=&v"(fn[1][1])
            : "v"(a0), "v"(a1), "v"(b0), "v"(b1)
            : "memory");
    };
    auto compute = [&]() {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fn[t][j]), __builtin_bit_cast(half8_t, fm[t][i]), acc[i][j], 0, 0, 0);
    };

    // ---- pipeline (the host guarantees K % 32 == 0 and K / 32 >= AHEAD) ----
    const int nc = p.K / 32;
#pragma unroll
    for (int c = 0; c < AHEAD; ++c) issue(c);
    WaitVmcnt<(AHEAD - 1) * LPC>();  // this wave's share of chunk 0 has landed
    __builtin_amdgcn_s_barrier();
    if (grp == 1) __builtin_amdgcn_s_barrier();  // the second group runs half a period behind
    auto iteration = [&](int c, auto issue_tag, auto wait_tag) {
        constexpr bool ISSUE = decltype(issue_tag)::value;
        constexpr int WAIT = decltype(wait_tag)::value;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (ISSUE) issue(c + AHEAD);  // into the stage both groups finished reading a phase ago
        read_frags(c);
        WaitVmcnt<WAIT>();  // chunk c + 1 (this wave's share) must have landed before the barrier behind which it is read
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        compute();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    int c = 0;
    for (; c + AHEAD < nc; ++c) iteration(c, std::true_type{}, std::integral_constant<int, (AHEAD - 1) * LPC>{});
    // tail: nothing left to issue; with tt chunks behind c in flight, chunk c + 1 has landed when tt - 1 are outstanding
    StaticFor<0, AHEAD>([&](auto i_tag) {
        constexpr int tt = AHEAD - 1 - decltype(i_tag)::value;
        iteration(c, std::false_type{}, std::integral_constant<int, (tt >= 1 ? tt - 1 : 0) * LPC>{});
        ++c;
    });
    if (grp == 0) __builtin_amdgcn_s_barrier();

    // ---- epilogue: lane holds m = r, n = 8 * (v / 4) + 4 * h + v % 4 of each 32 x 32 block ----
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 128 + i * 32 + r;
        if (m >= p.M) continue;
        half_t* const crow = p.c + static_cast<int64_t>(m) * p.ldc;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * 64 + j * 32 + q * 8 + h * 4;
                if (n >= p.N) continue;  // N % 4 == 0: a group of four is inside or outside
                PVecH<4> o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o.e[e] = static_cast<half_t>(acc[i][j][q * 4 + e]);
                *reinterpret_cast<PVecH<4>*>(crow + n) = o;
            }
        }
    }
}
}  // namespace gemm_pp
}  // namespace hipcx
