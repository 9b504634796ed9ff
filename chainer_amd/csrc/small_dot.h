// Matrix product for small outputs (batch-sized Linear layers: 100-128 rows, K up to a few thousand):
// out[M,N] = a[M,K] . b[K,N] with M*N so small that 128x128 tiles would occupy a handful of CUs.
//
// A workgroup owns one 32x32 tile of `out`; its 8 waves split the reduction axis, each feeding the MFMA straight
// from global memory (operands this small live in L2; no LDS staging), and the 8 partial tiles are summed through
// LDS.  For float the reduction index is dealt to the v_mfma_f32_32x32x2_f32 steps so that a lane's four steps use
// four consecutive k (one 16-byte load when k is the contiguous axis of the operand, which is the case for
// Linear's x and W^T view); for float16 a lane's v_mfma_f32_32x32x16_f16 operand is 8 consecutive k.
// Rows / columns beyond M / N and the tail of K are served as zeros by the buffer bounds check or explicit masks.
#pragma once

#include "nchw_conv.h"

namespace hipcx {

struct SmallDotArgs {
    const void* a;
    const void* b;
    void* out;
    int M, N, K;
    int64_t a_row, a_k;  // element strides of a along m and k
    int64_t b_k, b_col;  // element strides of b along k and n
    int64_t o_row, o_col;
    unsigned a_bytes, b_bytes;  // spans, for the buffer descriptors
    int a_vec, b_vec;           // k is the unit-stride axis of the operand and 16-byte runs are dword aligned
    int tiles_n;
    int nw;  // SmallDotRowsKernel: waves per workgroup = ways the reduction axis is split
};

// Workgroups are dealt to the 8 XCDs round-robin, and each XCD has its own L2: give every XCD one contiguous range of
// tiles, row tiles fastest, so that the workgroups sharing a slice of b (the weights) share an L2 and the whole of b is
// fetched into the L2s once instead of once per XCD.
__device__ __forceinline__ void SmallDotTile(int tiles_m, int& tm, int& tn) {
    const int nblk = gridDim.x;
    const int bid = blockIdx.x;
    const int xcd = bid & 7, loc = bid >> 3;
    const int q = nblk >> 3, r = nblk & 7;
    const int tile = xcd * q + min(xcd, r) + loc;
    tn = tile / tiles_m;
    tm = tile - tn * tiles_m;
}

template <typename T>
struct SmallDotTraits;
template <>
struct SmallDotTraits<float> {
    static constexpr int KG = 8;  // k values one "group step" of a wave consumes (4 MFMAs x 2)
    static constexpr int PER_LANE = 4;
    static constexpr int STEPS_IN_FLIGHT = 3;  // per register stage (two stages)
};
template <>
struct SmallDotTraits<half_t> {
    static constexpr int KG = 16;  // one MFMA
    static constexpr int PER_LANE = 8;
    static constexpr int STEPS_IN_FLIGHT = 2;  // per register stage (two stages)
};

// PER_LANE consecutive-k elements of one operand row/column as raw dwords; `contig`: k is the unit-stride axis.
template <typename T>
__device__ __forceinline__ Bytes16 LoadRun(__amdgpu_buffer_rsrc_t r, const T* base, int64_t line_off, int64_t kstride, int k, int kend, bool line_ok,
                                           bool contig) {
    constexpr int PL = SmallDotTraits<T>::PER_LANE;
    Bytes16 v = Bytes16(0);
    if (!line_ok) return v;
    if (contig && k + PL <= kend) {
        return __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>((line_off + k) * static_cast<int64_t>(sizeof(T))), 0, 0);
    }
    T e[PL];
#pragma unroll
    for (int i = 0; i < PL; ++i) e[i] = (k + i < kend) ? base[line_off + (k + i) * kstride] : T(0);
    if constexpr (sizeof(T) == 4) {
        v.x = __builtin_bit_cast(unsigned, e[0]);
        v.y = __builtin_bit_cast(unsigned, e[1]);
        v.z = __builtin_bit_cast(unsigned, e[2]);
        v.w = __builtin_bit_cast(unsigned, e[3]);
    } else {
        auto pk = [](T lo, T hi) {
            return static_cast<unsigned>(__builtin_bit_cast(unsigned short, lo)) | (static_cast<unsigned>(__builtin_bit_cast(unsigned short, hi)) << 16);
        };
        v.x = pk(e[0], e[1]);
        v.y = pk(e[2], e[3]);
        v.z = pk(e[4], e[5]);
        v.w = pk(e[6], e[7]);
    }
    return v;
}

// The same run when k is the unit-stride axis, without a branch: lines beyond the operand come back as zeros from the
// buffer bounds check, elements beyond kend (they belong to the next line) are masked.  Loads written this way can all be
// issued before the first one is waited for.
template <typename T>
__device__ __forceinline__ Bytes16 LoadRunContig(__amdgpu_buffer_rsrc_t r, int64_t line_off, int k, int kend, bool line_ok) {
    constexpr int PL = SmallDotTraits<T>::PER_LANE;
    const int off = line_ok && k < kend ? static_cast<int>((line_off + k) * static_cast<int64_t>(sizeof(T))) : 0x7fffffff;
    Bytes16 v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    const int c = kend - k;  // valid elements of the run (>= PL for all but the last run of a line)
    if constexpr (sizeof(T) == 4) {
        v.y = c > 1 ? v.y : 0u;
        v.z = c > 2 ? v.z : 0u;
        v.w = c > 3 ? v.w : 0u;
    } else {
        auto m = [c](int d) { return c > 2 * d + 1 ? 0xffffffffu : (c > 2 * d ? 0x0000ffffu : 0u); };
        v.x &= m(0);
        v.y &= m(1);
        v.z &= m(2);
        v.w &= m(3);
    }
    return v;
}

template <typename T>
__global__ __launch_bounds__(512) void SmallDotKernel(SmallDotArgs p) {
    constexpr int NW = 8;
    constexpr int KG = SmallDotTraits<T>::KG;
    constexpr int PL = SmallDotTraits<T>::PER_LANE;
    __shared__ float part[NW][32 * 33];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: the K loop below runs on scalar control flow
    const int lr = lane & 31;
    const int g = lane >> 5;
    int tm, tn;
    SmallDotTile((p.M + 31) / 32, tm, tn);
    const int m = tm * 32 + lr;
    const int n = tn * 32 + lr;
    const T* a = static_cast<const T*>(p.a);
    const T* b = static_cast<const T*>(p.b);
    const __amdgpu_buffer_rsrc_t ar = MakeRsrc(p.a, p.a_bytes);
    const __amdgpu_buffer_rsrc_t br = MakeRsrc(p.b, p.b_bytes);
    const bool a_contig = p.a_vec != 0, b_contig = p.b_vec != 0;
    const bool m_ok = m < p.M, n_ok = n < p.N;
    const int64_t a_off = static_cast<int64_t>(m) * p.a_row;
    const int64_t b_off = static_cast<int64_t>(n) * p.b_col;

    // this wave's share of K, in whole group steps
    const int groups = (p.K + KG - 1) / KG;
    const int per_wave = (groups + NW - 1) / NW;
    const int k_begin = wave * per_wave * KG;
    const int k_end = min(p.K, k_begin + per_wave * KG);

    float16_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
    constexpr int U = SmallDotTraits<T>::STEPS_IN_FLIGHT;
    if (a_contig && b_contig) {  // Linear's x and W^T: every operand load is one branch-free 16-byte buffer load
        // Two register stages of U group steps: the loads of the next stage are issued before the MFMAs of the current one,
        // so that a wave's matrix work overlaps its own loads (all waves of a workgroup run in lockstep otherwise).
        // Stages made of whole runs inside K need no masking, so nothing but the MFMAs depends on a load and the waits
        // land where the data is consumed; the (masked) remainder of a wave's share is done afterwards.
        Bytes16 av[2][U], bv[2][U];
        const int a_base = m_ok ? static_cast<int>(a_off * static_cast<int64_t>(sizeof(T))) : 0x7fffffff;
        const int b_base = n_ok ? static_cast<int>(b_off * static_cast<int64_t>(sizeof(T))) : 0x7fffffff;
        auto load_stage = [&](int st, int k) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int koff = (k + u * KG + g * PL) * static_cast<int>(sizeof(T));
                av[st][u] = __builtin_amdgcn_raw_buffer_load_b128(ar, m_ok ? a_base + koff : 0x7fffffff, 0, 0);
                bv[st][u] = __builtin_amdgcn_raw_buffer_load_b128(br, n_ok ? b_base + koff : 0x7fffffff, 0, 0);
            }
        };
        auto mfma_stage = [&](int st) {
#pragma unroll
            for (int u = 0; u < U; ++u) MfmaTile<T>(av[st][u], bv[st][u], acc);
        };
        constexpr int STEP = U * KG;
        const int nfull = k_end > k_begin ? (k_end - k_begin) / STEP : 0;  // stages whose every run ends inside K
        int k = k_begin;
        if (nfull > 0) {
            // The steady-state body has no conditional loads: the wait in front of a stage's MFMAs then only covers that
            // stage (the other stage's loads, issued later, stay in flight).  One or two stages are left for after the loop.
            load_stage(0, k);
            int i = 0;
            for (; i + 2 <= nfull - 1; i += 2) {
                load_stage(1, k + STEP);
                mfma_stage(0);
                load_stage(0, k + 2 * STEP);
                mfma_stage(1);
                k += 2 * STEP;
            }
            if (nfull - i == 2) {
                load_stage(1, k + STEP);
                mfma_stage(0);
                mfma_stage(1);
            } else {
                mfma_stage(0);
            }
            k = k_begin + nfull * STEP;
        }
        for (; k < k_end; k += KG) {
            const int kk = k + g * PL;
            Bytes16 ta = LoadRunContig<T>(ar, a_off, kk, k_end, m_ok);
            Bytes16 tb = LoadRunContig<T>(br, b_off, kk, k_end, n_ok);
            MfmaTile<T>(ta, tb, acc);
        }
    } else {
        for (int k = k_begin; k < k_end; k += 2 * KG) {
            Bytes16 av[2], bv[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                int kk = k + u * KG + g * PL;
                av[u] = LoadRun<T>(ar, a, a_off, p.a_k, kk, k_end, m_ok, a_contig);
                bv[u] = LoadRun<T>(br, b, b_off, p.b_k, kk, k_end, n_ok, b_contig);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) MfmaTile<T>(av[u], bv[u], acc);
        }
    }
    // lane holds column lr, rows 8*(v/4) + 4*g + v%4
#pragma unroll
    for (int v = 0; v < 16; ++v) part[wave][(8 * (v / 4) + 4 * g + (v % 4)) * 33 + lr] = acc[v];
    __syncthreads();
    T* out = static_cast<T*>(p.out);
    for (int e = tid; e < 32 * 32; e += 512) {
        int row = e >> 5, col = e & 31;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += part[w][row * 33 + col];
        int om = tm * 32 + row, on = tn * 32 + col;
        if (om < p.M && on < p.N) out[om * p.o_row + on * p.o_col] = static_cast<T>(s);
    }
}

// The same product when k is the unit-stride axis of both operands (Linear: x rows and W rows).  Lanes load whole
// 128-byte lines -- 8 lanes x 16 bytes per row, 8 rows per instruction -- instead of 32-byte pieces of 32 rows, and the
// wave regroups them into the MFMA operand layout through its own LDS region (no workgroup barrier in the loop).
// The loads of step s+1 are in flight while step s is multiplied.  p.nw waves split K in whole 128-byte steps.
template <typename T>
__global__ __launch_bounds__(512) void SmallDotRowsKernel(SmallDotArgs p) {
    constexpr int PL = 16 / sizeof(T);   // elements per 16-byte piece
    constexpr int KS = 8 * PL;           // k per step: one 128-byte line per row
    constexpr int PITCH = 144;           // bytes per staged row: 16 consecutive rows start on 16 different bank groups
    constexpr int REGION = 2 * 32 * PITCH;
    extern __shared__ __align__(16) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31;
    const int g = lane >> 5;
    const int piece = lane & 7;
    const int sub = lane >> 3;  // row within a group of 8
    int tm, tn;
    SmallDotTile((p.M + 31) / 32, tm, tn);
    const __amdgpu_buffer_rsrc_t ar = MakeRsrc(p.a, p.a_bytes);
    const __amdgpu_buffer_rsrc_t br = MakeRsrc(p.b, p.b_bytes);
    char* wa = lds + wave * REGION;
    char* wb = wa + 32 * PITCH;

    const int steps = (p.K + KS - 1) / KS;
    const int per_wave = (steps + p.nw - 1) / p.nw;
    const int k_begin = wave * per_wave * KS;
    const int k_end = min(p.K, k_begin + per_wave * KS);

    int abase[4], bbase[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int m = tm * 32 + j * 8 + sub, n = tn * 32 + j * 8 + sub;
        abase[j] = m < p.M ? static_cast<int>((static_cast<int64_t>(m) * p.a_row + piece * PL) * static_cast<int64_t>(sizeof(T))) : -1;
        bbase[j] = n < p.N ? static_cast<int>((static_cast<int64_t>(n) * p.b_col + piece * PL) * static_cast<int64_t>(sizeof(T))) : -1;
    }
    Bytes16 areg[4], breg[4];
    auto load_step = [&](int k) {
        const int koff = k * static_cast<int>(sizeof(T));
        const bool inside = k + piece * PL < k_end;  // pieces wholly beyond the share (or K) come back as zeros
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            areg[j] = __builtin_amdgcn_raw_buffer_load_b128(ar, (abase[j] >= 0 && inside) ? abase[j] + koff : 0x7fffffff, 0, 0);
            breg[j] = __builtin_amdgcn_raw_buffer_load_b128(br, (bbase[j] >= 0 && inside) ? bbase[j] + koff : 0x7fffffff, 0, 0);
        }
    };
    auto mask_piece = [](Bytes16 v, int c) {  // keep the first c elements of the piece (they end at K; what follows is the next row)
        if constexpr (sizeof(T) == 4) {
            v.y = c > 1 ? v.y : 0u;
            v.z = c > 2 ? v.z : 0u;
            v.w = c > 3 ? v.w : 0u;
        } else {
            auto m = [c](int d) { return c > 2 * d + 1 ? 0xffffffffu : (c > 2 * d ? 0x0000ffffu : 0u); };
            v.x &= m(0);
            v.y &= m(1);
            v.z &= m(2);
            v.w &= m(3);
        }
        return v;
    };
    auto stage_step = [&](int k) {
        const int c = k_end - (k + piece * PL);
        char* da = wa + sub * PITCH + piece * 16;
        char* db = wb + sub * PITCH + piece * 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<Bytes16*>(da + j * 8 * PITCH) = c < PL ? mask_piece(areg[j], c) : areg[j];
            *reinterpret_cast<Bytes16*>(db + j * 8 * PITCH) = c < PL ? mask_piece(breg[j], c) : breg[j];
        }
    };

    float16_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
    if (k_begin < k_end) {
        load_step(k_begin);
        for (int k = k_begin; k < k_end; k += KS) {
            stage_step(k);                           // waits for this step's loads only
            if (k + KS < k_end) load_step(k + KS);   // next step in flight during the MFMAs below
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int gs = 0; gs < 4; ++gs) {
                const Bytes16 fa = *reinterpret_cast<const Bytes16*>(wa + lr * PITCH + (2 * gs + g) * 16);
                const Bytes16 fb = *reinterpret_cast<const Bytes16*>(wb + lr * PITCH + (2 * gs + g) * 16);
                MfmaTile<T>(fa, fb, acc);
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
    __syncthreads();  // every wave is done with its staging region: it becomes the partial-sum area
    float* part = reinterpret_cast<float*>(lds);
#pragma unroll
    for (int v = 0; v < 16; ++v) part[wave * (32 * 33) + (8 * (v / 4) + 4 * g + (v % 4)) * 33 + lr] = acc[v];
    __syncthreads();
    T* out = static_cast<T*>(p.out);
    for (int e = tid; e < 32 * 32; e += 64 * p.nw) {
        const int row = e >> 5, col = e & 31;
        float s = 0.f;
        for (int w = 0; w < p.nw; ++w) s += part[w * (32 * 33) + row * 33 + col];
        const int om = tm * 32 + row, on = tn * 32 + col;
        if (om < p.M && on < p.N) out[om * p.o_row + on * p.o_col] = static_cast<T>(s);
    }
}

}  // namespace hipcx
