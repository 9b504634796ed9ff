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
};

template <typename T>
struct SmallDotTraits;
template <>
struct SmallDotTraits<float> {
    static constexpr int KG = 8;  // k values one "group step" of a wave consumes (4 MFMAs x 2)
    static constexpr int PER_LANE = 4;
    static constexpr int STEPS_IN_FLIGHT = 6;
};
template <>
struct SmallDotTraits<half_t> {
    static constexpr int KG = 16;  // one MFMA
    static constexpr int PER_LANE = 8;
    static constexpr int STEPS_IN_FLIGHT = 4;
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
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int g = lane >> 5;
    const int tm = blockIdx.x / p.tiles_n;
    const int tn = blockIdx.x - tm * p.tiles_n;
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
    // U group steps in flight: a wave's share of K is short (K / 8), and every round trip to L2 it spends is exposed
    constexpr int U = SmallDotTraits<T>::STEPS_IN_FLIGHT;
    if (a_contig && b_contig) {  // Linear's x and W^T: every operand load is one branch-free 16-byte buffer load
        for (int k = k_begin; k < k_end; k += U * KG) {
            Bytes16 av[U], bv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                int kk = k + u * KG + g * PL;
                av[u] = LoadRunContig<T>(ar, a_off, kk, k_end, m_ok);
                bv[u] = LoadRunContig<T>(br, b_off, kk, k_end, n_ok);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) MfmaTile<T>(av[u], bv[u], acc);
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

}  // namespace hipcx
