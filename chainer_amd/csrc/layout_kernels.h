// Gather of an NCHW-shaped activation (any strides) into dense channels-last memory
// [N][H'][W'][Cpad], optionally sub-sampling the spatial axes (for strided 1x1 convolutions) and
// zero-padding the channel axis up to Cpad.  A 64(c) x 64(pixel) tile goes through LDS so that both
// the global reads (along pixels) and the global writes (along channels) are coalesced.
#pragma once

#include "common.h"

namespace hipcx {

struct ToChannelsLastArgs {
    const void* x;
    void* out;
    int N, C, Cpad;
    int Ho, Wo;          // output plane extents
    int step_h, step_w;  // input pixel = (h * step_h, w * step_w)
    int64_t xsN, xsC, xsH, xsW;  // elements
    int vec_in;          // 1: plane is dense along pixels (xsW == 1, xsH == Wo, steps 1) and 16-byte loads are aligned
};

template <typename T>
__global__ __launch_bounds__(256) void ToChannelsLastKernel(ToChannelsLastArgs a) {
    constexpr int TILE = 64;
    constexpr int EPV = 16 / sizeof(T);  // elements per 16 bytes
    constexpr int ROW = TILE + EPV;      // padded LDS row, elements
    __shared__ __align__(16) T tile[TILE * ROW];  // [pixel][channel]
    const T* x = static_cast<const T*>(a.x);
    T* out = static_cast<T*>(a.out);
    const int tid = threadIdx.x;
    const int64_t plane = static_cast<int64_t>(a.Ho) * a.Wo;
    const int64_t p0 = static_cast<int64_t>(blockIdx.x) * TILE;
    const int c0 = blockIdx.y * TILE;
    const int n = blockIdx.z;
    const T* xn = x + n * a.xsN;

    if (a.vec_in) {
        // thread: channel row = tid / (TILE/EPV) + i * rows_per_pass, pixel chunk = tid % (TILE/EPV)
        constexpr int CHUNKS = TILE / EPV;
        constexpr int ROWS_PER_PASS = 256 / CHUNKS;
        struct alignas(16) V {
            T e[EPV];
        };
        const int pc = tid % CHUNKS;
#pragma unroll
        for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) {
            int cl = tid / CHUNKS + i * ROWS_PER_PASS;
            int c = c0 + cl;
            int64_t p = p0 + pc * EPV;
            V v = {};
            if (c < a.C && p < plane) v = *reinterpret_cast<const V*>(xn + c * a.xsC + p);  // plane % EPV == 0: no partial chunk
#pragma unroll
            for (int e = 0; e < EPV; ++e) tile[(pc * EPV + e) * ROW + cl] = v.e[e];
        }
    } else {
        for (int e = tid; e < TILE * TILE; e += 256) {
            int pl = e % TILE;
            int cl = e / TILE;
            int c = c0 + cl;
            int64_t p = p0 + pl;
            T v = T(0);
            if (c < a.C && p < plane) {
                int w = static_cast<int>(p % a.Wo);
                int h = static_cast<int>(p / a.Wo);
                v = xn[c * a.xsC + static_cast<int64_t>(h) * a.step_h * a.xsH + static_cast<int64_t>(w) * a.step_w * a.xsW];
            }
            tile[pl * ROW + cl] = v;
        }
    }
    __syncthreads();
    {
        constexpr int CHUNKS = TILE / EPV;
        constexpr int ROWS_PER_PASS = 256 / CHUNKS;
        struct alignas(16) V {
            T e[EPV];
        };
        const int cc = tid % CHUNKS;
#pragma unroll
        for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) {
            int pl = tid / CHUNKS + i * ROWS_PER_PASS;
            int64_t p = p0 + pl;
            int c = c0 + cc * EPV;
            if (p < plane && c < a.Cpad) {  // Cpad % EPV == 0
                V v = *reinterpret_cast<const V*>(&tile[pl * ROW + cc * EPV]);
                *reinterpret_cast<V*>(out + (static_cast<int64_t>(n) * plane + p) * a.Cpad + c) = v;
            }
        }
    }
}

template <typename T>
inline void LaunchToChannelsLast(const ToChannelsLastArgs& a, hipStream_t stream) {
    int64_t plane = static_cast<int64_t>(a.Ho) * a.Wo;
    if (plane == 0 || a.N == 0 || a.Cpad == 0) return;
    dim3 grid(static_cast<unsigned>((plane + 63) / 64), static_cast<unsigned>((a.Cpad + 63) / 64), static_cast<unsigned>(a.N));
    HIPCX_REQUIRE(grid.y <= 65535 && grid.z <= 65535, HIPCX_NOT_IMPLEMENTED_ERROR, "too many channels or images for the layout kernel");
    hipLaunchKernelGGL((ToChannelsLastKernel<T>), grid, dim3(256), 0, stream, a);
    CheckLaunch("to_channels_last");
}

// dst[r][c] (dense, row pitch dst_pitch elements, columns c >= cols zero-filled up to dst_pitch) = src[r * sr + c * sc]:
// brings a matrix operand whose reduction axis is not the unit-stride one into the layout the MFMA kernels read.
// 64x64 tiles through LDS; reads walk the source's faster axis, writes walk dst rows.
template <typename T>
__global__ __launch_bounds__(256) void StageMatrixKernel(const T* src, int64_t sr, int64_t sc, T* dst, int64_t dst_pitch, int rows, int cols,
                                                         int read_rows_fast) {
    constexpr int TILE = 64;
    __shared__ T tile[TILE][TILE + 2];
    const int r0 = blockIdx.y * TILE, c0 = blockIdx.x * TILE;
    const int tid = threadIdx.x;
    for (int e = tid; e < TILE * TILE; e += 256) {
        // consecutive threads take consecutive rows when the source is contiguous along r, consecutive columns otherwise
        const int rl = read_rows_fast ? e % TILE : e / TILE;
        const int cl = read_rows_fast ? e / TILE : e % TILE;
        const int r = r0 + rl, c = c0 + cl;
        tile[rl][cl] = (r < rows && c < cols) ? src[r * sr + c * sc] : T(0);
    }
    __syncthreads();
    for (int e = tid; e < TILE * TILE; e += 256) {
        const int rl = e / TILE, cl = e % TILE;
        const int r = r0 + rl, c = c0 + cl;
        if (r < rows && c < dst_pitch) dst[r * dst_pitch + c] = tile[rl][cl];
    }
}

template <typename T>
void StageMatrix(const T* src, int64_t sr, int64_t sc, T* dst, int64_t dst_pitch, int64_t rows, int64_t cols, hipStream_t stream) {
    const int64_t asr = sr < 0 ? -sr : sr, asc = sc < 0 ? -sc : sc;
    dim3 grid(static_cast<unsigned>((dst_pitch + 63) / 64), static_cast<unsigned>((rows + 63) / 64));
    HIPCX_REQUIRE(grid.y < 65536, HIPCX_NOT_IMPLEMENTED_ERROR, "matrix operand has too many rows to stage in one launch");
    hipLaunchKernelGGL((StageMatrixKernel<T>), grid, dim3(256), 0, stream, src, sr, sc, dst, dst_pitch, static_cast<int>(rows),
                       static_cast<int>(cols), asr < asc ? 1 : 0);
    CheckLaunch("stage_matrix");
}

}  // namespace hipcx
