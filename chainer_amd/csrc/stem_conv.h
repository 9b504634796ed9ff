// 7x7 stride-2 pad-3 convolution over few input channels (the stem of ImageNet networks): float16, dense NCHW in
// and out, C input channels (template), 64 output channels.
//
// With so few channels the reduction cannot run along C.  It runs along (c, r, s) with the filter row s padded from 7
// to 8 taps: for output pixel (oh, ow) and filter row (c, r) the 8 taps are the 8 *consecutive* input pixels
// x[c][2*oh - 3 + r][2*ow - 3 .. 2*ow + 4], i.e. one 16-byte MFMA operand group (the 8th meets a zero filter tap and is
// masked to zero so that a stray Inf/NaN there cannot leak in).  Two filter rows make one v_mfma_f32_32x32x16_f16 step.
//
// A workgroup computes two output rows of one image (2*OW consecutive output pixels x 64 channels).  The 9 input rows
// per channel that they touch are staged in LDS four times, shifted by 0, 2, 4 and 6 pixels, so that the group of
// pixel ow starts on a 16-byte boundary of copy (ow & 3): every operand is a single aligned ds_read_b128, and 16
// neighbouring lanes read 16 different bank groups (the copies are 64 bytes apart modulo 256).  The shifted copies are
// built in registers from aligned global loads with v_alignbit.  Filters stay in registers for the whole workgroup
// (waves 0-1 own output channels 0-31, waves 2-3 channels 32-63).  The output tile leaves through LDS as
// [channel][pixel] so that stores are whole cache lines, with the optional batch-norm / ReLU tail applied on the way.
// A workgroup walks tiles (the host launches as many workgroups as the device holds at a time): filters are loaded once, and
// the global loads of the next tile's rows are issued before the current tile is multiplied and written out, so that their
// latency runs under that work instead of in front of the next tile.
#pragma once

#include "nchw_conv.h"

namespace hipcx {

struct StemConvArgs {
    const half_t* x;
    const half_t* wp;  // packed filters [ksteps][2][64][8]: pair = 2*ks + g -> (c, r) = (pair / 7, pair % 7), tap 7 and pairs beyond C*7 are zero
    const half_t* bias;
    half_t* out;
    int N, H, W, OH, OW;
    int64_t bias_stride;
    unsigned x_bytes, wp_bytes;
    int rowp;   // bytes of one staged row: (W / 8) * 16
    int copyb;  // bytes of one shifted copy, == 64 (mod 256)
    const half_t* bn_gamma;
    const half_t* bn_beta;
    const half_t* bn_mean;
    const half_t* bn_var;
    int64_t bn_stride;
    float bn_eps;
    int relu;
};

template <int C>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void StemConv7x7s2Kernel(StemConvArgs p) {
    constexpr int K = 64;
    constexpr int NPAIR = C * 7;
    constexpr int KSTEPS = (NPAIR + 1) / 2;
    constexpr int NROW = C * 9;  // staged rows per copy; rows NROW .. NROW+2 stay zero (operand of the padding pair)
    constexpr int MAXSUB = 4;    // 32-pixel sub-tiles per wave (2*OW <= 256)
    extern __shared__ __align__(16) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int g = lane >> 5;
    const int chalf = wave >> 1;  // which 32 output channels
    const int sub0 = wave & 1;    // first pixel sub-tile; the wave takes every second one
    const int tiles_per_img = (p.OH + 1) / 2;
    const int total_tiles = p.N * tiles_per_img;
    const int nsub = (2 * p.OW + 31) / 32;
    const int ch = p.W / 8;  // 16-byte chunks per input row

    const __amdgpu_buffer_rsrc_t xr = MakeRsrc(p.x, p.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = MakeRsrc(p.wp, p.wp_bytes);

    // ---- filters -> registers ----
    Bytes16 wf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        wf[ks] = __builtin_amdgcn_raw_buffer_load_b128(wr, ((ks * 2 + g) * K + chalf * 32 + lr) * 16, 0, 0);
    }

    // Thread (tr, tj) stages 16-byte chunk tj of rows tr, tr + 8, ... (W <= 256: one chunk per thread and row): no divisions by
    // run-time values, and all loads of a tile are issued before the first is used.
    constexpr int kRowsPerThread = (NROW + 7) / 8;
    const int tj = tid & 31, tr = tid >> 5;
    Bytes16 g1[kRowsPerThread];
    Bytes8 g0[kRowsPerThread], g2[kRowsPerThread];
    auto issue_rows = [&](int tile) {  // global loads of the tile's input rows into registers
        const int n = tile / tiles_per_img;
        const int oh0 = 2 * (tile - n * tiles_per_img);
#pragma unroll
        for (int u = 0; u < kRowsPerThread; ++u) {
            const int rr = tr + 8 * u;
            const int c = rr / 9;
            const int ih = 2 * oh0 - 3 + (rr - c * 9);
            const bool row_ok = tj < ch && rr < NROW && ih >= 0 && ih < p.H;
            const int base = (((n * C + c) * p.H + ih) * p.W + tj * 8) * 2;
            g1[u] = __builtin_amdgcn_raw_buffer_load_b128(xr, row_ok ? base : 0x7fffffff, 0, 0);
            g0[u] = __builtin_amdgcn_raw_buffer_load_b64(xr, (row_ok && tj > 0) ? base - 8 : 0x7fffffff, 0, 0);
            g2[u] = __builtin_amdgcn_raw_buffer_load_b64(xr, (row_ok && tj + 1 < ch) ? base + 16 : 0x7fffffff, 0, 0);
        }
    };
    auto stage_rows = [&]() {  // zero rows, then the loaded rows as four shifted copies
        for (int off = tid * 16; off < 3 * p.rowp; off += 256 * 16) {
#pragma unroll
            for (int k = 0; k < 4; ++k) *reinterpret_cast<Bytes16*>(lds + k * p.copyb + NROW * p.rowp + off) = Bytes16(0);
        }
        if (tj >= ch) return;
#pragma unroll
        for (int u = 0; u < kRowsPerThread; ++u) {
            const int rr = tr + 8 * u;
            if (rr >= NROW) continue;
            // d[i] holds input pixels 8*tj - 8 + 2*i, +1 of this row (i = 2 .. 9)
            unsigned d[10] = {0, 0, g0[u].x, g0[u].y, g1[u].x, g1[u].y, g1[u].z, g1[u].w, g2[u].x, g2[u].y};
            char* dst = lds + rr * p.rowp + tj * 16;
#pragma unroll
            for (int k = 0; k < 4; ++k) {  // copy k, chunk tj = padded pixels 8*tj + 2*k .. +7 = input pixels 8*tj + 2*k - 3 .. +4
                Bytes16 v;
                v.x = __builtin_amdgcn_alignbit(d[3 + k], d[2 + k], 16);
                v.y = __builtin_amdgcn_alignbit(d[4 + k], d[3 + k], 16);
                v.z = __builtin_amdgcn_alignbit(d[5 + k], d[4 + k], 16);
                v.w = __builtin_amdgcn_alignbit(d[6 + k], d[5 + k], 16);
                *reinterpret_cast<Bytes16*>(dst + k * p.copyb) = v;
            }
        }
    };

    int poff[KSTEPS];  // staged row of this lane's filter row (c, r) in each step
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        int pair = 2 * ks + g;
        int c = pair / 7, r = pair - c * 7;
        poff[ks] = (pair < NPAIR ? c * 9 + r : NROW) * p.rowp;
    }
    // per-channel constants of the epilogue
    const int nch = chalf * 32 + lr;
    const float bias = p.bias != nullptr ? static_cast<float>(p.bias[nch * p.bias_stride]) : 0.f;
    const bool has_bn = p.bn_gamma != nullptr;
    float bn_mean = 0.f, bn_inv = 1.f, bn_gamma = 1.f, bn_beta = 0.f;
    if (has_bn) {
        bn_mean = static_cast<float>(p.bn_mean[nch * p.bn_stride]);
        bn_inv = 1.0f / sqrtf(static_cast<float>(p.bn_var[nch * p.bn_stride]) + p.bn_eps);
        bn_gamma = static_cast<float>(p.bn_gamma[nch * p.bn_stride]);
        bn_beta = static_cast<float>(p.bn_beta[nch * p.bn_stride]);
    }

    int tile = blockIdx.x;
    if (tile >= total_tiles) return;
    issue_rows(tile);
    for (; tile < total_tiles; tile += gridDim.x) {
    const int n = tile / tiles_per_img;
    const int oh0 = 2 * (tile - n * tiles_per_img);
    const int npix = min(2, p.OH - oh0) * p.OW;  // valid pixels of this tile
    stage_rows();
    if (tile + static_cast<int>(gridDim.x) < total_tiles) issue_rows(tile + gridDim.x);  // in flight during the rest of this tile

    // ---- operand addresses ----
    int abase[MAXSUB];
#pragma unroll
    for (int s = 0; s < MAXSUB; ++s) {
        int q = (sub0 + 2 * s) * 32 + lr;
        if (q >= npix) q = npix - 1;  // rows of the MFMA that are never stored
        int orow = q >= p.OW ? 1 : 0;  // the tile holds two output rows
        int ow = q - (orow ? p.OW : 0);
        abase[s] = (ow & 3) * p.copyb + 2 * orow * p.rowp + (ow >> 2) * 16;
    }
    float16_t acc[MAXSUB];
#pragma unroll
    for (int s = 0; s < MAXSUB; ++s) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[s][v] = 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < MAXSUB; ++s) {
        if (sub0 + 2 * s < nsub) {  // wave-uniform
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                Bytes16 a = *reinterpret_cast<const Bytes16*>(lds + abase[s] + poff[ks]);
                a.w &= 0x0000ffffu;  // tap 7 does not exist
                MfmaTile<half_t>(a, wf[ks], acc[s]);
            }
        }
    }
    __syncthreads();  // every operand read is done: the staging area becomes the output tile

    // ---- epilogue: [channel][pixel] tile, then coalesced rows ----
    const int opitch = 2 * p.OW * 2 + 16;
    {
#pragma unroll
        for (int s = 0; s < MAXSUB; ++s) {
            if (sub0 + 2 * s >= nsub) continue;
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                const int col = (sub0 + 2 * s) * 32 + vq * 8 + g * 4;
                if (col >= 2 * p.OW) continue;  // OW % 4 == 0: a group of four is inside or outside as a whole
                PVecH<4> pack;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = acc[s][vq * 4 + e] + bias;
                    if (has_bn) v = ((v - bn_mean) * bn_inv) * bn_gamma + bn_beta;
                    if (p.relu) v = v < 0.f ? 0.f : v;
                    pack.e[e] = static_cast<half_t>(v);
                }
                *reinterpret_cast<PVecH<4>*>(lds + nch * opitch + col * 2) = pack;
            }
        }
    }
    __syncthreads();
    const int cpr = npix / 8;  // 16-byte chunks per channel row (OW % 8 == 0)
    for (int cc = tj; cc < cpr; cc += 32) {
        half_t* dst = p.out + (static_cast<int64_t>(n) * K * p.OH + oh0) * p.OW + cc * 8;
#pragma unroll 4
        for (int row = tr; row < K; row += 8) {
            Bytes16 v = *reinterpret_cast<const Bytes16*>(lds + row * opitch + cc * 16);
            *reinterpret_cast<Bytes16*>(dst + static_cast<int64_t>(row) * p.OH * p.OW) = v;
        }
    }
    __syncthreads();  // the output tile has been read: the next tile's rows may be staged over it
    }  // tiles
}

// w[64][C][7][7] (element strides) -> wp[ksteps][2][64][8] with zero padding.
__global__ __launch_bounds__(256) void StemRepackFiltersKernel(const half_t* w, half_t* wp, int C, int ksteps, int64_t wsK, int64_t wsC,
                                                               int64_t wsR, int64_t wsS) {
    int idx = blockIdx.x * 256 + threadIdx.x;  // one 16-byte group each
    if (idx >= ksteps * 2 * 64) return;
    int k = idx % 64;
    int pair = idx / 64;
    int c = pair / 7, r = pair - c * 7;
    PVecH<8> grp;
#pragma unroll
    for (int s = 0; s < 8; ++s) grp.e[s] = (pair < C * 7 && s < 7) ? w[k * wsK + c * wsC + r * wsR + s * wsS] : half_t(0);
    *reinterpret_cast<PVecH<8>*>(wp + idx * 8) = grp;
}

}  // namespace hipcx
