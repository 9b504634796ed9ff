// NStepLstm forward (RnnKernel, CX/kernels/rnn.h:34-49, mode LSTM, one direction) for float32, as one entry point.
//
// What the routine composition computes (CX/routines/n_step_rnn.cc:41-54,97-115,185-215): for every layer and time step
//     gates = (x W_x^T + b_x) + (h W_h^T + b_h),   rows of the stacked matrices ordered unit * 4 + gate with
//     gate 0 = candidate (matrix 2 of the eight), 1 = input (0), 2 = forget (1), 3 = output (3); then the Lstm cell.
// It restacks the eight matrices and launches ~30 kernels per step.  Here:
//   * the eight matrices of a layer are packed once per call into one [4H][Xp + Hp] matrix (reduction axes zero-padded to
//     multiples of 16 floats, so rows are 16-byte granules) and the two bias sets are added up;
//   * one launch advances every layer by one time step: the layers run as a wavefront (layer l works on step s - l at stage s),
//     so a 2-layer, 35-step sequence is 36 launches;
//   * the inputs of layer 0 are copied once into one padded, 16-byte aligned array (one launch for all time steps); the layers
//     above read the padded outputs of the layer below;
//   * a workgroup owns 64 batch rows x 8 hidden units (32 gate columns): its weight slice goes through LDS in chunks of 128
//     reduction elements (two buffers), the activations [x_t ; h_{t-1}] are read straight into v_mfma_f32_16x16x4f32 operands
//     (a lane's 16-byte load feeds four consecutive MFMA steps; weights use the same assignment of k to steps), and the cell
//     (tanh / sigmoid / state update) runs on the accumulators: the gate pre-activations never reach memory.
// State rows beyond a step's batch size keep their values, as in the composition.  Sums run in another order than Dot + Add
// (float accumulation): equal to float32 tolerance, not bit for bit.
#include <algorithm>
#include <vector>

#include "common.h"

namespace hipcx {
namespace {

constexpr int kRows = 64;          // batch rows per workgroup (4 waves x 16)
constexpr int kUnits = 8;          // hidden units per workgroup
constexpr int kCols = 4 * kUnits;  // gate columns per workgroup
constexpr int kChunk = 128;        // reduction elements per LDS buffer
constexpr int kLdsRow = kChunk + 4;  // floats: 16-lane groups of 16-byte reads then hit 16 different bank quads
constexpr int kMaxJobs = 4;

using float4_t = __attribute__((ext_vector_type(4))) float;

struct LstmJob {
    const float* x;  // this step's input rows [Bt][Xp]: padded to a multiple of 16 columns with zeros, 16-byte aligned
    int Xp;
    const float* h_prev;  // [B][Hp], padding columns zero
    float* h_next;
    float* c;  // [B][H], updated in place
    int64_t c_stride;
    const float* w;  // packed [4H][Xp + Hp rounded up to whole chunks], zero beyond the two segments
    const float* bias;  // [4H]
    float* y;  // [Bt][..]: this step's output rows
    int64_t y_stride;
    int Bt;
};

struct LstmStepArgs {
    int njobs, B, H, Hp;
    LstmJob job[kMaxJobs];
};

__device__ __forceinline__ float TanhF(float v) { return tanhf(v); }
__device__ __forceinline__ float SigmoidF(float v) { return 1.0f / (1.0f + expf(-v)); }  // CX/routines/activation.cc:74-78

template <int SRC>
__device__ __forceinline__ float QuadBroadcast(float v) {  // the value of lane SRC of the lane's group of four
    constexpr int ctrl = SRC | (SRC << 2) | (SRC << 4) | (SRC << 6);  // quad_perm:[SRC,SRC,SRC,SRC]
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true));
}

__global__ __launch_bounds__(256) void LstmStepKernel(LstmStepArgs args) {
    __shared__ __attribute__((aligned(16))) float Bs[2][kCols][kLdsRow];
    const LstmJob& job = args.job[blockIdx.z];
    const int H = args.H, Hp = args.Hp, B = args.B;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int u0 = blockIdx.x * kUnits;
    const int r0 = blockIdx.y * kRows;
    const int Bt = job.Bt;
    const int lm = lane & 15, lq = lane >> 4;

    // the cell's view of the accumulators: lane <-> (row 4 * lq + (lane & 3), unit (lane & 15) / 4 (+4 for the second tile))
    const int cell_row = r0 + wave * 16 + 4 * lq + (lane & 3);
    const int cell_unit = u0 + (lm >> 2);

    if (r0 >= Bt) {  // (uniform) no row of this tile takes part in the step: the state is carried over
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int unit = cell_unit + 4 * t;
            if (cell_row < B && unit < H) job.h_next[static_cast<int64_t>(cell_row) * Hp + unit] = job.h_prev[static_cast<int64_t>(cell_row) * Hp + unit];
        }
        return;
    }

    const int Kp = job.Xp + Hp;
    const int nchunks = (Kp + kChunk - 1) / kChunk;
    const int Kw = nchunks * kChunk;  // length of a packed weight row: zero beyond Kp, so that no block needs a bounds check
    const int a_row = r0 + wave * 16 + lm;
    const bool a_ok = a_row < Bt;
    const float* xrow = job.x + static_cast<int64_t>(a_ok ? a_row : 0) * job.Xp;
    const float* hrow = job.h_prev + static_cast<int64_t>(a_ok ? a_row : 0) * Hp;

    // weights: 32 columns x 128 k = 1024 16-byte pieces per chunk, four per thread
    auto load_w = [&](int kc, float4_t* wreg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int piece = tid + 256 * i;
            const int col = piece >> 5, k = kc + 4 * (piece & 31);
            int n = u0 * 4 + col;
            if (n > 4 * H - 1) n = 4 * H - 1;  // columns past the last unit repeat the last row: their results are never stored
            wreg[i] = *reinterpret_cast<const float4_t*>(job.w + static_cast<int64_t>(n) * Kw + k);
        }
    };
    auto store_w = [&](int buf, const float4_t* wreg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int piece = tid + 256 * i;
            *reinterpret_cast<float4_t*>(&Bs[buf][piece >> 5][4 * (piece & 31)]) = wreg[i];
        }
    };
    // Activations: a lane's operand for block kb of a chunk is four consecutive k of its row, one 16-byte load; the eight loads of
    // a chunk are issued together.  Blocks past the end load the row's first block (a valid address) and are then replaced by
    // zeros: their weights are zero as well, but 0 * inf would be NaN where the reference forms no product at all.  Rows past the
    // step's batch read row 0: their products stay in accumulator rows that are never stored.
    constexpr int kBlocks = kChunk / 16;
    auto load_a = [&](int kc, float4_t* a) {
#pragma unroll
        for (int kb = 0; kb < kBlocks; ++kb) {
            const int kglob = kc + kb * 16;
            const float* p = kglob < job.Xp ? xrow + kglob : (kglob < Kp ? hrow + (kglob - job.Xp) : hrow);  // (uniform selects)
            const float4_t v = *reinterpret_cast<const float4_t*>(p + 4 * lq);
            a[kb] = kglob < Kp ? v : float4_t{0.f, 0.f, 0.f, 0.f};
        }
    };

    float4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    // Two operand register sets used in turn (the chunk loop is unrolled by two, so no set is ever copied into the other: a copy
    // would wait for the loads it copies and put the memory latency back in front of the products).
    float4_t a_even[kBlocks], a_odd[kBlocks];
    // No branch inside: chunks after the last are the last one read again (into buffers nobody uses any more).  Activations
    // (shared by every workgroup, so near) are fetched one chunk ahead; a workgroup's weight slice is its own and comes from
    // farther away: two chunks ahead, held in registers for one chunk before it goes to LDS.
    float4_t w_even[4], w_odd[4];
    auto chunk = [&](int ch, const float4_t* a_now, float4_t* a_later, const float4_t* w_next, float4_t* w_after) {
        const int cur = ch & 1;
        const int last = nchunks - 1;
        load_w((ch + 2 < last ? ch + 2 : last) * kChunk, w_after);
        load_a((ch + 1 < last ? ch + 1 : last) * kChunk, a_later);
#pragma unroll
        for (int kb = 0; kb < kBlocks; ++kb) {
            const float4_t b0 = *reinterpret_cast<const float4_t*>(&Bs[cur][lm][kb * 16 + 4 * lq]);
            const float4_t b1 = *reinterpret_cast<const float4_t*>(&Bs[cur][16 + lm][kb * 16 + 4 * lq]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_now[kb][j], b0[j], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_now[kb][j], b1[j], acc[1], 0, 0, 0);
            }
        }
        store_w(cur ^ 1, w_next);  // chunk ch + 1, loaded during chunk ch - 1; the buffer's readers passed the previous barrier
        __syncthreads();
    };
    load_w(0, w_even);
    load_a(0, a_even);
    load_w((nchunks > 1 ? 1 : 0) * kChunk, w_odd);
    store_w(0, w_even);
    __syncthreads();
    int ch = 0;
    for (; ch + 1 < nchunks; ch += 2) {
        chunk(ch, a_even, a_odd, w_odd, w_even);      // stores chunk ch + 1 (w_odd), fetches chunk ch + 2 into w_even
        chunk(ch + 1, a_odd, a_even, w_even, w_odd);  // stores chunk ch + 2 (w_even), fetches chunk ch + 3 into w_odd
    }
    if (ch < nchunks) chunk(ch, a_even, a_odd, w_odd, w_even);

    // ---- the cell: accumulator register i of a lane is (row 4 * lq + i, column lm); the four lanes of a group of four hold the four
    // gates of one unit, so lane r of the group collects the gates of row 4 * lq + r ----
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int n = u0 * 4 + 16 * t + lm;
        const float bias = n < 4 * H ? job.bias[n] : 0.f;
        float g[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float v = acc[t][i] + bias;
            const float v0 = QuadBroadcast<0>(v), v1 = QuadBroadcast<1>(v), v2 = QuadBroadcast<2>(v), v3 = QuadBroadcast<3>(v);
            if ((lane & 3) == i) {
                g[0] = v0;
                g[1] = v1;
                g[2] = v2;
                g[3] = v3;
            }
        }
        const int unit = cell_unit + 4 * t;
        if (unit >= H || cell_row >= B) continue;
        const int64_t hoff = static_cast<int64_t>(cell_row) * Hp + unit;
        if (cell_row < Bt) {
            const float ga = TanhF(g[0]), gi = SigmoidF(g[1]), gf = SigmoidF(g[2]), go = SigmoidF(g[3]);
            float* cp = job.c + static_cast<int64_t>(cell_row) * job.c_stride + unit;
            const float cn = ga * gi + gf * *cp;
            const float hn = go * TanhF(cn);
            *cp = cn;
            job.h_next[hoff] = hn;
            job.y[static_cast<int64_t>(cell_row) * job.y_stride + unit] = hn;
        } else {
            job.h_next[hoff] = job.h_prev[hoff];
        }
    }
}

struct LstmPackArgs {
    const float* w[8];
    int64_t w_row[8], w_col[8];  // element strides
    const float* b[8];
    int64_t b_stride[8];
    float* w_out;  // [4H][Xp + Hp rounded up to whole chunks]
    float* b_out;  // [4H]
    int H, I, Xp, Hp;
};

__global__ __launch_bounds__(256) void LstmPackKernel(LstmPackArgs p) {
    const int Kp = (p.Xp + p.Hp + kChunk - 1) / kChunk * kChunk;  // rows are padded to whole chunks with zeros
    const int64_t total = static_cast<int64_t>(4) * p.H * Kp;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        const int n = static_cast<int>(idx / Kp), k = static_cast<int>(idx - static_cast<int64_t>(n) * Kp);
        const int u = n >> 2, g = n & 3;
        const int mi = g == 0 ? 2 : (g == 1 ? 0 : (g == 2 ? 1 : 3));  // StackWeight order: matrices 2, 0, 1, 3 (and 6, 4, 5, 7)
        float v = 0.f;
        if (k < p.Xp) {
            if (k < p.I) v = p.w[mi][u * p.w_row[mi] + k * p.w_col[mi]];
        } else if (k - p.Xp < p.H) {
            v = p.w[4 + mi][u * p.w_row[4 + mi] + (k - p.Xp) * p.w_col[4 + mi]];
        }
        p.w_out[idx] = v;
        if (k == 0) p.b_out[n] = p.b[mi][u * p.b_stride[mi]] + p.b[4 + mi][u * p.b_stride[4 + mi]];
    }
}

// The inputs of layer 0, one array per time step, gathered into one array of padded rows.
constexpr int kMaxPadItems = 96;
struct LstmPadArgs {
    int n, I, Xp;
    float* dst;  // [sum of rows][Xp]
    struct Item {
        const float* src;
        int64_t stride;   // elements between rows
        int64_t dst_row;  // first row in dst
        int rows;
    } item[kMaxPadItems];
};

__global__ __launch_bounds__(256) void LstmPadKernel(LstmPadArgs p) {
    const LstmPadArgs::Item& it = p.item[blockIdx.y];
    const int64_t total = static_cast<int64_t>(it.rows) * p.Xp;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t r = idx / p.Xp;
        const int k = static_cast<int>(idx - r * p.Xp);
        p.dst[(it.dst_row + r) * p.Xp + k] = k < p.I ? it.src[r * it.stride + k] : 0.f;
    }
}

size_t Round256(size_t v) { return (v + 255) / 256 * 256; }
int RoundUp16(int64_t v) { return static_cast<int>((v + 15) / 16 * 16); }
int64_t PackedRow(int64_t k) { return (k + kChunk - 1) / kChunk * kChunk; }

void CheckStatus(int status) {
    if (status != HIPCX_OK) throw Error(status, hipcx_last_error());
}

struct LstmPlan {
    int L = 0, T = 0;
    int64_t B = 0, H = 0, I = 0, Hp = 0;
    int64_t rows = 0;  // sum of the steps' batch sizes
    std::vector<int64_t> row_start;
    std::vector<size_t> w_off, b_off, h_off, y_off;  // per layer
    size_t x_off = 0;                                  // the padded inputs of layer 0
    size_t total = 0;
};

LstmPlan PlanLstm(int n_layers, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps) {
    HIPCX_REQUIRE(n_layers >= 1 && n_steps >= 1, HIPCX_DIMENSION_ERROR, "n_step_lstm: at least one layer and one time step are required");
    HIPCX_REQUIRE(xs != nullptr, HIPCX_CHAINERX_ERROR, "xs is null");
    ValidateArray(hx, "hx");
    HIPCX_REQUIRE(hx->ndim == 3 && hx->shape[0] == n_layers, HIPCX_DIMENSION_ERROR, "hx must have the shape [n_layers, batch, units], got " + ShapeStr(hx));
    HIPCX_REQUIRE(hx->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: float32 only (compose the routine for other dtypes)");
    LstmPlan pl;
    pl.L = n_layers;
    pl.T = n_steps;
    pl.B = hx->shape[1];
    pl.H = hx->shape[2];
    HIPCX_REQUIRE(pl.B > 0 && pl.H > 0 && pl.B < (1 << 24) && pl.H < (1 << 24), HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: empty or oversized state");
    pl.Hp = RoundUp16(pl.H);
    for (int t = 0; t < n_steps; ++t) {
        ValidateArray(xs[t], "xs[t]");
        HIPCX_REQUIRE(xs[t]->ndim == 2, HIPCX_DIMENSION_ERROR, "every xs[t] must be a matrix");
        HIPCX_REQUIRE(xs[t]->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: float32 only");
        if (t == 0) pl.I = xs[0]->shape[1];
        HIPCX_REQUIRE(xs[t]->shape[1] == pl.I && pl.I > 0 && pl.I < (1 << 24), HIPCX_DIMENSION_ERROR, "every xs[t] must have the same number of columns");
        HIPCX_REQUIRE(xs[t]->shape[0] <= pl.B, HIPCX_DIMENSION_ERROR, "The batch size of x must be equal to or less than the size of state");
        HIPCX_REQUIRE(xs[t]->shape[0] > 0, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: empty time step");
        pl.row_start.push_back(pl.rows);
        pl.rows += xs[t]->shape[0];
    }
    size_t off = 0;
    pl.x_off = off;
    off += Round256(static_cast<size_t>(pl.rows * RoundUp16(pl.I)) * 4);
    for (int l = 0; l < n_layers; ++l) {
        const int64_t Xp = RoundUp16(l == 0 ? pl.I : pl.H);
        pl.w_off.push_back(off);
        off += Round256(static_cast<size_t>(4 * pl.H * PackedRow(Xp + pl.Hp)) * 4);
        pl.b_off.push_back(off);
        off += Round256(static_cast<size_t>(4 * pl.H) * 4);
        pl.h_off.push_back(off);
        off += Round256(static_cast<size_t>(2 * pl.B * pl.Hp) * 4);
        pl.y_off.push_back(off);
        if (l + 1 < n_layers) off += Round256(static_cast<size_t>(pl.rows * pl.Hp) * 4);
    }
    pl.total = off;
    return pl;
}

hipcx_array Matrix(void* data, int64_t rows, int64_t cols, int64_t row_stride_elems) {
    hipcx_array a{};
    a.data = data;
    a.dtype = HIPCX_FLOAT32;
    a.ndim = 2;
    a.shape[0] = rows;
    a.shape[1] = cols;
    a.strides[0] = row_stride_elems * 4;
    a.strides[1] = 4;
    return a;
}

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

size_t hipcx_n_step_lstm_workspace_size(int n_layers, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps) {
    try {
        return PlanLstm(n_layers, hx, xs, n_steps).total;
    } catch (...) {
        return 0;
    }
}

int hipcx_n_step_lstm(int n_layers, const hipcx_array* hx, const hipcx_array* cx, const hipcx_array* const* ws, const hipcx_array* const* bs,
                      const hipcx_array* const* xs, int n_steps, const hipcx_array* hy, const hipcx_array* cy, const hipcx_array* const* ys,
                      void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        const LstmPlan pl = PlanLstm(n_layers, hx, xs, n_steps);
        const int64_t B = pl.B, H = pl.H, Hp = pl.Hp;
        HIPCX_REQUIRE(ws != nullptr && bs != nullptr && ys != nullptr, HIPCX_CHAINERX_ERROR, "ws, bs or ys is null");
        auto state = [&](const hipcx_array* a, const char* name) {
            ValidateArray(a, name);
            HIPCX_REQUIRE(a->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: float32 only");
            HIPCX_REQUIRE(a->ndim == 3 && a->shape[0] == n_layers && a->shape[1] == B && a->shape[2] == H, HIPCX_DIMENSION_ERROR,
                          std::string(name) + " must have hx's shape, got " + ShapeStr(a));
            HIPCX_REQUIRE(a->strides[2] == 4 && a->strides[1] % 4 == 0 && a->strides[0] % 4 == 0, HIPCX_NOT_IMPLEMENTED_ERROR,
                          std::string(name) + ": unit stride along the last axis required");
        };
        state(hx, "hx");
        state(cx, "cx");
        state(hy, "hy");
        state(cy, "cy");
        for (int l = 0; l < n_layers; ++l) {
            const int64_t in = l == 0 ? pl.I : H;
            for (int i = 0; i < 8; ++i) {
                const hipcx_array* w = ws[l * 8 + i];
                const hipcx_array* b = bs[l * 8 + i];
                ValidateArray(w, "ws[i]");
                ValidateArray(b, "bs[i]");
                HIPCX_REQUIRE(w->dtype == HIPCX_FLOAT32 && b->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: float32 only");
                HIPCX_REQUIRE(w->ndim == 2 && w->shape[0] == H && w->shape[1] == (i < 4 ? in : H), HIPCX_DIMENSION_ERROR,
                              "n_step_lstm: weight matrix " + std::to_string(i) + " of layer " + std::to_string(l) + " has the wrong shape " + ShapeStr(w));
                HIPCX_REQUIRE(b->ndim == 1 && b->shape[0] == H, HIPCX_DIMENSION_ERROR, "n_step_lstm: every bias must have one value per unit");
                HIPCX_REQUIRE(w->strides[0] % 4 == 0 && w->strides[1] % 4 == 0 && b->strides[0] % 4 == 0, HIPCX_NOT_IMPLEMENTED_ERROR,
                              "byte strides must be multiples of the item size");
            }
        }
        for (int t = 0; t < n_steps; ++t) {
            ValidateArray(ys[t], "ys[t]");
            HIPCX_REQUIRE(ys[t]->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: float32 only");
            HIPCX_REQUIRE(ys[t]->ndim == 2 && ys[t]->shape[0] == xs[t]->shape[0] && ys[t]->shape[1] == H, HIPCX_DIMENSION_ERROR,
                          "ys[t] must have the shape [batch of step t, units]");
            HIPCX_REQUIRE(ys[t]->strides[1] == 4 && ys[t]->strides[0] % 4 == 0 && xs[t]->strides[1] == 4 && xs[t]->strides[0] % 4 == 0,
                          HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_lstm: xs[t] and ys[t] need unit stride along their last axis");
        }
        HIPCX_REQUIRE(workspace != nullptr && workspace_bytes >= pl.total, HIPCX_CHAINERX_ERROR,
                      "n_step_lstm workspace too small: need " + std::to_string(pl.total) + " bytes");
        HIPCX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, HIPCX_CHAINERX_ERROR, "workspace must be 256-byte aligned");
        char* base = static_cast<char*>(workspace);
        hipStream_t st = AsStream(stream);
        hipcx_scalar zero{};
        zero.kind = HIPCX_KIND_INT;

        // ---- set-up: packed weights, zeroed (padded) state and layer outputs, the initial state ----
        CheckStatus(hipcx_copy(cx, cy, stream));  // the cell state lives in cy and is updated in place
        const int Xp0 = RoundUp16(pl.I);
        int max_rows = 0;
        for (int t0 = 0; t0 < n_steps; t0 += kMaxPadItems) {
            LstmPadArgs pa{};
            pa.I = static_cast<int>(pl.I);
            pa.Xp = Xp0;
            pa.dst = reinterpret_cast<float*>(base + pl.x_off);
            max_rows = 0;
            for (int t = t0; t < n_steps && t < t0 + kMaxPadItems; ++t) {
                LstmPadArgs::Item& it = pa.item[pa.n++];
                it.src = static_cast<const float*>(xs[t]->data);
                it.stride = xs[t]->strides[0] / 4;
                it.dst_row = pl.row_start[t];
                it.rows = static_cast<int>(xs[t]->shape[0]);
                max_rows = std::max(max_rows, it.rows);
            }
            const int64_t blocks = (static_cast<int64_t>(max_rows) * Xp0 + 255) / 256;
            hipLaunchKernelGGL(LstmPadKernel, dim3(static_cast<unsigned>(blocks > 4096 ? 4096 : blocks), static_cast<unsigned>(pa.n)), dim3(256), 0,
                               st, pa);
            CheckLaunch("lstm_pad_inputs");
        }
        for (int l = 0; l < n_layers; ++l) {
            const int64_t in = l == 0 ? pl.I : H;
            LstmPackArgs pa{};
            for (int i = 0; i < 8; ++i) {
                const hipcx_array* w = ws[l * 8 + i];
                const hipcx_array* b = bs[l * 8 + i];
                pa.w[i] = static_cast<const float*>(w->data);
                pa.w_row[i] = w->strides[0] / 4;
                pa.w_col[i] = w->strides[1] / 4;
                pa.b[i] = static_cast<const float*>(b->data);
                pa.b_stride[i] = b->strides[0] / 4;
            }
            pa.w_out = reinterpret_cast<float*>(base + pl.w_off[l]);
            pa.b_out = reinterpret_cast<float*>(base + pl.b_off[l]);
            pa.H = static_cast<int>(H);
            pa.I = static_cast<int>(in);
            pa.Xp = RoundUp16(in);
            pa.Hp = static_cast<int>(Hp);
            const int64_t total = 4 * H * PackedRow(pa.Xp + Hp);
            int64_t blocks = (total + 255) / 256;
            const int64_t cap = static_cast<int64_t>(NumCUs()) * 16;
            hipLaunchKernelGGL(LstmPackKernel, dim3(static_cast<unsigned>(blocks > cap ? cap : blocks)), dim3(256), 0, st, pa);
            CheckLaunch("lstm_pack");
            // both state buffers zero (the padding columns stay zero for good), then hx[l] into the first
            hipcx_array hbuf = Matrix(base + pl.h_off[l], 2 * B, Hp, Hp);
            CheckStatus(hipcx_fill(&hbuf, zero, stream));
            hipcx_array h0 = Matrix(base + pl.h_off[l], B, H, Hp);
            hipcx_array hsrc = Matrix(static_cast<char*>(hx->data) + l * hx->strides[0], B, H, hx->strides[1] / 4);
            CheckStatus(hipcx_copy(&hsrc, &h0, stream));
            if (l + 1 < n_layers) {
                hipcx_array ybuf = Matrix(base + pl.y_off[l], pl.rows, Hp, Hp);
                CheckStatus(hipcx_fill(&ybuf, zero, stream));
            }
        }

        // ---- the wavefront: stage s runs (layer l, step s - l) for every layer that has such a step ----
        const dim3 block(256);
        for (int s = 0; s < n_steps + n_layers - 1; ++s) {
            LstmStepArgs a{};
            a.B = static_cast<int>(B);
            a.H = static_cast<int>(H);
            a.Hp = static_cast<int>(Hp);
            auto flush = [&]() {
                if (a.njobs == 0) return;
                const dim3 grid(static_cast<unsigned>((H + kUnits - 1) / kUnits), static_cast<unsigned>((B + kRows - 1) / kRows),
                                static_cast<unsigned>(a.njobs));
                hipLaunchKernelGGL(LstmStepKernel, grid, block, 0, st, a);
                CheckLaunch("lstm_step");
                a.njobs = 0;
            };
            for (int l = 0; l < n_layers; ++l) {
                const int t = s - l;
                if (t < 0 || t >= n_steps) continue;
                LstmJob& j = a.job[a.njobs++];
                const int64_t bt = xs[t]->shape[0];
                if (l == 0) {
                    j.Xp = Xp0;
                    j.x = reinterpret_cast<const float*>(base + pl.x_off) + pl.row_start[t] * Xp0;
                } else {
                    j.Xp = static_cast<int>(Hp);
                    j.x = reinterpret_cast<const float*>(base + pl.y_off[l - 1]) + pl.row_start[t] * Hp;
                }
                float* hbuf = reinterpret_cast<float*>(base + pl.h_off[l]);
                j.h_prev = hbuf + (t & 1) * B * Hp;
                j.h_next = hbuf + ((t + 1) & 1) * B * Hp;
                j.c = reinterpret_cast<float*>(static_cast<char*>(cy->data) + l * cy->strides[0]);
                j.c_stride = cy->strides[1] / 4;
                j.w = reinterpret_cast<const float*>(base + pl.w_off[l]);
                j.bias = reinterpret_cast<const float*>(base + pl.b_off[l]);
                if (l + 1 < n_layers) {
                    j.y = reinterpret_cast<float*>(base + pl.y_off[l]) + pl.row_start[t] * Hp;
                    j.y_stride = Hp;
                } else {
                    j.y = static_cast<float*>(ys[t]->data);
                    j.y_stride = ys[t]->strides[0] / 4;
                }
                j.Bt = static_cast<int>(bt);
                if (a.njobs == kMaxJobs) flush();
            }
            flush();
        }

        // ---- the final hidden state of every layer ----
        for (int l = 0; l < n_layers; ++l) {
            float* hbuf = reinterpret_cast<float*>(base + pl.h_off[l]);
            hipcx_array hfin = Matrix(hbuf + (n_steps & 1) * B * Hp, B, H, Hp);
            hipcx_array hdst = Matrix(static_cast<char*>(hy->data) + l * hy->strides[0], B, H, hy->strides[1] / 4);
            CheckStatus(hipcx_copy(&hfin, &hdst, stream));
        }
    });
}

}  // extern "C"
