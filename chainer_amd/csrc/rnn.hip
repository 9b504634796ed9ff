// RnnKernel and RnnBackwardKernel (CX/kernels/rnn.h:34-66) for float32: every mode NStepRnnImpl hands to the kernel
// (CX/routines/n_step_rnn.cc:434-497) -- LSTM (mode 1), GRU (mode 0), plain RNN with tanh or relu (mode 2) -- in one or both
// directions, with the gradients of a forward pass that kept its reserve.
//
// The forward pass computes what the routine composition computes (GruImpl / LstmImpl / RnnImpl, n_step_rnn.cc:57-131; the layer
// and direction wiring of NStepRnnImpl, :362-426).  Per layer and direction:
//   * the x-side matrices are stacked once into [G*H][in] (G gates, gate-major rows) and every time step's input projection is one
//     product  XW = X_all [rows, in] . Wx^T  over the rows of all steps (rows = sum of the steps' batch sizes);
//   * a time step is the recurrent product  HW = h[:Bt] . Wh^T  and one cell kernel that adds the biases, applies the gate
//     functions and updates h (and c) in place for the Bt rows the step holds; rows beyond Bt keep their state, as in
//     OneDirectionalLoop (:133-175).  The backward direction walks the steps from the last to the first on its own state.
//   * the outputs go to columns [d*H, (d+1)*H) of the layer's output rows, which are the next layer's input (the Concatenate of
//     :398-404), or to the caller's ys[t] for the top layer.
// With a reserve (training) the cell kernel also stores what the gradient needs: the gate activations, the state rows before the
// step, and the outputs of the lower layers.  The one-direction LSTM without reserve is handed to hipcx_n_step_lstm (lstm.hip), which
// keeps the gates in MFMA accumulators.
//
// The backward pass is backpropagation through time written out over the same buffers: per step one cell-gradient kernel (gate
// pre-activation gradients from dh, dc, dy and the saved activations), one product with Wh for dh of the step before; per layer
// and direction the weight gradients as products over all rows at once (dWx[g] = dG[:, g]^T . X_all, dWh[g] = dG[:, g]^T . Hprev_all),
// the bias gradients as column sums, and the input gradient dX_all = dG . Wx, which is the dy of the layer below.
// The reference's cuda backend gets these numbers from cuDNN (CX/cuda/cuda_device/rnn.cu); every other backend from autograd over the
// composition.  Sums run in another order than either: equal to float32 tolerance.
#include <algorithm>
#include <vector>

#include "common.h"

extern "C" {
size_t hipcx_n_step_lstm_workspace_size(int n_layers, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps);
int hipcx_n_step_lstm(int n_layers, const hipcx_array* hx, const hipcx_array* cx, const hipcx_array* const* ws, const hipcx_array* const* bs,
                      const hipcx_array* const* xs, int n_steps, const hipcx_array* hy, const hipcx_array* cy, const hipcx_array* const* ys,
                      void* workspace, size_t workspace_bytes, void* stream);
}

namespace hipcx {
namespace {

enum RnnMode { kGru = 0, kLstm = 1, kRnn = 2 };  // the `mode` argument of RnnKernel::Call as NStepRnnImpl's callers pass it

int NumGates(int mode) { return mode == kLstm ? 4 : (mode == kGru ? 3 : 1); }        // matrices per side; ws holds twice as many
int ReserveGates(int mode) { return mode == kRnn ? 1 : 4; }  // saved values per unit and row: LSTM i f g o; GRU r z n hh; RNN h

struct CellArgs {
    int mode, relu;
    int Bt, H;
    const float* xw;    // [Bt][G*H]: this step's rows of the input projection
    const float* hw;    // [Bt][G*H]: h . Wh^T
    const float* bx;    // [G*H]
    const float* bh;    // [G*H]
    float* h;           // [B][H] state, rows < Bt updated in place
    float* c;           // [B][H] (LSTM)
    float* y;           // output rows
    int64_t y_stride;
    float* gates;       // reserve, this step's rows [Bt][GR*H]; null: inference
    float* hprev;       // reserve [Bt][H]
    float* cprev;       // reserve [Bt][H] (LSTM)
};

__device__ __forceinline__ float Sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }  // CX/routines/activation.cc:74-78

__global__ __launch_bounds__(256) void RnnCellKernel(CellArgs p) {
    const int total = p.Bt * p.H;
    const int GH = p.H * (p.mode == kLstm ? 4 : (p.mode == kGru ? 3 : 1));
    for (int idx = blockIdx.x * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
        const int r = idx / p.H, u = idx - r * p.H;
        const float* xw = p.xw + static_cast<int64_t>(r) * GH + u;
        const float* hw = p.hw + static_cast<int64_t>(r) * GH + u;
        auto pre = [&](int g) { return (xw[g * p.H] + p.bx[g * p.H + u]) + (hw[g * p.H] + p.bh[g * p.H + u]); };  // Linear(x) + Linear(h)
        float* hs = p.h + static_cast<int64_t>(r) * p.H + u;
        const float h_old = *hs;
        float h_new;
        if (p.mode == kLstm) {
            float* cs = p.c + static_cast<int64_t>(r) * p.H + u;
            const float c_old = *cs;
            const float gi = Sigmoid(pre(0)), gf = Sigmoid(pre(1)), gg = tanhf(pre(2)), go = Sigmoid(pre(3));
            const float c_new = gg * gi + gf * c_old;
            h_new = go * tanhf(c_new);
            *cs = c_new;
            if (p.gates != nullptr) {
                float* q = p.gates + static_cast<int64_t>(r) * 4 * p.H + u;
                q[0] = gi, q[p.H] = gf, q[2 * p.H] = gg, q[3 * p.H] = go;
                p.cprev[idx] = c_old;
            }
        } else if (p.mode == kGru) {
            const float gr = Sigmoid(pre(0)), gz = Sigmoid(pre(1));
            const float hh = hw[2 * p.H] + p.bh[2 * p.H + u];
            const float gn = tanhf((xw[2 * p.H] + p.bx[2 * p.H + u]) + gr * hh);
            h_new = (1.0f - gz) * gn + gz * h_old;
            if (p.gates != nullptr) {
                float* q = p.gates + static_cast<int64_t>(r) * 4 * p.H + u;
                q[0] = gr, q[p.H] = gz, q[2 * p.H] = gn, q[3 * p.H] = hh;
            }
        } else {
            const float s = pre(0);
            h_new = p.relu ? fmaxf(s, 0.0f) : tanhf(s);
            if (p.gates != nullptr) p.gates[idx] = h_new;
        }
        if (p.gates != nullptr) p.hprev[idx] = h_old;
        *hs = h_new;
        p.y[static_cast<int64_t>(r) * p.y_stride + u] = h_new;
    }
}

struct CellGradArgs {
    int mode, relu;
    int Bt, H;
    const float* dy;  // this step's rows of the gradient of the layer's output, this direction's columns
    int64_t dy_stride;
    float* dh;        // [B][H]: in, the gradient of the state after the step; out, the part of the gradient of the state before
                      // the step that does not pass through Wh (GRU: dh * z, else 0) -- the caller adds dGh . Wh
    float* dc;        // [B][H] (LSTM), updated in place
    const float* gates;
    const float* hprev;
    const float* cprev;
    float* dgx;       // [Bt][G*H]: gradient of x . Wx^T + bx
    float* dgh;       // [Bt][G*H]: gradient of h . Wh^T + bh (the same array as dgx unless GRU)
};

__global__ __launch_bounds__(256) void RnnCellGradKernel(CellGradArgs p) {
    const int total = p.Bt * p.H;
    for (int idx = blockIdx.x * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
        const int r = idx / p.H, u = idx - r * p.H;
        float* dhs = p.dh + static_cast<int64_t>(r) * p.H + u;
        const float dh = *dhs + p.dy[static_cast<int64_t>(r) * p.dy_stride + u];
        if (p.mode == kLstm) {
            const float* q = p.gates + static_cast<int64_t>(r) * 4 * p.H + u;
            const float gi = q[0], gf = q[p.H], gg = q[2 * p.H], go = q[3 * p.H];
            const float c_old = p.cprev[idx];
            const float tc = tanhf(gg * gi + gf * c_old);
            float* dcs = p.dc + static_cast<int64_t>(r) * p.H + u;
            const float dc = *dcs + dh * go * (1.0f - tc * tc);
            float* g = p.dgx + static_cast<int64_t>(r) * 4 * p.H + u;
            g[0] = dc * gg * gi * (1.0f - gi);
            g[p.H] = dc * c_old * gf * (1.0f - gf);
            g[2 * p.H] = dc * gi * (1.0f - gg * gg);
            g[3 * p.H] = dh * tc * go * (1.0f - go);
            *dcs = dc * gf;
            *dhs = 0.0f;
        } else if (p.mode == kGru) {
            const float* q = p.gates + static_cast<int64_t>(r) * 4 * p.H + u;
            const float gr = q[0], gz = q[p.H], gn = q[2 * p.H], hh = q[3 * p.H];
            const float h_old = p.hprev[idx];
            const float dn_pre = dh * (1.0f - gz) * (1.0f - gn * gn);
            const float dz_pre = dh * (h_old - gn) * gz * (1.0f - gz);
            const float dr_pre = dn_pre * hh * gr * (1.0f - gr);
            float* gx = p.dgx + static_cast<int64_t>(r) * 3 * p.H + u;
            float* gh = p.dgh + static_cast<int64_t>(r) * 3 * p.H + u;
            gx[0] = dr_pre, gx[p.H] = dz_pre, gx[2 * p.H] = dn_pre;
            gh[0] = dr_pre, gh[p.H] = dz_pre, gh[2 * p.H] = dn_pre * gr;
            *dhs = dh * gz;
        } else {
            const float h_new = p.gates[idx];
            p.dgx[idx] = p.relu ? (h_new > 0.0f ? dh : 0.0f) : dh * (1.0f - h_new * h_new);
            *dhs = 0.0f;
        }
    }
}

size_t Round256(size_t v) { return (v + 255) / 256 * 256; }

void CheckStatus(int status) {
    if (status != HIPCX_OK) throw Error(status, hipcx_last_error());
}

hipcx_array Matrix(const void* data, int64_t rows, int64_t cols, int64_t row_stride, int64_t col_stride = 1) {
    hipcx_array a{};
    a.data = const_cast<void*>(data);
    a.dtype = HIPCX_FLOAT32;
    a.ndim = 2;
    a.shape[0] = rows, a.shape[1] = cols;
    a.strides[0] = row_stride * 4, a.strides[1] = col_stride * 4;
    return a;
}

hipcx_array Vector(const void* data, int64_t n, int64_t stride = 1) {
    hipcx_array a{};
    a.data = const_cast<void*>(data);
    a.dtype = HIPCX_FLOAT32;
    a.ndim = 1;
    a.shape[0] = n;
    a.strides[0] = stride * 4;
    return a;
}

// Shapes of a call and the layout of its workspace and reserve.  Offsets are bytes.
struct RnnPlan {
    int L = 0, D = 1, T = 0, mode = 0, G = 1, GR = 1;
    int64_t B = 0, H = 0, I = 0, rows = 0, max_in = 0;
    std::vector<int64_t> row_start, bt;
    // reserve (forward writes, backward reads): per layer-direction the gate activations and the states before each step; per
    // layer below the top its output rows
    std::vector<size_t> r_gates, r_hprev, r_cprev, r_y;
    size_t reserve_total = 0;
    int64_t In(int layer) const { return layer == 0 ? I : D * H; }
};

RnnPlan MakePlan(int n_layers, int bidirectional, int mode, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps) {
    HIPCX_REQUIRE(mode == kGru || mode == kLstm || mode == kRnn, HIPCX_CHAINERX_ERROR, "n_step_rnn: mode must be 0 (GRU), 1 (LSTM) or 2 (RNN)");
    HIPCX_REQUIRE(n_layers >= 1 && n_steps >= 1, HIPCX_DIMENSION_ERROR, "n_step_rnn: at least one layer and one time step are required");
    HIPCX_REQUIRE(xs != nullptr, HIPCX_CHAINERX_ERROR, "xs is null");
    ValidateArray(hx, "hx");
    RnnPlan pl;
    pl.L = n_layers, pl.D = bidirectional ? 2 : 1, pl.T = n_steps, pl.mode = mode;
    pl.G = NumGates(mode), pl.GR = ReserveGates(mode);
    HIPCX_REQUIRE(hx->ndim == 3 && hx->shape[0] == n_layers * pl.D, HIPCX_DIMENSION_ERROR,
                  "hx must have the shape [n_layers * directions, batch, units], got " + ShapeStr(hx));
    HIPCX_REQUIRE(hx->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: float32 only (compose the routine for other dtypes)");
    pl.B = hx->shape[1], pl.H = hx->shape[2];
    HIPCX_REQUIRE(pl.B > 0 && pl.H > 0 && pl.B < (1 << 24) && pl.H < (1 << 24), HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: empty or oversized state");
    for (int t = 0; t < n_steps; ++t) {
        ValidateArray(xs[t], "xs[t]");
        HIPCX_REQUIRE(xs[t]->ndim == 2, HIPCX_DIMENSION_ERROR, "every xs[t] must be a matrix");
        HIPCX_REQUIRE(xs[t]->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: float32 only");
        if (t == 0) pl.I = xs[0]->shape[1];
        HIPCX_REQUIRE(xs[t]->shape[1] == pl.I && pl.I > 0 && pl.I < (1 << 24), HIPCX_DIMENSION_ERROR, "every xs[t] must have the same number of columns");
        HIPCX_REQUIRE(xs[t]->shape[0] <= pl.B, HIPCX_DIMENSION_ERROR, "The batch size of x must be equal to or less than the size of state");
        HIPCX_REQUIRE(xs[t]->shape[0] > 0, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: empty time step");
        pl.row_start.push_back(pl.rows);
        pl.bt.push_back(xs[t]->shape[0]);
        pl.rows += xs[t]->shape[0];
    }
    HIPCX_REQUIRE(pl.rows * std::max<int64_t>(pl.I, 4 * pl.D * pl.H) < (int64_t{1} << 31), HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: sequence batch too large");
    pl.max_in = std::max(pl.I, pl.D * pl.H);
    size_t off = 0;
    for (int idx = 0; idx < pl.L * pl.D; ++idx) {
        pl.r_gates.push_back(off);
        off += Round256(static_cast<size_t>(pl.rows * pl.GR * pl.H) * 4);
        pl.r_hprev.push_back(off);
        off += Round256(static_cast<size_t>(pl.rows * pl.H) * 4);
        pl.r_cprev.push_back(off);
        if (mode == kLstm) off += Round256(static_cast<size_t>(pl.rows * pl.H) * 4);
    }
    for (int l = 0; l + 1 < pl.L; ++l) {
        pl.r_y.push_back(off);
        off += Round256(static_cast<size_t>(pl.rows * pl.D * pl.H) * 4);
    }
    pl.reserve_total = off;
    return pl;
}

// Hands out pieces of the workspace and runs the library calls of a pass.  In a dry run (base == nullptr) nothing is launched: the
// pieces get addresses relative to an aligned dummy base and the scratch need of every product / sum is recorded, which is how
// the workspace size of a pass is computed from the same code that later runs it.
class Pass {
public:
    Pass(void* base, size_t bytes, void* stream) : base_(static_cast<char*>(base)), bytes_(bytes), stream_(stream), dry_(base == nullptr) {
        if (dry_) base_ = reinterpret_cast<char*>(uintptr_t{1} << 20);
    }
    bool dry() const { return dry_; }
    hipStream_t hip_stream() const { return AsStream(stream_); }
    float* Take(int64_t floats) {
        float* p = reinterpret_cast<float*>(base_ + used_);
        used_ += Round256(static_cast<size_t>(floats) * 4);
        return p;
    }
    // everything after the pieces is scratch for the library calls; call once all pieces are taken
    void StartScratch() { scratch_off_ = used_; }
    size_t Need() const { return scratch_off_ + scratch_need_; }
    void CheckFits() const {
        HIPCX_REQUIRE(dry_ || Need() <= bytes_, HIPCX_CHAINERX_ERROR, "n_step_rnn workspace too small: need " + std::to_string(Need()) + " bytes");
    }
    void Dot(const hipcx_array& a, const hipcx_array& b, const hipcx_array& out) {
        const size_t need = hipcx_dot_workspace_size(&a, &b, &out);
        if (dry_) {
            scratch_need_ = std::max(scratch_need_, Round256(need));
            return;
        }
        HIPCX_REQUIRE(scratch_off_ + need <= bytes_, HIPCX_CHAINERX_ERROR, "n_step_rnn workspace too small for a matrix product");
        CheckStatus(hipcx_dot(&a, &b, &out, base_ + scratch_off_, bytes_ - scratch_off_, stream_));
    }
    void SumRows(const hipcx_array& a, const hipcx_array& out) {
        const int8_t axis = 0;
        const size_t need = hipcx_reduce_workspace_size(&a, &axis, 1, &out);
        if (dry_) {
            scratch_need_ = std::max(scratch_need_, Round256(need));
            return;
        }
        HIPCX_REQUIRE(scratch_off_ + need <= bytes_, HIPCX_CHAINERX_ERROR, "n_step_rnn workspace too small for a sum");
        CheckStatus(hipcx_sum(&a, &axis, 1, &out, base_ + scratch_off_, bytes_ - scratch_off_, stream_));
    }
    void Copy(const hipcx_array& a, const hipcx_array& out) {
        if (!dry_) CheckStatus(hipcx_copy(&a, &out, stream_));
    }
    void Add(const hipcx_array& a, const hipcx_array& b, const hipcx_array& out) {
        if (!dry_) CheckStatus(hipcx_add(&a, &b, &out, stream_));
    }
    void Zero(const hipcx_array& out) {
        hipcx_scalar zero{};
        zero.kind = HIPCX_KIND_INT;
        if (!dry_) CheckStatus(hipcx_fill(&out, zero, stream_));
    }

private:
    char* base_;
    size_t bytes_;
    void* stream_;
    bool dry_;
    size_t used_ = 0, scratch_off_ = 0, scratch_need_ = 0;
};

struct PackedWeights {
    std::vector<float*> wx, wh, bx, bh;  // per layer-direction: [G*H][in], [G*H][H], [G*H], [G*H]
};

// Stacks the matrices and biases of every layer-direction, gate-major: rows [g*H, (g+1)*H) of wx are ws[idx][g], of wh ws[idx][G + g].
PackedWeights PackWeights(Pass& pass, const RnnPlan& pl, const hipcx_array* const* ws, const hipcx_array* const* bs) {
    PackedWeights pw;
    const int G = pl.G;
    for (int idx = 0; idx < pl.L * pl.D; ++idx) {
        const int64_t in = pl.In(idx / pl.D);
        pw.wx.push_back(pass.Take(G * pl.H * in));
        pw.wh.push_back(pass.Take(G * pl.H * pl.H));
        pw.bx.push_back(pass.Take(G * pl.H));
        pw.bh.push_back(pass.Take(G * pl.H));
        if (pass.dry()) continue;
        for (int g = 0; g < 2 * G; ++g) {
            const hipcx_array* w = ws[idx * 2 * G + g];
            const hipcx_array* b = bs[idx * 2 * G + g];
            const bool xside = g < G;
            const int64_t cols = xside ? in : pl.H;
            float* wdst = (xside ? pw.wx[idx] : pw.wh[idx]) + static_cast<int64_t>(g % G) * pl.H * cols;
            float* bdst = (xside ? pw.bx[idx] : pw.bh[idx]) + static_cast<int64_t>(g % G) * pl.H;
            pass.Copy(*w, Matrix(wdst, pl.H, cols, cols));
            pass.Copy(*b, Vector(bdst, pl.H));
        }
    }
    return pw;
}

void CheckParameters(const RnnPlan& pl, const hipcx_array* const* ws, const hipcx_array* const* bs, const char* what) {
    HIPCX_REQUIRE(ws != nullptr && bs != nullptr, HIPCX_CHAINERX_ERROR, std::string(what) + " is null");
    for (int idx = 0; idx < pl.L * pl.D; ++idx) {
        const int64_t in = pl.In(idx / pl.D);
        for (int g = 0; g < 2 * pl.G; ++g) {
            const hipcx_array* w = ws[idx * 2 * pl.G + g];
            const hipcx_array* b = bs[idx * 2 * pl.G + g];
            ValidateArray(w, "ws[i]");
            ValidateArray(b, "bs[i]");
            HIPCX_REQUIRE(w->dtype == HIPCX_FLOAT32 && b->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: float32 only");
            HIPCX_REQUIRE(w->ndim == 2 && w->shape[0] == pl.H && w->shape[1] == (g < pl.G ? in : pl.H), HIPCX_DIMENSION_ERROR,
                          std::string(what) + ": matrix " + std::to_string(g) + " of layer-direction " + std::to_string(idx) + " has the wrong shape " +
                                  ShapeStr(w));
            HIPCX_REQUIRE(b->ndim == 1 && b->shape[0] == pl.H, HIPCX_DIMENSION_ERROR, std::string(what) + ": every bias must have one value per unit");
        }
    }
}

void CheckState(const RnnPlan& pl, const hipcx_array* a, const char* name) {
    ValidateArray(a, name);
    HIPCX_REQUIRE(a->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: float32 only");
    HIPCX_REQUIRE(a->ndim == 3 && a->shape[0] == pl.L * pl.D && a->shape[1] == pl.B && a->shape[2] == pl.H, HIPCX_DIMENSION_ERROR,
                  std::string(name) + " must have hx's shape, got " + ShapeStr(a));
}

hipcx_array StateSlice(const hipcx_array* a, int idx) {  // [B][H] view of a[idx]
    hipcx_array m{};
    m.data = static_cast<char*>(a->data) + idx * a->strides[0];
    m.dtype = HIPCX_FLOAT32;
    m.ndim = 2;
    m.shape[0] = a->shape[1], m.shape[1] = a->shape[2];
    m.strides[0] = a->strides[1], m.strides[1] = a->strides[2];
    return m;
}

void CheckStepArrays(const RnnPlan& pl, const hipcx_array* const* arrays, int64_t cols, const char* name, bool nullable) {
    HIPCX_REQUIRE(arrays != nullptr, HIPCX_CHAINERX_ERROR, std::string(name) + " is null");
    for (int t = 0; t < pl.T; ++t) {
        if (arrays[t] == nullptr && nullable) continue;
        ValidateArray(arrays[t], name);
        HIPCX_REQUIRE(arrays[t]->dtype == HIPCX_FLOAT32, HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn: float32 only");
        HIPCX_REQUIRE(arrays[t]->ndim == 2 && arrays[t]->shape[0] == pl.bt[t] && arrays[t]->shape[1] == cols, HIPCX_DIMENSION_ERROR,
                      std::string(name) + "[t] must have the shape [batch of step t, " + std::to_string(cols) + "], got " + ShapeStr(arrays[t]));
    }
}

unsigned CellBlocks(int64_t items) {
    int64_t b = (items + 255) / 256;
    const int64_t cap = static_cast<int64_t>(NumCUs()) * 8;
    return static_cast<unsigned>(b > cap ? cap : (b < 1 ? 1 : b));
}

// ---- forward ----
void RunForward(Pass& pass, const RnnPlan& pl, int activation, const hipcx_array* hx, const hipcx_array* cx, const hipcx_array* const* ws,
                const hipcx_array* const* bs, const hipcx_array* const* xs, const hipcx_array* hy, const hipcx_array* cy,
                const hipcx_array* const* ys, char* reserve) {
    const int64_t B = pl.B, H = pl.H, GH = pl.G * H, DH = pl.D * H, rows = pl.rows;
    PackedWeights pw = PackWeights(pass, pl, ws, bs);
    float* x_all = pass.Take(rows * pl.I);
    float* y_buf[2] = {nullptr, nullptr};
    if (reserve == nullptr && pl.L > 1) {
        y_buf[0] = pass.Take(rows * DH);
        if (pl.L > 2) y_buf[1] = pass.Take(rows * DH);
    }
    float* xw_all = pass.Take(rows * GH);
    float* hw = pass.Take(B * GH);
    float* h_state = pass.Take(B * H);
    float* c_state = pl.mode == kLstm ? pass.Take(B * H) : nullptr;
    pass.StartScratch();
    for (int t = 0; t < pl.T; ++t) pass.Copy(*xs[t], Matrix(x_all + pl.row_start[t] * pl.I, pl.bt[t], pl.I, pl.I));
    for (int l = 0; l < pl.L; ++l) {
        const int64_t in = pl.In(l);
        const float* x_in = l == 0 ? x_all : (reserve != nullptr ? reinterpret_cast<float*>(reserve + pl.r_y[l - 1]) : y_buf[(l - 1) & 1]);
        float* y_out = l + 1 == pl.L ? nullptr : (reserve != nullptr ? reinterpret_cast<float*>(reserve + pl.r_y[l]) : y_buf[l & 1]);
        for (int d = 0; d < pl.D; ++d) {
            const int idx = l * pl.D + d;
            // the input projection of every step at once
            pass.Dot(Matrix(x_in, rows, in, in), Matrix(pw.wx[idx], in, GH, 1, in), Matrix(xw_all, rows, GH, GH));
            pass.Copy(StateSlice(hx, idx), Matrix(h_state, B, H, H));
            if (pl.mode == kLstm) pass.Copy(StateSlice(cx, idx), Matrix(c_state, B, H, H));
            for (int s = 0; s < pl.T; ++s) {
                const int t = d == 0 ? s : pl.T - 1 - s;
                const int64_t bt = pl.bt[t], r0 = pl.row_start[t];
                pass.Dot(Matrix(h_state, bt, H, H), Matrix(pw.wh[idx], H, GH, 1, H), Matrix(hw, bt, GH, GH));
                if (pass.dry()) continue;
                CellArgs a{};
                a.mode = pl.mode, a.relu = activation == 1;
                a.Bt = static_cast<int>(bt), a.H = static_cast<int>(H);
                a.xw = xw_all + r0 * GH;
                a.hw = hw;
                a.bx = pw.bx[idx], a.bh = pw.bh[idx];
                a.h = h_state, a.c = c_state;
                if (y_out != nullptr) {
                    a.y = y_out + r0 * DH + d * H;
                    a.y_stride = DH;
                } else {
                    a.y = static_cast<float*>(ys[t]->data) + d * H;
                    a.y_stride = ys[t]->strides[0] / 4;
                }
                if (reserve != nullptr) {
                    a.gates = reinterpret_cast<float*>(reserve + pl.r_gates[idx]) + r0 * pl.GR * H;
                    a.hprev = reinterpret_cast<float*>(reserve + pl.r_hprev[idx]) + r0 * H;
                    a.cprev = pl.mode == kLstm ? reinterpret_cast<float*>(reserve + pl.r_cprev[idx]) + r0 * H : nullptr;
                }
                hipLaunchKernelGGL(RnnCellKernel, dim3(CellBlocks(bt * H)), dim3(256), 0, pass.hip_stream(), a);
                CheckLaunch("rnn_cell");
            }
            pass.Copy(Matrix(h_state, B, H, H), StateSlice(hy, idx));
            if (pl.mode == kLstm) pass.Copy(Matrix(c_state, B, H, H), StateSlice(cy, idx));
        }
    }
    pass.CheckFits();
}

// ---- backward ----
void RunBackward(Pass& pass, const RnnPlan& pl, int activation, const hipcx_array* const* ws, const hipcx_array* const* bs,
                 const hipcx_array* const* xs, const hipcx_array* dhy, const hipcx_array* dcy, const hipcx_array* const* dys, const char* reserve,
                 const hipcx_array* dhx, const hipcx_array* dcx, const hipcx_array* const* dws, const hipcx_array* const* dbs,
                 const hipcx_array* const* dxs) {
    const int64_t B = pl.B, H = pl.H, GH = pl.G * H, DH = pl.D * H, rows = pl.rows;
    PackedWeights pw = PackWeights(pass, pl, ws, bs);
    float* x_all = pass.Take(rows * pl.I);
    float* dy_cur = pass.Take(rows * pl.max_in);   // gradient of the current layer's output rows [rows][D*H]
    float* dx_acc = pass.Take(rows * pl.max_in);   // gradient of its input rows [rows][in]
    float* dx_tmp = pl.D == 2 ? pass.Take(rows * pl.max_in) : nullptr;
    float* dgx_all = pass.Take(rows * GH);
    float* dgh_all = pl.mode == kGru ? pass.Take(rows * GH) : dgx_all;
    float* dh = pass.Take(B * H);
    float* dc = pl.mode == kLstm ? pass.Take(B * H) : nullptr;
    float* tmp = pass.Take(B * H);
    pass.StartScratch();
    for (int t = 0; t < pl.T; ++t) pass.Copy(*xs[t], Matrix(x_all + pl.row_start[t] * pl.I, pl.bt[t], pl.I, pl.I));
    for (int t = 0; t < pl.T; ++t) {
        const hipcx_array dst = Matrix(dy_cur + pl.row_start[t] * DH, pl.bt[t], DH, DH);
        if (dys[t] != nullptr) pass.Copy(*dys[t], dst);
        else pass.Zero(dst);
    }
    for (int l = pl.L - 1; l >= 0; --l) {
        const int64_t in = pl.In(l);
        const float* x_in = l == 0 ? x_all : reinterpret_cast<const float*>(reserve + pl.r_y[l - 1]);
        for (int d = 0; d < pl.D; ++d) {
            const int idx = l * pl.D + d;
            const float* gates = reinterpret_cast<const float*>(reserve + pl.r_gates[idx]);
            const float* hprev = reinterpret_cast<const float*>(reserve + pl.r_hprev[idx]);
            const float* cprev = pl.mode == kLstm ? reinterpret_cast<const float*>(reserve + pl.r_cprev[idx]) : nullptr;
            pass.Copy(StateSlice(dhy, idx), Matrix(dh, B, H, H));
            if (pl.mode == kLstm) {
                if (dcy != nullptr) pass.Copy(StateSlice(dcy, idx), Matrix(dc, B, H, H));
                else pass.Zero(Matrix(dc, B, H, H));
            }
            for (int s = pl.T - 1; s >= 0; --s) {  // the forward order of this direction, backwards
                const int t = d == 0 ? s : pl.T - 1 - s;
                const int64_t bt = pl.bt[t], r0 = pl.row_start[t];
                if (!pass.dry()) {
                    CellGradArgs a{};
                    a.mode = pl.mode, a.relu = activation == 1;
                    a.Bt = static_cast<int>(bt), a.H = static_cast<int>(H);
                    a.dy = dy_cur + r0 * DH + d * H;
                    a.dy_stride = DH;
                    a.dh = dh, a.dc = dc;
                    a.gates = gates + r0 * pl.GR * H;
                    a.hprev = hprev + r0 * H;
                    a.cprev = cprev != nullptr ? cprev + r0 * H : nullptr;
                    a.dgx = dgx_all + r0 * GH;
                    a.dgh = dgh_all + r0 * GH;
                    hipLaunchKernelGGL(RnnCellGradKernel, dim3(CellBlocks(bt * H)), dim3(256), 0, pass.hip_stream(), a);
                    CheckLaunch("rnn_cell_grad");
                }
                // dh of the state before the step: what the cell left there plus dGh . Wh
                pass.Dot(Matrix(dgh_all + r0 * GH, bt, GH, GH), Matrix(pw.wh[idx], GH, H, H), Matrix(tmp, bt, H, H));
                pass.Add(Matrix(dh, bt, H, H), Matrix(tmp, bt, H, H), Matrix(dh, bt, H, H));
            }
            pass.Copy(Matrix(dh, B, H, H), StateSlice(dhx, idx));
            if (pl.mode == kLstm) pass.Copy(Matrix(dc, B, H, H), StateSlice(dcx, idx));
            // parameter gradients over all rows at once
            for (int g = 0; g < pl.G; ++g) {
                const hipcx_array gx_t = Matrix(dgx_all + g * H, H, rows, 1, GH);  // dGx[:, g]^T
                const hipcx_array gh_t = Matrix(dgh_all + g * H, H, rows, 1, GH);
                pass.Dot(gx_t, Matrix(x_in, rows, in, in), *dws[idx * 2 * pl.G + g]);
                pass.Dot(gh_t, Matrix(hprev, rows, H, H), *dws[idx * 2 * pl.G + pl.G + g]);
                pass.SumRows(Matrix(dgx_all + g * H, rows, H, GH), *dbs[idx * 2 * pl.G + g]);
                pass.SumRows(Matrix(dgh_all + g * H, rows, H, GH), *dbs[idx * 2 * pl.G + pl.G + g]);
            }
            // gradient of the layer's input rows; the second direction adds to the first
            if (d == 0) {
                pass.Dot(Matrix(dgx_all, rows, GH, GH), Matrix(pw.wx[idx], GH, in, in), Matrix(dx_acc, rows, in, in));
            } else {
                pass.Dot(Matrix(dgx_all, rows, GH, GH), Matrix(pw.wx[idx], GH, in, in), Matrix(dx_tmp, rows, in, in));
                pass.Add(Matrix(dx_acc, rows, in, in), Matrix(dx_tmp, rows, in, in), Matrix(dx_acc, rows, in, in));
            }
        }
        std::swap(dy_cur, dx_acc);  // the layer below produced these rows
    }
    for (int t = 0; t < pl.T; ++t) pass.Copy(Matrix(dy_cur + pl.row_start[t] * pl.I, pl.bt[t], pl.I, pl.I), *dxs[t]);
    pass.CheckFits();
}

bool FastLstmApplies(const RnnPlan& pl, const void* reserve) { return pl.mode == kLstm && pl.D == 1 && reserve == nullptr; }

}  // namespace
}  // namespace hipcx

using namespace hipcx;

extern "C" {

size_t hipcx_n_step_rnn_reserve_size(int n_layers, int bidirectional, int mode, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps) {
    try {
        return MakePlan(n_layers, bidirectional, mode, hx, xs, n_steps).reserve_total;
    } catch (...) {
        return 0;
    }
}

size_t hipcx_n_step_rnn_workspace_size(int n_layers, int bidirectional, int mode, int training, const hipcx_array* hx, const hipcx_array* const* xs,
                                       int n_steps) {
    try {
        const RnnPlan pl = MakePlan(n_layers, bidirectional, mode, hx, xs, n_steps);
        if (!training && pl.mode == kLstm && pl.D == 1) return hipcx_n_step_lstm_workspace_size(n_layers, hx, xs, n_steps);
        // a dry run over stand-ins for the caller's arrays: dense arrays of the right shapes
        std::vector<hipcx_array> w, b, y;
        std::vector<const hipcx_array*> pw, pb, py;
        for (int idx = 0; idx < pl.L * pl.D; ++idx) {
            for (int g = 0; g < 2 * pl.G; ++g) {
                const int64_t cols = g < pl.G ? pl.In(idx / pl.D) : pl.H;
                w.push_back(Matrix(reinterpret_cast<void*>(uintptr_t{1} << 20), pl.H, cols, cols));
                b.push_back(Vector(reinterpret_cast<void*>(uintptr_t{1} << 20), pl.H));
            }
        }
        for (int t = 0; t < pl.T; ++t) y.push_back(Matrix(reinterpret_cast<void*>(uintptr_t{1} << 20), pl.bt[t], pl.D * pl.H, pl.D * pl.H));
        for (auto& a : w) pw.push_back(&a);
        for (auto& a : b) pb.push_back(&a);
        for (auto& a : y) py.push_back(&a);
        char* fake_reserve = training ? reinterpret_cast<char*>(uintptr_t{1} << 30) : nullptr;
        Pass fwd(nullptr, 0, nullptr);
        RunForward(fwd, pl, 0, hx, hx, pw.data(), pb.data(), xs, hx, hx, py.data(), fake_reserve);
        size_t need = fwd.Need();
        if (training) {
            Pass bwd(nullptr, 0, nullptr);
            RunBackward(bwd, pl, 0, pw.data(), pb.data(), xs, hx, hx, py.data(), fake_reserve, hx, hx, pw.data(), pb.data(), xs);
            need = std::max(need, bwd.Need());
        }
        return need + 4096;  // the caller's arrays may be aligned differently from the stand-ins
    } catch (...) {
        return 0;
    }
}

int hipcx_n_step_rnn(int n_layers, int bidirectional, int mode, int activation, const hipcx_array* hx, const hipcx_array* cx,
                     const hipcx_array* const* ws, const hipcx_array* const* bs, const hipcx_array* const* xs, int n_steps, const hipcx_array* hy,
                     const hipcx_array* cy, const hipcx_array* const* ys, void* reserve, size_t reserve_bytes, void* workspace,
                     size_t workspace_bytes, void* stream) {
    return Guard([&] {
        const RnnPlan pl = MakePlan(n_layers, bidirectional, mode, hx, xs, n_steps);
        HIPCX_REQUIRE(activation == 0 || activation == 1, HIPCX_CHAINERX_ERROR, "n_step_rnn: activation must be 0 (tanh) or 1 (relu)");
        CheckParameters(pl, ws, bs, "ws / bs");
        CheckState(pl, hx, "hx");
        CheckState(pl, hy, "hy");
        if (pl.mode == kLstm) {
            CheckState(pl, cx, "cx");
            CheckState(pl, cy, "cy");
        }
        CheckStepArrays(pl, ys, pl.D * pl.H, "ys", false);
        for (int t = 0; t < pl.T; ++t) {
            HIPCX_REQUIRE(ys[t]->strides[1] == 4 && ys[t]->strides[0] % 4 == 0, HIPCX_NOT_IMPLEMENTED_ERROR,
                          "hip n_step_rnn: ys[t] needs unit stride along its last axis");
        }
        HIPCX_REQUIRE(workspace != nullptr && reinterpret_cast<uintptr_t>(workspace) % 256 == 0, HIPCX_CHAINERX_ERROR,
                      "n_step_rnn: workspace must be 256-byte aligned device memory");
        HIPCX_REQUIRE(reserve == nullptr || (reserve_bytes >= pl.reserve_total && reinterpret_cast<uintptr_t>(reserve) % 256 == 0),
                      HIPCX_CHAINERX_ERROR, "n_step_rnn: reserve too small or not 256-byte aligned: need " + std::to_string(pl.reserve_total) + " bytes");
        if (FastLstmApplies(pl, reserve)) {
            CheckStatus(hipcx_n_step_lstm(n_layers, hx, cx, ws, bs, xs, n_steps, hy, cy, ys, workspace, workspace_bytes, stream));
            return;
        }
        Pass pass(workspace, workspace_bytes, stream);
        RunForward(pass, pl, activation, hx, cx, ws, bs, xs, hy, cy, ys, static_cast<char*>(reserve));
    });
}

int hipcx_n_step_rnn_backward(int n_layers, int bidirectional, int mode, int activation, const hipcx_array* hx, const hipcx_array* const* ws,
                              const hipcx_array* const* bs, const hipcx_array* const* xs, int n_steps, const hipcx_array* dhy,
                              const hipcx_array* dcy, const hipcx_array* const* dys, const void* reserve, size_t reserve_bytes,
                              const hipcx_array* dhx, const hipcx_array* dcx, const hipcx_array* const* dws, const hipcx_array* const* dbs,
                              const hipcx_array* const* dxs, void* workspace, size_t workspace_bytes, void* stream) {
    return Guard([&] {
        const RnnPlan pl = MakePlan(n_layers, bidirectional, mode, hx, xs, n_steps);
        HIPCX_REQUIRE(activation == 0 || activation == 1, HIPCX_CHAINERX_ERROR, "n_step_rnn: activation must be 0 (tanh) or 1 (relu)");
        CheckParameters(pl, ws, bs, "ws / bs");
        CheckParameters(pl, dws, dbs, "dws / dbs");
        for (int i = 0; i < pl.L * pl.D * 2 * pl.G; ++i) {
            HIPCX_REQUIRE(IsContiguous(dws[i]) && IsContiguous(dbs[i]), HIPCX_NOT_IMPLEMENTED_ERROR, "hip n_step_rnn_backward: dws and dbs must be C-contiguous");
        }
        CheckState(pl, dhy, "dhy");
        CheckState(pl, dhx, "dhx");
        if (pl.mode == kLstm) {
            if (dcy != nullptr) CheckState(pl, dcy, "dcy");
            CheckState(pl, dcx, "dcx");
        }
        CheckStepArrays(pl, dys, pl.D * pl.H, "dys", true);
        CheckStepArrays(pl, dxs, pl.I, "dxs", false);
        HIPCX_REQUIRE(reserve != nullptr && reserve_bytes >= pl.reserve_total, HIPCX_CHAINERX_ERROR,
                      "n_step_rnn_backward: needs the reserve the forward pass filled (" + std::to_string(pl.reserve_total) + " bytes)");
        HIPCX_REQUIRE(workspace != nullptr && reinterpret_cast<uintptr_t>(workspace) % 256 == 0, HIPCX_CHAINERX_ERROR,
                      "n_step_rnn_backward: workspace must be 256-byte aligned device memory");
        Pass pass(workspace, workspace_bytes, stream);
        RunBackward(pass, pl, activation, ws, bs, xs, dhy, dcy, dys, static_cast<const char*>(reserve), dhx, dcx, dws, dbs, dxs);
    });
}

}  // extern "C"
