/*
 * CPU restatement of the ChainerX *native* backend for the kernels on the hip backend's path.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the parity oracle and the "cpu_baseline" of bench.py.
 * Nothing in the product (chainer_amd/) links, imports or calls it.
 *
 * Every function names the reference code it follows (paths relative to the reference tree,
 * CX/ = chainerx_cc/chainerx/).  Single-threaded scalar loops, like the native backend itself.
 * Build: see oracle/Makefile (-ffp-contract=off so that only the explicit fmaf/fma calls fuse).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------
 * Float16 <-> float: CX/float16.cc:27-89 (FloatbitsToHalfbits, round-to-nearest-even with
 * subnormals, overflow to inf, NaN payload kept) and :161-193 (HalfbitsToFloatbits).
 * ------------------------------------------------------------------------------------------ */
static uint16_t float_to_half_bits(float value) {
    uint32_t f;
    memcpy(&f, &value, 4);
    uint16_t sign = (uint16_t)((f >> 16) & 0x8000u);
    uint32_t expo = f & 0x7f800000u;
    uint32_t mant = f & 0x007fffffu;
    if (expo >= 0x47800000u) { /* too large for half, inf or NaN */
        if (expo == 0x7f800000u && mant != 0) {
            uint16_t r = (uint16_t)(0x7c00u + (mant >> 13));
            if (r == 0x7c00u) r++; /* keep it a NaN */
            return (uint16_t)(sign + r);
        }
        return (uint16_t)(sign + 0x7c00u);
    }
    if (expo <= 0x38000000u) { /* half subnormal or zero */
        if (expo < 0x33000000u) return sign;
        uint32_t e = expo >> 23;
        uint32_t sig = (0x00800000u + mant) >> (113 - e);
        if (((sig & 0x00003fffu) != 0x00001000u) || ((f & 0x000007ffu) != 0)) sig += 0x00001000u;
        return (uint16_t)(sign + (uint16_t)(sig >> 13));
    }
    uint16_t hexp = (uint16_t)((expo - 0x38000000u) >> 13);
    if ((mant & 0x00003fffu) != 0x00001000u) mant += 0x00001000u; /* ties to even */
    return (uint16_t)(sign + hexp + (uint16_t)(mant >> 13));
}

static float half_bits_to_float(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint16_t expo = h & 0x7c00u;
    uint32_t out;
    if (expo == 0) {
        uint16_t sig = h & 0x03ffu;
        if (sig == 0) {
            out = sign;
        } else {
            int shift = 0;
            sig <<= 1;
            while ((sig & 0x0400u) == 0) {
                sig <<= 1;
                shift++;
            }
            out = sign + ((uint32_t)(127 - 15 - shift) << 23) + ((uint32_t)(sig & 0x03ffu) << 13);
        }
    } else if (expo == 0x7c00u) {
        out = sign + 0x7f800000u + ((uint32_t)(h & 0x03ffu) << 13);
    } else {
        out = sign + (((uint32_t)(h & 0x7fffu) + 0x1c000u) << 13);
    }
    float r;
    memcpy(&r, &out, 4);
    return r;
}

void oracle_float_to_half(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = float_to_half_bits(in[i]);
}

void oracle_half_to_float(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = half_bits_to_float(in[i]);
}

/* ------------------------------------------------------------------------------------------
 * Pairwise reduction order of CX/native/reduce.h:46-83 (ExpandLen 4, SerialLen 8, binary-counter
 * tree), instantiated for Sum (CX/native/native_device/reduction.cc:96-119), AMax
 * (CX/native/native_device/statistics.cc:27-48) and ArgMax (reduction.cc:34-61).
 *
 * The macro below restates PairwiseReduction for an accumulator type ACC, given
 *   IDENT           -- impl.Identity()
 *   MAP(i)          -- impl.MapIn(in[i], i)
 *   REDUCE(next,acc)-- impl.Reduce(next, accum)   (a statement updating `acc`)
 * `in` is one row of `len` elements with element stride 1.
 * ------------------------------------------------------------------------------------------ */
#define PAIRWISE_BODY(ACC, IDENT, MAP, REDUCE)                                              \
    ACC accum = IDENT;                                                                      \
    ACC tree[64];                                                                           \
    int64_t i = 0;                                                                          \
    const int64_t main_len = len - (len % 4);                                               \
    while (i < main_len) {                                                                  \
        if (i != 0 && i % 32 == 0) {                                                        \
            int lvl = 0;                                                                    \
            for (int64_t k = i >> 1; k % 32 == 0; k >>= 1, ++lvl) {                         \
                ACC nx = tree[lvl];                                                         \
                REDUCE(nx, accum);                                                          \
            }                                                                               \
            tree[lvl] = accum;                                                              \
            accum = IDENT;                                                                  \
        }                                                                                   \
        /* expanded group of four: (e0 . e1) . (e2 . e3), later element is `next` */        \
        ACC p0 = MAP(i);                                                                    \
        {                                                                                   \
            ACC nx = MAP(i + 1);                                                            \
            REDUCE(nx, p0);                                                                 \
        }                                                                                   \
        ACC p1 = MAP(i + 2);                                                                \
        {                                                                                   \
            ACC nx = MAP(i + 3);                                                            \
            REDUCE(nx, p1);                                                                 \
        }                                                                                   \
        REDUCE(p1, p0);                                                                     \
        REDUCE(p0, accum);                                                                  \
        i += 4;                                                                             \
    }                                                                                       \
    while (i < len) {                                                                       \
        ACC nx = MAP(i);                                                                    \
        REDUCE(nx, accum);                                                                  \
        ++i;                                                                                \
    }                                                                                       \
    {                                                                                       \
        int lvl = 0;                                                                        \
        for (int64_t k = (len / 4 - 1) / 8; k > 0; k >>= 1, ++lvl) {                        \
            if (k & 1) {                                                                    \
                ACC nx = tree[lvl];                                                         \
                REDUCE(nx, accum);                                                          \
            }                                                                               \
        }                                                                                   \
    }

#define SUM_REDUCE(next, acc) acc += next

#define DEFINE_SUM(NAME, IN_T, ACC_T, LOAD)                                       \
    static ACC_T NAME(const IN_T* in, int64_t len) {                              \
        PAIRWISE_BODY(ACC_T, (ACC_T)0, LOAD, SUM_REDUCE)                          \
        return accum;                                                             \
    }

#define LOAD_F32(i) ((float)in[i])
#define LOAD_F64(i) ((double)in[i])
#define LOAD_I64(i) ((int64_t)in[i])
#define LOAD_H32(i) (half_bits_to_float(in[i]))

DEFINE_SUM(sum_row_f32, float, float, LOAD_F32)
DEFINE_SUM(sum_row_f64, double, double, LOAD_F64)
DEFINE_SUM(sum_row_i64, int64_t, int64_t, LOAD_I64)
DEFINE_SUM(sum_row_f16, uint16_t, float, LOAD_H32) /* Accum = float when Out is Float16 (reduction.cc:105) */

/* rows x len, contiguous; out[r] */
void oracle_sum_f32(const float* in, int64_t rows, int64_t len, float* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = sum_row_f32(in + r * len, len);
}
void oracle_sum_f64(const double* in, int64_t rows, int64_t len, double* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = sum_row_f64(in + r * len, len);
}
void oracle_sum_i64(const int64_t* in, int64_t rows, int64_t len, int64_t* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = sum_row_i64(in + r * len, len);
}
void oracle_sum_f16(const uint16_t* in, int64_t rows, int64_t len, uint16_t* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = float_to_half_bits(sum_row_f16(in + r * len, len));
}

/* AMax: Reduce(next, accum): if (IsNan(next) || accum < next) accum = next; identity = lowest/-inf */
#define AMAX_REDUCE_F(next, acc) \
    if (isnan(next) || acc < next) acc = next
#define AMAX_REDUCE_I(next, acc) \
    if (acc < next) acc = next

static float amax_row_f32(const float* in, int64_t len) {
    PAIRWISE_BODY(float, -HUGE_VALF, LOAD_F32, AMAX_REDUCE_F)
    return accum;
}
static double amax_row_f64(const double* in, int64_t len) {
    PAIRWISE_BODY(double, -HUGE_VAL, LOAD_F64, AMAX_REDUCE_F)
    return accum;
}
static int64_t amax_row_i64(const int64_t* in, int64_t len, int64_t lowest) {
    PAIRWISE_BODY(int64_t, lowest, LOAD_I64, AMAX_REDUCE_I)
    return accum;
}
void oracle_amax_f32(const float* in, int64_t rows, int64_t len, float* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = amax_row_f32(in + r * len, len);
}
void oracle_amax_f64(const double* in, int64_t rows, int64_t len, double* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = amax_row_f64(in + r * len, len);
}
/* integer dtypes are widened to int64 by the caller; `lowest` is the dtype's minimum */
void oracle_amax_i64(const int64_t* in, int64_t rows, int64_t len, int64_t lowest, int64_t* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = amax_row_i64(in + r * len, len, lowest);
}

/* ArgMax: accumulator {max, argmax}; identity {0, -1};
 * Reduce(next, accum): if (accum.argmax < 0 || accum.max < next.max) accum = next. */
typedef struct {
    double max; /* every dtype on the path converts to double exactly (int64 inputs beyond 2^53 excluded) */
    int64_t argmax;
} max_and_argmax;
#define ARG_MAP(i) ((max_and_argmax){(double)in[i], (i)})
#define ARG_REDUCE(next, acc) \
    if (acc.argmax < 0 || acc.max < next.max) acc = next
static const max_and_argmax kArgIdentity = {0.0, -1};

static int64_t argmax_row_f64(const double* in, int64_t len) {
    PAIRWISE_BODY(max_and_argmax, kArgIdentity, ARG_MAP, ARG_REDUCE)
    return accum.argmax;
}
/* the caller widens the row to double (exact for bool, (u)int8/16/32, float16/32/64) */
void oracle_argmax(const double* in, int64_t rows, int64_t len, int64_t* out) {
    for (int64_t r = 0; r < rows; ++r) out[r] = argmax_row_f64(in + r * len, len);
}

/* ------------------------------------------------------------------------------------------
 * Dot without BLAS: CX/native/native_device/dot.cc:181-227.  i, l, j loop order, one fused
 * multiply-add per term into an accumulator array that starts at zero; float16 inputs are
 * multiplied as floats into a float accumulator and rounded once at the end.
 * a[m,k], b[k,n], out[m,n] contiguous.
 * ------------------------------------------------------------------------------------------ */
void oracle_dot_f32(const float* a, const float* b, float* out, int64_t m, int64_t k, int64_t n) {
    memset(out, 0, sizeof(float) * (size_t)(m * n));
    for (int64_t i = 0; i < m; ++i) {
        float* acc = out + i * n;
        for (int64_t l = 0; l < k; ++l) {
            const float av = a[i * k + l];
            const float* brow = b + l * n;
            for (int64_t j = 0; j < n; ++j) acc[j] = fmaf(av, brow[j], acc[j]);
        }
    }
}

void oracle_dot_f64(const double* a, const double* b, double* out, int64_t m, int64_t k, int64_t n) {
    memset(out, 0, sizeof(double) * (size_t)(m * n));
    for (int64_t i = 0; i < m; ++i) {
        double* acc = out + i * n;
        for (int64_t l = 0; l < k; ++l) {
            const double av = a[i * k + l];
            const double* brow = b + l * n;
            for (int64_t j = 0; j < n; ++j) acc[j] = fma(av, brow[j], acc[j]);
        }
    }
}

/* float16: returns half bits; `acc` scratch is allocated here */
int oracle_dot_f16(const uint16_t* a, const uint16_t* b, uint16_t* out, int64_t m, int64_t k, int64_t n) {
    float* bf = (float*)malloc(sizeof(float) * (size_t)(k * n > 0 ? k * n : 1));
    float* acc = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    if (!bf || !acc) {
        free(bf);
        free(acc);
        return -1;
    }
    for (int64_t e = 0; e < k * n; ++e) bf[e] = half_bits_to_float(b[e]);
    for (int64_t i = 0; i < m; ++i) {
        for (int64_t j = 0; j < n; ++j) acc[j] = 0.f;
        for (int64_t l = 0; l < k; ++l) {
            const float av = half_bits_to_float(a[i * k + l]);
            const float* brow = bf + l * n;
            for (int64_t j = 0; j < n; ++j) acc[j] = fmaf(av, brow[j], acc[j]);
        }
        for (int64_t j = 0; j < n; ++j) out[i * n + j] = float_to_half_bits(acc[j]);
    }
    free(bf);
    free(acc);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Conv forward: CX/native/native_device/conv.cc:41-89 = Im2Col with zero padding
 * (CX/native/im2col.cc:82-149) + TensorDot over (channel, kh, kw) (CX/native/tensor_dot.cc:63-99,
 * i.e. the Dot above with l running over c, kh, kw in that order) + bias added to the rounded
 * result (`y += b`, in the output dtype) .  x[N,C,H,W], w[K,C,kh,kw] contiguous; out is written
 * as contiguous NCHW (the native result is the same values seen through an NHWC-backed view).
 * cover_all only changes OH/OW (CX/routines/connection.cc:37-49); positions beyond the padded
 * input read zeros (im2col.cc:93-97).
 * ------------------------------------------------------------------------------------------ */
#define DEFINE_CONV(NAME, IN_T, ACC_T, LOADX, FMA, STORE_ADD_BIAS)                                                     \
    int NAME(const IN_T* x, const IN_T* w, const IN_T* b, IN_T* out, int64_t N, int64_t C, int64_t H, int64_t W,       \
             int64_t K, int64_t R, int64_t S, int64_t sh, int64_t sw, int64_t ph, int64_t pw, int64_t OH, int64_t OW) { \
        const int64_t L = C * R * S;                                                                                   \
        ACC_T* wt = (ACC_T*)malloc(sizeof(ACC_T) * (size_t)(L * K > 0 ? L * K : 1)); /* [L][K]: b of the Dot */       \
        ACC_T* acc = (ACC_T*)malloc(sizeof(ACC_T) * (size_t)(K > 0 ? K : 1));                                          \
        if (!wt || !acc) {                                                                                             \
            free(wt);                                                                                                  \
            free(acc);                                                                                                 \
            return -1;                                                                                                 \
        }                                                                                                              \
        for (int64_t k = 0; k < K; ++k)                                                                                \
            for (int64_t l = 0; l < L; ++l) wt[l * K + k] = LOADX(w[k * L + l]);                                       \
        for (int64_t n = 0; n < N; ++n)                                                                                \
            for (int64_t oh = 0; oh < OH; ++oh)                                                                        \
                for (int64_t ow = 0; ow < OW; ++ow) {                                                                  \
                    for (int64_t k = 0; k < K; ++k) acc[k] = 0;                                                        \
                    for (int64_t c = 0; c < C; ++c)                                                                    \
                        for (int64_t r = 0; r < R; ++r)                                                                \
                            for (int64_t s = 0; s < S; ++s) {                                                          \
                                const int64_t ih = oh * sh - ph + r, iw = ow * sw - pw + s;                            \
                                ACC_T xv = 0;                                                                          \
                                if (ih >= 0 && ih < H && iw >= 0 && iw < W) xv = LOADX(x[((n * C + c) * H + ih) * W + iw]); \
                                const ACC_T* wrow = wt + ((c * R + r) * S + s) * K;                                    \
                                for (int64_t k = 0; k < K; ++k) acc[k] = FMA(xv, wrow[k], acc[k]);                     \
                            }                                                                                          \
                    for (int64_t k = 0; k < K; ++k) {                                                                  \
                        IN_T* o = out + ((n * K + k) * OH + oh) * OW + ow;                                             \
                        STORE_ADD_BIAS                                                                                 \
                    }                                                                                                  \
                }                                                                                                      \
        free(wt);                                                                                                      \
        free(acc);                                                                                                     \
        return 0;                                                                                                      \
    }

#define ID(v) (v)
#define STORE_F32 *o = b ? acc[k] + b[k] : acc[k];
#define STORE_F16                                                                                   \
    {                                                                                               \
        uint16_t y = float_to_half_bits(acc[k]);                                                    \
        if (b) y = float_to_half_bits(half_bits_to_float(y) + half_bits_to_float(b[k]));            \
        *o = y;                                                                                     \
    }
DEFINE_CONV(oracle_conv_f32, float, float, ID, fmaf, STORE_F32)
DEFINE_CONV(oracle_conv_f64, double, double, ID, fma, STORE_F32)
DEFINE_CONV(oracle_conv_f16, uint16_t, float, half_bits_to_float, fmaf, STORE_F16)

int oracle_has_hw_fma(void) {
#if defined(__FMA__)
    return __builtin_cpu_supports("fma") ? 1 : 0;
#else
    return -1; /* built without -mfma: fmaf/fma go through libm and are exact but slow */
#endif
}
