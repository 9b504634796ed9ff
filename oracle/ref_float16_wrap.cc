// C entry points over the reference's own chainerx::Float16 (compiled from the reference tree,
// see oracle/Makefile).  Used only to pin the oracle's float16 conversions.
#include <cstdint>

#include "chainerx/float16.h"

extern "C" {
void ref_float_to_half(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = chainerx::Float16{in[i]}.data();
}
void ref_double_to_half(const double* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = chainerx::Float16{in[i]}.data();
}
void ref_half_to_float(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = static_cast<float>(chainerx::Float16::FromData(in[i]));
}
void ref_half_to_double(const uint16_t* in, double* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = static_cast<double>(chainerx::Float16::FromData(in[i]));
}
// Float16 arithmetic as the native backend's functors see it: operator+ etc. via float.
void ref_half_add(const uint16_t* a, const uint16_t* b, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (chainerx::Float16::FromData(a[i]) + chainerx::Float16::FromData(b[i])).data();
}
void ref_half_mul(const uint16_t* a, const uint16_t* b, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (chainerx::Float16::FromData(a[i]) * chainerx::Float16::FromData(b[i])).data();
}
}
