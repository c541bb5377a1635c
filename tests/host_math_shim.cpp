// Host build of polarquant_amd/csrc/pq_math.h for the CPU tests: the same scalar
// code the quantizer kernel runs on the GPU, exported over arrays.
#include "../polarquant_amd/csrc/pq_math.h"

extern "C" {
void pqh_atan2f(const float* y, const float* x, float* out, long n) {
    for (long i = 0; i < n; i++) out[i] = pq::math::atan2f_sleef_u10(y[i], x[i]);
}
void pqh_half_to_float(const uint16_t* h, float* out, long n) {
    for (long i = 0; i < n; i++) out[i] = pq::math::half_bits_to_float(h[i]);
}
void pqh_float_to_half(const float* f, uint16_t* out, long n) {
    for (long i = 0; i < n; i++) out[i] = pq::math::float_to_half_bits(f[i]);
}
void pqh_float_to_bf16(const float* f, uint16_t* out, long n) {
    for (long i = 0; i < n; i++) out[i] = pq::math::float_to_bf16_bits(f[i]);
}
}
