// Scalar math of the polar quantizer, usable from device code and from a plain
// host C++ build (the host build exists so the arithmetic can be checked
// against eager torch-CPU on millions of inputs without a GPU).
//
// Eager torch evaluates atan2 on half/bfloat16 CPU tensors as
//     round_to_dtype( Sleef_atan2f_u10( float(y), float(x) ) ).
// SLEEF is a third-party dependency of PyTorch that is not part of the
// reference tree (PyTorch vendors SLEEF 3.x; the routine is xatan2f_u1 /
// atan2kf_u1 in sleefsp.c / sleefsimdsp.c).  atan2f_sleef_u10 below restates
// that published algorithm — double-float (two-float) division and Horner
// evaluation with fused multiply-adds — with the same operations in the same
// order, so that its fp32 result is bit-identical and the angle code of a key
// cannot differ from eager torch's by a last-ulp effect of the arctangent.
// It relies on: IEEE fp32 add/mul/div with round-to-nearest-even, a true fused
// multiply-add, and NO implicit contraction of a*b+c (compile with
// -ffp-contract=off).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define PQ_HD __host__ __device__ __forceinline__
#else
#include <cmath>
#include <cstring>
#define PQ_HD inline
#endif

namespace pq {
namespace math {

PQ_HD uint32_t f2u(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(f);
#else
    uint32_t u; __builtin_memcpy(&u, &f, 4); return u;
#endif
}
PQ_HD float u2f(uint32_t u) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(u);
#else
    float f; __builtin_memcpy(&f, &u, 4); return f;
#endif
}
PQ_HD float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
PQ_HD float mulsign(float x, float y) { return u2f(f2u(x) ^ (f2u(y) & 0x80000000u)); }
PQ_HD float fabs_(float x) { return u2f(f2u(x) & 0x7fffffffu); }
PQ_HD bool isinf_(float x) { return (f2u(x) & 0x7fffffffu) == 0x7f800000u; }
PQ_HD bool isnan_(float x) { return (f2u(x) & 0x7fffffffu) > 0x7f800000u; }
PQ_HD bool isfinite_(float x) { return (f2u(x) & 0x7f800000u) != 0x7f800000u; }

struct F2 { float x, y; };

PQ_HD F2 df_div(F2 n, F2 d) {
    const float t = 1.0f / d.x;
    F2 q;
    q.x = n.x * t;
    const float u = fma_(t, n.x, -q.x);
    q.y = fma_(-d.y, t, fma_(-d.x, t, 1.0f));
    q.y = fma_(q.x, q.y, fma_(n.y, t, u));
    return q;
}
PQ_HD F2 df_squ(F2 a) {
    F2 r;
    r.x = a.x * a.x;
    r.y = fma_(a.x + a.x, a.y, fma_(a.x, a.x, -r.x));
    return r;
}
PQ_HD F2 df_mul(F2 a, F2 b) {
    F2 r;
    r.x = a.x * b.x;
    r.y = fma_(a.x, b.y, fma_(a.y, b.x, fma_(a.x, b.x, -r.x)));
    return r;
}
PQ_HD F2 df_mul_f(F2 a, float b) {
    F2 r;
    r.x = a.x * b;
    r.y = fma_(a.y, b, fma_(a.x, b, -r.x));
    return r;
}
PQ_HD F2 df_normalize(F2 t) {
    F2 s;
    s.x = t.x + t.y;
    s.y = t.x - s.x + t.y;
    return s;
}
PQ_HD F2 df_add_f_f(float a, float b) {
    F2 r;
    r.x = a + b;
    r.y = a - r.x + b;
    return r;
}
PQ_HD F2 df_add_f_f2(float a, F2 b) {
    F2 r;
    r.x = a + b.x;
    r.y = a - r.x + b.x + b.y;
    return r;
}
PQ_HD F2 df_add_f2_f2(F2 a, F2 b) {
    F2 r;
    r.x = a.x + b.x;
    r.y = a.x - r.x + b.x + a.y + b.y;
    return r;
}

// atan2(|y|, x) as a two-float, y >= 0.
PQ_HD F2 atan2k_u1(F2 y, F2 x) {
    int q = 0;
    if (x.x < 0.0f) { q = -2; x.x = -x.x; x.y = -x.y; }
    F2 s, t;
    if (x.x < y.x) { q += 1; s.x = -x.x; s.y = -x.y; t = y; }
    else { s = y; t = x; }
    s = df_div(s, t);
    t = df_squ(s);
    t = df_normalize(t);
    float u = -0.00176397908944636583328247f;
    u = fma_(u, t.x, 0.0107900900766253471374512f);
    u = fma_(u, t.x, -0.0309564601629972457885742f);
    u = fma_(u, t.x, 0.0577365085482597351074219f);
    u = fma_(u, t.x, -0.0838950723409652709960938f);
    u = fma_(u, t.x, 0.109463557600975036621094f);
    u = fma_(u, t.x, -0.142626821994781494140625f);
    u = fma_(u, t.x, 0.199983194470405578613281f);
    t = df_mul(t, df_add_f_f(-0.333332866430282592773438f, u * t.x));
    t = df_mul(s, df_add_f_f2(1.0f, t));
    F2 half_pi; half_pi.x = 1.5707963705062866211f; half_pi.y = -4.3711388286737928865e-08f;
    t = df_add_f2_f2(df_mul_f(half_pi, static_cast<float>(q)), t);
    return t;
}

PQ_HD float atan2f_sleef_u10(float y, float x) {
    const float kPi = 3.14159274101257324219f, kHalfPi = 1.57079637050628662109f, kQuarterPi = 0.785398185253143310547f;
    if (fabs_(x) < 2.9387372783541830947e-39f) { x *= 16777216.0f; y *= 16777216.0f; }
    F2 ay; ay.x = fabs_(y); ay.y = 0.0f;
    F2 xx; xx.x = x; xx.y = 0.0f;
    const F2 d = atan2k_u1(ay, xx);
    float r = d.x + d.y;
    r = mulsign(r, x);
    if (isinf_(x) || x == 0.0f) r = kHalfPi - (isinf_(x) ? mulsign(kHalfPi, x) : 0.0f);
    if (isinf_(y)) r = kHalfPi - (isinf_(x) ? mulsign(kQuarterPi, x) : 0.0f);
    if (y == 0.0f) r = (f2u(x) >> 31) ? kPi : 0.0f;
    if (isnan_(x) || isnan_(y)) return u2f(0x7fc00000u);
    return mulsign(r, y);
}

// ---- half / bfloat16 words <-> float, round-to-nearest-even (host versions;
// the device uses the hardware conversions, which agree) ----
PQ_HD float half_bits_to_float(uint16_t h) {
    const uint32_t s = static_cast<uint32_t>(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return u2f(s);
        int sh = 0;
        while (!(m & 0x400u)) { m <<= 1; sh++; }
        m &= 0x3ffu;
        return u2f(s | (static_cast<uint32_t>(113 - sh) << 23) | (m << 13));
    }
    if (e == 31) return u2f(s | 0x7f800000u | (m << 13));
    return u2f(s | ((e + 112) << 23) | (m << 13));
}
PQ_HD uint16_t float_to_half_bits(float f) {
    const uint32_t u = f2u(f);
    const uint32_t s = (u >> 16) & 0x8000u, e = (u >> 23) & 0xffu;
    uint32_t m = u & 0x7fffffu;
    if (e == 255) return static_cast<uint16_t>(s | 0x7c00u | (m ? 0x200u : 0u));
    const int ex = static_cast<int>(e) - 127 + 15;
    if (ex >= 31) return static_cast<uint16_t>(s | 0x7c00u);
    if (ex <= 0) {
        if (ex < -10) return static_cast<uint16_t>(s);
        m |= 0x800000u;
        const int sh = 14 - ex;
        uint32_t r = m >> sh;
        const uint32_t rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return static_cast<uint16_t>(s | r);
    }
    uint32_t r = (static_cast<uint32_t>(ex) << 10) | (m >> 13);
    const uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
    return static_cast<uint16_t>(s | r);
}
PQ_HD float bf16_bits_to_float(uint16_t h) { return u2f(static_cast<uint32_t>(h) << 16); }
PQ_HD uint16_t float_to_bf16_bits(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

}  // namespace math
}  // namespace pq
