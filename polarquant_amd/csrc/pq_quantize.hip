// Polar quantizer (quantize-on-append and prompt quantization): the HIP
// counterpart of quantize_and_pack_nbit (models/modeling_llama_polar.py:135-157).
//
// One 256-thread workgroup per (batch, KV head, 128-token group).  Thread
// (tl = tid/16, pq = tid%16) owns dimension pairs 4pq..4pq+3 of tokens
// tl, tl+16, ..., tl+112: each load is 8 bytes of x (dims [4pq,4pq+4)) and 8
// bytes of y (dims [64+4pq, ...)), so a wavefront reads four whole 256-byte key
// rows at a time, and each store is the 4 code bytes of one token, so a
// wavefront writes 256 contiguous bytes.  The key tile is read from HBM once:
// angles and radii stay in registers (packed as two 16-bit words) between the
// min/max pass and the code pass.
//
// Arithmetic follows eager torch on half tensors op by op: every reference op
// is evaluated in fp32 and rounded to the key dtype before the next.
#include "pq_device.h"
#include "pq_internal.h"
#include "pq_math.h"

namespace pq {

template <typename T>
__device__ __forceinline__ float rnd(float f) { return lo2f<T>(f2lo<T>(f)); }

// ---- angle and radius of one pair, rounded to the key dtype -------------------
// Eager torch gives round_dtype(atan2f_sleef(y, x)) and round_dtype(sqrt_rn(x*x + y*y)).
// The exact routines cost ~100 instructions per pair, so a cheap estimate is tried
// first: a 3.5-ulp arctangent (reciprocal, degree-8 polynomial in r^2, quadrant
// fix-up; it stays within 4 ulp of the exact routine) and the hardware square
// root (1 ulp).  Rounding the estimate to the key dtype gives the same word as
// rounding the exact value unless the estimate lies within its error bound of a
// rounding boundary of the dtype (a midpoint between two neighbouring dtype
// values, i.e. low fp32 mantissa bits == 100..0).  Only those lanes, plus the
// special operands (zeros, infinities, NaNs, results below the dtype's normal
// range), take the exact path.  That the two paths agree on EVERY pair of half /
// bfloat16 operands is checked exhaustively on the device by pq_selftest_quantizer_math.
template <typename T> struct DT;
template <> struct DT<F16> { static constexpr uint32_t kLowMask = 0x1fffu, kMid = 0x1000u; static constexpr float kMinNormal = 6.103515625e-05f; };
template <> struct DT<BF16> { static constexpr uint32_t kLowMask = 0xffffu, kMid = 0x8000u; static constexpr float kMinNormal = 1.17549435e-38f; };

constexpr uint32_t kAtanGuardUlps = 5;   // the fast arctangent stays within 4 ulp of the exact routine (exhaustive self-test)
constexpr uint32_t kSqrtGuardUlps = 2;   // v_sqrt_f32 is within 1 ulp

template <typename T>
__device__ __forceinline__ bool near_rounding_boundary(float a, uint32_t guard) {
    // |low mantissa bits - midpoint pattern| <= guard, computed without a branch
    const uint32_t low = (__float_as_uint(a) + (guard - DT<T>::kMid)) & DT<T>::kLowMask;
    return low <= 2u * guard;
}

__device__ __forceinline__ float atan2_fast(float y, float x) {
    const float ax = fabsf(x), ay = fabsf(y);
    const float mx = fmaxf(ax, ay), mn = fminf(ax, ay);
    const float r = mn * __builtin_amdgcn_rcpf(mx);
    const float s = r * r;
    float u = 0.00282363896258175373077393f;
    u = __builtin_fmaf(u, s, -0.0159569028764963150024414f);
    u = __builtin_fmaf(u, s, 0.0425049886107444763183594f);
    u = __builtin_fmaf(u, s, -0.0748900920152664184570312f);
    u = __builtin_fmaf(u, s, 0.106347933411598205566406f);
    u = __builtin_fmaf(u, s, -0.142027363181114196777344f);
    u = __builtin_fmaf(u, s, 0.199926957488059997558594f);
    u = __builtin_fmaf(u, s, -0.333331018686294555664062f);
    float a = __builtin_fmaf(u * s, r, r);
    a = ay > ax ? 1.57079637050628662109f - a : a;
    a = x < 0.0f ? 3.14159274101257324219f - a : a;
    return __builtin_copysignf(a, y);
}

// -> (angle in [-pi, pi], radius), both already rounded to the key dtype
template <typename T>
__device__ __forceinline__ void angle_radius(float x, float y, float* phi, float* rad) {
    const float ss = __builtin_fmaf(x, x, y * y);          // x*x, y*y are exact for half/bf16 operands
    float a = atan2_fast(y, x);
    float r = __builtin_amdgcn_sqrtf(ss);
    // zeros, infinities, NaNs, and magnitudes (bfloat16 only) at which the reciprocal or the
    // hardware square root leave their accurate range
    const bool special = !(ss > 0x1p-80f && ss < 0x1p80f) || fminf(fabsf(x), fabsf(y)) == 0.0f;
    const bool risky = special || fabsf(a) < DT<T>::kMinNormal || r < DT<T>::kMinNormal ||
                       near_rounding_boundary<T>(a, kAtanGuardUlps) || near_rounding_boundary<T>(r, kSqrtGuardUlps);
    if (__builtin_expect(risky, 0)) {
        a = math::atan2f_sleef_u10(y, x);
        r = __fsqrt_rn(ss);
    }
    *phi = rnd<T>(a);
    *rad = rnd<T>(r);
}

template <typename T>
__device__ __forceinline__ void angle_radius_exact(float x, float y, float* phi, float* rad) {
    *phi = rnd<T>(math::atan2f_sleef_u10(y, x));
    *rad = rnd<T>(__fsqrt_rn(__builtin_fmaf(x, x, y * y)));
}

template <typename T>
__device__ __forceinline__ uint32_t code_of(float v, float mn, float scale, int top) {
    const float d = rnd<T>(v - mn);
    float qf = rnd<T>(d / scale);
    qf = floorf(qf);
    if (!math::isfinite_(qf)) return 0u;   // 0/0 or x/0: undefined in the reference, 0 here
    qf = fminf(fmaxf(qf, 0.0f), 255.0f);
    const uint32_t c = static_cast<uint32_t>(qf);
    return c > static_cast<uint32_t>(top) ? static_cast<uint32_t>(top) : c;
}

constexpr int kQThreads = 256;
constexpr int kTokPerThread = kGroup / 16;   // 8

template <typename T>
__global__ __launch_bounds__(kQThreads) void quantize_kernel(
    const uint16_t* __restrict__ k, int64_t sb, int64_t sh, int64_t st, int Nk, int rbits, int tbits, float two_pi,
    uint8_t* __restrict__ codes, uint16_t* __restrict__ rscale, uint16_t* __restrict__ rmn,
    uint16_t* __restrict__ tscale, uint16_t* __restrict__ tmn, int cap, int off) {
    __shared__ float red[4][16][kPairs];      // stat, token lane, pair
    __shared__ float fin[4][kPairs];

    const int tid = threadIdx.x;
    const int pq4 = tid & 15, tl = tid >> 4;
    const int grp = blockIdx.x, bh = blockIdx.y;
    const int b = bh / Nk, h = bh - b * Nk;
    const uint16_t* kb = k + b * sb + h * sh + static_cast<int64_t>(grp) * kGroup * st;

    uint32_t pr[kTokPerThread][4];   // (phi word) | (radius word << 16)
    float pmx[4], pmn[4], rmx[4], rmn_[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { pmx[i] = -INFINITY; pmn[i] = INFINITY; rmx[i] = -INFINITY; rmn_[i] = INFINITY; }

#pragma unroll
    for (int it = 0; it < kTokPerThread; it++) {
        const int tok = it * 16 + tl;
        const uint16_t* row = kb + tok * st;
        const uint2 xw = *reinterpret_cast<const uint2*>(row + 4 * pq4);
        const uint2 yw = *reinterpret_cast<const uint2*>(row + kPairs + 4 * pq4);
        const uint16_t xs[4] = {static_cast<uint16_t>(xw.x), static_cast<uint16_t>(xw.x >> 16),
                                static_cast<uint16_t>(xw.y), static_cast<uint16_t>(xw.y >> 16)};
        const uint16_t ys[4] = {static_cast<uint16_t>(yw.x), static_cast<uint16_t>(yw.x >> 16),
                                static_cast<uint16_t>(yw.y), static_cast<uint16_t>(yw.y >> 16)};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float x = lo2f<T>(xs[i]), y = lo2f<T>(ys[i]);
            float phi, r;
            angle_radius<T>(x, y, &phi, &r);                           // :143, :150
            if (phi < 0.0f) phi = rnd<T>(phi + two_pi);                // :144
            pmx[i] = fmaxf(pmx[i], phi); pmn[i] = fminf(pmn[i], phi);
            rmx[i] = fmaxf(rmx[i], r);   rmn_[i] = fminf(rmn_[i], r);
            pr[it][i] = static_cast<uint32_t>(f2lo<T>(phi)) | (static_cast<uint32_t>(f2lo<T>(r)) << 16);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        red[0][tl][4 * pq4 + i] = pmx[i]; red[1][tl][4 * pq4 + i] = pmn[i];
        red[2][tl][4 * pq4 + i] = rmx[i]; red[3][tl][4 * pq4 + i] = rmn_[i];
    }
    __syncthreads();
    {
        const int s = tid >> 6, p = tid & 63;
        float v = red[s][0][p];
#pragma unroll
        for (int j = 1; j < 16; j++) v = (s & 1) ? fminf(v, red[s][j][p]) : fmaxf(v, red[s][j][p]);
        fin[s][p] = v;
    }
    __syncthreads();

    const float inv_t = static_cast<float>(1 << tbits), inv_r = static_cast<float>(1 << rbits);
    float ts[4], tm[4], rs[4], rm[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int p = 4 * pq4 + i;
        tm[i] = fin[1][p]; rm[i] = fin[3][p];
        ts[i] = rnd<T>(rnd<T>(fin[0][p] - tm[i]) / inv_t);              // :147
        rs[i] = rnd<T>(rnd<T>(fin[2][p] - rm[i]) / inv_r);              // :152
    }
    const size_t plane = static_cast<size_t>(bh) * cap + off + grp;
    if (tl == 0) {
        auto pack4 = [](const float (&v)[4]) {
            return make_uint2(static_cast<uint32_t>(f2lo<T>(v[0])) | (static_cast<uint32_t>(f2lo<T>(v[1])) << 16),
                              static_cast<uint32_t>(f2lo<T>(v[2])) | (static_cast<uint32_t>(f2lo<T>(v[3])) << 16));
        };
        const size_t mi = plane * kPairs + 4 * pq4;
        *reinterpret_cast<uint2*>(tscale + mi) = pack4(ts);
        *reinterpret_cast<uint2*>(tmn + mi) = pack4(tm);
        *reinterpret_cast<uint2*>(rscale + mi) = pack4(rs);
        *reinterpret_cast<uint2*>(rmn + mi) = pack4(rm);
    }
    const int ttop = (1 << tbits) - 1, rtop = (1 << rbits) - 1;
    uint8_t* cb = codes + plane * (kGroup * kPairs);
#pragma unroll
    for (int it = 0; it < kTokPerThread; it++) {
        const int tok = it * 16 + tl;
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float phi = lo2f<T>(static_cast<uint16_t>(pr[it][i] & 0xffffu));
            const float r = lo2f<T>(static_cast<uint16_t>(pr[it][i] >> 16));
            const uint32_t th = code_of<T>(phi, tm[i], ts[i], ttop);    // :148
            const uint32_t rh = code_of<T>(r, rm[i], rs[i], rtop);      // :153
            w |= (((rh << tbits) + th) & 0xffu) << (8 * i);             // :155
        }
        *reinterpret_cast<uint32_t*>(cb + tok * kPairs + 4 * pq4) = w;
    }
}

// Exhaustive check of angle_radius against angle_radius_exact: block == bit pattern of y,
// thread t covers x patterns t, t+256, ...; NaN operands are skipped.
template <typename T>
__global__ __launch_bounds__(256) void selftest_kernel(unsigned long long* mismatches, unsigned long long* slow_lanes) {
    const uint16_t yb = static_cast<uint16_t>(blockIdx.x);
    const float y = lo2f<T>(yb);
    unsigned int bad = 0, slow = 0;
    for (uint32_t xb = threadIdx.x; xb < 65536u; xb += 256u) {
        const float x = lo2f<T>(static_cast<uint16_t>(xb));
        if (x != x || y != y) continue;
        float p0, r0, p1, r1;
        angle_radius<T>(x, y, &p0, &r0);
        angle_radius_exact<T>(x, y, &p1, &r1);
        bad += (f2lo<T>(p0) != f2lo<T>(p1)) || (f2lo<T>(r0) != f2lo<T>(r1));
        const float a = atan2_fast(y, x), r = __builtin_amdgcn_sqrtf(__builtin_fmaf(x, x, y * y));
        slow += near_rounding_boundary<T>(a, kAtanGuardUlps) || near_rounding_boundary<T>(r, kSqrtGuardUlps);
    }
    if (bad) atomicAdd(mismatches, static_cast<unsigned long long>(bad));
    if (slow) atomicAdd(slow_lanes, static_cast<unsigned long long>(slow));
}

int launch_selftest(int dtype, unsigned long long* counters, hipStream_t st) {
    if (dtype == 0) hipLaunchKernelGGL(selftest_kernel<F16>, dim3(65536), dim3(256), 0, st, counters, counters + 1);
    else hipLaunchKernelGGL(selftest_kernel<BF16>, dim3(65536), dim3(256), 0, st, counters, counters + 1);
    return static_cast<int>(hipGetLastError());
}

int launch_quantize(const void* k, const int64_t* strides, int dtype, int B, int Nk, int Nb, int rbits, int tbits,
                    unsigned flags, uint8_t* codes, void* rscale, void* rmn, void* tscale, void* tmn,
                    int cap, int off, hipStream_t st) {
    dim3 grid(Nb, B * Nk), block(kQThreads);
    const float two_pi_f = 6.28318548202514648438f;   // (float)(2*pi)
    // eager torch-CPU casts the python scalar 2*pi to the tensor dtype first: 6.28125 in both dtypes
    const float two_pi = (flags & 1u) ? two_pi_f : 6.28125f;
    if (dtype == 0)
        hipLaunchKernelGGL(quantize_kernel<F16>, grid, block, 0, st, (const uint16_t*)k, strides[0], strides[1],
                           strides[2], Nk, rbits, tbits, two_pi, codes, (uint16_t*)rscale, (uint16_t*)rmn,
                           (uint16_t*)tscale, (uint16_t*)tmn, cap, off);
    else
        hipLaunchKernelGGL(quantize_kernel<BF16>, grid, block, 0, st, (const uint16_t*)k, strides[0], strides[1],
                           strides[2], Nk, rbits, tbits, two_pi, codes, (uint16_t*)rscale, (uint16_t*)rmn,
                           (uint16_t*)tscale, (uint16_t*)tmn, cap, off);
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
