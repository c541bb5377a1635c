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
template <typename T> struct IsHalf { static constexpr bool value = false; };
template <> struct IsHalf<F16> { static constexpr bool value = true; };
template <typename T> struct DT;
template <> struct DT<F16> { static constexpr uint32_t kLowMask = 0x1fffu, kMid = 0x1000u; static constexpr float kMinNormal = 6.103515625e-05f; };
template <> struct DT<BF16> { static constexpr uint32_t kLowMask = 0xffffu, kMid = 0x8000u; static constexpr float kMinNormal = 1.17549435e-38f; };

constexpr uint32_t kAtanGuardUlps = 5;   // the fast arctangent stays within 4 ulp of the exact routine (exhaustive self-test)
constexpr uint32_t kSqrtGuardUlps = 2;   // v_sqrt_f32 is within 1 ulp

// Which arctangent the angle must reproduce.  Eager torch evaluates atan2 on half tensors in fp32 and
// rounds once: on the CPU with SLEEF's Sleef_atan2f_u10 (restated in pq_math.h), on the GPU with the
// device math library's atan2f, which is what `atan2f` in device code here resolves to as well.  The
// two differ in the last fp32 bits on about a third of all operands, and after rounding to half on a
// few dozen per million.  LIBM = true selects the device library's routine as the exact one; it lies
// within 3 ulp of SLEEF's on every operand pair seen, so the estimate's guard band is widened by that
// (the exhaustive self-test checks the wider band against the library routine itself).
template <bool LIBM> struct Atan { static constexpr uint32_t kGuardUlps = LIBM ? kAtanGuardUlps + 4 : kAtanGuardUlps; };
template <bool LIBM>
__device__ __forceinline__ float atan2_exact(float y, float x) {
    if constexpr (LIBM) return atan2f(y, x);
    else return math::atan2f_sleef_u10(y, x);
}

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

// Cheap estimates of the angle (in [-pi, pi]) and radius, NOT yet rounded; returns true when
// the exact routines must be used instead (see above).
template <typename T, bool LIBM = false>
__device__ __forceinline__ bool angle_radius_fast(float x, float y, float* a_out, float* r_out) {
    const float ss = __builtin_fmaf(x, x, y * y);          // x*x, y*y are exact for half/bf16 operands
    const float a = atan2_fast(y, x);
    const float r = __builtin_amdgcn_sqrtf(ss);
    // Infinities, NaNs, and (bfloat16 only) magnitudes at which the reciprocal or the hardware
    // square root leave their accurate range: one comparison for half, whose finite squares all lie
    // inside (2^-80, 2^80).  Zeros need no test of their own: with one zero operand the estimate is
    // exactly 0, pi/2 or pi like the exact routine's (0 then fails the kMinNormal test below), and
    // x == y == 0 gives a NaN angle with radius 0, which fails that test as well.
    // (bitwise | on purpose: one straight-line predicate instead of a chain of exec-mask branches)
    int special = static_cast<int>(!(ss < 0x1p80f));
    if constexpr (!IsHalf<T>::value) special |= static_cast<int>(!(ss > 0x1p-80f));
    *a_out = a;
    *r_out = r;
    return (special | static_cast<int>(fminf(fabsf(a), r) < DT<T>::kMinNormal) |
            static_cast<int>(near_rounding_boundary<T>(a, Atan<LIBM>::kGuardUlps)) |
            static_cast<int>(near_rounding_boundary<T>(r, kSqrtGuardUlps))) != 0;
}

// Correctly rounded fp32 square root.  NOT __fsqrt_rn: HIP defines that as the native (1 ulp)
// instruction unless OCML_BASIC_ROUNDED_OPERATIONS is set; sqrtf() is expanded by the compiler to
// the correctly rounded sequence (the default of -fhip-fp32-correctly-rounded-divide-sqrt), and the
// device self-test checks every result against its two neighbours' midpoints in double precision.
__device__ __forceinline__ float sqrt_rn(float s) { return __builtin_sqrtf(s); }

// -> (angle in [-pi, pi], radius), both rounded to the key dtype
template <typename T, bool LIBM = false>
__device__ __forceinline__ void angle_radius(float x, float y, float* phi, float* rad) {
    float a, r;
    if (__builtin_expect(angle_radius_fast<T, LIBM>(x, y, &a, &r), 0)) {
        a = atan2_exact<LIBM>(y, x);
        r = sqrt_rn(__builtin_fmaf(x, x, y * y));
    }
    *phi = rnd<T>(a);
    *rad = rnd<T>(r);
}

template <typename T, bool LIBM = false>
__device__ __forceinline__ void angle_radius_exact(float x, float y, float* phi, float* rad) {
    *phi = rnd<T>(atan2_exact<LIBM>(y, x));
    *rad = rnd<T>(sqrt_rn(__builtin_fmaf(x, x, y * y)));
}

// floor(dtype((v - mn) / scale)) clamped to [0, top] (:148, :153).  `topf` is the clamp bound as a
// float, or 0 for a degenerate pair (scale == 0 or NaN: x/0 and 0/0 are undefined in the reference
// and defined as code 0 here).  v_med3_f32 returns the minimum of its operands when one is NaN, so
// a NaN quotient also comes out as 0 without a separate test.
template <typename T>
__device__ __forceinline__ uint32_t code_of(float v, float mn, float scale, float topf) {
    const float d = rnd<T>(v - mn);
    const float qf = floorf(rnd<T>(d / scale));
    return static_cast<uint32_t>(__builtin_amdgcn_fmed3f(qf, 0.0f, topf));
}
// The same with div_faithful in place of the division; `inv` = v_rcp_f32(scale), scale accepted by fast_div_ok.
template <typename T>
__device__ __forceinline__ uint32_t code_of_fast(float v, float mn, float scale, float inv, float topf) {
    const float d = rnd<T>(v - mn);
    const float qf = floorf(rnd<T>(div_faithful(d, scale, inv)));
    return static_cast<uint32_t>(__builtin_amdgcn_fmed3f(qf, 0.0f, topf));
}
__device__ __forceinline__ float clamp_bound(float scale, int top) { return scale > 0.0f ? static_cast<float>(top) : 0.0f; }

constexpr int kQThreads = 256;
constexpr int kTokPerThread = kGroup / 16;   // 8
constexpr int kEntries = kTokPerThread * 4;  // (token, pair) entries per thread

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));

// Packed min / max of two (angle word | radius word << 16) registers.  Both values are
// non-negative (the angle after the 2*pi wrap, the radius always) and their sign bits are
// cleared, so bfloat16 words order like unsigned integers; half words use v_pk_max/min_f16.
template <typename T> __device__ __forceinline__ uint32_t pk_max(uint32_t a, uint32_t b);
template <typename T> __device__ __forceinline__ uint32_t pk_min(uint32_t a, uint32_t b);
template <> __device__ __forceinline__ uint32_t pk_max<F16>(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(half2v, a), __builtin_bit_cast(half2v, b)));
}
template <> __device__ __forceinline__ uint32_t pk_min<F16>(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(half2v, a), __builtin_bit_cast(half2v, b)));
}
template <> __device__ __forceinline__ uint32_t pk_max<BF16>(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(ushort2v, a), __builtin_bit_cast(ushort2v, b)));
}
template <> __device__ __forceinline__ uint32_t pk_min<BF16>(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(ushort2v, a), __builtin_bit_cast(ushort2v, b)));
}
template <typename T> struct PkInit;   // identity elements of pk_max / pk_min
template <> struct PkInit<F16> { static constexpr uint32_t kMax = 0x00000000u, kMin = 0x7c007c00u; };   // 0 / +inf
template <> struct PkInit<BF16> { static constexpr uint32_t kMax = 0x00000000u, kMin = 0xffffffffu; };

// How the angle is binned.  Reference mode: 2^tbits bins over the group's own [min, max] of the
// angle wrapped to [0, 2*pi) (:144-148).  Uniform mode: fixed bins over [-pi, pi), i.e. the same
// formula with the constants tmn = -pi and tscale = 2*pi / 2^tbits (both rounded to the key dtype);
// the angle code is then known in the first pass and is what the angle word carries.
struct AngleMode {
    float two_pi;      // reference mode: the constant added to negative angles
    float tmn, tscale; // uniform mode
    int ttop;
};

// (angle word | radius word << 16) of one pair: wrap applied, sign bits cleared
template <typename T, bool UNIFORM>
__device__ __forceinline__ uint32_t pack_angle_radius(float a, float r, const AngleMode& am) {
    float phi = rnd<T>(a);
    uint32_t aw;
    if constexpr (UNIFORM) {
        aw = code_of_fast<T>(phi, am.tmn, am.tscale, __builtin_amdgcn_rcpf(am.tscale), static_cast<float>(am.ttop));
    } else {
        if (phi < 0.0f) phi = rnd<T>(phi + am.two_pi);             // :144
        aw = f2lo<T>(phi);
    }
    return (aw | (static_cast<uint32_t>(f2lo<T>(r)) << 16)) & 0x7fff7fffu;
}

template <typename T, bool UNIFORM, bool PK6, bool LIBM>
__global__ __launch_bounds__(kQThreads) void quantize_kernel(
    const uint16_t* __restrict__ k, int64_t sb, int64_t sh, int64_t st, int Nk, int rbits, int tbits, AngleMode am,
    uint8_t* __restrict__ codes, uint16_t* __restrict__ rscale, uint16_t* __restrict__ rmn,
    uint16_t* __restrict__ tscale, uint16_t* __restrict__ tmn, int cap, int off) {
    // angle/radius words of the tile, entry-major so that a wavefront's accesses are contiguous
    __shared__ uint32_t pr[kEntries][kQThreads];
    __shared__ uint32_t red[2][4][kPairs];      // max / min, wavefront, pair
    __shared__ uint32_t fin[2][kPairs];

    const int tid = threadIdx.x;
    const int pq4 = tid & 15, tl = tid >> 4;
    const int grp = blockIdx.x, bh = blockIdx.y;
    const int b = bh / Nk, h = bh - b * Nk;
    const uint16_t* kb = k + b * sb + h * sh + static_cast<int64_t>(grp) * kGroup * st;

    // ---- pass 1: cheap estimates for every entry; remember which entries need the exact routines
    uint32_t risky_mask = 0;
#pragma unroll
    for (int it = 0; it < kTokPerThread; it++) {
        const uint16_t* row = kb + (it * 16 + tl) * st;
        const uint2 xw = *reinterpret_cast<const uint2*>(row + 4 * pq4);
        const uint2 yw = *reinterpret_cast<const uint2*>(row + kPairs + 4 * pq4);
        const uint16_t xs[4] = {static_cast<uint16_t>(xw.x), static_cast<uint16_t>(xw.x >> 16),
                                static_cast<uint16_t>(xw.y), static_cast<uint16_t>(xw.y >> 16)};
        const uint16_t ys[4] = {static_cast<uint16_t>(yw.x), static_cast<uint16_t>(yw.x >> 16),
                                static_cast<uint16_t>(yw.y), static_cast<uint16_t>(yw.y >> 16)};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float a, r;
            const bool risky = angle_radius_fast<T, LIBM>(lo2f<T>(xs[i]), lo2f<T>(ys[i]), &a, &r);   // :143, :150
            risky_mask |= static_cast<uint32_t>(risky) << (it * 4 + i);
            pr[it * 4 + i][tid] = pack_angle_radius<T, UNIFORM>(a, rnd<T>(r), am);
        }
    }
    // ---- fix-up: each lane redoes ITS risky entries with the exact routines (a lane has ~0.1 of
    // them, so the wavefront makes one or two trips instead of branching at all 32 entries)
    while (risky_mask) {
        const int e = __builtin_ctz(risky_mask);
        risky_mask &= risky_mask - 1;
        const uint16_t* row = kb + ((e >> 2) * 16 + tl) * st;
        const float x = lo2f<T>(row[4 * pq4 + (e & 3)]), y = lo2f<T>(row[kPairs + 4 * pq4 + (e & 3)]);
        float a, r;
        angle_radius_exact<T, LIBM>(x, y, &a, &r);
        pr[e][tid] = pack_angle_radius<T, UNIFORM>(a, r, am);
    }
    // ---- per-pair max / min of angle and radius over the 128 tokens (packed: both at once)
    uint32_t vmax[4], vmin[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { vmax[i] = PkInit<T>::kMax; vmin[i] = PkInit<T>::kMin; }
#pragma unroll
    for (int e = 0; e < kEntries; e++) {
        const uint32_t w = pr[e][tid];
        vmax[e & 3] = pk_max<T>(vmax[e & 3], w);
        vmin[e & 3] = pk_min<T>(vmin[e & 3], w);
    }
    // the 16 token lanes of a pair: 4 inside the wavefront (lane bits 4,5), 4 wavefronts
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int o = 16; o <= 32; o <<= 1) {
            vmax[i] = pk_max<T>(vmax[i], static_cast<uint32_t>(__shfl_xor(static_cast<int>(vmax[i]), o)));
            vmin[i] = pk_min<T>(vmin[i], static_cast<uint32_t>(__shfl_xor(static_cast<int>(vmin[i]), o)));
        }
    }
    if ((tid & 48) == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) { red[0][tid >> 6][4 * pq4 + i] = vmax[i]; red[1][tid >> 6][4 * pq4 + i] = vmin[i]; }
    }
    __syncthreads();
    if (tid < 2 * kPairs) {
        const int s = tid >> 6, p = tid & 63;
        uint32_t v = red[s][0][p];
#pragma unroll
        for (int j = 1; j < 4; j++) v = s ? pk_min<T>(v, red[s][j][p]) : pk_max<T>(v, red[s][j][p]);
        fin[s][p] = v;
    }
    __syncthreads();

    const float inv_t = static_cast<float>(1 << tbits), inv_r = static_cast<float>(1 << rbits);
    float ts[4], tm[4], rs[4], rm[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t wmax = fin[0][4 * pq4 + i], wmin = fin[1][4 * pq4 + i];
        tm[i] = lo2f<T>(static_cast<uint16_t>(wmin & 0xffffu));
        rm[i] = lo2f<T>(static_cast<uint16_t>(wmin >> 16));
        ts[i] = rnd<T>(rnd<T>(lo2f<T>(static_cast<uint16_t>(wmax & 0xffffu)) - tm[i]) / inv_t);   // :147
        if constexpr (UNIFORM) { tm[i] = am.tmn; ts[i] = am.tscale; }
        rs[i] = rnd<T>(rnd<T>(lo2f<T>(static_cast<uint16_t>(wmax >> 16)) - rm[i]) / inv_r);       // :152
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
    // ---- pass 2: codes
    float ttop[4], rtop[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ttop[i] = clamp_bound(ts[i], (1 << tbits) - 1);
        rtop[i] = clamp_bound(rs[i], (1 << rbits) - 1);
    }
    uint8_t* cb = codes + plane * (kGroup * (PK6 ? kPackedRowBytes : kPairs));
    // scales of 0 (degenerate pairs), infinities and the far ends of the bfloat16 range take the division
    bool fast = true;
    float tinv[4], rinv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        fast = fast && fast_div_ok(ts[i]) && fast_div_ok(rs[i]);
        tinv[i] = __builtin_amdgcn_rcpf(ts[i]);
        rinv[i] = __builtin_amdgcn_rcpf(rs[i]);
    }
    auto store_codes = [&](int it, uint32_t w) {
        if constexpr (PK6) {
            // 4 codes -> 24 bits; the 4 lanes that share 12 bytes of the row assemble its 3 words:
            // lane 4k+0 writes x0 | x1 << 24, lane 4k+1 x1 >> 8 | x2 << 16, lane 4k+2 x2 >> 16 | x3 << 8
            const uint32_t x = (w & 0x3Fu) | ((w >> 2) & 0xFC0u) | ((w >> 4) & 0x3F000u) | ((w >> 6) & 0xFC0000u);
            const uint32_t nx = static_cast<uint32_t>(__shfl_down(static_cast<int>(x), 1));
            const int k = pq4 & 3;
            const uint32_t word = (x >> (8 * k)) | (nx << (24 - 8 * k));
            if (k < 3)
                *reinterpret_cast<uint32_t*>(cb + (it * 16 + tl) * kPackedRowBytes + 12 * (pq4 >> 2) + 4 * k) = word;
        } else {
            *reinterpret_cast<uint32_t*>(cb + (it * 16 + tl) * kPairs + 4 * pq4) = w;
        }
    };
    // PK6 exchanges words between lanes, so the whole wavefront takes one side together
    if (__builtin_expect(PK6 ? __all(fast) : fast, 1)) {
#pragma unroll
        for (int it = 0; it < kTokPerThread; it++) {
            uint32_t w = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t v = pr[it * 4 + i][tid];
                const float phi = lo2f<T>(static_cast<uint16_t>(v & 0xffffu));
                const float r = lo2f<T>(static_cast<uint16_t>(v >> 16));
                const uint32_t th = UNIFORM ? (v & 0xffffu) : code_of_fast<T>(phi, tm[i], ts[i], tinv[i], ttop[i]);    // :148
                const uint32_t rh = code_of_fast<T>(r, rm[i], rs[i], rinv[i], rtop[i]);      // :153
                w |= (((rh << tbits) + th) & 0xffu) << (8 * i);             // :155
            }
            store_codes(it, w);
        }
    } else {
#pragma unroll
        for (int it = 0; it < kTokPerThread; it++) {
            uint32_t w = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t v = pr[it * 4 + i][tid];
                const float phi = lo2f<T>(static_cast<uint16_t>(v & 0xffffu));
                const float r = lo2f<T>(static_cast<uint16_t>(v >> 16));
                const uint32_t th = UNIFORM ? (v & 0xffffu) : code_of<T>(phi, tm[i], ts[i], ttop[i]);    // :148
                const uint32_t rh = code_of<T>(r, rm[i], rs[i], rtop[i]);      // :153
                w |= (((rh << tbits) + th) & 0xffu) << (8 * i);             // :155
            }
            store_codes(it, w);
        }
    }
}

#ifdef PQ_PROBE_DIRECT_BINS
#include "pq_quantize_probe.h"
#endif

// Exhaustive check of angle_radius against angle_radius_exact: block == bit pattern of y,
// thread t covers x patterns t, t+256, ...; NaN operands are skipped.
template <typename T, bool LIBM>
__global__ __launch_bounds__(256) void selftest_kernel(unsigned long long* mismatches, unsigned long long* slow_lanes) {
    const uint16_t yb = static_cast<uint16_t>(blockIdx.x);
    const float y = lo2f<T>(yb);
    unsigned int bad = 0, slow = 0;
    for (uint32_t xb = threadIdx.x; xb < 65536u; xb += 256u) {
        const float x = lo2f<T>(static_cast<uint16_t>(xb));
        if (x != x || y != y) continue;
        float p0, r0, p1, r1;
        angle_radius<T, LIBM>(x, y, &p0, &r0);
        angle_radius_exact<T, LIBM>(x, y, &p1, &r1);
        bad += (f2lo<T>(p0) != f2lo<T>(p1)) || (f2lo<T>(r0) != f2lo<T>(r1));
        // the exact radius: s lies between the squares of the midpoints to the two neighbours of sqrt_rn(s)
        const float s = __builtin_fmaf(x, x, y * y);
        if (!LIBM && s > 0.0f && s < INFINITY) {
            const float rr = sqrt_rn(s);
            const double lo = 0.5 * (static_cast<double>(rr) + static_cast<double>(__uint_as_float(__float_as_uint(rr) - 1u)));
            const double hi = 0.5 * (static_cast<double>(rr) + static_cast<double>(__uint_as_float(__float_as_uint(rr) + 1u)));
            bad += !(lo * lo <= static_cast<double>(s) && static_cast<double>(s) <= hi * hi);
        }
        const float a = atan2_fast(y, x), r = __builtin_amdgcn_sqrtf(__builtin_fmaf(x, x, y * y));
        slow += near_rounding_boundary<T>(a, Atan<LIBM>::kGuardUlps) || near_rounding_boundary<T>(r, kSqrtGuardUlps);
    }
    if (bad) atomicAdd(mismatches, static_cast<unsigned long long>(bad));
    if (slow) atomicAdd(slow_lanes, static_cast<unsigned long long>(slow));
}

// Exhaustive check of div_faithful: block == bit pattern of the dividend d, thread t covers the
// divisor patterns t, t+256, ...  Pairs the quantizers can meet: divisor accepted by fast_div_ok,
// 0 <= d <= 1024 * sc (d is a distance from the group minimum and sc the group's range over at
// most 2^8 bins).  Quotients below 1/4 may differ in denormal digits; floor() and rint() of both
// are 0 there, which is all the quantizers take from them.
template <typename T>
__global__ __launch_bounds__(256) void selftest_div_kernel(unsigned long long* mismatches) {
    const float d = lo2f<T>(static_cast<uint16_t>(blockIdx.x));
    unsigned int bad = 0;
    if (d >= 0.0f && d < INFINITY) {
        for (uint32_t sb = threadIdx.x; sb < 65536u; sb += 256u) {
            const float sc = lo2f<T>(static_cast<uint16_t>(sb));
            if (!fast_div_ok(sc) || !(d <= 1024.0f * sc)) continue;
            const float exact = rnd<T>(d / sc);
            const float fast = rnd<T>(div_faithful(d, sc, __builtin_amdgcn_rcpf(sc)));
            bad += (exact != fast) && !(exact < 0.25f && fast < 0.25f);
        }
    }
    if (bad) atomicAdd(mismatches, static_cast<unsigned long long>(bad));
}

int launch_selftest(int dtype, unsigned long long* counters, hipStream_t st) {
    // counters: [0] mismatches, [1] exact-path pairs (SLEEF arctangent); [2] division mismatches;
    // [3] mismatches, [4] exact-path pairs with the device library's arctangent as the exact routine
    if (dtype == 0) {
        hipLaunchKernelGGL((selftest_kernel<F16, false>), dim3(65536), dim3(256), 0, st, counters, counters + 1);
        hipLaunchKernelGGL(selftest_div_kernel<F16>, dim3(65536), dim3(256), 0, st, counters + 2);
        hipLaunchKernelGGL((selftest_kernel<F16, true>), dim3(65536), dim3(256), 0, st, counters + 3, counters + 4);
    } else {
        hipLaunchKernelGGL((selftest_kernel<BF16, false>), dim3(65536), dim3(256), 0, st, counters, counters + 1);
        hipLaunchKernelGGL(selftest_div_kernel<BF16>, dim3(65536), dim3(256), 0, st, counters + 2);
        hipLaunchKernelGGL((selftest_kernel<BF16, true>), dim3(65536), dim3(256), 0, st, counters + 3, counters + 4);
    }
    return static_cast<int>(hipGetLastError());
}

int launch_quantize(const void* k, const int64_t* strides, int dtype, int B, int Nk, int Nb, int rbits, int tbits,
                    unsigned flags, uint8_t* codes, void* rscale, void* rmn, void* tscale, void* tmn,
                    int cap, int off, hipStream_t st) {
    dim3 grid(Nb, B * Nk), block(kQThreads);
    const float two_pi_f = 6.28318548202514648438f;   // (float)(2*pi)
    // eager torch-CPU casts the python scalar 2*pi to the tensor dtype first: 6.28125 in both dtypes
    AngleMode am;
    const bool uniform = (flags & 2u) != 0;
    am.two_pi = (flags & 1u) ? two_pi_f : 6.28125f;
    am.ttop = (1 << tbits) - 1;
    const bool bf = dtype != 0;
    auto round_dt = [bf](float f) {
        return bf ? math::bf16_bits_to_float(math::float_to_bf16_bits(f)) : math::half_bits_to_float(math::float_to_half_bits(f));
    };
    am.tmn = round_dt(-3.14159274101257324219f);
    am.tscale = round_dt(round_dt(two_pi_f) / static_cast<float>(1 << tbits));
    const bool packed6 = (flags & 4u) != 0;
    const bool libm = (flags & 8u) != 0;
#define PQ_LAUNCH_QPL(T, U, P, L)                                                                                    \
    hipLaunchKernelGGL((quantize_kernel<T, U, P, L>), grid, block, 0, st, (const uint16_t*)k, strides[0], strides[1], \
                       strides[2], Nk, rbits, tbits, am, codes, (uint16_t*)rscale, (uint16_t*)rmn,                  \
                       (uint16_t*)tscale, (uint16_t*)tmn, cap, off)
#define PQ_LAUNCH_QP(T, U, P)                                                                                        \
    do {                                                                                                             \
        if (libm) PQ_LAUNCH_QPL(T, U, P, true);                                                                      \
        else PQ_LAUNCH_QPL(T, U, P, false);                                                                          \
    } while (0)
#define PQ_LAUNCH_Q(T, U)                                                                                            \
    do {                                                                                                             \
        if (packed6) PQ_LAUNCH_QP(T, U, true);                                                                       \
        else PQ_LAUNCH_QP(T, U, false);                                                                              \
    } while (0)
#ifdef PQ_PROBE_DIRECT_BINS
    // the probe build: every launch in the reference's angle mode with byte-per-code rows runs the probe kernel
    if (!uniform && !packed6) {
        if (dtype == 0)
            hipLaunchKernelGGL(quantize_direct_bins_probe_kernel<F16>, grid, block, 0, st, (const uint16_t*)k, strides[0], strides[1],
                               strides[2], Nk, rbits, tbits, am.two_pi, codes, (uint16_t*)rscale, (uint16_t*)rmn, (uint16_t*)tscale, (uint16_t*)tmn, cap, off);
        else
            hipLaunchKernelGGL(quantize_direct_bins_probe_kernel<BF16>, grid, block, 0, st, (const uint16_t*)k, strides[0], strides[1],
                               strides[2], Nk, rbits, tbits, am.two_pi, codes, (uint16_t*)rscale, (uint16_t*)rmn, (uint16_t*)tscale, (uint16_t*)tmn, cap, off);
        return static_cast<int>(hipGetLastError());
    }
#endif
    if (dtype == 0) { if (uniform) PQ_LAUNCH_Q(F16, true); else PQ_LAUNCH_Q(F16, false); }
    else            { if (uniform) PQ_LAUNCH_Q(BF16, true); else PQ_LAUNCH_Q(BF16, false); }
#undef PQ_LAUNCH_Q
#undef PQ_LAUNCH_QP
#undef PQ_LAUNCH_QPL
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
