// Device-side building blocks shared by the polar-key kernels (gfx950, wave64).
//
// Work decomposition used by every kernel here:
//   * one wavefront owns one 128-token group at a time and works through it in
//     two 64-token tiles, lane == token;
//   * per group the wavefront first builds, with lane == dimension pair d, an
//     angle lookup table in its private slice of LDS:
//         LUT[d][theta][j] = rscale_d * (q_j[d] cos phi + q_j[d+64] sin phi),
//         phi = tscale_d * (theta + 0.5) + tmn_d          (kernel4group.py:67-69)
//     for the `rep` query heads j that share the KV head;
//   * in the tile loop every lane walks the 64 pair codes of its token.  All
//     lanes look at the same pair d at the same time, so the LDS address differs
//     between lanes only by theta: equal theta is a broadcast, different theta
//     are different banks.  The radius bin centre r = rscale*(rho+0.5)+rmn
//     (kernel4group.py:73) is applied as (rho + c_d) with the wave-uniform
//     c_d = (rmn_d + rscale_d/2)/rscale_d, because rscale_d is already folded
//     into the table.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace pq {

constexpr int kPairs = 64;
constexpr int kGroup = 128;
constexpr int kHeadDim = 128;
constexpr int kWave = 64;

struct F16 {};
struct BF16 {};

template <typename T> __device__ __forceinline__ float lo2f(uint16_t w);
template <> __device__ __forceinline__ float lo2f<F16>(uint16_t w) {
    return __half2float(__ushort_as_half(w));
}
template <> __device__ __forceinline__ float lo2f<BF16>(uint16_t w) {
    return __uint_as_float(static_cast<uint32_t>(w) << 16);
}
template <typename T> __device__ __forceinline__ uint16_t f2lo(float f);
template <> __device__ __forceinline__ uint16_t f2lo<F16>(float f) {
    return __half_as_ushort(__float2half_rn(f));
}
template <> __device__ __forceinline__ uint16_t f2lo<BF16>(float f) {
    // one v_cvt_pk_bf16_f32 on gfx950 (round to nearest even, NaN stays NaN)
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

// ---- division of two key-dtype values, rounded to the key dtype ----------------
// Eager torch evaluates a / b on half / bfloat16 tensors as round_dtype(fp32 quotient).  The
// IEEE fp32 division is ~10 instructions; the quantizers divide every element by a scale that
// is shared by many elements, so they use instead
//     q0 = d * inv,  r = fma(-q0, sc, d),  q1 = fma(r, inv, q0),      inv = v_rcp_f32(sc) (1 ulp)
// q1 is a faithful fp32 quotient (the residual r is exact, so q1 is the rounding of a value
// within 2^-46 of d / sc).  It may differ from the correctly rounded fp32 quotient in the last
// bit, but never across a rounding boundary of the dtype: such a boundary t has at most 12
// significant bits and sc 11 (9 and 8 for bfloat16), so t * sc is exact in fp32 arithmetic and
// d / sc is either exactly t (then q1 == t as well) or more than 2 fp32 ulps away from it.
// Hence round_dtype(q1) == round_dtype(RN32(d / sc)).  Conditions: sc finite, positive and far
// from the ends of the fp32 range (fast_div_ok), d finite with d / sc far below overflow; callers
// take the plain division otherwise.  pq_selftest_quantizer_math checks the identity on the
// device for every operand pair of the dtype that meets them.
__device__ __forceinline__ bool fast_div_ok(float sc) { return sc >= 0x1p-100f && sc <= 0x1p100f; }
__device__ __forceinline__ float div_faithful(float d, float sc, float inv) {
    const float q0 = d * inv;
    const float r = __builtin_fmaf(-q0, sc, d);
    return __builtin_fmaf(r, inv, q0);
}

// v of lane (l & ~15) | ((l + N) & 15): a rotation inside each row of 16 lanes, as a DPP
// modifier of a move instead of a trip through the LDS crossbar
template <int N>
__device__ __forceinline__ uint32_t row_rotate(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x120 | N, 0xf, 0xf, true));
}

// Compile-time loop: f(std::integral_constant<int, I>) for I in [0, N).  Unlike
// "#pragma unroll" the indices are constants when the body is instantiated, so
// register arrays indexed by them never fall back to scratch memory.
template <int I> struct IC { static constexpr int value = I; constexpr operator int() const { return I; } };
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) { f(IC<I>{}); static_for<N, I + 1>(f); }
}

__device__ __forceinline__ float readlane_f(float v, int lane) {
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}

// Geometry of the per-wave lookup table for TB angle bits and REPP (1..8) query heads per KV head.
// An entry holds the first min(REPP, 4) heads; with more than 4 heads a second table ("half") of the
// same geometry holds the others, REPP - 4 floats per entry: a lookup reads the heads that exist
// (ds_read_b32 / b64 / b128; three heads are read as four), and no padded head costs a multiply-add.
// Entries are 4 (one head), 8 (two) or 16 bytes apart.  Within pair d the entry of angle bin theta sits
// at slot theta ^ (d & (NB-1)): the XOR spreads the 64 lanes of the build phase (lane == d, fixed
// theta) over all banks, and is undone in the tile loop by XOR-ing four codes at a time with a
// compile-time constant.
template <int TB, int REPP>
struct Lut {
    static_assert(REPP >= 1 && REPP <= 8, "1..8 query heads per KV head");
    static constexpr int NB = 1 << TB;
    static constexpr int W0 = REPP < 4 ? REPP : 4;        // heads in the first half's entries
    static constexpr int W1 = REPP - W0;                  // heads in the second half's entries (0: no second half)
    static constexpr int HALVES = W1 > 0 ? 2 : 1;
    static constexpr int EB = REPP == 1 ? 4 : (REPP == 2 ? 8 : 16);   // entry stride in bytes
    static constexpr int SH = REPP == 1 ? 2 : (REPP == 2 ? 3 : 4);
    static constexpr int PB = NB * EB;            // bytes per pair
    static constexpr int HB = kPairs * PB;        // bytes per half
    static constexpr int BYTES = HALVES * HB;
    // theta * EB fits a byte: the four byte offsets of a code word are made by two instructions on the
    // whole word; beyond that (TB 5, 6 with 16-byte entries) each code's offset is shifted into place
    static constexpr bool PACKED_OFFSETS = TB + SH <= 8;
};

// LDS is addressed with 32-bit byte addresses in address space 3 so that the
// compiler emits ds_read_b128/ds_write_b128 with the pair offset folded into
// the instruction's immediate offset field.
struct __attribute__((aligned(16))) Entry4 { float x, y, z, w; };
struct __attribute__((aligned(8))) Entry2 { float x, y; };
typedef __attribute__((address_space(3))) Entry4 lds_e4;
typedef __attribute__((address_space(3))) Entry2 lds_e2;
typedef __attribute__((address_space(3))) float lds_f1;
typedef float float4_v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) float4_v lds_f4;
typedef __attribute__((address_space(3))) void lds_void;

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"

template <typename P>
__device__ __forceinline__ P* lds_ptr(uint32_t addr) { return (P*)(addr); }

__device__ __forceinline__ uint32_t lds_addr(void* p) {
    return (uint32_t)(uintptr_t)((lds_void*)p);
}

// W (1..4) consecutive floats of a table entry at LDS byte address `addr`, as one ds_read / ds_write of that width.
// Three floats move as four (entries are 16 bytes apart, the fourth word belongs to nobody): a 96-bit LDS access
// keeps the LDS busy longer than a 128-bit one (measured at 7 heads per KV head, 3-bit angles, ragged batch of 64:
// SQ_LDS_IDX_ACTIVE 22.1 M with ds_read_b96 against 18.7 M with two ds_read_b128 for the same lookups).
template <int W>
__device__ __forceinline__ void lds_load_w(uint32_t addr, float* e) {
    if constexpr (W == 1) {
        e[0] = *lds_ptr<lds_f1>(addr);
    } else if constexpr (W == 2) {
        const lds_e2* p = lds_ptr<lds_e2>(addr);
        e[0] = p->x; e[1] = p->y;
    } else if constexpr (W == 3) {
        const float4_v v = *lds_ptr<const lds_f4>(addr);           // one 128-bit access; the fourth word is not used
        e[0] = v.x; e[1] = v.y; e[2] = v.z;
    } else {
        const lds_e4* p = lds_ptr<lds_e4>(addr);
        e[0] = p->x; e[1] = p->y; e[2] = p->z; e[3] = p->w;
    }
}
template <int W>
__device__ __forceinline__ void lds_store_w(uint32_t addr, const float* e) {
    if constexpr (W == 1) {
        *lds_ptr<lds_f1>(addr) = e[0];
    } else if constexpr (W == 2) {
        lds_e2* p = lds_ptr<lds_e2>(addr);
        p->x = e[0]; p->y = e[1];
    } else if constexpr (W == 3) {
        lds_e4* p = lds_ptr<lds_e4>(addr);
        p->x = e[0]; p->y = e[1]; p->z = e[2]; p->w = 0.0f;
    } else {
        lds_e4* p = lds_ptr<lds_e4>(addr);
        p->x = e[0]; p->y = e[1]; p->z = e[2]; p->w = e[3];
    }
}

// sin and cos of a bin-centre angle.  Three-constant Cody-Waite reduction by
// pi/2 with fused multiply-adds (accurate for |x| up to ~1e6, far beyond any
// half-precision tscale*(theta+0.5)+tmn), then the classic single-precision
// minimax polynomials on [-pi/4, pi/4]; absolute error below 2e-7.  Straight-line
// code: the library sincosf carries a Payne-Hanek branch the table build
// neither needs nor can afford in registers.
__device__ __forceinline__ void sincos_bin(float x, float* sn, float* cs) {
    const float k = __builtin_rintf(x * 0.636619772367581343f);
    float r = __builtin_fmaf(-k, 0x1.921fb6p+0f, x);
    r = __builtin_fmaf(-k, -0x1.777a5cp-25f, r);
    r = __builtin_fmaf(-k, -0x1.ee59dap-50f, r);
    const float z = r * r;
    float ps = __builtin_fmaf(z, -1.9515295891e-4f, 8.3321608736e-3f);
    ps = __builtin_fmaf(ps, z, -1.6666654611e-1f);
    const float s0 = __builtin_fmaf(ps * z, r, r);
    float pc = __builtin_fmaf(z, 2.443315711809948e-5f, -1.388731625493765e-3f);
    pc = __builtin_fmaf(pc, z, 4.166664568298827e-2f);
    const float c0 = __builtin_fmaf(pc * z, z, __builtin_fmaf(z, -0.5f, 1.0f));
    const int q = static_cast<int>(k);
    const float ss = (q & 1) ? c0 : s0;
    const float cc = (q & 1) ? s0 : c0;
    *sn = (q & 2) ? -ss : ss;
    *cs = ((q + 1) & 2) ? -cc : cc;
}

// Build the table for one group.  lane == pair d.
//   qx[j], qy[j]: q_j[d], q_j[d+64]
//   returns c_d for this lane's pair.
template <typename T, int TB, int REPP>
__device__ __forceinline__ float build_lut(uint32_t lut, int lane, const float (&qx)[REPP], const float (&qy)[REPP],
                                           uint16_t w_rscale, uint16_t w_rmn, uint16_t w_tscale, uint16_t w_tmn) {
    using L = Lut<TB, REPP>;
    const float ts = lo2f<T>(w_tscale), tm = lo2f<T>(w_tmn);
    const float rs = lo2f<T>(w_rscale), rm = lo2f<T>(w_rmn);
    float s, c, sd, cd;
    sincos_bin(__builtin_fmaf(ts, 0.5f, tm), &s, &c);
    sincos_bin(ts, &sd, &cd);
    const float rmp = __builtin_fmaf(rs, 0.5f, rm);
    float a, cdv;
    if (rs != 0.0f) { a = rs; cdv = rmp / rs; }
    else            { a = rmp * 0x1p-40f; cdv = 0x1p40f; }   // (rho + 2^40) * 2^-40 == 1 exactly
    float ax[REPP], ay[REPP];
#pragma unroll
    for (int j = 0; j < REPP; j++) { ax[j] = qx[j] * a; ay[j] = qy[j] * a; }
    // slot of bin k inside this lane's pair: k ^ (d & (NB-1)).  Computed on the slot number, then scaled and added to the
    // pair's base: nothing here depends on how the table is aligned in LDS.
    const uint32_t pair_base = lut + lane * L::PB;
    const uint32_t swz = lane & (L::NB - 1);
#pragma unroll
    for (int k = 0; k < L::NB; k++) {
        float e[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) e[j] = __builtin_fmaf(ax[j], c, ay[j] * s);
        const uint32_t off = pair_base + ((swz ^ k) << L::SH);
        lds_store_w<L::W0>(off, e);
        if constexpr (L::W1 > 0) lds_store_w<L::W1>(off + L::HB, e + 4);
        const float c2 = __builtin_fmaf(c, cd, -(s * sd));
        const float s2 = __builtin_fmaf(s, cd, c * sd);
        c = c2; s = s2;
    }
    return cdv;
}

// Score one token against the table.  `codes` holds the token's 64 pair codes as
// 16 little-endian words; cds[d] are the wave-uniform c_d.  acc[j] += ...
// The 64 table reads are issued in batches of 4 or 8 codes, one batch ahead of the
// FMAs that consume them, so that 4-16 LDS reads are always in flight.
template <int TB, int REPP>
__device__ __forceinline__ void score_token(uint32_t lut, const uint32_t (&codes)[16], const float (&cds)[kPairs],
                                            float (&acc)[REPP]) {
    using L = Lut<TB, REPP>;
    constexpr uint32_t TM4 = ((1u << TB) - 1u) * 0x01010101u;
    constexpr uint32_t RM4 = (0xFFu >> TB) * 0x01010101u;
    constexpr int nbm = L::NB - 1;
    constexpr int BW = REPP >= 4 ? 1 : 2;      // code words per batch
    constexpr int NBATCH = 16 / BW;
    float e[2][BW * 4][REPP];
    uint32_t r4s[2][BW];

    auto load = [&](auto BI) {
        constexpr int bi = decltype(BI)::value, buf = bi & 1;
        static_for<BW>([&](auto CC) {
            constexpr int cc = decltype(CC)::value, c = bi * BW + cc;
            const uint32_t w = codes[c];
            // byte i of ks: XOR pattern (slot swizzle) of pair 4c+i
            constexpr uint32_t ks = ((uint32_t)((4 * c + 0) & nbm)) | ((uint32_t)((4 * c + 1) & nbm) << 8) |
                                    ((uint32_t)((4 * c + 2) & nbm) << 16) | ((uint32_t)((4 * c + 3) & nbm) << 24);
            uint32_t a4, r4 = (w >> TB) & RM4;         // r4 byte i: rho_i
            if constexpr (L::PACKED_OFFSETS) {
                a4 = ((w & TM4) ^ ks) << L::SH;        // byte i: LDS byte offset of theta_i inside pair 4c+i
            } else {
                a4 = (w & TM4) ^ ks;                   // byte i: swizzled slot of theta_i, shifted into place per code
            }
            // keep the packed forms: byte i is then picked by v_bfe_u32 / v_cvt_f32_ubyte<i>
            asm volatile("" : "+v"(a4), "+v"(r4));
            r4s[buf][cc] = r4;
            static_for<4>([&](auto II) {
                constexpr int i = decltype(II)::value, d = 4 * c + i;
                uint32_t off = (a4 >> (8 * i)) & 0xFFu;
                if constexpr (!L::PACKED_OFFSETS) off <<= L::SH;
                const uint32_t addr = lut + off + d * L::PB;
                lds_load_w<L::W0>(addr, &e[buf][cc * 4 + i][0]);
                if constexpr (L::W1 > 0) lds_load_w<L::W1>(addr + L::HB, &e[buf][cc * 4 + i][4]);
            });
        });
    };
    auto compute = [&](auto BI) {
        constexpr int bi = decltype(BI)::value, buf = bi & 1;
        static_for<BW>([&](auto CC) {
            constexpr int cc = decltype(CC)::value, c = bi * BW + cc;
            const uint32_t r4 = r4s[buf][cc];
            // consume the batch's reads youngest first: the first use then waits for the whole
            // batch at once (LDS returns in order) and the other three need no wait instruction
            static_for<4>([&](auto II) {
                constexpr int i = 3 - decltype(II)::value;
                const float t = static_cast<float>((r4 >> (8 * i)) & 0xFFu) + cds[4 * c + i];
                static_for<REPP>([&](auto JJ) {
                    constexpr int j = decltype(JJ)::value;
                    acc[j] = __builtin_fmaf(e[buf][cc * 4 + i][j], t, acc[j]);
                });
            });
        });
    };
    load(IC<0>{});
    __builtin_amdgcn_sched_barrier(0);
    static_for<NBATCH>([&](auto BI) {
        constexpr int bi = decltype(BI)::value;
        if constexpr (bi + 1 < NBATCH) load(IC<bi + 1>{});
        compute(BI);
        __builtin_amdgcn_sched_barrier(0);
    });
    // pin the sums here: otherwise the optimizer sinks the FMA chains into whatever
    // conditional code consumes them and keeps all 64 table entries alive until then
#pragma unroll
    for (int j = 0; j < REPP; j++) asm volatile("" : "+v"(acc[j]));
}
#pragma clang diagnostic pop

// Packed 6-bit code rows (PQ_CODES_PACKED6): a token's 64 pair codes, each (rho << tbits) + theta < 64,
// are stored as 384 consecutive bits (48 bytes, code i in bits [6i, 6i+6)) instead of one byte each.
// unpack6 rebuilds the byte-per-code words the score loop works on: word c holds codes 4c..4c+3.
constexpr int kPackedRowBytes = 48;
__device__ __forceinline__ void unpack6(const uint32_t (&p)[12], uint32_t (&cw)[16]) {
    static_for<16>([&](auto CC) {
        constexpr int c = decltype(CC)::value, bit = 24 * c, j = bit >> 5, sh = bit & 31;
        uint32_t x;
        if constexpr (sh == 0) x = p[j];
        else if constexpr (j + 1 < 12) x = __builtin_amdgcn_alignbit(p[j + 1], p[j], sh);
        else x = p[j] >> sh;
        cw[c] = (x & 0x3Fu) | ((x << 2) & 0x3F00u) | ((x << 4) & 0x3F0000u) | ((x << 6) & 0x3F000000u);
    });
}

// Broadcast the 64 per-pair c_d values (lane d holds c_d) into wave-uniform registers.
__device__ __forceinline__ void broadcast_cd(float cdv, float (&cds)[kPairs]) {
#pragma unroll
    for (int d = 0; d < kPairs; d++) cds[d] = readlane_f(cdv, d);
}

}  // namespace pq
