// Fused polar-key decode attention: quantized-key scores, fp16 residual-key
// scores, 1/sqrt(d), mask, softmax and P.V in one pass over HBM
// (reference decode branch: models/modeling_llama_polar.py:66-99), split over
// the context, followed by a small merge kernel.
//
// attn_kernel: grid n_splits * B*Nk (plane index fastest), one wavefront per block: a block works
// through one slice of its sequence's quantized groups; the last block of
// a (batch, KV head) then also takes the fp16 residual keys (0..128 tokens).
// The kernel is built for ONE resident wavefront per SIMD (4 per CU) with deep
// software prefetch instead of many wavefronts: V operands are double-buffered
// a whole 64-token tile ahead, which keeps ~40 KiB of loads in flight per
// wavefront; pq_decode_attn_plan sizes n_splits so that B*Nk*n_splits fills
// those slots exactly once.
// Each wavefront walks its tokens in 64-token tiles, lane == token, and keeps
// flash-style running state (m, l, acc) for the `rep` query heads of its KV
// head.  P.V runs on the matrix cores: for 16 tokens at a time
//     D[dim][head] += V^T[dim][token] * P[token][head]
// with v_mfma_f32_16x16x16 (f16 or bf16), heads padded to the 16 columns.
// The V operand is built from plain 16-byte row loads (lane (g,n) loads dims
// 8n..8n+7 of tokens 4g..4g+3) by a 4x4 in-register transpose with v_perm_b32;
// P goes through a 1 KiB LDS staging buffer.
// The running maximum m is only raised when a score exceeds it by more than
// kLazyThreshold (in log2 units): probabilities stay below 2^8, and the
// 32-register rescale of the accumulators is skipped on almost every tile.
//
// merge_kernel: grid B*N, 128 threads (one per output dim), or four / eight such
// groups that share the partials when there are 32 / 128 or more: combines the n_splits
// partials (m, l, acc[128]) of a query head and writes half words.
#include "pq_device.h"
#include "pq_internal.h"
#include <mutex>

// Measuring build only (-DPQ_ATTN_PHASE_TIMERS, `python -m polarquant_amd.build --phase-timers`): wall-clock
// (100 MHz) time of each phase of the group loop, summed per wavefront and printed by a few of them.
#ifdef PQ_ATTN_PHASE_TIMERS
#define PQ_T_ENTRY const long long pt_entry_ = wall_clock64(); long long pt_loop0_ = pt_entry_, pt_first_ = 0, pt_loop1_ = pt_entry_, pt_sum_[6] = {0, 0, 0, 0, 0, 0}; int pt_groups_ = 0
#define PQ_T_DECL long long pt_[6] = {0, 0, 0, 0, 0, 0}, pt_mark_ = 0; pt_loop0_ = wall_clock64()
#define PQ_T_MARK() pt_mark_ = wall_clock64()
#define PQ_T_ADD(i) do { const long long pt_now_ = wall_clock64(); pt_[i] += pt_now_ - pt_mark_; pt_mark_ = pt_now_; } while (0)
#define PQ_T_KEEP(x) asm volatile("" ::"v"(x))
#define PQ_T_FIRST_GROUP_DONE() do { if (pt_first_ == 0) pt_first_ = wall_clock64() - pt_loop0_; } while (0)
#define PQ_T_REPORT(n_groups)                                                                                        \
    do {                                                                                                             \
        pt_loop1_ = wall_clock64();                                                                                  \
        pt_groups_ = n_groups;                                                                                       \
        for (int i_ = 0; i_ < 6; i_++) pt_sum_[i_] = pt_[i_];                                                        \
    } while (0)
// Printed once per piece, after its partial has been handed to the memory system (a device printf takes
// milliseconds, so none may sit inside what is timed): the phase sums of the group loop, then the absolute entry
// and exit clocks (the 100 MHz counter is common to the chip, so the spread of entries and exits over the
// wavefronts can be read off), entry -> loop, the first group, the loop, loop -> exit.
#define PQ_T_EXIT()                                                                                                  \
    do {                                                                                                             \
        const long long pt_exit_ = wall_clock64();                                                                   \
        if (threadIdx.x == 0 && blockIdx.x % 97 == 0) {                                                              \
            printf("pq_phase block %d groups %d total %lld table %lld value_issue %lld code_wait %lld code_issue %lld score %lld softmax_pv %lld\n", \
                   static_cast<int>(blockIdx.x), pt_groups_, pt_loop1_ - pt_loop0_, pt_sum_[0], pt_sum_[1], pt_sum_[2], \
                   pt_sum_[3], pt_sum_[4], pt_sum_[5]);                                                              \
            printf("pq_piece block %d groups %d entry %lld exit %lld before_loop %lld first_group %lld loop %lld after_loop %lld\n", \
                   static_cast<int>(blockIdx.x), pt_groups_, pt_entry_, pt_exit_, pt_loop0_ - pt_entry_, pt_first_,   \
                   pt_loop1_ - pt_loop0_, pt_exit_ - pt_loop1_);                                                     \
        }                                                                                                            \
    } while (0)
#else
#define PQ_T_ENTRY
#define PQ_T_DECL
#define PQ_T_MARK()
#define PQ_T_ADD(i)
#define PQ_T_KEEP(x)
#define PQ_T_FIRST_GROUP_DONE()
#define PQ_T_REPORT(n_groups)
#define PQ_T_EXIT()
#endif

namespace pq {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr float kLazyThreshold = 8.0f;
constexpr int kPartialFloats = 132;   // m, l, pad, pad, acc[128]
constexpr float kLog2e = 1.44269504088896340736f;

template <typename T> __device__ __forceinline__ floatx4 mfma16(uint2 a, uint2 b, floatx4 c);
template <> __device__ __forceinline__ floatx4 mfma16<F16>(uint2 a, uint2 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ floatx4 mfma16<BF16>(uint2 a, uint2 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

template <int REPP>
struct AttnState {
    float m[REPP];        // running maximum (log2 units), wave-uniform
    float l[REPP];        // per-lane partial sum of probabilities
    floatx4 acc[8];       // lane (g,n): acc[e][i] = out_head_n[dim 8*(4g+i)+e]
    float zp[REPP];       // 4-bit values only: per-lane partial sum of p * zero-point of the token
};

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"

// Softmax update and P.V for one 64-token tile.
//   t[j]   scaled score (log2 units) of this lane's token for head j; -inf = masked/invalid
//   vv     this lane's V operand loads: vv[tb][i] = dims 8n..8n+7 of token 16*tb + 4*g + i
//   pbuf   LDS address of the [REPP][64] 16-bit staging buffer
template <typename T, int REPP>
__device__ __forceinline__ void softmax_pv_tile(AttnState<REPP>& st, float (&t)[REPP], const uint4 (&vv)[4][4],
                                                uint32_t pbuf, int lane) {
    bool raise = false;
#pragma unroll
    for (int j = 0; j < REPP; j++) raise |= t[j] > st.m[j] + kLazyThreshold;
    if (__any(raise)) {
        float alpha[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) {
            const float mn = fmaxf(st.m[j], wave_max(t[j]));
            alpha[j] = (mn == -INFINITY) ? 1.0f : exp2f(st.m[j] - mn);
            st.m[j] = mn;
            st.l[j] *= alpha[j];
        }
        float a = alpha[0];
#pragma unroll
        for (int j = 1; j < REPP; j++) a = ((lane & 15) == j) ? alpha[j] : a;
#pragma unroll
        for (int e = 0; e < 8; e++) st.acc[e] *= a;
    }
#pragma unroll
    for (int j = 0; j < REPP; j++) {
        const float ms = (st.m[j] == -INFINITY) ? 0.0f : st.m[j];
        const float p = exp2f(t[j] - ms);
        st.l[j] += p;
        *lds_ptr<__attribute__((address_space(3))) uint16_t>(pbuf + (j * kWave + lane) * 2) = f2lo<T>(p);
    }
    asm volatile("" ::: "memory");
    const int g = lane >> 4, n = lane & 15;
    const uint32_t prow = pbuf + ((n & (REPP - 1)) * kWave + 4 * g) * 2;
#pragma unroll
    for (int tb = 0; tb < 4; tb++) {
        const __attribute__((address_space(3))) uint2* pp = lds_ptr<__attribute__((address_space(3))) uint2>(prow + tb * 32);
        uint2 pb;
        pb.x = pp->x; pb.y = pp->y;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
            auto word = [&](const uint4& v) { return (e >> 1) == 0 ? v.x : (e >> 1) == 1 ? v.y : (e >> 1) == 2 ? v.z : v.w; };
            uint2 va;
            va.x = __builtin_amdgcn_perm(word(vv[tb][1]), word(vv[tb][0]), sel);
            va.y = __builtin_amdgcn_perm(word(vv[tb][3]), word(vv[tb][2]), sel);
            st.acc[e] = mfma16<T>(va, pb, st.acc[e]);
        }
    }
    asm volatile("" ::: "memory");
    // keep the next tile's loads behind this tile's matrix work: hoisting them
    // here would double the registers held by V operands
    __builtin_amdgcn_sched_barrier(0);
}

// ---- 4-bit values (the Mixed variant, models/modeling_llama_polar.py:158-292) ----
// A cached value row is 16 int32 words; word n holds dims 8n..8n+7, dim 8n+e in bits [4e, 4e+4),
// with one (scale, zero-point) pair per token and head: v^ = code * scale + zero.  Then
//     sum_t p_t v^_t[dim] = sum_t (p_t scale_t) code_t[dim]  +  sum_t p_t zero_t
// and only the first term needs the matrix cores.  Lane (g,n) owns exactly word n of its tokens,
// so the MFMA row for dim 8n+e is nibble e of that word.  A nibble isolated in a byte and
// zero-extended to 16 bits IS the half-precision subnormal code * 2^-24 (odd nibbles are left in
// the high half of their byte: 16 * code * 2^-24), which v_mfma_f32_16x16x16_f16 multiplies
// exactly; so the A operand costs two v_and per word and one v_perm per register, like the
// half-precision rows it replaces, and the accumulators are brought back to real units once,
// after the last quantized tile (finish_v4).  The probabilities go through half precision for
// this product whatever the model dtype.  The weight p * scale must stay inside half precision's
// range at both ends: the running maximum is allowed to lag by only 2^kLazyThresholdV4 here, so
// that weight <= 4 * scale (scale <= 8734 for any half-precision row), and no further pre-scaling
// is applied, so that the tail of the softmax keeps the resolution the reference's
// half-precision probabilities have (a weight below 2^-25 drops out; with a pre-scale of 2^-6 a
// long flat tail 12 nats under the peak, still 10 % of the mass over 32k tokens, was lost).
constexpr float kLazyThresholdV4 = 2.0f;
constexpr float kV4PostEven = 0x1p24f;   // subnormal nibble = code * 2^-24
constexpr float kV4PostOdd = 0x1p20f;    // odd nibbles are left at 16 * code

// Tokens of a 16-token block are handed to the MFMA k-index transposed (k = 4g+i <-> token 4i+g),
// so that one load instruction of a wavefront covers 4 whole consecutive rows (256 contiguous
// bytes).  v4_slot is where lane == token puts its probability so that the B operand agrees.
__device__ __forceinline__ int v4_slot(int lane) { return (lane & 48) | ((lane & 3) << 2) | ((lane >> 2) & 3); }

//   vq[tb][i]  word n of token 16*tb + 4*i + g
//   sc, zp     this lane's token's scale and zero-point (lane == token)
template <int REPP>
__device__ __forceinline__ void softmax_pv_tile_v4(AttnState<REPP>& st, float (&t)[REPP], const uint32_t (&vq)[4][4],
                                                   float sc, float zp, uint32_t pbuf, int lane) {
    bool raise = false;
#pragma unroll
    for (int j = 0; j < REPP; j++) raise |= t[j] > st.m[j] + kLazyThresholdV4;
    if (__any(raise)) {
        float alpha[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) {
            const float mn = fmaxf(st.m[j], wave_max(t[j]));
            alpha[j] = (mn == -INFINITY) ? 1.0f : exp2f(st.m[j] - mn);
            st.m[j] = mn;
            st.l[j] *= alpha[j];
            st.zp[j] *= alpha[j];
        }
        float a = alpha[0];
#pragma unroll
        for (int j = 1; j < REPP; j++) a = ((lane & 15) == j) ? alpha[j] : a;
#pragma unroll
        for (int e = 0; e < 8; e++) st.acc[e] *= a;
    }
    const int slot = v4_slot(lane);
    // The weight the matrix cores see is w = half(p * scale).  The zero-point term must use
    // the SAME rounded weight (w * zero / scale), not p: code * scale and zero are each a few
    // units large and cancel to a value of order 1, so a weight that differs between the two terms by
    // its rounding error (2^-11) would leave an error of that size times ~3 when one token dominates.
    // A constant row has scale 0 and all codes 0: any scale serves, take 1.
    const float scp = sc == 0.0f ? 1.0f : sc;
    const float zq = zp / scp;
#pragma unroll
    for (int j = 0; j < REPP; j++) {
        const float ms = (st.m[j] == -INFINITY) ? 0.0f : st.m[j];
        const float p = exp2f(t[j] - ms);
        st.l[j] += p;
        const uint16_t wh = f2lo<F16>(p * scp);
        st.zp[j] = __builtin_fmaf(lo2f<F16>(wh), zq, st.zp[j]);
        *lds_ptr<__attribute__((address_space(3))) uint16_t>(pbuf + (j * kWave + slot) * 2) = wh;
    }
    asm volatile("" ::: "memory");
    const int g = lane >> 4, n = lane & 15;
    const uint32_t prow = pbuf + ((n & (REPP - 1)) * kWave + 4 * g) * 2;
#pragma unroll
    for (int tb = 0; tb < 4; tb++) {
        const __attribute__((address_space(3))) uint2* pp = lds_ptr<__attribute__((address_space(3))) uint2>(prow + tb * 32);
        uint2 pb;
        pb.x = pp->x; pb.y = pp->y;
        uint32_t ev[4], od[4];
#pragma unroll
        for (int i = 0; i < 4; i++) { ev[i] = vq[tb][i] & 0x0f0f0f0fu; od[i] = vq[tb][i] & 0xf0f0f0f0u; }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            // byte e/2 of the even / odd words of two tokens -> two zero-extended 16-bit fields
            const uint32_t by = static_cast<uint32_t>(e >> 1);
            const uint32_t sel = 0x0c000c00u | ((4u + by) << 16) | by;
            const uint32_t (&src)[4] = (e & 1) ? od : ev;
            uint2 va;
            va.x = __builtin_amdgcn_perm(src[1], src[0], sel);
            va.y = __builtin_amdgcn_perm(src[3], src[2], sel);
            st.acc[e] = mfma16<F16>(va, pb, st.acc[e]);
        }
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// After the last 4-bit tile: accumulators back to real units, plus the zero-point term (the same
// for all 128 dims of a head).
template <int REPP>
__device__ __forceinline__ void finish_v4(AttnState<REPP>& st, int lane) {
    float z = 0.0f;
#pragma unroll
    for (int j = 0; j < REPP; j++) {
        const float zj = wave_sum(st.zp[j]);
        z = ((lane & 15) == j) ? zj : z;
        st.zp[j] = 0.0f;
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float k = (e & 1) ? kV4PostOdd : kV4PostEven;
#pragma unroll
        for (int i = 0; i < 4; i++) st.acc[e][i] = __builtin_fmaf(st.acc[e][i], k, z);
    }
}

// Hot-loop loads go through buffer resources: the address is a wave-uniform
// base held in scalar registers plus one fixed 32-bit lane offset plus a scalar
// offset that carries the loop position, so no per-lane 64-bit pointer has to
// be kept or advanced, and rows past the end of a tensor read as zero instead
// of faulting (which is what the partly filled residual tile relies on).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}
// Cache policy of the code and V streams: every byte is used exactly once, so the loads carry
// the non-temporal hint (aux bit 1, "nt" on gfx94x/gfx950) and do not displace what the caches
// could keep.  Measured on configs[1]: 237 -> 222 us.
constexpr int kAuxStream = 2;
__device__ __forceinline__ uint4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(voff), static_cast<int>(soff), kAuxStream);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// Issue the V operand loads of the 64-token tile that starts at byte offset
// `tile_off` of the (batch, KV head) plane: lane (g,n) loads dims 8n..8n+7 of
// tokens 16*tb + 4*g + i.  voff = g*1024 + n*16.
__device__ __forceinline__ void load_v_tile(uint4 (&vv)[4][4], __amdgpu_buffer_rsrc_t rv, uint32_t voff, uint32_t tile_off) {
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
        for (int i = 0; i < 4; i++)
            vv[tb][i] = buf_load16(rv, voff, tile_off + static_cast<uint32_t>((16 * tb + i) * kHeadDim * 2));
}

// 4-bit value words of the 64-token tile at byte offset `tile_off` of the (batch, KV head) plane
// of value codes (64 bytes per token): voff = g*64 + n*4.
__device__ __forceinline__ void load_v4_tile(uint32_t (&vq)[4][4], __amdgpu_buffer_rsrc_t rv, uint32_t voff, uint32_t tile_off) {
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
        for (int i = 0; i < 4; i++)
            vq[tb][i] = static_cast<uint32_t>(__builtin_amdgcn_raw_buffer_load_b32(
                rv, static_cast<int>(voff), static_cast<int>(tile_off + static_cast<uint32_t>((16 * tb + 4 * i) * 64)), kAuxStream));
}

template <bool V4> struct VTile { uint4 r[4][4]; };         // one 64-token tile of V operands, per lane
template <> struct VTile<true> { uint32_t r[4][4]; };

struct V4Args {
    const uint32_t* codes;     // [B,Nk,capacity,16]
    const uint16_t* scale;     // [B,Nk,capacity]
    const uint16_t* zero;      // [B,Nk,capacity]
    int64_t capacity;          // tokens per (batch, KV head) plane
};

// Everything a wavefront needs to know about the call (the kernels' arguments).
struct AttnParams {
    const uint16_t* q;
    const uint8_t* codes;
    const uint16_t *rscale, *rmn, *tscale, *tmn;
    int group_capacity, n_groups;
    const int32_t* n_groups_per_seq;
    const uint16_t* k_resid;
    int resid_capacity, n_resid;
    const int32_t* n_resid_per_seq;
    const uint16_t* v;
    int64_t v_capacity;
    const uint8_t* mask;
    int64_t mask_stride;
    float scale_log2;
    int B, N, Nk, rep, n_splits, min_gps;
    float* ws;
};

// Token counts of one sequence as the kernels use them: groups and residual keys clamped to the
// capacities, tokens clamped to what the value plane holds.
struct SeqCounts { int nb, nres; int64_t n_tokens; };
template <bool V4>
__device__ __forceinline__ SeqCounts seq_counts(const AttnParams& p, const V4Args& v4, int b) {
    SeqCounts c;
    int nb = p.n_groups_per_seq ? p.n_groups_per_seq[b] : p.n_groups;
    nb = nb < 0 ? 0 : (nb > p.group_capacity ? p.group_capacity : nb);
    int nres = p.n_resid_per_seq ? p.n_resid_per_seq[b] : p.n_resid;
    nres = nres < 0 ? 0 : (nres > p.resid_capacity ? p.resid_capacity : nres);
    int64_t n_tokens = static_cast<int64_t>(nb) * kGroup + nres;
    if (V4) {
        nb = static_cast<int64_t>(nb) * kGroup > v4.capacity ? static_cast<int>(v4.capacity / kGroup) : nb;
        nres = nres > p.v_capacity ? static_cast<int>(p.v_capacity) : nres;
        n_tokens = static_cast<int64_t>(nb) * kGroup + nres;
    } else {
        n_tokens = n_tokens > p.v_capacity ? p.v_capacity : n_tokens;   // never read past the (batch, head) plane of V
    }
    c.nb = nb; c.nres = nres; c.n_tokens = n_tokens;
    return c;
}

// One piece of work of a wavefront: the 64-token tiles [t0, t1) of the quantized part of (sequence b,
// KV head kvh) (tile t = half t & 1 of group t >> 1; a piece may begin or end in the middle of a group,
// whose table it then builds like any other), then the 64-key tiles [r0, r1) of that sequence's
// half-precision residual keys; the partial result (m, l, acc) of each of the `rep` query heads goes
// to partial slot `slot` of its head.
template <typename T, int TB, int REPP, bool V4, bool PK6, bool RESID_FIRST>
__device__ __forceinline__ void attn_piece(const AttnParams& p, const V4Args& v4, uint32_t lut, uint32_t pbuf, int lane,
                                           int b, int kvh, const SeqCounts& sc, int t0, int t1, int r0, int r1, int slot) {
    // V4: the values of the quantized groups are 4-bit (v4), and `v` holds only the rows of the
    // residual window, row 0 = first residual token; otherwise `v` holds every row.
    PQ_T_ENTRY;
    const int N = p.N, Nk = p.Nk, rep = p.rep, n_splits = p.n_splits;
    const int bh = b * Nk + kvh;
    const int nb = sc.nb, nres = sc.nres;
    const int64_t n_tokens = sc.n_tokens;
    const int64_t v_capacity = p.v_capacity;
    const int group_capacity = p.group_capacity, resid_capacity = p.resid_capacity;
    const float scale_log2 = p.scale_log2;
    float* ws = p.ws;

    const uint16_t* qb = p.q + (static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep) * kHeadDim;
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(p.v + static_cast<size_t>(bh) * v_capacity * kHeadDim,
                                                static_cast<uint32_t>((V4 ? nres : n_tokens) * (kHeadDim * 2)));
    const uint32_t voff_v = static_cast<uint32_t>(lane >> 4) * (4 * kHeadDim * 2) + static_cast<uint32_t>(lane & 15) * 16;
    const bool has_mask = p.mask != nullptr;
    const __amdgpu_buffer_rsrc_t rm = make_rsrc(has_mask ? p.mask + static_cast<size_t>(b) * p.mask_stride : nullptr,
                                                has_mask ? static_cast<uint32_t>(n_tokens < p.mask_stride ? n_tokens : p.mask_stride) : 0u);

    AttnState<REPP> st;
#pragma unroll
    for (int j = 0; j < REPP; j++) { st.m[j] = -INFINITY; st.l[j] = 0.0f; st.zp[j] = 0.0f; }
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    // ---------------- residual keys (model dtype), 64-key tiles [r0, r1) ----------------
    // RESID_FIRST: runs right after the first loads of the quantized part have been issued, so that its own
    // loads and arithmetic overlap with their latency instead of standing alone at the end of the piece (the
    // order of the tiles does not matter to the running softmax).  Measured: configs[1] 221.2 -> 219.2 us
    // with even slices, where the wavefront that holds the residual keys is the last to finish; with balanced
    // slices, where it is not, configs[2] 92.7 -> 94.2 us, so those keep the residual keys at the end.
    auto residual_tiles = [&]() {
        if (r0 >= r1) return;
        // scores = K . q^T on the matrix cores, as the reference's half-precision matmul (:79): for 16 tokens
        // at a time D[token][head] += K[token][16 dims] * q[head][16 dims], heads padded to the 16 columns.
        // Lane (g,n) supplies, for step (kb, hf), dims 32 kb + 8 g + 4 hf .. +3 of key row n and of query head
        // n: both operands use the same order of the contraction index, so one 16-byte load per lane feeds two
        // MFMAs, and the four lanes of a row read 64 contiguous bytes.  All 16 loads of a 64-token tile are
        // in flight at once.  The D tiles go through LDS (the table region) to the lane == token layout.
        asm volatile("" ::: "memory");
        const int g = lane >> 4, n = lane & 15;
        uint4 qv[4];
#pragma unroll
        for (int kb = 0; kb < 4; kb++) {
            qv[kb] = (n < rep) ? *reinterpret_cast<const uint4*>(qb + n * kHeadDim + 32 * kb + 8 * g) : make_uint4(0u, 0u, 0u, 0u);
        }
        const __amdgpu_buffer_rsrc_t rk = make_rsrc(p.k_resid + static_cast<size_t>(bh) * resid_capacity * kHeadDim,
                                                    static_cast<uint32_t>(nres) * (kHeadDim * 2));
        const uint32_t voff_k = static_cast<uint32_t>(n) * (kHeadDim * 2) + static_cast<uint32_t>(g) * 16;
        for (int tt = r0; tt < r1; tt++) {
            const int tok = tt * kWave + lane;
            const bool valid = tok < nres;
            const uint32_t arow = static_cast<uint32_t>(nb) * kGroup + tt * kWave;   // absolute row of lane 0
            uint4 kk[4][4];
#pragma unroll
            for (int tb = 0; tb < 4; tb++)
#pragma unroll
                for (int kb = 0; kb < 4; kb++)
                    kk[tb][kb] = buf_load16(rk, voff_k, static_cast<uint32_t>(tt * kWave + 16 * tb) * (kHeadDim * 2) + 64 * kb);
            uint4 vv[4][4];
            load_v_tile(vv, rv, voff_v, (V4 ? static_cast<uint32_t>(tt * kWave) : arow) * (kHeadDim * 2));
#pragma unroll
            for (int tb = 0; tb < 4; tb++) {
                floatx4 d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int kb = 0; kb < 4; kb++) {
                    d = mfma16<T>(make_uint2(kk[tb][kb].x, kk[tb][kb].y), make_uint2(qv[kb].x, qv[kb].y), d);
                    d = mfma16<T>(make_uint2(kk[tb][kb].z, kk[tb][kb].w), make_uint2(qv[kb].z, qv[kb].w), d);
                }
                // d[i] = score of token 16 tb + 4 g + i for head n
                if (n < REPP) {
                    lds_e4* dst = lds_ptr<lds_e4>(lut + (n * kWave + 16 * tb + 4 * g) * 4);
                    dst->x = d[0]; dst->y = d[1]; dst->z = d[2]; dst->w = d[3];
                }
            }
            asm volatile("" ::: "memory");
            const bool keep = valid && (has_mask ? (__builtin_amdgcn_raw_buffer_load_b8(rm, lane, static_cast<int>(arow), 0) != 0) : true);
            float s[REPP];
#pragma unroll
            for (int j = 0; j < REPP; j++) {
                // the reference multiplies q.K^T in the model dtype before promoting (:79)
                const float sr = lo2f<T>(f2lo<T>(*lds_ptr<lds_f1>(lut + (j * kWave + lane) * 4)));
                s[j] = keep ? sr * scale_log2 : -INFINITY;
            }
            asm volatile("" ::: "memory");
            softmax_pv_tile<T, REPP>(st, s, vv, pbuf, lane);
        }
    };

    {
        // ---------------- quantized tiles [t0, t1) ----------------
        if (t0 < t1) {
            const int g0 = t0 >> 1, g1 = (t1 + 1) >> 1;
            // the query rows of all heads are requested at once, and nothing waits for them before the table is
            // built: a load under `j < rep` would be a branch with its own wait, one memory round trip per head
            // before the first codes are even requested (a padded head re-reads row 0 and is zeroed afterwards)
            uint16_t qraw[REPP][2];
#pragma unroll
            for (int j = 0; j < REPP; j++) {
                const uint16_t* qrow = qb + (j < rep ? j : 0) * kHeadDim + lane;
                qraw[j][0] = qrow[0];
                qraw[j][1] = qrow[kPairs];
            }
            const size_t plane = static_cast<size_t>(bh) * group_capacity;
            // a token's code row: 64 bytes, or 48 when the 6-bit codes are stored packed
            constexpr int kRowB = PK6 ? kPackedRowBytes : kPairs, kRowLoads = kRowB / 16;
            const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.codes + plane * (kGroup * kRowB),
                                                        static_cast<uint32_t>(nb) * (kGroup * kRowB));
            const uint32_t voff_c = static_cast<uint32_t>(lane) * kRowB;
            // software pipeline: codes of the next tile and metadata of the next group are in flight
            uint4 cnext[kRowLoads];
#pragma unroll
            for (int i = 0; i < kRowLoads; i++) cnext[i] = buf_load16(rc, voff_c, static_cast<uint32_t>(t0) * (kWave * kRowB) + 16 * i);
            const uint16_t* prs = p.rscale + plane * kPairs + lane;
            const uint16_t* prm = p.rmn + plane * kPairs + lane;
            const uint16_t* pts = p.tscale + plane * kPairs + lane;
            const uint16_t* ptm = p.tmn + plane * kPairs + lane;
            uint16_t mrs = prs[g0 * kPairs], mrm = prm[g0 * kPairs], mts = pts[g0 * kPairs], mtm = ptm[g0 * kPairs];
            // V operands are double-buffered by tile parity: tile t+1 is requested before tile t is scored
            VTile<V4> vv[2];
            const size_t vplane = static_cast<size_t>(bh) * static_cast<size_t>(V4 ? v4.capacity : 0);
            const __amdgpu_buffer_rsrc_t rq = make_rsrc(V4 ? v4.codes + vplane * 16 : nullptr,
                                                        V4 ? static_cast<uint32_t>(nb) * (kGroup * 64) : 0u);
            const __amdgpu_buffer_rsrc_t rvs = make_rsrc(V4 ? v4.scale + vplane : nullptr, V4 ? static_cast<uint32_t>(nb) * (kGroup * 2) : 0u);
            const __amdgpu_buffer_rsrc_t rvz = make_rsrc(V4 ? v4.zero + vplane : nullptr, V4 ? static_cast<uint32_t>(nb) * (kGroup * 2) : 0u);
            const uint32_t voff_q = static_cast<uint32_t>(lane >> 4) * 64 + static_cast<uint32_t>(lane & 15) * 4;
            uint16_t vsz[2][2] = {{0, 0}, {0, 0}};             // (scale, zero-point) words of this lane's token, by tile parity
            auto load_values = [&](int buf, uint32_t tile_tok, bool in_range) {
                if constexpr (V4) {
                    load_v4_tile(vv[buf].r, rq, voff_q, in_range ? tile_tok * 64u : 0xFFFF0000u);
                    const int so = in_range ? static_cast<int>(tile_tok * 2u) : static_cast<int>(0x7FFFFF00);
                    vsz[buf][0] = __builtin_amdgcn_raw_buffer_load_b16(rvs, lane * 2, so, 0);
                    vsz[buf][1] = __builtin_amdgcn_raw_buffer_load_b16(rvz, lane * 2, so, 0);
                } else {
                    load_v_tile(vv[buf].r, rv, voff_v, in_range ? tile_tok * (kHeadDim * 2) : 0xFFFF0000u);
                }
            };
            if (t0 & 1) load_values(1, static_cast<uint32_t>(t0) * kWave, true);
            else load_values(0, static_cast<uint32_t>(t0) * kWave, true);
            // (with 4-bit values the accumulators are in scaled units until finish_v4: the residual tiles, whose
            // values are half precision, have to come after it)
            if constexpr (!V4 && RESID_FIRST) residual_tiles();
            float qx[REPP], qy[REPP];
#pragma unroll
            for (int j = 0; j < REPP; j++) {
                qx[j] = j < rep ? lo2f<T>(qraw[j][0]) : 0.0f;
                qy[j] = j < rep ? lo2f<T>(qraw[j][1]) : 0.0f;
            }
            PQ_T_DECL;
            for (int grp = g0; grp < g1; grp++) {
                PQ_T_MARK();
                asm volatile("" ::: "memory");
                const float cdv = build_lut<T, TB, REPP>(lut, lane, qx, qy, mrs, mrm, mts, mtm);
                float cds[kPairs];
                broadcast_cd(cdv, cds);
                asm volatile("" ::: "memory");
                PQ_T_ADD(0);
                if (grp + 1 < g1) {
                    const int o = (grp + 1) * kPairs;
                    mrs = prs[o]; mrm = prm[o]; mts = pts[o]; mtm = ptm[o];
                }
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    const int tt = 2 * grp + half;
                    if (tt < t0 || tt >= t1) continue;            // a piece may begin or end in the middle of a group
                    const uint32_t tok0 = static_cast<uint32_t>(tt) * kWave;
                    // past the last tile of this slice the loads run off the buffer's end and return zeros (the
                    // out-of-range offset leaves room for the 16 KiB of row offsets added to it: no 32-bit wrap)
                    PQ_T_MARK();
                    load_values(half ^ 1, tok0 + kWave, tt + 1 < t1);
                    PQ_T_ADD(1);
                    uint32_t cw[16];
                    if constexpr (PK6) {
                        uint32_t pk[12];
#pragma unroll
                        for (int i = 0; i < 3; i++) {
                            pk[4 * i] = cnext[i].x; pk[4 * i + 1] = cnext[i].y; pk[4 * i + 2] = cnext[i].z; pk[4 * i + 3] = cnext[i].w;
                        }
                        unpack6(pk, cw);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            cw[4 * i] = cnext[i].x; cw[4 * i + 1] = cnext[i].y; cw[4 * i + 2] = cnext[i].z; cw[4 * i + 3] = cnext[i].w;
                        }
                    }
                    PQ_T_KEEP(cw[0]);
                    PQ_T_KEEP(cw[15]);
                    PQ_T_ADD(2);
                    if (tt + 1 < t1) {
#pragma unroll
                        for (int i = 0; i < kRowLoads; i++)
                            cnext[i] = buf_load16(rc, voff_c, static_cast<uint32_t>(tt + 1) * (kWave * kRowB) + 16 * i);
                    }
                    PQ_T_ADD(3);
                    float s[REPP];
#pragma unroll
                    for (int j = 0; j < REPP; j++) s[j] = 0.0f;
                    score_token<TB, REPP>(lut, cw, cds, s);
                    PQ_T_KEEP(s[0]);
                    PQ_T_ADD(4);
                    const bool keep = has_mask ? (__builtin_amdgcn_raw_buffer_load_b8(rm, lane, static_cast<int>(tok0), 0) != 0) : true;
#pragma unroll
                    for (int j = 0; j < REPP; j++) s[j] = keep ? s[j] * scale_log2 : -INFINITY;
                    if constexpr (V4) {
                        softmax_pv_tile_v4<REPP>(st, s, vv[half].r, lo2f<T>(vsz[half][0]), lo2f<T>(vsz[half][1]), pbuf, lane);
                    } else {
                        softmax_pv_tile<T, REPP>(st, s, vv[half].r, pbuf, lane);
                    }
                    PQ_T_KEEP(st.acc[0][0]);
                    PQ_T_ADD(5);
                }
                PQ_T_FIRST_GROUP_DONE();
            }
            PQ_T_REPORT(g1 - g0);
            if constexpr (V4) finish_v4<REPP>(st, lane);
            if constexpr (V4 || !RESID_FIRST) residual_tiles();
        } else {
            residual_tiles();
        }
    }
    // ---------------- write the partial ----------------
    float lsum[REPP];
#pragma unroll
    for (int j = 0; j < REPP; j++) lsum[j] = wave_sum(st.l[j]);
    const int g = lane >> 4, n = lane & 15;
    if (n < rep) {
        float mm = st.m[0], ll = lsum[0];
#pragma unroll
        for (int j = 1; j < REPP; j++) { mm = (n == j) ? st.m[j] : mm; ll = (n == j) ? lsum[j] : ll; }
        float* pw = ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep + n) * n_splits + slot) * kPartialFloats;
        if (g == 0) { pw[0] = mm; pw[1] = ll; }
        float* pa = pw + 4 + 32 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<float4*>(pa + 8 * i) = make_float4(st.acc[0][i], st.acc[1][i], st.acc[2][i], st.acc[3][i]);
            *reinterpret_cast<float4*>(pa + 8 * i + 4) = make_float4(st.acc[4][i], st.acc[5][i], st.acc[6][i], st.acc[7][i]);
        }
    }
    PQ_T_EXIT();
}

// Mark the partial slots [first, n_splits) of the `rep` query heads of (b, kvh) as holding nothing.
// Both header words: the workspace is not cleared between calls, and the merge must not meet a
// stale probability sum (0 * NaN) in a slot that holds nothing.
__device__ __forceinline__ void mark_empty_slots(const AttnParams& p, int lane, int b, int kvh, int first) {
    const int count = (p.n_splits - first) * p.rep;
    for (int i = lane; i < count; i += kWave) {
        const int j = i / (p.n_splits - first), s = first + i % (p.n_splits - first);
        float* pw = p.ws + ((static_cast<size_t>(b) * p.N + static_cast<size_t>(kvh) * p.rep + j) * p.n_splits + s) * kPartialFloats;
        pw[0] = -INFINITY;
        pw[1] = 0.0f;
    }
}

#define PQ_ATTN_KERNEL_PARAMS                                                                                        \
    const uint16_t* __restrict__ q, const uint8_t* __restrict__ codes, const uint16_t* __restrict__ rscale,          \
        const uint16_t* __restrict__ rmn, const uint16_t* __restrict__ tscale, const uint16_t* __restrict__ tmn,     \
        int group_capacity, int n_groups, const int32_t* __restrict__ n_groups_per_seq,                              \
        const uint16_t* __restrict__ k_resid, int resid_capacity, int n_resid,                                       \
        const int32_t* __restrict__ n_resid_per_seq, const uint16_t* __restrict__ v, int64_t v_capacity,             \
        const uint8_t* __restrict__ mask, int64_t mask_stride, float scale_log2, int B, int N, int Nk, int rep,      \
        int n_splits, int min_gps, float* __restrict__ ws, V4Args v4
#define PQ_ATTN_KERNEL_PACK                                                                                          \
    AttnParams p;                                                                                                    \
    p.q = q; p.codes = codes; p.rscale = rscale; p.rmn = rmn; p.tscale = tscale; p.tmn = tmn;                        \
    p.group_capacity = group_capacity; p.n_groups = n_groups; p.n_groups_per_seq = n_groups_per_seq;                 \
    p.k_resid = k_resid; p.resid_capacity = resid_capacity; p.n_resid = n_resid; p.n_resid_per_seq = n_resid_per_seq; \
    p.v = v; p.v_capacity = v_capacity; p.mask = mask; p.mask_stride = mask_stride; p.scale_log2 = scale_log2;      \
    p.B = B; p.N = N; p.Nk = Nk; p.rep = rep; p.n_splits = n_splits; p.min_gps = min_gps; p.ws = ws

// Even slices: block (plane bh, slice `split`) takes groups [split * gps, (split + 1) * gps) of its
// sequence, gps = max(min_gps, ceil(groups / n_splits)); the block that holds the last group also
// takes the residual keys.
template <typename T, int TB, int REPP, bool V4, bool PK6>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu((V4 && REPP <= 4) ? 2 : 1, 2)))
void attn_kernel(PQ_ATTN_KERNEL_PARAMS) {
    using L = Lut<TB, REPP>;
    // the table region doubles as the staging buffer of the residual block's scores ([REPP][64] fp32)
    constexpr int kLutBytes = L::BYTES > REPP * kWave * 4 ? L::BYTES : REPP * kWave * 4;
    __shared__ __attribute__((aligned(16))) char lut_mem[kLutBytes];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[REPP * kWave];
    const uint32_t lut = lds_addr(lut_mem), pbuf = lds_addr(p_mem);
    PQ_ATTN_KERNEL_PACK;

    const int lane = threadIdx.x;
    // 1-D grid, (batch, KV head) index fastest.  Consecutive workgroup ids go to different XCDs, so
    // every XCD receives whole (batch, KV head) planes with all their slices; with the slice index
    // fastest an XCD would receive one slice index of every plane, and in a ragged batch the XCDs
    // that own the high slice indices would sit idle (measured: 165 us instead of 120 us).
    const int units = gridDim.x / n_splits;
    const int bh = blockIdx.x % units;
    const int split = blockIdx.x / units;
    const int b = bh / Nk, kvh = bh - b * Nk;
    const SeqCounts sc = seq_counts<V4>(p, v4, b);

    // groups per slice: an even split of this sequence, but never fewer than min_gps (ragged
    // batches: short sequences then use fewer slices, and the unused blocks return at once)
    int gps = (sc.nb + n_splits - 1) / n_splits;
    gps = gps < min_gps ? min_gps : gps;
    // slices past the end of a short sequence have nothing to do: mark their partials empty and leave
    if (split > 0 && split * gps >= sc.nb) {
        if (lane < rep) {
            float* pw = ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep + lane) * n_splits + split) * kPartialFloats;
            pw[0] = -INFINITY;
            pw[1] = 0.0f;
        }
        return;
    }
    const int g0 = split * gps;
    const int g1 = (g0 + gps) < sc.nb ? (g0 + gps) : sc.nb;
    // the residual keys go to the block that holds the last quantized group of the sequence
    const int last_split = sc.nb > 0 ? (sc.nb - 1) / gps : 0;
    attn_piece<T, TB, REPP, V4, PK6, true>(p, v4, lut, pbuf, lane, b, kvh, sc, 2 * g0, 2 * g1, 0,
                                     split == last_split ? (sc.nres + kWave - 1) / kWave : 0, split);
}

// Units a plane's start-up counts for when the balanced kernel cuts the line (query, first table, first loads, the
// partial's write: measured at configs[2], 0 / 1 / 2 / 3 units: 92.8 / 89.6 / 87.9 / 88.6 us).
constexpr int kStartUnits = 2;

__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// Balanced slices: the work of the whole batch is laid out as one line of units, plane after plane
// (plane = (sequence, KV head), sequence-major).  A plane is kStartUnits units that stand for its
// start-up, then one unit per tile of 64 tokens: two per quantized group, then one per 64 residual
// keys.  The line is cut into segments of `seg` units, the same for every wavefront; wavefront w
// works through segment w, which may end one plane and begin the next: every piece of a plane it
// touches becomes one partial.  The piece of plane P cut by segment w goes to slot
// w - floor(start of P / seg) of that plane's heads, and the piece that ends P marks the slots
// behind it empty.
//   seg = max(2 min_gps, ceil(line length / wavefronts),
//             ceil((2 group_capacity + ceil(resid_capacity / 64) + kStartUnits) / (n_splits - 1)))
// The last term guarantees that no plane is cut into more than n_splits pieces (n_splits >= 2: a
// plane shorter than a segment can still lie across one cut).  All of this is computed from the
// per-sequence counts in device memory, by every wavefront alike, so the slices follow the real
// lengths of a ragged or growing batch without the host knowing them.
// The walk of wavefront (or pair) `w` of `W` over its segment of the line: calls
// piece(b, kvh, counts, t0, t1, r0, r1, slot, ends_plane) for every piece, in order.  `walk` is the LDS byte address
// of 8 ints that belong to the calling wavefront: the state of the walk lives there between pieces, so that nothing
// of it occupies registers inside a piece (the group loop already uses every scalar register).
template <bool V4, typename F>
__device__ __forceinline__ void walk_segment(const AttnParams& p, const V4Args& v4, long long W, long long w, int lane,
                                             uint32_t walk, F&& piece) {
    const int B = p.B, Nk = p.Nk;
    // units of one plane of sequence bb: kStartUnits for the plane's start-up (they also make a sequence with
    // nothing at all a plane of its own, so that somebody writes its partials), then its tiles
    auto units_of = [&](int bb) {
        const SeqCounts c = seq_counts<V4>(p, v4, bb);
        return kStartUnits + 2 * c.nb + (c.nres + kWave - 1) / kWave;
    };
    // length of the line
    int mine = 0;
    for (int base = 0; base < B; base += kWave) mine += (base + lane < B) ? units_of(base + lane) : 0;
    const long long per_head = wave_sum_i(mine);          // units of one KV head's planes, all sequences
    const long long total = per_head * Nk;
    long long seg = (total + W - 1) / W;
    seg = seg < 2 * p.min_gps ? 2 * p.min_gps : seg;
    // the most units a plane can have (the residual window is 128 keys in the reference, but the interface takes
    // any resid_capacity)
    const long long cap_units = 2 * static_cast<long long>(p.group_capacity) + (p.resid_capacity + kWave - 1) / kWave + kStartUnits;
    const long long fit = (cap_units + p.n_splits - 2) / (p.n_splits - 1);      // n_splits >= 2 (checked on the host)
    seg = seg < fit ? fit : seg;
    const long long start = w * seg;
    if (start >= total) return;
    const long long end = (start + seg) < total ? (start + seg) : total;

    // the sequence that holds unit `start`: units before sequence bb are Nk * (sum of u over earlier sequences)
    int b = 0;
    long long before = 0;                                  // units of one head's planes before sequence b
    for (int base = 0; base < B; base += kWave) {
        const int u = (base + lane < B) ? units_of(base + lane) : 0;
        int incl = u;
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
            const int t = __shfl_up(incl, o);
            incl += (lane >= o) ? t : 0;
        }
        const long long chunk = __shfl(incl, kWave - 1);
        if (start < (before + chunk) * Nk) {
            const unsigned long long past = __ballot((before + incl) * Nk > start);
            const int l0 = __builtin_ctzll(past);
            b = base + l0;
            before += __shfl(incl - u, l0);
            break;
        }
        before += chunk;
    }
    typedef __attribute__((address_space(3))) int lds_i1;
    {
        const int u0 = units_of(b);
        const long long seq_start = before * Nk;            // line position of plane (b, 0)
        const int kvh0 = static_cast<int>((start - seq_start) / u0);
        const long long plane_start = seq_start + static_cast<long long>(kvh0) * u0;
        const long long span = end - start;
        if (lane == 0) {
            lds_i1* wk = lds_ptr<lds_i1>(walk);
            wk[0] = b; wk[1] = kvh0; wk[2] = static_cast<int>(start - plane_start); wk[3] = u0;
            wk[4] = static_cast<int>(span < 0x7fffffffLL ? span : 0x7fffffffLL);          // units left in the segment
            wk[5] = static_cast<int>(w - plane_start / seg);                               // slot of the first piece
        }
    }
    for (;;) {
        asm volatile("" ::: "memory");
        const lds_i1* wk = lds_ptr<lds_i1>(walk);
        const int cb = __builtin_amdgcn_readfirstlane(wk[0]), ckvh = __builtin_amdgcn_readfirstlane(wk[1]);
        const int ua = __builtin_amdgcn_readfirstlane(wk[2]), u = __builtin_amdgcn_readfirstlane(wk[3]);
        const int left = __builtin_amdgcn_readfirstlane(wk[4]), slot = __builtin_amdgcn_readfirstlane(wk[5]);
        if (left <= 0 || cb >= B) break;
        const int ub = (u - ua) < left ? u : ua + left;
        asm volatile("" ::: "memory");
        // the state of the next piece: a plane that begins inside this segment has its first piece here (slot 0)
        {
            int nb_ = cb, nk = ckvh, nu = u;
            if (ub == u) {
                if (++nk == Nk) { nk = 0; ++nb_; nu = nb_ < B ? units_of(nb_) : 1; }
            }
            if (lane == 0) {
                lds_i1* ww = lds_ptr<lds_i1>(walk);
                ww[0] = nb_; ww[1] = nk; ww[2] = ub == u ? 0 : ub; ww[3] = nu;
                ww[4] = left - (ub - ua); ww[5] = 0;
            }
        }
        const SeqCounts sc = seq_counts<V4>(p, v4, cb);
        // the first kStartUnits units of a plane stand for its start-up; then the tiles of the quantized part,
        // then the residual keys'
        const int ta = ua > kStartUnits ? ua - kStartUnits : 0, tb = ub > kStartUnits ? ub - kStartUnits : 0;
        const int qt = 2 * sc.nb;
        const int t0 = ta < qt ? ta : qt, t1 = tb < qt ? tb : qt;
        const int r0 = ta > qt ? ta - qt : 0, r1 = tb > qt ? tb - qt : 0;
        piece(cb, ckvh, sc, t0, t1, r0, r1, slot, ub == u);
    }
}

template <typename T, int TB, int REPP, bool V4, bool PK6>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu((V4 && REPP <= 4) ? 2 : 1, 2)))
void attn_balanced_kernel(PQ_ATTN_KERNEL_PARAMS) {
    using L = Lut<TB, REPP>;
    constexpr int kLutBytes = L::BYTES > REPP * kWave * 4 ? L::BYTES : REPP * kWave * 4;
    __shared__ __attribute__((aligned(16))) char lut_mem[kLutBytes];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[REPP * kWave];
    __shared__ int walk[8];
    const uint32_t lut = lds_addr(lut_mem), pbuf = lds_addr(p_mem);
    PQ_ATTN_KERNEL_PACK;
    const int lane = threadIdx.x;
    walk_segment<V4>(p, v4, gridDim.x, blockIdx.x, lane, lds_addr(walk),
                     [&](int cb, int ckvh, const SeqCounts& sc, int t0, int t1, int r0, int r1, int slot, bool ends_plane) {
                         // the piece that ends its plane marks the slots behind its own as holding nothing
                         if (ends_plane && slot + 1 < n_splits) mark_empty_slots(p, lane, cb, ckvh, slot + 1);
                         attn_piece<T, TB, REPP, V4, PK6, false>(p, v4, lut, pbuf, lane, cb, ckvh, sc, t0, t1, r0, r1, slot);
                     });
}

// ---------------------------------------------------------------------------------------------
// Paired wavefronts (PQ_PAIRED_WAVES): the work of one slice is shared by the two wavefronts that
// sit on one SIMD.  The SCORER reads the codes, builds the tables and produces the scores of a
// 64-token tile; the ACCUMULATOR streams the values, and does the mask, the softmax update and
// P.V; the scores cross over in LDS, double-buffered, so the scorer works on tile t+1 while the
// accumulator finishes tile t.  Inside one wavefront those phases can only follow each other, and
// their sum, not the memory system, sets the time per group (8 heads per KV head most of all).
//
// A workgroup is 8 wavefronts = one compute unit's worth at 256 registers each, so the hardware
// puts exactly two on every SIMD; which two is read from the hardware id register, and the two
// that share a SIMD form a pair (lower wavefront index = scorer).  If the ids do not come out in
// pairs the wavefronts are paired as (w, w + 4): the results are the same, only the overlap is lost.
// The two hand tiles over through two counters in LDS (tiles published / tiles consumed); a wait
// gives up after kSpinLimit polls, flags the slice as failed and lets both wavefronts run out.
constexpr int kPairsPerBlock = 4;
constexpr int kSpinLimit = 1 << 22;

struct PairMem {
    uint32_t lut;      // the scorer's table
    uint32_t sbuf;     // [2][REPP][64] fp32 scores
    uint32_t pbuf;     // the accumulator's probability staging
    uint32_t flags;    // int[4]: published, consumed, failed, -
};

typedef __attribute__((address_space(3))) volatile int lds_vi;

__device__ __forceinline__ bool pair_wait(uint32_t addr, int want) {
    bool seen = false;
    for (int i = 0; i < kSpinLimit; i++) {
        if (*lds_ptr<lds_vi>(addr) >= want) { seen = true; break; }
        __builtin_amdgcn_s_sleep(1);
    }
    asm volatile("" ::: "memory");       // nothing that follows may be read or written ahead of the counter
    return seen;
}

// Which pair of its workgroup a wavefront belongs to, and its role in it (0 scorer, 1 accumulator); also clears the
// pairs' counters.  All 8 wavefronts of the workgroup call this once, before anything else (it holds a barrier).
__device__ __forceinline__ void pair_roles(int* simd_of, int* flags, int wave, int lane, int& pair, int& role) {
    // HW_ID (register 4), bits [5:4]: the SIMD this wavefront runs on
    const int simd = static_cast<int>(__builtin_amdgcn_s_getreg((1 << 11) | (4 << 6) | 4));
    if (lane == 0) simd_of[wave] = simd;
    if (threadIdx.x < kPairsPerBlock * 4) flags[threadIdx.x] = 0;
    __syncthreads();
    int partner = -1, same = 0;
    bool paired = true;
#pragma unroll
    for (int w = 0; w < 2 * kPairsPerBlock; w++) {
        int cnt = 0;
#pragma unroll
        for (int u = 0; u < 2 * kPairsPerBlock; u++) cnt += simd_of[u] == simd_of[w];
        paired = paired && cnt == 2;
        if (w != wave && simd_of[w] == simd) { partner = w; same++; }
    }
    if (paired && same == 1) { pair = simd & (kPairsPerBlock - 1); role = wave > partner; }
    else                     { pair = wave & (kPairsPerBlock - 1); role = wave >> 2; }
    pair = __builtin_amdgcn_readfirstlane(pair);
    role = __builtin_amdgcn_readfirstlane(role);
}

// Scorer: quantized tiles [t0, t1), then residual tiles [r0, r1), of plane (b, kvh).  `k` counts the tiles this pair
// has handed over since the kernel began.  -> false if the partner stopped answering.
template <typename T, int TB, int REPP, bool PK6>
__device__ __forceinline__ bool pair_scorer(const AttnParams& p, const PairMem& pm, int lane, int b, int kvh, const SeqCounts& sc,
                                            int t0, int t1, int r0, int r1, int& k) {
    const int rep = p.rep;
    const int bh = b * p.Nk + kvh;
    const int nb = sc.nb, nres = sc.nres;
    const uint16_t* qb = p.q + (static_cast<size_t>(b) * p.N + static_cast<size_t>(kvh) * rep) * kHeadDim;
    bool ok = true;
    auto publish_begin = [&]() {            // the buffer of tile k is free once tile k - 2 has been consumed
        if (k >= 2) ok = ok && pair_wait(pm.flags + 4, k - 1);
        return pm.sbuf + (k & 1) * (REPP * kWave * 4);
    };
    auto publish_end = [&]() {
        asm volatile("" ::: "memory");
        k++;
        if (lane == 0) *lds_ptr<lds_vi>(pm.flags) = k;
        asm volatile("" ::: "memory");
    };
    if (t0 < t1) {
        const int g0 = t0 >> 1, g1 = (t1 + 1) >> 1;
        uint16_t qraw[REPP][2];
#pragma unroll
        for (int j = 0; j < REPP; j++) {
            const uint16_t* qrow = qb + (j < rep ? j : 0) * kHeadDim + lane;
            qraw[j][0] = qrow[0];
            qraw[j][1] = qrow[kPairs];
        }
        const size_t plane = static_cast<size_t>(bh) * p.group_capacity;
        constexpr int kRowB = PK6 ? kPackedRowBytes : kPairs, kRowLoads = kRowB / 16;
        const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.codes + plane * (kGroup * kRowB), static_cast<uint32_t>(nb) * (kGroup * kRowB));
        const uint32_t voff_c = static_cast<uint32_t>(lane) * kRowB;
        uint4 cnext[kRowLoads];
#pragma unroll
        for (int i = 0; i < kRowLoads; i++) cnext[i] = buf_load16(rc, voff_c, static_cast<uint32_t>(t0) * (kWave * kRowB) + 16 * i);
        const uint16_t* prs = p.rscale + plane * kPairs + lane;
        const uint16_t* prm = p.rmn + plane * kPairs + lane;
        const uint16_t* pts = p.tscale + plane * kPairs + lane;
        const uint16_t* ptm = p.tmn + plane * kPairs + lane;
        uint16_t mrs = prs[g0 * kPairs], mrm = prm[g0 * kPairs], mts = pts[g0 * kPairs], mtm = ptm[g0 * kPairs];
        float qx[REPP], qy[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) {
            qx[j] = j < rep ? lo2f<T>(qraw[j][0]) : 0.0f;
            qy[j] = j < rep ? lo2f<T>(qraw[j][1]) : 0.0f;
        }
        for (int grp = g0; grp < g1; grp++) {
            asm volatile("" ::: "memory");
            const float cdv = build_lut<T, TB, REPP>(pm.lut, lane, qx, qy, mrs, mrm, mts, mtm);
            float cds[kPairs];
            broadcast_cd(cdv, cds);
            asm volatile("" ::: "memory");
            if (grp + 1 < g1) {
                const int o = (grp + 1) * kPairs;
                mrs = prs[o]; mrm = prm[o]; mts = pts[o]; mtm = ptm[o];
            }
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int tt = 2 * grp + half;
                if (tt < t0 || tt >= t1) continue;
                uint32_t cw[16];
                if constexpr (PK6) {
                    uint32_t pk[12];
#pragma unroll
                    for (int i = 0; i < 3; i++) {
                        pk[4 * i] = cnext[i].x; pk[4 * i + 1] = cnext[i].y; pk[4 * i + 2] = cnext[i].z; pk[4 * i + 3] = cnext[i].w;
                    }
                    unpack6(pk, cw);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        cw[4 * i] = cnext[i].x; cw[4 * i + 1] = cnext[i].y; cw[4 * i + 2] = cnext[i].z; cw[4 * i + 3] = cnext[i].w;
                    }
                }
                if (tt + 1 < t1) {
#pragma unroll
                    for (int i = 0; i < kRowLoads; i++)
                        cnext[i] = buf_load16(rc, voff_c, static_cast<uint32_t>(tt + 1) * (kWave * kRowB) + 16 * i);
                }
                float s[REPP];
#pragma unroll
                for (int j = 0; j < REPP; j++) s[j] = 0.0f;
                score_token<TB, REPP>(pm.lut, cw, cds, s);
                const uint32_t dst = publish_begin();
#pragma unroll
                for (int j = 0; j < REPP; j++) *lds_ptr<lds_f1>(dst + (j * kWave + lane) * 4) = s[j];
                publish_end();
            }
        }
    }
    if (r0 < r1) {
        // residual keys: K . q^T on the matrix cores, as in attn_piece; the D tiles go straight to the score buffer
        const int g = lane >> 4, n = lane & 15;
        uint4 qv[4];
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
            qv[kb] = (n < rep) ? *reinterpret_cast<const uint4*>(qb + n * kHeadDim + 32 * kb + 8 * g) : make_uint4(0u, 0u, 0u, 0u);
        const __amdgpu_buffer_rsrc_t rk = make_rsrc(p.k_resid + static_cast<size_t>(bh) * p.resid_capacity * kHeadDim,
                                                    static_cast<uint32_t>(nres) * (kHeadDim * 2));
        const uint32_t voff_k = static_cast<uint32_t>(n) * (kHeadDim * 2) + static_cast<uint32_t>(g) * 16;
        for (int tt = r0; tt < r1; tt++) {
            uint4 kk[4][4];
#pragma unroll
            for (int tb = 0; tb < 4; tb++)
#pragma unroll
                for (int kb = 0; kb < 4; kb++)
                    kk[tb][kb] = buf_load16(rk, voff_k, static_cast<uint32_t>(tt * kWave + 16 * tb) * (kHeadDim * 2) + 64 * kb);
            floatx4 d[4];
#pragma unroll
            for (int tb = 0; tb < 4; tb++) {
                d[tb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int kb = 0; kb < 4; kb++) {
                    d[tb] = mfma16<T>(make_uint2(kk[tb][kb].x, kk[tb][kb].y), make_uint2(qv[kb].x, qv[kb].y), d[tb]);
                    d[tb] = mfma16<T>(make_uint2(kk[tb][kb].z, kk[tb][kb].w), make_uint2(qv[kb].z, qv[kb].w), d[tb]);
                }
            }
            const uint32_t dst = publish_begin();
            if (n < REPP) {
#pragma unroll
                for (int tb = 0; tb < 4; tb++) {
                    lds_e4* o = lds_ptr<lds_e4>(dst + (n * kWave + 16 * tb + 4 * g) * 4);
                    o->x = d[tb][0]; o->y = d[tb][1]; o->z = d[tb][2]; o->w = d[tb][3];
                }
            }
            publish_end();
        }
    }
    return ok;
}

// Accumulator: the same tiles in the same order; writes the partial of the piece to `slot`.
template <typename T, int REPP>
__device__ __forceinline__ bool pair_accumulator(const AttnParams& p, const PairMem& pm, int lane, int b, int kvh, const SeqCounts& sc,
                                                 int t0, int t1, int r0, int r1, int slot, int& k) {
    const int N = p.N, rep = p.rep;
    const int bh = b * p.Nk + kvh;
    const int nb = sc.nb, nres = sc.nres;
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(p.v + static_cast<size_t>(bh) * p.v_capacity * kHeadDim,
                                                static_cast<uint32_t>(sc.n_tokens * (kHeadDim * 2)));
    const uint32_t voff_v = static_cast<uint32_t>(lane >> 4) * (4 * kHeadDim * 2) + static_cast<uint32_t>(lane & 15) * 16;
    const bool has_mask = p.mask != nullptr;
    const __amdgpu_buffer_rsrc_t rm = make_rsrc(has_mask ? p.mask + static_cast<size_t>(b) * p.mask_stride : nullptr,
                                                has_mask ? static_cast<uint32_t>(sc.n_tokens < p.mask_stride ? sc.n_tokens : p.mask_stride) : 0u);
    AttnState<REPP> st;
#pragma unroll
    for (int j = 0; j < REPP; j++) { st.m[j] = -INFINITY; st.l[j] = 0.0f; st.zp[j] = 0.0f; }
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    bool ok = true;
    // tile i of the piece: quantized tile t0 + i, or residual tile r0 + (i - nq); -> absolute row of its first token
    const int nq = t1 > t0 ? t1 - t0 : 0, nr = r1 > r0 ? r1 - r0 : 0, nt = nq + nr;
    auto row_of = [&](int i) { return i < nq ? (t0 + i) * kWave : nb * kGroup + (r0 + i - nq) * kWave; };
    VTile<false> vv[2];
    if (nt > 0) load_v_tile(vv[0].r, rv, voff_v, static_cast<uint32_t>(row_of(0)) * (kHeadDim * 2));
    auto step = [&](auto BUF, int i) {
        constexpr int buf = decltype(BUF)::value;
        load_v_tile(vv[buf ^ 1].r, rv, voff_v, i + 1 < nt ? static_cast<uint32_t>(row_of(i + 1)) * (kHeadDim * 2) : 0xFFFF0000u);
        const int row = row_of(i);
        const bool resid = i >= nq;
        const bool valid = resid ? (r0 + i - nq) * kWave + lane < nres : true;
        const bool keep = valid && (has_mask ? (__builtin_amdgcn_raw_buffer_load_b8(rm, lane, row, 0) != 0) : true);
        ok = ok && pair_wait(pm.flags, k + 1);
        const uint32_t src = pm.sbuf + (k & 1) * (REPP * kWave * 4);
        float s[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) s[j] = *lds_ptr<lds_f1>(src + (j * kWave + lane) * 4);
        asm volatile("" ::: "memory");
        k++;
        if (lane == 0) *lds_ptr<lds_vi>(pm.flags + 4) = k;
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < REPP; j++) {
            // the reference multiplies q . K^T of the residual keys in the model dtype before promoting (:79)
            const float sr = resid ? lo2f<T>(f2lo<T>(s[j])) : s[j];
            s[j] = keep ? sr * p.scale_log2 : -INFINITY;
        }
        softmax_pv_tile<T, REPP>(st, s, vv[buf].r, pm.pbuf, lane);
    };
    for (int i = 0; i < nt; i += 2) {
        step(std::integral_constant<int, 0>{}, i);
        if (i + 1 < nt) step(std::integral_constant<int, 1>{}, i + 1);
    }
    float lsum[REPP];
#pragma unroll
    for (int j = 0; j < REPP; j++) lsum[j] = wave_sum(st.l[j]);
    const int g = lane >> 4, n = lane & 15;
    if (n < rep) {
        float mm = st.m[0], ll = lsum[0];
#pragma unroll
        for (int j = 1; j < REPP; j++) { mm = (n == j) ? st.m[j] : mm; ll = (n == j) ? lsum[j] : ll; }
        float* pw = p.ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep + n) * p.n_splits + slot) * kPartialFloats;
        if (g == 0) { pw[0] = mm; pw[1] = ll; }
        float* pa = pw + 4 + 32 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<float4*>(pa + 8 * i) = make_float4(st.acc[0][i], st.acc[1][i], st.acc[2][i], st.acc[3][i]);
            *reinterpret_cast<float4*>(pa + 8 * i + 4) = make_float4(st.acc[4][i], st.acc[5][i], st.acc[6][i], st.acc[7][i]);
        }
    }
    return ok;
}

// Even slices, one slice per pair: pair index = 4 * blockIdx.x + (pair within the block), laid out as attn_kernel's
// block index (plane fastest).
template <typename T, int TB, int REPP, bool PK6>
__global__ __launch_bounds__(kPairsPerBlock * 2 * kWave) void attn_pair_kernel(PQ_ATTN_KERNEL_PARAMS, int n_slices_total) {
    using L = Lut<TB, REPP>;
    __shared__ __attribute__((aligned(16))) char lut_mem[kPairsPerBlock][L::BYTES];
    __shared__ __attribute__((aligned(16))) float s_mem[kPairsPerBlock][2 * REPP * kWave];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[kPairsPerBlock][REPP * kWave];
    __shared__ int flag_mem[kPairsPerBlock][4];
    __shared__ int simd_of[2 * kPairsPerBlock];
    PQ_ATTN_KERNEL_PACK;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int pair, role;
    pair_roles(simd_of, &flag_mem[0][0], wave, lane, pair, role);
    PairMem pm;
    pm.lut = lds_addr(lut_mem[pair]);
    pm.sbuf = lds_addr(s_mem[pair]);
    pm.pbuf = lds_addr(p_mem[pair]);
    pm.flags = lds_addr(flag_mem[pair]);

    const int slice = blockIdx.x * kPairsPerBlock + pair;
    if (slice >= n_slices_total) return;
    const int units = n_slices_total / n_splits;
    const int bh = slice % units, split = slice / units;
    const int b = bh / Nk, kvh = bh - b * Nk;
    const V4Args v4none = v4;
    const SeqCounts sc = seq_counts<false>(p, v4none, b);
    int gps = (sc.nb + n_splits - 1) / n_splits;
    gps = gps < min_gps ? min_gps : gps;
    if (split > 0 && split * gps >= sc.nb) {
        if (role == 1 && lane < rep) {
            float* pw = ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep + lane) * n_splits + split) * kPartialFloats;
            pw[0] = -INFINITY;
            pw[1] = 0.0f;
        }
        return;
    }
    const int g0 = split * gps;
    const int g1 = (g0 + gps) < sc.nb ? (g0 + gps) : sc.nb;
    const int last_split = sc.nb > 0 ? (sc.nb - 1) / gps : 0;
    const int r1 = split == last_split ? (sc.nres + kWave - 1) / kWave : 0;
    int k = 0;
    if (role == 0) pair_scorer<T, TB, REPP, PK6>(p, pm, lane, b, kvh, sc, 2 * g0, 2 * g1, 0, r1, k);
    else           pair_accumulator<T, REPP>(p, pm, lane, b, kvh, sc, 2 * g0, 2 * g1, 0, r1, split, k);
}


// Balanced slices for pairs: both wavefronts of a pair walk the same segment and meet tile by tile.
template <typename T, int TB, int REPP, bool PK6>
__global__ __launch_bounds__(kPairsPerBlock * 2 * kWave) void attn_pair_balanced_kernel(PQ_ATTN_KERNEL_PARAMS, int n_pairs_total) {
    using L = Lut<TB, REPP>;
    __shared__ __attribute__((aligned(16))) char lut_mem[kPairsPerBlock][L::BYTES];
    __shared__ __attribute__((aligned(16))) float s_mem[kPairsPerBlock][2 * REPP * kWave];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[kPairsPerBlock][REPP * kWave];
    __shared__ int flag_mem[kPairsPerBlock][4];
    __shared__ int simd_of[2 * kPairsPerBlock];
    __shared__ int walk_mem[2 * kPairsPerBlock][8];
    PQ_ATTN_KERNEL_PACK;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int pair, role;
    pair_roles(simd_of, &flag_mem[0][0], wave, lane, pair, role);
    PairMem pm;
    pm.lut = lds_addr(lut_mem[pair]);
    pm.sbuf = lds_addr(s_mem[pair]);
    pm.pbuf = lds_addr(p_mem[pair]);
    pm.flags = lds_addr(flag_mem[pair]);
    const int w = blockIdx.x * kPairsPerBlock + pair;
    if (w >= n_pairs_total) return;
    int k = 0;
    bool ok = true;
    walk_segment<false>(p, v4, n_pairs_total, w, lane, lds_addr(walk_mem[wave]),
                        [&](int cb, int ckvh, const SeqCounts& sc, int t0, int t1, int r0, int r1, int slot, bool ends_plane) {
                            if (!ok) return;         // the partner stopped answering: run out without touching anything
                            if (role == 0) {
                                ok = pair_scorer<T, TB, REPP, PK6>(p, pm, lane, cb, ckvh, sc, t0, t1, r0, r1, k);
                            } else {
                                if (ends_plane && slot + 1 < n_splits) mark_empty_slots(p, lane, cb, ckvh, slot + 1);
                                ok = pair_accumulator<T, REPP>(p, pm, lane, cb, ckvh, sc, t0, t1, r0, r1, slot, k);
                            }
                        });
}

#pragma clang diagnostic pop

template <typename T, int G>
__global__ __launch_bounds__(kHeadDim * G) void merge_kernel(const float* __restrict__ ws, int n_part, uint16_t* __restrict__ out) {
    // one block per query head, G groups of 128 threads: thread (grp, d) sums output dim d over
    // the grp-th share of the partials, and the G sums are added in a fixed order through LDS.
    // The partial headers (m, l) are fetched by one thread each, so that all loads of the block
    // are issued at once instead of one dependent load per partial.
    constexpr int NT = kHeadDim * G, NW = NT / kWave;
    __shared__ float wgt[1024];
    __shared__ float red[2][NW];
    __shared__ float part[G][kHeadDim];
    const int bn = blockIdx.x, tid = threadIdx.x, d = tid & (kHeadDim - 1), grp = tid / kHeadDim;
    const float* p = ws + static_cast<size_t>(bn) * n_part * kPartialFloats;
    float M = -INFINITY;
    for (int s = tid; s < n_part; s += NT) M = fmaxf(M, p[static_cast<size_t>(s) * kPartialFloats]);
    M = wave_max(M);
    if ((tid & (kWave - 1)) == 0) red[0][tid / kWave] = M;
    __syncthreads();
    M = red[0][0];
#pragma unroll
    for (int i = 1; i < NW; i++) M = fmaxf(M, red[0][i]);
    float num = 0.0f, den = 0.0f;
    for (int s0 = 0; s0 < n_part; s0 += 1024) {
        const int cnt = (n_part - s0) < 1024 ? (n_part - s0) : 1024;
        __syncthreads();
        for (int s = tid; s < cnt; s += NT) {
            const float m = p[static_cast<size_t>(s0 + s) * kPartialFloats];
            const float w = (m == -INFINITY) ? 0.0f : exp2f(m - M);
            wgt[s] = w;
            // an empty slice contributes nothing, whatever its sum word holds
            den = w != 0.0f ? __builtin_fmaf(w, p[static_cast<size_t>(s0 + s) * kPartialFloats + 1], den) : den;
        }
        __syncthreads();
        const float* pa = p + static_cast<size_t>(s0) * kPartialFloats + 4 + d;
        const int per = (cnt + G - 1) / G;
        int s = grp * per;
        const int se = (s + per) < cnt ? (s + per) : cnt;
        for (; s + 16 <= se; s += 16) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; u++) v[u] = pa[static_cast<size_t>(s + u) * kPartialFloats];
#pragma unroll
            for (int u = 0; u < 16; u++) num = wgt[s + u] != 0.0f ? __builtin_fmaf(wgt[s + u], v[u], num) : num;
        }
        for (; s + 8 <= se; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = pa[static_cast<size_t>(s + u) * kPartialFloats];
#pragma unroll
            for (int u = 0; u < 8; u++) num = wgt[s + u] != 0.0f ? __builtin_fmaf(wgt[s + u], v[u], num) : num;
        }
        for (; s < se; s++) {
            const float v = pa[static_cast<size_t>(s) * kPartialFloats];
            num = wgt[s] != 0.0f ? __builtin_fmaf(wgt[s], v, num) : num;
        }
    }
    den = wave_sum(den);
    __syncthreads();
    if ((tid & (kWave - 1)) == 0) red[1][tid / kWave] = den;
    if (G > 1) part[grp][d] = num;
    __syncthreads();
    if (grp != 0) return;
    den = red[1][0];
#pragma unroll
    for (int i = 1; i < NW; i++) den += red[1][i];
#pragma unroll
    for (int i = 1; i < G; i++) num += part[i][d];
    out[static_cast<size_t>(bn) * kHeadDim + d] = f2lo<T>(den > 0.0f ? num / den : 0.0f);
}

// Wavefront slots of the current device for the balanced kernel: one wavefront per SIMD (4 per
// compute unit), two for the 4-bit-value kernel with up to 4 query heads per KV head.
static int device_compute_units() {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static int cus[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

template <typename T, int TB>
static int launch_attn_tb(const AttnArgs& a, hipStream_t st) {
    const int rep = a.N / a.Nk;
    dim3 grid(static_cast<unsigned>(a.n_splits) * static_cast<unsigned>(a.B * a.Nk)), block(kWave);
    if (a.balanced) {
        // as many wavefronts as the device holds at once, but never more than there are partial slots
        const long long slots = static_cast<long long>(device_compute_units()) * ((a.v4_codes && rep_pad(rep) <= 4) ? 8 : 4);
        const long long most = static_cast<long long>(a.n_splits) * a.B * a.Nk;
        grid = dim3(static_cast<unsigned>(slots < most ? slots : most));
    }
    const float scale_log2 = a.sm_scale * kLog2e;
    V4Args v4{static_cast<const uint32_t*>(a.v4_codes), static_cast<const uint16_t*>(a.v4_scale),
              static_cast<const uint16_t*>(a.v4_zero), a.v4_capacity};
#define PQ_LAUNCH_K(KERNEL, REPP, V4, PK6)                                                                           \
    hipLaunchKernelGGL((KERNEL<T, TB, REPP, V4, PK6>), grid, block, 0, st, (const uint16_t*)a.q, a.codes,            \
                       (const uint16_t*)a.rscale, (const uint16_t*)a.rmn, (const uint16_t*)a.tscale,                 \
                       (const uint16_t*)a.tmn, a.group_capacity, a.n_groups, a.n_groups_per_seq,                     \
                       (const uint16_t*)a.k_resid, a.resid_capacity, a.n_resid, a.n_resid_per_seq,                   \
                       (const uint16_t*)a.v, a.v_capacity, a.mask, a.mask_stride, scale_log2, a.B, a.N, a.Nk, rep,   \
                       a.n_splits, a.min_groups_per_split, a.workspace, v4)
#define PQ_LAUNCH_VP(REPP, V4, PK6)                                                                                  \
    do {                                                                                                             \
        if (a.balanced) PQ_LAUNCH_K(attn_balanced_kernel, REPP, V4, PK6);                                            \
        else PQ_LAUNCH_K(attn_kernel, REPP, V4, PK6);                                                                \
    } while (0)
    // packed 6-bit code rows exist for tbits == 3 only (the 3/3 configuration)
#define PQ_LAUNCH_V(REPP, V4)                                                                                        \
    do {                                                                                                             \
        if constexpr (TB == 3) {                                                                                     \
            if (a.packed6) PQ_LAUNCH_VP(REPP, V4, true);                                                             \
            else PQ_LAUNCH_VP(REPP, V4, false);                                                                      \
        } else {                                                                                                     \
            PQ_LAUNCH_VP(REPP, V4, false);                                                                           \
        }                                                                                                            \
    } while (0)
#define PQ_LAUNCH(REPP)                                                                                              \
    do {                                                                                                             \
        if (a.v4_codes) PQ_LAUNCH_V(REPP, true);                                                                     \
        else PQ_LAUNCH_V(REPP, false);                                                                               \
    } while (0)
    if (!a.v4_codes && !a.single_wave) {
        // one pair of wavefronts per slice (even slices) or per segment (balanced slices), four pairs to a workgroup
        const int total = static_cast<int>(grid.x);
        const dim3 pgrid((total + kPairsPerBlock - 1) / kPairsPerBlock), pblock(kPairsPerBlock * 2 * kWave);
#define PQ_LAUNCH_PAIR_K(KERNEL, REPP, PK6)                                                                          \
        hipLaunchKernelGGL((KERNEL<T, TB, REPP, PK6>), pgrid, pblock, 0, st, (const uint16_t*)a.q, a.codes,          \
                           (const uint16_t*)a.rscale, (const uint16_t*)a.rmn, (const uint16_t*)a.tscale,             \
                           (const uint16_t*)a.tmn, a.group_capacity, a.n_groups, a.n_groups_per_seq,                 \
                           (const uint16_t*)a.k_resid, a.resid_capacity, a.n_resid, a.n_resid_per_seq,               \
                           (const uint16_t*)a.v, a.v_capacity, a.mask, a.mask_stride, scale_log2, a.B, a.N, a.Nk, rep, \
                           a.n_splits, a.min_groups_per_split, a.workspace, v4, total)
#define PQ_LAUNCH_PAIR_P(REPP, PK6)                                                                                  \
        do {                                                                                                         \
            if (a.balanced) PQ_LAUNCH_PAIR_K(attn_pair_balanced_kernel, REPP, PK6);                                  \
            else PQ_LAUNCH_PAIR_K(attn_pair_kernel, REPP, PK6);                                                      \
        } while (0)
#define PQ_LAUNCH_PAIR(REPP)                                                                                         \
        do {                                                                                                         \
            if constexpr (TB == 3) {                                                                                 \
                if (a.packed6) PQ_LAUNCH_PAIR_P(REPP, true);                                                         \
                else PQ_LAUNCH_PAIR_P(REPP, false);                                                                  \
            } else {                                                                                                 \
                PQ_LAUNCH_PAIR_P(REPP, false);                                                                       \
            }                                                                                                        \
        } while (0)
        switch (rep_pad(rep)) {
            case 1: PQ_LAUNCH_PAIR(1); break;
            case 2: PQ_LAUNCH_PAIR(2); break;
            case 4: PQ_LAUNCH_PAIR(4); break;
            default: PQ_LAUNCH_PAIR(8); break;
        }
#undef PQ_LAUNCH_PAIR
#undef PQ_LAUNCH_PAIR_P
#undef PQ_LAUNCH_PAIR_K
        return static_cast<int>(hipGetLastError());
    }
    switch (rep_pad(rep)) {
        case 1: PQ_LAUNCH(1); break;
        case 2: PQ_LAUNCH(2); break;
        case 4: PQ_LAUNCH(4); break;
        default: PQ_LAUNCH(8); break;
    }
#undef PQ_LAUNCH
#undef PQ_LAUNCH_V
#undef PQ_LAUNCH_VP
#undef PQ_LAUNCH_K
    return static_cast<int>(hipGetLastError());
}

template <typename T>
static int launch_attn_t(const AttnArgs& a, hipStream_t st) {
    switch (a.tbits) {
        case 1: return launch_attn_tb<T, 1>(a, st);
        case 2: return launch_attn_tb<T, 2>(a, st);
        case 3: return launch_attn_tb<T, 3>(a, st);
        default: return launch_attn_tb<T, 4>(a, st);
    }
}

int launch_attn_partials(const AttnArgs& a, hipStream_t st) {
    return a.dtype == 0 ? launch_attn_t<F16>(a, st) : launch_attn_t<BF16>(a, st);
}

constexpr int kMergeWideFrom = 32, kMergeWidestFrom = 128;

int launch_attn_merge(const float* ws, int B, int N, int n_splits, int dtype, void* out, hipStream_t st) {
    // many partials per head (a long context cut into many slices): four or eight groups of threads share them
    if (n_splits >= kMergeWidestFrom) {
        if (dtype == 0)
            hipLaunchKernelGGL((merge_kernel<F16, 8>), dim3(B * N), dim3(kHeadDim * 8), 0, st, ws, n_splits, (uint16_t*)out);
        else
            hipLaunchKernelGGL((merge_kernel<BF16, 8>), dim3(B * N), dim3(kHeadDim * 8), 0, st, ws, n_splits, (uint16_t*)out);
    } else if (n_splits >= kMergeWideFrom) {
        if (dtype == 0)
            hipLaunchKernelGGL((merge_kernel<F16, 4>), dim3(B * N), dim3(kHeadDim * 4), 0, st, ws, n_splits, (uint16_t*)out);
        else
            hipLaunchKernelGGL((merge_kernel<BF16, 4>), dim3(B * N), dim3(kHeadDim * 4), 0, st, ws, n_splits, (uint16_t*)out);
    } else if (dtype == 0) {
        hipLaunchKernelGGL((merge_kernel<F16, 1>), dim3(B * N), dim3(kHeadDim), 0, st, ws, n_splits, (uint16_t*)out);
    } else {
        hipLaunchKernelGGL((merge_kernel<BF16, 1>), dim3(B * N), dim3(kHeadDim), 0, st, ws, n_splits, (uint16_t*)out);
    }
    return static_cast<int>(hipGetLastError());
}

// ---- scratch of the entry point that allocates nothing (pq_decode_attn_static) -----------------
// The split partials of that entry point live in this file-scope device array instead of a caller's
// workspace.  Every GPU the library runs on holds its own copy at its own address until the process
// ends; the array's name is only a host-side handle, so the device address is asked for once per
// device (with that device current) and kept.
static __device__ __align__(256) float scratch[static_cast<size_t>(kStaticMaxPartials) * kPartialFloats];

int attn_static_scratch(float** ptr) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static float* per_device[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!p) return static_cast<int>(hipErrorInvalidSymbol);
        per_device[dev] = static_cast<float*>(p);
    }
    *ptr = per_device[dev];
    return 0;
}

}  // namespace pq
