// Device code shared by the decode-attention kernels (pq_attn.hip: one wavefront per slice, and the kernels for
// 4-bit values; pq_attn_pair.hip: a scorer / accumulator pair of wavefronts per slice): the softmax + P.V step
// of a 64-token tile on the matrix cores, the loads of a value tile, the kernels' argument block, the per-sequence
// counts, and the walk of a wavefront over its segment when the slices are cut on the device.
#pragma once
#include "pq_device.h"
#include "pq_internal.h"

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

// 2^x as the bare v_exp_f32: exact to 1 ulp over the normal range and 0 below 2^-126, where the library's exp2f spends
// five more instructions to return a denormal.  Every use here is a softmax weight relative to a running maximum: a
// weight below 2^-126 is nothing against the maximum's weight of at least 2^-8.
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }

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
            alpha[j] = (mn == -INFINITY) ? 1.0f : exp2_raw(st.m[j] - mn);
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
        const float p = exp2_raw(t[j] - ms);
        st.l[j] += p;
        *lds_ptr<__attribute__((address_space(3))) uint16_t>(pbuf + (j * kWave + lane) * 2) = f2lo<T>(p);
    }
    asm volatile("" ::: "memory");
    const int g = lane >> 4, n = lane & 15;
    const uint32_t prow = pbuf + ((n < REPP ? n : 0) * kWave + 4 * g) * 2;      // columns past the last head: any row, never stored
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
            alpha[j] = (mn == -INFINITY) ? 1.0f : exp2_raw(st.m[j] - mn);
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
    // (a reciprocal to 1 ulp instead of the ten-instruction IEEE division: what matters is that both terms see the same
    // rounded weight, not the last bit of zero / scale)
    const float zq = zp * __builtin_amdgcn_rcpf(scp);
#pragma unroll
    for (int j = 0; j < REPP; j++) {
        const float ms = (st.m[j] == -INFINITY) ? 0.0f : st.m[j];
        const float p = exp2_raw(t[j] - ms);
        st.l[j] += p;
        const uint16_t wh = f2lo<F16>(p * scp);
        st.zp[j] = __builtin_fmaf(lo2f<F16>(wh), zq, st.zp[j]);
        *lds_ptr<__attribute__((address_space(3))) uint16_t>(pbuf + (j * kWave + slot) * 2) = wh;
    }
    asm volatile("" ::: "memory");
    const int g = lane >> 4, n = lane & 15;
    const uint32_t prow = pbuf + ((n < REPP ? n : 0) * kWave + 4 * g) * 2;      // columns past the last head: any row, never stored
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

// Probe builds only: the softmax bookkeeping of a tile (running maximum, probabilities, their sum) without any
// product with the values.
template <int REPP>
__device__ __forceinline__ void softmax_sums_only(AttnState<REPP>& st, float (&t)[REPP], float lazy) {
    bool raise = false;
#pragma unroll
    for (int j = 0; j < REPP; j++) raise |= t[j] > st.m[j] + lazy;
    if (__any(raise)) {
#pragma unroll
        for (int j = 0; j < REPP; j++) {
            const float mn = fmaxf(st.m[j], wave_max(t[j]));
            st.l[j] *= (mn == -INFINITY) ? 1.0f : exp2_raw(st.m[j] - mn);
            st.m[j] = mn;
        }
    }
#pragma unroll
    for (int j = 0; j < REPP; j++) st.l[j] += exp2_raw(t[j] - ((st.m[j] == -INFINITY) ? 0.0f : st.m[j]));
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
    // query heads from one KV head to the next in q and in the partials: rep, except when a call's heads are worked
    // through in two launches (128 angle bins: a table holds at most four heads)
    int rep_stride;
    float* ws;
};

// Token counts of one sequence as the kernels use them: groups and residual keys clamped to the
// capacities, tokens clamped to what the value plane holds.
struct SeqCounts { int nb, nres; int64_t n_tokens; };
// from the counts as the caller gave them (nb: quantized groups, nres: residual keys of the sequence)
template <bool V4>
__device__ __forceinline__ SeqCounts seq_counts_from(const AttnParams& p, const V4Args& v4, int nb, int nres) {
    SeqCounts c;
    nb = nb < 0 ? 0 : (nb > p.group_capacity ? p.group_capacity : nb);
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
template <bool V4>
__device__ __forceinline__ SeqCounts seq_counts(const AttnParams& p, const V4Args& v4, int b) {
    return seq_counts_from<V4>(p, v4, p.n_groups_per_seq ? p.n_groups_per_seq[b] : p.n_groups,
                               p.n_resid_per_seq ? p.n_resid_per_seq[b] : p.n_resid);
}

// Mark the partial slots [first, n_splits) of the `rep` query heads of (b, kvh) as holding nothing.
// Both header words: the workspace is not cleared between calls, and the merge must not meet a
// stale probability sum (0 * NaN) in a slot that holds nothing.
__device__ __forceinline__ void mark_empty_slots(const AttnParams& p, int lane, int b, int kvh, int first) {
    const int count = (p.n_splits - first) * p.rep;
    for (int i = lane; i < count; i += kWave) {
        const int j = i / (p.n_splits - first), s = first + i % (p.n_splits - first);
        float* pw = p.ws + ((static_cast<size_t>(b) * p.N + static_cast<size_t>(kvh) * p.rep_stride + j) * p.n_splits + s) * kPartialFloats;
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
        int n_splits, int min_gps, float* __restrict__ ws, V4Args v4, int rep_stride
#define PQ_ATTN_KERNEL_PACK                                                                                          \
    AttnParams p;                                                                                                    \
    p.q = q; p.codes = codes; p.rscale = rscale; p.rmn = rmn; p.tscale = tscale; p.tmn = tmn;                        \
    p.group_capacity = group_capacity; p.n_groups = n_groups; p.n_groups_per_seq = n_groups_per_seq;                 \
    p.k_resid = k_resid; p.resid_capacity = resid_capacity; p.n_resid = n_resid; p.n_resid_per_seq = n_resid_per_seq; \
    p.v = v; p.v_capacity = v_capacity; p.mask = mask; p.mask_stride = mask_stride; p.scale_log2 = scale_log2;      \
    p.B = B; p.N = N; p.Nk = Nk; p.rep = rep; p.n_splits = n_splits; p.min_gps = min_gps; p.ws = ws;         \
    p.rep_stride = rep_stride

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
// of kWalkInts ints that belong to the calling wavefront: the state of the walk lives in the first 8 between pieces, so
// that nothing of it occupies registers inside a piece (the group loop already uses every scalar register); behind them
// sit the counts of the first 64 sequences, fetched from device memory once: the cut, the first piece and every later
// piece would otherwise each wait for a dependent load of its own (four memory round trips before a wavefront's first
// code or value load; measured at 64 ragged sequences: 13 us from entry to the first tile against 7.7 us with even slices).
constexpr int kWalkInts = 8 + 2 * kWave;
template <bool V4, typename F>
__device__ __forceinline__ void walk_segment(const AttnParams& p, const V4Args& v4, unsigned W, unsigned w, int lane,
                                             uint32_t walk, F&& piece) {
    // All positions on the line are 32-bit: the host refuses a call whose capacities could hold 2^31 units (far beyond
    // what fits in device memory).  64-bit quotients here were a thousand instructions in front of every wavefront's
    // first load.
    const int B = p.B, Nk = p.Nk;
    typedef __attribute__((address_space(3))) int lds_i1;
    // the counts of sequences 0..63 as the caller gave them, one per lane, into this wavefront's LDS
    if (lane < B) {
        lds_i1* wc = lds_ptr<lds_i1>(walk);
        wc[8 + lane] = p.n_groups_per_seq ? p.n_groups_per_seq[lane] : p.n_groups;
        wc[8 + kWave + lane] = p.n_resid_per_seq ? p.n_resid_per_seq[lane] : p.n_resid;
    }
    asm volatile("" ::: "memory");
    auto counts_of = [&](int bb) {
        if (bb < kWave) {
            const lds_i1* wc = lds_ptr<lds_i1>(walk);
            return seq_counts_from<V4>(p, v4, wc[8 + bb], wc[8 + kWave + bb]);
        }
        return seq_counts<V4>(p, v4, bb);
    };
    // units of one plane of sequence bb: kStartUnits for the plane's start-up (they also make a sequence with
    // nothing at all a plane of its own, so that somebody writes its partials), then its tiles
    auto units_of = [&](int bb) {
        const SeqCounts c = counts_of(bb);
        return kStartUnits + 2 * c.nb + (c.nres + kWave - 1) / kWave;
    };
    // length of the line
    int mine = 0;
    for (int base = 0; base < B; base += kWave) mine += (base + lane < B) ? units_of(base + lane) : 0;
    const unsigned per_head = static_cast<unsigned>(wave_sum_i(mine));          // units of one KV head's planes, all sequences
    const unsigned total = per_head * static_cast<unsigned>(Nk);
    unsigned seg = (total + W - 1u) / W;
    seg = seg < 2u * static_cast<unsigned>(p.min_gps) ? 2u * static_cast<unsigned>(p.min_gps) : seg;
    // the most units a plane can have (the residual window is 128 keys in the reference, but the interface takes
    // any resid_capacity)
    const unsigned cap_units = 2u * static_cast<unsigned>(p.group_capacity) + static_cast<unsigned>((p.resid_capacity + kWave - 1) / kWave + kStartUnits);
    const unsigned fit = (cap_units + static_cast<unsigned>(p.n_splits) - 2u) / static_cast<unsigned>(p.n_splits - 1);      // n_splits >= 2 (checked on the host)
    seg = seg < fit ? fit : seg;
    // (w * seg can pass 2^32 only for wavefronts far behind the end of the line)
    if (static_cast<unsigned long long>(w) * seg >= total) return;
    const unsigned start = w * seg;
    const unsigned end = (total - start) > seg ? (start + seg) : total;

    // the sequence that holds unit `start`: units before sequence bb are Nk * (sum of u over earlier sequences)
    int b = 0;
    unsigned before = 0;                                   // units of one head's planes before sequence b
    for (int base = 0; base < B; base += kWave) {
        const int u = (base + lane < B) ? units_of(base + lane) : 0;
        int incl = u;
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
            const int t = __shfl_up(incl, o);
            incl += (lane >= o) ? t : 0;
        }
        const unsigned chunk = static_cast<unsigned>(__shfl(incl, kWave - 1));
        if (start < (before + chunk) * static_cast<unsigned>(Nk)) {
            const unsigned long long past = __ballot((before + static_cast<unsigned>(incl)) * static_cast<unsigned>(Nk) > start);
            const int l0 = __builtin_ctzll(past);
            b = base + l0;
            before += static_cast<unsigned>(__shfl(incl - u, l0));
            break;
        }
        before += chunk;
    }
    {
        const unsigned u0 = static_cast<unsigned>(units_of(b));
        const unsigned seq_start = before * static_cast<unsigned>(Nk);            // line position of plane (b, 0)
        const unsigned kvh0 = (start - seq_start) / u0;
        const unsigned plane_start = seq_start + kvh0 * u0;
        if (lane == 0) {
            lds_i1* wk = lds_ptr<lds_i1>(walk);
            wk[0] = b; wk[1] = static_cast<int>(kvh0); wk[2] = static_cast<int>(start - plane_start); wk[3] = static_cast<int>(u0);
            wk[4] = static_cast<int>(end - start);                                         // units left in the segment
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
        // (cb is the same in every lane: the counts are made wave-uniform before anything is derived from them, so that
        // sizes and offsets of the piece stay in scalar registers)
        SeqCounts sc;
        if (cb < kWave) {
            const lds_i1* wc = lds_ptr<lds_i1>(walk);
            sc = seq_counts_from<V4>(p, v4, __builtin_amdgcn_readfirstlane(wc[8 + cb]), __builtin_amdgcn_readfirstlane(wc[8 + kWave + cb]));
        } else {
            sc = seq_counts<V4>(p, v4, cb);
        }
        // the first kStartUnits units of a plane stand for its start-up; then the tiles of the quantized part,
        // then the residual keys'
        const int ta = ua > kStartUnits ? ua - kStartUnits : 0, tb = ub > kStartUnits ? ub - kStartUnits : 0;
        const int qt = 2 * sc.nb;
        const int t0 = ta < qt ? ta : qt, t1 = tb < qt ? tb : qt;
        const int r0 = ta > qt ? ta - qt : 0, r1 = tb > qt ? tb - qt : 0;
        piece(cb, ckvh, sc, t0, t1, r0, r1, slot, ub == u);
    }
}

#pragma clang diagnostic pop

}  // namespace pq
