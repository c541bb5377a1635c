// Fused polar-key decode attention, the kernels with ONE wavefront per slice: quantized-key scores,
// half-precision residual-key scores, 1/sqrt(d), mask, softmax and P.V in one pass over HBM
// (reference decode branch: models/modeling_llama_polar.py:66-99), split over the context; These kernels serve the 4-bit values of the
// Mixed variant and PQ_SINGLE_WAVEFRONT; with half-precision values the default kernels are the
// scorer / accumulator pairs of pq_attn_pair.hip, which share the device code of pq_attn_device.h.
//
// attn_kernel: grid n_splits * B*Nk (plane index fastest), one wavefront per block: a block works
// through one slice of its sequence's quantized groups; the last block of
// a (batch, KV head) then also takes the residual keys (0..128 tokens).
// The kernel is built for ONE resident wavefront per SIMD (4 per CU) with deep
// software prefetch instead of many wavefronts: V operands are double-buffered
// a whole 64-token tile ahead, which keeps ~40 KiB of loads in flight per
// wavefront; pq_decode_attn_plan sizes n_splits so that B*Nk*n_splits fills
// those slots exactly once.  (With 4-bit values at up to 4 heads per KV head: two per SIMD.)
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
// The merge kernel that follows every attention kernel is in pq_attn_common.hip.  This file is compiled once per
// dtype (-DPQ_DTYPE=0 float16, 1 bfloat16).
#include "pq_attn_device.h"

#ifndef PQ_DTYPE
#error "compile with -DPQ_DTYPE=0 (float16) or 1 (bfloat16)"
#endif

#include "pq_phase_timers.h"

namespace pq {

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"

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

    const uint16_t* qb = p.q + (static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * p.rep_stride) * kHeadDim;
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
                if constexpr (V4 && kProbeNoValues) {
                    return;                                    // probe build: the 4-bit-value kernel without its value path
                } else if constexpr (V4) {
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
                    if constexpr (V4 && kProbeNoValues) {
                        softmax_sums_only<REPP>(st, s, kLazyThresholdV4);
                    } else if constexpr (V4) {
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
        float* pw = ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * p.rep_stride + n) * n_splits + slot) * kPartialFloats;
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

// Even slices: block (plane bh, slice `split`) takes groups [split * gps, (split + 1) * gps) of its
// sequence, gps = max(min_gps, ceil(groups / n_splits)); the block that holds the last group also
// takes the residual keys.
template <typename T, int TB, int REPP, bool V4, bool PK6>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu((V4 && REPP <= 4 && TB <= 4) ? 2 : 1, 2)))
void attn_kernel(PQ_ATTN_KERNEL_PARAMS) {
    using L = Lut<TB, REPP>;
    // the table region doubles as the staging buffer of the residual block's scores ([REPP][64] fp32)
    constexpr int kLutBytes = L::BYTES > REPP * kWave * 4 ? L::BYTES : REPP * kWave * 4;
    __shared__ __attribute__((aligned(16))) char lut_mem[kLutBytes];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[REPP * kWave];
    const uint32_t lut = lds_addr(lut_mem), pbuf = lds_addr(p_mem);
    PQ_ATTN_KERNEL_PACK;

    const int lane = threadIdx.x;
    // Grid (KV head, sequence, slice): workgroups are handed out x first, so the (batch, KV head) index runs
    // fastest.  Consecutive workgroup ids go to different XCDs, so every XCD receives whole planes with all
    // their slices; with the slice index fastest an XCD would receive one slice index of every plane, and in a
    // ragged batch the XCDs that own the high slice indices would sit idle (measured: 165 us instead of 120 us).
    // (Three grid dimensions instead of one index taken apart: three integer divisions fewer in front of the first
    // loads, 0.3-0.7 us per launch.)
    const int kvh = blockIdx.x, b = blockIdx.y, split = blockIdx.z;
    const SeqCounts sc = seq_counts<V4>(p, v4, b);

    // groups per slice: an even split of this sequence, but never fewer than min_gps (ragged
    // batches: short sequences then use fewer slices, and the unused blocks return at once)
    int gps = (sc.nb + n_splits - 1) / n_splits;
    gps = gps < min_gps ? min_gps : gps;
    // slices past the end of a short sequence have nothing to do: mark their partials empty and leave
    if (split > 0 && split * gps >= sc.nb) {
        if (lane < rep) {
            float* pw = ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep_stride + lane) * n_splits + split) * kPartialFloats;
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

template <typename T, int TB, int REPP, bool V4, bool PK6>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu((V4 && REPP <= 4 && TB <= 4) ? 2 : 1, 2)))
void attn_balanced_kernel(PQ_ATTN_KERNEL_PARAMS) {
    using L = Lut<TB, REPP>;
    constexpr int kLutBytes = L::BYTES > REPP * kWave * 4 ? L::BYTES : REPP * kWave * 4;
    __shared__ __attribute__((aligned(16))) char lut_mem[kLutBytes];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[REPP * kWave];
    __shared__ int walk[kWalkInts];
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

#pragma clang diagnostic pop

template <typename T, int TB>
static int launch_attn_tb(const AttnArgs& a, int total, hipStream_t st) {
    // a.rep_count: this launch's share of the query heads of every KV head (0: all of them); q and the workspace then
    // point at the share's first head
    const int rep_stride = a.N / a.Nk, rep = a.rep_count ? a.rep_count : rep_stride;
    const dim3 grid(static_cast<unsigned>(total)), block(kWave);
    const float scale_log2 = a.sm_scale * kLog2e;
    V4Args v4{static_cast<const uint32_t*>(a.v4_codes), static_cast<const uint16_t*>(a.v4_scale),
              static_cast<const uint16_t*>(a.v4_zero), a.v4_capacity};
#define PQ_LAUNCH_K(KERNEL, REPP, V4, PK6)                                                                           \
    hipLaunchKernelGGL((KERNEL<T, TB, REPP, V4, PK6>), grid, block, 0, st, (const uint16_t*)a.q, a.codes,            \
                       (const uint16_t*)a.rscale, (const uint16_t*)a.rmn, (const uint16_t*)a.tscale,                 \
                       (const uint16_t*)a.tmn, a.group_capacity, a.n_groups, a.n_groups_per_seq,                     \
                       (const uint16_t*)a.k_resid, a.resid_capacity, a.n_resid, a.n_resid_per_seq,                   \
                       (const uint16_t*)a.v, a.v_capacity, a.mask, a.mask_stride, scale_log2, a.B, a.N, a.Nk, rep,   \
                       a.n_splits, a.min_groups_per_split, a.workspace, v4, rep_stride)
#define PQ_LAUNCH_VP(REPP, V4, PK6)                                                                                  \
    do {                                                                                                             \
        if (a.balanced) PQ_LAUNCH_K(attn_balanced_kernel, REPP, V4, PK6);                                            \
        else { const dim3 grid(a.Nk, a.B, a.n_splits); PQ_LAUNCH_K(attn_kernel, REPP, V4, PK6); }                    \
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
    // (128 angle bins: a table holds four heads at most, and the caller sends the heads in two launches)
    switch (rep_pad(rep)) {
        case 1: PQ_LAUNCH(1); break;
        case 2: PQ_LAUNCH(2); break;
        case 4: PQ_LAUNCH(4); break;
        default:
            if constexpr (TB <= 6) PQ_LAUNCH(8);
            else return static_cast<int>(hipErrorInvalidValue);
            break;
    }
#undef PQ_LAUNCH
#undef PQ_LAUNCH_V
#undef PQ_LAUNCH_VP
#undef PQ_LAUNCH_K
    return static_cast<int>(hipGetLastError());
}

#if PQ_DTYPE == 0
int launch_attn_one_f16(const AttnArgs& a, int total, hipStream_t st) {
    using T = F16;
#else
int launch_attn_one_bf16(const AttnArgs& a, int total, hipStream_t st) {
    using T = BF16;
#endif
    switch (a.tbits) {
        case 1: return launch_attn_tb<T, 1>(a, total, st);
        case 2: return launch_attn_tb<T, 2>(a, total, st);
        case 3: return launch_attn_tb<T, 3>(a, total, st);
        case 4: return launch_attn_tb<T, 4>(a, total, st);
        case 5: return launch_attn_tb<T, 5>(a, total, st);
        case 6: return launch_attn_tb<T, 6>(a, total, st);
        default: return launch_attn_tb<T, 7>(a, total, st);
    }
}

}  // namespace pq
