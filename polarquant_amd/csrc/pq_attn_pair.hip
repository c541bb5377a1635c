// Fused polar-key decode attention with half-precision values, the default kernels:
// the work of one slice is shared by the two wavefronts that sit on one SIMD.  The SCORER reads the codes, builds the tables and produces the scores of a
// 64-token tile; the ACCUMULATOR streams the values, and does the mask, the softmax update and
// P.V; the scores cross over in LDS, double-buffered, so the scorer works on tile t+1 while the
// accumulator finishes tile t.  Inside one wavefront those phases can only follow each other, and
// their sum, not the memory system, sets the time per group (8 heads per KV head most of all).
//
// A workgroup is 8 wavefronts = one compute unit's worth at 256 registers each, so the hardware
// puts exactly two on every SIMD; which two is read from the hardware id register, and the two
// that share a SIMD form a pair (lower wavefront index = scorer).  If the ids do not come out in
// pairs the wavefronts are paired as (w, w + 4): the results are the same, only the overlap is lost.
// The two hand tiles over through two counters in LDS (tiles published / tiles consumed).  A counter is stored only
// after `s_waitcnt lgkmcnt(0)`: the wavefront's own LDS writes of the tile (or its reads of it, for the "consumed"
// counter) have completed by then, so whoever sees the counter sees the tile, and the order in which the LDS serves
// requests of different wavefronts is not relied on (the wait costs 0.3 us per launch).  A wait
// gives up after kSpinLimit polls (about half a second), after which both wavefronts run out
// without waiting again, the accumulator writes NaN into the partial of this piece and of every
// later piece of its segment, and both set the caller's status word (if one was passed) with a plain
// vector store: a failed hand-over cannot pass for a result, the host can learn of it without
// scanning the output, and no wavefront can wait for ever.
// Test build only (-DPQ_TEST_HOOKS, libpolarquant_hip_testhooks.so): PQ_TEST_SILENT_SCORER makes the
// scorers publish nothing and the waits give up after 1000 polls, so that a test can see exactly
// that: every kernel ends, every output is NaN, the status word is set.  The shipping library
// refuses the flag and its kernels hold no such switch.
#include "pq_attn_device.h"
#include "pq_phase_timers.h"

#ifndef PQ_DTYPE
#error "compile with -DPQ_DTYPE=0 (float16) or 1 (bfloat16)"
#endif

namespace pq {

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"

constexpr int kPairsPerBlock = 4;
constexpr int kSpinLimit = 1 << 22;
constexpr int kSpinLimitSilent = 1000;      // with PQ_TEST_SILENT_SCORER: the waits' time-out is what is being tested
#ifdef PQ_TEST_HOOKS
constexpr bool kTestHooks = true;
#else
constexpr bool kTestHooks = false;
#endif
constexpr int kStatusHandoverTimeout = 1;   // == PQ_STATUS_HANDOVER_TIMEOUT

struct PairMem {
    uint32_t lut;      // the scorer's table
    uint32_t sbuf;     // [2][REPP][64] fp32 scores
    uint32_t pbuf;     // the accumulator's probability staging
    uint32_t flags;    // int[4]: tiles published by the scorer, tiles consumed by the accumulator, -, -
    int spin_limit;    // polls after which a wait gives up
    bool silent;       // PQ_TEST_SILENT_SCORER (test build only): the scorer publishes nothing
};

__device__ __forceinline__ PairMem pair_mem(uint32_t lut, uint32_t sbuf, uint32_t pbuf, uint32_t flags, int silent_scorer) {
    PairMem pm;
    pm.lut = lut; pm.sbuf = sbuf; pm.pbuf = pbuf; pm.flags = flags;
    pm.silent = kTestHooks && silent_scorer != 0;
    pm.spin_limit = pm.silent ? kSpinLimitSilent : kSpinLimit;
    return pm;
}

// A hand-over gave up: tell the host, if it passed a status word.  One lane, an ordinary vector store of a constant
// (every wavefront that fails writes the same value, so no atomic is needed).  The pointer waits in LDS (stash_status,
// before the workgroup's barrier) instead of in two scalar registers for the whole kernel: the scorer's group loop holds
// 64 wave-uniform radius offsets in scalar registers and has none to spare.
typedef __attribute__((address_space(3))) unsigned long long lds_u64;
__device__ __forceinline__ void stash_status(unsigned long long* slot, int* status) {
    if (threadIdx.x == 0) *slot = reinterpret_cast<unsigned long long>(status);
}
__device__ __forceinline__ void report_timeout(uint32_t slot, int lane) {
    int* status = reinterpret_cast<int*>(*lds_ptr<lds_u64>(slot));
    if (status != nullptr && lane == 0) *status = kStatusHandoverTimeout;
}

// The partial of a piece whose pair has already failed: a NaN maximum for every head, which the merge turns into a NaN
// output row whatever the body of the partial holds.
__device__ __forceinline__ void poison_slot(const AttnParams& p, int lane, int b, int kvh, int slot) {
    if (lane < p.rep) {
        float* pw = p.ws + ((static_cast<size_t>(b) * p.N + static_cast<size_t>(kvh) * p.rep + lane) * p.n_splits + slot) * kPartialFloats;
        pw[0] = __builtin_nanf("");
        pw[1] = 0.0f;
    }
}

typedef __attribute__((address_space(3))) volatile int lds_vi;

__device__ __forceinline__ bool pair_wait(uint32_t addr, int want, int spin_limit) {
    bool seen = false;
#pragma clang loop unroll(disable)
    for (int i = 0; i < spin_limit; i++) {
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
                                            int t0, int t1, int r0, int r1, int& k, PairTimes& pw_times_) {
    const int rep = p.rep;
    const int bh = b * p.Nk + kvh;
    const int nb = sc.nb, nres = sc.nres;
    const uint16_t* qb = p.q + (static_cast<size_t>(b) * p.N + static_cast<size_t>(kvh) * rep) * kHeadDim;
    // polls a wait may still make: after one wait has given up it is 0, and every later wait falls through at once.  (One
    // scalar register; a separate "all hand-overs succeeded so far" flag would be a second and third, which the group
    // loop, with its 64 wave-uniform radius offsets, does not have.)
    int spin = pm.spin_limit;
    PQ_PAIR_T_MARK(0, false);
    auto publish_begin = [&]() {            // the buffer of tile k is free once tile k - 2 has been consumed
        if (k >= 2 && !PQ_PAIR_T_WAIT(pair_wait(pm.flags + 4, k - 1, spin))) spin = 0;
        return pm.sbuf + (k & 1) * (REPP * kWave * 4);
    };
    auto publish_end = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        k++;
        if (lane == 0 && !pm.silent) *lds_ptr<lds_vi>(pm.flags) = k;
        asm volatile("" ::: "memory");
        PQ_PAIR_T_TILE();
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
            PQ_PAIR_T_MARK(1, true);
            const float cdv = build_lut<T, TB, REPP>(pm.lut, lane, qx, qy, mrs, mrm, mts, mtm);
            float cds[kPairs];
            broadcast_cd(cdv, cds);
            asm volatile("" ::: "memory");
            PQ_PAIR_T_MARK(2, false);
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
    return spin != 0;
}

// Accumulator: the same tiles in the same order; writes the partial of the piece to `slot`.
template <typename T, int REPP>
__device__ __forceinline__ bool pair_accumulator(const AttnParams& p, const PairMem& pm, int lane, int b, int kvh, const SeqCounts& sc,
                                                 int t0, int t1, int r0, int r1, int slot, int& k, PairTimes& pw_times_,
                                                 uint16_t* direct_out = nullptr) {
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
    int spin = pm.spin_limit;            // 0 once a wait has given up (see pair_scorer)
    PQ_PAIR_T_MARK(0, false);
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
        if (!PQ_PAIR_T_WAIT(pair_wait(pm.flags, k + 1, spin))) spin = 0;
        const uint32_t src = pm.sbuf + (k & 1) * (REPP * kWave * 4);
        float s[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) s[j] = *lds_ptr<lds_f1>(src + (j * kWave + lane) * 4);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        k++;
        if (lane == 0) *lds_ptr<lds_vi>(pm.flags + 4) = k;
        asm volatile("" ::: "memory");
        PQ_PAIR_T_TILE();
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
    const bool ok = spin != 0;
    float lsum[REPP];
#pragma unroll
    for (int j = 0; j < REPP; j++) lsum[j] = wave_sum(st.l[j]);
    const int g = lane >> 4, n = lane & 15;
    if (n < rep) {
        float mm = st.m[0], ll = lsum[0];
#pragma unroll
        for (int j = 1; j < REPP; j++) { mm = (n == j) ? st.m[j] : mm; ll = (n == j) ? lsum[j] : ll; }
        if (!ok) mm = __builtin_nanf("");            // the scorer stopped answering: poison the result
        if (direct_out) {
            // the only slice of its plane: what the merge kernel would make of this one partial, written directly
            // (weight exp2(m - m) = 1, so out = acc / l; no token to attend to -> zeros; a poisoned slice -> NaN)
            const float den = (mm != mm) ? mm : ll;
            uint16_t* po = direct_out + (static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep + n) * kHeadDim + 32 * g;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float lo = den > 0.0f ? st.acc[e][i] / den : (den == den ? 0.0f : den);
                    const float hi = den > 0.0f ? st.acc[e + 1][i] / den : (den == den ? 0.0f : den);
                    w[e >> 1] = static_cast<uint32_t>(f2lo<T>(lo)) | (static_cast<uint32_t>(f2lo<T>(hi)) << 16);
                }
                *reinterpret_cast<uint4*>(po + 8 * i) = make_uint4(w[0], w[1], w[2], w[3]);
            }
            return ok;
        }
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

// Even slices of one plane, in 64-token tiles: slice `split` of `n_splits` takes quantized tiles [t0, t1) and, if it is
// the slice that ends the plane, the residual tiles [0, r1).  Normally a slice is a whole number of groups,
// max(min_gps, ceil(groups / n_splits)), and the last one carries the residual keys on top of its share.  That share
// is a full one when the groups divide evenly, and a full residual window then makes the last slice of every plane the
// slowest of the launch (two more tiles that move 32 KB each where a quantized tile moves 20 KB: 19 tile times against
// 16 at 8 groups per slice: 69.9 us against 62.1 us at batch 8 x 16384 tokens).  So the residual keys are given a
// weight in tiles (3 per 128 keys, to the nearest tile) and, where that lowers the longest slice, the plane is cut into
// equal runs of [quantized tiles | residual weight] instead; such slices begin and end in the middle of groups, which the
// tile loops allow.  With one residual key (and whenever the even cut is already the better one) the slices are exactly
// the whole-group ones.  Only the paired kernels cut this way: in the one-wavefront kernels (4-bit values, wide angle
// tables) the same arithmetic ahead of the first loads cost more than the cut returned.
struct EvenSlice { int t0, t1, r1; bool nothing; };
__device__ __forceinline__ EvenSlice even_slice(const SeqCounts& sc, int n_splits, int min_gps, int split) {
    const int T = 2 * sc.nb, R = (sc.nres + kWave - 1) / kWave;
    EvenSlice e;
    if (T == 0) {                                  // nothing quantized yet: slice 0 has the residual keys, if any
        e.t0 = e.t1 = 0; e.r1 = split == 0 ? R : 0; e.nothing = split > 0;
        return e;
    }
    const int RW = (3 * sc.nres + kGroup / 2) / kGroup;     // to the nearest tile: 0 below 22 keys, 3 from 107
    int ups = 2 * ((sc.nb + n_splits - 1) / n_splits);
    ups = ups < 2 * min_gps ? 2 * min_gps : ups;
    const int last = (T - 1) / ups;
    const int tail = T - last * ups + RW;          // what the last whole-group slice carries
    const int worst = (last > 0 && ups > tail) ? ups : tail;
    int alt = (T + RW + n_splits - 1) / n_splits;
    alt = alt < 2 * min_gps ? 2 * min_gps : alt;
    const bool weighted = alt < worst;
    const int per = weighted ? alt : ups;
    const int lo = split * per, hi = lo + per;
    e.t0 = lo < T ? lo : T;
    e.t1 = hi < T ? hi : T;
    e.r1 = split == (weighted ? (T + RW - 1) / alt : last) ? R : 0;
    e.nothing = split > 0 && e.t0 >= e.t1 && e.r1 == 0;
    return e;
}

// Even slices, one slice per pair.  Grid (ceil(planes / 4), slices): a workgroup's four pairs take the same slice of four
// consecutive (sequence, KV head) planes, and workgroups are handed out x first, so the plane index runs fastest as in
// attn_kernel.  (One index taken apart by two more integer divisions cost 0.3-0.4 us ahead of the first loads; `n_slices_total`
// is what the balanced kernel takes in this place and is not used here.)
template <typename T, int TB, int REPP, bool PK6>
__global__ __launch_bounds__(kPairsPerBlock * 2 * kWave) void attn_pair_kernel(PQ_ATTN_KERNEL_PARAMS, int n_slices_total, int silent_scorer,
                                                                              int* __restrict__ status, uint16_t* __restrict__ direct_out) {
    using L = Lut<TB, REPP>;
    __shared__ __attribute__((aligned(16))) char lut_mem[kPairsPerBlock][L::BYTES];
    __shared__ __attribute__((aligned(16))) float s_mem[kPairsPerBlock][2 * REPP * kWave];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[kPairsPerBlock][REPP * kWave];
    __shared__ int flag_mem[kPairsPerBlock][4];
    __shared__ int simd_of[2 * kPairsPerBlock];
    __shared__ unsigned long long status_slot;
    PQ_ATTN_KERNEL_PACK;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int pair, role;
    stash_status(&status_slot, status);
    pair_roles(simd_of, &flag_mem[0][0], wave, lane, pair, role);
    const PairMem pm = pair_mem(lds_addr(lut_mem[pair]), lds_addr(s_mem[pair]), lds_addr(p_mem[pair]), lds_addr(flag_mem[pair]), silent_scorer);

    // grid (planes / 4, slices): workgroups are handed out x first, so the plane index runs fastest
    const int bh = blockIdx.x * kPairsPerBlock + pair, split = blockIdx.y;
    if (bh >= B * Nk) return;
    const int b = bh / Nk, kvh = bh - b * Nk;
    const V4Args v4none = v4;
    const SeqCounts sc = seq_counts<false>(p, v4none, b);
    const EvenSlice es = even_slice(sc, n_splits, min_gps, split);
    if (es.nothing) {
        if (role == 1 && lane < rep) {
            float* pw = ws + ((static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep + lane) * n_splits + split) * kPartialFloats;
            pw[0] = -INFINITY;
            pw[1] = 0.0f;
        }
        return;
    }
    int k = 0;
    PairTimes waited;
    PQ_PAIR_T_DECL;
    const bool ok = role == 0 ? pair_scorer<T, TB, REPP, PK6>(p, pm, lane, b, kvh, sc, es.t0, es.t1, 0, es.r1, k, waited)
                              : pair_accumulator<T, REPP>(p, pm, lane, b, kvh, sc, es.t0, es.t1, 0, es.r1, split, k, waited, direct_out);
    if (!ok) report_timeout(lds_addr(&status_slot), lane);
    PQ_PAIR_T_REPORT(role, k, waited);
}


// Balanced slices for pairs: both wavefronts of a pair walk the same segment and meet tile by tile.
template <typename T, int TB, int REPP, bool PK6>
__global__ __launch_bounds__(kPairsPerBlock * 2 * kWave) void attn_pair_balanced_kernel(PQ_ATTN_KERNEL_PARAMS, int n_pairs_total, int silent_scorer,
                                                                                       int* __restrict__ status) {
    using L = Lut<TB, REPP>;
    __shared__ __attribute__((aligned(16))) char lut_mem[kPairsPerBlock][L::BYTES];
    __shared__ __attribute__((aligned(16))) float s_mem[kPairsPerBlock][2 * REPP * kWave];
    __shared__ __attribute__((aligned(16))) uint16_t p_mem[kPairsPerBlock][REPP * kWave];
    __shared__ int flag_mem[kPairsPerBlock][4];
    __shared__ int simd_of[2 * kPairsPerBlock];
    __shared__ int walk_mem[2 * kPairsPerBlock][kWalkInts];
    __shared__ unsigned long long status_slot;
    PQ_ATTN_KERNEL_PACK;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int pair, role;
    stash_status(&status_slot, status);
    pair_roles(simd_of, &flag_mem[0][0], wave, lane, pair, role);
    const PairMem pm = pair_mem(lds_addr(lut_mem[pair]), lds_addr(s_mem[pair]), lds_addr(p_mem[pair]), lds_addr(flag_mem[pair]), silent_scorer);
    const int w = blockIdx.x * kPairsPerBlock + pair;
    if (w >= n_pairs_total) return;
    int k = 0;
    bool ok = true;
    PairTimes waited;
    PQ_PAIR_T_DECL;
    walk_segment<false>(p, v4, n_pairs_total, w, lane, lds_addr(walk_mem[wave]),
                        [&](int cb, int ckvh, const SeqCounts& sc, int t0, int t1, int r0, int r1, int slot, bool ends_plane) {
                            // once the partner has stopped answering, the pair runs out without loads, waits or
                            // arithmetic; the accumulator still owns the partial of every remaining piece of the
                            // segment (a NaN header) and the empty slots behind a plane's last piece, so that the merge
                            // never meets what an earlier call left in the workspace
                            if (role == 0) {
                                if (ok) ok = pair_scorer<T, TB, REPP, PK6>(p, pm, lane, cb, ckvh, sc, t0, t1, r0, r1, k, waited);
                            } else {
                                if (ends_plane && slot + 1 < n_splits) mark_empty_slots(p, lane, cb, ckvh, slot + 1);
                                if (ok) ok = pair_accumulator<T, REPP>(p, pm, lane, cb, ckvh, sc, t0, t1, r0, r1, slot, k, waited);
                                else poison_slot(p, lane, cb, ckvh, slot);
                            }
                        });
    if (!ok) report_timeout(lds_addr(&status_slot), lane);
    PQ_PAIR_T_REPORT(role, k, waited);
}

#pragma clang diagnostic pop

namespace {

template <typename T, int TB>
int launch_pair_tb(const AttnArgs& a, int total, hipStream_t st) {
    const int rep = a.N / a.Nk;
    const float scale_log2 = a.sm_scale * kLog2e;
    const V4Args v4{nullptr, nullptr, nullptr, 0};
    const dim3 grid((total + kPairsPerBlock - 1) / kPairsPerBlock), block(kPairsPerBlock * 2 * kWave);
#define PQ_LAUNCH_PAIR_K(KERNEL, REPP, PK6, ...)                                                                     \
    hipLaunchKernelGGL((KERNEL<T, TB, REPP, PK6>), grid, block, 0, st, (const uint16_t*)a.q, a.codes,                \
                       (const uint16_t*)a.rscale, (const uint16_t*)a.rmn, (const uint16_t*)a.tscale,                 \
                       (const uint16_t*)a.tmn, a.group_capacity, a.n_groups, a.n_groups_per_seq,                     \
                       (const uint16_t*)a.k_resid, a.resid_capacity, a.n_resid, a.n_resid_per_seq,                   \
                       (const uint16_t*)a.v, a.v_capacity, a.mask, a.mask_stride, scale_log2, a.B, a.N, a.Nk, rep,   \
                       a.n_splits, a.min_groups_per_split, a.workspace, v4, rep, total, a.silent_scorer ? 1 : 0, a.status, ##__VA_ARGS__)
#define PQ_LAUNCH_PAIR_P(REPP, PK6)                                                                                  \
    do {                                                                                                             \
        if (a.balanced) PQ_LAUNCH_PAIR_K(attn_pair_balanced_kernel, REPP, PK6);                                      \
        else {                                                                                                       \
            const dim3 grid((a.B * a.Nk + kPairsPerBlock - 1) / kPairsPerBlock, a.n_splits);                         \
            PQ_LAUNCH_PAIR_K(attn_pair_kernel, REPP, PK6, static_cast<uint16_t*>(a.out));                            \
        }                                                                                                            \
    } while (0)
    // packed 6-bit code rows exist for tbits == 3 only (the 3/3 configuration)
#define PQ_LAUNCH_PAIR(REPP)                                                                                         \
    do {                                                                                                             \
        if constexpr (TB == 3) {                                                                                     \
            if (a.packed6) PQ_LAUNCH_PAIR_P(REPP, true);                                                             \
            else PQ_LAUNCH_PAIR_P(REPP, false);                                                                      \
        } else {                                                                                                     \
            PQ_LAUNCH_PAIR_P(REPP, false);                                                                           \
        }                                                                                                            \
    } while (0)
    switch (rep) {                // every ratio has its own instantiation: no padded head costs LDS reads or FMAs
        case 1: PQ_LAUNCH_PAIR(1); break;
        case 2: PQ_LAUNCH_PAIR(2); break;
        case 3: PQ_LAUNCH_PAIR(3); break;
        case 4: PQ_LAUNCH_PAIR(4); break;
        case 5: PQ_LAUNCH_PAIR(5); break;
        case 6: PQ_LAUNCH_PAIR(6); break;
        case 7: PQ_LAUNCH_PAIR(7); break;
        default: PQ_LAUNCH_PAIR(8); break;
    }
#undef PQ_LAUNCH_PAIR
#undef PQ_LAUNCH_PAIR_P
#undef PQ_LAUNCH_PAIR_K
    return static_cast<int>(hipGetLastError());
}

}  // namespace

// `total`: slices (even split: n_splits * B * Nk) or segments (balanced slices: what the device holds at once), one pair each
#if PQ_DTYPE == 0
int launch_attn_pair_f16(const AttnArgs& a, int total, hipStream_t st) {
    using T = F16;
#else
int launch_attn_pair_bf16(const AttnArgs& a, int total, hipStream_t st) {
    using T = BF16;
#endif
    switch (a.tbits) {
        case 1: return launch_pair_tb<T, 1>(a, total, st);
        case 2: return launch_pair_tb<T, 2>(a, total, st);
        case 3: return launch_pair_tb<T, 3>(a, total, st);
        default: return launch_pair_tb<T, 4>(a, total, st);
    }
}

}  // namespace pq
