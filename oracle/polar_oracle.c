/* CPU oracle (plain C) for the polar-key decode path.  TEST INFRASTRUCTURE ONLY.
 *
 * An independent second restatement of the reference algorithm, written with
 * scalar loops and libm so that it shares no code with oracle/polar_oracle.py
 * (torch) or with the HIP product.  Only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load the library built from this file.
 *
 * Reference lines followed:
 *   po_quantize      models/modeling_llama_polar.py:135-157
 *   po_scores        models/kernel4group.py:64-77 (semantics), :151-155 (formula)
 *   po_decode_attn   models/modeling_llama_polar.py:77-99
 *
 * Pin status: see the header of oracle/polar_oracle.py; the two restatements
 * are checked against each other bit-for-bit (codes, metadata) and to 1e-6
 * (scores) in tests/test_oracle_pins.py.
 *
 * The angle: eager torch evaluates atan2 on half / bfloat16 CPU tensors as
 * round_dtype(Sleef_atan2f_u10(float y, float x)).  SLEEF is a dependency of PyTorch
 * that is not in the reference tree (PyTorch vendors SLEEF 3.x; the routine is
 * xatan2f_u1 with atan2kf_u1 in sleefsp.c).  sleef_atan2f_u10 below restates that
 * published algorithm in plain C (two-float division, Horner scheme with fused
 * multiply-adds); tests/test_oracle_pins.py checks it bit for bit against
 * torch.atan2 on float32.  Flag bit 2 of po_quantize takes libm's atan2f instead:
 * a third opinion whose last-ulp differences can move a code across a bin edge;
 * the tests count such flips.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- half / bfloat16 <-> float, round-to-nearest-even ---- */
static float h2f(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu, u;
    if (e == 0) {
        if (m == 0) u = s;
        else { int sh = 0; while (!(m & 0x400u)) { m <<= 1; sh++; } m &= 0x3ffu; u = s | ((uint32_t)(113 - sh) << 23) | (m << 13); }
    } else if (e == 31) u = s | 0x7f800000u | (m << 13);
    else u = s | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &u, 4); return f;
}
static uint16_t f2h(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    uint32_t s = (u >> 16) & 0x8000u, e = (u >> 23) & 0xff, m = u & 0x7fffffu;
    if (e == 255) return (uint16_t)(s | 0x7c00u | (m ? 0x200u : 0));
    int ex = (int)e - 127 + 15;
    if (ex >= 31) return (uint16_t)(s | 0x7c00u);
    if (ex <= 0) {
        if (ex < -10) return (uint16_t)s;
        m |= 0x800000u;
        int sh = 14 - ex;
        uint32_t r = m >> sh, rem = m & ((1u << sh) - 1), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1))) r++;
        return (uint16_t)(s | r);
    }
    uint32_t r = ((uint32_t)ex << 10) | (m >> 13), rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) r++;
    return (uint16_t)(s | r);
}
static float b2f(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }
static uint16_t f2b(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1);
    return (uint16_t)(u >> 16);
}
static inline float lo2f(uint16_t h, int bf) { return bf ? b2f(h) : h2f(h); }
static inline uint16_t f2lo(float f, int bf) { return bf ? f2b(f) : f2h(f); }
/* round a float through the low-precision type: one eager torch op's result */
static inline float rnd(float f, int bf) { return lo2f(f2lo(f, bf), bf); }

float po_half_to_float(uint16_t h) { return h2f(h); }
uint16_t po_float_to_half(float f) { return f2h(f); }

/* ---- Sleef_atan2f_u10 (SLEEF 3.x, sleefsp.c: xatan2f_u1 / atan2kf_u1), restated ---- */
typedef struct { float x, y; } f2;
static inline float mulsignf_(float x, float y) {
    uint32_t a, b; memcpy(&a, &x, 4); memcpy(&b, &y, 4); a ^= b & 0x80000000u; memcpy(&x, &a, 4); return x;
}
static inline f2 df(float x, float y) { f2 r; r.x = x; r.y = y; return r; }
static inline f2 dfnormalize(f2 t) { f2 s; s.x = t.x + t.y; s.y = t.x - s.x + t.y; return s; }
static inline f2 dfadd_f_f(float a, float b) { f2 r; r.x = a + b; r.y = a - r.x + b; return r; }
static inline f2 dfadd_f_f2(float a, f2 b) { f2 r; r.x = a + b.x; r.y = a - r.x + b.x + b.y; return r; }
static inline f2 dfadd_f2_f2(f2 a, f2 b) { f2 r; r.x = a.x + b.x; r.y = a.x - r.x + b.x + a.y + b.y; return r; }
static inline f2 dfmul_f2_f2(f2 a, f2 b) {
    f2 r; r.x = a.x * b.x; r.y = fmaf(a.x, b.y, fmaf(a.y, b.x, fmaf(a.x, b.x, -r.x))); return r;
}
static inline f2 dfmul_f2_f(f2 a, float b) { f2 r; r.x = a.x * b; r.y = fmaf(a.y, b, fmaf(a.x, b, -r.x)); return r; }
static inline f2 dfsqu(f2 a) { f2 r; r.x = a.x * a.x; r.y = fmaf(a.x + a.x, a.y, fmaf(a.x, a.x, -r.x)); return r; }
static inline f2 dfdiv(f2 n, f2 d) {
    float t = 1.0f / d.x, u;
    f2 q;
    q.x = n.x * t;
    u = fmaf(t, n.x, -q.x);
    q.y = fmaf(-d.y, t, fmaf(-d.x, t, 1.0f));
    q.y = fmaf(q.x, q.y, fmaf(n.y, t, u));
    return q;
}
static f2 atan2kf_u1(f2 y, f2 x) {
    int q = 0;
    f2 s, t;
    float u;
    if (x.x < 0) { x.x = -x.x; x.y = -x.y; q = -2; }
    if (x.x < y.x) { t = x; x = y; y.x = -t.x; y.y = -t.y; q += 1; }
    s = dfdiv(y, x);
    t = dfnormalize(dfsqu(s));
    u = -0.00176397908944636583328247f;
    u = fmaf(u, t.x, 0.0107900900766253471374512f);
    u = fmaf(u, t.x, -0.0309564601629972457885742f);
    u = fmaf(u, t.x, 0.0577365085482597351074219f);
    u = fmaf(u, t.x, -0.0838950723409652709960938f);
    u = fmaf(u, t.x, 0.109463557600975036621094f);
    u = fmaf(u, t.x, -0.142626821994781494140625f);
    u = fmaf(u, t.x, 0.199983194470405578613281f);
    t = dfmul_f2_f2(t, dfadd_f_f(-0.333332866430282592773438f, u * t.x));
    t = dfmul_f2_f2(s, dfadd_f_f2(1.0f, t));
    t = dfadd_f2_f2(dfmul_f2_f(df(1.5707963705062866211f, -4.3711388286737928865e-08f), (float)q), t);
    return t;
}
float po_sleef_atan2f_u10(float y, float x) {
    f2 d;
    float r;
    if (fabsf(x) < 2.9387372783541830947e-39f) { y *= 16777216.0f; x *= 16777216.0f; }   /* x denormal: scale both */
    d = atan2kf_u1(df(fabsf(y), 0), df(x, 0));
    r = d.x + d.y;
    r = mulsignf_(r, x);
    if (isinf(x) || x == 0) r = 1.570796326794896557998982f - (isinf(x) ? mulsignf_(1.570796326794896557998982f, x) : 0.0f);
    if (isinf(y)) r = 1.570796326794896557998982f - (isinf(x) ? mulsignf_(0.785398163397448278999491f, x) : 0.0f);
    if (y == 0) r = signbit(x) ? 3.141592653589793238462643f : 0.0f;
    if (isnan(x) || isnan(y)) return NAN;
    return mulsignf_(r, y);
}

static uint8_t code_of(float v, float mn, float scale, int bits, int bf) {
    float d = rnd(v - mn, bf);
    float q = rnd(d / scale, bf);
    q = floorf(q);
    if (!(q == q) || isinf(q)) return 0;          /* NaN/Inf -> 0 (defined here; UB in the reference) */
    if (q < 0) q = 0;
    if (q > 255) q = 255;
    int c = (int)q, top = (1 << bits) - 1;
    return (uint8_t)(c > top ? top : c);
}

/* k: [B,Nk,L,2D] contiguous low-precision words.  Outputs contiguous:
 * codes [B,Nk,Nb,G,D] u8; rscale,rmn,tscale,tmn [B,Nk,Nb,D] low-precision words. */
int po_quantize(const uint16_t *k, int bf, int flags, int B, int Nk, int L, int D, int G, int rbits, int tbits,
                uint8_t *codes, uint16_t *rscale, uint16_t *rmn, uint16_t *tscale, uint16_t *tmn) {
    if (L % G || rbits + tbits > 8) return -1;
    /* flags: bit 0 = wrap in fp32, bit 1 = uniform angle bins over [-pi, pi) (no reference
     * counterpart: tmn = -pi, tscale = 2*pi / 2^tbits as key-dtype constants, no wrap),
     * bit 2 = libm's atan2f instead of the SLEEF routine eager torch evaluates */
    const int wrap_fp32 = flags & 1, uniform = (flags >> 1) & 1, libm_atan = (flags >> 2) & 1;
    /* torch-CPU casts the python scalar 2*pi to the tensor dtype before the add
     * (6.28125 in both half and bfloat16); wrap_fp32 != 0 keeps it in fp32, which
     * is what an eager CUDA add of a half tensor and a python scalar does. */
    const float TWO_PI = wrap_fp32 ? (float)(2.0 * 3.14159265358979323846)
                                   : rnd((float)(2.0 * 3.14159265358979323846), bf);
    int Nb = L / G;
    float *phi = (float *)malloc(sizeof(float) * G), *rad = (float *)malloc(sizeof(float) * G);
    for (long bh = 0; bh < (long)B * Nk; bh++)
        for (int nb = 0; nb < Nb; nb++)
            for (int d = 0; d < D; d++) {
                const uint16_t *base = k + ((bh * L) + (long)nb * G) * 2 * D;
                float pmx = -INFINITY, pmn = INFINITY, rmx_ = -INFINITY, rmn_ = INFINITY;
                for (int g = 0; g < G; g++) {
                    float x = lo2f(base[(long)g * 2 * D + d], bf), y = lo2f(base[(long)g * 2 * D + D + d], bf);
                    float p = rnd(libm_atan ? atan2f(y, x) : po_sleef_atan2f_u10(y, x), bf);   /* :143 */
                    if (p < 0 && !uniform) p = rnd(p + TWO_PI, bf);        /* :144 */
                    float r = rnd(sqrtf(x * x + y * y), bf);               /* :150 */
                    phi[g] = p; rad[g] = r;
                    if (p > pmx) pmx = p;
                    if (p < pmn) pmn = p;
                    if (r > rmx_) rmx_ = r;
                    if (r < rmn_) rmn_ = r;
                }
                float ts = rnd(rnd(pmx - pmn, bf) / (float)(1 << tbits), bf);   /* :147 */
                if (uniform) {
                    pmn = rnd(-(float)3.14159265358979323846, bf);
                    ts = rnd(rnd((float)(2.0 * 3.14159265358979323846), bf) / (float)(1 << tbits), bf);
                }
                float rs = rnd(rnd(rmx_ - rmn_, bf) / (float)(1 << rbits), bf); /* :152 */
                long mi = (bh * Nb + nb) * D + d;
                tscale[mi] = f2lo(ts, bf); tmn[mi] = f2lo(pmn, bf);
                rscale[mi] = f2lo(rs, bf); rmn[mi] = f2lo(rmn_, bf);
                for (int g = 0; g < G; g++) {
                    uint8_t th = code_of(phi[g], pmn, ts, tbits, bf);      /* :148 */
                    uint8_t rh = code_of(rad[g], rmn_, rs, rbits, bf);     /* :153 */
                    codes[((bh * Nb + nb) * G + g) * D + d] = (uint8_t)((rh << tbits) + th);  /* :155 */
                }
            }
    free(phi); free(rad);
    return 0;
}

/* 4-bit values of the Mixed variant (models/modeling_llama_polar.py:236,275 call
 * triton_quantize_and_pack_along_last_dim(values, 128, 4) of a kivi_quant package that is not in
 * the reference tree; restated from KIVI's published quant/new_pack.py).
 * v: [rows, D] contiguous low-precision words, one quantization group per row (D == group size).
 * codes: [rows, D*bits/32] int32, element i of each run of 32/bits in bits [i*bits, (i+1)*bits);
 * scale, mn: [rows] low-precision words. */
int po_quantize_values(const uint16_t *v, int bf, long rows, int D, int bits, int32_t *codes, uint16_t *scale,
                       uint16_t *mn) {
    if (bits <= 0 || 32 % bits || D % (32 / bits)) return -1;
    const int per = 32 / bits, top = (1 << bits) - 1;
    for (long r = 0; r < rows; r++) {
        const uint16_t *row = v + r * D;
        float lo = INFINITY, hi = -INFINITY;
        for (int d = 0; d < D; d++) {
            float x = lo2f(row[d], bf);
            if (x < lo) lo = x;
            if (x > hi) hi = x;
        }
        float sc = rnd(rnd(hi - lo, bf) / (float)top, bf);
        scale[r] = f2lo(sc, bf); mn[r] = f2lo(lo, bf);
        for (int w = 0; w < D / per; w++) {
            uint32_t word = 0;
            for (int i = 0; i < per; i++) {
                float q = rnd(rnd(lo2f(row[w * per + i], bf) - lo, bf) / sc, bf);
                if (q < 0) q = 0;
                if (q > top) q = (float)top;
                q = nearbyintf(q);                        /* round half to even (default rounding mode) */
                uint32_t c = (q == q) ? (uint32_t)q : 0u; /* 0/0 on a constant row -> 0 (defined here) */
                word |= c << (i * bits);
            }
            codes[r * (D / per) + w] = (int32_t)word;
        }
    }
    return 0;
}

/* scores[b,h,l] = sum_d (q[d] cos phi^ + q[d+D] sin phi^) * r^ ; out [B,N,Nb*G] fp32 */
int po_scores(const uint16_t *q, int bf, const uint8_t *codes, const uint16_t *rscale, const uint16_t *rmn,
              const uint16_t *tscale, const uint16_t *tmn, float *out,
              int B, int N, int Nk, int Nb, int G, int D, int rbits, int tbits) {
    (void)rbits;
    int rep = N / Nk, nt = 1 << tbits;
    double *lc = (double *)malloc(sizeof(double) * D * nt), *ls = (double *)malloc(sizeof(double) * D * nt);
    for (int b = 0; b < B; b++)
        for (int h = 0; h < N; h++) {
            int kvh = h / rep;
            const uint16_t *qq = q + ((long)b * N + h) * 2 * D;
            for (int nb = 0; nb < Nb; nb++) {
                long mi = (((long)b * Nk + kvh) * Nb + nb) * D;
                for (int d = 0; d < D; d++)
                    for (int t = 0; t < nt; t++) {
                        double p = (double)lo2f(tscale[mi + d], bf) * (t + 0.5) + (double)lo2f(tmn[mi + d], bf);
                        lc[d * nt + t] = cos(p); ls[d * nt + t] = sin(p);
                    }
                for (int g = 0; g < G; g++) {
                    const uint8_t *c = codes + ((((long)b * Nk + kvh) * Nb + nb) * G + g) * D;
                    double acc = 0;
                    for (int d = 0; d < D; d++) {
                        int th = c[d] & (nt - 1), rh = c[d] >> tbits;
                        double r = (double)lo2f(rscale[mi + d], bf) * (rh + 0.5) + (double)lo2f(rmn[mi + d], bf);
                        acc += ((double)lo2f(qq[d], bf) * lc[d * nt + th] + (double)lo2f(qq[D + d], bf) * ls[d * nt + th]) * r;
                    }
                    out[((long)b * N + h) * Nb * G + (long)nb * G + g] = (float)acc;
                }
            }
        }
    free(lc); free(ls);
    return 0;
}

/* Full decode attention for one step (new k/v already appended by the caller).
 * q [B,N,2D]; codes/meta as above (Nb groups, may be 0); kres [B,Nk,res,2D]; v [B,Nk,Nb*G+res,2D];
 * mask [B,Nb*G+res] bytes (1 keep) or NULL; out [B,N,2D] low-precision words. */
int po_decode_attn(const uint16_t *q, int bf, const uint8_t *codes, const uint16_t *rscale, const uint16_t *rmn,
                   const uint16_t *tscale, const uint16_t *tmn, const uint16_t *kres, int res,
                   const uint16_t *v, const uint8_t *mask, uint16_t *out,
                   int B, int N, int Nk, int Nb, int G, int D, int rbits, int tbits) {
    int rep = N / Nk, Lq = Nb * G, Lt = Lq + res, hd = 2 * D;
    float *sq = (float *)malloc(sizeof(float) * (size_t)B * N * (Lq ? Lq : 1));
    if (Nb) po_scores(q, bf, codes, rscale, rmn, tscale, tmn, sq, B, N, Nk, Nb, G, D, rbits, tbits);
    double *s = (double *)malloc(sizeof(double) * Lt), *acc = (double *)malloc(sizeof(double) * hd);
    double isq = 1.0 / sqrt((double)hd);
    for (int b = 0; b < B; b++)
        for (int h = 0; h < N; h++) {
            int kvh = h / rep;
            const uint16_t *qq = q + ((long)b * N + h) * hd;
            for (int l = 0; l < Lq; l++) s[l] = (double)sq[((long)b * N + h) * Lq + l] * isq;
            for (int l = 0; l < res; l++) {
                const uint16_t *kk = kres + (((long)b * Nk + kvh) * res + l) * hd;
                float a = 0;
                for (int d = 0; d < hd; d++) a += lo2f(qq[d], bf) * lo2f(kk[d], bf);
                s[Lq + l] = (double)rnd(a, bf) * isq;                      /* half matmul then .to(float32), :79 */
            }
            double mx = -INFINITY;
            for (int l = 0; l < Lt; l++) {
                if (mask && !mask[(long)b * Lt + l]) s[l] = -INFINITY;
                if (s[l] > mx) mx = s[l];
            }
            double den = 0;
            for (int l = 0; l < Lt; l++) { s[l] = exp(s[l] - mx); den += s[l]; }
            for (int d = 0; d < hd; d++) acc[d] = 0;
            for (int l = 0; l < Lt; l++) {
                double p = (double)rnd((float)(s[l] / den), bf);           /* softmax(...).to(q.dtype), :97 */
                const uint16_t *vv = v + (((long)b * Nk + kvh) * Lt + l) * hd;
                for (int d = 0; d < hd; d++) acc[d] += p * lo2f(vv[d], bf);
            }
            for (int d = 0; d < hd; d++) out[((long)b * N + h) * hd + d] = f2lo((float)acc[d], bf);
        }
    free(sq); free(s); free(acc);
    return 0;
}
