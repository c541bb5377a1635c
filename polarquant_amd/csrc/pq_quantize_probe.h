// Timing-only probe of another quantizer algorithm (-DPQ_PROBE_DIRECT_BINS, `python -m polarquant_amd.build --probe
// direct_bins`; never part of the shipping library): bin the fp32 estimates of angle and radius directly,
//     code = floor((a - min) / scale),
// instead of rounding every intermediate to the key dtype as eager torch does, and only TEST whether an element lies so
// close to a bin edge that the dtype's roundings could move it across (those elements, and the candidates for a pair's
// minimum and maximum, would take the exact route in a complete implementation; here nobody does).  The codes it
// writes are therefore WRONG near bin edges: the kernel exists to measure the floor of that algorithm, i.e. what
// the estimates, the direct binning and the edge test cost without any exact path.
// Included by pq_quantize.hip inside namespace pq.
template <typename T>
__global__ __launch_bounds__(kQThreads) void quantize_direct_bins_probe_kernel(
    const uint16_t* __restrict__ k, int64_t sb, int64_t sh, int64_t st, int Nk, int rbits, int tbits, float two_pi,
    uint8_t* __restrict__ codes, uint16_t* __restrict__ rscale, uint16_t* __restrict__ rmn,
    uint16_t* __restrict__ tscale, uint16_t* __restrict__ tmn, int cap, int off) {
    __shared__ float red[4][4][kPairs];        // angle max / min, radius max / min; wavefront; pair
    __shared__ float fin[4][kPairs];
    const int tid = threadIdx.x;
    const int pq4 = tid & 15, tl = tid >> 4;
    const int grp = blockIdx.x, bh = blockIdx.y;
    const int b = bh / Nk, h = bh - b * Nk;
    const uint16_t* kb = k + b * sb + h * sh + static_cast<int64_t>(grp) * kGroup * st;
    float av[kEntries], rv[kEntries];
    float amax[4], amin[4], rmax[4], rmin[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { amax[i] = 0.0f; amin[i] = INFINITY; rmax[i] = 0.0f; rmin[i] = INFINITY; }
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
            const float x = lo2f<T>(xs[i]), y = lo2f<T>(ys[i]);
            // a short arctangent (degree 7 in r, ~1e-5 rad: far inside the edge test's band), wrapped to [0, 2 pi)
            const float ax = fabsf(x), ay = fabsf(y);
            const float mx = fmaxf(ax, ay), mn = fminf(ax, ay);
            const float r = mn * __builtin_amdgcn_rcpf(mx);
            const float s = r * r;
            float u = -0.0464964749f;
            u = __builtin_fmaf(u, s, 0.15931422f);
            u = __builtin_fmaf(u, s, -0.327622764f);
            float a = __builtin_fmaf(u * s, r, r);
            a = ay > ax ? 1.57079637f - a : a;
            a = x < 0.0f ? 3.14159274f - a : a;
            a = y < 0.0f ? two_pi - a : a;
            const float rad = __builtin_amdgcn_sqrtf(__builtin_fmaf(x, x, y * y));
            av[it * 4 + i] = a; rv[it * 4 + i] = rad;
            amax[i] = fmaxf(amax[i], a); amin[i] = fminf(amin[i], a);
            rmax[i] = fmaxf(rmax[i], rad); rmin[i] = fminf(rmin[i], rad);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int o = 16; o <= 32; o <<= 1) {
            amax[i] = fmaxf(amax[i], __shfl_xor(amax[i], o)); amin[i] = fminf(amin[i], __shfl_xor(amin[i], o));
            rmax[i] = fmaxf(rmax[i], __shfl_xor(rmax[i], o)); rmin[i] = fminf(rmin[i], __shfl_xor(rmin[i], o));
        }
    }
    if ((tid & 48) == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            red[0][tid >> 6][4 * pq4 + i] = amax[i]; red[1][tid >> 6][4 * pq4 + i] = amin[i];
            red[2][tid >> 6][4 * pq4 + i] = rmax[i]; red[3][tid >> 6][4 * pq4 + i] = rmin[i];
        }
    }
    __syncthreads();
    {
        const int s = tid >> 6, p = tid & 63;
        float v = red[s][0][p];
#pragma unroll
        for (int j = 1; j < 4; j++) v = (s & 1) ? fminf(v, red[s][j][p]) : fmaxf(v, red[s][j][p]);
        fin[s][p] = v;
    }
    __syncthreads();
    const float inv_t = static_cast<float>(1 << tbits), inv_r = static_cast<float>(1 << rbits);
    float ts[4], tm[4], rs[4], rm[4], tinv[4], rinv[4], tband[4], rband[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // (a complete implementation would take these four from the exactly evaluated extreme elements)
        tm[i] = rnd<T>(fin[1][4 * pq4 + i]); rm[i] = rnd<T>(fin[3][4 * pq4 + i]);
        ts[i] = rnd<T>(rnd<T>(rnd<T>(fin[0][4 * pq4 + i]) - tm[i]) / inv_t);
        rs[i] = rnd<T>(rnd<T>(rnd<T>(fin[2][4 * pq4 + i]) - rm[i]) / inv_r);
        tinv[i] = __builtin_amdgcn_rcpf(ts[i]); rinv[i] = __builtin_amdgcn_rcpf(rs[i]);
        // how far the dtype's roundings (of the value, of the difference, of the quotient) can move a quotient, in bins
        constexpr float kUlp = IsHalf<T>::value ? 0x1p-11f : 0x1p-8f;
        tband[i] = 2.0f * 6.2831853f * kUlp * tinv[i] + inv_t * kUlp;
        rband[i] = 2.0f * fin[2][4 * pq4 + i] * kUlp * rinv[i] + inv_r * kUlp;
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
    const float ttop = static_cast<float>((1 << tbits) - 1), rtop = static_cast<float>((1 << rbits) - 1);
    uint8_t* cb = codes + plane * (kGroup * kPairs);
    uint32_t near_edge = 0;
#pragma unroll
    for (int it = 0; it < kTokPerThread; it++) {
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float tq = (av[it * 4 + i] - tm[i]) * tinv[i], rq = (rv[it * 4 + i] - rm[i]) * rinv[i];
            const uint32_t th = static_cast<uint32_t>(__builtin_amdgcn_fmed3f(floorf(tq), 0.0f, ttop));
            const uint32_t rh = static_cast<uint32_t>(__builtin_amdgcn_fmed3f(floorf(rq), 0.0f, rtop));
            near_edge |= static_cast<uint32_t>(fabsf(tq - __builtin_rintf(tq)) < tband[i]) << (it * 4 + i);
            near_edge |= static_cast<uint32_t>(fabsf(rq - __builtin_rintf(rq)) < rband[i]) << (it * 4 + i);
            w |= (((rh << tbits) + th) & 0xffu) << (8 * i);
        }
        *reinterpret_cast<uint32_t*>(cb + (it * 16 + tl) * kPairs + 4 * pq4) = w;
    }
    // keep the edge test alive: the number of flagged entries of thread 0 goes into a byte nobody reads back as a code
    if (near_edge == 0xdeadbeefu) cb[0] = 0;
}
