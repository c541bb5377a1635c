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
            float phi = rnd<T>(math::atan2f_sleef_u10(y, x));          // :143
            if (phi < 0.0f) phi = rnd<T>(phi + two_pi);                // :144
            const float r = rnd<T>(__fsqrt_rn(__builtin_fmaf(x, x, y * y)));   // :150 (x*x, y*y are exact)
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
