// 4-bit value quantizer of the Mixed variant: values [B,Nk,T,128] are quantized
// per token and head along the 128 dims (one min/max group per row), 8 codes to
// an int32, element i in bits [4i, 4i+4).  HIP counterpart of the
// triton_quantize_and_pack_along_last_dim(values, 128, 4) calls at
// models/modeling_llama_polar.py:236 and :275 (the routine itself belongs to a
// kivi_quant package that is not in the reference tree; its published form is
// followed: scale = (max - min) / 15, q = round_half_even(clamp((x - min) / scale, 0, 15)),
// every op rounded to the value dtype as eager torch does).
//
// 16 lanes own one row: each loads 16 bytes (dims 8n..8n+7) and writes the row's
// n-th code word, so a wavefront reads four whole 256-byte rows and writes 256
// contiguous bytes of codes.
#include "pq_device.h"
#include "pq_internal.h"

namespace pq {

template <typename T>
__device__ __forceinline__ float rnd_v(float f) { return lo2f<T>(f2lo<T>(f)); }

template <typename T> struct IsF16 { static constexpr bool value = false; };
template <> struct IsF16<F16> { static constexpr bool value = true; };

constexpr int kVThreads = 256;
constexpr int kRowsPerBlock = kVThreads / 16;

constexpr int kRowsPerLane = 2;   // two independent 16-byte loads in flight per lane

template <typename T>
__device__ __forceinline__ void quantize_row(uint4 w, bool live, int n, int64_t row,
                                             int32_t* __restrict__ codes, uint16_t* __restrict__ scale, uint16_t* __restrict__ mn) {
    if constexpr (IsF16<T>::value) {
        // half precision: the eager ops ARE half-precision instructions here (v_pk_min/max_f16,
        // v_sub_f16, v_med3_f16, v_rndne_f16); the division is div_faithful
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        const half2v p0 = __builtin_bit_cast(half2v, w.x), p1 = __builtin_bit_cast(half2v, w.y);
        const half2v p2 = __builtin_bit_cast(half2v, w.z), p3 = __builtin_bit_cast(half2v, w.w);
        const half2v mn2 = __builtin_elementwise_min(__builtin_elementwise_min(p0, p1), __builtin_elementwise_min(p2, p3));
        const half2v mx2 = __builtin_elementwise_max(__builtin_elementwise_max(p0, p1), __builtin_elementwise_max(p2, p3));
        // (min, -max) in one register: both reduce with a packed min
        half2v red = {live ? (mn2.x < mn2.y ? mn2.x : mn2.y) : static_cast<_Float16>(INFINITY),
                      live ? -(mx2.x > mx2.y ? mx2.x : mx2.y) : static_cast<_Float16>(INFINITY)};
        {
            uint32_t rw = __builtin_bit_cast(uint32_t, red);
            static_for<4>([&](auto s) {
                const uint32_t other = row_rotate<(1 << decltype(s)::value)>(rw);
                rw = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(half2v, rw), __builtin_bit_cast(half2v, other)));
            });
            red = __builtin_bit_cast(half2v, rw);
        }
        if (!live) return;
        const _Float16 lo = red.x, hi = -red.y;
        const _Float16 sc = static_cast<_Float16>(hi - lo) / static_cast<_Float16>(15.0f);
        const half2v ps[4] = {p0, p1, p2, p3};
        const float scf = static_cast<float>(sc);
        uint32_t word = 0;
        if (__builtin_expect(fast_div_ok(scf), 1)) {
            const float inv = __builtin_amdgcn_rcpf(scf);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const _Float16 x = (i & 1) ? ps[i >> 1].y : ps[i >> 1].x;
                _Float16 q = static_cast<_Float16>(div_faithful(static_cast<float>(static_cast<_Float16>(x - lo)), scf, inv));
                q = __builtin_amdgcn_fmed3h(q, static_cast<_Float16>(0.0f), static_cast<_Float16>(15.0f));
                q = __builtin_rintf16(q);                      // round half to even
                word |= static_cast<uint32_t>(static_cast<unsigned short>(q)) << (4 * i);
            }
        } else {
            // constant rows (0/0), scales that underflow to 0 (x/0), infinities
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const _Float16 x = (i & 1) ? ps[i >> 1].y : ps[i >> 1].x;
                _Float16 q = static_cast<_Float16>(x - lo) / sc;
                q = __builtin_amdgcn_fmed3h(q, static_cast<_Float16>(0.0f), static_cast<_Float16>(15.0f));   // NaN (0/0) -> 0
                q = __builtin_rintf16(q);
                word |= static_cast<uint32_t>(static_cast<unsigned short>(q)) << (4 * i);
            }
        }
        codes[row * 16 + n] = static_cast<int32_t>(word);
        if (n == 0) { scale[row] = __builtin_bit_cast(uint16_t, sc); mn[row] = __builtin_bit_cast(uint16_t, lo); }
    } else {
        float x[8];
        float lo = INFINITY, hi = -INFINITY;
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[2 * i] = lo2f<T>(static_cast<uint16_t>(ww[i] & 0xffffu));
            x[2 * i + 1] = lo2f<T>(static_cast<uint16_t>(ww[i] >> 16));
        }
        if (live) {
#pragma unroll
            for (int i = 0; i < 8; i++) { lo = fminf(lo, x[i]); hi = fmaxf(hi, x[i]); }
        }
        static_for<4>([&](auto s) {
            lo = fminf(lo, __uint_as_float(row_rotate<(1 << decltype(s)::value)>(__float_as_uint(lo))));
            hi = fmaxf(hi, __uint_as_float(row_rotate<(1 << decltype(s)::value)>(__float_as_uint(hi))));
        });
        if (!live) return;
        const float sc = rnd_v<T>(rnd_v<T>(hi - lo) / 15.0f);
        uint32_t word = 0;
        if (__builtin_expect(fast_div_ok(sc), 1)) {
            const float inv = __builtin_amdgcn_rcpf(sc);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float q = rnd_v<T>(div_faithful(rnd_v<T>(x[i] - lo), sc, inv));
                q = __builtin_amdgcn_fmed3f(q, 0.0f, 15.0f);
                q = __builtin_rintf(q);                        // round half to even
                word |= static_cast<uint32_t>(q) << (4 * i);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float q = rnd_v<T>(rnd_v<T>(x[i] - lo) / sc);
                q = __builtin_amdgcn_fmed3f(q, 0.0f, 15.0f);   // NaN (0/0 on a constant row) comes out as the minimum, 0
                q = __builtin_rintf(q);
                word |= static_cast<uint32_t>(q) << (4 * i);
            }
        }
        codes[row * 16 + n] = static_cast<int32_t>(word);
        if (n == 0) { scale[row] = f2lo<T>(sc); mn[row] = f2lo<T>(lo); }
    }
}

template <typename T>
__global__ __launch_bounds__(kVThreads) void quantize_values_kernel(
    const uint16_t* __restrict__ v, int64_t sb, int64_t sh, int64_t st, int Nk, int n_tok,
    int32_t* __restrict__ codes, uint16_t* __restrict__ scale, uint16_t* __restrict__ mn, int64_t cap, int64_t off) {
    const int n = threadIdx.x & 15;
    const int bh = blockIdx.y;
    const int b = bh / Nk, h = bh - b * Nk;
    const uint16_t* vb = v + b * sb + h * sh + 8 * n;
    uint4 w[kRowsPerLane];
    int t[kRowsPerLane];
#pragma unroll
    for (int u = 0; u < kRowsPerLane; u++) {
        t[u] = (blockIdx.x * kRowsPerLane + u) * kRowsPerBlock + (threadIdx.x >> 4);
        w[u] = make_uint4(0, 0, 0, 0);
        if (t[u] < n_tok) w[u] = *reinterpret_cast<const uint4*>(vb + static_cast<int64_t>(t[u]) * st);   // whole 16-lane rows are live or not
    }
#pragma unroll
    for (int u = 0; u < kRowsPerLane; u++)
        quantize_row<T>(w[u], t[u] < n_tok, n, static_cast<int64_t>(bh) * cap + off + t[u], codes, scale, mn);
}

int launch_quantize_values(const void* v, const int64_t* strides, int dtype, int B, int Nk, int T,
                           int32_t* codes, void* scale, void* mn, int64_t cap, int64_t off, hipStream_t st) {
    dim3 grid((T + kRowsPerBlock * kRowsPerLane - 1) / (kRowsPerBlock * kRowsPerLane), B * Nk), block(kVThreads);
    if (dtype == 0)
        hipLaunchKernelGGL(quantize_values_kernel<F16>, grid, block, 0, st, (const uint16_t*)v, strides[0], strides[1],
                           strides[2], Nk, T, codes, (uint16_t*)scale, (uint16_t*)mn, cap, off);
    else
        hipLaunchKernelGGL(quantize_values_kernel<BF16>, grid, block, 0, st, (const uint16_t*)v, strides[0], strides[1],
                           strides[2], Nk, T, codes, (uint16_t*)scale, (uint16_t*)mn, cap, off);
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
