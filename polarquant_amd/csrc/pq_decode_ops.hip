// Small fused kernels for the decode step around the attention call
// (models/modeling_llama_polar.py:47-59 projections -> RoPE -> cache append, and the
// decoder layer's norms / MLP activation, :456-486), each replacing a chain of
// 8-12 eager elementwise launches on a [B, 1, hidden] activation:
//
//   rope_append_kernel  q/k rotation (HF rotate-half) + write of the new key into the residual
//                       window + write of the new value into the value cache, positions read
//                       from device memory so that the step can be replayed from a graph
//   rmsnorm_kernel      (optional residual add) + RMS norm
//   silu_mul_kernel     silu(gate) * up
//
// Arithmetic follows the eager modules op by op in the activation dtype: every
// product / sum is formed in fp32 and rounded to the dtype before the next op.
#include "pq_device.h"
#include "pq_internal.h"

namespace pq {

template <typename T>
__device__ __forceinline__ float rnd_a(float f) { return lo2f<T>(f2lo<T>(f)); }

// grid (N + 2*Nk, B), 64 threads: lane d owns the pair (d, d+64) of one head.
//   q_lin [B, N*128], k_lin / v_lin [B, Nk*128]: outputs of the projections for the new token; batch
//   rows are `lin_stride` elements apart (N*128 etc. when separate and dense, (N+2Nk)*128 when the
//   three are slices of one fused projection output)
//   cos_tab / sin_tab [max_pos, 128] in the dtype; *pos = position of the new token
//   q_out [B, N, 128]
//   k_dst [B, Nk, k_rows, 128]: row *k_row receives the rotated key
//   v_dst [B, Nk, v_rows, 128]: row *v_row receives the value
template <typename T>
__global__ __launch_bounds__(kWave) void rope_append_kernel(
    const uint16_t* __restrict__ q_lin, const uint16_t* __restrict__ k_lin, const uint16_t* __restrict__ v_lin,
    const uint16_t* __restrict__ cos_tab, const uint16_t* __restrict__ sin_tab, const int64_t* __restrict__ pos,
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_dst, int64_t k_rows, const int64_t* __restrict__ k_row,
    uint16_t* __restrict__ v_dst, int64_t v_rows, const int64_t* __restrict__ v_row, int N, int Nk, int64_t max_pos,
    int64_t q_stride, int64_t kv_stride) {
    const int d = threadIdx.x, h = blockIdx.x, b = blockIdx.y;
    if (h >= N + Nk) {                               // value head: plain copy into the cache row
        const int kvh = h - N - Nk;
        int64_t r = *v_row;
        r = r < 0 ? 0 : (r >= v_rows ? v_rows - 1 : r);
        const uint16_t* src = v_lin + static_cast<size_t>(b) * kv_stride + static_cast<size_t>(kvh) * kHeadDim;
        uint16_t* dst = v_dst + ((static_cast<size_t>(b) * Nk + kvh) * v_rows + r) * kHeadDim;
        dst[d] = src[d];
        dst[d + kPairs] = src[d + kPairs];
        return;
    }
    int64_t p = *pos;
    p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
    const float c1 = lo2f<T>(cos_tab[p * kHeadDim + d]), c2 = lo2f<T>(cos_tab[p * kHeadDim + kPairs + d]);
    const float s1 = lo2f<T>(sin_tab[p * kHeadDim + d]), s2 = lo2f<T>(sin_tab[p * kHeadDim + kPairs + d]);
    const bool is_q = h < N;
    const uint16_t* src = is_q ? q_lin + static_cast<size_t>(b) * q_stride + static_cast<size_t>(h) * kHeadDim
                               : k_lin + static_cast<size_t>(b) * kv_stride + static_cast<size_t>(h - N) * kHeadDim;
    const float x1 = lo2f<T>(src[d]), x2 = lo2f<T>(src[d + kPairs]);
    // (x * cos) + (rotate_half(x) * sin), rotate_half(x) = cat(-x2, x1)
    const float o1 = rnd_a<T>(rnd_a<T>(x1 * c1) + rnd_a<T>(-x2 * s1));
    const float o2 = rnd_a<T>(rnd_a<T>(x2 * c2) + rnd_a<T>(x1 * s2));
    uint16_t* dst;
    if (is_q) {
        dst = q_out + (static_cast<size_t>(b) * N + h) * kHeadDim;
    } else {
        int64_t r = *k_row;
        r = r < 0 ? 0 : (r >= k_rows ? k_rows - 1 : r);
        dst = k_dst + ((static_cast<size_t>(b) * Nk + (h - N)) * k_rows + r) * kHeadDim;
    }
    dst[d] = f2lo<T>(o1);
    dst[d + kPairs] = f2lo<T>(o2);
}

// RoPE over whole sequences (the prompt pass, models/modeling_llama_polar.py:56-59): one workgroup per token,
// all query and key heads of it; a thread takes dims c..c+7 and 64+c..64+c+7 of one head (two 16-byte loads), the
// token's cos / sin rows are shared by its heads.  Same arithmetic as rope_append_kernel, so the same bits as the
// eager (x * cos) + (rotate_half(x) * sin).
//   q_lin / k_lin: projection outputs, token t = b * L + l at q_lin + t * q_stride (k likewise)
//   cos / sin [1 or B, L, 128]: batch b at b * cs_batch_stride (0 when shared)
//   q_out [B, L, N, 128], k_out [B, L, Nk, 128] contiguous
template <typename T>
__global__ __launch_bounds__(256) void rope_qk_kernel(
    const uint16_t* __restrict__ q_lin, int64_t q_stride, const uint16_t* __restrict__ k_lin, int64_t k_stride,
    const uint16_t* __restrict__ cos_t, const uint16_t* __restrict__ sin_t, int64_t cs_batch_stride,
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out, int L, int N, int Nk) {
    const size_t tok = blockIdx.x;
    const size_t b = tok / L, l = tok - b * L;
    const size_t cs = b * cs_batch_stride + l * kHeadDim;
    for (int item = threadIdx.x; item < (N + Nk) * 8; item += 256) {
        const int head = item >> 3, c = (item & 7) * 8;
        const bool is_q = head < N;
        const uint16_t* src = is_q ? q_lin + tok * q_stride + static_cast<size_t>(head) * kHeadDim
                                   : k_lin + tok * k_stride + static_cast<size_t>(head - N) * kHeadDim;
        uint16_t* dst = is_q ? q_out + (tok * N + head) * kHeadDim : k_out + (tok * Nk + (head - N)) * kHeadDim;
        const uint4 a1 = *reinterpret_cast<const uint4*>(src + c), a2 = *reinterpret_cast<const uint4*>(src + kPairs + c);
        const uint4 vc1 = *reinterpret_cast<const uint4*>(cos_t + cs + c), vc2 = *reinterpret_cast<const uint4*>(cos_t + cs + kPairs + c);
        const uint4 vs1 = *reinterpret_cast<const uint4*>(sin_t + cs + c), vs2 = *reinterpret_cast<const uint4*>(sin_t + cs + kPairs + c);
        const uint32_t x1w[4] = {a1.x, a1.y, a1.z, a1.w}, x2w[4] = {a2.x, a2.y, a2.z, a2.w};
        const uint32_t c1w[4] = {vc1.x, vc1.y, vc1.z, vc1.w}, c2w[4] = {vc2.x, vc2.y, vc2.z, vc2.w};
        const uint32_t s1w[4] = {vs1.x, vs1.y, vs1.z, vs1.w}, s2w[4] = {vs2.x, vs2.y, vs2.z, vs2.w};
        uint32_t o1w[4], o2w[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t r1 = 0, r2 = 0;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
                const int sh = 16 * hh;
                const float x1 = lo2f<T>(static_cast<uint16_t>(x1w[j] >> sh)), x2 = lo2f<T>(static_cast<uint16_t>(x2w[j] >> sh));
                const float c1 = lo2f<T>(static_cast<uint16_t>(c1w[j] >> sh)), c2 = lo2f<T>(static_cast<uint16_t>(c2w[j] >> sh));
                const float s1 = lo2f<T>(static_cast<uint16_t>(s1w[j] >> sh)), s2 = lo2f<T>(static_cast<uint16_t>(s2w[j] >> sh));
                const float o1 = rnd_a<T>(x1 * c1) + rnd_a<T>(-x2 * s1);
                const float o2 = rnd_a<T>(x2 * c2) + rnd_a<T>(x1 * s2);
                r1 |= static_cast<uint32_t>(f2lo<T>(o1)) << sh;
                r2 |= static_cast<uint32_t>(f2lo<T>(o2)) << sh;
            }
            o1w[j] = r1; o2w[j] = r2;
        }
        *reinterpret_cast<uint4*>(dst + c) = make_uint4(o1w[0], o1w[1], o1w[2], o1w[3]);
        *reinterpret_cast<uint4*>(dst + kPairs + c) = make_uint4(o2w[0], o2w[1], o2w[2], o2w[3]);
    }
}

// One 256-thread block per row of `hidden` elements (hidden % 8 == 0).
//   s = x (+ res, rounded to the dtype; written to sum_out if given)
//   y = w * dtype( float(s) * rsqrt(mean(float(s)^2) + eps) )
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
                                                       const uint16_t* __restrict__ w, uint16_t* __restrict__ y,
                                                       uint16_t* __restrict__ sum_out, int hidden, float eps) {
    __shared__ float part[4];
    const size_t row = static_cast<size_t>(blockIdx.x) * hidden;
    float ss = 0.0f;
    for (int i = threadIdx.x * 8; i < hidden; i += 256 * 8) {
        const uint4 xv = *reinterpret_cast<const uint4*>(x + row + i);
        uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
        if (res) {
            const uint4 rv = *reinterpret_cast<const uint4*>(res + row + i);
            const uint32_t rw[4] = {rv.x, rv.y, rv.z, rv.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint16_t lo = f2lo<T>(lo2f<T>(static_cast<uint16_t>(xw[j] & 0xffffu)) + lo2f<T>(static_cast<uint16_t>(rw[j] & 0xffffu)));
                const uint16_t hi = f2lo<T>(lo2f<T>(static_cast<uint16_t>(xw[j] >> 16)) + lo2f<T>(static_cast<uint16_t>(rw[j] >> 16)));
                xw[j] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
            }
            if (sum_out) *reinterpret_cast<uint4*>(sum_out + row + i) = make_uint4(xw[0], xw[1], xw[2], xw[3]);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float a = lo2f<T>(static_cast<uint16_t>(xw[j] & 0xffffu)), c = lo2f<T>(static_cast<uint16_t>(xw[j] >> 16));
            ss = __builtin_fmaf(a, a, ss);
            ss = __builtin_fmaf(c, c, ss);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = rsqrtf((part[0] + part[1] + part[2] + part[3]) / static_cast<float>(hidden) + eps);
    const uint16_t* src = (res && sum_out) ? sum_out : nullptr;
    for (int i = threadIdx.x * 8; i < hidden; i += 256 * 8) {
        uint32_t xw[4];
        if (src) {                                   // re-read the rounded sums this thread wrote
            const uint4 sv = *reinterpret_cast<const uint4*>(src + row + i);
            xw[0] = sv.x; xw[1] = sv.y; xw[2] = sv.z; xw[3] = sv.w;
        } else {
            const uint4 xv = *reinterpret_cast<const uint4*>(x + row + i);
            xw[0] = xv.x; xw[1] = xv.y; xw[2] = xv.z; xw[3] = xv.w;
            if (res) {
                const uint4 rv = *reinterpret_cast<const uint4*>(res + row + i);
                const uint32_t rw[4] = {rv.x, rv.y, rv.z, rv.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint16_t lo = f2lo<T>(lo2f<T>(static_cast<uint16_t>(xw[j] & 0xffffu)) + lo2f<T>(static_cast<uint16_t>(rw[j] & 0xffffu)));
                    const uint16_t hi = f2lo<T>(lo2f<T>(static_cast<uint16_t>(xw[j] >> 16)) + lo2f<T>(static_cast<uint16_t>(rw[j] >> 16)));
                    xw[j] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
                }
            }
        }
        const uint4 wv = *reinterpret_cast<const uint4*>(w + i);
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
        uint32_t yo[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float a = rnd_a<T>(lo2f<T>(static_cast<uint16_t>(xw[j] & 0xffffu)) * inv);
            const float c = rnd_a<T>(lo2f<T>(static_cast<uint16_t>(xw[j] >> 16)) * inv);
            const uint16_t lo = f2lo<T>(lo2f<T>(static_cast<uint16_t>(ww[j] & 0xffffu)) * a);
            const uint16_t hi = f2lo<T>(lo2f<T>(static_cast<uint16_t>(ww[j] >> 16)) * c);
            yo[j] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        }
        *reinterpret_cast<uint4*>(y + row + i) = make_uint4(yo[0], yo[1], yo[2], yo[3]);
    }
}

// y[r][c] = dtype(silu(gate[r][c])) * up[r][c] for `rows` rows of `cols` elements (cols % 8 == 0); gate and
// up rows are `in_stride` elements apart (cols when dense, 2*cols when they are the two halves of one
// fused projection output), y is dense.  silu(x) = x / (1 + exp(-x)) in fp32.
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up,
                                                        uint16_t* __restrict__ y, int cols, int64_t in_stride) {
    const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (c >= cols) return;
    const size_t in = static_cast<size_t>(blockIdx.y) * in_stride + c, out = static_cast<size_t>(blockIdx.y) * cols + c;
    const uint4 gv = *reinterpret_cast<const uint4*>(gate + in), uv = *reinterpret_cast<const uint4*>(up + in);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t yo[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float g0 = lo2f<T>(static_cast<uint16_t>(gw[j] & 0xffffu)), g1 = lo2f<T>(static_cast<uint16_t>(gw[j] >> 16));
        const float a0 = rnd_a<T>(g0 / (1.0f + __expf(-g0))), a1 = rnd_a<T>(g1 / (1.0f + __expf(-g1)));
        const uint16_t lo = f2lo<T>(a0 * lo2f<T>(static_cast<uint16_t>(uw[j] & 0xffffu)));
        const uint16_t hi = f2lo<T>(a1 * lo2f<T>(static_cast<uint16_t>(uw[j] >> 16)));
        yo[j] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
    }
    *reinterpret_cast<uint4*>(y + out) = make_uint4(yo[0], yo[1], yo[2], yo[3]);
}

// Layout converters between byte-per-code rows (64 B per token, the reference's store) and packed
// 6-bit rows (48 B).  One thread converts a quarter row: 16 codes = 16 bytes <-> 12 bytes.
__global__ __launch_bounds__(256) void pack_codes6_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t n_quarters) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n_quarters) return;
    const uint4 v = *reinterpret_cast<const uint4*>(src + i * 16);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t x[4];
#pragma unroll
    for (int c = 0; c < 4; c++) x[c] = (w[c] & 0x3Fu) | ((w[c] >> 2) & 0xFC0u) | ((w[c] >> 4) & 0x3F000u) | ((w[c] >> 6) & 0xFC0000u);
    uint32_t* o = reinterpret_cast<uint32_t*>(dst + i * 12);
    o[0] = x[0] | (x[1] << 24);
    o[1] = (x[1] >> 8) | (x[2] << 16);
    o[2] = (x[2] >> 16) | (x[3] << 8);
}

__global__ __launch_bounds__(256) void unpack_codes6_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t n_quarters) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n_quarters) return;
    const uint32_t* p = reinterpret_cast<const uint32_t*>(src + i * 12);
    const uint32_t a = p[0], b = p[1], c = p[2];
    const uint32_t x[4] = {a & 0xFFFFFFu, (a >> 24) | ((b & 0xFFFFu) << 8), (b >> 16) | ((c & 0xFFu) << 16), c >> 8};
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) w[k] = (x[k] & 0x3Fu) | ((x[k] << 2) & 0x3F00u) | ((x[k] << 4) & 0x3F0000u) | ((x[k] << 6) & 0x3F000000u);
    *reinterpret_cast<uint4*>(dst + i * 16) = make_uint4(w[0], w[1], w[2], w[3]);
}

int launch_convert_codes6(const uint8_t* src, uint8_t* dst, size_t n_rows, bool pack, hipStream_t st) {
    const size_t nq = n_rows * 4;
    const unsigned blocks = static_cast<unsigned>((nq + 255) / 256);
    if (pack) hipLaunchKernelGGL(pack_codes6_kernel, dim3(blocks), dim3(256), 0, st, src, dst, nq);
    else hipLaunchKernelGGL(unpack_codes6_kernel, dim3(blocks), dim3(256), 0, st, src, dst, nq);
    return static_cast<int>(hipGetLastError());
}

int launch_rope_append(const void* q_lin, const void* k_lin, const void* v_lin, const void* cos_tab, const void* sin_tab,
                       const int64_t* pos, void* q_out, void* k_dst, int64_t k_rows, const int64_t* k_row,
                       void* v_dst, int64_t v_rows, const int64_t* v_row, int B, int N, int Nk, int64_t max_pos, int dtype,
                       int64_t q_stride, int64_t kv_stride, hipStream_t st) {
    dim3 grid(N + 2 * Nk, B), block(kWave);
#define PQ_RA(T)                                                                                                     \
    hipLaunchKernelGGL(rope_append_kernel<T>, grid, block, 0, st, (const uint16_t*)q_lin, (const uint16_t*)k_lin,    \
                       (const uint16_t*)v_lin, (const uint16_t*)cos_tab, (const uint16_t*)sin_tab, pos,              \
                       (uint16_t*)q_out, (uint16_t*)k_dst, k_rows, k_row, (uint16_t*)v_dst, v_rows, v_row, N, Nk, max_pos,   \
                       q_stride, kv_stride)
    if (dtype == 0) PQ_RA(F16); else PQ_RA(BF16);
#undef PQ_RA
    return static_cast<int>(hipGetLastError());
}

int launch_rope_qk(const void* q_lin, int64_t q_stride, const void* k_lin, int64_t k_stride, const void* cos_t,
                   const void* sin_t, int64_t cs_batch_stride, void* q_out, void* k_out, int B, int L, int N, int Nk,
                   int dtype, hipStream_t st) {
    dim3 grid(static_cast<unsigned>(static_cast<size_t>(B) * L)), block(256);
#define PQ_RQ(T)                                                                                                     \
    hipLaunchKernelGGL(rope_qk_kernel<T>, grid, block, 0, st, (const uint16_t*)q_lin, q_stride, (const uint16_t*)k_lin, \
                       k_stride, (const uint16_t*)cos_t, (const uint16_t*)sin_t, cs_batch_stride, (uint16_t*)q_out,   \
                       (uint16_t*)k_out, L, N, Nk)
    if (dtype == 0) PQ_RQ(F16); else PQ_RQ(BF16);
#undef PQ_RQ
    return static_cast<int>(hipGetLastError());
}

int launch_rmsnorm(const void* x, const void* res, const void* w, void* y, void* sum_out, int rows, int hidden, float eps,
                   int dtype, hipStream_t st) {
    if (dtype == 0)
        hipLaunchKernelGGL(rmsnorm_kernel<F16>, dim3(rows), dim3(256), 0, st, (const uint16_t*)x, (const uint16_t*)res,
                           (const uint16_t*)w, (uint16_t*)y, (uint16_t*)sum_out, hidden, eps);
    else
        hipLaunchKernelGGL(rmsnorm_kernel<BF16>, dim3(rows), dim3(256), 0, st, (const uint16_t*)x, (const uint16_t*)res,
                           (const uint16_t*)w, (uint16_t*)y, (uint16_t*)sum_out, hidden, eps);
    return static_cast<int>(hipGetLastError());
}

int launch_silu_mul(const void* gate, const void* up, void* y, int rows, int cols, int64_t in_stride, int dtype, hipStream_t st) {
    dim3 grid(static_cast<unsigned>((cols / 8 + 255) / 256), static_cast<unsigned>(rows)), block(256);
    if (dtype == 0)
        hipLaunchKernelGGL(silu_mul_kernel<F16>, grid, block, 0, st, (const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)y, cols, in_stride);
    else
        hipLaunchKernelGGL(silu_mul_kernel<BF16>, grid, block, 0, st, (const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)y, cols, in_stride);
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
