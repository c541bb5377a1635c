// Linear layers of the decode step: y[M, N] = x[M, K] . W[N, K]^T (+ bias) with M <= 16 rows
// (one new token per sequence), the q/k/v, o and MLP projections around the attention call
// (models/modeling_llama_polar.py:47-52, :131 and the decoder layer's MLP, :456-486).
//
// At M <= 16 the product is a stream of the weight matrix through HBM, 2*M flops per weight
// byte: the kernel is laid out for the stream, not for the matrix cores.  A workgroup owns
// 16 output columns (16 rows of W) and splits K over its KSPLIT wavefronts; each wavefront
// keeps two stages of kStage 16-byte loads per lane in flight (ping-pong) and feeds them to
// v_mfma_f32_16x16x32 with the W rows as the A operand and x (rows >= M unused) as the B operand:
// lane l holds W[n0 + l % 16][k + 8 * (l / 16) .. + 8) and x[l % 16][same k], so a 16-byte
// load per lane is one MFMA operand and a wavefront load covers 16 rows x 64 contiguous
// bytes.  The KSPLIT partial 16x16 tiles are added in a fixed order through LDS, so results
// do not depend on scheduling.  x (at most 16 x K) is re-read by every workgroup from L2.
//
// GATED: two weight matrices share the x operand and the epilogue applies
// silu(gate) * up with the eager modules' roundings (gate, up and silu(gate) each rounded
// to the activation dtype), which saves the [M, 2 * N] round trip and one launch.
#include "pq_device.h"
#include "pq_internal.h"

namespace pq {

typedef float floatx4_l __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_l __attribute__((ext_vector_type(4)));
typedef _Float16 half8_l __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_l __attribute__((ext_vector_type(8)));

template <typename T> __device__ __forceinline__ floatx4_l mfma32(u32x4_l a, u32x4_l b, floatx4_l c);
template <> __device__ __forceinline__ floatx4_l mfma32<F16>(u32x4_l a, u32x4_l b, floatx4_l c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_l, a), __builtin_bit_cast(half8_l, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ floatx4_l mfma32<BF16>(u32x4_l a, u32x4_l b, floatx4_l c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_l, a), __builtin_bit_cast(bf16x8_l, b), c, 0, 0, 0);
}

template <typename T>
__device__ __forceinline__ float rnd_l(float f) { return lo2f<T>(f2lo<T>(f)); }

template <bool GATED, int kStage>
struct StageT {
    u32x4_l w[kStage], x[kStage], u[GATED ? kStage : 1];
};

template <typename T, int KSPLIT, bool GATED, int kStage>
__global__ __launch_bounds__(kWave * KSPLIT) void small_m_linear_kernel(
    const uint16_t* __restrict__ x, int64_t x_stride, const uint16_t* __restrict__ w, const uint16_t* __restrict__ w_up,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, int64_t y_stride, int M, int K) {
    __shared__ float part[KSPLIT][GATED ? 2 : 1][4][kWave];
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int klen = K / KSPLIT, steps = klen / 32;
    const int m = r < M ? r : 0;                           // tile columns >= M repeat row 0 and are never stored
    const size_t koff = static_cast<size_t>(wv) * klen + 8 * g;
    const uint16_t* wp = w + static_cast<size_t>(n0 + r) * K + koff;
    const uint16_t* up = GATED ? w_up + static_cast<size_t>(n0 + r) * K + koff : nullptr;
    const uint16_t* xp = x + static_cast<size_t>(m) * x_stride + koff;

    floatx4_l acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}}, acu[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    // No branch may sit between a stage's loads and the MFMAs of the other stage: at a join the
    // compiler has to wait for every outstanding load, which would serialize the two stages.  So
    // whole stages run in a branch-free ping-pong loop, and only the tail is predicated.
    auto load = [&](StageT<GATED, kStage>& st, int s0) {
        static_for<kStage>([&](auto U) {
            constexpr int u = decltype(U)::value;
            st.w[u] = *reinterpret_cast<const u32x4_l*>(wp + (s0 + u) * 32);
            if constexpr (GATED) st.u[u] = *reinterpret_cast<const u32x4_l*>(up + (s0 + u) * 32);
            st.x[u] = *reinterpret_cast<const u32x4_l*>(xp + (s0 + u) * 32);
        });
    };
    auto compute = [&](const StageT<GATED, kStage>& st) {
        static_for<kStage>([&](auto U) {
            constexpr int u = decltype(U)::value;
            acc[u & 1] = mfma32<T>(st.w[u], st.x[u], acc[u & 1]);
            if constexpr (GATED) acu[u & 1] = mfma32<T>(st.u[u], st.x[u], acu[u & 1]);
        });
    };
    const int full = steps / kStage;          // whole stages
    if (full > 0) {
        StageT<GATED, kStage> sa, sb;
        load(sa, 0);
        int st = 0;
        while (st + 2 < full) {
            load(sb, (st + 1) * kStage);
            compute(sa);
            load(sa, (st + 2) * kStage);
            compute(sb);
            st += 2;
        }
        if (full - st == 2) {
            load(sb, (st + 1) * kStage);
            compute(sa);
            compute(sb);
        } else {
            compute(sa);
        }
    }
    for (int s1 = full * kStage; s1 < steps; s1++) {      // fewer than kStage steps left
        const u32x4_l wv1 = *reinterpret_cast<const u32x4_l*>(wp + s1 * 32);
        const u32x4_l xv1 = *reinterpret_cast<const u32x4_l*>(xp + s1 * 32);
        acc[0] = mfma32<T>(wv1, xv1, acc[0]);
        if constexpr (GATED) acu[0] = mfma32<T>(*reinterpret_cast<const u32x4_l*>(up + s1 * 32), xv1, acu[0]);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        part[wv][0][i][lane] = acc[0][i] + acc[1][i];
        if constexpr (GATED) part[wv][1][i][lane] = acu[0][i] + acu[1][i];
    }
    __syncthreads();
    if (wv != 0 || r >= M) return;
    // the MFMA result layout: lane (r, g) holds tile rows 4g + i (i < 4) of tile column r = outputs y[r][n0 + 4g + i]
    uint16_t out[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float s = part[0][0][i][lane];
#pragma unroll
        for (int k = 1; k < KSPLIT; k++) s += part[k][0][i][lane];
        if constexpr (GATED) {
            float t = part[0][1][i][lane];
#pragma unroll
            for (int k = 1; k < KSPLIT; k++) t += part[k][1][i][lane];
            const float gv = rnd_l<T>(s), uv = rnd_l<T>(t);
            const float a = rnd_l<T>(gv / (1.0f + __expf(-gv)));
            out[i] = f2lo<T>(a * uv);
        } else {
            if (bias) s += lo2f<T>(bias[n0 + 4 * g + i]);
            out[i] = f2lo<T>(s);
        }
    }
    *reinterpret_cast<uint2*>(y + static_cast<size_t>(r) * y_stride + n0 + 4 * g) =
        make_uint2(static_cast<uint32_t>(out[0]) | (static_cast<uint32_t>(out[1]) << 16),
                   static_cast<uint32_t>(out[2]) | (static_cast<uint32_t>(out[3]) << 16));
}

// Four wavefronts per workgroup and short stages measured best at the decode shapes of Llama-3-8B
// (K-split 4 / 8 / 16 and stages of 2 / 4 / 8 loads were swept); K / KSPLIT must stay a whole
// number of 32-wide steps.
int launch_small_m_linear(const void* x, int64_t x_stride, const void* w, const void* w_up, const void* bias, void* y,
                          int64_t y_stride, int M, int N, int K, int dtype, hipStream_t st) {
    int ks = 4;
    while (ks > 1 && (K % (32 * ks)) != 0) ks >>= 1;
    dim3 grid(N / 16), block(kWave * ks);
#define PQ_LAUNCH_L(T, KS, G, S)                                                                                     \
    hipLaunchKernelGGL((small_m_linear_kernel<T, KS, G, S>), grid, block, 0, st, (const uint16_t*)x, x_stride,     \
                       (const uint16_t*)w, (const uint16_t*)w_up, (const uint16_t*)bias, (uint16_t*)y, y_stride, M, K)
#define PQ_LAUNCH_LK(T, G, S)                                                                                        \
    do {                                                                                                             \
        if (ks == 4) PQ_LAUNCH_L(T, 4, G, S);                                                                        \
        else if (ks == 2) PQ_LAUNCH_L(T, 2, G, S);                                                                   \
        else PQ_LAUNCH_L(T, 1, G, S);                                                                                \
    } while (0)
    const bool gated = w_up != nullptr;
    if (dtype == 0) { if (gated) PQ_LAUNCH_LK(F16, true, 2); else PQ_LAUNCH_LK(F16, false, 4); }
    else            { if (gated) PQ_LAUNCH_LK(BF16, true, 2); else PQ_LAUNCH_LK(BF16, false, 4); }
#undef PQ_LAUNCH_LK
#undef PQ_LAUNCH_L
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
