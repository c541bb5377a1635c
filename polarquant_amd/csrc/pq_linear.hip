// Linear layers of the decode step: y[M, N] = x[M, K] . W[N, K]^T (+ bias) with M <= 16 rows
// (one new token per sequence), the q/k/v, o and MLP projections around the attention call
// (models/modeling_llama_polar.py:47-52, :131 and the decoder layer's MLP, :456-486).
//
// At M <= 16 the product is a stream of the weight matrix through HBM, 2*M flops per weight
// byte: the kernels are laid out for the stream, not for the matrix cores.  Two of them:
// small_m_linear_kernel (any M <= 16, described here) and small_m8_linear_kernel (M <= 8, further
// down: whole-line loads, half the x operand traffic).  A workgroup owns
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

// M <= 8: each 16 x 16 MFMA tile is used as two 8 x 8 tiles on its diagonal.  Tile rows 0-7 are 8 rows
// of W over the first 32 of a 64-wide k-step, tile rows 8-15 the SAME 8 rows over the second 32; tile
// columns 0-7 are the rows of x over the first 32, columns 8-15 over the second 32.  Then
// y[m][n] = C[n][m] + C[n + 8][m + 8] and the off-diagonal quarters are ignored.  No lane loads a
// duplicate row of x, a wavefront load of W covers 8 rows x 128 contiguous bytes (whole cache lines,
// which is what lets the weight stream carry the non-temporal hint: with half lines the hint drops a
// line before its second half is asked for), and the workgroup's 16 rows of W are two such tiles that
// share one x operand: per 64-wide step two W loads and one x load instead of four and four.
template <bool GATED, int kStage>
struct Stage8T {
    u32x4_l w[2][kStage], x[kStage], u[GATED ? 2 : 1][GATED ? kStage : 1];
};

template <typename T, int KSPLIT, bool GATED, int kStage>
__global__ __launch_bounds__(kWave * KSPLIT) void small_m8_linear_kernel(
    const uint16_t* __restrict__ x, int64_t x_stride, const uint16_t* __restrict__ w, const uint16_t* __restrict__ w_up,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, int64_t y_stride, int M, int K) {
    __shared__ float part[KSPLIT][GATED ? 4 : 2][4][kWave];
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int row = r & 7, chunk = (r >> 3) * 4 + g;       // W row inside an 8-row tile == x row; 16-byte piece of the step
    const int n0 = blockIdx.x * 16;
    const int klen = K / KSPLIT, steps = klen / 64;
    const int m = row < M ? row : 0;                       // tile columns >= M repeat row 0 and are never stored
    const size_t koff = static_cast<size_t>(wv) * klen + 8 * chunk;
    const uint16_t* wp = w + static_cast<size_t>(n0 + row) * K + koff;
    const uint16_t* up = GATED ? w_up + static_cast<size_t>(n0 + row) * K + koff : nullptr;
    const uint16_t* xp = x + static_cast<size_t>(m) * x_stride + koff;
    const size_t half_tile = static_cast<size_t>(8) * K;   // rows n0 + 8 .. n0 + 15

    floatx4_l acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}}, acu[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    auto ldw = [](const uint16_t* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4_l*>(p)); };
    auto load = [&](Stage8T<GATED, kStage>& st, int s0) {          // branch-free, see small_m_linear_kernel
        static_for<kStage>([&](auto U) {
            constexpr int u = decltype(U)::value;
            st.w[0][u] = ldw(wp + (s0 + u) * 64);
            st.w[1][u] = ldw(wp + half_tile + (s0 + u) * 64);
            if constexpr (GATED) {
                st.u[0][u] = ldw(up + (s0 + u) * 64);
                st.u[1][u] = ldw(up + half_tile + (s0 + u) * 64);
            }
            st.x[u] = *reinterpret_cast<const u32x4_l*>(xp + (s0 + u) * 64);
        });
    };
    auto compute = [&](const Stage8T<GATED, kStage>& st) {
        static_for<kStage>([&](auto U) {
            constexpr int u = decltype(U)::value;
            acc[0] = mfma32<T>(st.w[0][u], st.x[u], acc[0]);
            acc[1] = mfma32<T>(st.w[1][u], st.x[u], acc[1]);
            if constexpr (GATED) {
                acu[0] = mfma32<T>(st.u[0][u], st.x[u], acu[0]);
                acu[1] = mfma32<T>(st.u[1][u], st.x[u], acu[1]);
            }
        });
    };
    const int full = steps / kStage;
    if (full > 0) {
        Stage8T<GATED, kStage> sa, sb;
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
    for (int s1 = full * kStage; s1 < steps; s1++) {
        const u32x4_l xv1 = *reinterpret_cast<const u32x4_l*>(xp + s1 * 64);
        acc[0] = mfma32<T>(ldw(wp + s1 * 64), xv1, acc[0]);
        acc[1] = mfma32<T>(ldw(wp + half_tile + s1 * 64), xv1, acc[1]);
        if constexpr (GATED) {
            acu[0] = mfma32<T>(ldw(up + s1 * 64), xv1, acu[0]);
            acu[1] = mfma32<T>(ldw(up + half_tile + s1 * 64), xv1, acu[1]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        part[wv][0][i][lane] = acc[0][i];
        part[wv][1][i][lane] = acc[1][i];
        if constexpr (GATED) { part[wv][2][i][lane] = acu[0][i]; part[wv][3][i][lane] = acu[1][i]; }
    }
    __syncthreads();
    // lane (r < 8, g < 2) owns outputs y[r][n0 + 8h + 4g + i] (h: which 8-row tile), each the sum of the tile's
    // entry (row 4g + i, column r) and its diagonal partner (row + 8, column + 8), which lane + 40 holds
    if (wv != 0 || r >= 8 || r >= M || g >= 2) return;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        uint16_t out[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float s = 0.0f, t = 0.0f;
#pragma unroll
            for (int k = 0; k < KSPLIT; k++) {
                s += part[k][h][i][lane] + part[k][h][i][lane + 40];
                if constexpr (GATED) t += part[k][2 + h][i][lane] + part[k][2 + h][i][lane + 40];
            }
            if constexpr (GATED) {
                const float gv = rnd_l<T>(s), uv = rnd_l<T>(t);
                const float a = rnd_l<T>(gv / (1.0f + __expf(-gv)));
                out[i] = f2lo<T>(a * uv);
            } else {
                if (bias) s += lo2f<T>(bias[n0 + 8 * h + 4 * g + i]);
                out[i] = f2lo<T>(s);
            }
        }
        *reinterpret_cast<uint2*>(y + static_cast<size_t>(r) * y_stride + n0 + 8 * h + 4 * g) =
            make_uint2(static_cast<uint32_t>(out[0]) | (static_cast<uint32_t>(out[1]) << 16),
                       static_cast<uint32_t>(out[2]) | (static_cast<uint32_t>(out[3]) << 16));
    }
}

// The fused q|k|v projection of a decode step with RoPE and the cache appends in its epilogue (M <= 8):
// small_m8_linear_kernel's loop on the concatenated [(N + 2 Nk) * 128, K] weight, with the workgroup's two
// 8-row tiles 64 rows apart instead of adjacent, i.e. dims d..d+7 and d+64..d+71 of one head: the two halves of
// 8 rotation pairs.  The epilogue rounds both to the dtype (the projection's output), rotates q and k heads
// exactly as rope_append_kernel does (every product and sum rounded to the dtype), and writes the query to
// q_out [M, N, 128], the key to row *k_row of k_dst [M, Nk, k_rows, 128] and the value (unrotated) to row
// *v_row of v_dst [M, Nk, v_rows, 128].  One launch instead of two, no [M, (N + 2 Nk) * 128] round trip.
struct RopeAppendArgs {
    const uint16_t* cos_tab;
    const uint16_t* sin_tab;
    const int64_t* pos;
    uint16_t* q_out;
    uint16_t* k_dst;
    const int64_t* k_row;
    uint16_t* v_dst;
    const int64_t* v_row;
    int64_t max_pos, k_rows, v_rows;
    int N, Nk;
};

template <typename T, int KSPLIT, int kStage>
__global__ __launch_bounds__(kWave * KSPLIT) void qkv_rope_append_kernel(
    const uint16_t* __restrict__ x, int64_t x_stride, const uint16_t* __restrict__ w, const uint16_t* __restrict__ bias,
    int M, int K, RopeAppendArgs ra) {
    __shared__ float part[KSPLIT][2][4][kWave];
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int row = r & 7, chunk = (r >> 3) * 4 + g;
    const int head = blockIdx.x >> 3, c8 = (blockIdx.x & 7) * 8;       // dims c8 .. c8+7 and 64 + c8 .. of this head
    const int n0 = head * kHeadDim + c8;
    const int klen = K / KSPLIT, steps = klen / 64;
    const int m = row < M ? row : 0;
    const size_t koff = static_cast<size_t>(wv) * klen + 8 * chunk;
    const uint16_t* wp = w + static_cast<size_t>(n0 + row) * K + koff;
    const uint16_t* xp = x + static_cast<size_t>(m) * x_stride + koff;
    const size_t half_tile = static_cast<size_t>(kPairs) * K;           // rows n0 + 64 .. n0 + 71

    floatx4_l acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    auto ldw = [](const uint16_t* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4_l*>(p)); };
    auto load = [&](Stage8T<false, kStage>& st, int s0) {
        static_for<kStage>([&](auto U) {
            constexpr int u = decltype(U)::value;
            st.w[0][u] = ldw(wp + (s0 + u) * 64);
            st.w[1][u] = ldw(wp + half_tile + (s0 + u) * 64);
            st.x[u] = *reinterpret_cast<const u32x4_l*>(xp + (s0 + u) * 64);
        });
    };
    auto compute = [&](const Stage8T<false, kStage>& st) {
        static_for<kStage>([&](auto U) {
            constexpr int u = decltype(U)::value;
            acc[0] = mfma32<T>(st.w[0][u], st.x[u], acc[0]);
            acc[1] = mfma32<T>(st.w[1][u], st.x[u], acc[1]);
        });
    };
    const int full = steps / kStage;
    if (full > 0) {
        Stage8T<false, kStage> sa, sb;
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
    for (int s1 = full * kStage; s1 < steps; s1++) {
        const u32x4_l xv1 = *reinterpret_cast<const u32x4_l*>(xp + s1 * 64);
        acc[0] = mfma32<T>(ldw(wp + s1 * 64), xv1, acc[0]);
        acc[1] = mfma32<T>(ldw(wp + half_tile + s1 * 64), xv1, acc[1]);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        part[wv][0][i][lane] = acc[0][i];
        part[wv][1][i][lane] = acc[1][i];
    }
    __syncthreads();
    if (wv != 0 || r >= 8 || r >= M || g >= 2) return;
    // lane (r, g): batch row r, dims d = c8 + 4g + i (first half) and d + 64 (second half), i < 4
    const int N = ra.N, Nk = ra.Nk;
    const bool is_q = head < N, is_k = !is_q && head < N + Nk;
    int64_t p = *ra.pos;
    p = p < 0 ? 0 : (p >= ra.max_pos ? ra.max_pos - 1 : p);
    uint16_t o1[4], o2[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int k = 0; k < KSPLIT; k++) {
            s1 += part[k][0][i][lane] + part[k][0][i][lane + 40];
            s2 += part[k][1][i][lane] + part[k][1][i][lane + 40];
        }
        const int d = c8 + 4 * g + i;
        if (bias) { s1 += lo2f<T>(bias[n0 + 4 * g + i]); s2 += lo2f<T>(bias[n0 + kPairs + 4 * g + i]); }
        const float x1 = rnd_l<T>(s1), x2 = rnd_l<T>(s2);           // the projection's output in the dtype
        if (is_q || is_k) {
            const float c1 = lo2f<T>(ra.cos_tab[p * kHeadDim + d]), c2 = lo2f<T>(ra.cos_tab[p * kHeadDim + kPairs + d]);
            const float n1 = lo2f<T>(ra.sin_tab[p * kHeadDim + d]), n2 = lo2f<T>(ra.sin_tab[p * kHeadDim + kPairs + d]);
            // (x * cos) + (rotate_half(x) * sin), rotate_half(x) = cat(-x2, x1)
            o1[i] = f2lo<T>(rnd_l<T>(x1 * c1) + rnd_l<T>(-x2 * n1));
            o2[i] = f2lo<T>(rnd_l<T>(x2 * c2) + rnd_l<T>(x1 * n2));
        } else {
            o1[i] = f2lo<T>(x1);
            o2[i] = f2lo<T>(x2);
        }
    }
    uint16_t* dst;
    if (is_q) {
        dst = ra.q_out + (static_cast<size_t>(r) * N + head) * kHeadDim;
    } else if (is_k) {
        int64_t kr = *ra.k_row;
        kr = kr < 0 ? 0 : (kr >= ra.k_rows ? ra.k_rows - 1 : kr);
        dst = ra.k_dst + ((static_cast<size_t>(r) * Nk + (head - N)) * ra.k_rows + kr) * kHeadDim;
    } else {
        int64_t vr = *ra.v_row;
        vr = vr < 0 ? 0 : (vr >= ra.v_rows ? ra.v_rows - 1 : vr);
        dst = ra.v_dst + ((static_cast<size_t>(r) * Nk + (head - N - Nk)) * ra.v_rows + vr) * kHeadDim;
    }
    dst += c8 + 4 * g;
    *reinterpret_cast<uint2*>(dst) = make_uint2(static_cast<uint32_t>(o1[0]) | (static_cast<uint32_t>(o1[1]) << 16),
                                                static_cast<uint32_t>(o1[2]) | (static_cast<uint32_t>(o1[3]) << 16));
    *reinterpret_cast<uint2*>(dst + kPairs) = make_uint2(static_cast<uint32_t>(o2[0]) | (static_cast<uint32_t>(o2[1]) << 16),
                                                         static_cast<uint32_t>(o2[2]) | (static_cast<uint32_t>(o2[3]) << 16));
}

int launch_qkv_rope_append(const void* x, int64_t x_stride, const void* w, const void* bias, int M, int K, int dtype,
                           const void* cos_tab, const void* sin_tab, int64_t max_pos, const int64_t* pos, void* q_out,
                           void* k_dst, int64_t k_rows, const int64_t* k_row, void* v_dst, int64_t v_rows,
                           const int64_t* v_row, int N, int Nk, hipStream_t st) {
    RopeAppendArgs ra;
    ra.cos_tab = static_cast<const uint16_t*>(cos_tab); ra.sin_tab = static_cast<const uint16_t*>(sin_tab);
    ra.pos = pos; ra.q_out = static_cast<uint16_t*>(q_out); ra.k_dst = static_cast<uint16_t*>(k_dst); ra.k_row = k_row;
    ra.v_dst = static_cast<uint16_t*>(v_dst); ra.v_row = v_row; ra.max_pos = max_pos; ra.k_rows = k_rows; ra.v_rows = v_rows;
    ra.N = N; ra.Nk = Nk;
    // the split of K, and with it the order of the partial sums, is launch_small_m_linear's for M <= 8
    int ks = K >= 8192 ? 8 : 4;
    while (ks > 1 && (K % (64 * ks)) != 0) ks >>= 1;
    dim3 grid((N + 2 * Nk) * 8), block(kWave * ks);
#define PQ_LAUNCH_R(T, KS, S)                                                                                        \
    hipLaunchKernelGGL((qkv_rope_append_kernel<T, KS, S>), grid, block, 0, st, (const uint16_t*)x, x_stride,        \
                       (const uint16_t*)w, (const uint16_t*)bias, M, K, ra)
#define PQ_LAUNCH_RK(T)                                                                                              \
    do {                                                                                                             \
        if (ks == 8) PQ_LAUNCH_R(T, 8, 2);                                                                           \
        else if (ks == 4) PQ_LAUNCH_R(T, 4, 1);                                                                      \
        else if (ks == 2) PQ_LAUNCH_R(T, 2, 1);                                                                      \
        else PQ_LAUNCH_R(T, 1, 1);                                                                                   \
    } while (0)
    if (dtype == 0) PQ_LAUNCH_RK(F16);
    else PQ_LAUNCH_RK(BF16);
#undef PQ_LAUNCH_RK
#undef PQ_LAUNCH_R
    return static_cast<int>(hipGetLastError());
}

// Launch shapes measured at the decode shapes of Llama-3-8B (K-split 4 / 8 / 16 and stages of 1 / 2 / 4 / 8
// loads were swept): the 16-row kernel runs four wavefronts per workgroup with stages of 4 (2 when gated); the
// M <= 8 kernel four wavefronts with stages of 1, or eight with stages of 2 when K >= 8192 (down_proj).
// K / KSPLIT must stay a whole number of k-steps.
int launch_small_m_linear(const void* x, int64_t x_stride, const void* w, const void* w_up, const void* bias, void* y,
                          int64_t y_stride, int M, int N, int K, int dtype, hipStream_t st) {
    const bool gated = w_up != nullptr;
    const bool m8 = M <= 8 && (K % 64) == 0;
    const int kstep = m8 ? 64 : 32;
    int ks = (m8 && K >= 8192) ? 8 : 4;
    while (ks > 1 && (K % (kstep * ks)) != 0) ks >>= 1;
    dim3 grid(N / 16), block(kWave * ks);
#define PQ_LAUNCH_L(KERNEL, T, KS, G, S)                                                                             \
    hipLaunchKernelGGL((KERNEL<T, KS, G, S>), grid, block, 0, st, (const uint16_t*)x, x_stride,                      \
                       (const uint16_t*)w, (const uint16_t*)w_up, (const uint16_t*)bias, (uint16_t*)y, y_stride, M, K)
#define PQ_LAUNCH_M8(T, G)                                                                                           \
    do {                                                                                                             \
        if (ks == 8) PQ_LAUNCH_L(small_m8_linear_kernel, T, 8, G, 2);                                                \
        else if (ks == 4) PQ_LAUNCH_L(small_m8_linear_kernel, T, 4, G, 1);                                           \
        else if (ks == 2) PQ_LAUNCH_L(small_m8_linear_kernel, T, 2, G, 1);                                           \
        else PQ_LAUNCH_L(small_m8_linear_kernel, T, 1, G, 1);                                                        \
    } while (0)
#define PQ_LAUNCH_M16(T, G, S)                                                                                       \
    do {                                                                                                             \
        if (ks == 4) PQ_LAUNCH_L(small_m_linear_kernel, T, 4, G, S);                                                 \
        else if (ks == 2) PQ_LAUNCH_L(small_m_linear_kernel, T, 2, G, S);                                            \
        else PQ_LAUNCH_L(small_m_linear_kernel, T, 1, G, S);                                                         \
    } while (0)
#define PQ_LAUNCH_LM(T)                                                                                              \
    do {                                                                                                             \
        if (m8) { if (gated) PQ_LAUNCH_M8(T, true); else PQ_LAUNCH_M8(T, false); }                                   \
        else    { if (gated) PQ_LAUNCH_M16(T, true, 2); else PQ_LAUNCH_M16(T, false, 4); }                           \
    } while (0)
    if (dtype == 0) PQ_LAUNCH_LM(F16);
    else PQ_LAUNCH_LM(BF16);
#undef PQ_LAUNCH_LM
#undef PQ_LAUNCH_M16
#undef PQ_LAUNCH_M8
#undef PQ_LAUNCH_L
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
