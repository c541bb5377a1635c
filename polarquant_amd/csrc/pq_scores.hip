// Quantized-key decode scores: the HIP counterpart of the reference's Triton
// score kernel (models/kernel4group.py:14-80).  One wavefront per
// (batch, KV head, 128-token group); output fp32 [B,N,1,Nb*128].
#include "pq_device.h"
#include "pq_internal.h"

namespace pq {

template <typename T, int TB, int REPP, bool PK6>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(Lut<TB, REPP>::BYTES > 40960 ? 1 : 2, 4))) void scores_kernel(const uint16_t* __restrict__ q, const uint8_t* __restrict__ codes,
                                                       const uint16_t* __restrict__ rscale, const uint16_t* __restrict__ rmn,
                                                       const uint16_t* __restrict__ tscale, const uint16_t* __restrict__ tmn,
                                                       float* __restrict__ out, int N, int Nk, int Nb, int rep, int rep_stride) {
    // rep_stride: query heads from one KV head to the next (rep, unless the heads go in two launches: launch_tb)
    using L = Lut<TB, REPP>;
    __shared__ __attribute__((aligned(16))) char lut_mem[L::BYTES];
    const uint32_t lut = lds_addr(lut_mem);
    const int lane = threadIdx.x;
    const int grp = blockIdx.x;
    const int kvh = blockIdx.y, b = blockIdx.z;      // (grid dimensions of their own: no division ahead of the first loads)
    const int bh = b * Nk + kvh;
    const size_t gidx = static_cast<size_t>(bh) * Nb + grp;

    // token codes of tile 0 and 1 (issued first: longest latency); rows of 64 bytes, or 48 when the
    // 6-bit codes are stored packed
    constexpr int kRowB = PK6 ? kPackedRowBytes : kPairs, kRowLoads = kRowB / 16;
    const uint4* crow = reinterpret_cast<const uint4*>(codes + gidx * (kGroup * kRowB));
    uint4 cw[2][kRowLoads];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < kRowLoads; i++) cw[t][i] = crow[(t * kWave + lane) * kRowLoads + i];

    float qx[REPP], qy[REPP];
    const uint16_t* qb = q + (static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep_stride) * kHeadDim;
#pragma unroll
    for (int j = 0; j < REPP; j++) {
        const bool ok = j < rep;
        qx[j] = ok ? lo2f<T>(qb[j * kHeadDim + lane]) : 0.0f;
        qy[j] = ok ? lo2f<T>(qb[j * kHeadDim + kPairs + lane]) : 0.0f;
    }
    const size_t mi = gidx * kPairs + lane;
    const float cdv = build_lut<T, TB, REPP>(lut, lane, qx, qy, rscale[mi], rmn[mi], tscale[mi], tmn[mi]);
    float cds[kPairs];
    broadcast_cd(cdv, cds);
    __syncthreads();

    float* ob = out + (static_cast<size_t>(b) * N + static_cast<size_t>(kvh) * rep_stride) * (static_cast<size_t>(Nb) * kGroup) +
                static_cast<size_t>(grp) * kGroup + lane;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        uint32_t cwords[16];
        if constexpr (PK6) {
            uint32_t pk[12];
#pragma unroll
            for (int i = 0; i < 3; i++) {
                pk[4 * i + 0] = cw[t][i].x; pk[4 * i + 1] = cw[t][i].y;
                pk[4 * i + 2] = cw[t][i].z; pk[4 * i + 3] = cw[t][i].w;
            }
            unpack6(pk, cwords);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                cwords[4 * i + 0] = cw[t][i].x; cwords[4 * i + 1] = cw[t][i].y;
                cwords[4 * i + 2] = cw[t][i].z; cwords[4 * i + 3] = cw[t][i].w;
            }
        }
        float acc[REPP];
#pragma unroll
        for (int j = 0; j < REPP; j++) acc[j] = 0.0f;
        score_token<TB, REPP>(lut, cwords, cds, acc);
#pragma unroll
        for (int j = 0; j < REPP; j++)
            if (j < rep) ob[static_cast<size_t>(j) * Nb * kGroup + t * kWave] = acc[j];
    }
}

// One launch for `rep` (<= 8; <= 4 with 128 angle bins) query heads of every KV head, the first of them at q / out.
template <typename T, int TB>
static int launch_tb_heads(const uint16_t* q, const uint8_t* codes, const void* rscale, const void* rmn, const void* tscale,
                           const void* tmn, float* out, int N, int Nk, int Nb, int rep, int rep_stride, bool packed6,
                           dim3 grid, hipStream_t st) {
    const dim3 block(kWave);
#define PQ_LAUNCH_P(REPP, PK6)                                                                                  \
    hipLaunchKernelGGL((scores_kernel<T, TB, REPP, PK6>), grid, block, 0, st, q, codes,                         \
                       (const uint16_t*)rscale, (const uint16_t*)rmn, (const uint16_t*)tscale,                  \
                       (const uint16_t*)tmn, out, N, Nk, Nb, rep, rep_stride)
    // packed 6-bit code rows exist for tbits == 3 only
#define PQ_LAUNCH(REPP)                                                                                         \
    do {                                                                                                        \
        if constexpr (TB == 3) {                                                                                \
            if (packed6) PQ_LAUNCH_P(REPP, true);                                                               \
            else PQ_LAUNCH_P(REPP, false);                                                                      \
        } else {                                                                                                \
            PQ_LAUNCH_P(REPP, false);                                                                           \
        }                                                                                                       \
    } while (0)
    switch (rep) {
        case 1: PQ_LAUNCH(1); break;
        case 2: PQ_LAUNCH(2); break;
        case 3: PQ_LAUNCH(3); break;
        case 4: PQ_LAUNCH(4); break;
        default:
            // (the table of more than four heads does not exist for 128 angle bins: launch_tb sends those in two shares)
            if constexpr (TB <= 6) {
                switch (rep) {
                    case 5: PQ_LAUNCH(5); break;
                    case 6: PQ_LAUNCH(6); break;
                    case 7: PQ_LAUNCH(7); break;
                    default: PQ_LAUNCH(8); break;
                }
            } else {
                return static_cast<int>(hipErrorInvalidValue);
            }
            break;
    }
#undef PQ_LAUNCH
#undef PQ_LAUNCH_P
    return static_cast<int>(hipGetLastError());
}

template <typename T, int TB>
static int launch_tb(const void* q, const uint8_t* codes, const void* rscale, const void* rmn, const void* tscale,
                     const void* tmn, float* out, int B, int N, int Nk, int Nb, bool packed6, hipStream_t st) {
    const int rep_stride = N / Nk;
    int rep = rep_stride;
    const uint16_t* qp = static_cast<const uint16_t*>(q);
    float* op = out;
    const dim3 grid(Nb, Nk, B);
    if constexpr (TB == 7) {
        // 128 angle bins: a table holds four query heads at most (128 KiB); more heads per KV head go in two
        // launches, heads [0, 4) here and [4, rep) below
        if (rep_stride > kMaxHeadsWidestTable) {
            if (int rc = launch_tb_heads<T, TB>(qp, codes, rscale, rmn, tscale, tmn, op, N, Nk, Nb, kMaxHeadsWidestTable, rep_stride, packed6, grid, st))
                return rc;
            qp += static_cast<size_t>(kMaxHeadsWidestTable) * kHeadDim;
            op += static_cast<size_t>(kMaxHeadsWidestTable) * Nb * kGroup;
            rep = rep_stride - kMaxHeadsWidestTable;
        }
    }
    return launch_tb_heads<T, TB>(qp, codes, rscale, rmn, tscale, tmn, op, N, Nk, Nb, rep, rep_stride, packed6, grid, st);
}

template <typename T>
static int launch_t(const void* q, const uint8_t* codes, const void* rscale, const void* rmn, const void* tscale,
                    const void* tmn, float* out, int B, int N, int Nk, int Nb, int tbits, bool packed6, hipStream_t st) {
    switch (tbits) {
        case 1: return launch_tb<T, 1>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
        case 2: return launch_tb<T, 2>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
        case 3: return launch_tb<T, 3>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
        case 4: return launch_tb<T, 4>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
        case 5: return launch_tb<T, 5>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
        case 6: return launch_tb<T, 6>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
        default: return launch_tb<T, 7>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, packed6, st);
    }
}

int launch_scores(const void* q, const uint8_t* codes, const void* rscale, const void* rmn, const void* tscale,
                  const void* tmn, float* out, int B, int N, int Nk, int Nb, int tbits, int dtype, bool packed6, hipStream_t st) {
    return dtype == 0 ? launch_t<F16>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, tbits, packed6, st)
                      : launch_t<BF16>(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, tbits, packed6, st);
}

}  // namespace pq
