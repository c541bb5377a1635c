// What the decode-attention kernel families share on the host side: the choice of the family and of the grid
// (launch_attn_partials), the merge kernel that follows every attention kernel, and the scratch of the entry point
// that allocates nothing.
//
// merge_kernel: grid B*N, 128 threads (one per output dim), or four / eight such
// groups that share the partials when there are 32 / 128 or more: combines the n_splits
// partials (m, l, acc[128]) of a query head and writes half words.
#include "pq_attn_device.h"
#include <mutex>

namespace pq {

template <typename T, int G>
__global__ __launch_bounds__(kHeadDim * G) void merge_kernel(const float* __restrict__ ws, int n_part, uint16_t* __restrict__ out) {
    // one block per query head, G groups of 128 threads: thread (grp, d) sums output dim d over
    // the grp-th share of the partials, and the G sums are added in a fixed order through LDS.
    // The partial headers (m, l) are fetched by one thread each, so that all loads of the block
    // are issued at once instead of one dependent load per partial.
    constexpr int NT = kHeadDim * G, NW = NT / kWave;
    __shared__ float wgt[1024];
    __shared__ float red[2][NW];
    __shared__ float part[G][kHeadDim];
    const int bn = blockIdx.x, tid = threadIdx.x, d = tid & (kHeadDim - 1), grp = tid / kHeadDim;
    const float* p = ws + static_cast<size_t>(bn) * n_part * kPartialFloats;
    float M = -INFINITY;
    for (int s = tid; s < n_part; s += NT) M = fmaxf(M, p[static_cast<size_t>(s) * kPartialFloats]);
    M = wave_max(M);
    if ((tid & (kWave - 1)) == 0) red[0][tid / kWave] = M;
    __syncthreads();
    M = red[0][0];
#pragma unroll
    for (int i = 1; i < NW; i++) M = fmaxf(M, red[0][i]);
    float num = 0.0f, den = 0.0f;
    for (int s0 = 0; s0 < n_part; s0 += 1024) {
        const int cnt = (n_part - s0) < 1024 ? (n_part - s0) : 1024;
        __syncthreads();
        for (int s = tid; s < cnt; s += NT) {
            const float m = p[static_cast<size_t>(s0 + s) * kPartialFloats];
            const float w = (m == -INFINITY) ? 0.0f : exp2_raw(m - M);
            wgt[s] = w;
            // an empty slice contributes nothing, whatever its sum word holds
            den = w != 0.0f ? __builtin_fmaf(w, p[static_cast<size_t>(s0 + s) * kPartialFloats + 1], den) : den;
        }
        __syncthreads();
        const float* pa = p + static_cast<size_t>(s0) * kPartialFloats + 4 + d;
        const int per = (cnt + G - 1) / G;
        int s = grp * per;
        const int se = (s + per) < cnt ? (s + per) : cnt;
        for (; s + 16 <= se; s += 16) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; u++) v[u] = pa[static_cast<size_t>(s + u) * kPartialFloats];
#pragma unroll
            for (int u = 0; u < 16; u++) num = wgt[s + u] != 0.0f ? __builtin_fmaf(wgt[s + u], v[u], num) : num;
        }
        for (; s + 8 <= se; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = pa[static_cast<size_t>(s + u) * kPartialFloats];
#pragma unroll
            for (int u = 0; u < 8; u++) num = wgt[s + u] != 0.0f ? __builtin_fmaf(wgt[s + u], v[u], num) : num;
        }
        for (; s < se; s++) {
            const float v = pa[static_cast<size_t>(s) * kPartialFloats];
            num = wgt[s] != 0.0f ? __builtin_fmaf(wgt[s], v, num) : num;
        }
    }
    den = wave_sum(den);
    __syncthreads();
    if ((tid & (kWave - 1)) == 0) red[1][tid / kWave] = den;
    if (G > 1) part[grp][d] = num;
    __syncthreads();
    if (grp != 0) return;
    den = red[1][0];
#pragma unroll
    for (int i = 1; i < NW; i++) den += red[1][i];
#pragma unroll
    for (int i = 1; i < G; i++) num += part[i][d];
    // nothing to attend to (den == 0) gives zeros; a NaN among the partials (a poisoned slice) must stay visible
    out[static_cast<size_t>(bn) * kHeadDim + d] = f2lo<T>(den > 0.0f ? num / den : (den == den ? 0.0f : den));
}

// Wavefront slots of the current device for the balanced kernel: one wavefront per SIMD (4 per
// compute unit), two for the 4-bit-value kernel with up to 4 query heads per KV head.
static int device_compute_units() {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static int cus[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

int launch_attn_partials(const AttnArgs& a, hipStream_t st) {
    const int rep = a.N / a.Nk;
    // half-precision values and at most 16 angle bins: a scorer / accumulator pair of wavefronts per slice or segment.
    // (4-bit values stay with one wavefront per slice, two per SIMD: a paired form of that kernel at four wavefronts per
    // SIMD was measured no faster -- the vector ALU's total work bounds it, however it is spread over wavefronts.)
    const bool pairs = attn_runs_pairs(a.v4_codes, a.single_wave, a.tbits);
    long long total = static_cast<long long>(a.n_splits) * a.B * a.Nk;
    if (a.balanced) {
        // as many wavefronts (or pairs) as the device holds at once, but never more than there are partial slots
        const long long slots = static_cast<long long>(device_compute_units()) * ((a.v4_codes && rep_pad(rep) <= 4) ? 8 : 4);
        total = slots < total ? slots : total;
    }
    if (pairs) return a.dtype == 0 ? launch_attn_pair_f16(a, static_cast<int>(total), st) : launch_attn_pair_bf16(a, static_cast<int>(total), st);
    auto one = [&](const AttnArgs& x) {
        return x.dtype == 0 ? launch_attn_one_f16(x, static_cast<int>(total), st) : launch_attn_one_bf16(x, static_cast<int>(total), st);
    };
    if (a.tbits <= 6 || rep <= kMaxHeadsWidestTable) return one(a);
    // 128 angle bins: the table of four query heads is 128 KiB, all the LDS a workgroup can have.  More heads per KV
    // head go in two launches, heads [0, 4) and [4, rep) of every KV head, each writing its own heads' partials.
    AttnArgs lo = a, hi = a;
    lo.rep_count = kMaxHeadsWidestTable;
    hi.rep_count = rep - kMaxHeadsWidestTable;
    hi.q = static_cast<const uint16_t*>(a.q) + static_cast<size_t>(kMaxHeadsWidestTable) * kHeadDim;
    hi.workspace = a.workspace + static_cast<size_t>(kMaxHeadsWidestTable) * a.n_splits * kPartialFloats;
    if (int rc = one(lo)) return rc;
    return one(hi);
}

constexpr int kMergeWideFrom = 32, kMergeWidestFrom = 128;

int launch_attn_merge(const float* ws, int B, int N, int n_splits, int dtype, void* out, hipStream_t st) {
    // many partials per head (a long context cut into many slices): four or eight groups of threads share them
    if (n_splits >= kMergeWidestFrom) {
        if (dtype == 0)
            hipLaunchKernelGGL((merge_kernel<F16, 8>), dim3(B * N), dim3(kHeadDim * 8), 0, st, ws, n_splits, (uint16_t*)out);
        else
            hipLaunchKernelGGL((merge_kernel<BF16, 8>), dim3(B * N), dim3(kHeadDim * 8), 0, st, ws, n_splits, (uint16_t*)out);
    } else if (n_splits >= kMergeWideFrom) {
        if (dtype == 0)
            hipLaunchKernelGGL((merge_kernel<F16, 4>), dim3(B * N), dim3(kHeadDim * 4), 0, st, ws, n_splits, (uint16_t*)out);
        else
            hipLaunchKernelGGL((merge_kernel<BF16, 4>), dim3(B * N), dim3(kHeadDim * 4), 0, st, ws, n_splits, (uint16_t*)out);
    } else if (dtype == 0) {
        hipLaunchKernelGGL((merge_kernel<F16, 1>), dim3(B * N), dim3(kHeadDim), 0, st, ws, n_splits, (uint16_t*)out);
    } else {
        hipLaunchKernelGGL((merge_kernel<BF16, 1>), dim3(B * N), dim3(kHeadDim), 0, st, ws, n_splits, (uint16_t*)out);
    }
    return static_cast<int>(hipGetLastError());
}

// ---- scratch of the entry point that allocates nothing (pq_decode_attn_static) -----------------
// The split partials of that entry point live in this file-scope device array instead of a caller's
// workspace.  Every GPU the library runs on holds its own copy at its own address until the process
// ends; the array's name is only a host-side handle, so the device address is asked for once per
// device (with that device current) and kept.
static __device__ __align__(256) float scratch[static_cast<size_t>(kStaticMaxPartials) * kPartialFloats];

int attn_static_scratch(float** ptr) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static float* per_device[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!p) return static_cast<int>(hipErrorInvalidSymbol);
        per_device[dev] = static_cast<float*>(p);
    }
    *ptr = per_device[dev];
    return 0;
}

}  // namespace pq
