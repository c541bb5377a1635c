// Measurement aid: a plain streaming read of a device buffer, the access pattern every kernel of
// this library is compared against.  Each wavefront owns one contiguous slice and keeps 16 loads
// of 16 bytes per lane in flight (16 KiB per wavefront), with the same non-temporal buffer loads
// the decode kernels use for their code and value streams.  What it reaches on a given GPU is
// the bandwidth a read-once kernel can be delivered there; the published HBM peak is not.
#include "pq_device.h"
#include "pq_internal.h"

namespace pq {

typedef uint32_t u32x4_s __attribute__((ext_vector_type(4)));
constexpr int kStreamDepth = 16;

__global__ __launch_bounds__(kWave) void stream_read_kernel(const uint8_t* __restrict__ src, size_t bytes_per_wave,
                                                            uint32_t* __restrict__ sink) {
    const uint8_t* base = src + static_cast<size_t>(blockIdx.x) * bytes_per_wave;
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(base), 0,
                                                                       static_cast<int>(bytes_per_wave), 0x00020000);
    const int voff = static_cast<int>(threadIdx.x) * 16;
    u32x4_s acc = {0, 0, 0, 0};
    for (size_t off = 0; off < bytes_per_wave; off += kStreamDepth * 1024) {
        u32x4_s v[kStreamDepth];
#pragma unroll
        for (int i = 0; i < kStreamDepth; i++)
            v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, voff, static_cast<int>(off) + i * 1024, 2);
#pragma unroll
        for (int i = 0; i < kStreamDepth; i++) acc ^= v[i];
    }
    // keeps the loads alive; the comparison practically never holds, so nothing is written
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;
}

int launch_stream_read(const void* src, size_t bytes_per_wave, int n_waves, uint32_t* sink, hipStream_t st) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(n_waves), dim3(kWave), 0, st, static_cast<const uint8_t*>(src),
                       bytes_per_wave, sink);
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq
