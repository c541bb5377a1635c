// The bench-only library (libpolarquant_bench.so, declared in include/polarquant_bench.h): kernels that
// measure what the memory system delivers, for bench.py and the profiles.  Not part of the product
// library and not needed by any caller of the decode path.
//
// Measurement aid: a plain streaming read of a device buffer, the access pattern every kernel of
// this library is compared against.  Each wavefront owns one contiguous slice and keeps 16 loads
// of 16 bytes per lane in flight (16 KiB per wavefront), with the same non-temporal buffer loads
// the decode kernels use for their code and value streams.  What it reaches on a given GPU is
// the bandwidth a read-once kernel can be delivered there; the published HBM peak is not.
#include "../../include/polarquant_bench.h"
#include "pq_device.h"

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

// Measurement aid: the HBM access of attn_kernel (half-precision values, unpacked codes) without its arithmetic.
// Same grid (one wavefront per (plane, slice), plane index fastest), same buffer loads in the same order and
// depth: per 64-token tile four 16-byte code loads per lane (lane == token, 64-byte rows) one tile ahead, and
// sixteen 16-byte value loads (instruction (tb, i): lane (g, n) reads dims 8n..8n+7 of token 16 tb + 4 g + i)
// one tile ahead; the data is only XOR-ed together.  Its duration is what that access pattern costs on a given
// GPU; the kernel's own duration above it is what the table, score and softmax work adds.
__global__ __launch_bounds__(kWave) void attn_load_replica_kernel(const uint8_t* __restrict__ codes,
                                                                   const uint16_t* __restrict__ v, int planes,
                                                                   uint32_t code_plane_tokens, uint32_t v_plane_tokens,
                                                                   uint32_t tokens_per_slice, uint32_t* __restrict__ sink) {
    __shared__ char table_space[16384];              // the kernel's table: the same bound on resident workgroups
    const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
    const int plane = blockIdx.x % planes, slice = blockIdx.x / planes;
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(codes) + static_cast<size_t>(plane) * code_plane_tokens * 64, 0,
        static_cast<int>(code_plane_tokens * 64u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(v) + static_cast<size_t>(plane) * v_plane_tokens * kHeadDim, 0,
        static_cast<int>(v_plane_tokens * (kHeadDim * 2u)), 0x00020000);
    const int voff_v = g * 1024 + n * 16, voff_c = lane * 64;
    const uint32_t t0 = static_cast<uint32_t>(slice) * tokens_per_slice, n_tiles = tokens_per_slice / kWave;
    u32x4_s vv[2][16], cc[4];
    u32x4_s acc = {0, 0, 0, 0};
    auto load_v = [&](u32x4_s (&d)[16], uint32_t tok) {
#pragma unroll
        for (int tb = 0; tb < 4; tb++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[tb * 4 + i] = __builtin_amdgcn_raw_buffer_load_b128(rv, voff_v, static_cast<int>(tok * 256u + (16 * tb + i) * 256u), 2);
    };
    auto load_c = [&](uint32_t tok) {
#pragma unroll
        for (int i = 0; i < 4; i++) cc[i] = __builtin_amdgcn_raw_buffer_load_b128(rc, voff_c, static_cast<int>(tok * 64u + 16u * i), 2);
    };
    load_c(t0);
    load_v(vv[0], t0);
    for (uint32_t t = 0; t < n_tiles; t += 2) {      // tiles past the end of the slice read the next slice's rows or zeros
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t tok = t0 + (t + h) * kWave;
            load_v(vv[h ^ 1], tok + kWave);
            acc ^= cc[0] ^ cc[1] ^ cc[2] ^ cc[3];
            load_c(tok + kWave);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < 16; k++) acc ^= vv[h][k];
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) { sink[0] = acc.x; table_space[lane] = 1; }
}

int launch_attn_load_replica(const void* codes, const void* v, int planes, uint32_t code_plane_tokens,
                             uint32_t v_plane_tokens, uint32_t tokens_per_slice, int n_slices, uint32_t* sink, hipStream_t st) {
    hipLaunchKernelGGL(attn_load_replica_kernel, dim3(static_cast<unsigned>(planes) * n_slices), dim3(kWave), 0, st,
                       static_cast<const uint8_t*>(codes), static_cast<const uint16_t*>(v), planes, code_plane_tokens,
                       v_plane_tokens, tokens_per_slice, sink);
    return static_cast<int>(hipGetLastError());
}

int launch_stream_read(const void* src, size_t bytes_per_wave, int n_waves, uint32_t* sink, hipStream_t st) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(n_waves), dim3(kWave), 0, st, static_cast<const uint8_t*>(src),
                       bytes_per_wave, sink);
    return static_cast<int>(hipGetLastError());
}

}  // namespace pq

namespace {
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
}  // namespace

extern "C" {

size_t pq_stream_read(const void* src, size_t bytes, int n_wavefronts, uint32_t* sink, void* stream) {
    if (!src || !sink || n_wavefronts <= 0 || n_wavefronts > (1 << 20) || !aligned(src, 16) || !aligned(sink, 4)) return 0;
    const size_t chunk = 16 * 1024;                       // what one wavefront requests per trip
    size_t per_wave = bytes / static_cast<size_t>(n_wavefronts) / chunk * chunk;
    if (per_wave > (size_t{1} << 31) - chunk) per_wave = ((size_t{1} << 31) - chunk) / chunk * chunk;
    if (per_wave == 0) return 0;
    if (pq::launch_stream_read(src, per_wave, n_wavefronts, sink, static_cast<hipStream_t>(stream)) != 0) return 0;
    return per_wave * static_cast<size_t>(n_wavefronts);
}

size_t pq_attn_load_replica(const uint8_t* codes, const void* v, int planes, int64_t code_plane_tokens,
                            int64_t v_plane_tokens, int64_t tokens, int n_slices, uint32_t* sink, void* stream) {
    if (!codes || !v || !sink || !aligned(codes, 16) || !aligned(v, 16) || !aligned(sink, 4)) return 0;
    if (planes <= 0 || n_slices <= 0 || static_cast<long long>(planes) * n_slices > (1ll << 24)) return 0;
    if (tokens <= 0 || tokens > code_plane_tokens || tokens > v_plane_tokens) return 0;
    if (v_plane_tokens > ((int64_t{1} << 31) - 1) / 256 || code_plane_tokens > ((int64_t{1} << 31) - 1) / 64) return 0;
    const int64_t per_slice = tokens / n_slices / 128 * 128;          // whole pairs of 64-token tiles
    if (per_slice == 0) return 0;
    if (pq::launch_attn_load_replica(codes, v, planes, static_cast<uint32_t>(code_plane_tokens),
                                     static_cast<uint32_t>(v_plane_tokens), static_cast<uint32_t>(per_slice), n_slices, sink,
                                     static_cast<hipStream_t>(stream)) != 0)
        return 0;
    return static_cast<size_t>(per_slice) * n_slices * static_cast<size_t>(planes) * 320;
}

}  // extern "C"
