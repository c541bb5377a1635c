/* polarquant_bench.h — C ABI of libpolarquant_bench.so, the bench-only companion of libpolarquant_hip.so.
 *
 * Measurement aids for bench.py and the profiles: kernels that show what the GPU's memory system
 * delivers to a read-once access pattern.  None of them replaces a reference interface and no caller
 * of the decode path needs this library.  Conventions as in polarquant.h (device pointers, a
 * hipStream_t passed as void*, asynchronous, no allocation).
 */
#ifndef POLARQUANT_BENCH_H
#define POLARQUANT_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid (no reference counterpart): a plain streaming read of `bytes` bytes at `src` by
 * `n_wavefronts` wavefronts, each reading one contiguous slice with 16 KiB in flight, with the
 * non-temporal loads the decode kernels use.  Time it to learn what a read-once kernel can be
 * delivered on the GPU at hand.  Returns the number of bytes the launch reads (slices are whole
 * multiples of 16 KiB, so slightly fewer than `bytes`), 0 on a bad argument or a failed launch.
 * `sink`: 4 writable bytes on the device (practically never written). */
size_t pq_stream_read(const void *src, size_t bytes, int n_wavefronts, uint32_t *sink, void *stream);

/* Measurement aid (no reference counterpart): the HBM reads of pq_decode_attn's main kernel (byte-per-code
 * rows, half-precision values) without its arithmetic: `planes` (batch x KV head) planes of `tokens` tokens,
 * each cut into `n_slices` slices read by one wavefront with the kernel's own loads, order and prefetch depth.
 * codes: `planes` planes of `code_plane_tokens` 64-byte rows; v: `planes` planes of `v_plane_tokens`
 * 256-byte rows.  Returns the bytes one launch reads (320 per token; slices are whole multiples of 128
 * tokens), 0 on a bad argument or a failed launch.  Time it beside the kernel: the difference is what the
 * kernel's table, score and softmax work costs on top of its memory access. */
size_t pq_attn_load_replica(const uint8_t *codes, const void *v, int planes, int64_t code_plane_tokens,
                            int64_t v_plane_tokens, int64_t tokens, int n_slices, uint32_t *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* POLARQUANT_BENCH_H */
