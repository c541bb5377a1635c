/* polarquant.h — C ABI of the MI355X (gfx950) polar-key decode path.
 *
 * The reference has no C/FFI boundary for this path: its Python attention
 * classes call a Triton JIT kernel and eager torch ops.  Each entry point below
 * names the reference interface it replaces; the Python classes in
 * polarquant_amd/ bind them through ctypes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller, unless it is
 *     documented as a host pointer;
 *   - every call is asynchronous on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream), performs no allocation and no
 *     synchronisation, and never throws;
 *   - the return value is PQ_OK (0) or a negative pq_status; argument errors are
 *     detected on the host before anything is launched, so they can be tested
 *     without a GPU;
 *   - "half word" means a 16-bit float in the dtype given by `dtype`
 *     (PQ_F16 = IEEE binary16, PQ_BF16 = bfloat16);
 *   - head_dim is 128 (D = 64 dimension pairs (d, d+64)) and the group size G is
 *     128 tokens, as in the reference (models/modeling_llama_polar.py:34-37).
 */
#ifndef POLARQUANT_H
#define POLARQUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PQ_HEAD_DIM 128
#define PQ_PAIRS 64
#define PQ_GROUP 128
#define PQ_MAX_REP 8          /* query heads per KV head (GQA ratio) supported by the kernels */
#define PQ_MAX_TBITS 7        /* angle bits: every split the reference takes (rbits + tbits <= 8,
                                 models/kernel4group.py:83-109).  Up to 4 angle bits run the tuned kernels; 5 to 7
                                 run the one-wavefront kernels with a 32-128 KiB table (correct, not tuned); with 7
                                 (128 bins: 128 KiB for four query heads, all the LDS a workgroup can have) a KV
                                 head's query heads are worked through four at a time, in two launches. */
#define PQ_PARTIAL_FLOATS 132 /* floats per split-K partial: m, l, 2 pad, acc[128] */
#define PQ_MAX_PLANE_TOKENS 16776960 /* 2^24 - 256: most value rows (v_capacity, v4_capacity) or residual
                                        keys (resid_capacity) of one (batch, KV head) plane */

typedef enum {
    PQ_OK = 0,
    PQ_ERR_NULL_POINTER = -1,
    PQ_ERR_BAD_SHAPE = -2,      /* non-positive size, N % Nk != 0, rep > PQ_MAX_REP ... */
    PQ_ERR_BAD_BITS = -3,       /* rbits/tbits outside [1,..], rbits + tbits > 8 */
    PQ_ERR_BAD_DTYPE = -4,
    PQ_ERR_MISALIGNED = -5,     /* a pointer or stride breaks the alignment a kernel needs */
    PQ_ERR_BAD_STRIDE = -6,
    PQ_ERR_WORKSPACE = -7,      /* workspace too small / bad split count */
    PQ_ERR_LAUNCH = -8,         /* hipLaunchKernel reported an error */
    PQ_ERR_NO_DEVICE = -9
} pq_status;

typedef enum { PQ_F16 = 0, PQ_BF16 = 1 } pq_dtype;

/* flags for pq_quantize_groups */
#define PQ_WRAP_FP32 1u /* add 2*pi in fp32 (eager CUDA semantics) instead of the
                           dtype-rounded 6.28125 that eager CPU torch adds */
#define PQ_DEVICE_ATAN2 8u /* the angle is round_dtype(atan2f(y, x)) with the GPU math library's atan2f, which
                              is what eager torch evaluates on device tensors, instead of SLEEF's
                              Sleef_atan2f_u10, which eager torch evaluates on the CPU */
#define PQ_EAGER_GPU (PQ_WRAP_FP32 | PQ_DEVICE_ATAN2) /* codes and metadata as the reference's lines produce them
                              when they run on the GPU (where the reference runs them): both switches */
#define PQ_ANGLE_UNIFORM 2u /* fixed angle bins over [-pi, pi) instead of the group's own
                               [min, max]: the reference formula (:148) with the constants
                               tmn = -pi and tscale = 2*pi / 2^tbits, both rounded to the key
                               dtype and written to the metadata tensors like any other, so
                               the decode kernels need no switch.  No reference counterpart. */

/* flag for the decode entry points (and for pq_quantize_groups): the code rows hold 64 packed 6-bit
 * codes (48 bytes per token, code i in bits [6i, 6i+6) of the row) instead of one byte per code.
 * For rbits + tbits <= 6; the decode kernels take it for tbits == 3 (the 3/3 configuration).  The
 * reference stores one byte per pair for every bit width (models/kernel4group.py:1-3); this is the
 * sub-byte store it announces there.  Code tensors are then [B,Nk,capacity,128,48]. */
#define PQ_CODES_PACKED6 4u

/* flag for the attention entry points (pq_decode_attn and its variants): the context slices are cut on
 * the device from the per-sequence counts, so that every wavefront gets the same amount of work
 * whatever the lengths are (ragged batches; batches that grow under a replayed graph).  All planes
 * ((sequence, KV head) pairs) are laid end to end in tiles of 64 tokens (two per quantized group, then
 * one per 64 residual keys, behind three units that stand for a plane's start-up), and the line is cut into equal segments, one per wavefront the device holds
 * at once; a segment may end one plane and begin the next, and may cut a group in half.  n_splits is
 * then the number of partial slots per query head (>= 2): no plane is cut into more pieces than that (the
 * segment length is raised to ceil((2 group_capacity + ceil(resid_capacity / 64) + 3) / (n_splits - 1)) tiles if it has
 * to be),
 * min_groups_per_split a lower bound on the segment length in groups.  Results do not depend on how the
 * line is cut beyond fp32 summation order.  No reference counterpart (the reference has no split over
 * the context at all). */
#define PQ_BALANCED_SLICES 16u

/* flag for the attention entry points with half-precision values: one wavefront per slice does everything
 * (codes, tables, scores, then values, softmax, P.V in turn), as the kernels for 4-bit values do.  Without it
 * (the default) a slice is shared by the two wavefronts that sit on one SIMD: a scorer (codes, tables, scores)
 * and an accumulator (values, mask, softmax, P.V) that hand 64-token tiles of scores over through LDS, so the
 * two halves of the work overlap; the results differ only as two split counts differ (fp32 summation order
 * is the same: the tiles are accumulated in the same order).  Kept for comparison and as the fall-back.
 * No reference counterpart. */
#define PQ_SINGLE_WAVEFRONT 32u

/* What the optional `status` word of the attention entry points can hold after the call's kernels have run. */
#define PQ_STATUS_HANDOVER_TIMEOUT 1 /* a scorer / accumulator hand-over gave up waiting; the output rows of every plane
                                        the failing pair worked on are NaN */

/* Test hook of pq_decode_attn / _partials / _static (scorer / accumulator kernels only; refused together with
 * PQ_SINGLE_WAVEFRONT, whose kernels have no hand-over, and by the 4-bit-value entry point): the scorers publish nothing,
 * and the bounded waits of the hand-over give up after 1000 polls instead of 2^22.  Every kernel still ends normally;
 * every output of the call is NaN and the status word is set.  For the test that a hand-over which fails can neither
 * hang the GPU nor pass for a result.  ONLY the test build of the library (compiled with -DPQ_TEST_HOOKS:
 * libpolarquant_hip_testhooks.so, which the package never loads) honours it, and only for PQ_F16; the shipping library
 * refuses the flag with PQ_ERR_BAD_SHAPE like any unknown flag, and its kernels contain no such switch. */
#define PQ_TEST_SILENT_SCORER 0x40000000u

/* Linear layer of a decode step: y[M, N] = x[M, K] . w[N, K]^T (+ bias[N]), M <= 16 rows (one new
 * token per sequence), fp32 accumulation, one rounding to the dtype.  Replaces the q/k/v, o and MLP
 * projections (`nn.Linear`) the decode step calls around the attention
 * (models/modeling_llama_polar.py:47-52, :131, and the decoder layer's MLP, :456-486): at this M they
 * are streams of the weight matrix through HBM, which the kernel is laid out for.
 *   x [M, K] rows `x_row_stride` elements apart, w [N, K] dense row-major (the nn.Linear weight),
 *   y [M, N] rows `y_row_stride` apart; N % 16 == 0, K % 32 == 0, x and w 16-byte aligned.
 *   w_up != NULL: the gated MLP input in one call, y = silu(x.w^T) * (x.w_up^T) with the eager
 *   modules' roundings (both products and silu rounded to the dtype first); no bias then. */
int pq_linear_small_m(const void *x, int64_t x_row_stride, const void *w, const void *w_up, const void *bias,
                      void *y, int64_t y_row_stride, int M, int N, int K, int dtype, void *stream);
int pq_validate_linear_small_m(const void *x, int64_t x_row_stride, const void *w, const void *w_up, const void *bias,
                               const void *y, int64_t y_row_stride, int M, int N, int K, int dtype);

/* The q, k, v projections of a decode step as ONE product with the concatenated weight
 * w_qkv [(N + 2 Nk) * 128, K] (q heads, then k heads, then v heads; optional bias of the same length),
 * with RoPE and the two cache appends in its epilogue: pq_linear_small_m followed by pq_rope_append in
 * one launch, bit-identical to that pair (models/modeling_llama_polar.py:47-59,77,98).  M <= 8 rows
 * (sequences), K % 64 == 0.  cos / sin tables, pos, q_out, k_dst / k_row, v_dst / v_row: as for
 * pq_rope_append, with B = M. */
int pq_qkv_rope_append(const void *x, int64_t x_row_stride, const void *w_qkv, const void *bias, int M, int K, int dtype,
                       const void *cos_table, const void *sin_table, int64_t table_rows, const int64_t *pos, void *q_out,
                       void *k_dst, int64_t k_rows, const int64_t *k_row, void *v_dst, int64_t v_rows,
                       const int64_t *v_row, int N, int Nk, void *stream);
int pq_validate_qkv_rope_append(const void *x, int64_t x_row_stride, const void *w_qkv, const void *bias, int M, int K,
                                int dtype, const void *cos_table, const void *sin_table, int64_t table_rows,
                                const int64_t *pos, const void *q_out, const void *k_dst, int64_t k_rows,
                                const int64_t *k_row, const void *v_dst, int64_t v_rows, const int64_t *v_row, int N, int Nk);

/* Layout converter for code rows: pack != 0 turns `n_rows` byte-per-code rows (64 bytes each, every
 * code < 64) into packed 6-bit rows (48 bytes each), pack == 0 the reverse.  For caches built by the
 * reference (always byte-per-code) that are to be kept packed, and back.  No reference counterpart. */
int pq_convert_codes6(const uint8_t *src, uint8_t *dst, size_t n_rows, int pack, void *stream);

/* Library version (major*10000 + minor*100 + patch). No reference counterpart. */
int pq_version(void);

/* Human-readable text for a pq_status. Host-only. */
const char *pq_status_string(int status);

/* ---------------------------------------------------------------------------
 * S — quantized-key decode scores.
 * Replaces attention_decode_forward_triton_impl(query_states, indices, rscale,
 * rmn, tscale, tmn, rbits, tbits) -> fp32 [B,N,1,Nb*G]
 * (models/kernel4group.py:83-109, kernel :14-80).
 *
 *   q       [B,N,1,128]      half words, contiguous
 *   codes   [B,Nk,Nb,128,64] u8, contiguous, code = (rho << tbits) + theta
 *   rscale, rmn, tscale, tmn [B,Nk,Nb,1,64] half words, contiguous
 *   out     [B,N,1,Nb*128]   fp32, contiguous
 * out[b, kvh*rep + j, 0, g*128 + t] = sum_d (q[d] cos phi + q[d+64] sin phi) * r,
 *   phi = tscale_d*(theta+0.5)+tmn_d, r = rscale_d*(rho+0.5)+rmn_d.  No 1/sqrt(d).
 * Query head h reads KV head h / (N/Nk) (repeat-interleave, as HF repeat_kv).
 * ------------------------------------------------------------------------- */
int pq_decode_scores(const void *q, const uint8_t *codes, const void *rscale, const void *rmn,
                     const void *tscale, const void *tmn, float *out,
                     int B, int N, int Nk, int Nb, int rbits, int tbits, int dtype, unsigned flags, void *stream);

/* Host-only argument check of pq_decode_scores (same return codes, launches nothing). */
int pq_validate_decode_scores(const void *q, const uint8_t *codes, const void *rscale, const void *rmn,
                              const void *tscale, const void *tmn, const float *out,
                              int B, int N, int Nk, int Nb, int rbits, int tbits, int dtype, unsigned flags);

/* ---------------------------------------------------------------------------
 * Q — polar quantizer (quantize-on-append and prompt quantization).
 * Replaces LlamaPolarGroupAttention.quantize_and_pack_nbit(key_states)
 * (models/modeling_llama_polar.py:135-157; models/modeling_qwen_polar.py:134-156).
 *
 *   k          post-RoPE keys, logical shape [B,Nk,Nb*128,128] half words, addressed
 *              with element strides k_strides[4] = {batch, head, token, dim};
 *              dim stride must be 1 (a transposed [B,L,Nk,128] view is fine)
 *   k_strides  HOST pointer to 4 int64
 *   codes      [B,Nk,Nb,128,64] u8 — written with group stride 128*64 inside a
 *              (batch, head) plane of `out_group_capacity` groups, i.e. the plane
 *              stride is out_group_capacity*128*64 (pass Nb for a dense output);
 *              writing starts at group `out_group_offset` of each plane
 *   rscale, rmn, tscale, tmn  [B,Nk,out_group_capacity,1,64] half words, same rule
 * Arithmetic: every reference op is evaluated in fp32 and rounded to the key
 * dtype before the next, which is what eager torch does on half tensors.
 * Degenerate groups (scale == 0, quotient NaN/Inf) yield code 0.
 * ------------------------------------------------------------------------- */
int pq_quantize_groups(const void *k, const int64_t *k_strides, int dtype,
                       int B, int Nk, int Nb, int rbits, int tbits, unsigned flags,
                       uint8_t *codes, void *rscale, void *rmn, void *tscale, void *tmn,
                       int out_group_capacity, int out_group_offset, void *stream);

int pq_validate_quantize_groups(const void *k, const int64_t *k_strides, int dtype,
                                int B, int Nk, int Nb, int rbits, int tbits, unsigned flags,
                                const uint8_t *codes, const void *rscale, const void *rmn,
                                const void *tscale, const void *tmn,
                                int out_group_capacity, int out_group_offset);

/* Device self-test of the quantizer's arithmetic (no reference counterpart).
 * The kernel takes a cheap arctangent / square root first and the exact,
 * eager-torch-identical routines only near a rounding boundary; this runs both on
 * ALL 2^32 (y, x) operand pairs of the dtype (NaNs skipped) and adds to
 * counters[0] the number of pairs whose rounded angle or radius differ, plus the
 * pairs whose exact radius is not the correctly rounded square root (checked in
 * double precision against the midpoints to its two neighbours); must stay 0.
 * counters[1] receives the number of pairs that needed the exact routine.
 * Both quantizers also replace the fp32 division by a scale with a reciprocal and
 * two fused multiply-adds; counters[2] receives the number of (dividend, scale)
 * pairs of the dtype, over the whole range the quantizers can meet, whose
 * quotient rounded to the dtype differs from the divided one (must stay 0).
 * counters[3] and [4]: as [0] and [1] with PQ_DEVICE_ATAN2 (the GPU math library's
 * arctangent as the exact routine, a wider guard band); [3] must stay 0.
 * `counters`: device uint64[5], zeroed by the caller. Takes ~0.2 s. */
int pq_selftest_quantizer_math(int dtype, uint64_t *counters, void *stream);

/* ---------------------------------------------------------------------------
 * R+M+X+V — fused decode attention over the polar key cache.
 * Replaces the decode branch of LlamaPolarGroupAttention.forward between the
 * RoPE and o_proj (models/modeling_llama_polar.py:66-99; qwen :65-98): quantized
 * scores, residual fp16 scores, concat, /sqrt(d), mask, fp32 softmax, P.V — in
 * one pass over HBM with a split over the context and a merge kernel.
 *
 * The caller has already appended the step's new key to the residual buffer
 * and the new value to the V cache (reference :77,98).
 *
 *   q        [B,N,128] half words, contiguous, 16-byte aligned
 *   codes    u8, (batch,head) plane stride = group_capacity*128*64; meta likewise
 *            with plane stride group_capacity*64; may be NULL when no sequence has
 *            a quantized group
 *   n_groups number of quantized groups of every sequence (used when
 *            n_groups_per_seq == NULL)
 *   n_groups_per_seq  optional device int32 [B]: per-sequence group count (ragged)
 *   k_resid  [B,Nk,resid_capacity,128] half words: fp16 keys not yet quantized
 *   n_resid / n_resid_per_seq  residual key count, uniform or device int32 [B];
 *            0..128
 *   v        [B,Nk,v_capacity,128] half words; token t of sequence b is row t;
 *            rows [0, n_groups*128 + n_resid) are read
 *   mask     optional device u8 [B, mask_stride]: 1 = attend, 0 = masked; column t
 *            is token t (reference attention_mask, :94-95); NULL = no mask
 *   sm_scale multiplier applied to every score (1/sqrt(128) in the reference)
 *   n_splits context slices (blocks) per (batch, KV head) for the quantized part, >= 1;
 *            use pq_decode_attn_plan to choose
 *   min_groups_per_split  0, or a lower bound on the groups one slice takes.  For ragged
 *            batches pass ceil(total groups of all (batch, KV head) planes / (4 * CUs)) and
 *            n_splits = ceil(group_capacity / that): every wavefront then gets about the same
 *            number of groups whatever its sequence's length, and a short sequence uses only
 *            its first few slices (the others return at once).  n_splits * max(this,
 *            ceil(groups / n_splits)) always covers the sequence.
 *   workspace  device fp32 buffer of pq_decode_attn_workspace_bytes(...) bytes
 *   out      [B,N,128] half words.  With n_splits == 1 and a 16-byte aligned `out` the default kernels (tbits <= 4,
 *            no PQ_SINGLE_WAVEFRONT, no PQ_BALANCED_SLICES) write it themselves (bit for bit what pq_decode_attn_merge
 *            makes of the one partial) and no merge is launched; the workspace then stays untouched
 *   flags    0, or PQ_CODES_PACKED6 (code plane stride is then group_capacity*128*48) and / or
 *            PQ_BALANCED_SLICES (slices cut on the device from the per-sequence counts, see above) and / or
 *            PQ_SINGLE_WAVEFRONT (one wavefront per slice instead of a scorer / accumulator pair)
 *   status   NULL, or one device int32 that the CALLER has set to 0 (the library never clears it): the kernels with a
 *            scorer / accumulator pair per slice store PQ_STATUS_HANDOVER_TIMEOUT there when a hand-over between the
 *            two wavefronts gives up (2^22 polls, about half a second, without an answer: a wavefront that never got
 *            to run, which no correct execution produces).  The affected output rows are NaN as well; the word lets a
 *            host learn of it, after synchronizing with the stream, without scanning the output.  It stays untouched
 *            by the one-wavefront kernels, which have no hand-over.
 * Limits: v_capacity <= PQ_MAX_PLANE_TOKENS tokens and group_capacity <= 2^17 groups per (batch, KV head)
 * plane (32-bit byte sizes and offsets inside a plane), B*Nk <= 65535, N/Nk <= 8.
 * ------------------------------------------------------------------------- */
int pq_decode_attn(const void *q,
                   const uint8_t *codes, const void *rscale, const void *rmn,
                   const void *tscale, const void *tmn, int group_capacity,
                   int n_groups, const int32_t *n_groups_per_seq,
                   const void *k_resid, int resid_capacity, int n_resid, const int32_t *n_resid_per_seq,
                   const void *v, int64_t v_capacity,
                   const uint8_t *mask, int64_t mask_stride,
                   float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                   int n_splits, int min_groups_per_split, void *workspace, size_t workspace_bytes,
                   void *out, unsigned flags, int32_t *status, void *stream);

int pq_validate_decode_attn(const void *q,
                            const uint8_t *codes, const void *rscale, const void *rmn,
                            const void *tscale, const void *tmn, int group_capacity,
                            int n_groups, const int32_t *n_groups_per_seq,
                            const void *k_resid, int resid_capacity, int n_resid, const int32_t *n_resid_per_seq,
                            const void *v, int64_t v_capacity,
                            const uint8_t *mask, int64_t mask_stride,
                            float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                            int n_splits, int min_groups_per_split, const void *workspace, size_t workspace_bytes,
                            const void *out, unsigned flags);

/* The two launches of pq_decode_attn as separate calls, same arguments and
 * checks: pq_decode_attn_partials writes the n_splits partial results
 * (running maximum, probability sum, un-normalised output) of every query head
 * into `workspace`; pq_decode_attn_merge combines them into `out`.  They exist so
 * that a caller can time, overlap or graph-capture the two kernels separately;
 * pq_decode_attn(...) == partials(...) followed by merge(...) on the same stream.
 * No reference counterpart beyond that of pq_decode_attn. */
int pq_decode_attn_partials(const void *q,
                            const uint8_t *codes, const void *rscale, const void *rmn,
                            const void *tscale, const void *tmn, int group_capacity,
                            int n_groups, const int32_t *n_groups_per_seq,
                            const void *k_resid, int resid_capacity, int n_resid, const int32_t *n_resid_per_seq,
                            const void *v, int64_t v_capacity,
                            const uint8_t *mask, int64_t mask_stride,
                            float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                            int n_splits, int min_groups_per_split, void *workspace, size_t workspace_bytes,
                            unsigned flags, int32_t *status, void *stream);

int pq_decode_attn_merge(const void *workspace, size_t workspace_bytes, int B, int N, int n_splits, int dtype,
                         void *out, void *stream);

/* pq_decode_attn for callers that cannot allocate device memory and have no workspace to pass:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments, checks and results as pq_decode_attn (the same two
 * kernels), but the split partials go to a buffer inside the library: a file-scope device array of
 * PQ_STATIC_MAX_PARTIALS partials (8.25 MiB, held by every GPU the library runs on until the process
 * ends).  The call allocates and frees nothing.  B * N * n_splits above PQ_STATIC_MAX_PARTIALS is
 * rejected with PQ_ERR_WORKSPACE.  All calls on one GPU share that buffer: calls that overlap on one
 * GPU (different streams, several threads) race on it; calls on one stream do not.  The first call
 * on a device asks the runtime for the array's device address; make that call outside a capture. */
#define PQ_STATIC_MAX_PARTIALS 16384
int pq_decode_attn_static(const void *q,
                          const uint8_t *codes, const void *rscale, const void *rmn,
                          const void *tscale, const void *tmn, int group_capacity,
                          int n_groups, const int32_t *n_groups_per_seq,
                          const void *k_resid, int resid_capacity, int n_resid, const int32_t *n_resid_per_seq,
                          const void *v, int64_t v_capacity,
                          const uint8_t *mask, int64_t mask_stride,
                          float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                          int n_splits, int min_groups_per_split, void *out, unsigned flags, int32_t *status,
                          void *stream);

/* ---------------------------------------------------------------------------
 * 4-bit values: the reference's Mixed variant (LlamaPolarMixedGroupAttention,
 * models/modeling_llama_polar.py:158-292).
 *
 * pq_quantize_values replaces triton_quantize_and_pack_along_last_dim(values, 128, 4)
 * at :236 and :275 (a routine of the kivi_quant package, which is not in the
 * reference tree; its published form is followed): per token and head, over the
 * 128 dims, scale = (max - min) / 15, code = round_half_even(clamp((x - min) / scale, 0, 15)),
 * each op rounded to the value dtype; 8 codes per int32, dim 8w+i in bits [4i, 4i+4)
 * of word w.  A constant row (0/0) yields code 0.
 *   v        [B,Nk,T,128] half words, element strides v_strides[4] (dim stride 1,
 *            the others multiples of 8), 16-byte aligned
 *   codes    int32 [B,Nk,out_token_capacity,16]; scale, zero [B,Nk,out_token_capacity]
 *            (the reference's [..., 1] tensors); rows out_token_offset .. +T are written
 *
 * pq_decode_attn_v4 replaces the decode branch :185-241 between RoPE and o_proj:
 * as pq_decode_attn, but the values of the quantized groups are 4-bit
 * (v_codes / v_scale / v_zero, token t of a sequence is row t, rows
 * [0, n_groups*128) are read; :229-236 cuda_bmm_fA_qB_outer) and `v_resid`
 * [B,Nk,resid_capacity,128] holds the half-precision values of the residual
 * window only, row r belonging to residual key r (:238).  Keys and values
 * share the window's fill (n_resid) and are flushed together (:207,:243).
 * flags, status: as for pq_decode_attn.  The kernels for 4-bit values run one wavefront per slice whatever
 * the flags say; PQ_SINGLE_WAVEFRONT and `status` matter only while no group has been quantized yet, when the
 * call is served by the half-precision-value kernels over the residual window.
 * ------------------------------------------------------------------------- */
int pq_quantize_values(const void *v, const int64_t *v_strides, int dtype, int B, int Nk, int T,
                       int32_t *codes, void *scale, void *zero,
                       int64_t out_token_capacity, int64_t out_token_offset, void *stream);

int pq_validate_quantize_values(const void *v, const int64_t *v_strides, int dtype, int B, int Nk, int T,
                                const int32_t *codes, const void *scale, const void *zero,
                                int64_t out_token_capacity, int64_t out_token_offset);

int pq_decode_attn_v4(const void *q,
                      const uint8_t *codes, const void *rscale, const void *rmn,
                      const void *tscale, const void *tmn, int group_capacity,
                      int n_groups, const int32_t *n_groups_per_seq,
                      const void *k_resid, int resid_capacity, int n_resid, const int32_t *n_resid_per_seq,
                      const void *v_resid,
                      const int32_t *v_codes, const void *v_scale, const void *v_zero, int64_t v4_capacity,
                      const uint8_t *mask, int64_t mask_stride,
                      float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                      int n_splits, int min_groups_per_split, void *workspace, size_t workspace_bytes,
                      void *out, unsigned flags, int32_t *status, void *stream);

/* RoPE over whole sequences, the prompt pass's `apply_rotary_pos_emb(query_states, key_states, cos, sin)`
 * (models/modeling_llama_polar.py:56-59) in one launch, bit-identical to the eager
 * (x * cos) + (rotate_half(x) * sin) in the model dtype.  q_lin / k_lin: outputs of q_proj / k_proj, token
 * t = b * L + l at element offset t * token_stride (0 = dense, N * 128 resp. Nk * 128; multiples of 8);
 * cos_rows / sin_rows [1 or B, L, 128] in the dtype, batch b at b * cos_sin_batch_stride (0 when shared);
 * q_out [B, L, N, 128], k_out [B, L, Nk, 128] contiguous (read them as [B, heads, L, 128] by a transposed view,
 * as the reference's .view().transpose(1, 2) does). */
int pq_rope_qk(const void *q_lin, int64_t q_token_stride, const void *k_lin, int64_t k_token_stride, const void *cos_rows,
               const void *sin_rows, int64_t cos_sin_batch_stride, void *q_out, void *k_out, int B, int L, int N, int Nk,
               int dtype, void *stream);

/* ---------------------------------------------------------------------------
 * A — the elementwise steps around the attention call of one decode step, each a
 * chain of 8-12 eager launches on a [B,1,hidden] activation in the reference.
 * Arithmetic follows the eager modules op by op (fp32 result rounded to the
 * dtype after every op).
 *
 * pq_rope_append: HF apply_rotary_pos_emb on the new token's q and k
 * (models/modeling_llama_polar.py:56-59), the key's append to the residual
 * window (:77) and the value's append to the value cache (:98), in one launch.
 * The position and the destination rows are read from device memory, so the
 * launch can be replayed from a captured graph.
 *   q_lin [B,N*128], k_lin / v_lin [B,Nk*128]  projection outputs; batch rows q_row_stride /
 *            kv_row_stride elements apart (0 = dense; (N+2Nk)*128 when the three are slices of
 *            one fused projection output)
 *   cos_table / sin_table [table_rows,128]     in the dtype; row *pos is used
 *   q_out [B,N,128]
 *   k_dst [B,Nk,k_rows,128], row *k_row <- rotated key
 *   v_dst [B,Nk,v_rows,128], row *v_row <- value
 *
 * pq_rmsnorm: y = weight * dtype(float(s) * rsqrt(mean(float(s)^2) + eps)) with
 * s = x, or s = dtype(x + residual) (also written to sum_out if given; sum_out may
 * alias x): the decoder layer's residual add + LlamaRMSNorm (:466-484).
 *
 * pq_silu_mul: y = dtype(silu(gate)) * up for `rows` rows of `cols` elements (LlamaMLP, called at
 * :483); gate / up rows are in_row_stride elements apart (0 = dense; 2*cols when they are the two
 * halves of one fused gate|up projection output), y is dense.
 * ------------------------------------------------------------------------- */
int pq_rope_append(const void *q_lin, const void *k_lin, const void *v_lin,
                   const void *cos_table, const void *sin_table, int64_t table_rows, const int64_t *pos,
                   void *q_out, void *k_dst, int64_t k_rows, const int64_t *k_row,
                   void *v_dst, int64_t v_rows, const int64_t *v_row,
                   int B, int N, int Nk, int dtype, int64_t q_row_stride, int64_t kv_row_stride, void *stream);

int pq_rmsnorm(const void *x, const void *residual, const void *weight, void *y, void *sum_out,
               int rows, int hidden, float eps, int dtype, void *stream);

int pq_silu_mul(const void *gate, const void *up, void *y, int rows, int cols, int64_t in_row_stride,
                int dtype, void *stream);

/* Split count for pq_decode_attn_v4 (as pq_decode_attn_plan, which see; the 4-bit
 * kernel runs two wavefronts per SIMD when N/Nk <= 4). No reference counterpart. */
int pq_decode_attn_v4_plan(int B, int N, int Nk, int max_groups, int n_cus);

int pq_validate_decode_attn_v4(const void *q,
                               const uint8_t *codes, const void *rscale, const void *rmn,
                               const void *tscale, const void *tmn, int group_capacity,
                               int n_groups, const int32_t *n_groups_per_seq,
                               const void *k_resid, int resid_capacity, int n_resid, const int32_t *n_resid_per_seq,
                               const void *v_resid,
                               const int32_t *v_codes, const void *v_scale, const void *v_zero, int64_t v4_capacity,
                               const uint8_t *mask, int64_t mask_stride,
                               float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                               int n_splits, int min_groups_per_split, const void *workspace, size_t workspace_bytes,
                               const void *out, unsigned flags);

/* Suggested n_splits for a shape (host-only; `max_groups` = largest group count
 * of any sequence, `n_cus` = compute units of the device or 0 for 256). */
int pq_decode_attn_plan(int B, int Nk, int max_groups, int n_cus);

/* Bytes of workspace pq_decode_attn needs for (B, N, n_splits). Host-only. */
size_t pq_decode_attn_workspace_bytes(int B, int N, int n_splits);

#ifdef __cplusplus
}
#endif
#endif /* POLARQUANT_H */
