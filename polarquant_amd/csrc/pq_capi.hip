// C ABI of the polar-key decode path: host-side argument validation and
// dispatch to the kernel launchers.  Declarations and the reference interfaces
// they replace are in include/polarquant.h.
#include "../../include/polarquant.h"
#include "pq_internal.h"

namespace {

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int check_bits(int rbits, int tbits) {
    if (rbits < 1 || tbits < 1 || rbits + tbits > 8) return PQ_ERR_BAD_BITS;
    // (7 angle bits: one byte per code leaves one radius bit; the decode kernels then work through a KV head's query
    // heads four at a time, see kMaxHeadsWidestTable)
    if (tbits > PQ_MAX_TBITS) return PQ_ERR_BAD_BITS;
    return PQ_OK;
}

// decode-side flags: the packed 6-bit code layout, which exists for tbits == 3 (rbits <= 3); for the attention entry
// points the two kernel choices; for the entry points that run the scorer / accumulator pairs, in the test build only,
// the hook that silences the scorers
enum class Entry { Scores, Attention, AttentionV4 };
int check_decode_flags(unsigned flags, int rbits, int tbits, Entry entry = Entry::Scores) {
    // the score op has one slice per group; only the attention entry points cut the context
    unsigned known = PQ_CODES_PACKED6;
    if (entry != Entry::Scores) known |= PQ_BALANCED_SLICES;
    if (entry != Entry::Scores) known |= PQ_SINGLE_WAVEFRONT;
    // (the test hook exists where a call runs the scorer / accumulator pairs: half-precision values, up to 4 angle bits)
#ifdef PQ_TEST_HOOKS
    if (entry == Entry::Attention && pq::attn_runs_pairs(false, (flags & PQ_SINGLE_WAVEFRONT) != 0, tbits))
        known |= PQ_TEST_SILENT_SCORER;
#endif
    if (flags & ~known) return PQ_ERR_BAD_SHAPE;
    if ((flags & PQ_CODES_PACKED6) && (tbits != 3 || rbits + tbits > 6)) return PQ_ERR_BAD_BITS;
    return PQ_OK;
}

int check_heads(int B, int N, int Nk) {
    if (B <= 0 || N <= 0 || Nk <= 0 || N % Nk != 0) return PQ_ERR_BAD_SHAPE;
    if (N / Nk > PQ_MAX_REP) return PQ_ERR_BAD_SHAPE;
    return PQ_OK;
}

}  // namespace

extern "C" {

int pq_version(void) { return 100; }

const char* pq_status_string(int status) {
    switch (status) {
        case PQ_OK: return "ok";
        case PQ_ERR_NULL_POINTER: return "null pointer argument";
        case PQ_ERR_BAD_SHAPE: return "bad shape (non-positive size, N % Nk != 0, or N/Nk > 8)";
        case PQ_ERR_BAD_BITS: return "bad bit widths (need rbits >= 1, tbits >= 1, rbits + tbits <= 8; packed 6-bit rows need tbits == 3)";
        case PQ_ERR_BAD_DTYPE: return "bad dtype (0 = float16, 1 = bfloat16)";
        case PQ_ERR_MISALIGNED: return "pointer or stride not aligned as the kernel requires";
        case PQ_ERR_BAD_STRIDE: return "bad stride or capacity";
        case PQ_ERR_WORKSPACE: return "workspace too small or bad split count";
        case PQ_ERR_LAUNCH: return "kernel launch failed";
        case PQ_ERR_NO_DEVICE: return "no HIP device";
        default: return "unknown status";
    }
}

int pq_validate_decode_scores(const void* q, const uint8_t* codes, const void* rscale, const void* rmn,
                              const void* tscale, const void* tmn, const float* out,
                              int B, int N, int Nk, int Nb, int rbits, int tbits, int dtype, unsigned flags) {
    if (!q || !codes || !rscale || !rmn || !tscale || !tmn || !out) return PQ_ERR_NULL_POINTER;
    if (int rc = check_decode_flags(flags, rbits, tbits)) return rc;
    if (int rc = check_heads(B, N, Nk)) return rc;
    if (Nb <= 0 || Nb > 65535 || static_cast<long long>(B) * Nk > 0x7fffffffLL) return PQ_ERR_BAD_SHAPE;
    if (int rc = check_bits(rbits, tbits)) return rc;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (!aligned(codes, 16) || !aligned(q, 2) || !aligned(rscale, 2) || !aligned(rmn, 2) || !aligned(tscale, 2) ||
        !aligned(tmn, 2) || !aligned(out, 4))
        return PQ_ERR_MISALIGNED;
    return PQ_OK;
}

int pq_decode_scores(const void* q, const uint8_t* codes, const void* rscale, const void* rmn,
                     const void* tscale, const void* tmn, float* out,
                     int B, int N, int Nk, int Nb, int rbits, int tbits, int dtype, unsigned flags, void* stream) {
    if (int rc = pq_validate_decode_scores(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, rbits, tbits, dtype, flags))
        return rc;
    // grid is (Nb, B*Nk): y is limited to 65535 blocks
    if (static_cast<long long>(B) * Nk > 65535) return PQ_ERR_BAD_SHAPE;
    const int err = pq::launch_scores(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, tbits, dtype,
                                      (flags & PQ_CODES_PACKED6) != 0, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

}  // extern "C"

extern "C" {

int pq_validate_quantize_groups(const void* k, const int64_t* k_strides, int dtype,
                                int B, int Nk, int Nb, int rbits, int tbits, unsigned flags,
                                const uint8_t* codes, const void* rscale, const void* rmn,
                                const void* tscale, const void* tmn,
                                int out_group_capacity, int out_group_offset) {
    if (!k || !k_strides || !codes || !rscale || !rmn || !tscale || !tmn) return PQ_ERR_NULL_POINTER;
    if (B <= 0 || Nk <= 0 || Nb <= 0 || Nb > 65535 * 32 || static_cast<long long>(B) * Nk > 65535)
        return PQ_ERR_BAD_SHAPE;
    // the same bit widths as the decode entry points: no cache is written that nothing here can read
    if (int rc = check_bits(rbits, tbits)) return rc;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (flags & ~static_cast<unsigned>(PQ_WRAP_FP32 | PQ_ANGLE_UNIFORM | PQ_CODES_PACKED6 | PQ_DEVICE_ATAN2)) return PQ_ERR_BAD_SHAPE;
    if ((flags & PQ_CODES_PACKED6) && rbits + tbits > 6) return PQ_ERR_BAD_BITS;
    if (k_strides[3] != 1) return PQ_ERR_BAD_STRIDE;
    if (k_strides[0] < 0 || k_strides[1] < 0 || k_strides[2] < PQ_HEAD_DIM) return PQ_ERR_BAD_STRIDE;
    if (out_group_offset < 0 || out_group_capacity < out_group_offset + Nb) return PQ_ERR_BAD_STRIDE;
    // 8-byte vector loads of 4 halves: base and every stride must keep that alignment
    if (!aligned(k, 8) || (k_strides[0] & 3) || (k_strides[1] & 3) || (k_strides[2] & 3)) return PQ_ERR_MISALIGNED;
    if (!aligned(codes, 4) || !aligned(rscale, 8) || !aligned(rmn, 8) || !aligned(tscale, 8) || !aligned(tmn, 8))
        return PQ_ERR_MISALIGNED;
    return PQ_OK;
}

int pq_quantize_groups(const void* k, const int64_t* k_strides, int dtype,
                       int B, int Nk, int Nb, int rbits, int tbits, unsigned flags,
                       uint8_t* codes, void* rscale, void* rmn, void* tscale, void* tmn,
                       int out_group_capacity, int out_group_offset, void* stream) {
    if (int rc = pq_validate_quantize_groups(k, k_strides, dtype, B, Nk, Nb, rbits, tbits, flags, codes, rscale, rmn,
                                             tscale, tmn, out_group_capacity, out_group_offset))
        return rc;
    if (Nb > 65535 * 32) return PQ_ERR_BAD_SHAPE;
    const int err = pq::launch_quantize(k, k_strides, dtype, B, Nk, Nb, rbits, tbits, flags, codes, rscale, rmn,
                                        tscale, tmn, out_group_capacity, out_group_offset,
                                        static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

}  // extern "C"

extern "C" {

int pq_selftest_quantizer_math(int dtype, uint64_t* counters, void* stream) {
    if (!counters) return PQ_ERR_NULL_POINTER;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (!aligned(counters, 8)) return PQ_ERR_MISALIGNED;
    const int err = pq::launch_selftest(dtype, reinterpret_cast<unsigned long long*>(counters),
                                        static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_decode_attn_plan(int B, int Nk, int max_groups, int n_cus) {
    if (B <= 0 || Nk <= 0 || max_groups <= 0) return 1;
    if (n_cus <= 0) n_cus = 256;
    // one wavefront per (batch, KV head, split), and the kernel keeps one wavefront per SIMD
    // (4 per CU).  Fill those slots exactly once, so that all slices run concurrently and
    // finish together; a few more blocks than slots would cost a whole second round.
    const long long slots = static_cast<long long>(n_cus) * 4;
    long long n = slots / (static_cast<long long>(B) * Nk);
    if (n < 1) n = 1;
    if (n > max_groups) n = max_groups;
    if (n > 65534) n = 65534;
    return static_cast<int>(n);
}

size_t pq_decode_attn_workspace_bytes(int B, int N, int n_splits) {
    if (B <= 0 || N <= 0 || n_splits <= 0) return 0;
    return static_cast<size_t>(B) * N * static_cast<size_t>(n_splits) * PQ_PARTIAL_FLOATS * sizeof(float);
}

}  // extern "C"

namespace {
int validate_attn(const void* q,
                  const uint8_t* codes, const void* rscale, const void* rmn,
                  const void* tscale, const void* tmn, int group_capacity,
                  int n_groups, const int32_t* n_groups_per_seq,
                  const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                  const void* v, int64_t v_capacity,
                  const uint8_t* mask, int64_t mask_stride,
                  float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                  int n_splits, int min_groups_per_split, const void* workspace, size_t workspace_bytes,
                  const void* out, unsigned flags, bool v4_entry) {
    if (!q || !v || !workspace || !out) return PQ_ERR_NULL_POINTER;
    if (int rc = check_decode_flags(flags, rbits, tbits, v4_entry ? Entry::AttentionV4 : Entry::Attention)) return rc;
    if (int rc = check_heads(B, N, Nk)) return rc;
    if (static_cast<long long>(B) * Nk > 65535) return PQ_ERR_BAD_SHAPE;
    if (int rc = check_bits(rbits, tbits)) return rc;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (group_capacity < 0 || resid_capacity < 0 || n_groups < 0 || n_resid < 0 || v_capacity <= 0)
        return PQ_ERR_BAD_STRIDE;
    // the kernels address one (batch, KV head) plane through a buffer resource with a 32-bit size and
    // 32-bit byte offsets, and park loads that must read nothing at offset 0xFFFF0000, which therefore
    // has to lie past the end of every plane: at most PQ_MAX_PLANE_TOKENS (2^24 - 256) rows of 256 bytes
    // of values or residual keys, and 2^17 groups of 8 KiB of codes
    if (v_capacity > PQ_MAX_PLANE_TOKENS || group_capacity > (1 << 17) || resid_capacity > PQ_MAX_PLANE_TOKENS)
        return PQ_ERR_BAD_SHAPE;
    const bool any_groups = n_groups_per_seq ? group_capacity > 0 : n_groups > 0;
    if (any_groups && (!codes || !rscale || !rmn || !tscale || !tmn)) return PQ_ERR_NULL_POINTER;
    const bool any_resid = n_resid_per_seq ? resid_capacity > 0 : n_resid > 0;
    if (any_resid && !k_resid) return PQ_ERR_NULL_POINTER;
    if (!n_groups_per_seq && n_groups > group_capacity) return PQ_ERR_BAD_STRIDE;
    if (!n_resid_per_seq && n_resid > resid_capacity) return PQ_ERR_BAD_STRIDE;
    if (!n_groups_per_seq && !n_resid_per_seq &&
        static_cast<int64_t>(n_groups) * PQ_GROUP + n_resid > v_capacity) return PQ_ERR_BAD_STRIDE;
    // with per-sequence counts (device arrays) the kernel clamps each sequence to the capacities instead
    if (mask && mask_stride <= 0) return PQ_ERR_BAD_STRIDE;
    if (mask && !n_groups_per_seq && !n_resid_per_seq &&
        mask_stride < static_cast<int64_t>(n_groups) * PQ_GROUP + n_resid) return PQ_ERR_BAD_STRIDE;
    if (!(sm_scale == sm_scale)) return PQ_ERR_BAD_SHAPE;
    if (n_splits < 1 || n_splits > 65534 || min_groups_per_split < 0) return PQ_ERR_WORKSPACE;
    // balanced slices: a plane shorter than a segment can still lie across one cut, i.e. two partials
    if ((flags & PQ_BALANCED_SLICES) && n_splits < 2) return PQ_ERR_WORKSPACE;
    // ... and the kernels count the batch's units (64-token tiles plus the start-up units of every plane) in 32 bits
    if ((flags & PQ_BALANCED_SLICES) &&
        (2LL * group_capacity + (resid_capacity + 63) / 64 + pq::kStartUnits) * B * Nk > 0x7fffffffLL) return PQ_ERR_BAD_SHAPE;
    if (workspace_bytes < pq_decode_attn_workspace_bytes(B, N, n_splits)) return PQ_ERR_WORKSPACE;
    // q rows are read as 16-byte pieces (operands of the residual keys' matrix product)
    if (!aligned(q, 16) || !aligned(v, 16) || !aligned(out, 2) || !aligned(workspace, 16)) return PQ_ERR_MISALIGNED;
    if (codes && !aligned(codes, 16)) return PQ_ERR_MISALIGNED;
    if (k_resid && !aligned(k_resid, 16)) return PQ_ERR_MISALIGNED;
    return PQ_OK;
}
}  // namespace

extern "C" {

int pq_validate_decode_attn(const void* q,
                            const uint8_t* codes, const void* rscale, const void* rmn,
                            const void* tscale, const void* tmn, int group_capacity,
                            int n_groups, const int32_t* n_groups_per_seq,
                            const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                            const void* v, int64_t v_capacity,
                            const uint8_t* mask, int64_t mask_stride,
                            float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                            int n_splits, int min_groups_per_split, const void* workspace, size_t workspace_bytes,
                            const void* out, unsigned flags) {
    return validate_attn(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups, n_groups_per_seq, k_resid,
                         resid_capacity, n_resid, n_resid_per_seq, v, v_capacity, mask, mask_stride, sm_scale, B, N, Nk,
                         rbits, tbits, dtype, n_splits, min_groups_per_split, workspace, workspace_bytes, out, flags, false);
}

namespace {
// The attention launch of pq_decode_attn_partials.  direct_out != nullptr (one slice per plane, default kernels): the
// kernel writes the finished output there and no partial, so that no merge has to follow.
int run_attn_partials(const void* q,
                      const uint8_t* codes, const void* rscale, const void* rmn,
                      const void* tscale, const void* tmn, int group_capacity,
                      int n_groups, const int32_t* n_groups_per_seq,
                      const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                      const void* v, int64_t v_capacity,
                      const uint8_t* mask, int64_t mask_stride,
                      float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                      int n_splits, int min_groups_per_split, void* workspace, size_t workspace_bytes,
                      unsigned flags, int32_t* status, void* stream, void* direct_out) {
    // `out` is not touched by the partials: validate with a stand-in non-null, aligned pointer
    if (int rc = pq_validate_decode_attn(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups, n_groups_per_seq,
                                         k_resid, resid_capacity, n_resid, n_resid_per_seq, v, v_capacity, mask,
                                         mask_stride, sm_scale, B, N, Nk, rbits, tbits, dtype, n_splits, min_groups_per_split,
                                         workspace, workspace_bytes, workspace, flags))
        return rc;
    if (status && !aligned(status, 4)) return PQ_ERR_MISALIGNED;
#ifdef PQ_TEST_HOOKS
    // only the float16 kernels of the test build carry the hook
    if ((flags & PQ_TEST_SILENT_SCORER) && dtype != PQ_F16) return PQ_ERR_BAD_DTYPE;
#endif
    pq::AttnArgs a;
    a.q = q; a.codes = codes; a.rscale = rscale; a.rmn = rmn; a.tscale = tscale; a.tmn = tmn;
    a.group_capacity = group_capacity; a.n_groups = n_groups; a.n_groups_per_seq = n_groups_per_seq;
    a.k_resid = k_resid; a.resid_capacity = resid_capacity; a.n_resid = n_resid; a.n_resid_per_seq = n_resid_per_seq;
    a.v = v; a.v_capacity = v_capacity; a.mask = mask; a.mask_stride = mask_stride; a.sm_scale = sm_scale;
    a.B = B; a.N = N; a.Nk = Nk; a.tbits = tbits; a.dtype = dtype; a.n_splits = n_splits;
    a.min_groups_per_split = min_groups_per_split;
    a.packed6 = (flags & PQ_CODES_PACKED6) != 0;
    a.balanced = (flags & PQ_BALANCED_SLICES) != 0;
    a.single_wave = (flags & PQ_SINGLE_WAVEFRONT) != 0;
    a.silent_scorer = (flags & PQ_TEST_SILENT_SCORER) != 0;
    a.status = status;
    a.workspace = static_cast<float*>(workspace); a.out = direct_out;
    const int err = pq::launch_attn_partials(a, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}
}  // namespace

int pq_decode_attn_partials(const void* q,
                            const uint8_t* codes, const void* rscale, const void* rmn,
                            const void* tscale, const void* tmn, int group_capacity,
                            int n_groups, const int32_t* n_groups_per_seq,
                            const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                            const void* v, int64_t v_capacity,
                            const uint8_t* mask, int64_t mask_stride,
                            float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                            int n_splits, int min_groups_per_split, void* workspace, size_t workspace_bytes,
                            unsigned flags, int32_t* status, void* stream) {
    return run_attn_partials(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups, n_groups_per_seq, k_resid,
                             resid_capacity, n_resid, n_resid_per_seq, v, v_capacity, mask, mask_stride, sm_scale, B, N, Nk,
                             rbits, tbits, dtype, n_splits, min_groups_per_split, workspace, workspace_bytes, flags, status,
                             stream, nullptr);
}

int pq_decode_attn_merge(const void* workspace, size_t workspace_bytes, int B, int N, int n_splits, int dtype,
                         void* out, void* stream) {
    if (!workspace || !out) return PQ_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0) return PQ_ERR_BAD_SHAPE;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (n_splits < 1 || n_splits > 65534) return PQ_ERR_WORKSPACE;
    if (workspace_bytes < pq_decode_attn_workspace_bytes(B, N, n_splits)) return PQ_ERR_WORKSPACE;
    if (!aligned(workspace, 16) || !aligned(out, 2)) return PQ_ERR_MISALIGNED;
    const int err = pq::launch_attn_merge(static_cast<const float*>(workspace), B, N, n_splits, dtype, out,
                                          static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_decode_attn(const void* q,
                   const uint8_t* codes, const void* rscale, const void* rmn,
                   const void* tscale, const void* tmn, int group_capacity,
                   int n_groups, const int32_t* n_groups_per_seq,
                   const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                   const void* v, int64_t v_capacity,
                   const uint8_t* mask, int64_t mask_stride,
                   float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                   int n_splits, int min_groups_per_split, void* workspace, size_t workspace_bytes,
                   void* out, unsigned flags, int32_t* status, void* stream) {
    if (!out) return PQ_ERR_NULL_POINTER;
    if (!aligned(out, 2)) return PQ_ERR_MISALIGNED;
    // one slice per plane (a batch large enough to fill the device by itself): the default kernels write the output
    // themselves and the merge launch is saved
    // (only the paired kernels do that: angle widths that run the one-wavefront kernels keep the merge)
    const bool direct = n_splits == 1 && !(flags & PQ_BALANCED_SLICES) && aligned(out, 16) &&
                        pq::attn_runs_pairs(false, (flags & PQ_SINGLE_WAVEFRONT) != 0, tbits);
    if (int rc = run_attn_partials(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups, n_groups_per_seq,
                                   k_resid, resid_capacity, n_resid, n_resid_per_seq, v, v_capacity, mask,
                                   mask_stride, sm_scale, B, N, Nk, rbits, tbits, dtype, n_splits, min_groups_per_split,
                                   workspace, workspace_bytes, flags, status, stream, direct ? out : nullptr))
        return rc;
    if (direct) return PQ_OK;
    return pq_decode_attn_merge(workspace, workspace_bytes, B, N, n_splits, dtype, out, stream);
}

int pq_decode_attn_static(const void* q,
                          const uint8_t* codes, const void* rscale, const void* rmn,
                          const void* tscale, const void* tmn, int group_capacity,
                          int n_groups, const int32_t* n_groups_per_seq,
                          const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                          const void* v, int64_t v_capacity,
                          const uint8_t* mask, int64_t mask_stride,
                          float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                          int n_splits, int min_groups_per_split, void* out, unsigned flags, int32_t* status,
                          void* stream) {
    static_assert(PQ_STATIC_MAX_PARTIALS == pq::kStaticMaxPartials, "header and library disagree");
    if (B <= 0 || N <= 0 || n_splits < 1) return PQ_ERR_BAD_SHAPE;
    if (static_cast<long long>(B) * N * n_splits > PQ_STATIC_MAX_PARTIALS) return PQ_ERR_WORKSPACE;
    float* ws = nullptr;
    if (pq::attn_static_scratch(&ws) != 0) return PQ_ERR_NO_DEVICE;
    // every (query head, slice) partial header is rewritten by each call and the merge skips the
    // body of an empty one, so nothing of the previous call's contents needs clearing
    return pq_decode_attn(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups, n_groups_per_seq, k_resid,
                          resid_capacity, n_resid, n_resid_per_seq, v, v_capacity, mask, mask_stride, sm_scale, B, N, Nk,
                          rbits, tbits, dtype, n_splits, min_groups_per_split, ws,
                          static_cast<size_t>(PQ_STATIC_MAX_PARTIALS) * PQ_PARTIAL_FLOATS * sizeof(float), out, flags, status,
                          stream);
}

// ---- fused elementwise steps of the decode layer -----------------------------------------------
int pq_rope_append(const void* q_lin, const void* k_lin, const void* v_lin, const void* cos_table, const void* sin_table,
                   int64_t table_rows, const int64_t* pos, void* q_out, void* k_dst, int64_t k_rows, const int64_t* k_row,
                   void* v_dst, int64_t v_rows, const int64_t* v_row, int B, int N, int Nk, int dtype,
                   int64_t q_row_stride, int64_t kv_row_stride, void* stream) {
    if (!q_lin || !k_lin || !v_lin || !cos_table || !sin_table || !pos || !q_out || !k_dst || !k_row || !v_dst || !v_row)
        return PQ_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || Nk <= 0 || B > 65535) return PQ_ERR_BAD_SHAPE;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (table_rows <= 0 || k_rows <= 0 || v_rows <= 0) return PQ_ERR_BAD_STRIDE;
    if (q_row_stride == 0) q_row_stride = static_cast<int64_t>(N) * PQ_HEAD_DIM;          // dense
    if (kv_row_stride == 0) kv_row_stride = static_cast<int64_t>(Nk) * PQ_HEAD_DIM;
    if (q_row_stride < static_cast<int64_t>(N) * PQ_HEAD_DIM || kv_row_stride < static_cast<int64_t>(Nk) * PQ_HEAD_DIM)
        return PQ_ERR_BAD_STRIDE;
    const int err = pq::launch_rope_append(q_lin, k_lin, v_lin, cos_table, sin_table, pos, q_out, k_dst, k_rows, k_row, v_dst,
                                           v_rows, v_row, B, N, Nk, table_rows, dtype, q_row_stride, kv_row_stride,
                                           static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_rope_qk(const void* q_lin, int64_t q_token_stride, const void* k_lin, int64_t k_token_stride, const void* cos_rows,
               const void* sin_rows, int64_t cos_sin_batch_stride, void* q_out, void* k_out, int B, int L, int N, int Nk,
               int dtype, void* stream) {
    if (!q_lin || !k_lin || !cos_rows || !sin_rows || !q_out || !k_out) return PQ_ERR_NULL_POINTER;
    if (B <= 0 || L <= 0 || N <= 0 || Nk <= 0 || static_cast<long long>(B) * L > 0x7fffffffll || N + Nk > 4096)
        return PQ_ERR_BAD_SHAPE;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (q_token_stride == 0) q_token_stride = static_cast<int64_t>(N) * PQ_HEAD_DIM;      // dense
    if (k_token_stride == 0) k_token_stride = static_cast<int64_t>(Nk) * PQ_HEAD_DIM;
    if (q_token_stride < static_cast<int64_t>(N) * PQ_HEAD_DIM || k_token_stride < static_cast<int64_t>(Nk) * PQ_HEAD_DIM ||
        (q_token_stride % 8) != 0 || (k_token_stride % 8) != 0 ||
        (cos_sin_batch_stride != 0 && (cos_sin_batch_stride < static_cast<int64_t>(L) * PQ_HEAD_DIM || (cos_sin_batch_stride % 8) != 0)))
        return PQ_ERR_BAD_STRIDE;
    if (!aligned(q_lin, 16) || !aligned(k_lin, 16) || !aligned(cos_rows, 16) || !aligned(sin_rows, 16) || !aligned(q_out, 16) ||
        !aligned(k_out, 16))
        return PQ_ERR_MISALIGNED;
    const int err = pq::launch_rope_qk(q_lin, q_token_stride, k_lin, k_token_stride, cos_rows, sin_rows, cos_sin_batch_stride,
                                       q_out, k_out, B, L, N, Nk, dtype, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_rmsnorm(const void* x, const void* residual, const void* weight, void* y, void* sum_out, int rows, int hidden,
               float eps, int dtype, void* stream) {
    if (!x || !weight || !y) return PQ_ERR_NULL_POINTER;
    if (rows <= 0 || hidden <= 0 || hidden % 8) return PQ_ERR_BAD_SHAPE;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (!aligned(x, 16) || !aligned(weight, 16) || !aligned(y, 16) || (residual && !aligned(residual, 16)) ||
        (sum_out && !aligned(sum_out, 16)))
        return PQ_ERR_MISALIGNED;
    const int err = pq::launch_rmsnorm(x, residual, weight, y, sum_out, rows, hidden, eps, dtype, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_silu_mul(const void* gate, const void* up, void* y, int rows, int cols, int64_t in_row_stride, int dtype, void* stream) {
    if (!gate || !up || !y) return PQ_ERR_NULL_POINTER;
    if (rows <= 0 || rows > 65535 || cols <= 0 || cols % 8) return PQ_ERR_BAD_SHAPE;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (in_row_stride == 0) in_row_stride = cols;                                       // dense
    if (in_row_stride < cols) return PQ_ERR_BAD_STRIDE;
    if (!aligned(gate, 16) || !aligned(up, 16) || !aligned(y, 16) || in_row_stride % 8) return PQ_ERR_MISALIGNED;
    const int err = pq::launch_silu_mul(gate, up, y, rows, cols, in_row_stride, dtype, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_convert_codes6(const uint8_t* src, uint8_t* dst, size_t n_rows, int pack, void* stream) {
    if (!src || !dst) return PQ_ERR_NULL_POINTER;
    if (n_rows == 0 || n_rows > (size_t{1} << 40)) return PQ_ERR_BAD_SHAPE;
    if (!aligned(src, pack ? 16 : 4) || !aligned(dst, pack ? 4 : 16)) return PQ_ERR_MISALIGNED;
    const int err = pq::launch_convert_codes6(src, dst, n_rows, pack != 0, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_validate_linear_small_m(const void* x, int64_t x_row_stride, const void* w, const void* w_up, const void* bias,
                               const void* y, int64_t y_row_stride, int M, int N, int K, int dtype) {
    if (!x || !w || !y) return PQ_ERR_NULL_POINTER;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (M < 1 || M > 16 || N < 16 || (N % 16) != 0 || K < 32 || (K % 32) != 0) return PQ_ERR_BAD_SHAPE;
    if (static_cast<long long>(N) * K > (1LL << 40)) return PQ_ERR_BAD_SHAPE;
    if (x_row_stride < K || (x_row_stride % 8) != 0 || y_row_stride < N || (y_row_stride % 4) != 0) return PQ_ERR_BAD_STRIDE;
    if (w_up && bias) return PQ_ERR_BAD_SHAPE;       // the gated form has no bias
    if (!aligned(x, 16) || !aligned(w, 16) || (w_up && !aligned(w_up, 16)) || !aligned(y, 8) || (bias && !aligned(bias, 2)))
        return PQ_ERR_MISALIGNED;
    return PQ_OK;
}

int pq_linear_small_m(const void* x, int64_t x_row_stride, const void* w, const void* w_up, const void* bias,
                      void* y, int64_t y_row_stride, int M, int N, int K, int dtype, void* stream) {
    const int rc = pq_validate_linear_small_m(x, x_row_stride, w, w_up, bias, y, y_row_stride, M, N, K, dtype);
    if (rc != PQ_OK) return rc;
    const int err = pq::launch_small_m_linear(x, x_row_stride, w, w_up, bias, y, y_row_stride, M, N, K, dtype,
                                              static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_validate_qkv_rope_append(const void* x, int64_t x_row_stride, const void* w_qkv, const void* bias, int M, int K,
                                int dtype, const void* cos_table, const void* sin_table, int64_t table_rows,
                                const int64_t* pos, const void* q_out, const void* k_dst, int64_t k_rows,
                                const int64_t* k_row, const void* v_dst, int64_t v_rows, const int64_t* v_row, int N, int Nk) {
    if (!x || !w_qkv || !cos_table || !sin_table || !pos || !q_out || !k_dst || !k_row || !v_dst || !v_row)
        return PQ_ERR_NULL_POINTER;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (M < 1 || M > 8 || K < 64 || (K % 64) != 0 || N < 1 || Nk < 1 || N + 2 * Nk > 8191) return PQ_ERR_BAD_SHAPE;
    if (x_row_stride < K || (x_row_stride % 8) != 0 || table_rows <= 0 || k_rows <= 0 || v_rows <= 0) return PQ_ERR_BAD_STRIDE;
    if (!aligned(x, 16) || !aligned(w_qkv, 16) || !aligned(q_out, 8) || !aligned(k_dst, 8) || !aligned(v_dst, 8) ||
        !aligned(cos_table, 2) || !aligned(sin_table, 2) || (bias && !aligned(bias, 2)) || !aligned(pos, 8) ||
        !aligned(k_row, 8) || !aligned(v_row, 8))
        return PQ_ERR_MISALIGNED;
    return PQ_OK;
}

int pq_qkv_rope_append(const void* x, int64_t x_row_stride, const void* w_qkv, const void* bias, int M, int K, int dtype,
                       const void* cos_table, const void* sin_table, int64_t table_rows, const int64_t* pos, void* q_out,
                       void* k_dst, int64_t k_rows, const int64_t* k_row, void* v_dst, int64_t v_rows,
                       const int64_t* v_row, int N, int Nk, void* stream) {
    const int rc = pq_validate_qkv_rope_append(x, x_row_stride, w_qkv, bias, M, K, dtype, cos_table, sin_table, table_rows,
                                               pos, q_out, k_dst, k_rows, k_row, v_dst, v_rows, v_row, N, Nk);
    if (rc != PQ_OK) return rc;
    const int err = pq::launch_qkv_rope_append(x, x_row_stride, w_qkv, bias, M, K, dtype, cos_table, sin_table, table_rows,
                                               pos, q_out, k_dst, k_rows, k_row, v_dst, v_rows, v_row, N, Nk,
                                               static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

// ---- 4-bit values (Mixed variant) ------------------------------------------------------------
int pq_decode_attn_v4_plan(int B, int N, int Nk, int max_groups, int n_cus) {
    if (B <= 0 || Nk <= 0 || N <= 0 || max_groups <= 0) return 1;
    if (n_cus <= 0) n_cus = 256;
    // with 4-bit values the kernel holds 32 instead of 128 registers of value operands and runs
    // two wavefronts per SIMD (for up to 4 query heads per KV head): twice the slots
    const int rep = N / Nk;
    const long long slots = static_cast<long long>(n_cus) * (pq::rep_pad(rep) <= 4 ? 8 : 4);
    long long n = slots / (static_cast<long long>(B) * Nk);
    if (n < 1) n = 1;
    if (n > max_groups) n = max_groups;
    if (n > 65534) n = 65534;
    return static_cast<int>(n);
}

int pq_validate_quantize_values(const void* v, const int64_t* v_strides, int dtype, int B, int Nk, int T,
                                const int32_t* codes, const void* scale, const void* zero,
                                int64_t out_token_capacity, int64_t out_token_offset) {
    if (!v || !v_strides || !codes || !scale || !zero) return PQ_ERR_NULL_POINTER;
    if (B <= 0 || Nk <= 0 || T <= 0 || static_cast<long long>(B) * Nk > 65535) return PQ_ERR_BAD_SHAPE;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (v_strides[3] != 1) return PQ_ERR_BAD_STRIDE;
    for (int i = 0; i < 3; i++)
        if (v_strides[i] < 0) return PQ_ERR_BAD_STRIDE;
    if (v_strides[2] < PQ_HEAD_DIM) return PQ_ERR_BAD_STRIDE;
    if (out_token_offset < 0 || out_token_capacity < out_token_offset + T) return PQ_ERR_BAD_STRIDE;
    // rows are read as 16-byte pieces
    if (!aligned(v, 16) || v_strides[0] % 8 || v_strides[1] % 8 || v_strides[2] % 8) return PQ_ERR_MISALIGNED;
    if (!aligned(codes, 4) || !aligned(scale, 2) || !aligned(zero, 2)) return PQ_ERR_MISALIGNED;
    return PQ_OK;
}

int pq_quantize_values(const void* v, const int64_t* v_strides, int dtype, int B, int Nk, int T,
                       int32_t* codes, void* scale, void* zero,
                       int64_t out_token_capacity, int64_t out_token_offset, void* stream) {
    if (int rc = pq_validate_quantize_values(v, v_strides, dtype, B, Nk, T, codes, scale, zero, out_token_capacity,
                                             out_token_offset))
        return rc;
    const int err = pq::launch_quantize_values(v, v_strides, dtype, B, Nk, T, codes, scale, zero, out_token_capacity,
                                               out_token_offset, static_cast<hipStream_t>(stream));
    return err == 0 ? PQ_OK : PQ_ERR_LAUNCH;
}

int pq_validate_decode_attn_v4(const void* q,
                               const uint8_t* codes, const void* rscale, const void* rmn,
                               const void* tscale, const void* tmn, int group_capacity,
                               int n_groups, const int32_t* n_groups_per_seq,
                               const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                               const void* v_resid,
                               const int32_t* v_codes, const void* v_scale, const void* v_zero, int64_t v4_capacity,
                               const uint8_t* mask, int64_t mask_stride,
                               float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                               int n_splits, int min_groups_per_split, const void* workspace, size_t workspace_bytes,
                               const void* out, unsigned flags) {
    // the residual window of values has the same capacity and fill as that of the keys
    const bool any_resid = n_resid_per_seq ? resid_capacity > 0 : n_resid > 0;
    if (any_resid && !v_resid) return PQ_ERR_NULL_POINTER;
    const bool any_groups = n_groups_per_seq ? group_capacity > 0 : n_groups > 0;
    if (any_groups && (!v_codes || !v_scale || !v_zero)) return PQ_ERR_NULL_POINTER;
    if (v4_capacity < 0) return PQ_ERR_BAD_STRIDE;
    // (only whole groups of the 4-bit planes are read, at most group_capacity <= 2^17 of them, so their
    // 32-bit sizes cannot wrap; the limit keeps the two value entry points alike)
    if (v4_capacity > PQ_MAX_PLANE_TOKENS) return PQ_ERR_BAD_SHAPE;
    if (!n_groups_per_seq && static_cast<int64_t>(n_groups) * PQ_GROUP > v4_capacity) return PQ_ERR_BAD_STRIDE;
    if ((v_codes && !aligned(v_codes, 4)) || (v_resid && !aligned(v_resid, 16))) return PQ_ERR_MISALIGNED;
    // everything else as in the fp16-value entry point; its V-capacity rule is met by construction here
    static const char dummy_v[16] __attribute__((aligned(16))) = {0};
    // (a stand-in, not memory: no more than the limit, so that the largest code and value stores pass as they should)
    int64_t vcap = static_cast<int64_t>(group_capacity > n_groups ? group_capacity : n_groups) * PQ_GROUP + resid_capacity + 1;
    vcap = vcap > PQ_MAX_PLANE_TOKENS ? PQ_MAX_PLANE_TOKENS : vcap;
    return validate_attn(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups, n_groups_per_seq,
                         k_resid, resid_capacity, n_resid, n_resid_per_seq, dummy_v, vcap, mask, mask_stride,
                         sm_scale, B, N, Nk, rbits, tbits, dtype, n_splits, min_groups_per_split, workspace,
                         workspace_bytes, out, flags, true);
}

int pq_decode_attn_v4(const void* q,
                      const uint8_t* codes, const void* rscale, const void* rmn,
                      const void* tscale, const void* tmn, int group_capacity,
                      int n_groups, const int32_t* n_groups_per_seq,
                      const void* k_resid, int resid_capacity, int n_resid, const int32_t* n_resid_per_seq,
                      const void* v_resid,
                      const int32_t* v_codes, const void* v_scale, const void* v_zero, int64_t v4_capacity,
                      const uint8_t* mask, int64_t mask_stride,
                      float sm_scale, int B, int N, int Nk, int rbits, int tbits, int dtype,
                      int n_splits, int min_groups_per_split, void* workspace, size_t workspace_bytes,
                      void* out, unsigned flags, int32_t* status, void* stream) {
    if (int rc = pq_validate_decode_attn_v4(q, codes, rscale, rmn, tscale, tmn, group_capacity, n_groups,
                                            n_groups_per_seq, k_resid, resid_capacity, n_resid, n_resid_per_seq,
                                            v_resid, v_codes, v_scale, v_zero, v4_capacity, mask, mask_stride, sm_scale,
                                            B, N, Nk, rbits, tbits, dtype, n_splits, min_groups_per_split, workspace,
                                            workspace_bytes, out, flags))
        return rc;
    if (status && !aligned(status, 4)) return PQ_ERR_MISALIGNED;
    const bool any_groups = n_groups_per_seq ? group_capacity > 0 : n_groups > 0;
    pq::AttnArgs a;
    a.q = q; a.codes = codes; a.rscale = rscale; a.rmn = rmn; a.tscale = tscale; a.tmn = tmn;
    a.group_capacity = group_capacity; a.n_groups = n_groups; a.n_groups_per_seq = n_groups_per_seq;
    a.k_resid = k_resid; a.resid_capacity = resid_capacity; a.n_resid = n_resid; a.n_resid_per_seq = n_resid_per_seq;
    a.mask = mask; a.mask_stride = mask_stride; a.sm_scale = sm_scale;
    a.B = B; a.N = N; a.Nk = Nk; a.tbits = tbits; a.dtype = dtype; a.n_splits = n_splits;
    a.min_groups_per_split = min_groups_per_split;
    a.packed6 = (flags & PQ_CODES_PACKED6) != 0;
    a.balanced = (flags & PQ_BALANCED_SLICES) != 0;
    a.single_wave = (flags & PQ_SINGLE_WAVEFRONT) != 0;
    a.status = status;
    a.workspace = static_cast<float*>(workspace); a.out = nullptr;
    if (any_groups) {
        a.v = v_resid; a.v_capacity = resid_capacity;      // residual rows only, row 0 = first residual token
        a.v4_codes = v_codes; a.v4_scale = v_scale; a.v4_zero = v_zero; a.v4_capacity = v4_capacity;
    } else {
        a.v = v_resid; a.v_capacity = resid_capacity;      // nothing quantized yet: the plain kernel over the window
    }
    const int err = pq::launch_attn_partials(a, static_cast<hipStream_t>(stream));
    if (err != 0) return PQ_ERR_LAUNCH;
    return pq_decode_attn_merge(workspace, workspace_bytes, B, N, n_splits, dtype, out, stream);
}

}  // extern "C"
