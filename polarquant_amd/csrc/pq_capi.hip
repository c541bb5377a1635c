// C ABI of the polar-key decode path: host-side argument validation and
// dispatch to the kernel launchers.  Declarations and the reference interfaces
// they replace are in include/polarquant.h.
#include "../../include/polarquant.h"
#include "pq_internal.h"

namespace {

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int check_bits(int rbits, int tbits) {
    if (rbits < 1 || tbits < 1 || rbits + tbits > 8) return PQ_ERR_BAD_BITS;
    if (tbits > 4) return PQ_ERR_BAD_BITS;  // the angle table is sized for at most 16 bins
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
        case PQ_ERR_BAD_BITS: return "bad bit widths (need 1 <= tbits <= 4, rbits >= 1, rbits + tbits <= 8)";
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
                              int B, int N, int Nk, int Nb, int rbits, int tbits, int dtype) {
    if (!q || !codes || !rscale || !rmn || !tscale || !tmn || !out) return PQ_ERR_NULL_POINTER;
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
                     int B, int N, int Nk, int Nb, int rbits, int tbits, int dtype, void* stream) {
    if (int rc = pq_validate_decode_scores(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, rbits, tbits, dtype))
        return rc;
    // grid is (Nb, B*Nk): y is limited to 65535 blocks
    if (static_cast<long long>(B) * Nk > 65535) return PQ_ERR_BAD_SHAPE;
    const int err = pq::launch_scores(q, codes, rscale, rmn, tscale, tmn, out, B, N, Nk, Nb, tbits, dtype,
                                      static_cast<hipStream_t>(stream));
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
    if (rbits < 1 || tbits < 1 || rbits + tbits > 8) return PQ_ERR_BAD_BITS;
    if (dtype != PQ_F16 && dtype != PQ_BF16) return PQ_ERR_BAD_DTYPE;
    if (flags & ~static_cast<unsigned>(PQ_WRAP_FP32)) return PQ_ERR_BAD_SHAPE;
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

// ---- TEMPORARY: remaining entry points are filled in next ----
extern "C" {
int pq_decode_attn(const void*, const uint8_t*, const void*, const void*, const void*, const void*, int, int, const int32_t*, const void*, int, int, const int32_t*, const void*, int64_t, const uint8_t*, int64_t, float, int, int, int, int, int, int, int, void*, size_t, void*, void*) { return PQ_ERR_LAUNCH; }
int pq_validate_decode_attn(const void*, const uint8_t*, const void*, const void*, const void*, const void*, int, int, const int32_t*, const void*, int, int, const int32_t*, const void*, int64_t, const uint8_t*, int64_t, float, int, int, int, int, int, int, int, const void*, size_t, const void*) { return PQ_ERR_LAUNCH; }
int pq_decode_attn_plan(int, int, int, int) { return 1; }
size_t pq_decode_attn_workspace_bytes(int, int, int) { return 0; }
}
