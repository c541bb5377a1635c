/* A plain C program against include/polarquant.h and libpolarquant_hip.so: the header must compile
 * as C, the library must link without Python or torch, and the host-only entry points must work
 * with no GPU present.  Built and run by tests/test_capi_cpu.py. */
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "polarquant.h"

int main(void) {
    static char buf[64] __attribute__((aligned(16)));
    void *p = buf;
    int64_t strides[4] = {8 * 256 * 128, 256 * 128, 128, 1};
    if (pq_version() <= 0) return 1;
    if (strcmp(pq_status_string(PQ_OK), pq_status_string(PQ_ERR_BAD_BITS)) == 0) return 2;
    if (pq_validate_decode_scores(p, p, p, p, p, p, p, 2, 32, 8, 4, 4, 4, PQ_F16, 0) != PQ_OK) return 3;
    if (pq_validate_decode_scores(NULL, p, p, p, p, p, p, 2, 32, 8, 4, 4, 4, PQ_F16, 0) != PQ_ERR_NULL_POINTER) return 4;
    if (pq_validate_quantize_groups(p, strides, PQ_BF16, 2, 8, 2, 4, 4, PQ_ANGLE_UNIFORM, p, p, p, p, p, 2, 0) != PQ_OK) return 5;
    if (pq_validate_quantize_groups(p, strides, PQ_BF16, 2, 8, 2, 5, 4, 0, p, p, p, p, p, 2, 0) != PQ_ERR_BAD_BITS) return 6;
    if (pq_validate_quantize_values(p, strides, PQ_F16, 2, 8, 256, p, p, p, 256, 0) != PQ_OK) return 7;
    if (pq_decode_attn_plan(16, 8, 256, 256) != 8 || pq_decode_attn_v4_plan(16, 32, 8, 256, 256) != 16) return 8;
    if (pq_decode_attn_workspace_bytes(2, 32, 4) != (size_t)2 * 32 * 4 * PQ_PARTIAL_FLOATS * sizeof(float)) return 9;
    /* the compute entry points refuse bad arguments before touching the device */
    if (pq_rmsnorm(NULL, NULL, p, p, NULL, 1, 128, 1e-5f, PQ_F16, NULL) != PQ_ERR_NULL_POINTER) return 10;
    if (pq_decode_attn(NULL, p, p, p, p, p, 4, 3, NULL, p, 128, 5, NULL, p, 1024, NULL, 0, 0.088f, 2, 32, 8, 4, 4, PQ_F16, 4, 0,
                       p, 1u << 20, p, 0, NULL, NULL) != PQ_ERR_NULL_POINTER) return 11;
    if (pq_validate_decode_scores(p, p, p, p, p, p, p, 2, 28, 4, 4, 3, 3, PQ_F16, PQ_CODES_PACKED6) != PQ_OK) return 12;
    if (pq_validate_decode_scores(p, p, p, p, p, p, p, 2, 28, 4, 4, 4, 4, PQ_F16, PQ_CODES_PACKED6) != PQ_ERR_BAD_BITS) return 13;
    printf("capi ok, version %d, group %d, head_dim %d\n", pq_version(), PQ_GROUP, PQ_HEAD_DIM);
    return 0;
}
