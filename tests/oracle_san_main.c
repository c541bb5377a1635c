/* Drives the plain-C oracle on small seeded inputs; built with -fsanitize=address,undefined by
 * tests/test_oracle_sanitizers.py.  Prints a checksum so that the run cannot be optimised away. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

int po_quantize(const uint16_t *k, int bf, int flags, int B, int Nk, int L, int D, int G, int rbits, int tbits,
                uint8_t *codes, uint16_t *rscale, uint16_t *rmn, uint16_t *tscale, uint16_t *tmn);
int po_scores(const uint16_t *q, int bf, const uint8_t *codes, const uint16_t *rscale, const uint16_t *rmn,
              const uint16_t *tscale, const uint16_t *tmn, float *out, int B, int N, int Nk, int Nb, int G, int D,
              int rbits, int tbits);
int po_quantize_values(const uint16_t *v, int bf, long rows, int D, int bits, int32_t *codes, uint16_t *scale, uint16_t *mn);
uint16_t po_float_to_half(float f);

static uint32_t rng = 12345u;
static float frand(void) { rng = rng * 1664525u + 1013904223u; return ((rng >> 8) / 8388608.0f) - 1.0f; }

int main(void) {
    enum { B = 2, N = 4, Nk = 2, L = 256, D = 64, G = 128, Nb = L / G };
    uint16_t *k = malloc(sizeof(uint16_t) * B * Nk * L * 2 * D), *q = malloc(sizeof(uint16_t) * B * N * 2 * D);
    for (int i = 0; i < B * Nk * L * 2 * D; i++) k[i] = po_float_to_half(3.0f * frand());
    for (int i = 0; i < 2 * D; i++) k[i] = po_float_to_half(0.5f);            /* a constant pair column start: degenerate paths */
    for (int i = 0; i < B * N * 2 * D; i++) q[i] = po_float_to_half(frand());
    uint8_t *codes = malloc((size_t)B * Nk * Nb * G * D);
    uint16_t *meta[4];
    for (int i = 0; i < 4; i++) meta[i] = malloc(sizeof(uint16_t) * B * Nk * Nb * D);
    float *out = malloc(sizeof(float) * B * N * L);
    int32_t *vc = malloc(sizeof(int32_t) * B * Nk * L * 16);
    uint16_t *vs = malloc(sizeof(uint16_t) * B * Nk * L), *vm = malloc(sizeof(uint16_t) * B * Nk * L);
    double sum = 0;
    for (int flags = 0; flags < 4; flags++)
        for (int bits = 3; bits <= 4; bits++) {
            if (po_quantize(k, 0, flags, B, Nk, L, D, G, bits, bits, codes, meta[0], meta[1], meta[2], meta[3])) return 1;
            if (po_scores(q, 0, codes, meta[0], meta[1], meta[2], meta[3], out, B, N, Nk, Nb, G, D, bits, bits)) return 2;
            for (int i = 0; i < B * N * L; i++) sum += out[i];
        }
    if (po_quantize_values(k, 0, (long)B * Nk * L, 2 * D, 4, vc, vs, vm)) return 3;
    for (int i = 0; i < B * Nk * L * 16; i++) sum += (double)(vc[i] & 0xff);
    printf("checksum %.6e\n", sum);
    free(k); free(q); free(codes); free(out); free(vc); free(vs); free(vm);
    for (int i = 0; i < 4; i++) free(meta[i]);
    return 0;
}
