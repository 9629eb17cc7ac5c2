/* Test infrastructure: a driver that runs every function of tq_oracle.c on small, ragged inputs, meant to be built
 * with -fsanitize=address,undefined (tests/test_oracle.py does that and runs it).  It checks only what the sanitizers
 * cannot: that packing round-trips and that compress -> decompress returns something of the right size; the numerical
 * pins of the oracle live in tests/test_oracle.py. */
#include "tq_oracle.c"

#include <stdio.h>
#include <stdlib.h>

static unsigned long long rng_state = 0x9e3779b97f4a7c15ull;
static float rnd(void) {   /* uniform in (-1, 1) */
    rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((double)(rng_state >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

int main(void) {
    const int dims[] = {1, 6, 7, 64, 128, 130};
    for (unsigned di = 0; di < sizeof(dims) / sizeof(dims[0]); ++di) {
        const int D = dims[di];
        for (int bits = 1; bits <= 8; ++bits) {
            const int L = 1 << bits, N = 37;
            const long long G = tqo_bytes_per_vector(D, bits);
            if (G <= 0 || tqo_indices_per_byte(bits) <= 0) { fprintf(stderr, "size arithmetic D=%d bits=%d\n", D, bits); return 1; }
            float *Pi = malloc(sizeof(float) * D * D), *cent = malloc(sizeof(float) * L), *x = malloc(sizeof(float) * N * D);
            float *rot = malloc(sizeof(float) * N * D), *rec = malloc(sizeof(float) * N * D);
            uint8_t *bytes = malloc((size_t)N * G), *idx = malloc(D), *idx2 = malloc(D), *one = malloc(G);
            uint16_t *norms = malloc(sizeof(uint16_t) * N);
            for (int i = 0; i < D * D; ++i) Pi[i] = (i / D == i % D) ? 1.f : 0.01f * rnd();
            for (int i = 0; i < L; ++i) cent[i] = -1.f + 2.f * (i + 0.5f) / L;
            for (int i = 0; i < N * D; ++i) x[i] = rnd() * (i % 11 == 0 ? 1e4f : 1.f);
            for (int i = 0; i < D; ++i) x[i] = 0.f;                         /* the all-zero vector */
            for (int i = 0; i < D; ++i) idx[i] = (uint8_t)((i * 7 + bits) & (L - 1));
            tqo_pack(idx, D, bits, one);
            tqo_unpack(one, D, bits, idx2);
            for (int i = 0; i < D; ++i)
                if (idx[i] != idx2[i]) { fprintf(stderr, "pack/unpack D=%d bits=%d at %d\n", D, bits, i); return 1; }
            for (int dbl = 0; dbl < 2; ++dbl) {
                if (tqo_compress(x, N, D, Pi, cent, bits, dbl, bytes, norms, rot)) { fprintf(stderr, "compress failed\n"); return 1; }
                if (tqo_compress(x, N, D, Pi, cent, bits, dbl, bytes, norms, NULL)) { fprintf(stderr, "compress failed\n"); return 1; }
                if (tqo_decompress(bytes, norms, N, D, Pi, cent, bits, dbl, rec)) { fprintf(stderr, "decompress failed\n"); return 1; }
            }
            for (int i = 0; i < D; ++i)
                if (rec[i] != 0.f) { fprintf(stderr, "zero vector D=%d bits=%d\n", D, bits); return 1; }
            uint8_t *codes = malloc((size_t)N * D);
            tqo_nearest(rot, (long long)N * D, cent, L, codes);
            free(codes);
            free(Pi); free(cent); free(x); free(rot); free(rec); free(bytes); free(idx); free(idx2); free(one); free(norms);
        }
    }
    /* every fp16 bit pattern through both conversions */
    uint16_t *h = malloc(65536 * sizeof(uint16_t)), *h2 = malloc(65536 * sizeof(uint16_t));
    float *f = malloc(65536 * sizeof(float));
    for (int i = 0; i < 65536; ++i) h[i] = (uint16_t)i;
    tqo_f16_to_f32(h, f, 65536);
    tqo_f32_to_f16(f, h2, 65536);
    for (int i = 0; i < 65536; ++i) {
        const int nan = (i & 0x7c00) == 0x7c00 && (i & 0x3ff);
        if (!nan && h[i] != h2[i]) { fprintf(stderr, "fp16 round trip at %04x\n", i); return 1; }
    }
    free(h); free(h2); free(f);
    tqo_set_threads(tqo_max_threads());
    puts("ok");
    return 0;
}
