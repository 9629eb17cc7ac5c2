/*
 * TEST INFRASTRUCTURE ONLY -- not part of the product.
 *
 * Scalar CPU restatement of the TurboQuant V3 KV codec, used as the checker for
 * the HIP kernels (tests/, the smoke check) and as the timed CPU baseline of the
 * benchmark.  Nothing in the shipped package may link or load this file.
 *
 * Algorithm followed (upstream reference, read as text):
 *   compress    turboquant/compressors_v3.py:46-81
 *   decompress  turboquant/compressors_v3.py:84-105
 *
 * Pinned by: tests/golden/{mse_roundtrip,config1,v3}.npz (outputs of the real
 * reference on seeded inputs), by exhaustive pack/unpack checks, by brute-force
 * argmin on tiny inputs and by the independent numpy restatement in
 * oracle/tq_oracle.py.  The only float steps whose last bits the reference
 * leaves open are the summation orders inside torch.norm and sgemm (third-party
 * BLAS): those are "parity unpinned" at the 1-ulp level and are compared through
 * the decision-boundary window instead (see tqo_compress's `rotated` output).
 *
 * Build:  gcc -O2 -fopenmp -ffp-contract=off -shared -fPIC tq_oracle.c -o _build/libtq_oracle.so -lm
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

/* ---- fp16 <-> fp32, round-to-nearest-even, as torch's .to(float16) ---------- */
static uint16_t f32_to_f16_bits(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t e = (x >> 23) & 0xffu;
    uint32_t m = x & 0x7fffffu;
    if (e == 0xff) return (uint16_t)(sign | 0x7c00u | (m ? 0x200u | (m >> 13) : 0));
    int32_t exp = (int32_t)e - 127 + 15;
    if (exp >= 31) return (uint16_t)(sign | 0x7c00u);          /* overflow -> inf */
    if (exp <= 0) {                                           /* subnormal / zero */
        if (exp < -10) return (uint16_t)sign;
        m |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - exp);
        uint32_t h = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)exp << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;   /* may carry into exponent: correct */
    return (uint16_t)(sign | h);
}

static float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) { x = sign; }
        else {
            int s = 0;
            while (!(m & 0x400u)) { m <<= 1; s++; }
            m &= 0x3ffu;
            x = sign | ((uint32_t)(127 - 15 - s + 1) << 23) | (m << 13);
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e - 15 + 127) << 23) | (m << 13);
    }
    float f; memcpy(&f, &x, 4);
    return f;
}

void tqo_f32_to_f16(const float *src, uint16_t *dst, long long n) {
    for (long long i = 0; i < n; i++) dst[i] = f32_to_f16_bits(src[i]);
}
void tqo_f16_to_f32(const uint16_t *src, float *dst, long long n) {
    for (long long i = 0; i < n; i++) dst[i] = f16_bits_to_f32(src[i]);
}

/* indices per byte = floor(8 / bits); bytes per vector = ceil(D / ipb)  (compressors_v3.py:64-69) */
int tqo_indices_per_byte(int bits) { return (bits >= 1 && bits <= 8) ? 8 / bits : 0; }
long long tqo_bytes_per_vector(int D, int bits) {
    int ipb = tqo_indices_per_byte(bits);
    return ipb ? (D + ipb - 1) / ipb : -1;
}

/* nearest centroid, first minimum wins on ties (argmin semantics, compressors_v3.py:60-61) */
static inline int nearest(float r, const float *cent, int L) {
    int best = 0;
    float bd = fabsf(r - cent[0]);
    for (int j = 1; j < L; j++) {
        float dj = fabsf(r - cent[j]);
        if (dj < bd) { bd = dj; best = j; }
    }
    return best;
}
void tqo_nearest(const float *r, long long n, const float *cent, int L, uint8_t *idx) {
    for (long long i = 0; i < n; i++) idx[i] = (uint8_t)nearest(r[i], cent, L);
}

/* MSB-first packing of one vector's indices (compressors_v3.py:64-74) */
void tqo_pack(const uint8_t *idx, int D, int bits, uint8_t *out) {
    int ipb = 8 / bits;
    int G = (D + ipb - 1) / ipb;
    for (int g = 0; g < G; g++) {
        unsigned v = 0;
        for (int k = 0; k < ipb; k++) {
            int c = g * ipb + k;
            unsigned code = c < D ? idx[c] : 0u;           /* zero padding, :65-68 */
            v += code << (bits * (ipb - 1 - k));
        }
        out[g] = (uint8_t)v;                               /* .to(uint8) wraps mod 256 */
    }
}
/* inverse (compressors_v3.py:93-101) */
void tqo_unpack(const uint8_t *bytes, int D, int bits, uint8_t *idx) {
    int ipb = 8 / bits;
    unsigned mask = (1u << bits) - 1u;
    for (int c = 0; c < D; c++) {
        int g = c / ipb, k = c % ipb;
        idx[c] = (uint8_t)((bytes[g] >> (bits * (ipb - 1 - k))) & mask);
    }
}

/*
 * compress: x [N,D] fp32 (callers widen fp16/bf16 exactly) ->
 *   idx_bytes [N,G] u8, norms [N] fp16 bits, optionally rotated [N,D] fp32
 *   (the unit-sphere coordinates the codes were chosen from, so a checker can
 *   measure the distance to the nearest decision boundary).
 * accum_double = 0: float accumulation throughout, like the reference's fp32 ops.
 * accum_double = 1: the D-term dot products are summed in double and rounded
 *   once, giving the centre of the rounding-error cloud any fp32 order lands in.
 */
int tqo_compress(const float *x, long long N, int D, const float *Pi, const float *cent,
                 int bits, int accum_double, uint8_t *idx_bytes, uint16_t *norms, float *rotated) {
    if (bits < 1 || bits > 8 || D < 1 || D > 4096 || N < 0) return -1;
    const int L = 1 << bits;
    const long long G = tqo_bytes_per_vector(D, bits);
    int fail = 0;
#pragma omp parallel
    {
        float *u = (float *)malloc(sizeof(float) * (size_t)D * 2);
        uint8_t *codes = (uint8_t *)malloc((size_t)D);
        if (!u || !codes) {
#pragma omp atomic write
            fail = 1;
        } else {
            float *r = u + D;
#pragma omp for schedule(static)
            for (long long n = 0; n < N; n++) {
                const float *xv = x + n * (long long)D;
                float nrm;
                if (accum_double) {
                    double s = 0.0;
                    for (int k = 0; k < D; k++) s += (double)xv[k] * (double)xv[k];
                    nrm = (float)sqrt(s);
                } else {
                    float s = 0.0f;
                    for (int k = 0; k < D; k++) s += xv[k] * xv[k];
                    nrm = sqrtf(s);
                }
                const float denom = nrm + 1e-8f;                 /* :56 eps on the divisor only */
                for (int k = 0; k < D; k++) u[k] = xv[k] / denom;
                for (int j = 0; j < D; j++) {                    /* rotated = u @ Pi.T  (:59) */
                    const float *row = Pi + (long long)j * D;
                    if (accum_double) {
                        double s = 0.0;
                        for (int k = 0; k < D; k++) s += (double)u[k] * (double)row[k];
                        r[j] = (float)s;
                    } else {
                        float s = 0.0f;
                        for (int k = 0; k < D; k++) s += u[k] * row[k];
                        r[j] = s;
                    }
                    codes[j] = (uint8_t)nearest(r[j], cent, L);
                }
                tqo_pack(codes, D, bits, idx_bytes + n * G);
                norms[n] = f32_to_f16_bits(nrm);                 /* :78 */
                if (rotated) memcpy(rotated + n * (long long)D, r, sizeof(float) * (size_t)D);
            }
        }
        free(u); free(codes);
    }
    return fail ? -2 : 0;
}

/* decompress: idx_bytes [N,G], norms [N] fp16 bits -> out [N,D] fp32 (compressors_v3.py:84-105) */
int tqo_decompress(const uint8_t *idx_bytes, const uint16_t *norms, long long N, int D,
                   const float *Pi, const float *cent, int bits, int accum_double, float *out) {
    if (bits < 1 || bits > 8 || D < 1 || D > 4096 || N < 0) return -1;
    const long long G = tqo_bytes_per_vector(D, bits);
    int fail = 0;
#pragma omp parallel
    {
        float *y = (float *)malloc(sizeof(float) * (size_t)D);
        uint8_t *codes = (uint8_t *)malloc((size_t)D);
        double *accd = (double *)malloc(sizeof(double) * (size_t)D);
        float *accf = (float *)malloc(sizeof(float) * (size_t)D);
        if (!y || !codes || !accd || !accf) {
#pragma omp atomic write
            fail = 1;
        } else {
#pragma omp for schedule(static)
            for (long long n = 0; n < N; n++) {
                tqo_unpack(idx_bytes + n * G, D, bits, codes);
                for (int j = 0; j < D; j++) y[j] = cent[codes[j]];
                const float nrm = f16_bits_to_f32(norms[n]);
                float *o = out + n * (long long)D;
                /* reconstructed = (y @ Pi) * norm : out[k] = sum_j y[j] * Pi[j][k] */
                if (accum_double) {
                    for (int k = 0; k < D; k++) accd[k] = 0.0;
                    for (int j = 0; j < D; j++) {
                        const float *row = Pi + (long long)j * D;
                        const double yj = y[j];
                        for (int k = 0; k < D; k++) accd[k] += yj * (double)row[k];
                    }
                    for (int k = 0; k < D; k++) o[k] = (float)accd[k] * nrm;
                } else {
                    for (int k = 0; k < D; k++) accf[k] = 0.0f;
                    for (int j = 0; j < D; j++) {
                        const float *row = Pi + (long long)j * D;
                        const float yj = y[j];
                        for (int k = 0; k < D; k++) accf[k] += yj * row[k];
                    }
                    for (int k = 0; k < D; k++) o[k] = accf[k] * nrm;
                }
            }
        }
        free(y); free(codes); free(accd); free(accf);
    }
    return fail ? -2 : 0;
}

#ifdef _OPENMP
#include <omp.h>
int tqo_max_threads(void) { return omp_get_max_threads(); }
void tqo_set_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int tqo_max_threads(void) { return 1; }
void tqo_set_threads(int n) { (void)n; }
#endif
