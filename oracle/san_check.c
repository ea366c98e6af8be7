/* Runs the oracle's functions over small ragged shapes with exactly sized heap buffers, for a build with the
 * address and undefined-behaviour sanitizers (make -C oracle san): an access past a buffer or a shift or
 * conversion with undefined behaviour in the restatement ends the run with a report. Test infrastructure, like
 * the oracle itself. Prints a checksum so that nothing is optimised away. */
#include "mtq_oracle.c"

#include <stdio.h>

static uint64_t rng_state = 0x243F6A8885A308D3ull;
static uint32_t rnd(void) {
    rng_state ^= rng_state >> 12;
    rng_state ^= rng_state << 25;
    rng_state ^= rng_state >> 27;
    return (uint32_t)((rng_state * 0x2545F4914F6CDD1Dull) >> 32);
}
static float rndf(void) { return (float)(rnd() >> 8) / 8388608.0f - 1.0f; }
static float *falloc(size_t n) {
    float *p = (float *)malloc((n ? n : 1) * sizeof(float));
    for (size_t i = 0; i < n; i++) p[i] = rndf();
    return p;
}
static uint32_t *walloc(size_t n) {
    uint32_t *p = (uint32_t *)malloc((n ? n : 1) * sizeof(uint32_t));
    for (size_t i = 0; i < n; i++) p[i] = rnd();
    return p;
}

int main(void) {
    double sum = 0.0;
    for (uint32_t bits = 2; bits <= 8; bits++) {
        const size_t G = 32, K = 96, N = 5, M = 3, E = 3, T = 7;   /* K * bits % 32 == 0 for every width */
        const size_t wpr = K * bits / 32, gpr = K / G;
        uint32_t *w = walloc(E * N * wpr);
        float *s = falloc(E * N * gpr), *b = falloc(E * N * gpr), *x = falloc(T * K);
        float *o = falloc(T * N);
        double *o64 = (double *)malloc(T * N * sizeof(double));
        mtq_oracle_qmm(w, s, b, x, M, N, K, bits, G, o, 1);
        sum += o[M * N - 1];
        mtq_oracle_qmm(w, s, b, x, M, N, K, bits, G, o, 3);
        mtq_oracle_qmm_f64(w, s, b, x, M, N, K, bits, G, o64, 2);
        sum += o64[M * N - 1];
        for (int dt = 0; dt < 3; dt++) {
            mtq_oracle_qmm_mma(w, s, b, x, M, N, K, bits, G, dt, o64, 2);
            sum += o64[0];
        }
        uint32_t off[4] = {0, 2, 2, 5};           /* expert 1 empty, rows 5 and 6 past every offset */
        uint32_t idx[7] = {2, 0, 1, 1, 0, 2, 0};
        mtq_oracle_gather_qmm(x, w, s, b, off, NULL, T, K, N, E, bits, G, o, o64, 2);
        sum += o[T * N - 1];
        mtq_oracle_gather_qmm(x, w, s, b, NULL, idx, T, K, N, E, bits, G, o, NULL, 1);
        sum += o[0];
        /* qvm: W [K][N] packed along N, N * bits % 32 == 0 */
        const size_t Nv = 32, Kv = 64;
        uint32_t *wv = walloc(Kv * Nv * bits / 32);
        float *sv = falloc(Kv / G * Nv), *bv = falloc(Kv / G * Nv), *xv = falloc(2 * Kv), *ov = falloc(2 * Nv);
        mtq_oracle_qvm(wv, sv, bv, xv, 2, Nv, Kv, bits, G, ov, NULL);
        sum += ov[2 * Nv - 1];
        /* codes: unpack, pack back, same words */
        uint8_t *codes = (uint8_t *)malloc(N * K);
        uint32_t *w2 = walloc(N * wpr);
        mtq_oracle_unpack_codes(w, N, K, bits, codes);
        mtq_oracle_pack_codes(codes, N, K, bits, w2);
        if (memcmp(w, w2, N * wpr * 4) != 0) { fprintf(stderr, "pack(unpack(w)) != w at %u bits\n", bits); return 1; }
        /* affine quantize / dequantize of 6 groups */
        float *v = falloc(6 * G), *qs = falloc(6), *qb = falloc(6), *dq = falloc(6 * G);
        uint8_t *qc = (uint8_t *)malloc(6 * G);
        for (int dt = 0; dt < 3; dt++) mtq_oracle_affine_quantize(v, 6, G, bits, dt, qc, qs, qb);
        uint32_t *qw = walloc(6 * G * bits / 32);
        mtq_oracle_pack_codes(qc, 1, 6 * G, bits, qw);
        mtq_oracle_affine_dequantize(qw, qs, qb, 6 * G, G, bits, dq);
        sum += dq[6 * G - 1];
        free(w); free(s); free(b); free(x); free(o); free(o64); free(wv); free(sv); free(bv); free(xv); free(ov);
        free(codes); free(w2); free(v); free(qs); free(qb); free(dq); free(qc); free(qw);
    }
    /* conversions over awkward values */
    const float specials[] = {0.0f, -0.0f, 1.0f, 65504.0f, 65520.0f, 1e-8f, 6e-8f, 3.3895314e38f, -1e30f, 1.0f / 0.0f};
    for (size_t i = 0; i < sizeof(specials) / sizeof(specials[0]); i++) {
        sum += mtq_oracle_bf16_to_f32(mtq_oracle_f32_to_bf16(specials[i])) == specials[i];
        sum += mtq_oracle_f16_to_f32(mtq_oracle_f32_to_f16(specials[i])) == specials[i];
    }
    double st[7], samples[5] = {3.0, 1.0, 2.0, 5.0, 4.0};
    mtq_oracle_bench_stats(samples, 5, st);
    sum += st[0];
    printf("oracle san_check: ok (%g)\n", sum);
    return 0;
}
