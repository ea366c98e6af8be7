/*
 * mtq_oracle.c -- CPU restatement of metaltile-std's affine-quantized matmul
 * reference semantics.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are
 * compared against and the "cpu_baseline" leg of the benchmark. Nothing in
 * the shipped library links, loads or calls it: only tests/, the smoke check
 * and bench.py's cpu_baseline may use it.
 *
 * Every function cites the reference file:line (relative to the reference
 * checkout root) whose algorithm it restates. The reference is Rust; Rust
 * never contracts a*b+c into an FMA, so this file must be compiled with
 * -ffp-contract=off to keep the same f32 rounding sequence.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   dtype packers     reference unit-test values (utils.rs:72-127), exhaustive
 *                     bf16/f16 round trips, numpy's IEEE float16 as a second
 *                     implementation, closed-form ties-to-even cases.
 *   code extraction   brute force against a pure-Python bit-stream reader,
 *                     pack(unpack) identity, all bit widths 2..8.
 *   qmm / gemv        numpy f64 `X @ dequant(W).T` (library matmul), closed
 *                     forms (all-zero codes, unit scale constant code),
 *                     linearity, M=1 qmm == qmv, split form == direct form.
 *   gather / expert   single expert == plain qmm, CSR == indices after
 *                     expansion, row permutation, expert e == slab e gemv.
 *   quantize          round trip within one step, constant group -> scale 1.
 *   rms_norm_qgemv    numpy restatement (dequant matrix @ normalised row), unit norm
 *                     weights with a constant row (inv_rms in closed form), scale
 *                     invariance in x, eps -> large limit.
 *   gated_rms_norm_qgemv  numpy f64 restatement with the library's logistic function; one row with a constant
 *                     gate == that gate x the (pinned) rms_norm_qgemv; z = 0 -> zero output; silu(ln 3) = 0.75 ln 3;
 *                     scaling one row of y leaves the output unchanged at eps = 0 (the sums of squares are per
 *                     row); norm weights repeat per row (index d, not r * dv + d).
 *   dequant_gather    (oracle.py: the pinned dequantiser over the table and a numpy row take) brute-force bit
 *                     extraction per element on the reference test's table generator.
 *   qvm               numpy f64 `x @ dequant(W)` on the [K, N] layout, and qvm(W) == qmv of the
 *                     transposed, repacked matrix.
 *   moe routing       numpy stable argsort + library softmax, the reference tests' tie-break,
 *                     k = 1 and NaN/Inf cases; unpermute against a numpy einsum; permute and
 *                     the expert sort are numpy one-liners (take, stable argsort) in oracle.py.
 *   moe_down_swiglu   numpy silu + the (pinned) expert-indexed GEMV + numpy slot sum; one slot with
 *                     weight 1 == expert-indexed GEMV of the swiglu row; zero gates -> zero output.
 *   stats             reference unit-test values (stats.rs:57-84).
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MTQ_ORACLE_API __attribute__((visibility("default")))

enum { MTQ_F32 = 0, MTQ_F16 = 1, MTQ_BF16 = 2 };

/* ------------------------------------------------------------------ */
/* dtype conversion                                                    */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float v) { uint32_t u; memcpy(&u, &v, 4); return u; }
static inline float bits_f32(uint32_t u) { float v; memcpy(&v, &u, 4); return v; }

/* f32 -> bf16, round to nearest even on the raw bits.
 * Reference: crates/metaltile-std/src/runner.rs:521-525 (f32_to_bf16), the same
 * rule the `half` crate applies for every non-NaN input (utils.rs:29). NaN is
 * quieted instead of rounded so it cannot turn into Inf. */
MTQ_ORACLE_API uint16_t mtq_oracle_f32_to_bf16(float v) {
    uint32_t x = f32_bits(v);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t r = x + 0x7FFFu + ((x >> 16) & 1u);
    return (uint16_t)(r >> 16);
}

/* bf16 -> f32. Reference: crates/metaltile-std/src/runner.rs:387 (bits << 16). */
MTQ_ORACLE_API float mtq_oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* f32 -> f16, IEEE round to nearest even INCLUDING subnormal results.
 * Reference: crates/metaltile-std/src/utils.rs:28 packs through
 * `half::f16::from_f32`, which is IEEE RNE with gradual underflow; the
 * hand-rolled runner.rs:498-519 agrees for every normal result and differs
 * only by flushing subnormal results to zero. The packer on the test/bench
 * path is utils.rs, so that behaviour is the one restated here. */
MTQ_ORACLE_API uint16_t mtq_oracle_f32_to_f16(float v) {
    uint32_t x = f32_bits(v);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x1FFu)); /* NaN */
    if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536 -> Inf (incl. Inf) */
    if (ax >= 0x38800000u) { /* normal f16 result: exponent >= -14 */
        uint32_t mant = ax & 0x7FFFFFu;
        uint32_t e16 = (ax >> 23) - 112u; /* rebias 127 -> 15 */
        uint32_t h = (e16 << 10) | (mant >> 13);
        uint32_t rem = mant & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++; /* may carry into exponent/Inf */
        return (uint16_t)(sign | h);
    }
    if (ax < 0x33000000u) return sign; /* < 2^-25 rounds to zero */
    /* subnormal f16 result: value = m * 2^-24, m in [0,1024) */
    uint32_t e = ax >> 23;                     /* biased f32 exponent, 102..112 */
    uint32_t mant = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t shift = 126u - e;                 /* 14..24 */
    uint32_t h = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

/* f16 -> f32, exact (subnormals preserved), as `half::f16::to_f32`
 * (crates/metaltile-std/src/utils.rs:50). */
MTQ_ORACLE_API float mtq_oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0x1Fu) return bits_f32(sign | 0x7F800000u | (m << 13));
    if (e != 0) return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
    if (m == 0) return bits_f32(sign);
    float mag = (float)m * 5.9604644775390625e-08f; /* m * 2^-24, exact */
    return bits_f32(f32_bits(mag) | sign);
}



/* pack_f32: f32 values -> little-endian bytes of dtype `dt`.
 * Reference: crates/metaltile-std/src/utils.rs:26-37. */
MTQ_ORACLE_API void mtq_oracle_pack_f32(const float *vals, size_t n, int dt, void *out) {
    if (dt == MTQ_F32) { memcpy(out, vals, n * 4); return; }
    uint16_t *o = (uint16_t *)out;
    for (size_t i = 0; i < n; i++)
        o[i] = dt == MTQ_F16 ? mtq_oracle_f32_to_f16(vals[i]) : mtq_oracle_f32_to_bf16(vals[i]);
}

/* unpack_f32: inverse of pack_f32. Reference: crates/metaltile-std/src/utils.rs:46-65. */
MTQ_ORACLE_API void mtq_oracle_unpack_f32(const void *bytes, size_t n, int dt, float *out) {
    if (dt == MTQ_F32) { memcpy(out, bytes, n * 4); return; }
    const uint16_t *b = (const uint16_t *)bytes;
    for (size_t i = 0; i < n; i++)
        out[i] = dt == MTQ_F16 ? mtq_oracle_f16_to_f32(b[i]) : mtq_oracle_bf16_to_f32(b[i]);
}

/* Round an f32 array through dtype `dt` in place (the reference's
 * `unpack_f32(&pack_f32(v, dt), dt)`, crates/metaltile-std/src/mlx/quantized.rs:5428-5430). */
MTQ_ORACLE_API void mtq_oracle_round_through(float *vals, size_t n, int dt) {
    if (dt == MTQ_F32) return;
    for (size_t i = 0; i < n; i++)
        vals[i] = dt == MTQ_F16 ? mtq_oracle_f16_to_f32(mtq_oracle_f32_to_f16(vals[i]))
                                : mtq_oracle_bf16_to_f32(mtq_oracle_f32_to_bf16(vals[i]));
}

/* ------------------------------------------------------------------ */
/* packed-weight synthesis used by the reference's own tests           */
/* ------------------------------------------------------------------ */

/* Deterministic [n,k] packed weights, code = (p*2654435761 + s) & mask for
 * pack p, slot s. Reference: crates/metaltile-std/src/mlx/quantized.rs:5355-5369. */
MTQ_ORACLE_API void mtq_oracle_synth_packed_w(size_t n, size_t k, uint32_t bits, uint32_t *out) {
    uint32_t pf = 32u / bits, mask = (1u << bits) - 1u;
    size_t n_packs = n * k / pf;
    for (size_t p = 0; p < n_packs; p++) {
        uint32_t v = 0;
        for (uint32_t s = 0; s < pf; s++) {
            uint32_t code = ((uint32_t)p * 2654435761u + s) & mask;
            v |= code << (s * bits);
        }
        out[p] = v;
    }
}

/* Bit-stream packed [out_dim,in_dim] weights for any width 2..8, code =
 * ((row*in_dim+d)*2654435761 + d) & mask written at bit offset d*bits.
 * Reference: crates/metaltile-std/src/ffai/dequant_gemv.rs:389-414. */
MTQ_ORACLE_API void mtq_oracle_synth_bitstream_w(size_t out_dim, size_t in_dim, uint32_t bits,
                                                 uint32_t *out) {
    uint32_t mask = (1u << bits) - 1u;
    size_t u32_per_row = in_dim * bits / 32;
    memset(out, 0, out_dim * u32_per_row * 4);
    for (size_t row = 0; row < out_dim; row++) {
        uint32_t *r = out + row * u32_per_row;
        for (size_t d = 0; d < in_dim; d++) {
            uint32_t code = ((uint32_t)(row * in_dim + d) * 2654435761u + (uint32_t)d) & mask;
            uint32_t bit_off = (uint32_t)(d * bits);
            uint32_t word = bit_off / 32, in_w = bit_off & 31u, bits_in_w0 = 32u - in_w;
            r[word] |= code << in_w;
            if (bits_in_w0 < bits) r[word + 1] |= code >> bits_in_w0;
        }
    }
}

/* Stacked [E,out,in] int4 weights, code = ((e*out*in + row*in + d)*2654435761) & 15.
 * Reference: crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:131-148. */
MTQ_ORACLE_API void mtq_oracle_synth_stacked_w(size_t n_experts, size_t out_dim, size_t in_dim,
                                               uint32_t *out) {
    size_t ppr = in_dim / 8;
    memset(out, 0, n_experts * out_dim * ppr * 4);
    for (size_t e = 0; e < n_experts; e++)
        for (size_t row = 0; row < out_dim; row++) {
            uint32_t *r = out + (e * out_dim + row) * ppr;
            for (size_t d = 0; d < in_dim; d++) {
                uint32_t code =
                    ((uint32_t)(e * out_dim * in_dim + row * in_dim + d) * 2654435761u) & 0xFu;
                r[d / 8] |= code << ((d % 8) * 4);
            }
        }
}

/* ------------------------------------------------------------------ */
/* code extraction                                                     */
/* ------------------------------------------------------------------ */

/* Code j of a row stored as a little-endian bit stream of `bits`-wide fields;
 * for bits in {2,4,8} this is (word >> ((j % pf)*bits)) & mask
 * (crates/metaltile-std/src/mlx/quantized.rs:5393-5396); other widths may
 * straddle two words (crates/metaltile-std/src/ffai/dequant_gemv.rs:436-449). */
static inline uint32_t extract_code(const uint32_t *row_w, size_t j, uint32_t bits) {
    uint64_t mask = (1ull << bits) - 1ull;
    uint32_t bit_off = (uint32_t)(j * bits);
    uint32_t word = bit_off / 32, in_w = bit_off & 31u, bits_in_w0 = 32u - in_w;
    if (bits_in_w0 >= bits) return (uint32_t)(((uint64_t)row_w[word] >> in_w) & mask);
    uint32_t lo_bits = bits_in_w0, spill = bits - lo_bits;
    uint64_t lo = ((uint64_t)row_w[word] >> in_w) & ((1ull << lo_bits) - 1ull);
    uint64_t hi = ((uint64_t)row_w[word + 1] & ((1ull << spill) - 1ull)) << lo_bits;
    return (uint32_t)(lo | hi);
}

/* Unpack an [n,k] packed matrix to one code per u8 (test helper for the
 * brute-force checks). */
MTQ_ORACLE_API void mtq_oracle_unpack_codes(const uint32_t *w, size_t n, size_t k, uint32_t bits,
                                            uint8_t *codes) {
    size_t wpr = k * bits / 32;
    for (size_t r = 0; r < n; r++)
        for (size_t j = 0; j < k; j++) codes[r * k + j] = (uint8_t)extract_code(w + r * wpr, j, bits);
}

/* Pack one code per u8 into the bit-stream layout (inverse of unpack_codes).
 * Reference packers: crates/metaltile-std/src/ffai/moe.rs:3558-3569 (int4),
 * crates/metaltile-std/src/ffai/dequant_gemv.rs:400-409 (any width). */
MTQ_ORACLE_API void mtq_oracle_pack_codes(const uint8_t *codes, size_t n, size_t k, uint32_t bits,
                                          uint32_t *w) {
    size_t wpr = k * bits / 32;
    uint32_t mask = (1u << bits) - 1u;
    memset(w, 0, n * wpr * 4);
    for (size_t r = 0; r < n; r++)
        for (size_t j = 0; j < k; j++) {
            uint32_t code = codes[r * k + j] & mask;
            uint32_t bit_off = (uint32_t)(j * bits);
            uint32_t word = bit_off / 32, in_w = bit_off & 31u, bits_in_w0 = 32u - in_w;
            w[r * wpr + word] |= code << in_w;
            if (bits_in_w0 < bits) w[r * wpr + word + 1] |= code >> bits_in_w0;
        }
}

/* ------------------------------------------------------------------ */
/* qmv / qmm                                                           */
/* ------------------------------------------------------------------ */

/* One output element, the reference's loop body: f32 accumulate in k order of
 * (q*scale + bias) * x. crates/metaltile-std/src/mlx/quantized.rs:5390-5400. */
static inline float dot_row_f32(const uint32_t *row_w, const float *s, const float *b,
                                const float *x, size_t k, uint32_t bits, size_t group_size) {
    float acc = 0.0f;
    for (size_t j = 0; j < k; j++) {
        size_t g = j / group_size;
        float q = (float)extract_code(row_w, j, bits);
        acc += (q * s[g] + b[g]) * x[j];
    }
    return acc;
}

/* qmm_oracle: out[m,n] = sum_k (q*s_g + b_g) * x[m,k], f32 sequential.
 * Reference: crates/metaltile-std/src/mlx/quantized.rs:5374-5404; identical
 * loop in tests/mt_qmv_gpu_correctness.rs:62-88 (naive_qmv_f32) and
 * ffai/dequant_gemv.rs:419-456 (dequant_gemv_oracle, any bit width).
 * Inputs are f32 values already rounded through the element dtype.
 * `threads` > 1 splits the independent output rows over OpenMP threads (used
 * only by the benchmark's cpu_baseline; results do not depend on it). */
MTQ_ORACLE_API void mtq_oracle_qmm(const uint32_t *w, const float *scales, const float *biases,
                                   const float *x, size_t m, size_t n, size_t k, uint32_t bits,
                                   size_t group_size, float *out, int threads) {
    size_t wpr = k * bits / 32, gpr = k / group_size;
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static) if (threads > 1)
    for (ptrdiff_t nc = 0; nc < (ptrdiff_t)n; nc++)
        for (size_t mr = 0; mr < m; mr++)
            out[mr * n + nc] = dot_row_f32(w + nc * wpr, scales + nc * gpr, biases + nc * gpr,
                                           x + mr * k, k, bits, group_size);
}

/* Same sum accumulated in f64 (dequantised weight still formed in f32 as the
 * reference does). This is the judge both the f32 oracle and the GPU are
 * measured against when the tolerance is tight. */
MTQ_ORACLE_API void mtq_oracle_qmm_f64(const uint32_t *w, const float *scales, const float *biases,
                                       const float *x, size_t m, size_t n, size_t k, uint32_t bits,
                                       size_t group_size, double *out, int threads) {
    size_t wpr = k * bits / 32, gpr = k / group_size;
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static) if (threads > 1)
    for (ptrdiff_t nc = 0; nc < (ptrdiff_t)n; nc++)
        for (size_t mr = 0; mr < m; mr++) {
            const uint32_t *rw = w + nc * wpr;
            double acc = 0.0;
            for (size_t j = 0; j < k; j++) {
                size_t g = j / group_size;
                float q = (float)extract_code(rw, j, bits);
                float wv = q * scales[nc * gpr + g] + biases[nc * gpr + g];
                acc += (double)wv * (double)x[mr * k + j];
            }
            out[mr * n + nc] = acc;
        }
}

/* Algebraic-split form: acc += s * sum(q*x) + b * sum(x) per group.
 * Reference: crates/metaltile-std/tests/qmm_gpu_correctness.rs:73-108
 * (cpu_qmm_reference; int4, group of 8 packs). Generalised over bits/group. */
MTQ_ORACLE_API void mtq_oracle_qmm_split(const uint32_t *w, const float *scales,
                                         const float *biases, const float *x, size_t m, size_t n,
                                         size_t k, uint32_t bits, size_t group_size, float *out) {
    size_t wpr = k * bits / 32, gpr = k / group_size;
    for (size_t mr = 0; mr < m; mr++)
        for (size_t nc = 0; nc < n; nc++) {
            float acc = 0.0f;
            for (size_t g = 0; g < gpr; g++) {
                float q_dot = 0.0f, x_sum = 0.0f;
                for (size_t i = 0; i < group_size; i++) {
                    size_t j = g * group_size + i;
                    float q = (float)extract_code(w + nc * wpr, j, bits);
                    float xv = x[mr * k + j];
                    q_dot += q * xv;
                    x_sum += xv;
                }
                acc += scales[nc * gpr + g] * q_dot + biases[nc * gpr + g] * x_sum;
            }
            out[mr * n + nc] = acc;
        }
}

/* MMA-path semantics: the dequantised weight is rounded to the element dtype
 * before the multiply, products accumulate in f32.
 * Reference: crates/metaltile-std/src/mlx/quantized.rs:2267-2274
 * (`(s*q+b).cast::<T>()` stored to threadgroup memory) and :2157-2168 (f32
 * accumulator fragments). */
MTQ_ORACLE_API void mtq_oracle_qmm_mma(const uint32_t *w, const float *scales, const float *biases,
                                       const float *x, size_t m, size_t n, size_t k, uint32_t bits,
                                       size_t group_size, int dt, double *out, int threads) {
    size_t wpr = k * bits / 32, gpr = k / group_size;
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static) if (threads > 1)
    for (ptrdiff_t nc = 0; nc < (ptrdiff_t)n; nc++) {
        float *wrow = (float *)malloc(k * sizeof(float));
        for (size_t j = 0; j < k; j++) {
            size_t g = j / group_size;
            float q = (float)extract_code(w + nc * wpr, j, bits);
            wrow[j] = q * scales[nc * gpr + g] + biases[nc * gpr + g];
        }
        mtq_oracle_round_through(wrow, k, dt);
        for (size_t mr = 0; mr < m; mr++) {
            double acc = 0.0;
            for (size_t j = 0; j < k; j++) acc += (double)wrow[j] * (double)x[mr * k + j];
            out[mr * n + nc] = acc;
        }
        free(wrow);
    }
}

/* ------------------------------------------------------------------ */
/* gather (MoE) family                                                 */
/* ------------------------------------------------------------------ */

/* Expert of row t under the CSR ABI: first e with t < expert_offsets[e+1],
 * 0 if none. Reference: crates/metaltile-std/src/ffai/moe.rs:3593-3600
 * (oracle) and :376-385 (kernel). */
MTQ_ORACLE_API uint32_t mtq_oracle_csr_expert(const uint32_t *expert_offsets, size_t n_experts,
                                              uint32_t t) {
    for (size_t e = 0; e < n_experts; e++)
        if (t < expert_offsets[e + 1]) return (uint32_t)e;
    return 0;
}

/* cpu_gather_qmm_int4 generalised over bits: out[t,m] = sum_k x[t,k] * W[E(t),m,k].
 * Reference: crates/metaltile-std/src/ffai/moe.rs:3577-3622. `indices` (per-row
 * expert id, crates/metaltile-std/src/ffai/moe.rs:2229-2236) is used when
 * expert_offsets is NULL. */
MTQ_ORACLE_API void mtq_oracle_gather_qmm(const float *x, const uint32_t *weight_packed,
                                          const float *scales, const float *biases,
                                          const uint32_t *expert_offsets, const uint32_t *indices,
                                          size_t t_rows, size_t k_in, size_t m_out,
                                          size_t n_experts, uint32_t bits, size_t group_size,
                                          float *out, double *out_f64, int threads) {
    size_t wpr = k_in * bits / 32, gpr = k_in / group_size;
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static) if (threads > 1)
    for (ptrdiff_t row = 0; row < (ptrdiff_t)t_rows; row++) {
        size_t e = expert_offsets ? mtq_oracle_csr_expert(expert_offsets, n_experts, (uint32_t)row)
                                  : indices[row];
        for (size_t mo = 0; mo < m_out; mo++) {
            const uint32_t *rw = weight_packed + (e * m_out + mo) * wpr;
            const float *s = scales + (e * m_out + mo) * gpr;
            const float *b = biases + (e * m_out + mo) * gpr;
            if (out) out[row * m_out + mo] = dot_row_f32(rw, s, b, x + row * k_in, k_in, bits, group_size);
            if (out_f64) {
                double acc = 0.0;
                for (size_t j = 0; j < k_in; j++) {
                    float q = (float)extract_code(rw, j, bits);
                    float wv = q * s[j / group_size] + b[j / group_size];
                    acc += (double)wv * (double)x[row * k_in + j];
                }
                out_f64[row * m_out + mo] = acc;
            }
        }
    }
}

/* One GEMV against slab `expert` of stacked weights.
 * Reference: crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:154-184. */
MTQ_ORACLE_API void mtq_oracle_expert_indexed(const uint32_t *weight, const float *scales,
                                              const float *biases, const float *input,
                                              size_t expert, size_t out_dim, size_t in_dim,
                                              size_t group_size, float *out) {
    size_t ppr = in_dim / 8, ng = in_dim / group_size;
    for (size_t row = 0; row < out_dim; row++)
        out[row] = dot_row_f32(weight + (expert * out_dim + row) * ppr,
                               scales + (expert * out_dim + row) * ng,
                               biases + (expert * out_dim + row) * ng, input, in_dim, 4, group_size);
}

/* Fused RMSNorm + quantized GEMV: normed[d] = x[d] * norm_weight[d] * inv_rms with
 * inv_rms = 1 / sqrt(sum(x^2) / in_dim + eps), then the f32-sequential dequant dot.
 * Reference: crates/metaltile-std/tests/rms_norm_qgemv_gpu_correctness.rs:59-91 (CPU form)
 * and crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:64-77,92-106 (kernel). `normed`
 * (in_dim floats, may be NULL) receives the normalised activation. When out_f64 is not
 * NULL the dot is also accumulated in f64 from the same f32 `normed` and f32 weights. */
MTQ_ORACLE_API void mtq_oracle_rms_norm_qgemv(const uint32_t *weight, const float *scales, const float *biases,
                                              const float *x, const float *norm_weight, size_t in_dim,
                                              size_t group_size, size_t out_dim, uint32_t bits, float eps,
                                              float *out, double *out_f64, float *normed) {
    float ssq = 0.0f;
    for (size_t d = 0; d < in_dim; d++) ssq += x[d] * x[d];
    float inv_rms = 1.0f / sqrtf(ssq / (float)in_dim + eps);
    size_t wpr = in_dim * bits / 32, ng = in_dim / group_size;
    float *nx = (float *)malloc(in_dim * sizeof(float));
    for (size_t d = 0; d < in_dim; d++) nx[d] = x[d] * norm_weight[d] * inv_rms;
    if (normed) memcpy(normed, nx, in_dim * sizeof(float));
    for (size_t row = 0; row < out_dim; row++) {
        const uint32_t *rw = weight + row * wpr;
        const float *rs = scales + row * ng, *rb = biases + row * ng;
        float acc = 0.0f;
        double acc64 = 0.0;
        for (size_t d = 0; d < in_dim; d++) {
            float w_real = (float)extract_code(rw, d, bits) * rs[d / group_size] + rb[d / group_size];
            acc += w_real * nx[d];
            acc64 += (double)w_real * (double)nx[d];
        }
        out[row] = acc;
        if (out_f64) out_f64[row] = acc64;
    }
    free(nx);
}

/* Fused gated RMSNorm + 4-bit GEMV: inner[r * dv + d] = y[r, d] * inv_rms[r] * norm_weight[d] * silu(z[r, d]) with
 * inv_rms[r] = 1 / sqrt(sum_d(y[r, d]^2) / dv + eps) and silu(v) = v / (1 + exp(-v)), all in f32 and in that order,
 * then the f32-sequential dequant dot over in_dim = hv * dv.
 * Reference: crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:322-366 (CPU form) and :120-151 (kernel).
 * `inner` (hv * dv floats, may be NULL) receives the gated, normalised activation. When out_f64 is not NULL the dot
 * is also accumulated in f64 from the same f32 `inner` and f32 weights. */
MTQ_ORACLE_API void mtq_oracle_gated_rms_norm_qgemv(const uint32_t *weight, const float *scales, const float *biases,
                                                    const float *y, const float *z, const float *norm_weight, size_t hv,
                                                    size_t dv, size_t group_size, size_t out_dim, float eps, float *out,
                                                    double *out_f64, float *inner) {
    size_t in_dim = hv * dv, wpr = in_dim / 8, ng = in_dim / group_size;
    float *nx = (float *)malloc(in_dim * sizeof(float));
    for (size_t r = 0; r < hv; r++) {
        const float *yr = y + r * dv, *zr = z + r * dv;
        float ssq = 0.0f;
        for (size_t d = 0; d < dv; d++) ssq += yr[d] * yr[d];
        float inv_rms = 1.0f / sqrtf(ssq / (float)dv + eps);
        for (size_t d = 0; d < dv; d++) {
            float gate = zr[d] / (1.0f + expf(-zr[d]));
            nx[r * dv + d] = yr[d] * inv_rms * norm_weight[d] * gate;
        }
    }
    if (inner) memcpy(inner, nx, in_dim * sizeof(float));
    for (size_t row = 0; row < out_dim; row++) {
        const uint32_t *rw = weight + row * wpr;
        const float *rs = scales + row * ng, *rb = biases + row * ng;
        float acc = 0.0f;
        double acc64 = 0.0;
        for (size_t d = 0; d < in_dim; d++) {
            float w_real = (float)extract_code(rw, d, 4) * rs[d / group_size] + rb[d / group_size];
            acc += w_real * nx[d];
            acc64 += (double)w_real * (double)nx[d];
        }
        out[row] = acc;
        if (out_f64) out_f64[row] = acc64;
    }
    free(nx);
}

/* Vector-matrix product against a transposed packed weight: out[m, c] = sum_d w_hat[d, c] * x[m, d],
 * W [K, N] packed along N (row d holds N codes), scales / biases [K/G, N] (groups along K).
 * f32 sequential in d; out_f64 (may be NULL) accumulates the same f32 weights in f64.
 * Reference: crates/metaltile-std/src/mlx/quantized.rs:5613-5635 (qvm_oracle) and :4397-4522 (kernels). */
MTQ_ORACLE_API void mtq_oracle_qvm(const uint32_t *w, const float *scales, const float *biases, const float *x,
                                   size_t m, size_t n, size_t k, uint32_t bits, size_t group_size, float *out,
                                   double *out_f64) {
    size_t wpr = n * bits / 32;
    for (size_t row = 0; row < m; row++)
        for (size_t c = 0; c < n; c++) {
            float acc = 0.0f;
            double acc64 = 0.0;
            for (size_t d = 0; d < k; d++) {
                size_t g = d / group_size;
                float wv = (float)extract_code(w + d * wpr, c, bits) * scales[g * n + c] + biases[g * n + c];
                acc += wv * x[row * k + d];
                acc64 += (double)wv * (double)x[row * k + d];
            }
            out[row * n + c] = acc;
            if (out_f64) out_f64[row * n + c] = acc64;
        }
}

/* ------------------------------------------------------------------ */
/* MoE routing around the gathered matmul                              */
/* ------------------------------------------------------------------ */

/* Top-k experts per token row and their softmax weights.
 * k passes of argmax with strict '>' from (-inf, index 0), already-chosen experts masked,
 * so ties go to the smaller index and NaN never wins; weight = exp(v - max_all) / divisor
 * with divisor = sum over the chosen k (norm_topk_prob = 1) or over all experts (0).
 * Reference: crates/metaltile-std/src/ffai/moe.rs:65-199 (kernel) and
 * crates/metaltile-std/tests/moe_gpu_correctness.rs:55-93 (its CPU form). */
MTQ_ORACLE_API void mtq_oracle_moe_router_topk(const float *logits, size_t n_rows, size_t n_experts, size_t k,
                                               int norm_topk_prob, uint32_t *indices, float *weights) {
    for (size_t row = 0; row < n_rows; row++) {
        const float *z = logits + row * n_experts;
        float max_all = -INFINITY;
        for (size_t j = 0; j < n_experts; j++)
            if (z[j] > max_all) max_all = z[j];
        float sum_all = 0.0f;
        for (size_t j = 0; j < n_experts; j++) sum_all += expf(z[j] - max_all);
        uint32_t *idx = indices + row * k;
        float vals[32];
        for (size_t it = 0; it < k; it++) {
            float best = -INFINITY;
            uint32_t bi = 0;
            for (size_t j = 0; j < n_experts; j++) {
                int taken = 0;
                for (size_t p = 0; p < it; p++) taken |= idx[p] == (uint32_t)j;
                if (taken) continue;
                if (z[j] > best) { best = z[j]; bi = (uint32_t)j; }
            }
            idx[it] = bi;
            vals[it] = best;
        }
        float e[32], sum_chosen = 0.0f;
        for (size_t j = 0; j < k; j++) { e[j] = expf(vals[j] - max_all); sum_chosen += e[j]; }
        float divisor = norm_topk_prob == 1 ? sum_chosen : sum_all;
        for (size_t j = 0; j < k; j++) weights[row * k + j] = e[j] / divisor;
    }
}

/* out[token, h] = sum_j w[token, j] * expert_outputs[inv_perm[token, j], h], f32, j ascending,
 * product and sum rounded separately.
 * Reference: crates/metaltile-std/src/ffai/moe.rs:225-251. */
MTQ_ORACLE_API void mtq_oracle_moe_unpermute(const float *expert_outputs, const uint32_t *inv_perm, const float *w,
                                             size_t n_tokens, size_t hidden, size_t k, float *out) {
    for (size_t t = 0; t < n_tokens; t++)
        for (size_t h = 0; h < hidden; h++) {
            float acc = 0.0f;
            for (size_t j = 0; j < k; j++) {
                float prod = w[t * k + j] * expert_outputs[(size_t)inv_perm[t * k + j] * hidden + h];
                acc = acc + prod;
            }
            out[t * hidden + h] = acc;
        }
}

/* Fused MoE decode step: out[i] = sum_k slot_w[k] * sum_d dequant(W[expert[k]][i][d]) * silu(gate_k[d]) * up_k[d],
 * silu(g) = g / (1 + exp(-g)), as the unfused chain in f32: swiglu, one 4-bit GEMV per slot
 * (f32 sequential), then acc[i] += slot_w[k] * down[i]. gates / ups: n_slots rows of in_dim.
 * out_f64 (may be NULL): same inner activations, dots and the slot sum accumulated in f64.
 * Reference: crates/metaltile-std/tests/moe_down_swiglu_accum_gpu_correctness.rs:99-183 and
 * crates/metaltile-std/src/ffai/moe_down_swiglu_accum.rs:240-275. */
MTQ_ORACLE_API void mtq_oracle_moe_down_swiglu_accum(const float *gates, const float *ups, const uint32_t *experts,
                                                     const float *slot_w, size_t n_slots, const uint32_t *weights,
                                                     const float *scales, const float *biases, size_t in_dim,
                                                     size_t out_dim, size_t group_size, float *out, double *out_f64) {
    size_t ppr = in_dim / 8, ng = in_dim / group_size;
    float *inner = (float *)malloc(in_dim * sizeof(float));
    for (size_t i = 0; i < out_dim; i++) { out[i] = 0.0f; if (out_f64) out_f64[i] = 0.0; }
    for (size_t k = 0; k < n_slots; k++) {
        for (size_t d = 0; d < in_dim; d++) {
            float g = gates[k * in_dim + d];
            float silu = g / (1.0f + expf(-g));
            inner[d] = silu * ups[k * in_dim + d];
        }
        size_t e = experts[k];
        for (size_t row = 0; row < out_dim; row++) {
            const uint32_t *rw = weights + (e * out_dim + row) * ppr;
            const float *rs = scales + (e * out_dim + row) * ng, *rb = biases + (e * out_dim + row) * ng;
            float acc = 0.0f;
            double acc64 = 0.0;
            for (size_t d = 0; d < in_dim; d++) {
                float wv = (float)extract_code(rw, d, 4) * rs[d / group_size] + rb[d / group_size];
                acc += wv * inner[d];
                acc64 += (double)wv * (double)inner[d];
            }
            out[row] += slot_w[k] * acc;
            if (out_f64) out_f64[row] += (double)slot_w[k] * acc64;
        }
    }
    free(inner);
}

/* ------------------------------------------------------------------ */
/* affine quantise / dequantise (producers of the packed format)       */
/* ------------------------------------------------------------------ */

/* Per group: scale = (max-min)/(2^b-1) (1.0 when < 1e-7), bias = min,
 * q = trunc(clamp((v-bias)*(1/scale) + 0.5, 0, 2^b-1)) formed with the f32
 * scale/bias; the stored scale/bias are then rounded to the element dtype.
 * Reference: crates/metaltile-std/src/mlx/quantized.rs:3642-3671 (kernel) and
 * :5296-5303 (oracle of the scale/bias derivation). */
MTQ_ORACLE_API void mtq_oracle_affine_quantize(const float *v, size_t n_groups, size_t group_size,
                                               uint32_t bits, int dt, uint8_t *codes,
                                               float *scales, float *biases) {
    float qmax = (float)((1u << bits) - 1u);
    for (size_t g = 0; g < n_groups; g++) {
        const float *gv = v + g * group_size;
        float mn = gv[0], mx = gv[0];
        for (size_t i = 1; i < group_size; i++) {
            if (gv[i] < mn) mn = gv[i];
            if (gv[i] > mx) mx = gv[i];
        }
        float scale = (mx - mn) / qmax;
        if (scale < 1e-7f) scale = 1.0f;
        float bias = mn, inv_scale = 1.0f / scale;
        for (size_t i = 0; i < group_size; i++) {
            float t = (gv[i] - bias) * inv_scale + 0.5f;
            if (t < 0.0f) t = 0.0f;
            if (t > qmax) t = qmax;
            codes[g * group_size + i] = (uint8_t)t;
        }
        scales[g] = scale;
        biases[g] = bias;
    }
    mtq_oracle_round_through(scales, n_groups, dt);
    mtq_oracle_round_through(biases, n_groups, dt);
}

/* out[i] = scale_g * q_i + bias_g. Reference: crates/metaltile-std/src/mlx/quantized.rs:3599-3604. */
MTQ_ORACLE_API void mtq_oracle_affine_dequantize(const uint32_t *w, const float *scales,
                                                 const float *biases, size_t n_elem,
                                                 size_t group_size, uint32_t bits, float *out) {
    for (size_t i = 0; i < n_elem; i++) {
        float q = (float)extract_code(w, i, bits);
        out[i] = scales[i / group_size] * q + biases[i / group_size];
    }
}

/* ------------------------------------------------------------------ */
/* bench statistics                                                    */
/* ------------------------------------------------------------------ */

static int cmp_double(const void *a, const void *b) {
    double x = *(const double *)a, y = *(const double *)b;
    return (x > y) - (x < y);
}

/* BenchStats::from_samples -> {min, mean, median, p95, p99, stddev, cv%}.
 * Reference: crates/metaltile-std/src/stats.rs:25-46. */
MTQ_ORACLE_API void mtq_oracle_bench_stats(const double *samples, size_t n, double out[7]) {
    double *s = (double *)malloc(n * sizeof(double));
    memcpy(s, samples, n * sizeof(double));
    qsort(s, n, sizeof(double), cmp_double);
    double mean = 0.0;
    for (size_t i = 0; i < n; i++) mean += s[i];
    mean /= (double)n;
    double var = 0.0;
    for (size_t i = 0; i < n; i++) var += (s[i] - mean) * (s[i] - mean);
    var /= (double)n;
    size_t i95 = n * 95 / 100, i99 = n * 99 / 100;
    if (i95 > n - 1) i95 = n - 1;
    if (i99 > n - 1) i99 = n - 1;
    out[0] = s[0];
    out[1] = mean;
    out[2] = s[n / 2];
    out[3] = s[i95];
    out[4] = s[i99];
    out[5] = sqrt(var);
    out[6] = mean > 0.0 ? out[5] / mean * 100.0 : 0.0;
    free(s);
}
