/*
 * mtq.h -- C-ABI of libmtq_hip.so: MI355X (gfx950) affine-quantized matmul.
 *
 * This is the boundary a HIP backend of the reference's runtime binds. The
 * reference reaches its GPU through two Rust call sites, both of which move
 * flat byte buffers bound by position:
 *   - Context::dispatch_with_grid(kernel, buffers, fn_consts, grid, tpg)
 *       crates/metaltile-runtime/src/context.rs:269-283   (tests)
 *   - GpuRunner::{new, compile, buffer_bytes, buffer_zeros, read_bytes,
 *       measure, flush_slc}
 *       crates/metaltile-std/src/runner.rs:253,287,317,324,354,413,455 (bench)
 * Each entry point below names the reference interface it replaces.
 *
 * Conventions
 *   - Every function returns 0 on success or a negative MTQ_ERR_* code; the
 *     message for the calling thread's last failure is mtq_last_error().
 *     Nothing throws or aborts across this boundary (the reference builds with
 *     panic = "abort", Cargo.toml:87).
 *   - Device pointers are plain `void*` obtained from mtq_alloc (or any other
 *     HIP allocation on the same device). The caller owns host memory; the
 *     library copies in and out (reference: single_dispatch.rs:163-171, 100-117).
 *   - Kernels are enqueued on the library's stream and do not block the host
 *     unless stated; mtq_download and mtq_sync wait for them.
 *   - Element dtype T of scales / biases / x / out is MTQ_F32, MTQ_F16 or
 *     MTQ_BF16. Weights are unsigned codes packed LSB-first into little-endian
 *     u32 words, row-major [N][K*bits/32]; w_hat = scale_g*q + bias_g with
 *     g = k / group_size; sums are f32; results are rounded to T on store
 *     (crates/metaltile-std/src/mlx/quantized.rs:5374-5404).
 *   - There is no CPU fallback: without a usable GPU every call fails with
 *     MTQ_ERR_NO_DEVICE.
 *   - Single-threaded use per process, like the reference's runner
 *     (crates/metaltile-std/src/runner.rs:209-229).
 */
#ifndef MTQ_H
#define MTQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MTQ_API __attribute__((visibility("default")))

/* element dtypes (reference: metaltile_core::dtype::DType F32 / F16 / BF16) */
enum { MTQ_F32 = 0, MTQ_F16 = 1, MTQ_BF16 = 2 };

/* error codes -- counterpart of MetalTileError, crates/metaltile-runtime/src/error.rs:8-55 */
enum {
    MTQ_OK = 0,
    MTQ_ERR_NO_DEVICE = -1,      /* NoDevice */
    MTQ_ERR_BAD_ARG = -2,        /* Buffer / invalid argument */
    MTQ_ERR_SHAPE = -3,          /* Dispatch: shape violates a kernel precondition */
    MTQ_ERR_BUFFER_SIZE = -4,    /* BufferSize{param, expected, actual} */
    MTQ_ERR_UNKNOWN_KERNEL = -5, /* no kernel of that name: caller may fall back */
    MTQ_ERR_HIP = -6,            /* Dispatch: runtime failure */
    MTQ_ERR_UNSUPPORTED = -7     /* valid request without a kernel in this build */
};

/* A bound buffer: device pointer plus its length in bytes (the reference binds
 * `Vec<u8>` and checks lengths, single_dispatch.rs:154-158). */
typedef struct mtq_buf {
    void *ptr;
    size_t bytes;
} mtq_buf;

typedef struct mtq_device_info {
    char name[128];
    char arch[32];          /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int compute_units;
    int clock_khz;          /* engine clock reported by the runtime */
    int memory_clock_khz;
    int memory_bus_bits;
    size_t total_memory;    /* bytes */
    int l2_bytes;
    int lds_per_cu_bytes;
} mtq_device_info;

/* ---- lifetime / device -------------------------------------------------- */

/* Replaces GpuRunner::new (crates/metaltile-std/src/runner.rs:253-285) and
 * Context::new (crates/metaltile-runtime/src/context.rs:174): pick the device,
 * create the stream and timing events. Idempotent for the same device. */
MTQ_API int mtq_init(int device);
MTQ_API int mtq_shutdown(void);
/* Thread-local message of the last failing call ("" if none). */
MTQ_API const char *mtq_last_error(void);
/* Replaces GpuRunner::device_name (crates/metaltile-std/src/runner.rs:95). */
MTQ_API int mtq_device_name(char *out, size_t cap);
MTQ_API int mtq_get_device_info(mtq_device_info *out);
/* Use a caller-owned hipStream_t (passed as void*) for all later launches;
 * NULL restores the library's own stream. Waits for the work queued on the stream
 * being left: several ops share one library-owned scratch buffer, so launches of
 * such ops must not overlap across streams. */
MTQ_API int mtq_set_stream(void *hip_stream);

/* ---- buffers ------------------------------------------------------------ */

/* Replace GpuRunner::buffer_zeros / buffer_bytes / read_bytes
 * (crates/metaltile-std/src/runner.rs:317-360) and Context::upload_resident
 * (crates/metaltile-runtime/src/context.rs:330-337). mtq_alloc zero-fills. */
MTQ_API int mtq_alloc(size_t bytes, void **dptr);
MTQ_API int mtq_free(void *dptr);
MTQ_API int mtq_upload(void *dptr, const void *host, size_t bytes);
MTQ_API int mtq_download(void *host, const void *dptr, size_t bytes);
MTQ_API int mtq_memset(void *dptr, int byte_value, size_t bytes);
MTQ_API int mtq_sync(void);

/* ---- typed entry points (device pointers) ------------------------------- */

/* qmv: out[m,n] = sum_k w_hat[n,k] * x[m,k] for a small batch of rows (M >= 1).
 * Replaces mt_qmv / mt_qmv_int8_fast / mt_qmm / mt_qmm_bm2 / mt_qmm_bm4 and the
 * int8 trio (crates/metaltile-std/src/mlx/quantized.rs:8, 1475, 343, 650,
 * 1072, 1602, 1719, 1870), dequant_gemv_int{2..8} and _int4_fast
 * (crates/metaltile-std/src/ffai/dequant_gemv.rs:52-341) and mt_qmv_b* / mt_qmm_b*
 * (quantized.rs:4273-4392). bits in 2..8; group_size divides K. */
MTQ_API int mtq_qmv(int dtype, int bits, uint32_t group_size, const void *w, const void *scales,
                    const void *biases, const void *x, void *out, uint32_t M, uint32_t N,
                    uint32_t K);

/* qmm: same product for any M; routes by M like mt_qmm_for
 * (crates/metaltile-std/src/mlx/quantized.rs:5040-5065): from 9 rows (from 5 where the
 * rows are long) the MFMA tile kernel (replaces mt_qmm_mma / _m16 / _int8 / _int2 / _b3 /
 * _b5 / _b6, quantized.rs:2106, 2408, 2731, 3330, 3560-3900; w_hat rounded to the element
 * type before the multiply, as there), below that the qmv family (exact w_hat). MTQ_F32
 * batches run on the f32 matrix cores from 5 rows. Short, wide matrices split K over
 * workgroups through a library-owned buffer (allocated on first use). */
MTQ_API int mtq_qmm(int dtype, int bits, uint32_t group_size, const void *w, const void *scales,
                    const void *biases, const void *x, void *out, uint32_t M, uint32_t N,
                    uint32_t K);

/* gather_qmv, CSR view: out[t,n] = sum_k x[t,k] * w_hat[E(t)][n,k], E(t) = first
 * e with t < expert_offsets[e+1] (0 if none). Replaces
 * mt_moe_gather_qmm_int4{,_m8,_m16,_m32} and _b* (crates/metaltile-std/src/ffai/moe.rs:358,
 * 634, 900, 1363, 461-605). w is [E][N][K*bits/32], scales/biases [E][N][K/G],
 * x [T][K], expert_offsets u32[E+1], out [T][N].
 * Both row views: while experts average at most 8 rows, each expert's rows run on the
 * GEMV kernels (exact w_hat = s*q + b in f32); above that the rows are grouped by expert
 * into 64-row tiles on the MFMA tile kernel, where w_hat is rounded to the element type
 * first, as in the reference's MMA gathers (moe.rs:2256); MTQ_F32 rows always run grouped, in
 * 32-row tiles on the f32 matrix-core kernel (f32 rounding only). The grouping tables live in a
 * library-owned buffer (allocated on first use). Option "gather.grouped": 0 this rule,
 * 1 never grouped, 2 always grouped. Through mtq_dispatch the reference's kernel name decides instead:
 * mt_moe_gather_qmm_int4{,_m8,_m16,_m32} and mt_moe_gather_qmm_b* multiply by the exact s*q + b in the
 * reference and stay on the GEMV kernels here at any number of rows per expert (option
 * "gather.names_exact"); mt_moe_gather_qmm_mma_* round w_hat to T in the reference and follow the rule above. */
MTQ_API int mtq_gather_qmv_csr(int dtype, int bits, uint32_t group_size, const void *x,
                               const void *w, const void *scales, const void *biases,
                               const uint32_t *expert_offsets, void *out, uint32_t T, uint32_t N,
                               uint32_t K, uint32_t E);

/* gather_qmv, per-row view: E(t) = indices[t]; rows need not be sorted; rows
 * whose index is >= E are left untouched. Replaces mt_moe_gather_qmm_mma_int4 /
 * _bm16 / _mma_int8 / _mma_b* (crates/metaltile-std/src/ffai/moe.rs:2256, 2857, 3231,
 * 2552-2835). */
MTQ_API int mtq_gather_qmv_indices(int dtype, int bits, uint32_t group_size, const void *x,
                                   const void *w, const void *scales, const void *biases,
                                   const uint32_t *indices, void *out, uint32_t T, uint32_t N,
                                   uint32_t K, uint32_t E);

/* gather_qmv, single view: one row against slab expert_index[0] (read on the
 * device, no host round trip; ids >= E are clamped to E-1). Replaces
 * dequant_gemv_int4_expert_indexed
 * (crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:58-105). */
MTQ_API int mtq_gather_qmv_single(int dtype, int bits, uint32_t group_size, const void *w,
                                  const void *scales, const void *biases, const void *input,
                                  const uint32_t *expert_index, void *output, uint32_t N,
                                  uint32_t K, uint32_t E);

/* qvm: out[m, c] = sum_d w_hat[d, c] * x[m, d] against the TRANSPOSED packed weight: w u32 [K, N*bits/32]
 * (row d holds the N codes of K-position d), scales / biases T [K/G, N] (groups along K), x T [M, K],
 * out T [M, N]. bits 2..8. Replaces mt_qvm_b{3,4,5,6,8} (crates/metaltile-std/src/mlx/quantized.rs:4397-4530)
 * and mt_qvm_int4_fast (:4582-4700). K is cut into slices whose f32 partial rows go through a
 * library-owned buffer (allocated on first use, grown on demand). */
MTQ_API int mtq_qvm(int dtype, int bits, uint32_t group_size, const void *w, const void *scales, const void *biases,
                    const void *x, void *out, uint32_t M, uint32_t N, uint32_t K);

/* mtq_qvm for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same
 * arguments, same kernels and bit-identical results as mtq_qvm, but the f32 partial rows go
 * through a 4 MiB array that is part of the library's code object instead of a library-owned
 * allocation: the call makes no hipMalloc / hipFree. Shapes whose partial rows
 * (M * slices * N * 4 bytes, slices = about 512 / (ceil(N / 512) * M) workgroups' worth) exceed
 * 4 MiB fail with MTQ_ERR_UNSUPPORTED. Every call on a GPU shares that GPU's array: calls that
 * overlap on one GPU (two streams, two threads) race; calls on one stream are ordered. */
MTQ_API int mtq_qvm_noalloc(int dtype, int bits, uint32_t group_size, const void *w, const void *scales,
                            const void *biases, const void *x, void *out, uint32_t M, uint32_t N, uint32_t K);

/* Batched qmv: n_mats (1..4) weight matrices of the same K, code width and group size
 * against ONE activation row, in one launch: outs[j][n] = sum_k w_hat_j[n,k] * x[k].
 * Replaces ffai_batched_qkv_qgemv / _fast (three matrices, one concatenated output:
 * pass outs[j] = out + offset; crates/metaltile-std/src/ffai/batched_qkv_qgemv.rs:42-59,
 * 157-174) and ffai_batched_4_qgemv_fast (four matrices, four outputs;
 * crates/metaltile-std/src/ffai/batched_4_qgemv.rs:60-84), and fuses e.g. the gate and
 * up projections of an MLP. w / scales / biases / outs / N are host arrays of n_mats
 * device pointers / row counts. */
MTQ_API int mtq_qmv_batched(int dtype, int bits, uint32_t group_size, int n_mats, const void *const *w,
                            const void *const *scales, const void *const *biases, const void *x,
                            void *const *outs, const uint32_t *N, uint32_t K);

/* The same over M activation rows (a prefill step's Q / K / V or four projections): x T[M, K], outs[j] T[M, N[j]],
 * row m of every output the GEMV of activation row m, 1..4 matrices. Replaces ffai_batched_qkv_qmm_fast
 * (crates/metaltile-std/src/ffai/batched_qkv_qmm.rs:49-68) and ffai_batched_4_qmm_fast
 * (crates/metaltile-std/src/ffai/batched_4_qmm.rs:61-85), whose row count is the grid's second dimension (under those
 * names here too when mtq_dispatch is given a grid other than the all-ones placeholder, and `x` may then hold more rows;
 * without one: the rows `x` holds) and whose constraints (K % 512 == 0, N % 8 == 0, group 64, 4-bit) are not required.
 * One mtq_qmm per matrix, in order, with mtq_qmm's routing and arithmetic: outputs are bit-equal to single calls.
 * Dispatched under the reference names the matrices run on the qmv family at every M, which keeps those kernels'
 * exact-dequant arithmetic (as the `mt_qmm*` names do). w / scales / biases / outs / N are HOST arrays of device pointers / row counts. */
MTQ_API int mtq_qmm_batched(int dtype, int bits, uint32_t group_size, int n_mats, const void *const *w,
                            const void *const *scales, const void *const *biases, const void *x,
                            void *const *outs, const uint32_t *N, uint32_t M, uint32_t K);

/* RMSNorm fused into qmv: out[n] = sum_k w_hat[n,k] * (x[k] * norm_weight[k] * inv_rms),
 * inv_rms = 1 / sqrt(mean(x^2) + eps_buf[0]); eps_buf is a DEVICE pointer to one f32, as in the
 * reference. Replaces ffai_rms_norm_qgemv / _fast (4-bit) and ffai_rms_norm_qgemv_int8_fast
 * (crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:53-125, 128-456, 459-...). The normalised
 * activation is an f32 value as in the reference; the f16 / bf16 kernels carry it as a rounded
 * value plus a rounded remainder (16 significant bits). Rows the fused kernel does not take are
 * normalised into a library-owned buffer first (allocated on first use, grown on demand). */
MTQ_API int mtq_rms_norm_qmv(int dtype, int bits, uint32_t group_size, const void *x, const void *norm_weight,
                             const void *w, const void *scales, const void *biases, void *out, const float *eps_buf,
                             uint32_t N, uint32_t K);

/* Gated RMSNorm fused into a 4-bit qmv (the tail of a gated-delta-net layer): with y f32 [hv, dv], z T [hv, dv],
 * norm_weight T [dv], inner[r, d] = y[r, d] * inv_rms[r] * norm_weight[d] * silu(z[r, d]),
 * inv_rms[r] = 1 / sqrt(mean_d(y[r]^2) + eps_buf[0]), silu(v) = v / (1 + exp(-v)), and
 * out[n] = sum_i w_hat[n, i] * inner_flat[i] over i = r * dv + d in [0, hv * dv). y is f32 for every dtype;
 * eps_buf is a DEVICE pointer to one f32. Replaces ffai_gated_rms_norm_qgemv_int4_fast
 * (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:88-291), whose invariants (hv * dv % 512 == 0,
 * N % 8 == 0, group_size 64, dv % 32 == 0, hv even, hv * dv <= 8192) are not required here: any hv, dv >= 1 with
 * group_size dividing hv * dv. inner is an f32 value as in the reference (never rounded to T); the f16 / bf16 kernels
 * carry it as a rounded value plus a rounded remainder (16 significant bits). One launch for f16 / bf16 when hv * dv is a
 * multiple of 2048 (at most 16384) and dv is 32 .. 2048 in powers of two; otherwise inner is written to a library-owned
 * buffer first (allocated on first use, grown on demand) and an ordinary qmv follows. */
MTQ_API int mtq_gated_rms_norm_qmv(int dtype, uint32_t group_size, const float *y, const void *z, const void *norm_weight,
                                   const float *eps_buf, const void *w, const void *scales, const void *biases, void *out,
                                   uint32_t hv, uint32_t dv, uint32_t N);

/* ---- MoE routing around gather_qmv -------------------------------------------------- */

/* Top-k experts per token row and their softmax weights. logits T[n_rows, n_experts] ->
 * indices_out u32[n_rows, k], weights_out T[n_rows, k]. norm_topk_prob 1: softmax over the chosen
 * k; 0: softmax over all experts, not renormalised. n_experts <= 1024, k <= 32. Ties go to the
 * smaller index; NaN is never chosen. Replaces mt_moe_router_topk
 * (crates/metaltile-std/src/ffai/moe.rs:65-199). */
MTQ_API int mtq_moe_router_topk(int dtype, const void *router_logits, uint32_t *indices_out, void *weights_out,
                                uint32_t n_rows, uint32_t n_experts, uint32_t k, uint32_t norm_topk_prob);

/* Stable sort of the n_tokens * k (token, slot) entries of `indices` by expert, on the device:
 * sort_token_idx u32[n*k] (source token of each sorted row: input of mtq_moe_permute),
 * inv_perm u32[n_tokens, k] (sorted row of each entry: input of mtq_moe_unpermute) and
 * expert_offsets u32[n_experts + 1] (CSR bounds: input of mtq_gather_qmv_csr). The reference has
 * no kernel for this step: its callers sort on the host (crates/metaltile-std/src/ffai/moe.rs:
 * 256-275 describes the two permutations). Up to 2048 experts: any number of entries (counting
 * sort); more experts: at most 32768 entries (sorting network). Expert ids >= n_experts are treated
 * as n_experts - 1. */
MTQ_API int mtq_moe_sort_by_expert(const uint32_t *indices, uint32_t n_tokens, uint32_t k, uint32_t n_experts,
                                   uint32_t *sort_token_idx, uint32_t *inv_perm, uint32_t *expert_offsets);

/* permuted[p, :] = tokens[sort_token_idx[p], :], p < n_permuted. A source index >= n_tokens gives
 * a zero row. Replaces mt_moe_permute (crates/metaltile-std/src/ffai/moe.rs:282-302). */
MTQ_API int mtq_moe_permute(int dtype, const void *tokens, const uint32_t *sort_token_idx, void *permuted,
                            uint32_t n_tokens, uint32_t n_permuted, uint32_t hidden);

/* out[t, h] = sum_j top_k_weights[t, j] * expert_outputs[inv_perm[t, j], h] (f32, j ascending).
 * A position >= n_permuted contributes nothing. Replaces mt_moe_unpermute
 * (crates/metaltile-std/src/ffai/moe.rs:225-251). */
MTQ_API int mtq_moe_unpermute(int dtype, const void *expert_outputs, const uint32_t *inv_perm,
                              const void *top_k_weights, void *out, uint32_t n_tokens, uint32_t n_permuted,
                              uint32_t hidden, uint32_t k);

/* Fused MoE decode step for one token: out[i] = sum_k slot_weights[k] * sum_d w_hat[expert_indices[k]][i][d] *
 * silu(gate_k[d]) * up_k[d], 4-bit weights stacked [n_experts, out_dim, in_dim/8]. gates / ups: host arrays of
 * n_slots (1..8) device pointers to T[in_dim]; expert_indices u32[n_slots] and slot_weights T[n_slots] on the
 * device (the outputs of the router). in_dim % 32 == 0, in_dim <= 4096, group_size a power of two >= 32.
 * Replaces ffai_moe_down_swiglu_accum_int4_chain8 (8 slots;
 * crates/metaltile-std/src/ffai/moe_down_swiglu_accum.rs:146-282). */
MTQ_API int mtq_moe_down_swiglu_accum(int dtype, uint32_t group_size, uint32_t n_slots, const void *const *gates,
                                      const void *const *ups, const uint32_t *expert_indices, const void *slot_weights,
                                      const void *w, const void *scales, const void *biases, void *out, uint32_t in_dim,
                                      uint32_t out_dim, uint32_t n_experts);

/* ---- the packed format's writer and reader ------------------------------ */

/* Affine quantise: per group of `group_size` consecutive elements of w (T[n_elem]),
 * scale = (max - min) / (2^bits - 1) (1 when below 1e-7), bias = min,
 * code = trunc(clamp((v - bias) * (1 / scale) + 0.5, 0, 2^bits - 1)); codes go to
 * `out` as an LSB-first bit stream of u32 words (n_elem * bits / 32 of them),
 * scale and bias to scales / biases (T[n_elem / group_size]). Replaces
 * mt_affine_quantize_int{2,3,4,5,6,8}
 * (crates/metaltile-std/src/mlx/quantized.rs:3629-3671, 3707, 3793, 3871, 3935, 4005).
 * bits in 2..8; group_size a multiple of 8 (4-, 8-bit), 16 (2-bit) or 32 (other
 * widths) with a power-of-two quotient; n_elem a multiple of group_size. */
MTQ_API int mtq_affine_quantize(int dtype, int bits, uint32_t group_size, const void *w, void *out,
                                void *scales, void *biases, size_t n_elem);

/* Affine dequantise: out[i] = scales[i / group_size] * code_i + biases[i / group_size]
 * rounded to T. Replaces mt_affine_dequantize_int{2,3,4,5,6,8}
 * (crates/metaltile-std/src/mlx/quantized.rs:3575-3611, 3681, 3762, 4081, 4127, 4179).
 * Same constraints as mtq_affine_quantize. */
MTQ_API int mtq_affine_dequantize(int dtype, int bits, uint32_t group_size, const void *w,
                                  const void *scales, const void *biases, void *out, size_t n_elem);

/* Dequantising gather (a quantized embedding table): out[t, d] = scales[id, d / group_size] * code[id, d] +
 * biases[id, d / group_size] rounded to T, id = indices[t]; weight u32[vocab, hidden * bits / 32] (each row a bit
 * stream, element d at bits [d * bits, (d + 1) * bits)), scales / biases T[vocab, hidden / group_size], indices
 * u32[n_tokens], out T[n_tokens, hidden]. Replaces dequant_gather_int{2,3,4,5,6,8}
 * (crates/metaltile-std/src/ffai/dequant_gather.rs:45-100; under those names vocab is what `weight` holds and n_tokens
 * what `indices` holds). An id >= vocab names no row: that output row keeps its bytes (the reference reads past the
 * table). hidden and group_size multiples of 8 (4-, 8-bit), 16 (2-bit) or 32 (other widths), group_size / that a
 * power of two; hidden a multiple of group_size. */
MTQ_API int mtq_dequant_gather(int dtype, int bits, uint32_t group_size, const void *weight, const void *scales,
                               const void *biases, const uint32_t *indices, void *out, uint32_t n_tokens,
                               uint32_t hidden, uint32_t vocab);

/* ---- name-keyed dispatch (the reference's binding convention) ----------- */

/* Replaces Context::dispatch_with_grid (crates/metaltile-runtime/src/context.rs:269-283)
 * and GpuRunner::compile + measure(.., 0, 1) (crates/metaltile-std/src/runner.rs:287, 413):
 * `kernel_name` is the reference kernel's `name` ("mt_qmv", "mt_qmm_mma",
 * "dequant_gemv_int4", "mt_moe_gather_qmm_int4", ...), `bufs` are its tensor
 * parameters in signature order, `consts` its constexprs in signature order
 * (crates/metaltile-std/src/run_kernel.rs:183-188, 210-234). grid/tpg describe
 * the Metal launch and are accepted for compatibility; the HIP launch is
 * derived from name, dtype, constexprs and buffer lengths (one exception: the
 * ffai_batched_*_qmm_fast names take their row count from grid[1], as the
 * reference does). Buffers shorter
 * than the op needs fail with MTQ_ERR_BUFFER_SIZE. Blocks until the kernel has
 * finished; *elapsed_us (may be NULL) receives its GPU duration. An unknown
 * name fails with MTQ_ERR_UNKNOWN_KERNEL so a caller can fall back. */
MTQ_API int mtq_dispatch(const char *kernel_name, int dtype, const mtq_buf *bufs, int n_bufs,
                         const uint32_t *consts, int n_consts, const uint32_t grid[3],
                         const uint32_t tpg[3], double *elapsed_us);

/* Replaces GpuRunner::measure (crates/metaltile-std/src/runner.rs:198-231, 413): `warmup`
 * untimed launches, then `iters` launches whose individual GPU durations (us)
 * are written to samples_us[iters]. */
MTQ_API int mtq_measure(const char *kernel_name, int dtype, const mtq_buf *bufs, int n_bufs,
                        const uint32_t *consts, int n_consts, const uint32_t grid[3],
                        const uint32_t tpg[3], int warmup, int iters, double *samples_us);

/* One entry of a dispatch chain: the arguments of mtq_dispatch minus grid/tpg. */
typedef struct mtq_dispatch_spec {
    const char *kernel_name;
    int dtype;
    const mtq_buf *bufs;
    int n_bufs;
    const uint32_t *consts;
    int n_consts;
} mtq_dispatch_spec;

/* Replaces Context::dispatch_chain over resident buffers
 * (crates/metaltile-runtime/src/context.rs:363-401; used with upload_resident by the
 * reference's perf tests, crates/metaltile-std/tests/qmm_gpu_correctness.rs:587-621):
 * enqueue the `n` dispatches in order, `repeat` times over, with no host wait
 * in between, then wait for the last. per_kernel_us (NULL or n*repeat entries)
 * receives each dispatch's own GPU duration; wall_us (may be NULL) the host
 * clock from the first enqueue to completion of the last; stream_us (may be
 * NULL) the time between two events recorded on the stream before the first
 * and after the last dispatch. Attaching per-kernel events costs host time per
 * launch, so ask for per_kernel_us and for the bracketing times in separate calls. */
MTQ_API int mtq_dispatch_chain(const mtq_dispatch_spec *specs, int n, int repeat,
                               double *per_kernel_us, double *wall_us, double *stream_us);

/* ---- planning without a device ------------------------------------------- */

/* What a call WOULD launch, computed by the same routing and geometry code as the call itself, with no device, no
 * mtq_init and no allocation: the counterpart of the reference's host-side checks before encoding a dispatch
 * (crates/metaltile-runtime/src/dispatch/single_dispatch.rs:142-158, buffer_plan.rs:62-77). Returns what the typed
 * entry point of `op` would return for these arguments as far as shapes decide it (MTQ_OK, MTQ_ERR_BAD_ARG,
 * MTQ_ERR_SHAPE, MTQ_ERR_UNSUPPORTED) and fills `info` with every kernel launch in order (name, grid, block, dynamic
 * LDS bytes) and the library-owned scratch bytes the call would need. M is the activation row count (qmv, qmm, qvm),
 * T the routed row count and E the expert count of the gathers; unused ones are ignored. The compute-unit count
 * that some geometries depend on is the current device's, or 256 without one. Options set with mtq_set_option apply. */
enum mtq_op {
    MTQ_OP_QMV = 0,
    MTQ_OP_QMM = 1,             /* mt_qmm*: exact dequantisation, any row count */
    MTQ_OP_QMM_MMA = 2,         /* mt_qmm_mma*: weights rounded to the element type first */
    MTQ_OP_QVM = 3,
    MTQ_OP_GATHER_CSR = 4,
    MTQ_OP_GATHER_INDICES = 5,
    MTQ_OP_GATHER_SINGLE = 6,
    MTQ_OP_RMS_NORM_QMV = 7
};
#define MTQ_PLAN_MAX_LAUNCHES 8
typedef struct mtq_plan_launch {
    char kernel[192];           /* demangled kernel name with its template arguments */
    uint32_t grid[3];           /* workgroups */
    uint32_t block[3];          /* threads per workgroup */
    size_t lds_bytes;           /* dynamic LDS per workgroup */
} mtq_plan_launch;
typedef struct mtq_plan_info {
    int n_launches;             /* launches the call makes; only the first MTQ_PLAN_MAX_LAUNCHES are described */
    mtq_plan_launch launch[MTQ_PLAN_MAX_LAUNCHES];
    size_t scratch_bytes;       /* library-owned device scratch the call needs (0 if none) */
} mtq_plan_info;
MTQ_API int mtq_plan(int op, int dtype, int bits, uint32_t group_size, uint32_t M, uint32_t N, uint32_t K, uint32_t E,
                     uint32_t T, mtq_plan_info *info);

/* 1 if mtq_dispatch knows `kernel_name`, else 0. */
MTQ_API int mtq_kernel_supported(const char *kernel_name);
/* Number of names mtq_dispatch knows, and the i-th of them (NULL past the end). */
MTQ_API int mtq_kernel_count(void);
MTQ_API const char *mtq_kernel_name(int i);

/* Replaces mt_qmm_for (crates/metaltile-std/src/mlx/quantized.rs:5040-5065): the name of
 * the reference kernel its selector would pick for M rows. */
MTQ_API const char *mtq_qmm_for(int dtype, uint32_t m);

/* Replaces GpuRunner::flush_slc (crates/metaltile-std/src/runner.rs:444-475): 16 read-modify-
 * write dispatches (the reference's SLC_FLUSH_DISPATCHES, runner.rs:245) over a scratch region
 * three times the size of the last-level cache, the last four of which touch every byte of it, so
 * that the next launch starts cold and follows sustained full-grid load. Waits for the dispatches. */
MTQ_API int mtq_flush_cache(void);

/* Tuning knobs (no counterpart in the reference). Known names:
 *   "qmv.kernel"           0 = choose per shape (default), 1 = one-shot kernel, 2 = streaming kernel, 3 = the wave-per-four-rows /
 *                          wave-per-row kernels wherever they apply (2- and 4-bit codes, f16 / bf16), 4 = the kernel whose
 *                          waves walk the rows wherever it applies (one row of x, rows of 2048 to 8192 4-bit codes in steps of 1024, or 3584, in
 *                          groups of 32 / 64 / 128, f16 / bf16; also the batched form of mtq_qmv_batched)
 *   "qmv.rows_per_thread"  one-shot kernel: 0 = choose per shape, or 4 / 7 / 8
 *   "qmv.stream_depth"     streaming kernel: 0 = choose per shape, or 4 / 8 loads in flight per thread
 *   "qmv.stream_batches"   streaming kernel: 0 = choose per shape, or 1..16 batches per thread
 *   "qmv.mfma"             matrix-core GEMV kernel: 0 = choose per shape, 1 = never, 2 = wherever it applies
 *   "qmv.mfma_kp" / "qmv.mfma_rbw" / "qmv.mfma_nrb" / "qmv.mfma_sets"
 *                          matrix-core GEMV geometry: K parts per row, row blocks side by side and one
 *                          after the other per workgroup, 4-row activation sets per pass; 0 = choose
 *   "qmv.gated_fused"      mtq_gated_rms_norm_qmv as one launch of the streaming kernel (hv * dv a multiple of 2048 up to
 *                          16384, dv = 32 .. 2048 in powers of two): 0 = for f16 / bf16, 1 = never (the activation is staged
 *                          in the library's buffer), 2 = wherever the shape allows
 *   "qmv.norm_mfma"        mtq_rms_norm_qmv with the norm applied inside the matrix-core GEMV (4-bit codes, f16 / bf16):
 *                          0 = where it is faster than the streaming kernel's fused form, 1 = never, 2 = wherever the
 *                          shape allows
 *   "gather.wide"          expert-routed rows on the 16-row matrix-core GEMV (4-bit g64 f16 / bf16, K <= 4608): 0 = where
 *                          it is the fastest kernel (large experts, at least 4 rows per expert, below the tile
 *                          kernel's crossover or under an exact-dequant name), 1 = never, 2 = wherever the shape allows
 *   "qmv.wide"             16-row matrix-core GEMV for batches of 5..16 rows (4-bit codes, f16 / bf16, K % 512 == 0):
 *                          0 = where it is the fastest kernel, 1 = never, 2 = wherever the shape allows
 *   "qmv.wide_kp"          that kernel: waves that share a row block, 0 = choose, or 1 / 2 / 4 / 8 / 16
 *   "qmv.wide_nb"          that kernel: row blocks per wave, 0 = choose, or 1 / 2
 *   "qmm.kernel"           0 = choose per shape, 1 = tile kernel with both operands through LDS, 2 = tile
 *                          kernel with the weights converted in registers
 *   "qmm.kgroups"          register-operand tile kernel: K-groups per workgroup, 0 = choose, or 1 / 2 / 4
 *   "qmm.tile_rows"        activation rows per tile, 0 = choose, or 32 (4 K-groups only) / 64 / 128 / 256 (4- and 8-bit
 *                          codes on 2 K-groups only)
 *   "qmm.dma"              tile instances that bring the activation tile in by load-to-LDS instructions (4- and 8-bit
 *                          codes): 0 = where the shape allows and it pays (8-bit codes: rows of 8192 codes and more, or
 *                          launches that fill the chip), 1 = never (the register-staged instances; same results bit for
 *                          bit), 2 = with the scales and biases in windows even where whole rows fit, 3 = wherever the
 *                          shape allows
 *   "qmm.by_m"             order in which workgroups walk the tiles: 0 = choose, 1 = the N-tiles of one M-tile
 *                          first, 2 = the M-tiles of one N-tile first
 *   "qmm.splits"           LDS tile kernel: 0 = choose per shape, or the number of K slices per output tile
 *   "qmm.ksplit"           register-operand tile kernel: 0 = choose, 1 = never split K, n = n splits (f32 partial
 *                          tiles in the library-owned buffer, added in split order by a second kernel)
 *   "qmm.f32_tiles"        f32 batches on the f32 matrix-core kernel: 0 = choose by rows, 1 = never, 2 = always
 *   "gather.grouped"       gather_qmv with many rows per expert on the tile kernel: 0 = choose, 1 = never, 2 = always
 *   "gather.names_exact"   the exact-dequant gather names of mtq_dispatch (mt_moe_gather_qmm_int4, _m8, _m16, _m32, _b3 ..
 *                          _b8): 0 = always on the GEMV kernels (exact s*q + b, as those reference kernels compute), 1 = grouped
 *                          on the tile kernel above 8 rows per expert like the typed entry points (w_hat rounded to T first)
 *   "qvm.wgs"              qvm: workgroups to aim for when K is sliced, 0 = choose
 *   "moe.sort"             expert sort: 0 = choose by size, 1 = always the bitonic network
 *   "moe_down.rows"        fused MoE down projection: output rows per workgroup, 0 = choose
 * Results do not depend on any of them beyond the order of floating-point sums.
 * Unknown names or values fail with MTQ_ERR_BAD_ARG. */
MTQ_API int mtq_set_option(const char *name, int value);

/* Timing helper for callers that launch through the typed entry points: the
 * next launch made by this thread attaches GPU timestamps; mtq_timed_last_us
 * waits for it and returns its duration. */
MTQ_API int mtq_timed_begin(void);
MTQ_API int mtq_timed_last_us(double *elapsed_us);

#ifdef __cplusplus
}
#endif
#endif /* MTQ_H */
