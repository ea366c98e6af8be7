// Host-side declarations shared between the kernel launchers and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "mtq_types.h"

namespace mtq {

// Error codes returned across the C-ABI (0 = success).
enum : int {
    ERR_OK = 0,
    ERR_NO_DEVICE = -1,      // no usable GPU / library not initialised
    ERR_BAD_ARG = -2,        // null pointer, zero size, unsupported dtype/bits
    ERR_SHAPE = -3,          // shape violates the kernel's preconditions
    ERR_BUFFER_SIZE = -4,    // a bound buffer is shorter than the op requires
    ERR_UNKNOWN_KERNEL = -5, // name-keyed dispatch: name not in the table
    ERR_HIP = -6,            // a HIP runtime call failed
    ERR_UNSUPPORTED = -7,    // valid request this build has no kernel for
};

// Sets the calling thread's last-error string and returns `code`.
int fail(int code, const std::string& msg);
int hip_fail(hipError_t e, const char* what);

#define MTQ_HIP(call)                                      \
    do {                                                   \
        hipError_t e__ = (call);                           \
        if (e__ != hipSuccess) return ::mtq::hip_fail(e__, #call); \
    } while (0)

// Optional per-launch timing hooks: when both events are set they are attached
// to the kernel dispatch itself, so their difference is the kernel's own GPU
// duration (no launch gap, no host time).
struct LaunchCtx {
    hipStream_t stream = nullptr;
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};

hipError_t launch_kernel(const void* fn, dim3 grid, dim3 block, void** args, size_t shmem,
                         const LaunchCtx& lc);
// Raises a kernel's dynamic LDS limit (needed above 48 KB).
hipError_t set_max_dynamic_lds(const void* fn, size_t bytes);
// Planning (mtq_plan): the routing and geometry code runs as for a real call, but launch_kernel and
// set_max_dynamic_lds only record what they are given and nothing touches a device. Code that would allocate
// device scratch of its own asks planning() first and reports the bytes with plan_note_scratch instead.
bool planning();
void plan_note_scratch(size_t bytes);

// How the x/out rows of a GEMV-family launch are selected.
enum GatherMode : int {
    GATHER_NONE = 0,     // x[M,K] against one weight matrix
    GATHER_CSR = 1,      // rows sorted by expert, expert_offsets[E+1]
    GATHER_INDICES = 2,  // indices[T] gives the expert of each row
    GATHER_SINGLE = 3,   // one row against slab expert_index[0]
    GATHER_NORM = 4,     // matrix-core GEMV only: one row, RMS-normalised as it is staged (QmvParams::norm_w, norm_eps)
};

struct QmvParams {
    int dtype = 0;            // DT_F32 / DT_F16 / DT_BF16
    int bits = 4;             // 2..8
    uint32_t group_size = 64;
    const void* w = nullptr;       // u32 [E?][N][K*bits/32]
    const void* scales = nullptr;  // T   [E?][N][K/G]
    const void* biases = nullptr;
    const void* x = nullptr;       // T [M or T][K]
    void* out = nullptr;           // T [M or T][N]
    uint32_t M = 1, N = 0, K = 0;
    int gather = GATHER_NONE;
    const uint32_t* route = nullptr;  // expert_offsets / indices / expert_index
    uint32_t T = 0;                   // rows (gather modes)
    uint32_t E = 1;                   // experts
    const void* norm_w = nullptr;     // matrix-core GEMV: weights of an RMS norm applied to the one row of x first
    const float* norm_eps = nullptr;  // its epsilon (device memory)
};

// Several weight matrices with the same K, code width and group size against one
// activation row (the fused projections of a decode step).
struct QmvBatch {
    int n = 0;                       // 2..4 matrices
    const void* w[4] = {};
    const void* scales[4] = {};
    const void* biases[4] = {};
    void* out[4] = {};
    uint32_t N[4] = {};
};

// Tuning overrides set through mtq_set_option (0 = automatic).
struct Options {
    int moe_sort = 0;             // expert sort: 0 automatic, 1 bitonic network only
    int qvm_wgs = 0;              // qvm: target workgroup count (0 = 1024)
    int moe_down_rows = 0;        // fused MoE down projection: rows per workgroup (0 = automatic)
    int qmv_rows_per_thread = 0;  // one-shot kernel: weight rows per thread
    int qmv_kernel = 0;           // 0 auto, 1 one-shot only, 2 prefer streaming, 3 the wave-per-four-rows kernel wherever it applies
    int qmv_stream_depth = 0;     // streaming kernel: ring depth (4 / 8)
    int qmv_stream_batches = 0;   // streaming kernel: batches per thread
    int qmm_splits = 0;           // MFMA qmm: K splits per tile (0 = choose per shape)
    int qmm_kernel = 0;           // MFMA qmm: 0 auto, 1 both operands through LDS, 2 weights direct to registers
    int qmm_kgroups = 0;          // direct qmm: K-groups per workgroup (0 = choose; 1, 2, 4)
    int qmm_by_m = 0;             // direct qmm: 1 = an XCD keeps its M-tiles' activations and streams all weights
    int gather_grouped = 0;       // expert-routed rows on the tile kernel: 0 = choose by rows per expert, 1 = never, 2 = always
    int gather_names_exact = 0;   // name-keyed exact-dequant gathers (mt_moe_gather_qmm_int4*, _b*): 0 = never on the rounding tile kernel, 1 = by rows per expert
    int qmm_ksplit = 0;           // direct qmm: 0 = choose, 1 = never split K, n = n splits
    int qmm_f32_tiles = 0;        // f32 batches on the f32 matrix cores: 0 = choose by rows, 1 = never, 2 = always
    int qmm_tile_rows = 0;        // direct qmm: activation rows per tile (0 = choose; 32, 64, 128, 256)
    int qmm_dma = 0;              // direct qmm: activation tiles by load-to-LDS instructions: 0 = where it pays, 1 = never, 2 = with the scales in windows even where whole rows fit, 3 = wherever the shape allows
    int qmv_mfma = 0;             // matrix-core qmv: 0 auto, 1 never, 2 whenever the shape fits
    int qmv_mfma_kp = 0;          // matrix-core qmv: K parts per row block
    int qmv_mfma_rbw = 0;         // matrix-core qmv: row blocks walked in parallel per workgroup
    int qmv_mfma_nrb = 0;         // matrix-core qmv: row blocks per wave
    int qmv_mfma_sets = 0;        // matrix-core gather: 4-row MFMA sets per pass (0 = choose; 1, 2, 4)
    int qmv_gated_fused = 0;      // gated RMS norm inside the streaming kernel: 0 = choose, 1 = never (stage the row), 2 = wherever the shape allows
    int qmv_norm_mfma = 0;        // RMS norm fused into the matrix-core GEMV (4-bit f16 / bf16): 0 = choose, 1 = never, 2 = wherever the shape allows
    int qmv_wide_kp = 0;          // 16-row matrix-core GEMV: waves sharing a row block (0 = choose; 1, 2, 4, 8, 16)
    int qmv_wide_nb = 0;          // 16-row matrix-core GEMV: row blocks per wave (0 = choose; 1, 2)
    int gather_wide = 0;          // expert-routed rows on the 16-row matrix-core GEMV: 0 = choose, 1 = never, 2 = wherever the shape allows
    int qmv_wide = 0;             // 16-row matrix-core GEMV for batches of 5..16 rows: 0 = choose per shape, 1 = never, 2 = wherever the shape allows
};
Options& options();

// Fast LDS/dot2 GEMV family (qmv.hip). Returns ERR_UNSUPPORTED when the shape
// does not fit its geometry so the caller can fall back to the generic kernel.
int launch_qmv_fast(const QmvParams& p, const LaunchCtx& lc);
// One launch for all matrices of `b` (p carries dtype, bits, group size, x, K; its
// w / scales / biases / out / N are ignored). ERR_UNSUPPORTED when the shape does not
// fit the streaming kernel: the caller then runs the matrices one by one.
// RMSNorm of the activation row fused into the streaming qmv (eps: device f32).
// ERR_UNSUPPORTED when the shape does not fit: the caller normalises into scratch first.
int launch_qmv_norm(const QmvParams& p, const void* norm_w, const float* eps, const LaunchCtx& lc);
int launch_qmv_gated_norm(const QmvParams& p, const void* gate_z, const void* norm_w, const float* eps, uint32_t dv,
                          const LaunchCtx& lc);
// Standalone x'[k] = x[k] * norm_w[k] * rsqrt(mean(x^2) + eps): one f32 row, or for f16 / bf16
// two rows of K elements (rounded value, rounded remainder).
int launch_rms_norm(int dtype, const void* x, const void* norm_w, const float* eps, void* out, uint32_t K, const LaunchCtx& lc);
int launch_gated_rms_norm(int dtype, const float* y, const void* z, const void* norm_w, const float* eps, void* out,
                          uint32_t hv, uint32_t dv, const LaunchCtx& lc);
// MoE routing (moe.hip)
int launch_moe_router_topk(int dtype, const void* logits, uint32_t* indices, void* weights, uint32_t n_rows,
                           uint32_t n_experts, uint32_t k, uint32_t norm_topk_prob, const LaunchCtx& lc);
int launch_moe_sort(const uint32_t* indices, uint32_t n_tokens, uint32_t k, uint32_t n_experts, uint32_t* sort_token_idx,
                    uint32_t* inv_perm, uint32_t* expert_offsets, const LaunchCtx& lc);
int launch_moe_permute(int dtype, const void* tokens, const uint32_t* sort_token_idx, void* permuted, uint32_t n_tokens,
                       uint32_t n_permuted, uint32_t hidden, const LaunchCtx& lc);
int launch_moe_unpermute(int dtype, const void* expert_outputs, const uint32_t* inv_perm, const void* weights, void* out,
                         uint32_t n_tokens, uint32_t n_permuted, uint32_t hidden, uint32_t k, const LaunchCtx& lc);
int launch_moe_down_swiglu(int dtype, uint32_t group_size, uint32_t n_slots, const void* const* gates, const void* const* ups,
                           const uint32_t* experts, const void* slot_w, const void* w, const void* scales, const void* biases,
                           void* out, uint32_t in_dim, uint32_t out_dim, uint32_t n_experts, const LaunchCtx& lc);
// qvm (qvm.hip): p.w is [K, N] packed along N, p.scales / p.biases [K/G, N]; scratch holds
// qvm_scratch_bytes() of f32 partial rows.
size_t qvm_scratch_bytes(int bits, uint32_t group_size, uint32_t M, uint32_t N, uint32_t K);
int launch_qvm(const QmvParams& p, void* scratch, const LaunchCtx& lc);
int launch_add_rows(int dtype, const void* a, const void* b, void* out, uint32_t n, const LaunchCtx& lc);
int launch_qmv_batched(const QmvParams& p, const QmvBatch& b, const LaunchCtx& lc);
// Matrix-core streaming GEMV family for f16/bf16 (qmv_mfma.hip); same contract.
int launch_qmv_mfma(const QmvParams& p, const LaunchCtx& lc);
// One-wave-per-output kernel for any bit width 2..8 and any group size (generic.hip).
int launch_qmv_generic(const QmvParams& p, const LaunchCtx& lc);

struct QmmParams {
    int dtype = 0;
    int bits = 4;
    uint32_t group_size = 64;
    const void* w = nullptr;
    const void* scales = nullptr;
    const void* biases = nullptr;
    const void* x = nullptr;  // T [M][K]
    void* out = nullptr;      // T [M][N]
    uint32_t M = 0, N = 0, K = 0;
};
// Tiled MFMA GEMM with weights dequantised into LDS (qmm.hip).
int launch_qmm_mfma(const QmmParams& p, const LaunchCtx& lc);
// 64x128 tiles, weights converted in MFMA operand registers, activations through LDS (qmm_direct.hip).
// scratch: qmm_direct_scratch_bytes(p) bytes (0 when K is not split: then scratch may be null).
size_t qmm_direct_scratch_bytes(const QmmParams& p);
int launch_qmm_direct(const QmmParams& p, const LaunchCtx& lc, void* scratch);
// 16-row matrix-core GEMV (qmv_wide.hip): 4-bit codes, f16 / bf16, at most 16 rows, K % 512 == 0.
// scratch: qmv_wide_scratch_bytes(p) bytes (0 when K is not split: then scratch may be null).
bool qmv_wide_takes(const QmmParams& p);
size_t qmv_wide_scratch_bytes(const QmmParams& p);
int launch_qmv_wide(const QmmParams& p, const LaunchCtx& lc, void* scratch);
// The same kernel on expert-routed rows (p.gather = GATHER_CSR / GATHER_INDICES), 16 rows of an expert per pass.
int launch_qmv_wide_gather(const QmvParams& p, const LaunchCtx& lc);
// f32 operands on the f32 matrix cores, any code width (qmm_f32.hip).
// scratch: qmm_f32_scratch_bytes(p) bytes (0 when K is not split: then scratch may be null).
size_t qmm_f32_scratch_bytes(const QmmParams& p);
int launch_qmm_f32(const QmmParams& p, const LaunchCtx& lc, void* scratch);
// Expert-routed rows on the same kernel (many rows per expert): p holds one expert's shapes (N, K),
// x [T][K], out [T][N], w / scales / biases the stacked experts. `route` = CSR offsets [E + 1], or one
// expert id per row when per_row_ids. scratch: qmm_grouped_scratch_bytes() bytes.
size_t qmm_grouped_scratch_bytes(uint32_t T, uint32_t E, bool sort_rows, uint32_t tile_rows = 64);
int launch_qmm_grouped(const QmmParams& p, const uint32_t* route, bool per_row_ids, uint32_t T, uint32_t E, void* scratch,
                       const LaunchCtx& lc);
// The table of row tiles behind both grouped launchers: tiles[0] = count, tiles[1 + i] = (expert,
// first row in the row order, rows, 0); rowlist maps the row order to rows of x / out (null: identity).
struct GatherTiles {
    uint32_t* tiles = nullptr;
    const uint32_t* rowlist = nullptr;
    uint32_t max_tiles = 0;
    LaunchCtx last;
};
int build_gather_tiles(const uint32_t* route, bool per_row_ids, uint32_t T, uint32_t E, uint32_t tile_rows, void* scratch,
                       const LaunchCtx& lc, GatherTiles& out);
// The same for f32 operands, 32-row tiles on the f32 matrix-core kernel (qmm_f32.hip);
// scratch: qmm_grouped_scratch_bytes(T, E, per_row_ids, 32).
int launch_qmm_f32_grouped(const QmmParams& p, const uint32_t* route, bool per_row_ids, uint32_t T, uint32_t E, void* scratch,
                           const LaunchCtx& lc);

// The wave-per-row kernels (qmv_rows.hip): one activation row, f16 / bf16; rows of 4096 4-bit codes in groups of 64 (one wave per
// four rows), or 2- / 4-bit codes in groups of 32 / 64 / 128 on rows of 8192, 14336 (4-bit) or 16384 (2-bit) codes (one wave per row).
bool qmv_rows_takes(const QmvParams& p);
bool qmv_rows_preferred(const QmvParams& p);
int launch_qmv_rows(const QmvParams& p, const LaunchCtx& lc);
// RMS norm fused into the one-row-per-wave kernel (4-bit codes, rows of 4096 or 8192 codes, f16 / bf16).
bool qmv_rows_norm_takes(const QmvParams& p, const void* norm_w);
int launch_qmv_rows_norm(const QmvParams& p, const void* norm_w, const float* eps, const LaunchCtx& lc);
// The same walk without the norm (one activation row): qmv.kernel = 4 takes it wherever it applies.
bool qmv_rows_walk_takes(const QmvParams& p);
bool qmv_rows_walk_preferred(const QmvParams& p);
int launch_qmv_rows_walk(const QmvParams& p, const LaunchCtx& lc);
bool qmv_rows_walk_batched_takes(const QmvParams& p, const QmvBatch& b);       // (p: dtype, bits, group size, x, K)
bool qmv_rows_walk_batched_preferred(const QmvParams& p, const QmvBatch& b);
int launch_qmv_rows_walk_batched(const QmvParams& p, const QmvBatch& b, const LaunchCtx& lc);
// Two to four activation rows (qmv_rows_few.hip): one wave per four weight rows; 4096 or 8192 4-bit codes or 8192 2-bit codes per
// row, groups of 32 / 64 / 128, f16 / bf16.
bool qmv_rows_few_takes(const QmvParams& p);
bool qmv_rows_few_preferred(const QmvParams& p);
int launch_qmv_rows_few(const QmvParams& p, const LaunchCtx& lc);
// The same kernel as a measurement aid (bf16; mode 0 / 1 / 2 = full / no arithmetic / weight loads only; stamps may be null).
int launch_rows_probe(const void* w, const void* s, const void* b, const void* x, void* out, uint32_t N, int mode, uint64_t* stamps,
                      const LaunchCtx& lc);

// Affine quantise (quantize = true: T[n_elem] -> packed words + scales + biases) and
// dequantise (packed words + scales + biases -> T[n_elem]) (affine.hip).
int launch_affine(bool quantize, int dtype, int bits, uint32_t group_size, const void* in, void* out,
                  void* scales, void* biases, uint64_t n_elem, const LaunchCtx& lc);
int launch_dequant_gather(int dtype, int bits, uint32_t group_size, const void* weight, const void* scales, const void* biases,
                          const uint32_t* ids, void* out, uint32_t n_tokens, uint32_t hidden, uint32_t vocab, const LaunchCtx& lc);

}  // namespace mtq
