// Generic affine-quantized GEMV: one wave per output element, any code width
// 2..8 (bit-stream packing, codes may straddle two words) and any group size
// that divides K. Correctness-first counterpart of the reference's scalar
// kernels mt_qmv_b{3,4,5,6,8} / mt_qmm_b*
// (crates/metaltile-std/src/mlx/quantized.rs:4273-4392), dequant_gemv_int{3,5,6}
// (crates/metaltile-std/src/ffai/dequant_gemv.rs:109-161) and
// mt_moe_gather_qmm_b{3,5,6,8} (crates/metaltile-std/src/ffai/moe.rs:461-605);
// also the fallback for shapes the tiled kernel's geometry does not cover.
#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

struct GenArgs {
    const uint32_t* w;
    const void* scales;
    const void* biases;
    const void* x;
    void* out;
    const uint32_t* route;
    uint32_t rows, N, K, bits, G, T, E;
};

template <int DT, int MODE> __global__ __launch_bounds__(64) void qmv_generic_kernel(GenArgs a) {
    const uint32_t n = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    uint32_t e = 0;
    if constexpr (MODE == GATHER_CSR) {
        // first e with t < off[e+1], else 0 (crates/metaltile-std/src/ffai/moe.rs:376-385)
        for (uint32_t j = 0; j < a.E; j++)
            if (t < a.route[j + 1]) { e = j; break; }
    } else if constexpr (MODE == GATHER_INDICES) {
        e = a.route[t];
        if (e >= a.E) return;  // never read outside the stacked slabs
    } else if constexpr (MODE == GATHER_SINGLE) {
        e = min(a.route[0], a.E - 1);
    }
    const uint32_t wpr = a.K * a.bits / 32, gpr = a.K / a.G;
    const size_t orow = (size_t)e * a.N + n;
    const uint32_t* rw = a.w + orow * wpr;
    const uint32_t mask = (1u << a.bits) - 1u;
    float acc = 0.f;
    for (uint32_t j = lane; j < a.K; j += 64) {
        uint32_t bit_off = j * a.bits;
        uint32_t word = bit_off >> 5, in_w = bit_off & 31u;
        uint64_t two = rw[word];
        if (in_w + a.bits > 32) two |= (uint64_t)rw[word + 1] << 32;
        float q = (float)((uint32_t)(two >> in_w) & mask);
        uint32_t g = j / a.G;
        float s = load_elem<DT>(a.scales, orow * gpr + g);
        float b = load_elem<DT>(a.biases, orow * gpr + g);
        acc = fmaf(fmaf(q, s, b), load_elem<DT>(a.x, (size_t)t * a.K + j), acc);
    }
    acc = seg_allreduce(acc, 64);
    if (lane == 0) store_elem<DT>(a.out, (size_t)t * a.N + n, acc);
}

template <int DT> static int launch_gen(GenArgs& a, int mode, const LaunchCtx& lc) {
    const void* fn;
    switch (mode) {
        case GATHER_NONE: fn = (const void*)qmv_generic_kernel<DT, GATHER_NONE>; break;
        case GATHER_CSR: fn = (const void*)qmv_generic_kernel<DT, GATHER_CSR>; break;
        case GATHER_INDICES: fn = (const void*)qmv_generic_kernel<DT, GATHER_INDICES>; break;
        default: fn = (const void*)qmv_generic_kernel<DT, GATHER_SINGLE>; break;
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3(a.N, a.rows, 1), dim3(64), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "generic qmv kernel launch");
    return ERR_OK;
}

int launch_qmv_generic(const QmvParams& p, const LaunchCtx& lc) {
    if (p.bits < 2 || p.bits > 8) return fail(ERR_BAD_ARG, "bits must be in 2..8");
    if (p.N == 0 || p.K == 0 || p.group_size == 0) return fail(ERR_SHAPE, "N, K and group_size must be non-zero");
    if (p.K % p.group_size) return fail(ERR_SHAPE, "group_size must divide K");
    if ((uint64_t)p.K * p.bits % 32) return fail(ERR_SHAPE, "K*bits must be a multiple of 32");
    GenArgs a;
    a.w = (const uint32_t*)p.w;
    a.scales = p.scales;
    a.biases = p.biases;
    a.x = p.x;
    a.out = p.out;
    a.route = p.route;
    const bool gather = p.gather == GATHER_CSR || p.gather == GATHER_INDICES;
    a.rows = gather ? p.T : (p.gather == GATHER_SINGLE ? 1u : p.M);
    a.N = p.N;
    a.K = p.K;
    a.bits = (uint32_t)p.bits;
    a.G = p.group_size;
    a.T = p.T;
    a.E = p.E;
    if (a.rows == 0) return ERR_OK;
    if (a.rows > 65535) return fail(ERR_UNSUPPORTED, "generic qmv: more than 65535 rows in one launch");
    switch (p.dtype) {
        case DT_F32: return launch_gen<DT_F32>(a, p.gather, lc);
        case DT_F16: return launch_gen<DT_F16>(a, p.gather, lc);
        case DT_BF16: return launch_gen<DT_BF16>(a, p.gather, lc);
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
}

}  // namespace mtq
