// Fused MoE decode step: SwiGLU of each routed slot, the 4-bit down projection against that
// slot's expert, and the routing-weighted sum over slots, in one launch
// (reference: ffai_moe_down_swiglu_accum_int4_chain8,
// crates/metaltile-std/src/ffai/moe_down_swiglu_accum.rs:146-282).
//
// A workgroup stages slot_w[k] * silu(gate_k) * up_k for every slot in LDS as f32 (the
// reference keeps the activation in f32 too), then each of its four waves takes output rows:
// the 64 lanes split the (slot, 16-byte weight chunk) pairs of a row between them, so one
// wave-wide load covers whole 16-byte pieces of up to eight different experts' rows.
#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

struct MoeDownArgs {
    const void* gate[8];
    const void* up[8];
    const uint32_t* experts;
    const void* slot_w;
    const uint32_t* w;
    const void* scales;
    const void* biases;
    void* out;
    uint32_t in_dim, out_dim, log2g, n_experts, n_slots, rows_per_wg, wide_acts;
};

template <int DT> __global__ __launch_bounds__(256) void moe_down_swiglu_kernel(MoeDownArgs a) {
    extern __shared__ __align__(16) float inner[];  // [n_slots][in_dim]
    __shared__ uint32_t expert_of[8];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    if (tid < a.n_slots) expert_of[tid] = min(a.experts[tid], a.n_experts - 1);
    // Every (slot, 16-byte piece) of the gate / up rows is one item; a thread issues the loads of
    // up to four items before it touches any of them, so the staging costs one memory round trip.
    // Pointers are picked with compare-selects: an indexed read of the argument arrays would go
    // through scratch memory.
    auto gate_of = [&](uint32_t k) {
        return k == 0 ? a.gate[0] : k == 1 ? a.gate[1] : k == 2 ? a.gate[2] : k == 3 ? a.gate[3]
             : k == 4 ? a.gate[4] : k == 5 ? a.gate[5] : k == 6 ? a.gate[6] : a.gate[7];
    };
    auto up_of = [&](uint32_t k) {
        return k == 0 ? a.up[0] : k == 1 ? a.up[1] : k == 2 ? a.up[2] : k == 3 ? a.up[3]
             : k == 4 ? a.up[4] : k == 5 ? a.up[5] : k == 6 ? a.up[6] : a.up[7];
    };
    typedef typename Elem<DT>::type elem_t;
    if (a.wide_acts) {
        constexpr int V = DT == DT_F32 ? 4 : 8;  // elements per 16-byte load (in_dim % 32 == 0)
        const uint32_t per_slot = a.in_dim / V, total = a.n_slots * per_slot;
        for (uint32_t base = 0; base < total; base += 1024) {
            uint4 gv[4], uv[4];
            float sw[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint32_t it = min(base + u * 256 + tid, total - 1);
                const uint32_t k = it / per_slot, d = (it - k * per_slot) * V;
                gv[u] = *(const uint4*)((const elem_t*)gate_of(k) + d);
                uv[u] = *(const uint4*)((const elem_t*)up_of(k) + d);
                sw[u] = load_elem<DT>(a.slot_w, k);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint32_t it = base + u * 256 + tid;
                if (it >= total) break;
                const uint32_t k = it / per_slot, d = (it - k * per_slot) * V;
#pragma unroll
                for (int i = 0; i < V; i++) {
                    const float g = load_elem<DT>(&gv[u], i), up = load_elem<DT>(&uv[u], i);
                    const float silu = g / (1.0f + expf(0.0f - g));
                    inner[k * a.in_dim + d + i] = sw[u] * (silu * up);
                }
            }
        }
    } else {
        for (uint32_t it = tid; it < a.n_slots * a.in_dim; it += 256) {
            const uint32_t k = it / a.in_dim, d = it - k * a.in_dim;
            const float g = load_elem<DT>(gate_of(k), d), up = load_elem<DT>(up_of(k), d);
            const float silu = g / (1.0f + expf(0.0f - g));
            inner[it] = load_elem<DT>(a.slot_w, k) * (silu * up);
        }
    }
    __syncthreads();
    const uint32_t chunks = a.in_dim / 32;      // 16-byte pieces of a 4-bit row
    const uint32_t items = a.n_slots * chunks;
    const uint32_t ng = a.in_dim >> a.log2g;
    for (uint32_t r = wave; r < a.rows_per_wg; r += 4) {
        const uint32_t row = blockIdx.x * a.rows_per_wg + r;
        if (row >= a.out_dim) break;  // uniform per wave
        float acc = 0.f;
        for (uint32_t it = lane; it < items; it += 64) {
            const uint32_t k = it / chunks, c = it - k * chunks;
            const size_t erow = (size_t)expert_of[k] * a.out_dim + row;
            const uint4 wv = *(const uint4*)(a.w + erow * (a.in_dim / 8) + c * 4);
            const uint32_t g = (c * 32) >> a.log2g;
            const float sc = load_elem<DT>(a.scales, erow * ng + g), bi = load_elem<DT>(a.biases, erow * ng + g);
            const float4* xv = (const float4*)(inner + k * a.in_dim + c * 32);
            const uint32_t wd[4] = {wv.x, wv.y, wv.z, wv.w};
            float dot = 0.f, xs = 0.f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const float4 x0 = xv[2 * d], x1 = xv[2 * d + 1];
                const uint32_t q = wd[d];
                dot = fmaf((float)(q & 15u), x0.x, dot);
                dot = fmaf((float)((q >> 4) & 15u), x0.y, dot);
                dot = fmaf((float)((q >> 8) & 15u), x0.z, dot);
                dot = fmaf((float)((q >> 12) & 15u), x0.w, dot);
                dot = fmaf((float)((q >> 16) & 15u), x1.x, dot);
                dot = fmaf((float)((q >> 20) & 15u), x1.y, dot);
                dot = fmaf((float)((q >> 24) & 15u), x1.z, dot);
                dot = fmaf((float)(q >> 28), x1.w, dot);
                xs += (x0.x + x0.y) + (x0.z + x0.w) + (x1.x + x1.y) + (x1.z + x1.w);
            }
            acc += sc * dot + bi * xs;
        }
        acc = seg_allreduce(acc, 64);
        if (lane == 0) store_elem<DT>(a.out, row, acc);
    }
}

int launch_moe_down_swiglu(int dtype, uint32_t group_size, uint32_t n_slots, const void* const* gates, const void* const* ups,
                           const uint32_t* experts, const void* slot_w, const void* w, const void* scales, const void* biases,
                           void* out, uint32_t in_dim, uint32_t out_dim, uint32_t n_experts, const LaunchCtx& lc) {
    if (n_slots == 0 || n_slots > 8) return fail(ERR_SHAPE, "moe down: 1..8 slots");
    if (in_dim == 0 || out_dim == 0 || n_experts == 0) return fail(ERR_SHAPE, "in_dim, out_dim and n_experts must be non-zero");
    if (in_dim % 32 || in_dim > 4096) return fail(ERR_UNSUPPORTED, "moe down: in_dim must be a multiple of 32, at most 4096");
    if (group_size < 32 || (group_size & (group_size - 1)) || in_dim % group_size)
        return fail(ERR_UNSUPPORTED, "moe down: group_size must be a power of two >= 32 that divides in_dim");
    if (!gates || !ups || !experts || !slot_w || !w || !scales || !biases || !out) return fail(ERR_BAD_ARG, "null buffer");
    if ((uintptr_t)w % 16) return fail(ERR_UNSUPPORTED, "moe down: weights must be 16-byte aligned");
    MoeDownArgs a;
    bool wide = true;  // 16-byte loads of the gate / up rows
    for (uint32_t k = 0; k < 8; k++) {
        const uint32_t j = k < n_slots ? k : 0;
        if (!gates[j] || !ups[j]) return fail(ERR_BAD_ARG, "null gate / up buffer");
        a.gate[k] = gates[j];
        a.up[k] = ups[j];
        if ((uintptr_t)gates[j] % 16 || (uintptr_t)ups[j] % 16) wide = false;
    }
    a.wide_acts = wide ? 1u : 0u;
    a.experts = experts;
    a.slot_w = slot_w;
    a.w = (const uint32_t*)w;
    a.scales = scales;
    a.biases = biases;
    a.out = out;
    a.in_dim = in_dim;
    a.out_dim = out_dim;
    uint32_t lg = 0;
    while ((1u << lg) < group_size) lg++;
    a.log2g = lg;
    a.n_experts = n_experts;
    a.n_slots = n_slots;
    // about two workgroups per CU: the SwiGLU staging is repeated by every workgroup
    int dev = 0, n_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0)
        n_cu = 256;
    const uint32_t cus = (uint32_t)n_cu;
    uint32_t rpw = (out_dim + 2 * cus - 1) / (2 * cus);
    rpw = (rpw + 3) / 4 * 4;
    a.rows_per_wg = rpw;
    const size_t shmem = (size_t)n_slots * in_dim * sizeof(float);
    const void* fn;
    switch (dtype) {
        case DT_F32: fn = (const void*)moe_down_swiglu_kernel<DT_F32>; break;
        case DT_F16: fn = (const void*)moe_down_swiglu_kernel<DT_F16>; break;
        case DT_BF16: fn = (const void*)moe_down_swiglu_kernel<DT_BF16>; break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    if (shmem > 48 * 1024) {
        hipError_t e = set_max_dynamic_lds(fn, (size_t)shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3((out_dim + rpw - 1) / rpw), dim3(256), args, shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "moe down + swiglu kernel launch");
    return ERR_OK;
}

}  // namespace mtq
