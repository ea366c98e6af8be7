// MoE routing around the gathered matmul: router top-k, the expert sort, permute and
// unpermute (reference kernels: crates/metaltile-std/src/ffai/moe.rs:65-302). All four are
// small latency- or bandwidth-bound kernels; none of them touches the matrix cores.
#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

// ---- router top-k -----------------------------------------------------------------------
// One 64-lane wave per token row, four rows per workgroup. Lane l holds experts l, l+64, ...
// in registers (NPL of them), so the k argmax passes run without touching memory again.

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = min(v, (uint32_t)__shfl_xor((int)v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

struct RouterArgs {
    const void* logits;
    uint32_t* indices;
    void* weights;
    uint32_t n_rows, n_experts, k, norm_topk_prob;
};

template <int DT, int NPL> __global__ __launch_bounds__(256) void moe_router_topk_kernel(RouterArgs a) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= a.n_rows) return;  // whole waves leave together; no barrier below
    const float NEG_INF = -__builtin_huge_valf();
    const size_t base = (size_t)row * a.n_experts;
    float v[NPL];
#pragma unroll
    for (int r = 0; r < NPL; r++) {
        const uint32_t j = r * 64u + lane;
        v[r] = j < a.n_experts ? load_elem<DT>(a.logits, base + j) : NEG_INF;
    }
    // softmax denominator over all experts (used when norm_topk_prob == 0)
    float m = NEG_INF;
#pragma unroll
    for (int r = 0; r < NPL; r++)
        if (v[r] > m) m = v[r];
    const float max_all = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < NPL; r++)
        if (r * 64u + lane < a.n_experts) s += expf(v[r] - max_all);
    const float sum_all = wave_sum(s);

    // k argmax passes; strict '>' from (-inf, 0), ties to the smaller index, NaN never wins
    uint32_t taken = 0, my_idx = 0;
    float my_val = NEG_INF;
    for (uint32_t it = 0; it < a.k; it++) {
        float best = NEG_INF;
        uint32_t bi = 0;
#pragma unroll
        for (int r = 0; r < NPL; r++) {
            const uint32_t j = r * 64u + lane;
            const float cand = (taken >> r) & 1u ? NEG_INF : v[r];
            if (j < a.n_experts && cand > best) {
                best = cand;
                bi = j;
            }
        }
        const float gbest = wave_max(best);
        const uint32_t gidx = wave_min_u32(best == gbest ? bi : 0xFFFFFFFFu);
        if ((gidx & 63u) == lane) taken |= 1u << (gidx >> 6);
        if (lane == it) {
            my_idx = gidx;
            my_val = gbest;
        }
    }
    const float e = lane < a.k ? expf(my_val - max_all) : 0.f;
    const float sum_chosen = wave_sum(e);
    const float w = e / (a.norm_topk_prob == 1u ? sum_chosen : sum_all);
    if (lane < a.k) {
        a.indices[(size_t)row * a.k + lane] = my_idx;
        store_elem<DT>(a.weights, (size_t)row * a.k + lane, w);
    }
}

template <int DT> static const void* router_fn(uint32_t npl) {
    switch (npl) {
        case 1: return (const void*)moe_router_topk_kernel<DT, 1>;
        case 2: return (const void*)moe_router_topk_kernel<DT, 2>;
        case 4: return (const void*)moe_router_topk_kernel<DT, 4>;
        case 8: return (const void*)moe_router_topk_kernel<DT, 8>;
        default: return (const void*)moe_router_topk_kernel<DT, 16>;
    }
}

int launch_moe_router_topk(int dtype, const void* logits, uint32_t* indices, void* weights, uint32_t n_rows,
                           uint32_t n_experts, uint32_t k, uint32_t norm_topk_prob, const LaunchCtx& lc) {
    if (n_experts == 0 || n_experts > 1024) return fail(ERR_SHAPE, "router: n_experts must be in 1..1024");
    if (k == 0 || k > 32 || k > n_experts) return fail(ERR_SHAPE, "router: k must be in 1..32 and <= n_experts");
    if (norm_topk_prob > 1) return fail(ERR_BAD_ARG, "router: norm_topk_prob must be 0 or 1");
    if (n_rows == 0) return ERR_OK;
    if (!logits || !indices || !weights) return fail(ERR_BAD_ARG, "null buffer");
    uint32_t npl = 1;
    while (npl * 64 < n_experts) npl *= 2;
    RouterArgs a{logits, indices, weights, n_rows, n_experts, k, norm_topk_prob};
    const void* fn;
    switch (dtype) {
        case DT_F32: fn = router_fn<DT_F32>(npl); break;
        case DT_F16: fn = router_fn<DT_F16>(npl); break;
        case DT_BF16: fn = router_fn<DT_BF16>(npl); break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3((n_rows + 3) / 4), dim3(256), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "router top-k kernel launch");
    return ERR_OK;
}

// ---- expert sort ------------------------------------------------------------------------
// Stable sort of the flattened (token * k + slot) entries by expert id: the step the
// reference leaves to its caller (crates/metaltile-std/src/ffai/moe.rs:256-275). One
// workgroup sorts the unique keys expert * 32768 + entry with a bitonic network in LDS
// (up to 32768 entries = 128 KB), then writes the permutation both ways and the CSR bounds.

struct SortArgs {
    const uint32_t* indices;    // [n] expert of each entry
    uint32_t* sort_token_idx;   // [n] source token of each sorted position
    uint32_t* inv_perm;         // [n] sorted position of each entry
    uint32_t* expert_offsets;   // [E + 1]
    uint32_t n, n_pad, k, n_experts;
};

__global__ __launch_bounds__(1024) void moe_sort_kernel(SortArgs a) {
    extern __shared__ uint32_t keys[];
    const uint32_t tid = threadIdx.x;
    for (uint32_t i = tid; i < a.n_pad; i += 1024)
        keys[i] = i < a.n ? min(a.indices[i], a.n_experts - 1) * 32768u + i : 0xFFFFFFFFu;
    __syncthreads();
    for (uint32_t size = 2; size <= a.n_pad; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t t = tid; t < a.n_pad / 2; t += 1024) {
                const uint32_t i = 2 * t - (t & (stride - 1));
                const uint32_t j = i + stride;
                const uint32_t x = keys[i], y = keys[j];
                if ((x > y) == ((i & size) == 0)) {
                    keys[i] = y;
                    keys[j] = x;
                }
            }
            __syncthreads();
        }
    }
    for (uint32_t p = tid; p < a.n; p += 1024) {
        const uint32_t key = keys[p], e = key >> 15, entry = key & 32767u;
        a.sort_token_idx[p] = entry / a.k;
        a.inv_perm[entry] = p;
        // experts (prev, e] start at p
        const uint32_t first = p == 0 ? 0u : (keys[p - 1] >> 15) + 1u;
        for (uint32_t x = first; x <= e; x++) a.expert_offsets[x] = p;
    }
    const uint32_t after = a.n == 0 ? 0u : (keys[a.n - 1] >> 15) + 1u;
    for (uint32_t x = after + tid; x <= a.n_experts; x += 1024) a.expert_offsets[x] = a.n;
}

// Counting sort, stable, for up to 2048 experts and any number of entries. The 16 waves of one
// workgroup own consecutive segments of the entries. Pass 1: per-wave histograms in LDS. Pass 2: the
// experts' CSR offsets (scan over experts) and, per wave and expert, where that wave's first entry
// of the expert goes. Pass 3: each wave walks its segment 64 entries at a time; an entry's place is
// its wave's cursor for the expert plus its rank among the equal entries of the 64 (the lanes with the
// same expert are found with one ballot per bit of the expert id), and the cursors move on. Waves never wait for each other after pass 2.
__global__ __launch_bounds__(1024) void moe_count_sort_kernel(SortArgs a) {
    extern __shared__ uint32_t tab[];            // [16][E] counts, then cursors
    const uint32_t E = a.n_experts, W = 16;
    uint32_t* offs = tab + W * E;                // [E] totals, then exclusive offsets
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const uint32_t seg = ((a.n + W - 1) / W + 63u) & ~63u;
    const uint32_t lo = min(a.n, w * seg), hi = min(a.n, lo + seg);
    for (uint32_t i = tid; i < W * E; i += 1024) tab[i] = 0;
    __syncthreads();
    for (uint32_t base = lo; base < hi; base += 64) {
        const uint32_t i = base + lane;
        if (i < hi) atomicAdd(&tab[w * E + min(a.indices[i], E - 1)], 1u);
    }
    __syncthreads();
    for (uint32_t e = tid; e < E; e += 1024) {
        uint32_t t = 0;
        for (uint32_t v = 0; v < W; v++) t += tab[v * E + e];
        offs[e] = t;
    }
    __syncthreads();
    if (w == 0) {  // exclusive scan over experts: each lane a run of consecutive experts, then across lanes
        const uint32_t per = (E + 63) / 64, e0 = lane * per, e1 = min(E, e0 + per);
        uint32_t sum = 0;
        for (uint32_t e = e0; e < e1; e++) sum += offs[e];
        uint32_t incl = sum;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, o, 64);
            if (lane >= (uint32_t)o) incl += up;
        }
        uint32_t run = incl - sum;
        for (uint32_t e = e0; e < e1; e++) {
            const uint32_t t = offs[e];
            offs[e] = run;
            run += t;
        }
    }
    __syncthreads();
    for (uint32_t e = tid; e < E; e += 1024) {
        uint32_t run = offs[e];
        a.expert_offsets[e] = run;
        for (uint32_t v = 0; v < W; v++) {
            const uint32_t c = tab[v * E + e];
            tab[v * E + e] = run;
            run += c;
        }
    }
    if (tid == 0) a.expert_offsets[E] = a.n;
    __syncthreads();
    uint32_t* cur = tab + w * E;
    uint32_t nbits = 0;
    while ((1u << nbits) < E) nbits++;
    uint32_t e_next = lo + lane < hi ? min(a.indices[lo + lane], E - 1) : 0u;  // one step ahead of its use
    for (uint32_t base = lo; base < hi; base += 64) {
        const uint32_t i = base + lane;
        const bool valid = i < hi;
        const uint32_t e = e_next;
        if (base + 64 + lane < hi) e_next = min(a.indices[base + 64 + lane], E - 1);
        // lanes holding the same expert: one ballot per bit of the expert id
        unsigned long long same = __ballot(valid);
        for (uint32_t bit = 0; bit < nbits; bit++) {
            const unsigned long long ones = __ballot((e >> bit) & 1u);
            same &= ((e >> bit) & 1u) ? ones : ~ones;
        }
        const uint32_t rank = (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
        if (valid) {
            const uint32_t pos = cur[e] + rank;
            a.sort_token_idx[pos] = i / a.k;
            a.inv_perm[i] = pos;
        }
        if (valid && rank == 0) cur[e] += (uint32_t)__popcll(same);  // after every lane of the wave has read its cursor
    }
}

int launch_moe_sort(const uint32_t* indices, uint32_t n_tokens, uint32_t k, uint32_t n_experts, uint32_t* sort_token_idx,
                    uint32_t* inv_perm, uint32_t* expert_offsets, const LaunchCtx& lc) {
    if (k == 0 || n_experts == 0 || n_experts > 65536) return fail(ERR_SHAPE, "expert sort: k >= 1, n_experts in 1..65536");
    const uint64_t n64 = (uint64_t)n_tokens * k;
    if (!expert_offsets || (n64 && (!indices || !sort_token_idx || !inv_perm))) return fail(ERR_BAD_ARG, "null buffer");
    if (n_experts <= 2048 && n64 > 128 && options().moe_sort != 1) {
        // counting sort: no limit on the entries held in LDS, 10 x faster than the network at 32768 entries
        if (n64 >= (1ull << 31)) return fail(ERR_UNSUPPORTED, "expert sort: too many entries");
        SortArgs a{indices, sort_token_idx, inv_perm, expert_offsets, (uint32_t)n64, 0, k, n_experts};
        const size_t shmem = (size_t)17 * n_experts * 4;
        if (shmem > 48 * 1024) {
            hipError_t e = set_max_dynamic_lds((const void*)moe_count_sort_kernel, (size_t)shmem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
        }
        void* args[] = {&a};
        hipError_t e = launch_kernel((const void*)moe_count_sort_kernel, dim3(1), dim3(1024), args, shmem, lc);
        if (e != hipSuccess) return hip_fail(e, "expert sort kernel launch");
        return ERR_OK;
    }
    if (n64 > 32768) return fail(ERR_UNSUPPORTED, "expert sort: more than 32768 (token, slot) entries with more than 2048 experts; sort on the host");
    uint32_t n_pad = 2;
    while (n_pad < n64) n_pad *= 2;
    SortArgs a{indices, sort_token_idx, inv_perm, expert_offsets, (uint32_t)n64, n_pad, k, n_experts};
    const size_t shmem = (size_t)n_pad * 4;
    if (shmem > 48 * 1024) {
        hipError_t e = set_max_dynamic_lds((const void*)moe_sort_kernel, (size_t)shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel((const void*)moe_sort_kernel, dim3(1), dim3(1024), args, shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "expert sort kernel launch");
    return ERR_OK;
}

// ---- permute / unpermute ----------------------------------------------------------------

struct PermuteArgs {
    const void* tokens;
    const uint32_t* sort_token_idx;
    void* permuted;
    uint32_t n_tokens, row_units;  // row length in copy units of UB bytes
};

// permuted[p, :] = tokens[sort_token_idx[p], :]; a source index past the token count gives a zero row.
template <typename U> __global__ __launch_bounds__(256) void moe_permute_kernel(PermuteArgs a) {
    const uint32_t p = blockIdx.x;
    const uint32_t token = a.sort_token_idx[p];
    const U* src = (const U*)a.tokens + (size_t)token * a.row_units;
    U* dst = (U*)a.permuted + (size_t)p * a.row_units;
    const bool ok = token < a.n_tokens;
    for (uint32_t i = threadIdx.x; i < a.row_units; i += 256) {
        U v = {};
        if (ok) v = src[i];
        dst[i] = v;
    }
}

int launch_moe_permute(int dtype, const void* tokens, const uint32_t* sort_token_idx, void* permuted, uint32_t n_tokens,
                       uint32_t n_permuted, uint32_t hidden, const LaunchCtx& lc) {
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "unknown dtype");
    if (hidden == 0) return fail(ERR_SHAPE, "hidden must be non-zero");
    if (n_permuted == 0) return ERR_OK;
    if (!tokens || !sort_token_idx || !permuted) return fail(ERR_BAD_ARG, "null buffer");
    const size_t row_bytes = (size_t)hidden * (dtype == DT_F32 ? 4 : 2);
    PermuteArgs a{tokens, sort_token_idx, permuted, n_tokens, 0};
    const void* fn;
    if (row_bytes % 16 == 0 && (uintptr_t)tokens % 16 == 0 && (uintptr_t)permuted % 16 == 0) {
        a.row_units = (uint32_t)(row_bytes / 16);
        fn = (const void*)moe_permute_kernel<uint4>;
    } else if (row_bytes % 4 == 0 && (uintptr_t)tokens % 4 == 0 && (uintptr_t)permuted % 4 == 0) {
        a.row_units = (uint32_t)(row_bytes / 4);
        fn = (const void*)moe_permute_kernel<uint32_t>;
    } else {
        a.row_units = (uint32_t)(row_bytes / 2);
        fn = (const void*)moe_permute_kernel<uint16_t>;
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3(n_permuted), dim3(256), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "permute kernel launch");
    return ERR_OK;
}

struct UnpermuteArgs {
    const void* expert_outputs;
    const uint32_t* inv_perm;
    const void* weights;
    void* out;
    uint32_t n_permuted, hidden, k;
};

// out[t, h] = sum_j w[t, j] * expert_outputs[inv_perm[t, j], h] in f32, j ascending, product and
// sum rounded separately; a position past the permuted row count contributes nothing.
// VEC elements per thread and step (16-byte loads when the row length and the pointers allow).
template <int DT, int VEC> __global__ __launch_bounds__(256) void moe_unpermute_kernel(UnpermuteArgs a) {
#pragma clang fp contract(off)
    typedef typename Elem<DT>::type elem_t;
    __shared__ uint32_t pos[32];
    __shared__ float wt[32];
    const uint32_t t = blockIdx.x;
    if (threadIdx.x < a.k) {
        const uint32_t p = a.inv_perm[(size_t)t * a.k + threadIdx.x];
        pos[threadIdx.x] = p < a.n_permuted ? p : 0xFFFFFFFFu;  // out-of-range slots are skipped below
        wt[threadIdx.x] = load_elem<DT>(a.weights, (size_t)t * a.k + threadIdx.x);
    }
    __syncthreads();
    for (uint32_t h = threadIdx.x * VEC; h < a.hidden; h += 256 * VEC) {
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] = 0.f;
        for (uint32_t j = 0; j < a.k; j++) {
            if (pos[j] == 0xFFFFFFFFu) continue;  // uniform over the workgroup
            elem_t v[VEC];
            const elem_t* src = (const elem_t*)a.expert_outputs + (size_t)pos[j] * a.hidden + h;
            if constexpr (VEC > 1) {
                *(uint4*)v = *(const uint4*)src;
            } else {
                v[0] = src[0];
            }
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const float prod = wt[j] * load_elem<DT>(v, i);
                acc[i] = acc[i] + prod;
            }
        }
        elem_t o[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) store_elem<DT>(o, i, acc[i]);
        elem_t* dst = (elem_t*)a.out + (size_t)t * a.hidden + h;
        if constexpr (VEC > 1) {
            *(uint4*)dst = *(const uint4*)o;
        } else {
            dst[0] = o[0];
        }
    }
}

template <int DT> static const void* unpermute_fn(bool vec) {
    constexpr int V = DT == DT_F32 ? 4 : 8;
    return vec ? (const void*)moe_unpermute_kernel<DT, V> : (const void*)moe_unpermute_kernel<DT, 1>;
}

int launch_moe_unpermute(int dtype, const void* expert_outputs, const uint32_t* inv_perm, const void* weights, void* out,
                         uint32_t n_tokens, uint32_t n_permuted, uint32_t hidden, uint32_t k, const LaunchCtx& lc) {
    if (hidden == 0) return fail(ERR_SHAPE, "hidden must be non-zero");
    if (k == 0 || k > 32) return fail(ERR_SHAPE, "unpermute: k must be in 1..32");
    if (n_tokens == 0) return ERR_OK;
    if (!expert_outputs || !inv_perm || !weights || !out) return fail(ERR_BAD_ARG, "null buffer");
    UnpermuteArgs a{expert_outputs, inv_perm, weights, out, n_permuted, hidden, k};
    const uint32_t vec = dtype == DT_F32 ? 4 : 8;
    const bool wide = hidden % vec == 0 && (uintptr_t)expert_outputs % 16 == 0 && (uintptr_t)out % 16 == 0;
    const void* fn;
    switch (dtype) {
        case DT_F32: fn = unpermute_fn<DT_F32>(wide); break;
        case DT_F16: fn = unpermute_fn<DT_F16>(wide); break;
        case DT_BF16: fn = unpermute_fn<DT_BF16>(wide); break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3(n_tokens), dim3(256), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "unpermute kernel launch");
    return ERR_OK;
}

}  // namespace mtq
