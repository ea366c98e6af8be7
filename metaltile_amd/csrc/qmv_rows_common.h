// Device helpers shared by the GEMV kernels that feed the 4x4x4 matrix instruction straight from registers:
// lane 4 b + i of block b supplies row i of the first operand (four 16-bit values along the reduction), lane 4 b + j
// column j of the second, and lane 4 b + j receives column j of the block's 4 x 4 result in four registers (register i =
// row i).
#pragma once

#include <hip/hip_runtime.h>

#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

typedef uint32_t rp_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned rp_u32x2 __attribute__((ext_vector_type(2)));
typedef short rp_s16x4 __attribute__((ext_vector_type(4)));
typedef float rp_f32x4 __attribute__((ext_vector_type(4)));

#define RP_KEEP_ORDER() do { asm volatile("" ::: "memory"); __builtin_amdgcn_sched_barrier(0); } while (0)

typedef _Float16 rp_f16x4 __attribute__((ext_vector_type(4)));
template <int DT> __device__ __forceinline__ rp_f32x4 rp_mfma(rp_u32x2 a, rp_u32x2 b, rp_f32x4 c) {
    if constexpr (DT == DT_BF16) return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(rp_s16x4, a), __builtin_bit_cast(rp_s16x4, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(rp_f16x4, a), __builtin_bit_cast(rp_f16x4, b), c, 0, 0, 0);
}
// a 16-bit element (zero-extended) as f32
template <int DT> __device__ __forceinline__ float rp_up(uint32_t h) {
    if constexpr (DT == DT_BF16) return __uint_as_float(h << 16);
    else return f16_bits_to_f32(h);
}
// register (lane % 4) of a block's result: the lane's own product
__device__ __forceinline__ float rp_diag(rp_f32x4 v, bool b0, bool b1) {
    const float lo = b0 ? v.y : v.x, hi = b0 ? v.w : v.z;
    return b1 ? hi : lo;
}
__device__ __forceinline__ float rp_swap32_add(float a, float b) {
    rp_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}
__device__ __forceinline__ float rp_swap16_add(float a, float b) {
    rp_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}
// position class of pair i of a 2-bit weight dword and the shift that brings it there
template <int DT> __host__ __device__ constexpr int rp_crumb_class(int i) { return DT == DT_F16 ? (i < 5 ? i : i - 5) : i % 3; }
template <int DT> __host__ __device__ constexpr int rp_crumb_shift(int i) { return DT == DT_F16 ? (i < 5 ? 0 : 10) : 6 * (i / 3); }
// the OR-constant of class p: 2^(MB - 2 p) in both halves (f16: exponent bias 15, 10 mantissa bits; bf16: 127, 7)
template <int DT> __host__ __device__ constexpr uint32_t rp_crumb_kor(int p) {
    const uint32_t h = DT == DT_F16 ? (uint32_t)(15 + 10 - 2 * p) << 10 : (uint32_t)(127 + 7 - 2 * p) << 7;
    return h | (h << 16);
}

// Routed rows (GM = GATHER_CSR / GATHER_INDICES; a decode step of a few tokens through a mixture-of-experts layer, fewer
// rows than experts): grid row blockIdx.y serves the blockIdx.y-th expert that has a row and runs the kernel's body once
// per row of that expert -- one row each when a token's experts are distinct, as top-k routing makes them. The same
// rules as the streaming kernel's routed form (at most 64 experts and 64 rows: the routing is read by one wave-wide load).
struct RowsRoute {
    uint32_t expert = 0, n_pass = 1;
    unsigned long long mask = 1;   // the rows of x routed to the expert, one bit per row
};
template <int GM> __device__ __forceinline__ bool rows_route(const uint32_t* route, uint32_t E, uint32_t T, uint32_t lane, RowsRoute& r) {
    if constexpr (GM == GATHER_CSR) {
        uint32_t lo, n1, lo2;
        if (E <= 64u) {   // (one read of the offsets)
            if (csr_route64(route, E, T, blockIdx.y, true, lane, r.expert, lo, n1, lo2) == 0) return false;
        } else {          // (more experts than lanes: the offsets scanned 64 at a time, once for the slot's expert and once for its rows)
            r.expert = csr_slot_expert(route, E, T, blockIdx.y, lane);
            if (r.expert == 0xFFFFFFFFu) return false;
            if (csr_expert_rows(route, E, T, r.expert, lane, lo, n1, lo2) == 0) return false;
        }
        // (the same in every lane; said so, the pass loop and everything in it stay uniform control flow on scalar registers)
        r.expert = __builtin_amdgcn_readfirstlane(r.expert);
        lo = __builtin_amdgcn_readfirstlane(lo);
        n1 = __builtin_amdgcn_readfirstlane(n1);
        lo2 = __builtin_amdgcn_readfirstlane(lo2);
        // the expert's rows lo .. lo + n1 - 1 and, for expert 0, the rows past the last offset lo2 .. T - 1 (T <= 64), as a mask
        // like the one the per-row ids give, so that both views share the code behind this point
        const unsigned long long all = T >= 64u ? ~0ull : (1ull << T) - 1ull;
        unsigned long long m = n1 ? ((n1 >= 64u ? ~0ull : (1ull << n1) - 1ull) << lo) : 0ull;
        if (r.expert == 0u && lo2 < T) m |= (~0ull << lo2);
        r.mask = m & all;
        r.n_pass = (uint32_t)__popcll(r.mask);
        if (r.n_pass == 0) return false;
    }
    if constexpr (GM == GATHER_SINGLE) r.expert = min(route[0], E - 1u);   // one row on the expert named on the device; an id past the last expert names the last
    if constexpr (GM == GATHER_INDICES) {
        r.expert = __builtin_amdgcn_readfirstlane(ids_slot_expert(route, E, T, blockIdx.y, lane));
        if (r.expert == 0xFFFFFFFFu) return false;
        r.mask = __ballot(lane < T && route[lane] == r.expert);
        r.n_pass = (uint32_t)__popcll(r.mask);
    }
    return true;
}
// the activation (and output) row of a pass
template <int GM> __device__ __forceinline__ uint32_t rows_route_row(const RowsRoute& r, uint32_t pass) {
    if constexpr (GM == GATHER_CSR || GM == GATHER_INDICES) {
        unsigned long long m = r.mask;
        for (uint32_t i = 0; i < pass; i++) m &= m - 1ull;
        return (uint32_t)__ffsll((long long)m) - 1u;
    }
    return 0u;
}

}  // namespace mtq
