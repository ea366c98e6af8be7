// Device-side building blocks shared by the affine-quantized kernels (gfx950).
//
// Packed-weight format (reference: crates/metaltile-std/src/mlx/quantized.rs:5393-5396):
// codes q in [0, 2^bits) packed LSB-first into little-endian u32 words,
// row-major [N, K*bits/32]; dequantised weight = scale_g * q + bias_g with
// g = k / group_size; every load is widened to f32 and all sums are f32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mtq_types.h"

namespace mtq {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;

template <int DT> struct Elem;
template <> struct Elem<DT_F32> { typedef float type; };
template <> struct Elem<DT_F16> { typedef uint16_t type; };
template <> struct Elem<DT_BF16> { typedef uint16_t type; };

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    uint16_t u = (uint16_t)h;
    _Float16 f;
    __builtin_memcpy(&f, &u, 2);
    return (float)f;
}

template <int DT> __device__ __forceinline__ float load_elem(const void* p, size_t i) {
    if constexpr (DT == DT_F32) return ((const float*)p)[i];
    else if constexpr (DT == DT_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
    else return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}

// f32 -> element store, round to nearest even (the reference's `.cast::<T>()`
// on store, crates/metaltile-std/src/mlx/quantized.rs:303-306).
template <int DT> __device__ __forceinline__ void store_elem(void* p, size_t i, float v) {
    if constexpr (DT == DT_F32) {
        ((float*)p)[i] = v;
    } else if constexpr (DT == DT_F16) {
        _Float16 h = (_Float16)v;
        uint16_t u;
        __builtin_memcpy(&u, &h, 2);
        ((uint16_t*)p)[i] = u;
    } else {
        __bf16 h = (__bf16)v;
        uint16_t u;
        __builtin_memcpy(&u, &h, 2);
        ((uint16_t*)p)[i] = u;
    }
}

template <int DT> __device__ __forceinline__ uint16_t f32_to_elem_bits(float v) {
    uint16_t u;
    if constexpr (DT == DT_F16) {
        _Float16 h = (_Float16)v;
        __builtin_memcpy(&u, &h, 2);
    } else {
        __bf16 h = (__bf16)v;
        __builtin_memcpy(&u, &h, 2);
    }
    return u;
}

// An f32 value carried as two 16-bit operands: `hi`, the element-type value nearest to it, and `lo`, the rounded
// remainder times kRemScale, so that hi + lo / kRemScale holds 16 significant bits of v (the f16 remainder is scaled by
// 2^11: it then has the magnitude of v and stays a normal number with all its bits where v is small).
// The value, and each half once converted, pass through an empty asm: every later use must see the same bits. The
// optimiser otherwise materialises f16(a * b) more than once, with different roundings - contracted into a
// mixed-precision FMA (one rounding of the exact product) for one use, converted from the rounded f32 product (two
// roundings) for another. The two differ by one f16 ulp when the f32 product lands on an f16 tie, about once in 8192
// values; when the dot operand and the f32 sum of the same row (the bias term of the split dot) got different copies,
// the output was off by 1024 x scale x ulp, the same sign in every output row: 0.11 on the parity metric for one data
// set in three of the gated norm, nothing for the others.
template <int DT> struct RemSplit {
    static constexpr float kRemScale = DT == DT_F16 ? 2048.0f : 1.0f;
    static __device__ __forceinline__ float up(uint32_t b) { return DT == DT_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b); }
    static __device__ __forceinline__ void split(float v, uint32_t& hi, uint32_t& lo) {
        asm volatile("" : "+v"(v));
        hi = f32_to_elem_bits<DT>(v);
        asm volatile("" : "+v"(hi));
        lo = f32_to_elem_bits<DT>((v - up(hi)) * kRemScale);
        asm volatile("" : "+v"(lo));
    }
};

// One 16-byte vector of activations (4 f32 or 8 16-bit elements): sum of squares, and
// in-place (x * w) * inv rounded to the element type.
template <int DT> __device__ __forceinline__ float raw_sumsq(uint4 v) {
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if constexpr (DT == DT_F32) {
            const float f = __uint_as_float(u[j]);
            s += f * f;
        } else {
            const float lo = DT == DT_BF16 ? bf16_bits_to_f32(u[j] & 0xFFFFu) : f16_bits_to_f32(u[j] & 0xFFFFu);
            const float hi = DT == DT_BF16 ? bf16_bits_to_f32(u[j] >> 16) : f16_bits_to_f32(u[j] >> 16);
            s += lo * lo;
            s += hi * hi;
        }
    }
    return s;
}
// (x * w) * inv of one vector, as the element-type value `hi` nearest to it and (16-bit
// types) the rounded, scaled remainder `lo` (RemSplit): hi + lo / kRemScale carries 16 significant bits of the f32 product.
template <int DT> __device__ __forceinline__ void raw_normed(uint4 xv, uint4 wv, float inv, uint4& hi, uint4& lo) {
    const uint32_t x[4] = {xv.x, xv.y, xv.z, xv.w};
    const uint32_t w[4] = {wv.x, wv.y, wv.z, wv.w};
    uint32_t h[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if constexpr (DT == DT_F32) {
            h[j] = __float_as_uint(__uint_as_float(x[j]) * __uint_as_float(w[j]) * inv);
            l[j] = 0;
        } else {
            auto up = [](uint32_t b) { return DT == DT_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b); };
            const float v0 = up(x[j] & 0xFFFFu) * up(w[j] & 0xFFFFu) * inv;
            const float v1 = up(x[j] >> 16) * up(w[j] >> 16) * inv;
            uint32_t h0, h1, l0, l1;
            RemSplit<DT>::split(v0, h0, l0);
            RemSplit<DT>::split(v1, h1, l1);
            h[j] = h0 | (h1 << 16);
            l[j] = l0 | (l1 << 16);
        }
    }
    hi = make_uint4(h[0], h[1], h[2], h[3]);
    lo = make_uint4(l[0], l[1], l[2], l[3]);
}

// ---- cross-lane sums -------------------------------------------------------

template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over aligned segments of `seg` lanes (seg a power of two, 1..64); every
// lane of a segment ends up holding the segment's sum. Lanes exchange with
// their xor-partners, so the summation order is fixed by the lane layout.
__device__ __forceinline__ float seg_allreduce(float v, int seg) {
    if (seg >= 2) v += dpp_f32<0xB1>(v);    // quad_perm [1,0,3,2]
    if (seg >= 4) v += dpp_f32<0x4E>(v);    // quad_perm [2,3,0,1]
    if (seg >= 8) v += dpp_f32<0x141>(v);   // row_half_mirror
    if (seg >= 16) v += dpp_f32<0x140>(v);  // row_mirror
    if (seg >= 32) v += __shfl_xor(v, 16, 64);
    if (seg >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// ---- x-slice holders and the per-chunk dot ---------------------------------
//
// A "chunk" is 16 bytes of packed weights (one dwordx4 load): CPC = 128/bits
// codes. A thread owns one chunk position of the row and keeps the matching
// CPC activations in registers for every row it visits.
//
// Two arithmetic paths:
//  * dot2 path (f16/bf16 activations, 2- and 4-bit codes): a masked pair of
//    codes OR-ed into the mantissa of 2^7 (bf16) or 2^10 (f16; 4-bit codes: into
//    mantissa bits 4-7 of 2^6, where the dword's second nibble already is, so the
//    f32 sums carry a sixteenth of the offset for the same instructions) is the pair
//    (MAGIC+q_a, MAGIC+q_b) in element format; v_dot2_f32_{bf16,f16} multiplies
//    it with the matching activation pair and accumulates in f32. The MAGIC
//    offset is folded into the bias: s*(dot - MAGIC*sum_x) + b*sum_x =
//    s*dot + (b - MAGIC*s)*sum_x.
//  * cvt path (f32 activations, or 8-bit codes): byte -> f32 convert and an f32
//    FMA per code.

template <int DT, int BITS> struct PathSel {
    static constexpr bool kDot2 = (DT != DT_F32) && (BITS == 2 || BITS == 4);
    static constexpr float kMagic = kDot2 ? (DT == DT_BF16 ? 128.0f : BITS == 4 ? 64.0f : 1024.0f) : 0.0f;
};

template <int DT> __device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float acc) {
    if constexpr (DT == DT_BF16) {
        bf16x2_t av, bv;
        __builtin_memcpy(&av, &a, 4);
        __builtin_memcpy(&bv, &b, 4);
        return __builtin_amdgcn_fdot2_f32_bf16(av, bv, acc, false);
    } else {
        half2_t av, bv;
        __builtin_memcpy(&av, &a, 4);
        __builtin_memcpy(&bv, &b, 4);
        return __builtin_amdgcn_fdot2(av, bv, acc, false);
    }
}

// MAGIC pair (2^7 twice in bf16, 2^10 twice in f16; SIXTY_FOUR: 2^6 twice in f16, for codes in mantissa bits 4-7) as an
// opaque VGPR value.
template <int DT, bool SIXTY_FOUR = false> __device__ __forceinline__ uint32_t magic_or_vgpr() {
    uint32_t k = DT == DT_BF16 ? 0x43004300u : SIXTY_FOUR ? 0x54005400u : 0x64006400u;
    asm volatile("" : "+v"(k));
    return k;
}

template <int DT, int BITS, bool DOT2 = PathSel<DT, BITS>::kDot2> struct XSlice;

// dot2 path: activations kept as 16-bit pairs arranged to match the code pairs
// a single mask extracts from one weight dword.
template <int DT, int BITS> struct XSlice<DT, BITS, true> {
    static constexpr int CPC = 128 / BITS;   // codes per 16-byte chunk
    static constexpr int CPD = 32 / BITS;    // codes per dword
    uint32_t xp[CPC / 2];
    float xsum[2];  // sum of the activations of dwords {0,1} and {2,3}
    uint32_t kor;   // MAGIC pair, held in a VGPR (set by prepare / zero)

    static constexpr int NRAW = CPC / 8;  // 16-byte vectors of activations per chunk
    // The chunk's CPC activations start at element `i0` of `x` (16-byte aligned).
    // load_raw only issues the loads; prepare() does the register shuffling, so a
    // caller can put other loads between the two.
    __device__ __forceinline__ void load_raw(const void* x, size_t i0, uint4 (&raw)[NRAW]) const {
        const uint4* xv = (const uint4*)((const uint16_t*)x + i0);
#pragma unroll
        for (int i = 0; i < NRAW; i++) raw[i] = xv[i];
    }
    __device__ __forceinline__ void prepare(const uint4 (&raw)[NRAW]) {
        kor = magic_or_vgpr<DT, BITS == 4>();
        float s01 = 0.f, s23 = 0.f;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int d = 0; d < 4; d++) {  // dword d of the chunk <-> 8 activations
                uint4 v = raw[d];
                xp[4 * d + 0] = (v.x & 0xFFFFu) | (v.z << 16);          // (x0,x4)
                xp[4 * d + 1] = (v.x >> 16) | (v.z & 0xFFFF0000u);      // (x1,x5)
                xp[4 * d + 2] = (v.y & 0xFFFFu) | (v.w << 16);          // (x2,x6)
                xp[4 * d + 3] = (v.y >> 16) | (v.w & 0xFFFF0000u);      // (x3,x7)
                float s = sum8(v);
                if (d < 2) s01 += s; else s23 += s;
            }
        } else {  // BITS == 2: dword d <-> 16 activations, pairs (x_i, x_{i+8})
#pragma unroll
            for (int d = 0; d < 4; d++) {
                uint4 a = raw[2 * d], b = raw[2 * d + 1];
                xp[8 * d + 0] = (a.x & 0xFFFFu) | (b.x << 16);
                xp[8 * d + 1] = (a.x >> 16) | (b.x & 0xFFFF0000u);
                xp[8 * d + 2] = (a.y & 0xFFFFu) | (b.y << 16);
                xp[8 * d + 3] = (a.y >> 16) | (b.y & 0xFFFF0000u);
                xp[8 * d + 4] = (a.z & 0xFFFFu) | (b.z << 16);
                xp[8 * d + 5] = (a.z >> 16) | (b.z & 0xFFFF0000u);
                xp[8 * d + 6] = (a.w & 0xFFFFu) | (b.w << 16);
                xp[8 * d + 7] = (a.w >> 16) | (b.w & 0xFFFF0000u);
                float s = sum8(a) + sum8(b);
                if (d < 2) s01 += s; else s23 += s;
            }
        }
        xsum[0] = s01;
        xsum[1] = s23;
    }
    __device__ __forceinline__ void load(const void* x, size_t i0) {
        uint4 raw[NRAW];
        load_raw(x, i0, raw);
        prepare(raw);
    }
    __device__ __forceinline__ void zero() {
        kor = magic_or_vgpr<DT, BITS == 4>();
#pragma unroll
        for (int i = 0; i < CPC / 2; i++) xp[i] = 0;
        xsum[0] = xsum[1] = 0.f;
    }
    static __device__ __forceinline__ float cvt(uint32_t h) {
        return DT == DT_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
    }
    static __device__ __forceinline__ float sum8(uint4 v) {
        float s = cvt(v.x & 0xFFFFu) + cvt(v.x >> 16);
        s += cvt(v.y & 0xFFFFu) + cvt(v.y >> 16);
        s += cvt(v.z & 0xFFFFu) + cvt(v.z >> 16);
        s += cvt(v.w & 0xFFFFu) + cvt(v.w >> 16);
        return s;
    }
    // sum over the codes of dword d of (MAGIC + q) * x
    __device__ __forceinline__ float dot_dword(uint32_t w, int d, float acc) const {
        // The OR constant lives in a VGPR the optimiser cannot see through: with
        // the mask as the one scalar/literal operand, (w & mask) | k then fits a
        // single v_and_or_b32 (two literal constants would not).
        const uint32_t kOr = kor;
        if constexpr (BITS == 4 && DT == DT_BF16) {
            acc = dot2_acc<DT>((w & 0x000F000Fu) | kOr, xp[4 * d + 0], acc);
            acc = dot2_acc<DT>(((w >> 4) & 0x000F000Fu) | kOr, xp[4 * d + 1], acc);
            acc = dot2_acc<DT>(((w >> 8) & 0x000F000Fu) | kOr, xp[4 * d + 2], acc);
            acc = dot2_acc<DT>(((w >> 12) & 0x000F000Fu) | kOr, xp[4 * d + 3], acc);
        } else if constexpr (BITS == 4) {   // f16: the codes into mantissa bits 4-7
            acc = dot2_acc<DT>(((w << 4) & 0x00F000F0u) | kOr, xp[4 * d + 0], acc);
            acc = dot2_acc<DT>((w & 0x00F000F0u) | kOr, xp[4 * d + 1], acc);
            acc = dot2_acc<DT>(((w >> 4) & 0x00F000F0u) | kOr, xp[4 * d + 2], acc);
            acc = dot2_acc<DT>(((w >> 8) & 0x00F000F0u) | kOr, xp[4 * d + 3], acc);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++)
                acc = dot2_acc<DT>(((w >> (2 * i)) & 0x00030003u) | kOr, xp[8 * d + i], acc);
        }
        return acc;
    }
};

// cvt path: activations kept as f32.
template <int DT, int BITS> struct XSlice<DT, BITS, false> {
    static constexpr int CPC = 128 / BITS;
    static constexpr int CPD = 32 / BITS;
    float xf[CPC];
    float xsum[2];

    // raw activations: 16-byte vectors of element storage
    static constexpr int NRAW = DT == DT_F32 ? CPC / 4 : CPC / 8;
    __device__ __forceinline__ void load_raw(const void* x, size_t i0, uint4 (&raw)[NRAW]) const {
        const uint4* xv = DT == DT_F32 ? (const uint4*)((const float*)x + i0)
                                       : (const uint4*)((const uint16_t*)x + i0);
#pragma unroll
        for (int i = 0; i < NRAW; i++) raw[i] = xv[i];
    }
    __device__ __forceinline__ void prepare(const uint4 (&raw)[NRAW]) {
#pragma unroll
        for (int i = 0; i < NRAW; i++) {
            const uint32_t u[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (DT == DT_F32) {
                    xf[4 * i + j] = __uint_as_float(u[j]);
                } else if constexpr (DT == DT_F16) {
                    xf[8 * i + 2 * j] = f16_bits_to_f32(u[j] & 0xFFFFu);
                    xf[8 * i + 2 * j + 1] = f16_bits_to_f32(u[j] >> 16);
                } else {
                    xf[8 * i + 2 * j] = bf16_bits_to_f32(u[j] & 0xFFFFu);
                    xf[8 * i + 2 * j + 1] = bf16_bits_to_f32(u[j] >> 16);
                }
            }
        }
        float s01 = 0.f, s23 = 0.f;
#pragma unroll
        for (int i = 0; i < CPC; i++) {
            if (i < CPC / 2) s01 += xf[i]; else s23 += xf[i];
        }
        xsum[0] = s01;
        xsum[1] = s23;
    }
    __device__ __forceinline__ void load(const void* x, size_t i0) {
        uint4 raw[NRAW];
        load_raw(x, i0, raw);
        prepare(raw);
    }
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < CPC; i++) xf[i] = 0.f;
        xsum[0] = xsum[1] = 0.f;
    }
    __device__ __forceinline__ float dot_dword(uint32_t w, int d, float acc) const {
        const float* x = xf + d * CPD;
        if constexpr (BITS == 8) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc = fmaf((float)((w >> (8 * j)) & 0xFFu), x[j], acc);
        } else if constexpr (BITS == 4) {
            uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc = fmaf((float)((lo >> (8 * j)) & 0xFFu), x[2 * j], acc);
                acc = fmaf((float)((hi >> (8 * j)) & 0xFFu), x[2 * j + 1], acc);
            }
        } else {  // BITS == 2: byte j of (w >> 2s) & 0x03030303 is code 4j+s
#pragma unroll
            for (int s = 0; s < 4; s++) {
                uint32_t m = (w >> (2 * s)) & 0x03030303u;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc = fmaf((float)((m >> (8 * j)) & 0xFFu), x[4 * j + s], acc);
            }
        }
        return acc;
    }
};

// Rows of one expert under the reference's CSR rule (crates/metaltile-std/src/ffai/moe.rs:376-385):
// row t belongs to the first expert e with t < off[e + 1], rows past every offset to expert 0. So
// expert e owns [max(off[1..e]), min(off[e + 1], T)) and expert 0 also the tail [max(off), T).
// Called by whole waves with a uniform expert; each wave scans the offsets 64 at a time. An expert
// whose own offsets already leave it empty returns before the scan: with many experts and few rows
// most workgroups are such, and a per-workgroup scan of every offset was the whole cost of the launch
// (256 experts, 8 rows: 408 us, against 27 us for the same routing as per-row ids).
__device__ __forceinline__ uint32_t csr_expert_rows(const uint32_t* off, uint32_t E, uint32_t T, uint32_t expert, uint32_t lane,
                                                    uint32_t& lo, uint32_t& n1, uint32_t& lo2) {
    const uint32_t o_hi = off[expert + 1];
    lo = n1 = lo2 = 0;
    if (expert != 0 && o_hi <= off[expert]) return 0;  // hi <= off[e] <= max(off[1..e]): no row
    uint32_t l = 0, mx = 0;
    for (uint32_t j0 = 1; j0 <= E; j0 += 64) {
        const uint32_t j = j0 + lane;
        const uint32_t o = j <= E ? off[j] : 0u;
        if (j <= expert) l = max(l, o);
        mx = max(mx, o);
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        l = max(l, (uint32_t)__shfl_xor((int)l, d, 64));
        mx = max(mx, (uint32_t)__shfl_xor((int)mx, d, 64));
    }
    const uint32_t hi = min(o_hi, T);
    lo = l;
    n1 = hi > lo ? hi - lo : 0;
    lo2 = min(mx, T);
    const uint32_t n2 = expert == 0 ? T - lo2 : 0;
    return n1 + n2;
}

// Gathers with fewer rows than experts launch one grid row per activation row instead of one per expert (most
// experts are not hit, and a workgroup that only finds that out holds its compute unit's LDS and wave slots while its
// loads of the routing come back: 8 experts of 14336 x 4096 with one row took 17 us, the same bytes as one matrix 8).
// Grid row `slot` serves the slot-th expert, in ascending order, that has a row; 0xFFFFFFFF if there are fewer.
// The same in every lane. CSR view, the reference's rule E(t) = first e with t < off[e + 1], else 0
// (crates/metaltile-std/src/ffai/moe.rs:376-385): expert e has rows iff min(off[e + 1], T) > min(max(off[1 .. e]), T),
// and expert 0 also takes the rows past every offset.
__device__ __forceinline__ uint32_t csr_slot_expert(const uint32_t* off, uint32_t E, uint32_t T, uint32_t slot, uint32_t lane) {
    uint32_t mx = 0;
    for (uint32_t j0 = 1; j0 <= E; j0 += 64) mx = max(mx, j0 + lane <= E ? off[j0 + lane] : 0u);
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, d, 64));
    const bool tail = min(mx, T) < T;
    uint32_t seen = 0, carry = 0;   // carry: max(off[1 .. e0])
    for (uint32_t e0 = 0; e0 < E; e0 += 64) {
        const uint32_t e = e0 + lane;
        const uint32_t o_hi = e < E ? off[e + 1] : 0u;
        uint32_t incl = o_hi;   // inclusive prefix maximum over the lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, d, 64);
            if (lane >= (uint32_t)d) incl = max(incl, up);
        }
        uint32_t before = (uint32_t)__shfl_up((int)incl, 1, 64);
        before = max(lane ? before : 0u, carry);
        const bool hit = e < E && (min(o_hi, T) > min(before, T) || (e == 0 && tail));
        unsigned long long m = __ballot(hit);
        const uint32_t c = (uint32_t)__popcll(m);
        if (slot < seen + c) {
            for (uint32_t i = seen; i < slot; i++) m &= m - 1ull;
            return e0 + (uint32_t)__ffsll((long long)m) - 1u;
        }
        seen += c;
        carry = max(carry, (uint32_t)__shfl((int)incl, 63, 64));
    }
    return 0xFFFFFFFFu;
}
// Both of the above from one read of the offsets, for at most 64 experts (lane e holds off[e + 1]; everything else is
// exchanged between lanes): which expert this grid row serves (`sel` is the expert, or with by_slot the slot) and its
// rows. Returns the expert's row count and sets expert (0xFFFFFFFF: a slot past the experts that have rows), lo, n1,
// lo2 as csr_expert_rows does. One trip to memory instead of three or four ahead of the first activation load.
__device__ __forceinline__ uint32_t csr_route64(const uint32_t* off, uint32_t E, uint32_t T, uint32_t sel, bool by_slot, uint32_t lane,
                                                uint32_t& expert, uint32_t& lo, uint32_t& n1, uint32_t& lo2) {
    const uint32_t o_hi = lane < E ? off[lane + 1] : 0u;
    uint32_t incl = o_hi;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, d, 64);
        if (lane >= (uint32_t)d) incl = max(incl, up);
    }
    uint32_t before = (uint32_t)__shfl_up((int)incl, 1, 64);   // max(off[1 .. e])
    if (lane == 0) before = 0;
    const uint32_t mx = (uint32_t)__shfl((int)incl, 63, 64);
    lo = n1 = lo2 = 0;
    expert = sel;
    if (by_slot) {
        const bool hit = lane < E && (min(o_hi, T) > min(before, T) || (lane == 0 && min(mx, T) < T));
        unsigned long long m = __ballot(hit);
        if (sel >= (uint32_t)__popcll(m)) { expert = 0xFFFFFFFFu; return 0; }
        for (uint32_t i = 0; i < sel; i++) m &= m - 1ull;
        expert = (uint32_t)__ffsll((long long)m) - 1u;
    }
    const uint32_t l = (uint32_t)__shfl((int)before, (int)expert, 64), oh = (uint32_t)__shfl((int)o_hi, (int)expert, 64);
    const uint32_t hi = min(oh, T);
    lo = l;
    n1 = hi > lo ? hi - lo : 0;
    lo2 = min(mx, T);
    return n1 + (expert == 0 ? T - lo2 : 0u);
}
// Per-row ids (at most 64 rows): the slot-th smallest id below E that a row names.
__device__ __forceinline__ uint32_t ids_slot_expert(const uint32_t* ids, uint32_t E, uint32_t T, uint32_t slot, uint32_t lane) {
    uint32_t v = lane < T ? ids[lane] : 0xFFFFFFFFu;
    if (v >= E) v = 0xFFFFFFFFu;
    uint32_t cur = 0xFFFFFFFFu;
    for (uint32_t i = 0; i <= slot; i++) {
        uint32_t c = (i == 0 || v > cur) ? v : 0xFFFFFFFFu;   // ids above the last one found
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) c = min(c, (uint32_t)__shfl_xor((int)c, d, 64));
        if (c == 0xFFFFFFFFu) return c;
        cur = c;
    }
    return cur;
}

}  // namespace mtq
