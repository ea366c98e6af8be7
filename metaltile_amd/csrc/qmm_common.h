// Pieces shared by the two matrix-core qmm kernels (qmm.hip, qmm_direct.hip):
// the 32x32x16 MFMA wrapper, round-to-nearest-even packing and the conversion
// of eight packed codes into eight elements s*q + b rounded to the element
// dtype (the reference's mma semantics,
// crates/metaltile-std/src/mlx/quantized.rs:2267-2274).
#pragma once
#include "mtq_device.h"

namespace mtq {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t q_u32x4 __attribute__((ext_vector_type(4)));

template <int DT> __device__ __forceinline__ f32x16 mfma32(uint4 a, uint4 b, f32x16 c) {
    if constexpr (DT == DT_BF16) {
        bf16x8_t av, bv;
        __builtin_memcpy(&av, &a, 16);
        __builtin_memcpy(&bv, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, c, 0, 0, 0);
    } else {
        f16x8_t av, bv;
        __builtin_memcpy(&av, &a, 16);
        __builtin_memcpy(&bv, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, c, 0, 0, 0);
    }
}

// two f32 -> two elements packed in one dword, round to nearest even
template <int DT> __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    uint32_t u;
    if constexpr (DT == DT_BF16) {
        typedef __attribute__((ext_vector_type(2))) __bf16 v2;
        v2 p;
        p.x = (__bf16)lo;
        p.y = (__bf16)hi;
        __builtin_memcpy(&u, &p, 4);
    } else {
        typedef __attribute__((ext_vector_type(2))) _Float16 v2;
        v2 p;
        p.x = (_Float16)lo;
        p.y = (_Float16)hi;
        __builtin_memcpy(&u, &p, 4);
    }
    return u;
}

template <int DT> __device__ __forceinline__ float elem_bits_to_f32(uint32_t h) {
    return DT == DT_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}

// 8 consecutive codes starting at code index 8*i of the thread's run -> 8
// elements s*q+b rounded to DT, packed in one 16-byte vector.
template <int DT, int BITS>
__device__ __forceinline__ uint4 dequant8(const uint32_t* wr, int i, float s, float b) {
    float v[8];
    if constexpr (BITS == 4) {
        const uint32_t w = wr[i];
        // Even codes sit in the low nibbles of the four bytes, odd codes in the high nibbles. The high
        // nibbles are converted where they are (as 16 * q) and multiplied by s / 16, which is exact, so
        // no shift is needed. The masked copies are opaque to the optimiser: it would otherwise fold the
        // masks into one bit-field extract per code and then convert byte 0; kept as they are, the
        // byte-select converts (v_cvt_f32_ubyte0..3) take the codes straight out of `e` and `o`.
        uint32_t e = w & 0x0F0F0F0Fu, o = w & 0xF0F0F0F0u;
        asm volatile("" : "+v"(e), "+v"(o));
        const float s16 = s * 0.0625f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[2 * j] = fmaf((float)((e >> (8 * j)) & 0xFFu), s, b);
            v[2 * j + 1] = fmaf((float)((o >> (8 * j)) & 0xFFu), s16, b);
        }
    } else if constexpr (BITS == 8) {
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int j = 0; j < 4; j++) v[4 * d + j] = fmaf((float)((wr[2 * i + d] >> (8 * j)) & 0xFFu), s, b);
    } else if constexpr (BITS == 2) {  // 16 codes per dword, this call takes half of dword i/2
        const uint32_t w = wr[i / 2] >> (16 * (i & 1));
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = fmaf((float)((w >> (2 * j)) & 3u), s, b);
    } else {  // bit-stream widths: code c of the run sits at bit c * BITS of the BITS words, LSB first
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int o = (8 * i + j) * BITS, lo = o >> 5, sh = o & 31;
            uint32_t q = wr[lo] >> sh;
            if (sh + BITS > 32) q |= wr[lo + 1] << (32 - sh);
            v[j] = fmaf((float)(q & ((1u << BITS) - 1u)), s, b);
        }
    }
    return make_uint4(pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3]), pack2<DT>(v[4], v[5]), pack2<DT>(v[6], v[7]));
}

}  // namespace mtq
