// Affine quantise / dequantise for gfx950: the writer and the reader of the
// packed weight format the matmul kernels consume.
//
// Replaces mt_affine_quantize_int{2,3,4,5,6,8} and mt_affine_dequantize_int{2,3,4,5,6,8}
// (crates/metaltile-std/src/mlx/quantized.rs:3575-3866, 3871-4230).
//
// Quantise, per group of `group_size` consecutive elements
// (quantized.rs:3642-3671): mn/mx = min/max of the group as f32,
// scale = (mx - mn) / (2^bits - 1), replaced by 1 when below 1e-7; bias = mn;
// code = trunc(clamp((v - bias) * (1 / scale) + 0.5, 0, 2^bits - 1)) formed with
// the f32 scale and bias; scale and bias are then stored rounded to the element
// dtype. Codes are integers and must not depend on instruction selection, so
// the subtract, multiply and add are issued as separately rounded operations
// (never contracted into an FMA) and the divisions are IEEE-correct.
// Dequantise: out = scale * code + bias, multiply and add rounded separately,
// then rounded to the element dtype (quantized.rs:3599-3604).
//
// Both are bandwidth kernels. A lane owns EPL consecutive elements: 8 for 4- and
// 8-bit codes, 16 for 2-bit, 32 for the widths whose codes straddle words (32
// codes of any width are a whole number of words). Its packed words and its
// elements are contiguous, so neighbouring lanes read and write neighbouring
// bytes; the G/EPL lanes of a group find the group's min and max with xor
// shuffles.
#include "mtq_device.h"
#include "mtq_internal.h"

// Every a*b+c in this file is two rounded operations, as in the reference's CPU
// loops (crates/metaltile-std/src/mlx/quantized.rs:5296-5303): a fused multiply-add can move a quantised value across a code
// boundary and changes the last bit of a dequantised one.
#pragma STDC FP_CONTRACT OFF

namespace mtq {

typedef uint32_t a_u32x4 __attribute__((ext_vector_type(4)));

struct AffineArgs {
    const void* in;     // quantise: T[n_elem]; dequantise: u32 words
    void* out;          // quantise: u32 words;  dequantise: T[n_elem]
    void* scales;       // T[n_elem / G]
    void* biases;
    uint64_t n_elem;
    uint32_t group_size;
    uint32_t lanes_per_group;  // G / EPL, a power of two
    uint32_t log2g;            // G is EPL * lanes_per_group: a power of two as well
    // Gathering dequantise (a quantized embedding table): output row t is table row row_ids[t]; rows of
    // lanes_per_row lanes; ids from n_rows on name no row and their output rows keep their bytes.
    const uint32_t* row_ids;
    uint32_t lanes_per_row;
    uint32_t n_rows;
};

template <int BITS> struct AffineGeom {
    static constexpr int EPL = (BITS == 4 || BITS == 8) ? 8 : (BITS == 2 ? 16 : 32);
    static constexpr int NW = EPL * BITS / 32;  // packed words per lane
};

// EPL consecutive elements -> f32
template <int DT, int EPL> __device__ __forceinline__ void load_elems(const void* p, uint64_t i0, float (&v)[EPL]) {
    if constexpr (DT == DT_F32) {
        const float4* s = (const float4*)((const float*)p + i0);
#pragma unroll
        for (int j = 0; j < EPL / 4; j++) {
            const float4 t = s[j];
            v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
        }
    } else {
        const a_u32x4* s = (const a_u32x4*)((const uint16_t*)p + i0);
#pragma unroll
        for (int j = 0; j < EPL / 8; j++) {
            const a_u32x4 t = s[j];
#pragma unroll
            for (int d = 0; d < 4; d++) {
                if constexpr (DT == DT_BF16) {
                    v[8 * j + 2 * d] = bf16_bits_to_f32(t[d] & 0xFFFFu);
                    v[8 * j + 2 * d + 1] = bf16_bits_to_f32(t[d] >> 16);
                } else {
                    v[8 * j + 2 * d] = f16_bits_to_f32(t[d] & 0xFFFFu);
                    v[8 * j + 2 * d + 1] = f16_bits_to_f32(t[d] >> 16);
                }
            }
        }
    }
}

template <int DT, int EPL> __device__ __forceinline__ void store_elems(void* p, uint64_t i0, const float (&v)[EPL]) {
    if constexpr (DT == DT_F32) {
        float4* d = (float4*)((float*)p + i0);
#pragma unroll
        for (int j = 0; j < EPL / 4; j++) d[j] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
    } else {
        a_u32x4* d = (a_u32x4*)((uint16_t*)p + i0);
#pragma unroll
        for (int j = 0; j < EPL / 8; j++) {
            a_u32x4 t;
#pragma unroll
            for (int k = 0; k < 4; k++)
                t[k] = (uint32_t)f32_to_elem_bits<DT>(v[8 * j + 2 * k]) | ((uint32_t)f32_to_elem_bits<DT>(v[8 * j + 2 * k + 1]) << 16);
            d[j] = t;
        }
    }
}

// Chunks per thread (a chunk = one lane's EPL elements): several independent 16-byte loads in
// flight per thread, issued before any of them is used. Chunk u of a thread is 256 lanes after
// chunk u - 1, so every load and store instruction still covers contiguous bytes.
template <int BITS> struct AffineUnroll {
    static constexpr int U = AffineGeom<BITS>::EPL == 8 ? 4 : (AffineGeom<BITS>::EPL == 16 ? 2 : 1);
};

template <int DT, int BITS>
__global__ __launch_bounds__(256) void affine_quantize_kernel(AffineArgs a) {
#pragma clang fp contract(off)
    constexpr int EPL = AffineGeom<BITS>::EPL, NW = AffineGeom<BITS>::NW, U = AffineUnroll<BITS>::U;
    const uint64_t n_lanes = a.n_elem / EPL;  // whole groups: n_elem is a multiple of G, G of EPL
    uint64_t t[U];
    bool live[U];
    float v[U][EPL];
#pragma unroll
    for (int u = 0; u < U; u++) {
        t[u] = ((uint64_t)blockIdx.x * U + u) * 256u + threadIdx.x;
        live[u] = t[u] < n_lanes;  // the lanes of a group are live or not together (256 is a multiple of their count)
        load_elems<DT, EPL>(a.in, (live[u] ? t[u] : n_lanes - 1) * EPL, v[u]);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        float mn = v[u][0], mx = v[u][0];
#pragma unroll
        for (int i = 1; i < EPL; i++) {
            mn = v[u][i] < mn ? v[u][i] : mn;
            mx = v[u][i] > mx ? v[u][i] : mx;
        }
        // the group's lanes are consecutive and aligned to their (power-of-two) count
        for (uint32_t d = 1; d < a.lanes_per_group; d <<= 1) {
            const float omn = __shfl_xor(mn, (int)d, 64), omx = __shfl_xor(mx, (int)d, 64);
            mn = omn < mn ? omn : mn;
            mx = omx > mx ? omx : mx;
        }
        constexpr float QMAX = (float)((1u << BITS) - 1u);
        float scale = (mx - mn) / QMAX;
        if (scale < 1.0e-7f) scale = 1.0f;
        const float inv = 1.0f / scale, bias = mn;
        uint32_t words[NW];
#pragma unroll
        for (int j = 0; j < NW; j++) words[j] = 0u;
#pragma unroll
        for (int i = 0; i < EPL; i++) {
            const float d = v[u][i] - bias;
            const float p = d * inv;
            float q = p + 0.5f;
            q = q < 0.0f ? 0.0f : q;
            q = q > QMAX ? QMAX : q;
            const uint32_t c = (uint32_t)q;
            const int pos = i * BITS, wi = pos / 32, sh = pos % 32;
            words[wi] |= c << sh;
            if (sh + BITS > 32) words[wi + 1] |= c >> (32 - sh);
        }
        if (!live[u]) continue;
        uint32_t* dst = (uint32_t*)a.out + t[u] * NW;
        if constexpr (NW == 1) {
            dst[0] = words[0];
        } else if constexpr (NW == 2) {
            *(uint2*)dst = make_uint2(words[0], words[1]);
        } else {
#pragma unroll
            for (int j = 0; j < NW; j++) dst[j] = words[j];
        }
        if ((t[u] & (a.lanes_per_group - 1)) == 0) {
            const uint64_t g = (t[u] * EPL) >> a.log2g;
            store_elem<DT>(a.scales, g, scale);
            store_elem<DT>(a.biases, g, bias);
        }
    }
}

// GATHER: crates/metaltile-std/src/ffai/dequant_gather.rs:45-93 (one thread per element there; a lane's run of
// elements here, the same bit stream and the same q * scale + bias).
template <int DT, int BITS, bool GATHER = false>
__global__ __launch_bounds__(256) void affine_dequantize_kernel(AffineArgs a) {
#pragma clang fp contract(off)
    constexpr int EPL = AffineGeom<BITS>::EPL, NW = AffineGeom<BITS>::NW, U = AffineUnroll<BITS>::U;
    const uint64_t n_lanes = a.n_elem / EPL;
    uint64_t t[U];
    bool live[U];
    uint32_t words[U][NW];
    float scale[U], bias[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        t[u] = ((uint64_t)blockIdx.x * U + u) * 256u + threadIdx.x;
        live[u] = t[u] < n_lanes;
        uint64_t tc = live[u] ? t[u] : n_lanes - 1;
        if constexpr (GATHER) {   // from the output lane to the lane of the table that holds its codes
            const uint32_t tc32 = (uint32_t)tc;   // (the host keeps the lane count below 2^32: a 64-bit quotient costs four times this one)
            const uint32_t row = tc32 / a.lanes_per_row;
            const uint32_t id = a.row_ids[row];
            live[u] = live[u] && id < a.n_rows;
            tc = (uint64_t)(id < a.n_rows ? id : 0u) * a.lanes_per_row + (tc32 - row * a.lanes_per_row);
        }
        const uint32_t* src = (const uint32_t*)a.in + tc * NW;
        if constexpr (NW == 2) {
            const uint2 w2 = *(const uint2*)src;
            words[u][0] = w2.x;
            words[u][1] = w2.y;
        } else {
#pragma unroll
            for (int j = 0; j < NW; j++) words[u][j] = src[j];
        }
        const uint64_t g = (tc * EPL) >> a.log2g;
        scale[u] = load_elem<DT>(a.scales, g);
        bias[u] = load_elem<DT>(a.biases, g);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (!live[u]) continue;
        float v[EPL];
#pragma unroll
        for (int i = 0; i < EPL; i++) {
            const int pos = i * BITS, wi = pos / 32, sh = pos % 32;
            uint32_t c = words[u][wi] >> sh;
            if (sh + BITS > 32) c |= words[u][wi + 1] << (32 - sh);
            c &= (1u << BITS) - 1u;
            const float p = scale[u] * (float)c;
            v[i] = p + bias[u];
        }
        store_elems<DT, EPL>(a.out, t[u] * EPL, v);
    }
}

template <int DT, int BITS> static int launch_one(bool quantize, AffineArgs& a, const LaunchCtx& lc) {
    constexpr int EPL = AffineGeom<BITS>::EPL;
    if (a.group_size % EPL) return fail(ERR_UNSUPPORTED, "affine: group_size must be a multiple of the lane's run (8, 16 or 32 elements)");
    a.lanes_per_group = a.group_size / EPL;
    if (a.lanes_per_group & (a.lanes_per_group - 1) || a.lanes_per_group > 64)
        return fail(ERR_UNSUPPORTED, "affine: group_size / run must be a power of two up to 64");
    a.log2g = 0;
    while ((1u << a.log2g) < a.group_size) a.log2g++;
    const uint64_t lanes = a.n_elem / EPL;
    const uint64_t per_block = 256ull * AffineUnroll<BITS>::U;
    const uint64_t blocks = (lanes + per_block - 1) / per_block;
    if (blocks == 0) return ERR_OK;
    if (blocks > 0x7FFFFFFFull) return fail(ERR_SHAPE, "affine: too many elements for one launch");
    const void* fn = quantize ? (const void*)affine_quantize_kernel<DT, BITS> : (const void*)affine_dequantize_kernel<DT, BITS>;
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3((uint32_t)blocks), dim3(256), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "affine kernel launch");
    return ERR_OK;
}

template <int DT> static int launch_bits(bool quantize, int bits, AffineArgs& a, const LaunchCtx& lc) {
    switch (bits) {
        case 2: return launch_one<DT, 2>(quantize, a, lc);
        case 3: return launch_one<DT, 3>(quantize, a, lc);
        case 4: return launch_one<DT, 4>(quantize, a, lc);
        case 5: return launch_one<DT, 5>(quantize, a, lc);
        case 6: return launch_one<DT, 6>(quantize, a, lc);
        case 7: return launch_one<DT, 7>(quantize, a, lc);
        default: return launch_one<DT, 8>(quantize, a, lc);
    }
}

template <int DT, int BITS> static int launch_gather_one(AffineArgs& a, uint32_t hidden, const LaunchCtx& lc) {
    constexpr int EPL = AffineGeom<BITS>::EPL;
    if (a.group_size % EPL || hidden % EPL) return fail(ERR_UNSUPPORTED, "dequant gather: group_size and hidden must be multiples of the lane's run (8, 16 or 32 elements)");
    a.lanes_per_group = a.group_size / EPL;
    if (a.lanes_per_group & (a.lanes_per_group - 1)) return fail(ERR_UNSUPPORTED, "dequant gather: group_size / run must be a power of two");
    a.log2g = 0;
    while ((1u << a.log2g) < a.group_size) a.log2g++;
    a.lanes_per_row = hidden / EPL;
    const uint64_t lanes = a.n_elem / EPL;
    const uint64_t per_block = 256ull * AffineUnroll<BITS>::U;
    const uint64_t blocks = (lanes + per_block - 1) / per_block;
    if (blocks > 0x7FFFFFFFull || lanes > 0xFFFFFFFFull) return fail(ERR_SHAPE, "dequant gather: too many elements for one launch");
    void* args[] = {&a};
    hipError_t e = launch_kernel((const void*)affine_dequantize_kernel<DT, BITS, true>, dim3((uint32_t)blocks), dim3(256), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "dequant gather kernel launch");
    return ERR_OK;
}

template <int DT> static int launch_gather_bits(int bits, AffineArgs& a, uint32_t hidden, const LaunchCtx& lc) {
    switch (bits) {
        case 2: return launch_gather_one<DT, 2>(a, hidden, lc);
        case 3: return launch_gather_one<DT, 3>(a, hidden, lc);
        case 4: return launch_gather_one<DT, 4>(a, hidden, lc);
        case 5: return launch_gather_one<DT, 5>(a, hidden, lc);
        case 6: return launch_gather_one<DT, 6>(a, hidden, lc);
        case 7: return launch_gather_one<DT, 7>(a, hidden, lc);
        default: return launch_gather_one<DT, 8>(a, hidden, lc);
    }
}

// out[t, :] = dequantised row ids[t] of a table [vocab, hidden] in the packed format (weight rows of hidden * bits / 32
// words, scales / biases rows of hidden / group_size).
int launch_dequant_gather(int dtype, int bits, uint32_t group_size, const void* weight, const void* scales, const void* biases,
                          const uint32_t* ids, void* out, uint32_t n_tokens, uint32_t hidden, uint32_t vocab, const LaunchCtx& lc) {
    if (bits < 2 || bits > 8) return fail(ERR_BAD_ARG, "bits must be in 2..8");
    if (hidden == 0 || vocab == 0) return fail(ERR_SHAPE, "hidden and vocab must be non-zero");
    if (group_size == 0 || hidden % group_size) return fail(ERR_SHAPE, "group_size must be non-zero and divide hidden");
    if ((uint64_t)hidden * bits % 32) return fail(ERR_SHAPE, "hidden*bits must be a multiple of 32");
    if (n_tokens == 0) return ERR_OK;
    if (!weight || !scales || !biases || !ids || !out) return fail(ERR_BAD_ARG, "null buffer");
    if ((uintptr_t)weight % 16 || (uintptr_t)out % 16) return fail(ERR_UNSUPPORTED, "dequant gather: buffers must be 16-byte aligned");
    AffineArgs a;
    a.in = weight;
    a.out = out;
    a.scales = const_cast<void*>(scales);
    a.biases = const_cast<void*>(biases);
    a.n_elem = (uint64_t)n_tokens * hidden;
    a.group_size = group_size;
    a.lanes_per_group = 1;
    a.row_ids = ids;
    a.n_rows = vocab;
    switch (dtype) {
        case DT_F32: return launch_gather_bits<DT_F32>(bits, a, hidden, lc);
        case DT_F16: return launch_gather_bits<DT_F16>(bits, a, hidden, lc);
        case DT_BF16: return launch_gather_bits<DT_BF16>(bits, a, hidden, lc);
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
}

int launch_affine(bool quantize, int dtype, int bits, uint32_t group_size, const void* in, void* out,
                  void* scales, void* biases, uint64_t n_elem, const LaunchCtx& lc) {
    if (bits < 2 || bits > 8) return fail(ERR_BAD_ARG, "bits must be in 2..8");
    if (group_size == 0 || n_elem % group_size) return fail(ERR_SHAPE, "n_elem must be a whole number of groups");
    if (n_elem == 0) return ERR_OK;
    if (!in || !out || !scales || !biases) return fail(ERR_BAD_ARG, "null buffer");
    if ((uintptr_t)in % 16 || (uintptr_t)out % 16) return fail(ERR_UNSUPPORTED, "affine: buffers must be 16-byte aligned");
    AffineArgs a;
    a.in = in;
    a.out = out;
    a.scales = scales;
    a.biases = biases;
    a.n_elem = n_elem;
    a.group_size = group_size;
    a.lanes_per_group = 1;
    a.row_ids = nullptr;
    a.lanes_per_row = 0;
    a.n_rows = 0;
    switch (dtype) {
        case DT_F32: return launch_bits<DT_F32>(quantize, bits, a, lc);
        case DT_F16: return launch_bits<DT_F16>(quantize, bits, a, lc);
        case DT_BF16: return launch_bits<DT_BF16>(quantize, bits, a, lc);
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
}

}  // namespace mtq
