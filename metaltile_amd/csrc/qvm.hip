// Vector-matrix product against a transposed packed weight (reference: mt_qvm_b{3,4,5,6,8} and
// mt_qvm_int4_fast, crates/metaltile-std/src/mlx/quantized.rs:4397-4522, 4582-4700):
// out[m, c] = sum_d w_hat[d, c] * x[m, d], W [K, N] packed along N, scales / biases [K/G, N].
//
// The packed axis is the output axis, so a thread owns the columns of one weight dword (or one
// column for the bit-stream widths) and walks down K. K is split twice: over the 16 K-lanes of a
// workgroup (added through LDS) and over workgroups, each of which writes an f32 partial row that
// a second small kernel adds in a fixed order (no atomics: the result does not depend on
// scheduling).
#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

struct QvmArgs {
    const uint32_t* w;
    const void* scales;
    const void* biases;
    const void* x;
    float* part;   // [M][ks][N]
    void* out;     // [M][N]
    uint32_t M, N, K, G, wpr, rows_per_slice, ks;
};

// 1024 threads = 64 column slots x 16 K-lanes. K-lane ty takes rows d0 + ty, d0 + ty + 16, ... of
// the workgroup's K slice (at each step the workgroup reads 16 consecutive rows), the 16 lanes
// of a column slot are added through LDS in lane order, and the slice's partial row goes to
// global memory.
template <int DT, int BITS> __global__ __launch_bounds__(1024) void qvm_partial_kernel(QvmArgs a) {
    constexpr bool kPow2 = 32 % BITS == 0;
    constexpr int CPT = kPow2 ? 32 / BITS : 1;   // columns per thread
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    __shared__ float red[16][64 * CPT + 1];
    const uint32_t tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;
    const uint32_t tcol = blockIdx.x * 64 + tx;
    const uint32_t c0 = tcol * CPT;
    const bool live = c0 < a.N;
    const uint32_t slice = blockIdx.y, m = blockIdx.z;
    const uint32_t d0 = slice * a.rows_per_slice;
    const uint32_t d1 = min(a.K, d0 + a.rows_per_slice);
    const uint32_t bit_off = c0 * BITS, wi = kPow2 ? tcol : bit_off >> 5, sh = bit_off & 31u;
    float acc[CPT];
#pragma unroll
    for (int j = 0; j < CPT; j++) acc[j] = 0.f;
    if (live) {
        // groups the slice touches; inside a group this lane's rows are those congruent to d0 + ty mod 16
        for (uint32_t gs = d0; gs < d1; gs = (gs / a.G + 1) * a.G) {
            const uint32_t ge = min((gs / a.G + 1) * a.G, d1);
            uint32_t d = gs + ((d0 + ty + 16u - (gs & 15u)) & 15u);   // first row >= gs of this lane
            if (d >= ge) continue;
            float qdot[CPT];
#pragma unroll
            for (int j = 0; j < CPT; j++) qdot[j] = 0.f;
            float xs = 0.f;
            for (; d < ge; d += 16) {
                const float xv = load_elem<DT>(a.x, (size_t)m * a.K + d);
                const uint32_t* row = a.w + (size_t)d * a.wpr;
                if constexpr (kPow2) {
                    const uint32_t word = row[wi];
#pragma unroll
                    for (int j = 0; j < CPT; j++) qdot[j] = fmaf((float)((word >> (j * BITS)) & MASK), xv, qdot[j]);
                } else {
                    uint32_t q = row[wi] >> sh;
                    if (sh + BITS > 32) q |= row[wi + 1] << (32 - sh);
                    qdot[0] = fmaf((float)(q & MASK), xv, qdot[0]);
                }
                xs += xv;
            }
            const size_t sb = (size_t)(gs / a.G) * a.N + c0;
#pragma unroll
            for (int j = 0; j < CPT; j++)
                acc[j] += load_elem<DT>(a.scales, sb + j) * qdot[j] + load_elem<DT>(a.biases, sb + j) * xs;
        }
    }
#pragma unroll
    for (int j = 0; j < CPT; j++) red[ty][tx * CPT + j] = acc[j];
    __syncthreads();
    // 64 * CPT columns of the workgroup, one thread each, K-lanes added in order
    for (uint32_t c = threadIdx.x; c < 64 * CPT; c += 1024) {
        const uint32_t col = blockIdx.x * 64 * CPT + c;
        if (col >= a.N) continue;
        float sum = 0.f;
#pragma unroll
        for (int l = 0; l < 16; l++) sum += red[l][c];
        a.part[((size_t)m * a.ks + slice) * a.N + col] = sum;
    }
}

// 32 consecutive elements starting at element i (a multiple of 32; the base is 16-byte aligned) as f32
template <int DT> __device__ __forceinline__ void load_elems32(const void* p, size_t i, float* out) {
    if constexpr (DT == DT_F32) {
        const float4* v = (const float4*)((const float*)p + i);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float4 t = v[k];
            out[4 * k] = t.x; out[4 * k + 1] = t.y; out[4 * k + 2] = t.z; out[4 * k + 3] = t.w;
        }
    } else {
        const uint4* v = (const uint4*)((const uint16_t*)p + i);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint4 t = v[k];
            const uint32_t wds[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int h = 0; h < 4; h++) {
                if constexpr (DT == DT_F16) {
                    out[8 * k + 2 * h] = f16_bits_to_f32(wds[h] & 0xFFFFu);
                    out[8 * k + 2 * h + 1] = f16_bits_to_f32(wds[h] >> 16);
                } else {
                    out[8 * k + 2 * h] = __uint_as_float(wds[h] << 16);
                    out[8 * k + 2 * h + 1] = __uint_as_float(wds[h] & 0xFFFF0000u);
                }
            }
        }
    }
}

// The kernel for N % 32 == 0: a thread owns 32 columns, which are BITS whole words of a row at any
// code width (4 * BITS contiguous bytes, codes extracted with constant shifts). 256 threads = 16
// column slots x 16 K-lanes; a wave reads 4 rows x 64 * BITS contiguous bytes per load. K-lane ty
// takes rows congruent to d0 + ty mod 16 of the workgroup's K slice, four rows of a group at a time
// with their loads issued together. The 16 K-lanes of a column slot are added through LDS in lane
// order.
template <int DT, int BITS> __global__ __launch_bounds__(256) void qvm32_partial_kernel(QvmArgs a) {
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    __shared__ float red[16][16 * 32 + 1];
    const uint32_t tx = threadIdx.x & 15u, ty = threadIdx.x >> 4;
    const uint32_t c0 = (blockIdx.x * 16 + tx) * 32;
    const bool live = c0 < a.N;
    const uint32_t slice = blockIdx.y, m = blockIdx.z;
    const uint32_t d0 = slice * a.rows_per_slice;
    const uint32_t d1 = min(a.K, d0 + a.rows_per_slice);
    const uint32_t wi = c0 / 32 * BITS;
    float acc[32];
#pragma unroll
    for (int j = 0; j < 32; j++) acc[j] = 0.f;
    if (live) {
        for (uint32_t gs = d0; gs < d1; gs = (gs / a.G + 1) * a.G) {
            const uint32_t ge = min((gs / a.G + 1) * a.G, d1);
            uint32_t d = gs + ((d0 + ty + 16u - (gs & 15u)) & 15u);   // first row >= gs of this lane
            if (d >= ge) continue;
            // this group's scales and biases of the 32 columns: loads in flight with the first rows
            const size_t sb = (size_t)(gs / a.G) * a.N + c0;
            float sc[32], bi[32];
            load_elems32<DT>(a.scales, sb, sc);
            load_elems32<DT>(a.biases, sb, bi);
            float qdot[32];
#pragma unroll
            for (int j = 0; j < 32; j++) qdot[j] = 0.f;
            float xs = 0.f;
            for (; d < ge; d += 64) {
                uint32_t cw[4][BITS];
                float xv[4];
                // The four activations first, as loaded, then the rows' words, and only then the conversions: the order is
                // pinned (left to itself the compiler converts each activation behind its load, a wait per row; loaded under
                // a condition of its own it would sit in a branch). Rows past the group read row d again and count as zero.
                uint32_t xbits[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const uint32_t dr = d + 16 * r;
                    const size_t xi = (size_t)m * a.K + (dr < ge ? dr : d);
                    if constexpr (DT == DT_F32) xbits[r] = ((const uint32_t*)a.x)[xi];
                    else xbits[r] = ((const uint16_t*)a.x)[xi];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const uint32_t dr = d + 16 * r;
                    const uint32_t* row = a.w + (size_t)(dr < ge ? dr : d) * a.wpr + wi;
#pragma unroll
                    for (int i = 0; i < BITS; i++) cw[r][i] = row[i];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float xr = DT == DT_F32 ? __uint_as_float(xbits[r]) : DT == DT_BF16 ? bf16_bits_to_f32(xbits[r]) : f16_bits_to_f32(xbits[r]);
                    xv[r] = d + 16 * r < ge ? xr : 0.f;
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
#pragma unroll
                    for (int j = 0; j < 32; j++) {
                        const int o = j * BITS, lo = o >> 5, sh = o & 31;
                        uint32_t q = cw[r][lo] >> sh;
                        if (sh + BITS > 32) q |= cw[r][lo + 1] << (32 - sh);
                        qdot[j] = fmaf((float)(q & MASK), xv[r], qdot[j]);
                    }
                    xs += xv[r];
                }
            }
#pragma unroll
            for (int j = 0; j < 32; j++) acc[j] += sc[j] * qdot[j] + bi[j] * xs;
        }
    }
#pragma unroll
    for (int j = 0; j < 32; j++) red[ty][tx * 32 + j] = acc[j];
    __syncthreads();
    // 512 columns of the workgroup, two per thread, K-lanes added in order
    for (uint32_t c = threadIdx.x; c < 512; c += 256) {
        const uint32_t col = blockIdx.x * 512 + c;
        if (col >= a.N) continue;
        float sum = 0.f;
#pragma unroll
        for (int l = 0; l < 16; l++) sum += red[l][c];
        a.part[((size_t)m * a.ks + slice) * a.N + col] = sum;
    }
}

// Adds the slices' partial rows in a fixed order: 1024 threads = 64 columns x 16 slice-lanes; lane l
// adds slices l, l + 16, ... in that order (independent loads, all in flight), then the 16 lanes are
// added through LDS in lane order.
template <int DT> __global__ __launch_bounds__(1024) void qvm_reduce_kernel(QvmArgs a) {
    __shared__ float red[16][64];
    const uint32_t tx = threadIdx.x & 63u, l = threadIdx.x >> 6;
    const uint32_t c = blockIdx.x * 64 + tx, m = blockIdx.y;
    float sum = 0.f;
    if (c < a.N)
        for (uint32_t sl = l; sl < a.ks; sl += 16) sum += a.part[((size_t)m * a.ks + sl) * a.N + c];
    red[l][tx] = sum;
    __syncthreads();
    if (l == 0 && c < a.N) {
        float r = red[0][tx];
#pragma unroll
        for (int u = 1; u < 16; u++) r += red[u][tx];
        store_elem<DT>(a.out, (size_t)m * a.N + c, r);
    }
}

template <int DT> static const void* qvm32_fn(int bits) {
    switch (bits) {
        case 2: return (const void*)qvm32_partial_kernel<DT, 2>;
        case 3: return (const void*)qvm32_partial_kernel<DT, 3>;
        case 4: return (const void*)qvm32_partial_kernel<DT, 4>;
        case 5: return (const void*)qvm32_partial_kernel<DT, 5>;
        case 6: return (const void*)qvm32_partial_kernel<DT, 6>;
        case 7: return (const void*)qvm32_partial_kernel<DT, 7>;
        default: return (const void*)qvm32_partial_kernel<DT, 8>;
    }
}

template <int DT> static const void* qvm_fn(int bits) {
    switch (bits) {
        case 2: return (const void*)qvm_partial_kernel<DT, 2>;
        case 3: return (const void*)qvm_partial_kernel<DT, 3>;
        case 4: return (const void*)qvm_partial_kernel<DT, 4>;
        case 5: return (const void*)qvm_partial_kernel<DT, 5>;
        case 6: return (const void*)qvm_partial_kernel<DT, 6>;
        case 7: return (const void*)qvm_partial_kernel<DT, 7>;
        default: return (const void*)qvm_partial_kernel<DT, 8>;
    }
}

static constexpr int QVM32_WGS = 512;

// Slices of K across workgroups: enough workgroups to fill the chip, at least 64 rows (4 per
// K-lane) in a slice. The scale / bias terms are linear in the rows, so a slice need not hold
// whole groups.
uint32_t qvm_slices(int bits, uint32_t group_size, uint32_t M, uint32_t N, uint32_t K) {
    (void)group_size;
    const uint32_t cpt = 32 % bits == 0 ? 32u / (uint32_t)bits : 1u;
    const bool wide = N % 32 == 0;  // the 32-columns-per-thread kernel, 512 columns per workgroup of 256 threads
    const uint32_t col_wgs = wide ? (N + 511) / 512 : (N / cpt + 63) / 64;
    uint32_t ks = (uint32_t)(options().qvm_wgs ? options().qvm_wgs : (wide ? QVM32_WGS : 256)) / (col_wgs * (M ? M : 1u));
    if (ks < 1) ks = 1;
    if (ks > (K + 63) / 64) ks = (K + 63) / 64;
    return ks;
}

size_t qvm_scratch_bytes(int bits, uint32_t group_size, uint32_t M, uint32_t N, uint32_t K) {
    return (size_t)M * qvm_slices(bits, group_size, M, N, K) * N * sizeof(float);
}

int launch_qvm(const QmvParams& p, void* scratch, const LaunchCtx& lc) {
    const uint32_t G = p.group_size, cpt = 32 % p.bits == 0 ? 32u / (uint32_t)p.bits : 1u;
    if ((uint64_t)p.N * p.bits % 32) return fail(ERR_SHAPE, "qvm: N*bits must be a multiple of 32");
    if (p.M > 65535) return fail(ERR_UNSUPPORTED, "qvm: at most 65535 activation rows");
    QvmArgs a;
    a.w = (const uint32_t*)p.w;
    a.scales = p.scales;
    a.biases = p.biases;
    a.x = p.x;
    a.part = (float*)scratch;
    a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K; a.G = G;
    a.wpr = (uint32_t)((uint64_t)p.N * p.bits / 32);
    a.ks = qvm_slices(p.bits, G, p.M, p.N, p.K);
    a.rows_per_slice = ((p.K + a.ks - 1) / a.ks + 15) / 16 * 16;
    a.ks = (p.K + a.rows_per_slice - 1) / a.rows_per_slice;   // no empty slice
    const bool wide = p.N % 32 == 0 && (uintptr_t)p.scales % 16 == 0 && (uintptr_t)p.biases % 16 == 0;
    const void *fn, *rfn;
    switch (p.dtype) {
        case DT_F32: fn = qvm_fn<DT_F32>(p.bits); rfn = (const void*)qvm_reduce_kernel<DT_F32>; break;
        case DT_F16: fn = qvm_fn<DT_F16>(p.bits); rfn = (const void*)qvm_reduce_kernel<DT_F16>; break;
        case DT_BF16: fn = qvm_fn<DT_BF16>(p.bits); rfn = (const void*)qvm_reduce_kernel<DT_BF16>; break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    if (wide) fn = p.dtype == DT_F32 ? qvm32_fn<DT_F32>(p.bits) : p.dtype == DT_F16 ? qvm32_fn<DT_F16>(p.bits) : qvm32_fn<DT_BF16>(p.bits);
    LaunchCtx l1 = lc, l2 = lc;
    l1.stop = nullptr;
    l2.start = nullptr;
    void* args[] = {&a};
    hipError_t e = wide ? launch_kernel(fn, dim3((p.N + 511) / 512, a.ks, p.M), dim3(256), args, 0, l1)
                        : launch_kernel(fn, dim3((p.N / cpt + 63) / 64, a.ks, p.M), dim3(1024), args, 0, l1);
    if (e != hipSuccess) return hip_fail(e, "qvm kernel launch");
    e = launch_kernel(rfn, dim3((p.N + 63) / 64, p.M), dim3(1024), args, 0, l2);
    if (e != hipSuccess) return hip_fail(e, "qvm reduce kernel launch");
    return ERR_OK;
}

}  // namespace mtq
