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

template <int DT> __global__ __launch_bounds__(256) void qvm_reduce_kernel(QvmArgs a) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
    if (c >= a.N) return;
    float sum = 0.f;
    for (uint32_t sl = 0; sl < a.ks; sl++) sum += a.part[((size_t)m * a.ks + sl) * a.N + c];
    store_elem<DT>(a.out, (size_t)m * a.N + c, sum);
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

// Slices of K across workgroups: enough workgroups to fill the chip, at least 64 rows (4 per
// K-lane) in a slice. The scale / bias terms are linear in the rows, so a slice need not hold
// whole groups.
uint32_t qvm_slices(int bits, uint32_t group_size, uint32_t M, uint32_t N, uint32_t K) {
    (void)group_size;
    const uint32_t cpt = 32 % bits == 0 ? 32u / (uint32_t)bits : 1u;
    const uint32_t col_wgs = (N / cpt + 63) / 64;
    uint32_t ks = (uint32_t)(options().qvm_wgs ? options().qvm_wgs : 256) / (col_wgs * (M ? M : 1u));
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
    const void *fn, *rfn;
    switch (p.dtype) {
        case DT_F32: fn = qvm_fn<DT_F32>(p.bits); rfn = (const void*)qvm_reduce_kernel<DT_F32>; break;
        case DT_F16: fn = qvm_fn<DT_F16>(p.bits); rfn = (const void*)qvm_reduce_kernel<DT_F16>; break;
        case DT_BF16: fn = qvm_fn<DT_BF16>(p.bits); rfn = (const void*)qvm_reduce_kernel<DT_BF16>; break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    LaunchCtx l1 = lc, l2 = lc;
    l1.stop = nullptr;
    l2.start = nullptr;
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3((p.N / cpt + 63) / 64, a.ks, p.M), dim3(1024), args, 0, l1);
    if (e != hipSuccess) return hip_fail(e, "qvm kernel launch");
    e = launch_kernel(rfn, dim3((p.N + 255) / 256, p.M), dim3(256), args, 0, l2);
    if (e != hipSuccess) return hip_fail(e, "qvm reduce kernel launch");
    return ERR_OK;
}

}  // namespace mtq
