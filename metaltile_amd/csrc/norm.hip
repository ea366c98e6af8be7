// RMS normalisation of one activation row: the first phase of the reference's fused
// norm + quantized GEMV (crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:64-77 and
// mt_rms_inv_scalar, crates/metaltile-std/src/mlx/rms_norm.rs:86-96), used on its own
// for row lengths the fused streaming kernel does not take.
#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

struct NormArgs {
    const void* x;
    const void* w;
    const float* eps;
    void* out;
    uint32_t K;
};

// One workgroup; v[k] = (x[k] * w[k]) * (1 / sqrt(sum(x^2) / K + eps)) in f32. f32 rows are
// stored as they are; f16 / bf16 rows are stored as two rows of K elements, the rounded
// value and the rounded remainder, so that a two-row qmv followed by add_rows_kernel sees
// 16 significant bits of v.
template <int DT> __global__ __launch_bounds__(1024) void rms_norm_kernel(NormArgs a) {
    __shared__ float part[16];
    const uint32_t tid = threadIdx.x;
    float ssq = 0.f;
    for (uint32_t k = tid; k < a.K; k += blockDim.x) {
        const float v = load_elem<DT>(a.x, k);
        ssq += v * v;
    }
    ssq = seg_allreduce(ssq, 64);
    if ((tid & 63u) == 0) part[tid >> 6] = ssq;
    __syncthreads();
    float tot = 0.f;
    for (uint32_t wv = 0; wv < (blockDim.x >> 6); wv++) tot += part[wv];
    const float inv = 1.0f / sqrtf(tot / (float)a.K + a.eps[0]);
    for (uint32_t k = tid; k < a.K; k += blockDim.x) {
        const float v = load_elem<DT>(a.x, k) * load_elem<DT>(a.w, k) * inv;
        store_elem<DT>(a.out, k, v);
        if constexpr (DT != DT_F32) {
            const float hi = load_elem<DT>(a.out, k);  // this thread's own store
            store_elem<DT>(a.out, (size_t)a.K + k, v - hi);
        }
    }
}

// out[n] = a[n] + b[n] (f32 sum, rounded to the element type)
template <int DT> __global__ __launch_bounds__(256) void add_rows_kernel(const void* a, const void* b, void* out, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) store_elem<DT>(out, i, load_elem<DT>(a, i) + load_elem<DT>(b, i));
}

int launch_add_rows(int dtype, const void* a, const void* b, void* out, uint32_t n, const LaunchCtx& lc) {
    const void* fn;
    switch (dtype) {
        case DT_F16: fn = (const void*)add_rows_kernel<DT_F16>; break;
        case DT_BF16: fn = (const void*)add_rows_kernel<DT_BF16>; break;
        default: fn = (const void*)add_rows_kernel<DT_F32>; break;
    }
    void* args[] = {&a, &b, &out, &n};
    hipError_t e = launch_kernel(fn, dim3((n + 255) / 256), dim3(256), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "add rows kernel launch");
    return ERR_OK;
}

int launch_rms_norm(int dtype, const void* x, const void* norm_w, const float* eps, void* out, uint32_t K,
                    const LaunchCtx& lc) {
    if (!x || !norm_w || !eps || !out) return fail(ERR_BAD_ARG, "null buffer");
    if (K == 0) return fail(ERR_SHAPE, "in_dim must be non-zero");
    NormArgs a{x, norm_w, eps, out, K};
    const void* fn;
    switch (dtype) {
        case DT_F32: fn = (const void*)rms_norm_kernel<DT_F32>; break;
        case DT_F16: fn = (const void*)rms_norm_kernel<DT_F16>; break;
        case DT_BF16: fn = (const void*)rms_norm_kernel<DT_BF16>; break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    uint32_t tpb = 64;
    while (tpb < 1024 && tpb * 4 < K) tpb *= 2;
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3(1), dim3(tpb), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "rms norm kernel launch");
    return ERR_OK;
}

}  // namespace mtq
