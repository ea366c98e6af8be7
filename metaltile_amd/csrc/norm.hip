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
// value and the rounded, scaled remainder (RemSplit), so that a two-row qmv followed by
// add_rows_kernel sees 16 significant bits of v.
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
        if constexpr (DT == DT_F32) {
            store_elem<DT>(a.out, k, v);
        } else {
            uint32_t hi, lo;
            RemSplit<DT>::split(v, hi, lo);
            ((uint16_t*)a.out)[k] = (uint16_t)hi;
            ((uint16_t*)a.out)[(size_t)a.K + k] = (uint16_t)lo;
        }
    }
}

struct GatedNormArgs {
    const float* y;
    const void* z;
    const void* w;
    const float* eps;
    void* out;
    uint32_t hv, dv;
};

// Gated RMS normalisation, the first phase of the reference's fused gated-norm + 4-bit GEMV
// (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:120-151): one workgroup per row r of hv,
// v[r, d] = y[r, d] * (1 / sqrt(sum_d(y[r]^2) / dv + eps)) * w[d] * silu(z[r, d]), in f32 and in that order;
// y is f32 whatever the element type, z and w are of the element type. Stored flat (index r * dv + d) the way
// rms_norm_kernel stores its row: as it is for f32, as value and remainder rows of hv * dv for f16 / bf16.
template <int DT> __global__ __launch_bounds__(256) void gated_rms_norm_kernel(GatedNormArgs a) {
    __shared__ float part[4];
    const uint32_t tid = threadIdx.x, r = blockIdx.x;
    const float* yr = a.y + (size_t)r * a.dv;
    float ssq = 0.f;
    for (uint32_t d = tid; d < a.dv; d += blockDim.x) ssq += yr[d] * yr[d];
    ssq = seg_allreduce(ssq, 64);
    if ((tid & 63u) == 0) part[tid >> 6] = ssq;
    __syncthreads();
    float tot = 0.f;
    for (uint32_t wv = 0; wv < (blockDim.x >> 6); wv++) tot += part[wv];
    const float inv = 1.0f / sqrtf(tot / (float)a.dv + a.eps[0]);
    const size_t K = (size_t)a.hv * a.dv;
    for (uint32_t d = tid; d < a.dv; d += blockDim.x) {
        const size_t idx = (size_t)r * a.dv + d;
        const float zv = load_elem<DT>(a.z, idx);
        const float gate = zv / (1.0f + expf(0.0f - zv));
        const float v = yr[d] * inv * load_elem<DT>(a.w, d) * gate;
        if constexpr (DT == DT_F32) {
            store_elem<DT>(a.out, idx, v);
        } else {
            uint32_t hi, lo;
            RemSplit<DT>::split(v, hi, lo);
            ((uint16_t*)a.out)[idx] = (uint16_t)hi;
            ((uint16_t*)a.out)[K + idx] = (uint16_t)lo;
        }
    }
}

// out[n] = a[n] + b[n] / kRemScale (f32 sum, rounded to the element type): the outputs of a value row and of its
// scaled remainder row
template <int DT> __global__ __launch_bounds__(256) void add_rows_kernel(const void* a, const void* b, void* out, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) store_elem<DT>(out, i, load_elem<DT>(a, i) + load_elem<DT>(b, i) * (1.0f / RemSplit<DT>::kRemScale));
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

int launch_gated_rms_norm(int dtype, const float* y, const void* z, const void* norm_w, const float* eps, void* out,
                          uint32_t hv, uint32_t dv, const LaunchCtx& lc) {
    if (!y || !z || !norm_w || !eps || !out) return fail(ERR_BAD_ARG, "null buffer");
    if (hv == 0 || dv == 0) return fail(ERR_SHAPE, "hv and dv must be non-zero");
    GatedNormArgs a{y, z, norm_w, eps, out, hv, dv};
    const void* fn;
    switch (dtype) {
        case DT_F32: fn = (const void*)gated_rms_norm_kernel<DT_F32>; break;
        case DT_F16: fn = (const void*)gated_rms_norm_kernel<DT_F16>; break;
        case DT_BF16: fn = (const void*)gated_rms_norm_kernel<DT_BF16>; break;
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
    uint32_t tpb = 64;
    while (tpb < 256 && tpb < dv) tpb *= 2;
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3(hv), dim3(tpb), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "gated rms norm kernel launch");
    return ERR_OK;
}

}  // namespace mtq
