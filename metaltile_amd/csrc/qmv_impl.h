// qmv / small-batch qmm / gather_qmv kernel family for gfx950 (device code and
// the per-dtype launch switch). Included by qmv_f32.hip, qmv_f16.hip and
// qmv_bf16.hip, which each instantiate one element dtype so the three compile in
// parallel; qmv.hip holds the host-side geometry choice.
//
// Replaces, on the reference side, mt_qmv / mt_qmm / mt_qmm_bm{2,4} and their
// int8 trio (crates/metaltile-std/src/mlx/quantized.rs:8-308, 343-621, 650,
// 1072, 1475-1870), dequant_gemv_int{2,4,8} and _int4_fast
// (crates/metaltile-std/src/ffai/dequant_gemv.rs:52-100, 212-341), the CSR
// gather kernels mt_moe_gather_qmm_int4{,_m8,_m16,_m32} / _b8
// (crates/metaltile-std/src/ffai/moe.rs:358-433, 634, 900, 1363, 461-523), the
// per-row-index gather ABI (moe.rs:2256-2550) at decode-sized row counts, and
// dequant_gemv_int4_expert_indexed
// (crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:58-105).
//
// Geometry. A row of packed weights is C = K*bits/128 chunks of 16 bytes. A
// workgroup of TPB = C*rps threads owns a tile of R = RT*rps consecutive rows,
// which is one contiguous R*C*16-byte block of HBM. Thread t keeps chunk
// position c = t % C for its whole life and owns exactly one chunk of every row
// it visits (rows rsub + i*rps, rsub = t / C).
//
// Order of work in a thread. All global loads are issued up front in
// straight-line code, smallest first, because loads return in issue order:
// the tile's scales and biases (four elements per load), the thread's CPC
// activations, then RT independent 128-bit non-temporal weight loads. Scales and
// biases go through LDS as (s, b - MAGIC*s) float pairs. Rows are then consumed
// in load order -- the compiler's s_waitcnt vmcnt(n) counts down one row at a
// time -- so the arithmetic and the cross-lane reduction of row i overlap the
// arrival of rows i+1..RT-1. Addresses of out-of-range rows are clamped rather
// than branched around, which keeps the load sequence free of control flow.
//
// Per-row sums are reduced across the C lanes of a row with DPP butterflies
// inside each wave and a small LDS exchange across waves.
//
// Gather modes run the same tile against several activation rows: blockIdx.y
// is the expert; the workgroup finds the rows routed to that expert, exits at
// once if there are none (so only experts that are hit are streamed from
// HBM), keeps its weight tile in registers and walks the rows MB at a time.
#pragma once
#include "mtq_device.h"
#include <type_traits>

#include "mtq_internal.h"

namespace mtq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Loads return in issue order, so the order they are issued in is part of the
// design. The empty asm keeps the optimiser from sinking or hoisting memory
// operations across this point; the scheduling barrier does the same for the
// machine scheduler. Neither emits an instruction.
#define MTQ_KEEP_LOAD_ORDER()                \
    do {                                     \
        asm volatile("" ::: "memory");       \
        __builtin_amdgcn_sched_barrier(0);   \
    } while (0)

struct QmvKArgs {
    const u32x4* w;
    const void* scales;
    const void* biases;
    const void* x;
    void* out;
    const uint32_t* route;
    uint32_t M, N, K, C;
    uint32_t log2g, rps, T, E;
    uint32_t gpr;          // groups per row = K / G
    uint32_t lds_sb_pairs; // capacity of the sb area in float2
    uint32_t wpr;          // waves per row (C / 64), 0 when C < 64
    uint32_t list_cap;     // capacity of the row list (indices mode)
};

// Launch geometry chosen on the host (qmv.hip).
struct QmvGeom {
    int mb;        // activation rows per pass: 1..4
    int rt;        // weight rows per thread: 4 or 8 (7 for balance when it divides better)
    int sbi;       // vector loads of scales (and of biases) per thread: 1, 2, 4; 0 = element-wise
    uint32_t tpb;
    size_t shmem;
    dim3 grid;
};

// Four consecutive scale (or bias) elements as one load.
template <int DT> struct SbVec;
template <> struct SbVec<DT_F32> {
    typedef float4 type;
    static __device__ __forceinline__ void unpack(const float4& v, float (&o)[4]) {
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct SbVec<DT_F16> {
    typedef uint2 type;
    static __device__ __forceinline__ void unpack(const uint2& v, float (&o)[4]) {
        o[0] = f16_bits_to_f32(v.x & 0xFFFFu); o[1] = f16_bits_to_f32(v.x >> 16);
        o[2] = f16_bits_to_f32(v.y & 0xFFFFu); o[3] = f16_bits_to_f32(v.y >> 16);
    }
};
template <> struct SbVec<DT_BF16> {
    typedef uint2 type;
    static __device__ __forceinline__ void unpack(const uint2& v, float (&o)[4]) {
        o[0] = bf16_bits_to_f32(v.x & 0xFFFFu); o[1] = bf16_bits_to_f32(v.x >> 16);
        o[2] = bf16_bits_to_f32(v.y & 0xFFFFu); o[3] = bf16_bits_to_f32(v.y >> 16);
    }
};

// SBI: vector loads of scales per thread (0 = element-wise staging for tiles
// whose scale block is not 4-aligned).
template <int DT, int BITS, int MB, int RT, int MODE, int MAXT, int SBI>
__global__ __launch_bounds__(MAXT) void qmv_kernel(QmvKArgs a) {
    typedef XSlice<DT, BITS> XS;
    typedef typename Elem<DT>::type elem_t;
    typedef typename SbVec<DT>::type sbvec_t;
    constexpr int CPC = XS::CPC;
    constexpr float MAGIC = PathSel<DT, BITS>::kMagic;
    constexpr uint32_t NOROW = 0xFFFFFFFFu;
    constexpr bool kOneBatch = MODE == GATHER_NONE || MODE == GATHER_SINGLE;
    constexpr int SBN = SBI > 0 ? SBI : 1;

    extern __shared__ __align__(16) unsigned char smem[];
    float2* sb = (float2*)smem;                            // [R][gpr] (s, b - MAGIC*s)
    float* part = (float*)(sb + a.lds_sb_pairs);           // [R*MB][wpr]
    uint32_t* rowlist = (uint32_t*)(part + RT * a.rps * MB * (a.wpr ? a.wpr : 1));
    __shared__ uint32_t s_meta[4];

    const uint32_t tid = threadIdx.x;
    const uint32_t TPB = blockDim.x;
    const uint32_t c = tid % a.C;
    const uint32_t rsub = tid / a.C;
    const uint32_t R = RT * a.rps;
    const uint32_t row0 = blockIdx.x * R;
    const uint32_t lane = tid & 63u;

    // ---- routing: which activation rows does this workgroup serve? ----------
    uint32_t expert = 0, cnt = a.M, lo = 0, n1 = a.M, lo2 = 0;
    if constexpr (MODE == GATHER_CSR) {
        expert = blockIdx.y;
        // E(t) = first e with t < off[e+1], else 0
        // (crates/metaltile-std/src/ffai/moe.rs:376-385): for expert e that is
        // t in [max(off[1..e]), off[e+1]); rows past every offset fall to expert 0.
        cnt = csr_expert_rows(a.route, a.E, a.T, expert, lane, lo, n1, lo2);
        if (cnt == 0) return;
    } else if constexpr (MODE == GATHER_INDICES) {
        expert = blockIdx.y;
        if (tid < 64) {
            uint32_t n = 0;
            for (uint32_t t0 = 0; t0 < a.T; t0 += 64) {
                uint32_t t = t0 + lane;
                bool hit = t < a.T && a.route[t] == expert;
                unsigned long long m = __ballot(hit);
                if (hit) rowlist[n + __popcll(m & ((1ull << lane) - 1ull))] = t;
                n += (uint32_t)__popcll(m);
            }
            if (lane == 0) s_meta[0] = n;
        }
        __syncthreads();
        cnt = s_meta[0];
        if (cnt == 0) return;
    } else if constexpr (MODE == GATHER_SINGLE) {
        expert = min(a.route[0], a.E - 1);  // an out-of-range id must not fault the GPU
        cnt = 1;
    }

    auto batch_row = [&](uint32_t j) -> uint32_t {
        if (j >= cnt) return NOROW;
        if constexpr (MODE == GATHER_CSR) return j < n1 ? lo + j : lo2 + (j - n1);
        else if constexpr (MODE == GATHER_INDICES) return rowlist[j];
        else return j;
    };

    const size_t slab_rows = (size_t)expert * a.N;  // row offset of this expert's slab
    const u32x4* wbase = a.w + slab_rows * a.C;
    const uint32_t rows_in_tile = min(R, a.N - row0);
    const uint32_t k0 = c * CPC;

    // ---- (1) scales / biases of the tile ------------------------------------
    const size_t sb0 = (slab_rows + row0) * a.gpr;
    const uint32_t n_sb = rows_in_tile * a.gpr;
    sbvec_t sraw[SBN], braw[SBN];
    if constexpr (SBI > 0) {
        const sbvec_t* sp = (const sbvec_t*)((const elem_t*)a.scales + sb0);
        const sbvec_t* bp = (const sbvec_t*)((const elem_t*)a.biases + sb0);
        const uint32_t last = n_sb / 4 - 1;  // n_sb is a non-zero multiple of 4 here
#pragma unroll
        for (int j = 0; j < SBI; j++) {
            const uint32_t v = min(tid + j * TPB, last);
            sraw[j] = sp[v];
            braw[j] = bp[v];
        }
    }
    MTQ_KEEP_LOAD_ORDER();
    // ---- (2) activations of the first (or only) batch -----------------------
    uint32_t xrow[MB];
    XS xs[MB];
    uint4 xraw[MB][XS::NRAW];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        xrow[mb] = batch_row(mb);
        const uint32_t t = xrow[mb] == NOROW ? batch_row(0) : xrow[mb];  // row 0 of the batch always exists
        xs[mb].load_raw(a.x, (size_t)t * a.K + k0, xraw[mb]);
    }
    MTQ_KEEP_LOAD_ORDER();
    // ---- (3) weights: RT independent 128-bit non-temporal streams -----------
    u32x4 wv[RT];
#pragma unroll
    for (int i = 0; i < RT; i++) {
        const uint32_t row = min(row0 + i * a.rps + rsub, a.N - 1);
        wv[i] = __builtin_nontemporal_load(wbase + (size_t)row * a.C + c);
    }

    MTQ_KEEP_LOAD_ORDER();

    // ---- stage (s, b - MAGIC*s) pairs in LDS --------------------------------
    if constexpr (SBI > 0) {
#pragma unroll
        for (int j = 0; j < SBI; j++) {
            const uint32_t v = tid + j * TPB;
            float sv[4], bv[4];
            SbVec<DT>::unpack(sraw[j], sv);
            SbVec<DT>::unpack(braw[j], bv);
            if (v * 4 < n_sb) {
                float4* dst = (float4*)(sb + v * 4);
                dst[0] = make_float4(sv[0], bv[0] - MAGIC * sv[0], sv[1], bv[1] - MAGIC * sv[1]);
                dst[1] = make_float4(sv[2], bv[2] - MAGIC * sv[2], sv[3], bv[3] - MAGIC * sv[3]);
            }
        }
    } else {
        for (uint32_t i = tid; i < n_sb; i += TPB) {
            float sv = load_elem<DT>(a.scales, sb0 + i);
            float bv = load_elem<DT>(a.biases, sb0 + i);
            sb[i] = make_float2(sv, bv - MAGIC * sv);
        }
    }
    __syncthreads();

    const uint32_t g0 = k0 >> a.log2g;
    const uint32_t g1 = (k0 + CPC / 2) >> a.log2g;  // == g0 unless a chunk spans two groups
    const int seg = a.C >= 64 ? 64 : (int)a.C;

    // Plain and single-expert launches carry at most MB rows: exactly one batch.
    const uint32_t n_batches = kOneBatch ? 1u : (cnt + MB - 1) / MB;
    for (uint32_t bi = 0; bi < n_batches; bi++) {
        const uint32_t base = bi * MB;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            if (bi > 0) {
                xrow[mb] = batch_row(base + mb);
                const uint32_t t = xrow[mb] == NOROW ? batch_row(base) : xrow[mb];
                xs[mb].load_raw(a.x, (size_t)t * a.K + k0, xraw[mb]);
            }
            xs[mb].prepare(xraw[mb]);
        }

        float acc[RT][MB];
#pragma unroll
        for (int i = 0; i < RT; i++) {
            const uint32_t rl = min(i * a.rps + rsub, rows_in_tile - 1);
            const float2 p0 = sb[rl * a.gpr + g0];
            const float2 p1 = sb[rl * a.gpr + g1];
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                float d01 = xs[mb].dot_dword(wv[i].x, 0, 0.f);
                d01 = xs[mb].dot_dword(wv[i].y, 1, d01);
                float d23 = xs[mb].dot_dword(wv[i].z, 2, 0.f);
                d23 = xs[mb].dot_dword(wv[i].w, 3, d23);
                float v = p0.x * d01 + p0.y * xs[mb].xsum[0];
                v += p1.x * d23 + p1.y * xs[mb].xsum[1];
                acc[i][mb] = seg_allreduce(v, seg);
            }
        }

        if (a.wpr <= 1) {
            // the whole row lives in one wave (or one segment of it)
            if (c == 0) {
#pragma unroll
                for (int i = 0; i < RT; i++) {
                    const uint32_t row = row0 + i * a.rps + rsub;
#pragma unroll
                    for (int mb = 0; mb < MB; mb++)
                        if (row < a.N && xrow[mb] != NOROW)
                            store_elem<DT>(a.out, (size_t)xrow[mb] * a.N + row, acc[i][mb]);
                }
            }
        } else {
            if (bi) __syncthreads();  // previous batch's readers are done with `part`
            if ((c & 63u) == 0) {
                const uint32_t wir = c >> 6;
#pragma unroll
                for (int i = 0; i < RT; i++) {
                    const uint32_t rl = i * a.rps + rsub;
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) part[(rl * MB + mb) * a.wpr + wir] = acc[i][mb];
                }
            }
            __syncthreads();
            for (uint32_t o = tid; o < rows_in_tile * MB; o += TPB) {
                const uint32_t rl = o / MB, mb = o % MB;
                const uint32_t t = batch_row(base + mb);
                if (t == NOROW) continue;
                float sum = 0.f;
                for (uint32_t wi = 0; wi < a.wpr; wi++) sum += part[o * a.wpr + wi];
                store_elem<DT>(a.out, (size_t)t * a.N + row0 + rl, sum);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Streaming variant for rows of at least one wave (C % 64 == 0), plain and
// single-expert modes.
//
// The one-shot kernel above issues all of a thread's weight loads at once, so
// a wave that is dispatched late receives all its rows at the very end of the
// stream and its whole arithmetic becomes the tail of the kernel. Here each
// workgroup owns a contiguous range of rows and every thread walks its rows
// through a ring of D registers-resident 16-byte chunks: the load for row j+D
// is issued right after row j has been consumed, so each wave's traffic is
// spread over the kernel's lifetime, D loads stay in flight per thread, and
// only one batch of arithmetic remains once the last byte has arrived. The
// scales and biases of the whole row range are staged in LDS once. Row sums
// are reduced D at a time: v_permlane32_swap / v_permlane16_swap fold pairs of
// partial sums across half-waves and 16-lane rows (one add per pair) before a
// four-step DPP butterfly inside the rows, 2.5 instructions per row instead
// of 6. Partial sums of the waves that share a row meet in LDS at the end.
// ---------------------------------------------------------------------------

struct QmvSArgs {
    const u32x4* w;
    const void* scales;
    const void* biases;
    const void* x;
    void* out;
    const uint32_t* route;   // expert_index (single mode) or null
    uint32_t M, N, K, C;
    uint32_t log2g, rps, gpr, wpr;
    uint32_t rows_per_wg;    // multiple of D*rps
    uint32_t nb;             // batches of D rows per thread
    uint32_t E;
    uint32_t T;              // routed modes: activation rows (fewer than experts; blockIdx.y counts the experts that have rows)
    // Batched launch (several weight matrices against the same activations, blockIdx.y
    // = matrix): per-matrix operands; nmat = 0 for a plain launch.
    uint32_t nmat;
    uint32_t mn[4];
    const void* mw[4];
    const void* ms[4];
    const void* mbias[4];
    void* mo[4];
    // Fused RMSNorm (NORM kernels): per-element norm weights T[K] and a device f32 holding eps.
    const void* norm_w;
    const float* eps;
    // Fused gated RMSNorm (NORM = 2): x is f32 [K / dv, dv] whatever the element type, gate_z T[K], norm_w T[dv].
    const void* gate_z;
    uint32_t dv;
};

typedef unsigned u32x2v __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float swap32_add(float a, float b) {
    // lanes 0..31 end up with a[l] + a[l+32], lanes 32..63 with b[l-32] + b[l]
    u32x2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}
__device__ __forceinline__ float swap16_add(float a, float b) {
    // 16-lane rows: [a0+a1, b0+b1, a2+a3, b2+b3]
    u32x2v r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}
__device__ __forceinline__ float row16_allreduce(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    return v;
}
// Sums four per-lane values over the wave. Returns, in every lane of 16-lane
// row r, the wave total of value kSlotOfRow[r] = {0, 2, 1, 3}[r].
__device__ __forceinline__ float wave_reduce4(float v0, float v1, float v2, float v3) {
    return row16_allreduce(swap16_add(swap32_add(v0, v1), swap32_add(v2, v3)));
}

// One vector of the gated, normalised activation: element e = y[e] * inv * w[e] * silu(z[e]) in f32
// (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:138-149), y in f32 (two vectors of 4 for a 16-bit vector of
// 8, one for an f32 vector of 4), z and w of the element type; split into `hi` and `lo` as in raw_normed.
template <int DT> __device__ __forceinline__ void raw_gated(const uint4* yv, uint4 zv, uint4 wv, float inv, uint4& hi, uint4& lo) {
    const uint32_t z[4] = {zv.x, zv.y, zv.z, zv.w};
    const uint32_t w[4] = {wv.x, wv.y, wv.z, wv.w};
    // (the hardware's exponential and reciprocal, about 1 ulp each: a full-precision quotient is a dozen instructions per
    // element, and every workgroup gates its whole slice before its first dot product)
    auto gated = [&](float y, float zf, float wf) { return y * inv * wf * (zf * __builtin_amdgcn_rcpf(1.0f + __expf(0.0f - zf))); };
    uint32_t h[4], l[4];
    if constexpr (DT == DT_F32) {
        const uint32_t y[4] = {yv[0].x, yv[0].y, yv[0].z, yv[0].w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            h[j] = __float_as_uint(gated(__uint_as_float(y[j]), __uint_as_float(z[j]), __uint_as_float(w[j])));
            l[j] = 0;
        }
    } else {
        const uint32_t y[8] = {yv[0].x, yv[0].y, yv[0].z, yv[0].w, yv[1].x, yv[1].y, yv[1].z, yv[1].w};
        auto up = [](uint32_t b) { return DT == DT_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b); };
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float v0 = gated(__uint_as_float(y[2 * j]), up(z[j] & 0xFFFFu), up(w[j] & 0xFFFFu));
            const float v1 = gated(__uint_as_float(y[2 * j + 1]), up(z[j] >> 16), up(w[j] >> 16));
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

// NORM: the activation row is RMS-normalised on the fly, x'[k] = x[k] * norm_w[k] *
// rsqrt(mean(x^2) + eps) (crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:64-77,104-106),
// every workgroup recomputing the row's sum of squares from the slice its threads hold.
// The dot2 path takes 16-bit operands: for f16 / bf16 the f32 x' is carried as two rows,
// its rounded value and the rounded remainder (MB = 2), whose dots are added.
// NORM = 2: the gated form (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:120-151). The activation is hv rows
// of dv f32 values y, each row normalised by its own sum of squares and gated by silu(z): a thread's chunk lies within
// one such row (dv a multiple of the chunk), the row's dv / CPC threads are neighbours in a wave, so the sum of squares
// is a segmented lane reduction and needs no LDS.
// NORM = 3: the same with four row slots per workgroup (rows of 2048 values in 256 threads): the four threads that
// hold the same chunk gate a quarter of it each (one vector of 8) and pass the halves through LDS behind the barrier
// the staging needs anyway, instead of each gating all 32 values ahead of its first dot product.
template <int DT, int BITS, int MB, int D, int MODE, int MAXT, int SBI, int NORM = 0>
__global__ __launch_bounds__(MAXT) void qmv_stream_kernel(QmvSArgs a) {
    static_assert(!NORM || (MB == (DT == DT_F32 ? 1 : 2) && MODE == GATHER_NONE), "the fused norm takes one plain activation row");
    static_assert(NORM != 3 || (DT != DT_F32 && BITS == 4), "the dealt gate: 16-bit types, 4-bit codes");
    constexpr bool GATED = NORM == 2 || NORM == 3;
    constexpr int MBR = NORM ? 1 : MB;  // activation rows as the caller sees them
    static_assert(D == 4 || D == 8, "ring depth");
    typedef XSlice<DT, BITS> XS;
    typedef typename Elem<DT>::type elem_t;
    typedef typename SbVec<DT>::type sbvec_t;
    constexpr int CPC = XS::CPC;
    constexpr float MAGIC = PathSel<DT, BITS>::kMagic;

    extern __shared__ __align__(16) unsigned char smem[];
    float2* sb = (float2*)smem;                                   // [rows_per_wg][gpr]
    float* part = (float*)(sb + (size_t)a.rows_per_wg * a.gpr);   // [rows_per_wg][MB][wpr]
    float* ssq_part = part + (size_t)a.rows_per_wg * MBR * a.wpr;  // [waves] (NORM only)

    const uint32_t tid = threadIdx.x;
    const uint32_t TPB = blockDim.x;
    const uint32_t c = tid % a.C;
    const uint32_t rsub = tid / a.C;
    const uint32_t lane = tid & 63u;
    const uint32_t rb = blockIdx.x * a.rows_per_wg;
    // operands of this workgroup's matrix (selected with scalar compares: an indexed
    // read of the argument arrays would go through scratch memory)
    const u32x4* Wm = a.w;
    const void* Sm = a.scales;
    const void* Bm = a.biases;
    void* Om = a.out;
    uint32_t Nm = a.N;
    if (a.nmat) {
        const uint32_t j = blockIdx.y;
        Wm = (const u32x4*)(j == 0 ? a.mw[0] : j == 1 ? a.mw[1] : j == 2 ? a.mw[2] : a.mw[3]);
        Sm = j == 0 ? a.ms[0] : j == 1 ? a.ms[1] : j == 2 ? a.ms[2] : a.ms[3];
        Bm = j == 0 ? a.mbias[0] : j == 1 ? a.mbias[1] : j == 2 ? a.mbias[2] : a.mbias[3];
        Om = j == 0 ? a.mo[0] : j == 1 ? a.mo[1] : j == 2 ? a.mo[2] : a.mo[3];
        Nm = j == 0 ? a.mn[0] : j == 1 ? a.mn[1] : j == 2 ? a.mn[2] : a.mn[3];
        if (rb >= Nm) return;  // the grid is sized for the tallest matrix
    }
    const uint32_t rows_here = min(a.rows_per_wg, Nm - rb);      // >= 1 by construction of the grid
    const uint32_t k0 = c * CPC;

    // Routed rows (one or two rows on at most 64 experts: a decode step of one token through a mixture-of-experts
    // layer): grid row blockIdx.y serves the blockIdx.y-th expert that has a row and runs the whole kernel once per row
    // of that expert - one row each when a token's experts are distinct, as top-k routing makes them.
    constexpr bool ROUTED = MODE == GATHER_CSR || MODE == GATHER_INDICES;
    uint32_t expert = 0, n_pass = 1, r_lo = 0, r_n1 = 1, r_lo2 = 0;
    unsigned long long r_mask = 0;
    if constexpr (MODE == GATHER_SINGLE) expert = min(a.route[0], a.E - 1);
    if constexpr (MODE == GATHER_CSR) {
        n_pass = csr_route64(a.route, a.E, a.T, blockIdx.y, true, lane, expert, r_lo, r_n1, r_lo2);
        if (n_pass == 0) return;
        expert = __builtin_amdgcn_readfirstlane(expert);
    }
    if constexpr (MODE == GATHER_INDICES) {
        expert = __builtin_amdgcn_readfirstlane(ids_slot_expert(a.route, a.E, a.T, blockIdx.y, lane));
        if (expert == 0xFFFFFFFFu) return;
        r_mask = __ballot(lane < a.T && a.route[lane] == expert);
        n_pass = (uint32_t)__popcll(r_mask);
    }
    const size_t slab_rows = (size_t)expert * Nm;
    const u32x4* wbase = Wm + (slab_rows + rb) * a.C + c;
    for (uint32_t pass = 0; pass < (ROUTED ? n_pass : 1u); pass++) {
    uint32_t trow = 0;   // the activation row (and output row) of this pass
    if constexpr (MODE == GATHER_CSR) trow = pass < r_n1 ? r_lo + pass : r_lo2 + (pass - r_n1);
    if constexpr (MODE == GATHER_INDICES) {
        unsigned long long m = r_mask;
        for (uint32_t i = 0; i < pass; i++) m &= m - 1ull;
        trow = (uint32_t)__ffsll((long long)m) - 1u;
    }

    // ---- loads, smallest first ----------------------------------------------
    const size_t sb0 = (slab_rows + rb) * a.gpr;
    const uint32_t n_sb = rows_here * a.gpr;
    sbvec_t sraw[SBI], braw[SBI];
    {
        const sbvec_t* sp = (const sbvec_t*)((const elem_t*)Sm + sb0);
        const sbvec_t* bp = (const sbvec_t*)((const elem_t*)Bm + sb0);
        const uint32_t last = n_sb / 4 - 1;
#pragma unroll
        for (int j = 0; j < SBI; j++) {
            const uint32_t v = min(tid + j * TPB, last);
            sraw[j] = sp[v];
            braw[j] = bp[v];
        }
    }
    MTQ_KEEP_LOAD_ORDER();
    XS xs[MB];
    uint4 xraw[MB][XS::NRAW];
    uint4 yraw[GATED ? CPC / 4 : 1];
    if constexpr (GATED) {
        const uint4* yp = (const uint4*)((const float*)a.x + k0);
#pragma unroll
        for (int i = 0; i < CPC / 4; i++) yraw[i] = yp[i];
        if constexpr (NORM == 3) xraw[0][0] = ((const uint4*)((const uint16_t*)a.gate_z + k0))[rsub];   // this row slot's quarter
        else xs[0].load_raw(a.gate_z, k0, xraw[0]);
    } else {
#pragma unroll
        for (int mb = 0; mb < MBR; mb++) {
            const uint32_t t = ROUTED ? trow : (mb < (int)a.M ? mb : 0);
            xs[mb].load_raw(a.x, (size_t)t * a.K + k0, xraw[mb]);
        }
    }
    uint4 nraw[NORM ? XS::NRAW : 1];
    float eps = 0.f;
    if constexpr (NORM) {
        // issued ahead of the weight stream: loads return in order, so a late load of eps
        // would wait for the whole first ring
        eps = a.eps[0];
        if constexpr (NORM == 3) nraw[0] = ((const uint4*)((const uint16_t*)a.norm_w + k0 % a.dv))[rsub];
        else xs[0].load_raw(a.norm_w, NORM == 2 ? k0 % a.dv : k0, nraw);
    }
    MTQ_KEEP_LOAD_ORDER();
    u32x4 ring[D];
#pragma unroll
    for (int d = 0; d < D; d++) {
        const uint32_t rl = min(d * a.rps + rsub, rows_here - 1);
        ring[d] = __builtin_nontemporal_load(wbase + (size_t)rl * a.C);
    }
    MTQ_KEEP_LOAD_ORDER();

    // ---- stage (s, b - MAGIC*s) pairs of the whole row range in LDS ----------
#pragma unroll
    for (int j = 0; j < SBI; j++) {
        const uint32_t v = tid + j * TPB;
        float sv[4], bv[4];
        SbVec<DT>::unpack(sraw[j], sv);
        SbVec<DT>::unpack(braw[j], bv);
        if (v * 4 < n_sb) {
            float4* dst = (float4*)(sb + v * 4);
            dst[0] = make_float4(sv[0], bv[0] - MAGIC * sv[0], sv[1], bv[1] - MAGIC * sv[1]);
            dst[1] = make_float4(sv[2], bv[2] - MAGIC * sv[2], sv[3], bv[3] - MAGIC * sv[3]);
        }
    }
    uint4* gx = (uint4*)(((uintptr_t)(ssq_part + 16) + 15) & ~(uintptr_t)15);   // NORM = 3: [C][4] value vectors, then [C][4] remainders
    if constexpr (NORM == 3) {
        float ssq = 0.f;
#pragma unroll
        for (int i = 0; i < CPC / 4; i++) ssq += raw_sumsq<DT_F32>(yraw[i]);
        ssq = seg_allreduce(ssq, (int)(a.dv / CPC));
        const float inv = 1.0f / sqrtf(ssq / (float)a.dv + eps);
        // this row slot's two vectors of y, loaded again (picking them out of yraw by rsub is an indexed read of a
        // register array, which goes through scratch memory)
        uint4 yq[2];
        {
            const uint4* yp = (const uint4*)((const float*)a.x + k0) + 2u * rsub;
            yq[0] = yp[0];
            yq[1] = yp[1];
        }
        uint4 hi, lo;
        raw_gated<DT>(yq, xraw[0][0], nraw[0], inv, hi, lo);
        gx[c * 4u + rsub] = hi;
        gx[(a.C + c) * 4u + rsub] = lo;
    }
    if constexpr (NORM == 2) {
        float ssq = 0.f;
#pragma unroll
        for (int i = 0; i < CPC / 4; i++) ssq += raw_sumsq<DT_F32>(yraw[i]);
        ssq = seg_allreduce(ssq, (int)(a.dv / CPC));
        const float inv = 1.0f / sqrtf(ssq / (float)a.dv + eps);
        constexpr int YPV = (CPC / 4) / XS::NRAW;   // y vectors per vector of the element type
#pragma unroll
        for (int i = 0; i < XS::NRAW; i++) {
            uint4 hi, lo;
            raw_gated<DT>(&yraw[i * YPV], xraw[0][i], nraw[i], inv, hi, lo);
            xraw[0][i] = hi;
            if constexpr (MB == 2) xraw[1][i] = lo;
        }
    }
    if constexpr (NORM == 1) {
        // threads of the first row slot hold the whole activation row between them
        float ssq = 0.f;
        if (rsub == 0) {
#pragma unroll
            for (int i = 0; i < XS::NRAW; i++) ssq += raw_sumsq<DT>(xraw[0][i]);
        }
        ssq = seg_allreduce(ssq, 64);
        if (lane == 0) ssq_part[tid >> 6] = ssq;
    }
    __syncthreads();
    if constexpr (NORM == 3) {
#pragma unroll
        for (int i = 0; i < XS::NRAW; i++) {
            xraw[0][i] = gx[c * 4u + i];
            xraw[1][i] = gx[(a.C + c) * 4u + i];
        }
    }
    if constexpr (NORM == 1) {
        float tot = 0.f;
        for (uint32_t wv = 0; wv < (TPB >> 6); wv++) tot += ssq_part[wv];
        const float inv = 1.0f / sqrtf(tot / (float)a.K + eps);
#pragma unroll
        for (int i = 0; i < XS::NRAW; i++) {
            uint4 hi, lo;
            raw_normed<DT>(xraw[0][i], nraw[i], inv, hi, lo);
            xraw[0][i] = hi;
            if constexpr (MB == 2) xraw[1][i] = lo;
        }
    }
#pragma unroll
    for (int mb = 0; mb < MB; mb++) xs[mb].prepare(xraw[mb]);

    const uint32_t g0 = k0 >> a.log2g;
    const uint32_t g1 = (k0 + CPC / 2) >> a.log2g;
    const uint32_t wir = c >> 6;
    // which ring slot's total this lane holds after wave_reduce4
    const uint32_t my_slot = ((lane >> 4) & 1u) * 2u + (lane >> 5);

    auto batch = [&](uint32_t b, auto issue_next) {
        float acc[D][MB];
#pragma unroll
        for (int d = 0; d < D; d++) {
            const uint32_t j = b * D + d;
            const uint32_t rl = min(j * a.rps + rsub, rows_here - 1);
            const float2 p0 = sb[rl * a.gpr + g0];
            const float2 p1 = sb[rl * a.gpr + g1];
            const u32x4 wv = ring[d];
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                float d01 = xs[mb].dot_dword(wv.x, 0, 0.f);
                d01 = xs[mb].dot_dword(wv.y, 1, d01);
                float d23 = xs[mb].dot_dword(wv.z, 2, 0.f);
                d23 = xs[mb].dot_dword(wv.w, 3, d23);
                float v = p0.x * d01 + p0.y * xs[mb].xsum[0];
                v += p1.x * d23 + p1.y * xs[mb].xsum[1];
                acc[d][mb] = v;
            }
            if constexpr (NORM != 0 && MB == 2) acc[d][0] += acc[d][1] * (1.0f / RemSplit<DT>::kRemScale);
            if constexpr (decltype(issue_next)::value) {
                const uint32_t rn = min((j + D) * a.rps + rsub, rows_here - 1);
                ring[d] = __builtin_nontemporal_load(wbase + (size_t)rn * a.C);
                // (kept where it is written: left to itself the scheduler gathers a batch's reloads behind its last
                // slot, and the ring is then empty once per batch; 8192 x 8192 8-bit 12.9 -> 12.55 us, 57344 x 4096 22.7 -> 22.0)
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // reduce D rows x MB values; lane (16*r) of each wave writes slot {0,2,1,3}[r]
#pragma unroll
        for (int h = 0; h < D / 4; h++) {
#pragma unroll
            for (int mb = 0; mb < MBR; mb++) {
                const float tot = wave_reduce4(acc[4 * h + 0][mb], acc[4 * h + 1][mb], acc[4 * h + 2][mb],
                                               acc[4 * h + 3][mb]);
                if ((lane & 15u) == 0) {
                    const uint32_t j = b * D + 4 * h + my_slot;
                    const uint32_t rl = j * a.rps + rsub;
                    if (rl < rows_here) part[(rl * MBR + mb) * a.wpr + wir] = tot;
                }
            }
        }
    };

    for (uint32_t b = 0; b + 1 < a.nb; b++) batch(b, std::true_type{});
    batch(a.nb - 1, std::false_type{});

    __syncthreads();
    for (uint32_t o = tid; o < rows_here * MBR; o += TPB) {
        const uint32_t rl = o / MBR, mb = o % MBR;
        if (mb >= a.M) continue;
        float sum = 0.f;
        for (uint32_t wi = 0; wi < a.wpr; wi++) sum += part[o * a.wpr + wi];
        store_elem<DT>(Om, (size_t)(ROUTED ? trow : mb) * Nm + rb + rl, sum);
    }
    if (ROUTED && pass + 1 < n_pass) __syncthreads();   // the next row stages into the same LDS
    }   // pass
}

// ---------------------------------------------------------------------------
// per-dtype launch switch (instantiated once per dtype)
// ---------------------------------------------------------------------------

template <int DT, int BITS, int MB, int RT, int MODE, int MAXT, int SBI>
static int qmv_launch_inst(QmvKArgs& a, const QmvGeom& g, const LaunchCtx& lc) {
    auto fn = qmv_kernel<DT, BITS, MB, RT, MODE, MAXT, SBI>;
    if (g.shmem > 48 * 1024) {
        hipError_t e = set_max_dynamic_lds((const void*)fn, (size_t)g.shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel((const void*)fn, g.grid, dim3(g.tpb), args, g.shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "qmv kernel launch");
    return ERR_OK;
}

template <int DT, int BITS, int MB, int RT, int MODE, int MAXT>
static int qmv_launch_sbi(QmvKArgs& a, const QmvGeom& g, const LaunchCtx& lc) {
    switch (g.sbi) {
        case 1: return qmv_launch_inst<DT, BITS, MB, RT, MODE, MAXT, 1>(a, g, lc);
        case 2: return qmv_launch_inst<DT, BITS, MB, RT, MODE, MAXT, 2>(a, g, lc);
        case 4: return qmv_launch_inst<DT, BITS, MB, RT, MODE, MAXT, 4>(a, g, lc);
        default: return qmv_launch_inst<DT, BITS, MB, RT, MODE, MAXT, 0>(a, g, lc);
    }
}

// (MB, RT, MAXT) combinations the host may ask for; see qmv_pick_geometry.
template <int DT, int BITS>
static int qmv_launch_bits(QmvKArgs& a, int mode, const QmvGeom& g, const LaunchCtx& lc) {
    switch (mode) {
        case GATHER_NONE:
            if (g.mb == 1 && g.rt == 8) return qmv_launch_sbi<DT, BITS, 1, 8, GATHER_NONE, 1024>(a, g, lc);
            if (g.mb == 1 && g.rt == 7) return qmv_launch_sbi<DT, BITS, 1, 7, GATHER_NONE, 1024>(a, g, lc);
            if (g.mb == 1 && g.rt == 4) return qmv_launch_sbi<DT, BITS, 1, 4, GATHER_NONE, 1024>(a, g, lc);
            if (g.mb == 2 && g.rt == 8) return qmv_launch_sbi<DT, BITS, 2, 8, GATHER_NONE, 512>(a, g, lc);
            if (g.mb == 3 && g.rt == 4) return qmv_launch_sbi<DT, BITS, 3, 4, GATHER_NONE, 512>(a, g, lc);
            if (g.mb == 4 && g.rt == 4) return qmv_launch_sbi<DT, BITS, 4, 4, GATHER_NONE, 512>(a, g, lc);
            break;
        case GATHER_CSR:
            if (g.mb == 4 && g.rt == 4) return qmv_launch_sbi<DT, BITS, 4, 4, GATHER_CSR, 512>(a, g, lc);
            break;
        case GATHER_INDICES:
            if (g.mb == 4 && g.rt == 4) return qmv_launch_sbi<DT, BITS, 4, 4, GATHER_INDICES, 512>(a, g, lc);
            break;
        case GATHER_SINGLE:
            if (g.mb == 1 && g.rt == 8) return qmv_launch_sbi<DT, BITS, 1, 8, GATHER_SINGLE, 1024>(a, g, lc);
            break;
    }
    return fail(ERR_UNSUPPORTED, "fast qmv: no kernel instance for this geometry");
}

struct QmvSGeom {
    int mb;     // 1..4
    int d;      // ring depth: 4 or 8
    int sbi;    // 1, 2 or 4
    uint32_t tpb;
    size_t shmem;
    dim3 grid;
};

template <int DT, int BITS, int MB, int D, int MODE, int MAXT>
static int qmv_stream_launch_sbi(QmvSArgs& a, const QmvSGeom& g, const LaunchCtx& lc) {
    const void* fn;
    switch (g.sbi) {
        case 1: fn = (const void*)qmv_stream_kernel<DT, BITS, MB, D, MODE, MAXT, 1>; break;
        case 2: fn = (const void*)qmv_stream_kernel<DT, BITS, MB, D, MODE, MAXT, 2>; break;
        default: fn = (const void*)qmv_stream_kernel<DT, BITS, MB, D, MODE, MAXT, 4>; break;
    }
    if (g.shmem > 48 * 1024) {
        hipError_t e = set_max_dynamic_lds(fn, (size_t)g.shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, g.grid, dim3(g.tpb), args, g.shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "qmv stream kernel launch");
    return ERR_OK;
}

// Fused-RMSNorm instances: one activation row, 4- or 8-bit codes (NORMK = 1); the gated form, 4-bit codes (NORMK = 2).
template <int DT, int BITS, int D, int NORMK = 1, int MAXT = 1024>
static int qmv_stream_norm_launch_d(QmvSArgs& a, const QmvSGeom& g, const LaunchCtx& lc) {
    constexpr int MBN = DT == DT_F32 ? 1 : 2;  // 16-bit types carry the normalised row as value + remainder
    const void* fn;
    switch (g.sbi) {
        case 1: fn = (const void*)qmv_stream_kernel<DT, BITS, MBN, D, GATHER_NONE, MAXT, 1, NORMK>; break;
        case 2: fn = (const void*)qmv_stream_kernel<DT, BITS, MBN, D, GATHER_NONE, MAXT, 2, NORMK>; break;
        default: fn = (const void*)qmv_stream_kernel<DT, BITS, MBN, D, GATHER_NONE, MAXT, 4, NORMK>; break;
    }
    if (g.shmem > 48 * 1024) {
        hipError_t e = set_max_dynamic_lds(fn, (size_t)g.shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, g.grid, dim3(g.tpb), args, g.shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "norm + qmv stream kernel launch");
    return ERR_OK;
}

template <int DT> int qmv_stream_norm_launch_dtype(QmvSArgs& a, int bits, const QmvSGeom& g, const LaunchCtx& lc) {
    if (g.mb != 1 || g.d != 4) return fail(ERR_UNSUPPORTED, "norm + qmv: no kernel instance for this geometry");
    if (a.gate_z) {
        if (bits != 4 || g.d != 4) return fail(ERR_UNSUPPORTED, "gated norm + qmv: 4-bit codes, ring of four");
        if constexpr (DT != DT_F32) {
            if (a.rps == 4) return qmv_stream_norm_launch_d<DT, 4, 4, 3, 512>(a, g, lc);   // the gate dealt over the four row slots
        }
        // (workgroups of at most 512 threads: with the register budget of 1024 the gate's 32 values spill)
        if (g.tpb > 512) return fail(ERR_UNSUPPORTED, "gated norm + qmv: rows of at most 16384 values");
        return qmv_stream_norm_launch_d<DT, 4, 4, 2, 512>(a, g, lc);
    }
    if (bits == 4) return qmv_stream_norm_launch_d<DT, 4, 4>(a, g, lc);   // (the host plans the norm on the ring of four only)
    if (bits == 8) return qmv_stream_norm_launch_d<DT, 8, 4>(a, g, lc);
    return fail(ERR_UNSUPPORTED, "norm + qmv: 4- or 8-bit codes");
}

template <int DT, int BITS, int MODE>
static int qmv_stream_launch_mode(QmvSArgs& a, const QmvSGeom& g, const LaunchCtx& lc) {
    if (g.d == 4) {
        if (g.mb == 1) return qmv_stream_launch_sbi<DT, BITS, 1, 4, MODE, 1024>(a, g, lc);
        if constexpr (MODE == GATHER_NONE) {
            switch (g.mb) {
                case 2: return qmv_stream_launch_sbi<DT, BITS, 2, 4, MODE, 512>(a, g, lc);
                case 3: return qmv_stream_launch_sbi<DT, BITS, 3, 4, MODE, 512>(a, g, lc);
                case 4: return qmv_stream_launch_sbi<DT, BITS, 4, 4, MODE, 512>(a, g, lc);
            }
        }
    } else if (g.d == 8 && g.mb == 1) {
        // (routed rows keep the ring of four: with eight loads in flight their instances spill)
        if constexpr (MODE != GATHER_CSR && MODE != GATHER_INDICES) return qmv_stream_launch_sbi<DT, BITS, 1, 8, MODE, 1024>(a, g, lc);
    }
    return fail(ERR_UNSUPPORTED, "stream qmv: no kernel instance for this geometry");
}

template <int DT> int qmv_stream_launch_dtype(QmvSArgs& a, int bits, int mode, const QmvSGeom& g, const LaunchCtx& lc) {
    if (mode == GATHER_NONE) {
        switch (bits) {
            case 2: return qmv_stream_launch_mode<DT, 2, GATHER_NONE>(a, g, lc);
            case 4: return qmv_stream_launch_mode<DT, 4, GATHER_NONE>(a, g, lc);
            default: return qmv_stream_launch_mode<DT, 8, GATHER_NONE>(a, g, lc);
        }
    }
    if (g.mb != 1) return fail(ERR_UNSUPPORTED, "stream qmv: the expert modes take one row at a time");
    if (mode == GATHER_CSR || mode == GATHER_INDICES) {   // (4-bit codes: the width mixture-of-experts weights come in)
        if (bits != 4) return fail(ERR_UNSUPPORTED, "stream qmv: routed rows take 4-bit codes");
        return mode == GATHER_CSR ? qmv_stream_launch_mode<DT, 4, GATHER_CSR>(a, g, lc) : qmv_stream_launch_mode<DT, 4, GATHER_INDICES>(a, g, lc);
    }
    switch (bits) {
        case 2: return qmv_stream_launch_mode<DT, 2, GATHER_SINGLE>(a, g, lc);
        case 4: return qmv_stream_launch_mode<DT, 4, GATHER_SINGLE>(a, g, lc);
        default: return qmv_stream_launch_mode<DT, 8, GATHER_SINGLE>(a, g, lc);
    }
}

template <int DT> int qmv_launch_dtype(QmvKArgs& a, int bits, int mode, const QmvGeom& g, const LaunchCtx& lc) {
    switch (bits) {
        case 2: return qmv_launch_bits<DT, 2>(a, mode, g, lc);
        case 4: return qmv_launch_bits<DT, 4>(a, mode, g, lc);
        default: return qmv_launch_bits<DT, 8>(a, mode, g, lc);
    }
}

}  // namespace mtq
