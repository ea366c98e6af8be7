// qmv / small-batch qmm / gather_qmv for gfx950: one kernel family.
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
// position c = t % C for its whole life: it issues RT independent 128-bit
// non-temporal loads (rows rsub + i*rps, rsub = t / C) before doing anything
// else, loads its CPC activations once into registers, and then owns exactly
// one chunk of every row it visits. Scales and biases of the tile are staged
// through LDS as (s, b - MAGIC*s) float pairs while the weight loads fly.
// Per-row sums are reduced across the C lanes of a row with DPP/permute
// butterflies inside each wave and a tiny LDS exchange across waves.
//
// Gather modes run the same tile against several activation rows: blockIdx.y
// is the expert; the workgroup finds the rows routed to that expert, exits at
// once if there are none (so only experts that are hit are streamed from
// HBM), keeps its weight tile in registers and walks the rows MB at a time.
#include "mtq_device.h"
#include "mtq_internal.h"

namespace mtq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

template <int DT, int BITS, int MB, int RT, int MODE, int MAXT>
__global__ __launch_bounds__(MAXT) void qmv_kernel(QmvKArgs a) {
    typedef XSlice<DT, BITS> XS;
    constexpr int CPC = XS::CPC;
    constexpr float MAGIC = PathSel<DT, BITS>::kMagic;

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
        uint32_t mx = 0, l = 0;
        for (uint32_t j = 1; j <= a.E; j++) {
            uint32_t o = a.route[j];
            if (j <= expert) l = max(l, o);
            mx = max(mx, o);
        }
        uint32_t hi = min(a.route[expert + 1], a.T);
        lo = l;
        n1 = hi > lo ? hi - lo : 0;
        lo2 = min(mx, a.T);
        uint32_t n2 = expert == 0 ? a.T - lo2 : 0;
        cnt = n1 + n2;
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

    const size_t slab_rows = (size_t)expert * a.N;  // row offset of this expert's slab
    const u32x4* wbase = a.w + slab_rows * a.C;

    // ---- weight loads first: RT independent 128-bit streams per thread ------
    u32x4 wv[RT];
#pragma unroll
    for (int i = 0; i < RT; i++) {
        uint32_t row = row0 + i * a.rps + rsub;
        if (row < a.N) wv[i] = __builtin_nontemporal_load(wbase + (size_t)row * a.C + c);
        else wv[i] = (u32x4)(0u);
    }

    // ---- stage the tile's scales / biases in LDS ----------------------------
    const uint32_t rows_in_tile = min(R, a.N - row0);
    {
        const size_t sb0 = (slab_rows + row0) * a.gpr;
        const uint32_t n_sb = rows_in_tile * a.gpr;
        for (uint32_t i = tid; i < n_sb; i += TPB) {
            float s = load_elem<DT>(a.scales, sb0 + i);
            float b = load_elem<DT>(a.biases, sb0 + i);
            sb[i] = make_float2(s, b - MAGIC * s);
        }
    }
    __syncthreads();

    const uint32_t k0 = c * CPC;
    const uint32_t g0 = k0 >> a.log2g;
    const uint32_t g1 = (k0 + CPC / 2) >> a.log2g;  // == g0 unless a chunk spans two groups
    const int seg = a.C >= 64 ? 64 : (int)a.C;

    // Plain and single-expert launches carry at most MB rows: exactly one batch.
    constexpr bool kOneBatch = MODE == GATHER_NONE || MODE == GATHER_SINGLE;
    const uint32_t n_batches = kOneBatch ? 1u : (cnt + MB - 1) / MB;
    for (uint32_t bi = 0; bi < n_batches; bi++) {
        const uint32_t base = bi * MB;
        // activation rows of this batch
        uint32_t xrow[MB];
        XS xs[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            uint32_t j = base + mb;
            uint32_t t = 0xFFFFFFFFu;
            if (j < cnt) {
                if constexpr (MODE == GATHER_CSR) t = j < n1 ? lo + j : lo2 + (j - n1);
                else if constexpr (MODE == GATHER_INDICES) t = rowlist[j];
                else t = j;
            }
            xrow[mb] = t;
            if (t != 0xFFFFFFFFu) xs[mb].load(a.x, (size_t)t * a.K + k0);
            else xs[mb].zero();
        }

        float acc[RT][MB];
#pragma unroll
        for (int i = 0; i < RT; i++) {
            const uint32_t rl = i * a.rps + rsub;
            float2 p0 = make_float2(0.f, 0.f), p1 = p0;
            if (rl < rows_in_tile) {
                p0 = sb[rl * a.gpr + g0];
                p1 = sb[rl * a.gpr + g1];
            }
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
                    uint32_t row = row0 + i * a.rps + rsub;
#pragma unroll
                    for (int mb = 0; mb < MB; mb++)
                        if (row < a.N && xrow[mb] != 0xFFFFFFFFu)
                            store_elem<DT>(a.out, (size_t)xrow[mb] * a.N + row, acc[i][mb]);
                }
            }
        } else {
            if (base) __syncthreads();  // previous batch's readers are done with `part`
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
                uint32_t j = base + mb;
                if (j >= cnt) continue;
                uint32_t t;
                if constexpr (MODE == GATHER_CSR) t = j < n1 ? lo + j : lo2 + (j - n1);
                else if constexpr (MODE == GATHER_INDICES) t = rowlist[j];
                else t = j;
                float s = 0.f;
                for (uint32_t wi = 0; wi < a.wpr; wi++) s += part[o * a.wpr + wi];
                store_elem<DT>(a.out, (size_t)t * a.N + row0 + rl, s);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

static bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }
static uint32_t ilog2(uint32_t v) { uint32_t l = 0; while ((1u << l) < v) l++; return l; }

template <int DT, int BITS, int MB, int RT, int MODE, int MAXT>
static int launch_inst(QmvKArgs& a, dim3 grid, uint32_t tpb, size_t shmem, const LaunchCtx& lc) {
    auto fn = qmv_kernel<DT, BITS, MB, RT, MODE, MAXT>;
    if (shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel((const void*)fn, grid, dim3(tpb), args, shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "qmv kernel launch");
    return ERR_OK;
}

template <int DT, int BITS, int MODE>
static int launch_mode(QmvKArgs& a, int mb, dim3 grid, uint32_t tpb, size_t shmem,
                       const LaunchCtx& lc) {
    if constexpr (MODE == GATHER_NONE) {
        switch (mb) {
            case 1: return launch_inst<DT, BITS, 1, 8, MODE, 1024>(a, grid, tpb, shmem, lc);
            case 2: return launch_inst<DT, BITS, 2, 8, MODE, 512>(a, grid, tpb, shmem, lc);
            case 3: return launch_inst<DT, BITS, 3, 4, MODE, 512>(a, grid, tpb, shmem, lc);
            default: return launch_inst<DT, BITS, 4, 4, MODE, 512>(a, grid, tpb, shmem, lc);
        }
    } else if constexpr (MODE == GATHER_SINGLE) {
        return launch_inst<DT, BITS, 1, 8, MODE, 1024>(a, grid, tpb, shmem, lc);
    } else {
        return launch_inst<DT, BITS, 4, 4, MODE, 512>(a, grid, tpb, shmem, lc);
    }
}

template <int DT, int BITS>
static int launch_bits(QmvKArgs& a, int mode, int mb, dim3 grid, uint32_t tpb, size_t shmem,
                       const LaunchCtx& lc) {
    switch (mode) {
        case GATHER_NONE: return launch_mode<DT, BITS, GATHER_NONE>(a, mb, grid, tpb, shmem, lc);
        case GATHER_CSR: return launch_mode<DT, BITS, GATHER_CSR>(a, mb, grid, tpb, shmem, lc);
        case GATHER_INDICES: return launch_mode<DT, BITS, GATHER_INDICES>(a, mb, grid, tpb, shmem, lc);
        default: return launch_mode<DT, BITS, GATHER_SINGLE>(a, mb, grid, tpb, shmem, lc);
    }
}

template <int DT>
static int launch_dt(QmvKArgs& a, int bits, int mode, int mb, dim3 grid, uint32_t tpb, size_t shmem,
                     const LaunchCtx& lc) {
    switch (bits) {
        case 2: return launch_bits<DT, 2>(a, mode, mb, grid, tpb, shmem, lc);
        case 4: return launch_bits<DT, 4>(a, mode, mb, grid, tpb, shmem, lc);
        default: return launch_bits<DT, 8>(a, mode, mb, grid, tpb, shmem, lc);
    }
}

int launch_qmv_fast(const QmvParams& p, const LaunchCtx& lc) {
    if (p.bits != 2 && p.bits != 4 && p.bits != 8)
        return fail(ERR_UNSUPPORTED, "fast qmv: bits must be 2, 4 or 8");
    const uint32_t cpc = 128u / (uint32_t)p.bits;
    if (p.K == 0 || p.N == 0 || p.K % cpc) return fail(ERR_UNSUPPORTED, "fast qmv: K*bits % 128 != 0");
    const uint32_t G = p.group_size;
    if (!is_pow2(G) || G * 2 < cpc || p.K % G) return fail(ERR_UNSUPPORTED, "fast qmv: group size");
    const uint32_t C = p.K / cpc;
    const bool gather = p.gather == GATHER_CSR || p.gather == GATHER_INDICES;
    const uint32_t rows = gather ? p.T : (p.gather == GATHER_SINGLE ? 1u : p.M);
    if (rows == 0) return ERR_OK;  // nothing to compute
    const uint32_t maxt = (gather || rows > 1) ? 512u : 1024u;
    if (C > maxt) return fail(ERR_UNSUPPORTED, "fast qmv: row too long for one workgroup");
    if (!(C % 64 == 0 || (C < 64 && is_pow2(C)))) return fail(ERR_UNSUPPORTED, "fast qmv: chunk count");
    // threads per workgroup: a whole number of rows per step, >= 256 threads when possible
    uint32_t rps = 1;
    while (C * rps < 256 && C * rps * 2 <= maxt) rps *= 2;
    const uint32_t tpb = C * rps;
    if (tpb % 64) return fail(ERR_UNSUPPORTED, "fast qmv: workgroup not a whole number of waves");

    if (!gather && p.gather != GATHER_SINGLE && rows > 4) {
        // more activation rows than one pass holds: run passes of up to 4 rows
        const size_t esz = p.dtype == DT_F32 ? 4 : 2;
        for (uint32_t m0 = 0; m0 < rows; m0 += 4) {
            QmvParams q = p;
            q.M = rows - m0 < 4 ? rows - m0 : 4;
            q.x = (const char*)p.x + (size_t)m0 * p.K * esz;
            q.out = (char*)p.out + (size_t)m0 * p.N * esz;
            LaunchCtx l2 = lc;
            if (m0) l2.start = nullptr;
            if (m0 + 4 < rows) l2.stop = nullptr;
            int rc = launch_qmv_fast(q, l2);
            if (rc) return rc;
        }
        return ERR_OK;
    }

    const int mb = gather ? 4 : (int)rows;
    const int rt = (p.gather == GATHER_NONE && mb <= 2) || p.gather == GATHER_SINGLE ? 8 : 4;
    const uint32_t R = (uint32_t)rt * rps;

    QmvKArgs a;
    a.w = (const u32x4*)p.w;
    a.scales = p.scales;
    a.biases = p.biases;
    a.x = p.x;
    a.out = p.out;
    a.route = p.route;
    a.M = rows;
    a.N = p.N;
    a.K = p.K;
    a.C = C;
    a.log2g = ilog2(G);
    a.rps = rps;
    a.T = p.T;
    a.E = p.E;
    a.gpr = p.K / G;
    a.lds_sb_pairs = R * a.gpr;
    a.wpr = C >= 64 ? C / 64 : 0;
    a.list_cap = p.gather == GATHER_INDICES ? p.T : 0;
    const size_t shmem = (size_t)a.lds_sb_pairs * 8 + (size_t)R * 4 * (a.wpr ? a.wpr : 1) * 4 +
                         (size_t)a.list_cap * 4;
    if (shmem > 64 * 1024) return fail(ERR_UNSUPPORTED, "fast qmv: tile does not fit in LDS");

    dim3 grid((p.N + R - 1) / R, gather ? p.E : 1, 1);
    switch (p.dtype) {
        case DT_F32: return launch_dt<DT_F32>(a, p.bits, p.gather, mb, grid, tpb, shmem, lc);
        case DT_F16: return launch_dt<DT_F16>(a, p.bits, p.gather, mb, grid, tpb, shmem, lc);
        case DT_BF16: return launch_dt<DT_BF16>(a, p.bits, p.gather, mb, grid, tpb, shmem, lc);
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
}

}  // namespace mtq
