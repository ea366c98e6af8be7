// Host side of the qmv / gather_qmv kernel family: checks that a request fits
// the tiled kernel's geometry, picks the launch shape and calls the per-dtype
// instantiation (qmv_impl.h). Requests that do not fit return ERR_UNSUPPORTED
// so the caller falls back to the generic kernel.
#include "qmv_impl.h"

namespace mtq {

extern template int qmv_launch_dtype<DT_F32>(QmvKArgs&, int, int, const QmvGeom&, const LaunchCtx&);
extern template int qmv_launch_dtype<DT_F16>(QmvKArgs&, int, int, const QmvGeom&, const LaunchCtx&);
extern template int qmv_launch_dtype<DT_BF16>(QmvKArgs&, int, int, const QmvGeom&, const LaunchCtx&);
extern template int qmv_stream_launch_dtype<DT_F32>(QmvSArgs&, int, int, const QmvSGeom&, const LaunchCtx&);
extern template int qmv_stream_launch_dtype<DT_F16>(QmvSArgs&, int, int, const QmvSGeom&, const LaunchCtx&);
extern template int qmv_stream_launch_dtype<DT_BF16>(QmvSArgs&, int, int, const QmvSGeom&, const LaunchCtx&);
extern template int qmv_stream_norm_launch_dtype<DT_F32>(QmvSArgs&, int, const QmvSGeom&, const LaunchCtx&);
extern template int qmv_stream_norm_launch_dtype<DT_F16>(QmvSArgs&, int, const QmvSGeom&, const LaunchCtx&);
extern template int qmv_stream_norm_launch_dtype<DT_BF16>(QmvSArgs&, int, const QmvSGeom&, const LaunchCtx&);

static bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }
static uint32_t ilog2(uint32_t v) { uint32_t l = 0; while ((1u << l) < v) l++; return l; }

static int g_num_cus = 0;
static int num_cus() {
    if (g_num_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_num_cus = n;
        else
            g_num_cus = 256;
    }
    return g_num_cus;
}

// Streaming kernel: picks ring depth D, batches per thread nb and the grid so
// that every workgroup gets the same contiguous range of D*nb*rps rows, the
// workgroup count is a whole multiple of the CU count where the shape allows,
// and at least two batches are pipelined. Returns ERR_UNSUPPORTED when the
// shape is better served by the one-shot kernel.
static int launch_qmv_stream(const QmvParams& p, uint32_t C, uint32_t rps, uint32_t tpb, uint32_t rows,
                             const LaunchCtx& lc, const QmvBatch* batch = nullptr,
                             const void* norm_w = nullptr, const float* eps = nullptr, const void* gate_z = nullptr,
                             uint32_t dv = 0) {
    const uint32_t G = p.group_size, gpr = p.K / G;
    if (C % 64 || gpr % 4 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)
        return fail(ERR_UNSUPPORTED, "stream qmv: geometry");
    const uint32_t cus = (uint32_t)num_cus();
    const Options& opt = options();
    double best = 1e30;
    uint32_t best_d = 0, best_nb = 0;
    const bool routed_rows = p.gather == GATHER_CSR || p.gather == GATHER_INDICES;
    for (uint32_t d : {4u, 8u}) {
        if (d == 8 && (rows != 1 || routed_rows)) continue;
        if (opt.qmv_stream_depth && (uint32_t)opt.qmv_stream_depth != d) continue;
        for (uint32_t nb = 1; nb <= 16; nb++) {
            if (opt.qmv_stream_batches && (uint32_t)opt.qmv_stream_batches != nb) continue;
            const uint32_t rpw = d * nb * rps;
            if (rpw > p.N + d * rps) break;
            uint32_t grid = (p.N + rpw - 1) / rpw;
            if (batch) {  // workgroups that do work, over all matrices
                grid = 0;
                for (int j = 0; j < batch->n; j++) grid += (batch->N[j] + rpw - 1) / rpw;
            }
            const uint64_t vecs = (uint64_t)rpw * gpr / 4;
            if ((vecs + tpb - 1) / tpb > 4) break;
            const size_t lds = (size_t)rpw * gpr * 8 + (size_t)rpw * rows * (C / 64) * 4;
            if (lds > 64 * 1024) break;
            uint64_t n_all = p.N;
            if (batch) {
                n_all = 0;
                for (int j = 0; j < batch->n; j++) n_all += batch->N[j];
            }
            const double waste = (double)((uint64_t)grid * rpw - n_all) / n_all;
            const uint32_t rounds = (grid + cus - 1) / cus;
            const double idle = (double)(rounds * cus - grid) / (rounds * cus);
            const double waves_per_cu = (double)grid / cus * (tpb / 64);
            double score = waste + idle;
            if (waves_per_cu < 8.0) score += (8.0 - waves_per_cu) * 0.04;
            if (waves_per_cu > 32.0) score += (waves_per_cu - 32.0) * 0.02;
            // Measured on the 14336x4096 / 4096x14336 shapes: small workgroups do
            // best one batch deep (more, shorter-lived workgroups), wide ones two.
            if (nb == 1) score += tpb > 256 ? 0.15 : -0.05;
            if (norm_w) {
                // Every workgroup repeats the normalisation of the row, which costs about as
                // much vector work as 8 weight rows per thread: take the longest workgroups
                // that still leave 7 waves per CU (measured on 14336x4096, 4096x14336, 4096x4096).
                if (d != 4) continue;
                score = waste + (waves_per_cu >= 7.0 ? 1.0 / nb : 10.0 + (7.0 - waves_per_cu));
            }
            if (score < best) { best = score; best_d = d; best_nb = nb; }
        }
    }
    if (!best_d) return fail(ERR_UNSUPPORTED, "stream qmv: no geometry");

    QmvSArgs a;
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
    a.gpr = gpr;
    a.wpr = C / 64;
    a.rows_per_wg = best_d * best_nb * rps;
    a.nb = best_nb;
    a.E = p.E;
    a.T = p.T;
    a.norm_w = norm_w;
    a.eps = eps;
    a.gate_z = gate_z;
    a.dv = dv;
    a.nmat = 0;
    if (batch) {
        a.nmat = (uint32_t)batch->n;
        for (int j = 0; j < 4; j++) {
            const int k = j < batch->n ? j : 0;  // unused slots repeat matrix 0
            a.mw[j] = batch->w[k];
            a.ms[j] = batch->scales[k];
            a.mbias[j] = batch->biases[k];
            a.mo[j] = batch->out[k];
            a.mn[j] = batch->N[k];
        }
    }
    QmvSGeom g;
    g.mb = (int)rows;
    g.d = (int)best_d;
    const uint64_t vecs = (uint64_t)a.rows_per_wg * gpr / 4;
    const uint64_t per_thread = (vecs + tpb - 1) / tpb;
    g.sbi = per_thread <= 1 ? 1 : per_thread <= 2 ? 2 : 4;
    g.tpb = tpb;
    g.shmem = (size_t)a.rows_per_wg * gpr * 8 + (size_t)a.rows_per_wg * rows * a.wpr * 4;
    const bool routed = p.gather == GATHER_CSR || p.gather == GATHER_INDICES;   // a grid row per activation row
    g.grid = dim3((p.N + a.rows_per_wg - 1) / a.rows_per_wg, batch ? (uint32_t)batch->n : routed ? p.T : 1u, 1);
    if (norm_w) {
        g.shmem += 16 * sizeof(float);  // one partial sum of squares per wave
        if (gate_z && rps == 4 && p.dtype != DT_F32) g.shmem += 16 + (size_t)C * 4 * 16 * 2;   // the gated halves, dealt over the row slots
        switch (p.dtype) {
            case DT_F32: return qmv_stream_norm_launch_dtype<DT_F32>(a, p.bits, g, lc);
            case DT_F16: return qmv_stream_norm_launch_dtype<DT_F16>(a, p.bits, g, lc);
            case DT_BF16: return qmv_stream_norm_launch_dtype<DT_BF16>(a, p.bits, g, lc);
            default: return fail(ERR_BAD_ARG, "unknown dtype");
        }
    }
    switch (p.dtype) {
        case DT_F32: return qmv_stream_launch_dtype<DT_F32>(a, p.bits, p.gather, g, lc);
        case DT_F16: return qmv_stream_launch_dtype<DT_F16>(a, p.bits, p.gather, g, lc);
        case DT_BF16: return qmv_stream_launch_dtype<DT_BF16>(a, p.bits, p.gather, g, lc);
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
}

int launch_qmv_batched(const QmvParams& p0, const QmvBatch& b, const LaunchCtx& lc) {
    if (b.n < 2 || b.n > 4) return fail(ERR_BAD_ARG, "batched qmv takes 2 to 4 matrices");
    // Rows of 2048 ... 8192 4-bit codes: the matrices' rows one after the other on the kernel whose waves walk the rows,
    // sized as the one matrix of all of them would be.
    if ((options().qmv_kernel == 0 && qmv_rows_walk_batched_preferred(p0, b)) || (options().qmv_kernel == 4 && qmv_rows_walk_batched_takes(p0, b))) {
        int rc = launch_qmv_rows_walk_batched(p0, b, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    if (p0.bits != 2 && p0.bits != 4 && p0.bits != 8) return fail(ERR_UNSUPPORTED, "batched qmv: bits must be 2, 4 or 8");
    QmvParams p = p0;
    p.gather = GATHER_NONE;
    p.M = 1;
    p.N = 0;
    for (int j = 0; j < b.n; j++) {
        if (!b.w[j] || !b.scales[j] || !b.biases[j] || !b.out[j] || b.N[j] == 0) return fail(ERR_BAD_ARG, "batched qmv: null buffer or empty matrix");
        if ((uintptr_t)b.w[j] % 16 || (uintptr_t)b.scales[j] % 16 || (uintptr_t)b.biases[j] % 16)
            return fail(ERR_UNSUPPORTED, "batched qmv: operands must be 16-byte aligned");
        if (b.N[j] > p.N) p.N = b.N[j];  // the geometry (and the grid) follow the tallest matrix
    }
    p.w = b.w[0];
    p.scales = b.scales[0];
    p.biases = b.biases[0];
    p.out = b.out[0];
    const uint32_t cpc = 128u / (uint32_t)p.bits;
    if (p.K == 0 || p.K % cpc) return fail(ERR_UNSUPPORTED, "batched qmv: K*bits % 128 != 0");
    const uint32_t G = p.group_size;
    if (!is_pow2(G) || G * 2 < cpc || p.K % G) return fail(ERR_UNSUPPORTED, "batched qmv: group size");
    const uint32_t C = p.K / cpc;
    if (C > 1024 || C % 64 || (uintptr_t)p.x % 16) return fail(ERR_UNSUPPORTED, "batched qmv: row geometry");
    uint32_t rps = 1;
    while (C * rps < 256 && C * rps * 2 <= 1024) rps *= 2;
    return launch_qmv_stream(p, C, rps, C * rps, 1, lc, &b);
}

int launch_qmv_norm(const QmvParams& p0, const void* norm_w, const float* eps, const LaunchCtx& lc) {
    if (p0.bits != 4 && p0.bits != 8) return fail(ERR_UNSUPPORTED, "norm + qmv: bits must be 4 or 8");
    QmvParams p = p0;
    p.gather = GATHER_NONE;
    p.M = 1;
    const uint32_t cpc = 128u / (uint32_t)p.bits;
    if (p.K == 0 || p.N == 0 || p.K % cpc) return fail(ERR_UNSUPPORTED, "norm + qmv: K*bits % 128 != 0");
    const uint32_t G = p.group_size;
    if (!is_pow2(G) || G * 2 < cpc || p.K % G) return fail(ERR_UNSUPPORTED, "norm + qmv: group size");
    const uint32_t C = p.K / cpc;
    if (C > 1024 || C % 64) return fail(ERR_UNSUPPORTED, "norm + qmv: row geometry");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)norm_w % 16)
        return fail(ERR_UNSUPPORTED, "norm + qmv: w, x and norm_weight must be 16-byte aligned");
    uint32_t rps = 1;
    while (C * rps < 256 && C * rps * 2 <= 1024) rps *= 2;
    return launch_qmv_stream(p, C, rps, C * rps, 1, lc, nullptr, norm_w, eps);
}

// The gated form of the fused norm (4-bit codes): p.x is the f32 activation y [hv, dv], K = hv * dv. A thread's chunk of
// 32 values must lie within one row of dv, and the dv / 32 threads of a row must be neighbours within a wave.
int launch_qmv_gated_norm(const QmvParams& p0, const void* gate_z, const void* norm_w, const float* eps, uint32_t dv,
                          const LaunchCtx& lc) {
    QmvParams p = p0;
    p.gather = GATHER_NONE;
    p.M = 1;
    p.bits = 4;
    const uint32_t cpc = 32;
    if (p.K == 0 || p.N == 0 || dv == 0 || p.K % dv || dv % cpc || !is_pow2(dv / cpc) || dv / cpc > 64)
        return fail(ERR_UNSUPPORTED, "gated norm + qmv: dv must be 32 times a power of two up to 2048");
    const uint32_t G = p.group_size;
    if (!is_pow2(G) || G * 2 < cpc || p.K % G) return fail(ERR_UNSUPPORTED, "gated norm + qmv: group size");
    const uint32_t C = p.K / cpc;
    if (C > 512 || C % 64) return fail(ERR_UNSUPPORTED, "gated norm + qmv: row geometry");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)norm_w % 16 || (uintptr_t)gate_z % 16)
        return fail(ERR_UNSUPPORTED, "gated norm + qmv: w, y, z and norm_weight must be 16-byte aligned");
    uint32_t rps = 1;
    while (C * rps < 256 && C * rps * 2 <= 512) rps *= 2;
    return launch_qmv_stream(p, C, rps, C * rps, 1, lc, nullptr, norm_w, eps, gate_z, dv);
}

static int launch_qmv_dot2(const QmvParams& p, const LaunchCtx& lc);

// Routed rows the one-row streaming kernel takes: one row (two when the streaming kernel is asked for by option),
// fewer than the experts, at most 64 experts (the routing is read by one wave-wide load), 4-bit codes, f16 / bf16.
static bool qmv_few_routed_rows(const QmvParams& p) {
    const uint32_t most = options().qmv_kernel == 2 ? 2u : 1u;
    // (and only rows the streaming kernel can tile: whole waves of 16-byte chunks, scales in whole 4-vectors, 16-byte aligned;
    // other rows keep the gather instances of the one-shot and matrix-core kernels)
    const bool tiles = p.group_size && p.K % 2048 == 0 && p.K % p.group_size == 0 && (p.K / p.group_size) % 4 == 0 &&
                       (uintptr_t)p.scales % 16 == 0 && (uintptr_t)p.biases % 16 == 0;
    return (p.gather == GATHER_CSR || p.gather == GATHER_INDICES) && p.T >= 1 && p.T <= most && p.T < p.E && p.E <= 64 && p.bits == 4 &&
           p.dtype != DT_F32 && options().qmv_kernel != 1 && tiles;   // (f32 rows stay where they were: measured for f16 / bf16 only)
}

int launch_qmv_fast(const QmvParams& p, const LaunchCtx& lc) {
    // The matrix-core kernel wins as soon as more than one activation row shares
    // the weight stream (and for every gather); a single row is as fast on the
    // dot2 kernels.
    // Widths 3, 5 and 6 have no dot2 kernel: the matrix-core kernel is their fast path.
    const bool many = p.gather == GATHER_CSR || p.gather == GATHER_INDICES || (p.gather == GATHER_NONE && p.M >= 2) ||
                      p.bits == 3 || p.bits == 5 || p.bits == 6;
    const int mode = options().qmv_mfma;
    bool tried_mfma = false;
    // One routed row: the one-row streaming kernel, each grid row once per row of the expert it finds. 8 experts of
    // 14336 x 4096, us, matrix-core GEMV -> this: 1 row 14.9 -> 10.6 (the plain one-row launch on one expert: 8.3; the
    // routing sits ahead of the first weight load); 2 rows on 2 experts 17.6 -> 18.1, so those stay where they were.
    // One row of 4096 4-bit codes (the gate / up shapes of the headline): the wave-per-four-rows kernel, 3 % ahead of the
    // streaming kernel in the same run (14336 x 4096 bf16: 7.86 against 8.11 us).
    if (mode != 2 && ((options().qmv_kernel == 0 && qmv_rows_walk_preferred(p)) || (options().qmv_kernel == 4 && qmv_rows_walk_takes(p)))) {
        int rc = launch_qmv_rows_walk(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    if (mode != 2 && ((options().qmv_kernel == 0 && qmv_rows_preferred(p)) || (options().qmv_kernel == 3 && qmv_rows_takes(p)))) {
        int rc = launch_qmv_rows(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    if (mode != 2 && ((options().qmv_kernel == 0 && qmv_rows_few_preferred(p)) || (options().qmv_kernel == 3 && qmv_rows_few_takes(p)))) {
        int rc = launch_qmv_rows_few(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    if (qmv_few_routed_rows(p) && mode != 2) {
        int rc = launch_qmv_dot2(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    if (mode == 2 || (mode == 0 && many)) {
        int rc = launch_qmv_mfma(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
        tried_mfma = true;
    }
    int rc = launch_qmv_dot2(p, lc);
    // Rows the dot2 kernels cannot tile (a chunk count that is neither whole waves nor a power of
    // two, e.g. K = 3584 or 18944 with 4-bit codes) still fit the matrix-core kernel when they are
    // whole 512-code segments: 18944x3584, one row, 98 us on the generic kernel against 12 us.
    if (rc == ERR_UNSUPPORTED && !tried_mfma && mode != 1) {
        const int rc2 = launch_qmv_mfma(p, lc);
        if (rc2 != ERR_UNSUPPORTED) return rc2;
    }
    return rc;
}

static int launch_qmv_dot2(const QmvParams& p, const LaunchCtx& lc) {
    if (p.bits != 2 && p.bits != 4 && p.bits != 8)
        return fail(ERR_UNSUPPORTED, "fast qmv: bits must be 2, 4 or 8");
    const uint32_t cpc = 128u / (uint32_t)p.bits;
    if (p.K == 0 || p.N == 0 || p.K % cpc) return fail(ERR_UNSUPPORTED, "fast qmv: K*bits % 128 != 0");
    const uint32_t G = p.group_size;
    if (!is_pow2(G) || G * 2 < cpc || p.K % G) return fail(ERR_UNSUPPORTED, "fast qmv: group size");
    const uint32_t C = p.K / cpc;
    const bool gather = p.gather == GATHER_CSR || p.gather == GATHER_INDICES;
    const bool few = qmv_few_routed_rows(p);   // worked one row at a time
    const uint32_t rows = few ? 1u : gather ? p.T : (p.gather == GATHER_SINGLE ? 1u : p.M);
    if (rows == 0) return ERR_OK;  // nothing to compute
    const uint32_t maxt = ((gather && !few) || rows > 1) ? 512u : 1024u;
    if (C > maxt) return fail(ERR_UNSUPPORTED, "fast qmv: row too long for one workgroup");
    if (!(C % 64 == 0 || (C < 64 && is_pow2(C)))) return fail(ERR_UNSUPPORTED, "fast qmv: chunk count");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16) return fail(ERR_UNSUPPORTED, "fast qmv: w and x must be 16-byte aligned");
    // threads per workgroup: a whole number of rows per step, >= 256 threads when possible
    uint32_t rps = 1;
    while (C * rps < 256 && C * rps * 2 <= maxt) rps *= 2;
    const uint32_t tpb = C * rps;
    if (tpb % 64) return fail(ERR_UNSUPPORTED, "fast qmv: workgroup not a whole number of waves");

    // Rows per pass: 4, except that a thread's slice of an f32 activation row for 2-bit codes is 64
    // floats, and two of those no longer fit the register file (2 rows: 35 us against 2 x 5.6).
    const uint32_t pass_rows = (p.dtype == DT_F32 && p.bits == 2) ? 1u : 4u;
    if (!gather && p.gather != GATHER_SINGLE && rows > pass_rows) {
        // more activation rows than one pass holds
        const size_t esz = p.dtype == DT_F32 ? 4 : 2;
        for (uint32_t m0 = 0; m0 < rows; m0 += pass_rows) {
            QmvParams q = p;
            q.M = rows - m0 < pass_rows ? rows - m0 : pass_rows;
            q.x = (const char*)p.x + (size_t)m0 * p.K * esz;
            q.out = (char*)p.out + (size_t)m0 * p.N * esz;
            LaunchCtx l2 = lc;
            if (m0) l2.start = nullptr;
            if (m0 + pass_rows < rows) l2.stop = nullptr;
            int rc = launch_qmv_fast(q, l2);
            if (rc) return rc;
        }
        return ERR_OK;
    }

    if ((!gather || few) && options().qmv_kernel != 1) {
        int rc = launch_qmv_stream(p, C, rps, tpb, rows, lc);
        if (rc != ERR_UNSUPPORTED || few) return rc;
    }

    QmvGeom g;
    g.mb = gather ? 4 : (int)rows;
    g.rt = (p.gather == GATHER_NONE && g.mb <= 2) || p.gather == GATHER_SINGLE ? 8 : 4;
    if (p.gather == GATHER_NONE && g.mb == 1) {
        // Even work per compute unit beats the deepest load queue: prefer the
        // rows-per-thread count whose tile count is a multiple of the CU count.
        const uint32_t cus = (uint32_t)num_cus();
        const int cand[3] = {8, 7, 4};
        for (int rt : cand) {
            const uint32_t R = (uint32_t)rt * rps;
            if (p.N % R == 0 && (p.N / R) % cus == 0) { g.rt = rt; break; }
        }
        if (options().qmv_rows_per_thread) g.rt = options().qmv_rows_per_thread;
    }
    const uint32_t R = (uint32_t)g.rt * rps;
    g.tpb = tpb;

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
    // Scales/biases are staged four elements per load when every tile's block of
    // them (R*gpr elements from a multiple of R*gpr) is 4-aligned.
    g.sbi = 0;
    if (a.gpr % 4 == 0 && (uintptr_t)p.scales % 16 == 0 && (uintptr_t)p.biases % 16 == 0) {
        const uint64_t vecs = (uint64_t)R * a.gpr / 4;
        const uint64_t per_thread = (vecs + tpb - 1) / tpb;
        g.sbi = per_thread <= 1 ? 1 : per_thread <= 2 ? 2 : per_thread <= 4 ? 4 : 0;
    }
    g.shmem = (size_t)a.lds_sb_pairs * 8 + (size_t)R * 4 * (a.wpr ? a.wpr : 1) * 4 + (size_t)a.list_cap * 4;
    if (g.shmem > 64 * 1024) return fail(ERR_UNSUPPORTED, "fast qmv: tile does not fit in LDS");
    g.grid = dim3((p.N + R - 1) / R, gather ? p.E : 1, 1);

    switch (p.dtype) {
        case DT_F32: return qmv_launch_dtype<DT_F32>(a, p.bits, p.gather, g, lc);
        case DT_F16: return qmv_launch_dtype<DT_F16>(a, p.bits, p.gather, g, lc);
        case DT_BF16: return qmv_launch_dtype<DT_BF16>(a, p.bits, p.gather, g, lc);
        default: return fail(ERR_BAD_ARG, "unknown dtype");
    }
}

}  // namespace mtq
