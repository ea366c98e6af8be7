// Host side of the matrix-core qmv / gather_qmv kernel (qmv_mfma_impl.h): checks
// that a request fits its geometry, picks the launch shape and calls the
// per-dtype instantiation. Requests that do not fit return ERR_UNSUPPORTED so
// the caller can use the dot2 family or the generic kernel.
#include "qmv_mfma_impl.h"

namespace mtq {

extern template int qmv_mfma_launch_dtype<DT_F16>(QmvMArgs&, int, int, const QmvMGeom&, const LaunchCtx&);
extern template int qmv_mfma_launch_dtype<DT_BF16>(QmvMArgs&, int, int, const QmvMGeom&, const LaunchCtx&);
extern template int qmv_mfma_launch_dtype_odd<DT_F16>(QmvMArgs&, int, int, const QmvMGeom&, const LaunchCtx&);
extern template int qmv_mfma_launch_dtype_odd<DT_BF16>(QmvMArgs&, int, int, const QmvMGeom&, const LaunchCtx&);

namespace {
bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }
uint32_t ilog2(uint32_t v) { uint32_t l = 0; while ((1u << l) < v) l++; return l; }
constexpr size_t kLdsBudget = 150 * 1024;  // of the 160 KB per CU

int num_cus_mfma() {
    static int n = 0;
    if (n == 0) {
        int dev = 0, v = 0;
        n = (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) ? v : 256;
    }
    return n;
}

// waves = KP * RBW; gpw = (scale, bias) pairs per row in a wave's window
size_t lds_bytes(uint32_t R, uint32_t K /* padded to whole steps */, uint32_t nch, uint32_t gpr, uint32_t rows_wg, uint32_t waves, uint32_t gpw, uint32_t KP, uint32_t list_cap) {
    return (size_t)R * K * 2 + (size_t)R * gpr * 4 + ((size_t)waves * 4 * gpw + 1) * 8 +
           (size_t)KP * rows_wg * R * 4 + (size_t)list_cap * 4 + 64;
}

// Pairs per row that a wave's window must hold: the groups its K part touches, from a
// multiple of 4 (8-byte loads) up to a whole number of 4-vectors. Parts are spp wave-wide
// steps of 16 * cpc codes; the last part ends with the row (K codes).
uint32_t window_pairs(uint32_t kp_count, uint32_t spp, uint32_t cpc, uint32_t log2g, uint32_t K) {
    uint32_t need = 4;
    for (uint32_t kp = 0; kp < kp_count; kp++) {
        const uint64_t end = (uint64_t)(kp + 1) * spp * 16u * cpc;
        const uint32_t first = (kp * spp * 16u * cpc) >> log2g, last = (uint32_t)(((end < K ? end : K) - 1u) >> log2g);
        const uint32_t lo = first & ~3u, n = (last + 1 - lo + 3) / 4 * 4;
        if (n > need) need = n;
    }
    return need;
}
}  // namespace

int launch_qmv_mfma(const QmvParams& p, const LaunchCtx& lc) {
    if (p.dtype != DT_F16 && p.dtype != DT_BF16) return fail(ERR_UNSUPPORTED, "mfma qmv: f16/bf16 only");
    // 2-bit codes in groups of 32: a 16-byte lane chunk (64 codes) would straddle two groups, so the lanes take
    // 8 bytes (32 codes) each, like the widths whose chunk is 32 codes of the bit stream
    const bool half2 = p.bits == 2 && p.group_size == 32;
    const bool odd = p.bits == 3 || p.bits == 5 || p.bits == 6 || half2;
    if (!(p.bits == 2 || p.bits == 4 || p.bits == 8 || odd))
        return fail(ERR_UNSUPPORTED, "mfma qmv: bits");
    if (p.N == 0 || p.K == 0) return fail(ERR_UNSUPPORTED, "mfma qmv: empty");
    // a lane's chunk: 16 bytes (128/bits codes), or 32 codes = bits dwords where codes straddle words
    const uint32_t cpc = odd ? 32u : 128u / (uint32_t)p.bits, cb = odd ? 4u * (uint32_t)p.bits : 16u;
    const uint64_t rb64 = (uint64_t)p.K * p.bits / 8;
    if (p.K % cpc || rb64 > (1u << 24)) return fail(ERR_UNSUPPORTED, "mfma qmv: row is not whole lane chunks");
    if (rb64 * p.N >= (1ull << 32) || (uint64_t)p.N * (p.K / p.group_size) >= (1ull << 31))
        return fail(ERR_UNSUPPORTED, "mfma qmv: a weight matrix of 4 GiB or more");
    // A wave-wide step covers 16 lane chunks of each of 4 rows; a row that is not a whole number of
    // steps ends with a partial one (its idle lanes are fed zeros).
    const uint32_t RB = (uint32_t)rb64, nch = p.K / cpc, nseg = (nch + 15u) / 16u, nchp = nseg * 16u;
    (void)cb;
    const uint32_t G = p.group_size;
    if (!is_pow2(G) || G < cpc || G > 16u * cpc || p.K % G) return fail(ERR_UNSUPPORTED, "mfma qmv: group size");
    const uint32_t gpr = p.K / G;
    if ((uintptr_t)p.w % (odd ? 4 : 16) || (uintptr_t)p.x % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16 ||
        (rb64 % 16 && !odd) || (p.K * 2) % 16)
        return fail(ERR_UNSUPPORTED, "mfma qmv: operands must be 16-byte aligned");
    const bool gather = p.gather == GATHER_CSR || p.gather == GATHER_INDICES;
    const bool norm = p.norm_w != nullptr;   // one row, staged as two (rounded value and remainder)
    if (norm && (p.gather != GATHER_NONE || p.M != 1 || p.bits != 4 || !p.norm_eps || (uintptr_t)p.norm_w % 16))
        return fail(ERR_UNSUPPORTED, "mfma qmv: the fused norm takes one row of 4-bit codes");
    const uint32_t rows = gather ? p.T : (p.gather == GATHER_SINGLE ? 1u : (norm ? 2u : p.M));
    if (rows == 0) return ERR_OK;
    const Options& opt = options();

    // K parts: keep 4..8 segments per wave and row block where the row allows
    uint32_t KP = 1;
    if (opt.qmv_mfma_kp) {
        KP = (uint32_t)opt.qmv_mfma_kp;
        if ((uint64_t)(KP - 1) * ((nseg + KP - 1) / KP) >= nseg) return fail(ERR_BAD_ARG, "qmv.mfma_kp leaves a K part empty");
    } else {
        uint32_t best = 1;
        double best_score = 1e30;
        for (uint32_t kp = 1; kp <= nseg && kp <= 16; kp++) {
            // parts of spp steps each; the last may be shorter but not empty
            const uint32_t spp = (nseg + kp - 1) / kp, padded = (spp + 3) / 4 * 4;
            if ((uint64_t)(kp - 1) * spp >= nseg) continue;
            if (window_pairs(kp, spp, cpc, ilog2(G), p.K) > 64) continue;  // a lane refills one 4-vector of its wave's window
            double score = (double)((uint64_t)kp * padded - nseg) / nseg;  // wasted ring slots over all parts
            if (spp > 8) score += 0.05 * (spp - 8);               // long walks: few waves per row block
            if (spp < 4) score += 0.5;
            score += 0.01 * kp;
            if (score < best_score) { best_score = score; best = kp; }
        }
        KP = best;
    }
    const uint32_t spp = (nseg + KP - 1) / KP;
    const uint32_t gpw = window_pairs(KP, spp, cpc, ilog2(G), p.K);
    if (gpw > 64) return fail(ERR_UNSUPPORTED, "mfma qmv: K part spans more than 64 groups");

    // activation rows per pass
    int mp = 4, s = 1;
    uint32_t rows_per_launch = rows;
    if (p.gather == GATHER_NONE) {
        if (rows == 1) mp = 1; else if (rows == 2) mp = 2;
        if (rows > 4) s = rows > 8 ? 4 : 2;
        rows_per_launch = rows > 16 ? 16 : rows;
    } else if (p.gather == GATHER_SINGLE) {
        mp = 1;
    } else {
        const uint32_t avg = (rows + p.E - 1) / (p.E ? p.E : 1);
        // 8 rows per pass from an average of 3 rows per expert: with uneven routing some expert
        // then has more than 4, and a second pass would stream its weights again (measured on
        // 8 experts x 14336x4096 with 2..6 rows each: 1.29 x the algorithmic traffic at 4 rows
        // per pass, 1.01 x at 8).
        s = avg > 8 ? 4 : (avg >= 3 ? 2 : 1);
        if (p.bits == 2 && s > 2) s = 2;  // the 16-row 2-bit variant does not fit the register file
        if (opt.qmv_mfma_sets) s = opt.qmv_mfma_sets;
    }
    // Rows per workgroup. Every workgroup stages all activation rows of a pass (R x K elements)
    // before it streams, so the weight rows are dealt to one workgroup per compute unit, as many of
    // its row blocks side by side as the workgroup size allows, the rest one after the other.
    // Measured with 8 activation rows, 4-bit bf16: 128256x4096 63 us at 251 workgroups against
    // 129 us at 4008; 57344x4096 33 against 57; 14336x4096 12.8 against 16.8.
    // A gather workgroup additionally should live long: as many row blocks one after the other as
    // leave one workgroup (two when 4 rows are staged) per CU over the experts that can be hit.
    // Measured on 8 experts x 14336x4096, 32 rows: 61 us with 7 row blocks of 64 rows per
    // workgroup, 74 us with 4, 98 us with 14. Short rows (few steps per row block) want the row
    // blocks one after the other in a narrow workgroup rather than side by side in a wide one: at
    // least 16 steps per wave (E = 128 x 256x2048 with one row per expert: 15 us with 2 blocks side
    // by side x 4 in sequence, 30 us with 16 side by side).
    // When the staged rows leave too little LDS: a narrower workgroup with the row blocks moved one
    // after the other (the number of workgroups stays) down to 8 waves, which a CU needs to keep
    // enough loads in flight (28672x8192, 8 rows: 100 us with 4-wave workgroups in one pass, 54 us
    // in two passes of 16-wave ones); then up to half the rows per workgroup; then half the
    // activation rows per pass, planned afresh, although every further pass streams the weights again.
    const uint32_t rbw_cap = 16u;
    const uint32_t list_cap = p.gather == GATHER_INDICES ? p.T : 0;
    uint32_t RBW = 1, nrb = 1;
    for (;; s /= 2) {
        const uint32_t maxt = s >= 2 ? 512u : 1024u;
        if (64u * KP > maxt) {
            if (s > 1) continue;
            return fail(ERR_UNSUPPORTED, "mfma qmv: too many K parts");
        }
        uint32_t rbw_max = rbw_cap;
        while (64u * KP * rbw_max > maxt && rbw_max > 1) rbw_max /= 2;
        const uint64_t blocks = ((uint64_t)p.N + 3) / 4;  // 4-row blocks of one matrix
        if (gather) {
            const uint64_t e_eff = p.E < rows ? p.E : rows;
            const uint64_t slots = (uint64_t)num_cus_mfma() * (s == 1 ? 2 : 1);
            uint64_t per_wg = (blocks * e_eff + slots - 1) / slots;
            if (per_wg > blocks) per_wg = blocks;
            const uint32_t min_nrb = spp >= 16 ? 1u : (16u + spp - 1) / spp;
            RBW = 1;
            while (RBW * 2 <= rbw_max && (uint64_t)RBW * 2 * min_nrb <= per_wg) RBW *= 2;
            const uint64_t n = (per_wg + RBW - 1) / RBW;
            nrb = n > 64 ? 64u : (n < 1 ? 1u : (uint32_t)n);
        } else {
            const uint64_t slots = (uint64_t)num_cus_mfma();
            const uint64_t per_wg = (blocks + slots - 1) / slots;
            RBW = 1;
            while (RBW < rbw_max && RBW < per_wg) RBW *= 2;
            const uint64_t n = (per_wg + RBW - 1) / RBW;
            nrb = n > 64 ? 64u : (uint32_t)n;
        }
        if (opt.qmv_mfma_rbw) {
            RBW = (uint32_t)opt.qmv_mfma_rbw;
            if (64u * KP * RBW > maxt) return fail(ERR_BAD_ARG, "qmv.mfma_rbw: workgroup too large");
        }
        if (opt.qmv_mfma_nrb) nrb = (uint32_t)opt.qmv_mfma_nrb;
        auto need = [&]() { return lds_bytes((uint32_t)(mp * s), nchp * cpc, nch, gpr, 4 * RBW * nrb, KP * RBW, gpw, KP, list_cap); };
        const uint32_t nrb_planned = nrb;
        const bool last = s == 1;  // nothing left to halve: shrink as far as it takes
        while (need() > kLdsBudget) {
            if (RBW > 1 && !opt.qmv_mfma_rbw && (last || KP * RBW / 2 >= 8)) { RBW /= 2; nrb = nrb * 2 > 64 ? 64 : nrb * 2; }
            else if (nrb > 1 && (last || nrb * 2 > nrb_planned)) nrb--;
            else break;
        }
        if (need() <= kLdsBudget) break;
        if (last) {
            // Not even one set of 4 rows: a plain batch can still go 2 rows, then 1 row, per pass
            // (3584x18944 with 4 rows: two passes of 12 us against 343 us on the generic kernel).
            if (p.gather == GATHER_NONE && mp > 1) {
                mp /= 2;
                s = 2;  // halved to 1 by the loop
                continue;
            }
            return fail(ERR_UNSUPPORTED, "mfma qmv: activations do not fit in LDS");
        }
    }
    const uint32_t R = (uint32_t)(mp * s);
    if (p.gather == GATHER_NONE && rows_per_launch > R) rows_per_launch = R;

    if (p.gather == GATHER_NONE && rows > rows_per_launch) {
        // more activation rows than one pass holds: one launch per R rows
        for (uint32_t m0 = 0; m0 < rows; m0 += rows_per_launch) {
            QmvParams q2 = p;
            q2.M = rows - m0 < rows_per_launch ? rows - m0 : rows_per_launch;
            q2.x = (const char*)p.x + (size_t)m0 * p.K * 2;
            q2.out = (char*)p.out + (size_t)m0 * p.N * 2;
            LaunchCtx l2 = lc;
            if (m0) l2.start = nullptr;
            if (m0 + rows_per_launch < rows) l2.stop = nullptr;
            int rc = launch_qmv_mfma(q2, l2);
            if (rc) return rc;
        }
        return ERR_OK;
    }

    QmvMArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = p.scales;
    a.biases = p.biases;
    a.x = p.x;
    a.out = p.out;
    a.route = p.route;
    a.M = rows;
    a.N = p.N;
    a.K = p.K;
    a.T = p.T;
    a.E = p.E;
    a.RB = RB;
    a.nch = nch;
    a.nchp = nchp;
    a.nseg = nseg;
    a.spp = spp;
    a.KP = KP;
    a.RBW = RBW;
    a.nrb = nrb;
    a.gpr = gpr;
    a.gpw = gpw;
    a.log2g = ilog2(G);
    a.list_cap = list_cap;
    // fewer rows than experts: a grid row per row, each finding the expert it serves (at most T experts have rows)
    const bool by_slot = (p.gather == GATHER_CSR || p.gather == GATHER_INDICES) && p.T < p.E && p.T <= 32;
    a.by_slot = by_slot ? 1u : 0u;
    a.norm_w = p.norm_w;
    a.norm_eps = p.norm_eps;
    const int mode = norm ? (int)GATHER_NORM : p.gather;
    QmvMGeom g;
    g.mp = mp;
    g.s = s;
    g.tpb = 64u * KP * RBW;
    const uint32_t rows_wg = 4 * RBW * nrb;
    g.shmem = lds_bytes(R, nchp * cpc, nch, gpr, rows_wg, KP * RBW, gpw, KP, list_cap);
    g.grid = dim3((p.N + rows_wg - 1) / rows_wg, by_slot ? p.T : gather ? p.E : 1, 1);
    if (odd)
        return p.dtype == DT_F16 ? qmv_mfma_launch_dtype_odd<DT_F16>(a, half2 ? 22 : p.bits, mode, g, lc)
                                 : qmv_mfma_launch_dtype_odd<DT_BF16>(a, half2 ? 22 : p.bits, mode, g, lc);
    switch (p.dtype) {
        case DT_F16: return qmv_mfma_launch_dtype<DT_F16>(a, p.bits, mode, g, lc);
        default: return qmv_mfma_launch_dtype<DT_BF16>(a, p.bits, mode, g, lc);
    }
}

}  // namespace mtq
