// Host side of the 16-row matrix-core GEMV (kernel in qmv_wide_impl.h): which shapes it takes, its geometry, the
// instances for plain batches (the expert-routed ones are built in qmv_wide_gather.hip).
#include "qmv_wide_impl.h"

namespace mtq {

// Adds the K slices' partial rows in slice order and rounds to the element type.
template <int DT> __global__ __launch_bounds__(256) void qmv_wide_reduce_kernel(const float* part, void* out, uint32_t total, uint32_t ksplit) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float r = part[i];
    for (uint32_t sp = 1; sp < ksplit; sp++) r += part[(size_t)sp * total + i];
    ((uint16_t*)out)[i] = f32_to_elem_bits<DT>(r);
}

struct QmvWPlan {
    uint32_t kslice, ksplit, nb, kp, log2kp, tpk, sets, grid_x;
    size_t lds;
};

static int wide_cus() {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    return cus;
}

// 16 rows of activations (32 bytes per code position) and a row of group sums (64 bytes per group) in 160 KB
static uint32_t wide_bytes_per_turn(uint32_t G) { return 512u * 32u + (512u / G) * 64u; }

// A workgroup's 16 waves take 16 * NB / KP row blocks: two per wave once that still gives every compute unit a
// workgroup, else one, and on shorter matrices KP waves share a row block, each with a run of the turns.
// tps: turns per K slice; nrb: row blocks of the matrix; want: workgroups per matrix (and K slice) that fill the chip.
static bool wide_geometry(uint32_t G, uint32_t tps, uint32_t nrb, uint32_t want, QmvWPlan& pl) {
    pl.nb = (nrb + 15u) / 16u > want + want / 4u && G != 32 ? 2u : 1u;   // (two row blocks of 32-code groups do not fit the registers)
    pl.kp = 1;
    pl.log2kp = 0;
    while (pl.nb == 1u && pl.kp < 16u && pl.kp * 2u <= tps && (nrb * pl.kp * 2u + 15u) / 16u <= want) {
        pl.kp *= 2u;
        pl.log2kp++;
    }
    if (options().qmv_wide_kp) {
        pl.nb = 1;
        pl.kp = (uint32_t)options().qmv_wide_kp;
        pl.log2kp = 0;
        while ((1u << pl.log2kp) < pl.kp) pl.log2kp++;
    }
    if (options().qmv_wide_nb) pl.nb = G == 32 ? 1u : (uint32_t)options().qmv_wide_nb;
    // A wave keeps the scales and biases of its whole run of turns in registers, a set per 4 turns: at most 3 sets
    // (2 with two row blocks per wave, 1 for groups of 32 codes, whose turns hold twice the groups).
    const uint32_t max_sets = G == 32 ? 1u : 3u;
    while (pl.kp < 16u && (tps + pl.kp - 1) / pl.kp > 4u * max_sets) {
        pl.kp *= 2u;
        pl.log2kp++;
    }
    pl.tpk = (tps + pl.kp - 1) / pl.kp;
    pl.sets = (pl.tpk + 3u) / 4u;
    if (pl.sets > max_sets) return false;
    if (pl.nb == 2u && pl.sets > 2u) pl.nb = 1;
    if (pl.nb == 2u && pl.sets == 1u && G == 128) pl.nb = 1;   // (that instance does not fit 128 registers; runs of at most 4 turns on very many rows)
    if (pl.kp > 1u && pl.lds < (size_t)16 * pl.nb * 1024) pl.lds = (size_t)16 * pl.nb * 1024;   // the K parts' sums, a KB per wave and row block
    const uint32_t per_wg = 16u * pl.nb / pl.kp;
    pl.grid_x = (nrb + per_wg - 1) / per_wg;
    return true;
}

// Shapes the kernel takes: f16 / bf16, 4-bit codes, groups of 32 / 64 / 128, at most 16 rows, rows of whole turns.
static bool plan_wide(const QmmParams& p, QmvWPlan& pl) {
    const uint32_t G = p.group_size;
    if ((p.dtype != DT_F16 && p.dtype != DT_BF16) || p.bits != 4 || (G != 32 && G != 64 && G != 128)) return false;
    if (p.M == 0 || p.M > 16 || p.N == 0 || p.K == 0 || p.K % 512) return false;
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16) return false;
    if ((uint64_t)p.M * p.N >= (1ull << 31) || (uint64_t)p.N * p.K / 2 >= (1ull << 32)) return false;
    const uint32_t cus = (uint32_t)wide_cus();
    const uint32_t per_turn = wide_bytes_per_turn(G);
    const uint32_t max_turns = (160u * 1024u - 64u) / per_turn;   // (64 bytes left for the kernel's statically allocated row counter)
    const uint32_t turns = p.K / 512u;
    uint32_t ks = (turns + max_turns - 1) / max_turns;
    const uint32_t tps = (turns + ks - 1) / ks;
    ks = (turns + tps - 1) / tps;
    pl.kslice = tps * 512u;
    pl.ksplit = ks;
    pl.lds = (size_t)tps * per_turn;
    const uint32_t nrb = (p.N + 15u) / 16u;
    const uint32_t want = cus / ks > 0 ? cus / ks : 1u;   // workgroups per K slice
    return wide_geometry(G, tps, nrb, want, pl);
}

bool qmv_wide_takes(const QmmParams& p) {
    QmvWPlan pl;
    return plan_wide(p, pl);
}

size_t qmv_wide_scratch_bytes(const QmmParams& p) {
    QmvWPlan pl;
    if (!plan_wide(p, pl) || pl.ksplit <= 1) return 0;
    return (size_t)pl.ksplit * p.M * p.N * sizeof(float);
}

int launch_qmv_wide(const QmmParams& p, const LaunchCtx& lc, void* scratch) {
    QmvWPlan pl;
    if (!plan_wide(p, pl)) return fail(ERR_UNSUPPORTED, "wide qmv: shape not taken");
    if (pl.ksplit > 1 && !scratch) return fail(ERR_BAD_ARG, "wide qmv: K split without a scratch buffer");
    QmvWArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = (const uint16_t*)p.scales;
    a.biases = (const uint16_t*)p.biases;
    a.x = (const uint16_t*)p.x;
    a.out = p.out;
    a.part = (float*)scratch;
    a.M = p.M;
    a.N = p.N;
    a.K = p.K;
    a.gpr = p.K / p.group_size;
    a.kslice = pl.kslice;
    a.kp = pl.kp;
    a.log2kp = pl.log2kp;
    a.tpk = pl.tpk;
    a.route = nullptr;
    a.T = p.M;
    a.E = 1;
    const void* fn = nullptr;
#define QW_PICK3(DTv, Gv, NBv) (pl.sets == 1 ? (const void*)qmv_wide_kernel<DTv, Gv, (Gv == 128 ? 1 : NBv), 1> : pl.sets == 2 ? (const void*)qmv_wide_kernel<DTv, Gv, NBv, 2> : NBv == 1 ? (const void*)qmv_wide_kernel<DTv, Gv, 1, 3> : nullptr)
#define QW_PICK2(DTv, NBv) (p.group_size == 32 ? (const void*)qmv_wide_kernel<DTv, 32, 1, 1> : p.group_size == 64 ? QW_PICK3(DTv, 64, NBv) : QW_PICK3(DTv, 128, NBv))
#define QW_PICK(DTv) (pl.nb == 2 ? QW_PICK2(DTv, 2) : QW_PICK2(DTv, 1))
    fn = p.dtype == DT_BF16 ? QW_PICK(DT_BF16) : QW_PICK(DT_F16);
#undef QW_PICK
#undef QW_PICK2
#undef QW_PICK3
    if (!fn) return fail(ERR_UNSUPPORTED, "wide qmv: geometry not built");
    hipError_t e = set_max_dynamic_lds(fn, pl.lds);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    void* args[] = {&a};
    LaunchCtx l1 = lc, l2 = lc;
    if (pl.ksplit > 1) { l1.stop = nullptr; l2.start = nullptr; }
    e = launch_kernel(fn, dim3(pl.grid_x, pl.ksplit), dim3(1024), args, pl.lds, l1);
    if (e != hipSuccess) return hip_fail(e, "wide qmv kernel launch");
    if (pl.ksplit > 1) {
        const float* part = a.part;
        void* out = a.out;
        uint32_t total = p.M * p.N, ks = pl.ksplit;
        void* rargs[] = {&part, &out, &total, &ks};
        const void* rf = p.dtype == DT_BF16 ? (const void*)qmv_wide_reduce_kernel<DT_BF16> : (const void*)qmv_wide_reduce_kernel<DT_F16>;
        e = launch_kernel(rf, dim3((total + 255) / 256), dim3(256), rargs, 0, l2);
        if (e != hipSuccess) return hip_fail(e, "wide qmv reduce kernel launch");
    }
    return ERR_OK;
}

// Expert-routed rows (CSR offsets or one expert id per row) on the same kernel: blockIdx.y is the expert, whose rows
// are worked 16 per pass. Replaces mt_moe_gather_qmm_int4* (crates/metaltile-std/src/ffai/moe.rs:358-433) and the
// decode side of the per-row-id gathers with the same exact-dequant arithmetic as the GEMV family. Groups of 64 codes,
// rows of at most 4608 codes (no K slices: their partial rows would need the routing on the host).
const void* qmv_wide_gather_pick(int dtype, int mode, uint32_t nb, uint32_t sets);

int launch_qmv_wide_gather(const QmvParams& p, const LaunchCtx& lc) {
    const uint32_t G = p.group_size;
    if (p.gather != GATHER_CSR && p.gather != GATHER_INDICES) return fail(ERR_UNSUPPORTED, "wide gather: routing view");
    if ((p.dtype != DT_F16 && p.dtype != DT_BF16) || p.bits != 4 || G != 64) return fail(ERR_UNSUPPORTED, "wide gather: 4-bit g64 f16 / bf16");
    if (p.N == 0 || p.K == 0 || p.K % 512 || p.E == 0 || p.T == 0 || !p.route) return fail(ERR_UNSUPPORTED, "wide gather: shape");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16) return fail(ERR_UNSUPPORTED, "wide gather: alignment");
    if ((uint64_t)p.N * p.K / 2 >= (1ull << 32) || (uint64_t)p.E >= 65536) return fail(ERR_UNSUPPORTED, "wide gather: size");
    const uint32_t per_turn = wide_bytes_per_turn(G), turns = p.K / 512u;
    if (turns > (160u * 1024u - 64u) / per_turn) return fail(ERR_UNSUPPORTED, "wide gather: rows too long for one slice");
    QmvWPlan pl;
    pl.kslice = p.K;
    pl.ksplit = 1;
    pl.lds = (size_t)turns * per_turn;
    const uint32_t e_eff = p.E < p.T ? p.E : p.T;
    const uint32_t cus = (uint32_t)wide_cus(), want = cus / e_eff > 0 ? cus / e_eff : 1u;
    if (!wide_geometry(G, turns, (p.N + 15u) / 16u, want, pl)) return fail(ERR_UNSUPPORTED, "wide gather: geometry");
    if (p.gather == GATHER_INDICES) pl.lds += (size_t)p.T * 4;
    // (the kernel's statically allocated row counter shares the 160 KB with the dynamic part)
    if (pl.lds + 64 > 160 * 1024) return fail(ERR_UNSUPPORTED, "wide gather: the row list does not fit LDS");
    const void* fn = qmv_wide_gather_pick(p.dtype, p.gather, pl.nb, pl.sets);
    if (!fn) return fail(ERR_UNSUPPORTED, "wide gather: geometry not built");
    QmvWArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = (const uint16_t*)p.scales;
    a.biases = (const uint16_t*)p.biases;
    a.x = (const uint16_t*)p.x;
    a.out = p.out;
    a.part = nullptr;
    a.M = p.T;
    a.N = p.N;
    a.K = p.K;
    a.gpr = p.K / G;
    a.kslice = pl.kslice;
    a.kp = pl.kp;
    a.log2kp = pl.log2kp;
    a.tpk = pl.tpk;
    a.route = p.route;
    a.T = p.T;
    a.E = p.E;
    hipError_t e = set_max_dynamic_lds(fn, pl.lds);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    void* args[] = {&a};
    e = launch_kernel(fn, dim3(pl.grid_x, p.E), dim3(1024), args, pl.lds, lc);
    if (e != hipSuccess) return hip_fail(e, "wide gather kernel launch");
    return ERR_OK;
}

}  // namespace mtq

