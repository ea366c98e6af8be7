// qmm for gfx950, second tiling: weights go from global memory straight into
// MFMA operand registers; only the activation tile passes through LDS.
//
// Replaces the same reference kernels as qmm.hip (mt_qmm_mma / _m16 / _int8 /
// _m16_int8 / _int2, crates/metaltile-std/src/mlx/quantized.rs:2106-2405, 2408,
// 2731, 2990, 3330) with the same semantics: s*q + b is rounded to the element
// dtype before the multiply (quantized.rs:2267-2274), products accumulate in
// f32, the result is rounded on store.
//
// Why a second tiling. LDS on this part reads ~230 B/clk per compute unit but
// writes only ~70 B/clk, so a tile that writes both operands to LDS is bound by
// those writes; and at M = 512 a 128x128 tiling yields 128 workgroups for 256
// compute units. Here a workgroup of 512 threads (8 waves) owns a 64 (M) x 128
// (N) tile: 256 workgroups at M = 512. The eight waves are 2 K-groups x 4
// N-waves: per iteration of 128 k, K-group g takes k in [64g, 64g+64) and wave
// wn the weight rows [32wn, 32wn+32). A lane of the 32x32x16 MFMA layout (row
// l%32, k-half l/32) loads exactly its own 32 codes of that 64-k slice (one
// 4*bits-byte load), its row's scale and bias for that slice, converts eight
// codes per MFMA step and never shares them: no weight byte is written to LDS
// and no code is converted twice. The 64 x 128 activation tile is written to LDS
// once per iteration (32 bytes per thread) and read by every wave of the
// matching K-group. Two waves per SIMD (one of each K-group) let one wave's
// conversions run under the other's MFMAs. The K-groups' accumulators meet in
// LDS once, at the end.
//
// Loads run two iterations ahead (two register sets); the activation tile is
// double-buffered in LDS; one barrier per iteration. Workgroup ids are remapped
// so that an XCD (ids congruent mod 8) works on all M-tiles of a contiguous run
// of N-tiles: its L2 holds its slice of W once and X once.
#include "qmm_direct_impl.h"

namespace mtq {

// The kernel itself lives in qmm_direct_impl.h; the instances for 3-, 5-, 6- and 7-bit codes are built in
// qmm_direct_odd.hip (a translation unit of their own, so the two compile side by side).

// LDS of one workgroup: two activation tiles, the tile's scales and biases, and at the
// end the K-groups' partial sums followed by the element tile.
static size_t lds_need(uint32_t rows, uint32_t kg, uint32_t gpr, bool sbl) {
    const uint32_t dbn = kg == 1 ? 128 : 32 * (8 / kg), dbk = 64 * kg;
    size_t main_loop = 2 * (size_t)rows * (dbk * 2 + 16) + (sbl ? (size_t)2 * dbn * (gpr + 2) * 2 : 0);
    size_t epilogue = (size_t)(kg - 1) * rows * dbn * 4 + (size_t)rows * dbn * 2;
    return main_loop > epilogue ? main_loop : epilogue;
}

// Adds the K splits' partial tiles in split order and rounds to the element type.
template <int DT> __global__ __launch_bounds__(256) void qmm_split_reduce_kernel(const float* part, void* out, uint32_t total, uint32_t ksplit) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float r = part[i];
    for (uint32_t sp = 1; sp < ksplit; sp++) r += part[(size_t)sp * total + i];
    ((uint16_t*)out)[i] = f32_to_elem_bits<DT>(r);
}

// Shapes the load-to-LDS instances take: 4- or 8-bit codes, 2 K-groups, whole iterations of 128 k, whole 8-element
// vectors of scales per row, one launch (no K split, no expert routing), and the ring of tiles beside the tile's
// scales and biases within the 160 KB.
// Returns 0 (not taken), 1 (the tile's whole rows of scales and biases in LDS) or 2 (two windows of 32 groups,
// refilled along K: rows too long for 1; groups of 64 or 128 codes).
static int dma_mode(int bits, uint32_t rows, uint32_t kgroups, uint32_t K, uint32_t gpr) {
    if (options().qmm_dma == 1 || (bits != 4 && bits != 8) || kgroups != 2 || K % 128 || gpr % 2) return 0;
    if (rows != 64 && rows != 128 && rows != 256) return 0;
    // whole rows are staged as 8-group vectors; the windows take them two groups at a time (K = 11008 at g64: 172 groups)
    if (options().qmm_dma != 2 && gpr % 8 == 0 && qmm_dma_lds_bytes(rows, gpr, false, false) <= 160 * 1024) return 1;
    const uint32_t G = K / gpr;
    if (bits == 8 && rows == 256) return 0;   // that instance does not fit the register file
    return (G == 64 || G == 128) && gpr >= 32 ? 2 : 0;
}
static bool dma_fits(int bits, uint32_t rows, uint32_t kgroups, uint32_t K, uint32_t gpr) { return dma_mode(bits, rows, kgroups, K, gpr) != 0; }

// K-split load-to-LDS instances on 2 K-groups (64 x 128 and 128 x 128 tiles): every split stages its own share of
// the tile's scales and biases (whole 8-group vectors, or pairs of groups where rows are not whole vectors) beside the
// ring of three tiles. Returns the LDS bytes, or 0
// where the shape is not taken.
static size_t dma_split_lds(int bits, uint32_t rows, uint32_t kgroups, uint32_t K, uint32_t gpr, uint32_t iters_per_split, uint32_t ksplit) {
    if (options().qmm_dma == 1 || (bits != 4 && bits != 8) || kgroups != 2 || K % 128 || gpr % 2 || ksplit < 2) return 0;
    if (rows != 64 && rows != 128) return 0;
    const uint32_t G = K / gpr, iters = K / 128;
    uint32_t most = 0;   // the kernel's own count of groups per split, at its largest
    for (uint32_t sp = 0; sp < ksplit; sp++) {
        const uint32_t it0 = sp * iters_per_split, its = iters - it0 < iters_per_split ? iters - it0 : iters_per_split;
        const uint32_t al = gpr % 8 ? 1u : 7u;
        const uint32_t g0 = (it0 * 128 / G) & ~al, ng_all = ((((it0 + its) * 128 - 1) / G + 1 - g0) + al) & ~al;
        const uint32_t ng = ng_all < gpr - g0 ? ng_all : gpr - g0;
        most = ng > most ? ng : most;
    }
    const size_t need = qmm_dma_split_lds_bytes(rows, most);
    return need <= 160 * 1024 ? need : 0;
}

template <int DT> static int launch_dt(QmmDArgs& a, int bits, uint32_t kgroups, const LaunchCtx& lc, bool grouped = false) {
    const void* fn = nullptr;
    // 8-bit codes on short rows gain nothing where the launch leaves compute units idle (14336 x 4096, 128 rows:
    // 36.3 against 34.3 us) or on the 4-K-group tiles (4096 x 4096, 16 / 64 rows 11.6 / 15.3 against 10.9 / 14.6;
    // 4096 x 14336 20.2 / 28.7 against 31.6 / 37.4): those stay on the register-staged instances
    const bool b8_short = bits == 8 && a.K < 8192 && options().qmm_dma < 2;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (const size_t shmem = grouped ? 0 : dma_split_lds(bits, a.m_tile_rows, kgroups, a.K, a.gpr, a.iters_per_split, a.ksplit)) {
        fn = qmm_dma_split_pick(bits, DT, a.m_tile_rows);
        hipError_t e = set_max_dynamic_lds(fn, shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
        void* args[] = {&a};
        LaunchCtx l1 = lc, l2 = lc;
        l1.stop = nullptr;
        l2.start = nullptr;
        e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles, a.ksplit), dim3(512), args, shmem, l1);
        if (e != hipSuccess) return hip_fail(e, "qmm load-to-LDS kernel launch");
        const float* part = a.part;
        void* out = a.out;
        uint32_t total = a.M * a.N, ks = a.ksplit;
        void* rargs[] = {&part, &out, &total, &ks};
        e = launch_kernel((const void*)qmm_split_reduce_kernel<DT>, dim3((total + 255) / 256), dim3(256), rargs, 0, l2);
        if (e != hipSuccess) return hip_fail(e, "qmm split reduce kernel launch");
        return ERR_OK;
    }
    if (a.ksplit <= 1 && dma_fits(bits, a.m_tile_rows, kgroups, a.K, a.gpr) && (!grouped || a.m_tile_rows == 64) &&
        !(b8_short && !grouped && a.m_tile_rows != 256 && (uint64_t)a.m_tiles * a.n_tiles < (uint64_t)cus)) {
        const bool windowed = dma_mode(bits, a.m_tile_rows, kgroups, a.K, a.gpr) == 2;
        const bool shallow = grouped || (uint64_t)a.m_tiles * a.n_tiles > (uint64_t)cus;
        fn = qmm_dma_pick(bits, DT, a.m_tile_rows, grouped, windowed, shallow);
        const size_t shmem = qmm_dma_lds_bytes(a.m_tile_rows, a.gpr, windowed, shallow);
        hipError_t e = set_max_dynamic_lds(fn, (size_t)shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
        void* args[] = {&a};
        e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles), dim3(512), args, shmem, lc);
        if (e != hipSuccess) return hip_fail(e, "qmm load-to-LDS kernel launch");
        return ERR_OK;
    }
    // The same transport on the 4-K-group tilings of few rows (32 x 64 and 64 x 64 tiles, plain, K-split or grouped
    // by expert): bit-equal results; 4096 x 14336, 16 / 32 / 64 / 128 rows 23.7 / 24.8 / 29.0 / 46.5 -> 16.0 / 17.6 /
    // 22.9 / 34.0 us, 14336 x 4096 15.4 / 15.9 / 21.5 / 28.8 -> 13.9 / 14.3 / 19.0 / 27.0, 4096 x 4096 128 / 256 rows
    // 17.1 / 20.9 -> 16.3 / 17.1 (64 rows and fewer: the same within 1 %).
    if (options().qmm_dma != 1 && (bits == 4 || bits == 8) && !b8_short && kgroups == 4 && (a.m_tile_rows == 32 || a.m_tile_rows == 64) && a.K % 256 == 0 &&
        a.gpr % 8 == 0 && qmm_dma4_lds_bytes(a.m_tile_rows, a.gpr) <= 160 * 1024 && !(grouped && a.ksplit > 1)) {
        const bool split = a.ksplit > 1;
        fn = qmm_dma4_pick(bits, DT, a.m_tile_rows, split, grouped);
        const size_t shmem = qmm_dma4_lds_bytes(a.m_tile_rows, a.gpr);
        hipError_t e = set_max_dynamic_lds(fn, (size_t)shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
        void* args[] = {&a};
        LaunchCtx l1 = lc, l2 = lc;
        if (split) { l1.stop = nullptr; l2.start = nullptr; }
        e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles, split ? a.ksplit : 1), dim3(512), args, shmem, l1);
        if (e != hipSuccess) return hip_fail(e, "qmm load-to-LDS kernel launch");
        if (split) {
            const float* part = a.part;
            void* out = a.out;
            uint32_t total = a.M * a.N, ks = a.ksplit;
            void* rargs[] = {&part, &out, &total, &ks};
            e = launch_kernel((const void*)qmm_split_reduce_kernel<DT>, dim3((total + 255) / 256), dim3(256), rargs, 0, l2);
            if (e != hipSuccess) return hip_fail(e, "qmm split reduce kernel launch");
        }
        return ERR_OK;
    }
    if (a.m_tile_rows == 256) return fail(ERR_UNSUPPORTED, "direct qmm: 256-row tiles need 4- or 8-bit codes, K % 128 == 0 and rows whose scales fit LDS (or, 4-bit codes, groups of 64 or 128 codes)");
    const bool tall = a.m_tile_rows == 128;
    const uint32_t dbn = kgroups == 1 ? 128 : 32 * (8 / kgroups);
    // scales and biases of the tile's rows in LDS when they fit beside the activation tiles
    const bool sbl = a.gpr % 8 == 0 && (size_t)2 * dbn * (a.gpr + 2) * 2 <= 48 * 1024;
    const size_t shmem = lds_need(a.m_tile_rows, kgroups, a.gpr, sbl);
    if (shmem > 160 * 1024) return fail(ERR_UNSUPPORTED, "direct qmm: tile does not fit in LDS");
#define QD_PICK3(B, MBv, KGv) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, MBv, true, KGv> : (const void*)qmm_direct_kernel<DT, B, 2, MBv, false, KGv>)
#define QD_PICK(B)                                                                      \
    fn = kgroups == 4   ? (tall ? QD_PICK3(B, 4, 4) : a.m_tile_rows == 32 ? QD_PICK3(B, 1, 4) : QD_PICK3(B, 2, 4)) \
         : kgroups == 1 ? (tall ? QD_PICK3(B, 4, 1) : QD_PICK3(B, 2, 1))                \
                        : (tall ? QD_PICK3(B, 4, 2) : QD_PICK3(B, 2, 2))
    const bool odd = bits != 2 && bits != 4 && bits != 8;
    switch (bits) {
        case 2: QD_PICK(2); break;
        case 4: QD_PICK(4); break;
        case 8: QD_PICK(8); break;
        default: fn = qmm_direct_pick_odd(DT, bits, kgroups, a.m_tile_rows, sbl, grouped, a.ksplit > 1); break;
    }
    if (a.ksplit > 1 && !grouped && !odd) {  // the K-split instances: the tilings qmm_direct_split_built() names
#define QD_S3(B, MBv, KGv) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, MBv, true, KGv, false, true> : (const void*)qmm_direct_kernel<DT, B, 2, MBv, false, KGv, false, true>)
#define QD_SPLIT(B) fn = kgroups == 4 ? (a.m_tile_rows == 32 ? QD_S3(B, 1, 4) : QD_S3(B, 2, 4)) : QD_S3(B, 4, 1)
        switch (bits) {
            case 2: QD_SPLIT(2); break;
            case 4: QD_SPLIT(4); break;
            default: QD_SPLIT(8); break;
        }
#undef QD_SPLIT
#undef QD_S3
    }
    if (!fn) return fail(ERR_UNSUPPORTED, "direct qmm: tiling not built for this code width");
#undef QD_PICK
#undef QD_PICK3
    if (grouped && !odd) {  // 64-row tiles, 2 or 4 K-groups
#define QD_G(B, KGv) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, 2, true, KGv, true> : (const void*)qmm_direct_kernel<DT, B, 2, 2, false, KGv, true>)
#define QD_G1(B) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, 1, true, 4, true> : (const void*)qmm_direct_kernel<DT, B, 2, 1, false, 4, true>)
        if (!(a.m_tile_rows == 64 && (kgroups == 2 || kgroups == 4)) && !(a.m_tile_rows == 32 && kgroups == 4))
            return fail(ERR_UNSUPPORTED, "grouped qmm: tile shape");
        switch (bits) {
            case 2: fn = a.m_tile_rows == 32 ? QD_G1(2) : kgroups == 4 ? QD_G(2, 4) : QD_G(2, 2); break;
            case 4: fn = a.m_tile_rows == 32 ? QD_G1(4) : kgroups == 4 ? QD_G(4, 4) : QD_G(4, 2); break;
            default: fn = a.m_tile_rows == 32 ? QD_G1(8) : kgroups == 4 ? QD_G(8, 4) : QD_G(8, 2); break;
        }
#undef QD_G1
#undef QD_G
    }
    hipError_t e = set_max_dynamic_lds(fn, (size_t)shmem);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    void* args[] = {&a};
    if (a.ksplit > 1 && !grouped) {
        LaunchCtx l1 = lc, l2 = lc;
        l1.stop = nullptr;
        l2.start = nullptr;
        e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles, a.ksplit), dim3(kgroups == 1 ? 256 : 512), args, shmem, l1);
        if (e != hipSuccess) return hip_fail(e, "qmm direct kernel launch");
        const float* part = a.part;
        void* out = a.out;
        uint32_t total = a.M * a.N, ks = a.ksplit;
        void* rargs[] = {&part, &out, &total, &ks};
        e = launch_kernel((const void*)qmm_split_reduce_kernel<DT>, dim3((total + 255) / 256), dim3(256), rargs, 0, l2);
        if (e != hipSuccess) return hip_fail(e, "qmm split reduce kernel launch");
        return ERR_OK;
    }
    e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles), dim3(kgroups == 1 ? 256 : 512), args, shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "qmm direct kernel launch");
    return ERR_OK;
}

// rows of k-iterations below which a K split is not worth its second launch
static constexpr uint32_t QMM_SPLIT_MIN_ITERS = 16;

// Tilings whose K-split instances are built: 32 x 64 and 64 x 64 on 4 K-groups, 128 x 128 on 1.
static bool qmm_direct_split_built(uint32_t rows, uint32_t kgroups) {
    return (kgroups == 4 && (rows == 32 || rows == 64)) || (kgroups == 1 && rows == 128);
}

struct QmmDPlan {
    uint32_t rows, kgroups, ksplit, iters_per_split;
};

// Checks the shape and picks the tile, the K-groups and the K split.
static int plan_direct(const QmmParams& p, QmmDPlan& pl) {
    if (p.dtype != DT_F16 && p.dtype != DT_BF16)
        return fail(ERR_UNSUPPORTED, "direct qmm: f16 / bf16 activations only");
    if (p.bits < 2 || p.bits > 8) return fail(ERR_UNSUPPORTED, "direct qmm: bits must be in 2..8");
    const bool odd_bits = p.bits != 2 && p.bits != 4 && p.bits != 8;
    const uint32_t G = p.group_size;
    if (p.M == 0 || p.N == 0 || p.K % 64 || G < 32 || (G & (G - 1)) || p.K % G)
        return fail(ERR_UNSUPPORTED, "direct qmm: K % 64 or group size");
    if ((uint64_t)p.M * p.K * 2 >= (1ull << 32) || (uint64_t)p.N * p.K * p.bits / 8 >= (1ull << 32))
        return fail(ERR_UNSUPPORTED, "direct qmm: operand larger than 4 GiB");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.out % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)
        return fail(ERR_UNSUPPORTED, "direct qmm: operands must be 16-byte aligned");
    // Tile choice, measured at N = K = 4096: 128 x 128 tiles (each converted weight
    // feeds 4 MFMAs) win once they fill the chip (M >= 1024: 42-47 us against 50);
    // below that 64 x 128 (M = 512: 29 us against 37-42); and when even those leave
    // half the chip idle, 64 x 64 tiles on 4 K-groups (M = 128: 18.6 us against 26).
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const uint64_t tall_wide = (uint64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
    const uint64_t short_wide = (uint64_t)((p.M + 63) / 64) * ((p.N + 127) / 128);
    uint32_t rows = 64, kgroups = 2;
    // Few rows never take a taller tile than they fill, however many column tiles there are: a
    // 128-row tile for 16 rows streams the weights at a quarter of the rate (128256 x 4096, 16 rows:
    // 162 us on 128 x 128 tiles, 86 us on 32 x 64; 28672 x 8192: 72 against 38 us). Up to 64 rows the
    // 64 x 64 tiles on 4 K-groups stay ahead until there are more 128-column tiles than compute
    // units (28672 x 8192, 32 rows on 64-row tiles: 58 us against 68; 128256 x 4096: 132 against 85).
    if (p.M <= 32) { rows = 32; kgroups = 4; }
    else if (p.M <= 64) { rows = 64; kgroups = short_wide <= (uint64_t)cus ? 4 : 2; }
    else if (tall_wide >= 2 * (uint64_t)cus) { rows = 128; kgroups = 1; }  // two 4-wave workgroups per CU (M = 2048: 72-75 us against 80-84; M = 4096: 160-170 against 180-190)
    // Between one and two tall tiles per compute unit the 8-wave workgroups (one per compute unit) run
    // a second, mostly empty round unless the count is an exact multiple; the 4-wave ones share compute
    // units and do not (1024 rows: 5120 x 5120 100 -> 82 us, 6144 x 4096 79 -> 68, 5120 x 13824 316 -> 233;
    // 4096 x 4096, exactly 256 tiles, stays: 42.9 against 47.2).
    else if (tall_wide >= (uint64_t)cus) { rows = 128; kgroups = tall_wide % (uint64_t)cus == 0 ? 2 : 1; }
    // Long rows with too few 128 x 128 tiles for the chip (a down projection at 256..512 rows): the
    // tall tile on 4-wave workgroups with K split so that two of them share a compute unit beats the
    // 64-row tiles (512 rows, 4096 x 14336: 131 -> 95 us; 4096 x 11008: 99 -> 78; 5120 x 13824: 213 -> 114;
    // 384 rows, 8192 x 28672: 446 -> 305; at K = 4096 it loses, 29 -> 36).
    else if (p.M >= 256 && p.K >= 8192) { rows = 128; kgroups = 1; }
    // More 64 x 128 tiles than compute units but at most one 128 x 128 tile each: one round of tall
    // tiles instead of a second, part-empty round of short ones (4096 x 4096: 768 rows 43.5 -> 40.5 us,
    // 640 rows 42.2 -> 39.4; 6144 x 4096, 384 rows: 41.9 -> 38.6).
    else if (short_wide > (uint64_t)cus) { rows = 128; kgroups = 2; }
    else if (short_wide * 2 <= (uint64_t)cus) {  // few tiles: halve their width, and their height for up to 32 rows
        rows = p.M <= 32 ? 32 : 64;
        kgroups = 4;
    }
    // Shapes the load-to-LDS instances take, with enough 64 x 128 tiles for half the chip: the tile height with
    // the lowest estimate. A round of tiles (one per compute unit) costs, at K = 4096, 20.6 / 28.0 / 48.5 us on
    // 64- / 128- / 256-row tiles when at most half the compute units are busy, 16 / 35 / 45 % more when all are
    // (the clock drops under full matrix load), and another 15 / 10 / 0 % when more rounds follow. Measured at
    // 4096 x 4096: 384 rows 26.7 -> 22.9 us, 512 rows 28.7 -> 23.8, 768 rows 38.3 -> 31.6, 1024 rows 43.0 -> 37.8,
    // 1536 rows 68.7 -> 56.8, 2048 rows 79.2 -> 70.6, 4096 rows 152 -> 141; 14336 x 4096: 512 rows 75.3 -> 65.1,
    // 4096 rows 513 -> 459; 4096 x 8192, 512 rows: 61.1 -> 43.8.
    // (long rows that leave even the 64-row tiles short of one per compute unit keep the K-split tall tiles chosen
    // above: 300 rows, 4096 x 11008 63 us against 68, 4096 x 14336 79 against 81)
    const bool underfilled_long = p.M >= 256 && p.K > 8192 && short_wide < (uint64_t)cus;   // (at K = 8192 the 64-row tiles win: 300 rows 38 us against 49)
    if (p.M > 64 && short_wide * 2 > (uint64_t)cus && !underfilled_long && !options().qmm_tile_rows && !options().qmm_kgroups) {
        static const uint32_t heights[3] = {64, 128, 256};
        static const double base[3] = {20.6, 28.0, 48.5}, full[3] = {0.16, 0.35, 0.45}, more[3] = {1.15, 1.10, 1.0};
        double best = 0.0;
        // long rows leave room for 64-row tiles only: past two rounds of them the 128-row tiles on 4-wave workgroups
        // stay ahead (4096 x 8192, 2048 rows: 188 us against 203)
        const bool short_only = !dma_fits(p.bits, 128, 2, p.K, p.K / G) && short_wide > 2 * (uint64_t)cus;
        for (int i = 0; i < 3 && !short_only; i++) {
            if (!dma_fits(p.bits, heights[i], 2, p.K, p.K / G)) continue;
            const uint64_t tiles = (uint64_t)((p.M + heights[i] - 1) / heights[i]) * ((p.N + 127) / 128);
            const uint64_t whole = tiles / (uint64_t)cus, rest = tiles % (uint64_t)cus;
            double est = (double)whole * base[i] * (1.0 + full[i]) * (whole + (rest ? 1 : 0) > 1 ? more[i] : 1.0);
            if (rest) {
                double f = ((double)rest / cus - 0.5) * 2.0;
                f = f < 0.0 ? 0.0 : f;
                est += base[i] * (1.0 + full[i] * f);
            }
            if (best == 0.0 || est < best) { best = est; rows = heights[i]; kgroups = 2; }
        }
    }
    // Long rows and too few 128 x 128 tiles for the chip (a down projection at 100..512 rows): the load-to-LDS tall
    // tile with K split so that every compute unit has one workgroup. us, the choice above -> this one:
    // 4096 x 14336, 128 / 256 / 384 / 512 rows 36.3 / 60.7 / 82.0 / 97.4 -> 31.7 / 47.3 / 75.5 / 80.7 (8-bit codes
    // 44.5 / 72.7 / 96.7 / 116.9 -> 39.1 / 56.1 / 86.8 / 92.7); 4096 x 8192, 256 / 384 / 512 rows 39.8 / 43.4 / 50.9 ->
    // 31.3 / 40.4 / 48.4 (128 rows lose, 22.0 -> 24.3); 5120 x 13824, 128 / 256 / 384 rows 47.9 / 70.7 / 92.2 -> 37.4 /
    // 55.6 / 75.9; 8192 x 28672 (a split's scales fit LDS from 4 splits on), 128 / 256 rows 163.5 / 184.4 -> 84.7 / 156.7.
    uint32_t dma_ks = 0;
    if (!options().qmm_tile_rows && !options().qmm_kgroups && options().qmm_ksplit == 0 && p.K >= 8192 &&
        (p.M > 128 || (p.M > 96 && p.K > 8192)) && tall_wide * 2 <= (uint64_t)cus && (uint64_t)p.M * p.N < (1ull << 31)) {
        uint32_t ks = (uint32_t)((uint64_t)cus / tall_wide);
        ks = ks > 8 ? 8 : ks;
        for (int attempt = 0; attempt < 2 && !dma_ks && ks <= 8; attempt++, ks *= 2) {
            const uint32_t its = p.K / 128, ips = (its + ks - 1) / ks, eff = (its + ips - 1) / ips;
            if (eff >= 2 && dma_split_lds(p.bits, 128, 2, p.K, p.K / G, ips, eff)) dma_ks = ks;
        }
        if (dma_ks) { rows = 128; kgroups = 2; }
    }
    if (options().qmm_tile_rows) rows = (uint32_t)options().qmm_tile_rows;
    if (options().qmm_kgroups) kgroups = (uint32_t)options().qmm_kgroups;
    // An iteration covers 64 k per K-group: K must be a multiple of 64 * K-groups (an odd number of
    // iterations is fine). Rows that are not (K = 11008 = 43 * 256 is, 11072 = 173 * 64 is not for 2 or
    // 4 K-groups) take fewer K-groups.
    while (kgroups > 1 && p.K % (64u * kgroups)) {
        if (options().qmm_kgroups) return fail(ERR_BAD_ARG, "qmm.kgroups: K must be a multiple of 64 * K-groups");
        kgroups /= 2;
    }
    // the bit-stream widths are built with 128-row tiles on 1 K-group only
    if (odd_bits && rows == 128 && !options().qmm_kgroups) kgroups = 1;
    if (rows == 256 && !dma_fits(p.bits, 256, kgroups, p.K, p.K / G))
        return fail(ERR_BAD_ARG, "qmm.tile_rows 256 needs 4- or 8-bit codes, 2 K-groups, K % 128 == 0 and rows whose scales fit LDS (or, 4-bit codes, groups of 64 or 128 codes)");
    if (rows == 32 && kgroups != 4) {
        if (options().qmm_tile_rows) return fail(ERR_BAD_ARG, "qmm.tile_rows 32 needs 4 K-groups");
        rows = 64;
    }
    pl.rows = rows;
    pl.kgroups = kgroups;
    // Few tiles and long rows (a down projection at 9..64 rows: 4096 x 14336 gives 64 tiles for 256
    // compute units): K is cut into splits, one workgroup per (tile, split), whose f32 partial tiles a
    // second kernel adds in split order.
    const uint32_t tile_cols = kgroups == 1 ? 128 : 32 * (8 / kgroups);
    const uint64_t tiles = (uint64_t)((p.M + rows - 1) / rows) * ((p.N + tile_cols - 1) / tile_cols);
    const uint32_t iters = p.K / (64 * kgroups);
    uint32_t ks = 1;
    if (options().qmm_ksplit > 1) ks = (uint32_t)options().qmm_ksplit;
    else if (dma_ks) ks = dma_ks;
    else if (options().qmm_ksplit == 0 && rows == 128 && kgroups == 1 && p.K >= 8192 && tiles < 2 * (uint64_t)cus) {
        // tall tiles on long rows: splits to about two 4-wave workgroups per compute unit, rounded
        ks = (uint32_t)((4 * (uint64_t)cus / tiles + 1) / 2);
        if (ks > 8) ks = 8;
        if (ks > iters / 16) ks = iters / 16;
    } else if (options().qmm_ksplit == 0 && kgroups != 2 && tiles * 2 <= (uint64_t)cus && iters >= QMM_SPLIT_MIN_ITERS) {
        // one workgroup per compute unit, at least 4 iterations each (measured optimum: 4096 x 14336,
        // 32 rows, 64 tiles: 1 / 2 / 4 / 8 / 16 splits 57 / 34 / 23 / 27 / 32 us; 2048 x 8192, 32 tiles:
        // 23 / 17 / 12 / 11 / 12 us; 8192 x 28672, 128 tiles: 108 / 63 / 62 / 66 / 80 us)
        ks = (uint32_t)((kgroups == 1 ? 2 : 1) * (uint64_t)cus / tiles);  // two 4-wave workgroups share a compute unit
        if (ks > iters / 4) ks = iters / 4;
        if (ks > 16) ks = 16;
    }
    if (ks > iters) ks = iters;
    if (ks < 1 || (uint64_t)p.M * p.N >= (1ull << 31)) ks = 1;  // the reduction indexes the output with 32 bits
    pl.iters_per_split = (iters + ks - 1) / ks;
    pl.ksplit = (iters + pl.iters_per_split - 1) / pl.iters_per_split;  // no empty split
    if (!qmm_direct_split_built(rows, kgroups) && !dma_split_lds(p.bits, rows, kgroups, p.K, p.K / G, pl.iters_per_split, pl.ksplit)) {
        pl.ksplit = 1;
        pl.iters_per_split = iters;
    }
    return ERR_OK;
}

size_t qmm_direct_scratch_bytes(const QmmParams& p) {
    QmmDPlan pl;
    if (plan_direct(p, pl) != ERR_OK || pl.ksplit <= 1) return 0;
    return (size_t)pl.ksplit * p.M * p.N * sizeof(float);
}

int launch_qmm_direct(const QmmParams& p, const LaunchCtx& lc, void* scratch) {
    QmmDPlan pl;
    int rc = plan_direct(p, pl);
    if (rc) return rc;
    const uint32_t G = p.group_size, rows = pl.rows, kgroups = pl.kgroups;
    if (pl.ksplit > 1 && !scratch) return fail(ERR_BAD_ARG, "direct qmm: K split without a scratch buffer");
    QmmDArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = (const unsigned char*)p.scales;
    a.biases = (const unsigned char*)p.biases;
    a.x = (const unsigned char*)p.x;
    a.out = p.out;
    a.M = p.M;
    a.N = p.N;
    a.K = p.K;
    uint32_t l = 0;
    while ((1u << l) < G) l++;
    a.log2g = l;
    a.gpr = p.K / G;
    a.m_tile_rows = rows;
    // Workgroup ids congruent mod 8 share an XCD and its L2. Whichever operand is smaller is
    // streamed by every XCD and the larger one is split between them (activations larger than the
    // packed weights: 14336x4096 with 8192 rows 1116 -> 941 us, 4096x4096 with 4096 rows 166 -> 154).
    const uint64_t x_bytes = (uint64_t)p.M * p.K * 2, w_bytes = (uint64_t)p.N * p.K * p.bits / 8;
    a.by_m = options().qmm_by_m == 1 || (options().qmm_by_m == 0 && x_bytes > w_bytes);
    a.m_tiles = (p.M + rows - 1) / rows;
    const uint32_t tile_cols = kgroups == 1 ? 128 : 32 * (8 / kgroups);
    a.n_tiles = (p.N + tile_cols - 1) / tile_cols;  // the last one may hang over N
    a.iters = p.K / (64 * kgroups);
    a.ksplit = pl.ksplit;
    a.iters_per_split = pl.iters_per_split;
    a.part = (float*)scratch;
    a.tiles = nullptr;
    a.rowlist = nullptr;
    a.w_expert_bytes = a.sb_expert_elems = 0;
    return p.dtype == DT_BF16 ? launch_dt<DT_BF16>(a, p.bits, kgroups, lc) : launch_dt<DT_F16>(a, p.bits, kgroups, lc);
}

// ---- expert-routed rows on the tile kernel ---------------------------------------------------
// Builds the table of row tiles: for every expert, its rows in the row order cut into tiles of
// `tile_rows`. CSR routing follows the reference's rule (crates/metaltile-std/src/ffai/moe.rs:376-385):
// row t belongs to the first expert e with t < off[e + 1], rows past every offset to expert 0; so
// expert e owns [max(off[1..e]), min(off[e + 1], T)) and expert 0 also the tail [max(off), T).
// With tail_to_0 == 0 (offsets from the sort of per-row ids) rows past the last offset are rows
// whose id names no expert: they get no tile, so their output rows stay untouched.
struct TileTabArgs {
    const uint32_t* off;  // [E + 1]
    uint32_t* tiles;      // [4 + 4 * max_tiles]
    uint32_t E, T, tile_rows, max_tiles, tail_to_0;
};
__global__ __launch_bounds__(64) void gather_tiles_kernel(TileTabArgs a) {
    // One wave, 64 experts at a time: lane l takes expert base + l. The rule needs, per expert, the
    // largest offset before it (a running maximum) and the number of tiles before it (a running sum);
    // both are wave scans, carried from one batch of 64 to the next, so the table comes out in expert
    // order exactly as a serial walk would write it, without a chain of dependent loads.
    const uint32_t lane = threadIdx.x;
    uint32_t n = 0, mx = 0;  // carried: tiles so far, largest offset so far (wave-uniform)
    uint4* tab = (uint4*)a.tiles + 1;
    auto emit = [&](uint32_t first, uint32_t e, uint32_t lo, uint32_t hi) {
        uint32_t i = first;
        for (uint32_t r = lo; r < hi && i < a.max_tiles; r += a.tile_rows, i++) tab[i] = make_uint4(e, r, min(a.tile_rows, hi - r), 0u);
    };
    for (uint32_t base = 0; base < a.E; base += 64) {
        const uint32_t e = base + lane;
        const uint32_t o1 = e < a.E ? a.off[e + 1] : 0u;
        // inclusive running maximum over the lanes
        uint32_t pm = o1;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t t = __shfl_up(pm, d, 64);
            if (lane >= (uint32_t)d) pm = max(pm, t);
        }
        uint32_t before = __shfl_up(pm, 1, 64);  // largest offset of the earlier lanes of this batch
        before = lane == 0 ? mx : max(mx, before);
        const uint32_t lo = min(before, a.T), hi = min(o1, a.T);
        const uint32_t cnt = (e < a.E && hi > lo) ? (hi - lo + a.tile_rows - 1) / a.tile_rows : 0u;
        uint32_t ps = cnt;  // inclusive running sum of tile counts
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t t = __shfl_up(ps, d, 64);
            if (lane >= (uint32_t)d) ps += t;
        }
        if (cnt) emit(n + ps - cnt, e, lo, hi);
        n += __shfl(ps, 63, 64);
        mx = max(mx, __shfl(pm, 63, 64));
    }
    if (lane == 0) {
        if (a.tail_to_0 && mx < a.T) {
            const uint32_t cnt = (a.T - mx + a.tile_rows - 1) / a.tile_rows;
            emit(n, 0u, mx, a.T);
            n += cnt;
        }
        a.tiles[0] = min(n, a.max_tiles);
    }
}

// Row-tile height of a grouped launch: 64, or 32 (on 4 K-groups, K % 256 == 0) for large experts with at
// most 24 rows each on average, where the 64-row tiles are mostly padding (random routing, 12 / 24 rows per
// expert, 64- against 32-row tiles: 8 x 14336 x 4096 100 / 99 against 85 / 88 us, 8 x 4096 x 4096 43 / 42
// against 36 / 43). With more rows, or many small experts, the 32-row tiles lose (every weight is converted
// once per 32 rows instead of 64: 128 x 2048 x 768, 48 rows each: 75 against 137 us).
static uint32_t grouped_tile_rows(const QmmParams& p, uint32_t T, uint32_t E) {
    if (p.K % 256 || (p.bits != 2 && p.bits != 4 && p.bits != 8)) return 64u;
    if (options().qmm_tile_rows == 32) return 32u;
    if (options().qmm_tile_rows == 64) return 64u;
    return ((uint64_t)T <= 24ull * E && (uint64_t)p.N * p.K >= (1ull << 24)) ? 32u : 64u;
}

size_t qmm_grouped_scratch_bytes(uint32_t T, uint32_t E, bool sort_rows, uint32_t tile_rows) {
    const size_t max_tiles = (size_t)(T + tile_rows - 1) / tile_rows + E + 1;
    size_t b = 16 + max_tiles * 16;
    if (sort_rows) b += ((size_t)2 * T + E + 2 + 3) / 4 * 16;  // sorted row list, inverse permutation, offsets of E + 1 buckets
    return b;
}

// Sorts per-row ids by expert where needed and launches the tile table kernel into `scratch`
// (sized by qmm_grouped_scratch_bytes for the same tile_rows). `out.last` is the launch context for
// the kernel that consumes the table (it carries the caller's stop event).
int build_gather_tiles(const uint32_t* route, bool per_row_ids, uint32_t T, uint32_t E, uint32_t tile_rows, void* scratch,
                       const LaunchCtx& lc, GatherTiles& out) {
    if (E >= 2048) return fail(ERR_UNSUPPORTED, "grouped qmm: 2048 experts or more");
    const uint32_t max_tiles = (T + tile_rows - 1) / tile_rows + E + 1;
    uint32_t* tiles = (uint32_t*)scratch;
    const uint32_t* off = route;
    const uint32_t* rowlist = nullptr;
    LaunchCtx first = lc, mid = lc;
    out.last = lc;
    first.stop = nullptr;
    mid.start = mid.stop = nullptr;
    out.last.start = nullptr;
    bool started = false;
    if (per_row_ids) {
        uint32_t* sorted = tiles + 4 + (size_t)max_tiles * 4;
        uint32_t* inv = sorted + T;
        uint32_t* offs = inv + T;
        // one bucket more than experts: the sort clamps ids to its last bucket, which so collects the
        // rows whose id names no expert
        int rc = launch_moe_sort(route, T, 1, E + 1, sorted, inv, offs, first);
        if (rc) return rc;
        started = true;
        off = offs;
        rowlist = sorted;
    }
    TileTabArgs ta{off, tiles, E, T, tile_rows, max_tiles, per_row_ids ? 0u : 1u};
    void* targs[] = {&ta};
    hipError_t e = launch_kernel((const void*)gather_tiles_kernel, dim3(1), dim3(64), targs, 0, started ? mid : first);
    if (e != hipSuccess) return hip_fail(e, "gather tile table kernel launch");
    out.tiles = tiles;
    out.rowlist = rowlist;
    out.max_tiles = max_tiles;
    return ERR_OK;
}

// x [T][K], out [T][N], stacked w / scales / biases [E][N][...]; route = CSR offsets [E + 1] or,
// with per_row_ids, one expert id per row (sorted by expert here, on the device).
int launch_qmm_grouped(const QmmParams& p, const uint32_t* route, bool per_row_ids, uint32_t T, uint32_t E, void* scratch,
                       const LaunchCtx& lc) {
    if (p.dtype != DT_F16 && p.dtype != DT_BF16) return fail(ERR_UNSUPPORTED, "grouped qmm: f16 / bf16 only");
    if (p.bits < 2 || p.bits > 8) return fail(ERR_UNSUPPORTED, "grouped qmm: bits must be in 2..8");
    const uint32_t G = p.group_size;
    if (T == 0 || p.N == 0 || p.K % 128 || G < 32 || (G & (G - 1)) || p.K % G)
        return fail(ERR_UNSUPPORTED, "grouped qmm: K % 128 or group size");
    if ((uint64_t)T * p.K * 2 >= (1ull << 32) || (uint64_t)p.N * p.K * p.bits / 8 >= (1ull << 32) || (uint64_t)T * p.N * 2 >= (1ull << 34))
        return fail(ERR_UNSUPPORTED, "grouped qmm: operand too large");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.out % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)
        return fail(ERR_UNSUPPORTED, "grouped qmm: operands must be 16-byte aligned");
    // 32-row tiles (on 4 K-groups) where the experts' rows would leave the 64-row tiles mostly padding
    const uint32_t tile_rows = grouped_tile_rows(p, T, E);
    GatherTiles gt;
    int rc = build_gather_tiles(route, per_row_ids, T, E, tile_rows, scratch, lc, gt);
    if (rc) return rc;
    const uint32_t max_tiles = gt.max_tiles;
    uint32_t* tiles = gt.tiles;
    const uint32_t* rowlist = gt.rowlist;
    const LaunchCtx& last = gt.last;

    QmmDArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = (const unsigned char*)p.scales;
    a.biases = (const unsigned char*)p.biases;
    a.x = (const unsigned char*)p.x;
    a.out = p.out;
    a.M = T;
    a.N = p.N;
    a.K = p.K;
    uint32_t l = 0;
    while ((1u << l) < G) l++;
    a.log2g = l;
    a.gpr = p.K / G;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    // 64 x 128 tiles; 64 x 64 on 4 K-groups when that still leaves fewer tiles than compute units. Row
    // tiles: every expert's last tile is partial, half an expert's worth on average (128 experts x
    // 768 x 2048, 10 rows each: 68 us on 4 K-groups, 44 us on 2).
    const uint64_t row_tiles = (uint64_t)(T + 63) / 64 + (E < T ? E : T) / 2;
    uint32_t kgroups = (row_tiles * ((p.N + 127) / 128) * 2 <= (uint64_t)cus && p.K % 256 == 0) ? 4 : 2;
    if (tile_rows == 32) kgroups = 4;
    a.m_tile_rows = tile_rows;
    a.m_tiles = max_tiles;
    a.n_tiles = (p.N + 32 * (8 / kgroups) - 1) / (32 * (8 / kgroups));
    a.iters = p.K / (64 * kgroups);
    a.by_m = 1;
    a.ksplit = 1;
    a.iters_per_split = a.iters;
    a.part = nullptr;
    a.tiles = tiles;
    a.rowlist = rowlist;
    a.w_expert_bytes = (uint64_t)p.N * p.K * p.bits / 8;
    a.sb_expert_elems = (uint64_t)p.N * a.gpr;
    return p.dtype == DT_BF16 ? launch_dt<DT_BF16>(a, p.bits, kgroups, last, true) : launch_dt<DT_F16>(a, p.bits, kgroups, last, true);
}

}  // namespace mtq
