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
#include "mtq_internal.h"
#include "qmm_common.h"

namespace mtq {

// Keeps memory operations from being moved across this point by the optimiser
// and the machine scheduler (loads must be issued a full iteration before the
// values are needed); emits no instruction.
#define QD_KEEP_ORDER()                     \
    do {                                    \
        asm volatile("" ::: "memory");      \
        __builtin_amdgcn_sched_barrier(0);  \
    } while (0)

struct QmmDArgs {
    const unsigned char* w;
    const unsigned char* scales;
    const unsigned char* biases;
    const unsigned char* x;
    void* out;
    uint32_t M, N, K;
    uint32_t log2g, gpr;
    uint32_t m_tiles, n_tiles, iters;
    uint32_t m_tile_rows;  // 32 (4 K-groups only), 64 or 128
    uint32_t by_m;         // consecutive workgroup ids walk the N-tiles of one M-tile (else the M-tiles of one N-tile)
    // grouped mode (expert-routed rows): tiles[0] = number of row tiles, then one uint4 per tile
    // (expert, first row of the tile in the row order, rows in the tile, 0); rowlist maps the row
    // order to rows of x / out (null: the identity). w / scales / biases are the stacked experts'.
    const uint32_t* tiles;
    const uint32_t* rowlist;
    uint64_t w_expert_bytes, sb_expert_elems;
};


// MB = 32-row activation blocks per wave (tile height DBM = 32*MB): every
// converted weight fragment feeds MB MFMAs, so the conversion cost per MFMA
// falls with MB; MB = 4 is the compute-bound shape, MB = 2 gives twice the
// workgroups for small M.
// SBL: the scales and biases of the tile's 128 weight rows are staged once in LDS
// (coalesced, one line per row) instead of being fetched per lane and iteration:
// a wave-wide 2-byte load from 32 different rows costs the L1 as many tag lookups
// as the weight load itself.
// KG: K-groups per workgroup (1, 2 or 4). For 2 and 4 the 8 waves are KG K-groups x 8/KG N-waves;
// the tile is 32*MB rows x 32*(8/KG) columns and an iteration covers 64*KG k. KG = 4
// halves the tile width, which doubles the number of 128-row tiles for small M.
// KG = 1 is the half-size workgroup: 4 waves, all N-waves of one K-group, 32*MB x 128 tile,
// 64 k per iteration and no partial sums to combine. Two such workgroups share a compute unit
// and are not in step with each other, so one's LDS traffic runs under the other's MFMAs.
template <int DT, int BITS, int PD, int MB, bool SBL, int KG, bool GR = false>
__global__ __launch_bounds__(KG == 1 ? 256 : 512) void qmm_direct_kernel(QmmDArgs a) {
    constexpr int NW = KG == 1 ? 4 : 8;      // waves
    constexpr int NT = 64 * NW;              // threads
    constexpr int NWV = NW / KG;             // N-waves
    constexpr int DBN = 32 * NWV, DBK = 64 * KG;
    constexpr int DLD = DBK * 2 + 16;        // LDS row stride in bytes
    constexpr int TPR = DBK * 2 / 32;        // threads per activation row (32 bytes each)
    constexpr int RS = NT / TPR;            // rows covered by one pass of the workgroup
    constexpr int DBM = 32 * MB;
    constexpr int DBUF = DBM * DLD;          // one activation tile
    constexpr int XV = DBM * DBK * 2 / NT / 16;  // 16-byte vectors of the tile per thread
    extern __shared__ __align__(16) unsigned char lds[];  // 2 * DBUF bytes
    // the epilogue needs DBM*DBN*(4+2) bytes: partial sums, then the element tile (checked on the host)

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t kg = wave / NWV, wn = wave % NWV;
    const uint32_t fr = lane & 31u, fh = lane >> 5;

    const uint32_t total = a.m_tiles * a.n_tiles;
    uint32_t vid = blockIdx.x;
    if (!GR && total % 8 == 0) vid = (blockIdx.x & 7u) * (total / 8) + (blockIdx.x >> 3);
    uint32_t nt = a.by_m ? vid % a.n_tiles : vid / a.m_tiles, mt = a.by_m ? vid / a.n_tiles : vid % a.m_tiles;
    // rows of this tile: row j of the tile is row (row_first + j) of the row order, j < row_count
    uint32_t row_first = mt * DBM, row_count = a.M > row_first ? min((uint32_t)DBM, a.M - row_first) : 0u;
    if constexpr (GR) {
        nt = blockIdx.x % a.n_tiles;
        mt = blockIdx.x / a.n_tiles;
        if (mt >= a.tiles[0]) return;  // the grid is sized for the worst routing
        const uint4 t = ((const uint4*)a.tiles)[1 + mt];
        row_first = t.y;
        row_count = t.z;
        a.w += (size_t)t.x * a.w_expert_bytes;
        a.scales += (size_t)t.x * a.sb_expert_elems * 2;
        a.biases += (size_t)t.x * a.sb_expert_elems * 2;
    }
    auto row_of = [&](uint32_t j) -> uint32_t {  // j < row_count
        if constexpr (GR) return a.rowlist ? a.rowlist[row_first + j] : row_first + j;
        else return row_first + j;
    };
    const uint32_t n0 = nt * DBN;

    // activations: thread t moves 32 bytes of row t/TPR (bytes [32*(t%TPR), +32) of the iteration's row)
    const uint32_t xr = tid / TPR, xc = tid % TPR;
    uint32_t xoff[XV / 2];
#pragma unroll
    for (int i = 0; i < XV / 2; i++) xoff[i] = row_of(min(xr + RS * i, row_count - 1)) * (a.K * 2) + xc * 32;
    // weights: row n0 + 32*wn + fr, codes [64*kg + 32*fh, +32) of the iteration
    // the last tile of a ragged N works its missing rows on row N - 1 and stores none of their columns
    const uint32_t wrow = min(n0 + wn * 32 + fr, a.N - 1);
    const uint32_t woff = wrow * (a.K * BITS / 8) + (kg * 64 + fh * 32) * BITS / 8;
    const uint32_t soff = wrow * a.gpr * 2;
    const uint32_t kofs = kg * 64 + fh * 32;  // k offset of this lane's codes inside an iteration

    // PD register sets: the loads of iteration it + PD are issued at the top of
    // iteration it, so PD iterations of work cover the memory latency.
    q_u32x4 px[PD][XV];
    uint32_t pw[PD][BITS];
    uint32_t ps[PD], pb[PD];
    // LDS after the two activation tiles: [DBN rows][gpr + 2] scales, then the same for biases
    const uint32_t sbld = a.gpr + 2;  // row stride in elements; (gpr + 2) / 2 dwords is odd for gpr % 4 == 0: rows spread over the banks
    uint16_t* sbS = (uint16_t*)(lds + 2 * DBUF);
    uint16_t* sbB = sbS + DBN * sbld;
    const uint32_t sbrow = (wn * 32 + fr) * sbld;

#define QD_LOAD(IT, SET)                                                                 \
    do {                                                                                 \
        const uint32_t it_ = min((uint32_t)(IT), a.iters - 1);                           \
        const unsigned char* xs_ = a.x + (size_t)it_ * (DBK * 2);                        \
        _Pragma("unroll") for (int i = 0; i < XV / 2; i++) {                             \
            px[SET][2 * i] = *(const q_u32x4*)(xs_ + xoff[i]);                           \
            px[SET][2 * i + 1] = *(const q_u32x4*)(xs_ + xoff[i] + 16);                  \
        }                                                                                \
        const unsigned char* ws_ = a.w + (size_t)it_ * (DBK * BITS / 8) + woff;          \
        if constexpr (BITS == 2) {                                                       \
            const uint2 t_ = *(const uint2*)(ws_);                                       \
            pw[SET][0] = t_.x;                                                           \
            pw[SET][1] = t_.y;                                                           \
        } else {                                                                         \
            _Pragma("unroll") for (int i = 0; i < BITS / 4; i++) {                       \
                const q_u32x4 t_ = *(const q_u32x4*)(ws_ + 16 * i);                      \
                pw[SET][4 * i] = t_.x;                                                   \
                pw[SET][4 * i + 1] = t_.y;                                               \
                pw[SET][4 * i + 2] = t_.z;                                               \
                pw[SET][4 * i + 3] = t_.w;                                               \
            }                                                                            \
        }                                                                                \
        if constexpr (!SBL) {                                                            \
            const uint32_t g_ = (it_ * DBK + kofs) >> a.log2g;                           \
            ps[SET] = *(const uint16_t*)(a.scales + soff + (size_t)g_ * 2);              \
            pb[SET] = *(const uint16_t*)(a.biases + soff + (size_t)g_ * 2);              \
        }                                                                                \
    } while (0)

#define QD_STORE_X(BUF, SET)                                                             \
    do {                                                                                 \
        unsigned char* d_ = lds + (BUF) * DBUF + xr * DLD + xc * 32;                     \
        _Pragma("unroll") for (int i = 0; i < XV / 2; i++) {                             \
            *(q_u32x4*)(d_ + RS * i * DLD) = px[SET][2 * i];                             \
            *(q_u32x4*)(d_ + RS * i * DLD + 16) = px[SET][2 * i + 1];                    \
        }                                                                                \
    } while (0)

    auto scale_bias = [&](uint32_t it_, int set, float& s_, float& b_) {
        if constexpr (SBL) {
            const uint32_t g_ = (min(it_, a.iters - 1) * DBK + kofs) >> a.log2g;
            s_ = elem_bits_to_f32<DT>(sbS[sbrow + g_]);
            b_ = elem_bits_to_f32<DT>(sbB[sbrow + g_]);
        } else {
            s_ = elem_bits_to_f32<DT>(ps[set]);
            b_ = elem_bits_to_f32<DT>(pb[set]);
        }
        // The loop runs whole pairs of iterations; with an odd count the one past the end works on
        // re-read operands and must add nothing: zero scale and bias make its weights zero.
        if (it_ >= a.iters) s_ = b_ = 0.f;
    };

    f32x16 acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0.f;

#pragma unroll
    for (int j = 0; j < PD; j++) QD_LOAD(j, j);
    QD_STORE_X(0, 0);
    if constexpr (SBL) {
        // DBN rows x gpr elements each of scales and biases, 16 bytes per load: vector v of
        // the tile covers elements [8*(v % vpr), +8) of row v / vpr
        const uint32_t vpr = a.gpr / 8, nvec = DBN * vpr;
        for (uint32_t v = tid; v < nvec; v += NT) {
            const uint32_t row = v / vpr, c0 = (v - row * vpr) * 8;
            const uint32_t grow = min(n0 + row, a.N - 1);
            const q_u32x4 sv = *(const q_u32x4*)((const uint16_t*)a.scales + (size_t)grow * a.gpr + c0);
            const q_u32x4 bv = *(const q_u32x4*)((const uint16_t*)a.biases + (size_t)grow * a.gpr + c0);
            uint32_t* ds = (uint32_t*)(sbS + row * sbld + c0);
            uint32_t* db = (uint32_t*)(sbB + row * sbld + c0);
            ds[0] = sv.x; ds[1] = sv.y; ds[2] = sv.z; ds[3] = sv.w;
            db[0] = bv.x; db[1] = bv.y; db[2] = bv.z; db[3] = bv.w;
        }
        __syncthreads();
    }
    // Software pipeline: the weights of iteration it+1 are converted while the
    // MFMAs of iteration it run, one conversion group behind every MFMA, so the
    // matrix cores and the vector ALU are busy at the same time inside one wave.
    uint4 bq[2][4];  // converted fragments: [it & 1][MFMA step]
    {
        float s0, b0;
        scale_bias(0, 0, s0, b0);
#pragma unroll
        for (int j = 0; j < 4; j++) bq[0][j] = dequant8<DT, BITS>(pw[0], j, s0, b0);
    }
    __syncthreads();

    // fragment of activation row (32*bi + fr), k = kofs + 8*j .. +8 of the iteration
    const unsigned char* Abase = lds + fr * DLD + kofs * 2;
    for (uint32_t it0 = 0; it0 < a.iters; it0 += PD) {
#pragma unroll
        for (int par = 0; par < PD; par++) {
            const uint32_t it = it0 + par;
            const int nx = (par + 1) % PD;  // set holding iteration it+1 (loaded PD-1 iterations ago)
            // set `par` held iteration `it`, whose weights were converted during iteration it-1
            // and whose activations are in LDS: refill it with iteration it+PD
            uint32_t cw[BITS];
#pragma unroll
            for (int i = 0; i < BITS; i++) cw[i] = pw[nx][i];
            float s, b;
            scale_bias(it + 1, nx, s, b);
            QD_LOAD(it + PD, par);
            QD_KEEP_ORDER();
            const unsigned char* A0 = Abase + (par & 1) * DBUF;
            // Activation fragments: all four MFMA steps' worth up front (fastest), or two
            // steps ahead of their use where the register file would not hold them all.
            constexpr bool kAllUpFront = !(MB == 4 && KG == 4);
            if constexpr (kAllUpFront) {
                uint4 af[4][MB];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int bi = 0; bi < MB; bi++) af[j][bi] = *(const uint4*)(A0 + bi * 32 * DLD + j * 16);
#pragma unroll
                for (int j = 0; j < 4; j++) {
#pragma unroll
                    for (int bi = 0; bi < MB; bi++) acc[bi] = mfma32<DT>(af[j][bi], bq[par & 1][j], acc[bi]);
                    bq[(par + 1) & 1][j] = dequant8<DT, BITS>(cw, j, s, b);
                }
                __builtin_amdgcn_sched_group_barrier(0x100, 4 * MB, 0);
            } else {
                uint4 af[2][MB];
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int bi = 0; bi < MB; bi++) af[j][bi] = *(const uint4*)(A0 + bi * 32 * DLD + j * 16);
#pragma unroll
                for (int j = 0; j < 4; j++) {
#pragma unroll
                    for (int bi = 0; bi < MB; bi++) acc[bi] = mfma32<DT>(af[j & 1][bi], bq[par & 1][j], acc[bi]);
                    if (j + 2 < 4) {
#pragma unroll
                        for (int bi = 0; bi < MB; bi++) af[j & 1][bi] = *(const uint4*)(A0 + bi * 32 * DLD + (j + 2) * 16);
                    }
                    bq[(par + 1) & 1][j] = dequant8<DT, BITS>(cw, j, s, b);
                }
            }
            // ask the scheduler for one MFMA followed by its share of the conversion's
            // vector instructions, 4*MB times
#pragma unroll
            for (int g = 0; g < 4 * MB; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, (96 + 4 * MB - 1) / (4 * MB), 0);
            }
            // activations of it+1 go to the other buffer
            QD_KEEP_ORDER();
            QD_STORE_X((par + 1) & 1, nx);
            __syncthreads();
        }
    }
#undef QD_LOAD
#undef QD_STORE_X

    // ---- the other K-groups hand their accumulators to K-group 0 through LDS ---
    float* red = (float*)lds;  // [kg - 1][wn][bi][v][lane]
    constexpr int GRP = NWV * MB * 16 * 64;  // floats per K-group
    if (kg != 0) {
#pragma unroll
        for (int bi = 0; bi < MB; bi++)
#pragma unroll
            for (int v = 0; v < 16; v++) red[(kg - 1) * GRP + ((wn * MB + bi) * 16 + v) * 64 + lane] = acc[bi][v];
    }
    __syncthreads();
    // accumulator layout: column j = lane%32, row i = 8*(v/4) + 4*(lane/32) + v%4.
    // K-group 0 adds, rounds to the element dtype and writes the tile to LDS as
    // [row][DBN columns], behind the partial sums.
    uint16_t* otile = (uint16_t*)(lds + (KG - 1) * GRP * 4);
    if (kg == 0) {
#pragma unroll
        for (int bi = 0; bi < MB; bi++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const uint32_t lrow = bi * 32 + 8 * (v / 4) + 4 * fh + (v % 4);
                float r = acc[bi][v];
#pragma unroll
                for (int g = 0; g < KG - 1; g++) r += red[g * GRP + ((wn * MB + bi) * 16 + v) * 64 + lane];
                otile[lrow * DBN + wn * 32 + fr] = f32_to_elem_bits<DT>(r);
            }
    }
    __syncthreads();
    // all threads store the tile, 16 bytes each, whole rows
    constexpr int VPR = DBN / 8;                    // 16-byte vectors per tile row
    constexpr int VPT = (DBM * VPR + NT - 1) / NT;  // vectors per thread
    if ((a.N & 7u) == 0) {
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const uint32_t v = tid + i * NT, lrow = v / VPR, col = n0 + (v % VPR) * 8;
            if (lrow < row_count && col < a.N)
                *(q_u32x4*)((uint16_t*)a.out + (size_t)row_of(lrow) * a.N + col) = *(const q_u32x4*)(otile + lrow * DBN + (v % VPR) * 8);
        }
    } else {
        // output rows that are not whole 16-byte vectors: element stores, neighbouring lanes on
        // neighbouring columns
        for (uint32_t e = tid; e < (uint32_t)(DBM * DBN); e += NT) {
            const uint32_t lrow = e / DBN, col = n0 + e % DBN;
            if (lrow < row_count && col < a.N) ((uint16_t*)a.out)[(size_t)row_of(lrow) * a.N + col] = otile[e];
        }
    }
}

// LDS of one workgroup: two activation tiles, the tile's scales and biases, and at the
// end the K-groups' partial sums followed by the element tile.
static size_t lds_need(uint32_t rows, uint32_t kg, uint32_t gpr, bool sbl) {
    const uint32_t dbn = kg == 1 ? 128 : 32 * (8 / kg), dbk = 64 * kg;
    size_t main_loop = 2 * (size_t)rows * (dbk * 2 + 16) + (sbl ? (size_t)2 * dbn * (gpr + 2) * 2 : 0);
    size_t epilogue = (size_t)(kg - 1) * rows * dbn * 4 + (size_t)rows * dbn * 2;
    return main_loop > epilogue ? main_loop : epilogue;
}

template <int DT> static int launch_dt(QmmDArgs& a, int bits, uint32_t kgroups, const LaunchCtx& lc, bool grouped = false) {
    const void* fn;
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
    switch (bits) {
        case 2: QD_PICK(2); break;
        case 4: QD_PICK(4); break;
        default: QD_PICK(8); break;
    }
#undef QD_PICK
#undef QD_PICK3
    if (grouped) {  // 64-row tiles, 2 or 4 K-groups
#define QD_G(B, KGv) (sbl ? (const void*)qmm_direct_kernel<DT, B, 2, 2, true, KGv, true> : (const void*)qmm_direct_kernel<DT, B, 2, 2, false, KGv, true>)
        if (a.m_tile_rows != 64 || (kgroups != 2 && kgroups != 4)) return fail(ERR_UNSUPPORTED, "grouped qmm: tile shape");
        switch (bits) {
            case 2: fn = kgroups == 4 ? QD_G(2, 4) : QD_G(2, 2); break;
            case 4: fn = kgroups == 4 ? QD_G(4, 4) : QD_G(4, 2); break;
            default: fn = kgroups == 4 ? QD_G(8, 4) : QD_G(8, 2); break;
        }
#undef QD_G
    }
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    void* args[] = {&a};
    e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles), dim3(kgroups == 1 ? 256 : 512), args, shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "qmm direct kernel launch");
    return ERR_OK;
}

int launch_qmm_direct(const QmmParams& p, const LaunchCtx& lc) {
    if (p.dtype != DT_F16 && p.dtype != DT_BF16)
        return fail(ERR_UNSUPPORTED, "direct qmm: f16 / bf16 activations only");
    if (p.bits != 2 && p.bits != 4 && p.bits != 8) return fail(ERR_UNSUPPORTED, "direct qmm: bits must be 2, 4 or 8");
    const uint32_t G = p.group_size;
    if (p.M == 0 || p.N == 0 || p.K % 64 || G < 32 || (G & (G - 1)) || p.K % G)
        return fail(ERR_UNSUPPORTED, "direct qmm: K % 64 or group size");
    if ((uint64_t)p.M * p.K * 2 >= (1ull << 32) || (uint64_t)p.N * p.K * p.bits / 8 >= (1ull << 32))
        return fail(ERR_UNSUPPORTED, "direct qmm: operand larger than 4 GiB");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.out % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)
        return fail(ERR_UNSUPPORTED, "direct qmm: operands must be 16-byte aligned");
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
    // Tile choice, measured at N = K = 4096: 128 x 128 tiles (each converted weight
    // feeds 4 MFMAs) win once they fill the chip (M >= 1024: 42-47 us against 50);
    // below that 64 x 128 (M = 512: 29 us against 37-42); and when even those leave
    // half the chip idle, 64 x 64 tiles on 4 K-groups (M = 128: 18.6 us against 26).
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const uint64_t tall_wide = (uint64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
    const uint64_t short_wide = (uint64_t)((p.M + 63) / 64) * ((p.N + 127) / 128);
    uint32_t rows = 64, kgroups = 2;
    if (tall_wide >= 2 * (uint64_t)cus) { rows = 128; kgroups = 1; }  // two 4-wave workgroups per CU (M = 2048: 72-75 us against 80-84; M = 4096: 160-170 against 180-190)
    else if (tall_wide >= (uint64_t)cus) { rows = 128; kgroups = 2; }
    else if (short_wide * 2 <= (uint64_t)cus) {  // few tiles: halve their width, and their height for up to 32 rows
        rows = p.M <= 32 ? 32 : 64;
        kgroups = 4;
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
    if (rows == 32 && kgroups != 4) {
        if (options().qmm_tile_rows) return fail(ERR_BAD_ARG, "qmm.tile_rows 32 needs 4 K-groups");
        rows = 64;
    }
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
    if (threadIdx.x != 0) return;  // E is small next to the GEMM that follows: one lane, in order
    uint32_t n = 0, mx = 0;
    uint4* tab = (uint4*)a.tiles + 1;
    auto emit = [&](uint32_t e, uint32_t lo, uint32_t hi) {
        for (uint32_t r = lo; r < hi && n < a.max_tiles; r += a.tile_rows, n++) tab[n] = make_uint4(e, r, min(a.tile_rows, hi - r), 0u);
    };
    for (uint32_t e = 0; e < a.E; e++) {
        const uint32_t lo = min(mx, a.T), hi = min(a.off[e + 1], a.T);
        if (hi > lo) emit(e, lo, hi);
        mx = max(mx, a.off[e + 1]);
    }
    if (a.tail_to_0 && mx < a.T) emit(0u, mx, a.T);
    a.tiles[0] = n;
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
    if (p.bits != 2 && p.bits != 4 && p.bits != 8) return fail(ERR_UNSUPPORTED, "grouped qmm: bits must be 2, 4 or 8");
    const uint32_t G = p.group_size;
    if (T == 0 || p.N == 0 || p.K % 128 || G < 32 || (G & (G - 1)) || p.K % G)
        return fail(ERR_UNSUPPORTED, "grouped qmm: K % 128 or group size");
    if ((uint64_t)T * p.K * 2 >= (1ull << 32) || (uint64_t)p.N * p.K * p.bits / 8 >= (1ull << 32) || (uint64_t)T * p.N * 2 >= (1ull << 34))
        return fail(ERR_UNSUPPORTED, "grouped qmm: operand too large");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.out % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)
        return fail(ERR_UNSUPPORTED, "grouped qmm: operands must be 16-byte aligned");
    GatherTiles gt;
    int rc = build_gather_tiles(route, per_row_ids, T, E, 64u, scratch, lc, gt);
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
    // 64 x 128 tiles; 64 x 64 on 4 K-groups when that still leaves fewer tiles than compute units
    uint32_t kgroups = ((uint64_t)((T + 63) / 64) * ((p.N + 127) / 128) * 2 <= (uint64_t)cus && p.K % 256 == 0) ? 4 : 2;
    a.m_tile_rows = 64;
    a.m_tiles = max_tiles;
    a.n_tiles = (p.N + 32 * (8 / kgroups) - 1) / (32 * (8 / kgroups));
    a.iters = p.K / (64 * kgroups);
    a.by_m = 1;
    a.tiles = tiles;
    a.rowlist = rowlist;
    a.w_expert_bytes = (uint64_t)p.N * p.K * p.bits / 8;
    a.sb_expert_elems = (uint64_t)p.N * a.gpr;
    return p.dtype == DT_BF16 ? launch_dt<DT_BF16>(a, p.bits, kgroups, last, true) : launch_dt<DT_F16>(a, p.bits, kgroups, last, true);
}

}  // namespace mtq
