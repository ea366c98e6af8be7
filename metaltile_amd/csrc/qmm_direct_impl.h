// The register-operand tile kernel of qmm_direct.hip, in a header so that its instances can be spread
// over translation units. See qmm_direct.hip for the design.
#pragma once
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
    // split K (few tiles, long rows): workgroup (x, y) works iterations [y * iters_per_split, +iters_per_split)
    // of tile x and writes its f32 partial tile to part[y][M][N]; a second kernel adds the splits in order.
    uint32_t ksplit, iters_per_split;
    float* part;
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
template <int DT, int BITS, int PD, int MB, bool SBL, int KG, bool GR = false, bool SP = false>
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
    uint32_t it_base = 0;  // first iteration of this workgroup's share of K
    if constexpr (SP) {
        it_base = blockIdx.y * a.iters_per_split;
        a.iters = min(a.iters_per_split, a.iters - it_base);
        a.x += (size_t)it_base * (DBK * 2);
        a.w += (size_t)it_base * (DBK * BITS / 8);
    }
    // groups of scales / biases this workgroup needs: [sb_g0, sb_g0 + sb_ng), whole 8-element vectors
    const uint32_t sb_g0 = ((it_base * DBK) >> a.log2g) & ~7u;
    const uint32_t sb_ng = min(a.gpr - sb_g0, (((((it_base + a.iters) * DBK - 1) >> a.log2g) + 1 - sb_g0) + 7u) & ~7u);

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
    // this lane's row in the staged window, less the window's first group: indexed with absolute group numbers
    const int sbrow = (int)((wn * 32 + fr) * sbld) - (int)sb_g0;
    const uint32_t kofs_abs = it_base * DBK + kofs;  // k of this lane's codes counted from the start of the row

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
        } else if constexpr (BITS % 4 != 0) { /* 3-, 5-, 6-, 7-bit: BITS words, 4-byte aligned */ \
            _Pragma("unroll") for (int i = 0; i < BITS; i++) pw[SET][i] = ((const uint32_t*)ws_)[i]; \
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
            const uint32_t g_ = (it_ * DBK + kofs_abs) >> a.log2g;                       \
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
            const int g_ = (int)((min(it_, a.iters - 1) * DBK + kofs_abs) >> a.log2g);
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
        const uint32_t vpr = sb_ng / 8, nvec = DBN * vpr;
        for (uint32_t v = tid; v < nvec; v += NT) {
            const uint32_t row = v / vpr, c0 = (v - row * vpr) * 8;
            const uint32_t grow = min(n0 + row, a.N - 1);
            const q_u32x4 sv = *(const q_u32x4*)((const uint16_t*)a.scales + (size_t)grow * a.gpr + sb_g0 + c0);
            const q_u32x4 bv = *(const q_u32x4*)((const uint16_t*)a.biases + (size_t)grow * a.gpr + sb_g0 + c0);
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
                if constexpr (SP) {  // this split's f32 partial sums, 32 consecutive columns per half wave
                    const uint32_t col = n0 + wn * 32 + fr;
                    if (lrow < row_count && col < a.N) a.part[((size_t)blockIdx.y * a.M + row_first + lrow) * a.N + col] = r;
                } else {
                    otile[lrow * DBN + wn * 32 + fr] = f32_to_elem_bits<DT>(r);
                }
            }
    }
    if constexpr (SP) return;  // split instances end here: the second kernel rounds and stores
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

// Kernel for 3-, 5-, 6- and 7-bit codes (qmm_direct_odd.hip); null when the combination is not built.
const void* qmm_direct_pick_odd(int dtype, int bits, uint32_t kgroups, uint32_t tile_rows, bool sbl, bool grouped, bool split);
// The instances with load-to-LDS activation tiles (qmm_dma.hip, qmm_dma_b8.hip): 4- and 8-bit codes, 2 K-groups, 64 / 128 / 256 rows, K a
// multiple of 128, whole 8-element vectors of scales per row; nullptr for other tile heights.
// `windowed`: the scales and biases as two windows of 32 groups refilled along K (groups of 64 or 128 codes) instead of
// the tile's whole rows.
// `shallow` (64-row tiles): a ring of two tiles instead of three, two workgroups per compute unit; grouped launches
// always take it.
const void* qmm_dma_pick(int bits, int dtype, uint32_t tile_rows, bool grouped, bool windowed, bool shallow);
size_t qmm_dma_lds_bytes(uint32_t tile_rows, uint32_t gpr, bool windowed, bool shallow);
// The same on 4 K-groups (32 x 64 and 64 x 64 tiles, K a multiple of 256), plain or K-split.
size_t qmm_dma_split_lds_bytes(uint32_t tile_rows, uint32_t groups);
const void* qmm_dma_split_pick(int bits, int dtype, uint32_t tile_rows);
const void* qmm_dma4_pick(int bits, int dtype, uint32_t tile_rows, bool split, bool grouped);
size_t qmm_dma4_lds_bytes(uint32_t tile_rows, uint32_t gpr);

}  // namespace mtq
