// qmm for f32 operands on gfx950: batches of f32 activation rows on the f32 matrix cores.
//
// Replaces, for the f32 element type, the reference's batch kernels mt_qmm_mma / _m16 / _int8 /
// _int2 / _b3 / _b5 / _b6 (crates/metaltile-std/src/mlx/quantized.rs:2106, 2408, 2731, 3330,
// 3560-3900) and the multi-row GEMV forms mt_qmm / mt_qmm_b* (quantized.rs:1330-1500). With T = f32
// their rounding of s*q + b to T is the f32 rounding itself, so one kernel serves both families:
// w_hat = fma(s, q, b) in f32, products and sums in f32 on v_mfma_f32_32x32x2_f32.
//
// Layout of the work. A wave owns a 32-row x (32 * NB)-column block of the output over a slice of
// K; the NW (4 or 16) waves of a workgroup take every NW-th 64-k step of the same block and meet in
// LDS at the end. In the 32x32x2 operand layout lane l holds row (or column) l % 32 and k-half l / 32, so
// a lane reads exactly its own operands from global memory: 32 consecutive f32 of activation row
// l % 32 (one 128-byte line) and the 32 codes (4 * bits bytes) of weight row l % 32 of each column
// block, for k in [64 * step + 32 * (l / 32), +32). Nothing passes through LDS in the loop and no
// code is converted twice. Any code width 2..8 works: the 32 codes of a lane are `bits` whole words.
// Loads run one step ahead in a second register set.
#include "mtq_internal.h"
#include "qmm_common.h"

namespace mtq {

typedef __attribute__((ext_vector_type(16))) float qf_f32x16;
typedef __attribute__((ext_vector_type(4))) float qf_f32x4;

struct QmmFArgs {
    const unsigned char* w;
    const float* scales;
    const float* biases;
    const float* x;
    float* out;
    uint32_t M, N, K, gpr, log2g, steps, m_tiles, n_tiles, by_m;
    // expert-routed rows (GR): the table of row tiles, the row order, the experts' strides
    const uint32_t* tiles;
    const uint32_t* rowlist;
    uint64_t w_expert_bytes, sb_expert_elems;
    // split K (few tiles): workgroup (x, y) takes steps [y * steps_per_split, +steps_per_split) and writes
    // its partial tile to part[y][M][N]; qmm_f32_split_reduce_kernel adds the splits in order
    uint32_t ksplit, steps_per_split;
    float* part;
};

// code j of 32 codes of BITS bits packed LSB-first into BITS words; j is a constant after unrolling
template <int BITS> __device__ __forceinline__ uint32_t qf_code(const uint32_t* cw, int j) {
    const int o = j * BITS, lo = o >> 5, sh = o & 31;
    uint32_t v = cw[lo] >> sh;
    if (sh + BITS > 32) v |= cw[lo + 1] << (32 - sh);
    return v & ((1u << BITS) - 1u);
}

template <int BITS, int NB, int NW, bool GR = false>
__global__ __launch_bounds__(64 * NW) void qmm_f32_kernel(QmmFArgs a) {
    __shared__ float red[NW][NB * 16][64];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t fr = lane & 31u, fh = lane >> 5;

    // workgroup ids congruent mod 8 share an XCD: give each XCD a contiguous run of tiles
    const uint32_t total = a.m_tiles * a.n_tiles;
    uint32_t vid = blockIdx.x;
    if (!GR && total % 8 == 0) vid = (blockIdx.x & 7u) * (total / 8) + (blockIdx.x >> 3);
    uint32_t nt = a.by_m ? vid % a.n_tiles : vid / a.m_tiles, mt = a.by_m ? vid / a.n_tiles : vid % a.m_tiles;
    // rows of this tile: row j of the tile is row (row_first + j) of the row order, j < row_count
    uint32_t row_first = mt * 32, row_count = a.M > row_first ? min(32u, a.M - row_first) : 0u;
    if constexpr (GR) {
        nt = blockIdx.x % a.n_tiles;
        mt = blockIdx.x / a.n_tiles;
        if (mt >= a.tiles[0]) return;  // the grid is sized for the worst routing; the whole workgroup leaves
        const uint4 t = ((const uint4*)a.tiles)[1 + mt];
        row_first = t.y;
        row_count = t.z;
        a.w += (size_t)t.x * a.w_expert_bytes;
        a.scales += (size_t)t.x * a.sb_expert_elems;
        a.biases += (size_t)t.x * a.sb_expert_elems;
    }
    auto row_of = [&](uint32_t j) -> uint32_t {  // j < row_count
        if constexpr (GR) return a.rowlist ? a.rowlist[row_first + j] : row_first + j;
        else return row_first + j;
    };

    uint32_t step0 = 0;  // first step of this workgroup's share of K
    if (!GR && a.ksplit > 1) {
        step0 = blockIdx.y * a.steps_per_split;
        a.steps = min(a.steps_per_split, a.steps - step0);
    }
    // rows and columns past the edge are worked on the last one and not stored
    const uint32_t row = row_of(min(fr, row_count - 1));
    const float* xp = a.x + (size_t)row * a.K + 32 * fh + (size_t)step0 * 64;
    const unsigned char* wp[NB];
    const float* sp[NB];
    const float* bp[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const uint32_t n = min((nt * NB + nb) * 32 + fr, a.N - 1);
        wp[nb] = a.w + (size_t)n * ((size_t)a.K * BITS / 8) + fh * 4 * BITS + (size_t)step0 * (8 * BITS);
        sp[nb] = a.scales + (size_t)n * a.gpr;
        bp[nb] = a.biases + (size_t)n * a.gpr;
    }

    qf_f32x4 px[2][8];
    uint32_t pw[2][NB][BITS];
    float ps[2][NB], pb[2][NB];
    auto load = [&](uint32_t step, int set) {
        step = min(step, a.steps - 1);
        const float* xs = xp + (size_t)step * 64;
#pragma unroll
        for (int i = 0; i < 8; i++) px[set][i] = *(const qf_f32x4*)(xs + 4 * i);
        const uint32_t g = ((step0 + step) * 64 + 32 * fh) >> a.log2g;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const uint32_t* ws = (const uint32_t*)(wp[nb] + (size_t)step * (8 * BITS));
#pragma unroll
            for (int i = 0; i < BITS; i++) pw[set][nb][i] = ws[i];
            ps[set][nb] = sp[nb][g];
            pb[set][nb] = bp[nb][g];
        }
    };

    // two accumulators per column block (even and odd k): consecutive MFMAs never wait on each other
    qf_f32x16 acc[NB][2];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[nb][h][v] = 0.f;

    auto work = [&](int set) {
#pragma unroll
        for (int j = 0; j < 32; j++) {
            const float xv = px[set][j >> 2][j & 3];
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                const float wv = __builtin_fmaf(ps[set][nb], (float)qf_code<BITS>(pw[set][nb], j), pb[set][nb]);
                acc[nb][j & 1] = __builtin_amdgcn_mfma_f32_32x32x2f32(xv, wv, acc[nb][j & 1], 0, 0, 0);
            }
        }
    };

    // steps wave, wave + NW, ... ; loads past the end re-read the last step, their work is skipped by a
    // wave-uniform test
    load(wave, 0);
    for (uint32_t s0 = wave; s0 < a.steps; s0 += 2 * NW) {
        load(s0 + NW, 1);
        work(0);
        load(s0 + 2 * NW, 0);
        if (s0 + NW < a.steps) work(1);
    }

    // the waves' K-slices meet in LDS; wave w adds (in wave order) and stores accumulator values
    // [w * 16 / NW, +16 / NW) of every column block. Accumulator layout: column lane % 32,
    // row 8 * (v / 4) + 4 * (lane / 32) + v % 4.
    constexpr int VPW = 16 / NW;
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int v = 0; v < 16; v++) red[wave][nb * 16 + v][lane] = acc[nb][0][v] + acc[nb][1][v];
    __syncthreads();
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const uint32_t col = (nt * NB + nb) * 32 + fr;
#pragma unroll
        for (int i = 0; i < VPW; i++) {
            const uint32_t v = wave * VPW + i;
            float r = red[0][nb * 16 + v][lane];
#pragma unroll
            for (int u = 1; u < NW; u++) r += red[u][nb * 16 + v][lane];
            const uint32_t lrow = 8 * (v / 4) + 4 * fh + (v % 4);
            if (lrow < row_count && col < a.N) {
                if (!GR && a.ksplit > 1) a.part[((size_t)blockIdx.y * a.M + row_first + lrow) * a.N + col] = r;
                else a.out[(size_t)row_of(lrow) * a.N + col] = r;
            }
        }
    }
}

// Adds the K splits' partial tiles in split order.
__global__ __launch_bounds__(256) void qmm_f32_split_reduce_kernel(const float* part, float* out, uint32_t total, uint32_t ksplit) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float r = part[i];
    for (uint32_t sp = 1; sp < ksplit; sp++) r += part[(size_t)sp * total + i];
    out[i] = r;
}

// K splits for a shape: tiles of 32 x 32 fewer than the compute units and rows long enough to give
// every split 16 steps (4096 x 4096, 32 rows: 128 tiles, the MFMA work of 128 compute units).
static uint32_t f32_ksplit(const QmmParams& p, int cus) {
    const uint64_t tiles = (uint64_t)((p.M + 31) / 32) * ((p.N + 31) / 32);
    const uint32_t steps = p.K / 64;
    if (options().qmm_ksplit == 1 || tiles * 2 > (uint64_t)cus || steps < 32 || (uint64_t)p.M * p.N >= (1ull << 31)) return 1;
    uint32_t ks = options().qmm_ksplit > 1 ? (uint32_t)options().qmm_ksplit : (uint32_t)((uint64_t)cus / tiles);
    if (ks > steps / 16) ks = steps / 16;
    if (ks > 8) ks = 8;
    return ks < 1 ? 1 : ks;
}

size_t qmm_f32_scratch_bytes(const QmmParams& p) {
    if (p.dtype != DT_F32 || p.K % 64 || p.M == 0 || p.N == 0) return 0;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const uint32_t ks = f32_ksplit(p, cus);
    return ks > 1 ? (size_t)ks * p.M * p.N * sizeof(float) : 0;
}

int launch_qmm_f32(const QmmParams& p, const LaunchCtx& lc, void* scratch) {
    const uint32_t G = p.group_size;
    if (p.dtype != DT_F32) return fail(ERR_UNSUPPORTED, "f32 qmm: element type");
    if (p.M == 0 || p.N == 0 || p.K == 0 || p.K % 64 || G < 32 || (G & (G - 1)) || p.K % G)
        return fail(ERR_UNSUPPORTED, "f32 qmm: K % 64 or group size");
    if (p.bits < 2 || p.bits > 8) return fail(ERR_UNSUPPORTED, "f32 qmm: code width");
    if ((uintptr_t)p.w % 4 || (uintptr_t)p.x % 16 || (uintptr_t)p.out % 4 || (uintptr_t)p.scales % 4 || (uintptr_t)p.biases % 4)
        return fail(ERR_UNSUPPORTED, "f32 qmm: operand alignment");
    QmmFArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = (const float*)p.scales;
    a.biases = (const float*)p.biases;
    a.x = (const float*)p.x;
    a.out = (float*)p.out;
    a.M = p.M;
    a.N = p.N;
    a.K = p.K;
    uint32_t l = 0;
    while ((1u << l) < G) l++;
    a.log2g = l;
    a.gpr = p.K / G;
    a.steps = p.K / 64;
    a.tiles = nullptr;
    a.rowlist = nullptr;
    a.w_expert_bytes = a.sb_expert_elems = 0;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    uint32_t ks = f32_ksplit(p, cus);
    if (ks > 1 && !scratch) ks = 1;
    a.steps_per_split = (a.steps + ks - 1) / ks;
    a.ksplit = (a.steps + a.steps_per_split - 1) / a.steps_per_split;  // no empty split
    a.part = (float*)scratch;
    a.m_tiles = (p.M + 31) / 32;
    // two column blocks per wave halve the activation traffic; taken once that still leaves two
    // workgroups for every compute unit. Below that, and with rows long enough to give every wave
    // work, while the blocks leave compute units idle anyway, 16 waves share a block: four waves per
    // SIMD hide each other's load latency (4096 x 4096, 32 rows: 42 us with 4 waves, 32 us with 16;
    // 128 rows: 62 us with 4 waves, 67 us with 16).
    const int nb = (uint64_t)a.m_tiles * ((p.N + 63) / 64) >= 2 * (uint64_t)cus ? 2 : 1;
    const int nw = (nb == 1 && a.steps_per_split >= 32 && (uint64_t)a.m_tiles * ((p.N + 31) / 32) * a.ksplit <= (uint64_t)cus) ? 16 : 4;
    a.n_tiles = (p.N + 32 * nb - 1) / (32 * nb);
    if ((uint64_t)a.m_tiles * a.n_tiles >= (1ull << 31)) return fail(ERR_UNSUPPORTED, "f32 qmm: too many tiles");
    const uint64_t x_bytes = (uint64_t)p.M * p.K * 4, w_bytes = (uint64_t)p.N * p.K * p.bits / 8;
    a.by_m = x_bytes > w_bytes;
    const void* fn = nullptr;
#define QF_PICK(B)                                                                              \
    case B:                                                                                     \
        fn = nb == 2 ? (const void*)qmm_f32_kernel<B, 2, 4>                                     \
             : nw == 16 ? (const void*)qmm_f32_kernel<B, 1, 16> : (const void*)qmm_f32_kernel<B, 1, 4>; \
        break;
    switch (p.bits) {
        QF_PICK(2)
        QF_PICK(3)
        QF_PICK(4)
        QF_PICK(5)
        QF_PICK(6)
        QF_PICK(7)
        QF_PICK(8)
    }
#undef QF_PICK
    void* args[] = {&a};
    if (a.ksplit > 1) {
        LaunchCtx l1 = lc, l2 = lc;
        l1.stop = nullptr;
        l2.start = nullptr;
        hipError_t e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles, a.ksplit), dim3(64 * nw), args, 0, l1);
        if (e != hipSuccess) return hip_fail(e, "f32 qmm kernel launch");
        const float* part = a.part;
        float* out = a.out;
        uint32_t total = a.M * a.N, nsp = a.ksplit;
        void* rargs[] = {&part, &out, &total, &nsp};
        e = launch_kernel((const void*)qmm_f32_split_reduce_kernel, dim3((total + 255) / 256), dim3(256), rargs, 0, l2);
        if (e != hipSuccess) return hip_fail(e, "f32 qmm split reduce kernel launch");
        return ERR_OK;
    }
    hipError_t e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles), dim3(64 * nw), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "f32 qmm kernel launch");
    return ERR_OK;
}

// x [T][K], out [T][N], stacked w / scales / biases [E][N][...]; route = CSR offsets [E + 1] or, with
// per_row_ids, one expert id per row (sorted by expert on the device). Rows of one expert share 32-row
// tiles; replaces, for T = f32, the reference's gather kernels (crates/metaltile-std/src/ffai/moe.rs:358,
// 2256 and their per-width forms).
int launch_qmm_f32_grouped(const QmmParams& p, const uint32_t* route, bool per_row_ids, uint32_t T, uint32_t E, void* scratch,
                           const LaunchCtx& lc) {
    const uint32_t G = p.group_size;
    if (p.dtype != DT_F32) return fail(ERR_UNSUPPORTED, "f32 grouped qmm: element type");
    if (T == 0 || p.N == 0 || p.K == 0 || p.K % 64 || G < 32 || (G & (G - 1)) || p.K % G)
        return fail(ERR_UNSUPPORTED, "f32 grouped qmm: K % 64 or group size");
    if (p.bits < 2 || p.bits > 8) return fail(ERR_UNSUPPORTED, "f32 grouped qmm: code width");
    if ((uintptr_t)p.w % 4 || (uintptr_t)p.x % 16 || (uintptr_t)p.out % 4 || (uintptr_t)p.scales % 4 || (uintptr_t)p.biases % 4)
        return fail(ERR_UNSUPPORTED, "f32 grouped qmm: operand alignment");
    if (((uint64_t)p.N * p.K * p.bits / 8) % 4) return fail(ERR_UNSUPPORTED, "f32 grouped qmm: expert stride");
    GatherTiles gt;
    int rc = build_gather_tiles(route, per_row_ids, T, E, 32u, scratch, lc, gt);
    if (rc) return rc;
    QmmFArgs a;
    a.w = (const unsigned char*)p.w;
    a.scales = (const float*)p.scales;
    a.biases = (const float*)p.biases;
    a.x = (const float*)p.x;
    a.out = (float*)p.out;
    a.M = T;
    a.N = p.N;
    a.K = p.K;
    uint32_t l = 0;
    while ((1u << l) < G) l++;
    a.log2g = l;
    a.gpr = p.K / G;
    a.steps = p.K / 64;
    a.ksplit = 1;
    a.steps_per_split = a.steps;
    a.part = nullptr;
    a.tiles = gt.tiles;
    a.rowlist = gt.rowlist;
    a.w_expert_bytes = (uint64_t)p.N * p.K * p.bits / 8;
    a.sb_expert_elems = (uint64_t)p.N * a.gpr;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    a.m_tiles = gt.max_tiles;
    const int nb = (uint64_t)((T + 31) / 32) * ((p.N + 63) / 64) >= 2 * (uint64_t)cus ? 2 : 1;
    a.n_tiles = (p.N + 32 * nb - 1) / (32 * nb);
    if ((uint64_t)a.m_tiles * a.n_tiles >= (1ull << 31)) return fail(ERR_UNSUPPORTED, "f32 grouped qmm: too many tiles");
    a.by_m = 1;
    const void* fn = nullptr;
#define QF_PICK(B)                                                                                                   \
    case B:                                                                                                          \
        fn = nb == 2 ? (const void*)qmm_f32_kernel<B, 2, 4, true> : (const void*)qmm_f32_kernel<B, 1, 4, true>;      \
        break;
    switch (p.bits) {
        QF_PICK(2)
        QF_PICK(3)
        QF_PICK(4)
        QF_PICK(5)
        QF_PICK(6)
        QF_PICK(7)
        QF_PICK(8)
    }
#undef QF_PICK
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles), dim3(256), args, 0, gt.last);
    if (e != hipSuccess) return hip_fail(e, "f32 grouped qmm kernel launch");
    return ERR_OK;
}

}  // namespace mtq
