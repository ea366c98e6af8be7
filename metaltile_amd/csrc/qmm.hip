// qmm for gfx950: Y[M,N] = X[M,K] * W_hat[N,K]^T with affine-quantized W,
// weight tiles dequantised into LDS and multiplied on the matrix cores.
//
// Replaces mt_qmm_mma / _m16 / _int8 / _m16_int8 / _int2
// (crates/metaltile-std/src/mlx/quantized.rs:2106-2405, 2408, 2731, 2990, 3330).
// Semantics follow that family: the dequantised weight s*q + b is rounded to
// the element dtype before the multiply (quantized.rs:2267-2274), products are
// accumulated in f32 (quantized.rs:2157-2168), the result is rounded to the
// element dtype on store.
//
// Tiling. One workgroup of 256 threads (4 waves, 2 x 2) computes a
// 128 (M) x 128 (N) tile of Y over a contiguous range of K; each wave owns
// 64 x 64 of it as four v_mfma_f32_32x32x16 accumulator blocks. Wide-N tiles
// are the cheap direction here: a weight column costs half a byte per k where
// an activation row costs two. K is walked in stages of 64; per stage the
// workgroup brings in
//   X: 128 rows x 64 elements (16 KB), four 16-byte loads per thread, each
//      row's 128 bytes coalesced, stored to LDS as is;
//   W: 128 rows x 64 codes, 32 codes per thread (one 4*bits-byte load) plus
//      that row's scale and bias; the thread turns its codes into elements
//      (byte extract, f32 FMA, round-to-nearest-even pack) and stores 64 bytes.
// Both LDS tiles use a 144-byte row stride, which makes the 16-byte per-lane
// fragment reads of the MFMA layout (lane l: row l%32, k-half l/32) bank-
// conflict free. Global loads run two stages ahead of the MFMAs through two
// register sets and a double-buffered LDS tile: one barrier per stage.
//
// When the tile count is below the number of compute units (M = 512 gives 128
// tiles), K is split across `splits` workgroups per tile. Each writes its f32
// partial tile to a library-owned scratch buffer and takes a ticket; the last
// arriver adds the partials in split order (so the sum does not depend on
// arrival order), stores the tile and resets the ticket counter.
//
// Workgroup ids are remapped so that the compute units of an XCD (ids
// congruent mod 8) work on consecutive N-tiles of one (split, M-tile) and share
// its X rows in that XCD's L2.
#include "mtq_internal.h"
#include "qmm_common.h"

namespace mtq {

struct QmmKArgs {
    const uint32_t* w;
    const uint16_t* scales;
    const uint16_t* biases;
    const uint16_t* x;
    uint16_t* out;
    float* scratch;        // [tiles][splits][64][256] partial accumulators
    uint32_t* tickets;     // [tiles], zero between launches
    uint32_t M, N, K;
    uint32_t log2g, gpr;
    uint32_t m_tiles, n_tiles, splits;
    uint32_t stages_per_split;
};

constexpr int QBM = 128, QBN = 128, QBK = 64;
constexpr int QLD = 144;                         // LDS row stride in bytes (64 elements * 2 + 16)
constexpr int QBUF = (QBM + QBN) * QLD;          // one stage: X tile then W tile
constexpr int QLDS = 2 * QBUF;

template <int DT, int BITS>
__global__ __launch_bounds__(256) void qmm_kernel(QmmKArgs a) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ uint32_t s_ticket;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;

    // XCD-aware order: ids congruent mod 8 share an XCD; give each XCD a
    // contiguous run of (split, m-tile, n-tile) triples with n fastest.
    const uint32_t tiles = a.m_tiles * a.n_tiles, total = tiles * a.splits;
    uint32_t vid = blockIdx.x;
    if (total % 8 == 0) vid = (blockIdx.x & 7u) * (total / 8) + (blockIdx.x >> 3);
    const uint32_t split = vid / tiles, tile = vid % tiles;
    const uint32_t mt = tile / a.n_tiles, nt = tile % a.n_tiles;
    const uint32_t m0 = mt * QBM, n0 = nt * QBN;
    const uint32_t stage0 = split * a.stages_per_split, stages = a.stages_per_split;

    // ---- per-thread global addresses ----------------------------------------
    // Every address is a wave-uniform base (advanced per stage on the scalar
    // unit) plus a per-lane 32-bit byte offset fixed for the whole kernel, so the
    // loop issues its loads without any vector address arithmetic.
    // X: 4 loads of 16 bytes; row tid/8 + 32*i, 16-byte chunk tid%8 of the stage's 128-byte row
    const uint32_t xr = tid >> 3, xc = tid & 7u;
    uint32_t xoff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) xoff[i] = min(m0 + xr + 32 * i, a.M - 1) * (a.K * 2) + xc * 16;
    // W: row n0 + tid/2, codes [32*(tid%2), +32) of the stage
    const uint32_t wrow = min(n0 + (tid >> 1), a.N - 1), wq = tid & 1u;
    const uint32_t woff = wrow * (a.K * BITS / 8) + wq * (4 * BITS);
    // scale / bias: group of this thread's 32 codes = (stage*64 + wq*32) / G
    const bool half_groups = a.log2g == 5;  // G = 32: the two halves of a stage are two groups
    const uint32_t soff = (wrow * a.gpr + (half_groups ? wq : 0u)) * 2;
    const unsigned char* xb = (const unsigned char*)a.x;
    const unsigned char* wb = (const unsigned char*)a.w;
    const unsigned char* sb = (const unsigned char*)a.scales;
    const unsigned char* bb = (const unsigned char*)a.biases;

    // Prefetch registers: two sets, indexed only by compile-time constants so
    // they stay in VGPRs. Stage t uses set t%2.
    q_u32x4 px[2][4];
    uint32_t pw[2][BITS];  // 32 codes = BITS dwords
    uint32_t ps[2], pb[2];

    // Loads past the last stage re-read the last one (harmless, keeps the loop branch-free).
#define QMM_LOAD_STAGE(S, SET)                                                          \
    do {                                                                                \
        const uint32_t st_ = stage0 + min((uint32_t)(S), stages - 1);                   \
        const unsigned char* xs_ = xb + (size_t)st_ * (QBK * 2);                        \
        _Pragma("unroll") for (int i = 0; i < 4; i++) px[SET][i] = *(const q_u32x4*)(xs_ + xoff[i]); \
        const unsigned char* ws_ = wb + (size_t)st_ * (QBK * BITS / 8);                 \
        if constexpr (BITS == 2) {                                                      \
            const uint2 t_ = *(const uint2*)(ws_ + woff);                               \
            pw[SET][0] = t_.x;                                                          \
            pw[SET][1] = t_.y;                                                          \
        } else {                                                                        \
            _Pragma("unroll") for (int i = 0; i < BITS / 4; i++) {                      \
                const q_u32x4 t_ = *(const q_u32x4*)(ws_ + woff + 16 * i);              \
                pw[SET][4 * i] = t_.x;                                                  \
                pw[SET][4 * i + 1] = t_.y;                                              \
                pw[SET][4 * i + 2] = t_.z;                                              \
                pw[SET][4 * i + 3] = t_.w;                                              \
            }                                                                           \
        }                                                                               \
        const uint32_t g_ = half_groups ? st_ * 2 : (st_ * QBK) >> a.log2g;             \
        ps[SET] = *(const uint16_t*)(sb + (size_t)g_ * 2 + soff);                       \
        pb[SET] = *(const uint16_t*)(bb + (size_t)g_ * 2 + soff);                       \
    } while (0)

#define QMM_STORE_STAGE(BUF, SET)                                                       \
    do {                                                                                \
        unsigned char* A_ = lds + (BUF) * QBUF;                                         \
        unsigned char* B_ = A_ + QBM * QLD;                                             \
        _Pragma("unroll") for (int i = 0; i < 4; i++)                                   \
            *(q_u32x4*)(A_ + (xr + 32 * i) * QLD + xc * 16) = px[SET][i];               \
        const float s_ = elem_bits_to_f32<DT>(ps[SET]), b_ = elem_bits_to_f32<DT>(pb[SET]); \
        unsigned char* dst_ = B_ + (tid >> 1) * QLD + wq * 64;                          \
        _Pragma("unroll") for (int i = 0; i < 4; i++)                                   \
            *(uint4*)(dst_ + 16 * i) = dequant8<DT, BITS>(pw[SET], i, s_, b_);          \
    } while (0)

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // Stage t is loaded during iteration t-2, converted and stored to LDS at the
    // end of iteration t-1 and multiplied in iteration t. `stages` is even.
    QMM_LOAD_STAGE(0, 0);
    QMM_LOAD_STAGE(1, 1);
    QMM_STORE_STAGE(0, 0);
    __syncthreads();

    const uint32_t fr = lane & 31u, fh = lane >> 5;  // fragment row / k-half of this lane
    const unsigned char* Abase = lds + (wm * 64 + fr) * QLD + fh * 16;
    const unsigned char* Bbase = lds + QBM * QLD + (wn * 64 + fr) * QLD + fh * 16;
    for (uint32_t s2 = 0; s2 < stages; s2 += 2) {
#pragma unroll
        for (int par = 0; par < 2; par++) {
            const uint32_t s = s2 + par;
            // set `par` held stage s, which is already in LDS: refill it with stage s+2
            QMM_LOAD_STAGE(s + 2, par);
            const unsigned char* A0 = Abase + par * QBUF;
            const unsigned char* B0 = Bbase + par * QBUF;
#pragma unroll
            for (int ks = 0; ks < QBK / 16; ks++) {
                const uint4 a0 = *(const uint4*)(A0 + ks * 32);
                const uint4 a1 = *(const uint4*)(A0 + 32 * QLD + ks * 32);
                const uint4 b0 = *(const uint4*)(B0 + ks * 32);
                const uint4 b1 = *(const uint4*)(B0 + 32 * QLD + ks * 32);
                // D[i][j] = sum_k A[i][k] B[k][j]: i = activation row, j = weight row
                acc[0][0] = mfma32<DT>(a0, b0, acc[0][0]);
                acc[0][1] = mfma32<DT>(a0, b1, acc[0][1]);
                acc[1][0] = mfma32<DT>(a1, b0, acc[1][0]);
                acc[1][1] = mfma32<DT>(a1, b1, acc[1][1]);
            }
            // stage s+1 (set par^1) goes to the other buffer; after the last stage this
            // writes a duplicate nobody reads
            QMM_STORE_STAGE(par ^ 1, par ^ 1);
            __syncthreads();
        }
    }
#undef QMM_LOAD_STAGE
#undef QMM_STORE_STAGE

    // ---- epilogue ------------------------------------------------------------
    // accumulator layout: column j = lane%32, row i = 8*(v/4) + 4*(lane/32) + v%4
    auto store_tile = [&]() {
#pragma unroll
        for (int bi = 0; bi < 2; bi++)
#pragma unroll
            for (int bj = 0; bj < 2; bj++) {
                const uint32_t col = n0 + wn * 64 + bj * 32 + fr;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const uint32_t row = m0 + wm * 64 + bi * 32 + 8 * (v / 4) + 4 * fh + (v % 4);
                    if (row < a.M && col < a.N) store_elem<DT>(a.out, (size_t)row * a.N + col, acc[bi][bj][v]);
                }
            }
    };
    if (a.splits == 1) {
        store_tile();
        return;
    }
    // split-K: publish the partial tile, take a ticket, last arriver sums in split order
    float* mine = a.scratch + ((size_t)tile * a.splits + split) * (64 * 256);
#pragma unroll
    for (int bi = 0; bi < 2; bi++)
#pragma unroll
        for (int bj = 0; bj < 2; bj++)
#pragma unroll
            for (int v = 0; v < 16; v++) mine[((bi * 2 + bj) * 16 + v) * 256 + tid] = acc[bi][bj][v];
    __threadfence();
    __syncthreads();
    if (tid == 0) s_ticket = atomicAdd(&a.tickets[tile], 1u);
    __syncthreads();
    if (s_ticket != a.splits - 1) return;
    __threadfence();
#pragma unroll
    for (int bi = 0; bi < 2; bi++)
#pragma unroll
        for (int bj = 0; bj < 2; bj++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[bi][bj][v] = 0.f;
    for (uint32_t p = 0; p < a.splits; p++) {
        const float* src = a.scratch + ((size_t)tile * a.splits + p) * (64 * 256);
#pragma unroll
        for (int bi = 0; bi < 2; bi++)
#pragma unroll
            for (int bj = 0; bj < 2; bj++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    acc[bi][bj][v] += __builtin_nontemporal_load(src + ((bi * 2 + bj) * 16 + v) * 256 + tid);
    }
    store_tile();
    if (tid == 0) a.tickets[tile] = 0;  // ready for the next launch
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct QmmScratch {
    float* partials = nullptr;
    size_t partial_bytes = 0;
    uint32_t* tickets = nullptr;
    size_t ticket_count = 0;
};
static QmmScratch g_scratch;

static int ensure_scratch(size_t partial_bytes, size_t tiles, hipStream_t stream) {
    if (planning()) {
        plan_note_scratch(partial_bytes + (tiles < 1024 ? 1024 : tiles) * sizeof(uint32_t));
        return ERR_OK;
    }
    if (g_scratch.partial_bytes < partial_bytes) {
        if (g_scratch.partials) {
            MTQ_HIP(hipStreamSynchronize(stream));
            MTQ_HIP(hipFree(g_scratch.partials));
            g_scratch.partials = nullptr;
            g_scratch.partial_bytes = 0;
        }
        MTQ_HIP(hipMalloc((void**)&g_scratch.partials, partial_bytes));
        g_scratch.partial_bytes = partial_bytes;
    }
    if (g_scratch.ticket_count < tiles) {
        if (g_scratch.tickets) {
            MTQ_HIP(hipStreamSynchronize(stream));
            MTQ_HIP(hipFree(g_scratch.tickets));
            g_scratch.tickets = nullptr;
            g_scratch.ticket_count = 0;
        }
        const size_t n = tiles < 1024 ? 1024 : tiles;
        MTQ_HIP(hipMalloc((void**)&g_scratch.tickets, n * sizeof(uint32_t)));
        MTQ_HIP(hipMemsetAsync(g_scratch.tickets, 0, n * sizeof(uint32_t), stream));
        g_scratch.ticket_count = n;
    }
    return ERR_OK;
}

template <int DT> static int launch_qmm_dt(QmmKArgs& a, int bits, const LaunchCtx& lc) {
    const void* fn;
    switch (bits) {
        case 2: fn = (const void*)qmm_kernel<DT, 2>; break;
        case 4: fn = (const void*)qmm_kernel<DT, 4>; break;
        default: fn = (const void*)qmm_kernel<DT, 8>; break;
    }
    hipError_t e = set_max_dynamic_lds(fn, (size_t)QLDS);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    void* args[] = {&a};
    e = launch_kernel(fn, dim3(a.m_tiles * a.n_tiles * a.splits), dim3(256), args, QLDS, lc);
    if (e != hipSuccess) return hip_fail(e, "qmm kernel launch");
    return ERR_OK;
}

int launch_qmm_mfma(const QmmParams& p, const LaunchCtx& lc) {
    if (p.dtype != DT_F16 && p.dtype != DT_BF16)
        return fail(ERR_UNSUPPORTED, "mfma qmm: f16 / bf16 activations only");
    if (p.bits != 2 && p.bits != 4 && p.bits != 8) return fail(ERR_UNSUPPORTED, "mfma qmm: bits must be 2, 4 or 8");
    const uint32_t G = p.group_size;
    if (p.K % (2 * QBK) || G % 32 || (G & (G - 1)) || p.K % G) return fail(ERR_UNSUPPORTED, "mfma qmm: K % 128 or group size");
    if ((uint64_t)p.M * p.K * 2 >= (1ull << 32) || (uint64_t)p.N * p.K * p.bits / 8 >= (1ull << 32))
        return fail(ERR_UNSUPPORTED, "mfma qmm: operand larger than 4 GiB");
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16) return fail(ERR_UNSUPPORTED, "mfma qmm: w and x must be 16-byte aligned");
    QmmKArgs a;
    a.w = (const uint32_t*)p.w;
    a.scales = (const uint16_t*)p.scales;
    a.biases = (const uint16_t*)p.biases;
    a.x = (const uint16_t*)p.x;
    a.out = (uint16_t*)p.out;
    a.M = p.M;
    a.N = p.N;
    a.K = p.K;
    uint32_t l = 0;
    while ((1u << l) < G) l++;
    a.log2g = l;
    a.gpr = p.K / G;
    a.m_tiles = (p.M + QBM - 1) / QBM;
    a.n_tiles = (p.N + QBN - 1) / QBN;
    // K is split only on request: the ticketed reduction needs device-scope
    // fences (an L2 write-back and invalidate per workgroup on this multi-die
    // part), which measured slower than leaving half the CUs idle at M = 512.
    const uint32_t stages = p.K / QBK, tiles = a.m_tiles * a.n_tiles;
    uint32_t splits = 1;
    if (options().qmm_splits) {
        const uint32_t s = (uint32_t)options().qmm_splits;
        if (stages % (2 * s) == 0) splits = s;
    }
    a.splits = splits;
    a.stages_per_split = stages / splits;
    a.scratch = nullptr;
    a.tickets = nullptr;
    if (splits > 1) {
        int rc = ensure_scratch((size_t)tiles * splits * 64 * 256 * sizeof(float), tiles, lc.stream);
        if (rc) return rc;
        a.scratch = g_scratch.partials;
        a.tickets = g_scratch.tickets;
    }
    return p.dtype == DT_BF16 ? launch_qmm_dt<DT_BF16>(a, p.bits, lc) : launch_qmm_dt<DT_F16>(a, p.bits, lc);
}

}  // namespace mtq
