// The GEMV whose waves walk the rows: out[n] = sum_k (s q + b)[n, k] x[k] for one row of x against rows of 2048 ... 8192
// 4-bit codes in steps of 1024, or 3584 (mt_qmv and the affine_qmv family, crates/metaltile-std/src/mlx/quantized.rs:8-308;
// dequant_gemv_int2 / int4, crates/metaltile-std/src/ffai/dequant_gemv.rs:52-100), f16 / bf16, groups of 32 / 64 / 128; a row
// that ends inside a group of 64 chunks is the *_ragged_kernel instances' (TAIL). On the same body
//   - the RMS norm fused in front of it, x'[k] = x[k] norm_w[k] / sqrt(mean(x^2) + eps) (ffai_rms_norm_qgemv / _fast,
//     crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:53-125, 128-456),
//   - two to four matrices against the one row in one launch (the fused projections of a decode step),
//   - expert-routed rows, fewer than the experts, and the single-index expert GEMV (rows of 2048 / 4096 / 5120 / 6144 / 7168 /
//     8192 codes in groups of 64),
//   - 2-bit codes (rows of 8192).
//
// The make of the one-row-per-wave kernel (qmv_rows.hip): a wave owns a weight row, lane l its 16-byte chunks l, 64 + l, ...,
// codes become operands of the 4x4x4 matrix instruction in place, the activations are put into operand order once per
// workgroup in LDS. What differs is that a workgroup stays: the launch is at most two workgroups of eight waves per
// compute unit (one of sixteen from 2049 to 4096 rows), wave g of G takes rows g, g + G, g + 2 G, ..., each row's loads issued
// while the row before it is worked on, so the activations are read and prepared once per few dozen rows. With the norm,
// the activations are normalised on the way into LDS: every workgroup works out the row's sum of squares itself
// (thread t from chunk t, one more barrier), and x', an f32 value in the reference, is carried as the element-type value
// nearest to it and the rounded (f16: scaled) remainder -- two operand sets whose products are added, 16 significant
// bits, as in the streaming kernel's fused form.
#include <hip/hip_runtime.h>

#include "../../include/mtq.h"
#include "mtq_device.h"
#include "mtq_internal.h"
#include "qmv_rows_common.h"

namespace mtq {

struct QmvRowsNArgs {
    const rp_u32x4* w;
    const uint16_t* s;
    const uint16_t* b;
    const uint16_t* x;
    uint16_t* out;
    uint32_t N;
    uint32_t slot_major;      // wave w of workgroup g starts at row w * gridDim.x + g instead of g * waves + w
    const uint16_t* norm_w;   // [K]
    const float* norm_eps;    // one f32 on the device
    // Several matrices against the one activation row (the batched instances): the rows of matrix m are rows
    // first[m] .. first[m + 1] - 1 of the launch, N is their total; unused slots hold the total.
    const rp_u32x4* mw[4];
    const uint16_t* ms[4];
    const uint16_t* mb[4];
    uint16_t* mo[4];
    uint32_t first[5];
    // Routed rows (the routed instances): expert_offsets[E + 1], indices[T] or the one expert id; w / s / b then hold E
    // matrices of N rows, x and out T rows.
    const uint32_t* route;
    uint32_t E, T;
};

// One row's loads of one lane, as they come from memory: whatever has to be done to a loaded value (picking the 16-bit
// half, widening) is done where the row is worked on. An operation on the value where it is loaded would be carried
// round the row loop with it, and the wait for the load with that operation.
template <int CH> struct RowsNormBuf {
    rp_u32x4 wv[CH];
    uint32_t sc[CH];         // the dword that holds the scale of chunk 64 i + lane
    uint32_t sw[2], bw[2];   // the lane's groups of the bias term, two 16-bit elements per dword (one group per lane: the dword that holds it)
};

// TAIL: the chunks of the last 64 a row has (0: all 64; a row of 3584 codes is 112 chunks, CH = 2 and TAIL = 48). The lanes
// past them load the row's last chunk and add nothing.
template <int DT, int CH, int LOG2G, int NWV, bool NORM, bool BATCH = false, int BITS = 4, int GM = GATHER_NONE, int TAIL = 0>
__device__ __forceinline__ void qmv_rows_walk_body(const QmvRowsNArgs& a) {
    static_assert(BITS == 4 || (BITS == 2 && !NORM && !BATCH), "4-bit codes; 2-bit codes on the plain walk");
    constexpr bool ROUTED = GM != GATHER_NONE;
    static_assert(!ROUTED || (!NORM && !BATCH && BITS == 4), "routed rows: the plain walk on 4-bit codes");
    static_assert(TAIL == 0 || (TAIL > 0 && TAIL < 64 && TAIL % 16 == 0 && BITS == 4), "ragged rows: 4-bit codes, whole 4-lane blocks");
    constexpr float MAGIC = DT == DT_BF16 ? 128.0f : 64.0f;   // 4-bit codes: one offset for every pair
    constexpr float REM = 1.0f / RemSplit<DT>::kRemScale;
    constexpr int CPC = 128 / BITS, Q = CPC / 8;   // codes per 16-byte chunk; 16-byte quarters of a chunk's activations in operand order
    constexpr int C = TAIL ? 64 * (CH - 1) + TAIL : 64 * CH, K = C * CPC;   // chunks and codes per row
    constexpr int GPR = K >> LOG2G;          // groups per row
    constexpr int GPL = GPR > 128 ? 4 : GPR > 64 ? 2 : 1;   // groups a lane owns in the bias term (lanes below GPR / GPL)
    constexpr int NH = (1 << LOG2G) < CPC ? 2 : 1;           // groups a chunk spans (2-bit codes in groups of 32: its halves are accumulated and scaled apart)
    constexpr int SPG = NH == 2 ? 1 : (1 << LOG2G) / (CPC / 2);   // half chunks per group
    static_assert(C <= 64 * NWV && LOG2G >= 5 && LOG2G <= 7 && GPR % GPL == 0 && GPR / GPL <= 64, "one thread per chunk; groups of 32, 64 or 128 codes, at most 256 per row");
    __shared__ __align__(16) uint32_t xp_lds[Q][C][4];   // [quarter][chunk][4 pair dwords]: the rounded values
    __shared__ __align__(16) uint32_t xl_lds[NORM ? Q : 1][NORM ? C : 1][4];   // the remainders
    __shared__ __align__(16) float xs_lds[2 * C];        // sum of x' over each half chunk
    __shared__ __align__(16) float xm_lds[BITS == 2 ? 2 * C : 4];   // 2-bit codes: that sum weighted with the pairs' offsets
    __shared__ float ssq_lds[NWV];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // (the same in every lane: row numbers stay in scalar registers) A turn's rows go to the launch's waves workgroup by
    // workgroup (a workgroup's waves on consecutive rows), or wave slot by wave slot (a workgroup's waves gridDim.x rows
    // apart): which of the two the launch picks is a measured rule, stated where it is set.
    const uint32_t GW = gridDim.x * (uint32_t)NWV;
    const uint32_t gw = a.slot_major ? wave * gridDim.x + blockIdx.x : blockIdx.x * (uint32_t)NWV + wave;
    const uint32_t last = a.N - 1u;
    const uint32_t gl = min(lane, (uint32_t)(GPR / GPL - 1));
    // Routed rows: grid row blockIdx.y serves the blockIdx.y-th expert that has a row, and the walk below runs once per
    // row of that expert (a pass), on that expert's matrix.
    RowsRoute rt;
    if constexpr (ROUTED) {
        if (!rows_route<GM>(a.route, a.E, a.T, lane, rt)) return;   // (the same for every wave of the workgroup: no barrier is left waiting)
    }
    const size_t eoff = ROUTED ? (size_t)rt.expert * a.N : (size_t)0;   // the expert's first row among the rows of all experts
    auto load_row = [&](uint32_t row, RowsNormBuf<CH>& r) {   // row <= last
        row = min(row, last);   // (it is; a scalar instruction keeps the loads inside the matrix whatever the caller does)
        const uint16_t *sp, *bp;
        const rp_u32x4* wrow;
        if constexpr (BATCH) {   // (row numbers are the same in every lane: the matrix is picked by scalar code)
            const uint32_t m = (uint32_t)(row >= a.first[1]) + (uint32_t)(row >= a.first[2]) + (uint32_t)(row >= a.first[3]);
            const uint32_t local = row - a.first[m];   // < the rows of matrix m, as row < first[m + 1]
            sp = a.ms[m] + (size_t)local * GPR;
            bp = a.mb[m] + (size_t)local * GPR;
            wrow = a.mw[m] + (size_t)local * C;
        } else {
            sp = a.s + (eoff + row) * GPR;
            bp = a.b + (eoff + row) * GPR;
            wrow = a.w + (eoff + row) * C;
        }
        uint32_t ci[CH];   // this lane's chunks (past the row's end: its last chunk)
#pragma unroll
        for (int i = 0; i < CH; i++) ci[i] = TAIL && i == CH - 1 ? min((uint32_t)(i * 64) + lane, (uint32_t)(C - 1)) : (uint32_t)(i * 64) + lane;
#pragma unroll
        for (int i = 0; i < CH; i++) r.sc[i] = ((const uint32_t*)sp)[(ci[i] * CPC) >> (LOG2G + 1)];   // (a chunk that spans two groups: both of them)
        r.sw[0] = r.sw[1] = r.bw[0] = r.bw[1] = 0u;
        if constexpr (GPL == 4) {
            const uint2 sv = ((const uint2*)sp)[gl], bv = ((const uint2*)bp)[gl];
            r.sw[0] = sv.x; r.sw[1] = sv.y; r.bw[0] = bv.x; r.bw[1] = bv.y;
        } else if constexpr (GPL == 2) {
            r.sw[0] = ((const uint32_t*)sp)[gl];
            r.bw[0] = ((const uint32_t*)bp)[gl];
        } else {
            r.sw[0] = ((const uint32_t*)sp)[gl >> 1];
            r.bw[0] = ((const uint32_t*)bp)[gl >> 1];
        }
        const rp_u32x4* wbase = wrow + lane;
#pragma unroll
        for (int i = 0; i < CH; i++) r.wv[i] = TAIL && i == CH - 1 ? __builtin_nontemporal_load(wrow + ci[i]) : __builtin_nontemporal_load(wbase + i * 64);
    };
    for (uint32_t pass = 0; pass < rt.n_pass; pass++) {   // (one pass unless routed)
    const uint32_t trow = rows_route_row<GM>(rt, pass);
    const uint16_t* const xrow = a.x + (size_t)trow * K;
    uint16_t* const orow = a.out + (size_t)trow * a.N;
    // ---- this thread's chunk of the activations and of the norm weights; the first row's loads ---------------------
    uint4 xraw[Q], nraw[Q];
    if (tid < (uint32_t)C) {
        const uint4* xv = (const uint4*)(xrow + (size_t)tid * CPC);
        const uint4* nv = (const uint4*)(a.norm_w + (size_t)tid * CPC);
#pragma unroll
        for (int v = 0; v < Q; v++) xraw[v] = xv[v];
        if constexpr (NORM) {
#pragma unroll
            for (int v = 0; v < Q; v++) nraw[v] = nv[v];
        }
    }
    float eps = 0.f;
    if constexpr (NORM) eps = a.norm_eps[0];
    RP_KEEP_ORDER();
    RowsNormBuf<CH> bufA, bufB;
    load_row(min(gw, last), bufA);   // (idle waves of a short launch load the last row and store nothing)
    RP_KEEP_ORDER();
    const bool j0 = lane & 1u, j1 = lane & 2u;
    // (2^7, 2^7) in bf16, a code OR-ed into mantissa bits 0-3; (2^6, 2^6) in f16, a code in mantissa bits 4-7 (where the second nibble
    // already is: the same three shifts per dword as for bits 0-3, and a sixteenth of the offset that the f32 sums carry): MAGIC + q
    uint32_t kor = DT == DT_BF16 ? 0x43004300u : 0x54005400u;
    asm volatile("" : "+v"(kor));
    // 2-bit codes: a pair of crumbs masked where it sits (bit 2 p) and OR-ed into 2^(MB - 2 p) is that power of two
    // plus the code (qmv_rows_common.h); one constant per position class, kept opaque so that an and-or has one literal
    uint32_t kor2[BITS == 2 ? (DT == DT_F16 ? 5 : 3) : 1] = {};
    if constexpr (BITS == 2) {
#pragma unroll
        for (int p = 0; p < (DT == DT_F16 ? 5 : 3); p++) {
            kor2[p] = rp_crumb_kor<DT>(p);
            asm volatile("" : "+v"(kor2[p]));
        }
    }
    // ---- the row's sum of squares ------------------------------------------------------------------------------------
    float inv = 1.0f;
    if constexpr (NORM) {
        float ssq = 0.f;
        if (tid < (uint32_t)C) {
#pragma unroll
            for (int v = 0; v < Q; v++) ssq += raw_sumsq<DT>(xraw[v]);
        }
        ssq = seg_allreduce(ssq, 64);
        if (lane == 0) ssq_lds[wave] = ssq;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int wv_ = 0; wv_ < NWV; wv_++) tot += ssq_lds[wv_];
        inv = 1.0f / sqrtf(tot / (float)K + eps);
    }
    // ---- the normalised chunk into operand order, into LDS --------------------------------------------------------------
    if (tid < (uint32_t)C) {
        rp_u32x2 ones;
        ones.x = ones.y = DT == DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
        rp_f32x4 sx[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, sl[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        rp_f32x4 sm[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        if constexpr (BITS == 4) {
#pragma unroll
        for (int d = 0; d < 4; d++) {       // weight dword d: activations 8 d .. 8 d + 7, pairs (j, j + 4)
            uint4 v = xraw[d], rem = make_uint4(0u, 0u, 0u, 0u);
            if constexpr (NORM) raw_normed<DT>(xraw[d], nraw[d], inv, v, rem);
            uint4 o, ol;
            o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
            o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
            o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
            o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
            ol.x = __builtin_amdgcn_perm(rem.z, rem.x, 0x05040100u);
            ol.y = __builtin_amdgcn_perm(rem.z, rem.x, 0x07060302u);
            ol.z = __builtin_amdgcn_perm(rem.w, rem.y, 0x05040100u);
            ol.w = __builtin_amdgcn_perm(rem.w, rem.y, 0x07060302u);
            *(uint4*)xp_lds[d][tid] = o;
            if constexpr (NORM) *(uint4*)xl_lds[d][tid] = ol;
            rp_u32x2 a0, a1, l0, l1;
            a0.x = o.x; a0.y = o.y; a1.x = o.z; a1.y = o.w;
            l0.x = ol.x; l0.y = ol.y; l1.x = ol.z; l1.y = ol.w;
            sx[d / 2] = rp_mfma<DT>(a0, ones, sx[d / 2]);
            sx[d / 2] = rp_mfma<DT>(a1, ones, sx[d / 2]);
            if constexpr (NORM) {
                sl[d / 2] = rp_mfma<DT>(l0, ones, sl[d / 2]);
                sl[d / 2] = rp_mfma<DT>(l1, ones, sl[d / 2]);
            }
        }
        } else {
#pragma unroll
            for (int d = 0; d < 4; d++) {       // weight dword d: activations 16 d .. 16 d + 15, pairs (i, i + 8)
                const uint4 lo = xraw[2 * d], hi = xraw[2 * d + 1];
                uint4 o[2];
                o[0].x = __builtin_amdgcn_perm(hi.x, lo.x, 0x05040100u);
                o[0].y = __builtin_amdgcn_perm(hi.x, lo.x, 0x07060302u);
                o[0].z = __builtin_amdgcn_perm(hi.y, lo.y, 0x05040100u);
                o[0].w = __builtin_amdgcn_perm(hi.y, lo.y, 0x07060302u);
                o[1].x = __builtin_amdgcn_perm(hi.z, lo.z, 0x05040100u);
                o[1].y = __builtin_amdgcn_perm(hi.z, lo.z, 0x07060302u);
                o[1].z = __builtin_amdgcn_perm(hi.w, lo.w, 0x05040100u);
                o[1].w = __builtin_amdgcn_perm(hi.w, lo.w, 0x07060302u);
                *(uint4*)xp_lds[2 * d][tid] = o[0];
                *(uint4*)xp_lds[2 * d + 1][tid] = o[1];
                const uint32_t pw[8] = {o[0].x, o[0].y, o[0].z, o[0].w, o[1].x, o[1].y, o[1].z, o[1].w};
#pragma unroll
                for (int m = 0; m < 4; m++) {   // pairs 2 m, 2 m + 1
                    rp_u32x2 av, kv;
                    av.x = pw[2 * m]; av.y = pw[2 * m + 1];
                    kv.x = kor2[rp_crumb_class<DT>(2 * m)]; kv.y = kor2[rp_crumb_class<DT>(2 * m + 1)];
                    sx[d / 2] = rp_mfma<DT>(av, ones, sx[d / 2]);
                    sm[d / 2] = rp_mfma<DT>(av, kv, sm[d / 2]);
                }
            }
        }
        // (a lane's own sum is the diagonal entry of its block: its first operand against its own second operand)
        xs_lds[2 * tid] = fmaf(rp_diag(sl[0], j0, j1), REM, rp_diag(sx[0], j0, j1));
        xs_lds[2 * tid + 1] = fmaf(rp_diag(sl[1], j0, j1), REM, rp_diag(sx[1], j0, j1));
        if constexpr (BITS == 2) {
            xm_lds[2 * tid] = rp_diag(sm[0], j0, j1);
            xm_lds[2 * tid + 1] = rp_diag(sm[1], j0, j1);
        }
    }
    __syncthreads();
    if (gw <= last) {
    // the activation sums of this lane's GPL groups of the bias term (the same for every row)
    float X[GPL], XM[GPL];   // (XM: the sum weighted with the codes' offsets; 4-bit codes have the one offset)
#pragma unroll
    for (int v = 0; v < GPL; v++) {
        X[v] = XM[v] = 0.f;
#pragma unroll
        for (int h = 0; h < SPG; h++) {
            X[v] += xs_lds[(gl * GPL + (uint32_t)v) * SPG + (uint32_t)h];
            if constexpr (BITS == 2) XM[v] += xm_lds[(gl * GPL + (uint32_t)v) * SPG + (uint32_t)h];
        }
        if constexpr (BITS == 4) XM[v] = MAGIC * X[v];
    }
    auto work_row = [&](uint32_t row, const RowsNormBuf<CH>& r) {
        float t = 0.f;
        // (the lane number, made opaque once per row: the operand reads from LDS below are the same for every row, and
        // lifted out of the row loop they would hold 32 registers per chunk)
        uint32_t ln = lane;
        asm volatile("" : "+v"(ln));
        if (lane < (uint32_t)(GPR / GPL)) {
#pragma unroll
            for (int v = 0; v < GPL; v++) {
                const uint32_t sh = GPL == 1 ? 16u * (gl & 1u) : 16u * (uint32_t)(v & 1);
                const float sf = rp_up<DT>((r.sw[v >> 1] >> sh) & 0xFFFFu), bf = rp_up<DT>((r.bw[v >> 1] >> sh) & 0xFFFFu);
                t = fmaf(bf, X[v], t);
                t = fmaf(0.f - sf, XM[v], t);
            }
        }
#pragma unroll
        for (int i = 0; i < CH; i++) {
            if constexpr (BITS == 4) {
                rp_f32x4 dh = {0.f, 0.f, 0.f, 0.f}, dl = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    const uint32_t w = r.wv[i][d];
                    const uint4 xo = *(const uint4*)xp_lds[d][TAIL && i == CH - 1 ? min((uint32_t)(i * 64) + ln, (uint32_t)(C - 1)) : (uint32_t)(i * 64) + ln];
                    uint4 xl = make_uint4(0u, 0u, 0u, 0u);
                    if constexpr (NORM) xl = *(const uint4*)xl_lds[d][TAIL && i == CH - 1 ? min((uint32_t)(i * 64) + ln, (uint32_t)(C - 1)) : (uint32_t)(i * 64) + ln];
                    rp_u32x2 b0, b1, a0, a1, l0, l1;
                    if constexpr (DT == DT_BF16) {
                        b0.x = (w & 0x000F000Fu) | kor;
                        b0.y = ((w >> 4) & 0x000F000Fu) | kor;
                        b1.x = ((w >> 8) & 0x000F000Fu) | kor;
                        b1.y = ((w >> 12) & 0x000F000Fu) | kor;
                    } else {   // (the second nibble is where it has to be)
                        b0.x = ((w << 4) & 0x00F000F0u) | kor;
                        b0.y = (w & 0x00F000F0u) | kor;
                        b1.x = ((w >> 4) & 0x00F000F0u) | kor;
                        b1.y = ((w >> 8) & 0x00F000F0u) | kor;
                    }
                    a0.x = xo.x; a0.y = xo.y; a1.x = xo.z; a1.y = xo.w;
                    l0.x = xl.x; l0.y = xl.y; l1.x = xl.z; l1.y = xl.w;
                    dh = rp_mfma<DT>(a0, b0, dh);
                    dh = rp_mfma<DT>(a1, b1, dh);
                    if constexpr (NORM) {
                        dl = rp_mfma<DT>(l0, b0, dl);
                        dl = rp_mfma<DT>(l1, b1, dl);
                    }
                }
                const uint32_t sch = 16u * ((((TAIL && i == CH - 1 ? min((uint32_t)(i * 64) + lane, (uint32_t)(C - 1)) : (uint32_t)(i * 64) + lane) * CPC) >> LOG2G) & 1u);   // the half of the dword the chunk's group is in
                const float ti = fmaf(rp_up<DT>((r.sc[i] >> sch) & 0xFFFFu), fmaf(rp_diag(dl, j0, j1), REM, rp_diag(dh, j0, j1)), t);
                t = TAIL && i == CH - 1 && lane >= (uint32_t)TAIL ? t : ti;   // (lanes past the row's end hold its last chunk again)
            } else {
                rp_f32x4 dq[NH];
#pragma unroll
                for (int h = 0; h < NH; h++) dq[h] = rp_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    const uint32_t w = r.wv[i][d];
                    constexpr int HSH = NH == 2 ? 1 : 2;   // dword d adds to half d >> HSH
                    const uint4 xo0 = *(const uint4*)xp_lds[2 * d][i * 64 + ln], xo1 = *(const uint4*)xp_lds[2 * d + 1][i * 64 + ln];
                    const uint32_t xa[8] = {xo0.x, xo0.y, xo0.z, xo0.w, xo1.x, xo1.y, xo1.z, xo1.w};
                    uint32_t pq[8];
#pragma unroll
                    for (int pi = 0; pi < 8; pi++) {
                        constexpr uint32_t M2 = 0x00030003u;
                        const int p = rp_crumb_class<DT>(pi), sh = rp_crumb_shift<DT>(pi);
                        pq[pi] = ((w >> sh) & (M2 << (2 * p))) | kor2[p];
                    }
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        rp_u32x2 av, bvv;
                        av.x = xa[2 * m]; av.y = xa[2 * m + 1];
                        bvv.x = pq[2 * m]; bvv.y = pq[2 * m + 1];
                        dq[d >> HSH] = rp_mfma<DT>(av, bvv, dq[d >> HSH]);
                    }
                }
                if constexpr (NH == 2) {   // the dword holds the chunk's two groups: half h is group h
                    t = fmaf(rp_up<DT>(r.sc[i] & 0xFFFFu), rp_diag(dq[0], j0, j1), t);
                    t = fmaf(rp_up<DT>(r.sc[i] >> 16), rp_diag(dq[NH - 1], j0, j1), t);
                } else {
                    const uint32_t sch = 16u * ((((uint32_t)(i * 64 + (int)lane) * CPC) >> LOG2G) & 1u);
                    t = fmaf(rp_up<DT>((r.sc[i] >> sch) & 0xFFFFu), rp_diag(dq[0], j0, j1), t);
                }
            }
        }
        t += __shfl_xor(t, 32, 64);
        t += dpp_f32<0xB1>(t);
        t += dpp_f32<0x4E>(t);
        t += dpp_f32<0x141>(t);
        t += dpp_f32<0x140>(t);
        t += __shfl_xor(t, 16, 64);
        if (lane == 0 && row <= last) {
            if constexpr (BATCH) {
                const uint32_t m = (uint32_t)(row >= a.first[1]) + (uint32_t)(row >= a.first[2]) + (uint32_t)(row >= a.first[3]);
                a.mo[m][row - a.first[m]] = f32_to_elem_bits<DT>(t);
            } else {
                orow[row] = f32_to_elem_bits<DT>(t);
            }
        }
    };
    // ---- this wave's rows, each row's loads in flight while the row before it is worked on ------------------------------
    // A row's loads and the work on the row before it stand in one block of straight-line code, in a counted loop with
    // no way out but its end: the wait that the compiler puts before the first use of a buffer then leaves the loads
    // just issued in flight. (With the loads under a condition of their own, or with a way out of the loop between
    // them, that wait has to hold for the path that issued nothing, and waits for them.)
    const uint32_t cnt = (last - gw) / GW + 1u;   // rows of this wave: gw, gw + GW, ... (gw <= last here)
    uint32_t row = gw;
    // (The norm's instances for rows of 8192 codes have no register to spare for a second way of ending: they run
    // whole turns, the last of which loads the matrix's last row once more for nobody, and end on the odd row.)
    constexpr bool WHOLE_TURNS = NORM && CH == 4;
    if (WHOLE_TURNS && cnt == 1u) {
        work_row(row, bufA);
    } else {
        for (uint32_t it = WHOLE_TURNS ? cnt >> 1 : (cnt - 1u) >> 1; it != 0u; it--) {   // two rows a turn (while a third is there to be loaded)
            load_row(row + GW, bufB);
            RP_KEEP_ORDER();
            work_row(row, bufA);
            load_row(row + 2u * GW, bufA);
            RP_KEEP_ORDER();
            work_row(row + GW, bufB);
            row += 2u * GW;
        }
        if constexpr (WHOLE_TURNS) {
            if (cnt & 1u) work_row(row, bufA);
        } else if (cnt & 1u) {   // one row is left, or two; the first of them is loaded
            RP_KEEP_ORDER();     // (both ways start behind a fence of their own, so that the work on the first row is not lifted above the branch)
            work_row(row, bufA);
        } else {
            load_row(row + GW, bufB);
            RP_KEEP_ORDER();
            work_row(row, bufA);
            RP_KEEP_ORDER();
            work_row(row + GW, bufB);
        }
    }
    }   // this wave has rows
    if constexpr (ROUTED) {
        if (pass + 1u < rt.n_pass) __syncthreads();   // the next pass overwrites the activations in LDS
    }
    }   // pass
}

// (four waves per SIMD: two workgroups of eight waves, or one of sixteen, per compute unit)
template <int DT, int CH, int LOG2G, int NWV> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_norm_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, true>(a);
}
template <int DT, int CH, int LOG2G, int NWV, int TAIL> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_norm_ragged_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, true, false, 4, GATHER_NONE, TAIL>(a);   // (rows that end inside a group of 64 chunks)
}
// The same walk without the norm: out[n] = sum_k (s q + b)[n, k] x[k], the activations as they are (one operand set).
template <int DT, int CH, int LOG2G, int NWV> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_walk_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, false>(a);
}
// Rows that do not fill whole groups of 64 chunks (3072 / 3584 / 5120 / 7168 codes: the hidden sizes of other models).
template <int DT, int CH, int LOG2G, int NWV, int TAIL> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_walk_ragged_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, false, false, 4, GATHER_NONE, TAIL>(a);
}

// 2-bit codes (rows of 8192: 128 chunks of 64 codes), made operands in place as in the one-row-per-wave kernel.
template <int DT, int CH, int LOG2G, int NWV> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_walk2_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, false, false, 2>(a);
}
// Routed rows (a decode step of a few tokens through a mixture-of-experts layer: fewer rows than experts, or the one
// row of dequant_gemv_int4_expert_indexed, crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:58-105; the
// routing rules of mt_moe_gather_qmm_int4, crates/metaltile-std/src/ffai/moe.rs:376-385): grid row y walks the rows of the
// y-th expert that has a row, once per row of x routed to it.
template <int DT, int CH, int LOG2G, int GM> __global__ __launch_bounds__(512, 4) void qmv_rows_walk_routed_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, 8, false, false, 4, GM>(a);
}
// Two to four matrices against the one activation row in one launch (the fused projections of a decode step:
// ffai_batched_qkv_qgemv_fast, crates/metaltile-std/src/ffai/batched_qkv_qgemv.rs:157; ffai_batched_4_qgemv_fast,
// crates/metaltile-std/src/ffai/batched_4_qgemv.rs:60): the launch's rows are the matrices' rows one after the other.
template <int DT, int CH, int LOG2G, int NWV> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_walk_batched_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, false, true>(a);
}

// 4-bit codes, rows of 2048 ... 8192 codes in steps of 1024 or 3584, groups of 32 / 64 / 128, f16 / bf16
bool qmv_rows_norm_takes(const QmvParams& p, const void* norm_w) {
    if ((p.dtype != DT_F16 && p.dtype != DT_BF16) || p.bits != 4 || p.N == 0 || p.N > (1u << 24)) return false;   // (row numbers plus the launch's waves stay below 2^32)
    if (p.K != 3584 && (p.K < 2048 || p.K > 8192 || p.K % 1024)) return false;
    const uint32_t G = p.group_size;
    if (G != 32 && G != 64 && G != 128) return false;
    return !((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)norm_w % 16 || (uintptr_t)p.scales % 8 || (uintptr_t)p.biases % 8 || (uintptr_t)p.out % 2);
}

template <int DT, int CH, int LOG2G, int NWV, int TAIL> __global__ __launch_bounds__(64 * NWV, 4) void qmv_rows_walk_batched_ragged_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, NWV, false, true, 4, GATHER_NONE, TAIL>(a);   // (rows that end inside a group of 64 chunks)
}
template <int DT, int LOG2G> static const void* rows_walk_batched_fn(uint32_t K, bool sixteen) {
    if (K == 2048) return sixteen ? (const void*)qmv_rows_walk_batched_kernel<DT, 1, LOG2G, 16> : (const void*)qmv_rows_walk_batched_kernel<DT, 1, LOG2G, 8>;
    if (K == 6144) return sixteen ? (const void*)qmv_rows_walk_batched_kernel<DT, 3, LOG2G, 16> : (const void*)qmv_rows_walk_batched_kernel<DT, 3, LOG2G, 8>;
    if (K == 3072) return sixteen ? (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 2, LOG2G, 16, 32> : (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 2, LOG2G, 8, 32>;
    if (K == 3584) return sixteen ? (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 2, LOG2G, 16, 48> : (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 2, LOG2G, 8, 48>;
    if (K == 5120) return sixteen ? (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 3, LOG2G, 16, 32> : (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 3, LOG2G, 8, 32>;
    if (K == 7168) return sixteen ? (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 4, LOG2G, 16, 32> : (const void*)qmv_rows_walk_batched_ragged_kernel<DT, 4, LOG2G, 8, 32>;
    if (sixteen) return K == 4096 ? (const void*)qmv_rows_walk_batched_kernel<DT, 2, LOG2G, 16> : (const void*)qmv_rows_walk_batched_kernel<DT, 4, LOG2G, 16>;
    return K == 4096 ? (const void*)qmv_rows_walk_batched_kernel<DT, 2, LOG2G, 8> : (const void*)qmv_rows_walk_batched_kernel<DT, 4, LOG2G, 8>;
}

template <int DT, int LOG2G> static const void* rows_walk2_fn(bool sixteen) {   // 2-bit codes, rows of 8192
    return sixteen ? (const void*)qmv_rows_walk2_kernel<DT, 2, LOG2G, 16> : (const void*)qmv_rows_walk2_kernel<DT, 2, LOG2G, 8>;
}

template <int DT, int CH, int LOG2G, int GM, int TAIL> __global__ __launch_bounds__(512, 4) void qmv_rows_walk_routed_ragged_kernel(QmvRowsNArgs a) {
    qmv_rows_walk_body<DT, CH, LOG2G, 8, false, false, 4, GM, TAIL>(a);   // (rows that end inside a group of 64 chunks)
}
template <int DT, int GM> static const void* rows_walk_routed_fn(uint32_t K) {   // groups of 64
    if (K == 2048) return (const void*)qmv_rows_walk_routed_kernel<DT, 1, 6, GM>;
    if (K == 6144) return (const void*)qmv_rows_walk_routed_kernel<DT, 3, 6, GM>;
    if (K == 5120) return (const void*)qmv_rows_walk_routed_ragged_kernel<DT, 3, 6, GM, 32>;
    if (K == 7168) return (const void*)qmv_rows_walk_routed_ragged_kernel<DT, 4, 6, GM, 32>;
    return K == 4096 ? (const void*)qmv_rows_walk_routed_kernel<DT, 2, 6, GM> : (const void*)qmv_rows_walk_routed_kernel<DT, 4, 6, GM>;
}

template <int DT, int LOG2G, bool NORM> static const void* rows_walk_fn(uint32_t K, bool sixteen) {
    if constexpr (NORM) {
        if (K == 2048) return sixteen ? (const void*)qmv_rows_norm_kernel<DT, 1, LOG2G, 16> : (const void*)qmv_rows_norm_kernel<DT, 1, LOG2G, 8>;
        if (K == 6144) return sixteen ? (const void*)qmv_rows_norm_kernel<DT, 3, LOG2G, 16> : (const void*)qmv_rows_norm_kernel<DT, 3, LOG2G, 8>;
        if (K == 3072) return sixteen ? (const void*)qmv_rows_norm_ragged_kernel<DT, 2, LOG2G, 16, 32> : (const void*)qmv_rows_norm_ragged_kernel<DT, 2, LOG2G, 8, 32>;
        if (K == 3584) return sixteen ? (const void*)qmv_rows_norm_ragged_kernel<DT, 2, LOG2G, 16, 48> : (const void*)qmv_rows_norm_ragged_kernel<DT, 2, LOG2G, 8, 48>;
        if (K == 5120) return sixteen ? (const void*)qmv_rows_norm_ragged_kernel<DT, 3, LOG2G, 16, 32> : (const void*)qmv_rows_norm_ragged_kernel<DT, 3, LOG2G, 8, 32>;
        if (K == 7168) return sixteen ? (const void*)qmv_rows_norm_ragged_kernel<DT, 4, LOG2G, 16, 32> : (const void*)qmv_rows_norm_ragged_kernel<DT, 4, LOG2G, 8, 32>;
        if (sixteen) return K == 4096 ? (const void*)qmv_rows_norm_kernel<DT, 2, LOG2G, 16> : (const void*)qmv_rows_norm_kernel<DT, 4, LOG2G, 16>;
        return K == 4096 ? (const void*)qmv_rows_norm_kernel<DT, 2, LOG2G, 8> : (const void*)qmv_rows_norm_kernel<DT, 4, LOG2G, 8>;
    } else {
        if (K == 2048) return sixteen ? (const void*)qmv_rows_walk_kernel<DT, 1, LOG2G, 16> : (const void*)qmv_rows_walk_kernel<DT, 1, LOG2G, 8>;
        if (K == 3072) return sixteen ? (const void*)qmv_rows_walk_ragged_kernel<DT, 2, LOG2G, 16, 32> : (const void*)qmv_rows_walk_ragged_kernel<DT, 2, LOG2G, 8, 32>;
        if (K == 3584) return sixteen ? (const void*)qmv_rows_walk_ragged_kernel<DT, 2, LOG2G, 16, 48> : (const void*)qmv_rows_walk_ragged_kernel<DT, 2, LOG2G, 8, 48>;
        if (K == 5120) return sixteen ? (const void*)qmv_rows_walk_ragged_kernel<DT, 3, LOG2G, 16, 32> : (const void*)qmv_rows_walk_ragged_kernel<DT, 3, LOG2G, 8, 32>;
        if (K == 7168) return sixteen ? (const void*)qmv_rows_walk_ragged_kernel<DT, 4, LOG2G, 16, 32> : (const void*)qmv_rows_walk_ragged_kernel<DT, 4, LOG2G, 8, 32>;
        if (K == 6144) return sixteen ? (const void*)qmv_rows_walk_kernel<DT, 3, LOG2G, 16> : (const void*)qmv_rows_walk_kernel<DT, 3, LOG2G, 8>;
        if (sixteen) return K == 4096 ? (const void*)qmv_rows_walk_kernel<DT, 2, LOG2G, 16> : (const void*)qmv_rows_walk_kernel<DT, 4, LOG2G, 16>;
        return K == 4096 ? (const void*)qmv_rows_walk_kernel<DT, 2, LOG2G, 8> : (const void*)qmv_rows_walk_kernel<DT, 4, LOG2G, 8>;
    }
}

// p.N is the launch's rows: the matrix's, or the total of the batch's matrices
template <bool NORM> static int launch_rows_walk(const QmvParams& p, const void* norm_w, const float* eps, const LaunchCtx& lc, const QmvBatch* batch = nullptr) {
    QmvRowsNArgs a{};
    a.w = (const rp_u32x4*)p.w; a.s = (const uint16_t*)p.scales; a.b = (const uint16_t*)p.biases; a.x = (const uint16_t*)p.x; a.out = (uint16_t*)p.out;
    a.N = p.N; a.norm_w = (const uint16_t*)norm_w; a.norm_eps = eps;
    a.route = p.route; a.E = p.E; a.T = p.T;
    // Rows of 4096 4-bit codes in groups of 64, from 16384 rows: slot by slot (bf16, us per launch in a chain, workgroup by
    // workgroup -> slot by slot, two machines: 16384 rows 8.44 -> 8.05 and 8.28 -> 7.93, 28672 13.0 -> 12.4 and 12.7 -> 12.3, 40960
    // 17.8 -> 16.7, 57344 23.5 -> 22.3 and 23.1 -> 22.2, 98304 37.2 -> 36.6; 14336 rows 7.47 -> 7.55 and 7.40 -> 7.43, 8192 rows the
    // same). Other shapes stay workgroup by workgroup: groups of 32 / 128 on 28672 x 4096 13.2 -> 13.2, 12.2 -> 12.3 (11.8 -> 12.2
    // on the other machine); rows of 8192 codes 14336 / 28672 / 57344 rows 12.9 -> 13.0, 22.1 -> 24.0, 42.3 -> 46.0.
    // The norm's and the batched instances alike (norm 16384 / 28672 / 32768 rows 9.9 -> 9.8, 14.3 -> 14.2, 16.0 -> 15.8; two matrices
    // of 14336 rows 13.0 -> 12.6, three of 8192 11.5 -> 11.2). The kernels that work one long row per wave and end lose by it
    // (4096 x 14336 7.33 -> 7.42, 8192 x 8192 8.0 -> 8.2).
    // 2-bit codes (rows of 8192, the same 2 KB): groups of 32 and 64 gain from 16384 rows (f16, 16384 / 28672 rows: g32 10.8 -> 10.6,
    // 17.0 -> 16.4; g64 10.6 -> 10.1, 17.7 -> 17.1), groups of 128 do not (10.7 -> 10.7, 16.8 -> 16.9), 8192 rows are the same.
    a.slot_major = p.gather == GATHER_NONE && p.N >= 16384 &&
                   ((p.bits == 4 && p.K == 4096 && p.group_size == 64) || (p.bits == 2 && p.group_size <= 64));
    if (batch) {
        uint32_t at = 0;
        for (int j = 0; j < 4; j++) {
            const int k = j < batch->n ? j : 0;   // (unused slots repeat matrix 0 and start at the total: no row reaches them)
            a.mw[j] = (const rp_u32x4*)batch->w[k]; a.ms[j] = (const uint16_t*)batch->scales[k]; a.mb[j] = (const uint16_t*)batch->biases[k];
            a.mo[j] = (uint16_t*)batch->out[k];
            a.first[j] = at;
            if (j < batch->n) at += batch->N[j];
        }
        a.first[4] = at;
        if (at != p.N) return fail(ERR_BAD_ARG, "qmv walking rows kernel: the batch's rows do not add up");
    }
    void* args[] = {&a};
    const uint32_t G = p.group_size;
    // From 2049 to 4096 rows one workgroup of sixteen waves per 16 rows (norm, 4096 x 4096 bf16: 4.5 us against 5.6 in
    // workgroups of eight); beyond, two workgroups of eight waves per compute unit, which walk the rows (14336 x 4096: the
    // same either way; eight hold on the machines where a launch of exactly one large workgroup per compute unit falls
    // behind). Up to 2048 rows workgroups of eight again: sixteen rows per workgroup would leave compute units without one
    // (bf16 g64, sixteen -> eight: 2048 x 7168 4.32 -> 3.66, 1024 x 7168 4.15 -> 3.26, 2048 x 5120 3.79 -> 3.29, 2048 x 4096
    // 3.2 - 3.4 -> 3.0, 1024 x 3072 3.05 - 3.35 -> 2.76).
    const bool sixteen = p.N > 2048 && p.N <= 4096;
    const uint32_t nwv = sixteen ? 16u : 8u, cap = sixteen ? 256u : 512u;
    const void* fn = p.dtype == DT_BF16 ? (G == 32 ? rows_walk_fn<DT_BF16, 5, NORM>(p.K, sixteen) : G == 64 ? rows_walk_fn<DT_BF16, 6, NORM>(p.K, sixteen) : rows_walk_fn<DT_BF16, 7, NORM>(p.K, sixteen))
                                        : (G == 32 ? rows_walk_fn<DT_F16, 5, NORM>(p.K, sixteen) : G == 64 ? rows_walk_fn<DT_F16, 6, NORM>(p.K, sixteen) : rows_walk_fn<DT_F16, 7, NORM>(p.K, sixteen));
    if (p.bits == 2) {
        if (NORM || batch || p.K != 8192) return fail(ERR_UNSUPPORTED, "qmv walking rows kernel: 2-bit codes on one matrix with rows of 8192 codes");
        fn = p.dtype == DT_BF16 ? (G == 32 ? rows_walk2_fn<DT_BF16, 5>(sixteen) : G == 64 ? rows_walk2_fn<DT_BF16, 6>(sixteen) : rows_walk2_fn<DT_BF16, 7>(sixteen))
                                : (G == 32 ? rows_walk2_fn<DT_F16, 5>(sixteen) : G == 64 ? rows_walk2_fn<DT_F16, 6>(sixteen) : rows_walk2_fn<DT_F16, 7>(sixteen));
    }
    if (batch) {
        if constexpr (NORM) return fail(ERR_UNSUPPORTED, "norm + qmv rows kernel: one matrix");
        fn = p.dtype == DT_BF16 ? (G == 32 ? rows_walk_batched_fn<DT_BF16, 5>(p.K, sixteen) : G == 64 ? rows_walk_batched_fn<DT_BF16, 6>(p.K, sixteen) : rows_walk_batched_fn<DT_BF16, 7>(p.K, sixteen))
                                : (G == 32 ? rows_walk_batched_fn<DT_F16, 5>(p.K, sixteen) : G == 64 ? rows_walk_batched_fn<DT_F16, 6>(p.K, sixteen) : rows_walk_batched_fn<DT_F16, 7>(p.K, sixteen));
    }
    if (p.gather != GATHER_NONE) {
        // a grid row per expert that can have a row, workgroups of eight waves, about two of them per compute unit over all grid rows
        if (NORM || batch || p.bits != 4 || G != 64) return fail(ERR_UNSUPPORTED, "qmv walking rows kernel: routed rows on the plain 4-bit walk, groups of 64");
        const uint32_t slots = p.gather == GATHER_SINGLE ? 1u : (p.T < p.E ? p.T : p.E);
        fn = p.gather == GATHER_CSR       ? (p.dtype == DT_BF16 ? rows_walk_routed_fn<DT_BF16, GATHER_CSR>(p.K) : rows_walk_routed_fn<DT_F16, GATHER_CSR>(p.K))
             : p.gather == GATHER_INDICES ? (p.dtype == DT_BF16 ? rows_walk_routed_fn<DT_BF16, GATHER_INDICES>(p.K) : rows_walk_routed_fn<DT_F16, GATHER_INDICES>(p.K))
                                          : (p.dtype == DT_BF16 ? rows_walk_routed_fn<DT_BF16, GATHER_SINGLE>(p.K) : rows_walk_routed_fn<DT_F16, GATHER_SINGLE>(p.K));
        const uint32_t per_slot = 512u / slots > 0u ? 512u / slots : 1u, all = (p.N + 7u) / 8u;
        hipError_t e = launch_kernel(fn, dim3(all < per_slot ? all : per_slot, slots), dim3(512), args, 0, lc);
        if (e != hipSuccess) return hip_fail(e, "qmv walking rows kernel launch (routed)");
        return ERR_OK;
    }
    const uint32_t wgs = (p.N + nwv - 1u) / nwv;
    hipError_t e = launch_kernel(fn, dim3(wgs < cap ? wgs : cap), dim3(64u * nwv), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, NORM ? "norm + qmv rows kernel launch" : "qmv walking rows kernel launch");
    return ERR_OK;
}

int launch_qmv_rows_norm(const QmvParams& p, const void* norm_w, const float* eps, const LaunchCtx& lc) {
    if (!qmv_rows_norm_takes(p, norm_w) || !eps) return fail(ERR_UNSUPPORTED, "norm + qmv rows kernel: 4-bit codes, rows of 2048 to 8192 codes in steps of 1024 (and 3584), f16 / bf16");
    return launch_rows_walk<true>(p, norm_w, eps, lc);
}

// The plain GEMV on the same walk: one activation row against one matrix.
bool qmv_rows_walk_takes(const QmvParams& p) {
    if (p.gather != GATHER_NONE) {
        // routed rows: at most 64 rows (a wave-wide mask of an expert's rows) on any number of experts, 4-bit codes in groups
        // of 64, every expert's block of scales as aligned as the first
        if (p.gather != GATHER_CSR && p.gather != GATHER_INDICES && p.gather != GATHER_SINGLE) return false;
        if (!p.route || p.E == 0 || p.bits != 4 || p.group_size != 64) return false;
        if (p.gather != GATHER_SINGLE && (p.T == 0 || p.T > 64)) return false;
        if (((size_t)p.N * (p.K / 64u) * 2u) % 8u) return false;
        return (p.K == 4096 || p.K == 8192 || p.K == 2048 || p.K == 5120 || p.K == 6144 || p.K == 7168) && qmv_rows_norm_takes(p, p.x);   // (the widths of expert layers it is built for)
    }
    if (p.M != 1) return false;
    if (p.bits == 2) {   // rows of 8192 2-bit codes: the 4-bit instance's conditions on a matrix of that width
        QmvParams q = p;
        q.bits = 4;
        return p.K == 8192 && qmv_rows_norm_takes(q, p.x);
    }
    return qmv_rows_norm_takes(p, p.x);   // (the alignment of x stands in for that of the norm weights)
}

// Where it is ahead of the kernels that work a row block per wave and end (bf16 g64, us, those -> this, same run):
// rows of 4096 codes, 1536 / 2048 / 4096 / 6144 / 8192 / 14336 / 16384 / 28672 / 32768 weight rows 3.35 -> 3.25, 3.46 -> 3.30,
// 4.14 -> 3.82, 5.07 -> 4.38, 5.58 -> 5.02, 7.93 -> 7.45, 8.35 -> 8.27, 13.07 -> 12.72, 14.32 -> 14.0 (1024 rows: 3.15 -> 3.19), level
// at 40960, behind between (49152 / 57344 / 65536 rows 19.98 -> 20.2, 22.57 -> 23.19, 25.3 -> 25.65: the streaming kernel's
// sizes) and ahead again from 81920 (30.8 against 32.1; 98304 36.0 / 37.5; 128256 45.96 / 47.45); other group sizes alike
// (14336 x 4096: f16 g32 8.71 -> 7.7, bf16 g128 8.05 -> 7.2 - 7.5). Rows of 8192 codes from 10240 weight rows (10240 /
// 12288 / 14336 / 16384 / 20480 / 28672 / 40960 / 57344: 10.7 -> 9.65, 11.4 -> 10.8, 13.8 -> 12.6, 14.5 -> 14.15, 18.3 -> 16.4, 22.5 -> 21.8,
// 32.1 -> 30.4, 41.9 -> 41.3; f16 g32 14336 / 28672 14.3 -> 13.6, 24.9 -> 23.5); below that the one-row-per-wave kernel
// holds (8192 x 8192 f16 g32 / g64 / g128 8.70 / 8.84, 8.4 / 8.37, 7.68 / 8.12; 4096 x 8192 5.04 / 5.42), and so it does
// in groups of 128 (14336 x 8192: 12.59 / 12.80).
bool qmv_rows_walk_preferred(const QmvParams& p) {
    if (!qmv_rows_walk_takes(p)) return false;
    // Routed rows, fewer than the experts (8 experts, bf16, us per launch in a chain of launches, the routed wave-per-row
    // kernels or, from three rows of 4096 codes, the matrix-core GEMV -> this): experts of 14336 x 4096, 1 / 2 / 3 / 4 / 5 / 7 rows
    // on distinct experts 8.1 - 8.3 -> 7.9 - 8.2, 14.9 -> 12.8, 22.3 -> 18.7, 28.4 -> 24.1, 41.2 -> 28.6, 51.2 -> 39.2; of 4096 x 8192 5.9 -> 5.4,
    // 10.3 -> 8.8, (5 / 7 rows) 25.2 -> 17.3, 31.3 -> 23.2. Launched alone, with a host wait behind each launch, the gains are
    // larger (14336 x 4096 one row 8.6 -> 7.4; 14336 x 8192, 1 / 4 rows 18.0 -> 12.5, 63.4 -> 41.4). Two rows on one expert are two
    // passes over its matrix: 13.4 -> 14.2 alone on 14336 x 4096 (the older kernel's second pass is shorter), 9.8 -> 8.6 and
    // 29.9 -> 22.2 on the others. The single-index form is routed as the plain launch of the same matrix (in a chain:
    // 14336 x 4096 7.4 -> 6.7, 14336 x 8192 13.8 -> 12.8, 4096 x 8192 5.0 -> 5.4).
    // Small experts too (8 experts, 1 / 2 / 4 / 7 rows: 768 x 2048 4.13 -> 4.16, 4.47 -> 4.05, 6.14 -> 3.97, 7.46 -> 4.30; 768 x 8192 4.09 -> 4.00,
    // 7.49 -> 4.03, 10.7 -> 5.27, 13.1 -> 6.69; 96 experts of 768 x 2048 5.37 -> 4.19, 5.82 -> 4.71, 7.17 -> 5.71, 8.55 -> 6.67 at 1 / 2 / 4 / 8 rows).
    // More rows than eight, on many small experts (96 experts, rows on distinct ones, 12 / 16 / 32 / 64 rows: experts of 2048 x 7168
    // 31.1 -> 19.1, 27.1 -> 22.8, 52.9 -> 43.8, 90.2 -> 84.1; of 768 x 2048 11.3 -> 7.58, 12.8 -> 7.94, 15.0 -> 10.7, 15.8 -> 16.8; of 7168 x 2048
    // 23.4 -> 24.0, 26.8 -> 29.5, 55.1 -> 56.5, 90.5 -> 110): up to 32 rows where an expert has at most 2048 rows and the experts are
    // at least twice the rows.
    if (p.gather != GATHER_NONE && p.gather != GATHER_SINGLE)
        return p.N >= 256 && p.T < p.E && (p.T <= 8 || (p.T <= 32 && p.N <= 2048 && p.E >= 2u * p.T));
    // 2-bit codes (rows of 8192), the one-row-per-wave kernel -> this: 8192 rows f16 g32 / g64 / g128 6.76 -> 6.30, 6.27 -> 5.91,
    // 6.09 -> 5.61; bf16 g64 14336 / 28672 rows 9.51 -> 8.75, 16.2 -> 14.4; 2048 / 4096 rows 3.62 -> 3.84, 4.01 -> 4.30
    if (p.bits == 2) return p.N >= 8192;
    // Rows of 2048 / 6144 codes (bf16 g64, the kernels that end after a row block -> this): 2048 codes, 1024 / 2048 / 4096 / 8192 /
    // 16384 / 20480 rows 3.4 - 3.7 -> 3.2, 3.4 - 3.6 -> 2.7 - 3.3, 3.5 -> 2.9 - 3.3, 4.56 -> 3.80, 5.87 -> 5.57, 6.66 -> 6.54, level at
    // 24576 and behind beyond (128256 rows 24.8 -> 29.2: a wave's two rows in flight are 2 KB; four workgroups per compute unit
    // bring that to 26.6 and cost the sizes below 16384 rows 5 %); 6144 codes, 1024 / 2048 / 4096 / 8192 / 16384 / 32768 / 102400 rows
    // 4.22 -> 3.66, 4.59 -> 3.83, 5.66 -> 4.38, 7.68 -> 6.56, 12.0 -> 11.4, 20.3 -> 19.7, 60.5 -> 57.8; groups of 32 / 128 alike
    // (8192 x 2048 f16 4.60 -> 3.89, 4.58 -> 3.81; 16384 x 6144 12.7 -> 11.8, 12.0 -> 11.3).
    // Rows that end inside a group of 64 chunks (bf16 g64, the streaming kernel -> this): 3072 codes, 1024 / 4096 / 8192 / 18944 /
    // 57344 rows 5.01 -> 3.30, 4.57 -> 3.38, 6.00 -> 4.56, 12.8 -> 8.45, 23.1 -> 19.9; 3584 codes 4.93 -> 3.3, 4.64 -> 3.46, 6.19 -> 4.83,
    // 12.9 -> 8.85, 23.5 -> 21.0 (151936 rows 55.6 -> 51.1); 5120 codes 3.86 -> 3.62, 5.91 -> 4.15, 8.27 -> 6.21, 13.8 -> 12.4, 32.2 -> 28.3
    // (13824 rows f16 g32 / g128 12.2 -> 9.85, 11.0 -> 10.5); 7168 codes 5.31 -> 4.15, 6.22 -> 4.94, 9.56 -> 7.65, 17.9 -> 15.4, 41.5 -> 39.2
    // (129280 rows 91.9 -> 86.4).
    // (fewer rows too: 256 / 512 x 7168 5.24 -> 3.2, 256 / 768 x 3072 4.84 -> 2.7 - 3.2, 4.87 -> 2.7 - 3.4, 512 x 3584 4.97 -> 2.7 - 3.3, 512 x 5120 3.85 -> 3.0 - 3.3)
    if (p.K == 3072 || p.K == 3584 || p.K == 5120 || p.K == 7168) return p.N >= 256;
    if (p.K == 2048) return p.N >= 1024 && p.N <= 20480;
    if (p.K == 6144) return p.N >= 256;   // (256 / 512 / 768 rows 5.31 -> 2.93, 4.19 -> 2.94, 4.18 -> 2.96)
    if (p.K == 4096) return p.N >= 1536 && (p.N <= 40960 || p.N >= 81920);
    return p.N >= 10240 && p.group_size != 128;
}

// The batch on one walk: every matrix as the single one would have to be, the rows counted together.
static bool rows_walk_batch_as_one(const QmvParams& p0, const QmvBatch& b, QmvParams& p) {
    if (b.n < 2 || b.n > 4 || p0.bits != 4) return false;
    p = p0;
    p.gather = GATHER_NONE;
    p.M = 1;
    uint64_t total = 0;
    for (int j = 0; j < b.n; j++) {
        p.w = b.w[j]; p.scales = b.scales[j]; p.biases = b.biases[j]; p.out = b.out[j]; p.N = b.N[j];
        if (!b.w[j] || !b.scales[j] || !b.biases[j] || !b.out[j] || !qmv_rows_walk_takes(p)) return false;
        total += b.N[j];
    }
    if (total > (1u << 24)) return false;
    p.N = (uint32_t)total;
    return true;
}
bool qmv_rows_walk_batched_takes(const QmvParams& p0, const QmvBatch& b) {
    QmvParams p;
    return rows_walk_batch_as_one(p0, b, p);
}
bool qmv_rows_walk_batched_preferred(const QmvParams& p0, const QmvBatch& b) {
    QmvParams p;
    return rows_walk_batch_as_one(p0, b, p) && qmv_rows_walk_preferred(p);   // (sized as one matrix of all the rows)
}
int launch_qmv_rows_walk_batched(const QmvParams& p0, const QmvBatch& b, const LaunchCtx& lc) {
    QmvParams p;
    if (!rows_walk_batch_as_one(p0, b, p)) return fail(ERR_UNSUPPORTED, "qmv walking rows kernel: 2 to 4 matrices of 4-bit codes, rows of 2048 to 8192 codes in steps of 1024 (and 3584), f16 / bf16");
    return launch_rows_walk<false>(p, nullptr, nullptr, lc, &b);
}

int launch_qmv_rows_walk(const QmvParams& p, const LaunchCtx& lc) {
    if (!qmv_rows_walk_takes(p)) return fail(ERR_UNSUPPORTED, "qmv walking rows kernel: one activation row, 4-bit codes, rows of 2048 to 8192 codes in steps of 1024 (and 3584), f16 / bf16");
    return launch_rows_walk<false>(p, nullptr, nullptr, lc);
}

}  // namespace mtq
