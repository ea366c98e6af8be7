// Quantized GEMV for two to four activation rows (out[i, n] = sum_k x[i, k] (s q + b)[n, k]): one wave per four weight
// rows, the 4x4x4 matrix instruction used as it is meant. Replaces the small-batch launches of the reference's
// affine_qmv family (crates/metaltile-std/src/mlx/quantized.rs:141-240 with more than one row of x bound) for rows of
// 4096 or 8192 4-bit codes and 8192 2-bit codes, groups of 32 / 64 / 128, f16 / bf16.
//
// A workgroup of sixteen waves owns 32 consecutive weight rows: eight groups of four rows, each shared by two waves that
// take one half of the reduction each and meet through LDS at the end (sixteen waves per compute unit hide the LDS
// latency of the operand reads that eight do not). Lane 4 b + j of a wave holds the codes of weight row j at the 16-byte
// chunks b, 16 + b, 32 + b, ... of its half of that row, loaded four chunks ahead of use (a wave's load instruction
// covers 256 consecutive bytes of each of its four rows). The same lane supplies, as the first operand,
// activation row j at the same chunks, read from LDS where the workgroup has put the (at most four) activation rows into
// operand order once; block b of the instruction then yields the 4 x 4 products of four activation rows with four weight
// rows over that chunk, every entry of which is wanted. Scales and biases of the 32 rows are staged in LDS by a few
// 16-byte loads per thread instead of one small load per chunk.
//
// Codes become operands as in the one-row kernels: OR-ed into the mantissa of a power of two (MAGIC + q), the offset
// taken out again through the activation sums: out = sum_h s_h dot_h + sum_g (b_g X_g - s_g XM_g), X the plain sum of a
// group's activations and XM the sum weighted with the offsets (4-bit codes: XM = MAGIC X; 2-bit codes carry an offset
// that depends on the pair's position in the dword).
#pragma once

#include <hip/hip_runtime.h>

#include "mtq_device.h"
#include "qmv_rows_common.h"

namespace mtq {

struct QmvRowsFArgs {
    const rp_u32x4* w;
    const uint16_t* s;
    const uint16_t* b;
    const uint16_t* x;
    uint16_t* out;
    uint32_t N;
    uint32_t M;   // 1..4 activation rows
    uint64_t* stamps;   // timeline instances only: [workgroup][wave][ROWS_FEW_STAMPS] readings of the 100 MHz counter, else null
};
#define ROWS_FEW_STAMPS 8


// Shape constants and the LDS layout (bytes) of one instance: T 16-byte chunks per lane and weight row.
template <int BITS, int T, int LOG2G> struct RowsFewGeom {
    static constexpr int CPC = 128 / BITS;                 // codes per chunk
    static constexpr int Q = CPC / 8;                      // 16-byte quarters of a chunk's activations in operand order
    static constexpr int C = 16 * T;                       // chunks per row
    static constexpr int K = C * CPC;
    static constexpr int GPR = K >> LOG2G;                 // groups per row
    static constexpr int SPG = (1 << LOG2G) / (CPC / 2);   // half chunks per group
    static constexpr int NH = (1 << LOG2G) < CPC ? 2 : 1;  // groups a chunk spans
    static constexpr int ROWS = 32;                        // weight rows per workgroup
    static constexpr int THREADS = 1024;
    static constexpr int KP = 2;                           // waves that share four weight rows, one part of the reduction each
    static constexpr int TW = T / KP;                      // chunks per lane, weight row and wave
    static constexpr int SP = GPR + 16;                    // staged scales: elements per row, padded so that four rows fall on different banks
    static constexpr int XP = 0;                           // uint4 [Q][C][4 activation rows]
    static constexpr int XS = XP + Q * C * 4 * 16;         // float [2 C][4]: activation sum of each half chunk
    static constexpr int XM = XS + 2 * C * 16;             // float [2 C][4]: the offset-weighted sums (2-bit codes)
    static constexpr int XG = XM + (BITS == 2 ? 2 * C * 16 : 0);   // float [GPR][4]: sums per group
    static constexpr int XMG = XG + GPR * 16;
    static constexpr int SS = XMG + (BITS == 2 ? GPR * 16 : 0);    // 16-bit [ROWS][SP] scales
    static constexpr int SB = SS + ROWS * SP * 2;                  // biases
    static constexpr int TOTAL = SB + ROWS * SP * 2;
    static constexpr int NPT = C / 64;                     // (weight dword, activation row) pairs each thread prepares: 16 C of them
    static constexpr int SVEC = ROWS * GPR / 8;            // 16-byte vectors of scales (and of biases) to stage
    static constexpr int SPT = (SVEC + THREADS - 1) / THREADS;
    static_assert(C % 64 == 0 && T % KP == 0 && (GPR / 16) % KP == 0, "every thread prepares as much; the reduction and the groups split evenly");
    static_assert(GPR % 16 == 0 && SPG >= 1 && TOTAL <= 160 * 1024 && XS % 16 == 0 && SS % 16 == 0 && SB % 16 == 0, "layout");
};

template <int DT, int BITS, int T, int LOG2G, bool TL = false>
__global__ __launch_bounds__(1024) void qmv_rows_few_kernel(QmvRowsFArgs a) {
    static_assert(BITS == 2 || BITS == 4, "2- or 4-bit codes");
    using Geo = RowsFewGeom<BITS, T, LOG2G>;
    constexpr float MAGIC = DT == DT_BF16 ? 128.0f : 64.0f;   // 4-bit codes: one offset for every pair
    constexpr int CPC = Geo::CPC, Q = Geo::Q, C = Geo::C, K = Geo::K, GPR = Geo::GPR, SPG = Geo::SPG, NH = Geo::NH, SP = Geo::SP;
    uint64_t st[ROWS_FEW_STAMPS];
    auto stamp = [&](int i) {
        if constexpr (TL) {
            RP_KEEP_ORDER();
            st[i] = wall_clock64();
            RP_KEEP_ORDER();
        }
    };
    stamp(0);                                            // wave started
    extern __shared__ __align__(16) unsigned char lds[];
    uint4* const xp = (uint4*)(lds + Geo::XP);       // [(q C + c) 4 + i]
    float* const xs = (float*)(lds + Geo::XS);       // [(2 c + h) 4 + i]
    float* const xm = (float*)(lds + Geo::XM);
    float* const xg = (float*)(lds + Geo::XG);       // [g 4 + i]
    float* const xmg = (float*)(lds + Geo::XMG);
    uint16_t* const ss = (uint16_t*)(lds + Geo::SS); // [r SP + g]
    uint16_t* const sb = (uint16_t*)(lds + Geo::SB);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t blk = lane >> 2, j = lane & 3u;
    const uint32_t quad = wave & 7u, kh = wave >> 3;   // which four rows, which half of the reduction
    const uint32_t row0 = blockIdx.x * (uint32_t)Geo::ROWS;
    const uint32_t row = row0 + quad * 4u + j;
    const uint32_t last = a.N - 1u;
    const uint32_t rowc = min(row, last);            // rows past the end repeat the last one and store nothing
    __builtin_amdgcn_s_setprio(3);
    // ---- loads, all issued before anything is waited for ---------------------------------------------------------
    // A task is the activations that meet one weight dword (8 or 16 values: 16 or 32 bytes) of one activation row. Lane
    // 4 u + i of a wave takes tasks of row i, sixteen consecutive ones per pass, so that a load instruction covers
    // 256 (512) consecutive bytes of each of the four rows, as the weight loads do.
    constexpr int NPT = Geo::NPT, VPT = Q / 4;   // tasks per thread, 16-byte vectors per task
    uint4 xraw[NPT][VPT];
#pragma unroll
    for (int n = 0; n < NPT; n++) {
        const uint32_t pr = (wave * (uint32_t)NPT + (uint32_t)n) * 16u + blk;   // task within the row: chunk pr / 4, dword pr % 4
        if (j < a.M) {
            const uint4* xv = (const uint4*)(a.x + (size_t)j * K + (size_t)pr * (CPC / 4));
#pragma unroll
            for (int v = 0; v < VPT; v++) xraw[n][v] = xv[v];
        } else {
#pragma unroll
            for (int v = 0; v < VPT; v++) xraw[n][v] = make_uint4(0u, 0u, 0u, 0u);
        }
    }
    RP_KEEP_ORDER();
    uint4 sraw[Geo::SPT], braw[Geo::SPT];
#pragma unroll
    for (int n = 0; n < Geo::SPT; n++) {
        const uint32_t v = tid + (uint32_t)(n * Geo::THREADS);
        sraw[n] = braw[n] = make_uint4(0u, 0u, 0u, 0u);
        if (Geo::SVEC % Geo::THREADS == 0 || v < (uint32_t)Geo::SVEC) {
            const uint32_t r = v / (uint32_t)(GPR / 8), c8 = v % (uint32_t)(GPR / 8);
            const size_t off = (size_t)min(row0 + r, last) * GPR + c8 * 8u;
            sraw[n] = *(const uint4*)(a.s + off);
            braw[n] = *(const uint4*)(a.b + off);
        }
    }
    RP_KEEP_ORDER();
    constexpr int TW = Geo::TW;
    const rp_u32x4* wbase = a.w + (size_t)rowc * C + kh * (uint32_t)(TW * 16) + blk;
    // Weight loads run W0 chunks ahead of the chunk being worked on, the first PRE of them issued here. A compute
    // unit takes loads only as fast as earlier ones return: with all of them issued here the slowest wave is still
    // issuing when most of the data is there, and the barriers below, which a wave reaches only after its last load is
    // issued, come that late (8192 x 8192 4-bit, four rows: 12.5 us against 10.4). Measured in one run, us per launch,
    // PRE / W0 = 0/4, 1/4, 4/4, 1/8, 2/8: 4-bit g64 11.1, 11.0, 10.5, 11.3, 10.9; 2-bit g64 8.7, 8.0, 9.1, 8.0, 8.1.
    constexpr int PRE = BITS == 2 ? 1 : (TW < 4 ? TW : 4);
    constexpr int W0 = TW < 4 ? TW : 4;
    static_assert(PRE <= W0, "the first loads are part of the ring");
    rp_u32x4 wv[TW];
#pragma unroll
    for (int t = 0; t < PRE; t++) wv[t] = __builtin_nontemporal_load(wbase + t * 16);
    RP_KEEP_ORDER();
    stamp(1);                                            // first loads issued
    __builtin_amdgcn_s_setprio(0);
    const bool j0 = lane & 1u, j1 = lane & 2u;
    // OR-constants in registers the optimiser cannot see through (an and-or then has one literal operand, its mask)
    uint32_t kor[BITS == 2 ? (DT == DT_F16 ? 5 : 3) : 1];
    if constexpr (BITS == 4) kor[0] = DT == DT_BF16 ? 0x43004300u : 0x54005400u;
    else {
#pragma unroll
        for (int p = 0; p < (DT == DT_F16 ? 5 : 3); p++) kor[p] = rp_crumb_kor<DT>(p);
    }
#pragma unroll
    for (int p = 0; p < (int)(sizeof(kor) / 4); p++) asm volatile("" : "+v"(kor[p]));
    // ---- activations into operand order, into LDS; the sums of each half chunk beside them ---------------------------
    {
        rp_u32x2 ones;
        ones.x = ones.y = DT == DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
#pragma unroll
        for (int n = 0; n < NPT; n++) {
            const uint32_t pr = (wave * (uint32_t)NPT + (uint32_t)n) * 16u + blk, c = pr >> 2, d = pr & 3u;
            rp_f32x4 sx = {0.f, 0.f, 0.f, 0.f}, sm = {0.f, 0.f, 0.f, 0.f};
            if constexpr (BITS == 4) {                // activations 8 d .. 8 d + 7 of the chunk, pairs (e, e + 4)
                const uint4 v = xraw[n][0];
                uint4 o;
                o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
                o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
                o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
                o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
                xp[(d * (uint32_t)C + c) * 4u + j] = o;
                rp_u32x2 a0, a1;
                a0.x = o.x; a0.y = o.y; a1.x = o.z; a1.y = o.w;
                sx = rp_mfma<DT>(a0, ones, sx);
                sx = rp_mfma<DT>(a1, ones, sx);
            } else {                                  // activations 16 d .. 16 d + 15, pairs (e, e + 8)
                const uint4 lo = xraw[n][0], hi = xraw[n][1];
                uint4 o[2];
                o[0].x = __builtin_amdgcn_perm(hi.x, lo.x, 0x05040100u);
                o[0].y = __builtin_amdgcn_perm(hi.x, lo.x, 0x07060302u);
                o[0].z = __builtin_amdgcn_perm(hi.y, lo.y, 0x05040100u);
                o[0].w = __builtin_amdgcn_perm(hi.y, lo.y, 0x07060302u);
                o[1].x = __builtin_amdgcn_perm(hi.z, lo.z, 0x05040100u);
                o[1].y = __builtin_amdgcn_perm(hi.z, lo.z, 0x07060302u);
                o[1].z = __builtin_amdgcn_perm(hi.w, lo.w, 0x05040100u);
                o[1].w = __builtin_amdgcn_perm(hi.w, lo.w, 0x07060302u);
                xp[(2u * d * (uint32_t)C + c) * 4u + j] = o[0];
                xp[((2u * d + 1u) * (uint32_t)C + c) * 4u + j] = o[1];
                const uint32_t pw[8] = {o[0].x, o[0].y, o[0].z, o[0].w, o[1].x, o[1].y, o[1].z, o[1].w};
#pragma unroll
                for (int m = 0; m < 4; m++) {   // pairs 2 m, 2 m + 1
                    rp_u32x2 av, kv;
                    av.x = pw[2 * m]; av.y = pw[2 * m + 1];
                    kv.x = kor[rp_crumb_class<DT>(2 * m)]; kv.y = kor[rp_crumb_class<DT>(2 * m + 1)];
                    sx = rp_mfma<DT>(av, ones, sx);
                    sm = rp_mfma<DT>(av, kv, sm);
                }
            }
            // A lane's own sum is the diagonal entry of its block (its first operand against its own second operand);
            // the other dword of the half chunk is four lanes on.
            float hs = rp_diag(sx, j0, j1);
            hs += __shfl_xor(hs, 4, 64);
            if ((d & 1u) == 0u) xs[(2u * c + (d >> 1)) * 4u + j] = hs;
            if constexpr (BITS == 2) {
                float hm = rp_diag(sm, j0, j1);
                hm += __shfl_xor(hm, 4, 64);
                if ((d & 1u) == 0u) xm[(2u * c + (d >> 1)) * 4u + j] = hm;
            }
        }
    }
#pragma unroll
    for (int n = 0; n < Geo::SPT; n++) {
        const uint32_t v = tid + (uint32_t)(n * Geo::THREADS);
        if (Geo::SVEC % Geo::THREADS == 0 || v < (uint32_t)Geo::SVEC) {
            const uint32_t r = v / (uint32_t)(GPR / 8), c8 = v % (uint32_t)(GPR / 8);
            *(uint4*)(ss + r * SP + c8 * 8u) = sraw[n];
            *(uint4*)(sb + r * SP + c8 * 8u) = braw[n];
        }
    }
    stamp(2);                                            // this thread's chunks prepared, scales stored
    __syncthreads();
    stamp(3);                                            // the workgroup's
    // sums per group: a group is SPG consecutive half chunks
#pragma unroll
    for (int n = 0; n < (GPR * 4 + Geo::THREADS - 1) / Geo::THREADS; n++) {
        const uint32_t idx = tid + (uint32_t)(n * Geo::THREADS);
        if (idx < (uint32_t)(GPR * 4)) {
            const uint32_t g = idx >> 2, i = idx & 3u;
            float X = 0.f, XM = 0.f;
#pragma unroll
            for (int h = 0; h < SPG; h++) {
                X += xs[(g * SPG + h) * 4u + i];
                if constexpr (BITS == 2) XM += xm[(g * SPG + h) * 4u + i];
            }
            xg[idx] = X;
            if constexpr (BITS == 2) xmg[idx] = XM;
        }
    }
    __syncthreads();
    stamp(4);                                            // sums per group there
#pragma unroll
    for (int t = PRE; t < W0; t++) wv[t] = __builtin_nontemporal_load(wbase + t * 16);
    RP_KEEP_ORDER();
    // ---- this wave's four weight rows against the activation rows ------------------------------------------------------
    const uint16_t* const srow = ss + (quad * 4u + j) * SP;
    const uint16_t* const brow = sb + (quad * 4u + j) * SP;
    rp_f32x4 acc = {0.f, 0.f, 0.f, 0.f};   // [activation row] for weight row j, over this lane's chunks
    // bias term over groups blk + 16 kh, blk + 16 kh + 32, ...: b X - s XM (the two waves of a row group take every other
    // run of sixteen groups, whichever half of the reduction those lie in)
#pragma unroll
    for (int gi = 0; gi < GPR / 32; gi++) {
        const uint32_t g = blk + 16u * kh + (uint32_t)(gi * 32);
        const float sf = rp_up<DT>(srow[g]), bf = rp_up<DT>(brow[g]);
        const float4 X = *(const float4*)(xg + g * 4u);
        float4 XM;
        if constexpr (BITS == 2) XM = *(const float4*)(xmg + g * 4u);
        else XM = make_float4(MAGIC * X.x, MAGIC * X.y, MAGIC * X.z, MAGIC * X.w);
        acc.x = fmaf(bf, X.x, acc.x); acc.x = fmaf(0.f - sf, XM.x, acc.x);
        acc.y = fmaf(bf, X.y, acc.y); acc.y = fmaf(0.f - sf, XM.y, acc.y);
        acc.z = fmaf(bf, X.z, acc.z); acc.z = fmaf(0.f - sf, XM.z, acc.z);
        acc.w = fmaf(bf, X.w, acc.w); acc.w = fmaf(0.f - sf, XM.w, acc.w);
    }
    stamp(5);                                            // bias term done
#pragma unroll
    for (int t = 0; t < TW; t++) {
        if (t + W0 < TW) wv[t + W0] = __builtin_nontemporal_load(wbase + (t + W0) * 16);
        RP_KEEP_ORDER();
        const uint32_t c = blk + 16u * (kh * (uint32_t)TW + (uint32_t)t);
        const uint32_t g0 = (c * CPC) >> LOG2G;
        rp_f32x4 dh[NH];
#pragma unroll
        for (int h = 0; h < NH; h++) dh[h] = rp_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t w = wv[t][d];
            constexpr int HSH = NH == 2 ? 1 : 2;   // dword d adds to half d >> HSH
            if constexpr (BITS == 4) {
                const uint4 xo = xp[((uint32_t)(d * C) + c) * 4u + j];
                rp_u32x2 b0, b1, a0, a1;
                if constexpr (DT == DT_BF16) {
                    b0.x = (w & 0x000F000Fu) | kor[0];
                    b0.y = ((w >> 4) & 0x000F000Fu) | kor[0];
                    b1.x = ((w >> 8) & 0x000F000Fu) | kor[0];
                    b1.y = ((w >> 12) & 0x000F000Fu) | kor[0];
                } else {   // (f16: the codes into mantissa bits 4-7, where the second nibble already is)
                    b0.x = ((w << 4) & 0x00F000F0u) | kor[0];
                    b0.y = (w & 0x00F000F0u) | kor[0];
                    b1.x = ((w >> 4) & 0x00F000F0u) | kor[0];
                    b1.y = ((w >> 8) & 0x00F000F0u) | kor[0];
                }
                a0.x = xo.x; a0.y = xo.y;
                a1.x = xo.z; a1.y = xo.w;
                dh[d >> HSH] = rp_mfma<DT>(a0, b0, dh[d >> HSH]);
                dh[d >> HSH] = rp_mfma<DT>(a1, b1, dh[d >> HSH]);
            } else {
                const uint4 xo0 = xp[((uint32_t)(2 * d * C) + c) * 4u + j], xo1 = xp[((uint32_t)((2 * d + 1) * C) + c) * 4u + j];
                const uint32_t xa[8] = {xo0.x, xo0.y, xo0.z, xo0.w, xo1.x, xo1.y, xo1.z, xo1.w};
                uint32_t pq[8];
#pragma unroll
                for (int pi = 0; pi < 8; pi++) {
                    constexpr uint32_t M2 = 0x00030003u;
                    const int p = rp_crumb_class<DT>(pi), sh = rp_crumb_shift<DT>(pi);
                    pq[pi] = ((w >> sh) & (M2 << (2 * p))) | kor[p];
                }
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    rp_u32x2 av, bvv;
                    av.x = xa[2 * m]; av.y = xa[2 * m + 1];
                    bvv.x = pq[2 * m]; bvv.y = pq[2 * m + 1];
                    dh[d >> HSH] = rp_mfma<DT>(av, bvv, dh[d >> HSH]);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < NH; h++) {
            const float sf = rp_up<DT>(srow[g0 + (uint32_t)h]);
            acc.x = fmaf(sf, dh[h].x, acc.x);
            acc.y = fmaf(sf, dh[h].y, acc.y);
            acc.z = fmaf(sf, dh[h].z, acc.z);
            acc.w = fmaf(sf, dh[h].w, acc.w);
        }
    }
    stamp(6);                                            // last chunk done
    // ---- the sixteen lanes that share a weight row add up (lanes j, 4 + j, ..., 60 + j) ------------------------------
    float r[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float v = r[i];
        v += dpp_f32<0x124>(v);            // row_ror:4
        v += dpp_f32<0x128>(v);            // row_ror:8
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        r[i] = v;
    }
    // the wave of the second half hands over through LDS (the half-chunk sums are no longer needed: their space is reused)
    float* const red = xs;   // [(quad 4 + j) 4 + i]
    if (kh == 1u && lane < 4u) *(float4*)(red + (quad * 4u + j) * 4u) = make_float4(r[0], r[1], r[2], r[3]);
    __syncthreads();
    if (kh == 0u && lane < 4u && row <= last) {
        const float4 o = *(const float4*)(red + (quad * 4u + j) * 4u);
        const float other[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
        for (int i = 0; i < 4; i++)
            if ((uint32_t)i < a.M) a.out[(size_t)i * a.N + row] = f32_to_elem_bits<DT>(r[i] + other[i]);
    }
    if constexpr (TL) {
        stamp(7);                                        // stored
        if (lane == 0) {
            uint64_t* dst = a.stamps + ((size_t)blockIdx.x * 16u + wave) * ROWS_FEW_STAMPS;
#pragma unroll
            for (int i = 0; i < ROWS_FEW_STAMPS; i++) dst[i] = st[i];
        }
    }
}

}  // namespace mtq
