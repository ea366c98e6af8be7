// qmv_rows_kernel: the 4-bit, group-of-64 GEMV for rows of 4096 codes, f16 / bf16, one activation row (mt_qmv,
// crates/metaltile-std/src/mlx/quantized.rs:8-308, at the Llama MLP gate / up shape), in a make where nothing is shared
// between waves. One wave owns four consecutive weight rows and issues every load it will ever make at once
// (activations, scales, biases, 8 x 16 bytes of weights per lane); there is no LDS staging, no barrier and no loop.
//   * lane l holds chunks l and 64 + l of a row (16 bytes = 32 codes each: one wave-wide load is 1 KB of one row) and the
//     64 activations that go with them, in registers, in the order the nibble masks deliver the codes;
//   * the dot products run on the matrix cores: v_mfma_f32_4x4x4_16b_{bf16,f16} is sixteen independent 4x4x4 products,
//     and in block b lane 4b + i supplies row i of A (its own activations) and lane 4b + j column j of B (its own codes),
//     so the diagonal element D[j][j], register j % 4 of lane 4b + j, is that lane's own partial dot product: 7 vector
//     instructions per weight dword (4 mask-or, 3 shifts) and 2 matrix instructions, against 11 (4 of them double-length
//     dot2) on the vector ALU;
//   * a chunk lies in one group, so its eight matrix instructions are followed by one multiply with the group's scale
//     (each lane loads the two scales of its own chunks); the bias term is sum_g (b_g - MAGIC s_g) * sum(x_g) with lane
//     g holding the activation sum of group g, exchanged between lanes once per wave;
//   * four rows are summed over the wave with lane swaps and stored by four lanes.
// Arithmetic as everywhere in the GEMV family: exact codes times element-type activations, f32 sums, s * dot + b * sum(x).
// The same source gives the measurement entry point mtq_probe_qmv_rows (include/mtq_measure.h): MODE switches parts off
// (1: no arithmetic, only loads, reduction and stores; 2: weight loads only), and a stamped launch writes per-wave
// readings of the constant-rate counter at six points of a wave's life.
#include <hip/hip_runtime.h>

#include "../../include/mtq.h"
#include "../../include/mtq_measure.h"
#include "mtq_device.h"
#include "mtq_internal.h"
#include "qmv_rows_common.h"

namespace mtq {

struct QmvRowsArgs {
    const rp_u32x4* w;
    const uint16_t* s;
    const uint16_t* b;
    const uint16_t* x;
    uint16_t* out;
    uint32_t N;
    uint64_t* stamps;   // [N / 4][MTQ_ROWS_PROBE_STAMPS] or null
    const uint32_t* route;   // routed instances: expert_offsets[E + 1] or indices[T]; w / s / b then hold E matrices, x and out T rows
    uint32_t E, T;
};

template <bool TL> __device__ __forceinline__ void rp_stamp(uint64_t (&st)[MTQ_ROWS_PROBE_STAMPS], int i) {
    if constexpr (TL) {
        RP_KEEP_ORDER();
        st[i] = wall_clock64();
        RP_KEEP_ORDER();
    }
}

template <int DT, int MODE, bool TL, int GM>
__device__ __forceinline__ void qmv_rows_body(const QmvRowsArgs& a) {
    static_assert(GM == GATHER_NONE || (MODE == 0 && !TL), "routed instances are product instances");
    constexpr float MAGIC = DT == DT_BF16 ? 128.0f : 64.0f;
    constexpr int GPR = 64, C = 128, R = 4;
    uint64_t st[MTQ_ROWS_PROBE_STAMPS];
    rp_stamp<TL>(st, 0);                                  // wave started
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t gw = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const uint32_t r0 = gw * R;
    if (r0 >= a.N) return;
    RowsRoute rt;
    if (!rows_route<GM>(a.route, a.E, a.T, lane, rt)) return;
    const size_t er0 = (size_t)rt.expert * a.N + r0;   // this wave's first row among the rows of all experts
    for (uint32_t pass = 0; pass < rt.n_pass; pass++) {
    const uint32_t trow = rows_route_row<GM>(rt, pass);
    const uint16_t* const xrow = a.x + (size_t)trow * 4096u;
    uint16_t* const orow = a.out + (size_t)trow * a.N;
    __builtin_amdgcn_s_setprio(3);
    uint4 xraw[2][4];
    if constexpr (MODE != 2) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint4* xv = (const uint4*)(xrow + ((size_t)i * 64 + lane) * 32);
#pragma unroll
            for (int v = 0; v < 4; v++) xraw[i][v] = xv[v];
        }
    }
    RP_KEEP_ORDER();
    uint32_t s0[R], s1[R], bb[R];
    if constexpr (MODE != 2) {
        const uint16_t* sp = a.s + er0 * GPR + (lane >> 1);
        const uint16_t* bp = a.b + er0 * GPR + lane;
#pragma unroll
        for (int r = 0; r < R; r++) { s0[r] = sp[r * GPR]; s1[r] = sp[r * GPR + 32]; bb[r] = bp[r * GPR]; }
    }
    RP_KEEP_ORDER();
    const rp_u32x4* wbase = a.w + er0 * C + lane;
    rp_u32x4 wv[R][2];
    // (Every load at once is the fastest form here: with the loads of only one, two or three rows ahead of the row
    // being worked on, 14336 x 4096 bf16 takes 8.3, 8.5 and 9.1 us against 7.75 in the same run.)
#pragma unroll
    for (int r = 0; r < R; r++) {
        wv[r][0] = __builtin_nontemporal_load(wbase + r * C);
        wv[r][1] = __builtin_nontemporal_load(wbase + r * C + 64);
    }
    RP_KEEP_ORDER();
    __builtin_amdgcn_s_setprio(0);
    rp_stamp<TL>(st, 1);                                  // every load issued
    const bool j0 = lane & 1u, j1 = lane & 2u;
    uint32_t xp[2][16];
    float gsum = 0.f;
    uint32_t kor = DT == DT_BF16 ? 0x43004300u : 0x54005400u;   // (2^7, 2^7) in bf16, a code OR-ed into mantissa bits 0-3; (2^6, 2^6) in f16, a code in mantissa bits 4-7: MAGIC + q
    asm volatile("" : "+v"(kor));
    if constexpr (MODE == 0) {
        rp_u32x2 ones;
        ones.x = ones.y = DT == DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
        float xsum[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            rp_f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint4 v = xraw[i][d];   // activations 8 d .. 8 d + 7 of the chunk; pairs (j, j + 4) match the masks
                xp[i][4 * d + 0] = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
                xp[i][4 * d + 1] = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
                xp[i][4 * d + 2] = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
                xp[i][4 * d + 3] = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
                rp_u32x2 a0, a1;
                a0.x = v.x; a0.y = v.y; a1.x = v.z; a1.y = v.w;
                sacc = rp_mfma<DT>(a0, ones, sacc);
                sacc = rp_mfma<DT>(a1, ones, sacc);
            }
            xsum[i] = rp_diag(sacc, j0, j1);
        }
        // group g = chunks 2g and 2g + 1: lanes 2 (g % 32) and + 1 of chunk set g / 32; lane g keeps the sum of group g
        const uint32_t gl = (lane & 31u) * 8u;
        const float t0 = __int_as_float(__builtin_amdgcn_ds_bpermute((int)gl, __float_as_int(xsum[0]))) +
                         __int_as_float(__builtin_amdgcn_ds_bpermute((int)gl + 4, __float_as_int(xsum[0])));
        const float t1 = __int_as_float(__builtin_amdgcn_ds_bpermute((int)gl, __float_as_int(xsum[1]))) +
                         __int_as_float(__builtin_amdgcn_ds_bpermute((int)gl + 4, __float_as_int(xsum[1])));
        gsum = lane < 32 ? t0 : t1;
    }
    rp_stamp<TL>(st, 2);                                  // activations in operand order
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        if constexpr (MODE == 0) {
            const float sf0 = rp_up<DT>(s0[r]), sf1 = rp_up<DT>(s1[r]);
            rp_f32x4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < 4; q++) {
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const uint32_t w = wv[r][i][q];
                    rp_u32x2 b0, b1, a0, a1;
                    if constexpr (DT == DT_BF16) {
                        b0.x = (w & 0x000F000Fu) | kor;
                        b0.y = ((w >> 4) & 0x000F000Fu) | kor;
                        b1.x = ((w >> 8) & 0x000F000Fu) | kor;
                        b1.y = ((w >> 12) & 0x000F000Fu) | kor;
                    } else {   // (f16: the codes into mantissa bits 4-7, where the second nibble already is)
                        b0.x = ((w << 4) & 0x00F000F0u) | kor;
                        b0.y = (w & 0x00F000F0u) | kor;
                        b1.x = ((w >> 4) & 0x00F000F0u) | kor;
                        b1.y = ((w >> 8) & 0x00F000F0u) | kor;
                    }
                    a0.x = xp[i][4 * q + 0]; a0.y = xp[i][4 * q + 1];
                    a1.x = xp[i][4 * q + 2]; a1.y = xp[i][4 * q + 3];
                    if (i == 0) { d0 = rp_mfma<DT>(a0, b0, d0); d0 = rp_mfma<DT>(a1, b1, d0); }
                    else { d1 = rp_mfma<DT>(a0, b0, d1); d1 = rp_mfma<DT>(a1, b1, d1); }
                }
            }
            acc[r] = fmaf(sf1, rp_diag(d1, j0, j1), sf0 * rp_diag(d0, j0, j1));
        } else {
            uint32_t f = wv[r][0][0] ^ wv[r][0][1] ^ wv[r][0][2] ^ wv[r][0][3] ^ wv[r][1][0] ^ wv[r][1][1] ^ wv[r][1][2] ^ wv[r][1][3];
            float t = __uint_as_float(f & 0x3FFFFFFFu);
            if constexpr (MODE == 1)
                t += rp_up<DT>(s0[r]) + rp_up<DT>(s1[r]) + rp_up<DT>(bb[r]) + __uint_as_float(xraw[0][0].x << 16);
            acc[r] = t;
        }
        if (r == 0) rp_stamp<TL>(st, 3);                  // first row done
    }
    if constexpr (MODE == 0) {
        // (b - MAGIC s) of group `lane` times that group's activation sum; the group's scale is held by lane 2 (lane % 32)
        const uint32_t src = (lane & 31u) * 8u;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float sa = rp_up<DT>((uint32_t)__builtin_amdgcn_ds_bpermute((int)src, (int)s0[r]));
            const float sb = rp_up<DT>((uint32_t)__builtin_amdgcn_ds_bpermute((int)src, (int)s1[r]));
            acc[r] = fmaf(rp_up<DT>(bb[r]) - MAGIC * (lane < 32 ? sa : sb), gsum, acc[r]);
        }
    }
    rp_stamp<TL>(st, 4);                                  // all rows done
    float tot = rp_swap16_add(rp_swap32_add(acc[0], acc[1]), rp_swap32_add(acc[2], acc[3]));
    tot += dpp_f32<0xB1>(tot);
    tot += dpp_f32<0x4E>(tot);
    tot += dpp_f32<0x141>(tot);
    tot += dpp_f32<0x140>(tot);
    // 16-lane row r of the wave now holds the total of row {0, 2, 1, 3}[r]
    const uint32_t slot = ((lane >> 4) & 1u) * 2u + (lane >> 5);
    if ((lane & 15u) == 0) orow[r0 + slot] = f32_to_elem_bits<DT>(tot);
    rp_stamp<TL>(st, 5);                                  // stored
    if constexpr (TL) {
        if (lane == 0)
            for (int i = 0; i < MTQ_ROWS_PROBE_STAMPS; i++) a.stamps[(size_t)gw * MTQ_ROWS_PROBE_STAMPS + i] = st[i];
    }
    }   // pass
}
template <int DT, int MODE, bool TL>
__global__ __launch_bounds__(1024) void qmv_rows_kernel(QmvRowsArgs a) { qmv_rows_body<DT, MODE, TL, GATHER_NONE>(a); }
template <int DT, int GM>
__global__ __launch_bounds__(1024) void qmv_rows_routed_kernel(QmvRowsArgs a) { qmv_rows_body<DT, 0, false, GM>(a); }

// ---- one wave per row, activations shared by the workgroup: other row lengths, group sizes and 2-bit codes -----------
// The same ownership (lane l holds chunks l, 64 + l, ... of a row, the diagonal of the 4x4x4 blocks, scales loaded per
// lane), with what longer rows change. A lane's share of the activations grows with the row (112 registers for 14336
// 4-bit codes), so a wave owns one row and a workgroup of sixteen waves owns sixteen - one workgroup per compute unit at
// 4096 rows. And the activations are put into operand order once per workgroup, not once per wave: thread t prepares
// chunk t (its values and their sums) into LDS while the first weights are in flight, and after the one barrier of the
// kernel every lane takes its operands from there (laid out by 16-byte quarter, so that consecutive lanes read
// consecutive 16 bytes). Measured in one run on 4096 x 14336 bf16: streaming kernel 8.60 us, this with two rows per wave
// on eight waves 8.34, one row per wave and every load issued at the start 8.11, as here (loads four chunks ahead, see
// below) 7.2. (The same sharing for rows of 4096 4-bit codes gains nothing over one preparation per wave: 8.00 against
// 7.95 us.)
//
// A chunk is 16 bytes: CPC = 32 4-bit or 64 2-bit codes. Groups of 32, 64 or 128 codes: the two halves of a chunk are
// accumulated apart and each takes the scale of its own group (the same one unless 2-bit codes come in groups of 32).
// 2-bit codes are made operands without moving them: a masked pair of crumbs (i, i + 8) of a weight dword, left at
// its bit position 2 p inside the two 16-bit halves and OR-ed into the mantissa of 2^(MB - 2 p) (MB = 10 mantissa bits
// for f16, 7 for bf16), is the pair (2^(MB - 2p) + q_i, 2^(MB - 2p) + q_(i+8)) exactly: five positions fit an f16
// mantissa and three a bf16 one, so a dword's eight pairs cost 8 mask-or and one shift (f16) or two (bf16) instead of
// eight shifts. The offset each pair carries depends on its position; sum(offset_k x_k) over a half chunk is worked out
// once per workgroup by the same matrix instruction with the OR-constants as its second operand, and leaves with the
// bias term: out = sum_h s_h dot_h + sum_g (b_g X_g - s_g XM_g), X the plain and XM the offset-weighted activation sums.
struct QmvRowsLArgs {
    const rp_u32x4* w;
    const uint16_t* s;
    const uint16_t* b;
    const uint16_t* x;
    uint16_t* out;
    uint32_t N;
    const uint32_t* route;   // routed instances (see RowsRoute): expert_offsets[E + 1] or indices[T]
    uint32_t E, T;
};

// TAIL: the chunks of the last 64 a row has (0: all 64; a row of 11008 codes is 344 chunks, CH = 6 and TAIL = 24). The lanes
// past them load the row's last chunk and add nothing.
template <int DT, int BITS, int CH, int LOG2G, int GM, int TAIL = 0>
__device__ __forceinline__ void qmv_rows_long_body(const QmvRowsLArgs& a) {
    static_assert(BITS == 2 || BITS == 4, "2- or 4-bit codes");
    static_assert(TAIL == 0 || (TAIL > 0 && TAIL < 64 && TAIL % 4 == 0 && BITS == 4 && GM == GATHER_NONE), "ragged rows: 4-bit codes, unrouted, whole 4-lane blocks");
    constexpr float MAGIC = DT == DT_BF16 ? 128.0f : 64.0f;   // 4-bit codes: one offset for every pair
    constexpr int CPC = 128 / BITS;        // codes per chunk
    constexpr int Q = CPC / 8;             // 16-byte quarters of a chunk's activations in operand order (4 pair dwords each)
    constexpr int C = TAIL ? 64 * (CH - 1) + TAIL : 64 * CH;   // chunks per row
    constexpr int K = C * CPC;
    constexpr int GPR = K >> LOG2G;        // groups per row
    constexpr int GPL = GPR > 256 ? 8 : GPR > 128 ? 4 : GPR > 64 ? 2 : 1;   // groups a lane owns in the bias term (lanes below GPR / GPL)
    constexpr int SPG = (1 << LOG2G) / (CPC / 2);            // half chunks per group
    constexpr int NH = (1 << LOG2G) < CPC ? 2 : 1;           // groups a chunk spans: its halves are then accumulated and scaled apart
    static_assert(C <= 1024, "one thread per chunk");
    static_assert(LOG2G >= 5 && LOG2G <= 7 && GPR % GPL == 0 && GPR / GPL <= 64 && SPG >= 1, "groups of 32, 64 or 128 codes, at most 512 per row");
    __shared__ __align__(16) uint32_t xp_lds[Q][C][4];   // [quarter][chunk][4 pair dwords]
    __shared__ __align__(16) float xs_lds[2 * C];        // activation sum of each half chunk
    __shared__ __align__(16) float xm_lds[BITS == 2 ? 2 * C : 4];   // 2-bit codes: the sum weighted with the pairs' offsets
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t r0 = blockIdx.x * (blockDim.x >> 6) + wave;   // (a workgroup is 8 or 16 waves, at least C threads)
    const bool live = r0 < a.N;
    RowsRoute rt;
    if (!rows_route<GM>(a.route, a.E, a.T, lane, rt)) return;   // (the same for every wave of the workgroup: no barrier is left waiting)
    const size_t rr = (size_t)rt.expert * a.N + (live ? r0 : 0u);   // idle waves of the last workgroup still prepare their chunks
    for (uint32_t pass = 0; pass < rt.n_pass; pass++) {
    const uint32_t trow = rows_route_row<GM>(rt, pass);
    const uint16_t* const xrow = a.x + (size_t)trow * K;
    uint16_t* const orow = a.out + (size_t)trow * a.N;
    __builtin_amdgcn_s_setprio(3);
    // this thread's chunk of the activations
    uint4 xraw[Q];
    if (tid < (uint32_t)C) {
        const uint4* xv = (const uint4*)(xrow + (size_t)tid * CPC);
#pragma unroll
        for (int v = 0; v < Q; v++) xraw[v] = xv[v];
    }
    RP_KEEP_ORDER();
    // scales of the two halves of this lane's CH chunks, and for the bias term scales and biases of groups GPL lane .. + GPL - 1
    uint32_t sc[CH][NH];
    uint32_t sw[4] = {0u, 0u, 0u, 0u}, bw[4] = {0u, 0u, 0u, 0u};   // GPL elements each, two per dword
    const uint32_t gl = min(lane, (uint32_t)(GPR / GPL - 1));
    {
        const uint16_t* sp = a.s + rr * GPR;
        const uint16_t* bp = a.b + rr * GPR;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t k0 = (TAIL && i == CH - 1 ? min((uint32_t)(i * 64) + lane, (uint32_t)(C - 1)) : (uint32_t)(i * 64) + lane) * CPC;   // (past the row's end: its last chunk)
            sc[i][0] = sp[k0 >> LOG2G];
            if constexpr (NH == 2) sc[i][1] = sp[(k0 + CPC / 2) >> LOG2G];
        }
        if constexpr (GPL == 8) {   // (rows of 448 groups: 896 bytes, the operands 16-byte aligned)
            const uint4 sv = ((const uint4*)sp)[gl], bv = ((const uint4*)bp)[gl];
            sw[0] = sv.x; sw[1] = sv.y; sw[2] = sv.z; sw[3] = sv.w;
            bw[0] = bv.x; bw[1] = bv.y; bw[2] = bv.z; bw[3] = bv.w;
        } else if constexpr (GPL == 4) {
            const uint2 sv = ((const uint2*)sp)[gl], bv = ((const uint2*)bp)[gl];
            sw[0] = sv.x; sw[1] = sv.y; bw[0] = bv.x; bw[1] = bv.y;
        } else if constexpr (GPL == 2) {
            sw[0] = ((const uint32_t*)sp)[gl];
            bw[0] = ((const uint32_t*)bp)[gl];
        } else {
            sw[0] = sp[gl];
            bw[0] = bp[gl];
        }
    }
    RP_KEEP_ORDER();
    const rp_u32x4* wbase = a.w + rr * C + lane;
    const rp_u32x4* wlast = a.w + rr * C + min((uint32_t)((CH - 1) * 64) + lane, (uint32_t)(C - 1));   // the lane's chunk of the last group, inside the row
    rp_u32x4 wv[CH];
    // Rows of more than four chunks per lane: the loads run four chunks ahead of the chunk being worked on and only two
    // are issued before the activations are prepared. A compute unit takes loads only as fast as earlier ones return, so
    // with all seven issued here the slowest wave reaches the barrier below when most of the data has arrived, and all
    // the arithmetic follows in one piece (4096 x 14336 bf16, same run: 8.40 us; two ahead of the barrier and four in
    // flight 7.17; 1 / 4 7.21, 3 / 4 7.39, 2 / 3 7.3, 2 / 5 7.55). Rows of two or four chunks are faster with every load
    // at once (8192 x 8192 4-bit: 7.82 us against 9.05 with one ahead of the barrier, 10.2 with two).
    constexpr int W0 = CH > 4 ? 4 : CH, PRE = CH > 4 ? 2 : CH;
#pragma unroll
    for (int i = 0; i < PRE; i++) wv[i] = TAIL && i == CH - 1 ? __builtin_nontemporal_load(wlast) : __builtin_nontemporal_load(wbase + i * 64);
    RP_KEEP_ORDER();
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
    // ---- the chunk into operand order, into LDS ------------------------------------------------------------------
    if (tid < (uint32_t)C) {
        rp_u32x2 ones;
        ones.x = ones.y = DT == DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
        rp_f32x4 sx[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, sm[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        if constexpr (BITS == 4) {
#pragma unroll
            for (int d = 0; d < 4; d++) {       // weight dword d: activations 8 d .. 8 d + 7, pairs (j, j + 4)
                const uint4 v = xraw[d];
                uint4 o;
                o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
                o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
                o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
                o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
                *(uint4*)xp_lds[d][tid] = o;
                rp_u32x2 a0, a1;
                a0.x = o.x; a0.y = o.y; a1.x = o.z; a1.y = o.w;
                sx[d / 2] = rp_mfma<DT>(a0, ones, sx[d / 2]);
                sx[d / 2] = rp_mfma<DT>(a1, ones, sx[d / 2]);
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
                    kv.x = kor[rp_crumb_class<DT>(2 * m)]; kv.y = kor[rp_crumb_class<DT>(2 * m + 1)];
                    sx[d / 2] = rp_mfma<DT>(av, ones, sx[d / 2]);
                    sm[d / 2] = rp_mfma<DT>(av, kv, sm[d / 2]);
                }
            }
        }
        xs_lds[2 * tid] = rp_diag(sx[0], j0, j1);
        xs_lds[2 * tid + 1] = rp_diag(sx[1], j0, j1);
        if constexpr (BITS == 2) {
            xm_lds[2 * tid] = rp_diag(sm[0], j0, j1);
            xm_lds[2 * tid + 1] = rp_diag(sm[1], j0, j1);
        }
    }
    __syncthreads();
    if constexpr (GM == GATHER_NONE) {
        if (!live) return;
    }
    if (GM == GATHER_NONE || live) {
#pragma unroll
    for (int i = PRE; i < W0; i++) wv[i] = TAIL && i == CH - 1 ? __builtin_nontemporal_load(wlast) : __builtin_nontemporal_load(wbase + i * 64);
    RP_KEEP_ORDER();
    // bias term: over this lane's GPL groups, b X - s XM (4-bit codes: XM = MAGIC X). A group is SPG half chunks, so the
    // lane's groups are a run of GPL SPG consecutive half-chunk sums.
    float t = 0.f;
    if (lane < (uint32_t)(GPR / GPL)) {
        constexpr int RUN = GPL * SPG;
        float xs[RUN], xm[RUN];
        if constexpr (RUN % 4 == 0) {
#pragma unroll
            for (int h = 0; h < RUN / 4; h++) {
                const float4 v = *(const float4*)&xs_lds[lane * RUN + 4 * h];
                xs[4 * h] = v.x; xs[4 * h + 1] = v.y; xs[4 * h + 2] = v.z; xs[4 * h + 3] = v.w;
                if constexpr (BITS == 2) {
                    const float4 m = *(const float4*)&xm_lds[lane * RUN + 4 * h];
                    xm[4 * h] = m.x; xm[4 * h + 1] = m.y; xm[4 * h + 2] = m.z; xm[4 * h + 3] = m.w;
                }
            }
        } else {
#pragma unroll
            for (int h = 0; h < RUN; h++) {
                xs[h] = xs_lds[lane * RUN + h];
                if constexpr (BITS == 2) xm[h] = xm_lds[lane * RUN + h];
            }
        }
#pragma unroll
        for (int v = 0; v < GPL; v++) {
            float X = 0.f, XM = 0.f;
#pragma unroll
            for (int h = 0; h < SPG; h++) {
                X += xs[v * SPG + h];
                if constexpr (BITS == 2) XM += xm[v * SPG + h];
            }
            if constexpr (BITS == 4) XM = MAGIC * X;
            const float sf = rp_up<DT>((sw[v >> 1] >> (16 * (v & 1))) & 0xFFFFu), bf = rp_up<DT>((bw[v >> 1] >> (16 * (v & 1))) & 0xFFFFu);
            t = fmaf(bf, X, t);
            t = fmaf(0.f - sf, XM, t);
        }
    }
#pragma unroll
    for (int i = 0; i < CH; i++) {
        if (i + W0 < CH) wv[i + W0] = TAIL && i + W0 == CH - 1 ? __builtin_nontemporal_load(wlast) : __builtin_nontemporal_load(wbase + (i + W0) * 64);
        RP_KEEP_ORDER();
        rp_f32x4 dh[NH];
#pragma unroll
        for (int h = 0; h < NH; h++) dh[h] = rp_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t w = wv[i][d];
            constexpr int HSH = NH == 2 ? 1 : 2;   // dword d adds to half d >> HSH
            if constexpr (BITS == 4) {
                const uint4 xo = *(const uint4*)xp_lds[d][TAIL && i == CH - 1 ? min((uint32_t)(i * 64) + lane, (uint32_t)(C - 1)) : (uint32_t)(i * 64) + lane];
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
                const uint4 xo0 = *(const uint4*)xp_lds[2 * d][i * 64 + lane], xo1 = *(const uint4*)xp_lds[2 * d + 1][i * 64 + lane];
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
            const float ti = fmaf(rp_up<DT>(sc[i][h]), rp_diag(dh[h], j0, j1), t);
            t = TAIL && i == CH - 1 && lane >= (uint32_t)TAIL ? t : ti;   // (lanes past the row's end hold its last chunk again)
        }
    }
    t += __shfl_xor(t, 32, 64);
    t += dpp_f32<0xB1>(t);
    t += dpp_f32<0x4E>(t);
    t += dpp_f32<0x141>(t);
    t += dpp_f32<0x140>(t);
    t += __shfl_xor(t, 16, 64);
    if (lane == 0) orow[r0] = f32_to_elem_bits<DT>(t);
    }   // live
    if constexpr (GM != GATHER_NONE) {
        if (pass + 1 < rt.n_pass) __syncthreads();   // the next pass overwrites the activations in LDS
    }
    }   // pass
}
template <int DT, int BITS, int CH, int LOG2G>
__global__ __launch_bounds__(1024) void qmv_rows_long_kernel(QmvRowsLArgs a) { qmv_rows_long_body<DT, BITS, CH, LOG2G, GATHER_NONE>(a); }
// 4-bit codes on rows that end inside a group of 64 chunks (11008 / 13824 / 18944 / 27648 codes: the widths of other models).
template <int DT, int CH, int LOG2G, int TAIL>
__global__ __launch_bounds__(1024) void qmv_rows_long_ragged_kernel(QmvRowsLArgs a) { qmv_rows_long_body<DT, 4, CH, LOG2G, GATHER_NONE, TAIL>(a); }
template <int DT, int BITS, int CH, int LOG2G, int GM>
__global__ __launch_bounds__(1024) void qmv_rows_long_routed_kernel(QmvRowsLArgs a) { qmv_rows_long_body<DT, BITS, CH, LOG2G, GM>(a); }

template <int DT> static const void* qmv_rows_fn(int mode, bool tl) {
    switch (mode) {
        case 0: return tl ? (const void*)qmv_rows_kernel<DT, 0, true> : (const void*)qmv_rows_kernel<DT, 0, false>;
        case 1: return tl ? (const void*)qmv_rows_kernel<DT, 1, true> : (const void*)qmv_rows_kernel<DT, 1, false>;
        default: return tl ? (const void*)qmv_rows_kernel<DT, 2, true> : (const void*)qmv_rows_kernel<DT, 2, false>;
    }
}

template <int DT> static const void* qmv_rows_routed_fn(int gather) {
    return gather == GATHER_CSR       ? (const void*)qmv_rows_routed_kernel<DT, GATHER_CSR>
           : gather == GATHER_INDICES ? (const void*)qmv_rows_routed_kernel<DT, GATHER_INDICES>
                                      : (const void*)qmv_rows_routed_kernel<DT, GATHER_SINGLE>;
}

// slots: grid rows of a routed launch (the experts that can have a row), 1 for a plain one
static int launch_rows(int dtype, const void* w, const void* s, const void* b, const void* x, void* out, uint32_t N, int mode,
                       uint64_t* stamps, const LaunchCtx& lc, int gather = GATHER_NONE, const uint32_t* route = nullptr, uint32_t E = 1,
                       uint32_t T = 1, uint32_t slots = 1) {
    QmvRowsArgs a{(const rp_u32x4*)w, (const uint16_t*)s, (const uint16_t*)b, (const uint16_t*)x, (uint16_t*)out, N, stamps, route, E, T};
    void* args[] = {&a};
    const void* fn = gather != GATHER_NONE ? (dtype == DT_BF16 ? qmv_rows_routed_fn<DT_BF16>(gather) : qmv_rows_routed_fn<DT_F16>(gather))
                     : dtype == DT_BF16    ? qmv_rows_fn<DT_BF16>(mode, stamps != nullptr)
                                           : qmv_rows_fn<DT_F16>(mode, stamps != nullptr);
    // A workgroup is only a container here (no LDS, no barrier). It is sized so that the workgroups are a whole number
    // per compute unit: one of up to 16 waves up to 16384 rows (14336 rows: 256 workgroups of 14 waves, 7.88 us against
    // 7.97 as 896 workgroups of 4; 1024 rows: 256 single waves, 3.15 against 3.60), beyond that as few rounds of at most
    // 8 waves as it takes (28672 rows: 1024 workgroups of 7 waves, 13.25 us against 14.1 as 1792 of 4).
    // (a routed launch counts the waves of every grid row: two rows on experts of 14336 rows run as 2 x 512 workgroups
    // of 7 waves, 15.3 us against 15.7 as 2 x 256 of 14, four rows 29.3 against 31.1)
    const uint32_t waves = (N + 3u) / 4u, total = waves * slots;
    const uint32_t rounds = total <= 256u * 16u ? 1u : (total + 256u * 8u - 1u) / (256u * 8u);
    const uint32_t per_slot = (256u * rounds + slots - 1u) / slots;   // workgroups per grid row
    uint32_t wpw = (waves + per_slot - 1u) / per_slot;
    if (wpw > 16u) wpw = 16u;
    hipError_t e = launch_kernel(fn, dim3((waves + wpw - 1u) / wpw, slots), dim3(wpw * 64u), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "qmv rows kernel launch");
    return ERR_OK;
}

// chunks of 16 bytes per lane and row for the one-row-per-wave kernel, or 0 if it has no instance for the shape
// (rows whose last group of 64 chunks is not full count that group)
static int rows_long_ch(const QmvParams& p) {
    if (p.bits != 2 && p.bits != 4) return 0;
    const uint32_t G = p.group_size, cpc = 128u / (uint32_t)p.bits;
    if (G != 32 && G != 64 && G != 128) return 0;
    // 4-bit codes in groups of 64 / 128 on the row lengths of other models: 10240, 12288, 18432 codes (whole groups of 64
    // chunks) and 11008, 13824, 18944, 27648 (the last group partly filled). Every lane's groups of the bias term are one
    // aligned load: up to 256 groups per row the rows' scales are 8-byte multiples, beyond that 16-byte multiples.
    if (p.bits == 4 && G >= 64 && p.gather == GATHER_NONE) {
        static const struct { uint32_t K; int ch; } kMore[] = {{10240, 5}, {12288, 6}, {18432, 9}, {11008, 6}, {13824, 7}, {18944, 10}, {27648, 14}};
        for (const auto& m : kMore) {
            if (p.K != m.K) continue;
            if (p.K / G > 256u && ((uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)) return 0;
            return m.ch;
        }
    }
    if (p.K % (64u * cpc) || p.K / G > 512u || (p.K / G) % 8u) return 0;
    const uint32_t ch = p.K / (64u * cpc);
    if (p.K / G > 256u && ((uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16)) return 0;   // (a lane's eight groups of the bias term: one 16-byte load)
    // 8192, 14336, 28672 codes (16384, in workgroups of eight rows as for 14336, is behind the streaming kernel:
    // 8192 x 16384 16.5 us against 14.8)
    if (p.bits == 4 && (ch == 4 || ((ch == 7 || ch == 14) && G >= 64))) return (int)ch;
    if (p.bits == 2 && (ch == 2 || ch == 4) && p.K / G <= 256u) return (int)ch;     // 8192, 16384 codes
    return 0;
}

bool qmv_rows_takes(const QmvParams& p) {
    if ((p.dtype != DT_F16 && p.dtype != DT_BF16) || p.N == 0) return false;
    const bool routed = p.gather == GATHER_CSR || p.gather == GATHER_INDICES || p.gather == GATHER_SINGLE;
    if (routed) {
        // at most 64 experts and 64 rows (the routing is read by one wave-wide load; the single-index form reads one id
        // and takes any number of experts); 4-bit codes in groups of 64 on rows of 4096, 8192 or 14336 codes (the
        // instances that exist); every expert's block of scales as aligned as the first
        if (!p.route || p.E == 0 || p.bits != 4 || p.group_size != 64) return false;
        if (p.gather != GATHER_SINGLE && (p.E > 64 || p.T == 0 || p.T > 64)) return false;
        if (((size_t)p.N * (p.K / 64u) * 2u) % 8u) return false;
    } else if (p.gather != GATHER_NONE || p.M != 1) {
        return false;
    }
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.scales % 8 || (uintptr_t)p.biases % 8 || (uintptr_t)p.out % 2) return false;
    if (p.bits == 4 && p.group_size == 64 && p.K == 4096) return p.N % 4 == 0;   // one wave per four rows
    const int ch = rows_long_ch(p);
    return routed ? (p.K == 8192 || p.K == 14336) && (ch == 4 || ch == 7) : ch != 0;
}

// Where these kernels are the fastest the library has (measured against the streaming kernel in one run, f16 / bf16, us):
// 14336 x 4096 4-bit g64 8.11 -> 7.86; 4096 x 14336 8.60 -> 8.11 on one machine, 8.63 -> 8.73 on another; 8192 x 8192:
// 2-bit g32 / g64 / g128 8.98 / 8.55 / 8.41 -> 6.65 / 6.16 / 6.03, 4-bit 9.63 / 9.47 / 9.27 -> 8.53 / 7.90 / 7.78.
// Small matrices stay where they were (a workgroup here is sixteen rows: few rows leave compute units idle).
bool qmv_rows_preferred(const QmvParams& p) {
    // (rows of 8192 4-bit codes from 256 weight rows: 256 / 512 / 768 rows 3.51 -> 3.15, 3.56 -> 3.17, 3.61 -> 3.22)
    if (!qmv_rows_takes(p) || p.N < (p.bits == 4 && p.K == 8192 && p.gather == GATHER_NONE ? 256u : 1024u)) return false;
    // Routed rows: fewer rows than experts, each streaming its expert's matrix on its own grid row. 8 experts, bf16, us,
    // against the kernels that served these before (the one-row streaming kernel for one row, the matrix-core GEMV
    // beyond): 14336 x 4096, 1 / 2 / 3 / 4 rows on distinct experts 10.8 -> 8.4, 17.6 -> 15.8, 22.4 -> 23.3, 28.0 -> 31.1,
    // two rows on one expert 16.4 -> 14.0; 4096 x 14336: 9.0 -> 8.0, 16.6 -> 14.6, 41.8 -> 21.0, 34.8 -> 27.8, 15.8 -> 13.4.
    if (p.gather == GATHER_SINGLE) return true;   // (one row, as the plain launch)
    if (p.gather != GATHER_NONE) return p.T < p.E && p.T <= (p.K == 4096 ? 2u : 4u);
    // Large launches have a steady state, and there the streaming kernel is ahead again (bf16, us, streaming / these):
    // rows of 4096 codes, 28672 / 57344 / 128256 rows 13.1 / 13.5, 22.6 / 24.1, 47.6 / 50.4 (14336 rows: 8.1 / 7.85);
    // rows of 8192, 16384 / 28672 rows 14.7 / 14.3, 22.5 / 23.0. Longer rows stay here at every size (14336 codes, 8192 /
    // 14336 / 28672 rows 14.2 / 12.65, 21.5 / 20.35, 37.8 / 36.5; 28672 codes, 4096 / 8192 / 16384 rows 14.6 / 12.1, 24.5 /
    // 22.3, 51.8 / 42.1), and so do 2-bit codes (28672 x 8192: 19.7 / 17.6).
    // The row lengths of other models (bf16 g64, us in a chain, the streaming kernel or the matrix-core GEMV -> these): 4096 x 10240 7.20 -> 5.83, 1024 /
    // 4096 / 8192 x 11008 5.53 -> 3.65, 7.91 -> 6.35, 12.0 -> 11.9 (g128 7.92 -> 6.22), 4096 x 12288 7.98 -> 6.45, 2048 / 5120 / 16384 x
    // 13824 6.98 -> 4.69, 11.67 -> 9.36, 24.8 -> 22.3, 7168 x 18432 15.6 -> 14.3, 3584 x 18944 10.97 -> 8.44 (g128 10.7 -> 8.43);
    // 5120 x 27648 is level (18.6 / 18.8) and stays.
    if (p.bits == 4 && p.K != 4096 && p.K != 8192 && p.K != 14336 && p.K != 28672) return p.K != 27648;
    if (p.bits == 4 && p.K == 4096) return p.N <= 16384;
    if (p.bits == 4 && p.K == 8192) return p.N <= 20480;
    return true;
}

template <int DT, int LOG2G> static const void* rows_long_fn_g(int bits, int ch) {
    if (bits == 4) {
        if (ch == 4) return (const void*)qmv_rows_long_kernel<DT, 4, 4, LOG2G>;
        if constexpr (LOG2G >= 6) {   // (14336 / 28672 codes in groups of 32: 448 / 896 groups per row, 448 of which need 16-byte aligned scales)
            if (ch == 7) return (const void*)qmv_rows_long_kernel<DT, 4, 7, LOG2G>;
            if (ch == 14) return (const void*)qmv_rows_long_kernel<DT, 4, 14, LOG2G>;
        }
        return nullptr;
    }
    if (ch == 2) return (const void*)qmv_rows_long_kernel<DT, 2, 2, LOG2G>;
    if constexpr (LOG2G >= 6) return (const void*)qmv_rows_long_kernel<DT, 2, 4, LOG2G>;       // (16384 codes in groups of 32: 512)
    return nullptr;
}
template <int DT, int LOG2G> static const void* rows_long_more_fn(uint32_t K) {   // groups of 64 / 128
    switch (K) {
        case 10240: return (const void*)qmv_rows_long_kernel<DT, 4, 5, LOG2G>;
        case 12288: return (const void*)qmv_rows_long_kernel<DT, 4, 6, LOG2G>;
        case 18432: return (const void*)qmv_rows_long_kernel<DT, 4, 9, LOG2G>;
        case 11008: return (const void*)qmv_rows_long_ragged_kernel<DT, 6, LOG2G, 24>;
        case 13824: return (const void*)qmv_rows_long_ragged_kernel<DT, 7, LOG2G, 48>;
        case 18944: return (const void*)qmv_rows_long_ragged_kernel<DT, 10, LOG2G, 16>;
        case 27648: return (const void*)qmv_rows_long_ragged_kernel<DT, 14, LOG2G, 32>;
        default: return nullptr;
    }
}
template <int DT> static const void* rows_long_fn(int bits, int ch, uint32_t G) {
    return G == 32 ? rows_long_fn_g<DT, 5>(bits, ch) : G == 64 ? rows_long_fn_g<DT, 6>(bits, ch) : rows_long_fn_g<DT, 7>(bits, ch);
}
template <int DT, int GM> static const void* rows_long_routed_fn(int ch) {   // 4-bit codes in groups of 64
    return ch == 4 ? (const void*)qmv_rows_long_routed_kernel<DT, 4, 4, 6, GM> : ch == 7 ? (const void*)qmv_rows_long_routed_kernel<DT, 4, 7, 6, GM> : nullptr;
}

int launch_qmv_rows(const QmvParams& p, const LaunchCtx& lc) {
    if (!qmv_rows_takes(p)) return fail(ERR_UNSUPPORTED, "qmv rows kernels: one activation row, 2- or 4-bit codes, f16 / bf16, rows of 4096, 8192, 14336, 16384 or 28672 codes or one of the other lengths it is built for");
    const bool routed = p.gather != GATHER_NONE;
    const uint32_t slots = routed && p.gather != GATHER_SINGLE ? (p.T < p.E ? p.T : p.E) : 1u;   // the experts that can have a row
    if (p.bits == 4 && p.group_size == 64 && p.K == 4096)
        return launch_rows(p.dtype, p.w, p.scales, p.biases, p.x, p.out, p.N, 0, nullptr, lc, p.gather, p.route, p.E, p.T, slots);
    const int ch = rows_long_ch(p);
    QmvRowsLArgs a{(const rp_u32x4*)p.w, (const uint16_t*)p.scales, (const uint16_t*)p.biases, (const uint16_t*)p.x, (uint16_t*)p.out, p.N, p.route, p.E, p.T};
    void* args[] = {&a};
    const void* fn = p.gather == GATHER_CSR       ? (p.dtype == DT_BF16 ? rows_long_routed_fn<DT_BF16, GATHER_CSR>(ch) : rows_long_routed_fn<DT_F16, GATHER_CSR>(ch))
                     : p.gather == GATHER_INDICES ? (p.dtype == DT_BF16 ? rows_long_routed_fn<DT_BF16, GATHER_INDICES>(ch) : rows_long_routed_fn<DT_F16, GATHER_INDICES>(ch))
                     : p.gather == GATHER_SINGLE  ? (p.dtype == DT_BF16 ? rows_long_routed_fn<DT_BF16, GATHER_SINGLE>(ch) : rows_long_routed_fn<DT_F16, GATHER_SINGLE>(ch))
                     : p.dtype == DT_BF16         ? rows_long_fn<DT_BF16>(p.bits, ch, p.group_size)
                                                  : rows_long_fn<DT_F16>(p.bits, ch, p.group_size);
    if (p.gather == GATHER_NONE && p.bits == 4 && p.K != 8192 && p.K != 14336 && p.K != 28672)   // the other models' row lengths
        fn = p.dtype == DT_BF16 ? (p.group_size == 64 ? rows_long_more_fn<DT_BF16, 6>(p.K) : p.group_size == 128 ? rows_long_more_fn<DT_BF16, 7>(p.K) : nullptr)
                                : (p.group_size == 64 ? rows_long_more_fn<DT_F16, 6>(p.K) : p.group_size == 128 ? rows_long_more_fn<DT_F16, 7>(p.K) : nullptr);
    if (!fn) return fail(ERR_UNSUPPORTED, "qmv rows kernels: no instance for this row length and group size");
    // Sixteen rows per workgroup, eight for the long rows. One workgroup of sixteen per compute unit (4096 x 14336: 256
    // of them) is the fastest form on some machines of the pool and 9 % behind on others, where the same launch as 512
    // workgroups of eight holds (same run, 1024 / 512 threads: 7.34 / 7.40 us on one machine, 8.19 / 7.48 and 8.60 /
    // 7.70 on two others); shorter rows keep sixteen (8192 x 8192: 4-bit 8.00 / 7.97, 2-bit 6.27 / 6.95).
    // From 8192 rows on (two or more workgroups of sixteen per compute unit) sixteen are ahead again: 8192 x 14336 13.2 ->
    // 12.65 us, 14336 x 14336 21.25 -> 20.35. (28672 codes: 896 chunks to prepare, always sixteen.)
    // Few rows of up to four chunks per lane: workgroups of eight rows up to 2048 rows, so that every compute unit has one
    // (8192 4-bit codes, 1024 / 2048 rows 3.98 -> 3.27, 4.16 -> 3.78 us; 3072 / 4096 rows 4.55 -> 4.87, 5.02 -> 5.22: sixteen again;
    // 2-bit codes, 1024 / 2048 rows of 8192 3.52 -> 3.25, 3.57 -> 3.23, of 16384 5.56 -> 4.27, 5.70 -> 4.62).
    const uint32_t block = ch > 8 || (ch == 7 && p.N >= 8192u) ? 1024u : ch > 4 ? 512u : (p.N <= 2048u ? 512u : 1024u);
    if (block < 64u * (uint32_t)ch) return fail(ERR_UNSUPPORTED, "qmv rows kernels: workgroup smaller than the row's chunks");   // (thread t prepares chunk t)
    hipError_t e = launch_kernel(fn, dim3((p.N + block / 64u - 1u) / (block / 64u), slots), dim3(block), args, 0, lc);
    if (e != hipSuccess) return hip_fail(e, "qmv long rows kernel launch");
    return ERR_OK;
}

int launch_rows_probe(const void* w, const void* s, const void* b, const void* x, void* out, uint32_t N, int mode, uint64_t* stamps,
                      const LaunchCtx& lc) {
    return launch_rows(DT_BF16, w, s, b, x, out, N, mode, stamps, lc);
}

}  // namespace mtq
