// The 16-row matrix-core GEMV (see qmv_wide.hip for the routing and the geometry): kernel and argument block, shared
// by the translation units that instantiate it.
#pragma once
// Matrix-core GEMV for 5..16 activation rows on the 16x16x32 MFMA: 4-bit codes, f16 / bf16, long weight matrices.
// Replaces, for those batches, the reference's multi-row GEMV forms mt_qmm / mt_qmm_mma at small M
// (crates/metaltile-std/src/mlx/quantized.rs:1330-1500, 2106-2405; routed by mt_qmm_for, quantized.rs:5040-5065)
// with exact-dequant arithmetic: out[m][n] = sum_g (s[n][g] * sum_k q[n][k] x[m][k] + b[n][g] * sum_k x[m][k]).
//
// Why another GEMV: the 4x4x4 MFMA of qmv_mfma_kernel issues every 16 clk and covers 4 activation rows x 256 codes,
// so two row sets (5..8 rows) are bound by the matrix pipe at about 3.2 TB/s, and the 32-row tile kernel streams
// long matrices no faster. One 16x16x32 MFMA covers 16 rows x 16 weight rows x 32 codes in the same 16 clk.
//
// Layout of the work. A wave owns row blocks of 16 weight rows; lane (j, q) = (lane % 16, lane / 16) loads, per
// step of 128 codes, the 16 bytes (32 codes) at code 32 q of weight row j: a wave-wide load is 16 rows x 64 bytes.
// An MFMA has to stay inside one group of codes (one scale), so the step's dwords are transposed among the four
// lanes of a weight row (two v_permlane32_swap and two v_permlane16_swap per step): dword u of lane (j, q) is then
// codes [32 u + 8 q, +8) of the step, MFMA u multiplies the 32 consecutive codes [32 u, +32), and the activations
// are staged in LDS in that order (16-byte pieces [step][u][q][row], elements inside a piece in the order the nibble
// masks deliver the codes), so the A operand of lane (j, q) is one conflict-free ds_read_b128. A pair of codes becomes a pair of elements with
// one v_and_or_b32 (MAGIC | code: 128 + q in bf16, 1024 + q in f16); the MAGIC share is taken out with the group
// sums of the activations, as in qmv_mfma_kernel. The accumulator of lane (j, q) holds activation rows 4 q .. 4 q + 3
// of weight row j: the lane's own scale applies, and no cross-lane reduction is needed.
// The K range of a workgroup (the whole row, or a slice of it when 16 rows of K activations do not fit LDS: then
// blockIdx.y picks the slice and f32 partial rows go to a scratch buffer that a second kernel adds up) is walked
// in turns of 512 codes; weights are loaded a turn ahead, the scales and biases of a wave's whole run once.
#include "mtq_device.h"
#include "vm_schedule.h"
#include "mtq_internal.h"

#include <type_traits>

namespace mtq {

struct QmvWArgs {
    const unsigned char* w;
    const uint16_t* scales;
    const uint16_t* biases;
    const uint16_t* x;
    void* out;
    float* part;          // [ksplit][M][N] when gridDim.y > 1
    uint32_t M, N, K, gpr;
    uint32_t kslice;      // codes per K slice (blockIdx.y), a multiple of 512
    uint32_t kp, log2kp;  // waves that share a wave's row blocks, each with a run of the slice's turns (a power of two)
    uint32_t tpk;         // turns per such wave
    const uint32_t* route;   // gathers: CSR offsets [E + 1] or one expert id per row [T]; blockIdx.y is the expert
    uint32_t T, E;           // w / scales / biases then hold E matrices, x and out T rows
};

typedef uint32_t qw_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t qw_u32x2 __attribute__((ext_vector_type(2)));
typedef float qw_f32x4 __attribute__((ext_vector_type(4)));

template <int DT> __device__ __forceinline__ qw_f32x4 mfma16(qw_u32x4 a, qw_u32x4 b, qw_f32x4 c) {
    if constexpr (DT == DT_BF16) {
        typedef __attribute__((ext_vector_type(8))) __bf16 v8;
        v8 av, bv;
        __builtin_memcpy(&av, &a, 16);
        __builtin_memcpy(&bv, &b, 16);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, c, 0, 0, 0);
    } else {
        typedef __attribute__((ext_vector_type(8))) _Float16 v8;
        v8 av, bv;
        __builtin_memcpy(&av, &a, 16);
        __builtin_memcpy(&bv, &b, 16);
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, c, 0, 0, 0);
    }
}

// f(integral_constant<int, I>) for I = B .. E-1: loop indices that are constant expressions in the body.
template <int B, int E, class F> __device__ __forceinline__ void qw_static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        qw_static_for<B + 1, E>(f);
    }
}
// 16 (or 8) bytes per lane from sbase + voff + OFF into registers. The result is valid only after a qw_wait that
// covers it and a qw_tie behind that wait; until then the registers must not be read or copied. The destination is
// declared as read and written, so that the new value lives in the registers of the old one: a loop that carries
// such registers from one iteration to the next then needs no copies of registers whose loads are still in flight.
template <int OFF> __device__ __forceinline__ void qw_load(qw_u32x4& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}
// The same for data read once (the weights): the line is the first to leave the caches.
template <int OFF> __device__ __forceinline__ void qw_load_once(qw_u32x4& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void qw_load(qw_u32x2& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}
// Waits until at most N vector memory loads of this wave are outstanding (they complete in order).
// The stream loop's vector-memory schedule and the one wait count that follows from it. A turn's weights are two
// lines (steps 0-1 and 2-3) of 2 NB loads each; the prologue issues both lines of the first turn; turn n waits for its
// line 0, issues line 0 of turn n + 1 behind step 1, waits for its line 1 and issues line 1 of turn n + 1 behind step 3.
// Whenever a line is needed the loads younger than it are exactly the other line's: 2 NB. holds() replays that order.
template <int NB> struct QmvWideWaits {
    static constexpr int line = 2 * NB;
    static constexpr bool holds() {
        VmQueue q;
        q.issue(vm_tag(0, 0), 2 * NB);
        q.issue(vm_tag(1, 0), 2 * NB);
        for (int n = 0; n < 12; n++)
            for (int p = 0; p < 2; p++) {
                if (q.younger_than(vm_tag(p, n)) != line) return false;   // neither too early nor later than need be
                q.wait(line);
                if (!q.landed(vm_tag(p, n))) return false;
                q.issue(vm_tag(p, n + 1), 2 * NB);
            }
        return true;
    }
};
template <int N> __device__ __forceinline__ void qw_wait() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Placed behind a wait: no read of r is scheduled above it.
template <class T> __device__ __forceinline__ void qw_tie(T& r) { asm volatile("" : "+v"(r)::"memory"); }

// element `odd` of a dword of two packed elements
template <int DT> __device__ __forceinline__ float qw_elem(uint32_t dw, int odd) {
    if constexpr (DT == DT_BF16) return __uint_as_float(odd ? (dw & 0xFFFF0000u) : (dw << 16));
    else return f16_bits_to_f32(odd ? (dw >> 16) : (dw & 0xFFFFu));
}

// MODE: GATHER_NONE (rows 0 .. M - 1 against one matrix), or GATHER_CSR / GATHER_INDICES: blockIdx.y is an expert,
// its rows (the reference's CSR rule, crates/metaltile-std/src/ffai/moe.rs:376-385, or the rows whose id names it) are
// worked 16 at a time, each pass staging its rows and streaming the workgroup's share of the expert's weights.
template <int DT, int G, int NB, int SETS, int MODE = GATHER_NONE> __global__ __launch_bounds__(1024) void qmv_wide_kernel(QmvWArgs a) {
    static_assert(G == 32 || G == 64 || G == 128, "group size");
    static_assert(NB == 1 || NB == 2, "row blocks per wave");
    static_assert(SETS >= 1 && SETS <= 3, "a wave works on at most 4 * SETS turns");
    constexpr int NW = 16;
    constexpr int GPT = 512 / G;       // groups per turn
    constexpr int DPT = GPT / 2;       // dwords of packed scales (and of biases) per turn and weight row
    constexpr int UPG = G / 32;        // MFMAs per group
    constexpr int MAXG = G == 32 ? 9 : G == 64 ? 5 : 3;   // groups a wave stages at most: a slice is at most 4608 codes
    constexpr float MAGIC = DT == DT_BF16 ? 128.0f : 1024.0f;
    extern __shared__ __align__(16) unsigned char lds[];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t j = lane & 15u, q = lane >> 4;
    constexpr bool GATHER = MODE != GATHER_NONE;
    const uint32_t k0 = GATHER ? 0u : blockIdx.y * a.kslice, klen = min(a.kslice, a.K - k0);
    const uint32_t turns = klen / 512u, ng = klen / (uint32_t)G;
    qw_u32x4* XL = (qw_u32x4*)lds;                                   // [klen / 8 pieces][16 rows]
    float* XG = (float*)(lds + (size_t)(klen / 8u) * 256u);          // [ng][16 rows]
    // GATHER_INDICES: the expert's rows, [T], behind everything that is written while they are needed
    const uint32_t x_end = (klen / 8u) * 256u + ng * 64u, red_end = a.kp > 1u ? (uint32_t)(NW * NB) * 1024u : 0u;
    uint32_t* rowlist = (uint32_t*)(lds + (x_end > red_end ? x_end : red_end));
    __shared__ uint32_t s_cnt;

    // ---- routing: which activation rows does this workgroup serve? ------------------------------------------------
    uint32_t expert = 0, nrows = a.M, lo = 0, n1 = a.M, lo2 = 0;
    if constexpr (MODE == GATHER_CSR) {
        expert = blockIdx.y;
        if (a.E <= 64u) {
            uint32_t same;
            nrows = csr_route64(a.route, a.E, a.T, expert, false, lane, same, lo, n1, lo2);   // (one read of the offsets)
        } else {
            nrows = csr_expert_rows(a.route, a.E, a.T, expert, lane, lo, n1, lo2);
        }
        // (the same in every lane: kept in scalar registers, the vector ones are all spoken for)
        nrows = __builtin_amdgcn_readfirstlane(nrows);
        lo = __builtin_amdgcn_readfirstlane(lo);
        n1 = __builtin_amdgcn_readfirstlane(n1);
        lo2 = __builtin_amdgcn_readfirstlane(lo2);
        if (nrows == 0) return;
    } else if constexpr (MODE == GATHER_INDICES) {
        expert = blockIdx.y;
        if (tid < 64) {
            uint32_t n = 0;
            for (uint32_t tb = 0; tb < a.T; tb += 64) {
                const uint32_t t = tb + lane;
                const bool hit = t < a.T && a.route[t] == expert;
                const unsigned long long m = __ballot(hit);
                if (hit) rowlist[n + __popcll(m & ((1ull << lane) - 1ull))] = t;
                n += (uint32_t)__popcll(m);
            }
            if (lane == 0) s_cnt = n;
        }
        __syncthreads();
        nrows = __builtin_amdgcn_readfirstlane(s_cnt);
        if (nrows == 0) return;
    }
    auto batch_row = [&](uint32_t jj) -> uint32_t {   // jj < nrows
        if constexpr (MODE == GATHER_CSR) return jj < n1 ? lo + jj : lo2 + (jj - n1);
        else if constexpr (MODE == GATHER_INDICES) return rowlist[jj];
        else return jj;
    };
    if constexpr (GATHER) {
        a.w += (size_t)expert * a.N * (a.K / 2u);
        a.scales += (size_t)expert * a.N * a.gpr;
        a.biases += (size_t)expert * a.N * a.gpr;
    }

    // KP waves share a set of NB row blocks, each taking a run of the slice's turns
    const uint32_t kp = wave & (a.kp - 1u), wr = wave >> a.log2kp;
    const uint32_t t0 = min(kp * a.tpk, turns), t1 = min(t0 + a.tpk, turns), cnt = t1 - t0;   // cnt <= 4 * SETS (host)
    const uint32_t rb0 = (blockIdx.x * (NW >> a.log2kp) + wr) * NB;
    const uint32_t n_pass = GATHER ? (nrows + 15u) / 16u : 1u;
    // A weight load covers whole 128-byte lines: eight lanes share a row's line, so one instruction takes the line of
    // rows 0 .. 7 of the block (woff[i][0]) and a second that of rows 8 .. 15 (woff[i][1]); lane (j, q) holds piece
    // q + 4 (j / 8) of row j % 8 (or 8 + j % 8). (Four lanes to a row, 64 bytes of 16 lines per instruction, the same
    // bytes streamed at 5.2 - 5.5 TB/s in a read-only kernel of this shape; whole lines at 6.3 - 6.5.)
    uint32_t row[NB], woff[NB][2];   // woff: byte offsets of this lane's two loads in turn 0 of the slice
#pragma unroll
    for (int i = 0; i < NB; i++) {   // row blocks past the matrix work on its last row and store nothing
        row[i] = (rb0 + i) * 16u + j;
#pragma unroll
        for (int h = 0; h < 2; h++)
            woff[i][h] = min((rb0 + i) * 16u + 8u * h + (j & 7u), a.N - 1u) * (a.K / 2u) + (q + 4u * (j >> 3)) * 16u;
    }
    const unsigned char* wbase = a.w + k0 / 2u;   // + 256 bytes per turn

    // ---- scales and biases of the wave's whole run, read once ------------------------------------------------------
    // A row's scales are 16 bytes per turn of one 128-byte line; read turn by turn, the line had left the L2 by the
    // next turn and was fetched from memory again (4.8 x the bytes). The four lanes of a weight row take the turns
    // q, q + 4, q + 8 of the run (one 128-byte line per instruction and row); at turn n the lanes fetch the pairs from
    // lane quarter n % 4, register set n / 4, with ds_bpermute.
    // With 16 bytes per turn (groups of 64 codes) and two sets, the first two are read as the weights are: eight lanes
    // to a row, pieces q + 4 (j / 8) of rows j % 8 and 8 + j % 8, whole lines per instruction; the half rows change
    // places behind the barrier below.
    constexpr bool PAIRED = DPT == 4 && SETS >= 2;
    uint32_t sreg[NB][SETS][DPT], breg[NB][SETS][DPT];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        [[maybe_unused]] const size_t e0 = (size_t)min(row[i], a.N - 1u) * a.gpr + k0 / (uint32_t)G;
        if constexpr (PAIRED) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const size_t eh = (size_t)min((rb0 + i) * 16u + 8u * h + (j & 7u), a.N - 1u) * a.gpr + k0 / (uint32_t)G;
                const uint32_t n = min(q + 4u * (j >> 3), cnt ? cnt - 1u : 0u);
                const size_t e = eh + (size_t)min(t0 + n, turns - 1u) * GPT;
                const qw_u32x4 sv = *(const qw_u32x4*)(a.scales + e), bv = *(const qw_u32x4*)(a.biases + e);
                sreg[i][h][0] = sv.x; sreg[i][h][1] = sv.y; sreg[i][h][2] = sv.z; sreg[i][h][3] = sv.w;
                breg[i][h][0] = bv.x; breg[i][h][1] = bv.y; breg[i][h][2] = bv.z; breg[i][h][3] = bv.w;
            }
        }
#pragma unroll
        for (int st = PAIRED ? 2 : 0; st < SETS; st++) {
            const uint32_t n = min(4u * st + q, cnt ? cnt - 1u : 0u);   // a turn past the run: any valid address, never used
            const size_t e = e0 + (size_t)min(t0 + n, turns - 1u) * GPT;
            if constexpr (DPT == 2) {
                const qw_u32x2 sv = *(const qw_u32x2*)(a.scales + e), bv = *(const qw_u32x2*)(a.biases + e);
                sreg[i][st][0] = sv.x; sreg[i][st][1] = sv.y; breg[i][st][0] = bv.x; breg[i][st][1] = bv.y;
            } else {
#pragma unroll
                for (int h = 0; h < DPT / 4; h++) {
                    const qw_u32x4 sv = *(const qw_u32x4*)(a.scales + e + 8 * h), bv = *(const qw_u32x4*)(a.biases + e + 8 * h);
                    sreg[i][st][4 * h] = sv.x; sreg[i][st][4 * h + 1] = sv.y; sreg[i][st][4 * h + 2] = sv.z; sreg[i][st][4 * h + 3] = sv.w;
                    breg[i][st][4 * h] = bv.x; breg[i][st][4 * h + 1] = bv.y; breg[i][st][4 * h + 2] = bv.z; breg[i][st][4 * h + 3] = bv.w;
                }
            }
        }
    }

    static_assert(QmvWideWaits<NB>::holds(), "the hand-counted vmcnt wait does not match the order in which the stream loop issues its loads");
    qw_u32x4 ring[NB][4];
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int d = 0; d < 4; d++) ring[i][d] = qw_u32x4{0u, 0u, 0u, 0u};
    for (uint32_t pass = 0; pass < n_pass; pass++) {
    const uint32_t row_base = pass * 16u, live = min(16u, nrows - row_base);   // activation rows of this pass
    // (With several passes, addresses that do not change from pass to pass - of the staged operands, of the K parts'
    // sums, of the final stores - are worked out ahead of the pass loop and live across every stream in registers there
    // are none left for: each wave spills them. They are worked out from the lane's coordinates plus a zero that the
    // optimiser cannot tell from a value that changes with the pass.)
    const uint32_t pz = GATHER ? pass & (a.log2kp >> 16) : 0u;
    // ---- the first turn's weights: in flight while the activations are staged --------------------------------------
    // The weight loads of the stream are issued by hand, in a fixed order, and waited for with "at most N loads
    // outstanding": the compiler would sink the loads to the end of a turn and wait for all of them at its top.
    // The loop below is the only code that touches registers with loads in flight, and every turn issues its loads
    // (those of a wave's last turn, for a turn that does not exist, all read the slice's first bytes): a register
    // allocator that had to join several copies of the turn would move such registers about while their loads fly.
    {
        const uint32_t tc = min(t0, turns - 1u);   // a wave without turns loads a valid address and uses nothing
        qw_static_for<0, 4>([&](auto d_c) {
            constexpr int d = decltype(d_c)::value;
#pragma unroll
            for (int i = 0; i < NB; i++) qw_load_once<(d / 2) * 128>(ring[i][d], woff[i][d % 2], wbase + tc * 256u);
        });
    }

    // ---- stage the activations: wave w takes groups w, w + 16, ...; a block is 32 codes x 16 rows -----------------
    {
        const uint16_t* xr = a.x + (size_t)batch_row(row_base + min(j, live - 1u)) * a.K + k0;   // rows past the last repeat it; their results are not stored
        qw_u32x4 xs[MAXG * UPG];
#pragma unroll
        for (int gi = 0; gi < MAXG; gi++) {
            const uint32_t g = min(wave + gi * NW, ng - 1u);
#pragma unroll
            for (int b = 0; b < UPG; b++) xs[gi * UPG + b] = *(const qw_u32x4*)(xr + (g * UPG + b) * 32u + q * 8u);
        }
#pragma unroll
        for (int gi = 0; gi < MAXG; gi++) {
            const uint32_t g = wave + gi * NW;
            if (g < ng) {
                float sum = 0.f;
#pragma unroll
                for (int b = 0; b < UPG; b++) {
                    const uint32_t blk = g * UPG + b;   // codes [32 blk, +32) of the slice = one MFMA; this lane stages its k part q
                    const qw_u32x4 v = xs[gi * UPG + b];
                    sum += qw_elem<DT>(v.x, 0) + qw_elem<DT>(v.x, 1) + qw_elem<DT>(v.y, 0) + qw_elem<DT>(v.y, 1) + qw_elem<DT>(v.z, 0) +
                           qw_elem<DT>(v.z, 1) + qw_elem<DT>(v.w, 0) + qw_elem<DT>(v.w, 1);
                    // the masks deliver codes (0, 4), (1, 5), (2, 6), (3, 7) of a dword as element pairs
                    qw_u32x4 o;
                    o.x = (v.x & 0xFFFFu) | (v.z << 16);
                    o.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
                    o.z = (v.y & 0xFFFFu) | (v.w << 16);
                    o.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
                    XL[(blk * 4u + q) * 16u + j] = o;
                }
                sum += __shfl_xor(sum, 16, 64);
                sum += __shfl_xor(sum, 32, 64);
                if (q == 0) XG[g * 16u + j] = sum;
            }
        }
        // (loads whose group does not exist are waited for here too: left pending, the compiler waits for them where
        // it next uses their registers, inside the loop, and with them for the loop's own loads)
#pragma unroll
        for (int k = 0; k < MAXG * UPG; k++) qw_tie(xs[k]);
    }
    __syncthreads();
    // (the compiler's own wait for the scales and biases belongs here, not inside the loop, where it would wait for
    // the loop's loads as well)
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int st = 0; st < SETS; st++)
#pragma unroll
            for (int k = 0; k < DPT; k++) { qw_tie(sreg[i][st][k]); qw_tie(breg[i][st][k]); }
    if (PAIRED && pass == 0u) {
        // set 0 = turn q, set 1 = turn 4 + q of row j: lanes j >= 8 take set 0 from the second load of lane j - 8,
        // lanes j < 8 take set 1 from the first load of lane j + 8
        constexpr int ROR8 = 0x128;
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int k = 0; k < DPT; k++) {
                const uint32_t s0 = sreg[i][0][k], s1 = sreg[i][1][k], b0 = breg[i][0][k], b1 = breg[i][1][k];
                sreg[i][0][k] = (uint32_t)__builtin_amdgcn_update_dpp((int)s0, (int)s1, ROR8, 0xF, 0xC, false);
                sreg[i][1][k] = (uint32_t)__builtin_amdgcn_update_dpp((int)s1, (int)s0, ROR8, 0xF, 0x3, false);
                breg[i][0][k] = (uint32_t)__builtin_amdgcn_update_dpp((int)b0, (int)b1, ROR8, 0xF, 0xC, false);
                breg[i][1][k] = (uint32_t)__builtin_amdgcn_update_dpp((int)b1, (int)b0, ROR8, 0xF, 0x3, false);
            }
    }

    // ---- stream ---------------------------------------------------------------------------------------------------
    const uint32_t kor = magic_or_vgpr<DT>();
    const uint32_t msk = 0x000F000Fu;
    const unsigned char* xl_lane = lds + (q * 16u + j + pz) * 16u;
    const unsigned char* xg_lane = (const unsigned char*)(XG + 4u * (q + pz));
    float tot[NB][4];
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) tot[i][r] = 0.f;
    // One turn: 512 codes of every row block of the wave, in four steps of 128. ring[i][2 p] and ring[i][2 p + 1] hold
    // line p of the turn (steps 2 p and 2 p + 1) for rows 0 .. 7 and 8 .. 15 of block i; both are reloaded for the next
    // turn behind step 2 p + 1. Loads outstanding at the top of a turn: its weights, 4 NB; when line p is needed, the
    // younger ones are the other line's, of this turn (p = 0) or the next (p = 1): 2 NB.
    for (uint32_t n = 0; n < cnt; n++) {
        const uint32_t t = t0 + n;
        const bool has_next = n + 1u < cnt;
        const uint32_t tn = has_next ? t + 1u : t;
        const unsigned char* xl_t = xl_lane + t * 16384u;
        const unsigned char* xg_t = xg_lane + t * (uint32_t)(GPT * 64);
        const int src_lane4 = (int)((j + 16u * (n & 3u)) * 4u);   // the lane that holds this turn's scales and biases of row j
        uint32_t m4 = (n & 4u) ? ~0u : 0u, m8 = (n & 8u) ? ~0u : 0u;   // register set n / 4: all-ones masks for sets 1 and 2
        asm volatile("" : "+s"(m4), "+s"(m8));
        qw_f32x4 acc[NB];
        qw_static_for<0, 4>([&](auto d_c) {
            constexpr int d = decltype(d_c)::value;
            if constexpr (d % 2 == 0) {
                qw_wait<QmvWideWaits<NB>::line>();
#pragma unroll
                for (int i = 0; i < NB; i++) { qw_tie(ring[i][d]); qw_tie(ring[i][d + 1]); }
            }
            uint32_t v[NB][4];
#pragma unroll
            for (int i = 0; i < NB; i++) {
                // The step's 64 bytes of row j: lanes j < 8 hold the line's first half of their own row in the first
                // register and the first half of row j + 8 in the second; lanes j >= 8 hold the second half of row
                // j - 8 and of their own. Each half row changes places with the lane 8 further on (a rotation by 8
                // within the 16 lanes, written to half of them).
                qw_u32x4 w4;
                {
                    const qw_u32x4 ra = ring[i][d & ~1], rb = ring[i][d | 1];
                    constexpr int ROR8 = 0x128;
                    if constexpr (d % 2 == 0) {   // first half: lanes j >= 8 take it from the second register of lane j - 8
                        w4.x = (uint32_t)__builtin_amdgcn_update_dpp((int)ra.x, (int)rb.x, ROR8, 0xF, 0xC, false);
                        w4.y = (uint32_t)__builtin_amdgcn_update_dpp((int)ra.y, (int)rb.y, ROR8, 0xF, 0xC, false);
                        w4.z = (uint32_t)__builtin_amdgcn_update_dpp((int)ra.z, (int)rb.z, ROR8, 0xF, 0xC, false);
                        w4.w = (uint32_t)__builtin_amdgcn_update_dpp((int)ra.w, (int)rb.w, ROR8, 0xF, 0xC, false);
                    } else {                      // second half: lanes j < 8 take it from the first register of lane j + 8
                        w4.x = (uint32_t)__builtin_amdgcn_update_dpp((int)rb.x, (int)ra.x, ROR8, 0xF, 0x3, false);
                        w4.y = (uint32_t)__builtin_amdgcn_update_dpp((int)rb.y, (int)ra.y, ROR8, 0xF, 0x3, false);
                        w4.z = (uint32_t)__builtin_amdgcn_update_dpp((int)rb.z, (int)ra.z, ROR8, 0xF, 0x3, false);
                        w4.w = (uint32_t)__builtin_amdgcn_update_dpp((int)rb.w, (int)ra.w, ROR8, 0xF, 0x3, false);
                    }
                }
                // 4 x 4 transpose of the step's dwords among the lanes j, j + 16, j + 32, j + 48: before, dword u of
                // lane quarter q is codes [32 q + 8 u, +8) of the step; after, codes [32 u + 8 q, +8)
                const auto a02 = __builtin_amdgcn_permlane32_swap(w4.x, w4.z, false, false);
                const auto a13 = __builtin_amdgcn_permlane32_swap(w4.y, w4.w, false, false);
                const auto b01 = __builtin_amdgcn_permlane16_swap(a02[0], a13[0], false, false);
                const auto b23 = __builtin_amdgcn_permlane16_swap(a02[1], a13[1], false, false);
                v[i][0] = b01[0]; v[i][1] = b01[1]; v[i][2] = b23[0]; v[i][3] = b23[1];
            }
            if constexpr (d % 2 == 1) {
#pragma unroll
                for (int i = 0; i < NB; i++) {
                    qw_load_once<(d / 2) * 128>(ring[i][d - 1], has_next ? woff[i][0] : 0u, wbase + tn * 256u);
                    qw_load_once<(d / 2) * 128>(ring[i][d], has_next ? woff[i][1] : 0u, wbase + tn * 256u);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const qw_u32x4 aop = *(const qw_u32x4*)(xl_t + (d * 4 + u) * 1024);
                const qw_f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < NB; i++) {
                    const uint32_t dw = v[i][u];
                    const qw_u32x4 bop = {(dw & msk) | kor, ((dw >> 4) & msk) | kor, ((dw >> 8) & msk) | kor, ((dw >> 12) & msk) | kor};
                    acc[i] = mfma16<DT>(aop, bop, (d * 4 + u) % UPG == 0 ? zero : acc[i]);
                }
                if ((d * 4 + u) % UPG == UPG - 1) {   // a group is complete
                    const int gi = (d * 4 + u) / UPG;
                    const qw_f32x4 xg = *(const qw_f32x4*)(xg_t + gi * 64);
#pragma unroll
                    for (int i = 0; i < NB; i++) {
                        // (bitwise selection under masks the optimiser cannot see through: a conditional selection
                        // between array elements becomes an indexed read, and the arrays then live in scratch memory)
                        uint32_t sp = sreg[i][0][gi / 2], bp = breg[i][0][gi / 2];
                        if constexpr (SETS > 1) {
                            sp = (sp & ~m4) | (sreg[i][1][gi / 2] & m4);
                            bp = (bp & ~m4) | (breg[i][1][gi / 2] & m4);
                        }
                        if constexpr (SETS > 2) {
                            sp = (sp & ~m8) | (sreg[i][2][gi / 2] & m8);
                            bp = (bp & ~m8) | (breg[i][2][gi / 2] & m8);
                        }
                        // (an odd group's pair was fetched for the even group before it; the compiler keeps it)
                        const uint32_t spl = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane4, (int)sp);
                        const uint32_t bpl = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane4, (int)bp);
                        const float sv = qw_elem<DT>(spl, gi % 2), bv = qw_elem<DT>(bpl, gi % 2);
                        const float bm = fmaf(-MAGIC, sv, bv);
#pragma unroll
                        for (int r = 0; r < 4; r++) tot[i][r] = fmaf(bm, xg[r], fmaf(sv, acc[i][r], tot[i][r]));
                    }
                }
            }
        });
    }
    qw_wait<0>();   // the last turn's loads, or those of a wave without turns
    // (Nothing reads what those loads bring, so to the compiler their registers are free from the loop's end on, and it
    // may put other values there ahead of the wait, for the loads to overwrite when they land. Naming the registers
    // behind the wait keeps them taken until then.)
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int d = 0; d < 4; d++) qw_tie(ring[i][d]);

    // ---- the K parts of a row block meet in LDS (over the staged activations, which are done with) ---------------
    if (a.kp > 1u) {
        __syncthreads();
        float* red = (float*)lds;
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[((wave * NB + i) * 4u + r) * 64u + lane + pz] = tot[i][r];
        __syncthreads();
        if (kp == 0u)
        for (uint32_t o = 1; o < a.kp; o++)
#pragma unroll
            for (int i = 0; i < NB; i++)
#pragma unroll
                for (int r = 0; r < 4; r++) tot[i][r] += red[(((wave + o) * NB + i) * 4u + r) * 64u + lane + pz];
    }
    // activation rows 4 q .. 4 q + 3 of the pass, weight row `row`
    if (kp == 0u) {
        const uint32_t jp = j + pz, qp = q + pz;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t m = 4u * qp + r;
            if (m >= live) continue;
            const uint32_t orow = batch_row(row_base + m);
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const uint32_t wrow = (rb0 + i) * 16u + jp;   // (worked out again: one register fewer across the stream)
                if (wrow >= a.N) continue;
                if (!GATHER && gridDim.y > 1) a.part[((size_t)blockIdx.y * a.M + orow) * a.N + wrow] = tot[i][r];
                else ((uint16_t*)a.out)[(size_t)orow * a.N + wrow] = f32_to_elem_bits<DT>(tot[i][r]);
            }
        }
    }
    if (pass + 1u < n_pass) {
        qw_wait<0>();        // the stores are done before the next pass counts its loads
        __syncthreads();     // every wave is done with the staged rows
    }
    }   // pass
}

}  // namespace mtq
