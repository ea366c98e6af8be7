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
// in turns of 512 codes; weights are loaded two turns ahead, a row's scales and biases for a turn with one or two
// 16-byte loads per lane.
#include "mtq_device.h"
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

template <int DT, int G, int NB, int SETS> __global__ __launch_bounds__(1024) void qmv_wide_kernel(QmvWArgs a) {
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
    const uint32_t k0 = blockIdx.y * a.kslice, klen = min(a.kslice, a.K - k0);
    const uint32_t turns = klen / 512u, ng = klen / (uint32_t)G;
    qw_u32x4* XL = (qw_u32x4*)lds;                                   // [klen / 8 pieces][16 rows]
    float* XG = (float*)(lds + (size_t)(klen / 8u) * 256u);          // [ng][16 rows]

    // KP waves share a set of NB row blocks, each taking a run of the slice's turns
    const uint32_t kp = wave & (a.kp - 1u), wr = wave >> a.log2kp;
    const uint32_t t0 = min(kp * a.tpk, turns), t1 = min(t0 + a.tpk, turns), cnt = t1 - t0;   // cnt <= 4 * SETS (host)
    const uint32_t rb0 = (blockIdx.x * (NW >> a.log2kp) + wr) * NB;
    uint32_t row[NB], woff[NB];   // woff: byte offset of this lane's weights in turn 0 of the slice
#pragma unroll
    for (int i = 0; i < NB; i++) {   // row blocks past the matrix work on its last row and store nothing
        row[i] = (rb0 + i) * 16u + j;
        woff[i] = min(row[i], a.N - 1u) * (a.K / 2u) + q * 16u;
    }
    const unsigned char* wbase = a.w + k0 / 2u;   // + 256 bytes per turn

    // ---- scales and biases of the wave's whole run, read once ------------------------------------------------------
    // A row's scales are 16 bytes per turn of one 128-byte line; read turn by turn, the line had left the L2 by the
    // next turn and was fetched from memory again (4.8 x the bytes). The four lanes of a weight row take the turns
    // q, q + 4, q + 8 of the run (one 128-byte line per instruction and row); at turn n the lanes fetch the pairs from
    // lane quarter n % 4, register set n / 4, with ds_bpermute.
    uint32_t sreg[NB][SETS][DPT], breg[NB][SETS][DPT];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const size_t e0 = (size_t)min(row[i], a.N - 1u) * a.gpr + k0 / (uint32_t)G;
#pragma unroll
        for (int st = 0; st < SETS; st++) {
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

    // ---- the first turn's weights: in flight while the activations are staged --------------------------------------
    // The weight loads of the stream are issued by hand, in a fixed order, and waited for with "at most N loads
    // outstanding": the compiler would sink the loads to the end of a turn and wait for all of them at its top.
    // The loop below is the only code that touches registers with loads in flight, and every turn issues its loads
    // (those of a wave's last turn, for a turn that does not exist, all read the slice's first bytes): a register
    // allocator that had to join several copies of the turn would move such registers about while their loads fly.
    qw_u32x4 ring[NB][4];
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int d = 0; d < 4; d++) ring[i][d] = qw_u32x4{0u, 0u, 0u, 0u};
    {
        const uint32_t tc = min(t0, turns - 1u);   // a wave without turns loads a valid address and uses nothing
        qw_static_for<0, 4>([&](auto d_c) {
            constexpr int d = decltype(d_c)::value;
#pragma unroll
            for (int i = 0; i < NB; i++) qw_load_once<d * 64>(ring[i][d], woff[i], wbase + tc * 256u);
        });
    }

    // ---- stage the activations: wave w takes groups w, w + 16, ...; a block is 32 codes x 16 rows -----------------
    {
        const uint16_t* xr = a.x + (size_t)min(j, a.M - 1u) * a.K + k0;   // rows past M repeat the last one; their results are not stored
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

    // ---- stream ---------------------------------------------------------------------------------------------------
    const uint32_t kor = magic_or_vgpr<DT>();
    const uint32_t msk = 0x000F000Fu;
    const unsigned char* xl_lane = lds + (q * 16u + j) * 16u;
    const unsigned char* xg_lane = (const unsigned char*)(XG + 4u * q);
    float tot[NB][4];
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) tot[i][r] = 0.f;
    // One turn: 512 codes of every row block of the wave. The registers of two steps are reloaded for the next turn
    // together, behind steps 1 and 3, so that both 64-byte halves of a 128-byte line are asked for at the same time
    // (asked for a quarter turn apart, most lines were fetched from memory twice: the loads are marked as read
    // once). Loads outstanding at the top of a turn: its weights, 4 NB; when step d's are needed, the younger ones
    // are the rest of the turn's and the next turn's issued so far: 3 NB at steps 0 and 2, 2 NB at steps 1 and 3.
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
            qw_wait<(d % 2 ? 2 : 3) * NB>();
            uint32_t v[NB][4];
#pragma unroll
            for (int i = 0; i < NB; i++) {
                qw_tie(ring[i][d]);
                // 4 x 4 transpose of the step's dwords among the lanes j, j + 16, j + 32, j + 48: before, dword u of
                // lane quarter q is codes [32 q + 8 u, +8) of the step; after, codes [32 u + 8 q, +8)
                const qw_u32x4 w4 = ring[i][d];
                const auto a02 = __builtin_amdgcn_permlane32_swap(w4.x, w4.z, false, false);
                const auto a13 = __builtin_amdgcn_permlane32_swap(w4.y, w4.w, false, false);
                const auto b01 = __builtin_amdgcn_permlane16_swap(a02[0], a13[0], false, false);
                const auto b23 = __builtin_amdgcn_permlane16_swap(a02[1], a13[1], false, false);
                v[i][0] = b01[0]; v[i][1] = b01[1]; v[i][2] = b23[0]; v[i][3] = b23[1];
            }
            if constexpr (d % 2 == 1) {
#pragma unroll
                for (int i = 0; i < NB; i++) qw_load_once<(d - 1) * 64>(ring[i][d - 1], has_next ? woff[i] : 0u, wbase + tn * 256u);
#pragma unroll
                for (int i = 0; i < NB; i++) qw_load_once<d * 64>(ring[i][d], has_next ? woff[i] : 0u, wbase + tn * 256u);
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

    // ---- the K parts of a row block meet in LDS (over the staged activations, which are done with) ---------------
    if (a.kp > 1u) {
        __syncthreads();
        float* red = (float*)lds;
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[((wave * NB + i) * 4u + r) * 64u + lane] = tot[i][r];
        __syncthreads();
        if (kp != 0u) return;
        for (uint32_t o = 1; o < a.kp; o++)
#pragma unroll
            for (int i = 0; i < NB; i++)
#pragma unroll
                for (int r = 0; r < 4; r++) tot[i][r] += red[(((wave + o) * NB + i) * 4u + r) * 64u + lane];
    }
    // activation rows 4 q .. 4 q + 3 of weight row `row`
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t m = 4u * q + r;
            if (m < a.M && row[i] < a.N) {
                if (gridDim.y > 1) a.part[((size_t)blockIdx.y * a.M + m) * a.N + row[i]] = tot[i][r];
                else ((uint16_t*)a.out)[(size_t)m * a.N + row[i]] = f32_to_elem_bits<DT>(tot[i][r]);
            }
        }
}

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

// Shapes the kernel takes: f16 / bf16, 4-bit codes, groups of 32 / 64 / 128, at most 16 rows, rows of whole turns.
static bool plan_wide(const QmmParams& p, QmvWPlan& pl) {
    const uint32_t G = p.group_size;
    if ((p.dtype != DT_F16 && p.dtype != DT_BF16) || p.bits != 4 || (G != 32 && G != 64 && G != 128)) return false;
    if (p.M == 0 || p.M > 16 || p.N == 0 || p.K == 0 || p.K % 512) return false;
    if ((uintptr_t)p.w % 16 || (uintptr_t)p.x % 16 || (uintptr_t)p.scales % 16 || (uintptr_t)p.biases % 16) return false;
    if ((uint64_t)p.M * p.N >= (1ull << 31)) return false;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    // 16 rows of activations (32 bytes per code position) and a row of group sums (64 bytes per group) in 160 KB
    const uint32_t per_turn = 512u * 32u + (512u / G) * 64u;
    const uint32_t max_turns = (160u * 1024u) / per_turn;
    const uint32_t turns = p.K / 512u;
    uint32_t ks = (turns + max_turns - 1) / max_turns;
    const uint32_t tps = (turns + ks - 1) / ks;
    ks = (turns + tps - 1) / tps;
    pl.kslice = tps * 512u;
    pl.ksplit = ks;
    pl.lds = (size_t)tps * per_turn;
    // A workgroup's 16 waves take 16 * NB / KP row blocks: two per wave once that still gives every compute unit a
    // workgroup, else one, and on shorter matrices KP waves share a row block, each with a run of the turns.
    const uint32_t nrb = (p.N + 15u) / 16u;
    const uint32_t want = (uint32_t)cus / ks > 0 ? (uint32_t)cus / ks : 1u;   // workgroups per K slice
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
    if (pl.kp > 1u && pl.lds < (size_t)16 * pl.nb * 1024) pl.lds = (size_t)16 * pl.nb * 1024;   // the K parts' sums, a KB per wave and row block
    const uint32_t per_wg = 16u * pl.nb / pl.kp;
    pl.grid_x = (nrb + per_wg - 1) / per_wg;
    return true;
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
    const void* fn = nullptr;
#define QW_PICK3(DTv, Gv, NBv) (pl.sets == 1 ? (const void*)qmv_wide_kernel<DTv, Gv, NBv, 1> : pl.sets == 2 ? (const void*)qmv_wide_kernel<DTv, Gv, NBv, 2> : NBv == 1 ? (const void*)qmv_wide_kernel<DTv, Gv, 1, 3> : nullptr)
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

}  // namespace mtq
