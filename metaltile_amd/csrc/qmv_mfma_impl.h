// Streaming qmv / small-batch qmm / gather_qmv kernel for f16 and bf16
// activations on gfx950 that does its dot products on the matrix cores.
// Included by qmv_mfma_f16.hip and qmv_mfma_bf16.hip (one element dtype each).
//
// Replaces the same reference kernels as the dot2 family in qmv_impl.h
// (mt_qmv, mt_qmm, mt_qmm_bm{2,4}: crates/metaltile-std/src/mlx/quantized.rs:8-308,
// 343-621, 650, 1072; mt_moe_gather_qmm_int4{,_m8,_m16,_m32} and the per-row
// ABI: crates/metaltile-std/src/ffai/moe.rs:358-433, 634, 900, 1363, 2256-2550;
// dequant_gemv_int4_expert_indexed:
// crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:58-105) for shapes
// whose rows are a whole number of 256-byte segments.
//
// Geometry. v_mfma_f32_4x4x4_16b_{f16,bf16} is sixteen independent 4x4x4
// products: in block b (lanes 4b..4b+3), lane 4b+j supplies column j of B, lane
// 4b+i supplies row i of A, and lane 4b+j receives D[0..3][j]. Here B's column j
// is four codes of weight row r0+j, A's row i is the matching four activations
// of activation row i, so lane (j, b) accumulates, for ITS OWN 16 bytes of
// weights, the partial dot products with up to four activation rows at once.
// One wave-wide 128-bit load therefore covers 4 weight rows x 256 contiguous
// bytes (lane = 4*q + r: row r, 16-byte chunk q of the segment), which streams
// from HBM at the rate of a plain linear read.
//
// Codes never leave integer form: a masked pair of codes OR-ed into the mantissa
// of 2^7 (bf16) or 2^10 (f16) IS the pair (MAGIC+q_a, MAGIC+q_b) in element
// format and goes straight into the B operand. A chunk lies inside one
// quantisation group, so after the chunk's MFMAs
//     out += s * (D - MAGIC*sum_x) + b * sum_x = s*D + (b - MAGIC*s) * sum_x
// with sum_x the sum of the chunk's activations (precomputed once per
// workgroup). Activations live in LDS, permuted once into MFMA operand order,
// together with the per-chunk sums and the (s, b - MAGIC*s) pairs of the
// workgroup's rows.
//
// A wave walks along K for a block of four weight rows (optionally a 1/KP part
// of K), keeping D weight loads in flight in a register ring, then reduces its
// lanes' totals once per row block. Gather modes add blockIdx.y = expert and run
// the expert's activation rows R = MP*S at a time.
#pragma once
#include "mtq_device.h"
#include "mtq_internal.h"

#include <type_traits>

namespace mtq {

// Keeps memory operations from being moved across this point by the optimiser
// and by the machine scheduler; emits no instruction.
#define MTQ_MFMA_KEEP_ORDER()               \
    do {                                    \
        asm volatile("" ::: "memory");      \
        __builtin_amdgcn_sched_barrier(0);  \
    } while (0)

typedef uint32_t m_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t m_u32x2 __attribute__((ext_vector_type(2)));
typedef short m_s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 m_f16x4 __attribute__((ext_vector_type(4)));
typedef float m_f32x4 __attribute__((ext_vector_type(4)));

struct QmvMArgs {
    const unsigned char* w;
    const void* scales;
    const void* biases;
    const void* x;
    void* out;
    const uint32_t* route;
    uint32_t M, N, K, T, E;
    uint32_t RB;        // bytes per packed weight row
    uint32_t nch;       // lane chunks per row (K / CPC)
    uint32_t nchp;      // nch rounded up to whole wave-wide steps of 16 chunks
    uint32_t nseg;      // wave-wide steps per row (nchp / 16); the last one may be partial
    uint32_t spp;       // steps per K part (the last part may be shorter)
    uint32_t KP;        // K parts (waves sharing a row block)
    uint32_t RBW;       // row blocks walked in parallel by one workgroup
    uint32_t nrb;       // row blocks per wave, one after the other
    uint32_t gpr, log2g;
    uint32_t gpw;       // (scale, bias) pairs per row that a wave keeps in LDS: the groups of its K part, whole 4-vectors, <= 64
    uint32_t list_cap;  // capacity of the row list (indices mode)
    uint32_t by_slot;   // gathers: blockIdx.y counts the experts that have rows (fewer rows than experts), not all experts
    const void* norm_w;     // GATHER_NORM: the norm's weights [K] and its epsilon
    const float* norm_eps;
};

struct QmvMGeom {
    int mp, s;          // activation rows per MFMA set (1, 2, 4) and sets
    uint32_t tpb;
    size_t shmem;
    dim3 grid;
};

template <int DT> __device__ __forceinline__ m_f32x4 mfma4(m_u32x2 a, m_u32x2 b, m_f32x4 c) {
    if constexpr (DT == DT_BF16) {
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(m_s16x4, a), __builtin_bit_cast(m_s16x4, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(m_f16x4, a), __builtin_bit_cast(m_f16x4, b), c, 0, 0, 0);
    }
}

// How one lane's run of packed codes maps to MFMA B operands, per code width.
//   NWD   dwords a lane loads per step (its chunk)
//   CPC   codes in that chunk (a multiple of 8); the chunk must lie in one group
//   src() position, in the chunk's activations, of the element that multiplies
//         the o-th element of the chunk's operand sequence
// Widths that divide 32 (2, 4, 8): the chunk is 16 bytes and a masked dword gives
// pairs (code j, code j + PF/2) of one word, so MFMA t of a word multiplies codes
// (2t, 2t+PF/2, 2t+1, 2t+1+PF/2). Other widths (3, 5, 6, 7): the chunk is 32 codes
// = BITS whole dwords of the bit stream, codes are extracted one by one (bit-field
// extract, or a funnel shift where a code straddles two words) and paired in
// natural order.
// 8-bit codes do not fit the 7 mantissa bits of bf16: there the chunk is fed as
// two 4-bit planes (PLANES = 2), high nibbles first; the accumulator is scaled by
// 16 between the planes, so sum = 16*sum(hi*x) + sum(lo*x) and the offset to
// remove is MAGIC*(16+1) per activation.
// BITS = 22 stands for 2-bit codes taken 32 at a time (8 bytes per lane instead of 16): the form for groups of 32
// codes, which a 64-code chunk would straddle.
template <int DT, int BITS> struct MfmaCodec {
    static constexpr bool kHalf2 = BITS == 22;
    static constexpr int CBITS = kHalf2 ? 2 : BITS;       // bits per code
    static constexpr bool kPow2 = (32 % CBITS) == 0;
    static constexpr int PLANES = (DT == DT_BF16 && BITS == 8) ? 2 : 1;
    static constexpr float kMagic = (DT == DT_BF16 ? 128.0f : 1024.0f) * (PLANES == 2 ? 17.0f : 1.0f);
    static constexpr int PF = kPow2 ? 32 / CBITS : 0;    // codes per dword (power-of-two widths)
    static constexpr int NWD = kHalf2 ? 2 : kPow2 ? 4 : BITS;
    static constexpr int CPC = kPow2 ? NWD * PF : 32;
    static constexpr int CB = NWD * 4;                    // chunk bytes
    __host__ __device__ static constexpr int src(int o) {
        if (!kPow2) return o;
        const int wi = o / PF, oo = o % PF, t = oo / 4, e = oo % 4;
        return wi * PF + 2 * t + (e >> 1) + (e & 1) * (PF / 2);
    }
    // dwords of the chunk -> CPC/2 pair words (MAGIC+q_a | (MAGIC+q_b) << 16); MFMA m takes pairs 2m, 2m+1
    static __device__ __forceinline__ void pairs(const uint32_t (&w)[NWD], uint32_t kor, uint32_t (&pw)[PLANES * (CPC / 2)]) {
        if constexpr (PLANES == 2) {
            // plane 0 = high nibbles, plane 1 = low nibbles of the byte pairs (b_j, b_{j+2})
#pragma unroll
            for (int wi = 0; wi < 4; wi++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    pw[wi * 2 + j] = ((w[wi] >> (8 * j + 4)) & 0x000F000Fu) | kor;
                    pw[CPC / 2 + wi * 2 + j] = ((w[wi] >> (8 * j)) & 0x000F000Fu) | kor;
                }
        } else if constexpr (kPow2) {
            constexpr uint32_t MASK = ((1u << CBITS) - 1u) * 0x00010001u;
#pragma unroll
            for (int wi = 0; wi < NWD; wi++)
#pragma unroll
                for (int j = 0; j < PF / 2; j++) pw[wi * (PF / 2) + j] = ((w[wi] >> (CBITS * j)) & MASK) | kor;
        } else {
            constexpr uint32_t M1 = (1u << BITS) - 1u;
#pragma unroll
            for (int j = 0; j < CPC / 2; j++) {
                uint32_t c[2];
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const int pos = (2 * j + e) * BITS, wi = pos / 32, sh = pos % 32;
                    if (sh + BITS <= 32) c[e] = (w[wi] >> sh) & M1;
                    else c[e] = __builtin_amdgcn_alignbit(w[wi + 1 < NWD ? wi + 1 : wi], w[wi], sh) & M1;
                }
                pw[j] = (c[0] | (c[1] << 16)) | kor;
            }
        }
    }
    static __device__ __forceinline__ void load(const unsigned char* p, uint32_t (&w)[NWD]) {
        typedef uint32_t v4 __attribute__((ext_vector_type(4), aligned(4)));
        typedef uint32_t v3 __attribute__((ext_vector_type(3), aligned(4)));
        typedef uint32_t v2 __attribute__((ext_vector_type(2), aligned(4)));
        if constexpr (NWD == 2) {
            const v2 t = __builtin_nontemporal_load((const v2*)p);
            w[0] = t.x; w[1] = t.y;
        } else if constexpr (NWD == 3) {
            const v3 t = __builtin_nontemporal_load((const v3*)p);
            w[0] = t.x; w[1] = t.y; w[2] = t.z;
        } else {
            const v4 t = __builtin_nontemporal_load((const v4*)p);
            w[0] = t.x; w[1] = t.y; w[2] = t.z; w[3] = t.w;
            if constexpr (NWD == 5) {
                w[4] = __builtin_nontemporal_load((const uint32_t*)(p + 16));
            } else if constexpr (NWD == 6) {
                const v2 u = __builtin_nontemporal_load((const v2*)(p + 16));
                w[4] = u.x; w[5] = u.y;
            } else if constexpr (NWD == 7) {
                const v3 u = __builtin_nontemporal_load((const v3*)(p + 16));
                w[4] = u.x; w[5] = u.y; w[6] = u.z;
            }
        }
    }
};

__device__ __forceinline__ uint32_t waves_of(const QmvMArgs& a) { return a.KP * a.RBW; }  // waves per workgroup

// REFILL: the workgroup walks more than one row block (nrb > 1) and refills the waves' (scale, bias)
// windows as it goes; the single-block instance carries none of that state.
template <int DT, int BITS, int MP, int S, int D, int MODE, int MAXT, bool REFILL>
__global__ __launch_bounds__(MAXT) void qmv_mfma_kernel(QmvMArgs a) {
    typedef MfmaCodec<DT, BITS> Codec;
    constexpr int CPC = Codec::CPC;  // codes per lane chunk
    constexpr int NWD = Codec::NWD;  // dwords per lane chunk
    constexpr int NP = CPC / 8;      // 16-byte activation pieces per chunk
    constexpr int R = MP * S;       // activation rows per pass
    constexpr float MAGIC = Codec::kMagic;
    constexpr uint32_t NOROW = 0xFFFFFFFFu;
    static_assert(CPC % 8 == 0 && CPC / 2 >= 2, "chunk must be whole activation pieces");

    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t rows_wg = 4u * a.RBW * a.nrb;
    m_u32x4* XL = (m_u32x4*)smem;                                    // [S][nch / 16][NP][16][MP] pieces: one wave-wide step reads NP contiguous KB
    float* XG = (float*)(XL + (size_t)S * NP * a.nchp * MP);          // [S][gpr][MP] sums of the activations over each group
    float2* SB = (float2*)(XG + (size_t)S * a.gpr * MP);             // [waves][4 rows][gpw] + one zero pair
    const uint32_t sb_zero = (waves_of(a)) * 4u * a.gpw;               // index of the zero pair
    float* RED = (float*)(SB + (size_t)sb_zero + 1);                 // [KP][rows_wg][R]
    uint32_t* rowlist = (uint32_t*)(RED + (size_t)a.KP * rows_wg * R);
    __shared__ uint32_t s_meta[4];
    __shared__ float s_sq[16];

    const uint32_t tid = threadIdx.x, TPB = blockDim.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t r = lane & 3u, q = lane >> 2;
    const uint32_t kp = wave % a.KP, rbw = wave / a.KP;
    const uint32_t row0 = blockIdx.x * rows_wg;

    // ---- routing: which activation rows does this workgroup serve? ----------
    uint32_t expert = 0, cnt = a.M, lo = 0, n1 = a.M, lo2 = 0;
    if constexpr (MODE == GATHER_CSR) {
        expert = blockIdx.y;
        // E(t) = first e with t < off[e+1], else 0 (crates/metaltile-std/src/ffai/moe.rs:376-385)
        if (a.E <= 64u) {
            cnt = csr_route64(a.route, a.E, a.T, blockIdx.y, a.by_slot != 0u, lane, expert, lo, n1, lo2);
            expert = __builtin_amdgcn_readfirstlane(expert);   // (the same in every lane: a scalar)
        } else {
            if (a.by_slot) {
                expert = __builtin_amdgcn_readfirstlane(csr_slot_expert(a.route, a.E, a.T, blockIdx.y, lane));
                if (expert == NOROW) return;
            }
            cnt = csr_expert_rows(a.route, a.E, a.T, expert, lane, lo, n1, lo2);
        }
        if (cnt == 0) return;
    } else if constexpr (MODE == GATHER_INDICES) {
        expert = blockIdx.y;
        if (a.by_slot) {
            expert = __builtin_amdgcn_readfirstlane(ids_slot_expert(a.route, a.E, a.T, blockIdx.y, lane));
            if (expert == NOROW) return;
        }
        if (tid < 64) {
            uint32_t n = 0;
            for (uint32_t t0 = 0; t0 < a.T; t0 += 64) {
                uint32_t t = t0 + lane;
                bool hit = t < a.T && a.route[t] == expert;
                unsigned long long m = __ballot(hit);
                if (hit) rowlist[n + __popcll(m & ((1ull << lane) - 1ull))] = t;
                n += (uint32_t)__popcll(m);
            }
            if (lane == 0) s_meta[0] = n;
        }
        __syncthreads();
        cnt = s_meta[0];
        if (cnt == 0) return;
    } else if constexpr (MODE == GATHER_SINGLE) {
        expert = min(a.route[0], a.E - 1);  // an out-of-range id must not fault the GPU
        cnt = 1;
    }
    // GATHER_NORM: x' = (x * norm_w) * rsqrt(mean(x^2) + eps) in f32 (crates/metaltile-std/src/ffai/rms_norm_qgemv.rs:64-77,
    // 104-106) is staged as two rows, its value rounded to the element type and the rounded remainder (16 significant
    // bits in all), whose dot products are added at the end: rounding x' alone costs 3.5e-2 on the parity metric.
    float inv_rms = 1.0f;
    if constexpr (MODE == GATHER_NORM) {
        cnt = 2;
        float ss = 0.f;
        for (uint32_t c = tid; c < a.nch; c += TPB) {
            const m_u32x4* src = (const m_u32x4*)((const uint16_t*)a.x + (size_t)c * CPC);
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const m_u32x4 v = src[p];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float lo_ = DT == DT_BF16 ? bf16_bits_to_f32(v[k] & 0xFFFFu) : f16_bits_to_f32(v[k] & 0xFFFFu);
                    const float hi_ = DT == DT_BF16 ? bf16_bits_to_f32(v[k] >> 16) : f16_bits_to_f32(v[k] >> 16);
                    ss = fmaf(lo_, lo_, fmaf(hi_, hi_, ss));
                }
            }
        }
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        if (lane == 0) s_sq[wave] = ss;
        __syncthreads();
        ss = 0.f;
        for (uint32_t wv = 0; wv < TPB / 64u; wv++) ss += s_sq[wv];
        inv_rms = rsqrtf(ss / (float)a.K + a.norm_eps[0]);
    }
    auto batch_row = [&](uint32_t j) -> uint32_t {
        if (j >= cnt) return NOROW;
        if constexpr (MODE == GATHER_NORM) return 0u;
        if constexpr (MODE == GATHER_CSR) return j < n1 ? lo + j : lo2 + (j - n1);
        else if constexpr (MODE == GATHER_INDICES) return rowlist[j];
        else return j;
    };

    const size_t slab_rows = (size_t)expert * a.N;
    constexpr uint32_t SEGB = 16u * Codec::CB;  // bytes of one weight row covered by a wave-wide load
    // Uniform 64-bit bases (scalar registers) + 32-bit per-lane offsets inside the expert's slab
    // (the host checks N * RB < 4 GiB): per-lane 64-bit pointers would cost a register pair each.
    const unsigned char* wslab = a.w + slab_rows * a.RB;
    const uint16_t* sslab = (const uint16_t*)a.scales + slab_rows * a.gpr;
    const uint16_t* bslab = (const uint16_t*)a.biases + slab_rows * a.gpr;
    const uint32_t woff = (kp * a.spp) * SEGB + q * (uint32_t)Codec::CB;
    const uint32_t sppD = (a.spp + D - 1) / D * D;  // steps per row block, padded to whole rings
    // This wave's K part may be shorter than the others (the last one), and in the row's last step
    // only the first nch - 16 * (nseg - 1) lanes of a row have a chunk.
    const uint32_t spp_eff = min(a.spp, a.nseg - kp * a.spp);
    const bool short_lane = kp * a.spp + spp_eff == a.nseg && q >= a.nch - 16u * (a.nseg - 1u);
    const uint32_t lane_steps = spp_eff - (short_lane ? 1u : 0u);  // steps in which this lane's chunk exists
    // (scale, bias) pairs: every wave keeps those of its own 4 rows and its own K part in its own
    // LDS window and refills it when it moves to the next row block, so the number of row blocks
    // a workgroup walks is not bounded by LDS and no workgroup barrier sits in the refill.
    const uint32_t g_lo = ((kp * a.spp * 16u * (uint32_t)CPC) >> a.log2g) & ~3u;  // first group of the window
    const uint32_t sbw_off = wave * 4u * a.gpw;                 // this wave's window: [4 rows][gpw] pairs
    const uint32_t sb_row = sbw_off + r * a.gpw - g_lo;          // + g = this lane's row, group g
    // Lane l refills 4 pairs of the window: row l & 3, groups g_lo + 4 * (l >> 2) .. + 3 (gpw <= 64, so
    // one 8-byte load of scales and one of biases per lane and refill).
    struct SbRegs { uint2 s, b; };
    auto sbw_load = [&](uint32_t rb, SbRegs& o, uint32_t nudge = 0u) {  // nudge: an opaque zero, see the pass loop
        rb = min(rb, a.nrb - 1);
        const uint32_t row = min(row0 + (rb * a.RBW + rbw) * 4u + (lane & 3u), a.N - 1);
        if (a.gpr & 3u) {
            // rows of scales that are not a whole number of 8-byte vectors (K / G = 14, 18, 22, 45 ...):
            // element loads, each clamped to the row
            const uint32_t g0 = g_lo + (lane >> 2) * 4u, base = row * a.gpr + nudge;
            uint32_t e[4], f[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t idx = base + min(g0 + (uint32_t)j, a.gpr - 1);
                e[j] = sslab[idx];
                f[j] = bslab[idx];
            }
            o.s = make_uint2(e[0] | (e[1] << 16), e[2] | (e[3] << 16));
            o.b = make_uint2(f[0] | (f[1] << 16), f[2] | (f[3] << 16));
        } else {
            const uint32_t src = row * a.gpr + min(g_lo + (lane >> 2) * 4u, a.gpr - 4) + nudge;
            o.s = *(const uint2*)(sslab + src);
            o.b = *(const uint2*)(bslab + src);
        }
    };
    auto sbw_store = [&](const SbRegs& o) {
        if (lane < a.gpw) {  // gpw / 4 vectors for each of the 4 rows
            float s4[4], b4[4];
            if constexpr (DT == DT_BF16) {
                s4[0] = bf16_bits_to_f32(o.s.x & 0xFFFFu); s4[1] = bf16_bits_to_f32(o.s.x >> 16);
                s4[2] = bf16_bits_to_f32(o.s.y & 0xFFFFu); s4[3] = bf16_bits_to_f32(o.s.y >> 16);
                b4[0] = bf16_bits_to_f32(o.b.x & 0xFFFFu); b4[1] = bf16_bits_to_f32(o.b.x >> 16);
                b4[2] = bf16_bits_to_f32(o.b.y & 0xFFFFu); b4[3] = bf16_bits_to_f32(o.b.y >> 16);
            } else {
                s4[0] = f16_bits_to_f32(o.s.x & 0xFFFFu); s4[1] = f16_bits_to_f32(o.s.x >> 16);
                s4[2] = f16_bits_to_f32(o.s.y & 0xFFFFu); s4[3] = f16_bits_to_f32(o.s.y >> 16);
                b4[0] = f16_bits_to_f32(o.b.x & 0xFFFFu); b4[1] = f16_bits_to_f32(o.b.x >> 16);
                b4[2] = f16_bits_to_f32(o.b.y & 0xFFFFu); b4[3] = f16_bits_to_f32(o.b.y >> 16);
            }
            float4* dst = (float4*)(SB + sbw_off + (lane & 3u) * a.gpw + (lane >> 2) * 4u);
            dst[0] = make_float4(s4[0], b4[0] - MAGIC * s4[0], s4[1], b4[1] - MAGIC * s4[1]);
            dst[1] = make_float4(s4[2], b4[2] - MAGIC * s4[2], s4[3], b4[3] - MAGIC * s4[3]);
        }
    };

    // Address of the 16 bytes this lane loads at step (rb, sg). Steps past the
    // end of a row block or of the wave's work re-read a valid address; what they
    // load is multiplied by a zero scale.
    auto w_ptr = [&](uint32_t rb, uint32_t sg, uint32_t nudge = 0u) -> const unsigned char* {
        rb = min(rb, a.nrb - 1);
        sg = min(sg, spp_eff - 1);
        const uint32_t row = min(row0 + (rb * a.RBW + rbw) * 4u + r, a.N - 1);
        return wslab + (uint32_t)(row * a.RB + min(sg * SEGB + woff, a.RB - (uint32_t)Codec::CB) + nudge);
    };

    const uint32_t n_pass = (MODE == GATHER_CSR || MODE == GATHER_INDICES) ? (cnt + R - 1) / R : 1u;
    for (uint32_t pass = 0; pass < n_pass; pass++) {
        // Loads return in issue order, so the small ones go first: this thread's
        // first activation chunk and its first four (scale, bias) elements, then D
        // weight loads per lane, which stay in flight while the small data are
        // staged into LDS. All of it is straight-line code on clamped addresses so
        // that the waits count exactly.
        const uint32_t base_row = pass * R;
        const uint32_t live = min((uint32_t)R, cnt - base_row);
        // Rows past the pass's last live row are never staged: what the matrix
        // cores compute from their LDS slots lands in output rows nobody stores.
        const uint32_t ntask = live * a.nchp;  // chunks past the row's end are staged as zeros
        uint32_t raw[NP * 4];
        uint32_t nraw[MODE == GATHER_NORM ? NP * 4 : 1];   // the norm's weights for the chunk
        bool row_live;
        auto x_load = [&](uint32_t task) {
            const uint32_t i = task / a.nchp, c = task - i * a.nchp;
            uint32_t t = batch_row(base_row + i);
            row_live = t != NOROW && c < a.nch;
            if (t == NOROW) t = batch_row(base_row);  // the pass's first row always exists
            const m_u32x4* src = (const m_u32x4*)((const uint16_t*)a.x + (size_t)t * a.K + (size_t)min(c, a.nch - 1) * CPC);
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const m_u32x4 v = src[p];
                raw[4 * p] = v.x; raw[4 * p + 1] = v.y; raw[4 * p + 2] = v.z; raw[4 * p + 3] = v.w;
            }
            if constexpr (MODE == GATHER_NORM) {
                const m_u32x4* nsrc = (const m_u32x4*)((const uint16_t*)a.norm_w + (size_t)min(c, a.nch - 1) * CPC);
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    const m_u32x4 v = nsrc[p];
                    nraw[4 * p] = v.x; nraw[4 * p + 1] = v.y; nraw[4 * p + 2] = v.z; nraw[4 * p + 3] = v.w;
                }
            }
        };
        const uint32_t cpg = (1u << a.log2g) / (uint32_t)CPC;  // chunks per group: a power of two, at most 16
        auto x_store = [&](uint32_t task) {
            const uint32_t i = task / a.nchp, c = task - i * a.nchp;
            if (!row_live) {
#pragma unroll
                for (int j = 0; j < NP * 4; j++) raw[j] = 0u;
            }
            if constexpr (MODE == GATHER_NORM) {   // row 0: x' rounded; row 1: what the rounding left
#pragma unroll
                for (int j = 0; j < NP * 4; j++) {
                    uint32_t o2[2];
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const uint32_t xb = h ? raw[j] >> 16 : raw[j] & 0xFFFFu, wb = h ? nraw[j] >> 16 : nraw[j] & 0xFFFFu;
                        const float xf = DT == DT_BF16 ? bf16_bits_to_f32(xb) : f16_bits_to_f32(xb);
                        const float wf = DT == DT_BF16 ? bf16_bits_to_f32(wb) : f16_bits_to_f32(wb);
                        const float xn = (xf * wf) * inv_rms;
                        uint32_t hb, lb;
                        RemSplit<DT>::split(xn, hb, lb);   // (the f16 remainder scaled into the normal range)
                        o2[h] = i == 0 ? hb : lb;
                    }
                    raw[j] = o2[0] | (o2[1] << 16);
                }
            }
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < NP * 4; j++) {
                if constexpr (DT == DT_BF16) sum += bf16_bits_to_f32(raw[j] & 0xFFFFu) + bf16_bits_to_f32(raw[j] >> 16);
                else sum += f16_bits_to_f32(raw[j] & 0xFFFFu) + f16_bits_to_f32(raw[j] >> 16);
            }
            const uint32_t s = i / MP, i4 = i % MP;
            // A group is cpg consecutive chunks of one row, staged by cpg consecutive lanes (tasks are
            // dealt in order, a row is a multiple of 16 >= cpg chunks, and the lanes of such a block are
            // all staging or all idle): butterfly over them, one lane writes. The bias term of a row
            // block is then b' . (group sums), added once per row block instead of once per chunk.
            for (uint32_t o = 1; o < cpg; o <<= 1) sum += __shfl_xor(sum, (int)o, 64);
            if ((c & (cpg - 1u)) == 0u && c < a.nch) XG[((size_t)s * a.gpr + c / cpg) * MP + i4] = sum;
#pragma unroll
            for (int p = 0; p < NP; p++) {
                uint32_t o[4];
#pragma unroll
                for (int dw = 0; dw < 4; dw++) {
                    uint32_t h[2];
#pragma unroll
                    for (int e2 = 0; e2 < 2; e2++) {
                        const int oe = p * 8 + dw * 2 + e2;          // element of the chunk's operand sequence
                        const int se = Codec::src(oe);               // source element
                        h[e2] = (se & 1) ? (raw[se >> 1] >> 16) : (raw[se >> 1] & 0xFFFFu);
                    }
                    o[dw] = h[0] | (h[1] << 16);
                }
                m_u32x4 piece = {o[0], o[1], o[2], o[3]};
                XL[(size_t)s * NP * a.nchp * MP + ((((size_t)(c >> 4) * NP + p) * 16u + (c & 15u)) * MP + i4)] = piece;
            }
        };
        // In the gather modes this body is a loop over passes. Index math of the staging and of the
        // final store is cheap but would be hoisted out of that loop and then held in registers
        // all through the streaming; an opaque copy of the thread id keeps it inside.
        uint32_t ptid = tid, pzero = 0u;
        if constexpr (MODE == GATHER_CSR || MODE == GATHER_INDICES) asm volatile("" : "+v"(ptid), "+v"(pzero));
        x_load(min(ptid, ntask - 1));
        SbRegs sb_now, sb_next;
        sbw_load(0, sb_now, pzero);
        if constexpr (REFILL) sbw_load(1, sb_next, pzero);
        MTQ_MFMA_KEEP_ORDER();
        MTQ_MFMA_KEEP_ORDER();
        uint32_t ring[D][NWD];
#pragma unroll
        for (int d = 0; d < D; d++) Codec::load(w_ptr(0, d, pzero), ring[d]);
        MTQ_MFMA_KEEP_ORDER();
        if (ptid < ntask) x_store(ptid);
        sbw_store(sb_now);
        if (tid == 0) SB[sb_zero] = make_float2(0.f, 0.f);
        for (uint32_t task = ptid + TPB; task < ntask; task += TPB) {
            x_load(task);
            x_store(task);
        }
        __syncthreads();

        // ---- stream ------------------------------------------------------------
        const uint32_t arow = r & (uint32_t)(MP - 1);
        const uint32_t kor = magic_or_vgpr<DT>();
        // One ring turn = D steps. Every turn but the wave's last issues the loads
        // of the turn after it; the last one is a separate copy of the body without
        // loads, so no load is ever issued twice and the loop stays branch-free
        // around its loads.
        float tot[S][MP];
#pragma unroll
        for (int s = 0; s < S; s++)
#pragma unroll
            for (int i = 0; i < MP; i++) tot[s][i] = 0.f;
        uint32_t rb = 0, sg0 = 0;
        // LDS addresses as a per-lane constant plus a wave-uniform offset per step: the step index is
        // uniform, so its share is scalar arithmetic and each read costs one vector add. (A wave-wide
        // step covers 16 * CPC codes, a whole number of groups: the host checks G <= 16 * CPC.)
        const uint32_t c_lane = kp * a.spp * 16u + q;
        const unsigned char* xl_lane = (const unsigned char*)(XL + ((size_t)(kp * a.spp) * NP * 16u + q) * MP + arow);
        const uint32_t sb_idx = sb_row + ((c_lane * (uint32_t)CPC) >> a.log2g);  // 32-bit sum: sb_row alone may have wrapped
        const unsigned char* sb_lane = (const unsigned char*)(SB + sb_idx);
        const unsigned char* sb_zero_p = (const unsigned char*)(SB + sb_zero);
        const uint32_t xl_set = (uint32_t)NP * a.nchp * MP * 16u;  // bytes from one row set to the next
        const uint32_t part_g0 = (kp * a.spp * 16u * (uint32_t)CPC) >> a.log2g;  // this wave's K part: whole groups
        const uint32_t part_ng = min(a.gpr, ((kp * a.spp + spp_eff) * 16u * (uint32_t)CPC) >> a.log2g) - part_g0;
        // SE: row sets the pass works on. A pass of a gather whose expert has at most MP rows left skips the
        // second set's operand reads, MFMAs and scale terms (its rows are not live and are never stored).
        auto turn = [&](auto issue_tag, auto sets_tag) {
            constexpr bool ISSUE = decltype(issue_tag)::value;
            constexpr int SE = decltype(sets_tag)::value;
            const uint32_t row_local = (rb * a.RBW + rbw) * 4u + r;
            {
                const bool wrap = sg0 + D >= sppD;
                const uint32_t nrb_i = wrap ? rb + 1 : rb;
                const uint32_t nsg0 = wrap ? 0u : sg0 + D;
#pragma unroll
                for (int d = 0; d < D; d++) {
                    const uint32_t sg = sg0 + d;
                    const bool valid = sg < lane_steps;
                    const uint32_t sgc = min(sg, spp_eff - 1);  // uniform
                    // operands from LDS
                    m_u32x4 av[S][NP];
#pragma unroll
                    for (int s = 0; s < SE; s++) {
#pragma unroll
                        for (int p = 0; p < NP; p++)
                            av[s][p] = *(const m_u32x4*)(xl_lane + (sgc * ((uint32_t)NP * 16u * MP * 16u) + (uint32_t)s * xl_set) + p * (16 * MP * 16));
                    }
                    const uint32_t g_off = ((sgc * 16u * (uint32_t)CPC) >> a.log2g) * 8u;
                    const float2 sb = *(const float2*)(valid ? sb_lane + g_off : sb_zero_p);
                    uint32_t pw[Codec::PLANES * (CPC / 2)];
                    Codec::pairs(ring[d], kor, pw);
                    if constexpr (ISSUE) Codec::load(w_ptr(nrb_i, nsg0 + d), ring[d]);
                    // codes -> B operands, MFMAs
                    m_f32x4 acc[S];
#pragma unroll
                    for (int pl = 0; pl < Codec::PLANES; pl++) {
#pragma unroll
                        for (int m = 0; m < CPC / 4; m++) {  // MFMA m of the chunk: codes 4m .. 4m+3 of its operand sequence
                            const m_u32x2 b = {pw[pl * (CPC / 2) + 2 * m], pw[pl * (CPC / 2) + 2 * m + 1]};
#pragma unroll
                            for (int s = 0; s < SE; s++) {
                                const m_u32x4 piece = av[s][m / 2];
                                const m_u32x2 aop = (m & 1) ? m_u32x2{piece.z, piece.w} : m_u32x2{piece.x, piece.y};
                                const m_f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                                acc[s] = mfma4<DT>(aop, b, (m == 0 && pl == 0) ? zero : acc[s]);
                            }
                        }
                        if (pl + 1 < Codec::PLANES) {
#pragma unroll
                            for (int s = 0; s < SE; s++)
#pragma unroll
                                for (int i = 0; i < MP; i++) acc[s][i] *= 16.0f;  // only the live rows are read later
                        }
                    }
#pragma unroll
                    for (int s = 0; s < SE; s++)
#pragma unroll
                        for (int i = 0; i < MP; i++) {
                            tot[s][i] = fmaf(sb.x, acc[s][i], tot[s][i]);
                        }
                }
                if (wrap) {
                    // bias term of this row block: the 16 lanes of a weight row share its K part's groups
                    for (uint32_t gi = q; gi < part_ng; gi += 16u) {
                        const uint32_t g = part_g0 + gi;
                        const float bq = SB[sb_row + g].y;
#pragma unroll
                        for (int s = 0; s < SE; s++) {
                            const float* xg = XG + ((size_t)s * a.gpr + g) * MP;
#pragma unroll
                            for (int i = 0; i < MP; i++) tot[s][i] = fmaf(bq, xg[i], tot[s][i]);
                        }
                    }
                    // lanes of one weight row (same r, all q) add up: q spans lane bits 2..5
#pragma unroll
                    for (int s = 0; s < SE; s++)
#pragma unroll
                        for (int i = 0; i < MP; i++) {
                            float v = tot[s][i];
                            v += dpp_f32<0x124>(v);  // row_ror:4
                            v += dpp_f32<0x128>(v);  // row_ror:8
                            v += __shfl_xor(v, 16, 64);
                            v += __shfl_xor(v, 32, 64);
                            if (q == 0) RED[((size_t)kp * rows_wg + row_local) * R + s * MP + i] = v;
                            tot[s][i] = 0.f;
                        }
                    rb++;
                    sg0 = 0;
                    // the window now holds a finished row block: refill it with the next one's pairs,
                    // loaded one row block ago, and fetch the pairs of the block after that
                    if constexpr (REFILL) {
                        sbw_store(sb_next);
                        if constexpr (ISSUE) sbw_load(rb + 1, sb_next);
                    }
                } else {
                    sg0 += D;
                }
            }
        };
        const uint32_t n_turns = a.nrb * (sppD / D);
        if (S > 1 && live <= (uint32_t)MP) {
            for (uint32_t it = 0; it + 1 < n_turns; it++) turn(std::true_type{}, std::integral_constant<int, 1>{});
            turn(std::false_type{}, std::integral_constant<int, 1>{});
        } else {
            for (uint32_t it = 0; it + 1 < n_turns; it++) turn(std::true_type{}, std::integral_constant<int, S>{});
            turn(std::false_type{}, std::integral_constant<int, S>{});
        }
        __syncthreads();

        // ---- add the K parts and store ----------------------------------------
        uint32_t stid = tid;
        if constexpr (MODE == GATHER_CSR || MODE == GATHER_INDICES) asm volatile("" : "+v"(stid));
        if constexpr (MODE == GATHER_NORM) {   // one output row: the sum of the two staged rows' dot products
            for (uint32_t rl = stid; rl < rows_wg; rl += TPB) {
                const uint32_t row = row0 + rl;
                if (row >= a.N) continue;
                float v = 0.f;
                for (uint32_t k2 = 0; k2 < a.KP; k2++)
                    v += RED[((size_t)k2 * rows_wg + rl) * R] + RED[((size_t)k2 * rows_wg + rl) * R + 1] * (1.0f / RemSplit<DT>::kRemScale);
                store_elem<DT>(a.out, row, v);
            }
            return;
        }
        for (uint32_t idx = stid; idx < rows_wg * live; idx += TPB) {
            const uint32_t i = idx / rows_wg, rl = idx - i * rows_wg;
            const uint32_t row = row0 + rl;
            if (row >= a.N) continue;
            float v = 0.f;
            for (uint32_t k2 = 0; k2 < a.KP; k2++) v += RED[((size_t)k2 * rows_wg + rl) * R + i];
            const uint32_t t = batch_row(base_row + i);
            store_elem<DT>(a.out, (size_t)t * a.N + row, v);
        }
        if (pass + 1 < n_pass) __syncthreads();
    }
}

template <int DT, int BITS, int MP, int S, int MODE>
int qmv_mfma_launch_one(QmvMArgs& a, const QmvMGeom& g, const LaunchCtx& lc) {
    // Two row sets (8 rows per pass) at 1024 threads leave 128 registers per lane and the kernel spills; at 512
    // threads it has 256 and keeps eight weight loads in flight per lane instead of four: the same bytes in flight
    // per compute unit from half the waves.
    // A wave's steps per row block are walked in whole rings: with 4 steps (rows of 2048 4-bit codes) a ring of eight
    // is half padding, loads included (128 experts of 256 x 2048, 8 rows each: 17.9 -> 23.2 us). The deep ring is taken
    // where it pads no more than the ring of four does, and for 4-bit codes only (8-bit, 8 rows, 4096 x 4096: 10.2 us
    // on the ring of eight, 9.2 on that of four; larger matrices alike).
    constexpr int MAXT = S >= 2 ? 512 : 1024;
    constexpr bool DEEP = S == 2 && BITS == 4;
    if (g.tpb > (uint32_t)MAXT) return fail(ERR_UNSUPPORTED, "mfma qmv: workgroup too large for this row count");
    const void* fn = a.nrb > 1 ? (const void*)qmv_mfma_kernel<DT, BITS, MP, S, 4, MODE, MAXT, true>
                               : (const void*)qmv_mfma_kernel<DT, BITS, MP, S, 4, MODE, MAXT, false>;
    if constexpr (DEEP) {
        if ((a.spp + 7u) / 8u * 8u == (a.spp + 3u) / 4u * 4u)
            fn = a.nrb > 1 ? (const void*)qmv_mfma_kernel<DT, BITS, MP, S, 8, MODE, MAXT, true>
                           : (const void*)qmv_mfma_kernel<DT, BITS, MP, S, 8, MODE, MAXT, false>;
    }
    if (g.shmem > 48 * 1024) {
        hipError_t e = set_max_dynamic_lds(fn, (size_t)g.shmem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(max dynamic LDS)");
    }
    void* args[] = {&a};
    hipError_t e = launch_kernel(fn, g.grid, dim3(g.tpb), args, g.shmem, lc);
    if (e != hipSuccess) return hip_fail(e, "mfma qmv kernel launch");
    return ERR_OK;
}

template <int DT, int BITS, int MODE>
int qmv_mfma_launch_rows(QmvMArgs& a, const QmvMGeom& g, const LaunchCtx& lc) {
    if constexpr (MODE == GATHER_SINGLE) {
        return qmv_mfma_launch_one<DT, BITS, 1, 1, MODE>(a, g, lc);
    } else if constexpr (MODE == GATHER_NONE) {
        if (g.s == 1) {
            switch (g.mp) {
                case 1: return qmv_mfma_launch_one<DT, BITS, 1, 1, MODE>(a, g, lc);
                case 2: return qmv_mfma_launch_one<DT, BITS, 2, 1, MODE>(a, g, lc);
                default: return qmv_mfma_launch_one<DT, BITS, 4, 1, MODE>(a, g, lc);
            }
        }
        if (g.s == 2) return qmv_mfma_launch_one<DT, BITS, 4, 2, MODE>(a, g, lc);
        return qmv_mfma_launch_one<DT, BITS, 4, 4, MODE>(a, g, lc);
    } else {
        if (g.s == 1) return qmv_mfma_launch_one<DT, BITS, 4, 1, MODE>(a, g, lc);
        if (g.s == 2) return qmv_mfma_launch_one<DT, BITS, 4, 2, MODE>(a, g, lc);
        return qmv_mfma_launch_one<DT, BITS, 4, 4, MODE>(a, g, lc);
    }
}

template <int DT, int BITS>
int qmv_mfma_launch_mode(QmvMArgs& a, int mode, const QmvMGeom& g, const LaunchCtx& lc) {
    switch (mode) {
        case GATHER_NONE: return qmv_mfma_launch_rows<DT, BITS, GATHER_NONE>(a, g, lc);
        case GATHER_CSR: return qmv_mfma_launch_rows<DT, BITS, GATHER_CSR>(a, g, lc);
        case GATHER_INDICES: return qmv_mfma_launch_rows<DT, BITS, GATHER_INDICES>(a, g, lc);
        case GATHER_NORM:
            if constexpr (BITS == 4) return qmv_mfma_launch_one<DT, 4, 2, 1, GATHER_NORM>(a, g, lc);
            else return fail(ERR_UNSUPPORTED, "mfma qmv: the fused norm is built for 4-bit codes");
        default: return qmv_mfma_launch_rows<DT, BITS, GATHER_SINGLE>(a, g, lc);
    }
}

template <int DT> int qmv_mfma_launch_dtype(QmvMArgs& a, int bits, int mode, const QmvMGeom& g, const LaunchCtx& lc) {
    switch (bits) {
        case 2: return qmv_mfma_launch_mode<DT, 2>(a, mode, g, lc);
        case 4: return qmv_mfma_launch_mode<DT, 4>(a, mode, g, lc);
        default: return qmv_mfma_launch_mode<DT, 8>(a, mode, g, lc);
    }
}

// Widths whose codes straddle words (3, 5, 6): instantiated in their own translation units.
template <int DT> int qmv_mfma_launch_dtype_odd(QmvMArgs& a, int bits, int mode, const QmvMGeom& g, const LaunchCtx& lc) {
    switch (bits) {
        case 3: return qmv_mfma_launch_mode<DT, 3>(a, mode, g, lc);
        case 5: return qmv_mfma_launch_mode<DT, 5>(a, mode, g, lc);
        case 6: return qmv_mfma_launch_mode<DT, 6>(a, mode, g, lc);
        case 22: return qmv_mfma_launch_mode<DT, 22>(a, mode, g, lc);   // 2-bit codes in 8-byte chunks (groups of 32)
        default: return fail(ERR_UNSUPPORTED, "mfma qmv: code width");
    }
}

}  // namespace mtq
