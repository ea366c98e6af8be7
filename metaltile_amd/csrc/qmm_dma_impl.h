// The register-operand tile kernel with its activation tile brought in by load-to-LDS instructions
// (see qmm_direct.hip for the tiling; this header only differs in how the operands travel).
#pragma once
#include "qmm_direct_impl.h"
#include "vm_schedule.h"

#include <type_traits>

namespace mtq {

typedef uint32_t qm_u32x4 __attribute__((ext_vector_type(4)));
typedef float qm_f32x2 __attribute__((ext_vector_type(2)));

// f(integral_constant<int, I>) for I = B .. E-1: loop indices that are constant expressions in the body.
template <int B, int E, class F> __device__ __forceinline__ void qm_static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        qm_static_for<B + 1, E>(f);
    }
}

// One 16-byte-per-lane load from global memory straight into LDS: lane l's bytes land at
// lds_base + 16 * l (lds_base is wave-uniform and goes through M0); the global address is
// sbase + voff per lane. Counts in vmcnt like any vector memory load.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // M0 is a reserved register: naming it as clobbered is the point
__device__ __forceinline__ void qm_load_to_lds(uint32_t lds_base, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(sbase) : "memory", "m0");
}
// The same with 4 bytes per lane: lane l's dword lands at lds_base + 4 * l.
__device__ __forceinline__ void qm_load_to_lds_b32(uint32_t lds_base, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_base), "v"(voff), "s"(sbase) : "memory", "m0");
}
#pragma clang diagnostic pop
// 16 bytes per lane from sbase + voff into registers. The result is valid only after a qm_wait_vm
// that covers it; until then the registers must not be read or copied.
__device__ __forceinline__ void qm_load_regs(qm_u32x4& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
// Waits until at most N vector memory loads of this wave are outstanding (they complete in order).
template <int N> __device__ __forceinline__ void qm_wait_vm() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// The same, and ties the loaded registers to the wait so that no use of them is scheduled above it.
template <int N> __device__ __forceinline__ void qm_wait_vm_for(qm_u32x4& r) {
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r) : "n"(N) : "memory");
}
template <int N> __device__ __forceinline__ void qm_wait_vm_for2(qm_u32x4& r0, qm_u32x4& r1) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(r0), "+v"(r1) : "n"(N) : "memory");
}

// Four 4-bit codes -> four elements s * q + b rounded to T, as two dwords. e and o hold the even and the odd
// codes of a weight dword one per byte (e = w & 0x0F0F0F0F, o = (w >> 4) & 0x0F0F0F0F); `half` picks bytes
// 0, 1 or 2, 3. A byte 0..15 read as an fp8 (E4M3) number is exactly code / 512, so one packed fp8 -> f32
// convert yields two codes, and with s512 = 512 * s the fused multiply-add rounds the same exact value
// s * q + b as it would from the integer code.
template <int DT> __device__ __forceinline__ void qm_dequant4_b4(uint32_t e, uint32_t o, int half, float s512, float b, uint32_t& d0, uint32_t& d1) {
    const qm_f32x2 fe = half ? __builtin_amdgcn_cvt_pk_f32_fp8((int)e, true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)e, false);
    const qm_f32x2 fo = half ? __builtin_amdgcn_cvt_pk_f32_fp8((int)o, true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)o, false);
    d0 = pack2<DT>(fmaf(fe.x, s512, b), fmaf(fo.x, s512, b));
    d1 = pack2<DT>(fmaf(fe.y, s512, b), fmaf(fo.y, s512, b));
}

// The loop's vector-memory schedule and the waits that follow from it. Per iteration `it` a wave issues, in this order,
//   ring of three or more tiles: the weights of iteration it + WSN (NWL loads), its piece of the next scale window (NSB),
//                                its share of tile it + NBUF - 1 (IPW load-to-LDS instructions);
//   ring of two:                 the window piece, its share of tile it + 1, then the weights of iteration it + WSN;
// it needs the weights of iteration it + 1 before it converts them (next_weights) and its share of tile it + 1 before
// the iteration's barrier (next_tile). The prologue issues the first WSN weight sets, then the first NBUF - 1 tiles,
// and needs tile 0 and weight set 0 (first). holds() replays that order and checks every N against it.
template <int NBUF, int WSN, int IPW, int NWL, int NSB> struct QmmDmaWaits {
    static constexpr int next_weights = NBUF == 2 ? 2 * IPW + 2 * NWL + 2 * NSB : WSN * (IPW + NSB) + (WSN - 1) * NWL;
    static constexpr int next_tile = NBUF == 2 ? NWL : NBUF == 3 ? IPW + NWL + NSB : (NBUF - 2) * (IPW + NWL) - 1;
    static constexpr int first = (NBUF - 2) * IPW;
    enum { W = 1, X = 2, S = 3 };
    static constexpr bool holds() {
        VmQueue q;
        for (int i = 0; i < WSN; i++) q.issue(vm_tag(W, i), NWL);
        for (int i = 0; i < NBUF - 1; i++) q.issue(vm_tag(X, i), IPW);
        q.wait(first);
        if (!q.landed(vm_tag(X, 0)) || !q.landed(vm_tag(W, 0))) return false;
        for (int it = 0; it < 4 * (WSN > NBUF ? WSN : NBUF) + 4; it++) {
            if (NBUF == 2) {
                q.issue(vm_tag(S, it), NSB);
                q.issue(vm_tag(X, it + 1), IPW);
                q.issue(vm_tag(W, it + WSN), NWL);
            } else {
                q.issue(vm_tag(W, it + WSN), NWL);
                q.issue(vm_tag(S, it), NSB);
                q.issue(vm_tag(X, it + NBUF - 1), IPW);
            }
            const int w_exact = q.younger_than(vm_tag(W, it + 1)), x_exact = q.younger_than(vm_tag(X, it + 1));
            q.wait(next_weights);
            if (!q.landed(vm_tag(W, it + 1))) return false;   // the conversion would read weights still in flight
            q.wait(next_tile);
            if (!q.landed(vm_tag(X, it + 1))) return false;   // the barrier would release a tile still in flight
            // steady state: exactly what the schedule allows (rings deeper than three are allowed one less: their first
            // iterations follow the prologue's order)
            if (it >= WSN && next_weights != w_exact) return false;
            if (it >= NBUF && x_exact - next_tile > (NBUF > 3 ? 1 : 0)) return false;
            // a piece of a scale window is read two iterations after it was issued at the earliest
            if (NSB && it >= 2 && !q.landed(vm_tag(S, it - 2))) return false;
        }
        return true;
    }
};

// Same tiling and arguments as qmm_direct_kernel with 8 waves (KG = 2 or 4 K-groups x 8 / KG column waves,
// 4-bit codes, scales and biases of the tile staged in LDS), same results; what differs:
//   activations: the (32 * MB) x (64 * KG) tile of an iteration is MB * KG slots of 32 rows x 64 k (4 KB,
//     16-byte chunks XOR-swizzled so that the fragment reads are conflict free); the eight waves share its
//     load-to-LDS instructions (MB * KG / 2 each), issued two iterations ahead into a ring of three tiles: no
//     register, no LDS store instruction and no vector ALU work is spent on staging. A wave waits for its own
//     share of the next tile before the iteration's barrier, so past the barrier the whole tile is in LDS.
//   weights: 16 bytes per lane (the 32 codes it converts) straight into registers three iterations ahead;
//     converted one iteration ahead with the packed fp8 -> f32 convert (two codes per instruction).
// Every vector memory load of the loop is issued by hand in a fixed order, so the waits are "at most N loads
// outstanding" with compile-time N.
// NB is the depth of the ring of activation tiles (0: three, or two for 256-row tiles, whose tile is 64 KB): tile
// it + NB - 1 is issued during iteration it. Measured at 1024 x 4096 x 4096 the depth does not matter (2 / 3 / 4:
// 39.3 / 40.0 / 41.5 us): the loop is not waiting for latency.
// 256-row tiles (MB = 8) keep the scales and biases unpadded, row r rotated by 8 r elements, so that two tiles and the
// window fill the 160 KB exactly at 64 groups per row; their epilogue runs in two rounds of 128 rows.
// WIN: rows too long for their scales and biases to sit in LDS whole (K / G groups x 128 columns x 4 bytes). They
// are kept as two windows of 32 groups (16 KB each: [scales | biases][128 columns][32 groups], 16-byte chunks
// XOR-swizzled by column pair); while the loop reads one window, every wave brings 256 bytes of the next one in per
// iteration with a 4-byte-per-lane load-to-LDS (64 pieces = 8 iterations of the G / 4 a window lasts, so groups of
// 64 and 128 codes), as one more hand-counted load per iteration. The LDS footprint no longer depends on K.
// BITS: 4, or 8 (a lane's 32 codes are then 32 bytes: two 16-byte loads per iteration, bytes converted with the
// byte-select converts; everything else alike).
template <int DT, int MB, int KG, int NW, int NB = 0, bool GR = false, bool SP = false, bool WIN = false, int BITS = 4>
__global__ __launch_bounds__(64 * NW) void qmm_dma_kernel(QmmDArgs a) {
    static_assert(NW == 8 || NW == 16, "two or four waves per SIMD");
    static_assert(KG == 2 || KG == 4, "2 or 4 K-groups");
    static_assert(MB == 1 || MB == 2 || MB == 4 || MB == 8, "32 to 256 rows");
    static_assert(BITS == 4 || BITS == 8, "4- or 8-bit codes");
    constexpr int NWL = BITS / 4;              // 16-byte weight loads per lane and iteration
    constexpr float KSCALE = BITS == 4 ? 512.f : 1.f;   // 4-bit codes are read as fp8 = code / 512
    constexpr int NT = 64 * NW, NWV = NW / KG;
    constexpr int DBN = 32 * NWV, DBK = 64 * KG, DBM = 32 * MB;
    constexpr int NSLOT = MB * KG, SLOT = 4096, TILE = NSLOT * SLOT;
    constexpr int NBUF = NB ? NB : MB == 8 ? 2 : 3;
    static_assert(NBUF >= 2 && NBUF <= 6, "ring of 2 to 6 tiles");
    static_assert(!WIN || (KG == 2 && NW == 8 && !SP && NBUF <= 3), "windows: 128-k iterations, 8 waves, whole rows");
    constexpr int NSB = WIN ? 1 : 0;           // window loads per wave and iteration
    constexpr int WSN = NBUF < 3 ? 3 : NBUF;   // weight register sets: weights are issued WSN iterations ahead
    constexpr int IPW = NSLOT * 4 / NW;       // load-to-LDS instructions per wave and iteration
    static_assert(IPW >= 1 && NSLOT * 4 % NW == 0, "the tile's load instructions divide among the waves");
    constexpr int NM = 4 * MB;                // MFMAs per wave and iteration
    constexpr int UN = WSN % 2 ? 2 * WSN : WSN;   // unroll: a multiple of the ring, of the weight sets and of 2 (fragment parity)
    static_assert(UN % NBUF == 0 && UN % WSN == 0 && UN % 2 == 0, "unroll covers every ring");
    typedef QmmDmaWaits<NBUF, WSN, IPW, NWL, NSB> Waits;
    static_assert(Waits::holds(), "a hand-counted vmcnt wait does not match the order in which the loop issues its loads");
    extern __shared__ __align__(16) unsigned char lds[];  // NBUF tiles, then the scales / biases window

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t kg = wave / NWV, wn = wave % NWV;
    const uint32_t fr = lane & 31u, fh = lane >> 5;

    const uint32_t total = a.m_tiles * a.n_tiles;
    uint32_t vid = blockIdx.x;
    if (!GR && total % 8 == 0) vid = (blockIdx.x & 7u) * (total / 8) + (blockIdx.x >> 3);
    uint32_t nt = a.by_m ? vid % a.n_tiles : vid / a.m_tiles, mt = a.by_m ? vid / a.n_tiles : vid % a.m_tiles;
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
    const uint32_t ilast = a.iters - 1;
    // groups of scales / biases this workgroup needs: [sb_g0, sb_g0 + sb_ng), whole 8-element vectors (rows that are
    // not whole vectors, K-split instances only: whole dwords, two groups)
    const uint32_t sb_al = (a.gpr & 7u) ? 1u : 7u;
    const uint32_t sb_g0 = ((it_base * DBK) >> a.log2g) & ~sb_al;
    const uint32_t sb_ng = min(a.gpr - sb_g0, (((((it_base + a.iters) * DBK - 1) >> a.log2g) + 1 - sb_g0) + sb_al) & ~sb_al);

    // ---- per-lane offsets ---------------------------------------------------------------------------
    // this wave's load-to-LDS instructions: unit q = wave * IPW + i is quarter q % 4 of slot q / 4; slot sl holds
    // row block sl % MB, k-block sl / MB of the iteration; a quarter is 8 rows x 128 bytes, lane l moving chunk
    // (l % 8) ^ ((row / 2) % 8) of row 8 * quarter + l / 8
    auto x_offset = [&](int i) -> uint32_t {
        const uint32_t q = wave * IPW + i, sl = q / 4, t = q % 4;
        const uint32_t rr = 8 * t + (lane >> 3), c = (lane & 7u) ^ ((rr >> 1) & 7u);
        const uint32_t lrow = min((sl % MB) * 32 + rr, row_count - 1);
        return row_of(lrow) * (a.K * 2) + (sl / MB) * 128 + c * 16;
    };
    // 256-row tiles with windows have no register to spare (three of these offsets were spilled and reloaded inside
    // the loop, each reload with the compiler's wait for every load in flight): a wave's instructions 4 .. 7 there move
    // the row block after that of instructions 0 .. 3, 32 rows on, which in a full tile is the same lane offsets from
    // a base 32 rows on. Only those four are kept; a ragged last tile (rows clamped per lane) works its offsets out
    // again at every use.
    constexpr bool LEAN = MB == 8 && WIN && !GR && IPW == 8;
    constexpr int NXO = LEAN ? 4 : IPW;
    const bool full_tile = row_count == (uint32_t)DBM;
    uint32_t xoff[NXO];
#pragma unroll
    for (int i = 0; i < NXO; i++) xoff[i] = x_offset(i);
    // fragment reads: MFMA step j of lane (fr, fh) takes chunk 4 * fh + j of row fr of slot (bi, kg)
    uint32_t aoff[4];
#pragma unroll
    for (int j = 0; j < 4; j++) aoff[j] = kg * MB * SLOT + (fr * 8 + ((4 * fh + j) ^ ((fr >> 1) & 7u))) * 16;
    // weights: row n0 + 32 * wn + fr, codes [64 * kg + 32 * fh, +32) of the iteration; the last tile of a ragged N
    // works its missing rows on row N - 1 and stores none of their columns
    const uint32_t wrow = min(n0 + wn * 32 + fr, a.N - 1);
    const uint32_t woff = wrow * (a.K * BITS / 8) + (kg * 64 + fh * 32) * BITS / 8;
    const uint32_t kofs_abs = it_base * DBK + kg * 64 + fh * 32;  // k of this lane's codes counted from the start of the row
    const uint32_t ring = (uint32_t)(uintptr_t)lds;

    // LDS after the tiles: [DBN rows][gpr + 2] scales, then the same for biases
    // rows padded by two elements, or (256-row tiles: no room for padding) row r rotated by 8 r elements, so that
    // the 32 rows a wave reads one group of do not all fall into one bank
    constexpr bool ROT = NBUF != 3;
    const uint32_t sbld = ROT ? sb_ng : ((sb_ng + 3u) & ~3u) + 2;   // (a K split stages its own share of the groups only)
    uint16_t* sbS = (uint16_t*)(lds + NBUF * TILE);
    uint16_t* sbB = sbS + DBN * sbld;
    const int sbrow = (int)((wn * 32 + fr) * sbld) - (ROT ? 0 : (int)sb_g0);
    const uint32_t sbrot = ((wn * 32 + fr) * 8) % sbld - sb_g0 + sbld;   // ROT: position of group g is (g + sbrot) mod sbld
    // WIN: windows at the same place; this lane's column inside a window and its swizzle
    const unsigned char* sbW = lds + NBUF * TILE;
    const uint32_t wcol = wn * 32 + fr, wswz = (wcol >> 1) & 3u;
    const uint32_t log2p = a.log2g - 2;        // iterations a window lasts: 32 groups x G codes / 128
    // piece `pid` (256 bytes, LDS order) of window `wi`: where this lane's dword comes from
    auto issue_sb = [&](uint32_t it) {
        if constexpr (WIN) {
            const uint32_t t = (it + 2) & ((1u << log2p) - 1u), wi = ((it + 2) >> log2p) + 1;
            const uint32_t pid = (t * 8u + wave) & 63u;
            const uint32_t off = pid * 256u + 4u * lane;          // byte inside the window
            const uint32_t isb = off >> 13, rem = off & 8191u, col = rem >> 6, cpos = (rem >> 4) & 3u, dw = (rem >> 2) & 3u;
            const uint32_t c = cpos ^ ((col >> 1) & 3u);
            // two groups per dword; past the row's last group the load is clamped onto it (those positions are never read)
            const uint32_t grp = min(wi * 32u + c * 8u + dw * 2u, a.gpr - 2u);
            const uint32_t voff = (min(n0 + col, a.N - 1) * a.gpr + grp) * 2u;
            qm_load_to_lds_b32(ring + NBUF * TILE + (wi & 1u) * 16384u + pid * 256u, voff, isb ? a.biases : a.scales);
        }
    };

    auto issue_x = [&](uint32_t it, int buf) {
        const unsigned char* src = a.x + (size_t)min(it, ilast) * (DBK * 2);
#pragma unroll
        for (int i = 0; i < NXO; i++) qm_load_to_lds(ring + buf * TILE + (wave * IPW + i) * 1024, xoff[i], src);
        if constexpr (LEAN) {
            if (full_tile) {
#pragma unroll
                for (int i = 0; i < 4; i++) qm_load_to_lds(ring + buf * TILE + (wave * IPW + 4 + i) * 1024, xoff[i], src + (size_t)32 * a.K * 2);
            } else {
#pragma unroll
                for (int i = 4; i < 8; i++) qm_load_to_lds(ring + buf * TILE + (wave * IPW + i) * 1024, x_offset(i), src);
            }
        }
    };
    qm_u32x4 raw[WSN][NWL];
    auto issue_w = [&](uint32_t it, int set) {
        const unsigned char* src = a.w + (size_t)min(it, ilast) * (DBK * BITS / 8);
        qm_load_regs(raw[set][0], woff, src);
        if constexpr (NWL == 2) qm_load_regs(raw[set][1], woff, src + 16);
    };
    // waits until at most N loads are outstanding and ties a weight set to the wait
    auto wait_w = [&](auto n_c, int set) {
        constexpr int N = decltype(n_c)::value;
        if constexpr (NWL == 2) qm_wait_vm_for2<N>(raw[set][0], raw[set][NWL - 1]);
        else qm_wait_vm_for<N>(raw[set][0]);
    };
    // half fragment hf (4 codes) of weight set `set` -> two dwords of elements
    uint32_t ek = 0, ok = 0;
    auto convert_half = [&](int set, int hf, float sc, float bi, uint32_t& d0, uint32_t& d1) {
        if constexpr (BITS == 4) {
            const int jj = hf / 2, half = hf % 2;
            if (half == 0) {
                ek = raw[set][0][jj] & 0x0F0F0F0Fu;
                ok = (raw[set][0][jj] >> 4) & 0x0F0F0F0Fu;
            }
            qm_dequant4_b4<DT>(ek, ok, half, sc, bi, d0, d1);
        } else {
            const uint32_t w8 = raw[set][hf / 4][hf % 4];
            d0 = pack2<DT>(fmaf((float)(w8 & 0xFFu), sc, bi), fmaf((float)((w8 >> 8) & 0xFFu), sc, bi));
            d1 = pack2<DT>(fmaf((float)((w8 >> 16) & 0xFFu), sc, bi), fmaf((float)(w8 >> 24), sc, bi));
        }
    };
    // 512 * scale and bias of this lane's codes in iteration it (zero past the end: such an iteration adds nothing)
    auto scale_bias = [&](uint32_t it, float& s512, float& b) {
        int g = (int)((min(it, ilast) * DBK + kofs_abs) >> a.log2g);
        if constexpr (WIN) {
            const uint32_t gl = (uint32_t)g & 31u;
            const unsigned char* p = sbW + (((uint32_t)g >> 5) & 1u) * 16384u + wcol * 64u + (((gl >> 3) ^ wswz) << 4) + ((gl & 7u) << 1);
            s512 = elem_bits_to_f32<DT>(*(const uint16_t*)p) * KSCALE;
            b = elem_bits_to_f32<DT>(*(const uint16_t*)(p + 8192));
            if (it > ilast) s512 = b = 0.f;
            return;
        }
        if constexpr (ROT) {
            g += sbrot;                      // in [sbld, 3 sbld)
            if (g >= 2 * (int)sbld) g -= sbld;
            g -= sbld;
        }
        s512 = elem_bits_to_f32<DT>(sbS[sbrow + g]) * KSCALE;
        b = elem_bits_to_f32<DT>(sbB[sbrow + g]);
        if (it > ilast) s512 = b = 0.f;
    };

    f32x16 acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0.f;

    // ---- prologue ------------------------------------------------------------------------------------
    // issue order of the loop: iteration it issues W(it + 3), then X(it + 2) x IPW; the iterations before the
    // first issue W(0), W(1) | W(2), X(0) | W(3)... : here W(0), W(1), W(2), X(0), then (as iteration -1) X(1)
    qm_static_for<0, WSN>([&](auto i_c) { issue_w(decltype(i_c)::value, decltype(i_c)::value); });
    qm_static_for<0, NBUF - 1>([&](auto i_c) { issue_x(decltype(i_c)::value, decltype(i_c)::value); });
    if constexpr (WIN) {
        // windows 0 and 1, a dword (two groups) per load: 2 windows x (scales, biases) x 128 columns x 16 dwords; rows
        // need not be whole 8-group vectors (K / G even is enough), loads past a row's end are clamped onto its last dword
        for (uint32_t v = tid; v < 8192u; v += NT) {
            const uint32_t win = v >> 12, isb = (v >> 11) & 1u, col = (v >> 4) & 127u, c = (v >> 2) & 3u, dw = v & 3u;
            const uint32_t grp = min(win * 32u + c * 8u + dw * 2u, a.gpr - 2u);
            const uint32_t val = *(const uint32_t*)((const uint16_t*)(isb ? a.biases : a.scales) + (size_t)min(n0 + col, a.N - 1) * a.gpr + grp);
            *(uint32_t*)(lds + NBUF * TILE + win * 16384u + isb * 8192u + col * 64u + ((c ^ ((col >> 1) & 3u)) << 4) + dw * 4u) = val;
        }
    } else if (!ROT && (a.gpr & 7u)) {
        // rows of scales that are not whole 16-byte vectors: a dword (two groups) per load
        const uint32_t dpr = sb_ng / 2, ndw = DBN * dpr;
        for (uint32_t v = tid; v < ndw; v += NT) {
            const uint32_t row = v / dpr, c0 = (v - row * dpr) * 2;
            const uint32_t grow = min(n0 + row, a.N - 1);
            *(uint32_t*)(sbS + row * sbld + c0) = *(const uint32_t*)((const uint16_t*)a.scales + (size_t)grow * a.gpr + sb_g0 + c0);
            *(uint32_t*)(sbB + row * sbld + c0) = *(const uint32_t*)((const uint16_t*)a.biases + (size_t)grow * a.gpr + sb_g0 + c0);
        }
    } else {
        // DBN rows x sb_ng elements each of scales and biases, 16 bytes per load (ordinary loads: the compiler waits).
        // Two vectors of each per thread are loaded before the first is stored: the usual tile (128 columns x 64 groups on
        // 512 threads) is then one trip to memory behind the weight and activation loads above, not two in a row.
        const uint32_t vpr = sb_ng / 8, nvec = DBN * vpr;
        for (uint32_t v0 = 0; v0 < nvec; v0 += 2 * NT) {
            q_u32x4 sv[2], bv[2];
            uint32_t row[2], c0[2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const uint32_t v = min(v0 + u * NT + tid, nvec - 1);
                row[u] = v / vpr;
                c0[u] = (v - row[u] * vpr) * 8;
                const uint32_t grow = min(n0 + row[u], a.N - 1);
                sv[u] = *(const q_u32x4*)((const uint16_t*)a.scales + (size_t)grow * a.gpr + sb_g0 + c0[u]);
                bv[u] = *(const q_u32x4*)((const uint16_t*)a.biases + (size_t)grow * a.gpr + sb_g0 + c0[u]);
            }
#pragma unroll
            for (int u = 0; u < 2; u++) {
                if (v0 + u * NT + tid >= nvec) continue;
                const uint32_t cpos = ROT ? (c0[u] + row[u] * 8) % sbld : c0[u];   // whole 8-element vectors move together
                uint32_t* ds = (uint32_t*)(sbS + row[u] * sbld + cpos);
                uint32_t* db = (uint32_t*)(sbB + row[u] * sbld + cpos);
                ds[0] = sv[u].x; ds[1] = sv[u].y; ds[2] = sv[u].z; ds[3] = sv[u].w;
                db[0] = bv[u].x; db[1] = bv[u].y; db[2] = bv[u].z; db[3] = bv[u].w;
            }
        }
    }
    qm_wait_vm<Waits::first>();   // everything but X(1)..: the first tile's share and the first weight sets
    __syncthreads();      // tile 0 and the scales are in LDS
    uint32_t bq[2][4][4];  // converted fragments: [iteration parity][MFMA step][dword]
    float sn, bn;          // 512 * scale and bias of the iteration being converted (the next one)
    {
        wait_w(std::integral_constant<int, Waits::first>{}, 0);
        float s0, b0;
        scale_bias(0, s0, b0);
#pragma unroll
        for (int hf = 0; hf < 8; hf++) convert_half(0, hf, s0, b0, bq[0][hf / 2][2 * (hf % 2)], bq[0][hf / 2][2 * (hf % 2) + 1]);
        scale_bias(1, sn, bn);
    }
    qm_u32x4 af[2][4];  // activation fragments of one 32-row block: [row block parity][MFMA step]
#pragma unroll
    for (int j = 0; j < 4; j++) af[0][j] = *(const qm_u32x4*)(lds + aoff[j]);

    const uint32_t iters_up = (a.iters + UN - 1) / UN * UN;
    for (uint32_t it0 = 0; it0 < iters_up; it0 += UN) {
        qm_static_for<0, UN>([&](auto u_c) {
            constexpr int u = decltype(u_c)::value;
            constexpr int cur = u & 1, nxt = cur ^ 1;
            constexpr int buf = u % NBUF;
            const uint32_t it = it0 + u;
            if (it >= a.iters) return;   // (uniform) the unrolled run reaches past the last iteration
            // loads: this wave's share of the tile two iterations ahead into the buffer read during the last iteration,
            // weights three iterations ahead into the set whose weights have been converted
            if constexpr (NBUF == 2) {
                // ring of two: (window piece,) the next tile into the buffer read during the last iteration, then the weights
                issue_sb(it);
                issue_x(it + 1, (u + 1) % NBUF);
                issue_w(it + WSN, u % WSN);
            } else {
                issue_w(it + WSN, u % WSN);
                issue_sb(it);
                issue_x(it + NBUF - 1, (u + NBUF - 1) % NBUF);
            }
            float sn2, bn2;
            // weights of the next iteration, issued WSN - 1 iterations ago: the loads younger than they are the tiles
            // of WSN iterations and the weights of WSN - 1 (ring of two: tiles and weights of two iterations)
            wait_w(std::integral_constant<int, Waits::next_weights>{}, (u + 1) % WSN);
            qm_static_for<0, MB>([&](auto bi_c) {
                constexpr int bi = decltype(bi_c)::value;
                constexpr int par = bi & 1;
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[par][0]), "+v"(af[par][1]), "+v"(af[par][2]), "+v"(af[par][3])::"memory");
                if (bi + 1 < MB) {
#pragma unroll
                    for (int j = 0; j < 4; j++) af[par ^ 1][j] = *(const qm_u32x4*)(lds + buf * TILE + (bi + 1) * SLOT + aoff[j]);
                }
                if (bi == 0) scale_bias(it + 2, sn2, bn2);
                __builtin_amdgcn_sched_barrier(0);
                qm_static_for<0, 4>([&](auto j_c) {
                    constexpr int j = decltype(j_c)::value;
                    constexpr int m = bi * 4 + j;   // MFMA of the iteration
                    const uint4 bv = make_uint4(bq[cur][j][0], bq[cur][j][1], bq[cur][j][2], bq[cur][j][3]);
                    const uint4 av = make_uint4(af[par][j].x, af[par][j].y, af[par][j].z, af[par][j].w);
                    acc[bi] = mfma32<DT>(av, bv, acc[bi]);
                    // its share of the next iteration's conversion: half fragments [8 m / NM, 8 (m + 1) / NM)
#pragma unroll
                    for (int hf = 8 * m / NM; hf < 8 * (m + 1) / NM; hf++)
                        convert_half((u + 1) % WSN, hf, sn, bn, bq[nxt][hf / 2][2 * (hf % 2)], bq[nxt][hf / 2][2 * (hf % 2) + 1]);
                });
                __builtin_amdgcn_sched_barrier(0);
            });
            sn = sn2;
            bn = bn2;
            // this wave's share of the next tile (issued one iteration ago) is in LDS once at most this iteration's
            // loads are outstanding; past the barrier every wave's share is
            // (one less than the steady state allows: the first iterations follow the prologue's order)
            qm_wait_vm<Waits::next_tile>();
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 4; j++) af[0][j] = *(const qm_u32x4*)(lds + ((u + 1) % NBUF) * TILE + aoff[j]);
        });
    }
    qm_wait_vm<0>();   // loads still in flight write into the ring the epilogue is about to reuse
    // (The last weight loads are issued for iterations that do not exist and nothing reads them: to the compiler their
    // registers are free from the loop's end on, and a value put there ahead of the wait would be overwritten when the
    // load lands. Naming the registers behind the wait keeps them taken until then.)
#pragma unroll
    for (int ws = 0; ws < WSN; ws++)
#pragma unroll
        for (int k = 0; k < NWL; k++) asm volatile("" ::"v"(raw[ws][k]));
    __syncthreads();

    // ---- the K-groups add their accumulators through LDS, at most 128 rows at a time ------------------------------
    // A wave's accumulators of a round are U = 4 EPB units of four registers (unit u = row block u / 4, rows
    // 8 (u % 4) + 4 (lane / 32) + 0 .. 3 of it, column lane % 32). Unit u is summed by K-group u % KG: every other
    // K-group hands it over with one 16-byte LDS store, the owner adds the KG values in K-group order (its own in its
    // place: the sum is ((k0 + k1) + k2) + k3 whoever owns it), rounds and writes the four elements into the tile of
    // rows that leaves in whole 16-byte pieces. All eight waves share the adding, rounding and LDS traffic, and the
    // partial sums move 16 bytes per instruction.
    constexpr int EPB = MB == 8 ? 4 : MB;       // row blocks per round
    constexpr int GRP = NWV * EPB * 16 * 64;    // floats per handing-over K-group and round
    constexpr int U = 4 * EPB;
    typedef float qm_f32x4 __attribute__((ext_vector_type(4)));
    qm_f32x4* red4 = (qm_f32x4*)lds;            // [KG - 1 senders][wn][U][lane]
    uint16_t* otile = (uint16_t*)(lds + (KG - 1) * GRP * 4);   // the round's rows as [row][DBN columns], behind the partial sums
    qm_static_for<0, MB / EPB>([&](auto ph_c) {
        constexpr int ph = decltype(ph_c)::value;
        if constexpr (ph > 0) __syncthreads();   // the last round's tile has been stored
        qm_static_for<0, U>([&](auto u_c) {
            constexpr int u = decltype(u_c)::value;
            constexpr int owner = u % KG, bi = ph * EPB + u / 4, v0 = 4 * (u % 4);
            if (kg != (uint32_t)owner) {         // (uniform per wave)
                const uint32_t slot = kg < (uint32_t)owner ? kg : kg - 1u;
                const qm_f32x4 t = {acc[bi][v0], acc[bi][v0 + 1], acc[bi][v0 + 2], acc[bi][v0 + 3]};
                red4[((slot * NWV + wn) * U + u) * 64 + lane] = t;
            }
        });
        __syncthreads();
        // accumulator layout: column j = lane%32, row i = 8*(v/4) + 4*(lane/32) + v%4
        qm_static_for<0, U>([&](auto u_c) {
            constexpr int u = decltype(u_c)::value;
            constexpr int owner = u % KG, bl = u / 4, bi = ph * EPB + bl, v0 = 4 * (u % 4);
            if (kg == (uint32_t)owner) {
                qm_f32x4 r = {0.f, 0.f, 0.f, 0.f};
                qm_static_for<0, KG>([&](auto j_c) {
                    constexpr int j = decltype(j_c)::value;
                    qm_f32x4 val;
                    if constexpr (j == owner) val = qm_f32x4{acc[bi][v0], acc[bi][v0 + 1], acc[bi][v0 + 2], acc[bi][v0 + 3]};
                    else val = red4[(((j < owner ? j : j - 1) * NWV + wn) * U + u) * 64 + lane];
                    if constexpr (j == 0) r = val;
                    else r = r + val;
                });
#pragma unroll
                for (int vv = 0; vv < 4; vv++) {
                    const uint32_t trow = bl * 32 + 8 * (u % 4) + 4 * fh + vv, lrow = ph * EPB * 32 + trow;
                    if constexpr (SP) {  // this split's f32 partial sums, 32 consecutive columns per half wave
                        const uint32_t col = n0 + wn * 32 + fr;
                        if (lrow < row_count && col < a.N) a.part[((size_t)blockIdx.y * a.M + row_first + lrow) * a.N + col] = r[vv];
                    } else {
                        otile[trow * DBN + wn * 32 + fr] = f32_to_elem_bits<DT>(r[vv]);
                    }
                }
            }
        });
        if constexpr (!SP) {  // split instances end with the partial sums: the second kernel rounds and stores
            __syncthreads();
            // all threads store the rows, 16 bytes each, whole rows
            constexpr int VPR = DBN / 8;                         // 16-byte vectors per tile row
            constexpr int VPT = (EPB * 32 * VPR + NT - 1) / NT;  // vectors per thread
            if ((a.N & 7u) == 0) {
#pragma unroll
                for (int i = 0; i < VPT; i++) {
                    const uint32_t v = tid + i * NT, trow = v / VPR, lrow = ph * EPB * 32 + trow, col = n0 + (v % VPR) * 8;
                    if (trow < (uint32_t)(EPB * 32) && lrow < row_count && col < a.N)
                        *(q_u32x4*)((uint16_t*)a.out + (size_t)row_of(lrow) * a.N + col) = *(const q_u32x4*)(otile + trow * DBN + (v % VPR) * 8);
                }
            } else {
                for (uint32_t e = tid; e < (uint32_t)(EPB * 32 * DBN); e += NT) {
                    const uint32_t trow = e / DBN, lrow = ph * EPB * 32 + trow, col = n0 + e % DBN;
                    if (lrow < row_count && col < a.N) ((uint16_t*)a.out)[(size_t)row_of(lrow) * a.N + col] = otile[e];
                }
            }
        }
    });
}

}  // namespace mtq
