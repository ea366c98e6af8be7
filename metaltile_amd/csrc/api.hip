// C-ABI of libmtq_hip.so (declared in include/mtq.h): device lifetime, buffers,
// typed entry points, the reference's name-keyed dispatch and its measurement
// loop. There is deliberately no CPU path in this file: without a GPU every
// entry point fails with MTQ_ERR_NO_DEVICE.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <cxxabi.h>
#include <dlfcn.h>
#include <time.h>

#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/mtq.h"
#include "../../include/mtq_measure.h"
#include "mtq_internal.h"

namespace mtq {

static thread_local std::string g_err;

int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    g_err = std::string(what) + ": " + hipGetErrorString(e);
    // clear the sticky "last error" so an unrelated later call does not report it
    (void)hipGetLastError();
    return e == hipErrorNoDevice || e == hipErrorInvalidDevice ? ERR_NO_DEVICE : ERR_HIP;
}

// What mtq_plan records instead of launching.
struct PlanRecorder {
    bool on = false;
    int n = 0;                 // launches seen (may exceed the slots of the caller's struct)
    size_t scratch = 0;        // most library-owned scratch any step asked for
    mtq_plan_info* out = nullptr;
};
static PlanRecorder g_plan;
bool planning() { return g_plan.on; }
void plan_note_scratch(size_t bytes) {
    if (bytes > g_plan.scratch) g_plan.scratch = bytes;
}

hipError_t set_max_dynamic_lds(const void* fn, size_t bytes) {
    if (g_plan.on) return hipSuccess;
    return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// Name of a kernel from the address of its host-side stub, without asking the runtime (which needs a device).
static void kernel_name_of(const void* fn, char* out, size_t cap) {
    Dl_info di;
    if (dladdr(fn, &di) && di.dli_sname) {
        int st = 0;
        char* dm = abi::__cxa_demangle(di.dli_sname, nullptr, nullptr, &st);
        std::string s = st == 0 && dm ? dm : di.dli_sname;
        free(dm);
        const std::string stub = "__device_stub__";
        const size_t k = s.find(stub);
        if (k != std::string::npos) s.erase(k, stub.size());
        snprintf(out, cap, "%s", s.c_str());
    } else {
        snprintf(out, cap, "kernel@%p", fn);
    }
}

hipError_t launch_kernel(const void* fn, dim3 grid, dim3 block, void** args, size_t shmem,
                         const LaunchCtx& lc) {
    if (g_plan.on) {
        if (g_plan.out && g_plan.n < MTQ_PLAN_MAX_LAUNCHES) {
            mtq_plan_launch& l = g_plan.out->launch[g_plan.n];
            kernel_name_of(fn, l.kernel, sizeof(l.kernel));
            l.grid[0] = grid.x; l.grid[1] = grid.y; l.grid[2] = grid.z;
            l.block[0] = block.x; l.block[1] = block.y; l.block[2] = block.z;
            l.lds_bytes = shmem;
        }
        g_plan.n++;
        return hipSuccess;
    }
    if (lc.start || lc.stop)
        return hipExtLaunchKernel(fn, grid, block, args, shmem, lc.stream, lc.start, lc.stop, 0);
    return hipLaunchKernel(fn, grid, block, args, shmem, lc.stream);
}

Options& options() {
    static Options o;
    return o;
}

struct State {
    bool ready = false;
    int device = -1;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;  // stream in use (own_stream or the caller's)
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    void* flush_buf = nullptr;
    void* scratch_buf = nullptr;     // library-owned scratch: normalised rows, qvm partial sums
    size_t scratch_bytes = 0;
    size_t scratch_held = 0;         // bytes at the front of scratch_buf that the running op keeps for itself
    size_t flush_bytes = 0;
    uint64_t* probe_buf = nullptr;   // four u64 written by the clock probe
    hipDeviceProp_t prop;
    bool timed_armed = false;    // next typed launch attaches the events
    bool timed_pending = false;  // events attached, not yet read
};
static State g;

// Scratch of mtq_qvm_noalloc: part of the code object, so it exists on every GPU the library is
// loaded on without any allocation call. `noalloc_scratch` names the array for the host only as a
// symbol; its address on a device comes from hipGetSymbolAddress (looked up once per device in
// mtq_init) and that address is what the launches are given.
static constexpr size_t kNoallocScratchBytes = (size_t)4 << 20;
static __device__ __align__(256) unsigned char noalloc_scratch[kNoallocScratchBytes];
static constexpr int kMaxDevices = 64;
static void* g_noalloc_ptr[kMaxDevices] = {};

static int need_ready() {
    if (!g.ready) return fail(ERR_NO_DEVICE, "mtq_init has not succeeded (no usable GPU?)");
    return ERR_OK;
}

static LaunchCtx make_ctx() {
    LaunchCtx lc;
    lc.stream = g.stream;
    if (g.timed_armed) {
        lc.start = g.ev_start;
        lc.stop = g.ev_stop;
        g.timed_armed = false;
        g.timed_pending = true;
    }
    return lc;
}

__global__ __launch_bounds__(256) void flush_kernel(uint4* p, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint4 v = p[i];
        v.x += 1u;
        p[i] = v;
    }
}

// One wave, a chain of dependent adds between two readings of the constant-rate counter: the chain issues one add per
// four shader clocks whatever else the chip does, so its length on the constant-rate counter gives the shader clock.
#define MTQ_ADD16 "v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n" \
                  "v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n" \
                  "v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n" \
                  "v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n v_add_u32 %0, %0, %0\n"
static constexpr uint32_t kProbeAddsPerTurn = 512;
__global__ __launch_bounds__(64) void clock_probe_kernel(uint64_t* out, uint32_t turns) {
    uint32_t v = threadIdx.x | 1u;
    const uint64_t r0 = wall_clock64();
    const uint64_t c0 = clock64();
    for (uint32_t i = 0; i < turns; i++) {
        asm volatile(MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16
                     MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16
                     MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16
                     MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16 MTQ_ADD16
                     : "+v"(v));
    }
    const uint64_t c1 = clock64();
    const uint64_t r1 = wall_clock64();
    if (threadIdx.x == 0) {
        out[0] = r1 - r0;
        out[1] = c1 - c0;
        out[2] = (uint64_t)turns * kProbeAddsPerTurn;
        out[3] = v;
    }
}
#undef MTQ_ADD16

// Reads n 16-byte vectors and keeps nothing: the rate at which a launch of this size can pull bytes out of HBM
// at all, the ceiling of every weight-streaming kernel of the same size. B loads in flight per thread.
template <bool NT, int B> __global__ __launch_bounds__(256) void read_kernel(const uint4* __restrict__ src, size_t n, uint32_t* sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    auto ld = [&](size_t j) -> uint4 {
        if constexpr (NT) {
            typedef uint32_t u4v __attribute__((ext_vector_type(4)));
            const u4v v = __builtin_nontemporal_load((const u4v*)src + j);
            return make_uint4(v.x, v.y, v.z, v.w);
        } else {
            return src[j];
        }
    };
    // batches of up to B loads, all issued before the first is used; none past the end
    for (; i < n; i += B * stride) {
        uint4 v[B];
#pragma unroll
        for (int u = 0; u < B; u++) {
            v[u] = make_uint4(0, 0, 0, 0);
            if (i + u * stride < n) v[u] = ld(i + u * stride);
        }
#pragma unroll
        for (int u = 0; u < B; u++) { acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
    }
    // a store the compiler cannot rule out and that in practice never happens
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u && (acc.x + acc.y) == 0x7F4A7C15u) *sink = acc.z;
}

__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

// ---------------------------------------------------------------------------
// typed ops (shared by the C entry points and the name-keyed dispatch)
// ---------------------------------------------------------------------------

static size_t esize(int dt) { return dt == DT_F32 ? 4 : 2; }

static int check_common(int dtype, int bits, uint32_t G, uint32_t N, uint32_t K) {
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    if (bits < 2 || bits > 8) return fail(ERR_BAD_ARG, "bits must be in 2..8");
    if (N == 0 || K == 0) return fail(ERR_SHAPE, "N and K must be non-zero");
    if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must be non-zero and divide K");
    if ((uint64_t)K * bits % 32) return fail(ERR_SHAPE, "K*bits must be a multiple of 32");
    return ERR_OK;
}

static int run_gemv(const QmvParams& p, const LaunchCtx& lc) {
    int rc = launch_qmv_fast(p, lc);
    if (rc == ERR_UNSUPPORTED) rc = launch_qmv_generic(p, lc);
    return rc;
}

static int ensure_scratch(size_t need);

// f32 batches: the f32 matrix-core kernel works 32 activation rows per pass over the weights, the
// f32 dot kernels 4. Measured at 4096 x 4096 (tiles with K split over workgroups): 4-bit, 4 rows 16.6 us
// on the dot kernels against 16, 8 rows 33.6 against 16.4, 32 rows 133 against 24; 3-bit (5-, 6-, 7-bit
// alike: no f32 dot kernel, so every row count goes to the tiles), 1 row 25-35 against 15.4, 32 rows 534
// against 24. Returns ERR_UNSUPPORTED when the rows stay with the GEMV family.
static int try_f32_tiles(int bits, uint32_t G, const void* w, const void* s, const void* b, const void* x, void* out,
                         uint32_t M, uint32_t N, uint32_t K, const LaunchCtx& lc) {
    const int opt = options().qmm_f32_tiles;
    const bool odd = bits == 3 || bits == 5 || bits == 6 || bits == 7;
    if (opt == 1 || (opt == 0 && !odd && M < 5u)) return ERR_UNSUPPORTED;
    QmmParams q;
    q.dtype = DT_F32; q.bits = bits; q.group_size = G;
    q.w = w; q.scales = s; q.biases = b; q.x = x; q.out = out;
    q.M = M; q.N = N; q.K = K;
    const size_t need = qmm_f32_scratch_bytes(q);  // f32 partial tiles when K is split
    if (need) {
        // behind whatever the calling op holds at the front of the buffer (a normalised row)
        int rc = ensure_scratch(g.scratch_held + need);
        if (rc) return rc;
    }
    return launch_qmm_f32(q, lc, need ? (char*)g.scratch_buf + g.scratch_held : nullptr);
}


// Batches of 5..16 rows on the 16-row matrix-core GEMV where the shape allows and it is the fastest kernel;
// ERR_UNSUPPORTED otherwise. `exact`: the caller's alternative is the GEMV family (passes of up to 8 rows, the
// same exact-dequant arithmetic); else it is the tile kernel.
static int try_wide(int dtype, int bits, uint32_t G, const void* w, const void* s, const void* b, const void* x,
                    void* out, uint32_t M, uint32_t N, uint32_t K, bool exact, const LaunchCtx& lc) {
    if (M < 5 || M > 16 || options().qmv_wide == 1) return ERR_UNSUPPORTED;
    QmmParams q;
    q.dtype = dtype; q.bits = bits; q.group_size = G;
    q.w = w; q.scales = s; q.biases = b; q.x = x; q.out = out;
    q.M = M; q.N = N; q.K = K;
    if (!qmv_wide_takes(q)) return ERR_UNSUPPORTED;
    // Every workgroup stages its 16 rows of activations (128 KB at K = 4096), which pays once a compute unit streams
    // several times that in weights. us, 5 / 8 / 12 / 16 rows, the other kernels (GEMV passes of up to 8 rows | tiles)
    // against this one: 128256 x 4096 69 66 116 131 | 88 89 90 92 -> 54 53 55 55; 57344 x 4096 31 32 56 62 | 42 43 43
    // 44 -> 26 27 28 29; 28672 x 8192 50 52 77 103 | 45 45 45 45 -> 29 30 31 32; 32768 x 4096 21 22 38 43 | 27 27 27 28
    // -> 17.5 18.3 19.5 20.3; 8192 x 8192 19 22 32 42 | 17.4 16.9 17.1 17.4 -> 14.8 15.6 17.2 18.3; 14336 x 4096 13.1 13.6
    // 23 27 | 13.5 13.4 13.6 13.7 -> 12.3 12.9 13.8 14.7; 4096 x 14336 23 25 38 50 | 15.2 15.4 15.9 16.0 -> 14.8 15.1 16.2
    // 17.4; 4096 x 4096 7.6 8.3 10.7 12.6 | 9.4 9.6 9.9 10.1 -> 10.1 10.7 11.4 12.1.
    const uint64_t codes = (uint64_t)N * K;
    const bool pays = M <= 8 ? codes >= 50000000ull : exact ? codes >= (1ull << 25) : codes >= 100000000ull;
    if (options().qmv_wide != 2 && !pays) return ERR_UNSUPPORTED;
    const size_t need = qmv_wide_scratch_bytes(q);
    if (need) {
        int rc = ensure_scratch(g.scratch_held + need);
        if (rc) return rc;
    }
    return launch_qmv_wide(q, lc, need ? (char*)g.scratch_buf + g.scratch_held : nullptr);
}

static int op_qmv(int dtype, int bits, uint32_t G, const void* w, const void* s, const void* b,
                  const void* x, void* out, uint32_t M, uint32_t N, uint32_t K, const LaunchCtx& lc) {
    int rc = check_common(dtype, bits, G, N, K);
    if (rc) return rc;
    if (M == 0) return ERR_OK;
    if (!w || !s || !b || !x || !out) return fail(ERR_BAD_ARG, "null buffer");
    rc = try_wide(dtype, bits, G, w, s, b, x, out, M, N, K, true, lc);
    if (rc != ERR_UNSUPPORTED) return rc;
    if (dtype == DT_F32) {
        rc = try_f32_tiles(bits, G, w, s, b, x, out, M, N, K, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    QmvParams p;
    p.dtype = dtype; p.bits = bits; p.group_size = G;
    p.w = w; p.scales = s; p.biases = b; p.x = x; p.out = out;
    p.M = M; p.N = N; p.K = K;
    return run_gemv(p, lc);
}

// Kernel routing by M, the counterpart of mt_qmm_for
// (crates/metaltile-std/src/mlx/quantized.rs:5040-5065, which sends M = 16 and the multiples
// of 32 to its MMA kernels). Here the GEMV family takes 8 activation rows per pass over the
// weights, so it serves up to 8 rows; from 9 rows the MFMA tile kernel takes over: a second GEMV
// pass always loses to 32-row tiles once short matrices split K over workgroups (16 rows, GEMV
// against tiles: 4096 x 14336 50 / 23 us, 2048 x 8192 21 / 11, 1024 x 4096 24 / 11, 14336 x 4096
// 25 / 15, 128256 x 4096 134 / 98).
static int op_qmm(int dtype, int bits, uint32_t G, const void* w, const void* s, const void* b,
                  const void* x, void* out, uint32_t M, uint32_t N, uint32_t K, bool force_mma,
                  const LaunchCtx& lc) {
    int rc = check_common(dtype, bits, G, N, K);
    if (rc) return rc;
    if (M == 0) return ERR_OK;
    if (!w || !s || !b || !x || !out) return fail(ERR_BAD_ARG, "null buffer");
    if (dtype == DT_F32 && options().qmm_f32_tiles != 1) return op_qmv(dtype, bits, G, w, s, b, x, out, M, N, K, lc);
    // 7-bit codes have no GEMV kernel of their own (the reference has no 7-bit kernels either): any
    // number of rows beats the generic kernel on the tile kernel (4096 x 4096: 1 row 28 -> 17 us, 16 rows 236 -> 17).
    // 5..8 rows: rows too long for 8 of them in LDS make the GEMV take two passes, and short, wide
    // matrices leave it few row blocks; the split-K tiles are ahead there (8 rows, GEMV against tiles:
    // 4096 x 14336 26 / 22 us, 1024 x 4096 14 / 10, 8192 x 28672 107 / 62, 28672 x 8192 56 / 39; but
    // 14336 x 4096 12 / 14, 128256 x 4096 70 / 84).
    if (!force_mma) {
        rc = try_wide(dtype, bits, G, w, s, b, x, out, M, N, K, false, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    const bool long_rows = M >= 5 && ((uint64_t)K >= 2 * (uint64_t)N || (K >= 8192 && (uint64_t)N >= 3 * (uint64_t)K));
    if (M >= 9 || long_rows || force_mma || bits == 7) {
        QmmParams q;
        q.dtype = dtype; q.bits = bits; q.group_size = G;
        q.w = w; q.scales = s; q.biases = b; q.x = x; q.out = out;
        q.M = M; q.N = N; q.K = K;
        if (options().qmm_kernel != 1) {
            const size_t need = qmm_direct_scratch_bytes(q);  // f32 partial tiles when K is split
            if (need) {
                rc = ensure_scratch(g.scratch_held + need);
                if (rc) return rc;
            }
            rc = launch_qmm_direct(q, lc, need ? (char*)g.scratch_buf + g.scratch_held : nullptr);
            if (rc != ERR_UNSUPPORTED) return rc;
        }
        rc = launch_qmm_mfma(q, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    return op_qmv(dtype, bits, G, w, s, b, x, out, M, N, K, lc);
}

// Library-owned device scratch (normalised rows, qvm partial sums): grown on demand, never shrunk.
static int ensure_scratch(size_t need) {
    if (g_plan.on) {  // mtq_plan has put a stand-in address into scratch_buf; nothing is allocated
        plan_note_scratch(need);
        return ERR_OK;
    }
    if (g.scratch_bytes >= need) return ERR_OK;
    if (g.scratch_buf) {
        MTQ_HIP(hipStreamSynchronize(g.stream));  // earlier launches may still use the old buffer
        MTQ_HIP(hipFree(g.scratch_buf));
        g.scratch_buf = nullptr;
        g.scratch_bytes = 0;
    }
    const size_t cap = need < 65536 ? 65536 : need;
    MTQ_HIP(hipMalloc(&g.scratch_buf, cap));
    g.scratch_bytes = cap;
    return ERR_OK;
}

static int op_qvm(int dtype, int bits, uint32_t G, const void* w, const void* s, const void* b, const void* x, void* out,
                  uint32_t M, uint32_t N, uint32_t K, const LaunchCtx& lc) {
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    if (bits < 2 || bits > 8) return fail(ERR_BAD_ARG, "bits must be in 2..8");
    if (N == 0 || K == 0) return fail(ERR_SHAPE, "N and K must be non-zero");
    if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must be non-zero and divide K");
    if ((uint64_t)N * bits % 32) return fail(ERR_SHAPE, "N*bits must be a multiple of 32");
    if (M == 0) return ERR_OK;
    if (!w || !s || !b || !x || !out) return fail(ERR_BAD_ARG, "null buffer");
    int rc = ensure_scratch(qvm_scratch_bytes(bits, G, M, N, K));
    if (rc) return rc;
    QmvParams p;
    p.dtype = dtype; p.bits = bits; p.group_size = G; p.w = w; p.scales = s; p.biases = b; p.x = x; p.out = out;
    p.M = M; p.N = N; p.K = K;
    return launch_qvm(p, g.scratch_buf, lc);
}

// A qmv whose activation row some first launch writes into library-owned scratch: `stage(dst, ctx)` enqueues
// that launch (one row of K for f32; for f16 / bf16 two rows, the rounded values and the rounded remainders, so
// that the row carries 16 significant bits), an ordinary qmv follows, and for two rows the sum of their outputs.
template <class Stage>
static int qmv_of_staged_row(int dtype, int bits, uint32_t G, const void* w, const void* s, const void* b, void* out,
                             uint32_t N, uint32_t K, const LaunchCtx& lc, Stage&& stage) {
    int rc;
    // scratch: the normalised row(s), then for 16-bit types the two partial outputs
    const size_t sz = esize(dtype);
    const uint32_t rows = dtype == DT_F32 ? 1u : 2u;
    const size_t x_bytes = ((size_t)rows * K * sz + 255) & ~(size_t)255;
    const size_t held = (x_bytes + (rows == 2 ? (size_t)2 * N * sz : 0) + 255) & ~(size_t)255;
    // The qmv that follows may itself want scratch (f32 rows on the tile kernel split K into partial
    // tiles): size the buffer for both now, so that it is not reallocated under the normalised row, and
    // let that qmv work behind the held part, so that its partial tiles do not overwrite the row it reads.
    size_t inner = 0;
    if (dtype == DT_F32) {
        QmmParams q;
        q.dtype = dtype; q.bits = bits; q.group_size = G; q.w = w; q.scales = s; q.biases = b; q.x = g.scratch_buf; q.out = out;
        q.M = rows; q.N = N; q.K = K;
        inner = qmm_f32_scratch_bytes(q);
    }
    rc = ensure_scratch(held + inner);
    if (rc) return rc;
    LaunchCtx first = lc, mid = lc, last = lc;
    first.stop = nullptr;
    mid.start = mid.stop = nullptr;
    last.start = nullptr;
    rc = stage(g.scratch_buf, first);
    if (rc) return rc;
    g.scratch_held = held;
    if (rows == 1) {
        rc = op_qmv(dtype, bits, G, w, s, b, g.scratch_buf, out, 1, N, K, last);
        g.scratch_held = 0;
        return rc;
    }
    char* part = (char*)g.scratch_buf + x_bytes;
    rc = op_qmv(dtype, bits, G, w, s, b, g.scratch_buf, part, 2, N, K, mid);
    g.scratch_held = 0;
    if (rc) return rc;
    return launch_add_rows(dtype, part, part + (size_t)N * sz, out, N, last);
}

// RMSNorm fused into qmv: inside the streaming kernel when the row fits it, else the
// row is normalised into a library-owned buffer and an ordinary qmv follows.
static int op_rms_norm_qmv(int dtype, int bits, uint32_t G, const void* x, const void* norm_w, const void* w,
                           const void* s, const void* b, void* out, const float* eps, uint32_t N, uint32_t K,
                           const LaunchCtx& lc) {
    int rc = check_common(dtype, bits, G, N, K);
    if (rc) return rc;
    if (!x || !norm_w || !w || !s || !b || !out || !eps) return fail(ERR_BAD_ARG, "null buffer");
    QmvParams p;
    p.dtype = dtype; p.bits = bits; p.group_size = G; p.w = w; p.scales = s; p.biases = b; p.x = x; p.out = out;
    p.N = N; p.K = K;
    // 4-bit f16 / bf16: the norm applied as the matrix-core GEMV stages its row (two staged rows share one set of 4;
    // no per-workgroup renormalisation beyond the sum of squares). us, streaming kernel -> this: 14336 x 4096 12.6 ->
    // 10.6, 6144 x 4096 8.1 -> 7.3; it loses on short matrices and long rows (4096 x 4096 6.2 -> 6.4, 4096 x 14336 13.7 -> 14.1).
    // Rows of 2048 ... 8192 4-bit codes: the norm applied as the kernel whose waves walk the rows puts the activations into
    // LDS (qmv_rows_walk.hip). bf16, us, the better of the forms below -> this, same run: 1024 / 2048 / 4096 / 6144 / 8192 / 14336 /
    // 28672 x 4096 4.65 -> 4.41, 4.75 -> 4.42, 6.52 -> 4.57, 7.37 -> 5.90, 7.57 -> 6.93, 10.61 -> 8.91, 16.76 -> 15.79; 2048 / 4096 /
    // 6144 / 8192 / 14336 / 20480 / 28672 x 8192 6.81 -> 6.19, 8.73 -> 7.09, 11.01 -> 9.79, 11.73 -> 11.59, 17.17 -> 16.05, 22.28 -> 20.75,
    // 27.51 -> 26.48. On the largest matrices the matrix-core form is level or ahead (65536 x 4096 29.0 / 29.4 - 32.2, 65536 x 8192
    // 52.2 / 52.9 - 54.3). qmv.kernel = 2 keeps the older forms, = 3 takes this one wherever the shape allows.
    // The other row lengths it is built for (2048 / 3072 / 3584 / 5120 / 6144 / 7168 codes; bf16 g64, us, the forms below -> this):
    // 2048 codes, 2048 / 8192 / 16384 / 32768 rows 4.96 -> 4.51, 6.59 -> 5.04, 8.49 -> 6.78, 11.7 -> 10.7; 3072 codes, 512 / 3072 / 8192 /
    // 28672 rows 12.8 -> 4.15, 13.0 -> 4.61, 7.25 -> 6.88, 15.5 -> 13.8; 3584 codes, 1024 / 3584 / 18944 / 37888 rows 14.3 -> 4.26, 13.6 -> 4.73,
    // 14.7 -> 10.9, 20.1 -> 17.5; 5120 codes, 1024 / 5120 / 13824 / 27648 rows 12.4 -> 5.09, 9.56 -> 7.14, 13.9 -> 11.0, 19.6 -> 18.2; 6144
    // codes, 1024 / 6144 / 16384 rows 6.46 -> 5.22, 10.1 -> 7.74, 14.7 -> 14.1; 7168 codes, 2048 / 7168 / 18432 rows 14.2 -> 6.18, 11.0 -> 10.4,
    // 20.5 -> 18.3 (rows that the streaming kernel does not take whole were a norm launch and a GEMV). From 65536 rows the
    // forms below are ahead (65536 x 3584 26.1 / 27.5, 65536 x 7168 47.9 / 56.3, 151936 x 2048 32.6 / 38.9).
    const bool rows_norm = options().qmv_kernel == 3 ||
                           (options().qmv_kernel == 0 && ((K == 4096 || K == 8192) ? N >= (K == 4096 ? 1024u : 2048u) && N <= 32768u
                                                                                     : N >= 512u && N <= 40960u));
    if (options().qmv_norm_mfma != 2 && rows_norm && qmv_rows_norm_takes(p, norm_w)) {
        rc = launch_qmv_rows_norm(p, norm_w, eps, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    const bool norm_on_mfma = options().qmv_norm_mfma == 2 ||
                              (options().qmv_norm_mfma == 0 && K <= 8192 && (uint64_t)N * K >= 24000000ull);
    if (bits == 4 && dtype != DT_F32 && norm_on_mfma) {
        QmvParams pm = p;
        pm.M = 1;
        pm.norm_w = norm_w;
        pm.norm_eps = eps;
        rc = launch_qmv_mfma(pm, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    rc = launch_qmv_norm(p, norm_w, eps, lc);
    if (rc != ERR_UNSUPPORTED) return rc;
    return qmv_of_staged_row(dtype, bits, G, w, s, b, out, N, K, lc, [&](void* dst, const LaunchCtx& ctx) {
        return launch_rms_norm(dtype, x, norm_w, eps, dst, K, ctx);
    });
}

// Gated RMSNorm + 4-bit qmv (crates/metaltile-std/src/ffai/gated_rms_norm_qgemv.rs:88-291): the gated, normalised
// rows of y (hv rows of dv, flat: the GEMV's activation of hv * dv) are written into library-owned scratch, an
// ordinary qmv follows. The reference stages that activation in f32 and never rounds it to the element type;
// the two-row form of the staged qmv keeps 16 significant bits of it for f16 / bf16.
static int op_gated_rms_norm_qmv(int dtype, uint32_t G, const float* y, const void* z, const void* norm_w, const float* eps,
                                 const void* w, const void* s, const void* b, void* out, uint32_t hv, uint32_t dv, uint32_t N,
                                 const LaunchCtx& lc) {
    if (hv == 0 || dv == 0) return fail(ERR_SHAPE, "hv and dv must be non-zero");
    if ((uint64_t)hv * dv > 0xFFFFFFFFull) return fail(ERR_SHAPE, "hv * dv must fit 32 bits");
    const uint32_t K = hv * dv;
    int rc = check_common(dtype, 4, G, N, K);
    if (rc) return rc;
    if (!y || !z || !norm_w || !eps || !w || !s || !b || !out) return fail(ERR_BAD_ARG, "null buffer");
    // One launch: the streaming kernel gates and normalises the slice each thread holds. us per call, staged (three
    // launches; two for f32) -> one launch, dv 128: bf16 hv 16, 2048 rows 7.7 -> 5.1 (the plain qmv of that matrix: 3.3);
    // hv 32, 1024 rows 10.3 -> 5.7; hv 32, 4096 rows 9.3 -> 8.0; hv 64, 8192 rows 14.8 -> 14.5. f32 stays staged (6.3 -> 6.9,
    // 7.9 -> 11.5, 16.3 -> 19.3): its one-row streaming kernel is the slower one to begin with.
    if (options().qmv_gated_fused == 2 || (options().qmv_gated_fused == 0 && dtype != DT_F32)) {
        QmvParams p;
        p.dtype = dtype; p.bits = 4; p.group_size = G; p.w = w; p.scales = s; p.biases = b; p.x = y; p.out = out;
        p.N = N; p.K = K;
        rc = launch_qmv_gated_norm(p, z, norm_w, eps, dv, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    return qmv_of_staged_row(dtype, 4, G, w, s, b, out, N, K, lc, [&](void* dst, const LaunchCtx& ctx) {
        return launch_gated_rms_norm(dtype, y, z, norm_w, eps, dst, hv, dv, ctx);
    });
}

// Fused projections: one launch when the shape fits the streaming kernel, else one qmv per matrix.
static int op_qmv_batched(int dtype, int bits, uint32_t G, int n, const void* const* w, const void* const* s,
                          const void* const* b, const void* x, void* const* outs, const uint32_t* N, uint32_t K,
                          const LaunchCtx& lc) {
    if (n < 1 || n > 4 || !w || !s || !b || !outs || !N || !x) return fail(ERR_BAD_ARG, "batched qmv: 1..4 matrices, non-null arrays");
    for (int j = 0; j < n; j++) {
        int rc = check_common(dtype, bits, G, N[j], K);
        if (rc) return rc;
        if (!w[j] || !s[j] || !b[j] || !outs[j]) return fail(ERR_BAD_ARG, "null buffer");
    }
    if (n >= 2) {
        QmvParams p;
        p.dtype = dtype; p.bits = bits; p.group_size = G; p.x = x; p.K = K;
        QmvBatch qb;
        qb.n = n;
        for (int j = 0; j < n; j++) { qb.w[j] = w[j]; qb.scales[j] = s[j]; qb.biases[j] = b[j]; qb.out[j] = outs[j]; qb.N[j] = N[j]; }
        int rc = launch_qmv_batched(p, qb, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    for (int j = 0; j < n; j++) {
        LaunchCtx l2 = lc;
        if (j) l2.start = nullptr;
        if (j + 1 < n) l2.stop = nullptr;
        int rc = op_qmv(dtype, bits, G, w[j], s[j], b[j], x, outs[j], 1, N[j], K, l2);
        if (rc) return rc;
    }
    return ERR_OK;
}

// Several weight matrices against the same M activation rows (the prefill siblings of the batched GEMV,
// crates/metaltile-std/src/ffai/batched_qkv_qmm.rs:49-68, batched_4_qmm.rs:61-85): row m of every output is the
// GEMV of activation row m. One qmm per matrix, in order on the caller's stream; at prefill sizes a launch is
// long against its fixed cost, so one grid over all the matrices would buy nothing.
static int op_qmm_batched(int dtype, int bits, uint32_t G, int n, const void* const* w, const void* const* s,
                          const void* const* b, const void* x, void* const* outs, const uint32_t* N, uint32_t M, uint32_t K,
                          bool exact, const LaunchCtx& lc) {
    if (n < 1 || n > 4 || !w || !s || !b || !outs || !N) return fail(ERR_BAD_ARG, "batched qmm: 1..4 matrices, non-null arrays");
    for (int j = 0; j < n; j++) {
        int rc = check_common(dtype, bits, G, N[j], K);
        if (rc) return rc;
    }
    if (M == 0) return ERR_OK;
    if (!x) return fail(ERR_BAD_ARG, "null buffer");
    for (int j = 0; j < n; j++)
        if (!w[j] || !s[j] || !b[j] || !outs[j]) return fail(ERR_BAD_ARG, "null buffer");
    for (int j = 0; j < n; j++) {
        LaunchCtx l2 = lc;
        if (j) l2.start = nullptr;
        if (j + 1 < n) l2.stop = nullptr;
        // exact: the caller named a reference kernel, whose rows are GEMVs on the exact f32 s*q + b (as mt_qmm's are):
        // the GEMV family at every M; else mtq_qmm's routing, which takes batches to the tiles and their rounded weights
        int rc = exact ? op_qmv(dtype, bits, G, w[j], s[j], b[j], x, outs[j], M, N[j], K, l2)
                       : op_qmm(dtype, bits, G, w[j], s[j], b[j], x, outs[j], M, N[j], K, false, l2);
        if (rc) return rc;
    }
    return ERR_OK;
}

static int op_gather(int mode, int dtype, int bits, uint32_t G, const void* x, const void* w,
                     const void* s, const void* b, const uint32_t* route, void* out, uint32_t T,
                     uint32_t N, uint32_t K, uint32_t E, const LaunchCtx& lc, bool exact_only = false) {
    int rc = check_common(dtype, bits, G, N, K);
    if (rc) return rc;
    if (E == 0) return fail(ERR_SHAPE, "n_experts must be non-zero");
    if (mode != GATHER_SINGLE && T == 0) return ERR_OK;
    if (!w || !s || !b || !x || !out || !route) return fail(ERR_BAD_ARG, "null buffer");
    QmvParams p;
    p.dtype = dtype; p.bits = bits; p.group_size = G;
    p.w = w; p.scales = s; p.biases = b; p.x = x; p.out = out;
    p.M = 1; p.N = N; p.K = K;
    p.gather = mode; p.route = route; p.T = mode == GATHER_SINGLE ? 1 : T; p.E = E;
    // Many rows per expert (a prefill through an MoE layer): the GEMV family would stream every
    // expert's weights once per 8 of its rows, so the rows go to the tile kernel, grouped by expert,
    // like the reference's MMA gather kernels (crates/metaltile-std/src/ffai/moe.rs:2256). Measured
    // crossover: 8 rows per expert, the most one GEMV pass takes (GEMV / tiles, us, 10 rows each:
    // 128 experts x 2048x768 125 / 52, 768x2048 56 / 44, 64 x 1408x2048 51 / 41, 8 x 14336x4096
    // 118 / 94, 8 x 4096x2048 25 / 28; 6 rows each: 69 / 53, 36 / 44, 38 / 41, 64 / 134, 19 / 28).
    const int gopt = options().gather_grouped;
    // f32 rows always go grouped to the f32 matrix-core kernel: the f32 dot kernels take 4 rows per pass
    // and lose at any routing (128 experts x 256x2048: 64 rows 64 us against 48, 1024 rows 315 against 88;
    // 8 experts x 4096x4096: 8 rows 212 against 77, 128 rows 940 against 112, host time included).
    if (dtype == DT_F32 && mode != GATHER_SINGLE && gopt != 1 && options().qmm_f32_tiles != 1) {
        QmmParams q;
        q.dtype = dtype; q.bits = bits; q.group_size = G;
        q.w = w; q.scales = s; q.biases = b; q.x = x; q.out = out;
        q.M = T; q.N = N; q.K = K;
        const bool ids = mode == GATHER_INDICES;
        rc = ensure_scratch(qmm_grouped_scratch_bytes(T, E, ids, 32));
        if (rc) return rc;
        rc = launch_qmm_f32_grouped(q, route, ids, T, E, g.scratch_buf, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    // exact_only: the caller named a reference kernel that multiplies by the exact f32 s*q + b
    // (mt_moe_gather_qmm_int4* / _b*, crates/metaltile-std/src/ffai/moe.rs:358-433); the tile kernel rounds
    // that value to the element type first, so such a name stays on the GEMV kernels at any routing density.
    if (dtype != DT_F32 && mode != GATHER_SINGLE && options().gather_wide == 2) {
        rc = launch_qmv_wide_gather(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    if (dtype != DT_F32 && mode != GATHER_SINGLE && gopt != 1 && (gopt == 2 || (!exact_only && (uint64_t)T > (uint64_t)8 * (E < T ? E : T)))) {
        QmmParams q;
        q.dtype = dtype; q.bits = bits; q.group_size = G;
        q.w = w; q.scales = s; q.biases = b; q.x = x; q.out = out;
        q.M = T; q.N = N; q.K = K;
        const bool ids = mode == GATHER_INDICES;
        rc = ensure_scratch(qmm_grouped_scratch_bytes(T, E, ids, 32));  // sized for the smaller tile height: more tiles
        if (rc) return rc;
        rc = launch_qmm_grouped(q, route, ids, T, E, g.scratch_buf, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    // From 4 rows per expert on large experts, below the tile kernel's crossover or under a name that must stay
    // exact: the 16-row matrix-core GEMV, 16 rows of an expert per pass. 8 experts x 14336 x 4096, rows by random ids,
    // us, 8-row passes of the GEMV family -> this: 32 rows 58.6 -> 54.5 (CSR 63 -> 60), 64 rows 113 -> 56, 128 rows
    // 197 -> 105, 256 rows 345 -> 152 (the tiles, rounded weights: 82 and 99 at 128 and 256 rows). It loses below (16 rows
    // 53 -> 54.5: a workgroup stages 16 rows whatever the expert has) and on small experts.
    if (dtype != DT_F32 && mode != GATHER_SINGLE && options().gather_wide == 0 && (uint64_t)N * K >= (1ull << 24) &&
        (uint64_t)T >= (uint64_t)4 * (E < T ? E : T)) {
        rc = launch_qmv_wide_gather(p, lc);
        if (rc != ERR_UNSUPPORTED) return rc;
    }
    return run_gemv(p, lc);
}

// ---------------------------------------------------------------------------
// name-keyed dispatch table
// ---------------------------------------------------------------------------

enum Family { F_QMV, F_QMM, F_QMM_MMA, F_QB, F_DGEMV, F_EXPERT, F_GCSR, F_GIDX, F_AQ, F_ADQ, F_DGATHER, F_BQKV, F_B4, F_BQKV_QMM, F_B4_QMM, F_NORMQ, F_GNORMQ, F_ROUTER, F_PERMUTE, F_UNPERMUTE, F_MOEDOWN, F_QVM, F_QVM_FAST };

struct KernelDesc {
    const char* name;
    Family fam;
    int bits;
    int n_bufs;
    int n_consts;
};

// Names are the reference kernels' `name` fields; buffer / constexpr order is
// their signature order (files cited in include/mtq.h).
static const KernelDesc kTable[] = {
    // w, scales, biases, x, out | k, gs_per_row
    {"mt_qmv", F_QMV, 4, 5, 2},
    {"mt_qmv_int8_fast", F_QMV, 8, 5, 2},
    // w, scales, biases, x, out | k, n, gs_per_row
    {"mt_qmm", F_QMM, 4, 5, 3},
    {"mt_qmm_bm2", F_QMM, 4, 5, 3},
    {"mt_qmm_bm4", F_QMM, 4, 5, 3},
    {"mt_qmm_int8_fast", F_QMM, 8, 5, 3},
    {"mt_qmm_bm2_int8_fast", F_QMM, 8, 5, 3},
    {"mt_qmm_bm4_int8_fast", F_QMM, 8, 5, 3},
    {"mt_qmm_mma", F_QMM_MMA, 4, 5, 3},
    {"mt_qmm_mma_m16", F_QMM_MMA, 4, 5, 3},
    {"mt_qmm_mma_int8", F_QMM_MMA, 8, 5, 3},
    {"mt_qmm_mma_m16_int8", F_QMM_MMA, 8, 5, 3},
    {"mt_qmm_mma_int2", F_QMM_MMA, 2, 5, 3},
    {"mt_qmm_mma_b3", F_QMM_MMA, 3, 5, 3},
    {"mt_qmm_mma_b5", F_QMM_MMA, 5, 5, 3},
    {"mt_qmm_mma_b6", F_QMM_MMA, 6, 5, 3},
    // w, scales, biases, x, out | k, n, group_size
    {"mt_qmv_b3", F_QB, 3, 5, 3}, {"mt_qmv_b4", F_QB, 4, 5, 3}, {"mt_qmv_b5", F_QB, 5, 5, 3},
    {"mt_qmv_b6", F_QB, 6, 5, 3}, {"mt_qmv_b8", F_QB, 8, 5, 3},
    {"mt_qmm_b3", F_QB, 3, 5, 3}, {"mt_qmm_b4", F_QB, 4, 5, 3}, {"mt_qmm_b5", F_QB, 5, 5, 3},
    {"mt_qmm_b6", F_QB, 6, 5, 3}, {"mt_qmm_b8", F_QB, 8, 5, 3},
    // weight, scales, biases, input, output | in_dim, group_size
    {"dequant_gemv_int2", F_DGEMV, 2, 5, 2}, {"dequant_gemv_int3", F_DGEMV, 3, 5, 2},
    {"dequant_gemv_int4", F_DGEMV, 4, 5, 2}, {"dequant_gemv_int5", F_DGEMV, 5, 5, 2},
    {"dequant_gemv_int6", F_DGEMV, 6, 5, 2}, {"dequant_gemv_int8", F_DGEMV, 8, 5, 2},
    {"dequant_gemv_int4_fast", F_DGEMV, 4, 5, 2},
    // weights_stacked, scales_stacked, biases_stacked, input, expert_index, output | in_dim, out_dim, group_size
    {"dequant_gemv_int4_expert_indexed", F_EXPERT, 4, 6, 3},
    // x, weight_packed, scales, biases, expert_offsets, out | k_in, m_out, n_experts, group_size
    {"mt_moe_gather_qmm_int4", F_GCSR, 4, 6, 4}, {"mt_moe_gather_qmm_int4_m8", F_GCSR, 4, 6, 4},
    {"mt_moe_gather_qmm_int4_m16", F_GCSR, 4, 6, 4}, {"mt_moe_gather_qmm_int4_m32", F_GCSR, 4, 6, 4},
    {"mt_moe_gather_qmm_b3", F_GCSR, 3, 6, 4}, {"mt_moe_gather_qmm_b5", F_GCSR, 5, 6, 4},
    {"mt_moe_gather_qmm_b6", F_GCSR, 6, 6, 4}, {"mt_moe_gather_qmm_b8", F_GCSR, 8, 6, 4},
    // x, w, scales, biases, indices, out | m_total, n_out, k_in, group_size
    {"mt_moe_gather_qmm_mma_int4", F_GIDX, 4, 6, 4}, {"mt_moe_gather_qmm_mma_int4_bm16", F_GIDX, 4, 6, 4},
    {"mt_moe_gather_qmm_mma_int8", F_GIDX, 8, 6, 4}, {"mt_moe_gather_qmm_mma_b3", F_GIDX, 3, 6, 4},
    {"mt_moe_gather_qmm_mma_b5", F_GIDX, 5, 6, 4}, {"mt_moe_gather_qmm_mma_b6", F_GIDX, 6, 6, 4},
    {"mt_moe_gather_qmm_mma_b8", F_GIDX, 8, 6, 4},
    // weight, scales, biases, indices, out | hidden, group_size
    {"dequant_gather_int2", F_DGATHER, 2, 5, 2}, {"dequant_gather_int3", F_DGATHER, 3, 5, 2},
    {"dequant_gather_int4", F_DGATHER, 4, 5, 2}, {"dequant_gather_int5", F_DGATHER, 5, 5, 2},
    {"dequant_gather_int6", F_DGATHER, 6, 5, 2}, {"dequant_gather_int8", F_DGATHER, 8, 5, 2},
    // x, (w, scales, biases) x 3, out | out_q, out_k, out_v, in_dim, group_size
    {"ffai_batched_qkv_qgemv", F_BQKV, 4, 11, 5}, {"ffai_batched_qkv_qgemv_fast", F_BQKV, 4, 11, 5},
    // x, (w, scales, biases) x 4, a_out .. d_out | out_a .. out_d, in_dim, group_size
    {"ffai_batched_4_qgemv_fast", F_B4, 4, 17, 6},
    // x, (w, scales, biases) x 3, q_buf, k_buf, v_buf | out_q, out_k, out_v, in_dim, group_size (M rows: from x)
    {"ffai_batched_qkv_qmm_fast", F_BQKV_QMM, 4, 13, 5},
    // x, (w, scales, biases) x 4, a_buf .. d_buf | out_a .. out_d, in_dim, group_size
    {"ffai_batched_4_qmm_fast", F_B4_QMM, 4, 17, 6},
    // x, norm_weight, weight, scales, biases, output, eps_buf | in_dim, group_size
    {"ffai_rms_norm_qgemv", F_NORMQ, 4, 7, 2}, {"ffai_rms_norm_qgemv_fast", F_NORMQ, 4, 7, 2},
    {"ffai_rms_norm_qgemv_int8_fast", F_NORMQ, 8, 7, 2},
    // y (f32), z, norm_weight, eps_buf, q_weight, q_scales, q_biases, out | hv, dv, out_dim, group_size
    {"ffai_gated_rms_norm_qgemv_int4_fast", F_GNORMQ, 4, 8, 4},
    // router_logits, indices_out, weights_out | n_experts, k, norm_topk_prob
    {"mt_moe_router_topk", F_ROUTER, 0, 3, 3},
    // tokens, sort_token_idx, permuted | hidden
    {"mt_moe_permute", F_PERMUTE, 0, 3, 1},
    // expert_outputs, inv_perm, top_k_weights, out | hidden, k
    {"mt_moe_unpermute", F_UNPERMUTE, 0, 4, 2},
    // gate_0, up_0, ..., gate_7, up_7, expert_indices, slot_weights, weights_stacked, scales_stacked, biases_stacked,
    // output | in_dim, out_dim, group_size
    {"ffai_moe_down_swiglu_accum_int4_chain8", F_MOEDOWN, 4, 22, 3},
    // w, scales, biases, x, out | k, n, group_size (transposed weight [K, N])
    {"mt_qvm_b3", F_QVM, 3, 5, 3}, {"mt_qvm_b4", F_QVM, 4, 5, 3}, {"mt_qvm_b5", F_QVM, 5, 5, 3},
    {"mt_qvm_b6", F_QVM, 6, 5, 3}, {"mt_qvm_b8", F_QVM, 8, 5, 3},
    // w, scales, biases, x, out | k, n, gs_per_col
    {"mt_qvm_int4_fast", F_QVM_FAST, 4, 5, 3},
    // w, out, scales, biases | group_size
    {"mt_affine_quantize_int2", F_AQ, 2, 4, 1}, {"mt_affine_quantize_int3", F_AQ, 3, 4, 1},
    {"mt_affine_quantize_int4", F_AQ, 4, 4, 1}, {"mt_affine_quantize_int5", F_AQ, 5, 4, 1},
    {"mt_affine_quantize_int6", F_AQ, 6, 4, 1}, {"mt_affine_quantize_int8", F_AQ, 8, 4, 1},
    // w, scales, biases, out | group_size
    {"mt_affine_dequantize_int2", F_ADQ, 2, 4, 1}, {"mt_affine_dequantize_int3", F_ADQ, 3, 4, 1},
    {"mt_affine_dequantize_int4", F_ADQ, 4, 4, 1}, {"mt_affine_dequantize_int5", F_ADQ, 5, 4, 1},
    {"mt_affine_dequantize_int6", F_ADQ, 6, 4, 1}, {"mt_affine_dequantize_int8", F_ADQ, 8, 4, 1},
};
static const int kTableLen = (int)(sizeof(kTable) / sizeof(kTable[0]));

static const KernelDesc* find_kernel(const char* name) {
    if (!name) return nullptr;
    for (int i = 0; i < kTableLen; i++)
        if (!strcmp(kTable[i].name, name)) return &kTable[i];
    return nullptr;
}

static int need_bytes(const mtq_buf& b, const char* param, uint64_t expected) {
    if (!b.ptr && expected) return fail(ERR_BAD_ARG, std::string("buffer '") + param + "' is null");
    if (b.bytes < expected) {
        char m[200];
        snprintf(m, sizeof m, "buffer '%s' too small: expected %llu bytes, got %llu", param,
                 (unsigned long long)expected, (unsigned long long)b.bytes);
        return fail(ERR_BUFFER_SIZE, m);
    }
    return ERR_OK;
}

#define MTQ_NEED(buf, name, n)                      \
    do {                                            \
        int rc__ = need_bytes(buf, name, n);        \
        if (rc__) return rc__;                      \
    } while (0)

// Validates the bound buffers against the shape implied by (name, dtype,
// constexprs, buffer lengths) and enqueues the kernel.
static int dispatch_desc(const KernelDesc& d, int dtype, const mtq_buf* bufs, int n_bufs,
                         const uint32_t* consts, int n_consts, const LaunchCtx& lc, const uint32_t* grid = nullptr) {
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    if (n_bufs != d.n_bufs || n_consts != d.n_consts || !bufs || !consts) {
        char m[200];
        snprintf(m, sizeof m, "%s expects %d buffers and %d constexprs, got %d and %d", d.name,
                 d.n_bufs, d.n_consts, n_bufs, n_consts);
        return fail(ERR_BAD_ARG, m);
    }
    const uint64_t sz = esize(dtype);
    const uint64_t bits = (uint64_t)d.bits;
    switch (d.fam) {
        case F_QMV:
        case F_QMM:
        case F_QMM_MMA:
        case F_QB: {
            uint32_t K = consts[0], N, G, M;
            if (K == 0) return fail(ERR_SHAPE, "k must be non-zero");
            if (d.fam == F_QMV) {
                // mt_qmv has no `n` constexpr: N is the length of `out`
                // (crates/metaltile-std/src/mlx/quantized.rs:8-16).
                uint32_t gspr = consts[1];
                if (gspr == 0 || K % gspr) return fail(ERR_SHAPE, "gs_per_row must divide k");
                G = K / gspr;
                N = (uint32_t)(bufs[4].bytes / sz);
                M = 1;
            } else {
                N = consts[1];
                if (d.fam == F_QB) {
                    G = consts[2];
                } else {
                    uint32_t gspr = consts[2];
                    if (gspr == 0 || K % gspr) return fail(ERR_SHAPE, "gs_per_row must divide k");
                    G = K / gspr;
                }
                M = (uint32_t)(bufs[3].bytes / (K * sz));
            }
            if (N == 0) return fail(ERR_SHAPE, "n must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide k");
            if (M == 0) return fail(ERR_BUFFER_SIZE, "buffer 'x' holds less than one row");
            MTQ_NEED(bufs[0], "w", (uint64_t)N * K * bits / 8);
            MTQ_NEED(bufs[1], "scales", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[2], "biases", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[3], "x", (uint64_t)M * K * sz);
            MTQ_NEED(bufs[4], "out", (uint64_t)M * N * sz);
            if (d.fam == F_QMM_MMA)
                return op_qmm(dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr,
                              bufs[4].ptr, M, N, K, true, lc);
            return op_qmv(dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr,
                          bufs[4].ptr, M, N, K, lc);
        }
        case F_DGEMV: {
            uint32_t K = consts[0], G = consts[1];
            uint32_t N = (uint32_t)(bufs[4].bytes / sz);
            if (K == 0 || N == 0) return fail(ERR_SHAPE, "in_dim and out_dim must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide in_dim");
            MTQ_NEED(bufs[0], "weight", (uint64_t)N * K * bits / 8);
            MTQ_NEED(bufs[1], "scales", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[2], "biases", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[3], "input", (uint64_t)K * sz);
            return op_qmv(dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr,
                          bufs[4].ptr, 1, N, K, lc);
        }
        case F_EXPERT: {
            uint32_t K = consts[0], N = consts[1], G = consts[2];
            if (K == 0 || N == 0) return fail(ERR_SHAPE, "in_dim and out_dim must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide in_dim");
            uint64_t slab = (uint64_t)N * K * bits / 8;
            uint32_t E = (uint32_t)(bufs[0].bytes / slab);
            if (E == 0) return fail(ERR_BUFFER_SIZE, "buffer 'weights_stacked' holds less than one expert");
            MTQ_NEED(bufs[1], "scales_stacked", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[2], "biases_stacked", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[3], "input", (uint64_t)K * sz);
            MTQ_NEED(bufs[4], "expert_index", 4);
            MTQ_NEED(bufs[5], "output", (uint64_t)N * sz);
            return op_gather(GATHER_SINGLE, dtype, d.bits, G, bufs[3].ptr, bufs[0].ptr, bufs[1].ptr,
                             bufs[2].ptr, (const uint32_t*)bufs[4].ptr, bufs[5].ptr, 1, N, K, E, lc);
        }
        case F_GCSR: {
            uint32_t K = consts[0], N = consts[1], E = consts[2], G = consts[3];
            if (K == 0 || N == 0 || E == 0) return fail(ERR_SHAPE, "k_in, m_out and n_experts must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide k_in");
            uint32_t T = (uint32_t)(bufs[0].bytes / (K * sz));
            MTQ_NEED(bufs[1], "weight_packed", (uint64_t)E * N * K * bits / 8);
            MTQ_NEED(bufs[2], "scales", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[3], "biases", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[4], "expert_offsets", (uint64_t)(E + 1) * 4);
            MTQ_NEED(bufs[5], "out", (uint64_t)T * N * sz);
            return op_gather(GATHER_CSR, dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr,
                             bufs[3].ptr, (const uint32_t*)bufs[4].ptr, bufs[5].ptr, T, N, K, E, lc,
                             options().gather_names_exact == 0);
        }
        case F_GIDX: {
            uint32_t T = consts[0], N = consts[1], K = consts[2], G = consts[3];
            if (K == 0 || N == 0) return fail(ERR_SHAPE, "k_in and n_out must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide k_in");
            uint64_t slab = (uint64_t)N * K * bits / 8;
            uint32_t E = (uint32_t)(bufs[1].bytes / slab);
            if (E == 0) return fail(ERR_BUFFER_SIZE, "buffer 'w' holds less than one expert");
            MTQ_NEED(bufs[0], "x", (uint64_t)T * K * sz);
            MTQ_NEED(bufs[2], "scales", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[3], "biases", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[4], "indices", (uint64_t)T * 4);
            MTQ_NEED(bufs[5], "out", (uint64_t)T * N * sz);
            return op_gather(GATHER_INDICES, dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr,
                             bufs[3].ptr, (const uint32_t*)bufs[4].ptr, bufs[5].ptr, T, N, K, E, lc);
        }
        case F_ROUTER: {
            const uint32_t E = consts[0], k = consts[1];
            if (E == 0 || k == 0) return fail(ERR_SHAPE, "n_experts and k must be non-zero");
            const uint32_t rows = (uint32_t)(bufs[1].bytes / ((uint64_t)4 * k));
            MTQ_NEED(bufs[0], "router_logits", (uint64_t)rows * E * sz);
            MTQ_NEED(bufs[2], "weights_out", (uint64_t)rows * k * sz);
            return launch_moe_router_topk(dtype, bufs[0].ptr, (uint32_t*)bufs[1].ptr, bufs[2].ptr, rows, E, k, consts[2], lc);
        }
        case F_PERMUTE: {
            const uint32_t H = consts[0];
            if (H == 0) return fail(ERR_SHAPE, "hidden must be non-zero");
            const uint32_t n_perm = (uint32_t)(bufs[1].bytes / 4);
            const uint32_t n_tok = (uint32_t)(bufs[0].bytes / ((uint64_t)H * sz));
            MTQ_NEED(bufs[2], "permuted", (uint64_t)n_perm * H * sz);
            return launch_moe_permute(dtype, bufs[0].ptr, (const uint32_t*)bufs[1].ptr, bufs[2].ptr, n_tok, n_perm, H, lc);
        }
        case F_UNPERMUTE: {
            const uint32_t H = consts[0], k = consts[1];
            if (H == 0 || k == 0) return fail(ERR_SHAPE, "hidden and k must be non-zero");
            const uint32_t n_tok = (uint32_t)(bufs[3].bytes / ((uint64_t)H * sz));
            const uint32_t n_perm = (uint32_t)(bufs[0].bytes / ((uint64_t)H * sz));
            MTQ_NEED(bufs[1], "inv_perm", (uint64_t)n_tok * k * 4);
            MTQ_NEED(bufs[2], "top_k_weights", (uint64_t)n_tok * k * sz);
            return launch_moe_unpermute(dtype, bufs[0].ptr, (const uint32_t*)bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, n_tok,
                                        n_perm, H, k, lc);
        }
        case F_QVM:
        case F_QVM_FAST: {
            const uint32_t K = consts[0], N = consts[1];
            if (K == 0 || N == 0 || consts[2] == 0) return fail(ERR_SHAPE, "k, n and the group constexpr must be non-zero");
            uint32_t G = consts[2];
            if (d.fam == F_QVM_FAST) {
                if (K % consts[2]) return fail(ERR_SHAPE, "gs_per_col must divide k");
                G = K / consts[2];
            }
            if (K % G) return fail(ERR_SHAPE, "group_size must divide k");
            const uint32_t M = (uint32_t)(bufs[4].bytes / ((uint64_t)N * sz));
            if (M == 0) return fail(ERR_BUFFER_SIZE, "buffer 'out' holds less than one row");
            MTQ_NEED(bufs[0], "w", (uint64_t)K * N * bits / 8);
            MTQ_NEED(bufs[1], "scales", (uint64_t)(K / G) * N * sz);
            MTQ_NEED(bufs[2], "biases", (uint64_t)(K / G) * N * sz);
            MTQ_NEED(bufs[3], "x", (uint64_t)M * K * sz);
            return op_qvm(dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, bufs[4].ptr, M, N, K, lc);
        }
        case F_MOEDOWN: {
            const uint32_t K = consts[0], N = consts[1], G = consts[2];
            if (K == 0 || N == 0) return fail(ERR_SHAPE, "in_dim and out_dim must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide in_dim");
            const void *gates[8], *ups[8];
            for (int k = 0; k < 8; k++) {
                MTQ_NEED(bufs[2 * k], "gate_*", (uint64_t)K * sz);
                MTQ_NEED(bufs[2 * k + 1], "up_*", (uint64_t)K * sz);
                gates[k] = bufs[2 * k].ptr;
                ups[k] = bufs[2 * k + 1].ptr;
            }
            MTQ_NEED(bufs[16], "expert_indices", 32);
            MTQ_NEED(bufs[17], "slot_weights", 8 * sz);
            const uint64_t slab = (uint64_t)N * K / 2;
            const uint32_t E = (uint32_t)(bufs[18].bytes / slab);
            if (E == 0) return fail(ERR_BUFFER_SIZE, "buffer 'weights_stacked' holds less than one expert");
            MTQ_NEED(bufs[19], "scales_stacked", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[20], "biases_stacked", (uint64_t)E * N * (K / G) * sz);
            MTQ_NEED(bufs[21], "output", (uint64_t)N * sz);
            return launch_moe_down_swiglu(dtype, G, 8, gates, ups, (const uint32_t*)bufs[16].ptr, bufs[17].ptr, bufs[18].ptr,
                                          bufs[19].ptr, bufs[20].ptr, bufs[21].ptr, K, N, E, lc);
        }
        case F_NORMQ: {
            const uint32_t K = consts[0], G = consts[1];
            const uint32_t N = (uint32_t)(bufs[5].bytes / sz);
            if (K == 0 || N == 0) return fail(ERR_SHAPE, "in_dim and out_dim must be non-zero");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide in_dim");
            MTQ_NEED(bufs[0], "x", (uint64_t)K * sz);
            MTQ_NEED(bufs[1], "norm_weight", (uint64_t)K * sz);
            MTQ_NEED(bufs[2], "weight", (uint64_t)N * K * bits / 8);
            MTQ_NEED(bufs[3], "scales", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[4], "biases", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[6], "eps_buf", 4);
            return op_rms_norm_qmv(dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, bufs[4].ptr,
                                   bufs[5].ptr, (const float*)bufs[6].ptr, N, K, lc);
        }
        case F_DGATHER: {
            // the table's row count is what `weight` holds; the token count what `indices` holds
            const uint32_t H = consts[0], G = consts[1];
            if (H == 0 || G == 0 || H % G) return fail(ERR_SHAPE, "group_size must divide hidden");
            if ((uint64_t)H * bits % 32) return fail(ERR_SHAPE, "hidden*bits must be a multiple of 32");
            const uint64_t row_bytes = (uint64_t)H * bits / 8;
            const uint64_t vocab = bufs[0].bytes / row_bytes, T = bufs[3].bytes / 4;
            if (vocab == 0) return fail(ERR_BUFFER_SIZE, "buffer 'weight' holds less than one row");
            if (vocab > 0xFFFFFFFFull || T > 0xFFFFFFFFull) return fail(ERR_SHAPE, "too many rows");
            MTQ_NEED(bufs[1], "scales", vocab * (H / G) * sz);
            MTQ_NEED(bufs[2], "biases", vocab * (H / G) * sz);
            MTQ_NEED(bufs[4], "out", T * H * sz);
            return launch_dequant_gather(dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, (const uint32_t*)bufs[3].ptr,
                                         bufs[4].ptr, (uint32_t)T, H, (uint32_t)vocab, lc);
        }
        case F_BQKV_QMM:
        case F_B4_QMM: {
            // The reference takes the number of rows from the grid's second dimension (its grid is [max_out / 8, M, 1],
            // crates/metaltile-std/src/ffai/batched_qkv_qmm.rs:46-70): a grid that is more than the all-ones placeholder
            // decides, and x may then be longer than M rows (a buffer allocated for the longest sequence). Without one
            // the row count is what x holds.
            const int n = d.fam == F_BQKV_QMM ? 3 : 4;
            const uint32_t K = consts[n], G = consts[n + 1];
            if (K == 0 || G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide in_dim");
            uint64_t M;
            if (grid && grid[1] >= 1 && (grid[0] > 1 || grid[1] > 1)) {
                M = grid[1];
                MTQ_NEED(bufs[0], "x", M * K * sz);
            } else {
                if (bufs[0].bytes % ((uint64_t)K * sz)) return fail(ERR_BUFFER_SIZE, "'x' must hold whole rows of in_dim");
                M = bufs[0].bytes / ((uint64_t)K * sz);
            }
            if (M > 0xFFFFFFFFull) return fail(ERR_SHAPE, "too many rows");
            const void *w[4], *s[4], *b[4];
            void* outs[4];
            uint32_t N[4];
            for (int j = 0; j < n; j++) {
                N[j] = consts[j];
                if (N[j] == 0) return fail(ERR_SHAPE, "every out_* must be non-zero");
                MTQ_NEED(bufs[1 + 3 * j], "w_*", (uint64_t)N[j] * K * bits / 8);
                MTQ_NEED(bufs[2 + 3 * j], "scales_*", (uint64_t)N[j] * (K / G) * sz);
                MTQ_NEED(bufs[3 + 3 * j], "biases_*", (uint64_t)N[j] * (K / G) * sz);
                MTQ_NEED(bufs[1 + 3 * n + j], "*_buf", M * N[j] * sz);
                w[j] = bufs[1 + 3 * j].ptr;
                s[j] = bufs[2 + 3 * j].ptr;
                b[j] = bufs[3 + 3 * j].ptr;
                outs[j] = bufs[1 + 3 * n + j].ptr;
            }
            return op_qmm_batched(dtype, d.bits, G, n, w, s, b, bufs[0].ptr, outs, N, (uint32_t)M, K, true, lc);
        }
        case F_GNORMQ: {
            const uint32_t hv = consts[0], dv = consts[1], N = consts[2], G = consts[3];
            const uint64_t K = (uint64_t)hv * dv;
            if (K == 0 || N == 0) return fail(ERR_SHAPE, "hv, dv and out_dim must be non-zero");
            if (K > 0xFFFFFFFFull) return fail(ERR_SHAPE, "hv * dv must fit 32 bits");
            if (G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide hv * dv");
            MTQ_NEED(bufs[0], "y", K * 4);   // f32 whatever the element type
            MTQ_NEED(bufs[1], "z", K * sz);
            MTQ_NEED(bufs[2], "norm_weight", (uint64_t)dv * sz);
            MTQ_NEED(bufs[3], "eps_buf", 4);
            MTQ_NEED(bufs[4], "q_weight", (uint64_t)N * K / 2);
            MTQ_NEED(bufs[5], "q_scales", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[6], "q_biases", (uint64_t)N * (K / G) * sz);
            MTQ_NEED(bufs[7], "out", (uint64_t)N * sz);
            return op_gated_rms_norm_qmv(dtype, G, (const float*)bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, (const float*)bufs[3].ptr,
                                         bufs[4].ptr, bufs[5].ptr, bufs[6].ptr, bufs[7].ptr, hv, dv, N, lc);
        }
        case F_BQKV:
        case F_B4: {
            const int n = d.fam == F_BQKV ? 3 : 4;
            const uint32_t K = consts[n], G = consts[n + 1];
            if (K == 0 || G == 0 || K % G) return fail(ERR_SHAPE, "group_size must divide in_dim");
            MTQ_NEED(bufs[0], "x", (uint64_t)K * sz);
            const void *w[4], *s[4], *b[4];
            void* outs[4];
            uint32_t N[4];
            uint64_t off = 0, total = 0;
            for (int j = 0; j < n; j++) total += consts[j];
            if (d.fam == F_BQKV) MTQ_NEED(bufs[10], "out", total * sz);
            for (int j = 0; j < n; j++) {
                N[j] = consts[j];
                if (N[j] == 0) return fail(ERR_SHAPE, "every out_* must be non-zero");
                MTQ_NEED(bufs[1 + 3 * j], "w_*", (uint64_t)N[j] * K * bits / 8);
                MTQ_NEED(bufs[2 + 3 * j], "scales_*", (uint64_t)N[j] * (K / G) * sz);
                MTQ_NEED(bufs[3 + 3 * j], "biases_*", (uint64_t)N[j] * (K / G) * sz);
                w[j] = bufs[1 + 3 * j].ptr;
                s[j] = bufs[2 + 3 * j].ptr;
                b[j] = bufs[3 + 3 * j].ptr;
                if (d.fam == F_BQKV) {
                    outs[j] = (char*)bufs[10].ptr + off * sz;  // Q, K, V concatenated in that order
                    off += N[j];
                } else {
                    MTQ_NEED(bufs[13 + j], "*_out", (uint64_t)N[j] * sz);
                    outs[j] = bufs[13 + j].ptr;
                }
            }
            return op_qmv_batched(dtype, d.bits, G, n, w, s, b, bufs[0].ptr, outs, N, K, lc);
        }
        case F_AQ: {
            // element count = length of the input tensor (one workgroup per group in
            // the reference, crates/metaltile-std/src/mlx/quantized.rs:3636-3638)
            const uint32_t G = consts[0];
            if (G == 0) return fail(ERR_SHAPE, "group_size must be non-zero");
            const uint64_t n = bufs[0].bytes / sz;
            if (n % G) return fail(ERR_SHAPE, "'w' must hold a whole number of groups");
            MTQ_NEED(bufs[1], "out", n * bits / 8);
            MTQ_NEED(bufs[2], "scales", n / G * sz);
            MTQ_NEED(bufs[3], "biases", n / G * sz);
            return launch_affine(true, dtype, d.bits, G, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, n, lc);
        }
        case F_ADQ: {
            // element count = length of the output tensor (one thread per packed word
            // in the reference, crates/metaltile-std/src/mlx/quantized.rs:3582-3585)
            const uint32_t G = consts[0];
            if (G == 0) return fail(ERR_SHAPE, "group_size must be non-zero");
            const uint64_t n = bufs[3].bytes / sz;
            if (n % G) return fail(ERR_SHAPE, "'out' must hold a whole number of groups");
            MTQ_NEED(bufs[0], "w", n * bits / 8);
            MTQ_NEED(bufs[1], "scales", n / G * sz);
            MTQ_NEED(bufs[2], "biases", n / G * sz);
            return launch_affine(false, dtype, d.bits, G, bufs[0].ptr, bufs[3].ptr, bufs[1].ptr, bufs[2].ptr, n, lc);
        }
    }
    return fail(ERR_UNKNOWN_KERNEL, "unhandled kernel family");
}

}  // namespace mtq

using namespace mtq;

// ---------------------------------------------------------------------------
// extern "C"
// ---------------------------------------------------------------------------

extern "C" {

const char* mtq_last_error(void) { return g_err.c_str(); }

int mtq_init(int device) {
    if (g.ready && g.device == device) return MTQ_OK;
    if (g.ready) mtq_shutdown();
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(ERR_NO_DEVICE, "no HIP device available; this library has no CPU fallback");
    }
    if (device < 0 || device >= n) return fail(ERR_NO_DEVICE, "device index out of range");
    MTQ_HIP(hipSetDevice(device));
    MTQ_HIP(hipGetDeviceProperties(&g.prop, device));
    if (strncmp(g.prop.gcnArchName, "gfx950", 6) != 0)
        return fail(ERR_NO_DEVICE, std::string("kernels are built for gfx950 only, device is ") + g.prop.gcnArchName);
    if (device < kMaxDevices && !g_noalloc_ptr[device]) {
        void* sp = nullptr;
        MTQ_HIP(hipGetSymbolAddress(&sp, HIP_SYMBOL(noalloc_scratch)));
        g_noalloc_ptr[device] = sp;
    }
    MTQ_HIP(hipStreamCreateWithFlags(&g.own_stream, hipStreamNonBlocking));
    MTQ_HIP(hipEventCreate(&g.ev_start));
    MTQ_HIP(hipEventCreate(&g.ev_stop));
    g.stream = g.own_stream;
    g.device = device;
    g.ready = true;
    g.timed_armed = g.timed_pending = false;
    return MTQ_OK;
}

int mtq_shutdown(void) {
    if (!g.ready) return MTQ_OK;
    (void)hipStreamSynchronize(g.stream);
    if (g.flush_buf) (void)hipFree(g.flush_buf);
    if (g.probe_buf) (void)hipFree(g.probe_buf);
    if (g.scratch_buf) (void)hipFree(g.scratch_buf);
    g.scratch_buf = nullptr;
    g.scratch_bytes = 0;
    if (g.ev_start) (void)hipEventDestroy(g.ev_start);
    if (g.ev_stop) (void)hipEventDestroy(g.ev_stop);
    if (g.own_stream) (void)hipStreamDestroy(g.own_stream);
    g = State();
    return MTQ_OK;
}

int mtq_device_name(char* out, size_t cap) {
    int rc = need_ready();
    if (rc) return rc;
    if (!out || cap == 0) return fail(ERR_BAD_ARG, "null output");
    // some driver stacks report an empty marketing name: fall back to the ISA name
    snprintf(out, cap, "%s", g.prop.name[0] ? g.prop.name : g.prop.gcnArchName);
    return MTQ_OK;
}

int mtq_get_device_info(mtq_device_info* out) {
    int rc = need_ready();
    if (rc) return rc;
    if (!out) return fail(ERR_BAD_ARG, "null output");
    memset(out, 0, sizeof *out);
    snprintf(out->name, sizeof out->name, "%s", g.prop.name);
    snprintf(out->arch, sizeof out->arch, "%s", g.prop.gcnArchName);
    out->compute_units = g.prop.multiProcessorCount;
    out->clock_khz = g.prop.clockRate;
    out->memory_clock_khz = g.prop.memoryClockRate;
    out->memory_bus_bits = g.prop.memoryBusWidth;
    out->total_memory = g.prop.totalGlobalMem;
    out->l2_bytes = g.prop.l2CacheSize;
    out->lds_per_cu_bytes = (int)g.prop.maxSharedMemoryPerMultiProcessor;
    return MTQ_OK;
}

int mtq_set_stream(void* hip_stream) {
    int rc = need_ready();
    if (rc) return rc;
    hipStream_t next = hip_stream ? (hipStream_t)hip_stream : g.own_stream;
    // launches queued on the stream being left may still use the library-owned scratch buffer,
    // which the next stream's launches would reuse (or regrow) with no ordering between the two
    if (next != g.stream) MTQ_HIP(hipStreamSynchronize(g.stream));
    g.stream = next;
    return MTQ_OK;
}

int mtq_alloc(size_t bytes, void** dptr) {
    int rc = need_ready();
    if (rc) return rc;
    if (!dptr) return fail(ERR_BAD_ARG, "null output");
    *dptr = nullptr;
    // sub-4-byte buffers are padded to 4 bytes (reference: single_dispatch.rs:142-152)
    size_t n = bytes < 4 ? 4 : bytes;
    MTQ_HIP(hipMalloc(dptr, n));
    MTQ_HIP(hipMemsetAsync(*dptr, 0, n, g.stream));
    return MTQ_OK;
}

int mtq_free(void* dptr) {
    int rc = need_ready();
    if (rc) return rc;
    if (!dptr) return MTQ_OK;
    MTQ_HIP(hipStreamSynchronize(g.stream));
    MTQ_HIP(hipFree(dptr));
    return MTQ_OK;
}

int mtq_upload(void* dptr, const void* host, size_t bytes) {
    int rc = need_ready();
    if (rc) return rc;
    if (bytes == 0) return MTQ_OK;
    if (!dptr || !host) return fail(ERR_BAD_ARG, "null pointer");
    MTQ_HIP(hipMemcpyAsync(dptr, host, bytes, hipMemcpyHostToDevice, g.stream));
    MTQ_HIP(hipStreamSynchronize(g.stream));
    return MTQ_OK;
}

int mtq_download(void* host, const void* dptr, size_t bytes) {
    int rc = need_ready();
    if (rc) return rc;
    if (bytes == 0) return MTQ_OK;
    if (!dptr || !host) return fail(ERR_BAD_ARG, "null pointer");
    MTQ_HIP(hipMemcpyAsync(host, dptr, bytes, hipMemcpyDeviceToHost, g.stream));
    MTQ_HIP(hipStreamSynchronize(g.stream));
    return MTQ_OK;
}

int mtq_memset(void* dptr, int byte_value, size_t bytes) {
    int rc = need_ready();
    if (rc) return rc;
    if (bytes == 0) return MTQ_OK;
    if (!dptr) return fail(ERR_BAD_ARG, "null pointer");
    MTQ_HIP(hipMemsetAsync(dptr, byte_value, bytes, g.stream));
    return MTQ_OK;
}

int mtq_sync(void) {
    int rc = need_ready();
    if (rc) return rc;
    MTQ_HIP(hipStreamSynchronize(g.stream));
    return MTQ_OK;
}

int mtq_qmv(int dtype, int bits, uint32_t group_size, const void* w, const void* scales,
            const void* biases, const void* x, void* out, uint32_t M, uint32_t N, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    return op_qmv(dtype, bits, group_size, w, scales, biases, x, out, M, N, K, make_ctx());
}

int mtq_qmm(int dtype, int bits, uint32_t group_size, const void* w, const void* scales,
            const void* biases, const void* x, void* out, uint32_t M, uint32_t N, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    return op_qmm(dtype, bits, group_size, w, scales, biases, x, out, M, N, K, false, make_ctx());
}

int mtq_gather_qmv_csr(int dtype, int bits, uint32_t group_size, const void* x, const void* w,
                       const void* scales, const void* biases, const uint32_t* expert_offsets,
                       void* out, uint32_t T, uint32_t N, uint32_t K, uint32_t E) {
    int rc = need_ready();
    if (rc) return rc;
    return op_gather(GATHER_CSR, dtype, bits, group_size, x, w, scales, biases, expert_offsets, out,
                     T, N, K, E, make_ctx());
}

int mtq_gather_qmv_indices(int dtype, int bits, uint32_t group_size, const void* x, const void* w,
                           const void* scales, const void* biases, const uint32_t* indices,
                           void* out, uint32_t T, uint32_t N, uint32_t K, uint32_t E) {
    int rc = need_ready();
    if (rc) return rc;
    return op_gather(GATHER_INDICES, dtype, bits, group_size, x, w, scales, biases, indices, out, T,
                     N, K, E, make_ctx());
}

int mtq_gather_qmv_single(int dtype, int bits, uint32_t group_size, const void* w,
                          const void* scales, const void* biases, const void* input,
                          const uint32_t* expert_index, void* output, uint32_t N, uint32_t K,
                          uint32_t E) {
    int rc = need_ready();
    if (rc) return rc;
    return op_gather(GATHER_SINGLE, dtype, bits, group_size, input, w, scales, biases, expert_index,
                     output, 1, N, K, E, make_ctx());
}

int mtq_qvm(int dtype, int bits, uint32_t group_size, const void* w, const void* scales, const void* biases, const void* x,
            void* out, uint32_t M, uint32_t N, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    return op_qvm(dtype, bits, group_size, w, scales, biases, x, out, M, N, K, make_ctx());
}

int mtq_qvm_noalloc(int dtype, int bits, uint32_t group_size, const void* w, const void* scales, const void* biases,
                    const void* x, void* out, uint32_t M, uint32_t N, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    if (bits < 2 || bits > 8) return fail(ERR_BAD_ARG, "bits must be in 2..8");
    if (N == 0 || K == 0) return fail(ERR_SHAPE, "N and K must be non-zero");
    if (group_size == 0 || K % group_size) return fail(ERR_SHAPE, "group_size must be non-zero and divide K");
    if ((uint64_t)N * bits % 32) return fail(ERR_SHAPE, "N*bits must be a multiple of 32");
    if (M == 0) return ERR_OK;
    if (!w || !scales || !biases || !x || !out) return fail(ERR_BAD_ARG, "null buffer");
    void* sp = g.device >= 0 && g.device < kMaxDevices ? g_noalloc_ptr[g.device] : nullptr;
    if (!sp) return fail(ERR_UNSUPPORTED, "mtq_qvm_noalloc: no built-in scratch on this device index");
    const size_t need = qvm_scratch_bytes(bits, group_size, M, N, K);
    if (need > kNoallocScratchBytes) {
        char m[200];
        snprintf(m, sizeof m, "mtq_qvm_noalloc: the partial rows need %zu bytes, the built-in scratch holds %zu; use mtq_qvm",
                 need, kNoallocScratchBytes);
        return fail(ERR_UNSUPPORTED, m);
    }
    QmvParams p;
    p.dtype = dtype; p.bits = bits; p.group_size = group_size; p.w = w; p.scales = scales; p.biases = biases; p.x = x; p.out = out;
    p.M = M; p.N = N; p.K = K;
    // every partial row the reduction reads is written by the first kernel of this call: nothing to clear
    return launch_qvm(p, sp, make_ctx());
}

int mtq_qmv_batched(int dtype, int bits, uint32_t group_size, int n_mats, const void* const* w,
                    const void* const* scales, const void* const* biases, const void* x, void* const* outs,
                    const uint32_t* N, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    return op_qmv_batched(dtype, bits, group_size, n_mats, w, scales, biases, x, outs, N, K, make_ctx());
}

int mtq_dequant_gather(int dtype, int bits, uint32_t group_size, const void* weight, const void* scales, const void* biases,
                       const uint32_t* indices, void* out, uint32_t n_tokens, uint32_t hidden, uint32_t vocab) {
    int rc = need_ready();
    if (rc) return rc;
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    return launch_dequant_gather(dtype, bits, group_size, weight, scales, biases, indices, out, n_tokens, hidden, vocab, make_ctx());
}

int mtq_qmm_batched(int dtype, int bits, uint32_t group_size, int n_mats, const void* const* w, const void* const* scales,
                    const void* const* biases, const void* x, void* const* outs, const uint32_t* N, uint32_t M, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    return op_qmm_batched(dtype, bits, group_size, n_mats, w, scales, biases, x, outs, N, M, K, false, make_ctx());
}

int mtq_gated_rms_norm_qmv(int dtype, uint32_t group_size, const float* y, const void* z, const void* norm_weight,
                           const float* eps_buf, const void* w, const void* scales, const void* biases, void* out, uint32_t hv,
                           uint32_t dv, uint32_t N) {
    int rc = need_ready();
    if (rc) return rc;
    return op_gated_rms_norm_qmv(dtype, group_size, y, z, norm_weight, eps_buf, w, scales, biases, out, hv, dv, N, make_ctx());
}

int mtq_rms_norm_qmv(int dtype, int bits, uint32_t group_size, const void* x, const void* norm_weight, const void* w,
                     const void* scales, const void* biases, void* out, const float* eps_buf, uint32_t N, uint32_t K) {
    int rc = need_ready();
    if (rc) return rc;
    return op_rms_norm_qmv(dtype, bits, group_size, x, norm_weight, w, scales, biases, out, eps_buf, N, K, make_ctx());
}

int mtq_moe_router_topk(int dtype, const void* router_logits, uint32_t* indices_out, void* weights_out, uint32_t n_rows,
                        uint32_t n_experts, uint32_t k, uint32_t norm_topk_prob) {
    int rc = need_ready();
    if (rc) return rc;
    return launch_moe_router_topk(dtype, router_logits, indices_out, weights_out, n_rows, n_experts, k, norm_topk_prob, make_ctx());
}

int mtq_moe_sort_by_expert(const uint32_t* indices, uint32_t n_tokens, uint32_t k, uint32_t n_experts,
                           uint32_t* sort_token_idx, uint32_t* inv_perm, uint32_t* expert_offsets) {
    int rc = need_ready();
    if (rc) return rc;
    return launch_moe_sort(indices, n_tokens, k, n_experts, sort_token_idx, inv_perm, expert_offsets, make_ctx());
}

int mtq_moe_permute(int dtype, const void* tokens, const uint32_t* sort_token_idx, void* permuted, uint32_t n_tokens,
                    uint32_t n_permuted, uint32_t hidden) {
    int rc = need_ready();
    if (rc) return rc;
    return launch_moe_permute(dtype, tokens, sort_token_idx, permuted, n_tokens, n_permuted, hidden, make_ctx());
}

int mtq_moe_unpermute(int dtype, const void* expert_outputs, const uint32_t* inv_perm, const void* top_k_weights, void* out,
                      uint32_t n_tokens, uint32_t n_permuted, uint32_t hidden, uint32_t k) {
    int rc = need_ready();
    if (rc) return rc;
    return launch_moe_unpermute(dtype, expert_outputs, inv_perm, top_k_weights, out, n_tokens, n_permuted, hidden, k, make_ctx());
}

int mtq_moe_down_swiglu_accum(int dtype, uint32_t group_size, uint32_t n_slots, const void* const* gates, const void* const* ups,
                              const uint32_t* expert_indices, const void* slot_weights, const void* w, const void* scales,
                              const void* biases, void* out, uint32_t in_dim, uint32_t out_dim, uint32_t n_experts) {
    int rc = need_ready();
    if (rc) return rc;
    return launch_moe_down_swiglu(dtype, group_size, n_slots, gates, ups, expert_indices, slot_weights, w, scales, biases, out,
                                  in_dim, out_dim, n_experts, make_ctx());
}

int mtq_affine_quantize(int dtype, int bits, uint32_t group_size, const void* w, void* out,
                        void* scales, void* biases, size_t n_elem) {
    int rc = need_ready();
    if (rc) return rc;
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    return launch_affine(true, dtype, bits, group_size, w, out, scales, biases, n_elem, make_ctx());
}

int mtq_affine_dequantize(int dtype, int bits, uint32_t group_size, const void* w, const void* scales,
                          const void* biases, void* out, size_t n_elem) {
    int rc = need_ready();
    if (rc) return rc;
    if (dtype != DT_F32 && dtype != DT_F16 && dtype != DT_BF16) return fail(ERR_BAD_ARG, "dtype must be MTQ_F32, MTQ_F16 or MTQ_BF16");
    return launch_affine(false, dtype, bits, group_size, w, out, const_cast<void*>(scales),
                         const_cast<void*>(biases), n_elem, make_ctx());
}

int mtq_kernel_supported(const char* kernel_name) { return find_kernel(kernel_name) ? 1 : 0; }
int mtq_kernel_count(void) { return kTableLen; }
const char* mtq_kernel_name(int i) { return i >= 0 && i < kTableLen ? kTable[i].name : nullptr; }

const char* mtq_qmm_for(int dtype, uint32_t m) {
    (void)dtype;  // the reference's choice does not depend on dtype (only its LDS skew does)
    if (m >= 32 && m % 32 == 0) return "mt_qmm_mma";
    if (m == 16) return "mt_qmm_mma_m16";
    if (m >= 4 && m % 4 == 0) return "mt_qmm_bm4";
    if (m >= 2 && m % 2 == 0) return "mt_qmm_bm2";
    return "mt_qmm";
}

int mtq_dispatch(const char* kernel_name, int dtype, const mtq_buf* bufs, int n_bufs,
                 const uint32_t* consts, int n_consts, const uint32_t grid[3], const uint32_t tpg[3],
                 double* elapsed_us) {
    (void)grid;
    (void)tpg;
    int rc = need_ready();
    if (rc) return rc;
    const KernelDesc* d = find_kernel(kernel_name);
    if (!d) return fail(ERR_UNKNOWN_KERNEL, std::string("unknown kernel '") + (kernel_name ? kernel_name : "(null)") + "'");
    LaunchCtx lc;
    lc.stream = g.stream;
    lc.start = g.ev_start;
    lc.stop = g.ev_stop;
    rc = dispatch_desc(*d, dtype, bufs, n_bufs, consts, n_consts, lc, grid);
    if (rc) return rc;
    MTQ_HIP(hipStreamSynchronize(g.stream));
    if (elapsed_us) {
        float ms = 0.f;
        hipError_t e = hipEventElapsedTime(&ms, g.ev_start, g.ev_stop);
        if (e != hipSuccess) { (void)hipGetLastError(); ms = 0.f; }  // op enqueued no kernel
        *elapsed_us = (double)ms * 1000.0;
    }
    return MTQ_OK;
}

int mtq_measure(const char* kernel_name, int dtype, const mtq_buf* bufs, int n_bufs,
                const uint32_t* consts, int n_consts, const uint32_t grid[3], const uint32_t tpg[3],
                int warmup, int iters, double* samples_us) {
    (void)grid;
    (void)tpg;
    int rc = need_ready();
    if (rc) return rc;
    const KernelDesc* d = find_kernel(kernel_name);
    if (!d) return fail(ERR_UNKNOWN_KERNEL, std::string("unknown kernel '") + (kernel_name ? kernel_name : "(null)") + "'");
    if (warmup < 0 || iters < 0 || (iters > 0 && !samples_us)) return fail(ERR_BAD_ARG, "bad warmup/iters/samples");
    LaunchCtx plain;
    plain.stream = g.stream;
    for (int i = 0; i < warmup; i++) {
        rc = dispatch_desc(*d, dtype, bufs, n_bufs, consts, n_consts, plain, grid);
        if (rc) return rc;
    }
    MTQ_HIP(hipStreamSynchronize(g.stream));
    LaunchCtx timed = plain;
    timed.start = g.ev_start;
    timed.stop = g.ev_stop;
    for (int i = 0; i < iters; i++) {
        rc = dispatch_desc(*d, dtype, bufs, n_bufs, consts, n_consts, timed, grid);
        if (rc) return rc;
        MTQ_HIP(hipEventSynchronize(g.ev_stop));
        float ms = 0.f;
        MTQ_HIP(hipEventElapsedTime(&ms, g.ev_start, g.ev_stop));
        samples_us[i] = (double)ms * 1000.0;
    }
    return MTQ_OK;
}

int mtq_dispatch_chain(const mtq_dispatch_spec* specs, int n, int repeat, double* per_kernel_us,
                       double* wall_us, double* stream_us) {
    int rc = need_ready();
    if (rc) return rc;
    if (n < 0 || repeat < 0 || (n > 0 && !specs)) return fail(ERR_BAD_ARG, "bad chain arguments");
    const size_t total = (size_t)n * (size_t)repeat;
    if (total == 0) {
        if (wall_us) *wall_us = 0.0;
        if (stream_us) *stream_us = 0.0;
        return MTQ_OK;
    }
    if (per_kernel_us && total > 65536) return fail(ERR_BAD_ARG, "per-kernel timing is limited to 65536 dispatches per chain");
    std::vector<const KernelDesc*> descs((size_t)n);
    for (int i = 0; i < n; i++) {
        descs[i] = find_kernel(specs[i].kernel_name);
        if (!descs[i]) return fail(ERR_UNKNOWN_KERNEL, std::string("unknown kernel '") + (specs[i].kernel_name ? specs[i].kernel_name : "(null)") + "'");
    }
    std::vector<hipEvent_t> ev;
    auto drop_events = [&]() { for (hipEvent_t e : ev) (void)hipEventDestroy(e); };
    if (per_kernel_us) {
        ev.resize(total * 2, nullptr);
        for (size_t i = 0; i < ev.size(); i++) {
            hipError_t e = hipEventCreate(&ev[i]);
            if (e != hipSuccess) { ev.resize(i); drop_events(); return hip_fail(e, "hipEventCreate"); }
        }
    }
    hipError_t he = hipStreamSynchronize(g.stream);
    if (he != hipSuccess) { drop_events(); return hip_fail(he, "hipStreamSynchronize"); }
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    if (stream_us) {
        he = hipEventRecord(g.ev_start, g.stream);
        if (he != hipSuccess) { drop_events(); return hip_fail(he, "hipEventRecord"); }
    }
    size_t idx = 0;
    for (int r = 0; r < repeat; r++)
        for (int i = 0; i < n; i++, idx++) {
            LaunchCtx lc;
            lc.stream = g.stream;
            if (per_kernel_us) { lc.start = ev[2 * idx]; lc.stop = ev[2 * idx + 1]; }
            rc = dispatch_desc(*descs[i], specs[i].dtype, specs[i].bufs, specs[i].n_bufs, specs[i].consts,
                               specs[i].n_consts, lc);
            if (rc) { (void)hipStreamSynchronize(g.stream); drop_events(); return rc; }
        }
    if (stream_us) {
        he = hipEventRecord(g.ev_stop, g.stream);
        if (he != hipSuccess) { (void)hipStreamSynchronize(g.stream); drop_events(); return hip_fail(he, "hipEventRecord"); }
    }
    he = hipStreamSynchronize(g.stream);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    if (he != hipSuccess) { drop_events(); return hip_fail(he, "hipStreamSynchronize"); }
    if (stream_us) {
        float ms = 0.f;
        he = hipEventElapsedTime(&ms, g.ev_start, g.ev_stop);
        if (he != hipSuccess) { drop_events(); return hip_fail(he, "hipEventElapsedTime"); }
        *stream_us = (double)ms * 1000.0;
    }
    if (wall_us) *wall_us = (double)(t1.tv_sec - t0.tv_sec) * 1e6 + (double)(t1.tv_nsec - t0.tv_nsec) * 1e-3;
    if (per_kernel_us)
        for (size_t i = 0; i < total; i++) {
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]) != hipSuccess) { (void)hipGetLastError(); ms = 0.f; }
            per_kernel_us[i] = (double)ms * 1000.0;
        }
    drop_events();
    return MTQ_OK;
}

int mtq_read_kernel(const void* const* srcs, int n_srcs, size_t bytes, int repeat, int workgroups, int in_flight, int nontemporal, void* sink, double* avg_us) {
    int rc = need_ready();
    if (rc) return rc;
    if (!srcs || n_srcs < 1 || bytes == 0 || bytes % 16 || repeat < 1 || !sink || workgroups < 0 || workgroups > 65536)
        return fail(ERR_BAD_ARG, "read: need buffers, bytes % 16 == 0, repeat >= 1, a 4-byte sink, 0..65536 workgroups");
    if (in_flight != 0 && in_flight != 1 && in_flight != 2 && in_flight != 4 && in_flight != 8) return fail(ERR_BAD_ARG, "read: loads in flight per thread must be 0 (= 8), 1, 2, 4 or 8");
    const void* fn = nullptr;
    switch (in_flight) {
        case 1: fn = nontemporal ? (const void*)read_kernel<true, 1> : (const void*)read_kernel<false, 1>; break;
        case 2: fn = nontemporal ? (const void*)read_kernel<true, 2> : (const void*)read_kernel<false, 2>; break;
        case 4: fn = nontemporal ? (const void*)read_kernel<true, 4> : (const void*)read_kernel<false, 4>; break;
        default: fn = nontemporal ? (const void*)read_kernel<true, 8> : (const void*)read_kernel<false, 8>; break;
    }
    for (int i = 0; i < n_srcs; i++)
        if (!srcs[i] || (uintptr_t)srcs[i] % 16) return fail(ERR_BAD_ARG, "read: null or unaligned buffer");
    const size_t n = bytes / 16;
    const uint32_t wgs = workgroups ? (uint32_t)workgroups : 2048u;
    // every pass over the buffers enqueued back to back, one event pair around them all
    MTQ_HIP(hipEventRecord(g.ev_start, g.stream));
    for (int r = 0; r < repeat; r++)
        for (int i = 0; i < n_srcs; i++) {
            LaunchCtx lc;
            lc.stream = g.stream;
            const uint4* s = (const uint4*)srcs[i];
            uint32_t* k = (uint32_t*)sink;
            void* args[] = {&s, (void*)&n, &k};
            hipError_t e = launch_kernel(fn, dim3(wgs), dim3(256), args, 0, lc);
            if (e != hipSuccess) return hip_fail(e, "read kernel launch");
        }
    MTQ_HIP(hipEventRecord(g.ev_stop, g.stream));
    MTQ_HIP(hipEventSynchronize(g.ev_stop));
    float ms = 0.f;
    MTQ_HIP(hipEventElapsedTime(&ms, g.ev_start, g.ev_stop));
    if (avg_us) *avg_us = (double)ms * 1000.0 / ((double)repeat * n_srcs);
    return MTQ_OK;
}

int mtq_probe_qmv_rows(const void* const* sets, int n_sets, uint32_t N, int mode, int repeat, uint64_t* stamps, double* avg_us) {
    int rc = need_ready();
    if (rc) return rc;
    if (!sets || n_sets < 1 || N == 0 || N % 16 || mode < 0 || mode > 2 || repeat < 1)
        return fail(ERR_BAD_ARG, "rows probe: need operand sets, N a multiple of 16, mode 0..2, repeat >= 1");
    for (int i = 0; i < 5 * n_sets; i++)
        if (!sets[i] || (uintptr_t)sets[i] % 16) return fail(ERR_BAD_ARG, "rows probe: null or unaligned operand");
    LaunchCtx lc;
    lc.stream = g.stream;
    auto one = [&](int i, uint64_t* st) {
        const void* const* p = sets + 5 * i;
        return launch_rows_probe(p[0], p[1], p[2], p[3], (void*)p[4], N, mode, st, lc);
    };
    MTQ_HIP(hipEventRecord(g.ev_start, g.stream));
    for (int r = 0; r < repeat; r++)
        for (int i = 0; i < n_sets; i++)
            if ((rc = one(i, nullptr))) return rc;
    MTQ_HIP(hipEventRecord(g.ev_stop, g.stream));
    if (stamps) {
        if ((rc = one(0, stamps))) return rc;
        for (int i = 1; i < n_sets; i++)
            if ((rc = one(i, nullptr))) return rc;
    }
    MTQ_HIP(hipStreamSynchronize(g.stream));
    float ms = 0.f;
    MTQ_HIP(hipEventElapsedTime(&ms, g.ev_start, g.ev_stop));
    if (avg_us) *avg_us = (double)ms * 1000.0 / ((double)repeat * n_sets);
    return MTQ_OK;
}

int mtq_plan(int op, int dtype, int bits, uint32_t group_size, uint32_t M, uint32_t N, uint32_t K, uint32_t E, uint32_t T,
             mtq_plan_info* info) {
    if (!info) return fail(ERR_BAD_ARG, "plan: info must not be null");
    memset(info, 0, sizeof(*info));
    if (op < MTQ_OP_QMV || op > MTQ_OP_RMS_NORM_QMV) return fail(ERR_BAD_ARG, "plan: unknown op");
    // Stand-in operand addresses: distinct, 256-byte aligned, never dereferenced (no launch happens).
    auto at = [](int i) { return (void*)(uintptr_t)(0x100000000ull + ((uint64_t)i << 36)); };
    const void *w = at(1), *s = at(2), *b = at(3), *x = at(4), *aux = at(6), *aux2 = at(7);
    void* out = at(5);
    void* const real_scratch = g.scratch_buf;
    const size_t real_held = g.scratch_held;
    g.scratch_buf = at(8);
    g_plan = PlanRecorder{};
    g_plan.on = true;
    g_plan.out = info;
    LaunchCtx lc;  // null stream, no events: nothing is enqueued
    int rc;
    switch (op) {
        case MTQ_OP_QMV: rc = op_qmv(dtype, bits, group_size, w, s, b, x, out, M, N, K, lc); break;
        case MTQ_OP_QMM: rc = op_qmm(dtype, bits, group_size, w, s, b, x, out, M, N, K, false, lc); break;
        case MTQ_OP_QMM_MMA: rc = op_qmm(dtype, bits, group_size, w, s, b, x, out, M, N, K, true, lc); break;
        case MTQ_OP_QVM: rc = op_qvm(dtype, bits, group_size, w, s, b, x, out, M, N, K, lc); break;
        case MTQ_OP_GATHER_CSR: rc = op_gather(GATHER_CSR, dtype, bits, group_size, x, w, s, b, (const uint32_t*)aux, out, T, N, K, E, lc); break;
        case MTQ_OP_GATHER_INDICES: rc = op_gather(GATHER_INDICES, dtype, bits, group_size, x, w, s, b, (const uint32_t*)aux, out, T, N, K, E, lc); break;
        case MTQ_OP_GATHER_SINGLE: rc = op_gather(GATHER_SINGLE, dtype, bits, group_size, x, w, s, b, (const uint32_t*)aux, out, 1, N, K, E, lc); break;
        default: rc = op_rms_norm_qmv(dtype, bits, group_size, x, aux, w, s, b, out, (const float*)aux2, N, K, lc); break;
    }
    info->n_launches = g_plan.n;
    info->scratch_bytes = g_plan.scratch;
    g_plan = PlanRecorder{};
    g.scratch_buf = real_scratch;
    g.scratch_held = real_held;
    return rc;
}

int mtq_copy_kernel(void* dst, const void* src, size_t bytes, int repeat, double* avg_us) {
    int rc = need_ready();
    if (rc) return rc;
    if (!dst || !src || bytes == 0 || bytes % 16 || repeat < 1) return fail(ERR_BAD_ARG, "copy: need non-null pointers, bytes % 16 == 0, repeat >= 1");
    size_t n = bytes / 16;
    double sum = 0.0;
    for (int r = 0; r < repeat; r++) {
        LaunchCtx lc;
        lc.stream = g.stream;
        lc.start = g.ev_start;
        lc.stop = g.ev_stop;
        uint4* d = (uint4*)dst;
        const uint4* s = (const uint4*)src;
        void* args[] = {&d, &s, &n};
        hipError_t e = launch_kernel((const void*)copy_kernel, dim3(4096), dim3(256), args, 0, lc);
        if (e != hipSuccess) return hip_fail(e, "copy kernel launch");
        MTQ_HIP(hipEventSynchronize(g.ev_stop));
        float ms = 0.f;
        MTQ_HIP(hipEventElapsedTime(&ms, g.ev_start, g.ev_stop));
        sum += (double)ms * 1000.0;
    }
    if (avg_us) *avg_us = sum / repeat;
    return MTQ_OK;
}

static int ensure_flush_buf() {
    const size_t want = (size_t)768 << 20;  // three times the 256 MB last-level cache (+ 8 x 4 MB L2)
    if (!g.flush_buf) {
        MTQ_HIP(hipMalloc(&g.flush_buf, want));
        MTQ_HIP(hipMemsetAsync(g.flush_buf, 0, want, g.stream));
        g.flush_bytes = want;
    }
    return MTQ_OK;
}

// Read-modify-write dispatch number `turn` over a quarter of the flush region: four consecutive turns touch all of it.
static hipError_t enqueue_flush_quarter(unsigned turn) {
    const size_t quarter = g.flush_bytes / 4 / sizeof(uint4);
    hipLaunchKernelGGL(flush_kernel, dim3(2048), dim3(256), 0, g.stream, (uint4*)g.flush_buf + (size_t)(turn % 4) * quarter, quarter);
    return hipGetLastError();
}

int mtq_flush_cache(void) {
    int rc = need_ready();
    if (rc) return rc;
    if ((rc = ensure_flush_buf())) return rc;
    for (unsigned i = 0; i < 16; i++) MTQ_HIP(enqueue_flush_quarter(i));   // the reference's SLC_FLUSH_DISPATCHES
    MTQ_HIP(hipStreamSynchronize(g.stream));
    return MTQ_OK;
}

int mtq_wake_clocks(double min_gpu_ms, double* gpu_ms, int* dispatches) {
    int rc = need_ready();
    if (rc) return rc;
    if (!(min_gpu_ms >= 0.0) || min_gpu_ms > 2000.0) return fail(ERR_BAD_ARG, "wake: 0 <= min_gpu_ms <= 2000");
    if ((rc = ensure_flush_buf())) return rc;
    double total = 0.0;
    int n = 0;
    // batches of 16 dispatches, each batch between two events on the stream; the host only waits at a batch's end
    while (n < 4096 && (n == 0 || total < min_gpu_ms)) {
        MTQ_HIP(hipEventRecord(g.ev_start, g.stream));
        for (unsigned i = 0; i < 16; i++, n++) MTQ_HIP(enqueue_flush_quarter((unsigned)n));
        MTQ_HIP(hipEventRecord(g.ev_stop, g.stream));
        MTQ_HIP(hipEventSynchronize(g.ev_stop));
        float ms = 0.f;
        MTQ_HIP(hipEventElapsedTime(&ms, g.ev_start, g.ev_stop));
        total += (double)ms;
    }
    if (gpu_ms) *gpu_ms = total;
    if (dispatches) *dispatches = n;
    return MTQ_OK;
}

int mtq_clock_probe(mtq_clock_sample* out) {
    int rc = need_ready();
    if (rc) return rc;
    if (!out) return fail(ERR_BAD_ARG, "clock probe: out must not be null");
    if (!g.probe_buf) MTQ_HIP(hipMalloc((void**)&g.probe_buf, 4 * sizeof(uint64_t)));
    int wall_khz = 0;
    MTQ_HIP(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, g.device));
    if (wall_khz <= 0) return fail(ERR_HIP, "clock probe: the runtime reports no constant-rate counter");
    const uint32_t turns = 24;   // 12288 adds: about 20 us at 2.4 GHz
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, g.stream, g.probe_buf, turns);
    MTQ_HIP(hipGetLastError());
    uint64_t h[4] = {};
    MTQ_HIP(hipMemcpyAsync(h, g.probe_buf, sizeof(h), hipMemcpyDeviceToHost, g.stream));
    MTQ_HIP(hipStreamSynchronize(g.stream));
    if (h[0] == 0) return fail(ERR_HIP, "clock probe: the constant-rate counter did not advance");
    const double us = (double)h[0] / ((double)wall_khz * 1e-3);
    out->probe_us = us;
    out->wall_clock_mhz = (double)wall_khz * 1e-3;
    out->valu_ops = h[2];
    out->sclk_mhz = 4.0 * (double)h[2] / us;
    out->counter_mhz = (double)h[1] / us;
    return MTQ_OK;
}

int mtq_set_option(const char* name, int value) {
    if (!name) return fail(ERR_BAD_ARG, "null option name");
    if (!strcmp(name, "qmv.rows_per_thread")) {
        if (value != 0 && value != 4 && value != 7 && value != 8) return fail(ERR_BAD_ARG, "qmv.rows_per_thread must be 0, 4, 7 or 8");
        options().qmv_rows_per_thread = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "moe.sort")) {
        if (value < 0 || value > 1) return fail(ERR_BAD_ARG, "moe.sort must be 0 (automatic) or 1 (bitonic network)");
        options().moe_sort = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qvm.wgs")) {
        if (value < 0 || value > 65536) return fail(ERR_BAD_ARG, "qvm.wgs must be in 0..65536");
        options().qvm_wgs = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "moe_down.rows")) {
        if (value < 0 || value > 4096) return fail(ERR_BAD_ARG, "moe_down.rows must be in 0..4096");
        options().moe_down_rows = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.kernel")) {
        if (value < 0 || value > 4) return fail(ERR_BAD_ARG, "qmv.kernel must be 0 (auto), 1 (one-shot), 2 (streaming), 3 (wave per four rows / per row) or 4 (waves walking the rows)");
        options().qmv_kernel = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.mfma")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmv.mfma must be 0 (auto), 1 (off) or 2 (prefer)");
        options().qmv_mfma = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.gated_fused")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmv.gated_fused must be 0 (choose), 1 (never) or 2 (wherever the shape allows)");
        options().qmv_gated_fused = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.norm_mfma")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmv.norm_mfma must be 0 (choose), 1 (never) or 2 (wherever the shape allows)");
        options().qmv_norm_mfma = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.wide_kp")) {
        if (value < 0 || value > 16 || (value & (value - 1))) return fail(ERR_BAD_ARG, "qmv.wide_kp must be 0, 1, 2, 4, 8 or 16");
        options().qmv_wide_kp = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.wide_nb")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmv.wide_nb must be 0, 1 or 2");
        options().qmv_wide_nb = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.wide")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmv.wide must be 0 (choose), 1 (never) or 2 (wherever the shape allows)");
        options().qmv_wide = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.mfma_sets")) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return fail(ERR_BAD_ARG, "qmv.mfma_sets must be 0, 1, 2 or 4");
        options().qmv_mfma_sets = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.mfma_kp") || !strcmp(name, "qmv.mfma_rbw") || !strcmp(name, "qmv.mfma_nrb")) {
        if (value < 0 || value > 256) return fail(ERR_BAD_ARG, "qmv.mfma_* must be in 0..256");
        if (name[9] == 'k') options().qmv_mfma_kp = value;
        else if (name[9] == 'r') options().qmv_mfma_rbw = value;
        else options().qmv_mfma_nrb = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.kernel")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmm.kernel must be 0 (auto), 1 (LDS tiling) or 2 (direct)");
        options().qmm_kernel = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.kgroups")) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return fail(ERR_BAD_ARG, "qmm.kgroups must be 0, 1, 2 or 4");
        options().qmm_kgroups = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.by_m")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmm.by_m must be 0 (choose), 1 or 2 (off)");
        options().qmm_by_m = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "gather.wide")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "gather.wide must be 0 (choose), 1 (never) or 2 (wherever the shape allows)");
        options().gather_wide = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "gather.grouped")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "gather.grouped must be 0 (choose), 1 (never) or 2 (always)");
        options().gather_grouped = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "gather.names_exact")) {
        if (value < 0 || value > 1) return fail(ERR_BAD_ARG, "gather.names_exact must be 0 (exact-dequant names stay exact) or 1 (they may run grouped)");
        options().gather_names_exact = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.ksplit")) {
        if (value < 0 || value > 64) return fail(ERR_BAD_ARG, "qmm.ksplit must be 0 (choose), 1 (never) or a number of splits up to 64");
        options().qmm_ksplit = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.f32_tiles")) {
        if (value < 0 || value > 2) return fail(ERR_BAD_ARG, "qmm.f32_tiles must be 0 (choose), 1 (never) or 2 (always)");
        options().qmm_f32_tiles = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.tile_rows")) {
        if (value != 0 && value != 32 && value != 64 && value != 128 && value != 256) return fail(ERR_BAD_ARG, "qmm.tile_rows must be 0, 32, 64, 128 or 256");
        options().qmm_tile_rows = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.dma")) {
        if (value < 0 || value > 3)
            return fail(ERR_BAD_ARG, "qmm.dma must be 0 (where it pays), 1 (never), 2 (always with windowed scales) or 3 (wherever the shape allows)");
        options().qmm_dma = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmm.splits")) {
        if (value < 0 || value > 64) return fail(ERR_BAD_ARG, "qmm.splits must be in 0..64");
        options().qmm_splits = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.stream_depth")) {
        if (value != 0 && value != 4 && value != 8) return fail(ERR_BAD_ARG, "qmv.stream_depth must be 0, 4 or 8");
        options().qmv_stream_depth = value;
        return MTQ_OK;
    }
    if (!strcmp(name, "qmv.stream_batches")) {
        if (value < 0 || value > 16) return fail(ERR_BAD_ARG, "qmv.stream_batches must be in 0..16");
        options().qmv_stream_batches = value;
        return MTQ_OK;
    }
    return fail(ERR_BAD_ARG, std::string("unknown option '") + name + "'");
}

int mtq_timed_begin(void) {
    int rc = need_ready();
    if (rc) return rc;
    g.timed_armed = true;
    g.timed_pending = false;
    return MTQ_OK;
}

int mtq_timed_last_us(double* elapsed_us) {
    int rc = need_ready();
    if (rc) return rc;
    if (!elapsed_us) return fail(ERR_BAD_ARG, "null output");
    if (!g.timed_pending) return fail(ERR_BAD_ARG, "no timed launch pending (call mtq_timed_begin, then one op)");
    MTQ_HIP(hipEventSynchronize(g.ev_stop));
    float ms = 0.f;
    MTQ_HIP(hipEventElapsedTime(&ms, g.ev_start, g.ev_stop));
    *elapsed_us = (double)ms * 1000.0;
    g.timed_pending = false;
    return MTQ_OK;
}

}  // extern "C"
