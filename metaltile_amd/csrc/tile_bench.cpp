// tile_bench: a host-only driver over the C-ABI (include/mtq.h) that mirrors the
// reference's `tile bench -f <filter>` for the quantized-matmul path.
//
// Each entry below reproduces one `#[bench(name = ...)]` registration of the
// reference: its name, shape, kernel name, buffer list in signature order,
// constexprs and bytes-moved model
//   qmb           crates/metaltile-std/src/mlx/quantized.rs:5789-5820 (benches :5822-6153)
//   gb            crates/metaltile-std/src/ffai/dequant_gemv.rs:547-611
//   expert bench  crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:224-250
//   csr_bench     crates/metaltile-std/src/ffai/moe.rs:3709-3784, mma benches :3786-3944
// and runs it the way run_kernel_bench does
// (crates/metaltile-std/src/run_kernel.rs:197-257): resident buffers, one cache
// flush, 15 warm-up + 10 timed dispatches, throughput from the minimum sample
// (crates/metaltile-std/src/runner.rs:615-649). One JSON object per (bench, dtype)
// row in the shape of the reference's bench output
// (crates/metaltile-cli/src/cmd/bench.rs:361-468): op, subop, shape, metric, mt.
//
// Buffers hold seeded pseudo-random codes and finite scale / bias / activation
// values (the reference fills them with random bit patterns; timing does not
// depend on the values).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <string>
#include <vector>

#include "mtq.h"

namespace {

struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed ? seed : 0x9E3779B97F4A7C15ull) {}
    uint64_t next() {  // xorshift64*
        s ^= s >> 12;
        s ^= s << 25;
        s ^= s >> 27;
        return s * 0x2545F4914F6CDD1Dull;
    }
    float unit() { return (float)((next() >> 40) * (1.0 / 16777216.0)); }
};

std::vector<std::string>* g_snapshot_rows = nullptr;  // set when --snapshot is given

size_t esize(int dt) { return dt == MTQ_F32 ? 4 : 2; }
const char* dt_label(int dt) { return dt == MTQ_F32 ? "f32" : dt == MTQ_F16 ? "f16" : "bf16"; }

uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
uint16_t to_f16(float f) {  // finite, normal-range inputs only
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    int32_t e = (int32_t)((u >> 23) & 0xFF) - 127 + 15;
    uint32_t m = u & 0x7FFFFFu;
    if (e <= 0) return (uint16_t)sign;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    uint32_t h = sign | ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)h;
}

std::vector<unsigned char> typed_values(size_t n, int dt, float lo, float hi, Rng& r) {
    std::vector<unsigned char> out(n * esize(dt));
    for (size_t i = 0; i < n; i++) {
        const float v = lo + (hi - lo) * r.unit();
        if (dt == MTQ_F32) memcpy(&out[i * 4], &v, 4);
        else {
            const uint16_t h = dt == MTQ_F16 ? to_f16(v) : to_bf16(v);
            memcpy(&out[i * 2], &h, 2);
        }
    }
    return out;
}
std::vector<unsigned char> random_words(size_t n, Rng& r) {
    std::vector<unsigned char> out(n * 4);
    for (size_t i = 0; i < n; i++) {
        const uint32_t v = (uint32_t)(r.next() >> 16);
        memcpy(&out[i * 4], &v, 4);
    }
    return out;
}

enum Abi { ABI_QMV, ABI_QMM, ABI_QB, ABI_DGEMV, ABI_EXPERT, ABI_CSR, ABI_IDX };

struct Bench {
    const char* name;    // the reference's bench name
    const char* kernel;  // the reference kernel's `name`
    Abi abi;
    int bits;
    uint32_t m, n, k, g, e;  // m = rows (T / m_total for the gathers), e = experts
};

// Shapes as registered by the reference (files cited at the top).
const Bench kBenches[] = {
    {"mlx/quantized/qmv", "mt_qmv", ABI_QMV, 4, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmv_int8_fast", "mt_qmv_int8_fast", ABI_QMV, 8, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm", "mt_qmm", ABI_QMM, 4, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_bm2", "mt_qmm_bm2", ABI_QMM, 4, 8, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_bm4", "mt_qmm_bm4", ABI_QMM, 4, 8, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_int8_fast", "mt_qmm_int8_fast", ABI_QMM, 8, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_bm2_int8_fast", "mt_qmm_bm2_int8_fast", ABI_QMM, 8, 8, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_bm4_int8_fast", "mt_qmm_bm4_int8_fast", ABI_QMM, 8, 8, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma", "mt_qmm_mma", ABI_QMM, 4, 32, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_m16", "mt_qmm_mma_m16", ABI_QMM, 4, 16, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_int8", "mt_qmm_mma_int8", ABI_QMM, 8, 32, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_m16_int8", "mt_qmm_mma_m16_int8", ABI_QMM, 8, 16, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_int2", "mt_qmm_mma_int2", ABI_QMM, 2, 32, 4096, 4096, 64, 1},
    {"mlx/quantized/qmv_b3", "mt_qmv_b3", ABI_QB, 3, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmv_b4", "mt_qmv_b4", ABI_QB, 4, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmv_b5", "mt_qmv_b5", ABI_QB, 5, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmv_b6", "mt_qmv_b6", ABI_QB, 6, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmv_b8", "mt_qmv_b8", ABI_QB, 8, 1, 4096, 4096, 64, 1},
    // transposed weight [K, N]: same buffer totals as qmv at a square shape
    {"mlx/quantized/qvm_int4_fast", "mt_qvm_int4_fast", ABI_QMM, 4, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qvm_b3", "mt_qvm_b3", ABI_QB, 3, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qvm_b4", "mt_qvm_b4", ABI_QB, 4, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qvm_b5", "mt_qvm_b5", ABI_QB, 5, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qvm_b6", "mt_qvm_b6", ABI_QB, 6, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qvm_b8", "mt_qvm_b8", ABI_QB, 8, 1, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_b3", "mt_qmm_b3", ABI_QB, 3, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_b4", "mt_qmm_b4", ABI_QB, 4, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_b5", "mt_qmm_b5", ABI_QB, 5, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_b6", "mt_qmm_b6", ABI_QB, 6, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_b8", "mt_qmm_b8", ABI_QB, 8, 4, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_b3", "mt_qmm_mma_b3", ABI_QMM, 3, 32, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_b5", "mt_qmm_mma_b5", ABI_QMM, 5, 32, 4096, 4096, 64, 1},
    {"mlx/quantized/qmm_mma_b6", "mt_qmm_mma_b6", ABI_QMM, 6, 32, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int2", "dequant_gemv_int2", ABI_DGEMV, 2, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int3", "dequant_gemv_int3", ABI_DGEMV, 3, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int4", "dequant_gemv_int4", ABI_DGEMV, 4, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int5", "dequant_gemv_int5", ABI_DGEMV, 5, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int6", "dequant_gemv_int6", ABI_DGEMV, 6, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int8", "dequant_gemv_int8", ABI_DGEMV, 8, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv/int4_fast", "dequant_gemv_int4_fast", ABI_DGEMV, 4, 1, 4096, 4096, 64, 1},
    {"ffai/dequant_gemv_expert_indexed/int4", "dequant_gemv_int4_expert_indexed", ABI_EXPERT, 4, 1, 4096, 4096, 64, 8},
    {"ffai/moe/gather_qmm_int4", "mt_moe_gather_qmm_int4", ABI_CSR, 4, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_int4_m8", "mt_moe_gather_qmm_int4_m8", ABI_CSR, 4, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_int4_m16", "mt_moe_gather_qmm_int4_m16", ABI_CSR, 4, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_int4_m32", "mt_moe_gather_qmm_int4_m32", ABI_CSR, 4, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_b3", "mt_moe_gather_qmm_b3", ABI_CSR, 3, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_b5", "mt_moe_gather_qmm_b5", ABI_CSR, 5, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_b6", "mt_moe_gather_qmm_b6", ABI_CSR, 6, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_b8", "mt_moe_gather_qmm_b8", ABI_CSR, 8, 64, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_int4", "mt_moe_gather_qmm_mma_int4", ABI_IDX, 4, 1024, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_int4_bm16", "mt_moe_gather_qmm_mma_int4_bm16", ABI_IDX, 4, 1024, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_int8", "mt_moe_gather_qmm_mma_int8", ABI_IDX, 8, 1024, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_b3", "mt_moe_gather_qmm_mma_b3", ABI_IDX, 3, 1024, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_b5", "mt_moe_gather_qmm_mma_b5", ABI_IDX, 5, 1024, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_b6", "mt_moe_gather_qmm_mma_b6", ABI_IDX, 6, 1024, 256, 2048, 64, 128},
    {"ffai/moe/gather_qmm_mma_b8", "mt_moe_gather_qmm_mma_b8", ABI_IDX, 8, 1024, 256, 2048, 64, 128},
};

struct DevBuf {
    mtq_buf b{nullptr, 0};
    int upload(const std::vector<unsigned char>& h) {
        b.bytes = h.size();
        int rc = mtq_alloc(h.size(), &b.ptr);
        if (rc) return rc;
        return mtq_upload(b.ptr, h.data(), h.size());
    }
    int zeros(size_t n) {
        b.bytes = n;
        return mtq_alloc(n, &b.ptr);  // mtq_alloc zero-fills
    }
    ~DevBuf() {
        if (b.ptr) mtq_free(b.ptr);
    }
};

#define CHK(call)                                                        \
    do {                                                                 \
        int rc__ = (call);                                               \
        if (rc__) {                                                      \
            fprintf(stderr, "  %s -> %d: %s\n", #call, rc__, mtq_last_error()); \
            return rc__;                                                 \
        }                                                                \
    } while (0)

int run_one(const Bench& bn, int dt, int warmup, int iters) {
    const size_t sz = esize(dt);
    const size_t slab_words = (size_t)bn.n * bn.k * bn.bits / 32, gpr = bn.k / bn.g;
    const size_t slabs = (bn.abi == ABI_EXPERT || bn.abi == ABI_CSR || bn.abi == ABI_IDX) ? bn.e : 1;
    Rng r(0xC0FFEEull ^ ((uint64_t)bn.bits << 32) ^ bn.k ^ ((uint64_t)dt << 20));
    DevBuf w, s, b, x, out, route;
    CHK(w.upload(random_words(slabs * slab_words, r)));
    CHK(s.upload(typed_values(slabs * bn.n * gpr, dt, 0.001f, 0.03f, r)));
    CHK(b.upload(typed_values(slabs * bn.n * gpr, dt, -0.25f, 0.0f, r)));
    CHK(x.upload(typed_values((size_t)bn.m * bn.k, dt, -1.0f, 1.0f, r)));
    CHK(out.zeros((size_t)bn.m * bn.n * sz));
    std::vector<mtq_buf> bufs;
    std::vector<uint32_t> consts;
    uint64_t bytes = slabs * slab_words * 4 + 2 * slabs * bn.n * gpr * sz + (uint64_t)bn.m * bn.k * sz + (uint64_t)bn.m * bn.n * sz;
    char shape[96];
    snprintf(shape, sizeof shape, "m%u n%u k%u %s", bn.m, bn.n, bn.k, dt_label(dt));
    switch (bn.abi) {
        case ABI_QMV:
            bufs = {w.b, s.b, b.b, x.b, out.b};
            consts = {bn.k, (uint32_t)gpr};
            break;
        case ABI_QMM:
            bufs = {w.b, s.b, b.b, x.b, out.b};
            consts = {bn.k, bn.n, (uint32_t)gpr};
            break;
        case ABI_QB:
            bufs = {w.b, s.b, b.b, x.b, out.b};
            consts = {bn.k, bn.n, bn.g};
            break;
        case ABI_DGEMV:
            bufs = {w.b, s.b, b.b, x.b, out.b};
            consts = {bn.k, bn.g};
            snprintf(shape, sizeof shape, "%ux%u %s", bn.n, bn.k, dt_label(dt));
            break;
        case ABI_EXPERT: {
            std::vector<unsigned char> idx(4, 0);
            const uint32_t pick = 3;
            memcpy(idx.data(), &pick, 4);
            CHK(route.upload(idx));
            bufs = {w.b, s.b, b.b, x.b, route.b, out.b};
            consts = {bn.k, bn.n, bn.g};
            // one slab is streamed (crates/metaltile-std/src/ffai/dequant_gemv_expert_indexed.rs:231-232)
            bytes = slab_words * 4 + 2 * bn.n * gpr * sz + bn.k * sz + bn.n * sz;
            snprintf(shape, sizeof shape, "E%u %ux%u %s", bn.e, bn.n, bn.k, dt_label(dt));
            break;
        }
        case ABI_CSR: {
            // rows spread evenly over the experts (the reference binds all-zero offsets: every row -> expert 0)
            std::vector<unsigned char> off((bn.e + 1) * 4);
            for (uint32_t i = 0; i <= bn.e; i++) {
                const uint32_t v = (uint32_t)((uint64_t)bn.m * i / bn.e);
                memcpy(&off[i * 4], &v, 4);
            }
            CHK(route.upload(off));
            bufs = {x.b, w.b, s.b, b.b, route.b, out.b};
            consts = {bn.k, bn.n, bn.e, bn.g};
            snprintf(shape, sizeof shape, "T%u m%u k%u E%u %s", bn.m, bn.n, bn.k, bn.e, dt_label(dt));
            break;
        }
        case ABI_IDX: {
            std::vector<unsigned char> idx((size_t)bn.m * 4);
            for (uint32_t i = 0; i < bn.m; i++) {
                const uint32_t v = (uint32_t)((uint64_t)i * bn.e / bn.m);  // sorted by expert, as after a permute
                memcpy(&idx[(size_t)i * 4], &v, 4);
            }
            CHK(route.upload(idx));
            bufs = {x.b, w.b, s.b, b.b, route.b, out.b};
            consts = {bn.m, bn.n, bn.k, bn.g};
            snprintf(shape, sizeof shape, "M%u N%u K%u E%u %s", bn.m, bn.n, bn.k, bn.e, dt_label(dt));
            break;
        }
    }
    CHK(mtq_flush_cache());
    std::vector<double> us((size_t)iters);
    // The reference's Metal grid is not used by this backend: it derives its launch from the shape.
    const uint32_t grid[3] = {1, 1, 1}, tpg[3] = {64, 1, 1};
    CHK(mtq_measure(bn.kernel, dt, bufs.data(), (int)bufs.size(), consts.data(), (int)consts.size(), grid, tpg, warmup, iters, us.data()));
    std::sort(us.begin(), us.end());
    const double mn = us.front(), med = us[us.size() / 2];
    const char* slash = strrchr(bn.name, '/');
    const std::string op(bn.name, slash ? (size_t)(slash - bn.name) : strlen(bn.name));
    if (g_snapshot_rows) {
        // a row of the reference's snapshot file (crates/metaltile-cli/src/cmd/bench.rs:361-372, keys in serde_json's sorted order)
        char row[512];
        snprintf(row, sizeof row, "    {\n      \"metric\": \"GB/s\",\n      \"mt\": %.3f,\n      \"op\": \"%s\",\n      \"ref\": null,\n"
                 "      \"shape\": \"%s\",\n      \"subop\": \"%s\"\n    }", (double)bytes / mn / 1e3, op.c_str(), shape, slash ? slash + 1 : bn.name);
        g_snapshot_rows->push_back(row);
    }
    printf("{\"op\": \"%s\", \"subop\": \"%s\", \"shape\": \"%s\", \"metric\": \"GB/s\", \"ref\": null, \"mt\": %.1f, "
           "\"min_us\": %.2f, \"median_us\": %.2f, \"bytes_moved\": %llu, \"kernel\": \"%s\"}\n",
           op.c_str(), slash ? slash + 1 : bn.name, shape, (double)bytes / mn / 1e3, mn, med, (unsigned long long)bytes, bn.kernel);
    fflush(stdout);
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    std::string filter, snapshot, note;
    bool list = false;
    int warmup = 15, iters = 10, device = 0;
    std::vector<int> dtypes = {MTQ_F32, MTQ_F16, MTQ_BF16};
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        if ((a == "-f" || a == "--filter") && i + 1 < argc) filter = argv[++i];
        else if (a == "--list") list = true;
        else if (a == "--snapshot" && i + 1 < argc) snapshot = argv[++i];
        else if (a == "--note" && i + 1 < argc) note = argv[++i];
        else if (a == "--warmup" && i + 1 < argc) warmup = atoi(argv[++i]);
        else if (a == "--iters" && i + 1 < argc) iters = atoi(argv[++i]);
        else if (a == "--device" && i + 1 < argc) device = atoi(argv[++i]);
        else if (a == "--dtype" && i + 1 < argc) {
            const std::string d = argv[++i];
            dtypes = {d == "f32" ? MTQ_F32 : d == "f16" ? MTQ_F16 : MTQ_BF16};
        } else {
            fprintf(stderr, "usage: tile_bench [-f substring] [--dtype f32|f16|bf16] [--warmup N] [--iters N] [--device N] [--list]\n"
                            "                  [--snapshot out.json [--note text]]\n");
            return 2;
        }
    }
    if (iters < 1) iters = 1;
    if (list) {
        for (const Bench& b : kBenches) printf("%s\t%s\n", b.name, b.kernel);
        return 0;
    }
    if (int rc = mtq_init(device)) {
        fprintf(stderr, "mtq_init(%d) -> %d: %s\n", device, rc, mtq_last_error());
        return 1;
    }
    char name[128] = "";
    mtq_device_name(name, sizeof name);
    fprintf(stderr, "device: %s\n", name);
    int failed = 0, ran = 0;
    std::vector<std::string> rows;
    if (!snapshot.empty()) g_snapshot_rows = &rows;
    for (const Bench& b : kBenches) {
        if (!filter.empty() && !strstr(b.name, filter.c_str())) continue;
        if (!mtq_kernel_supported(b.kernel)) {
            fprintf(stderr, "%s: no kernel '%s' in this library, skipped\n", b.name, b.kernel);
            continue;
        }
        for (int dt : dtypes) {
            ran++;
            if (run_one(b, dt, warmup, iters)) {
                fprintf(stderr, "%s %s: failed\n", b.name, dt_label(dt));
                failed++;
            }
        }
    }
    if (!snapshot.empty()) {
        // the layout of the reference's `tile snap` files (crates/metaltile-cli/src/cmd/snap.rs:24-35), which `tile diff` reads
        FILE* f = fopen(snapshot.c_str(), "w");
        if (!f) {
            fprintf(stderr, "cannot write %s\n", snapshot.c_str());
            failed++;
        } else {
            mtq_device_info info;
            char arch[128] = "";
            if (mtq_get_device_info(&info) == 0) snprintf(arch, sizeof arch, "%s", info.arch);
            char stamp[32];
            const time_t now = time(nullptr);
            strftime(stamp, sizeof stamp, "%Y-%m-%dT%H:%M:%SZ", gmtime(&now));
            fprintf(f, "{\n  \"device\": \"%s\",\n  \"gpu_family\": \"%s\",\n  \"timestamp\": \"%s\",\n", name[0] ? name : arch, arch, stamp);
            if (!note.empty()) {
                std::string esc;
                for (char c : note) {
                    if (c == '"' || c == '\\') esc += '\\';
                    if ((unsigned char)c >= 0x20) esc += c;
                }
                fprintf(f, "  \"note\": \"%s\",\n", esc.c_str());
            }
            fprintf(f, "  \"results\": [\n");
            for (size_t i = 0; i < rows.size(); i++) fprintf(f, "%s%s\n", rows[i].c_str(), i + 1 < rows.size() ? "," : "");
            fprintf(f, "  ]\n}\n");
            fclose(f);
            fprintf(stderr, "snapshot: %zu rows -> %s\n", rows.size(), snapshot.c_str());
        }
    }
    mtq_shutdown();
    if (ran == 0) fprintf(stderr, "no bench matches '%s'\n", filter.c_str());
    return failed ? 1 : 0;
}
