// plan_sweep: walks mtq_plan over a grid of shapes on the host and checks every launch it reports against the
// limits of the part. Built with the address and undefined-behaviour sanitizers from the library's own host code
// (metaltile_amd/build.py, build_sanitized): it exercises the routing and geometry code of every entry point
// without a GPU. Exit code 0 = every plan within limits; otherwise the first violations are printed.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <initializer_list>

#include "mtq.h"

namespace {

long g_checked = 0, g_bad = 0;

void check(const char* what, int dtype, int bits, uint32_t G, uint32_t M, uint32_t N, uint32_t K, uint32_t E, uint32_t T,
           int rc, const mtq_plan_info& pi, bool must_succeed) {
    g_checked++;
    auto complain = [&](const char* why) {
        if (g_bad++ < 20)
            fprintf(stderr, "%s dtype %d bits %d g %u M %u N %u K %u E %u T %u: %s (rc %d, %d launches)\n", what, dtype, bits, G, M, N,
                    K, E, T, why, rc, pi.n_launches);
    };
    if (must_succeed && rc != MTQ_OK) return complain("valid shape refused");
    if (rc != MTQ_OK) {
        if (rc != MTQ_ERR_BAD_ARG && rc != MTQ_ERR_SHAPE && rc != MTQ_ERR_UNSUPPORTED) complain("unexpected error code");
        return;
    }
    const int n = pi.n_launches < MTQ_PLAN_MAX_LAUNCHES ? pi.n_launches : MTQ_PLAN_MAX_LAUNCHES;
    for (int i = 0; i < n; i++) {
        const mtq_plan_launch& l = pi.launch[i];
        const uint64_t threads = (uint64_t)l.block[0] * l.block[1] * l.block[2];
        if (threads == 0 || threads > 1024 || threads % 64) complain("block size");
        if (l.grid[0] == 0 || l.grid[1] == 0 || l.grid[2] == 0 || l.grid[0] >= (1u << 31) || l.grid[1] > 65535 || l.grid[2] > 65535)
            complain("grid");
        if (l.lds_bytes > 160 * 1024) complain("LDS");
        if (!memchr(l.kernel, 0, sizeof(l.kernel)) || !l.kernel[0]) complain("kernel name");
    }
}

}  // namespace

int main() {
    const uint32_t Ks[] = {64, 96, 128, 320, 576, 768, 1024, 1152, 2048, 2816, 3584, 4096, 5120, 8192, 11008, 14336, 18944, 28672};
    const uint32_t Ns[] = {1, 7, 64, 100, 131, 1000, 4096, 14336, 128256};
    const uint32_t Ms[] = {1, 2, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 128, 300, 512, 1024, 2048, 4096};
    const uint32_t Gs[] = {32, 64, 128};
    mtq_plan_info pi;
    for (int dtype = 0; dtype < 3; dtype++)
        for (int bits = 2; bits <= 8; bits++)
            for (uint32_t G : Gs)
                for (uint32_t K : Ks) {
                    const bool valid = K % G == 0 && ((uint64_t)K * bits) % 32 == 0;
                    for (uint32_t N : Ns) {
                        for (uint32_t M : Ms) {
                            if ((uint64_t)M * K * 4 >= (1ull << 32) || (uint64_t)M * N * 4 >= (1ull << 32)) continue;
                            for (int op : {MTQ_OP_QMV, MTQ_OP_QMM, MTQ_OP_QMM_MMA}) {
                                if (op == MTQ_OP_QMV && M > 8) continue;
                                const int rc = mtq_plan(op, dtype, bits, G, M, N, K, 1, 0, &pi);
                                check("qmv/qmm", dtype, bits, G, M, N, K, 1, 0, rc, pi, valid);
                            }
                        }
                        const uint32_t ET[][2] = {{8, 32}, {8, 2048}, {128, 8192}, {2047, 4096}, {2048, 64}, {1, 300}};
                        for (auto& et : ET)
                            for (int op : {MTQ_OP_GATHER_CSR, MTQ_OP_GATHER_INDICES}) {
                                const int rc = mtq_plan(op, dtype, bits, G, 1, N, K, et[0], et[1], &pi);
                                check("gather", dtype, bits, G, 1, N, K, et[0], et[1], rc, pi, valid);
                            }
                        int rc = mtq_plan(MTQ_OP_GATHER_SINGLE, dtype, bits, G, 1, N, K, 8, 1, &pi);
                        check("gather_single", dtype, bits, G, 1, N, K, 8, 1, rc, pi, valid);
                        rc = mtq_plan(MTQ_OP_RMS_NORM_QMV, dtype, bits, G, 1, N, K, 1, 0, &pi);
                        check("rms_norm_qmv", dtype, bits, G, 1, N, K, 1, 0, rc, pi, valid);
                        for (uint32_t M : {1u, 2u, 8u}) {
                            rc = mtq_plan(MTQ_OP_QVM, dtype, bits, G, M, N, K, 1, 0, &pi);
                            check("qvm", dtype, bits, G, M, N, K, 1, 0, rc, pi, valid && ((uint64_t)N * bits) % 32 == 0);
                        }
                    }
                }
    // argument validation reaches its error codes without a device
    struct { int op, dtype, bits; uint32_t G, M, N, K, E, T; int want; } bad[] = {
        {MTQ_OP_QMV, 7, 4, 64, 1, 4096, 4096, 1, 0, MTQ_ERR_BAD_ARG},   {MTQ_OP_QMV, 2, 9, 64, 1, 4096, 4096, 1, 0, MTQ_ERR_BAD_ARG},
        {MTQ_OP_QMV, 2, 4, 64, 1, 0, 4096, 1, 0, MTQ_ERR_SHAPE},        {MTQ_OP_QMV, 2, 4, 96, 1, 4096, 4096, 1, 0, MTQ_ERR_SHAPE},
        {MTQ_OP_GATHER_CSR, 2, 4, 64, 1, 4096, 4096, 0, 8, MTQ_ERR_SHAPE}, {99, 2, 4, 64, 1, 4096, 4096, 1, 0, MTQ_ERR_BAD_ARG},
    };
    for (auto& b : bad) {
        const int rc = mtq_plan(b.op, b.dtype, b.bits, b.G, b.M, b.N, b.K, b.E, b.T, &pi);
        g_checked++;
        if (rc != b.want && g_bad++ < 20) fprintf(stderr, "validation: op %d gave %d, expected %d\n", b.op, rc, b.want);
    }
    if (mtq_plan(MTQ_OP_QMV, 2, 4, 64, 1, 4096, 4096, 1, 0, nullptr) != MTQ_ERR_BAD_ARG) g_bad++;
    printf("plan_sweep: %ld plans checked, %ld violations\n", g_checked, g_bad);
    return g_bad ? 1 : 0;
}
