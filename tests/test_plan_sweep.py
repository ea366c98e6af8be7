"""Routing and launch geometry without a GPU: mtq_plan runs the same code as the typed entry points and records
what they would launch. A sweep over a few thousand shapes checks every recorded launch against the limits of the
part (1024 threads per workgroup, 160 KB of LDS, grid dimensions), that every valid shape is served (the generic
kernel stands behind every specialised one), that argument validation is reached without a device, and pins the
kernels the benchmark configurations are routed to.

Counterpart of the reference's host-side checks before a dispatch is encoded
(crates/metaltile-runtime/src/dispatch/single_dispatch.rs:142-158, buffer_plan.rs:62-77).
"""
import itertools

import pytest

from metaltile_amd import DType, ops

OK, BAD_ARG, SHAPE, UNSUPPORTED = 0, -2, -3, -7
LDS_MAX = 160 * 1024


def check_launches(tag, launches, n_launches, rows=1):
    # exact-dequant batches run as passes of up to 4 (f32 dot kernels) or 8 / 16 rows over the weights
    assert 1 <= n_launches <= max(8, rows // 4 + 2), f"{tag}: {n_launches} launches"
    assert len(launches) == min(n_launches, 8)
    for kernel, grid, block, lds in launches:
        threads = block[0] * block[1] * block[2]
        assert kernel.startswith(("void mtq::", "mtq::")), f"{tag}: kernel name {kernel!r}"
        assert 1 <= threads <= 1024 and threads % 64 == 0, f"{tag}: {kernel} block {block}"
        assert 1 <= grid[0] < 2 ** 31 and 1 <= grid[1] <= 65535 and 1 <= grid[2] <= 65535, f"{tag}: {kernel} grid {grid}"
        assert grid[0] * grid[1] * grid[2] < 2 ** 32, f"{tag}: {kernel} grid {grid}"
        assert lds <= LDS_MAX, f"{tag}: {kernel} asks for {lds} B of LDS"


def valid(bits, G, N, K):
    return N > 0 and K > 0 and G > 0 and K % G == 0 and (K * bits) % 32 == 0


# row lengths of the models named in the benchmark configurations and their neighbours, and awkward ones
KS = [64, 96, 128, 320, 576, 768, 1024, 1152, 1408, 2048, 2816, 3584, 4096, 5120, 6144, 8192, 11008, 13824, 14336, 18944, 28672]
NS = [1, 7, 64, 100, 131, 333, 768, 1000, 2048, 4096, 5120, 14336, 28672, 128256]
MS = [1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 32, 33, 64, 65, 100, 128, 256, 300, 512, 640, 1024, 1536, 2048, 3000, 4096]


def test_qmv_qmm_sweep():
    """Every valid (dtype, bits, group, M, N, K) is served by some kernel within the part's limits."""
    n = 0
    for dt in (DType.F32, DType.F16, DType.BF16):
        for bits, G in itertools.product((2, 3, 4, 5, 6, 8), (32, 64, 128)):
            for K in KS:
                if not valid(bits, G, 1, K):
                    continue
                for N in (NS if K in (4096, 14336, 576, 11008) else (100, 4096, 14336)):
                    for M in (MS if (K, N) in ((4096, 4096), (14336, 4096), (4096, 14336), (11008, 4096)) else (1, 4, 16, 300)):
                        if M * K * 4 >= 2 ** 32 or M * N * 4 >= 2 ** 32:
                            continue
                        for op in ("qmv", "qmm", "qmm_mma") if M > 1 else ("qmv",):
                            if op == "qmv" and M > 8:
                                continue
                            tag = f"{op} {dt.name} b{bits} g{G} M{M} N{N} K{K}"
                            rc, launches, scratch, nl = ops.plan(op, dt, bits, G, M, N, K)
                            assert rc == OK, f"{tag}: rc {rc}"
                            check_launches(tag, launches, nl, M)
                            assert scratch < 2 ** 34, tag
                            n += 1
    assert n > 3000


def test_gather_and_fused_sweep():
    n = 0
    for dt in (DType.F16, DType.BF16, DType.F32):
        for bits, G in ((4, 64), (8, 64), (2, 32), (3, 64), (6, 128)):
            for N, K in ((14336, 4096), (4096, 14336), (768, 2048), (2048, 768), (1408, 2048), (100, 576)):
                if not valid(bits, G, N, K):
                    continue
                for E, T in ((8, 32), (8, 2048), (128, 8192), (64, 1), (2047, 4096), (2048, 64), (1, 300), (8, 0)):
                    for op in ("gather_csr", "gather_indices"):
                        tag = f"{op} {dt.name} b{bits} g{G} N{N} K{K} E{E} T{T}"
                        rc, launches, scratch, nl = ops.plan(op, dt, bits, G, 1, N, K, E, T)
                        assert rc == OK, f"{tag}: rc {rc}"
                        if T:
                            check_launches(tag, launches, nl)
                        else:
                            assert nl == 0
                        n += 1
                rc, launches, _, nl = ops.plan("gather_single", dt, bits, G, 1, N, K, 8)
                assert rc == OK
                check_launches(f"gather_single {dt.name} b{bits} N{N} K{K}", launches, nl)
                rc, launches, _, nl = ops.plan("rms_norm_qmv", dt, bits, G, 1, N, K)
                assert rc == OK
                check_launches(f"rms_norm_qmv {dt.name} b{bits} N{N} K{K}", launches, nl)
                if (N * bits) % 32 == 0:
                    for M in (1, 2, 8):
                        rc, launches, scratch, nl = ops.plan("qvm", dt, bits, G, M, N, K)
                        assert rc == OK
                        check_launches(f"qvm {dt.name} b{bits} M{M} N{N} K{K}", launches, nl)
                n += 3
    assert n > 500


def test_validation_without_a_device():
    P = lambda op, *a, **k: ops.plan(op, *a, **k)[0]
    assert P("qmv", 7, 4, 64, 1, 4096, 4096) == BAD_ARG          # no such dtype
    assert P("qmv", DType.BF16, 9, 64, 1, 4096, 4096) == BAD_ARG  # bits
    assert P("qmv", DType.BF16, 1, 64, 1, 4096, 4096) == BAD_ARG
    assert P("qmv", DType.BF16, 4, 64, 1, 0, 4096) == SHAPE       # N == 0
    assert P("qmv", DType.BF16, 4, 64, 1, 4096, 0) == SHAPE
    assert P("qmv", DType.BF16, 4, 0, 1, 4096, 4096) == SHAPE     # group size
    assert P("qmv", DType.BF16, 4, 96, 1, 4096, 4096) == SHAPE    # K % G
    assert P("qmm", DType.BF16, 3, 4, 16, 64, 4) == SHAPE         # K * bits % 32
    assert P("gather_csr", DType.BF16, 4, 64, 1, 4096, 4096, 0, 8) == SHAPE   # no experts
    assert P("qvm", DType.BF16, 3, 64, 1, 100, 4096) == SHAPE     # N * bits % 32
    assert P("qmv", DType.BF16, 4, 64, 0, 4096, 4096) == OK       # no rows: nothing to do
    assert ops.plan("qmv", DType.BF16, 4, 64, 0, 4096, 4096)[3] == 0


def test_benchmark_configurations_are_routed_as_documented():
    def kernels(op, *a, **k):
        rc, launches, _, _ = ops.plan(op, *a, **k)
        assert rc == OK
        return [l[0] for l in launches], launches

    ks, ls = kernels("qmv", DType.BF16, 4, 64, 1, 14336, 4096)
    assert "qmv_rows_walk_kernel<2, 2, 6, 8>" in ks[0] and ls[0][1][0] == 512 and ls[0][2][0] == 512   # two workgroups of eight waves per compute unit walk the rows
    ks, ls = kernels("qmv", DType.F16, 4, 32, 1, 4096, 4096)
    assert "qmv_rows_walk_kernel<1, 2, 5, 16>" in ks[0] and ls[0][1][0] == 256 and ls[0][2][0] == 1024   # up to 4096 rows: sixteen rows per workgroup
    ks, _ = kernels("qmv", DType.BF16, 4, 64, 1, 128256, 4096)
    assert "qmv_rows_walk_kernel<2, 2, 6, 8>" in ks[0]
    ks, _ = kernels("qmv", DType.BF16, 4, 64, 1, 57344, 4096)      # the sizes between stay on the streaming kernel
    assert "qmv_stream_kernel" in ks[0]
    ks, ls = kernels("qmv", DType.BF16, 4, 64, 1, 28672, 8192)
    assert "qmv_rows_walk_kernel<2, 4, 6, 8>" in ks[0] and ls[0][1][0] == 512
    ks, _ = kernels("qmv", DType.F16, 4, 64, 1, 1100, 4096)        # below the walk's sizes: the wave-per-four-rows kernel
    assert "qmv_rows_kernel<1, 0, false>" in ks[0]
    for args in ((DType.BF16, 4, 64, 1, 1026, 4096), (DType.BF16, 4, 32, 1, 1024, 4096), (DType.BF16, 4, 64, 2, 4096, 4096),
                 (DType.BF16, 8, 64, 1, 4096, 4096), (DType.BF16, 4, 64, 1, 512, 4096)):
        assert "qmv_rows_kernel" not in kernels("qmv", *args)[0][0]          # what that kernel does not take
    for args in ((DType.BF16, 4, 64, 2, 14336, 4096), (DType.BF16, 8, 64, 1, 14336, 4096), (DType.BF16, 2, 64, 1, 14336, 8192),
                 (DType.F32, 4, 64, 1, 14336, 4096), (DType.BF16, 4, 64, 1, 14336, 2560), (DType.BF16, 4, 16, 1, 14336, 4096), (DType.BF16, 4, 64, 1, 24576, 2048)):
        assert "qmv_rows_walk_kernel" not in kernels("qmv", *args)[0][0]     # nor the walk: one row, 4-bit, 2048 ... 8192 codes in steps of 1024 or 3584 (2048: up to 20480 rows), groups of 32 / 64 / 128
    ks, ls = kernels("qmv", DType.BF16, 4, 64, 1, 8192, 2048)
    assert "qmv_rows_walk_kernel<2, 1, 6, 8>" in ks[0] and ls[0][1][0] == 512 and ls[0][2][0] == 512
    ks, ls = kernels("qmv", DType.BF16, 4, 64, 1, 18944, 3584)      # rows that end inside a group of 64 chunks
    assert "qmv_rows_walk_ragged_kernel<2, 2, 6, 8, 48>" in ks[0] and ls[0][1][0] == 512 and ls[0][2][0] == 512
    ks, ls = kernels("qmv", DType.F16, 4, 128, 1, 4096, 6144)
    assert "qmv_rows_walk_kernel<1, 3, 7, 16>" in ks[0] and ls[0][1][0] == 256 and ls[0][2][0] == 1024
    ks, ls = kernels("qmv", DType.BF16, 4, 64, 1, 4096, 14336)
    assert "qmv_rows_long_kernel<2, 4, 7, 6>" in ks[0] and ls[0][1][0] == 512 and ls[0][2][0] == 512   # workgroups of eight rows
    ks, ls = kernels("qmv", DType.BF16, 4, 64, 1, 4096, 11008)      # a long row that ends inside a group of 64 chunks
    assert "qmv_rows_long_ragged_kernel<2, 6, 6, 24>" in ks[0] and ls[0][1][0] == 512 and ls[0][2][0] == 512
    ks, ls = kernels("qmv", DType.F16, 4, 128, 1, 3584, 18944)
    assert "qmv_rows_long_ragged_kernel<1, 10, 7, 16>" in ks[0] and ls[0][1][0] == 224 and ls[0][2][0] == 1024
    ks, _ = kernels("qmv", DType.BF16, 4, 64, 1, 5120, 27648)       # built, level with the kernel that serves it, not routed
    assert "qmv_rows" not in ks[0]
    for bits, G, name in ((2, 32, "qmv_rows_walk2_kernel<1, 2, 5, 8>"), (2, 128, "qmv_rows_walk2_kernel<1, 2, 7, 8>"), (4, 64, "qmv_rows_long_kernel<1, 4, 4, 6>")):   # the one-row cells of the width / group sweep
        ks, ls = kernels("qmv", DType.F16, bits, G, 1, 8192, 8192)
        assert name in ks[0] and ls[0][1][0] == 512, ks
    ks, ls = kernels("qmv", DType.F16, 2, 64, 1, 4096, 8192)      # fewer rows of 2-bit codes: the one-row-per-wave kernel
    assert "qmv_rows_long_kernel<1, 2, 2, 6>" in ks[0], ks
    ks, _ = kernels("qmv", DType.F16, 8, 64, 1, 8192, 8192)
    assert "qmv_rows" not in ks[0]
    # the four-row cells of the sweep: one wave per four weight rows where that is ahead (2-bit codes, 4-bit in groups of 32,
    # three or four rows of 4-bit codes); two rows of 4-bit g64 / g128, fewer weight rows and 8-bit codes stay on the matrix-core GEMV
    for bits, G, M, name in ((2, 32, 4, "<1, 2, 8, 5, false>"), (2, 64, 2, "<1, 2, 8, 6, false>"), (4, 32, 2, "<1, 4, 16, 5, false>"), (4, 64, 4, "<1, 4, 16, 6, false>"),
                             (4, 128, 3, "<1, 4, 16, 7, false>")):
        ks, ls = kernels("qmv", DType.F16, bits, G, M, 8192, 8192)
        assert "qmv_rows_few_kernel" + name in ks[0] and ls[0][1][0] == 256 and ls[0][2][0] == 1024, ks
    for args in ((DType.F16, 4, 64, 2, 8192, 8192), (DType.F16, 4, 64, 4, 4096, 8192), (DType.F16, 8, 64, 4, 8192, 8192), (DType.BF16, 4, 64, 4, 14336, 4096),
                 (DType.F16, 2, 64, 5, 8192, 8192)):
        assert "qmv_mfma_kernel" in kernels("qmv", *args)[0][0]
    ks, _ = kernels("qmv", DType.F32, 4, 64, 1, 4096, 4096)
    assert "qmv_stream_kernel<0, 4" in ks[0] or "qmv_kernel<0, 4" in ks[0]
    for M, mb in ((512, 2), (1024, 4), (2048, 8)):     # 64-, 128-, 256-row load-to-LDS tiles
        ks, ls = kernels("qmm_mma", DType.BF16, 4, 64, M, 4096, 4096)
        assert f"qmm_dma_kernel<2, {mb}, 2, 8," in ks[0], ks
        assert ls[0][1][0] == 256 and ls[0][2][0] == 512
    ks, ls = kernels("qmm_mma", DType.BF16, 4, 64, 32, 4096, 4096)
    assert "qmm_dma_kernel<2, 1, 4, 8," in ks[0]       # 32-row tiles on 4 K-groups, K split: a reduce kernel follows
    assert "qmm_split_reduce_kernel" in ks[1]
    ks, _ = kernels("qmm_mma", DType.BF16, 8, 64, 512, 4096, 4096)
    assert "qmm_dma_kernel<2, 2, 2, 8," in ks[0] and ks[0].rstrip(">(mtq::QmmDArgs)").endswith(", 8")   # 8-bit codes: the same tiles
    for bits in (4, 8):     # a down projection at 512 rows: 128 tall tiles, K split in two so that every compute unit has one
        ks, ls = kernels("qmm_mma", DType.BF16, bits, 64, 512, 4096, 14336)
        assert "qmm_dma_kernel<2, 4, 2, 8, 0, false, true, false" in ks[0] and ls[0][1][:2] == (128, 2) and "qmm_split_reduce_kernel" in ks[1]
    ks, _ = kernels("qmm_mma", DType.BF16, 6, 64, 512, 4096, 4096)
    assert "qmm_direct_kernel<2, 6," in ks[0]          # other code widths stay on the register-staged tiles
    ks, ls = kernels("gather_indices", DType.BF16, 4, 64, 1, 14336, 4096, 8, 32)   # 4 rows per expert: the routed 16-row GEMV
    assert "qmv_wide_kernel<2, 64, 2, 2, 2>" in ks[0] and ls[0][1][:2] == (28, 8) and ls[0][2][0] == 1024
    for T in (1, 2, 4):   # the down projection's experts: up to four rows on the routed one-row-per-wave kernel, eight-row workgroups
        ks, ls = kernels("gather_csr", DType.BF16, 4, 64, 1, 4096, 14336, 8, T)
        assert "qmv_rows_long_routed_kernel<2, 4, 7, 6, 1>" in ks[0] and ls[0][1][:2] == (512, T) and ls[0][2][0] == 512, ls
    ks, _ = kernels("gather_csr", DType.BF16, 4, 64, 1, 4096, 14336, 8, 5)
    assert "qmv_mfma_kernel<2, 4," in ks[0]
    ks, ls = kernels("gather_indices", DType.BF16, 4, 64, 1, 2048, 2048, 8, 1)           # the expert widths of other models walk too
    assert "qmv_rows_walk_routed_kernel<2, 1, 6, 2>" in ks[0]
    ks, ls = kernels("gather_csr", DType.BF16, 4, 64, 1, 2048, 7168, 8, 4)
    assert "qmv_rows_walk_routed_ragged_kernel<2, 4, 6, 1, 32>" in ks[0] and ls[0][1][:2] == (128, 4), ls
    ks, ls = kernels("gather_indices", DType.BF16, 4, 64, 1, 2048, 3072, 8, 1)           # other row lengths: the kernels that served them before
    assert "qmv_rows" not in ks[0]
    ks, _ = kernels("gather_indices", DType.BF16, 4, 64, 1, 14336, 4096, 8, 16)           # 2 rows per expert: 8-row passes
    assert "qmv_mfma_kernel<2, 4," in ks[0]
    for view in ("gather_csr", "gather_indices"):      # fewer rows than experts: a grid row per row, not per expert
        for T, E in ((1, 8), (2, 8), (4, 8), (7, 8), (8, 128), (32, 128)):
            ks, ls = kernels(view, DType.BF16, 4, 64, 1, 14336, 4096, E, T)
            # up to eight rows on experts of 14336 x 4096: the routed walk, about 512 workgroups over the grid rows
            kernel = "qmv_rows_walk_routed_kernel<2, 2, 6, " if T <= 8 else "qmv_mfma_kernel<2, 4,"
            assert kernel in ks[0] and ls[0][1][1] == T, (view, T, E, ls)
            if T <= 8 and E <= 64:
                assert ls[0][1][0] == 512 // T and ls[0][2][0] == 512, ls
        ks, ls = kernels("gather_single", DType.BF16, 4, 64, 1, 14336, 4096, 8, 1)
        assert "qmv_rows_walk_routed_kernel<2, 2, 6, 3>" in ks[0] and ls[0][1][:2] == (512, 1)
        ks, ls = kernels(view, DType.BF16, 4, 64, 1, 4096, 14336, 8, 2)     # rows of 14336 codes: the routed one-row-per-wave kernel
        assert "qmv_rows_long_routed_kernel<2, 4, 7, 6, " in ks[0] and ls[0][1][1] == 2, ls
        ks, ls = kernels(view, DType.BF16, 4, 64, 1, 2048, 768, 128, 33)   # (more than 32 rows: a grid row per expert)
        assert ls[0][1][1] == 128
    ks, _ = kernels("gather_indices", DType.BF16, 4, 64, 1, 4096, 4096, 8, 2048)
    assert "moe_count_sort_kernel" in ks[0] and "gather_tiles_kernel" in ks[1] and "qmm_dma_kernel<2, 2, 2, 8, 2, true" in ks[2]
    for bits, M in itertools.product((2, 4, 8), (1, 4)):   # the sweep configuration's cells
        for G in (32, 64, 128):
            ks, _ = kernels("qmv", DType.F16, bits, G, M, 8192, 8192)
            assert "generic" not in ks[0], (bits, G, M, ks)
