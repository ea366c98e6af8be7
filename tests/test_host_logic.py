"""CPU-only checks of the host layer: selector, stats, packers, and that the
C-ABI library loads and exports every symbol include/*.h declares."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import metaltile_amd as m
from metaltile_amd import DType, _lib
from metaltile_amd.signatures import KERNEL_SIGNATURES

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _have_gpu() -> bool:
    return _lib.load().mtq_init(0) == 0


# ---- selector: crates/metaltile-std/src/mlx/quantized.rs:5128-5199 ----------

@pytest.mark.parametrize("impl", ["python", "c"])
def test_selector_routes_like_reference(impl):
    lib = _lib.load()
    pick = (lambda dt, mm: m.mt_qmm_for(dt, mm)) if impl == "python" else \
        (lambda dt, mm: lib.mtq_qmm_for(int(dt), mm).decode())
    for mm in (32, 64, 96, 128):
        assert pick(DType.F32, mm) == "mt_qmm_mma"
    assert pick(DType.F32, 16) == "mt_qmm_mma_m16"
    for mm in (4, 8, 12, 20, 24, 28, 36, 60):
        assert pick(DType.F32, mm) == "mt_qmm_bm4"
    for mm in (2, 6, 10, 14, 18, 22, 26, 30):
        assert pick(DType.F32, mm) == "mt_qmm_bm2"
    for mm in (1, 3, 5, 7, 9, 15, 31):
        assert pick(DType.F32, mm) == "mt_qmm"
    for dt in (DType.F32, DType.F16):
        assert pick(dt, 8) == "mt_qmm_bm4"


# ---- stats: crates/metaltile-std/src/stats.rs:57-84 --------------------------

def test_bench_stats_reference_cases():
    st = m.BenchStats.from_samples([1.0, 2.0, 3.0, 4.0, 10.0])
    assert (st.min_us, st.median_us, st.p95_us, st.p99_us) == (1.0, 3.0, 10.0, 10.0)
    assert st.stddev_us > 0.0
    slow = m.BenchStats.from_samples([250.0] * 5 + [120.0] * 5)
    fast = m.BenchStats.from_samples([250.0] * 4 + [120.0] * 6)
    assert slow.median_us - fast.median_us >= 100.0
    assert slow.min_us == 120.0 and fast.min_us == 120.0
    with pytest.raises(ValueError):
        m.BenchStats.from_samples([])


def test_throughput_uses_min_sample():
    st = m.BenchStats.from_samples([10.0, 5.0, 20.0])
    assert m.to_gbps(st, 5e3) == pytest.approx(1.0)        # 5000 B / 5 us = 1 GB/s
    assert m.to_gflops(st, 1e4) == pytest.approx(2.0)


# ---- packers: crates/metaltile-std/src/utils.rs:72-127 -----------------------

def test_pack_f32_reference_unit_values():
    assert m.unpack_f32(m.pack_f32([0.0, 1.5, -2.25, 1024.0], DType.F32), DType.F32).tolist() == [0.0, 1.5, -2.25, 1024.0]
    assert m.unpack_f32(m.pack_f32([0.0, 0.5, -0.5, 2.0], DType.F16), DType.F16).tolist() == [0.0, 0.5, -0.5, 2.0]
    assert m.unpack_f32(m.pack_f32([1.0, 2.0, -0.5, 0.0], DType.BF16), DType.BF16).tolist() == [1.0, 2.0, -0.5, 0.0]
    r = m.unpack_f32(m.pack_f32([0.1], DType.F16), DType.F16)[0]
    assert abs(r - 0.1) < 1e-3 and r != np.float32(0.1)
    for dt in (DType.F32, DType.F16, DType.BF16):
        assert m.pack_f32([], dt) == b"" and m.unpack_f32(b"", dt).size == 0
    assert m.unpack_f32(bytes([0, 0, 128, 63, 7]), DType.F32).tolist() == [1.0]
    assert m.pack_f32([1.0], DType.U32) == (1).to_bytes(4, "little")
    assert [len(m.pack_f32([1.0], dt)) for dt in (DType.F32, DType.F16, DType.BF16)] == [4, 2, 2]


def test_pack_codes_matches_oracle_layout(oracle):
    from metaltile_amd.synth import pack_codes
    rng = np.random.default_rng(3)
    for bits in (2, 3, 4, 5, 6, 8):
        codes = rng.integers(0, 1 << bits, size=(7, 96), dtype=np.uint8)
        assert np.array_equal(pack_codes(codes, bits), oracle.pack_codes(codes, bits))


# ---- C-ABI surface -----------------------------------------------------------

def _header_symbols():
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in sorted(os.listdir(os.path.join(ROOT, "include"))) if h.endswith(".h"))
    return re.findall(r"MTQ_API\s+[\w\s\*]+?\b(mtq_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    names = _header_symbols()
    assert len(names) >= 25
    lib = C.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/*.h but not exported"
    assert sorted(names) == sorted(_lib.SIGNATURES)


def test_kernel_table_matches_python_signatures():
    lib = _lib.load()
    c_names = [lib.mtq_kernel_name(i).decode() for i in range(lib.mtq_kernel_count())]
    assert sorted(c_names) == sorted(KERNEL_SIGNATURES)
    assert lib.mtq_kernel_name(lib.mtq_kernel_count()) is None
    assert lib.mtq_kernel_supported(b"mt_qmv") == 1 and lib.mtq_kernel_supported(b"mt_gemm") == 0
    # names the reference registers for this path (tests + benches)
    for n in ("mt_qmv", "mt_qmm", "mt_qmm_mma", "dequant_gemv_int2", "dequant_gemv_int4_expert_indexed",
              "mt_moe_gather_qmm_int4_m8", "mt_moe_gather_qmm_mma_int4"):
        assert n in c_names


def test_no_gpu_means_error_not_fallback():
    if _have_gpu():
        pytest.skip("a GPU is present; the no-device path cannot be observed")
    lib = _lib.load()
    assert lib.mtq_init(0) == -1
    assert b"no CPU fallback" in lib.mtq_last_error() or b"HIP device" in lib.mtq_last_error()
    assert lib.mtq_qmv(0, 4, 64, None, None, None, None, None, 1, 8, 512) == -1
    assert lib.mtq_sync() == -1
    with pytest.raises(m.MtqError) as ei:
        m.Context(0)
    assert ei.value.code == -1


def test_product_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "metaltile_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", ".hpp")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_bench_driver_lists_the_reference_registrations():
    """The C++ driver names every bench it mirrors; each maps to a kernel the library and the Python mirror know."""
    import subprocess
    from metaltile_amd.build import DRIVER
    from metaltile_amd.signatures import KERNEL_SIGNATURES
    if not os.path.exists(DRIVER):
        from metaltile_amd.build import build
        build(verbose=False)
    out = subprocess.run([DRIVER, "--list"], capture_output=True, text=True, check=True).stdout
    rows = [l.split("\t") for l in out.strip().splitlines()]
    assert len(rows) >= 55
    names = [r[0] for r in rows]
    assert len(set(names)) == len(names)
    for must in ("mlx/quantized/qmv", "mlx/quantized/qmm_mma", "ffai/dequant_gemv/int4_fast",
                 "ffai/dequant_gemv_expert_indexed/int4", "ffai/moe/gather_qmm_int4", "ffai/moe/gather_qmm_mma_int4"):
        assert must in names
    for _, kernel in rows:
        assert kernel in KERNEL_SIGNATURES, kernel


def test_bench_driver_fails_loudly_without_a_gpu():
    import subprocess
    import metaltile_amd as m
    from metaltile_amd.build import DRIVER
    try:
        m.GpuRunner(0)
    except m.MtqError:
        r = subprocess.run([DRIVER, "-f", "mlx/quantized/qmv"], capture_output=True, text=True)
        assert r.returncode != 0 and "no HIP device" in r.stderr
    else:
        pytest.skip("a GPU is present")


def test_dynamic_m_helpers_match_reference_values():
    """crates/metaltile-std/src/mlx/quantized_mma_dynamic_m.rs:116-160 (its unit tests)."""
    from metaltile_amd import dynamic_m as d
    assert [d.pad_t_to_bm(t) for t in (0, 1, 31, 32, 33, 37, 64, 4096, 4097)] == [0, 32, 32, 32, 64, 64, 64, 4096, 4128]
    assert d.dispatch_grid(1, 128) == [4, 1, 1]
    assert d.dispatch_grid(37, 128) == [4, 2, 1]
    assert d.dispatch_grid(4096, 2048) == [64, 128, 1]
    assert all(d.kernel_name_for(dt) == "mt_qmm_mma" for dt in (DType.F32, DType.F16, DType.BF16))
    with pytest.raises(ValueError):
        d.dispatch_grid(32, 100)
    x = b"\x01" * 16
    p = d.pad_x_rows_bytes(x, 2, 4, 2)
    assert len(p) == 32 * 4 * 2 and p[:16] == x and not any(p[16:])
    with pytest.raises(ValueError):
        d.pad_x_rows_bytes(x, 3, 4, 2)


def test_two_bit_operand_constants_are_exact():
    """The one-row-per-wave GEMV makes a pair of 2-bit codes an MFMA operand by masking it in place and OR-ing it into
    the mantissa of a power of two chosen by its bit position (csrc/qmv_rows_common.h: rp_crumb_class / _shift / _kor). The
    same constants, restated here, must give exactly offset + code in both halves for every pair of every dword."""
    def cls(dt, i): return (i if i < 5 else i - 5) if dt == "f16" else i % 3
    def sh(dt, i): return (0 if i < 5 else 10) if dt == "f16" else 6 * (i // 3)
    def kor(dt, p):
        h = ((15 + 10 - 2 * p) << 10) if dt == "f16" else ((127 + 7 - 2 * p) << 7)
        return h | (h << 16)
    def val(dt, h):
        if dt == "f16":
            return float(np.array([h], dtype=np.uint16).view(np.float16)[0])
        return float(np.array([h << 16], dtype=np.uint32).view(np.float32)[0])
    src = open(os.path.join(ROOT, "metaltile_amd", "csrc", "qmv_rows_common.h")).read()
    assert "DT == DT_F16 ? (i < 5 ? i : i - 5) : i % 3" in src and "DT == DT_F16 ? (i < 5 ? 0 : 10) : 6 * (i / 3)" in src
    assert "(uint32_t)(15 + 10 - 2 * p) << 10 : (uint32_t)(127 + 7 - 2 * p) << 7" in src
    rng = np.random.default_rng(1)
    for dt, mant in (("f16", 10), ("bf16", 7)):
        for w in [0, 0xFFFFFFFF, 0xAAAAAAAA, 0x55555555] + [int(v) for v in rng.integers(0, 2 ** 32, size=500)]:
            for i in range(8):
                p = cls(dt, i)
                v = ((w >> sh(dt, i)) & (0x00030003 << (2 * p))) | kor(dt, p)
                magic = 2.0 ** (mant - 2 * p)
                assert val(dt, v & 0xFFFF) == magic + ((w >> (2 * i)) & 3)
                assert val(dt, v >> 16) == magic + ((w >> (2 * (i + 8))) & 3)
