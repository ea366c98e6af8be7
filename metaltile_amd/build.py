"""Build libmtq_hip.so (HIP kernels + C-ABI) for gfx950 with hipcc.

Usage: python -m metaltile_amd.build [--force]

hipcc cross-compiles without a GPU. Objects go to metaltile_amd/_build/ and the
library to metaltile_amd/libmtq_hip.so (both git-ignored, both in-tree so the
library travels with the source tree).
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJDIR = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "libmtq_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 from float code.
HIPFLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
# per-source additions: the wave-per-four-rows GEMV keeps its matrix-core results in ordinary vector registers (no accumulator-register copies)
EXTRA_FLAGS = {"qmv_rows.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"], "qmv_rows_few.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"], "qmv_rows_walk.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}
SOURCES = ["api.hip", "qmv.hip", "qmv_f32.hip", "qmv_f16.hip", "qmv_bf16.hip", "qmv_mfma.hip", "qmv_mfma_f16.hip", "qmv_mfma_bf16.hip", "qmv_mfma_f16_odd.hip", "qmv_mfma_bf16_odd.hip", "qmv_wide.hip", "qmv_wide_gather.hip", "generic.hip", "qmm.hip", "qmm_direct.hip", "qmm_direct_odd.hip", "qmm_dma.hip", "qmm_dma_b8.hip", "qmm_f32.hip", "affine.hip", "norm.hip", "moe.hip", "moe_down.hip", "qvm.hip", "qmv_rows.hip", "qmv_rows_few.hip", "qmv_rows_walk.hip"]


def _headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(HERE, "..", "include", "mtq.h"))
    return hs


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def _compile(src, force):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if not force and not _stale(obj, [path] + _headers()):
        return obj, ""
    cmd = [HIPCC] + HIPFLAGS + EXTRA_FLAGS.get(src, []) + (["-x", "hip"] if src.endswith(".cpp") else []) + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only feature flag; that note is noise
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return obj, err


def build(force: bool = False, verbose: bool = True) -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in results]
    for _, err in results:
        if err.strip() and verbose:
            print(err, file=sys.stderr)
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    build_driver(force, verbose)
    return LIB


DRIVER = os.path.join(HERE, "tile_bench")


def build_driver(force: bool = False, verbose: bool = True) -> str:
    """Host-only bench driver over the C-ABI (csrc/tile_bench.cpp), linked against the library beside it."""
    src = os.path.join(CSRC, "tile_bench.cpp")
    inc = os.path.join(HERE, "..", "include")
    if force or _stale(DRIVER, [src, os.path.join(inc, "mtq.h"), LIB]):
        cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-I", inc, src, "-o", DRIVER, "-L", HERE, "-lmtq_hip",
               "-Wl,-rpath,$ORIGIN"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"driver build failed:\n{r.stderr}")
        if verbose:
            print(f"built {DRIVER}")
    return DRIVER


SAN_DIR = os.path.join(OBJDIR, "san")
SAN_FLAGS = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-fno-sanitize-recover=all"]


def build_sanitized(verbose: bool = True) -> dict:
    """The library's HOST code (routing, geometry, argument checks, the C-ABI) compiled with the address and
    undefined-behaviour sanitizers and linked into two programs under _build/san/: plan_sweep (walks mtq_plan over
    a grid of shapes, no GPU needed) and tile_bench. Only the host side of every source is compiled
    (--cuda-host-only: no device code, so nothing here can be launched); the GPU library is not touched."""
    os.makedirs(SAN_DIR, exist_ok=True)
    inc = os.path.join(HERE, "..", "include")
    flags = ["--offload-arch=gfx950", "--cuda-host-only", "-O1", "-g", "-std=c++17", "-Wall", "-Wno-unused-function", "-I", inc] + SAN_FLAGS

    def one(src):
        obj = os.path.join(SAN_DIR, os.path.splitext(src)[0] + ".o")
        r = subprocess.run([HIPCC] + flags + ["-c", os.path.join(CSRC, src), "-o", obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"sanitized compile of {src} failed:\n{r.stderr}")
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(one, SOURCES))
    out = {}
    # A host-only object still refers to the device code bundle its registration hands to the runtime at load
    # time. Give each an empty bundle (the bundle magic and an entry count of zero): nothing is ever launched here.
    names = set()
    for o in objs:
        r = subprocess.run(["nm", "-u", o], capture_output=True, text=True)
        names.update(l.split()[-1] for l in r.stdout.splitlines() if "__hip_fatbin_" in l)
    stub_c = os.path.join(SAN_DIR, "empty_bundles.c")
    with open(stub_c, "w") as f:
        for nm in sorted(names):
            f.write(f'__attribute__((section(".hip_fatbin"), aligned(4096))) const unsigned char {nm}[32] = "__CLANG_OFFLOAD_BUNDLE__";\n')
    stub_o = os.path.join(SAN_DIR, "empty_bundles.o")
    r = subprocess.run(["gcc", "-c", stub_c, "-o", stub_o], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"empty bundle stubs failed:\n{r.stderr}")
    objs = objs + [stub_o]
    clangxx = os.path.join(os.path.dirname(os.path.realpath(HIPCC)), "..", "lib", "llvm", "bin", "clang++")
    if not os.path.exists(clangxx):
        clangxx = "/opt/rocm/lib/llvm/bin/clang++"
    rocm_lib = os.path.join(os.path.dirname(os.path.realpath(HIPCC)), "..", "lib")
    for prog in ("plan_sweep", "tile_bench"):
        exe = os.path.join(SAN_DIR, prog)
        cmd = [clangxx, os.path.join(CSRC, prog + ".cpp")] + objs + \
              ["-O1", "-g", "-std=c++17", "-I", inc, "-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=all",
               "-L", rocm_lib, "-lamdhip64", "-ldl", f"-Wl,-rpath,{rocm_lib}", "-o", exe]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"sanitized link of {prog} failed:\n{r.stderr}")
        out[prog] = exe
        if verbose:
            print(f"built {exe}")
    return out


if __name__ == "__main__":
    if "--sanitized" in sys.argv:
        build_sanitized()
    else:
        build(force="--force" in sys.argv)
