"""The 16-row matrix-core GEMV issues its weight loads by hand and waits for them with hand-counted
`s_waitcnt vmcnt(N)`. That only pipelines if the compiler adds no wait of its own inside the stream loop: one
`vmcnt` wait it inserts there (for a register whose load it still believes pending, or for a spilled value it
reloads) also waits for every load in flight, silently, with correct results. This test compiles the kernel's two
translation units to assembly (no GPU needed) and checks, for every instance, that inside the loop that holds the
MFMAs the only `vmcnt` waits are the two written by hand and that nothing there touches scratch memory; and that
between the loop's end and the wait for its last loads (which nothing reads: dead registers to the compiler) nothing is
written to a register one of those loads is still on its way to."""
import concurrent.futures
import os
import re
import shutil
import subprocess
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "metaltile_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _units_including(header):
    """Every translation unit that instantiates the kernels of `header` (directly or through another header): an
    instance added in a new file is scanned without this test being told about it."""
    def includes(path, seen):
        out = set()
        for m in re.finditer(r'#include\s+"([^"]+)"', open(path).read()):
            name = os.path.basename(m.group(1))
            if name not in seen and os.path.exists(os.path.join(CSRC, name)):
                seen.add(name)
                out |= {name} | includes(os.path.join(CSRC, name), seen)
        return out
    units = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip") and header in includes(os.path.join(CSRC, f), set()))
    assert units, header
    return units


def _assembly(src, out):
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I" + os.path.join(HERE, "..", "include"), "--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return open(out).read().split("\n")


def _regs(operand):
    m = re.match(r"v\[(\d+):(\d+)\]", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", operand)
    return {int(m.group(1))} if m else set()


def _early_writes(body, loop_end):
    """The last turn's loads are still in flight when the loop ends and nothing reads them: to the compiler their
    registers are free. A value written to one of them before the wait is overwritten when the load lands."""
    ring = set()
    for i, l in enumerate(body):
        if "ASMSTART" in body[i - 1] and "global_load_dword" in l:
            ring |= _regs(l.split()[1].rstrip(","))
    assert ring
    hits = []
    for i in range(loop_end + 1, len(body)):
        l = body[i]
        if "s_waitcnt vmcnt(0)" in l and "ASMSTART" in body[i - 1]:
            return hits
        t = l.split()
        if not t or t[0].startswith((";", ".", "s_", "ds_write", "global_store", "scratch_store", "buffer_store", "v_cmp")) or len(t) < 2:
            continue
        if _regs(t[1].rstrip(",")) & ring:
            hits.append(l.strip())
    raise AssertionError("no hand-written vmcnt(0) behind the stream loop")


def _stream_loops(lines):
    """(kernel symbol, hand-written vmcnt waits, all vmcnt waits, scratch accesses, MFMAs, early writes) of each kernel's
    MFMA loop; early writes: instructions between the loop's end and the hand-written vmcnt(0) behind it that write a
    register some hand-issued load targets."""
    starts = [(i, l.split(":")[0]) for i, l in enumerate(lines) if l.startswith("_ZN3mtq15qmv_wide_kernel") and "; @" in l]
    starts.append((len(lines), ""))
    for (s0, name), (s1, _) in zip(starts, starts[1:]):
        body = lines[s0:s1]
        found = None
        for i, l in enumerate(body):
            if "Inner Loop Header" not in l:
                continue
            k = i
            while k >= 0 and not re.match(r"^\.LBB\d+_\d+:", body[k]):
                k -= 1
            label = body[k].split(":")[0]
            j, mine, every, scratch, mfma = k + 1, 0, 0, 0, 0
            while j < len(body) and not re.search(r"s_cbranch\w+ " + re.escape(label) + r"\b", body[j]):
                if "s_waitcnt vmcnt" in body[j]:
                    every += 1
                    mine += "ASMSTART" in body[j - 1]
                scratch += "scratch_" in body[j]
                mfma += "v_mfma" in body[j]
                j += 1
            if mfma and j < len(body):   # (a loop whose back edge is not a conditional branch to its header is not the stream loop)
                found = (name, mine, every, scratch, mfma, j)
        assert found, f"{name}: no loop with MFMAs"
        yield found[:5] + (_early_writes(body, found[5]),)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is needed to produce the assembly")
def test_only_hand_counted_waits_in_the_stream_loop():
    with tempfile.TemporaryDirectory() as tmp:
        with concurrent.futures.ThreadPoolExecutor(max_workers=2) as ex:
            units = _units_including("qmv_wide_impl.h")
            assert {"qmv_wide.hip", "qmv_wide_gather.hip"} <= set(units)
            outs = list(ex.map(lambda s: _assembly(s, os.path.join(tmp, s + ".s")), units))
    n = 0
    for lines in outs:
        for name, mine, every, scratch, mfma, early in _stream_loops(lines):
            assert mine == 2 and every == 2, f"{name}: {every} vmcnt waits in the stream loop, {mine} of them hand-written"
            assert scratch == 0, f"{name}: {scratch} scratch accesses in the stream loop"
            assert not early, f"{name}: registers with loads in flight are written before the wait behind the loop: {early[:3]}"
            assert mfma in (16, 32), name
            n += 1
    assert n >= 40


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is needed to produce the assembly")
def test_tile_kernels_wait_only_where_written():
    """The load-to-LDS tile kernel counts its loads by hand too. From its first MFMA to its last, every instance may
    wait on `vmcnt` only where the source says so, and may not touch scratch memory: one spilled tile offset reloaded
    in the loop cost the 256-row windowed instance 12 % (each reload is followed by the compiler's wait for it, which
    is a wait for every load in flight)."""
    with tempfile.TemporaryDirectory() as tmp:
        with concurrent.futures.ThreadPoolExecutor(max_workers=2) as ex:
            units = _units_including("qmm_dma_impl.h")
            assert {"qmm_dma.hip", "qmm_dma_b8.hip"} <= set(units)
            outs = list(ex.map(lambda s: _assembly(s, os.path.join(tmp, s + ".s")), units))
    n = 0
    for lines in outs:
        starts = [(i, l.split(":")[0]) for i, l in enumerate(lines) if l.startswith("_ZN3mtq14qmm_dma_kernel") and "; @" in l]
        starts.append((len(lines), ""))
        for (s0, name), (s1, _) in zip(starts, starts[1:]):
            body = lines[s0:s1]
            mf = [i for i, l in enumerate(body) if "v_mfma" in l]
            assert mf, name
            region = body[mf[0]:mf[-1] + 1]
            own = [l for i, l in enumerate(region) if "s_waitcnt vmcnt" in l and "ASMSTART" not in region[i - 1]]
            assert not own, f"{name}: {len(own)} vmcnt waits between the MFMAs that the source does not hold"
            assert not any("scratch_" in l for l in region), f"{name}: scratch memory touched between the MFMAs"
            n += 1
    assert n >= 60


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is needed to produce the assembly")
def test_one_row_streaming_instances_keep_their_values_in_registers():
    """The one-row streaming GEMV is a single pass of loads, dots and a reduction: a value spilled to scratch memory is
    reloaded in the middle of it, and the compiler's wait for that reload waits for every weight load in flight. Every
    bf16 instance that serves one or two activation rows - plain, single-expert, routed, with the RMS norm or the gated
    norm inside - must have a scratch size of zero (the routed instances on a ring of eight loads and the first form of
    the dealt gate did not, at a cost of up to 2 us per launch; 2-bit codes on three and four rows still spill and are
    not planned for)."""
    with tempfile.TemporaryDirectory() as tmp:
        lines = _assembly("qmv_bf16.hip", os.path.join(tmp, "qmv_bf16.s"))
    seen = 0
    for i, l in enumerate(lines):
        m = re.match(r"^_ZN3mtq17qmv_stream_kernelILi2ELi(\d)ELi(\d)ELi(\d)ELi(\d)ELi(\d+)ELi(\d)ELi(\d)EEEvNS_8QmvSArgsE:", l)
        if not m:
            continue
        bits, mb, depth, mode, maxt, sbi, norm = map(int, m.groups())
        if mb > 2:
            continue
        size = next(int(x.split(":")[1]) for x in lines[i:] if "; ScratchSize:" in x)
        assert size == 0, f"qmv_stream_kernel<bf16, {bits}-bit, {mb} rows, ring {depth}, mode {mode}, {maxt}, {sbi}, norm {norm}>: {size} bytes of scratch"
        seen += 1
    assert seen >= 30


def test_the_schedule_model_behind_the_static_asserts():
    """Both hand-waited kernels hold their vmcnt counts against a compile-time replay of their own issue order
    (csrc/vm_schedule.h: QmmDmaWaits, QmvWideWaits). The replay's queue is checked here on the host compiler, with
    cases it must accept and cases it must reject, and every schedule the library instantiates must hold."""
    src = r"""
#include "vm_schedule.h"
using namespace mtq;
constexpr bool accepts() {
    VmQueue q;
    q.issue(vm_tag(1, 0), 2); q.issue(vm_tag(1, 1), 2); q.issue(vm_tag(2, 0), 3);
    if (q.younger_than(vm_tag(1, 0)) != 5 || q.younger_than(vm_tag(1, 1)) != 3 || q.younger_than(vm_tag(2, 0)) != 0) return false;
    if (q.younger_than(vm_tag(3, 0)) != -1 || q.landed(vm_tag(1, 0))) return false;
    q.wait(5);                                    // the two oldest loads have landed
    if (!q.landed(vm_tag(1, 0)) || q.landed(vm_tag(1, 1))) return false;
    q.wait(6);                                    // a weaker wait later takes nothing back
    if (!q.landed(vm_tag(1, 0))) return false;
    q.wait(0);
    return q.landed(vm_tag(2, 0)) && !q.landed(vm_tag(3, 0));
}
static_assert(accepts(), "queue model");
// one load too many allowed in flight: the load that is needed may be the one still outstanding
constexpr bool too_weak() { VmQueue q; q.issue(vm_tag(1, 0), 1); q.issue(vm_tag(1, 1), 4); q.wait(5); return q.landed(vm_tag(1, 0)); }
static_assert(!too_weak(), "a wait that is too weak must be seen");
int main() { return 0; }
"""
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "q.cpp")
        open(path, "w").write(src)
        r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", CSRC, path], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
    # the kernels carry the static_asserts (a build of the library is their test)
    for header, name in (("qmm_dma_impl.h", "QmmDmaWaits"), ("qmv_wide_impl.h", "QmvWideWaits")):
        text = open(os.path.join(CSRC, header)).read()
        assert re.search(r"static_assert\(\s*(Waits|" + name + r"<[^>]*>)::holds\(\)", text), header
        assert "qm_wait_vm<(" not in text and "qw_wait<2" not in text, f"{header}: a wait count written as a literal expression"
