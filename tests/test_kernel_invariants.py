"""Compile-time invariants of the dense forward kernel that its hand-counted waits rely on.

The kernel leaves the output stores of a finished work item in flight and waits with
`s_waitcnt vmcnt(N)` for the loads of the next item; N must not exceed the number of
store instructions a full wave issues, and the registers that receive the next item's Q
operands (loaded from inline assembly, invisible to the compiler's own wait insertion)
must not be copied between the load and that wait.  Both are properties of the generated
code, so they are checked on the generated code: hipcc cross-compiles without a GPU.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tritonops_amd", "csrc", "prefill.hip")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.fixture(scope="module")
def prefill_asm(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm") / "prefill.s"
    cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O3", "-std=c++17",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "--cuda-device-only", "-S", SRC, "-o", str(out)]
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return out.read_text()


def _bodies(text, family, flag=None):
    """{(dtype, head_dim): lines} of the instantiations of a kernel template; `flag` picks the
    value of a third, boolean template argument where the template has one."""
    kernels = {}
    for m in re.finditer(r"^(_ZN2mi\S*\d%sI(\S+?)Li(\d+)E(?:Lb([01])E)?\S*):" % family, text, re.M):
        if m.group(4) != flag:
            continue
        body = text[m.end():text.index("s_endpgm", m.end())]
        kernels[(m.group(2), int(m.group(3)))] = body.split("\n")
    return kernels


@pytest.fixture(scope="module")
def dense_kernels(prefill_asm):
    kernels = _bodies(prefill_asm, "dense_kernel")
    assert len(kernels) == 6, sorted(kernels)          # bf16 / f16  x  64 / 96 / 128
    return kernels


@pytest.fixture(scope="module")
def short_kernels(prefill_asm):
    """The dense walk (dense_short_kernel<T, D, false>) and, under dtype + "/window", the same
    kernel walking the tiles of a token window (dense_short_kernel<T, D, true>): one protocol."""
    kernels = _bodies(prefill_asm, "dense_short_kernel", "0")
    assert len(kernels) == 6, sorted(kernels)          # bf16 / f16  x  64 / 96 / 128
    window = _bodies(prefill_asm, "dense_short_kernel", "1")
    assert len(window) == 6, sorted(window)
    kernels.update({(dtype + "/window", d): lines for (dtype, d), lines in window.items()})
    return kernels


def _regs(line):
    line = line.split(";")[0]
    found = set()
    for a, b in re.findall(r"v\[(\d+):(\d+)\]", line):
        found.update(range(int(a), int(b) + 1))
    found.update(int(x) for x in re.findall(r"\bv(\d+)\b", line))
    return found


def _significant(lines):
    """(index, text) of the instruction lines: no comments, directives or labels."""
    out = []
    for i, l in enumerate(lines):
        t = l.split(";")[0].strip()
        if t and not t.startswith(".") and not t.endswith(":"):
            out.append((i, t))
    return out


def test_output_store_count_matches_the_counted_wait(dense_kernels):
    # At an item boundary a wave issues: Q and tile 0, the first half of its
    # output stores, tile 1, the second half of the stores, tile 2.  The wait at
    # the top of the next item leaves that second half and the loads of tile 2
    # in flight: half the stores plus the loads of one tile per wave.  That wait
    # is the one site in the kernel where a counted wait and a full wait are the
    # two arms of one decision (all stores issued or not), joined in front of
    # the barrier that opens the item with no vector-memory instruction between.
    for (dtype, d), lines in dense_kernels.items():
        stores = [l for l in lines if "global_store_dwordx4" in l]
        expect = {64: 4, 96: 8, 128: 8}[d]
        assert len(stores) == expect, (dtype, d, len(stores))
        tile_loads = {64: 2, 96: 4, 128: 4}[d]      # K and V instructions of one tile per wave
        want = expect // 2 + tile_loads
        sig = _significant(lines)
        sites = []
        for k, (_, t) in enumerate(sig):
            if t != "s_waitcnt vmcnt(%d)" % want:
                continue
            arm = [x for _, x in sig[k + 1:k + 4]]
            if "s_waitcnt vmcnt(0)" not in arm:
                continue                                  # some other wait that happens to have the same count
            j = k + 1 + arm.index("s_waitcnt vmcnt(0)")
            nxt = next(x for _, x in sig[j + 1:] if x.startswith("s_barrier") or re.match(r"(global|buffer|scratch|flat)_", x))
            assert nxt.startswith("s_barrier"), (dtype, d, nxt)
            sites.append(k)
        assert len(sites) == 1, (dtype, d, want, sites)


def test_no_scratch_memory(dense_kernels, short_kernels):
    for key, lines in list(dense_kernels.items()) + list(short_kernels.items()):
        assert not any("scratch_" in l for l in lines), key


def test_short_form_register_budget_and_item_top_wait(prefill_asm, short_kernels):
    """At head_dim 64 three 4-wave workgroups share a CU, one wave of each per SIMD:
    512 registers in allocation units of 8 leave 168 per wave.  And the item-top
    wait of every instantiation: when the next item has a fourth tile its loads
    (one K and one V instruction per wave at head_dim 64, two of each otherwise)
    are the youngest and may stay in flight, else everything is waited for; the
    two arms meet in front of the barrier that opens the item."""
    seen = 0
    for block in prefill_asm.split("- .agpr_count:")[1:]:
        kern = re.search(r"\.name:\s+(\S+)", block).group(1)
        if "dense_short_kernel" in kern and "Li64E" in kern:
            assert int(re.search(r"\.vgpr_count:\s+(\d+)", block).group(1)) <= 168, kern
            seen += 1
    assert seen == 4                                   # bf16 / f16  x  dense / window
    for (dtype, d), lines in short_kernels.items():
        assert len([l for l in lines if "global_store_dwordx4" in l]) == {64: 4, 96: 8, 128: 8}[d], (dtype, d)
        tile_loads = {64: 2, 96: 4, 128: 4}[d]
        sig = _significant(lines)
        sites = []
        for k, (_, t) in enumerate(sig):
            if t != "s_waitcnt vmcnt(%d)" % tile_loads:
                continue
            near = [j for j in range(max(0, k - 5), min(len(sig), k + 6)) if sig[j][1] == "s_waitcnt vmcnt(0)"]
            if not near:
                continue                                  # (the waits at the top of a position also cover lgkmcnt)
            last = max(near + [k])
            nxt = next(x for _, x in sig[last + 1:] if x.startswith("s_barrier") or re.match(r"(global|buffer|scratch|flat)_", x))
            assert nxt.startswith("s_barrier"), (dtype, d, nxt)
            sites.append(k)
        assert len(sites) == 1, (dtype, d, sites)


def test_q_registers_are_untouched_between_load_and_wait(dense_kernels, short_kernels):
    for (dtype, d), lines in list(dense_kernels.items()) + list(short_kernels.items()):
        loads = [(i, l) for i, l in enumerate(lines)
                 if re.match(r"\s*global_load_dwordx4 v\[\d+:\d+\], v\[\d+:\d+\], off offset:", l)]
        ksteps = d // 16
        assert len(loads) == 2 * ksteps, (dtype, d, len(loads))
        dest = lambda grp: set().union(*[set(range(*map(int, re.search(r"v\[(\d+):(\d+)\]", l).groups()))) |
                                         {int(re.search(r"v\[(\d+):(\d+)\]", l).group(2))} for _, l in grp])
        first, second = loads[:ksteps], loads[ksteps:]
        q = dest(first)
        assert q == dest(second) and len(q) == 4 * ksteps, (dtype, d)
        barriers = [i for i, l in enumerate(lines) if "s_barrier" in l]
        top_barrier = min(i for i in barriers if i > first[-1][0])     # the barrier that opens an item
        # (a) first item: from its loads to the item's first barrier; (b) later items: from the loads at the
        # bottom of the item loop to the end of the loop body (it branches back above the same barrier);
        # (c) from the head of the item loop to that barrier.
        head = max(i for i, l in enumerate(lines[:top_barrier]) if re.match(r"\.LBB\d+_\d+:.*Loop Header", l))
        spans = [(first[-1][0] + 1, top_barrier), (second[-1][0] + 1, len(lines)), (head, top_barrier)]
        for lo, hi in spans:
            for i in range(lo, hi):
                l = lines[i]
                if "global_load_dwordx4" in l and "lds" not in l:
                    continue
                assert not (_regs(l) & q), (dtype, d, i, l.strip())


# ---------------------------------------------------------------------------
# Direct-to-LDS loads with a scalar base, issued from inline assembly.  A vector
# memory instruction that reads a scalar register written by a VECTOR
# instruction needs five wait states between the two, and the compiler cannot
# see into an assembly statement to add them.  The kernels therefore form every
# such base with scalar arithmetic (or read it to a scalar register well
# before); this checks the generated code of every kernel that uses the form.
@pytest.fixture(scope="module")
def saddr_sources(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out_dir = tmp_path_factory.mktemp("asm_all")
    texts = {}
    procs = []
    for name in ("prefill.hip", "bwd.hip", "xent.hip"):
        out = out_dir / (name + ".s")
        cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O3", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I", os.path.join(ROOT, "include"), "--cuda-device-only", "-S",
               os.path.join(ROOT, "tritonops_amd", "csrc", name), "-o", str(out)]
        procs.append((name, out, subprocess.Popen(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)))
    for name, out, proc in procs:
        assert proc.wait() == 0, name
        texts[name] = out.read_text()
    return texts


def test_scalar_bases_of_lds_loads_are_not_fresh_vector_results(saddr_sources):
    n_loads = 0
    for name, text in saddr_sources.items():
        lines = [l for l in text.split("\n")
                 if l.strip() and not l.strip().startswith(";") and not l.strip().startswith(".")]
        for k, line in enumerate(lines):
            m = re.search(r"global_load_lds_dword(?:x4)? v\d+, s\[(\d+):(\d+)\]", line)
            if not m:
                continue
            n_loads += 1
            lo, hi = int(m.group(1)), int(m.group(2))
            for back in range(1, 7):
                prev = lines[k - back]
                if prev.strip().endswith(":"):
                    break
                w = re.match(r"\s*(v_\S+)\s+s\[(\d+):(\d+)\]", prev) or re.match(r"\s*(v_\S+)\s+s(\d+)\b", prev)
                if w:
                    d0 = int(w.group(2))
                    d1 = int(w.group(3)) if (w.lastindex or 0) >= 3 else d0
                    assert not (d0 <= hi and d1 >= lo), (name, k, prev.strip(), line.strip())
    assert n_loads > 100   # the form is in use (dense forward, both backward kernels, cross-entropy)


def test_tile_loop_kernels_keep_their_state_in_registers(saddr_sources):
    """A spilled vector register is reloaded through vector memory, and the wait
    the compiler puts in front of its use also drains the tile loads that are
    meant to stay in flight.  The forward, backward and cross-entropy forward
    kernels must not spill; the cross-entropy gradient variant is known to
    (a few values around its epilogue) and is bounded instead."""
    seen = 0
    for name, text in saddr_sources.items():
        for block in text.split("- .agpr_count:")[1:]:
            kern = re.search(r"\.name:\s+(\S+)", block).group(1)
            spills = int(re.search(r"\.vgpr_spill_count:\s+(\d+)", block).group(1))
            seen += 1
            if "xent_gemm_kernel" in kern and kern.rstrip("E").endswith("Lb1EEEvNS_10XentParams"):
                assert spills <= 24, (kern, spills)
            else:
                assert spills == 0, (kern, spills)
    assert seen >= 30   # six instantiations of each attention kernel and more
