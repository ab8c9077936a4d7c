"""Static check of the GEMM kernels' ISA (no GPU needed: hipcc cross-compiles).

The scale-accumulate MFMA of csrc/jf_gemm.hip is written as inline asm (its accumulator input has to be an inline
constant), so the compiler's hazard recogniser does not know it is an MFMA.  A vector instruction that reads or
writes an MFMA's destination registers needs up to 19 wait states after the MFMA issues; the kernel guarantees
them by program order (the result is consumed one accumulation later).  This test compiles the file to assembly
and verifies that guarantee for every such MFMA in every instantiation, and that the kernels do not spill in
their main loops."""
import os
import re
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "jetfire-int8training_amd")
WAIT_STATES = 19


def _regs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


@pytest.fixture(scope="module")
def gemm_isa(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    sys.path.insert(0, PKG)
    import build_ext
    out = tmp_path_factory.mktemp("isa") / "jf_gemm.s"
    flags = [f for f in build_ext.HIP_FLAGS if f not in ("-shared", "-fPIC")]
    subprocess.check_call([hipcc] + flags + ["-S", "--cuda-device-only", "-o", str(out),
                                             os.path.join(PKG, "csrc", "jf_gemm.hip")], stderr=subprocess.DEVNULL)
    return out.read_text().split("\n")


def test_asm_mfma_results_are_not_touched_too_early(gemm_isa):
    lines = gemm_isa
    found = 0
    for i, line in enumerate(lines):
        code = line.split(";")[0]
        if "v_mfma" not in code or "0x3e22f983" not in code:
            continue
        found += 1
        dst = _regs(code.split(",")[0])
        ws, j = 0, i + 1
        while ws < WAIT_STATES and j < len(lines):
            t = lines[j].split(";")[0].strip()
            j += 1
            if not t or t.startswith(".") or t.endswith(":"):
                continue
            m = re.match(r"s_nop (\d+)", t)
            if m:
                ws += int(m.group(1)) + 1
                continue
            assert not t.startswith(("s_branch", "s_cbranch", "s_endpgm", "s_setpc")), \
                f"line {i + 1}: control flow {t!r} within {WAIT_STATES} wait states of an asm MFMA"
            assert not (_regs(t) & dst), f"line {i + 1}: {code.strip()!r} -> line {j}: {t!r} touches its destination"
            ws += 1
    assert found >= 16, "the scale-accumulate MFMAs were not found (did the kernel change?)"


def test_main_loops_do_not_spill(gemm_isa):
    """Scratch accesses are tolerated outside loops (a few values parked across the K loop in the binary16-scale
    kernels), never inside one."""
    in_loop_depth = None
    for i, line in enumerate(gemm_isa):
        m = re.search(r"Loop Header: Depth=(\d+)|in Loop: Header=\S+ Depth=(\d+)", line)
        if re.match(r"^\.LBB\d+_\d+:", line):
            in_loop_depth = int(m.group(1) or m.group(2)) if m else None
        if in_loop_depth and re.match(r"\s*scratch_(load|store)", line):
            raise AssertionError(f"line {i + 1}: scratch access inside a loop: {line.strip()}")
