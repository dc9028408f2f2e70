"""The software pipelines of the linear kernels, checked in the compiler's assembly output.

The int4 and dense GEMM kernels keep weight and activation requests several 64-k groups ahead of their use.
That distance exists only while no instruction inside the main loop waits for EVERY outstanding request
(``s_waitcnt vmcnt(0)``): one such wait per trip turns the prefetch back into load - wait - use.  The compiler
inserts it whenever a loop-carried register slot is loaded while its old contents are still being read (the
new value then lives in other registers and is copied into the slot at the end of the body, behind a full
wait), which no test of results can see.  This test compiles the two sources to assembly with the build's own
flags and looks at every loop of every GEMM kernel variant.
"""
import os
import re
import shutil
import subprocess

import pytest

from subspec_amd import build as build_mod


_ASSEMBLY = {}                                               # source path -> assembly text (one compilation per run)


def _assembly(src: str, tmp_path) -> str:
    if src not in _ASSEMBLY:
        _ASSEMBLY[src] = _compile_to_assembly(src, tmp_path)
    return _ASSEMBLY[src]


def _compile_to_assembly(src: str, tmp_path) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    out = str(tmp_path / (os.path.basename(src) + ".s"))
    flags = [f for f in build_mod.HIPCC_FLAGS if f != "-fPIC"]
    subprocess.run([hipcc, *flags, "-S", "--cuda-device-only", "-w", src, "-o", out], check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=600)
    with open(out) as f:
        return f.read()


def _loops_with_full_waits(asm: str, kernel_substring: str):
    """[(kernel, loop length in lines, offsets of full waits)] for every loop of every matching kernel."""
    found = []
    kernel = None
    open_loops = {}                                          # label -> (first line, offsets of full waits)
    for i, line in enumerate(asm.split("\n")):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, open_loops = m.group(1), {}
            continue
        if kernel is None or kernel_substring not in kernel:
            continue
        m = re.match(r"^(\.LBB\d+_\d+):.*Loop Header", line)
        if m:
            open_loops[m.group(1)] = (i, [])
        if "s_waitcnt" in line and re.search(r"vmcnt\(0\)", line):
            for start, waits in open_loops.values():
                waits.append(i - start)
        m = re.search(r"\bs_c?branch\w*\s+(\.LBB\d+_\d+)\b", line)
        if m and m.group(1) in open_loops:
            start, waits = open_loops.pop(m.group(1))
            found.append((kernel, i - start, waits))
    return found


@pytest.mark.parametrize("source, kernel, min_kernels", [
    ("int4.hip", "int4_gemm_kernel", 24),
    ("dense.hip", "dense_gemm_kernel", 12),
])
def test_main_loops_never_wait_for_every_request(source, kernel, min_kernels, tmp_path):
    asm = _assembly(os.path.join(build_mod.CSRC, source), tmp_path)
    loops = _loops_with_full_waits(asm, kernel)
    main_loops = [l for l in loops if l[1] >= 40]            # the pipelined loop; short loops are epilogue code
    assert len({l[0] for l in main_loops}) >= min_kernels, "the parser found too few kernel variants"
    stalled = [(k, n, w) for k, n, w in main_loops if w]
    assert not stalled, "a full wait inside the pipelined loop of: " + ", ".join(
        f"{k} (loop of {n} lines, at {w})" for k, n, w in stalled)


def _kernel_bodies(asm: str, kernel_substring: str):
    """{kernel: lines of its body} for every matching kernel."""
    bodies, kernel = {}, None
    for line in asm.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel = m.group(1) if kernel_substring in m.group(1) else None
            if kernel:
                bodies[kernel] = []
            continue
        if kernel:
            bodies[kernel].append(line)
            if "s_endpgm" in line:
                kernel = None
    return bodies


def test_the_8_row_kernel_keeps_its_requests_in_order_and_its_registers(tmp_path):
    """int4_rows8_kernel issues every request before its first wait and relies on three things no result can show:
    the activation blocks are requested before any weight word (vector memory returns in order, so a block requested
    after the weights could only be waited for together with them), the steps stream (their waits leave later requests
    outstanding), and nothing lives in scratch memory (without a pin the compiler sinks the accumulator updates of the
    two-round variants below the last MFMA and spills every raw product)."""
    asm = _assembly(os.path.join(build_mod.CSRC, "int4.hip"), tmp_path)
    bodies = _kernel_bodies(asm, "int4_rows8_kernel")
    assert len(bodies) >= 20, "the parser found too few kernel variants"
    for kernel, lines in bodies.items():
        assert not any("scratch_" in l for l in lines), f"{kernel} uses scratch memory"
        loads = [(i, l) for i, l in enumerate(lines) if re.search(r"\bbuffer_load_dword", l)]
        x_loads = [i for i, l in loads if "dwordx4" in l]                # activation blocks (and the gain piece)
        w_loads = [i for i, l in loads if "dwordx2" in l]                # weight words
        assert x_loads and w_loads, kernel
        assert max(x_loads) < min(w_loads), f"{kernel}: an activation block is requested after a weight word"
        first_mfma = next(i for i, l in enumerate(lines) if "v_mfma" in l)
        waits = [int(m.group(1)) for l in lines[:first_mfma + 40] for m in [re.search(r"vmcnt\((\d+)\)", l)] if m]
        # the wait in front of the first product leaves the weight words of the later steps on their way
        assert waits and min(waits) >= 4, f"{kernel}: the first step waits for (nearly) every request: {sorted(set(waits))}"


def test_no_hand_written_instruction_sits_next_to_an_mfma():
    """With MFMA results kept in ordinary vector registers (-amdgpu-mfma-vgpr-form=1) the compiler inserts the wait
    states between an MFMA and the vector ALU instruction that reads its result, but only for instructions it emitted
    itself: a vector ALU instruction written as inline assembly is opaque to that pass and has read half-written
    accumulators.  The kernels therefore contain no assembly TEXT at all -- every asm statement is an empty one that
    only pins a value to a register class (the constants of v_and_or_b32 are made opaque by arithmetic on run-time
    values instead) -- and this test keeps it that way."""
    pattern = re.compile(r"\basm\s*(?:volatile)?\s*\(\s*\"([^\"]*)\"")
    seen = 0
    for name in sorted(os.listdir(build_mod.CSRC)):
        if not name.endswith((".hip", ".h")):
            continue
        with open(os.path.join(build_mod.CSRC, name)) as f:
            text = f.read()
        for m in pattern.finditer(text):
            seen += 1
            line = text.count("\n", 0, m.start()) + 1
            assert m.group(1).strip() == "", f"{name}:{line}: inline assembly with instruction text: {m.group(1)!r}"
        assert "__asm__" not in text, f"{name}: __asm__ spelling is not covered by this check"
    assert seen >= 8, "the pattern no longer finds the register pins it is meant to inspect"
    assert "-amdgpu-mfma-vgpr-form=1" in build_mod.HIPCC_FLAGS
