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


def _recognised(asm: str, kernel_substring: str) -> None:
    """Skips the calling test when the assembly does not look like what these parsers were written against (another
    compiler release may name labels or annotate loops differently): a difference of the toolchain, not of the kernels."""
    kernels = [m.group(1) for m in re.finditer(r"^(_Z\w+):", asm, flags=re.M) if kernel_substring in m.group(1)]
    anchors = {"kernel labels": bool(kernels), "loop annotations": "Loop Header" in asm, "wait counters": "s_waitcnt" in asm,
               "end of program": "s_endpgm" in asm}
    missing = [name for name, ok in anchors.items() if not ok]
    if missing:
        pytest.skip("compiler output format not recognised (toolchain differs): no " + ", ".join(missing)
                    + f" found for {kernel_substring}")


def _loops_with_full_waits(asm: str, kernel_substring: str):
    """[(kernel, loop length in lines, offsets of full waits)] for every loop of every matching kernel.  A loop is its
    header block plus every block the compiler annotates as lying in it, wherever the block was placed (a rotated loop
    has its latch in front of the header and jumps back to the latch, not to the header)."""
    loops = {}                                               # (kernel, header) -> [lines, offsets of full waits]
    order = []
    kernel, current = None, None
    for line in asm.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, current = (m.group(1) if kernel_substring in m.group(1) else None), None
            continue
        if kernel is None:
            continue
        m = re.match(r"^\.L(BB\d+_\d+):(.*)$", line)
        if m:
            label, note = m.group(1), m.group(2)
            inside = re.search(r"in Loop: Header=(BB\d+_\d+)", note)
            current = (kernel, label) if "Loop Header" in note else (kernel, inside.group(1)) if inside else None
            if current is not None and current not in loops:
                loops[current] = [0, []]
                order.append(current)
            continue
        if current is not None:
            loops[current][0] += 1
            if "s_waitcnt" in line and re.search(r"vmcnt\(0\)", line):
                loops[current][1].append(loops[current][0])
        if "s_endpgm" in line and current is None:
            pass
    return [(k[0], loops[k][0], loops[k][1]) for k in order]


@pytest.mark.parametrize("source, kernel, min_kernels", [
    ("int4.hip", "int4_gemm_kernel", 24),
    ("dense.hip", "dense_gemm_kernel", 12),
])
def test_main_loops_never_wait_for_every_request(source, kernel, min_kernels, tmp_path):
    asm = _assembly(os.path.join(build_mod.CSRC, source), tmp_path)
    _recognised(asm, kernel)
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
    _recognised(asm, "int4_rows8_kernel")
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


def test_the_long_k_8_row_kernel_refills_its_registers_without_draining_them(tmp_path):
    """int4_rows8_long_kernel requests a step's weight words for the next round into the registers the step has just
    emptied.  Requested while the old words are still wanted they land in other registers, and the copy back at the
    end of the round waits for every request in flight -- a round trip per round that no result shows.  The loop must
    therefore hold no full wait, every wait inside it must leave at least the other steps' requests outstanding, and
    nothing may live in scratch memory."""
    asm = _assembly(os.path.join(build_mod.CSRC, "int4.hip"), tmp_path)
    _recognised(asm, "int4_rows8_long_kernel")
    bodies = _kernel_bodies(asm, "int4_rows8_long_kernel")
    assert len(bodies) >= 2, "the parser found too few kernel variants"
    for kernel, lines in bodies.items():
        assert not any("scratch_" in l for l in lines), f"{kernel} uses scratch memory"
    loops = [l for l in _loops_with_full_waits(asm, "int4_rows8_long_kernel") if l[1] >= 100]
    assert len({l[0] for l in loops}) >= 2, "the parser found no round loop"
    stalled = [(k, n, w) for k, n, w in loops if w]
    assert not stalled, "a full wait inside the round loop of: " + ", ".join(f"{k} (at {w})" for k, n, w in stalled)


def test_the_attention_kernels_keep_their_requests_in_flight(tmp_path):
    """The 32 x 32 attention kernels keep K / V requests of later blocks on their way while a block is multiplied: the
    ping-pong kernel through copies into LDS that it waits for by hand (vmcnt(4): the newest block stays outstanding),
    the plain kernel through two register sets.  A wait for EVERY request inside the block loop (the compiler adds one
    as soon as a request is issued on one path only, or a global load appears in the loop) serialises them again; so
    does anything living in scratch memory."""
    asm = _assembly(os.path.join(build_mod.CSRC, "attention.hip"), tmp_path)
    for kernel, min_kernels in (("tree_attention_pp_kernel", 4), ("tree_attention32_kernel", 8)):
        _recognised(asm, kernel)
        bodies = _kernel_bodies(asm, kernel)
        assert len(bodies) >= min_kernels, f"the parser found too few variants of {kernel}"
        for name, lines in bodies.items():
            assert not any("scratch_" in l for l in lines), f"{name} uses scratch memory"
        loops = [l for l in _loops_with_full_waits(asm, kernel) if l[1] >= 200]      # the block loop
        contiguous = [l for l in loops if "Lb1E" not in l[0]]                     # paged variants look up pages in the loop
        assert len({l[0] for l in contiguous}) >= min_kernels // 2, f"the parser found too few block loops of {kernel}"
        stalled = [(k, n, w) for k, n, w in contiguous if w]
        assert not stalled, "a full wait inside the block loop of: " + ", ".join(f"{k} (at {w})" for k, n, w in stalled)


def test_the_wide_dense_kernel_waits_only_where_it_says(tmp_path):
    """dense_wide_kernel copies weights and activations straight into LDS rings with requests the compiler does not know
    about, and waits for them by hand: the weight wavefronts for all but the newest chunks of their ring, the activation
    wavefronts likewise.  Any other wait for vector memory inside a K loop (the compiler adds one, for EVERY request, as
    soon as it sees a request of its own there) would drain the rings once per chunk; accumulators in scratch memory
    would do worse."""
    asm = _assembly(os.path.join(build_mod.CSRC, "dense.hip"), tmp_path)
    _recognised(asm, "dense_wide_kernel")
    bodies = _kernel_bodies(asm, "dense_wide_kernel")
    assert len(bodies) >= 12, "the parser found too few kernel variants"            # 3 shapes x SwiGLU or not x 2 dtypes
    for kernel, lines in bodies.items():
        assert not any("scratch_" in l for l in lines), f"{kernel} uses scratch memory"
        # template arguments <DT, WM, MG, NTMAX, SW, SX, NWW, WPER, NXW, XPER, SILU> from the mangled name
        args = [int(a) for a in re.findall(r"Li(\d+)E", kernel)]
        assert len(args) >= 10, kernel
        sw, sx, wper, xper = args[4], args[5], args[7], args[9]
        expected = {(sw - 2) * wper, (sx - 2) * xper}
        in_loop = [l for l in lines if "v_mfma" in l or "vmcnt" in l]
        first, last = next(i for i, l in enumerate(in_loop) if "v_mfma" in l), max(i for i, l in enumerate(in_loop) if "v_mfma" in l)
        waits = {int(m.group(1)) for l in in_loop[first:last] for m in [re.search(r"vmcnt\((\d+)\)", l)] if m}
        assert waits and waits <= expected, f"{kernel}: waits {sorted(waits)} between its products, expected {sorted(expected)}"


def test_no_hand_written_vector_instruction_sits_next_to_an_mfma():
    """With MFMA results kept in ordinary vector registers (-amdgpu-mfma-vgpr-form=1) the compiler inserts the wait
    states between an MFMA and the vector ALU instruction that reads its result, but only for instructions it emitted
    itself: a vector ALU instruction written as inline assembly is opaque to that pass and has read half-written
    accumulators.  The kernels therefore contain no vector ALU instruction as assembly TEXT -- asm statements are empty
    ones that only pin a value to a register class (the constants of v_and_or_b32 are made opaque by arithmetic on
    run-time values instead), waits, and the attention kernel's copies from memory into LDS (which the compiler must NOT
    know about: it would wait for all of them before every LDS read) -- and this test keeps it that way."""
    pattern = re.compile(r"\basm\s*(?:volatile)?\s*\(\s*\"([^\"]*)\"")
    allowed = re.compile(r"^(s_waitcnt\b|s_mov_b32 m0,|global_load_lds_dwordx4\b)")
    seen = 0
    for name in sorted(os.listdir(build_mod.CSRC)):
        if not name.endswith((".hip", ".h")):
            continue
        with open(os.path.join(build_mod.CSRC, name)) as f:
            text = f.read()
        for m in pattern.finditer(text):
            seen += 1
            line = text.count("\n", 0, m.start()) + 1
            for instruction in re.split(r"\\n|\\t|;", m.group(1)):
                instruction = instruction.strip()
                assert instruction == "" or allowed.match(instruction), \
                    f"{name}:{line}: inline assembly with instruction text: {instruction!r}"
    assert seen >= 10, "the pattern no longer finds the register-class pins"
