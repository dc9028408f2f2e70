"""Builds libsubspec_hip.so (gfx950) in-tree with hipcc.  ``python -m subspec_amd.build``."""
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libsubspec_hip.so")

# -packed-fp32-ops is switched off on purpose: packed fp32 VALU forms are not used in this build.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results that feed vector ALU work stay in VGPRs instead of bouncing through AGPRs
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-result", "-Wno-inline-asm",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = True, jobs: int = 8) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    procs, objs = [], []
    for src in sources():
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = [hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        noise = "is not a recognized feature for this target"
        out = "\n".join(l for l in out.splitlines() if noise not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if out.strip():
            print(out)


if __name__ == "__main__":
    build()
    print("built", LIB_PATH)
