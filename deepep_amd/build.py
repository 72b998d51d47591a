"""Compile the HIP sources for gfx950 into deepep_amd/libdeepep_amd.so (in-tree).

Usage: ``python -m deepep_amd.build``.  hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libdeepep_amd.so")
SOURCES = ("runtime.hip", "layout.hip", "dispatch.hip", "combine.hip", "megamoe.hip")
FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # plain IEEE arithmetic: correctly rounded fp32 divide, no contraction, no packed-fp32 forms
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # Registers that do not fit go to the stack, never into spare accumulation registers: the grouped GEMM keeps weight
    # fragments in accumulation registers that the compiler does not know to be in use (see csrc/megamoe.hip).
    "-mllvm", "-amdgpu-spill-vgpr-to-agpr=0",
)
# Per-file additions.  megamoe.hip: with the register allocator's default order of local assignments the 192-row GEMM
# kernels put loop-carried addresses on the stack although half the register file is free (every reload then waits for
# all the copies in flight); in reverse order nothing is spilled.  tests/test_gemm_registers.py checks the result.
FILE_FLAGS = {"megamoe.hip": ("-mllvm", "-greedy-reverse-local-assignment=1")}


def _hipcc():
    for candidate in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if candidate and (os.path.isabs(candidate) and os.path.exists(candidate) or not os.path.isabs(candidate)):
            return candidate
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(name):
        obj = os.path.join(objdir, name.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *FILE_FLAGS.get(name, ()), "-c", os.path.join(CSRC, name), "-o", obj]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {name}:\n{proc.stdout}\n{proc.stderr}")
        if verbose and proc.stderr.strip():
            noise = "is not a recognized feature for this target"
            kept = [line for line in proc.stderr.splitlines() if noise not in line]
            if kept:
                print("\n".join(kept), file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objects]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
