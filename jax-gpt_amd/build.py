"""Builds libmoe_hip.so (the C-ABI library of HIP kernels) for gfx950 with hipcc.

Run on the CPU host: hipcc cross-compiles without a GPU.  The library is written
next to this file so that it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libmoe_hip.so")
# the timing probe of the grouped GEMM's K loop (`python bench.py --probe`): its own library, nothing of the product links it
PROBE_PATH = os.path.join(HERE, "libmoe_probe.so")

SOURCES = ["moe_api.hip", "moe_route.hip", "moe_router.hip", "moe_permute.hip", "moe_quant.hip", "moe_gemm.hip",
           "moe_combine.hip"]
# no v_pk_*_f32 code generation (some packed-f32 forms misbehave on this hardware pool)
COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-fvisibility=hidden",    # only the functions include/moe_hip.h declares (MOE_API) are exported
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC]
# routing and combine promise individually rounded f32 operations (bit-reproducible on a CPU)
PER_FILE = {"moe_route.hip": ["-ffp-contract=off"], "moe_combine.hip": ["-ffp-contract=off"],
            "moe_router.hip": ["-ffp-contract=off", "-Wno-inline-asm"],
            # MFMA results go straight to VGPRs: the block-scale FMA consumes them on the vector ALU
            "moe_gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form", "-Wno-inline-asm"]}   # m0 is clobbered on purpose


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the MI355X kernels cannot be built")


def build(verbose: bool = True, jobs: int = 6) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc, *COMMON, *PER_FILE.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    probe = [hipcc, *COMMON, *PER_FILE["moe_gemm.hip"], "-shared", os.path.join(CSRC, "moe_probe.hip"), "-o", PROBE_PATH]
    if verbose:
        print(" ".join(probe), flush=True)
    procs.append(("moe_probe.hip", subprocess.Popen(probe, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    _drain(procs)
    return LIB_PATH


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if out:
            print(out, flush=True)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}")


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
