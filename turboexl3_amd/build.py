"""Builds libturboexl3_hip.so for gfx950 with hipcc, in-tree (turboexl3_amd/lib/).

    python -m turboexl3_amd.build [--force]

Cross-compiles without a GPU. Every HIP translation unit gets the packed-fp32 feature switched off.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libturboexl3_hip.so")

HIP_SOURCES = ["t3_dense.hip", "t3_dequant.hip", "t3_gemm.hip", "t3_moe.hip", "t3_prefill.hip", "t3_unrot.hip"]
HOST_SOURCES = ["t3_api.cpp", "t3_linear.cpp", "t3_moe.cpp", "t3_table.cpp"]

ARCH = "gfx950"
COMMON = ["-O3", "-std=c++20", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-function"]
# -amdgpu-mfma-vgpr-form: MFMA accumulators stay in VGPRs (these kernels need no AGPRs; the default shuffles
# accumulators through AGPR copies every loop iteration)
# -fma-mix-insts: no v_fma_mixlo_f16. The compiler folds f16(fma(a, b, c)) into that instruction where the fma's result
# has no other use, and the instruction rounds once where the two it replaces round twice (to f32, then to f16, as the
# format's own arithmetic does): whether a value met the fold depended on the code around it, and the same statements
# gave different bytes in different kernels (the routed chain's two-launch and five-launch forms, MUL1's map).
HIP_FLAGS = [f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Xclang", "-target-feature", "-Xclang", "-fma-mix-insts", "-mllvm", "-amdgpu-mfma-vgpr-form"]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _headers_mtime() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))]
    paths.append(os.path.join(HERE, "..", "include", "turboexl3_hip.h"))
    return max(os.path.getmtime(p) for p in paths)


# No kernel here may use scratch memory (a register spill, or a local array the compiler could not keep in registers):
# the GEMM that issues its loads from inline asm and waits with s_waitcnt vmcnt(N) counts them itself, and a spill would
# put the compiler's scratch loads and stores into the same counter; everywhere else scratch means a slower wave launch
# and memory traffic in a latency-bound chain. The build reads the compiler's resource remarks and fails on any.
def _check_no_scratch(src: str, remarks: str) -> None:
    name = None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif name and ("ScratchSize" in line or "VGPRs Spill" in line):
            if int(line.split(":")[-1].split()[0]) != 0:
                raise RuntimeError(f"{src}: {name} uses scratch memory ({line.strip()})")


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJDIR, src + ".o")
    path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), _headers_mtime()):
        return obj
    # T3_EXTRA_HIPCC_FLAGS: build-time switches of the measured variants (e.g. -DT3_GEMV_LDS_RING_FROM=0)
    extra = os.environ.get("T3_EXTRA_HIPCC_FLAGS", "").split()
    cmd = [hipcc(), "-x", "hip", *COMMON, *HIP_FLAGS, *extra, "-c", path, "-o", obj]
    cmd[-4:-4] = ["-Rpass-analysis=kernel-resource-usage", "-fno-caret-diagnostics"]  # remarks without source lines
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "fma-mix-insts" not in l and "kernel-resource-usage" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    _check_no_scratch(src, res.stderr)
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int = 8) -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    sources = HIP_SOURCES + HOST_SOURCES
    with cf.ThreadPoolExecutor(max_workers=min(jobs, len(sources))) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), sources))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB, *objs]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n" + res.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
