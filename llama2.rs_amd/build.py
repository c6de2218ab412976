"""Build libllama2_hip.so (HIP kernels + C ABI) for gfx950 with hipcc.

Cross-compiles without a GPU.  The library is written next to this file and
loaded from there by llama2_rs (ctypes); nothing is installed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libllama2_hip.so")

ARCH = "gfx950"
# -packed-fp32-ops off: v_pk_*_f32 forms are not used on this target.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", f"--offload-arch={ARCH}"]

SOURCES = {
    # file: extra flags
    "kernels_q4.hip": [],
    "kernels_q4_stream.hip": [],
    # MFMA accumulators in VGPRs: the per-group fold reads and writes them with plain FMAs
    "kernels_q4_gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    # the block kernels keep the reference's rounded-multiply-then-add where they restate it
    "kernels_misc.hip": ["-ffp-contract=off"],
    "kernels_attn.hip": ["-ffp-contract=off"],
    "host.cpp": ["-x", "hip", "-ffp-contract=off"],
    "textgen.cpp": ["-x", "hip", "-ffp-contract=off"],
}


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _compile(name: str, flags, verbose: bool) -> str:
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ, os.path.splitext(name)[0] + ".o")
    cmd = [hipcc(), *COMMON, *DEVICE_FLAGS, *flags, "-c", src, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {name}:\n{r.stdout}\n{r.stderr}")
    noise = "'-packed-fp32-ops' is not a recognized feature"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l and l.strip())
    if err and verbose:
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        objs = list(ex.map(lambda kv: _compile(kv[0], kv[1], verbose), SOURCES.items()))
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB + ".tmp", *objs, "-lpthread"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(LIB + ".tmp", LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
