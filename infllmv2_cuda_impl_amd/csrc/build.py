"""Builds libinfllmv2_hip.so (gfx950 code objects + C ABI) in-tree with hipcc.

Run as ``python infllmv2_cuda_impl_amd/csrc/build.py`` (a plain script: it must work when no
library exists yet, so it does not import the package).  There is exactly one target architecture.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
LIB_PATH = os.path.join(PKG, "libinfllmv2_hip.so")
OBJ_DIR = os.path.join(PKG, "build")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffast-math", "-fno-finite-math-only", *os.environ.get("IV2_EXTRA_FLAGS", "").split(),
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value", "-Wno-inline-asm",
    # keep MFMA accumulators in ordinary VGPRs: the default AGPR form makes this compiler shuffle accumulators
    # through v_accvgpr_read/write around every MFMA whose result the VALU touches
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
    cmd = ["hipcc", *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True, jobs: int | None = None) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), sources()))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build()
