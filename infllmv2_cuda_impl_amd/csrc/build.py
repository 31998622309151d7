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


def include_dir() -> str:
    """Directory that holds infllmv2_hip.h, the C-ABI header the sources include by name: `include/` beside the
    package in a source checkout, `include/` inside the package where it was installed from a built distribution
    (setup.py copies the header there)."""
    for cand in (os.path.join(PKG, "include"), os.path.join(os.path.dirname(PKG), "include")):
        if os.path.exists(os.path.join(cand, "infllmv2_hip.h")):
            return cand
    raise RuntimeError("infllmv2_hip.h not found: expected in " + os.path.join(PKG, "include") + " or "
                       + os.path.join(os.path.dirname(PKG), "include"))

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffast-math", "-fno-finite-math-only", *os.environ.get("IV2_EXTRA_FLAGS", "").split(),
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value", "-Wno-inline-asm",
    # keep MFMA accumulators in ordinary VGPRs: the default AGPR form makes this compiler shuffle accumulators
    # through v_accvgpr_read/write around every MFMA whose result the VALU touches
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


# translation units that hold attention kernels: compiled twice, for bfloat16 (plain entry-point names) and, with
# -DIV2_F16, for IEEE half (entry points with the suffix _f16); the other files are element-type independent or take
# the type at run time
PER_ELEMENT_TYPE = {"compress.hip", "decode.hip", "stage1.hip", "stage1_decode.hip", "stage2_bwd.hip",
                    "stage2_bwd_dkdv.hip", "stage2_bwd_dq.hip", "stage2_fwd.hip",
                    "stage2_fwd_hybrid.hip"}


def sources():
    """(source file, extra flags, object name) of every compilation."""
    out = []
    for f in sorted(f for f in os.listdir(CSRC) if f.endswith(".hip")):
        out.append((f, [], f[:-4] + ".o"))
        if f in PER_ELEMENT_TYPE:
            out.append((f, ["-DIV2_F16=1"], f[:-4] + "_f16.o"))
    return out


def _compile(unit, verbose: bool) -> str:
    src, extra, obj_name = unit
    obj = os.path.join(OBJ_DIR, obj_name)
    cmd = ["hipcc", *HIPCC_FLAGS, "-I", include_dir(), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
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


TORCH_MODULE = "_C"


def torch_module_path() -> str:
    import sysconfig
    return os.path.join(PKG, TORCH_MODULE + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_torch_module(verbose: bool = True) -> str:
    """Compiles csrc/torch_module.cpp, the native module `infllmv2_cuda_impl_amd._C` (`infllm_v2.C`): host code only
    (pybind11 + ATen for tensors and the current stream) that links against libinfllmv2_hip.so beside it."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce
    out = torch_module_path()
    torch_lib = ce.library_paths()[0]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-DTORCH_EXTENSION_NAME={TORCH_MODULE}", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch.compiled_with_cxx11_abi())}",
           *[f"-I{d}" for d in ce.include_paths()], "-I", sysconfig.get_paths()["include"], "-I", "/opt/rocm/include",
           "-I", include_dir(), os.path.join(CSRC, "torch_module.cpp"), "-o", out,
           f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", f"-L{PKG}", "-linfllmv2_hip",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the torch module failed:\n" + r.stderr)
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build()
    build_torch_module()
