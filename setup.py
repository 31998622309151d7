"""Packaging for the MI355X build of infllm_v2.

``pip install -e .`` (or ``python setup.py build_py``) compiles the HIP sources for gfx950 with hipcc into
``infllmv2_cuda_impl_amd/libinfllmv2_hip.so`` and installs two packages: ``infllmv2_cuda_impl_amd`` (the operators)
and ``infllm_v2`` (the reference's package name, re-exporting them).  No network access and no torch extension
build are involved: the library is a plain C-ABI shared object loaded with ctypes.
"""
import importlib.util
import os

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))


class BuildWithHip(build_py):
    def run(self):
        spec = importlib.util.spec_from_file_location(
            "infllmv2_build", os.path.join(ROOT, "infllmv2_cuda_impl_amd", "csrc", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build(verbose=True)
        mod.build_torch_module(verbose=True)
        # the sources include the C-ABI header by name: ship a copy inside the package so that an installed copy
        # can be rebuilt without the repository root
        import shutil
        dst = os.path.join(ROOT, "infllmv2_cuda_impl_amd", "include")
        os.makedirs(dst, exist_ok=True)
        shutil.copy2(os.path.join(ROOT, "include", "infllmv2_hip.h"), os.path.join(dst, "infllmv2_hip.h"))
        super().run()


setup(
    name="infllm_v2",
    version="0.1.0",
    description="InfLLM-V2 two-stage sparse attention for AMD MI355X (gfx950): hand-written HIP kernels behind a C ABI",
    packages=["infllmv2_cuda_impl_amd", "infllm_v2"],
    package_data={"infllmv2_cuda_impl_amd": ["libinfllmv2_hip.so", "_C*.so", "csrc/*.cpp", "csrc/*.hip", "csrc/*.h", "csrc/build.py", "include/*.h"]},
    include_package_data=True,
    python_requires=">=3.9",
    cmdclass={"build_py": BuildWithHip},
)
