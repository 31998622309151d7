"""The C-ABI library loads and exports every symbol that include/infllmv2_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "infllmv2_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(infllmv2_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported():
    names = _declared()
    assert len(names) >= 10
    lib = ctypes.CDLL(os.path.join(ROOT, "infllmv2_cuda_impl_amd", "libinfllmv2_hip.so"))
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared but not exported: {missing}"


def test_python_binding_matches_header():
    from infllmv2_cuda_impl_amd import _lib
    assert sorted(_lib.exported_names()) == _declared()
    assert _lib.lib.infllmv2_abi_version() == _lib.ABI_VERSION


def test_argument_errors_are_reported_without_gpu():
    """Host-side validation runs before any launch, so it can be exercised on a CPU-only box."""
    from infllmv2_cuda_impl_amd import _lib
    rc = _lib.lib.infllmv2_uint64_to_bool(None, None, None, 4, 200, 1)       # 1 word cannot hold 200 bits
    assert rc != 0
    assert b"cannot hold" in _lib.lib.infllmv2_last_error()
    rc = _lib.lib.infllmv2_topk_blocks(None, None, 9000, None, 1, 9000, 4)
    assert rc != 0 and b"exceeds" in _lib.lib.infllmv2_last_error()


def test_product_package_does_not_import_oracle():
    pkg = os.path.join(ROOT, "infllmv2_cuda_impl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src, f"{f} mentions the oracle"
