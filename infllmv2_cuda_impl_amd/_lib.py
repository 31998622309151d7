"""ctypes binding of libinfllmv2_hip.so (declared in include/infllmv2_hip.h).

The library is the only compute path: if it is missing or fails to load, importing this module
raises.  There is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libinfllmv2_hip.so")

ABI_VERSION = 11

_p, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> argtypes; every function returns int except the three noted below
SIGNATURES = {
    "infllmv2_check_device": [_i],
    "infllmv2_topk_to_uint64": [_p, _p, _p, _i64, _i, _i, _i],
    "infllmv2_uint64_to_bool": [_p, _p, _p, _i64, _i, _i],
    "infllmv2_blockmask_to_uint64": [_p, _p, _p, _i64, _i, _i],
    "infllmv2_transpose_blockmask": [_p, _p, _p, _i, _i64, _i, _i, _i],
    "infllmv2_max_pooling_1d": [_p, _p, _p] + [_i] * 12,
    "infllmv2_max_pooling_1d_strided": [_p, _p, _p, _i, _i, _i, _i, _i64, _i64] + [_i] * 8,
    "infllmv2_max_pooling_1d_varlen": [_p, _p, _p, _p, _p, _p] + [_i] * 12,
    "infllmv2_max_pooling_1d_varlen_strided": [_p, _p, _p, _p, _p, _p] + [_i] * 6 + [_i64, _i64] + [_i] * 7,
    "infllmv2_topk": [_p, _i, _i, _i, _i, _p, _p, _p],
    "infllmv2_topk_blocks": [_p, _p, _i64, _p, _i64, _i, _i],
    "infllmv2_topk_select": [_p, _p, _i64, _i, _p, _p, _i64, _i, _i, _i, _i, _i],
    "infllmv2_compress_keys": [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i, _i, _i],
    "infllmv2_compress_keys_cache": [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _p, _p, _i, _i, _i, _i],
    "infllmv2_compress_keys_cache_pair": [_p] * 8 + [_i] * 5 + [_p] * 3 + [_i] * 7,
    "infllmv2_varlen_fwd_stage1": [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i64, _i, _i, _i, _i, _i, _p, _p, _p, _i64, _i64, _f, _i],
    "infllmv2_varlen_fwd_stage1_pooled": [_p] * 9 + [_i, _i, _i64, _i, _i, _i, _i, _i, _p, _p, _p, _i, _f] + [_i] * 7,
    "infllmv2_stage1_decode": [_p] * 11 + [_sz] + [_i] * 6 + [_p] * 3 + [_i64, _i64, _f, _i, _i, _p] + [_i] * 8,
    "infllmv2_varlen_fwd": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _i, _i, _i64, _i64, _i, _i, _i, _i, _i,
                            _p, _p, _p, _p, _p, _i, _f, _i],
    "infllmv2_varlen_bwd": [_p] * 14 + [_sz, _i, _i64, _i64, _i, _i, _i, _i, _i] + [_p] * 9 + [_i, _f, _i, _i],
    "infllmv2_fwd_kvcache": [_p] * 11 + [_sz] + [_i] * 7 + [_p] * 6 + [_i, _i, _f, _p, _p, _p, _i64, _i, _p, _p, _i, _i],
    "infllmv2_fwd_kvcache_static": [_p] * 10 + [_i] * 7 + [_p] * 6 + [_i, _i, _f, _p, _p, _p, _i64, _i, _p, _p, _i, _i],
    "infllmv2_pack_kv": [_p, _p, _p, _p, _p, _sz, _i, _i64, _i, _i, _i, _p, _p],
}
# entry points that exist once per element type: the plain name takes bfloat16, name + "_f16" IEEE half
PER_ELEMENT_TYPE = ["infllmv2_compress_keys", "infllmv2_compress_keys_cache", "infllmv2_compress_keys_cache_pair", "infllmv2_varlen_fwd_stage1",
                    "infllmv2_varlen_fwd_stage1_pooled", "infllmv2_stage1_decode", "infllmv2_varlen_fwd",
                    "infllmv2_varlen_bwd", "infllmv2_fwd_kvcache"]
for _name in PER_ELEMENT_TYPE:
    SIGNATURES[_name + "_f16"] = SIGNATURES[_name]
OTHER = {
    "infllmv2_last_error": (C.c_char_p, []),
    "infllmv2_abi_version": (_i, []),
    "infllmv2_kv_image_bytes": (_sz, [_i64, _i, _i]),
    "infllmv2_stage1_decode_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "infllmv2_fwd_kvcache_workspace_bytes": (_sz, [_i, _i, _i]),
    "infllmv2_fwd_kvcache_num_splits": (_i, [_i, _i, _i]),
    "infllmv2_varlen_bwd_workspace_bytes": (_sz, [_i, _i64, _i64, _i, _i]),
    "infllmv2_varlen_bwd_deterministic_workspace_bytes": (_sz, [_i, _i64, _i64, _i, _i]),
}


def exported_names():
    return sorted(list(SIGNATURES) + list(OTHER))


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python infllmv2_cuda_impl_amd/csrc/build.py` "
            "(hipcc, --offload-arch=gfx950). There is no fallback path.")
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _i
    for name, (res, argtypes) in OTHER.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = res
    if lib.infllmv2_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI {lib.infllmv2_abi_version()}, expected {ABI_VERSION}; rebuild it")
    return lib


lib = _load()


def call(name: str, *args) -> None:
    """Call an int-returning entry point and raise RuntimeError with the library's message on failure."""
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(lib.infllmv2_last_error().decode("utf-8", "replace") or f"{name} failed with code {rc}")


def call_for(dtype, name: str, *args) -> None:
    """`call` of the instantiation of a per-element-type entry point for torch dtype `dtype` (bfloat16 or float16)."""
    import torch
    if dtype == torch.bfloat16:
        call(name, *args)
    elif dtype == torch.float16:
        call(name + "_f16", *args)
    else:
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")


def i64_array(values):
    return (C.c_int64 * len(values))(*[int(v) for v in values])
