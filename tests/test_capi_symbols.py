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


def _err(lib):
    return lib.infllmv2_last_error().decode()


def test_new_entry_points_validate_before_launch():
    """Argument checks of the fused front end, the compressed-key kernel and the decode options run on the host."""
    import ctypes as C
    from infllmv2_cuda_impl_amd import _lib
    lib = _lib.lib
    i64 = _lib.i64_array
    fake = 0x1000                                           # a non-null, 16-byte aligned "pointer"; nothing is launched
    # fused Stage-1/pool: only the 5/4/1 window on 64-token blocks
    rc = lib.infllmv2_varlen_fwd_stage1_pooled(None, fake, fake, fake, fake, fake, fake, fake, None, 0, 1, 128, 32, 2, 128,
                                               128, 7, i64([4096, 128, 2048]), i64([256, 128]), i64([256, 128]), 2,
                                               0.088, 1, 9, 8, 1, 128, 1, 1)
    assert rc != 0 and "only the 5/4/1 window" in _err(lib)
    # Stage 1: head_dim, group size, alignment
    rc = lib.infllmv2_varlen_fwd_stage1(None, fake, fake, fake, fake, fake, fake, fake, 1, 128, 32, 2, 64, 128, 7,
                                        i64([4096, 128, 2048]), i64([256, 128]), i64([256, 128]), 896, 7, 0.088, 1)
    assert rc != 0 and "head_dim 128" in _err(lib)
    rc = lib.infllmv2_varlen_fwd_stage1(None, fake, fake, fake, fake, fake, fake, fake, 1, 128, 24, 2, 128, 128, 7,
                                        i64([4096, 128, 2048]), i64([256, 128]), i64([256, 128]), 896, 7, 0.088, 1)
    assert rc != 0 and "g * num_heads_k" in _err(lib)
    rc = lib.infllmv2_varlen_fwd_stage1(None, fake + 2, fake, fake, fake, fake, fake, fake, 1, 128, 32, 2, 128, 128, 7,
                                        i64([4096, 128, 2048]), i64([256, 128]), i64([256, 128]), 896, 7, 0.088, 1)
    assert rc != 0 and "16-byte aligned" in _err(lib)
    # compressed keys
    rc = lib.infllmv2_compress_keys(None, fake, fake, fake, fake, 1, 128, 2, 128, 256, 128, 0, 16, 0)
    assert rc != 0 and "must be positive" in _err(lib)
    rc = lib.infllmv2_compress_keys(None, None, fake, fake, fake, 1, 128, 2, 128, 256, 128, 32, 16, 0)
    assert rc != 0 and "null pointer" in _err(lib)
    # compressed-key caches: the row capacities are arguments of the entry point and are checked before any launch
    rc = lib.infllmv2_compress_keys_cache(None, fake, fake, None, fake, None, 2, 1, 2, 128, i64([262144, 256, 128]),
                                          i64([16384, 256, 128]), 32, 16, 1024, -1)
    assert rc != 0 and "negative cache capacity" in _err(lib)
    # decode: option conflicts carry the reference's messages (flash_api.cpp:1596, 1763, 1774)
    def kv(**o):
        a = dict(knew=None, cbi=None, lp=None, bt=None, page=0, cos=None, sin=None, rd=0)
        a.update(o)
        return lib.infllmv2_fwd_kvcache(None, fake, fake, fake, a["knew"], a["knew"], fake, fake, fake, None, fake, 1 << 20,
                                        1, 1, 32, 2, 128, 512, 1 if a["knew"] else 0, i64([4096, 128]),
                                        i64([131072, 256, 128]), i64([131072, 256, 128]), i64([256, 256, 128]),
                                        i64([256, 256, 128]), i64([4096, 128]), 0, 1, 0.088, a["cbi"], a["lp"], a["bt"],
                                        8 if a["bt"] else 0, a["page"], a["cos"], a["sin"], a["rd"], 1)
    assert kv(bt=fake, page=256, cbi=fake) != 0 and "does not support cache_batch_idx" in _err(lib)
    assert kv(bt=fake, page=256, lp=fake) != 0 and "leftpad_k running at the same time" in _err(lib)
    assert kv(bt=fake, page=100) != 0 and "multiple of 64" in _err(lib)
    assert kv(cos=fake, sin=fake, rd=64) != 0 and "new key / value to be appended" in _err(lib)
    assert kv(cos=fake, sin=None, rd=64, knew=fake) != 0 and "rotary sin must also be provided" in _err(lib)
    assert kv(cos=fake, sin=fake, rd=24, knew=fake) != 0 and "divisible by 16" in _err(lib)
    assert kv(cos=fake, sin=fake, rd=256, knew=fake) != 0 and "rotary_dim must be <= headdim" in _err(lib)


def test_product_package_does_not_import_oracle():
    pkg = os.path.join(ROOT, "infllmv2_cuda_impl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src, f"{f} mentions the oracle"


def test_ctypes_signatures_have_the_headers_parameter_counts():
    """Every declaration of include/infllmv2_hip.h is parsed for its parameter list; the ctypes argtypes of the
    binding must have the same length and pointer / integer / float kinds in the same places (an argument added on
    one side only would shift every later one silently)."""
    import ctypes as C
    import re
    from infllmv2_cuda_impl_amd import _lib
    text = open(os.path.join(ROOT, "include", "infllmv2_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    decls = dict(re.findall(r"\b(infllmv2_\w+)\s*\(([^)]*)\)\s*;", text))
    assert len(decls) >= 10

    def kind_of_c(param):
        p = param.strip()
        if p in ("void", ""):
            return None
        if "*" in p:
            return "p"
        if re.search(r"\b(float|double)\b", p):
            return "f"
        return "i"

    def kind_of_ctype(t):
        if t in (C.c_void_p, C.c_char_p) or isinstance(t, type) and issubclass(t, C._Pointer):
            return "p"
        if t in (C.c_float, C.c_double):
            return "f"
        return "i"
    checked = 0
    for name, params in decls.items():
        want = [k for k in (kind_of_c(x) for x in params.split(",")) if k is not None]
        fn = getattr(_lib.lib, name)
        if fn.argtypes is None:
            continue
        got = [kind_of_ctype(t) for t in fn.argtypes]
        assert got == want, (name, "".join(got), "".join(want))
        checked += 1
    assert checked >= 10
