"""Host side of decode against a KV cache (mha_fwd_kvcache, csrc/flash_attn/flash_api.cpp:1549-1843)."""
from __future__ import annotations

import torch

from . import _lib
from ._util import ptr, require_gpu, stream_ptr

GROUP = 16


def _s3(t):
    return _lib.i64_array([t.stride(0), t.stride(1), t.stride(2)])


def decode_with_kvcache(q, k_cache, v_cache, k_new, v_new, cache_seqlens, softmax_scale, causal, num_splits, mask):
    """q (b, 1, Hq, 128); caches (b, capacity, Hk, 128); mask (b, Hk, 1, n64) int64 or None.
    Returns (out (b, 1, Hq, 128), lse (b, Hq, 1) fp32).  The caches are updated in place when k_new/v_new are given."""
    for name, t in (("q", q), ("k_cache", k_cache), ("v_cache", v_cache)):
        require_gpu(t, name)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    if k_cache.dtype != q.dtype:
        raise RuntimeError("query and key must have the same dtype")
    if v_cache.dtype != q.dtype:
        raise RuntimeError("query and value must have the same dtype")
    if q.dtype != torch.bfloat16:
        raise RuntimeError("this build only has bf16 kernels")
    if q.dim() != 4 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise RuntimeError("q, k_cache, v_cache must have 4 dimensions")
    batch, seqlen_q, Hq, d = q.shape
    cap, Hk = k_cache.shape[1], k_cache.shape[2]
    if batch <= 0:
        raise RuntimeError("batch size must be positive")
    if d != 128:
        raise RuntimeError("this build only supports head dimension 128")
    if Hq % Hk != 0:
        raise RuntimeError("Number of heads in key/value must divide number of heads in query")
    if Hq != GROUP * Hk:
        raise RuntimeError("this build requires 16 query heads per key/value head")
    if seqlen_q != 1:
        raise RuntimeError("this build only supports seqlen_q == 1 in infllmv2_attn_with_kvcache")
    if tuple(k_cache.shape) != (batch, cap, Hk, d) or tuple(v_cache.shape) != (batch, cap, Hk, d):
        raise RuntimeError("k_cache and v_cache must have shape (batch_size, seqlen_cache, num_heads_k, head_size)")
    seqlen_new = 0
    if k_new is not None:
        if v_new is None:
            raise RuntimeError("If key is supplied, value must also be passed in")
        if k_new.dtype != q.dtype or v_new.dtype != q.dtype:
            raise RuntimeError("Key and value must have the same dtype as query")
        seqlen_new = k_new.shape[1]
        if tuple(k_new.shape) != (batch, seqlen_new, Hk, d) or tuple(v_new.shape) != tuple(k_new.shape):
            raise RuntimeError("k and v must have shape (batch_size, seqlen_new, num_heads_k, head_size)")
    if cache_seqlens is not None:
        if cache_seqlens.dtype != torch.int32:
            raise RuntimeError("seqlens_k must have dtype int32")
        if tuple(cache_seqlens.shape) != (batch,):
            raise RuntimeError("seqlens_k must have shape (batch_size)")
        cache_seqlens = cache_seqlens.contiguous()
    n64 = 0
    if mask is not None:
        if tuple(mask.shape[:3]) != (batch, Hk, 1):
            raise RuntimeError("topk_idx must have shape (batch_size, num_heads_k, 1, k)")
        n64 = mask.shape[-1]
    out = torch.empty_like(q)
    lse = torch.empty((batch, Hq, 1), dtype=torch.float32, device=q.device)
    splits = _lib.lib.infllmv2_fwd_kvcache_num_splits(batch, Hk, int(num_splits))
    ws_bytes = _lib.lib.infllmv2_fwd_kvcache_workspace_bytes(batch, Hk, splits)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    two = lambda t: _lib.i64_array([t.stride(0), t.stride(2)])
    with torch.cuda.device(q.device):
        _lib.call("infllmv2_fwd_kvcache", stream_ptr(q.device), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                  ptr(k_new), ptr(v_new), ptr(cache_seqlens), out.data_ptr(), lse.data_ptr(), ptr(mask),
                  workspace.data_ptr(), workspace.numel(), batch, seqlen_q, Hq, Hk, d, cap, seqlen_new, two(q),
                  _s3(k_cache), _s3(v_cache), _s3(k_new) if k_new is not None else _lib.i64_array([0, 0, 0]),
                  _s3(v_new) if v_new is not None else _lib.i64_array([0, 0, 0]), two(out), n64, splits,
                  float(softmax_scale))
    return out, lse
