"""Host side of decode against a KV cache (mha_fwd_kvcache, csrc/flash_attn/flash_api.cpp:1549-1843)."""
from __future__ import annotations

import torch

from . import _lib
from ._util import ptr, require_gpu, stream_ptr

GROUP = 16


def _s3(t):
    return _lib.i64_array([t.stride(0), t.stride(1), t.stride(2)])


def _int32_vec(t, batch, name, what):
    if t.dtype != torch.int32:
        raise RuntimeError(f"{name} must have dtype int32")
    require_gpu(t, name)
    if tuple(t.shape) != (batch,):
        raise RuntimeError(f"{name} must have shape (batch_size)")
    return t.contiguous()


def decode_with_kvcache(q, k_cache, v_cache, k_new, v_new, cache_seqlens, softmax_scale, causal, num_splits, mask,
                        cache_batch_idx=None, cache_leftpad=None, block_table=None, rotary_cos=None, rotary_sin=None,
                        rotary_interleaved=True):
    """q (b, 1, Hq, 128); caches (b_cache, capacity, Hk, 128), or (pages, page_size, Hk, 128) with ``block_table``
    (b, pages per sequence) int32; mask (b, Hk, 1, n64) int64 or None.
    Returns (out (b, 1, Hq, 128), lse (b, Hq, 1) fp32).  The caches are updated in place when k_new/v_new are given.
    Checks and messages follow mha_fwd_kvcache (flash_api.cpp:1549-1843)."""
    for name, t in (("q", q), ("k_cache", k_cache), ("v_cache", v_cache)):
        require_gpu(t, name)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    if k_cache.dtype != q.dtype:
        raise RuntimeError("query and key must have the same dtype")
    if v_cache.dtype != q.dtype:
        raise RuntimeError("query and value must have the same dtype")
    if q.dim() != 4 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise RuntimeError("q, k_cache, v_cache must have 4 dimensions")
    batch, seqlen_q, Hq, d = q.shape
    Hk = k_cache.shape[2]
    paged = block_table is not None
    if paged:
        if cache_batch_idx is not None:
            raise RuntimeError("Paged KVcache does not support cache_batch_idx")
        if cache_leftpad is not None:
            raise RuntimeError("We don't support Paged KV and leftpad_k running at the same time yet")
        require_gpu(block_table, "block_table")
        if block_table.dtype != torch.int32:
            raise RuntimeError("block_table must have dtype torch.int32")
        if block_table.stride(-1) != 1:
            raise RuntimeError("block_table must have contiguous last dimension")
        if block_table.dim() != 2 or block_table.shape[0] != batch:
            raise RuntimeError("block_table must have shape (batch_size, max_num_blocks_per_seq)")
        page = k_cache.shape[1]
        if page % 64 != 0:
            raise RuntimeError("Paged KV cache block size must be divisible by 64")
        cap = block_table.shape[1] * page
        batch_c = batch
    else:
        cap = k_cache.shape[1]
        batch_c = k_cache.shape[0]
    if batch <= 0:
        raise RuntimeError("batch size must be positive")
    if d != 128:
        raise RuntimeError("this build only supports head dimension 128")
    if Hq % Hk != 0:
        raise RuntimeError("Number of heads in key/value must divide number of heads in query")
    if Hq // Hk not in (1, 2, 4, 8, 16):
        raise RuntimeError("this build requires 1, 2, 4, 8 or 16 query heads per key/value head")
    if seqlen_q != 1:
        raise RuntimeError("this build only supports seqlen_q == 1 in infllmv2_attn_with_kvcache")
    if paged:
        if tuple(k_cache.shape[1:]) != (page, Hk, d) or tuple(v_cache.shape) != tuple(k_cache.shape):
            raise RuntimeError("paged k_cache and v_cache must have shape (num_blocks, page_block_size, num_heads_k, head_size)")
    else:
        if tuple(k_cache.shape) != (batch_c, cap, Hk, d) or tuple(v_cache.shape) != (batch_c, cap, Hk, d):
            raise RuntimeError("k_cache and v_cache must have shape (batch_size, seqlen_cache, num_heads_k, head_size)")
        if cache_batch_idx is None and batch_c != batch:
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
    if k_new is not None and cache_seqlens is None:
        raise RuntimeError("If key is supplied, seqlens_k must also be passed in")
    if cache_batch_idx is not None:
        cache_batch_idx = _int32_vec(cache_batch_idx, batch, "cache_batch_idx", "cache_batch_idx")
    if cache_leftpad is not None:
        cache_leftpad = _int32_vec(cache_leftpad, batch, "leftpad_k", "leftpad_k")
    rotary_dim = 0
    if rotary_cos is not None:
        if k_new is None:
            raise RuntimeError("If rotary cos/sin are provided, new key / value to be appended to KV cache must also be provided")
        if rotary_sin is None:
            raise RuntimeError("If rotary cos is provided, rotary sin must also be provided")
        require_gpu(rotary_cos, "rotary_cos")
        require_gpu(rotary_sin, "rotary_sin")
        rotary_dim = rotary_cos.shape[1] * 2
        if rotary_dim > d:
            raise RuntimeError("rotary_dim must be <= headdim")
        if rotary_dim % 16 != 0:
            raise RuntimeError("Only rotary dimensions divisible by 16 are currently supported")
        if rotary_cos.shape[0] < cap:
            raise RuntimeError("cos/sin seqlen must be at least the seqlen of KV cache")
        if tuple(rotary_sin.shape) != tuple(rotary_cos.shape) or not rotary_cos.is_contiguous() or not rotary_sin.is_contiguous():
            raise RuntimeError("rotary_cos and rotary_sin must be contiguous (seqlen_ro, rotary_dim / 2) tensors")
        if rotary_cos.dtype != q.dtype or rotary_sin.dtype != q.dtype:
            raise RuntimeError("rotary_cos must have the same dtype as query")
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
        _lib.call_for(q.dtype, "infllmv2_fwd_kvcache", stream_ptr(q.device), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                  ptr(k_new), ptr(v_new), ptr(cache_seqlens), out.data_ptr(), lse.data_ptr(), ptr(mask),
                  workspace.data_ptr(), workspace.numel(), batch, seqlen_q, Hq, Hk, d, cap, seqlen_new, two(q),
                  _s3(k_cache), _s3(v_cache), _s3(k_new) if k_new is not None else _lib.i64_array([0, 0, 0]),
                  _s3(v_new) if v_new is not None else _lib.i64_array([0, 0, 0]), two(out), n64, splits,
                  float(softmax_scale), ptr(cache_batch_idx), ptr(cache_leftpad), ptr(block_table),
                  block_table.stride(0) if paged else 0, k_cache.shape[1] if paged else 0, ptr(rotary_cos),
                  ptr(rotary_sin), rotary_dim, int(bool(rotary_interleaved)))
    return out, lse
