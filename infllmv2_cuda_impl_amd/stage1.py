"""Host side of Stage-1 scoring (mha_varlen_fwd_stage1, csrc/flash_attn/flash_api.cpp:784-1049)."""
from __future__ import annotations

import torch

from . import _lib
from ._util import stream_ptr

GROUP = 16


def _readable(t: torch.Tensor) -> torch.Tensor:
    """A key set with no rows (sequences shorter than one window) still needs a valid pointer; no row of it is read."""
    return t if t.shape[0] > 0 else t.new_zeros((1,) + tuple(t.shape[1:]))


def _max_rows_bound(v, batch, max_seqlen_k):
    """Upper bound of the longest sequence's rows in the packed key set ``v`` (the operator's signature has no
    max_seqlen_v): a sequence's coarse keys are never more than its fine keys, and never more than all rows."""
    return min(int(v.shape[0]), int(max_seqlen_k)) if batch > 1 else int(v.shape[0])


def stage1_scores(q, k, v, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, max_seqlen_q, max_seqlen_k, softmax_scale,
                  causal, row_pad_to: int = 1):
    """Returns bf16 ``(nheads_k, total_q, max_seqlen_k)``.

    The reference allocates a zero-filled ``(Hk, T, round128(max_k))`` buffer, slices it and replaces NaNs
    in a further pass (flash_api.cpp:941, infllmv2_sparse_attention.py:587-589).  Here the kernel defines
    every element of the result once and can produce no NaN: rows with no visible coarse key are written
    as zeros.  ``row_pad_to`` > 1 lays rows out with a padded stride (a view of the first
    ``max_seqlen_k`` columns is returned) so that the pooling kernel can use aligned vector loads.
    """
    for t in (cu_seqlens_q, cu_seqlens_k, cu_seqlens_v):
        if not t.is_contiguous():
            raise RuntimeError("cu_seqlens must be contiguous")
    batch = cu_seqlens_q.numel() - 1
    if cu_seqlens_v.numel() != batch + 1:
        raise RuntimeError("cu_seqlens_v must have shape (batch_size + 1)")
    total_q, Hq, d = q.shape
    Hk = k.shape[1]
    if v.shape[1] != Hk or v.shape[2] != d:
        raise RuntimeError("v must have shape (total_v, num_heads_k, head_size)")
    k, v = _readable(k), _readable(v)
    row = (max_seqlen_k + row_pad_to - 1) // row_pad_to * row_pad_to
    buf = torch.empty((Hk, total_q, row), dtype=q.dtype, device=q.device)
    if max_seqlen_q == 1 and total_q > 0:
        # decode: one query per sequence, so the parallelism has to come from the keys
        stage1_decode(q, k, v, cu_seqlens_q=cu_seqlens_q, cu_seqlens_k=cu_seqlens_k, cu_seqlens_v=cu_seqlens_v,
                      max_seqlen_k=max_seqlen_k, max_seqlen_v=_max_rows_bound(v, batch, max_seqlen_k),
                      softmax_scale=softmax_scale, causal=causal, out=buf, out_head_stride=buf.stride(0),
                      out_row_stride=buf.stride(1))
        return buf if row == max_seqlen_k else buf[:, :, :max_seqlen_k]
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_fwd_stage1", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  buf.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), cu_seqlens_v.data_ptr(), batch,
                  total_q, Hq, Hk, d, max_seqlen_q, max_seqlen_k,
                  _lib.i64_array([q.stride(0), q.stride(1), (Hq // Hk) * q.stride(1)]),
                  _lib.i64_array([k.stride(0), k.stride(1)]), _lib.i64_array([v.stride(0), v.stride(1)]),
                  buf.stride(0), buf.stride(1), float(softmax_scale), int(bool(causal)))
    return buf if row == max_seqlen_k else buf[:, :, :max_seqlen_k]


def stage1_pooled(q, k, v, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, max_seqlen_q, max_seqlen_k, softmax_scale,
                  causal, out_len, cache_lens, cache_len, local_blocks, init_blocks, block_size, stride):
    """Stage-1 scores pooled onto key blocks in the same launch: bf16 ``(nheads_k, total_q, out_len)``."""
    for t in (cu_seqlens_q, cu_seqlens_k, cu_seqlens_v):
        if not t.is_contiguous():
            raise RuntimeError("cu_seqlens must be contiguous")
    batch = cu_seqlens_q.numel() - 1
    if cu_seqlens_v.numel() != batch + 1:
        raise RuntimeError("cu_seqlens_v must have shape (batch_size + 1)")
    if cache_lens is not None and (cache_lens.dtype != torch.int32 or cache_lens.numel() != batch
                                   or not cache_lens.is_contiguous()):
        raise RuntimeError("cache_lens must be a contiguous int32 tensor of shape (batch_size)")
    total_q, Hq, d = q.shape
    Hk = k.shape[1]
    if v.shape[1] != Hk or v.shape[2] != d:
        raise RuntimeError("v must have shape (total_v, num_heads_k, head_size)")
    k, v = _readable(k), _readable(v)
    per_block = block_size // stride
    out = torch.empty((Hk, total_q, out_len), dtype=q.dtype, device=q.device)
    if max_seqlen_q == 1 and total_q > 0 and out_len > 0:
        return stage1_decode(q, k, v, cu_seqlens_q=cu_seqlens_q, cu_seqlens_k=cu_seqlens_k, cu_seqlens_v=cu_seqlens_v,
                             max_seqlen_k=max_seqlen_k, max_seqlen_v=_max_rows_bound(v, batch, max_seqlen_k),
                             softmax_scale=softmax_scale, causal=causal, out=out, out_head_stride=out.stride(0),
                             out_row_stride=out.stride(1), pooled=True, cache_lens=cache_lens, cache_len=cache_len,
                             out_len=out_len, local_blocks=local_blocks, init_blocks=init_blocks,
                             block_size=block_size, stride=stride)
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_fwd_stage1_pooled", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  out.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), cu_seqlens_v.data_ptr(),
                  cache_lens.data_ptr() if cache_lens is not None else None, int(cache_len), batch, total_q, Hq, Hk, d,
                  max_seqlen_q, max_seqlen_k,
                  _lib.i64_array([q.stride(0), q.stride(1), (Hq // Hk) * q.stride(1)]),
                  _lib.i64_array([k.stride(0), k.stride(1)]), _lib.i64_array([v.stride(0), v.stride(1)]),
                  out_len, float(softmax_scale), int(bool(causal)), per_block + 1, per_block, 1, block_size,
                  local_blocks, init_blocks)
    return out


def stage1_decode(q, k, v, *, cu_seqlens_q=None, cu_seqlens_k=None, k_lens=None, cu_seqlens_v=None, v_lens=None,
                  max_seqlen_k, max_seqlen_v, softmax_scale, causal, out, out_head_stride, out_row_stride,
                  pooled=False, cache_lens=None, cache_len=0, out_len=0, local_blocks=0, init_blocks=0, block_size=64,
                  stride=16):
    """Stage 1 with one query token per sequence (infllmv2_stage1_decode): the compressed keys of every sequence are
    scored in parallel runs.  q ``(rows, nheads, 128)``; k/v either packed ``(sum L, nheads_k, 128)`` with
    ``cu_seqlens_*`` or caches ``(batch, capacity, nheads_k, 128)`` with ``*_lens``.  Writes into ``out`` (the caller
    chooses its layout through the two strides) and returns it."""
    batch = (cu_seqlens_q.numel() - 1) if cu_seqlens_q is not None else q.shape[0]
    Hq, d = q.shape[-2], q.shape[-1]
    Hk = k.shape[-2]
    k, v = _readable(k), _readable(v)

    def key_strides(t, packed):
        return _lib.i64_array([0, t.stride(0), t.stride(1)] if packed else [t.stride(0), t.stride(1), t.stride(2)])
    ws_bytes = _lib.lib.infllmv2_stage1_decode_workspace_bytes(batch, Hk, max_seqlen_k, max_seqlen_v)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    per_block = block_size // stride
    p = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_stage1_decode", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  out.data_ptr(), p(cu_seqlens_q), p(cu_seqlens_k), p(k_lens), p(cu_seqlens_v), p(v_lens),
                  workspace.data_ptr(), workspace.numel(), batch, Hq, Hk, d, max_seqlen_k, max_seqlen_v,
                  _lib.i64_array([q.stride(0), q.stride(-2), (Hq // Hk) * q.stride(-2)]),
                  key_strides(k, cu_seqlens_k is not None), key_strides(v, cu_seqlens_v is not None),
                  out_head_stride, out_row_stride, float(softmax_scale), int(bool(causal)), int(bool(pooled)),
                  p(cache_lens), int(cache_len), int(out_len), per_block + 1, per_block, 1, block_size,
                  local_blocks, init_blocks)
    return out
