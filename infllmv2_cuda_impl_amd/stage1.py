"""Host side of Stage-1 scoring (mha_varlen_fwd_stage1, csrc/flash_attn/flash_api.cpp:784-1049)."""
from __future__ import annotations

import torch

from . import _lib
from ._util import stream_ptr

GROUP = 16


def _readable(t: torch.Tensor) -> torch.Tensor:
    """A key set with no rows (sequences shorter than one window) still needs a valid pointer; no row of it is read."""
    return t if t.shape[0] > 0 else t.new_zeros((1,) + tuple(t.shape[1:]))


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
    buf = torch.empty((Hk, total_q, row), dtype=torch.bfloat16, device=q.device)
    with torch.cuda.device(q.device):
        _lib.call("infllmv2_varlen_fwd_stage1", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  buf.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), cu_seqlens_v.data_ptr(), batch,
                  total_q, Hq, Hk, d, max_seqlen_q, max_seqlen_k,
                  _lib.i64_array([q.stride(0), q.stride(1), GROUP * q.stride(1)]),
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
    out = torch.empty((Hk, total_q, out_len), dtype=torch.bfloat16, device=q.device)
    with torch.cuda.device(q.device):
        _lib.call("infllmv2_varlen_fwd_stage1_pooled", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  out.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), cu_seqlens_v.data_ptr(),
                  cache_lens.data_ptr() if cache_lens is not None else None, int(cache_len), batch, total_q, Hq, Hk, d,
                  max_seqlen_q, max_seqlen_k,
                  _lib.i64_array([q.stride(0), q.stride(1), GROUP * q.stride(1)]),
                  _lib.i64_array([k.stride(0), k.stride(1)]), _lib.i64_array([v.stride(0), v.stride(1)]),
                  out_len, float(softmax_scale), int(bool(causal)), per_block + 1, per_block, 1, block_size,
                  local_blocks, init_blocks)
    return out
