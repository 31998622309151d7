"""Block selection: compressed keys, top-k over pooled block scores, and the whole front end in one call.

The reference leaves this step to its callers (README.md:42,125-126 use ``torch.topk``); the only
order it states is the comparator of csrc/topk.cuh:17,26,37, which this operator implements:
larger score first, equal scores by ascending block index.
"""
from __future__ import annotations

import torch

from . import _lib
from ._util import flat_rows, require_gpu, stream_ptr


def topk_blocks(pooled: torch.Tensor, k: int, *, return_mask: bool = False, by_index: bool = False,
                drop_unreachable: bool = False, n_uint64_per_row: int | None = None):
    """pooled ``(..., n_blocks)`` fp16/bf16 -> int32 ``(..., k)``: the first ``k`` columns of a stable
    descending sort of every row; rows with fewer than ``k`` columns are padded with ``-1``.

    Options (all off by default, none changes WHICH blocks of reachable score are selected):
    ``return_mask`` also returns the packed selection ``(..., n_uint64_per_row)`` int64, equal to
    ``topk_to_uint64`` of the indices (default width ``ceil(n_blocks / 64)``), written by the same launch, so that
    Stage 2 (``block_mask=``) needs no packing launch; ``by_index`` lists the selected blocks in ascending block
    order (what the reference's callers sort them into) instead of score order; ``drop_unreachable`` never selects
    a block whose pooled score is ``-inf`` (no visible key: blocks in a causal query's future), so a query with
    fewer than ``k`` reachable blocks gets ``-1`` padding instead of unreachable blocks."""
    assert pooled.dtype == torch.float16 or pooled.dtype == torch.bfloat16
    require_gpu(pooled, "pooled")
    x = pooled if pooled.is_contiguous() else pooled.contiguous()
    n = x.shape[-1]
    out = torch.empty(tuple(x.shape[:-1]) + (k,), dtype=torch.int32, device=x.device)
    rows = flat_rows(x.shape[:-1])
    if not (return_mask or by_index or drop_unreachable):
        with torch.cuda.device(x.device):
            _lib.call("infllmv2_topk_blocks", stream_ptr(x.device), x.data_ptr(), n, out.data_ptr(), rows, n, k)
        return out
    n64 = (n + 63) // 64 if n_uint64_per_row is None else int(n_uint64_per_row)
    mask = torch.empty(tuple(x.shape[:-1]) + (n64,), dtype=torch.int64, device=x.device) if return_mask else None
    with torch.cuda.device(x.device):
        _lib.call("infllmv2_topk_select", stream_ptr(x.device), x.data_ptr(), n, int(x.dtype == torch.bfloat16),
                  out.data_ptr(), None if mask is None else mask.data_ptr(), rows, n, k, n64, int(bool(by_index)),
                  int(bool(drop_unreachable)))
    return (out, mask) if return_mask else out


def compress_keys(k: torch.Tensor, cu_seqlens_k: torch.Tensor, max_seqlen_k: int, kernel_size: int, stride: int,
                  out: torch.Tensor | None = None, first_row: int = 0):
    """Mean of ``k`` ``(total_k, nheads_k, d)`` bf16 over the full windows ``[stride*j, stride*j + kernel_size)`` of
    every packed sequence: the compressed keys of Stage 1, which the reference's callers build themselves
    (compress_tensor, tests/test_stage1_compressed_lse.py:56-99).

    Returns ``(k_cmp, cu_seqlens_cmp)``: ``k_cmp`` ``(rows, nheads_k, d)`` bf16 whose first ``cu_seqlens_cmp[-1]``
    rows are defined (``rows`` is that count for one sequence and an upper bound, ``total_k // stride + 1``, for a
    packed batch, so that no host read is needed) and ``cu_seqlens_cmp`` int32 ``(batch + 1)``.  With ``out`` (a
    buffer returned by an earlier call) and ``first_row`` only rows ``>= first_row`` of each sequence are written.
    """
    require_gpu(k, "k")
    if k.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    if k.dim() != 3 or k.stride(-1) != 1:
        raise RuntimeError("k must have shape (total_k, num_heads_k, head_size) with a contiguous last dimension")
    if cu_seqlens_k.dtype != torch.int32 or not cu_seqlens_k.is_contiguous():
        raise RuntimeError("cu_seqlens_k must be a contiguous int32 tensor")
    batch = cu_seqlens_k.numel() - 1
    total_k, Hk, d = k.shape
    if batch == 1:
        rows = (max_seqlen_k - kernel_size) // stride + 1 if max_seqlen_k >= kernel_size else 0
    else:
        rows = total_k // stride + 1
    if out is None:
        backing = torch.empty((max(rows, 1), Hk, d), dtype=k.dtype, device=k.device)      # never a null pointer
        out = backing[:rows]
    elif out.shape[0] < rows or tuple(out.shape[1:]) != (Hk, d) or not out.is_contiguous() or out.dtype != k.dtype:
        raise RuntimeError("out must be a contiguous (rows, num_heads_k, head_size) buffer of k's dtype")
    else:
        backing = out
    cu_out = torch.empty(batch + 1, dtype=torch.int32, device=k.device)
    with torch.cuda.device(k.device):
        _lib.call_for(k.dtype, "infllmv2_compress_keys", stream_ptr(k.device), k.data_ptr(), backing.data_ptr(), cu_seqlens_k.data_ptr(),
                  cu_out.data_ptr(), batch, max_seqlen_k, Hk, d, k.stride(0), k.stride(1), kernel_size, stride, first_row)
    return out, cu_out


def compress_keys_cache(k_cache: torch.Tensor, new_lens: torch.Tensor, kernel_size: int, stride: int, out: torch.Tensor,
                        old_lens: torch.Tensor | None = None, max_new_rows: int | None = None,
                        out_lens: torch.Tensor | None = None):
    """Compressed keys of per-sequence key caches, as a batched decode loop keeps them: ``k_cache``
    ``(batch, capacity, nheads_k, d)`` holds ``new_lens[b]`` keys of sequence b; rows of ``out``
    ``(batch, rows, nheads_k, d)`` whose windows were completed since ``old_lens[b]`` tokens (``None``: all of them)
    are written in place.  ``max_new_rows`` bounds the new rows per sequence (default: every row of ``out``; 1 suffices
    for a one-token step).  Returns ``out_lens`` int32 ``(batch,)``: the rows each compressed cache now holds - never
    more than ``out`` has rows or than this call covered (the kernels get both capacities and write nothing beyond)."""
    require_gpu(k_cache, "k_cache")
    if k_cache.dtype not in (torch.float16, torch.bfloat16) or out.dtype != k_cache.dtype:
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    if k_cache.dim() != 4 or out.dim() != 4 or k_cache.stride(-1) != 1 or out.stride(-1) != 1 or \
            out.shape[0] != k_cache.shape[0] or tuple(out.shape[2:]) != tuple(k_cache.shape[2:]):
        raise RuntimeError("k_cache and out must have shapes (batch, capacity, num_heads_k, head_size) and "
                           "(batch, rows, num_heads_k, head_size)")
    batch, cap, Hk, d = k_cache.shape
    for name, t in (("new_lens", new_lens), ("old_lens", old_lens)):
        if t is not None and (t.dtype != torch.int32 or tuple(t.shape) != (batch,) or not t.is_contiguous()):
            raise RuntimeError(f"{name} must be a contiguous int32 tensor of shape (batch_size)")
    if max_new_rows is None:
        if (cap - kernel_size) // stride + 1 > out.shape[1]:
            raise RuntimeError("out has fewer rows than the key cache has windows")
        max_new_rows = out.shape[1]
    elif max_new_rows < 0:
        raise RuntimeError("max_new_rows must not be negative")
    if out_lens is None:
        out_lens = torch.empty(batch, dtype=torch.int32, device=k_cache.device)
    s3 = lambda t: _lib.i64_array([t.stride(0), t.stride(1), t.stride(2)])
    with torch.cuda.device(k_cache.device):
        _lib.call_for(k_cache.dtype, "infllmv2_compress_keys_cache", stream_ptr(k_cache.device), k_cache.data_ptr(), out.data_ptr(),
                  None if old_lens is None else old_lens.data_ptr(), new_lens.data_ptr(), out_lens.data_ptr(), batch,
                  int(max_new_rows), Hk, d, s3(k_cache), s3(out), kernel_size, stride, cap, out.shape[1])
    return out_lens


def compress_keys_cache_pair(k_cache: torch.Tensor, new_lens: torch.Tensor, fine, coarse, old_lens: torch.Tensor | None = None,
                             max_new_rows: int | None = None, out_lens=(None, None)):
    """:func:`compress_keys_cache` for the two compressed caches Stage 1 reads, in one call (one launch when both are
    appends of a few rows, as in a decode step): ``fine`` and ``coarse`` are ``(kernel_size, stride, out)`` triples, e.g.
    ``(32, 16, k_fine)`` and ``(128, 64, k_coarse)``.  Same results as two separate calls.  Returns the two ``out_lens``."""
    require_gpu(k_cache, "k_cache")
    (ks_a, st_a, out_a), (ks_b, st_b, out_b) = fine, coarse
    if k_cache.dtype not in (torch.float16, torch.bfloat16) or out_a.dtype != k_cache.dtype or out_b.dtype != k_cache.dtype:
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    for out in (out_a, out_b):
        if k_cache.dim() != 4 or out.dim() != 4 or k_cache.stride(-1) != 1 or out.stride(-1) != 1 or \
                out.shape[0] != k_cache.shape[0] or tuple(out.shape[2:]) != tuple(k_cache.shape[2:]):
            raise RuntimeError("k_cache and out must have shapes (batch, capacity, num_heads_k, head_size) and "
                               "(batch, rows, num_heads_k, head_size)")
    batch, cap, Hk, d = k_cache.shape
    for name, t in (("new_lens", new_lens), ("old_lens", old_lens)):
        if t is not None and (t.dtype != torch.int32 or tuple(t.shape) != (batch,) or not t.is_contiguous()):
            raise RuntimeError(f"{name} must be a contiguous int32 tensor of shape (batch_size)")
    rows = []
    for ks, st, out in ((ks_a, st_a, out_a), (ks_b, st_b, out_b)):
        if max_new_rows is None:
            if (cap - ks) // st + 1 > out.shape[1]:
                raise RuntimeError("out has fewer rows than the key cache has windows")
            rows.append(out.shape[1])
        elif max_new_rows < 0:
            raise RuntimeError("max_new_rows must not be negative")
        else:
            rows.append(int(max_new_rows))
    lens_a, lens_b = [torch.empty(batch, dtype=torch.int32, device=k_cache.device) if t is None else t for t in out_lens]
    s3 = lambda t: _lib.i64_array([t.stride(0), t.stride(1), t.stride(2)])
    with torch.cuda.device(k_cache.device):
        _lib.call_for(k_cache.dtype, "infllmv2_compress_keys_cache_pair", stream_ptr(k_cache.device), k_cache.data_ptr(),
                      out_a.data_ptr(), out_b.data_ptr(), None if old_lens is None else old_lens.data_ptr(), new_lens.data_ptr(),
                      lens_a.data_ptr(), lens_b.data_ptr(), batch, rows[0], rows[1], Hk, d, s3(k_cache), s3(out_a), s3(out_b),
                      ks_a, st_a, ks_b, st_b, cap, out_a.shape[1], out_b.shape[1])
    return lens_a, lens_b


def select_blocks(q: torch.Tensor, k: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                  max_seqlen_q: int, max_seqlen_k: int, topk: int, local_blocks: int, init_blocks: int,
                  cache_lens: torch.Tensor | None = None, max_cache_len: int | None = None, softmax_scale=None,
                  causal: bool = True, kernel_size: int = 32, stride: int = 16, block_size: int = 64,
                  exact_lse: bool = False, return_mask: bool = False, by_index: bool = False,
                  drop_unreachable: bool = False):
    """The selection front end in one call: compressed keys (kernel ``kernel_size`` / stride ``stride``; the
    log-sum-exp over the 4x coarser set, or over the same set with ``exact_lse``), Stage-1 scores pooled onto
    ``block_size``-token key blocks in one launch, top-k.  Returns ``topk_idx`` int32 ``(nheads_k, total_q, topk)``
    for :func:`infllmv2_attn_varlen_func`, equal to what the reference's sequence of calls
    (compress, ``infllmv2_attn_stage1``, ``max_pooling_1d(_varlen)``, top-k) selects; the score tensor is never
    materialised.  Packed batches need ``cache_lens`` (zeros for plain prefill), as ``max_pooling_1d_varlen`` does.
    ``return_mask`` / ``by_index`` / ``drop_unreachable`` as in :func:`topk_blocks`; with ``return_mask`` the result is
    ``(topk_idx, block_mask)`` and the mask (as wide as ``max_seqlen_k`` needs) can be handed to
    ``infllmv2_attn_varlen_func(block_mask=...)``.
    """
    from .attention import infllmv2_attn_stage1_pooled, pad_head_dim, HEAD_DIM
    if q.shape[-1] != HEAD_DIM:
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        q, k = pad_head_dim(q, k)                              # the mean of zero columns is zero
    kf, cu_f = compress_keys(k, cu_seqlens_k, max_seqlen_k, kernel_size, stride)
    if exact_lse:
        kc, cu_c = kf, cu_f
    else:
        kc, cu_c = compress_keys(k, cu_seqlens_k, max_seqlen_k, 4 * kernel_size, 4 * stride)
    max_lk = (max_seqlen_k - kernel_size) // stride + 1 if max_seqlen_k >= kernel_size else 0
    pooled = infllmv2_attn_stage1_pooled(q, kf, kc, cu_seqlens_q, cu_f, cu_c, max_seqlen_q, max_lk, local_blocks,
                                         init_blocks, cache_lens=cache_lens, max_cache_len=max_cache_len,
                                         block_size=block_size, stride=stride, softmax_scale=softmax_scale,
                                         causal=causal)
    n64 = ((max_seqlen_k + block_size - 1) // block_size + 63) // 64
    if n64 * 64 < pooled.shape[-1]:                           # cached tokens widen the pooled rows beyond max_seqlen_k
        n64 = (pooled.shape[-1] + 63) // 64
    return topk_blocks(pooled, topk, return_mask=return_mask, by_index=by_index, drop_unreachable=drop_unreachable,
                       n_uint64_per_row=n64)
