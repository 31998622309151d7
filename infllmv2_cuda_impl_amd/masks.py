"""Block-mask conversions: index lists, bool masks and packed uint64 words.

Operator interface of infllm_v2/topk_to_uint64.py:5-72, infllm_v2/uint64_to_bool.py:5-39 and
infllm_v2/blockmask_to_uint64.py:5-43 of the reference.  Packed masks are int64 tensors (bit 63
set shows as a negative number), one word per 64 key blocks.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from ._util import flat_rows, require_gpu, stream_ptr


def topk_to_uint64(topk_idx: torch.Tensor, max_seqlen_k: int, block_size: int,
                   memory_buffer: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, int]:
    """Pack selected block indices into mask words.

    topk_idx: int32 ``(num_heads, total_seqlen, k)`` or ``(batch, num_heads, seqlen, k)``; ``-1``
    marks an unused slot.  Returns ``(words, k_blocks)`` where ``words`` has the leading dims of
    ``topk_idx`` and ``ceil(k_blocks / 64)`` int64 words per row, ``k_blocks =
    ceil(max_seqlen_k / block_size)``.  ``memory_buffer`` is reused as the output when it has the
    right shape, dtype and device.
    """
    assert topk_idx.dtype == torch.int32
    if topk_idx.dim() not in (3, 4):
        raise ValueError(f"topk_idx must have 3 or 4 dimensions, got {topk_idx.dim()}")
    require_gpu(topk_idx, "topk_idx")
    k_blocks = (max_seqlen_k + block_size - 1) // block_size
    n64 = (k_blocks + 63) // 64
    idx = topk_idx.contiguous()
    out_shape = tuple(idx.shape[:-1]) + (n64,)
    if (memory_buffer is not None and tuple(memory_buffer.shape) == out_shape and memory_buffer.dtype == torch.int64
            and memory_buffer.device == idx.device and memory_buffer.is_contiguous()):
        words = memory_buffer
    else:
        words = torch.empty(out_shape, dtype=torch.int64, device=idx.device)
    with torch.cuda.device(idx.device):
        _lib.call("infllmv2_topk_to_uint64", stream_ptr(idx.device), idx.data_ptr(), words.data_ptr(),
                  flat_rows(idx.shape[:-1]), idx.shape[-1], k_blocks, n64)
    return words, k_blocks


def uint64_to_bool(uint64_array: torch.Tensor, last_dim_size: int) -> torch.Tensor:
    """Unpack mask words into a bool tensor whose last dimension has ``last_dim_size`` entries."""
    require_gpu(uint64_array, "uint64_array")
    words = uint64_array.contiguous()
    if words.dtype != torch.int64:
        raise TypeError(f"uint64_array must be torch.int64, got {words.dtype}")
    n64 = words.shape[-1]
    out = torch.empty(tuple(words.shape[:-1]) + (last_dim_size,), dtype=torch.bool, device=words.device)
    with torch.cuda.device(words.device):
        _lib.call("infllmv2_uint64_to_bool", stream_ptr(words.device), words.data_ptr(), out.data_ptr(),
                  flat_rows(words.shape[:-1]), last_dim_size, n64)
    return out


def blockmask_to_uint64(blockmask: torch.Tensor) -> Tuple[torch.Tensor, int]:
    """Pack a bool mask along its last dimension.  Returns ``(words, last_dim_size)``."""
    require_gpu(blockmask, "blockmask")
    if blockmask.dtype != torch.bool:
        raise TypeError(f"blockmask must be torch.bool, got {blockmask.dtype}")
    m = blockmask.contiguous()
    last = m.shape[-1]
    n64 = (last + 63) // 64
    words = torch.empty(tuple(m.shape[:-1]) + (n64,), dtype=torch.int64, device=m.device)
    with torch.cuda.device(m.device):
        _lib.call("infllmv2_blockmask_to_uint64", stream_ptr(m.device), m.data_ptr(), words.data_ptr(),
                  flat_rows(m.shape[:-1]), last, n64)
    return words, last


def transpose_blockmask(fwd_words: torch.Tensor, k_blocks: int) -> torch.Tensor:
    """Forward mask ``(heads, total_q, n64)`` -> backward mask ``(heads, k_blocks, ceil(total_q/64))``.

    One launch instead of the reference's unpack / transpose / synchronize / repack sequence
    (infllm_v2/infllmv2_sparse_attention.py:344-350); same result bit for bit.
    """
    require_gpu(fwd_words, "fwd_words")
    if fwd_words.dim() != 3 or fwd_words.dtype != torch.int64:
        raise ValueError("fwd_words must be an int64 tensor of shape (heads, total_q, n64)")
    w = fwd_words.contiguous()
    heads, total_q, n64 = w.shape
    n64_bwd = (total_q + 63) // 64
    out = torch.empty((heads, k_blocks, n64_bwd), dtype=torch.int64, device=w.device)
    with torch.cuda.device(w.device):
        _lib.call("infllmv2_transpose_blockmask", stream_ptr(w.device), w.data_ptr(), out.data_ptr(),
                  heads, total_q, n64, k_blocks, n64_bwd)
    return out
