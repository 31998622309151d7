"""Max-pooling of Stage-1 scores onto 64-token key blocks.

Operator interface of infllm_v2/max_pooling_1d.py:4-46 (fixed length) and :49-137 (packed).
Forced blocks (the first ``init_blocks`` and the query's own block plus ``local_blocks`` before
it) come out as +inf, an empty window as -inf.
"""
from __future__ import annotations

import torch

from . import _lib
from ._util import require_gpu, stream_ptr


def _window(block_size: int, stride: int):
    s = block_size // stride          # compressed keys per block
    return s + 1, s, 1                # kernel_size, stride, padding  (max_pooling_1d.py:14-16)


def _row_strided(x: torch.Tensor) -> torch.Tensor:
    """Inputs whose last dim is dense and whose rows/heads are regularly strided are used in place."""
    if x.stride(-1) == 1 and x.stride(1) >= x.shape[2] and x.stride(0) >= 0:
        return x
    return x.contiguous()


def max_pooling_1d(input: torch.Tensor, cache_len: int, local_blocks: int, init_blocks: int,
                   block_size: int = 64, stride: int = 16) -> torch.Tensor:
    """input ``(num_heads, q_len, k_len)`` fp16/bf16 -> ``(num_heads, q_len, ceil((q_len+cache_len)/block_size))``."""
    assert input.dtype == torch.float16 or input.dtype == torch.bfloat16
    assert input.dim() == 3, f"Expected 3D input, got {input.dim()}D"
    require_gpu(input, "input")
    x = _row_strided(input)
    ksize, s, pad = _window(block_size, stride)
    num_heads, q_len, k_len = x.shape
    out_len = (q_len + cache_len + block_size - 1) // block_size
    out = torch.empty(num_heads, q_len, out_len, device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        _lib.call("infllmv2_max_pooling_1d_strided", stream_ptr(x.device), x.data_ptr(), out.data_ptr(),
                  int(x.dtype == torch.bfloat16), num_heads, q_len, k_len, x.stride(0), x.stride(1), out_len,
                  cache_len, ksize, s, pad, block_size, local_blocks, init_blocks)
    return out


def max_pooling_1d_varlen(input: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                          cache_lens: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, local_blocks: int,
                          init_blocks: int, block_size: int = 64, stride: int = 16,
                          max_cache_len: int | None = None) -> torch.Tensor:
    """Packed variant: input ``(num_heads, total_q, max_seqlen_k)``; ``cache_lens`` int32 per sequence.

    Output ``(num_heads, total_q, ceil((max_seqlen_q + max(cache_lens)) / block_size))``.  Passing
    ``max_cache_len`` (an extra, optional argument) avoids the one host read of ``cache_lens``.
    """
    assert input.dtype == torch.float16 or input.dtype == torch.bfloat16
    assert cu_seqlens_q.dtype == torch.int32
    assert cu_seqlens_k.dtype == torch.int32
    assert cache_lens.dtype == torch.int32
    assert input.dim() == 3, f"Expected 3D input, got {input.dim()}D"
    require_gpu(input, "input")
    x = _row_strided(input)
    cu_q, cu_k, cl = cu_seqlens_q.contiguous(), cu_seqlens_k.contiguous(), cache_lens.contiguous()
    batch = cu_q.shape[0] - 1
    num_heads, total_q, max_k = x.shape
    assert max_k == max_seqlen_k, f"max_k mismatch: {max_k} vs {max_seqlen_k}"
    assert cl.shape[0] == batch, f"cache_lens batch size mismatch: {cl.shape[0]} vs {batch}"
    if max_cache_len is None:
        max_cache_len = int(cl.max().item()) if batch > 0 else 0
    ksize, s, pad = _window(block_size, stride)
    out_len = (max_seqlen_q + max_cache_len + block_size - 1) // block_size
    out = torch.empty(num_heads, total_q, out_len, device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        _lib.call("infllmv2_max_pooling_1d_varlen_strided", stream_ptr(x.device), x.data_ptr(), out.data_ptr(),
                  cu_q.data_ptr(), cu_k.data_ptr(), cl.data_ptr(), int(x.dtype == torch.bfloat16), batch,
                  num_heads, total_q, max_seqlen_q, max_seqlen_k, x.stride(0), x.stride(1), out_len,
                  ksize, s, pad, block_size, local_blocks, init_blocks)
    return out
