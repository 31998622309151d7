"""Block selection (top-k over pooled block scores).

The reference leaves this step to its callers (README.md:42,125-126 use ``torch.topk``); the only
order it states is the comparator of csrc/topk.cuh:17,26,37, which this operator implements:
larger score first, equal scores by ascending block index.
"""
from __future__ import annotations

import torch

from . import _lib
from ._util import flat_rows, require_gpu, stream_ptr


def topk_blocks(pooled: torch.Tensor, k: int) -> torch.Tensor:
    """pooled ``(..., n_blocks)`` fp16/bf16 -> int32 ``(..., k)``: the first ``k`` columns of a stable
    descending sort of every row; rows with fewer than ``k`` columns are padded with ``-1``."""
    assert pooled.dtype == torch.float16 or pooled.dtype == torch.bfloat16
    require_gpu(pooled, "pooled")
    x = pooled if pooled.is_contiguous() else pooled.contiguous()
    n = x.shape[-1]
    out = torch.empty(tuple(x.shape[:-1]) + (k,), dtype=torch.int32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.call("infllmv2_topk_blocks", stream_ptr(x.device), x.data_ptr(), n, out.data_ptr(),
                  flat_rows(x.shape[:-1]), n, k)
    return out
