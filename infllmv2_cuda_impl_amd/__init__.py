"""InfLLM-V2 two-stage sparse attention for AMD MI355X (gfx950).

Same public names and argument meaning as the ``infllm_v2`` package of
OpenBMB/infllmv2_cuda_impl (infllm_v2/__init__.py:1-11); the compute is hand-written HIP behind
the C ABI declared in ``include/infllmv2_hip.h``.
"""
__version__ = "0.1.0"

from .masks import blockmask_to_uint64, topk_to_uint64, uint64_to_bool, transpose_blockmask
from .pooling import max_pooling_1d, max_pooling_1d_varlen
from .selection import topk_blocks, compress_keys, compress_keys_cache, compress_keys_cache_pair, select_blocks
from .attention import (
    infllmv2_attn_varlen_func,
    infllmv2_attn_stage1,
    infllmv2_attn_stage1_pooled,
    infllmv2_attn_stage1_kvcache,
    infllmv2_attn_with_kvcache,
)

from .layer import BatchCache, InfLLMv2Attention, SequenceCache

__all__ = [
    "BatchCache", "InfLLMv2Attention", "SequenceCache",
    "blockmask_to_uint64", "topk_to_uint64", "uint64_to_bool", "transpose_blockmask",
    "max_pooling_1d", "max_pooling_1d_varlen", "topk_blocks", "compress_keys", "compress_keys_cache", "compress_keys_cache_pair",
    "select_blocks",
    "infllmv2_attn_varlen_func", "infllmv2_attn_stage1", "infllmv2_attn_stage1_pooled",
    "infllmv2_attn_stage1_kvcache",    "infllmv2_attn_with_kvcache",
]
