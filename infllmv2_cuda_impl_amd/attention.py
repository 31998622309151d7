"""Stage-1 scoring, Stage-2 block-sparse attention (forward/backward) and decode.

Host-side counterpart of infllm_v2/infllmv2_sparse_attention.py of the reference: same function
names, arguments and results.  The reference re-lays-out q / out / dout into a
``(T*16, Hk, d)`` tensor before every kernel call (lines 71-95, 174-191, 551-559 there); here the
kernels address the caller's ``(T, Hq, d)`` tensors through strides, so no copy is made.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from . import _lib
from ._util import ptr, require_gpu, stream_ptr
from .masks import topk_to_uint64, transpose_blockmask

GROUP = 16          # query heads per KV head the reference build is hard-wired to (flash_api.cpp:941)
GROUPS = (1, 2, 4, 8, 16)     # group sizes served: smaller ones run on the same 16-row tiles


def group_size(num_heads: int, num_heads_k: int) -> int:
    """Query heads per KV head, checked against what the kernels serve."""
    if num_heads_k <= 0 or num_heads % num_heads_k != 0:
        raise RuntimeError("Number of heads in key/value must divide number of heads in query")
    if num_heads // num_heads_k not in GROUPS:
        raise RuntimeError("this build requires 1, 2, 4, 8 or 16 query heads per key/value head")
    return num_heads // num_heads_k
BLOCK_N = 64        # key-block size of the sparse mask (infllmv2_sparse_attention.py:93)


def _dense_last_dim(x):
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


def _reject_unsupported(dropout_p, window_size, softcap, alibi_slopes, causal, max_seqlen_k=None):
    """Options the reference build compiles out (setup.py:235-239) fail with its messages
    (flash_api.cpp:107-109, 131-133, 144-147, 330-332).  Returns the causal flag the kernels must run with, derived
    from the window the way the reference derives it: a window side that reaches ``max_seqlen_k`` is unbounded
    (flash_api.cpp:621-622), ``causal`` closes the right side (flash_api.cpp:600), and the launch is causal iff the
    left side is unbounded and the right side is 0 (flash_api.cpp:137) -- so ``window_size=(-1, 0)`` with
    ``causal=False`` runs causal."""
    if softcap > 0.0:
        raise RuntimeError("This flash attention build does not support softcap.")
    if not dropout_p < 1.0:
        raise RuntimeError("Expected p_dropout < 1.f to be true, but got false.")
    if dropout_p != 0.0:
        raise RuntimeError("This flash attention build does not support dropout.")
    is_causal = normalise_causal(causal, window_size, max_seqlen_k)
    if is_causal is None:
        raise RuntimeError("This flash attention build does not support local attention.")
    if alibi_slopes is not None:
        raise RuntimeError("This flash attention build does not support alibi.")
    return is_causal


def normalise_causal(causal, window_size, max_seqlen_k=None):
    """True / False: the causal flag of the launch; None: a sliding window that this build (like the reference's,
    FLASHATTENTION_DISABLE_LOCAL) does not have."""
    wl, wr = int(window_size[0]), int(window_size[1])
    if max_seqlen_k is not None:
        if wl >= max_seqlen_k:
            wl = -1
        if wr >= max_seqlen_k:
            wr = -1
    if causal:
        wr = 0
    if wl < 0 and wr == 0:
        return True
    if wl < 0 and wr < 0:
        return False
    return None


def _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k, same_kv_len=True):
    """Input checks of mha_varlen_fwd (flash_api.cpp:552-616) that apply to this build."""
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    if k.dtype != q.dtype:
        raise RuntimeError("query and key must have the same dtype")
    if v.dtype != q.dtype:
        raise RuntimeError("query and value must have the same dtype")
    if cu_seqlens_q.dtype != torch.int32:
        raise RuntimeError("cu_seqlens_q must have dtype int32")
    if cu_seqlens_k.dtype != torch.int32:
        raise RuntimeError("cu_seqlens_k must have dtype int32")
    for name, t in (("q", q), ("k", k), ("v", v), ("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        require_gpu(t, name)
    for t in (q, k, v):
        if t.numel() > 0 and t.stride(-1) != 1:
            raise RuntimeError("Input tensor must have contiguous last dimension")
    if not cu_seqlens_q.is_contiguous():
        raise RuntimeError("cu_seqlens_q must be contiguous")
    if not cu_seqlens_k.is_contiguous():
        raise RuntimeError("cu_seqlens_k must be contiguous")
    batch = cu_seqlens_q.numel() - 1
    if batch <= 0:
        raise RuntimeError("batch size must be positive")
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise RuntimeError("q, k, v must have shape (total, nheads, headdim)")
    head_size = q.shape[2]
    if head_size > 256:
        raise RuntimeError("FlashAttention forward only supports head dimension at most 256")
    if head_size % 8 != 0:
        raise RuntimeError("query, key, value, and out_ must have a head_size that is a multiple of 8")
    if q.shape[1] % k.shape[1] != 0:
        raise RuntimeError("Number of heads in key/value must divide number of heads in query")
    if k.shape[2] != head_size or tuple(v.shape[1:]) != tuple(k.shape[1:]) or (same_kv_len and v.shape[0] != k.shape[0]):
        raise RuntimeError("k and v must have shape (total_k, num_heads_k, head_size)")
    if cu_seqlens_k.numel() != batch + 1:
        raise RuntimeError("cu_seqlens_k must have shape (batch_size + 1)")
    if head_size != 128:
        raise RuntimeError("this build only supports head dimension 128")
    group_size(q.shape[1], k.shape[1])
    return batch


HEAD_DIM = 128      # the head size the kernels are laid out for (static_switch.h:79-89 instantiates the same one)


def pad_head_dim(*tensors):
    """Zero-pads the last dimension of every tensor to 128, as the reference's wrapper pads it to a multiple of 8 before
    its kernels and slices the result afterwards (infllmv2_sparse_attention.py:299-303, 336, 352-355, 381).  Zeros
    in q/k leave every dot product unchanged, zeros in v give zero output columns, and the padding is differentiable,
    so gradients come back at the original width.  Returns the tensors (unchanged objects when already 128 wide)."""
    d = tensors[0].shape[-1]
    if d == HEAD_DIM:
        return tensors
    if d > HEAD_DIM or d < 1:
        raise RuntimeError("this build only supports head dimension at most 128")
    return tuple(torch.nn.functional.pad(t, [0, HEAD_DIM - d]) for t in tensors)


def _natural_strides(t: torch.Tensor, group: int = GROUP):
    """{token, head-in-group, kv-head} element strides of a (T, Hq, d) tensor."""
    return _lib.i64_array([t.stride(0), t.stride(1), group * t.stride(1)])


def _sparse_forward(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal,
                    fwd_mask, lse_expanded: bool):
    """Runs the Stage-2 forward kernel.  Returns (out (T,Hq,d), lse)."""
    batch = cu_seqlens_q.numel() - 1
    total_q, Hq, d = q.shape
    total_k, Hk = k.shape[0], k.shape[1]
    out = torch.empty_like(q)
    grp = Hq // Hk
    if lse_expanded:
        lse = torch.empty((Hk, total_q * grp), dtype=torch.float32, device=q.device)         # flash_api.cpp:665
        lse_strides = _lib.i64_array([grp, 1, total_q * grp])
    else:
        lse = torch.empty((Hq, total_q), dtype=torch.float32, device=q.device)
        lse_strides = _lib.i64_array([1, total_q, grp * total_q])
    ws_bytes = _lib.lib.infllmv2_kv_image_bytes(total_k, batch, Hk)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    n64 = 0 if fwd_mask is None else fwd_mask.shape[-1]
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_fwd", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  out.data_ptr(), lse.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), ptr(fwd_mask),
                  workspace.data_ptr(), workspace.numel(), 0, batch, total_q, total_k, Hq, Hk, d, max_seqlen_q,
                  max_seqlen_k, _natural_strides(q, grp), _lib.i64_array([k.stride(0), k.stride(1)]),
                  _lib.i64_array([v.stride(0), v.stride(1)]), _natural_strides(out, grp), lse_strides, n64,
                  float(softmax_scale), int(bool(causal)))
    return out, lse


class Infllmv2AttnVarlenFunc(torch.autograd.Function):
    """Autograd wrapper (infllmv2_sparse_attention.py:275-385 of the reference)."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
                causal, window_size, softcap, alibi_slopes, deterministic, return_softmax, block_table, topk_idx,
                block_mask=None):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        causal = _reject_unsupported(dropout_p, window_size, softcap, alibi_slopes, causal, max_seqlen_k)
        if block_table is not None:
            raise RuntimeError("paged KV (block_table) is not supported by this build")
        q, k, v = [_dense_last_dim(x) for x in (q, k, v)]
        _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k)
        fwd_mask = None
        sparse = topk_idx is not None or block_mask is not None
        if block_mask is not None:
            # the packed selection itself (topk_blocks(return_mask=True)): nothing to pack
            # rows may be wider than max_seqlen_k needs (select_blocks widens them for cached tokens): the kernels take
            # the width as a row stride and never look at a block beyond the sequence
            n64 = ((max_seqlen_k + BLOCK_N - 1) // BLOCK_N + 63) // 64
            if block_mask.dtype != torch.int64 or block_mask.dim() != 3 or \
                    tuple(block_mask.shape[:2]) != (k.shape[1], q.shape[0]) or block_mask.shape[2] < n64:
                raise RuntimeError("block_mask must be int64 of shape (num_heads_k, total_q, words) with "
                                   "words >= ceil(ceil(max_seqlen_k / 64) / 64)")
            require_gpu(block_mask, "block_mask")
            fwd_mask = block_mask.contiguous()
        elif topk_idx is not None:
            assert topk_idx.dtype == torch.int32
            fwd_mask, _ = topk_to_uint64(topk_idx, max_seqlen_k, BLOCK_N)
            if fwd_mask.dim() != 3 or fwd_mask.shape[0] != k.shape[1] or fwd_mask.shape[1] != q.shape[0]:
                raise RuntimeError("topk_idx must have shape (num_heads_k, total_q, k)")
        out, lse = _sparse_forward(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                   softmax_scale, causal, fwd_mask, lse_expanded=sparse)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, fwd_mask)
        ctx.max_seqlen_q = max_seqlen_q
        ctx.max_seqlen_k = max_seqlen_k
        ctx.softmax_scale = softmax_scale
        ctx.causal = causal
        ctx.deterministic = deterministic
        ctx.sparse = sparse
        if not return_softmax:
            return out
        # S_dmask is only materialised with dropout, which this build rejects
        # (infllmv2_sparse_attention.py:319, flash_api.cpp:672-674): an empty tensor is returned.
        s_dmask = torch.empty((0,), dtype=q.dtype, device=q.device)
        ctx.mark_non_differentiable(lse, s_dmask)
        return out, lse, s_dmask

    @staticmethod
    def backward(ctx, dout, *args):
        from .backward import sparse_backward
        q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, fwd_mask = ctx.saved_tensors
        dq, dk, dv = sparse_backward(dout, q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, ctx.max_seqlen_q,
                                     ctx.max_seqlen_k, ctx.softmax_scale, ctx.causal, fwd_mask, ctx.sparse,
                                     ctx.deterministic)
        return (dq, dk, dv) + (None,) * 15


def infllmv2_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p=0.0,
                              softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                              alibi_slopes=None, deterministic=False, return_attn_probs=False, block_table=None,
                              topk_idx=None, block_mask=None):
    """Block-sparse (or, with ``topk_idx=None``, dense) attention over packed variable-length sequences.

    q ``(total_q, nheads, 128)``, k/v ``(total_k, nheads_k, 128)`` bf16 or fp16 with ``nheads == g*nheads_k``, g in 1, 2, 4, 8, 16
    (16 is what the reference build serves and what the kernels' tiles are laid out for);
    ``cu_seqlens_q/k`` int32 ``(batch+1,)``.  ``topk_idx`` int32 ``(nheads_k, total_q, k)`` lists, per KV head
    and packed query token, the 64-key blocks (indices local to the token's sequence, ``-1`` = unused) the
    token attends to; all query heads of a group share the row.  ``causal=True`` aligns the causal mask to
    the bottom-right corner; a query with no visible key yields zeros.  Differentiable w.r.t. q, k, v.

    Returns ``out (total_q, nheads, 128)``; with ``return_attn_probs`` the tuple ``(out, softmax_lse, S_dmask)``
    where ``softmax_lse`` is fp32 ``(nheads_k, total_q*g)`` with column ``t*g + head-in-group`` on the sparse path
    (``(nheads, total_q)`` on the dense path) and ``S_dmask`` is empty.  dropout, softcap, ALiBi, sliding
    windows and paged KV are rejected exactly as the reference build rejects them.
    ``block_mask`` (not in the reference's signature) is the packed form of the same selection, int64
    ``(nheads_k, total_q, ceil(ceil(max_seqlen_k / 64) / 64))`` as ``topk_to_uint64`` / ``topk_blocks(return_mask=True)``
    produce it; when given it is used as is and ``topk_idx`` is ignored.
    Head sizes below 128 are served by zero padding (see :func:`pad_head_dim`); ``softmax_scale`` then defaults to
    the caller's head size ``** -0.5``, as in the reference.
    """
    head_size_og = q.shape[-1]
    if head_size_og != HEAD_DIM and q.dim() == 3 and k.dim() == 3 and v.dim() == 3:
        if softmax_scale is None:
            softmax_scale = head_size_og ** (-0.5)
        q, k, v = pad_head_dim(q, k, v)
    res = Infllmv2AttnVarlenFunc.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                                       softmax_scale, causal, window_size, softcap, alibi_slopes, deterministic,
                                       return_attn_probs, block_table, topk_idx, block_mask)
    if head_size_og == HEAD_DIM:
        return res
    if isinstance(res, tuple):
        return (res[0][..., :head_size_og],) + tuple(res[1:])
    return res[..., :head_size_og]


def infllmv2_attn_stage1(q, k, v, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, max_seqlen_q, max_seqlen_k,
                         dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                         alibi_slopes=None, deterministic=False, return_attn_probs=True, block_table=None):
    """Stage-1 group scores over compressed keys.

    q ``(total_q, nheads, 128)``; k ``(sum Lk, nheads_k, 128)`` the stride-16 compressed keys; v
    ``(sum Lc, nheads_k, 128)`` the key set the log-sum-exp is taken over (the stride-64 compressed keys, or
    ``k`` itself for an exact softmax); ``cu_seqlens_{q,k,v}`` int32.  Returns bf16
    ``(nheads_k, total_q, max_seqlen_k)``: for every token and KV head the sum over the grouped heads of
    ``exp(scale*q.k_j - lse)`` on the keys the token may see, 0 elsewhere.
    """
    from .stage1 import stage1_scores
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    if q.shape[-1] != HEAD_DIM and q.dim() == 3 and k.dim() == 3 and v.dim() == 3:
        q, k, v = pad_head_dim(q, k, v)                        # scores depend on dot products only
    causal = _reject_unsupported(dropout_p, window_size, softcap, alibi_slopes, causal, max_seqlen_k)
    if block_table is not None:
        raise RuntimeError("paged KV (block_table) is not supported by this build")
    q, k, v = [_dense_last_dim(x) for x in (q, k, v)]
    _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k, same_kv_len=False)
    if cu_seqlens_v.dtype != torch.int32:
        raise RuntimeError("cu_seqlens_v must have dtype int32")
    return stage1_scores(q, k, v, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, max_seqlen_q, max_seqlen_k,
                         softmax_scale, causal)


def infllmv2_attn_stage1_pooled(q, k, v, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, max_seqlen_q, max_seqlen_k,
                                local_blocks, init_blocks, cache_lens=None, cache_len=0, max_cache_len=None,
                                block_size=64, stride=16, softmax_scale=None, causal=False):
    """Stage-1 scoring and the max-pooling onto key blocks, fused (no counterpart in the reference's API).

    Returns exactly what ``max_pooling_1d(infllmv2_attn_stage1(...), cache_len, local_blocks, init_blocks)`` (one
    sequence, ``cache_lens`` None) or ``max_pooling_1d_varlen(infllmv2_attn_stage1(...), cu_seqlens_q, cu_seqlens_k,
    cache_lens, max_seqlen_q, max_seqlen_k, local_blocks, init_blocks)`` (packed) return, bit for bit, in one
    launch and without materialising the ``(nheads_k, total_q, max_seqlen_k)`` score tensor: bf16
    ``(nheads_k, total_q, ceil((max_seqlen_q + cache) / block_size))`` with ``cache`` = ``cache_len`` or
    ``max(cache_lens)`` (pass ``max_cache_len`` to avoid the host read).  Only ``block_size`` 64 over stride-16
    compressed keys is fused.
    """
    from .stage1 import stage1_pooled
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    if q.shape[-1] != HEAD_DIM and q.dim() == 3 and k.dim() == 3 and v.dim() == 3:
        q, k, v = pad_head_dim(q, k, v)
    q, k, v = [_dense_last_dim(x) for x in (q, k, v)]
    _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k, same_kv_len=False)
    if cu_seqlens_v.dtype != torch.int32:
        raise RuntimeError("cu_seqlens_v must have dtype int32")
    if cache_lens is not None:
        if max_cache_len is None:
            max_cache_len = int(cache_lens.max().item()) if cache_lens.numel() > 0 else 0
    else:
        if cu_seqlens_q.numel() != 2:
            raise RuntimeError("packed sequences need cache_lens (as max_pooling_1d_varlen does)")
        max_cache_len = cache_len
    out_len = (max_seqlen_q + max_cache_len + block_size - 1) // block_size
    return stage1_pooled(q, k, v, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, max_seqlen_q, max_seqlen_k,
                         softmax_scale, causal, out_len, cache_lens, cache_len, local_blocks, init_blocks,
                         block_size, stride)


def infllmv2_attn_stage1_kvcache(q, k_fine_cache, k_coarse_cache, fine_lens, coarse_lens, cache_seqlens, local_blocks,
                                 init_blocks, max_cache_len=None, block_size=64, stride=16, softmax_scale=None,
                                 causal=False, pooled=True):
    """Stage 1 of a batched decode step against per-sequence compressed-key caches (no counterpart in the reference's
    API, whose varlen Stage 1 needs the compressed keys of all sequences packed into one tensor).

    q ``(batch, 1, nheads, 128)``; ``k_fine_cache`` ``(batch, rows, nheads_k, 128)`` holds ``fine_lens[b]`` stride-16
    compressed keys of sequence b, ``k_coarse_cache`` ``coarse_lens[b]`` keys of the log-sum-exp set (int32
    ``(batch,)`` device tensors).  ``cache_seqlens`` int32 ``(batch,)`` is the position of each sequence's query
    (its tokens before this one), as ``cache_lens`` of ``max_pooling_1d_varlen``.  With ``causal=False`` (a decode
    step) every compressed key is visible.

    ``pooled=True`` returns bf16 ``(batch, nheads_k, ceil((1 + max_cache_len) / block_size))``: the block scores
    ``max_pooling_1d_varlen`` gives for the rows ``infllmv2_attn_stage1`` computes on the packed equivalent, ready for
    ``topk_blocks`` (``max_cache_len`` defaults to the token capacity implied by the fine cache, which avoids a host
    read).  ``pooled=False`` returns the score rows ``(batch, nheads_k, rows)`` themselves."""
    from .stage1 import stage1_decode
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    if q.dim() != 4 or q.shape[1] != 1:
        raise RuntimeError("q must have shape (batch_size, 1, num_heads, head_size)")
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashAttention only support fp16 and bf16 data type")
    if k_fine_cache.dtype != q.dtype or k_coarse_cache.dtype != q.dtype:
        raise RuntimeError("query and key must have the same dtype")
    batch, _, Hq, d = q.shape
    for name, t in (("q", q), ("k_fine_cache", k_fine_cache), ("k_coarse_cache", k_coarse_cache)):
        require_gpu(t, name)
        if t.stride(-1) != 1:
            raise RuntimeError("Input tensor must have contiguous last dimension")
    if k_fine_cache.dim() != 4 or k_coarse_cache.dim() != 4 or k_fine_cache.shape[0] != batch or \
            k_coarse_cache.shape[0] != batch:
        raise RuntimeError("compressed-key caches must have shape (batch_size, rows, num_heads_k, head_size)")
    Hk = k_fine_cache.shape[2]
    group_size(Hq, Hk)
    if d != 128 or tuple(k_coarse_cache.shape[2:]) != (Hk, d) or k_fine_cache.shape[3] != d:
        raise RuntimeError("this build requires head dimension 128")
    for name, t in (("fine_lens", fine_lens), ("coarse_lens", coarse_lens), ("cache_seqlens", cache_seqlens)):
        if t.dtype != torch.int32 or tuple(t.shape) != (batch,) or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous int32 tensor of shape (batch_size)")
    rows_f, rows_c = k_fine_cache.shape[1], k_coarse_cache.shape[1]
    q3 = q[:, 0]
    if not pooled:
        out = torch.empty((batch, Hk, rows_f), dtype=q.dtype, device=q.device)
        return stage1_decode(q3, k_fine_cache, k_coarse_cache, k_lens=fine_lens, v_lens=coarse_lens,
                             max_seqlen_k=rows_f, max_seqlen_v=rows_c, softmax_scale=softmax_scale, causal=causal,
                             out=out, out_head_stride=out.stride(1), out_row_stride=out.stride(0))
    if max_cache_len is None:
        max_cache_len = (rows_f + 1) * stride + block_size
    out_len = (1 + max_cache_len + block_size - 1) // block_size
    out = torch.empty((batch, Hk, out_len), dtype=q.dtype, device=q.device)
    return stage1_decode(q3, k_fine_cache, k_coarse_cache, k_lens=fine_lens, v_lens=coarse_lens, max_seqlen_k=rows_f,
                         max_seqlen_v=rows_c, softmax_scale=softmax_scale, causal=causal, out=out,
                         out_head_stride=out.stride(1), out_row_stride=out.stride(0), pooled=True,
                         cache_lens=cache_seqlens, out_len=out_len, local_blocks=local_blocks, init_blocks=init_blocks,
                         block_size=block_size, stride=stride)


def infllmv2_attn_with_kvcache(q, k_cache, v_cache, k=None, v=None, rotary_cos=None, rotary_sin=None,
                               cache_seqlens: Optional[Union[int, torch.Tensor]] = None,
                               cache_batch_idx: Optional[torch.Tensor] = None,
                               cache_leftpad: Optional[torch.Tensor] = None,
                               block_table: Optional[torch.Tensor] = None, softmax_scale=None, causal=False,
                               window_size=(-1, -1), softcap=0.0, rotary_interleaved=True, alibi_slopes=None,
                               num_splits=0, return_softmax_lse=False, topk_idx=None, block_mask=None):
    """Decode step against a KV cache, restricted to the blocks in ``topk_idx``.

    q ``(batch, 1, nheads, 128)``; caches ``(batch, capacity, nheads_k, 128)``; ``cache_seqlens`` int or int32
    ``(batch,)``.  If ``k``/``v`` ``(batch, s_new, nheads_k, 128)`` are given they are written into the caches
    at ``cache_seqlens`` first (in place) and take part in the attention.  ``topk_idx`` int32
    ``(batch, nheads_k, 1, k)`` selects 64-key blocks of the cache (mask width from the cache capacity).
    Returns ``out (batch, 1, nheads, 128)`` or ``(out, softmax_lse (batch, nheads, 1))``.  No backward.
    ``rotary_cos``/``rotary_sin`` ``(seqlen_ro, rotary_dim / 2)`` turn the appended keys (at their cache rows) and
    the query (at ``cache_seqlens``); ``cache_batch_idx`` ``(batch,)`` picks each sequence's cache row;
    ``cache_leftpad`` ``(batch,)`` is the cache row a sequence's keys start at; ``block_table``
    ``(batch, pages)`` makes the caches ``(num_pages, page_size, nheads_k, 128)`` (page size a multiple of 64).
    """
    from .decode import decode_with_kvcache
    assert k_cache.stride(-1) == 1, "k_cache must have contiguous last dimension"
    assert v_cache.stride(-1) == 1, "v_cache must have contiguous last dimension"
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    _reject_unsupported(0.0, window_size, softcap, alibi_slopes, causal)
    q, k, v = [_dense_last_dim(x) for x in (q, k, v)]
    if cache_seqlens is not None and isinstance(cache_seqlens, int):
        cache_seqlens = torch.full((q.shape[0],), cache_seqlens, dtype=torch.int32, device=k_cache.device)
    mask = None
    if block_mask is not None:
        # the packed selection (batch, nheads_k, 1, words) as topk_blocks(return_mask=True) writes it
        require_gpu(block_mask, "block_mask")
        if block_mask.dtype != torch.int64 or block_mask.dim() != 4 or block_mask.shape[0] != q.shape[0] or \
                block_mask.shape[2] != 1 or block_mask.shape[1] != k_cache.shape[-2] or block_mask.device != q.device:
            raise RuntimeError("block_mask must be an int64 tensor of shape (batch_size, num_heads_k, 1, words) on q's device")
        mask = block_mask.contiguous()
    elif topk_idx is not None:
        assert topk_idx.dtype == torch.int32
        # the mask spans the sequence's whole key capacity; with a paged cache that is pages x page size (the
        # reference sizes it from k_cache.shape[1], which for a paged cache is one page)
        capacity = k_cache.shape[1] if block_table is None else block_table.shape[1] * k_cache.shape[1]
        mask, _ = topk_to_uint64(topk_idx, capacity, BLOCK_N)
    out, lse = decode_with_kvcache(q, k_cache, v_cache, k, v, cache_seqlens, softmax_scale, causal, num_splits, mask,
                                   cache_batch_idx, cache_leftpad, block_table, rotary_cos, rotary_sin,
                                   rotary_interleaved)
    return (out, lse) if return_softmax_lse else out
