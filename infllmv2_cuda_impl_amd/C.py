"""Mirror of the reference's native module ``infllm_v2.C`` (csrc/entry.cu:197-215) on top of the C ABI.

Code written against the reference's extension keeps working: same function names, argument order and
results.  The raw-pointer group takes ``uintptr_t`` pointers and a stream handle, validates nothing beyond
what the library checks, returns nothing and is asynchronous on the given stream (entry.cu:31-195).  The
tensor group (entry.cu:13-18, 209-214) takes torch tensors in the layouts the reference's Python wrappers
produce — for the sparse path q / out / dout re-laid-out as ``(total_q * 16, Hk, d)`` with
``cu_seqlens_q`` and ``max_seqlen_q`` multiplied by 16 — and is served by the same kernels through
strides, without copying.  ``fwd`` and ``bwd`` (fixed-length dense attention, never reached from the
reference's Python package) run the packed kernels with equal sequence lengths; ``get_probs`` (bound by
the reference, called by nothing) raises NotImplementedError.
"""
from __future__ import annotations

import torch

from . import _lib
from ._util import ptr, stream_ptr
from .attention import _reject_unsupported

GROUP = 16


# ---- raw-pointer group ----------------------------------------------------------------------------
def topk(stream, num_tokens, dim, top, dtype, x, topk_val, topk_pos):
    _lib.call("infllmv2_topk", stream, num_tokens, dim, top, dtype, x, topk_val, topk_pos)


def blockmask_to_uint64(stream, blockmask, result, batch_size, last_dim_size, n_uint64_per_row):
    _lib.call("infllmv2_blockmask_to_uint64", stream, blockmask, result, batch_size, last_dim_size, n_uint64_per_row)


def topk_to_uint64(stream, topk_idx, result, batch_size, k, k_blocks, n_uint64_per_row):
    _lib.call("infllmv2_topk_to_uint64", stream, topk_idx, result, batch_size, k, k_blocks, n_uint64_per_row)


def uint64_to_bool(stream, input, result, batch_size, last_dim_size, n_uint64_per_row):
    _lib.call("infllmv2_uint64_to_bool", stream, input, result, batch_size, last_dim_size, n_uint64_per_row)


def max_pooling_1d(stream, input, output, dtype, num_heads, q_len, k_len, out_len, cache_len, kernel_size, stride,
                   padding, block_size, local_blocks, init_blocks):
    _lib.call("infllmv2_max_pooling_1d", stream, input, output, int(dtype), num_heads, q_len, k_len, out_len,
              cache_len, kernel_size, stride, padding, block_size, local_blocks, init_blocks)


def max_pooling_1d_varlen(stream, input, output, cu_seqlens_q, cu_seqlens_k, cache_lens, dtype, batch_size,
                          num_heads, max_seqlen_q, max_seqlen_k, out_len, kernel_size, stride, padding, block_size,
                          local_blocks, init_blocks):
    _lib.call("infllmv2_max_pooling_1d_varlen", stream, input, output, cu_seqlens_q, cu_seqlens_k, cache_lens,
              int(dtype), batch_size, num_heads, max_seqlen_q, max_seqlen_k, out_len, kernel_size, stride, padding,
              block_size, local_blocks, init_blocks)


def get_probs(*args, **kwargs):
    raise NotImplementedError("get_probs is bound by the reference but unused by its package; not built here")


# ---- tensor group ---------------------------------------------------------------------------------
def _layout(t, expanded: bool):
    """{token, head-in-group, kv-head} strides and (total_q, Hq, Hk) of a q-like tensor."""
    if expanded:                                            # (T*16, Hk, d): row t*16+g, head h
        return _lib.i64_array([GROUP * t.stride(0), t.stride(0), t.stride(1)])
    return _lib.i64_array([t.stride(0), t.stride(1), GROUP * t.stride(1)])


def _kv(t):
    return _lib.i64_array([t.stride(0), t.stride(1)])


def _common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k):
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
    for t in (q, k, v):
        if not t.is_cuda:
            raise RuntimeError("Input tensor must be on CUDA device")
        if t.stride(-1) != 1:
            raise RuntimeError("Input tensor must have contiguous last dimension")
    if cu_seqlens_q.numel() - 1 <= 0:
        raise RuntimeError("batch size must be positive")


def varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k_, block_table_, alibi_slopes_,
               max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, window_size_left,
               window_size_right, softcap, return_softmax, gen_, blockmask_=None):
    """mha_varlen_fwd (flash_api.cpp:519-782).  Returns ``[out, softmax_lse, p, rng_state]``."""
    _common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k)
    is_causal = _reject_unsupported(p_dropout, (window_size_left, window_size_right), softcap, alibi_slopes_, is_causal,
                                    max_seqlen_k)
    for name, val in (("seqused_k", seqused_k), ("leftpad_k", leftpad_k_), ("block_table", block_table_)):
        if val is not None:
            raise RuntimeError(f"{name} is not supported by this build")
    if return_softmax:
        raise RuntimeError("return_softmax is only supported when p_dropout > 0.0")
    Hk = k.shape[1]
    expanded = blockmask_ is not None and q.shape[1] == Hk
    batch = cu_seqlens_q.numel() - 1
    if expanded:
        if q.shape[0] % GROUP != 0 or max_seqlen_q % GROUP != 0:
            raise RuntimeError("the re-laid-out query must hold 16 rows per token")
        total_q, Hq = q.shape[0] // GROUP, Hk * GROUP
        cu_q = torch.div(cu_seqlens_q, GROUP, rounding_mode="floor").to(torch.int32)
        max_q = max_seqlen_q // GROUP
        lse = torch.empty((Hk, total_q * GROUP), dtype=torch.float32, device=q.device)
        lse_strides = _lib.i64_array([GROUP, 1, total_q * GROUP])
    else:
        total_q, Hq = q.shape[0], q.shape[1]
        cu_q, max_q = cu_seqlens_q, max_seqlen_q
        lse = torch.empty((Hq, total_q), dtype=torch.float32, device=q.device)
        lse_strides = _lib.i64_array([1, total_q, GROUP * total_q])
    if max_q == 1:
        is_causal = False                                   # flash_api.cpp:599
    out = out_ if out_ is not None else torch.empty_like(q)
    if out.dtype != q.dtype:
        raise RuntimeError("Output must have the same dtype as inputs")
    if tuple(out.shape) != tuple(q.shape):
        raise RuntimeError("out must have the shape of q")
    total_k = k.shape[0]
    ws = torch.empty(max(_lib.lib.infllmv2_kv_image_bytes(total_k, batch, Hk), 16), dtype=torch.uint8, device=q.device)
    n64 = 0 if blockmask_ is None else blockmask_.shape[-1]
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_fwd", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                  lse.data_ptr(), cu_q.data_ptr(), cu_seqlens_k.data_ptr(), ptr(blockmask_), ws.data_ptr(), ws.numel(), 0,
                  batch, total_q, total_k, Hq, Hk, q.shape[-1], max_q, max_seqlen_k, _layout(q, expanded), _kv(k), _kv(v),
                  _layout(out, expanded), lse_strides, n64, float(softmax_scale), int(bool(is_causal)))
    p = torch.empty((0,), dtype=q.dtype, device=q.device)
    rng_state = torch.empty((2,), dtype=torch.int64, device=q.device)
    return [out, lse, p, rng_state]


def varlen_fwd_stage1(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, seqused_k, leftpad_k_, block_table_,
                      alibi_slopes_, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal,
                      window_size_left, window_size_right, softcap, return_softmax, gen_):
    """mha_varlen_fwd_stage1 (flash_api.cpp:784-1049): q is the re-laid-out ``(T*16, Hk, d)`` tensor.
    Returns ``[p]`` with p bf16 ``(Hk, T, round128(max_seqlen_k))`` like the reference's buffer
    (flash_api.cpp:941); columns >= max_seqlen_k are zero."""
    _common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k)
    is_causal = _reject_unsupported(p_dropout, (window_size_left, window_size_right), softcap, alibi_slopes_, is_causal,
                                    max_seqlen_k)
    Hk = k.shape[1]
    if q.shape[1] != Hk or q.shape[0] % GROUP != 0:
        raise RuntimeError("stage 1 expects the query re-laid-out as (total_q * 16, num_heads_k, head_size)")
    total_q = q.shape[0] // GROUP
    batch = cu_seqlens_q.numel() - 1
    cu_q = torch.div(cu_seqlens_q, GROUP, rounding_mode="floor").to(torch.int32)
    row = (max_seqlen_k + 127) // 128 * 128
    p = torch.zeros((Hk, total_q, row), dtype=q.dtype, device=q.device) if row != max_seqlen_k else \
        torch.empty((Hk, total_q, row), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_fwd_stage1", stream_ptr(q.device), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  p.data_ptr(), cu_q.data_ptr(), cu_seqlens_k.data_ptr(), cu_seqlens_v.data_ptr(), batch, total_q,
                  Hk * GROUP, Hk, q.shape[-1], max_seqlen_q // GROUP, max_seqlen_k, _layout(q, True), _kv(k), _kv(v),
                  p.stride(0), p.stride(1), float(softmax_scale), int(bool(is_causal)))
    return [p]


def varlen_bwd(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, cu_seqlens_q, cu_seqlens_k, alibi_slopes_, max_seqlen_q,
               max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, window_size_left, window_size_right,
               softcap, deterministic, col_blockmask_=None, gen_=None, rng_state=None):
    """mha_varlen_bwd (flash_api.cpp:1278-1547).  ``col_blockmask_`` is the transposed mask
    ``(Hk, k_blocks, ceil(T/64))`` the reference's Python wrapper builds; it is turned back into the row
    mask (the dQ kernel walks rows, the dK/dV kernel re-derives the columns).  dq, dk, dv are written in
    place and returned with an empty softmax_d."""
    _common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k)
    is_causal = _reject_unsupported(p_dropout, (window_size_left, window_size_right), softcap, alibi_slopes_, is_causal,
                                    max_seqlen_k)
    Hk = k.shape[1]
    expanded = col_blockmask_ is not None and q.shape[1] == Hk
    batch = cu_seqlens_q.numel() - 1
    if expanded:
        total_q, Hq = q.shape[0] // GROUP, Hk * GROUP
        cu_q = torch.div(cu_seqlens_q, GROUP, rounding_mode="floor").to(torch.int32)
        max_q = max_seqlen_q // GROUP
        lse_strides = _lib.i64_array([GROUP, 1, total_q * GROUP])
    else:
        total_q, Hq = q.shape[0], q.shape[1]
        cu_q, max_q = cu_seqlens_q, max_seqlen_q
        lse_strides = _lib.i64_array([1, total_q, GROUP * total_q])
    dq = dq_ if dq_ is not None else torch.empty_like(q)
    dk = dk_ if dk_ is not None else torch.empty_like(k)
    dv = dv_ if dv_ is not None else torch.empty_like(v)
    fwd_mask, n64 = None, 0
    if col_blockmask_ is not None:
        from .masks import transpose_blockmask
        k_blocks = (max_seqlen_k + 63) // 64
        if col_blockmask_.shape[1] < k_blocks:
            raise RuntimeError("col_blockmask has fewer rows than key blocks")
        fwd_mask = transpose_blockmask(col_blockmask_[:, :k_blocks].contiguous(), total_q)   # rows <-> columns
        n64 = fwd_mask.shape[-1]
    total_k = k.shape[0]
    size_query = (_lib.lib.infllmv2_varlen_bwd_deterministic_workspace_bytes if deterministic
                  else _lib.lib.infllmv2_varlen_bwd_workspace_bytes)
    ws_bytes = size_query(batch, total_q, total_k, Hk, max_seqlen_k)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_bwd", stream_ptr(q.device), dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                  out.data_ptr(), softmax_lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), cu_q.data_ptr(),
                  cu_seqlens_k.data_ptr(), ptr(fwd_mask), ws.data_ptr(), ws.numel(), batch, total_q, total_k, Hq, Hk,
                  q.shape[-1], max_q, max_seqlen_k, _layout(q, expanded), _kv(k), _kv(v), _layout(out, expanded),
                  _layout(dout, expanded), _layout(dq, expanded), _kv(dk), _kv(dv), lse_strides, n64,
                  float(softmax_scale), int(bool(is_causal)), int(bool(deterministic)))
    return [dq, dk, dv, torch.empty((0,), dtype=torch.float32, device=q.device)]


def fwd_kvcache(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_, leftpad_k_,
                block_table_, alibi_slopes_, out_, softmax_scale, is_causal, window_size_left, window_size_right,
                softcap, is_rotary_interleaved, num_splits, blockmask_=None):
    """mha_fwd_kvcache (flash_api.cpp:1549-1843).  Returns ``[out, softmax_lse]``."""
    from .decode import decode_with_kvcache
    _reject_unsupported(0.0, (window_size_left, window_size_right), softcap, alibi_slopes_, is_causal)
    out, lse = decode_with_kvcache(q, kcache, vcache, k_, v_, seqlens_k_, softmax_scale, is_causal, num_splits, blockmask_,
                                   cache_batch_idx_, leftpad_k_, block_table_, rotary_cos_, rotary_sin_,
                                   is_rotary_interleaved)
    if out_ is not None:
        out_.copy_(out)
        out = out_
    return [out, lse]


# ---- fixed-length batches: the packed entries with equal sequence lengths -----------------------------
def _packed(t, name):
    """(b, s, h, d) -> (b * s, h, d) sharing memory when the batch rows follow one another, else a copy."""
    if t.dim() != 4:
        raise RuntimeError(f"{name} must have shape (batch_size, seqlen, num_heads, head_size)")
    return t.reshape(t.shape[0] * t.shape[1], t.shape[2], t.shape[3])


def _cu(batch, seqlen, device):
    return torch.arange(batch + 1, dtype=torch.int32, device=device) * seqlen


def fwd(q, k, v, out_, alibi_slopes_, p_dropout, softmax_scale, is_causal, window_size_left, window_size_right,
        softcap, return_softmax, gen_=None):
    """mha_fwd (flash_api.cpp:349-517): dense attention over a fixed-length batch, q ``(b, sq, Hq, d)``, k/v
    ``(b, sk, Hk, d)``.  Runs the packed kernels with equal sequence lengths.  Returns
    ``[out, softmax_lse (b, Hq, sq) fp32, p, rng_state]``."""
    b, sq, Hq, d = q.shape
    sk = k.shape[1]
    if k.shape[0] != b or v.shape != k.shape:
        raise RuntimeError("k and v must have shape (batch_size, seqlen_k, num_heads_k, head_size)")
    if out_ is not None and tuple(out_.shape) != tuple(q.shape):
        raise RuntimeError("out must have the shape of q")
    out2 = None
    if out_ is not None:
        out2 = _packed(out_, "out")
        if out2.data_ptr() != out_.data_ptr() or out_.stride(0) != sq * out_.stride(1):
            out2 = None                                     # not viewable as packed rows: copy at the end
    res = varlen_fwd(_packed(q, "q"), _packed(k, "k"), _packed(v, "v"), out2, _cu(b, sq, q.device), _cu(b, sk, q.device),
                     None, None, None, alibi_slopes_, sq, sk, p_dropout, softmax_scale, False, is_causal,
                     window_size_left, window_size_right, softcap, return_softmax, gen_)
    out = res[0].view(b, sq, Hq, d)
    if out_ is not None:
        if out2 is None:
            out_.copy_(out)
        out = out_
    lse = res[1].view(Hq, b, sq).permute(1, 0, 2).contiguous()
    return [out, lse, res[2], res[3]]


def bwd(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, alibi_slopes_, p_dropout, softmax_scale, is_causal,
        window_size_left, window_size_right, softcap, deterministic, gen_=None, rng_state=None):
    """mha_bwd (flash_api.cpp:1062-1276): gradients of ``fwd``; softmax_lse ``(b, Hq, sq)``.  dq_, dk_, dv_ are
    filled in place when given.  Returns ``[dq, dk, dv, softmax_d]`` (softmax_d empty: D never leaves the
    workspace)."""
    b, sq, Hq, d = q.shape
    sk = k.shape[1]
    if tuple(softmax_lse.shape) != (b, Hq, sq):
        raise RuntimeError("softmax_lse must have shape (batch_size, num_heads, seqlen_q)")
    lse = softmax_lse.permute(1, 0, 2).reshape(Hq, b * sq).contiguous()
    given = (dq_, dk_, dv_)
    like = (q, k, v)
    packed = []
    for g, l in zip(given, like):
        if g is not None and tuple(g.shape) != tuple(l.shape):
            raise RuntimeError("dq, dk, dv must have the shapes of q, k, v")
        p2 = None
        if g is not None and g.stride(-1) == 1:
            p2 = _packed(g, "gradient")
            if p2.data_ptr() != g.data_ptr() or g.stride(0) != g.shape[1] * g.stride(1):
                p2 = None
        packed.append(p2)
    res = varlen_bwd(_packed(dout, "dout"), _packed(q, "q"), _packed(k, "k"), _packed(v, "v"), _packed(out, "out"), lse,
                     packed[0], packed[1], packed[2], _cu(b, sq, q.device), _cu(b, sk, q.device), alibi_slopes_, sq, sk,
                     p_dropout, softmax_scale, False, is_causal, window_size_left, window_size_right, softcap,
                     deterministic, None, gen_, rng_state)
    grads = []
    for r, g, l, p2 in zip(res[:3], given, like, packed):
        r = r.view(l.shape)
        if g is not None:
            if p2 is None:
                g.copy_(r)
            r = g
        grads.append(r)
    return grads + [res[3]]
