"""Host side of the Stage-2 backward (mha_varlen_bwd, csrc/flash_attn/flash_api.cpp:1278-1547, and
_infllmv2_attn_varlen_backward, infllm_v2/infllmv2_sparse_attention.py:140-264 of the reference).

The reference copies q, dout and out into the (T*16, Hk, d) layout, builds the expanded cu_seqlens in
a Python loop, transposes the mask through bool tensors with a device synchronisation and empties
the allocator cache twice.  Here one C-ABI call does everything on the caller's tensors; the mask is
transposed by a single kernel inside it.
"""
from __future__ import annotations

import torch

from . import _lib
from ._util import ptr, stream_ptr

GROUP = 16
HAVE_BACKWARD = True

def _nat(t, group=GROUP):
    return _lib.i64_array([t.stride(0), t.stride(1), group * t.stride(1)])


def sparse_backward(dout, q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale,
                    causal, fwd_mask, lse_expanded: bool, deterministic: bool = False):
    """Returns (dq, dk, dv) with the shapes and dtype of (q, k, v).  dq is always bit-reproducible; with
    ``deterministic`` dk and dv are too (slots + ordered sum instead of fp32 atomics, at the price of a large workspace)."""
    if dout.stride(-1) != 1:
        dout = dout.contiguous()
    if dout.dtype != q.dtype or tuple(dout.shape) != tuple(q.shape):
        raise RuntimeError("dout must have the shape and dtype of q")
    batch = cu_seqlens_q.numel() - 1
    total_q, Hq, d = q.shape
    total_k, Hk = k.shape[0], k.shape[1]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    grp = Hq // Hk
    if lse_expanded:
        lse_strides = _lib.i64_array([grp, 1, total_q * grp])
    else:
        lse_strides = _lib.i64_array([1, total_q, grp * total_q])
    n64 = 0 if fwd_mask is None else fwd_mask.shape[-1]
    size_query = (_lib.lib.infllmv2_varlen_bwd_deterministic_workspace_bytes if deterministic
                  else _lib.lib.infllmv2_varlen_bwd_workspace_bytes)
    workspace = torch.empty(max(size_query(batch, total_q, total_k, Hk, max_seqlen_k), 256), dtype=torch.uint8, device=q.device)
    kv = lambda t: _lib.i64_array([t.stride(0), t.stride(1)])
    with torch.cuda.device(q.device):
        _lib.call_for(q.dtype, "infllmv2_varlen_bwd", stream_ptr(q.device), dout.data_ptr(), q.data_ptr(), k.data_ptr(),
                  v.data_ptr(), out.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                  cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), ptr(fwd_mask), workspace.data_ptr(),
                  workspace.numel(), batch, total_q, total_k, Hq, Hk, d, max_seqlen_q, max_seqlen_k,
                  _nat(q, grp), kv(k), kv(v), _nat(out, grp), _nat(dout, grp), _nat(dq, grp), kv(dk), kv(dv), lse_strides, n64,
                  float(softmax_scale), int(bool(causal)), int(bool(deterministic)))
    return dq, dk, dv
