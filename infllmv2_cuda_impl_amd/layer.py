"""Caller-side glue: an attention layer that strings the operators together the way a MiniCPM4-style model does.

The reference ships only the operators; its callers (the model code, README.md:36-60, 118-140) build the
compressed keys, call ``infllmv2_attn_stage1``, pool, take the top-k and call ``infllmv2_attn_varlen_func`` (prefill)
or ``infllmv2_attn_with_kvcache`` (decode).  This module is that sequence, so that the kernels can be exercised and
validated inside one layer: a prefill over packed sequences, a single-sequence decode loop and a batched decode step
(``BatchCache`` / ``decode_batch``) that keep the K/V caches and the two compressed-key caches up to date (a new
compressed key every ``stride`` tokens).

Conventions (the ones the operators assume):
* block size 64, compressed keys kernel 32 / stride 16, log-sum-exp over kernel 128 / stride 64;
* ``topk`` counts the forced blocks (``init_blocks`` first ones, the query's own block and ``local_blocks`` before it);
* sequences of at most ``dense_len`` tokens skip the selection and attend densely (every block selected);
* in decode the single query scores every complete compressed key of the cache (non-causal Stage 1: all of them
  lie in its past), its block index is ``cache_len // 64`` (``max_pooling_1d`` with ``cache_len``), and the top-k
  indices go to the decode kernel as ``(1, nheads_k, 1, topk)``.  A decode step then selects and attends exactly as
  the prefill does for the last token of the same sequence, except at lengths L with L % 16 == 15 or
  L % 64 == 63, where the causal Stage-1 rule of the prefill (truncating division, mask.h:273-281) hides the newest
  compressed key from the last token.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import (infllmv2_attn_stage1_kvcache, infllmv2_attn_stage1_pooled, infllmv2_attn_varlen_func,
                        infllmv2_attn_with_kvcache)
from .pooling import max_pooling_1d_varlen
from .selection import compress_keys, compress_keys_cache, compress_keys_cache_pair, select_blocks, topk_blocks


@dataclass
class SequenceCache:
    """K/V cache of one sequence plus its compressed keys.  ``length`` tokens are valid."""
    k: torch.Tensor                  # (1, capacity, nheads_k, d)
    v: torch.Tensor
    k_fine: torch.Tensor             # (capacity // stride, nheads_k, d): stride-16 compressed keys
    k_coarse: torch.Tensor           # (capacity // (4 * stride), nheads_k, d)
    length: int = 0

    @staticmethod
    def empty(capacity: int, nheads_k: int, head_dim: int, device, stride: int = 16, dtype=torch.bfloat16):
        z = lambda n: torch.zeros((n, nheads_k, head_dim), dtype=dtype, device=device)
        return SequenceCache(z(capacity).unsqueeze(0), z(capacity).unsqueeze(0), z(capacity // stride + 1),
                             z(capacity // (4 * stride) + 1), 0)


@dataclass
class BatchCache:
    """K/V caches of a batch of sequences plus their compressed keys, for batched decoding.  All lengths live on the
    device (no host read per step); ``max_length`` is the host's upper bound of ``lengths``."""
    k: torch.Tensor                  # (batch, capacity, nheads_k, d)
    v: torch.Tensor
    k_fine: torch.Tensor             # (batch, capacity // stride + 1, nheads_k, d)
    k_coarse: torch.Tensor           # (batch, capacity // (4 * stride) + 1, nheads_k, d)
    lengths: torch.Tensor            # int32 (batch,): tokens held per sequence
    fine_lens: torch.Tensor          # int32 (batch,): rows of k_fine that are valid
    coarse_lens: torch.Tensor
    max_length: int = 0

    @staticmethod
    def empty(batch: int, capacity: int, nheads_k: int, head_dim: int, device, stride: int = 16, dtype=torch.bfloat16):
        z = lambda n: torch.zeros((batch, n, nheads_k, head_dim), dtype=dtype, device=device)
        i = lambda: torch.zeros(batch, dtype=torch.int32, device=device)
        return BatchCache(z(capacity), z(capacity), z(capacity // stride + 1), z(capacity // (4 * stride) + 1),
                          i(), i(), i(), 0)


class InfLLMv2Attention(torch.nn.Module):
    """Sparse attention over 64-token key blocks chosen per query token and KV head (no parameters).

    ``selection`` picks the branch a model layer runs: ``"sparse"`` (default) scores the compressed keys and takes the
    top-k blocks; ``"window"`` attends only the forced blocks (the first ``init_blocks`` and the query's own block with
    the ``local_blocks`` before it: a sliding window in 64-token blocks plus attention sinks, no scoring at all);
    ``"dense"`` attends everything.  Sequences of at most ``dense_len`` tokens are dense whatever the branch."""

    def __init__(self, topk: int = 64, local_blocks: int = 31, init_blocks: int = 1, dense_len: int = 0,
                 kernel_size: int = 32, stride: int = 16, block_size: int = 64, softmax_scale: float | None = None,
                 selection: str = "sparse"):
        super().__init__()
        if selection not in ("sparse", "window", "dense"):
            raise ValueError("selection must be 'sparse', 'window' or 'dense'")
        self.selection = selection
        self.topk, self.local_blocks, self.init_blocks = topk, local_blocks, init_blocks
        self.dense_len = dense_len
        self.kernel_size, self.stride, self.block_size = kernel_size, stride, block_size
        self.softmax_scale = softmax_scale

    def _window_blocks(self, nheads_k: int, rows: int, cu_seqlens_q, positions, max_seqlen_q: int, max_position: int,
                       device):
        """The forced blocks alone as a selection: what the pooling operator marks +inf on a score tensor with no
        columns, with every other block dropped.  ``rows``: packed query tokens; ``positions`` int32 (batch): tokens before each
        sequence's first query.  Returns ``(topk_idx, block_mask)`` with ``init_blocks + local_blocks + 1`` index slots."""
        batch = cu_seqlens_q.numel() - 1
        empty = torch.empty((nheads_k, rows, 0), dtype=torch.bfloat16, device=device)  # pooled scores: any 16-bit type
        no_keys = torch.zeros(batch + 1, dtype=torch.int32, device=device)
        pooled = max_pooling_1d_varlen(empty, cu_seqlens_q, no_keys, positions, max_seqlen_q, 0, self.local_blocks,
                                       self.init_blocks, block_size=self.block_size, stride=self.stride,
                                       max_cache_len=max_position)
        return topk_blocks(pooled, self.init_blocks + self.local_blocks + 1, return_mask=True, by_index=True,
                           drop_unreachable=True)

    # ---- prefill / training ----
    def forward(self, q, k, v, cu_seqlens, max_seqlen: int, cache: SequenceCache | None = None):
        """q ``(total, nheads, d)``, k/v ``(total, nheads_k, d)`` packed; returns ``(total, nheads, d)``.
        With ``cache`` (one sequence only) the keys, values and compressed keys are also stored for decoding."""
        topk_idx = mask = None
        batch = cu_seqlens.numel() - 1
        if self.selection == "window" and max_seqlen > self.dense_len:
            topk_idx, mask = self._window_blocks(k.shape[1], q.shape[0], cu_seqlens, torch.zeros(batch, dtype=torch.int32, device=q.device),
                                                 max_seqlen, 0, q.device)
        elif self.selection == "sparse" and max_seqlen > self.dense_len:
            cache_lens = torch.zeros(batch, dtype=torch.int32, device=q.device) if batch > 1 else None
            # the selection launch also writes the packed mask Stage 2 walks
            topk_idx, mask = select_blocks(q.detach(), k.detach(), cu_seqlens, cu_seqlens, max_seqlen, max_seqlen,
                                           self.topk, self.local_blocks, self.init_blocks, cache_lens=cache_lens,
                                           max_cache_len=0, softmax_scale=self.softmax_scale, causal=True,
                                           kernel_size=self.kernel_size, stride=self.stride,
                                           block_size=self.block_size, return_mask=True)
        out = infllmv2_attn_varlen_func(q, k, v, cu_seqlens, cu_seqlens, max_seqlen, max_seqlen,
                                        softmax_scale=self.softmax_scale, causal=True, topk_idx=topk_idx,
                                        block_mask=mask)
        if cache is not None:
            if cu_seqlens.numel() != 2:
                raise RuntimeError("a SequenceCache holds one sequence")
            n = k.shape[0]
            cache.k[0, :n], cache.v[0, :n] = k.detach(), v.detach()
            cache.length = n
            self._extend_compressed(cache, 0)
        return out

    def _extend_compressed(self, cache: SequenceCache, old_length: int):
        """Brings the compressed keys up to ``cache.length`` tokens; only windows completed since ``old_length`` are
        computed."""
        n = cache.length
        cu = torch.tensor([0, n], dtype=torch.int32, device=cache.k.device)
        rows = lambda length, ks, st: (length - ks) // st + 1 if length >= ks else 0
        for buf, ks, st in ((cache.k_fine, self.kernel_size, self.stride),
                            (cache.k_coarse, 4 * self.kernel_size, 4 * self.stride)):
            if rows(n, ks, st) > rows(old_length, ks, st):
                compress_keys(cache.k[0, :n], cu, n, ks, st, out=buf, first_row=rows(old_length, ks, st))

    # ---- decode ----
    def decode(self, q, k_new, v_new, cache: SequenceCache):
        """One token of one sequence: q ``(1, 1, nheads, d)``, k_new/v_new ``(1, 1, nheads_k, d)``.  Appends the token
        to the cache (K/V in the decode kernel itself, compressed keys when a window completes), selects blocks and
        attends.  Returns ``(1, 1, nheads, d)``."""
        dev = q.device
        old = cache.length
        pos = old                                              # position of the new token
        # the selection needs the new token's key inside the compressed keys, so K goes into the cache first; the
        # decode kernel's own append then rewrites the same row with the same bytes
        cache.k[0, pos], cache.v[0, pos] = k_new[0, 0], v_new[0, 0]
        cache.length = old + 1
        self._extend_compressed(cache, old)
        n = cache.length
        lens = torch.tensor([old], dtype=torch.int32, device=dev)
        topk_idx = None
        if self.selection == "window" and n > self.dense_len:
            topk_idx, _ = self._window_blocks(cache.k.shape[2], 1, torch.tensor([0, 1], dtype=torch.int32, device=dev), lens,
                                              1, pos, dev)
            topk_idx = topk_idx.unsqueeze(0)
        elif self.selection == "sparse" and n > self.dense_len:
            rows = lambda ks, st: (n - ks) // st + 1 if n >= ks else 0
            lf, lc = rows(self.kernel_size, self.stride), rows(4 * self.kernel_size, 4 * self.stride)
            one = lambda x: torch.tensor([0, x], dtype=torch.int32, device=dev)
            pooled = infllmv2_attn_stage1_pooled(q[0], cache.k_fine[:lf], cache.k_coarse[:lc], one(1), one(lf), one(lc),
                                                 1, lf, self.local_blocks, self.init_blocks, cache_len=pos,
                                                 block_size=self.block_size, stride=self.stride,
                                                 softmax_scale=self.softmax_scale, causal=False)
            topk_idx = topk_blocks(pooled, self.topk).unsqueeze(0)                  # (Hk, 1, topk) -> (1, Hk, 1, topk)
        return infllmv2_attn_with_kvcache(q, cache.k, cache.v, k=k_new, v=v_new, cache_seqlens=lens,
                                          softmax_scale=self.softmax_scale, topk_idx=topk_idx)

    # ---- batched decode ----
    def fill_cache(self, cache: BatchCache, k, v, seqlens):
        """Stores packed keys/values ``(total, nheads_k, d)`` of ``len(seqlens)`` sequences (host list of lengths) in
        ``cache`` and builds their compressed keys, as after a prefill."""
        if len(seqlens) != cache.k.shape[0]:
            raise RuntimeError("one length per cached sequence")
        start = 0
        for b, n in enumerate(seqlens):
            cache.k[b, :n], cache.v[b, :n] = k[start:start + n].detach(), v[start:start + n].detach()
            start += n
        cache.lengths.copy_(torch.tensor(list(seqlens), dtype=torch.int32))
        cache.max_length = max(seqlens)
        for buf, lens, ks, st in ((cache.k_fine, cache.fine_lens, self.kernel_size, self.stride),
                                  (cache.k_coarse, cache.coarse_lens, 4 * self.kernel_size, 4 * self.stride)):
            compress_keys_cache(cache.k, cache.lengths, ks, st, out=buf, out_lens=lens)

    def decode_batch(self, q, k_new, v_new, cache: BatchCache):
        """One token for every sequence of the batch: q ``(batch, 1, nheads, d)``, k_new/v_new
        ``(batch, 1, nheads_k, d)``.  Per sequence exactly what :meth:`decode` does, in a fixed number of launches
        for the whole batch and without reading anything back to the host: append, extend the compressed keys where a
        window completes, Stage 1 over each sequence's compressed-key cache, pooling at the sequence's own position,
        top-k, split decode attention.  Returns ``(batch, 1, nheads, d)``."""
        batch = q.shape[0]
        if cache.max_length + 1 > cache.k.shape[1]:
            raise RuntimeError("the K/V cache is full")
        old = cache.lengths
        new = old + 1
        # the selection needs the new key inside the compressed keys; the decode kernel's own append rewrites the row
        cache.k[torch.arange(batch, device=q.device), old.long()] = k_new[:, 0]
        compress_keys_cache_pair(cache.k, new, (self.kernel_size, self.stride, cache.k_fine),
                                 (4 * self.kernel_size, 4 * self.stride, cache.k_coarse), old_lens=old, max_new_rows=1,
                                 out_lens=(cache.fine_lens, cache.coarse_lens))
        mask = None
        if self.selection == "window" and cache.max_length + 1 > self.dense_len:
            cu_one = torch.arange(batch + 1, dtype=torch.int32, device=q.device)
            _, mask = self._window_blocks(cache.k.shape[2], batch, cu_one, old, 1, cache.max_length, q.device)
            mask = mask.transpose(0, 1).unsqueeze(2).contiguous()                    # (Hk, batch, words) -> (batch, Hk, 1, words)
        elif self.selection == "sparse" and cache.max_length + 1 > self.dense_len:
            pooled = infllmv2_attn_stage1_kvcache(q, cache.k_fine, cache.k_coarse, cache.fine_lens, cache.coarse_lens,
                                                  old, self.local_blocks, self.init_blocks,
                                                  max_cache_len=cache.max_length, block_size=self.block_size,
                                                  stride=self.stride, softmax_scale=self.softmax_scale, causal=False)
            _, mask = topk_blocks(pooled, self.topk, return_mask=True, by_index=True)
            mask = mask.unsqueeze(2)                                                 # (batch, Hk, 1, words)
        out = infllmv2_attn_with_kvcache(q, cache.k, cache.v, k=k_new, v=v_new, cache_seqlens=old,
                                         softmax_scale=self.softmax_scale, block_mask=mask)
        cache.lengths = new
        cache.max_length += 1
        return out
