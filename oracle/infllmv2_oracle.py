"""CPU oracle for the InfLLM-V2 two-stage sparse-attention path.

TEST INFRASTRUCTURE ONLY.  This module restates, in plain numpy, the arithmetic of
the reference kernels so that the HIP kernels can be checked against it.  Nothing in
the shipped package imports it; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and only as the checker.

Every function cites the reference file:line (paths relative to the reference
checkout) whose behaviour it follows.  Float functions compute in fp32/fp64 on
inputs that were already rounded to bf16 by the caller; integer/bit functions are
exact.

Pinning status (how each function is checked independently of its own formula, see
``tests/test_oracle.py``):

* bit packing / unpacking / transposition: brute-force Python-int loops, round trips,
  popcount invariants, the reference's own case tables
  (tests/test_topk_to_uint64.py:259-281, tests/test_uint64_to_bool.py:113-121,
  tests/test_blockmask.py:104-113).
* max-pool: brute force over every (q, kb) + reduction to a -inf padded
  kernel-5/stride-4 library max-pool; varlen == per-sequence fixed-length.
* top-k: equals the prefix of a stable descending sort; forced-block invariant.
* stage-1 exact mode: equals a textbook softmax summed over the 16 group heads with
  the visibility rule brute-forced from "compressed key j covers tokens
  [16j, 16j+32)"; row sums equal 16.
* stage-1 compressed LSE: closed form, reduces to exact mode when v is k.
* stage-2 forward: dense masked softmax; stage-2 backward: central finite
  differences in fp64 on tiny shapes + softmax-Jacobian identities; the one-key-block
  form used at full size (stage2_backward_key_block) equals slices of fp64 autograd gradients.
* decode: the stage-2 forward oracle with one query token; its options (paged cache,
  cache_batch_idx, left padding) are gathers checked by relabelling invariance, rotary by
  complex multiplication, norm preservation, angle addition and the identity at angle 0.

Parity unpinned (stated in the tests that touch it): the tie order of the *external*
``torch.topk`` the reference's callers use (PyTorch leaves it unspecified); this
build defines value-descending / index-ascending as csrc/topk.cuh:17,26,37 does.
"""
from __future__ import annotations

import numpy as np

GROUP = 16          # query heads per KV head, hard-wired by the reference (flash_api.cpp:941)
BLOCK = 64          # key-block size n_block_dim (flash_api.cpp:706-710)


# ----------------------------------------------------------------------------------------
# number formats
# ----------------------------------------------------------------------------------------
def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 to the nearest-even bf16 and return it as fp32 (NaN/inf preserved)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    special = (u & 0x7F800000) == 0x7F800000          # inf / NaN keep their top half
    r = np.where(special, u & 0xFFFF0000, r)
    return r.astype(np.uint32).view(np.float32).reshape(x.shape)


def f16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 to the nearest-even IEEE half and return it as fp32 (numpy's own conversion)."""
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def _trunc_div(a: int, b: int) -> int:
    """C++ integer division (rounds toward zero), as the kernels compute it."""
    q = abs(a) // abs(b)
    return q if (a >= 0) == (b > 0) else -q


# ----------------------------------------------------------------------------------------
# compressed keys (caller-side in the reference: tests/test_stage1_compressed_lse.py:11-99)
# ----------------------------------------------------------------------------------------
def compressed_len(seqlen: int, kernel: int, stride: int) -> int:
    return 0 if seqlen < kernel else (seqlen - kernel) // stride + 1


def compress_keys(k: np.ndarray, cu_seqlens, kernel: int, stride: int, rounding=bf16_round):
    """Mean over full windows [stride*j, stride*j + kernel) of every packed sequence.

    k: (total, H, d) fp32.  Returns (k_cmp (sum L, H, d) fp32 rounded to the element type (``rounding``: bf16_round or
    f16_round), cu_cmp int32).
    """
    cu = [int(c) for c in cu_seqlens]
    outs, cu_c = [], [0]
    for b in range(len(cu) - 1):
        seq = k[cu[b]:cu[b + 1]]
        L = compressed_len(seq.shape[0], kernel, stride)
        if L:
            idx = (np.arange(L)[:, None] * stride + np.arange(kernel)[None, :]).reshape(-1)
            win = seq[idx].reshape(L, kernel, *seq.shape[1:]).astype(np.float32)
            outs.append(rounding(win.mean(axis=1, dtype=np.float32)))
        cu_c.append(cu_c[-1] + L)
    if outs:
        kc = np.concatenate(outs, axis=0)
    else:
        kc = np.zeros((0,) + k.shape[1:], dtype=np.float32)
    return kc, np.asarray(cu_c, dtype=np.int32)


# ----------------------------------------------------------------------------------------
# Stage 1
# ----------------------------------------------------------------------------------------
def stage1_visible(i: int, stride: int, L: int, seqlen_q: int, causal: bool) -> int:
    """Number of compressed keys token ``i`` may see (mask.h:273-281).

    ``cq = (seqlen_q - stride + 1) / stride`` uses truncating division as in the kernel.
    """
    if not causal:
        return L
    cq = _trunc_div(seqlen_q - stride + 1, stride)
    return min(L, max(0, (i + 1) // stride - 1 + L - cq))


def stage1_scores(q, k_cmp, k_coarse, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v,
                  max_seqlen_k: int, softmax_scale: float, causal: bool,
                  round_output: bool = True, rounding=bf16_round) -> np.ndarray:
    """Stage-1 group scores (flash_fwd_kernel.h:1203-1744, softmax.h:94-121,198-237).

    q (T, Hq, d); k_cmp (sum Lk, Hk, d) fine compressed keys; k_coarse (sum Lc, Hk, d) the key
    set the log-sum-exp is taken over (the reference passes it in the ``v`` slot).  Returns
    (Hk, T, max_seqlen_k): ``sum_g exp(scale*q_g.k_j - lse_g)`` for visible j, else 0, rounded once
    to bf16 (flash_fwd_kernel.h:95-107).  A token with no visible coarse key gets an all-zero
    row (early exit flash_fwd_kernel.h:1271-1276 leaves the zero fill of flash_api.cpp:941).
    The LSE stride is 64, or 16 when both key sets have the same length
    (flash_fwd_kernel.h:1236-1240).
    """
    q = np.asarray(q, dtype=np.float32)
    T, Hq, d = q.shape
    Hk = k_cmp.shape[1]
    G = Hq // Hk
    out = np.zeros((Hk, T, max_seqlen_k), dtype=np.float32)
    cu_q = [int(c) for c in cu_seqlens_q]
    cu_k = [int(c) for c in cu_seqlens_k]
    cu_v = [int(c) for c in cu_seqlens_v]
    for b in range(len(cu_q) - 1):
        qb = q[cu_q[b]:cu_q[b + 1]].reshape(-1, Hk, G, d)
        kf = np.asarray(k_cmp[cu_k[b]:cu_k[b + 1]], dtype=np.float32)
        kc = np.asarray(k_coarse[cu_v[b]:cu_v[b + 1]], dtype=np.float32)
        Sq, Lk, Lc = qb.shape[0], kf.shape[0], kc.shape[0]
        if Sq == 0 or Lk == 0:
            continue
        s1 = 16 if Lk == Lc else 64
        i = np.arange(Sq)
        vis_f = np.array([stage1_visible(int(t), 16, Lk, Sq, causal) for t in i])
        vis_c = np.array([stage1_visible(int(t), s1, Lc, Sq, causal) for t in i])
        for h in range(Hk):
            sf = np.einsum("tgd,jd->tgj", qb[:, h], kf[:, h], dtype=np.float64) * softmax_scale
            sc = np.einsum("tgd,jd->tgj", qb[:, h], kc[:, h], dtype=np.float64) * softmax_scale
            mc = np.arange(Lc)[None, :] < vis_c[:, None]               # (Sq, Lc)
            mf = np.arange(Lk)[None, :] < vis_f[:, None]
            sc = np.where(mc[:, None, :], sc, -np.inf)
            with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
                m = sc.max(axis=-1, keepdims=True) if Lc else np.full((Sq, G, 1), -np.inf)
                m_safe = np.where(np.isfinite(m), m, 0.0)
                lse = m_safe + np.log(np.exp(sc - m_safe).sum(axis=-1, keepdims=True)) if Lc \
                    else np.full((Sq, G, 1), -np.inf)
                p = np.exp(sf - lse)
            p = np.where(mf[:, None, :], p, 0.0).sum(axis=1)             # sum over the G heads
            p = np.where((vis_c > 0)[:, None], p, 0.0)
            p = np.where(np.isnan(p), 0.0, p)                           # infllmv2_sparse_attention.py:589
            out[h, cu_q[b]:cu_q[b + 1], :Lk] = p.astype(np.float32)
    return rounding(out) if round_output else out


# ----------------------------------------------------------------------------------------
# max-pool onto 64-token blocks
# ----------------------------------------------------------------------------------------
def max_pool_out_len(q_len: int, cache_len: int, block_size: int = 64) -> int:
    return (q_len + cache_len + block_size - 1) // block_size        # max_pooling_1d.py:19-20


def max_pooling_1d(x: np.ndarray, cache_len: int, local_blocks: int, init_blocks: int,
                   block_size: int = 64, stride: int = 16) -> np.ndarray:
    """csrc/max_pooling_1d.cuh:107-160 with the wrapper's parameters (max_pooling_1d.py:14-22).

    x (H, q_len, k_len).  Output (H, q_len, ceil((q_len+cache_len)/block_size)).
    """
    H, q_len, k_len = x.shape
    s = block_size // stride                # 4
    ksize, pad = s + 1, 1
    out_len = max_pool_out_len(q_len, cache_len, block_size)
    out = np.empty((H, q_len, out_len), dtype=np.float32)
    kb = np.arange(out_len)
    start = np.maximum(kb * s - pad, 0)
    end = np.minimum(kb * s - pad + ksize, k_len)
    for qi in range(q_len):
        bq = (qi + cache_len) // block_size
        forced = (kb < init_blocks) | ((bq >= kb) & (bq <= kb + local_blocks))
        row = np.full((H, out_len), -np.inf, dtype=np.float32)
        for j in range(out_len):
            if not forced[j] and end[j] > start[j]:
                row[:, j] = x[:, qi, start[j]:end[j]].max(axis=-1)
        row[:, forced] = np.inf
        out[:, qi] = row
    return out


def max_pooling_1d_fast(x: np.ndarray, cache_len: int, local_blocks: int, init_blocks: int,
                        block_size: int = 64, stride: int = 16, row_cache_lens=None,
                        row_qidx=None, row_klen=None) -> np.ndarray:
    """Vectorised statement of the same rule (used for large parity cases); checked against
    :func:`max_pooling_1d` in the CPU tests.  ``row_*`` let the varlen wrapper give per-row
    values."""
    H, q_len, k_len = x.shape
    s = block_size // stride
    if row_qidx is None:
        row_qidx = np.arange(q_len)
        row_cache_lens = np.full(q_len, cache_len)
        row_klen = np.full(q_len, k_len)
        out_len = max_pool_out_len(q_len, cache_len, block_size)
    else:
        out_len = cache_len                                     # caller passes out_len here
    xp = np.full((H, q_len, s * out_len + s + 1), -np.inf, dtype=np.float32)
    ncopy = min(k_len, xp.shape[2] - 1)
    xv = np.where(np.arange(k_len)[None, None, :] < np.asarray(row_klen)[None, :, None], x, -np.inf)
    xp[:, :, 1:1 + ncopy] = xv[:, :, :ncopy]
    win = np.stack([xp[:, :, j:j + s * out_len:s] for j in range(s + 1)], axis=0).max(axis=0)
    kb = np.arange(out_len)[None, :]
    bq = ((np.asarray(row_qidx) + np.asarray(row_cache_lens)) // block_size)[:, None]
    forced = (kb < init_blocks) | ((bq >= kb) & (bq <= kb + local_blocks))
    return np.where(forced[None], np.float32(np.inf), win).astype(np.float32)


def max_pooling_1d_varlen(x: np.ndarray, cu_seqlens_q, cu_seqlens_k, cache_lens,
                          max_seqlen_q: int, max_seqlen_k: int, local_blocks: int,
                          init_blocks: int, block_size: int = 64, stride: int = 16) -> np.ndarray:
    """csrc/max_pooling_1d.cuh:12-103 + max_pooling_1d.py:92-108: packed rows, per-sequence
    cache_len, window clipped to that sequence's key length,
    out_len = ceil((max_seqlen_q + max(cache_lens)) / block_size)."""
    cu_q = [int(c) for c in cu_seqlens_q]
    cu_k = [int(c) for c in cu_seqlens_k]
    cl = [int(c) for c in cache_lens]
    H, total_q, _ = x.shape
    out_len = (max_seqlen_q + max(cl) + block_size - 1) // block_size
    qidx = np.zeros(total_q, dtype=np.int64)
    rcl = np.zeros(total_q, dtype=np.int64)
    rkl = np.zeros(total_q, dtype=np.int64)
    for b in range(len(cu_q) - 1):
        qidx[cu_q[b]:cu_q[b + 1]] = np.arange(cu_q[b + 1] - cu_q[b])
        rcl[cu_q[b]:cu_q[b + 1]] = cl[b]
        rkl[cu_q[b]:cu_q[b + 1]] = cu_k[b + 1] - cu_k[b]
    return max_pooling_1d_fast(x, out_len, local_blocks, init_blocks, block_size, stride,
                               row_cache_lens=rcl, row_qidx=qidx, row_klen=rkl)


# ----------------------------------------------------------------------------------------
# top-k block selection
# ----------------------------------------------------------------------------------------
def topk_blocks(pooled: np.ndarray, k: int) -> np.ndarray:
    """First k entries of a stable descending sort of each row (value descending, ties by
    ascending block index — the comparator of csrc/topk.cuh:17,26,37); ``-1`` pads rows with
    fewer than k columns.  Returns int32 (..., k)."""
    n = pooled.shape[-1]
    order = np.argsort(-pooled.astype(np.float32), axis=-1, kind="stable")[..., :k].astype(np.int32)
    if n < k:
        padw = [(0, 0)] * (pooled.ndim - 1) + [(0, k - n)]
        order = np.pad(order, padw, constant_values=-1)
    return order


# ----------------------------------------------------------------------------------------
# bit masks
# ----------------------------------------------------------------------------------------
def topk_to_uint64(topk_idx: np.ndarray, max_seqlen_k: int, block_size: int = 64):
    """csrc/topk_to_uint64.cuh:10-52: word w of a row = OR of 1 << (idx - 64w) over the row's
    indices in [64w, 64w+64); -1 (and any other negative) skipped; no upper-bound check against
    k_blocks beyond the number of words.  Returns (uint64 (..., n64), k_blocks)."""
    k_blocks = (max_seqlen_k + block_size - 1) // block_size
    n64 = (k_blocks + 63) // 64
    idx = np.asarray(topk_idx).astype(np.int64)
    flat = idx.reshape(-1, idx.shape[-1])
    out = np.zeros((flat.shape[0], n64), dtype=np.uint64)
    rows = np.repeat(np.arange(flat.shape[0]), flat.shape[1])
    v = flat.reshape(-1)
    ok = (v >= 0) & (v < 64 * n64)
    np.bitwise_or.at(out, (rows[ok], v[ok] // 64), np.uint64(1) << (v[ok] % 64).astype(np.uint64))
    return out.reshape(idx.shape[:-1] + (n64,)), k_blocks


def uint64_to_bool(words: np.ndarray, last_dim: int) -> np.ndarray:
    """csrc/uint64_to_bool.cuh:24-42: out[..., c] = bit (c % 64) of word c // 64, c < last_dim."""
    w = np.asarray(words).astype(np.uint64)
    c = np.arange(last_dim)
    return ((w[..., c // 64] >> (c % 64).astype(np.uint64)) & np.uint64(1)).astype(bool)


def blockmask_to_uint64(mask: np.ndarray):
    """csrc/blockmask_to_uint64.cuh:34-50: 64 bools -> one word, tail bits zero."""
    m = np.asarray(mask).astype(bool)
    last = m.shape[-1]
    n64 = (last + 63) // 64
    padded = np.zeros(m.shape[:-1] + (n64 * 64,), dtype=np.uint64)
    padded[..., :last] = m
    sh = np.arange(64, dtype=np.uint64)
    words = (padded.reshape(m.shape[:-1] + (n64, 64)) << sh).sum(axis=-1, dtype=np.uint64)
    return words, last


def transpose_blockmask(fwd_words: np.ndarray, k_blocks: int) -> np.ndarray:
    """The mask the backward walks (infllmv2_sparse_attention.py:344-350): unpack to
    (Hk, T, k_blocks) bool, swap the last two axes, repack: (Hk, k_blocks, ceil(T/64))."""
    b = uint64_to_bool(fwd_words, k_blocks)
    return blockmask_to_uint64(np.swapaxes(b, -1, -2))[0]


# ----------------------------------------------------------------------------------------
# Stage 2
# ----------------------------------------------------------------------------------------
def _token_mask(Sq, Sk, block_bits, causal):
    """(Sq, Sk) bool: key t allowed for token i.  block_bits (Sq, nblk) bool or None.
    Causal is aligned bottom-right in token units (mask.h:181-185, flash_fwd_kernel.h:169-177)."""
    t = np.arange(Sk)[None, :]
    allow = np.ones((Sq, Sk), dtype=bool)
    if causal:
        allow &= t <= (np.arange(Sq)[:, None] + Sk - Sq)
    if block_bits is not None:
        nb = (Sk + BLOCK - 1) // BLOCK
        bb = np.zeros((Sq, nb), dtype=bool)
        w = min(nb, block_bits.shape[1])
        bb[:, :w] = block_bits[:, :w]
        allow &= np.repeat(bb, BLOCK, axis=1)[:, :Sk]
    return allow


def stage2_forward(q, k, v, cu_seqlens_q, cu_seqlens_k, fwd_mask_words, softmax_scale: float,
                   causal: bool, dtype=np.float64):
    """Block-sparse attention forward (flash_fwd_kernel.h:137-602, softmax.h:240-256).

    q (T, Hq, d); k, v (total_k, Hk, d); fwd_mask_words (Hk, T, n64) uint64 with block indices
    local to each sequence and rows indexed by the packed token index, or None for dense.
    Returns out (T, Hq, d) and lse (Hk, T*G) in the expanded layout column t*G + g
    (flash_api.cpp:665).  Rows with no allowed key: out = 0, lse = +inf.
    """
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    T, Hq, d = q.shape
    Hk = k.shape[1]
    G = Hq // Hk
    out = np.zeros((T, Hq, d), dtype=dtype)
    lse = np.full((Hk, T * G), np.inf, dtype=dtype)
    cu_q = [int(c) for c in cu_seqlens_q]
    cu_k = [int(c) for c in cu_seqlens_k]
    for b in range(len(cu_q) - 1):
        q0, q1, k0, k1 = cu_q[b], cu_q[b + 1], cu_k[b], cu_k[b + 1]
        Sq, Sk = q1 - q0, k1 - k0
        if Sq == 0:
            continue
        nb = (Sk + BLOCK - 1) // BLOCK
        for h in range(Hk):
            bits = None if fwd_mask_words is None else uint64_to_bool(
                fwd_mask_words[h, q0:q1], max(nb, 1))
            allow = _token_mask(Sq, Sk, bits, causal)
            for g in range(G):
                hq = h * G + g
                s = (q[q0:q1, hq] @ k[k0:k1, h].T) * softmax_scale
                s = np.where(allow, s, -np.inf)
                with np.errstate(invalid="ignore", divide="ignore"):
                    m = s.max(axis=1, keepdims=True) if Sk else np.full((Sq, 1), -np.inf)
                    ms = np.where(np.isfinite(m), m, 0.0)
                    p = np.exp(s - ms)
                    l = p.sum(axis=1, keepdims=True)
                    o = (p @ v[k0:k1, h]) / np.where(l > 0, l, 1.0)
                    row_lse = np.where(l > 0, ms + np.log(np.where(l > 0, l, 1.0)), np.inf)
                out[q0:q1, hq] = np.where(l > 0, o, 0.0)
                lse[h, (np.arange(q0, q1)) * G + g] = row_lse[:, 0]
    return out, lse


def stage2_backward(q, k, v, dout, cu_seqlens_q, cu_seqlens_k, fwd_mask_words,
                    softmax_scale: float, causal: bool, dtype=np.float64):
    """Gradients of :func:`stage2_forward` (flash_bwd_kernel.h:498-794):
    D = rowsum(dO*O); P = exp(scale*S - LSE); dV = P^T dO; dP = dO V^T; dS = P*(dP - D);
    dQ = scale*dS K; dK = scale*dS^T Q, with the 16 group heads summed into their KV head."""
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    dout = np.asarray(dout, dtype=dtype)
    T, Hq, d = q.shape
    Hk = k.shape[1]
    G = Hq // Hk
    dq = np.zeros_like(q)
    dk = np.zeros_like(k)
    dv = np.zeros_like(v)
    cu_q = [int(c) for c in cu_seqlens_q]
    cu_k = [int(c) for c in cu_seqlens_k]
    for b in range(len(cu_q) - 1):
        q0, q1, k0, k1 = cu_q[b], cu_q[b + 1], cu_k[b], cu_k[b + 1]
        Sq, Sk = q1 - q0, k1 - k0
        if Sq == 0 or Sk == 0:
            continue
        nb = (Sk + BLOCK - 1) // BLOCK
        for h in range(Hk):
            bits = None if fwd_mask_words is None else uint64_to_bool(fwd_mask_words[h, q0:q1], nb)
            allow = _token_mask(Sq, Sk, bits, causal)
            for g in range(G):
                hq = h * G + g
                s = (q[q0:q1, hq] @ k[k0:k1, h].T) * softmax_scale
                s = np.where(allow, s, -np.inf)
                with np.errstate(invalid="ignore"):
                    m = s.max(axis=1, keepdims=True)
                    ms = np.where(np.isfinite(m), m, 0.0)
                    e = np.exp(s - ms)
                    l = e.sum(axis=1, keepdims=True)
                    p = e / np.where(l > 0, l, 1.0)
                o = p @ v[k0:k1, h]
                do = dout[q0:q1, hq]
                D = (do * o).sum(axis=1, keepdims=True)
                dp = do @ v[k0:k1, h].T
                ds = p * (dp - D)
                dv[k0:k1, h] += p.T @ do
                dq[q0:q1, hq] = softmax_scale * (ds @ k[k0:k1, h])
                dk[k0:k1, h] += softmax_scale * (ds.T @ q[q0:q1, hq])
    return dq, dk, dv


def stage2_backward_key_block(q, k, v, dout, row_words, kb: int, head: int, softmax_scale: float,
                              dtype=np.float32):
    """dK and dV of ONE 64-key block ``kb`` of ONE sequence and KV head (the unit a column-parallel backward works on,
    flash_bwd_kernel.h:80-856), computed token by token from the tokens whose mask row selects the block, so that a
    full-size problem costs only those tokens: for such a token i (causal, q_len == k_len) the keys are its selected
    blocks up to its own, cut at key i; P = softmax(scale * q K^T) over them, O = P V, D = rowsum(dO * O),
    dP = dO V_kb^T, dS = P_kb * (dP - D); dV_kb += P_kb^T dO, dK_kb += scale * dS^T q, summed over the 16 heads.

    q, dout (S, Hq, d), k, v (S, Hk, d): ONE sequence; row_words (S, n64) uint64: the mask rows of that sequence for
    KV head ``head``.  Returns (dk_block, dv_block, tokens) with the blocks (rows, d) and the contributing tokens."""
    S = q.shape[0]
    G = q.shape[1] // k.shape[1]
    lo, hi = kb * BLOCK, min((kb + 1) * BLOCK, S)
    nb = (S + BLOCK - 1) // BLOCK
    bits = uint64_to_bool(row_words, nb)                          # (S, nb)
    tokens = [i for i in range(lo, S) if bits[i, kb]]
    kh = np.asarray(k[:, head], dtype=dtype)
    vh = np.asarray(v[:, head], dtype=dtype)
    dk = np.zeros((hi - lo, k.shape[2]), dtype=np.float64)
    dv = np.zeros((hi - lo, k.shape[2]), dtype=np.float64)
    for i in tokens:
        blocks = np.nonzero(bits[i, :i // BLOCK + 1])[0]
        keys = np.concatenate([np.arange(b * BLOCK, min((b + 1) * BLOCK, i + 1)) for b in blocks])
        in_kb = (keys >= lo) & (keys < hi)
        qi = np.asarray(q[i, head * G:(head + 1) * G], dtype=dtype)       # (G, d)
        do = np.asarray(dout[i, head * G:(head + 1) * G], dtype=dtype)
        s = (qi @ kh[keys].T).astype(np.float64) * softmax_scale
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        o = p @ vh[keys].astype(np.float64)
        D = (do.astype(np.float64) * o).sum(axis=1, keepdims=True)
        pk = p[:, in_kb]                                                  # (G, rows of the block visible to i)
        rows = keys[in_kb] - lo
        dp = do.astype(np.float64) @ vh[lo + rows].astype(np.float64).T
        ds = pk * (dp - D)
        dv[rows] += pk.T @ do.astype(np.float64)
        dk[rows] += softmax_scale * (ds.T @ qi.astype(np.float64))
    return dk, dv, tokens


def decode_forward(q, k_cache, v_cache, cache_seqlens, fwd_mask_words, softmax_scale: float,
                   k_new=None, v_new=None, dtype=np.float64):
    """Decode against a KV cache (flash_api.cpp:1549-1843): q (b, 1, Hq, d); caches
    (b, cap, Hk, d); optional new k/v (b, s_new, Hk, d) are written at cache_seqlens[b] first
    (in place, like the reference); attention is non-causal over [0, cache_seqlens[b] + s_new)
    restricted to the blocks set in fwd_mask_words (b, Hk, 1, n64) (None = all).
    Returns out (b, 1, Hq, d), lse (b, Hq, 1)."""
    B, Sq, Hq, d = q.shape
    assert Sq == 1
    Hk = k_cache.shape[2]
    G = Hq // Hk
    out = np.zeros((B, 1, Hq, d), dtype=dtype)
    lse = np.full((B, Hq, 1), np.inf, dtype=dtype)
    for b in range(B):
        L = int(cache_seqlens[b])
        if k_new is not None:
            n = k_new.shape[1]
            k_cache[b, L:L + n] = k_new[b]
            v_cache[b, L:L + n] = v_new[b]
            L += n
        cu_q = [0, 1]
        cu_k = [0, L]
        words = None if fwd_mask_words is None else np.asarray(fwd_mask_words)[b]
        o, ls = stage2_forward(np.asarray(q[b], dtype=dtype), np.asarray(k_cache[b, :L], dtype=dtype),
                               np.asarray(v_cache[b, :L], dtype=dtype), cu_q, cu_k, words,
                               softmax_scale, False, dtype=dtype)
        out[b] = o
        lse[b, :, 0] = ls.reshape(Hk, 1, G).reshape(-1)
    return out, lse


def rotary_apply(x: np.ndarray, cos: np.ndarray, sin: np.ndarray, pos: int, interleaved: bool,
                 rounding=bf16_round) -> np.ndarray:
    """Rotary embedding of the rows of ``x`` (..., d) at position ``pos`` (csrc/flash_attn/src/rotary.h:19-82
    interleaved, :84-150 contiguous): only the first ``rotary_dim = 2 * cos.shape[1]`` columns turn.
    interleaved: pairs (2i, 2i+1); contiguous: pairs (i, i + rotary_dim/2);
    (a, b) -> (a cos_i - b sin_i, a sin_i + b cos_i), fp32 arithmetic, result rounded to the element type."""
    x = np.asarray(x, dtype=np.float32).copy()
    half = cos.shape[1]
    c = np.asarray(cos[pos], dtype=np.float32)
    s_ = np.asarray(sin[pos], dtype=np.float32)
    if interleaved:
        a, b = x[..., 0:2 * half:2].copy(), x[..., 1:2 * half:2].copy()
        x[..., 0:2 * half:2] = a * c - b * s_
        x[..., 1:2 * half:2] = a * s_ + b * c
    else:
        a, b = x[..., :half].copy(), x[..., half:2 * half].copy()
        x[..., :half] = a * c - b * s_
        x[..., half:2 * half] = a * s_ + b * c
    return rounding(x)


def decode_forward_ext(q, k_cache, v_cache, cache_seqlens, fwd_mask_words, softmax_scale: float, k_new=None,
                       v_new=None, cache_batch_idx=None, cache_leftpad=None, block_table=None, rotary_cos=None,
                       rotary_sin=None, rotary_interleaved=True, dtype=np.float64, rounding=bf16_round):
    """mha_fwd_kvcache with its remaining options (flash_api.cpp:1549-1843, flash_fwd_kernel.h:606-1199):
    * cache_batch_idx (b): sequence b lives in cache row cache_batch_idx[b];
    * cache_leftpad (b): the sequence's keys are cache rows [leftpad, cache_seqlens) (block_info.h:23-25, 41-43);
      mask block j covers rows leftpad + 64 j ...;
    * block_table (b, max_pages): the caches are (num_pages, page_size, Hk, d) and row r of sequence b is row
      r % page_size of page block_table[b, r // page_size];
    * rotary_cos/sin (seqlen_ro, rotary_dim/2): the new keys are turned at their cache rows cache_seqlens[b] + t and
      the query at cache_seqlens[b] (the non-causal rule, flash_fwd_kernel.h:899-901) before anything else.
    The caches are updated in place.  Returns out (b, 1, Hq, d), lse (b, Hq, 1)."""
    B, Sq, Hq, d = q.shape
    assert Sq == 1
    Hk = k_cache.shape[2]
    G = Hq // Hk
    out = np.zeros((B, 1, Hq, d), dtype=dtype)
    lse = np.full((B, Hq, 1), np.inf, dtype=dtype)

    def rows(b, lo, hi):
        """(cache index array, row index array) of rows lo..hi-1 of sequence b"""
        r = np.arange(lo, hi)
        if block_table is not None:
            page = k_cache.shape[1]
            return np.asarray(block_table)[b, r // page], r % page
        cb = b if cache_batch_idx is None else int(cache_batch_idx[b])
        return np.full(r.shape, cb), r

    for b in range(B):
        end = int(cache_seqlens[b])
        lp = 0 if cache_leftpad is None else int(cache_leftpad[b])
        qb = np.asarray(q[b], dtype=np.float32)
        if k_new is not None:
            n = k_new.shape[1]
            ci, ri = rows(b, end, end + n)
            kn = np.asarray(k_new[b], dtype=np.float32)
            if rotary_cos is not None:
                kn = np.stack([rotary_apply(kn[t], rotary_cos, rotary_sin, end + t, rotary_interleaved, rounding) for t in range(n)])
                qb = rotary_apply(qb, rotary_cos, rotary_sin, end, rotary_interleaved, rounding)
            k_cache[ci, ri] = kn
            v_cache[ci, ri] = v_new[b]
            end += n
        ci, ri = rows(b, lp, end)
        words = None if fwd_mask_words is None else np.asarray(fwd_mask_words)[b]
        o, ls = stage2_forward(np.asarray(qb, dtype=dtype), np.asarray(k_cache[ci, ri], dtype=dtype),
                               np.asarray(v_cache[ci, ri], dtype=dtype), [0, 1], [0, end - lp], words,
                               softmax_scale, False, dtype=dtype)
        out[b] = o
        lse[b, :, 0] = ls.reshape(Hk, 1, G).reshape(-1)
    return out, lse
