#!/usr/bin/env python3
"""Writes the known-answer fixtures of this folder: ``python tests/golden/make_golden.py``.

Where the vectors come from.  The reference (OpenBMB/infllmv2_cuda_impl) stores no golden vectors: all of its
tests compare a live CUDA run with PyTorch, and neither can run here (no CUDA, CUTLASS is an empty submodule, and
every Python module imports the compiled extension).  These fixtures are therefore produced by this repository's
CPU oracle (``oracle/infllmv2_oracle.py``), whose every function is pinned independently in ``tests/test_oracle.py``
(brute force, closed forms, library routines, finite differences).  They freeze those answers: a later change of
the oracle or of a kernel that moves a result shows up against a file, not only against the oracle of the day.

Each ``.npz`` holds the expected outputs of one small case that runs the whole path: compressed keys -> Stage-1
scores -> max-pool -> top-k -> uint64 mask (+ its transpose) -> Stage-2 forward -> backward, and one decode case.
To keep the files small the random inputs are not stored: ``prefill_inputs`` / ``decode_inputs`` rebuild them from
the seed (numpy's PCG64 stream) and the file keeps a CRC-32 of their bytes, which the tests check first; the
large outputs (out, dq) are stored for every ``SAMPLE``-th token, as float16 (relative error 2^-11, far below
the bf16 tolerances they are compared with).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import infllmv2_oracle as O  # noqa: E402


def bits(x):
    """fp32 array holding bf16-representable values -> uint16 bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert np.array_equal(O.bf16_round(x), x)
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def unbits(u):
    return (u.astype(np.uint32) << 16).view(np.float32)


SAMPLE = 8


def crc(*arrays):
    import zlib
    c = 0
    for a in arrays:
        c = zlib.crc32(np.ascontiguousarray(a).tobytes(), c)
    return np.array([c], np.uint32)


def prefill_inputs(seed, seqs, Hk):
    """q, k, v, dout (fp32 arrays of bf16-representable values) and cu_seqlens."""
    r = np.random.default_rng(seed)
    T = sum(seqs)
    cu = np.cumsum([0] + list(seqs)).astype(np.int32)
    mk = lambda *shape: O.bf16_round(r.standard_normal(shape).astype(np.float32))
    return mk(T, 16 * Hk, 128), mk(T, Hk, 128), mk(T, Hk, 128), mk(T, 16 * Hk, 128), cu


def prefill_case(seed, seqs, Hk, topk, local_blocks, init_blocks):
    q, k, v, dout, cu = prefill_inputs(seed, seqs, Hk)
    scale = 128 ** -0.5
    kf, cu_f = O.compress_keys(k, cu, 32, 16)
    kc, cu_c = O.compress_keys(k, cu, 128, 64)
    kf, kc = O.bf16_round(kf), O.bf16_round(kc)
    max_lk = int(max(np.diff(cu_f)))
    score = O.stage1_scores(q, kf, kc, cu, cu_f, cu_c, max_lk, scale, True)
    cache_lens = np.zeros(len(seqs), np.int32)
    pooled = O.max_pooling_1d_varlen(score, cu, cu_f, cache_lens, max(seqs), max_lk, local_blocks, init_blocks)
    idx = O.topk_blocks(pooled, topk)
    words, k_blocks = O.topk_to_uint64(idx, max(seqs), 64)
    col_words = O.transpose_blockmask(words, k_blocks)
    out, lse = O.stage2_forward(q, k, v, cu, cu, words, scale, True)
    dq, dk, dv = O.stage2_backward(q, k, v, dout, cu, cu, words, scale, True)
    f16 = lambda x: np.asarray(x, np.float64).astype(np.float16)
    return dict(seed=np.array([seed], np.int64), seqs=np.asarray(seqs, np.int32),
                params=np.array([Hk, topk, local_blocks, init_blocks], np.int32), input_crc=crc(q, k, v, dout),
                k_fine=bits(kf), k_coarse=bits(kc), cu_fine=np.asarray(cu_f, np.int32),
                cu_coarse=np.asarray(cu_c, np.int32), score=bits(score), pooled=pooled.astype(np.float32),
                topk_idx=idx.astype(np.int32), mask_words=words.astype(np.uint64),
                mask_words_transposed=col_words.astype(np.uint64), lse=lse.astype(np.float32),
                out_sampled=f16(out[::SAMPLE]), dq_sampled=f16(dq[::SAMPLE]), dk=f16(dk), dv=f16(dv))


def decode_inputs(seed, lens, cap, Hk, topk):
    r = np.random.default_rng(seed)
    B = len(lens)
    mk = lambda *shape: O.bf16_round(r.standard_normal(shape).astype(np.float32))
    q, kc, vc = mk(B, 1, 16 * Hk, 128), mk(B, cap, Hk, 128), mk(B, cap, Hk, 128)
    idx = np.full((B, Hk, 1, topk), -1, np.int32)
    for b in range(B):
        nb = (lens[b] + 63) // 64
        for h in range(Hk):
            sel = np.sort(r.permutation(nb)[:topk])
            idx[b, h, 0, :len(sel)] = sel
    return q, kc, vc, idx


def decode_case(seed, lens, cap, Hk, topk):
    q, kc, vc, idx = decode_inputs(seed, lens, cap, Hk, topk)
    words, _ = O.topk_to_uint64(idx, cap, 64)
    out, lse = O.decode_forward(q, kc.copy(), vc.copy(), np.asarray(lens), words, 128 ** -0.5)
    return dict(seed=np.array([seed], np.int64), cache_seqlens=np.asarray(lens, np.int32),
                params=np.array([cap, Hk, topk], np.int32), input_crc=crc(q, kc, vc, idx), topk_idx=idx,
                mask_words=words.astype(np.uint64), out=out.astype(np.float32), lse=lse.astype(np.float32))


CASES = {
    "prefill_two_sequences_hk1.npz": lambda: prefill_case(101, [200, 136], 1, 2, 0, 1),
    "prefill_one_sequence_hk2.npz": lambda: prefill_case(102, [256], 2, 3, 0, 1),
    "decode_three_sequences_hk1.npz": lambda: decode_case(103, [130, 257, 64], 320, 1, 3),
}

if __name__ == "__main__":
    for name, make in CASES.items():
        np.savez_compressed(os.path.join(HERE, name), **make())
        print(name, os.path.getsize(os.path.join(HERE, name)) // 1024, "KiB")
