"""GPU parity of the fused Stage-1 + max-pooling launch.

The fused launch must return, bit for bit, what the two calls it replaces return (Stage-1 scores, then
max_pooling_1d / max_pooling_1d_varlen, infllm_v2/max_pooling_1d.py:4-137): the pooled tensor is what top-k reads,
so one differing bit could change a selection.  Each case is checked three ways: against this library's two-call
path, against the CPU oracle's pooling of the same score tensor, and (loosely, scores are floating point) against
the oracle's own scores pooled."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np
from test_gpu_stage1 import inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def to_dev(a, dt=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t if dt is None else t.to(dt)).to("cuda:0")


def same_bits(a, b):
    return torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("S,causal,local,init", [(256, True, 1, 1), (1000, True, 2, 1), (2048, True, 1, 1),
                                                 (2048, True, 31, 1), (130, True, 0, 0), (1000, False, 1, 2),
                                                 (4160, True, 4, 1), (128, True, 1, 1), (150, True, 1, 1)])
def test_single_sequence(ops, S, causal, local, init):
    q, cu, kf, cu_f, kc, cu_c = inputs(5, [S])
    Lk = int(cu_f[-1])
    args = (q.to("cuda:0"), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16), to_dev(cu), to_dev(cu_f), to_dev(cu_c),
            S, Lk)
    score = ops.infllmv2_attn_stage1(*args, causal=causal)
    two_calls = ops.max_pooling_1d(score, 0, local, init)
    fused = ops.infllmv2_attn_stage1_pooled(*args, local, init, causal=causal)
    assert fused.dtype == torch.bfloat16 and tuple(fused.shape) == (2, S, (S + 63) // 64)
    assert same_bits(fused, two_calls)
    assert np.array_equal(bf16_np(fused), O.max_pooling_1d_fast(bf16_np(score), 0, local, init))
    # and against the oracle's own scores: finite entries within the score tolerance, forced / empty entries equal
    ref_score = O.stage1_scores(bf16_np(q), kf, kc, cu, cu_f, cu_c, Lk, 128 ** -0.5, causal, round_output=False)
    ref = O.max_pooling_1d_fast(ref_score.astype(np.float32), 0, local, init)
    got = bf16_np(fused)
    fin = np.isfinite(ref)
    assert np.array_equal(np.isposinf(got), np.isposinf(ref)) and np.array_equal(np.isneginf(got), np.isneginf(ref))
    assert (np.abs(got[fin] - ref[fin]) <= 2.0 ** -7 * np.abs(ref[fin]) + 2e-3).all()


@pytest.mark.parametrize("cache_len", [0, 64, 200])
def test_with_cache_len(ops, cache_len):
    """A chunk of queries against a longer key history (q_len < k_len): block of the query = (i + cache_len) / 64."""
    Sq, Sk = 192, 192 + cache_len
    g = torch.Generator(device="cpu").manual_seed(9)
    q = torch.randn(Sq, 32, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(Sk, 2, 128, generator=g).to(torch.bfloat16)
    cu_k = np.array([0, Sk], np.int32)
    kf, cu_f = O.compress_keys(bf16_np(k), cu_k, 32, 16)
    kc, cu_c = O.compress_keys(bf16_np(k), cu_k, 128, 64)
    Lk = int(cu_f[-1])
    args = (q.to("cuda:0"), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16), to_dev(np.array([0, Sq], np.int32)),
            to_dev(cu_f), to_dev(cu_c), Sq, Lk)
    score = ops.infllmv2_attn_stage1(*args, causal=True)
    two_calls = ops.max_pooling_1d(score, cache_len, 1, 1)
    fused = ops.infllmv2_attn_stage1_pooled(*args, 1, 1, cache_len=cache_len, causal=True)
    assert tuple(fused.shape) == tuple(two_calls.shape) and same_bits(fused, two_calls)


def test_packed_sequences(ops):
    seqs = [320, 1024, 64, 700, 150, 5]
    q, cu, kf, cu_f, kc, cu_c = inputs(6, seqs)
    max_k = max(int(cu_f[i + 1] - cu_f[i]) for i in range(len(seqs)))
    cache_lens = torch.tensor([0, 0, 64, 0, 128, 0], dtype=torch.int32, device="cuda:0")
    args = (q.to("cuda:0"), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16), to_dev(cu), to_dev(cu_f), to_dev(cu_c),
            max(seqs), max_k)
    score = ops.infllmv2_attn_stage1(*args, causal=True)
    two_calls = ops.max_pooling_1d_varlen(score, to_dev(cu), to_dev(cu_f), cache_lens, max(seqs), max_k, 2, 1)
    fused = ops.infllmv2_attn_stage1_pooled(*args, 2, 1, cache_lens=cache_lens, causal=True)
    assert tuple(fused.shape) == tuple(two_calls.shape) and same_bits(fused, two_calls)


def test_selection_from_fused_scores(ops):
    """BASELINE config 1 shape: top-k and the packed mask from the fused launch equal those of the three-call chain."""
    S = 2048
    q, cu, kf, cu_f, kc, cu_c = inputs(3, [S])
    Lk = int(cu_f[-1])
    args = (q.to("cuda:0"), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16), to_dev(cu), to_dev(cu_f), to_dev(cu_c),
            S, Lk)
    pooled = ops.infllmv2_attn_stage1_pooled(*args, 1, 1, causal=True)
    chain = ops.max_pooling_1d(ops.infllmv2_attn_stage1(*args, causal=True), 0, 1, 1)
    idx, idx_chain = ops.topk_blocks(pooled, 16), ops.topk_blocks(chain, 16)
    assert torch.equal(idx, idx_chain)
    assert np.array_equal(idx.cpu().numpy(), O.topk_blocks(bf16_np(pooled), 16))


def test_other_windows_are_rejected(ops):
    q, cu, kf, cu_f, kc, cu_c = inputs(5, [256])
    args = (q.to("cuda:0"), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16), to_dev(cu), to_dev(cu_f), to_dev(cu_c),
            256, int(cu_f[-1]))
    with pytest.raises(RuntimeError, match="only the 5/4/1 window"):
        ops.infllmv2_attn_stage1_pooled(*args, 1, 1, block_size=128, causal=True)
