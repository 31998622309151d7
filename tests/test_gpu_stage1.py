"""GPU parity of Stage-1 scoring against the CPU oracle, and of the whole selection chain
(scores -> pool -> top-k -> mask) on the kernel's own score tensor.

Tolerance: a score is a sum of up to 16 probabilities rounded once to bf16, so
|got - ref| <= 2^-7 * |ref| + 2e-3 against the unrounded fp64 oracle (the reference's own test accepts
a max difference of 1e-2 on softmax-normalised rows, tests/test_stage1.py:218).  Shapes follow
tests/test_stage1.py:223-231 and tests/test_stage1_compressed_lse.py:203-215."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np, words_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def close(got, ref):
    err = np.abs(got - ref)
    tol = 2.0 ** -7 * np.abs(ref) + 2e-3
    assert (err <= tol).all(), (err.max(), np.unravel_index(np.argmax(err - tol), err.shape))


def inputs(seed, seqs, Hk=2):
    g = torch.Generator(device="cpu").manual_seed(seed)
    T = sum(seqs)
    q = torch.randn(T, 16 * Hk, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(T, Hk, 128, generator=g).to(torch.bfloat16)
    cu = np.cumsum([0] + list(seqs)).astype(np.int32)
    kf, cu_f = O.compress_keys(bf16_np(k), cu, 32, 16)
    kc, cu_c = O.compress_keys(bf16_np(k), cu, 128, 64)
    return q, cu, kf, cu_f, kc, cu_c


def run(ops, q, cu_q, kf, cu_f, kc, cu_c, max_q, max_k, causal):
    dev = torch.device("cuda:0")
    t = lambda a, dt=None: torch.from_numpy(np.ascontiguousarray(a)).to(dev) if dt is None else torch.from_numpy(np.ascontiguousarray(a)).to(dt).to(dev)
    return ops.infllmv2_attn_stage1(q.to(dev), t(kf, torch.bfloat16), t(kc, torch.bfloat16), t(cu_q), t(cu_f), t(cu_c),
                                    max_q, max_k, causal=causal)


@pytest.mark.parametrize("S,causal", [(256, True), (256, False), (1000, True), (1000, False), (2048, True), (130, True)])
def test_compressed_lse(ops, S, causal):
    q, cu, kf, cu_f, kc, cu_c = inputs(0, [S])
    Lk = int(cu_f[-1])
    got = run(ops, q, cu, kf, cu_f, kc, cu_c, S, Lk, causal)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (2, S, Lk)
    ref = O.stage1_scores(bf16_np(q), kf, kc, cu, cu_f, cu_c, Lk, 128 ** -0.5, causal, round_output=False)
    close(bf16_np(got), ref)
    if causal:
        assert float(got[:, :127].abs().max()) == 0.0           # no visible coarse key -> zero rows


@pytest.mark.parametrize("Sq,L,causal", [(64, 15, False), (64, 16, False), (64, 17, False), (256, 15, False),
                                         (256, 16, True), (256, 17, True), (256, 40, True), (33, 70, True)])
def test_exact_mode_v_is_k(ops, Sq, L, causal):
    """v is k: plain softmax over the compressed keys summed over the 16 heads; q_len != k_len offsets."""
    g = torch.Generator(device="cpu").manual_seed(1)
    q = torch.randn(Sq, 32, 128, generator=g).to(torch.bfloat16)
    k = bf16_np(torch.randn(L, 2, 128, generator=g).to(torch.bfloat16))
    cu_q, cu_k = np.array([0, Sq], np.int32), np.array([0, L], np.int32)
    got = run(ops, q, cu_q, k, cu_k, k, cu_k, Sq, L, causal)
    ref = O.stage1_scores(bf16_np(q), k, k, cu_q, cu_k, cu_k, L, 128 ** -0.5, causal, round_output=False)
    close(bf16_np(got), ref)
    vis = np.array([O.stage1_visible(i, 16, L, Sq, causal) for i in range(Sq)])
    sums = bf16_np(got).sum(-1)
    assert np.allclose(sums[:, vis > 0], 16.0, atol=0.15) and np.all(sums[:, vis == 0] == 0)


def test_varlen_batch(ops):
    seqs = [320, 1024, 64, 700, 150]
    q, cu, kf, cu_f, kc, cu_c = inputs(2, seqs)
    max_k = max(int(cu_f[i + 1] - cu_f[i]) for i in range(len(seqs)))
    got = run(ops, q, cu, kf, cu_f, kc, cu_c, max(seqs), max_k, True)
    ref = O.stage1_scores(bf16_np(q), kf, kc, cu, cu_f, cu_c, max_k, 128 ** -0.5, True, round_output=False)
    close(bf16_np(got), ref)


def test_selection_chain_bit_exact_on_kernel_scores(ops):
    """BASELINE config 1 shape (2048 tokens, 32/2 heads, topk 16, init 1, local 1): pooled scores, top-k
    indices and packed masks are bit-exact against the oracle applied to the same score tensor."""
    S = 2048
    q, cu, kf, cu_f, kc, cu_c = inputs(3, [S])
    Lk = int(cu_f[-1])
    score = run(ops, q, cu, kf, cu_f, kc, cu_c, S, Lk, True)
    pooled = ops.max_pooling_1d(score, 0, 1, 1)
    ref_pooled = O.max_pooling_1d_fast(bf16_np(score), 0, 1, 1)
    assert np.array_equal(bf16_np(pooled), ref_pooled)
    idx = ops.topk_blocks(pooled, 16)
    ref_idx = O.topk_blocks(ref_pooled, 16)
    assert np.array_equal(idx.cpu().numpy(), ref_idx)
    words, kb = ops.topk_to_uint64(idx, S, 64)
    assert kb == 32 and np.array_equal(words_np(words), O.topk_to_uint64(ref_idx, S, 64)[0])
    # forced blocks (block 0, diagonal, previous) are always selected
    bits = ops.uint64_to_bool(words, 32).cpu().numpy()
    for t in (0, 63, 64, 700, 2047):
        b = t // 64
        assert bits[:, t, 0].all() and bits[:, t, b].all() and bits[:, t, max(b - 1, 0)].all()
