"""GPU parity of the Stage-2 block-sparse forward against the CPU oracle.

Tolerance (bf16 outputs vs an fp32/fp64 reference on the same bf16-rounded inputs): max-abs <= 2e-2,
mean-abs <= 1e-3; LSE (fp32) max-abs <= 2e-3.  Shapes follow tests/test_infllmv2.py:466-474 of the
reference (seqlens 128..2048, batch 1-2, GQA 32/2 and MQA 16/1, random padding lengths)."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np, words_np

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS, LSE_ABS = 2e-2, 1e-3, 2e-3


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def make_case(seed, sq, sk, Hk, k_sel, device, sort=True):
    g = torch.Generator(device="cpu").manual_seed(seed)
    cu_q = np.cumsum([0] + sq).astype(np.int32)
    cu_k = np.cumsum([0] + sk).astype(np.int32)
    T, Tk = int(cu_q[-1]), int(cu_k[-1])
    q = torch.randn(T, 16 * Hk, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(Tk, Hk, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(Tk, Hk, 128, generator=g).to(torch.bfloat16)
    idx = torch.full((Hk, T, k_sel), -1, dtype=torch.int32)
    for h in range(Hk):
        for b in range(len(sq)):
            nb = (sk[b] + 63) // 64
            for t in range(cu_q[b], cu_q[b + 1]):
                sel = torch.randperm(nb, generator=g)[:k_sel]
                if sort:
                    sel = sel.sort().values
                idx[h, t, :len(sel)] = sel.to(torch.int32)
    to = lambda x: x.to(device)
    return (to(q), to(k), to(v), to(torch.from_numpy(cu_q)), to(torch.from_numpy(cu_k)), to(idx))


def check(out, lse, ref_o, ref_lse):
    o = bf16_np(out).astype(np.float64)
    err = np.abs(o - ref_o)
    assert err.max() <= MAX_ABS and err.mean() <= MEAN_ABS, (err.max(), err.mean())
    l = lse.cpu().numpy().astype(np.float64)
    fin = np.isfinite(ref_lse)
    assert np.array_equal(np.isinf(l) & (l > 0), ~fin)
    assert np.abs(l[fin] - ref_lse[fin]).max() <= LSE_ABS


@pytest.mark.parametrize("sq,sk,Hk,k_sel,causal", [
    ([128], [128], 2, 1, True),
    ([256], [256], 2, 2, True),
    ([512, 300], [512, 300], 2, 3, True),
    ([1000], [1000], 2, 5, True),
    ([2048], [2048], 2, 10, True),
    ([100, 37, 64], [100, 37, 64], 2, 2, True),
    ([70], [200], 2, 2, True),             # q shorter than k: bottom-right aligned causal
    ([200], [70], 2, 1, True),             # q longer than k: first 130 tokens see nothing
    ([64], [130], 2, 3, False),
    ([256], [256], 1, 2, True),            # MQA 16/1
    ([1], [1], 2, 1, True),
])
def test_sparse_forward(ops, sq, sk, Hk, k_sel, causal):
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(42, sq, sk, Hk, k_sel, dev)
    out, lse, s_dmask = ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, max(sq), max(sk), causal=causal,
                                                     topk_idx=idx, return_attn_probs=True)
    assert out.shape == q.shape and out.dtype == torch.bfloat16
    assert tuple(lse.shape) == (Hk, q.shape[0] * 16) and s_dmask.numel() == 0
    words, _ = O.topk_to_uint64(idx.cpu().numpy(), max(sk), 64)
    ref_o, ref_lse = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_q.cpu().numpy(), cu_k.cpu().numpy(),
                                      words, 128 ** -0.5, causal)
    check(out, lse, ref_o, ref_lse)


def test_sparse_forward_unsorted_indices_and_scale(ops):
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(7, [300], [300], 2, 4, dev, sort=False)
    out = ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, 300, 300, softmax_scale=0.05, causal=True, topk_idx=idx)
    words, _ = O.topk_to_uint64(idx.cpu().numpy(), 300, 64)
    ref_o, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), [0, 300], [0, 300], words, 0.05, True)
    err = np.abs(bf16_np(out) - ref_o)
    assert err.max() <= MAX_ABS and err.mean() <= MEAN_ABS


def test_dense_forward(ops):
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, _ = make_case(9, [200, 131], [200, 131], 2, 1, dev)
    out, lse, _ = ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, 200, 200, causal=True, return_attn_probs=True)
    ref_o, ref_lse = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_q.cpu().numpy(), cu_k.cpu().numpy(),
                                      None, 128 ** -0.5, True)
    assert tuple(lse.shape) == (32, 331)                 # dense path: (nheads, total_q)
    ref_dense = ref_lse.reshape(2, 331, 16).transpose(0, 2, 1).reshape(32, 331)
    check(out, lse, ref_o, ref_dense)


def test_forward_noncontiguous_inputs(ops):
    """q/k/v given as slices of a fused qkv buffer (dense last dim, larger row stride)."""
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(11, [192], [192], 2, 2, dev)
    fused = torch.zeros(192, 32 + 2 + 2, 128, dtype=torch.bfloat16, device=dev)
    fused[:, :32], fused[:, 32:34], fused[:, 34:36] = q, k, v
    a = ops.infllmv2_attn_varlen_func(fused[:, :32], fused[:, 32:34], fused[:, 34:36], cu_q, cu_k, 192, 192,
                                      causal=True, topk_idx=idx)
    b = ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, 192, 192, causal=True, topk_idx=idx)
    assert torch.equal(a, b)


def test_rejected_options_raise_like_the_reference(ops):
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(1, [64], [64], 2, 1, dev)
    f = ops.infllmv2_attn_varlen_func
    with pytest.raises(RuntimeError, match="does not support dropout"):
        f(q, k, v, cu_q, cu_k, 64, 64, dropout_p=0.1, topk_idx=idx)
    with pytest.raises(RuntimeError, match="does not support softcap"):
        f(q, k, v, cu_q, cu_k, 64, 64, softcap=1.0, topk_idx=idx)
    with pytest.raises(RuntimeError, match="does not support local attention"):
        f(q, k, v, cu_q, cu_k, 64, 64, window_size=(16, 0), topk_idx=idx)
    with pytest.raises(RuntimeError, match="does not support alibi"):
        f(q, k, v, cu_q, cu_k, 64, 64, alibi_slopes=torch.ones(32, device=dev), topk_idx=idx)
    with pytest.raises(RuntimeError, match="same dtype"):
        f(q, k.float(), v, cu_q, cu_k, 64, 64, topk_idx=idx)
    with pytest.raises(RuntimeError, match="int32"):
        f(q, k, v, cu_q.long(), cu_k, 64, 64, topk_idx=idx)
    with pytest.raises(AssertionError):
        f(q, k, v, cu_q, cu_k, 64, 64, topk_idx=idx.long())


def test_causal_flag_follows_the_window_like_the_reference(ops):
    """flash_api.cpp:137, 600, 621-622: window (-1, 0) IS causal whatever the `causal` argument says, and a left window
    that reaches max_seqlen_k counts as unbounded."""
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(3, [200], [200], 2, 2, dev)
    f = ops.infllmv2_attn_varlen_func
    want = f(q, k, v, cu_q, cu_k, 200, 200, causal=True, topk_idx=idx)
    assert torch.equal(f(q, k, v, cu_q, cu_k, 200, 200, causal=False, window_size=(-1, 0), topk_idx=idx), want)
    assert torch.equal(f(q, k, v, cu_q, cu_k, 200, 200, causal=False, window_size=(200, 0), topk_idx=idx), want)
    assert torch.equal(f(q, k, v, cu_q, cu_k, 200, 200, causal=True, window_size=(4096, 4096), topk_idx=idx), want)
    non_causal = f(q, k, v, cu_q, cu_k, 200, 200, causal=False, topk_idx=idx)
    assert not torch.equal(non_causal, want)
    assert torch.equal(f(q, k, v, cu_q, cu_k, 200, 200, causal=False, window_size=(300, 200), topk_idx=idx), non_causal)
    with pytest.raises(RuntimeError, match="does not support local attention"):
        f(q, k, v, cu_q, cu_k, 200, 200, causal=False, window_size=(199, 0), topk_idx=idx)
