"""GPU parity of Stage-2 forward and backward on masks with InfLLM-V2's structure: every token selects the initial
block, a local window of recent blocks and a few scattered blocks (as max_pooling_1d's forced +inf entries plus
top-k produce, infllm_v2/max_pooling_1d.py:4-43).  Neighbouring tokens then share most of their blocks, which is the
case the kernels treat specially (common blocks staged once per 8 tokens, the rest walked per token; light 512-token
slices of the column walk merged), so these cases exercise the paths that random per-token selections do not:
long common runs (longer than the staging ring), token groups that straddle a sequence end or a query-block
boundary, rows wider than one mask word, q shorter than k, dense (mask-free) attention.

Tolerances as in test_gpu_stage2_fwd.py / test_gpu_stage2_bwd.py."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np
from test_gpu_stage2_fwd import check
from test_gpu_stage2_bwd import check_grad

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def window_case(seed, sq, sk, Hk, window, scattered, device):
    """idx (Hk, T, 1 + window + scattered): block 0, the `window` most recent causal blocks, `scattered` random ones."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    cu_q = np.cumsum([0] + sq).astype(np.int32)
    cu_k = np.cumsum([0] + sk).astype(np.int32)
    T, Tk = int(cu_q[-1]), int(cu_k[-1])
    q = torch.randn(T, 16 * Hk, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(Tk, Hk, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(Tk, Hk, 128, generator=g).to(torch.bfloat16)
    width = 1 + window + scattered
    idx = torch.full((Hk, T, width), -1, dtype=torch.int32)
    for h in range(Hk):
        for b in range(len(sq)):
            nb = (sk[b] + 63) // 64
            for i in range(sq[b]):
                last = min(nb - 1, max(0, (i + sk[b] - sq[b]) // 64))          # block of the causal diagonal
                sel = {0} | set(range(max(0, last - window + 1), last + 1))
                extra = torch.randperm(nb, generator=g)[:scattered].tolist()
                sel |= set(extra)
                sel = sorted(sel)[:width]
                idx[h, cu_q[b] + i, :len(sel)] = torch.tensor(sel, dtype=torch.int32)
    to = lambda x: x.to(device)
    return to(q), to(k), to(v), to(torch.from_numpy(cu_q)), to(torch.from_numpy(cu_k)), to(idx)


CASES = [
    ([1000], [1000], 2, 4, 3),
    ([700, 333], [700, 333], 2, 6, 2),          # token groups straddle the first sequence's end (700 % 8 != 0)
    ([130], [600], 2, 3, 2),                    # q shorter than k: the diagonal sits at block (i + 470) / 64
    ([5000], [5000], 1, 8, 5),                  # 79 key blocks: mask rows of two words
    ([64, 8, 1, 200], [64, 8, 1, 200], 2, 2, 1),
]


@pytest.mark.parametrize("sq,sk,Hk,window,scattered", CASES)
def test_forward_window_masks(ops, sq, sk, Hk, window, scattered):
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = window_case(7, sq, sk, Hk, window, scattered, dev)
    out, lse, _ = ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, max(sq), max(sk), causal=True, topk_idx=idx,
                                                return_attn_probs=True)
    words, _ = O.topk_to_uint64(idx.cpu().numpy(), max(sk), 64)
    ref_o, ref_lse = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_q.cpu().numpy(), cu_k.cpu().numpy(),
                                      words, 128 ** -0.5, True)
    check(out, lse, ref_o, ref_lse)


@pytest.mark.parametrize("sq,sk,Hk,window,scattered", CASES[:4])
def test_backward_window_masks(ops, sq, sk, Hk, window, scattered):
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = window_case(11, sq, sk, Hk, window, scattered, dev)
    g = torch.Generator(device="cpu").manual_seed(12)
    dout = torch.randn(q.shape, generator=g).to(torch.bfloat16).to(dev)
    qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
    out = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu_q, cu_k, max(sq), max(sk), causal=True, topk_idx=idx)
    out.backward(dout)
    words = O.topk_to_uint64(idx.cpu().numpy(), max(sk), 64)[0]
    dq, dk, dv = O.stage2_backward(bf16_np(q), bf16_np(k), bf16_np(v), bf16_np(dout), cu_q.cpu().numpy(),
                                   cu_k.cpu().numpy(), words, 128 ** -0.5, True)
    check_grad("dq", qg.grad, dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vg.grad, dv)


@pytest.mark.parametrize("sq,sk,causal", [([300], [300], True), ([100], [260], False), ([260, 75], [260, 75], True)])
def test_dense_forward_backward(ops, sq, sk, causal):
    """topk_idx=None: every causal block is common to a token group (all of the walk goes through the LDS ring)."""
    dev = torch.device("cuda:0")
    Hk = 2
    g = torch.Generator(device="cpu").manual_seed(3)
    cu_q = np.cumsum([0] + sq).astype(np.int32)
    cu_k = np.cumsum([0] + sk).astype(np.int32)
    q = torch.randn(int(cu_q[-1]), 16 * Hk, 128, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(int(cu_k[-1]), Hk, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(int(cu_k[-1]), Hk, 128, generator=g).to(torch.bfloat16).to(dev)
    dout = torch.randn(q.shape, generator=g).to(torch.bfloat16).to(dev)
    cq, ck = torch.from_numpy(cu_q).to(dev), torch.from_numpy(cu_k).to(dev)
    qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
    out, lse, _ = ops.infllmv2_attn_varlen_func(qg, kg, vg, cq, ck, max(sq), max(sk), causal=causal, topk_idx=None,
                                                return_attn_probs=True)
    ref_o, ref_lse = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_q, cu_k, None, 128 ** -0.5, causal)
    # the dense path returns the LSE as (nheads, total_q); the oracle uses the sparse path's (Hk, total_q * 16)
    assert tuple(lse.shape) == (16 * Hk, q.shape[0])
    lse_expanded = lse.view(Hk, 16, q.shape[0]).permute(0, 2, 1).reshape(Hk, q.shape[0] * 16)
    check(out.detach(), lse_expanded, ref_o, ref_lse)
    out.backward(dout)
    dq, dk, dv = O.stage2_backward(bf16_np(q), bf16_np(k), bf16_np(v), bf16_np(dout), cu_q, cu_k, None, 128 ** -0.5, causal)
    check_grad("dq", qg.grad, dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vg.grad, dv)
