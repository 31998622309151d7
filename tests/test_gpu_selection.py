"""GPU parity of the selection front end's extra entry points: compressed-key construction and the one-call
selection (compress -> fused Stage-1/pool -> top-k).

Compressed keys are bit-exact against the oracle (fp32 sum in window order, one rounding; the rule of
compress_tensor, tests/test_stage1_compressed_lse.py:56-99).  The one-call selection must pick exactly the blocks
the separate calls pick."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def rand_k(seed, total, Hk=2):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(total, Hk, 128, generator=g).to(torch.bfloat16)


@pytest.mark.parametrize("seqs,kernel,stride", [([2048], 32, 16), ([2048], 128, 64), ([1000], 32, 16), ([31], 32, 16),
                                                ([32], 32, 16), ([320, 1024, 64, 700, 150, 5], 32, 16),
                                                ([320, 1024, 64, 700, 150, 5], 128, 64), ([200, 100], 16, 16)])
def test_compress_keys_bit_exact(ops, seqs, kernel, stride):
    k = rand_k(1, sum(seqs))
    cu = np.cumsum([0] + seqs).astype(np.int32)
    ref, ref_cu = O.compress_keys(bf16_np(k), cu, kernel, stride)
    got, got_cu = ops.compress_keys(k.cuda(), torch.from_numpy(cu).cuda(), max(seqs), kernel, stride)
    assert np.array_equal(got_cu.cpu().numpy(), ref_cu)
    n = int(ref_cu[-1])
    assert got.shape[0] >= n and np.array_equal(bf16_np(got[:n]), ref)


@pytest.mark.parametrize("Hk", [1, 4, 40])
def test_compress_keys_other_head_counts(ops, Hk):
    k = rand_k(5, 300, Hk)
    cu = np.array([0, 300], np.int32)
    ref, _ = O.compress_keys(bf16_np(k), cu, 32, 16)
    got, _ = ops.compress_keys(k.cuda(), torch.from_numpy(cu).cuda(), 300, 32, 16)
    assert np.array_equal(bf16_np(got), ref)


def test_compress_keys_strided_input(ops):
    """k as a slice of a fused qkv projection output: row stride larger than heads * d."""
    g = torch.Generator(device="cpu").manual_seed(2)
    qkv = torch.randn(900, 36, 128, generator=g).to(torch.bfloat16).cuda()
    k = qkv[:, 32:34]
    cu = torch.tensor([0, 900], dtype=torch.int32, device="cuda")
    got, got_cu = ops.compress_keys(k, cu, 900, 32, 16)
    ref, ref_cu = O.compress_keys(bf16_np(k), np.array([0, 900], np.int32), 32, 16)
    assert np.array_equal(bf16_np(got), ref) and int(got_cu[-1]) == ref.shape[0]


def test_compress_keys_append(ops):
    """A decode loop extends the compressed keys as tokens arrive: rows below first_row stay as they were."""
    k = rand_k(3, 1024).cuda()
    cu = lambda n: torch.tensor([0, n], dtype=torch.int32, device="cuda")
    full, _ = ops.compress_keys(k, cu(1024), 1024, 32, 16)
    buf = torch.zeros_like(full)
    part, cu_part = ops.compress_keys(k[:512], cu(512), 512, 32, 16)
    buf[:part.shape[0]] = part
    rows_before = int(cu_part[-1])
    marker = buf[:rows_before].clone()
    _, cu_all = ops.compress_keys(k, cu(1024), 1024, 32, 16, out=buf, first_row=rows_before)
    assert int(cu_all[-1]) == full.shape[0]
    assert torch.equal(buf[:rows_before], marker) and torch.equal(buf, full)


@pytest.mark.parametrize("seqs,topk,local,init", [([2048], 16, 1, 1), ([4096], 64, 31, 1), ([700, 1300, 64, 300], 8, 2, 1)])
def test_select_blocks_equals_separate_calls(ops, seqs, topk, local, init):
    g = torch.Generator(device="cpu").manual_seed(4)
    T = sum(seqs)
    q = torch.randn(T, 32, 128, generator=g).to(torch.bfloat16).cuda()
    k = torch.randn(T, 2, 128, generator=g).to(torch.bfloat16).cuda()
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    cu = torch.from_numpy(cu_np).cuda()
    packed = len(seqs) > 1
    cache_lens = torch.zeros(len(seqs), dtype=torch.int32, device="cuda") if packed else None
    idx = ops.select_blocks(q, k, cu, cu, max(seqs), max(seqs), topk, local, init, cache_lens=cache_lens)
    # the reference's sequence of calls on caller-side (oracle) compressed keys
    kf, cu_f = O.compress_keys(bf16_np(k), cu_np, 32, 16)
    kc, cu_c = O.compress_keys(bf16_np(k), cu_np, 128, 64)
    dev = lambda a, dt=None: (torch.from_numpy(np.ascontiguousarray(a)) if dt is None else torch.from_numpy(np.ascontiguousarray(a)).to(dt)).cuda()
    max_lk = max(int(cu_f[i + 1] - cu_f[i]) for i in range(len(seqs)))
    score = ops.infllmv2_attn_stage1(q, dev(kf, torch.bfloat16), dev(kc, torch.bfloat16), cu, dev(cu_f), dev(cu_c),
                                     max(seqs), max_lk, causal=True)
    if packed:
        pooled = ops.max_pooling_1d_varlen(score, cu, dev(cu_f), cache_lens, max(seqs), max_lk, local, init)
    else:
        pooled = ops.max_pooling_1d(score, 0, local, init)
    chain = ops.topk_blocks(pooled, topk)
    assert idx.dtype == torch.int32 and tuple(idx.shape) == (2, T, topk)
    assert torch.equal(idx, chain)
    assert np.array_equal(idx.cpu().numpy(), O.topk_blocks(bf16_np(pooled), topk))
    # and the selection drives Stage 2
    out = ops.infllmv2_attn_varlen_func(q, k, k, cu, cu, max(seqs), max(seqs), causal=True, topk_idx=idx)
    assert torch.isfinite(out.float()).all()
