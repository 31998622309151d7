"""GPU parity of decode against a KV cache (infllmv2_attn_with_kvcache) with the CPU oracle.

Tolerance as for the Stage-2 forward: max-abs <= 2e-2, mean-abs <= 1e-3, LSE max-abs <= 2e-3.
The reference's own decode test (tests/test_kvcache_simple.py:17-78: cache_len 10000, half of the blocks
selected, batch 1, new k/v appended) only prints the difference to a dense masked softmax."""
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


def make(seed, B, cap, lens, k_sel, Hk=2, new=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, 1, 16 * Hk, 128, generator=g).to(torch.bfloat16)
    kc = torch.randn(B, cap, Hk, 128, generator=g).to(torch.bfloat16)
    vc = torch.randn(B, cap, Hk, 128, generator=g).to(torch.bfloat16)
    kn = torch.randn(B, new, Hk, 128, generator=g).to(torch.bfloat16) if new else None
    vn = torch.randn(B, new, Hk, 128, generator=g).to(torch.bfloat16) if new else None
    idx = torch.full((B, Hk, 1, k_sel), -1, dtype=torch.int32)
    for b in range(B):
        nb = (lens[b] + new + 63) // 64
        for h in range(Hk):
            sel = torch.randperm(nb, generator=g)[:k_sel]
            idx[b, h, 0, :len(sel)] = sel.sort().values.to(torch.int32)
    return q, kc, vc, kn, vn, torch.tensor(lens, dtype=torch.int32), idx


def run(ops, q, kc, vc, kn, vn, lens, idx, num_splits=0, scale=None):
    dev = torch.device("cuda:0")
    d = lambda t: None if t is None else t.to(dev)
    kcd, vcd = d(kc).clone(), d(vc).clone()
    out, lse = ops.infllmv2_attn_with_kvcache(d(q), kcd, vcd, k=d(kn), v=d(vn), cache_seqlens=d(lens), topk_idx=d(idx),
                                              num_splits=num_splits, return_softmax_lse=True, softmax_scale=scale)
    return out, lse, kcd, vcd


def reference(q, kc, vc, kn, vn, lens, idx, scale=128 ** -0.5):
    cap = kc.shape[1]
    words = None if idx is None else O.topk_to_uint64(idx.numpy(), cap, 64)[0]
    kc2, vc2 = bf16_np(kc).copy(), bf16_np(vc).copy()
    o, l = O.decode_forward(bf16_np(q), kc2, vc2, lens.numpy(), words, scale,
                            None if kn is None else bf16_np(kn), None if vn is None else bf16_np(vn))
    return o, l, kc2, vc2


def check(out, lse, ro, rl):
    err = np.abs(bf16_np(out) - ro)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    l = lse.cpu().numpy().astype(np.float64)
    fin = np.isfinite(rl)
    assert np.array_equal(np.isinf(l), ~fin) and np.abs(l[fin] - rl[fin]).max() <= 2e-3


@pytest.mark.parametrize("B,cap,lens,k_sel,new", [
    (3, 300, [100, 257, 64], 3, 0),
    (3, 300, [100, 256, 63], 3, 1),           # append one token, crossing a block boundary for sequence 1
    (1, 10048, [10000], 78, 1),               # tests/test_kvcache_simple.py:78 shape: half of 157 blocks
    (4, 2048, [2048, 1, 1000, 777], 8, 0),
    (2, 4096, [4000, 3000], 64, 0),
])
def test_decode(ops, B, cap, lens, k_sel, new):
    q, kc, vc, kn, vn, L, idx = make(0, B, cap, lens, k_sel, new=new)
    out, lse, kcd, vcd = run(ops, q, kc, vc, kn, vn, L, idx)
    ro, rl, kc2, vc2 = reference(q, kc, vc, kn, vn, L, idx)
    assert out.shape == q.shape and tuple(lse.shape) == (B, 32, 1)
    check(out, lse, ro, rl)
    if new:                                   # caches updated in place, nothing else touched
        assert np.array_equal(bf16_np(kcd), kc2) and np.array_equal(bf16_np(vcd), vc2)


def test_result_independent_of_split_count(ops):
    q, kc, vc, kn, vn, L, idx = make(1, 2, 8192, [8000, 5000], 40)
    ro, rl, _, _ = reference(q, kc, vc, kn, vn, L, idx)
    outs = []
    for s in (1, 2, 3, 7, 16, 64):
        out, lse, _, _ = run(ops, q, kc, vc, kn, vn, L, idx, num_splits=s)
        check(out, lse, ro, rl)
        outs.append(bf16_np(out))
    assert max(np.abs(o - outs[0]).max() for o in outs) <= 8e-3     # splits only regroup an fp32 sum


def test_dense_decode_and_int_cache_seqlens(ops):
    dev = torch.device("cuda:0")
    q, kc, vc, _, _, L, _ = make(2, 2, 512, [300, 300], 1)
    out = ops.infllmv2_attn_with_kvcache(q.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=300, softmax_scale=0.07)
    ro, rl = O.decode_forward(bf16_np(q), bf16_np(kc), bf16_np(vc), [300, 300], None, 0.07)
    err = np.abs(bf16_np(out) - ro)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3


def test_decode_rejects_unsupported(ops):
    dev = torch.device("cuda:0")
    q, kc, vc, _, _, L, idx = make(3, 1, 128, [100], 1)
    f = ops.infllmv2_attn_with_kvcache
    with pytest.raises(RuntimeError, match="not supported"):
        f(q.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=L.to(dev), topk_idx=idx.to(dev), rotary_cos=torch.ones(1, device=dev))
    with pytest.raises(RuntimeError, match="seqlen_q == 1"):
        f(torch.cat([q, q], 1).to(dev), kc.to(dev), vc.to(dev), cache_seqlens=L.to(dev))
