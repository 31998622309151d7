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
    with pytest.raises(RuntimeError, match="new key / value to be appended"):      # flash_api.cpp:1774
        f(q.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=L.to(dev), topk_idx=idx.to(dev),
          rotary_cos=torch.ones(128, 32, device=dev, dtype=torch.bfloat16), rotary_sin=torch.zeros(128, 32, device=dev, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="does not support cache_batch_idx"):    # flash_api.cpp:1596
        f(q.to(dev), kc.view(1, 128, 2, 128).to(dev), vc.view(1, 128, 2, 128).to(dev), cache_seqlens=L.to(dev),
          block_table=torch.zeros(1, 1, dtype=torch.int32, device=dev), cache_batch_idx=torch.zeros(1, dtype=torch.int32, device=dev))
    with pytest.raises(RuntimeError, match="seqlen_q == 1"):
        f(torch.cat([q, q], 1).to(dev), kc.to(dev), vc.to(dev), cache_seqlens=L.to(dev))


# ---------------------------------------------------------------------------------------------------------------
# the remaining options of mha_fwd_kvcache: cache_batch_idx, cache_leftpad, paged cache, rotary on append
# ---------------------------------------------------------------------------------------------------------------
def rotary_tables(seed, n_pos, half):
    g = torch.Generator(device="cpu").manual_seed(seed)
    theta = (torch.rand(n_pos, half, generator=g) * 2 - 1) * 3.14159
    return torch.cos(theta).to(torch.bfloat16), torch.sin(theta).to(torch.bfloat16)


def check_ext(ops, q, kc, vc, lens, idx, cap, new=None, num_splits=0, **opts):
    """Runs the operator and the oracle with the same options and compares outputs, LSE and the updated caches."""
    dev = torch.device("cuda:0")
    d = lambda t: None if t is None else t.to(dev)
    kcd, vcd = d(kc).clone(), d(vc).clone()
    kn, vn = new if new is not None else (None, None)
    out, lse = ops.infllmv2_attn_with_kvcache(d(q), kcd, vcd, k=d(kn), v=d(vn), cache_seqlens=d(lens), topk_idx=d(idx),
                                              num_splits=num_splits, return_softmax_lse=True,
                                              **{k: (d(v) if torch.is_tensor(v) else v) for k, v in opts.items()})
    words = None if idx is None else O.topk_to_uint64(idx.numpy(), cap, 64)[0]
    kc2, vc2 = bf16_np(kc).copy(), bf16_np(vc).copy()
    np_opts = {}
    for k_, v_ in opts.items():
        key = {"cache_leftpad": "cache_leftpad", "cache_batch_idx": "cache_batch_idx", "block_table": "block_table",
               "rotary_cos": "rotary_cos", "rotary_sin": "rotary_sin", "rotary_interleaved": "rotary_interleaved"}[k_]
        np_opts[key] = (bf16_np(v_) if v_.dtype == torch.bfloat16 else v_.numpy()) if torch.is_tensor(v_) else v_
    ro, rl = O.decode_forward_ext(bf16_np(q), kc2, vc2, lens.numpy(), words, 128 ** -0.5,
                                  None if kn is None else bf16_np(kn), None if vn is None else bf16_np(vn), **np_opts)
    check(out, lse, ro, rl)
    if kn is not None:
        # appended rows: V bit-exact, K within one bf16 rounding of the oracle's fp32 rotation
        assert np.array_equal(bf16_np(vcd), vc2)
        dk = np.abs(bf16_np(kcd) - kc2)
        assert (dk <= 2.0 ** -7 * np.abs(kc2) + 1e-6).all()
        if "rotary_cos" not in opts:
            assert np.array_equal(bf16_np(kcd), kc2)
    return out, lse


@pytest.mark.parametrize("num_splits", [0, 1, 3])
def test_cache_batch_idx(ops, num_splits):
    q, kc, vc, kn, vn, lens, idx = make(11, 3, 512, [200, 333, 448], 4, new=1)
    big_k = torch.randn(6, 512, 2, 128).to(torch.bfloat16)
    big_v = torch.randn(6, 512, 2, 128).to(torch.bfloat16)
    where = torch.tensor([4, 0, 2], dtype=torch.int32)
    big_k[where.long()], big_v[where.long()] = kc, vc
    check_ext(ops, q, big_k, big_v, lens, idx, 512, new=(kn, vn), num_splits=num_splits, cache_batch_idx=where)


@pytest.mark.parametrize("new", [0, 2])
def test_cache_leftpad(ops, new):
    """Keys of sequence b are cache rows [pad_b, cache_seqlens_b); mask block j starts at row pad_b + 64 j."""
    q, kc, vc, kn, vn, lens, idx = make(12, 3, 640, [200, 333, 448], 4, new=new)
    pad = torch.tensor([7, 64, 30], dtype=torch.int32)
    check_ext(ops, q, kc, vc, lens + pad, idx, 640, new=(kn, vn) if new else None, cache_leftpad=pad)


@pytest.mark.parametrize("page,new", [(64, 0), (128, 1), (256, 3)])
def test_paged_cache(ops, page, new):
    B, cap = 3, 1024
    q, kc, vc, kn, vn, lens, idx = make(13, B, cap, [500, 1000, 64], 6, new=new)
    n_pages = B * cap // page + 5
    g = torch.Generator(device="cpu").manual_seed(14)
    table = torch.randperm(n_pages, generator=g)[:B * cap // page].view(B, cap // page).to(torch.int32)
    pk = torch.randn(n_pages, page, 2, 128, generator=g).to(torch.bfloat16)
    pv = torch.randn(n_pages, page, 2, 128, generator=g).to(torch.bfloat16)
    pk[table.view(-1).long()] = kc.view(B * cap // page, page, 2, 128)
    pv[table.view(-1).long()] = vc.view(B * cap // page, page, 2, 128)
    out, lse = check_ext(ops, q, pk, pv, lens, idx, cap, new=(kn, vn) if new else None, block_table=table)
    # same sequences in a contiguous cache give the same answer
    o2, l2, _, _ = run(ops, q, kc, vc, kn, vn, lens, idx)
    assert torch.equal(out, o2) and torch.equal(lse, l2)


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("rotary_dim", [128, 64, 32])
def test_rotary_on_append(ops, interleaved, rotary_dim):
    q, kc, vc, kn, vn, lens, idx = make(15, 3, 512, [200, 333, 448], 4, new=2)
    cos, sin = rotary_tables(16, 512, rotary_dim // 2)
    check_ext(ops, q, kc, vc, lens, idx, 512, new=(kn, vn), rotary_cos=cos, rotary_sin=sin, rotary_interleaved=interleaved)


def test_rotary_with_leftpad_and_splits(ops):
    q, kc, vc, kn, vn, lens, idx = make(17, 2, 640, [300, 500], 5, new=1)
    pad = torch.tensor([16, 100], dtype=torch.int32)
    cos, sin = rotary_tables(18, 640, 64)
    check_ext(ops, q, kc, vc, lens + pad, idx, 640, new=(kn, vn), num_splits=4, cache_leftpad=pad, rotary_cos=cos,
              rotary_sin=sin, rotary_interleaved=False)
