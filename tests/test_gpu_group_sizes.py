"""Group sizes other than 16 (1, 2, 4, 8 query heads per KV head) through every attention entry point, and head
sizes below 128 through the wrappers that pad them.

The reference's Python is written for any group size (infllmv2_sparse_attention.py:76-88, 546-555) but its native code
divides by 16 everywhere (flash_api.cpp:706-710, 941, 1397): only 16 runs there.  Here smaller groups run on the same
16-row tiles, the spare rows repeating the group's last head with LSE = +inf so that they add nothing to the Stage-1
head sum or to dK / dV.  Checked against the CPU oracle, which is written for any group size.  Tolerances as for 16:
Stage-1 |err| <= 2^-7 |ref| + 2e-3; Stage-2 forward / decode max-abs <= 2e-2, mean-abs <= 1e-3, LSE <= 2e-3; gradients
max-abs <= 2e-2 s, mean-abs <= 1e-3 s with s = max(1, max|ref|); pooling / top-k bit-exact on the GPU's scores."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np, words_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF = torch.bfloat16


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def rand(shape, seed, dtype=BF):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def random_selection(seed, Hk, seqs, k_sel):
    g = torch.Generator(device="cpu").manual_seed(seed)
    idx = torch.full((Hk, sum(seqs), k_sel), -1, dtype=torch.int32)
    row = 0
    for s in seqs:
        nb = (s + 63) // 64
        for t in range(row, row + s):
            for h in range(Hk):
                sel = torch.randperm(nb, generator=g)[:k_sel].sort().values
                idx[h, t, :len(sel)] = sel.to(torch.int32)
        row += s
    return idx


@pytest.mark.parametrize("G,Hk", [(1, 3), (2, 2), (4, 2), (8, 1), (8, 3)])
@pytest.mark.parametrize("mode", ["atomics", "deterministic"])
def test_stage2_forward_backward(ops, G, Hk, mode):
    seqs = [300, 650]
    T = sum(seqs)
    q, k, v, dout = rand((T, G * Hk, 128), 1), rand((T, Hk, 128), 2), rand((T, Hk, 128), 3), rand((T, G * Hk, 128), 4)
    idx = random_selection(5, Hk, seqs, 4)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    cu = torch.from_numpy(cu_np).to(DEV)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out, lse, _ = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, max(seqs), max(seqs), causal=True,
                                                topk_idx=idx.to(DEV), return_attn_probs=True,
                                                deterministic=(mode == "deterministic"))
    out.backward(dout.to(DEV))
    assert tuple(lse.shape) == (Hk, T * G)
    words = O.topk_to_uint64(idx.numpy(), max(seqs), 64)[0]
    qn, kn, vn, dn = [bf16_np(t) for t in (q, k, v, dout)]
    ref_o, ref_lse = O.stage2_forward(qn, kn, vn, cu_np, cu_np, words, 128 ** -0.5, True)
    err = np.abs(bf16_np(out).astype(np.float64) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    l = lse.cpu().numpy().astype(np.float64)
    fin = np.isfinite(ref_lse)                               # a token none of whose selected blocks is visible: +inf
    assert np.array_equal(np.isinf(l) & (l > 0), ~fin) and np.abs(l[fin] - ref_lse[fin]).max() <= 2e-3
    dq, dk, dv = O.stage2_backward(qn, kn, vn, dn, cu_np, cu_np, words, 128 ** -0.5, True)
    for name, got, ref in (("dq", qg.grad, dq), ("dk", kg.grad, dk), ("dv", vg.grad, dv)):
        s = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got).astype(np.float64) - ref)
        assert e.max() <= 2e-2 * s and e.mean() <= 1e-3 * s, (name, e.max(), e.mean(), s)


def test_dense_and_noncausal_and_fp16(ops):
    """Dense attention (no mask), non-causal, in fp16, group size 4; and a group-16 run of the same heads regrouped
    must agree with it: 8 heads over 2 KV heads == the same 8 query heads when K/V heads are repeated to 8 with g = 1."""
    T, G, Hk = 333, 4, 2
    q, k, v = rand((T, G * Hk, 128), 6, torch.float16), rand((T, Hk, 128), 7, torch.float16), rand((T, Hk, 128), 8, torch.float16)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    out = ops.infllmv2_attn_varlen_func(q.to(DEV), k.to(DEV), v.to(DEV), cu, cu, T, T, causal=False)
    ref, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), [0, T], [0, T], None, 128 ** -0.5, False)
    err = np.abs(bf16_np(out).astype(np.float64) - ref)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3
    k1, v1 = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)          # MHA view of the same problem
    out1 = ops.infllmv2_attn_varlen_func(q.to(DEV), k1.to(DEV), v1.to(DEV), cu, cu, T, T, causal=False)
    assert float((out.float() - out1.float()).abs().max()) <= 2e-3


@pytest.mark.parametrize("G", [1, 2, 4, 8])
def test_stage1_scores_pooled_topk_and_decode_shape(ops, G):
    """Stage 1 (prefill kernel, the one-query kernel, fused pooling) sums over the group's heads only."""
    Hk = 2
    seqs = [900, 260]
    T = sum(seqs)
    q, k = rand((T, G * Hk, 128), 9), rand((T, Hk, 128), 10)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    kf, cu_f = O.compress_keys(bf16_np(k), cu_np, 32, 16)
    kc, cu_c = O.compress_keys(bf16_np(k), cu_np, 128, 64)
    Lk = int(max(np.diff(cu_f)))
    t = lambda x, dt=None: torch.from_numpy(np.ascontiguousarray(x)).to(DEV) if dt is None else torch.from_numpy(np.ascontiguousarray(x)).to(dt).to(DEV)
    args = (q.to(DEV), t(kf, BF), t(kc, BF), t(cu_np), t(cu_f), t(cu_c), max(seqs), Lk)
    score = ops.infllmv2_attn_stage1(*args, causal=True)
    ref = O.stage1_scores(bf16_np(q), kf, kc, cu_np, cu_f, cu_c, Lk, 128 ** -0.5, True, round_output=False)
    got = bf16_np(score).astype(np.float64)
    assert (np.abs(got - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3).all()
    assert got.max() > 0.05                                  # spare tile rows adding anything would break the bound above
    cache_lens = torch.zeros(2, dtype=torch.int32, device=DEV)
    sep = ops.max_pooling_1d_varlen(score, t(cu_np), t(cu_f), cache_lens, max(seqs), Lk, 1, 1)
    fused = ops.infllmv2_attn_stage1_pooled(*args, 1, 1, cache_lens=cache_lens, causal=True)
    assert torch.equal(sep.view(torch.int16), fused.view(torch.int16))
    # one query per sequence (the decode-shaped kernel): the last token of each sequence against all its keys
    last = torch.tensor([seqs[0] - 1, T - 1])
    q1 = q[last].to(DEV)
    cu1 = torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV)
    s1 = ops.infllmv2_attn_stage1(q1, t(kf, BF), t(kc, BF), cu1, t(cu_f), t(cu_c), 1, Lk, causal=False)
    ref1 = O.stage1_scores(bf16_np(q[last]), kf, kc, np.array([0, 1, 2], np.int32), cu_f, cu_c, Lk, 128 ** -0.5, False,
                           round_output=False)
    assert (np.abs(bf16_np(s1).astype(np.float64) - ref1) <= 2.0 ** -7 * np.abs(ref1) + 2e-3).all()


@pytest.mark.parametrize("G,splits", [(1, 1), (2, 4), (8, 0)])
def test_decode_with_append(ops, G, splits):
    B, cap, Hk = 3, 512, 2
    q, kc, vc = rand((B, 1, G * Hk, 128), 11), rand((B, cap, Hk, 128), 12), rand((B, cap, Hk, 128), 13)
    kn, vn = rand((B, 1, Hk, 128), 14), rand((B, 1, Hk, 128), 15)
    lens = np.array([70, 447, 256], dtype=np.int32)
    g = torch.Generator(device="cpu").manual_seed(16)
    nblk = cap // 64
    bits = torch.rand(B, Hk, 1, nblk, generator=g) < 0.6
    bits[..., 0] = True
    words = O.blockmask_to_uint64(bits.numpy())[0]
    idx = torch.full((B, Hk, 1, nblk), -1, dtype=torch.int32)
    for b in range(B):
        for h in range(Hk):
            sel = torch.nonzero(bits[b, h, 0]).flatten().to(torch.int32)
            idx[b, h, 0, :len(sel)] = sel
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    out, lse = ops.infllmv2_attn_with_kvcache(q.to(DEV), kcd, vcd, k=kn.to(DEV), v=vn.to(DEV),
                                              cache_seqlens=torch.from_numpy(lens).to(DEV), topk_idx=idx.to(DEV),
                                              return_softmax_lse=True, num_splits=splits)
    kc_np, vc_np = bf16_np(kc).copy(), bf16_np(vc).copy()
    ref_o, ref_lse = O.decode_forward_ext(bf16_np(q), kc_np, vc_np, lens, words, 128 ** -0.5, k_new=bf16_np(kn),
                                          v_new=bf16_np(vn))
    assert tuple(out.shape) == (B, 1, G * Hk, 128) and tuple(lse.shape) == (B, G * Hk, 1)
    err = np.abs(bf16_np(out).astype(np.float64) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 2e-3


def test_layer_decode_steps_equal_prefill_group4(ops):
    """The whole call sequence at group size 4: every decode step reproduces the prefill of the longer sequence."""
    G, Hk, start, steps = 4, 2, 600, 20
    total = start + steps
    q, k, v = rand((total, G * Hk, 128), 17).to(DEV), rand((total, Hk, 128), 18).to(DEV), rand((total, Hk, 128), 19).to(DEV)
    cu = lambda n: torch.tensor([0, n], dtype=torch.int32, device=DEV)
    layer = ops.InfLLMv2Attention(topk=5, local_blocks=1, init_blocks=1)
    full = layer(q, k, v, cu(total), total)
    cache = ops.SequenceCache.empty(total + 64, Hk, 128, DEV)
    layer(q[:start], k[:start], v[:start], cu(start), start, cache=cache)
    checked = 0
    for t in range(start, total):
        o1 = layer.decode(q[t][None, None], k[t][None, None], v[t][None, None], cache)
        L = t + 1
        if L % 16 == 15 or L % 64 == 63:
            continue
        e = (o1[0, 0].float() - full[t].float()).abs()
        assert float(e.max()) <= 2e-2 and float(e.mean()) <= 1e-3, t
        checked += 1
    assert checked >= steps * 3 // 4


def test_unsupported_group_is_rejected(ops):
    q, k, v = rand((64, 6, 128), 20).to(DEV), rand((64, 2, 128), 21).to(DEV), rand((64, 2, 128), 22).to(DEV)
    cu = torch.tensor([0, 64], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="1, 2, 4, 8 or 16"):
        ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, 64, 64, causal=True)


@pytest.mark.parametrize("d", [64, 80, 32])
def test_head_sizes_below_128_by_zero_padding(ops, d):
    """The wrapper pads the head dimension with zeros up to the kernels' 128, as the reference's wrapper pads it to a
    multiple of 8 (infllmv2_sparse_attention.py:299-303, 336, 381): forward, gradients (at the caller's width) and the
    selection front end against the oracle at the original head size, default scale d ** -0.5."""
    seqs = [400, 270]
    T, G, Hk = sum(seqs), 16, 2
    q, k, v, dout = rand((T, G * Hk, d), 30), rand((T, Hk, d), 31), rand((T, Hk, d), 32), rand((T, G * Hk, d), 33)
    idx = random_selection(34, Hk, seqs, 4)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    cu = torch.from_numpy(cu_np).to(DEV)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, max(seqs), max(seqs), causal=True, topk_idx=idx.to(DEV))
    assert tuple(out.shape) == (T, G * Hk, d)
    out.backward(dout.to(DEV))
    words = O.topk_to_uint64(idx.numpy(), max(seqs), 64)[0]
    qn, kn, vn, dn = [bf16_np(t) for t in (q, k, v, dout)]
    ref_o, _ = O.stage2_forward(qn, kn, vn, cu_np, cu_np, words, d ** -0.5, True)
    err = np.abs(bf16_np(out).astype(np.float64) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    dq, dk, dv = O.stage2_backward(qn, kn, vn, dn, cu_np, cu_np, words, d ** -0.5, True)
    for name, got, ref in (("dq", qg.grad, dq), ("dk", kg.grad, dk), ("dv", vg.grad, dv)):
        assert tuple(got.shape) == ref.shape
        s = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got).astype(np.float64) - ref)
        assert e.max() <= 2e-2 * s and e.mean() <= 1e-3 * s, (name, e.max(), e.mean(), s)
    # Stage 1 on compressed keys of the original width
    kf, cu_f = O.compress_keys(kn, cu_np, 32, 16)
    kc, cu_c = O.compress_keys(kn, cu_np, 128, 64)
    Lk = int(max(np.diff(cu_f)))
    t = lambda x, dt=None: torch.from_numpy(np.ascontiguousarray(x)).to(DEV) if dt is None else torch.from_numpy(np.ascontiguousarray(x)).to(dt).to(DEV)
    score = ops.infllmv2_attn_stage1(q.to(DEV), t(kf, BF), t(kc, BF), cu, t(cu_f), t(cu_c), max(seqs), Lk, causal=True)
    ref = O.stage1_scores(qn, kf, kc, cu_np, cu_f, cu_c, Lk, d ** -0.5, True, round_output=False)
    assert (np.abs(bf16_np(score).astype(np.float64) - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3).all()
    # the whole front end picks what top-k of the pooled oracle-side GPU scores gives
    cache_lens = torch.zeros(2, dtype=torch.int32, device=DEV)
    sel = ops.select_blocks(q.to(DEV), k.to(DEV), cu, cu, max(seqs), max(seqs), 5, 1, 1, cache_lens=cache_lens)
    pooled = ops.max_pooling_1d_varlen(score, cu, t(cu_f), cache_lens, max(seqs), Lk, 1, 1)
    assert torch.equal(sel, ops.topk_blocks(pooled, 5))


def test_head_size_above_128_is_rejected(ops):
    q, k, v = rand((64, 32, 256), 35).to(DEV), rand((64, 2, 256), 36).to(DEV), rand((64, 2, 256), 37).to(DEV)
    cu = torch.tensor([0, 64], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="at most 128"):
        ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, 64, 64, causal=True)
