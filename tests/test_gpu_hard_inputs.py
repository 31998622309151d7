"""Numerically hard inputs and BASELINE config 1 through the GPU path.

* Large logits: q scaled by 8 (logits ~ N(0, 64): the softmax is nearly one-hot, running maxima move a lot, the
  rescale-skip and the -inf paths of the online softmax are exercised), plus planted keys that hand chosen rows a
  dominant logit in their FIRST block (block 0: every later block must not move the maximum) and in their LAST block
  (the token's own key: the maximum arrives at the very end of the walk).  Forward, backward and decode against the
  oracle with the usual tolerances (outputs are convex combinations of V rows, so the absolute tolerance stands;
  gradients scale with max |ref|).
* Config 1 at its exact parameters (one sequence of 2048 tokens, topk 16, block 0 and the two most recent blocks
  forced, compressed keys 32/16, causal): every token of the forward against the oracle.
Reference tolerances for context: tests/test_infllmv2.py:331, 348-350."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np, words_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def planted_case(seed, S, k_sel, q_gain):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = (torch.randn(S, 32, 128, generator=g) * q_gain).to(torch.bfloat16)
    k = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16)
    nb = (S + 63) // 64
    idx = torch.full((2, S, k_sel), -1, dtype=torch.int32)
    for h in range(2):
        for t in range(S):
            bq = t // 64
            forced = {0, bq, max(bq - 1, 0)}
            rest = [b for b in torch.randperm(bq + 1, generator=g).tolist() if b not in forced][:k_sel - len(forced)]
            sel = sorted(forced | set(rest))
            idx[h, t, :len(sel)] = torch.tensor(sel, dtype=torch.int32)
    # planted keys: a key that is a multiple of one query head's vector gives that row a logit far above the rest
    planted = []
    for t, head, where in ((S - 1, 3, "last"), (S - 70, 20, "last"), (S - 5, 17, "first"), (S // 2 + 7, 9, "first"),
                           (S // 2 + 8, 30, "middle")):
        key = {"last": t, "first": 5 + len(planted), "middle": 64 * int(idx[head // 16, t, 1]) + 11}[where]
        unit = q[t, head].float() / q[t, head].float().norm()
        k[key, head // 16] = (unit * 40.0).to(torch.bfloat16)
        planted.append((t, head, key))
    return q, k, v, idx, planted


@pytest.mark.parametrize("S,k_sel,q_gain", [(1500, 6, 8.0), (700, 4, 1.0)])
def test_large_logits_forward_and_backward(ops, S, k_sel, q_gain):
    q, k, v, idx, planted = planted_case(3, S, k_sel, q_gain)
    scale = 128 ** -0.5
    cu = torch.tensor([0, S], dtype=torch.int32, device=DEV)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    dout = torch.randn(S, 32, 128, generator=torch.Generator(device="cpu").manual_seed(4)).to(torch.bfloat16)
    out, lse, _ = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, S, S, causal=True, topk_idx=idx.to(DEV),
                                                return_attn_probs=True)
    out.backward(dout.to(DEV))
    words, _ = O.topk_to_uint64(idx.numpy(), S, 64)
    ref_o, ref_lse = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), [0, S], [0, S], words, scale, True)
    err = np.abs(bf16_np(out) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    # the LSE of a row with logits in the hundreds: absolute 2e-3 on values around 1e2 is 2e-5 relative (fp32 holds 6e-8)
    assert np.abs(lse.detach().cpu().numpy() - ref_lse).max() <= 2e-3 * max(1.0, np.abs(ref_lse).max() / 16)
    # the planted rows really are dominated by their planted key
    probs_check = 0
    for t, head, key in planted:
        logits = (bf16_np(q[t, head]) @ bf16_np(k[:t + 1, head // 16]).T) * scale
        sel_blocks = set(int(x) for x in idx[head // 16, t].tolist() if x >= 0)
        if key // 64 in sel_blocks:
            assert logits[key] >= logits.max() - 1e-3 and logits[key] > 30
            probs_check += 1
    assert probs_check >= 4
    dq, dk, dv = O.stage2_backward(bf16_np(q), bf16_np(k), bf16_np(v), bf16_np(dout), [0, S], [0, S], words, scale, True)
    for name, got, ref in (("dq", qg.grad, dq), ("dk", kg.grad, dk), ("dv", vg.grad, dv)):
        sc = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got) - ref)
        assert e.max() <= 2e-2 * sc and e.mean() <= 1e-3 * sc, (name, e.max(), e.mean(), sc)


def test_large_logits_backward_deterministic(ops):
    deterministic = True
    S, k_sel = 900, 5
    q, k, v, idx, _ = planted_case(5, S, k_sel, 8.0)
    cu = torch.tensor([0, S], dtype=torch.int32, device=DEV)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    dout = torch.randn(S, 32, 128, generator=torch.Generator(device="cpu").manual_seed(6)).to(torch.bfloat16)
    ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, S, S, causal=True, topk_idx=idx.to(DEV),
                                  deterministic=deterministic).backward(dout.to(DEV))
    words, _ = O.topk_to_uint64(idx.numpy(), S, 64)
    dq, dk, dv = O.stage2_backward(bf16_np(q), bf16_np(k), bf16_np(v), bf16_np(dout), [0, S], [0, S], words, 128 ** -0.5, True)
    for name, got, ref in (("dq", qg.grad, dq), ("dk", kg.grad, dk), ("dv", vg.grad, dv)):
        sc = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got) - ref)
        assert e.max() <= 2e-2 * sc and e.mean() <= 1e-3 * sc, (name, e.max(), e.mean(), sc)


def test_large_logits_decode(ops):
    """Decode with q x 8 and, per sequence, a planted dominant key in the first / the last selected block; several
    split counts (the combine merges partial maxima that differ by tens of units)."""
    B, cap, k_sel = 4, 4096, 12
    lens = [4096, 3000, 1025, 700]
    g = torch.Generator(device="cpu").manual_seed(7)
    q = (torch.randn(B, 1, 32, 128, generator=g) * 8).to(torch.bfloat16)
    kc = torch.randn(B, cap, 2, 128, generator=g).to(torch.bfloat16)
    vc = torch.randn(B, cap, 2, 128, generator=g).to(torch.bfloat16)
    idx = torch.full((B, 2, 1, k_sel), -1, dtype=torch.int32)
    for b in range(B):
        nb = (lens[b] + 63) // 64
        for h in range(2):
            sel = sorted({0, nb - 1} | set(torch.randperm(nb, generator=g)[:k_sel - 2].tolist()))[:k_sel]
            idx[b, h, 0, :len(sel)] = torch.tensor(sel, dtype=torch.int32)
        for head, key in ((2, 3), (21, lens[b] - 1)):          # first block for head 2, the very last key for head 21
            unit = q[b, 0, head].float() / q[b, 0, head].float().norm()
            kc[b, key, head // 16] = (unit * 5.0).to(torch.bfloat16)
    L = torch.tensor(lens, dtype=torch.int32)
    words = O.topk_to_uint64(idx.numpy(), cap, 64)[0]
    ro, rl = O.decode_forward(bf16_np(q), bf16_np(kc), bf16_np(vc), L.numpy(), words, 128 ** -0.5)
    for splits in (0, 1, 3, 7):
        out, lse = ops.infllmv2_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), cache_seqlens=L.to(DEV),
                                                  topk_idx=idx.to(DEV), num_splits=splits, return_softmax_lse=True)
        err = np.abs(bf16_np(out) - ro)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3, (splits, err.max(), err.mean())
        assert np.abs(lse.cpu().numpy() - rl).max() <= 2e-3 * max(1.0, np.abs(rl).max() / 16)


def test_config1_all_tokens_forward(ops):
    """BASELINE config 1 on the GPU: 2048 tokens, topk 16, init 1, local 1 (block 0 and the two most recent blocks
    forced).  Scores to the Stage-1 tolerance; pooled / top-k / mask bit-exact functions of the GPU scores; the
    Stage-2 output of EVERY token against the oracle on the selected blocks; and the oracle's own end-to-end result
    (its scores, its selection): rows where both selections agree meet the tolerance, and nearly all rows agree."""
    S, topk, init, local = 2048, 16, 1, 1
    r = np.random.default_rng(0)
    mk = lambda h: torch.from_numpy(O.bf16_round(r.standard_normal((S, h, 128)).astype(np.float32))).to(torch.bfloat16)
    q, k, v = mk(32), mk(2), mk(2)
    cu_np = np.array([0, S], np.int32)
    kf, cu_f = O.compress_keys(bf16_np(k), cu_np, 32, 16)
    kc, cu_c = O.compress_keys(bf16_np(k), cu_np, 128, 64)
    Lk = int(cu_f[-1])
    to = lambda a, dt=None: (torch.from_numpy(np.ascontiguousarray(a)) if dt is None else torch.from_numpy(np.ascontiguousarray(a)).to(dt)).to(DEV)
    qd, kd, vd, cu = q.to(DEV), k.to(DEV), v.to(DEV), to(cu_np)
    score = ops.infllmv2_attn_stage1(qd, to(kf, torch.bfloat16), to(kc, torch.bfloat16), cu, to(cu_f), to(cu_c), S, Lk, causal=True)
    ref_score = O.stage1_scores(bf16_np(q), kf, kc, cu_np, cu_f, cu_c, Lk, 128 ** -0.5, True, round_output=False)
    got_score = bf16_np(score)
    assert (np.abs(got_score - ref_score) <= 2.0 ** -7 * np.abs(ref_score) + 2e-3).all()
    pooled = ops.max_pooling_1d(score, 0, local, init)
    assert np.array_equal(bf16_np(pooled), O.max_pooling_1d_fast(got_score, 0, local, init))
    idx = ops.topk_blocks(pooled, topk)
    assert np.array_equal(idx.cpu().numpy(), O.topk_blocks(bf16_np(pooled), topk))
    assert torch.equal(idx, ops.select_blocks(qd, kd, cu, cu, S, S, topk, local, init))       # the one-call front end
    words, _ = ops.topk_to_uint64(idx, S, 64)
    assert np.array_equal(words_np(words), O.topk_to_uint64(idx.cpu().numpy(), S, 64)[0])
    out, lse, _ = ops.infllmv2_attn_varlen_func(qd, kd, vd, cu, cu, S, S, causal=True, topk_idx=idx, return_attn_probs=True)
    ref_o, ref_lse = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_np, cu_np, words_np(words), 128 ** -0.5, True)
    err = np.abs(bf16_np(out) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 2e-3
    # the oracle alone, end to end
    o_idx = O.topk_blocks(O.max_pooling_1d_fast(O.bf16_round(ref_score.astype(np.float32)), 0, local, init), topk)
    o_words = O.topk_to_uint64(o_idx, S, 64)[0]
    same = (o_words == words_np(words)).all(axis=-1)                  # (Hk, S): identical selections
    assert same.mean() >= 0.98, same.mean()
    o_out, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_np, cu_np, o_words, 128 ** -0.5, True)
    e2 = np.abs(bf16_np(out) - o_out).reshape(S, 2, 16, 128)
    assert e2[same.T].max() <= 2e-2 and e2.mean() <= 1e-3
