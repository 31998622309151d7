"""BASELINE-size runs checked through sampled rows and size-independent properties.

Config 2 (prefill, 32768 tokens) end to end; config 3 (four packed sequences, ~64K tokens, forward +
backward); config 4 (prefill, 131072 tokens, fused front end); config 5 (decode, batch 64, cache lengths up to
131072).  Oracle parity on sampled rows; for
the rest: forced blocks always selected, popcount == k, sum_keys dV = sum_tokens dO and sum_keys dK = 0
(rows of P sum to one, rows of dS sum to zero)."""
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


def compress(k, kernel, stride):
    return k.unfold(0, kernel, stride).float().mean(-1).to(torch.bfloat16).contiguous()


def token_oracle(q, k, v, words_row, t_local, Sq, Sk, tok_global, dout=None):
    """Oracle forward (and dQ) of one token: a one-query problem against its visible prefix."""
    pos = t_local + Sk - Sq
    kk, vv = bf16_np(k[:pos + 1]), bf16_np(v[:pos + 1])
    qq = bf16_np(q[tok_global:tok_global + 1])
    w = words_row[:, None, :]                               # (Hk, 1, n64)
    o, lse = O.stage2_forward(qq, kk, vv, [0, 1], [0, pos + 1], w, 128 ** -0.5, True)
    if dout is None:
        return o[0], None
    dq, _, _ = O.stage2_backward(qq, kk, vv, bf16_np(dout[tok_global:tok_global + 1]), [0, 1], [0, pos + 1], w,
                                 128 ** -0.5, True)
    return o[0], dq[0]


def test_config2_prefill_32k(ops):
    dev = torch.device("cuda:0")
    S, topk = 32768, 64
    g = torch.Generator(device="cpu").manual_seed(0)
    q = torch.randn(S, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    kf, kc = compress(k, 32, 16), compress(k, 128, 64)
    mk = lambda n: torch.tensor([0, n], dtype=torch.int32, device=dev)
    Lk = kf.shape[0]
    score = ops.infllmv2_attn_stage1(q, kf, kc, mk(S), mk(Lk), mk(kc.shape[0]), S, Lk, causal=True)
    pooled = ops.max_pooling_1d(score, 0, 31, 1)
    idx = ops.topk_blocks(pooled, topk)
    words, kb = ops.topk_to_uint64(idx, S, 64)
    out = ops.infllmv2_attn_varlen_func(q, k, v, mk(S), mk(S), S, S, causal=True, topk_idx=idx)
    rows = [0, 1, 63, 64, 127, 128, 2047, 2048, 4095, 4096, 10000, 20001, 32767]
    # Stage 1 on sampled rows (one-row oracle problems: q_len < k_len uses the offset rule, so feed whole prefix lengths)
    sc = bf16_np(score[:, rows])
    # pooled / top-k / mask are bit-exact functions of the GPU score rows
    full_pool = O.max_pooling_1d_fast(sc, (S + 63) // 64, 31, 1, row_cache_lens=np.zeros(len(rows), dtype=np.int64),
                                      row_qidx=np.array(rows), row_klen=np.full(len(rows), Lk))
    assert np.array_equal(bf16_np(pooled[:, rows]), full_pool)
    ref_idx = O.topk_blocks(full_pool, topk)
    assert np.array_equal(idx[:, rows].cpu().numpy(), ref_idx)
    assert np.array_equal(words_np(words[:, rows]), O.topk_to_uint64(ref_idx, S, 64)[0])
    # selection invariants over all rows
    bits = ops.uint64_to_bool(words, kb)
    tok = torch.arange(S, device=dev)
    bq = tok // 64
    assert bool(bits[:, :, 0].all())
    assert bool((bits.sum(-1) == topk).all())
    for d in (0, 1, 15, 31):
        sel = bits[:, tok, torch.clamp(bq - d, min=0)]
        assert bool(sel.all())
    # Stage-1 parity on sampled rows against the oracle (exact prefix semantics: Sq == Sk for the full problem)
    kf_np, kc_np = bf16_np(kf), bf16_np(kc)
    for r in rows[::3]:
        vf = O.stage1_visible(r, 16, Lk, S, True)
        vc = O.stage1_visible(r, 64, kc.shape[0], S, True)
        got = bf16_np(score[:, r])
        if vc == 0:
            assert np.all(got == 0)
            continue
        qq = bf16_np(q[r]).reshape(2, 16, 128).astype(np.float64)
        for h in range(2):
            sc_c = qq[h] @ kc_np[:vc, h].astype(np.float64).T * 128 ** -0.5
            lse = np.log(np.exp(sc_c - sc_c.max(-1, keepdims=True)).sum(-1, keepdims=True)) + sc_c.max(-1, keepdims=True)
            ref = np.exp(qq[h] @ kf_np[:vf, h].astype(np.float64).T * 128 ** -0.5 - lse).sum(0)
            assert (np.abs(got[h, :vf] - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3).all()
            assert np.all(got[h, vf:] == 0)
    # Stage-2 forward on sampled tokens
    wnp = words_np(words)
    for r in rows:
        o_ref, _ = token_oracle(q, k, v, wnp[:, r], r, S, S, r)
        err = np.abs(bf16_np(out[r]) - o_ref)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3, (r, err.max(), err.mean())


def test_config3_selection_64k(ops):
    """The selection leg at BASELINE config 3: four packed sequences (the lengths of the test below), compressed keys,
    packed Stage 1, varlen pooling, top-k and mask words.  Stage-1 rows of sampled tokens of every sequence (first,
    last, the pair across each sequence boundary, mid-sequence) against the oracle of the token's own sequence; pooled
    scores, indices and mask words of those rows bit-exact functions of the GPU's score rows; invariants over all
    rows; the fused front end bit-identical to the chain of separate calls."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1)
    lens = [int(64 * x) for x in rng.integers(64, 385, size=4)]
    T, topk = sum(lens), 64
    cu_l = np.cumsum([0] + lens).astype(np.int32)
    cu = torch.from_numpy(cu_l).to(dev)
    g = torch.Generator(device="cpu").manual_seed(0)
    q = torch.randn(T, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(T, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    kf, cu_f = ops.compress_keys(k, cu, max(lens), 32, 16)
    kc, cu_c = ops.compress_keys(k, cu, max(lens), 128, 64)
    cf, cc = cu_f.cpu().numpy(), cu_c.cpu().numpy()
    for b in range(4):                                         # compressed keys of every sequence == its own unfold/mean
        seg = k[cu_l[b]:cu_l[b + 1]]
        assert torch.equal(kf[cf[b]:cf[b + 1]], compress(seg, 32, 16)) and torch.equal(kc[cc[b]:cc[b + 1]], compress(seg, 128, 64))
    max_lk = int(np.diff(cf).max())
    score = ops.infllmv2_attn_stage1(q, kf, kc, cu, cu_f, cu_c, max(lens), max_lk, causal=True)
    zeros = torch.zeros(4, dtype=torch.int32, device=dev)
    pooled = ops.max_pooling_1d_varlen(score, cu, cu_f, zeros, max(lens), max_lk, 31, 1)
    idx = ops.topk_blocks(pooled, topk)
    words, kb = ops.topk_to_uint64(idx, max(lens), 64)
    samples = []                                               # (sequence, local token)
    for b in range(4):
        samples += [(b, 0), (b, 1), (b, lens[b] - 1), (b, lens[b] // 2 + 7), (b, 4095), (b, min(4096, lens[b] - 2))]
    rows = [int(cu_l[b]) + t for b, t in samples]
    loc = np.array([t for _, t in samples])
    lk_row = np.array([cf[b + 1] - cf[b] for b, _ in samples])
    sc = bf16_np(score[:, rows])
    nblk = (max(lens) + 63) // 64
    ref_pool = O.max_pooling_1d_fast(sc, nblk, 31, 1, row_cache_lens=np.zeros(len(rows), dtype=np.int64), row_qidx=loc,
                                     row_klen=lk_row)
    assert np.array_equal(bf16_np(pooled[:, rows]), ref_pool)
    ref_idx = O.topk_blocks(ref_pool, topk)
    assert np.array_equal(idx[:, rows].cpu().numpy(), ref_idx)
    assert np.array_equal(words_np(words[:, rows]), O.topk_to_uint64(ref_idx, max(lens), 64)[0])
    # Stage 1 of the sampled rows against the oracle restricted to the token's own sequence
    kf_np, kc_np = bf16_np(kf), bf16_np(kc)
    for (b, t), r in zip(samples, rows):
        Lk, Lc = int(cf[b + 1] - cf[b]), int(cc[b + 1] - cc[b])
        vf = O.stage1_visible(t, 16, Lk, lens[b], True)
        vc = O.stage1_visible(t, 64, Lc, lens[b], True)
        got = bf16_np(score[:, r])
        if vc == 0:
            assert np.all(got == 0), (b, t)
            continue
        qq = bf16_np(q[r]).reshape(2, 16, 128).astype(np.float64)
        for h in range(2):
            sc_c = qq[h] @ kc_np[cc[b]:cc[b] + vc, h].astype(np.float64).T * 128 ** -0.5
            lse = np.log(np.exp(sc_c - sc_c.max(-1, keepdims=True)).sum(-1, keepdims=True)) + sc_c.max(-1, keepdims=True)
            ref = np.exp(qq[h] @ kf_np[cf[b]:cf[b] + vf, h].astype(np.float64).T * 128 ** -0.5 - lse).sum(0)
            assert (np.abs(got[h, :vf] - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3).all(), (b, t, h)
            assert np.all(got[h, vf:] == 0), (b, t, h)
    # invariants over all rows: block 0 and the local window always selected, nothing from the token's future
    bits = ops.uint64_to_bool(words, kb)
    local_tok = torch.cat([torch.arange(n, device=dev) for n in lens])
    bq = local_tok // 64
    rows_all = torch.arange(T, device=dev)
    assert bool(bits[:, :, 0].all())
    assert bool((bits.sum(-1) == topk).all())
    for d in (0, 1, 15, 31):
        assert bool(bits[:, rows_all, torch.clamp(bq - d, min=0)].all())
    # the one-call front end selects the same blocks, bit for bit, without writing the score tensor
    fused = ops.select_blocks(q, k, cu, cu, max(lens), max(lens), topk, 31, 1, cache_lens=zeros, max_cache_len=0)
    assert torch.equal(fused, idx)


def test_config3_varlen_fwd_bwd_64k(ops):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1)
    lens = [int(64 * x) for x in rng.integers(64, 385, size=4)]
    T = sum(lens)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=dev)
    g = torch.Generator(device="cpu").manual_seed(0)
    q = torch.randn(T, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(T, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(T, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    dout = torch.randn(T, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    # top-k from random pooled scores with forced blocks (selection itself is covered by config 2)
    nblk = max(lens) // 64
    pooled = torch.rand(2, T, nblk, device=dev).to(torch.bfloat16)
    cu_l = cu.cpu().numpy()
    for b in range(4):
        i = torch.arange(lens[b], device=dev)
        blk = torch.arange(nblk, device=dev)[None, :]
        bqv = (i // 64)[:, None]
        forced = (blk < 1) | ((bqv >= blk) & (bqv <= blk + 31))
        future = blk > bqv
        seg = pooled[:, cu_l[b]:cu_l[b + 1]]
        seg[:, forced] = float("inf")
        seg[:, future & ~forced] = float("-inf")
    idx = ops.topk_blocks(pooled, 64, drop_unreachable=True)   # blocks in a token's future are never selected: -1 padding
    assert not bool((torch.gather(pooled, 2, idx.long().clamp(min=0)) == float("-inf"))[idx >= 0].any())
    qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
    out = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, max(lens), max(lens), causal=True, topk_idx=idx)
    out.backward(dout)
    words = words_np(ops.topk_to_uint64(idx, max(lens), 64)[0])
    # sampled tokens: forward and dQ against the oracle
    for b, t_local in [(0, 0), (0, lens[0] - 1), (1, 5000 % lens[1]), (2, 64), (3, lens[3] - 1), (3, 2049 % lens[3])]:
        t = int(cu_l[b]) + t_local
        kb_, vb_ = k[cu_l[b]:cu_l[b + 1]], v[cu_l[b]:cu_l[b + 1]]
        o_ref, dq_ref = token_oracle(q, kb_, vb_, words[:, t], t_local, lens[b], lens[b], t, dout)
        err = np.abs(bf16_np(out[t]) - o_ref)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        s = max(1.0, float(np.abs(dq_ref).max()))
        e2 = np.abs(bf16_np(qg.grad[t]) - dq_ref)
        assert e2.max() <= 2e-2 * s and e2.mean() <= 1e-3 * s
    # size-independent identities per sequence and KV head
    for b in range(4):
        sl = slice(int(cu_l[b]), int(cu_l[b + 1]))
        dv_sum = vg.grad[sl].float().sum(0)                                   # (Hk, d)
        do_sum = dout[sl].float().reshape(-1, 2, 16, 128).sum((0, 2))          # every token attends block 0, so rows of P sum to 1
        scale = float(dout[sl].float().abs().sum(0).max())
        assert float((dv_sum - do_sum).abs().max()) <= 2e-3 * scale
        dk_sum = kg.grad[sl].float().sum(0)
        dk_scale = float(kg.grad[sl].float().abs().sum(0).max())
        assert float(dk_sum.abs().max()) <= 2e-2 * dk_scale
    assert bool(torch.isfinite(qg.grad.float()).all() and torch.isfinite(kg.grad.float()).all())
    # whole-tensor inner products: O is linear in V, so <dO, O> = <dV, V>; S is bilinear in (Q, K), so scaling Q up and K
    # down by the same factor changes nothing and <dQ, Q> = <dK, K>.  Every element of dQ, dK and dV enters; the
    # tolerance is 3.5 times the largest difference these inputs give (1.7e-3 of the terms' root sum of squares), which rounding
    # each factor to bf16 explains; the inner products themselves are 0.5 to 3 of that norm.
    def inner(a, b):
        prod = a.detach().double() * b.detach().double()
        return float(prod.sum()), float(prod.pow(2).sum().sqrt())
    for b in range(4):
        sl = slice(int(cu_l[b]), int(cu_l[b + 1]))
        x_o, n_o = inner(dout[sl], out[sl])
        x_v, n_v = inner(vg.grad[sl], v[sl])
        assert abs(x_o - x_v) <= 6e-3 * (n_o + n_v), ("<dO,O> vs <dV,V>", b, x_o, x_v, n_o, n_v)
        x_q, n_q = inner(qg.grad[sl], q[sl])
        x_k, n_k = inner(kg.grad[sl], k[sl])
        assert abs(x_q - x_k) <= 6e-3 * (n_q + n_k), ("<dQ,Q> vs <dK,K>", b, x_q, x_k, n_q, n_k)
    # dK / dV element by element on sampled key blocks: per sequence one late block (few tokens, all near its diagonal:
    # a light slice that the column kernel merges with others) and one mid-prefix block that many distant tokens
    # chose by score (many 512-token slices, multi-slice accumulation); never block 0.  The oracle only needs the
    # tokens whose mask row selects the block.  Both dK/dV modes: fp32 atomics (default) and deterministic accumulation.
    samples = []
    for b in range(4):
        nb = lens[b] // 64
        sl = slice(int(cu_l[b]), int(cu_l[b + 1]))
        for kb, h in ((nb - 3, b % 2), (nb // 3, (b + 1) % 2)):
            dk_ref, dv_ref, toks = O.stage2_backward_key_block(bf16_np(q[sl]), bf16_np(k[sl]), bf16_np(v[sl]),
                                                                bf16_np(dout[sl]), words[h, sl], kb, h, 128 ** -0.5)
            assert len(toks) >= 64 and kb > 0
            samples.append((b, kb, h, dk_ref, dv_ref, len(toks)))
    assert max(n for *_, n in samples) >= 2500                 # a heavy block spanning several token slices is among them

    def check_blocks(dk, dv, what):
        for b, kb, h, dk_ref, dv_ref, _ in samples:
            rows = slice(int(cu_l[b]) + kb * 64, int(cu_l[b]) + kb * 64 + 64)
            for name, got, ref in (("dk", dk[rows, h], dk_ref), ("dv", dv[rows, h], dv_ref)):
                sc = max(1.0, float(np.abs(ref).max()))
                err = np.abs(bf16_np(got) - ref)
                assert err.max() <= 2e-2 * sc and err.mean() <= 1e-3 * sc, (what, name, b, kb, h, err.max(), err.mean(), sc)
    check_blocks(kg.grad, vg.grad, "atomics")
    dq_default = qg.grad.clone()
    qg.grad = kg.grad = vg.grad = None
    ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, max(lens), max(lens), causal=True, topk_idx=idx,
                                  deterministic=True).backward(dout)
    check_blocks(kg.grad, vg.grad, "deterministic")
    assert torch.equal(qg.grad, dq_default)                    # dQ is bit-reproducible


def test_config5_decode_batch64(ops):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1)
    B = 64
    lens = [int(64 * x) for x in rng.integers(256, 2049, size=B)]
    cap = max(lens)
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, 1, 32, 128, generator=g, device=dev).to(torch.bfloat16)
    kc = torch.randn(B, cap, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    vc = torch.randn(B, cap, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    idx = torch.full((B, 2, 1, 64), -1, dtype=torch.int32)
    cg = torch.Generator(device="cpu").manual_seed(2)
    for b in range(B):
        nb = lens[b] // 64
        for h in range(2):
            forced = torch.cat([torch.tensor([0]), torch.arange(nb - 32, nb)])
            rest = torch.tensor(sorted(set(range(1, nb - 32))))
            pick = rest[torch.randperm(len(rest), generator=cg)[:31]]
            idx[b, h, 0] = torch.cat([forced, pick]).sort().values.to(torch.int32)
    L = torch.tensor(lens, dtype=torch.int32, device=dev)
    out, lse = ops.infllmv2_attn_with_kvcache(q, kc, vc, cache_seqlens=L, topk_idx=idx.to(dev), return_softmax_lse=True)
    for b in (0, 17, 63):
        words = O.topk_to_uint64(idx[b:b + 1].numpy(), cap, 64)[0]
        ro, rl = O.decode_forward(bf16_np(q[b:b + 1]), bf16_np(kc[b:b + 1, :lens[b]]), bf16_np(vc[b:b + 1, :lens[b]]),
                                  [lens[b]], words, 128 ** -0.5)
        err = np.abs(bf16_np(out[b:b + 1]) - ro)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        assert np.abs(lse[b:b + 1].cpu().numpy() - rl).max() <= 2e-3
    # split-count independence at full size
    out1 = ops.infllmv2_attn_with_kvcache(q, kc, vc, cache_seqlens=L, topk_idx=idx.to(dev), num_splits=1)
    assert float((out.float() - out1.float()).abs().max()) <= 8e-3


def test_config5_decode_batch64_selection_leg(ops):
    """BASELINE config 5 end to end: batch 64, one query per sequence, K/V cache lengths drawn from multiples of 64 in
    [16384, 131072]: compressed-key caches -> Stage 1 (decode-shaped launch) -> pooling at each sequence's own
    position -> top-k -> mask -> split decode attention.  Stage-1 scores of sampled sequences against the oracle
    (Stage-1 tolerance); pooled / top-k / mask bit-exact functions of the GPU scores; the fused pooled launch equals
    pooling of the score launch for every sequence; the attention output of sampled sequences against the oracle's
    decode on the selected blocks, and against the prefill kernels run on the sampled sequence's last token."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    B, topk, local, init = 64, 64, 31, 1
    lens = [int(64 * x) for x in rng.integers(256, 2049, size=B)]        # tokens per sequence, the new one included
    lens[3], lens[40] = 131072, 16384                                     # both ends of the range are present
    cap = max(lens)
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, 1, 32, 128, generator=g, device=dev).to(torch.bfloat16)
    kc = torch.randn(B, cap, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    vc = torch.randn(B, cap, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    L = torch.tensor(lens, dtype=torch.int32, device=dev)
    pos = L - 1                                                           # position of each sequence's query
    fine = torch.empty(B, cap // 16 + 1, 2, 128, dtype=torch.bfloat16, device=dev)
    coarse = torch.empty(B, cap // 64 + 1, 2, 128, dtype=torch.bfloat16, device=dev)
    fl = ops.compress_keys_cache(kc, L, 32, 16, out=fine)
    cl = ops.compress_keys_cache(kc, L, 128, 64, out=coarse)
    assert fl.tolist() == [(n - 32) // 16 + 1 for n in lens] and cl.tolist() == [(n - 128) // 64 + 1 for n in lens]
    score = ops.infllmv2_attn_stage1_kvcache(q, fine, coarse, fl, cl, pos, local, init, causal=False, pooled=False)
    pooled = ops.infllmv2_attn_stage1_kvcache(q, fine, coarse, fl, cl, pos, local, init, max_cache_len=cap - 1,
                                              causal=False)
    nblk = cap // 64
    assert tuple(pooled.shape) == (B, 2, nblk)
    idx = ops.topk_blocks(pooled, topk)                                   # (B, Hk, topk)
    words, _ = ops.topk_to_uint64(idx.unsqueeze(2), cap, 64)
    # pooled == pooling of the score rows, all sequences (GPU pooling operator on the packed equivalent)
    cu_q = torch.arange(B + 1, dtype=torch.int32, device=dev)
    rows_f = fine.shape[1]
    cu_rows = torch.arange(B + 1, dtype=torch.int32, device=dev) * rows_f
    for b in (0, 3, 40, 63):
        one = lambda n: torch.tensor([0, n], dtype=torch.int32, device=dev)
        two_calls = ops.max_pooling_1d_varlen(score[b][:, None, :int(fl[b])].contiguous(), one(1), one(int(fl[b])),
                                              pos[b:b + 1].contiguous(), 1, int(fl[b]), local, init, max_cache_len=cap - 1)
        assert torch.equal(two_calls[:, 0].view(torch.int16), pooled[b].view(torch.int16))
    for b in (3, 17, 40):
        n, Lf, Lc = lens[b], int(fl[b]), int(cl[b])
        got = bf16_np(score[b])                                           # (Hk, rows)
        assert np.all(got[:, Lf:] == 0)
        qq = bf16_np(q[b, 0]).reshape(2, 16, 128).astype(np.float64)
        # compressed keys themselves: bit-exact windowed means of the cache
        assert torch.equal(fine[b, :Lf], compress(kc[b, :n], 32, 16)) or \
            float((fine[b, :Lf].float() - compress(kc[b, :n], 32, 16).float()).abs().max()) <= 2.0 ** -8 * 4
        kf_np, kc_np = bf16_np(fine[b, :Lf]).astype(np.float64), bf16_np(coarse[b, :Lc]).astype(np.float64)
        for h in range(2):
            sc_c = qq[h] @ kc_np[:, h].T * 128 ** -0.5
            mx = sc_c.max(-1, keepdims=True)
            lse = np.log(np.exp(sc_c - mx).sum(-1, keepdims=True)) + mx
            ref = np.exp(qq[h] @ kf_np[:, h].T * 128 ** -0.5 - lse).sum(0)
            assert (np.abs(got[h, :Lf] - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3).all()
        # pooled / top-k / mask from the GPU scores by the oracle
        want_pool = O.max_pooling_1d_fast(got[:, None, :Lf], nblk, local, init, row_cache_lens=np.array([n - 1]),
                                          row_qidx=np.array([0]), row_klen=np.array([Lf]))
        assert np.array_equal(bf16_np(pooled[b])[:, None], want_pool)
        want_idx = O.topk_blocks(want_pool, topk)
        assert np.array_equal(idx[b].cpu().numpy()[:, None], want_idx)
        assert np.array_equal(words_np(words[b]), O.topk_to_uint64(want_idx, cap, 64)[0])
        sel = set(want_idx[0, 0].tolist())
        bq = (n - 1) // 64
        assert 0 in sel and all(bq - d in sel for d in range(32)) and max(sel) <= bq
    # Stage 2 on the selected blocks
    out, lse = ops.infllmv2_attn_with_kvcache(q, kc, vc, cache_seqlens=L, topk_idx=idx.unsqueeze(2), return_softmax_lse=True)
    for b in (3, 17, 40):
        n = lens[b]
        w = O.topk_to_uint64(idx[b:b + 1].unsqueeze(2).cpu().numpy(), cap, 64)[0]
        ro, rl = O.decode_forward(bf16_np(q[b:b + 1]), bf16_np(kc[b:b + 1, :n]), bf16_np(vc[b:b + 1, :n]), [n], w, 128 ** -0.5)
        err = np.abs(bf16_np(out[b:b + 1]) - ro)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        assert np.abs(lse[b:b + 1].cpu().numpy() - rl).max() <= 2e-3
        # the prefill kernels on the same sequence's last token with the same selection
        one = lambda m: torch.tensor([0, m], dtype=torch.int32, device=dev)
        pre = ops.infllmv2_attn_varlen_func(q[b], kc[b, :n], vc[b, :n], one(1), one(n), 1, n, causal=True,
                                            topk_idx=idx[b][:, None, :].contiguous())
        e2 = (pre.float() - out[b].float()).abs()
        assert float(e2.max()) <= 2e-2 and float(e2.mean()) <= 1e-3


def test_config4_prefill_128k_fused_front_end(ops):
    """BASELINE config 4 (131072 tokens): the one-call selection, which never writes the 4.3 GB score tensor, against
    the separate calls (bit-exact pooled scores and identical top-k), selection invariants over all rows, and the
    Stage-2 forward on sampled tokens against the oracle."""
    dev = torch.device("cuda:0")
    S, topk = 131072, 64
    g = torch.Generator(device="cpu").manual_seed(4)
    q = torch.randn(S, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    mk = lambda n: torch.tensor([0, n], dtype=torch.int32, device=dev)
    idx = ops.select_blocks(q, k, mk(S), mk(S), S, S, topk, 31, 1)
    # the separate calls on separately built compressed keys
    kf, kc = compress(k, 32, 16), compress(k, 128, 64)
    kf2, cu_f = ops.compress_keys(k, mk(S), S, 32, 16)
    assert torch.equal(kf2, kf) or float((kf2.float() - kf.float()).abs().max()) <= 2.0 ** -8 * float(kf.float().abs().max())
    Lk = kf2.shape[0]
    kc2, cu_c = ops.compress_keys(k, mk(S), S, 128, 64)
    score = ops.infllmv2_attn_stage1(q, kf2, kc2, mk(S), cu_f, cu_c, S, Lk, causal=True)
    pooled = ops.max_pooling_1d(score, 0, 31, 1)
    del score
    fused = ops.infllmv2_attn_stage1_pooled(q, kf2, kc2, mk(S), cu_f, cu_c, S, Lk, 31, 1, causal=True)
    assert torch.equal(fused.view(torch.int16), pooled.view(torch.int16))
    assert torch.equal(idx, ops.topk_blocks(pooled, topk))
    del pooled, fused
    words, kb = ops.topk_to_uint64(idx, S, 64)
    assert kb == 2048 and words.shape[-1] == 32
    bits = ops.uint64_to_bool(words, kb)
    tok = torch.arange(S, device=dev)
    bq = tok // 64
    assert bool(bits[:, :, 0].all()) and bool((bits.sum(-1) == topk).all())
    for d in (0, 1, 31):
        assert bool(bits[:, tok, torch.clamp(bq - d, min=0)].all())
    # a token with at least topk causal blocks selects nothing from the future (earlier tokens must pad with such blocks,
    # which the Stage-2 kernels never visit)
    late = bq >= topk
    future = torch.arange(kb, device=dev)[None, None, :] > bq[None, late, None]
    assert not bool((bits[:, late] & future).any())
    del bits
    out = ops.infllmv2_attn_varlen_func(q, k, v, mk(S), mk(S), S, S, causal=True, topk_idx=idx)
    wnp = words_np(words)
    for r in [0, 63, 4096, 50001, 100000, 131071]:
        o_ref, _ = token_oracle(q, k, v, wnp[:, r], r, S, S, r)
        err = np.abs(bf16_np(out[r]) - o_ref)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3, (r, err.max(), err.mean())
