"""Seeded sweep over shapes the fixed cases do not name: packed batches of odd lengths, queries shorter than the
keys, 1 to 3 KV heads, masks built like the selection front end builds them (initial block + a local window shared
by neighbouring tokens + score-chosen blocks, so that both the shared-block and the own-block walks of the
row-parallel kernels, heavy and merged light slices of the column kernel and multi-word mask rows all occur), with
-1 padding and repeated indices.  Forward, LSE and all three gradients against the fp64 oracle; tolerances as in
test_gpu_stage2_fwd.py / test_gpu_stage2_bwd.py."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np

pytestmark = pytest.mark.gpu


def random_case(seed):
    r = np.random.default_rng(seed)
    Hk = int(r.integers(1, 4))
    nseq = int(r.integers(1, 4))
    sk = [int(r.integers(1, 1400)) for _ in range(nseq)]
    if seed % 3 == 0:
        sk[0] = int(r.integers(4100, 5200))                      # more than 64 key blocks: two mask words per row
    same = seed % 2 == 0
    sq = list(sk) if same else [int(r.integers(1, s + 1)) for s in sk]
    if seed % 3 == 0:
        sq[0] = min(sq[0], 600)                                  # keep the oracle fast
    k_sel = int(r.integers(1, 12))
    local = int(r.integers(0, 4))
    T = sum(sq)
    idx = np.full((Hk, T, k_sel), -1, np.int32)
    t0 = 0
    for b in range(nseq):
        nb = (sk[b] + 63) // 64
        for i in range(sq[b]):
            bq = (i + sk[b] - sq[b]) // 64
            forced = [0] + [x for x in range(bq - local, bq + 1) if x > 0]
            for h in range(Hk):
                rest = r.permutation(nb)[:k_sel]
                row = (forced + [int(x) for x in rest])[:k_sel]       # repeats happen: packing is idempotent
                if r.random() < 0.2:
                    row = row[:max(1, len(row) // 2)]                 # short rows keep their -1 padding
                idx[h, t0 + i, :len(row)] = row
        t0 += sq[b]
    mk = lambda *shape: O.bf16_round(r.standard_normal(shape).astype(np.float32))
    return dict(Hk=Hk, sq=sq, sk=sk, k_sel=k_sel, idx=idx, q=mk(T, 16 * Hk, 128), k=mk(sum(sk), Hk, 128),
                v=mk(sum(sk), Hk, 128), dout=mk(T, 16 * Hk, 128), causal=bool(seed % 5 != 4) or not same)


@pytest.mark.parametrize("seed", list(range(200, 216)))
def test_random_case_forward_backward(seed):
    import infllmv2_cuda_impl_amd as ops
    c = random_case(seed)
    print(f"seed {seed}: Hk {c['Hk']} sq {c['sq']} sk {c['sk']} k {c['k_sel']} causal {c['causal']}", flush=True)
    dev = torch.device("cuda:0")
    t = lambda x: torch.from_numpy(x).to(torch.bfloat16).to(dev)
    cu_q = np.cumsum([0] + c["sq"]).astype(np.int32)
    cu_k = np.cumsum([0] + c["sk"]).astype(np.int32)
    q, k, v = [t(c[n]).requires_grad_(True) for n in ("q", "k", "v")]
    out, lse, _ = ops.infllmv2_attn_varlen_func(q, k, v, torch.from_numpy(cu_q).to(dev), torch.from_numpy(cu_k).to(dev),
                                                max(c["sq"]), max(c["sk"]), causal=c["causal"],
                                                topk_idx=torch.from_numpy(c["idx"]).to(dev), return_attn_probs=True)
    out.backward(t(c["dout"]))
    words, _ = O.topk_to_uint64(c["idx"], max(c["sk"]), 64)
    scale = 128 ** -0.5
    ref_o, ref_lse = O.stage2_forward(c["q"], c["k"], c["v"], cu_q, cu_k, words, scale, c["causal"])
    err = np.abs(bf16_np(out) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    l = lse.cpu().numpy().astype(np.float64)
    fin = np.isfinite(ref_lse)
    assert np.array_equal(np.isinf(l) & (l > 0), ~fin)
    if fin.any():
        assert np.abs(l[fin] - ref_lse[fin]).max() <= 2e-3
    dq, dk, dv = O.stage2_backward(c["q"], c["k"], c["v"], c["dout"], cu_q, cu_k, words, scale, c["causal"])
    for name, got, ref in (("dq", q.grad, dq), ("dk", k.grad, dk), ("dv", v.grad, dv)):
        s = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got).astype(np.float64) - ref)
        assert e.max() <= 2e-2 * s and e.mean() <= 1e-3 * s, (name, e.max(), e.mean(), s)


@pytest.mark.parametrize("seed", list(range(300, 312)))
def test_random_case_selection_front_end(seed):
    """Packed batches of arbitrary lengths (shorter than one compression window, not multiples of 16 or 64), 1 to 3
    KV heads, per-sequence cache lengths: Stage-1 scores against the oracle (2^-7 relative + 2e-3); pooling, top-k and
    the packed mask bit-exact against the oracle applied to the GPU's own scores; the fused launch and
    `select_blocks` bit-identical to the chain of separate calls."""
    import infllmv2_cuda_impl_amd as ops
    r = np.random.default_rng(seed)
    Hk = int(r.integers(1, 4))
    seqs = [int(r.integers(1, 900)) for _ in range(int(r.integers(1, 5)))]
    if seed % 4 == 0:
        seqs[0] = int(r.integers(1, 40))
    if max(seqs) < 32:                                         # at least one complete compression window in the batch
        seqs.append(int(r.integers(32, 900)))
    local, init, topk = int(r.integers(0, 4)), int(r.integers(0, 3)), int(r.integers(1, 20))
    use_cache = seed % 3 == 0
    cache = [int(64 * r.integers(0, 3)) if use_cache else 0 for _ in seqs]
    print(f"seed {seed}: Hk {Hk} seqs {seqs} local {local} init {init} topk {topk} cache {cache}", flush=True)
    T = sum(seqs)
    cu = np.cumsum([0] + seqs).astype(np.int32)
    q = O.bf16_round(r.standard_normal((T, 16 * Hk, 128)).astype(np.float32))
    k = O.bf16_round(r.standard_normal((T, Hk, 128)).astype(np.float32))
    kf, cu_f = O.compress_keys(k, cu, 32, 16)
    kc, cu_c = O.compress_keys(k, cu, 128, 64)
    kf, kc = O.bf16_round(kf), O.bf16_round(kc)
    max_lk = int(np.diff(cu_f).max())
    assert max_lk > 0
    dev = torch.device("cuda:0")
    tb = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16).to(dev)
    ti = lambda x: torch.from_numpy(np.asarray(x, np.int32)).to(dev)
    tq, tk = tb(q), tb(k)
    gkf, gcu_f = ops.compress_keys(tk, ti(cu), max(seqs), 32, 16)
    gkc, gcu_c = ops.compress_keys(tk, ti(cu), max(seqs), 128, 64)
    assert np.array_equal(gcu_f.cpu().numpy(), cu_f) and np.array_equal(gcu_c.cpu().numpy(), cu_c)
    assert np.array_equal(bf16_np(gkf[:int(cu_f[-1])]), kf) and np.array_equal(bf16_np(gkc[:int(cu_c[-1])]), kc)
    args = (tq, gkf, gkc, ti(cu), gcu_f, gcu_c, max(seqs), max_lk)
    score = ops.infllmv2_attn_stage1(*args, causal=True)
    ref = O.stage1_scores(q, kf, kc, cu, cu_f, cu_c, max_lk, 128 ** -0.5, True, round_output=False).astype(np.float64)
    assert np.all(np.abs(bf16_np(score) - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3)
    cache_lens = ti(cache)
    pooled = ops.max_pooling_1d_varlen(score, ti(cu), gcu_f, cache_lens, max(seqs), max_lk, local, init)
    ref_pooled = O.max_pooling_1d_varlen(bf16_np(score), cu, cu_f, np.asarray(cache), max(seqs), max_lk, local, init)
    assert pooled.shape == ref_pooled.shape and np.array_equal(bf16_np(pooled), ref_pooled)
    fused = ops.infllmv2_attn_stage1_pooled(*args, local, init, cache_lens=cache_lens, causal=True)
    assert torch.equal(fused.view(torch.int16), pooled.view(torch.int16))
    idx = ops.topk_blocks(pooled, topk)
    assert np.array_equal(idx.cpu().numpy(), O.topk_blocks(ref_pooled, topk))
    max_k_tokens = max(s + c for s, c in zip(seqs, cache))
    words, kb = ops.topk_to_uint64(idx, max_k_tokens, 64)
    ref_words, ref_kb = O.topk_to_uint64(idx.cpu().numpy(), max_k_tokens, 64)
    assert kb == ref_kb and np.array_equal(words.cpu().numpy().view(np.uint64), ref_words)
    if not use_cache:
        chosen = ops.select_blocks(tq, tk, ti(cu), ti(cu), max(seqs), max(seqs), topk, local, init, cache_lens=cache_lens,
                                   max_cache_len=0)
        assert torch.equal(chosen, idx)


@pytest.mark.parametrize("seed", list(range(400, 412)))
def test_random_case_decode_options(seed):
    """Random combinations of the decode options (where the sequences lie: plain, cache_batch_idx or paged; left
    padding; 0-3 appended tokens with or without rotary embedding, both pairings; forced split counts; 1-3 KV heads)
    against the extended decode oracle, caches included."""
    import infllmv2_cuda_impl_amd as ops
    import test_gpu_decode as D
    r = np.random.default_rng(seed)
    B, Hk = int(r.integers(1, 6)), int(r.integers(1, 4))
    page = int(r.choice([64, 128, 256]))
    cap = page * int(r.integers(2, 1 + 2048 // page))
    new = int(r.integers(0, 4))
    layout = ["plain", "batch_idx", "paged"][seed % 3]
    leftpad = layout != "paged" and bool(r.integers(0, 2))
    pad = [int(r.integers(0, cap // 4)) for _ in range(B)] if leftpad else [0] * B
    lens = [int(r.integers(1, cap - new - pad[b] + 1)) for b in range(B)]
    k_sel = int(r.integers(1, 10))
    q, kc, vc, kn, vn, L, idx = D.make(seed, B, cap, lens, k_sel, Hk=Hk, new=new)
    opts = {}
    g = torch.Generator(device="cpu").manual_seed(seed + 1)
    if leftpad:
        opts["cache_leftpad"] = torch.tensor(pad, dtype=torch.int32)
        L = L + opts["cache_leftpad"]
    if new and bool(r.integers(0, 2)):
        half = int(r.choice([16, 32, 64]))
        opts["rotary_cos"], opts["rotary_sin"] = D.rotary_tables(seed + 2, cap, half)
        opts["rotary_interleaved"] = bool(r.integers(0, 2))
    if layout == "batch_idx":
        rows = B + int(r.integers(0, 3))
        where = torch.randperm(rows, generator=g)[:B].to(torch.int32)
        big_k = torch.randn(rows, cap, Hk, 128, generator=g).to(torch.bfloat16)
        big_v = torch.randn(rows, cap, Hk, 128, generator=g).to(torch.bfloat16)
        big_k[where.long()], big_v[where.long()] = kc, vc
        kc, vc = big_k, big_v
        opts["cache_batch_idx"] = where
    elif layout == "paged":
        per_seq = cap // page
        n_pages = B * per_seq + 3
        table = torch.randperm(n_pages, generator=g)[:B * per_seq].view(B, per_seq).to(torch.int32)
        pk = torch.randn(n_pages, page, Hk, 128, generator=g).to(torch.bfloat16)
        pv = torch.randn(n_pages, page, Hk, 128, generator=g).to(torch.bfloat16)
        pk[table.view(-1).long()] = kc.view(B * per_seq, page, Hk, 128)
        pv[table.view(-1).long()] = vc.view(B * per_seq, page, Hk, 128)
        kc, vc = pk, pv
        opts["block_table"] = table
    num_splits = int(r.choice([0, 0, 1, 2, 5]))
    print(f"seed {seed}: B {B} Hk {Hk} cap {cap} page {page} new {new} layout {layout} pad {pad} lens {lens} "
          f"k {k_sel} splits {num_splits} rotary {'rotary_cos' in opts}", flush=True)
    D.check_ext(ops, q, kc, vc, L, idx, cap, new=(kn, vn) if new else None, num_splits=num_splits, **opts)


def test_empty_sequence_inside_a_packed_batch():
    """cu_seqlens with a zero-length sequence in the middle and at the end: every kernel skips it."""
    import infllmv2_cuda_impl_amd as ops
    r = np.random.default_rng(77)
    seqs = [150, 0, 200, 0]
    Hk, k_sel, T = 2, 3, 350
    cu = np.cumsum([0] + seqs).astype(np.int32)
    mk = lambda *shape: O.bf16_round(r.standard_normal(shape).astype(np.float32))
    q, k, v, dout = mk(T, 32, 128), mk(T, Hk, 128), mk(T, Hk, 128), mk(T, 32, 128)
    idx = np.full((Hk, T, k_sel), -1, np.int32)
    for b, s in enumerate(seqs):
        for i in range(s):
            nb = (s + 63) // 64
            for h in range(Hk):
                idx[h, cu[b] + i, :min(k_sel, nb)] = np.sort(r.permutation(nb)[:k_sel])
    dev = torch.device("cuda:0")
    t = lambda x: torch.from_numpy(x).to(torch.bfloat16).to(dev)
    tcu = torch.from_numpy(cu).to(dev)
    qg, kg, vg = [t(x).requires_grad_(True) for x in (q, k, v)]
    out, lse, _ = ops.infllmv2_attn_varlen_func(qg, kg, vg, tcu, tcu, max(seqs), max(seqs), causal=True,
                                                topk_idx=torch.from_numpy(idx).to(dev), return_attn_probs=True)
    out.backward(t(dout))
    words, _ = O.topk_to_uint64(idx, max(seqs), 64)
    ref_o, ref_lse = O.stage2_forward(q, k, v, cu, cu, words, 128 ** -0.5, True)
    assert np.abs(bf16_np(out) - ref_o).max() <= 2e-2
    dq, dk, dv = O.stage2_backward(q, k, v, dout, cu, cu, words, 128 ** -0.5, True)
    for got, ref in ((qg.grad, dq), (kg.grad, dk), (vg.grad, dv)):
        s = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got).astype(np.float64) - ref)
        assert e.max() <= 2e-2 * s and e.mean() <= 1e-3 * s
    # selection front end on the same batch
    tk = t(k)
    kf, cu_f = ops.compress_keys(tk, tcu, max(seqs), 32, 16)
    kc, cu_c = ops.compress_keys(tk, tcu, max(seqs), 128, 64)
    rkf, rcu_f = O.compress_keys(k, cu, 32, 16)
    rkc, rcu_c = O.compress_keys(k, cu, 128, 64)
    assert np.array_equal(cu_f.cpu().numpy(), rcu_f) and np.array_equal(cu_c.cpu().numpy(), rcu_c)
    max_lk = int(np.diff(rcu_f).max())
    score = ops.infllmv2_attn_stage1(t(q), kf, kc, tcu, cu_f, cu_c, max(seqs), max_lk, causal=True)
    ref = O.stage1_scores(q, O.bf16_round(rkf), O.bf16_round(rkc), cu, rcu_f, rcu_c, max_lk, 128 ** -0.5, True,
                          round_output=False).astype(np.float64)
    assert np.all(np.abs(bf16_np(score) - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3)
    cache_lens = torch.zeros(len(seqs), dtype=torch.int32, device=dev)
    pooled = ops.max_pooling_1d_varlen(score, tcu, cu_f, cache_lens, max(seqs), max_lk, 1, 1)
    fused = ops.infllmv2_attn_stage1_pooled(t(q), kf, kc, tcu, cu_f, cu_c, max(seqs), max_lk, 1, 1, cache_lens=cache_lens,
                                            causal=True)
    assert torch.equal(fused.view(torch.int16), pooled.view(torch.int16))
    assert np.array_equal(bf16_np(pooled), O.max_pooling_1d_varlen(bf16_np(score), cu, rcu_f, np.zeros(4, np.int32),
                                                                   max(seqs), max_lk, 1, 1))


def test_operators_follow_the_current_stream():
    """Everything is launched on torch's current stream (flash_api.cpp:764; topk_to_uint64.py:54-55): the same calls
    on a side stream (default priority) give the same bits, forward and backward."""
    import infllmv2_cuda_impl_amd as ops
    from test_gpu_stage2_fwd import make_case
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(55, [700, 300], [700, 300], 2, 5, dev)
    dout = torch.randn(q.shape, generator=torch.Generator(device="cpu").manual_seed(56)).to(torch.bfloat16).to(dev)

    def run():
        qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
        out = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu_q, cu_k, 700, 700, causal=True, topk_idx=idx, deterministic=True)
        out.backward(dout)
        sel = ops.select_blocks(q, k, cu_q, cu_k, 700, 700, 4, 1, 1,
                                cache_lens=torch.zeros(2, dtype=torch.int32, device=dev), max_cache_len=0)
        return out.detach(), qg.grad, kg.grad, vg.grad, sel
    ref = run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        got = run()
    side.synchronize()
    for a, b in zip(ref, got):
        assert torch.equal(a, b)


def test_forward_and_decode_replay_from_a_hip_graph():
    """The library launches kernels only (no allocation, memset, copy or synchronisation of its own), so a forward
    step and a decode step can be captured in a HIP graph.  Replayed three times, with eager work and
    synchronisations in between and new input values each time, every replay equals the eager result."""
    import infllmv2_cuda_impl_amd as ops
    from test_gpu_stage2_fwd import make_case
    import test_gpu_decode as D
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(61, [600, 424], [600, 424], 2, 5, dev)
    dq_, dkc, dvc, _, _, L, didx = D.make(62, 3, 512, [200, 333, 448], 4)
    dq_, dkc, dvc, L, didx = [t.to(dev) for t in (dq_, dkc, dvc, L, didx)]

    def step():
        sel = ops.select_blocks(q, k, cu_q, cu_k, 600, 600, 5, 1, 1,
                                cache_lens=torch.zeros(2, dtype=torch.int32, device=dev), max_cache_len=0)
        out = ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, 600, 600, causal=True, topk_idx=sel)
        dec = ops.infllmv2_attn_with_kvcache(dq_, dkc, dvc, cache_seqlens=L, topk_idx=didx)
        return sel, out, dec
    step()                                                     # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = step()
    torch.cuda.synchronize()
    gen = torch.Generator(device="cpu").manual_seed(63)
    for _ in range(3):
        q.copy_(torch.randn(q.shape, generator=gen).to(torch.bfloat16))       # new values in the captured tensors
        dq_.copy_(torch.randn(dq_.shape, generator=gen).to(torch.bfloat16))
        eager = step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, captured):
            assert torch.equal(a, b)


def test_kv_heads_can_be_computed_separately():
    """Sharding by KV head (the reference's tests/test_tp.py:25-33 reassembles such shards): each KV head with its 16
    query heads, given as strided slices of the full tensors, yields exactly the slice of the full result, forward
    and backward (deterministic mode, so that dK/dV compare bit for bit)."""
    import infllmv2_cuda_impl_amd as ops
    from test_gpu_stage2_fwd import make_case
    dev = torch.device("cuda:0")
    q, k, v, cu_q, cu_k, idx = make_case(71, [500, 260], [500, 260], 2, 4, dev)
    dout = torch.randn(q.shape, generator=torch.Generator(device="cpu").manual_seed(72)).to(torch.bfloat16).to(dev)

    def run(qs, ks, vs, ds, sel):
        qg, kg, vg = [t.clone().requires_grad_(True) for t in (qs, ks, vs)]     # clones keep the slices' strides
        out = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu_q, cu_k, 500, 500, causal=True, topk_idx=sel, deterministic=True)
        out.backward(ds)
        return out.detach(), qg.grad, kg.grad, vg.grad
    full = run(q, k, v, dout, idx)
    for h in range(2):
        hs = slice(16 * h, 16 * h + 16)
        part = run(q[:, hs], k[:, h:h + 1], v[:, h:h + 1], dout[:, hs], idx[h:h + 1].contiguous())
        assert torch.equal(part[0], full[0][:, hs]) and torch.equal(part[1], full[1][:, hs])
        assert torch.equal(part[2], full[2][:, h:h + 1]) and torch.equal(part[3], full[3][:, h:h + 1])


def test_query_chunk_against_the_full_prefix_equals_rows_of_the_full_run():
    """Sharding by query range (the reference's tests/test_stage1_cp_load.py scores a chunk of queries against the
    whole key history): the last 256 tokens of a 1024-token sequence as queries, all 1024 tokens as keys, give the
    same Stage-1 scores and the same attention output as those rows of the full computation (bit for bit: the chunk
    starts on a workgroup boundary, so every reduction runs in the same order)."""
    import infllmv2_cuda_impl_amd as ops
    from test_gpu_stage2_fwd import make_case
    dev = torch.device("cuda:0")
    S, C = 1024, 256
    q, k, v, cu, _, idx = make_case(81, [S], [S], 2, 6, dev)
    one = lambda n: torch.tensor([0, n], dtype=torch.int32, device=dev)
    kf, cu_f = ops.compress_keys(k, cu, S, 32, 16)
    kc, cu_c = ops.compress_keys(k, cu, S, 128, 64)
    lf = int(cu_f[-1])
    full_score = ops.infllmv2_attn_stage1(q, kf, kc, cu, cu_f, cu_c, S, lf, causal=True)
    part_score = ops.infllmv2_attn_stage1(q[S - C:], kf, kc, one(C), cu_f, cu_c, C, lf, causal=True)
    assert torch.equal(part_score.view(torch.int16), full_score[:, S - C:].contiguous().view(torch.int16))
    full_pool = ops.max_pooling_1d(full_score, 0, 1, 1)
    part_pool = ops.max_pooling_1d(part_score, S - C, 1, 1)     # cache_len = tokens before the chunk
    assert torch.equal(part_pool.view(torch.int16), full_pool[:, S - C:].contiguous().view(torch.int16))
    full_out = ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, S, S, causal=True, topk_idx=idx)
    part_out = ops.infllmv2_attn_varlen_func(q[S - C:], k, v, one(C), cu, C, S, causal=True,
                                             topk_idx=idx[:, S - C:].contiguous())
    assert torch.equal(part_out, full_out[S - C:])
