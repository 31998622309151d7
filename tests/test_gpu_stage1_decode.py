"""GPU parity of Stage 1 with one query per sequence (the selection half of a batched decode step).

Scores against the CPU oracle to the Stage-1 tolerance (|got - ref| <= 2^-7 |ref| + 2e-3); the pooled output bit for
bit against pooling the same launch's score rows (max_pooling_1d_varlen on the GPU and the oracle's pooling on the CPU:
one differing bit could change a selection); packed keys and per-sequence key caches give the same bits; the
batched decode step of the layer reproduces the single-sequence decode loop.  The reference covers this case with
its varlen Stage 1 on cu_seqlens_q = 0, 1, 2, ... and tests/test_cache_lens.py:4-98 (per-sequence cache_lens)."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def to_dev(a, dt=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t if dt is None else t.to(dt)).to(DEV)


def same_bits(a, b):
    return torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16))


def close(got, ref):
    err = np.abs(got - ref)
    tol = 2.0 ** -7 * np.abs(ref) + 2e-3
    assert (err <= tol).all(), (err.max(), np.unravel_index(np.argmax(err - tol), err.shape))


def batch_inputs(seed, lens, Hk=2, exact=False):
    """One query per sequence; the sequences' keys packed; compressed keys by the oracle."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    B = len(lens)
    q = torch.randn(B, 16 * Hk, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(sum(lens), Hk, 128, generator=g).to(torch.bfloat16)
    cu = np.cumsum([0] + list(lens)).astype(np.int32)
    kf, cu_f = O.compress_keys(bf16_np(k), cu, 32, 16)
    kc, cu_c = (kf, cu_f) if exact else O.compress_keys(bf16_np(k), cu, 128, 64)
    return q, k, cu, kf, cu_f, kc, cu_c


@pytest.mark.parametrize("lens,causal,exact", [
    ([1000, 40, 3000, 128, 129, 31, 2047], False, False),     # no fine key, no coarse key, one coarse key, ...
    ([1000, 40, 3000, 128, 129, 31, 2047], True, False),      # causal rule of a 1-token query: the last key of each set hidden
    ([20000], False, False),                                   # one sequence: many runs per (sequence, head)
    ([5000, 700], False, True),                                # exact softmax: the log-sum-exp over the fine keys themselves
    ([64 * 17 + 5] * 40, False, False),                       # more (sequence, head) pairs than runs wanted: short runs
    ([140000, 300], False, False),                            # over 128 fine tiles: runs of three tiles
    ([140000], True, True),                                    # ... and, the log-sum-exp over the same keys, coarse runs of three
])
def test_scores_pooled_and_layouts(ops, lens, causal, exact):
    q, k, cu, kf, cu_f, kc, cu_c = batch_inputs(1, lens, exact=exact)
    B = len(lens)
    Lk = int(np.diff(cu_f).max())
    cu_q = np.arange(B + 1, dtype=np.int32)
    qd, kfd, kcd = q.to(DEV), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16)
    args = (qd, kfd, kcd, to_dev(cu_q), to_dev(cu_f), to_dev(cu_c), 1, Lk)
    score = ops.infllmv2_attn_stage1(*args, causal=causal)
    assert tuple(score.shape) == (2, B, Lk) and score.dtype == torch.bfloat16
    ref = O.stage1_scores(bf16_np(q), kf, kc, cu_q, cu_f, cu_c, Lk, 128 ** -0.5, causal, round_output=False)
    close(bf16_np(score), ref)
    # pooled: the query of sequence b sits at position lens[b] - 1 (its cache holds the tokens before it)
    cache_lens = np.array([n - 1 for n in lens], dtype=np.int32)
    for local, init in ((1, 1), (31, 1), (0, 0)):
        fused = ops.infllmv2_attn_stage1_pooled(*args, local, init, cache_lens=to_dev(cache_lens), causal=causal)
        two_calls = ops.max_pooling_1d_varlen(score, to_dev(cu_q), to_dev(cu_f), to_dev(cache_lens), 1, Lk, local, init)
        assert tuple(fused.shape) == tuple(two_calls.shape) == (2, B, (max(lens) + 63) // 64)
        assert same_bits(fused, two_calls)
        want = O.max_pooling_1d_varlen(bf16_np(score), cu_q, cu_f, cache_lens, 1, Lk, local, init)
        assert np.array_equal(bf16_np(fused), want)
    # per-sequence compressed-key caches instead of packed keys: same bits
    rows_f = Lk + 3
    rows_c = int(np.diff(cu_c).max()) + 2
    fcache = torch.randn(B, rows_f, 2, 128).to(torch.bfloat16)          # stale rows beyond each sequence's keys
    ccache = torch.randn(B, rows_c, 2, 128).to(torch.bfloat16)
    for b in range(B):
        fcache[b, :cu_f[b + 1] - cu_f[b]] = torch.from_numpy(kf[cu_f[b]:cu_f[b + 1]]).to(torch.bfloat16)
        ccache[b, :cu_c[b + 1] - cu_c[b]] = torch.from_numpy(kc[cu_c[b]:cu_c[b + 1]]).to(torch.bfloat16)
    fl, cl = to_dev(np.diff(cu_f).astype(np.int32)), to_dev(np.diff(cu_c).astype(np.int32))
    if not exact:
        q4 = qd[:, None]
        sc2 = ops.infllmv2_attn_stage1_kvcache(q4, fcache.to(DEV), ccache.to(DEV), fl, cl, to_dev(cache_lens), 1, 1,
                                               causal=causal, pooled=False)
        assert same_bits(sc2[:, :, :Lk].transpose(0, 1), score)
        assert float(sc2[:, :, Lk:].abs().max()) == 0.0
        p2 = ops.infllmv2_attn_stage1_kvcache(q4, fcache.to(DEV), ccache.to(DEV), fl, cl, to_dev(cache_lens), 1, 1,
                                              max_cache_len=max(lens) - 1, causal=causal)
        fused = ops.infllmv2_attn_stage1_pooled(*args, 1, 1, cache_lens=to_dev(cache_lens), causal=causal)
        assert same_bits(p2.transpose(0, 1), fused)


def test_decode_kernel_agrees_with_the_prefill_shaped_kernel(ops):
    """The generic Stage-1 launch (C ABI infllmv2_varlen_fwd_stage1) on the same one-query sequences: different kernel,
    different summation order of the log-sum-exp, same scores to the Stage-1 tolerance."""
    from infllmv2_cuda_impl_amd import _lib
    lens = [3000, 500, 64 * 40]
    q, k, cu, kf, cu_f, kc, cu_c = batch_inputs(4, lens)
    B, Lk = len(lens), int(np.diff(cu_f).max())
    cu_q = to_dev(np.arange(B + 1, dtype=np.int32))
    qd, kfd, kcd, cfd, ccd = q.to(DEV), to_dev(kf, torch.bfloat16), to_dev(kc, torch.bfloat16), to_dev(cu_f), to_dev(cu_c)
    for causal in (False, True):
        fast = ops.infllmv2_attn_stage1(qd, kfd, kcd, cu_q, cfd, ccd, 1, Lk, causal=causal)
        slow = torch.empty_like(fast)
        _lib.call("infllmv2_varlen_fwd_stage1", torch.cuda.current_stream().cuda_stream, qd.data_ptr(), kfd.data_ptr(),
                  kcd.data_ptr(), slow.data_ptr(), cu_q.data_ptr(), cfd.data_ptr(), ccd.data_ptr(), B, B, 32, 2, 128, 1, Lk,
                  _lib.i64_array([qd.stride(0), qd.stride(1), 16 * qd.stride(1)]),
                  _lib.i64_array([kfd.stride(0), kfd.stride(1)]), _lib.i64_array([kcd.stride(0), kcd.stride(1)]),
                  slow.stride(0), slow.stride(1), 128 ** -0.5, int(causal))
        close(bf16_np(fast), bf16_np(slow).astype(np.float64))


def test_compressed_key_caches_follow_the_key_caches(ops):
    """compress_keys_cache == compress_keys of each sequence; a one-token step adds exactly the rows whose window the
    new token completes and touches nothing else."""
    lens = [100, 31, 32, 127, 128, 1000, 47]
    B, cap = len(lens), 1100
    g = torch.Generator(device="cpu").manual_seed(5)
    kcache = torch.randn(B, cap, 2, 128, generator=g).to(torch.bfloat16).to(DEV)
    L = torch.tensor(lens, dtype=torch.int32, device=DEV)
    for ks, st in ((32, 16), (128, 64)):
        out = torch.full((B, cap // st + 1, 2, 128), 7.0, dtype=torch.bfloat16, device=DEV)
        rows = ops.compress_keys_cache(kcache, L, ks, st, out=out)
        for b, n in enumerate(lens):
            one = torch.tensor([0, n], dtype=torch.int32, device=DEV)
            ref, _ = ops.compress_keys(kcache[b, :n], one, n, ks, st)
            r = ref.shape[0]
            assert int(rows[b]) == r == O.compressed_len(n, ks, st)
            assert torch.equal(out[b, :r], ref) and bool((out[b, r:] == 7.0).all())
        for step in range(1, 20):                              # one token at a time
            new = L + step
            rows2 = ops.compress_keys_cache(kcache, new, ks, st, out=out, old_lens=new - 1, max_new_rows=1)
            for b, n in enumerate(lens):
                r = O.compressed_len(n + step, ks, st)
                assert int(rows2[b]) == r
                if r:
                    ref, _ = ops.compress_keys(kcache[b, :n + step], torch.tensor([0, n + step], dtype=torch.int32, device=DEV),
                                               n + step, ks, st)
                    assert torch.equal(out[b, :r], ref)
                assert bool((out[b, r:] == 7.0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hk,d,ks,st,jump", [(8, 128, 32, 16, 40), (3, 64, 24, 8, 20), (2, 128, 128, 64, 200), (5, 128, 160, 32, 7)])
def test_append_of_a_few_rows_equals_the_full_build(ops, dtype, Hk, d, ks, st, jump):
    """The append path (at most 8 new rows per sequence, window staged in LDS; several workgroups per row when a row
    has more than 32 sixteen-byte units) and the general path (windows too large for it, or many new rows) write the
    same bits as a build from scratch, and nothing else."""
    lens = [0, 5, ks - 1, ks, 3 * ks + 1, 500]
    B, cap = len(lens), 800
    g = torch.Generator(device="cpu").manual_seed(17)
    kcache = torch.randn(B, cap, Hk, d, generator=g).to(dtype).to(DEV)
    old = torch.tensor(lens, dtype=torch.int32, device=DEV)
    new = old + jump
    rows_max = (cap - ks) // st + 1
    full = torch.full((B, rows_max, Hk, d), 7.0, dtype=dtype, device=DEV)
    rows_full = ops.compress_keys_cache(kcache, new, ks, st, out=full)
    inc = torch.full((B, rows_max, Hk, d), 7.0, dtype=dtype, device=DEV)
    ops.compress_keys_cache(kcache, old, ks, st, out=inc)
    max_new = max(O.compressed_len(n + jump, ks, st) - O.compressed_len(n, ks, st) for n in lens)
    rows_inc = ops.compress_keys_cache(kcache, new, ks, st, out=inc, old_lens=old, max_new_rows=max_new)
    assert torch.equal(rows_inc, rows_full)
    assert [int(r) for r in rows_full] == [O.compressed_len(n + jump, ks, st) for n in lens]
    assert torch.equal(inc, full)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_both_compressed_caches_in_one_call(ops, dtype):
    """compress_keys_cache_pair == two compress_keys_cache calls, bit for bit: the full build (two launches inside), a
    one-token step and a step of a few tokens (one launch for both caches), undersized second cache included."""
    lens = [0, 31, 32, 127, 128, 129, 1000, 47, 640]
    B, cap = len(lens), 1100
    g = torch.Generator(device="cpu").manual_seed(23)
    kcache = torch.randn(B, cap, 2, 128, generator=g).to(dtype).to(DEV)
    L = torch.tensor(lens, dtype=torch.int32, device=DEV)
    shapes = ((32, 16, cap // 16 + 1), (128, 64, 12))          # the coarse cache holds 12 rows only
    mk = lambda: [torch.full((B, r, 2, 128), 7.0, dtype=dtype, device=DEV) for _, _, r in shapes]
    one, two = mk(), mk()
    la, lb = ops.compress_keys_cache_pair(kcache, L, (32, 16, one[0]), (128, 64, one[1]), max_new_rows=cap)
    ra = ops.compress_keys_cache(kcache, L, 32, 16, out=two[0], max_new_rows=cap)
    rb = ops.compress_keys_cache(kcache, L, 128, 64, out=two[1], max_new_rows=cap)
    assert torch.equal(la, ra) and torch.equal(lb, rb) and torch.equal(one[0], two[0]) and torch.equal(one[1], two[1])
    for jump in (1, 1, 1, 40, 1, 100):
        new = L + jump
        la, lb = ops.compress_keys_cache_pair(kcache, new, (32, 16, one[0]), (128, 64, one[1]), old_lens=L, max_new_rows=7)
        ra = ops.compress_keys_cache(kcache, new, 32, 16, out=two[0], old_lens=L, max_new_rows=7)
        rb = ops.compress_keys_cache(kcache, new, 128, 64, out=two[1], old_lens=L, max_new_rows=7)
        assert torch.equal(la, ra) and torch.equal(lb, rb)
        assert torch.equal(one[0], two[0]) and torch.equal(one[1], two[1])
        L = new
    assert int(lb.max()) == 12 and int(la.max()) == O.compressed_len(cap, 32, 16)     # 1144 tokens read as the capacity


def test_compressed_cache_capacity_bounds_what_is_written(ops):
    """An undersized compressed cache, or a step that completes more windows than max_new_rows covers: nothing is
    written beyond the cache's rows, and out_lens counts only rows the call did write (the kernels get both
    capacities; the guard rows behind the view stay untouched)."""
    B, cap, ks, st = 3, 512, 32, 16
    g = torch.Generator(device="cpu").manual_seed(23)
    kcache = torch.randn(B, cap, 2, 128, generator=g).to(torch.bfloat16).to(DEV)
    backing = torch.full((B, 12, 2, 128), 7.0, dtype=torch.bfloat16, device=DEV)
    out = backing[:, :8]                                       # 8 rows of capacity, 4 guard rows behind each sequence
    new = torch.tensor([200, 400, 40], dtype=torch.int32, device=DEV)       # 11, 24 and 1 complete windows
    old = torch.tensor([128, 399, 0], dtype=torch.int32, device=DEV)        # 7, 23 and 0 rows held before
    rows = ops.compress_keys_cache(kcache, new, ks, st, out=out, old_lens=old, max_new_rows=1)
    assert [int(r) for r in rows] == [8, 8, 1]                 # 7 + 1; nothing fits (23 >= 8 rows): the capacity; 0 + 1
    assert bool((backing[:, 8:] == 7.0).all())
    ref0, _ = ops.compress_keys(kcache[0, :200], torch.tensor([0, 200], dtype=torch.int32, device=DEV), 200, ks, st)
    assert torch.equal(out[0, 7], ref0[7]) and bool((out[0, :7] == 7.0).all())
    assert bool((out[1] == 7.0).all())
    # a jump of several windows with max_new_rows = 2: two rows written, two reported
    rows = ops.compress_keys_cache(kcache, torch.tensor([200, 0, 0], dtype=torch.int32, device=DEV), ks, st, out=out,
                                   old_lens=torch.tensor([32, 0, 0], dtype=torch.int32, device=DEV), max_new_rows=2)
    assert [int(r) for r in rows] == [3, 0, 0]
    assert torch.equal(out[0, 1:3], ref0[1:3]) and bool((out[0, 3:7] == 7.0).all())
    # a length beyond the key cache is read as the capacity
    big = torch.full((B, 40, 2, 128), 7.0, dtype=torch.bfloat16, device=DEV)
    rows = ops.compress_keys_cache(kcache, torch.tensor([9999, 0, 0], dtype=torch.int32, device=DEV), ks, st, out=big)
    assert int(rows[0]) == (cap - ks) // st + 1
    with pytest.raises(RuntimeError, match="fewer rows"):
        ops.compress_keys_cache(kcache, new, ks, st, out=out)


def test_batched_decode_steps_equal_single_sequence_decode(ops):
    """decode_batch on sequences of different lengths == the single-sequence decode loop run on each of them: same
    caches afterwards (bit for bit), outputs to the Stage-2 tolerance (the two paths cut the compressed keys into
    different runs, so a score can differ in its last bit and tip a tie between two barely-selected blocks)."""
    lens, steps, cap = [1000, 300, 2047, 130], 20, 2200
    B = len(lens)
    g = torch.Generator(device="cpu").manual_seed(6)
    mk = lambda n, h: torch.randn(n, h, 128, generator=g).to(torch.bfloat16).to(DEV)
    total = [n + steps for n in lens]
    qs, ks, vs = [mk(n, 32) for n in total], [mk(n, 2) for n in total], [mk(n, 2) for n in total]
    layer = ops.InfLLMv2Attention(topk=8, local_blocks=2, init_blocks=1)
    singles = []
    for b in range(B):
        c = ops.SequenceCache.empty(cap, 2, 128, DEV)
        n = lens[b]
        layer(qs[b][:n], ks[b][:n], vs[b][:n], torch.tensor([0, n], dtype=torch.int32, device=DEV), n, cache=c)
        singles.append(c)
    cache = ops.BatchCache.empty(B, cap, 2, 128, DEV)
    layer.fill_cache(cache, torch.cat([ks[b][:lens[b]] for b in range(B)]), torch.cat([vs[b][:lens[b]] for b in range(B)]), lens)
    for b in range(B):
        assert torch.equal(cache.k_fine[b, :int(cache.fine_lens[b])], singles[b].k_fine[:int(cache.fine_lens[b])])
    for s in range(steps):
        q = torch.stack([qs[b][lens[b] + s] for b in range(B)])[:, None]
        kn = torch.stack([ks[b][lens[b] + s] for b in range(B)])[:, None]
        vn = torch.stack([vs[b][lens[b] + s] for b in range(B)])[:, None]
        out = layer.decode_batch(q, kn, vn, cache)
        assert tuple(out.shape) == (B, 1, 32, 128)
        for b in range(B):
            ref = layer.decode(q[b:b + 1], kn[b:b + 1], vn[b:b + 1], singles[b])
            err = (out[b].float() - ref[0].float()).abs()
            assert float(err.max()) <= 2e-2 and float(err.mean()) <= 1e-3, (s, b, float(err.max()))
    assert cache.max_length == max(lens) + steps
    assert cache.lengths.tolist() == total
    for b in range(B):
        n = total[b]
        assert torch.equal(cache.k[b, :n], singles[b].k[0, :n]) and torch.equal(cache.v[b, :n], singles[b].v[0, :n])
        rf, rc = O.compressed_len(n, 32, 16), O.compressed_len(n, 128, 64)
        assert int(cache.fine_lens[b]) == rf and int(cache.coarse_lens[b]) == rc
        assert torch.equal(cache.k_fine[b, :rf], singles[b].k_fine[:rf])
        assert torch.equal(cache.k_coarse[b, :rc], singles[b].k_coarse[:rc])
