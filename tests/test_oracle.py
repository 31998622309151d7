"""Pins the CPU oracle (oracle/infllmv2_oracle.py) by means other than its own formulas:
brute-force Python loops, library routines (torch softmax / max_pool1d / stable sort / autograd),
closed forms and invariants.  Case tables follow the reference's own tests
(tests/test_topk_to_uint64.py:259-281, tests/test_uint64_to_bool.py:113-121,
tests/test_blockmask.py:104-113, tests/test_stage1.py:223-231,
tests/test_stage1_compressed_lse.py:203-215, tests/test_cache_lens.py:10-37).  CPU only."""
import math

import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------------------------------------
# bit ops
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape,max_k,bs", [
    ((2, 128, 16), 256, 4), ((8, 64, 32), 1024, 16), ((4, 50, 64), 2048, 32),
    ((3, 40, 64), 8192, 16), ((2, 2, 16, 16), 256, 4)])
def test_topk_to_uint64_bruteforce(shape, max_k, bs):
    k_blocks = (max_k + bs - 1) // bs
    idx = rng(0).integers(-1, k_blocks, size=shape).astype(np.int32)
    words, kb = O.topk_to_uint64(idx, max_k, bs)
    assert kb == k_blocks and words.shape == shape[:-1] + ((k_blocks + 63) // 64,)
    flat = idx.reshape(-1, shape[-1])
    wf = words.reshape(flat.shape[0], -1)
    for r in range(flat.shape[0]):
        big = 0
        for v in flat[r]:
            if v != -1:
                big |= 1 << int(v)
        for w in range(wf.shape[1]):
            assert int(wf[r, w]) == (big >> (64 * w)) & (2 ** 64 - 1)
        assert sum(bin(int(x)).count("1") for x in wf[r]) == len({int(v) for v in flat[r] if v >= 0})


@pytest.mark.parametrize("shape,last", [((100, 1), 64), ((100, 1), 63), ((100, 2), 65), ((100, 2), 128),
                                        ((100, 4), 200), ((2, 3, 4, 2), 100), ((50, 16), 1000)])
def test_uint64_to_bool_bruteforce_and_roundtrip(shape, last):
    words = rng(1).integers(0, 2 ** 64, size=shape, dtype=np.uint64)
    b = O.uint64_to_bool(words, last)
    flat, bf = words.reshape(-1, shape[-1]), b.reshape(-1, last)
    for r in range(0, flat.shape[0], 7):
        for c in range(last):
            assert bool(bf[r, c]) == bool((int(flat[r, c // 64]) >> (c % 64)) & 1)
    back, l2 = O.blockmask_to_uint64(b)
    assert l2 == last
    keep = np.zeros(shape[-1] * 64, dtype=bool)
    keep[:last] = True
    keep_words = O.blockmask_to_uint64(keep)[0]
    assert np.array_equal(back, words & keep_words)           # tail bits zero, the rest identical
    assert np.array_equal(O.uint64_to_bool(back, last), b)


@pytest.mark.parametrize("shape", [(100, 64), (100, 63), (100, 65), (100, 128), (100, 200), (2, 3, 4, 100), (40, 1000)])
def test_blockmask_to_uint64_bruteforce(shape):
    m = rng(2).random(shape) < 0.5
    words, last = O.blockmask_to_uint64(m)
    assert last == shape[-1]
    mf, wf = m.reshape(-1, shape[-1]), words.reshape(-1, words.shape[-1])
    for r in range(0, mf.shape[0], 5):
        big = sum(1 << c for c in range(shape[-1]) if mf[r, c])
        for w in range(wf.shape[1]):
            assert int(wf[r, w]) == (big >> (64 * w)) & (2 ** 64 - 1)
    assert words.view(np.int64).min() < 0 or shape[-1] < 64   # bit 63 shows as a negative int64


def test_transpose_blockmask_definition():
    Hk, T, nblk = 2, 150, 70
    m = rng(3).random((Hk, T, nblk)) < 0.3
    fwd = O.blockmask_to_uint64(m)[0]
    bwd = O.transpose_blockmask(fwd, nblk)
    assert bwd.shape == (Hk, nblk, (T + 63) // 64)
    for h in range(Hk):
        for kb in range(nblk):
            for t in range(T):
                bit = (int(bwd[h, kb, t // 64]) >> (t % 64)) & 1
                assert bit == int(m[h, t, kb])
    # tail bits beyond T are zero
    assert all((int(bwd[h, kb, -1]) >> (T % 64)) == 0 for h in range(Hk) for kb in range(nblk))


# ---------------------------------------------------------------------------------------------
# max-pool
# ---------------------------------------------------------------------------------------------
def _pool_by_library(x, cache_len, local_blocks, init_blocks):
    """-inf padded kernel-5 / stride-4 / pad-1 library max-pool, then forced positions -> +inf."""
    H, q, kl = x.shape
    out_len = (q + cache_len + 63) // 64
    need = 4 * out_len + 3
    xp = torch.full((H, q, need), -math.inf)
    xp[:, :, :min(kl, need)] = torch.from_numpy(x)[:, :, :need]
    pooled = torch.nn.functional.max_pool1d(
        torch.nn.functional.pad(xp, (1, 0), value=-math.inf), kernel_size=5, stride=4)[:, :, :out_len]
    qi = torch.arange(q)[:, None]
    kb = torch.arange(out_len)[None, :]
    bq = (qi + cache_len) // 64
    forced = (kb < init_blocks) | ((bq >= kb) & (bq <= kb + local_blocks))
    return torch.where(forced[None], torch.tensor(math.inf), pooled).numpy()


@pytest.mark.parametrize("q,kl,cache,local,init", [(70, 127, 0, 1, 1), (130, 30, 0, 2, 1), (33, 17, 64, 4, 1),
                                                   (200, 51, 128, 0, 0), (5, 3, 0, 1, 2), (64, 0, 0, 1, 1)])
def test_max_pool_vs_library_and_fast(q, kl, cache, local, init):
    x = O.bf16_round(rng(4).standard_normal((2, q, kl)).astype(np.float32))
    a = O.max_pooling_1d(x, cache, local, init)
    assert a.shape == (2, q, (q + cache + 63) // 64)
    if kl > 0:
        assert np.array_equal(a, _pool_by_library(x, cache, local, init))
    assert np.array_equal(a, O.max_pooling_1d_fast(x, cache, local, init))
    # forced-block count: local_blocks = L forces L + 1 blocks (diagonal + L previous) where they exist
    bq = (np.arange(q) + cache) // 64
    n_forced = (a == np.inf).sum(axis=2)[0]
    out_len = a.shape[2]
    expect = [len(set(range(min(init, out_len))) | {kb for kb in range(out_len) if kb <= b <= kb + local}) for b in bq]
    assert list(n_forced) == expect


def test_max_pool_empty_window_is_neg_inf():
    x = np.ones((1, 300, 5), dtype=np.float32)          # only 5 compressed keys but 5 output blocks
    a = O.max_pooling_1d(x, 0, 0, 0)
    assert a.shape[2] == 5
    assert a[0, 0, 1] == 1.0 and a[0, 0, 2] == -np.inf and a[0, 299, 3] == -np.inf


def test_max_pool_varlen_equals_per_sequence():
    # tests/test_cache_lens.py:10-37 shapes
    sq, sk, cl = [10, 15, 8], [20, 25, 16], [0, 64, 128]
    cu_q, cu_k = np.cumsum([0] + sq), np.cumsum([0] + sk)
    x = O.bf16_round(rng(5).standard_normal((2, sum(sq), max(sk))).astype(np.float32))
    out = O.max_pooling_1d_varlen(x, cu_q, cu_k, cl, max(sq), max(sk), 4, 1)
    assert out.shape[2] == (max(sq) + max(cl) + 63) // 64
    for b in range(3):
        ref = O.max_pooling_1d(x[:, cu_q[b]:cu_q[b + 1], :sk[b]], cl[b], 4, 1)
        w = ref.shape[2]
        got = out[:, cu_q[b]:cu_q[b + 1]]
        assert np.array_equal(got[:, :, :w], ref)
        # columns past this sequence's own out_len: window empty or beyond -> follow the same rule
        full = O.max_pooling_1d(np.pad(x[:, cu_q[b]:cu_q[b + 1], :sk[b]], ((0, 0), (0, 0), (0, 0))), cl[b], 4, 1)
        assert np.array_equal(got[:, :, :full.shape[2]], full)


# ---------------------------------------------------------------------------------------------
# top-k
# ---------------------------------------------------------------------------------------------
def test_topk_is_stable_descending_sort_prefix():
    x = O.bf16_round(rng(6).standard_normal((3, 40, 100)).astype(np.float32))
    x[:, :, :3] = np.inf                 # forced blocks
    x[:, :, 50:60] = 0.0                 # exact ties
    x[:, :, 90:] = -np.inf
    got = O.topk_blocks(x, 16)
    ref = torch.sort(torch.from_numpy(x), dim=-1, descending=True, stable=True).indices[..., :16].numpy()
    assert np.array_equal(got, ref)
    assert (got[..., :3] == np.arange(3)).all()          # +inf first, by ascending index
    short = O.topk_blocks(x[..., :5], 8)
    assert (short[..., 5:] == -1).all() and sorted(short[0, 0, :5]) == [0, 1, 2, 3, 4]


# ---------------------------------------------------------------------------------------------
# stage 1
# ---------------------------------------------------------------------------------------------
def test_stage1_visibility_from_first_principles():
    """Sq == Sk: fine key j covers tokens [16j, 16j+32) and is visible iff 16j+31 <= i; coarse key j
    covers [64j, 64j+128) and is visible iff 64j+127 <= i."""
    for S in (64, 256, 1000, 2048):
        Lk, Lc = O.compressed_len(S, 32, 16), O.compressed_len(S, 128, 64)
        for i in range(S):
            assert O.stage1_visible(i, 16, Lk, S, True) == sum(1 for j in range(Lk) if 16 * j + 31 <= i)
            assert O.stage1_visible(i, 64, Lc, S, True) == sum(1 for j in range(Lc) if 64 * j + 127 <= i)
    assert O.stage1_visible(5, 16, 7, 100, False) == 7


def test_stage1_visibility_shorter_query():
    """q_len < k_len (context-parallel / decode): the last token sees all L keys, each earlier group of
    16 tokens one fewer (tests/stage1/naive_softmax.py:22-33 with floor division)."""
    Sq, L = 256, 40
    for i in range(Sq):
        expect = min(L, max(0, ((i - 15) // 16) + L - (Sq - 15) // 16))
        assert O.stage1_visible(i, 16, L, Sq, True) == expect
    assert O.stage1_visible(Sq - 1, 16, L, Sq, True) == L


def _torch_exact_stage1(q, k, causal):
    """Textbook statement: softmax over visible compressed keys, summed over the 16 group heads."""
    T, Hq, d = q.shape
    L, Hk = k.shape[0], k.shape[1]
    qt = torch.from_numpy(q).double().transpose(0, 1)
    kt = torch.from_numpy(k).double().transpose(0, 1).repeat_interleave(16, dim=0)
    s = qt @ kt.transpose(-1, -2) / math.sqrt(d)
    if causal:
        vis = torch.tensor([sum(1 for j in range(L) if 16 * j + 31 <= i) for i in range(T)])
        s = s.masked_fill(torch.arange(L)[None, :] >= vis[:, None], -math.inf)
    p = torch.softmax(s, dim=-1)
    p = torch.where(torch.isnan(p), torch.zeros_like(p), p)
    return p.reshape(Hk, 16, T, L).sum(1).numpy()


@pytest.mark.parametrize("S,causal", [(64, True), (256, True), (256, False), (500, True)])
def test_stage1_exact_mode_is_textbook_softmax(S, causal):
    r = rng(7)
    q = O.bf16_round(r.standard_normal((S, 32, 128)).astype(np.float32))
    kfull = O.bf16_round(r.standard_normal((S, 2, 128)).astype(np.float32))
    kc, cu_c = O.compress_keys(kfull, [0, S], 32, 16)
    L = kc.shape[0]
    got = O.stage1_scores(q, kc, kc, [0, S], cu_c, cu_c, L, 128 ** -0.5, causal, round_output=False)
    ref = _torch_exact_stage1(q, kc, causal)
    assert np.abs(got - ref).max() < 1e-5
    sums = got.sum(-1)
    vis = np.array([O.stage1_visible(i, 16, L, S, causal) for i in range(S)])
    assert np.allclose(sums[:, vis > 0], 16.0, atol=1e-4) and np.all(sums[:, vis == 0] == 0)


def test_stage1_non_causal_shapes_of_reference_tests():
    # tests/test_stage1.py:223-231: q in {64, 256}, k in {15, 16, 17} compressed keys, non-causal
    r = rng(8)
    for Sq in (64, 256):
        for L in (15, 16, 17):
            q = O.bf16_round(r.standard_normal((Sq, 32, 128)).astype(np.float32))
            k = O.bf16_round(r.standard_normal((L, 2, 128)).astype(np.float32))
            got = O.stage1_scores(q, k, k, [0, Sq], [0, L], [0, L], L, 128 ** -0.5, False, round_output=False)
            assert np.abs(got - _torch_exact_stage1(q, k, False)).max() < 1e-5


def test_stage1_compressed_lse_closed_form():
    """score[h,i,j] = sum_g exp(s_gj - logsumexp_{c < vis_c(i)} s^c_g); rows with no visible coarse key = 0;
    rows are not normalised."""
    S = 300
    r = rng(9)
    q = O.bf16_round(r.standard_normal((S, 32, 128)).astype(np.float32))
    kfull = O.bf16_round(r.standard_normal((S, 2, 128)).astype(np.float32))
    kf, cu_f = O.compress_keys(kfull, [0, S], 32, 16)
    kc, cu_c = O.compress_keys(kfull, [0, S], 128, 64)
    Lk, Lc = kf.shape[0], kc.shape[0]
    assert (Lk, Lc) == ((S - 32) // 16 + 1, (S - 128) // 64 + 1)
    scale = 128 ** -0.5
    got = O.stage1_scores(q, kf, kc, [0, S], cu_f, cu_c, Lk, scale, True, round_output=False)
    for i in (0, 31, 126, 127, 128, 191, 192, 255, 299):
        for h in (0, 1):
            vf = sum(1 for j in range(Lk) if 16 * j + 31 <= i)
            vc = sum(1 for j in range(Lc) if 64 * j + 127 <= i)
            row = np.zeros(Lk)
            if vc > 0:
                for g in range(16):
                    qv = q[i, 16 * h + g].astype(np.float64)
                    lse = math.log(sum(math.exp(scale * float(qv @ kc[c, h])) for c in range(vc)))
                    for j in range(vf):
                        row[j] += math.exp(scale * float(qv @ kf[j, h]) - lse)
            assert np.abs(got[h, i] - row).max() < 1e-4 * max(1.0, row.max())
    assert got[:, :127].max() == 0.0 and got[:, 127:].max() > 0.0


def test_compress_keys_is_windowed_mean():
    k = rng(10).standard_normal((100, 2, 8)).astype(np.float32)
    kc, cu = O.compress_keys(k, [0, 40, 100], 32, 16)
    assert list(cu) == [0, 1, 1 + (60 - 32) // 16 + 1]
    assert np.allclose(kc[0], O.bf16_round(k[0:32].mean(0)))
    assert np.allclose(kc[2], O.bf16_round(k[40 + 16:40 + 48].mean(0)))


# ---------------------------------------------------------------------------------------------
# stage 2
# ---------------------------------------------------------------------------------------------
def _torch_stage2(q, k, v, cu_q, cu_k, bits, scale, causal, dout=None):
    """Dense masked softmax with library softmax + autograd (fp64)."""
    qt = torch.from_numpy(q).double().requires_grad_(True)
    kt = torch.from_numpy(k).double().requires_grad_(True)
    vt = torch.from_numpy(v).double().requires_grad_(True)
    outs = []
    Hk = k.shape[1]
    for b in range(len(cu_q) - 1):
        q0, q1, k0, k1 = cu_q[b], cu_q[b + 1], cu_k[b], cu_k[b + 1]
        Sq, Sk = q1 - q0, k1 - k0
        allow = torch.ones(Hk, Sq, Sk, dtype=torch.bool)
        if causal:
            allow &= (torch.arange(Sk)[None, :] <= torch.arange(Sq)[:, None] + Sk - Sq)[None]
        if bits is not None:
            nb = (Sk + 63) // 64
            bb = torch.from_numpy(bits[:, q0:q1, :nb])
            allow &= bb.repeat_interleave(64, dim=2)[:, :, :Sk]
        allow = allow.repeat_interleave(16, dim=0)
        s = torch.einsum("thd,shd->hts", qt[q0:q1], kt[k0:k1].repeat_interleave(16, dim=1)) * scale
        s = s.masked_fill(~allow, -math.inf)
        p = torch.softmax(s, dim=-1)
        p = torch.where(allow.any(-1, keepdim=True), p, torch.zeros_like(p))
        outs.append(torch.einsum("hts,shd->thd", p, vt[k0:k1].repeat_interleave(16, dim=1)))
    out = torch.cat(outs, 0)
    if dout is None:
        return out.detach().numpy()
    out.backward(torch.from_numpy(dout).double())
    return out.detach().numpy(), qt.grad.numpy(), kt.grad.numpy(), vt.grad.numpy()


def _random_case(seed, sq, sk, k_sel, causal):
    r = rng(seed)
    cu_q, cu_k = np.cumsum([0] + sq), np.cumsum([0] + sk)
    T, Tk = cu_q[-1], cu_k[-1]
    q = O.bf16_round(r.standard_normal((T, 32, 128)).astype(np.float32))
    k = O.bf16_round(r.standard_normal((Tk, 2, 128)).astype(np.float32))
    v = O.bf16_round(r.standard_normal((Tk, 2, 128)).astype(np.float32))
    nblk = (max(sk) + 63) // 64
    idx = np.full((2, T, k_sel), -1, dtype=np.int32)
    for h in range(2):
        for b in range(len(sq)):
            nb = (sk[b] + 63) // 64
            for t in range(cu_q[b], cu_q[b + 1]):
                sel = r.permutation(nb)[:k_sel]
                idx[h, t, :len(sel)] = np.sort(sel)
    words, kb = O.topk_to_uint64(idx, max(sk), 64)
    bits = O.uint64_to_bool(words, nblk)
    return q, k, v, cu_q, cu_k, words, bits


@pytest.mark.parametrize("sq,sk,k_sel,causal", [([128], [128], 1, True), ([100, 37], [100, 37], 2, True),
                                                ([70], [200], 2, True), ([64], [130], 3, False),
                                                ([200], [70], 1, True)])
def test_stage2_forward_and_backward_vs_library(sq, sk, k_sel, causal):
    q, k, v, cu_q, cu_k, words, bits = _random_case(11, sq, sk, k_sel, causal)
    scale = 128 ** -0.5
    dout = rng(12).standard_normal(q.shape).astype(np.float32)
    ref_o, ref_dq, ref_dk, ref_dv = _torch_stage2(q, k, v, cu_q, cu_k, bits, scale, causal, dout)
    out, lse = O.stage2_forward(q, k, v, cu_q, cu_k, words, scale, causal)
    assert np.abs(out - ref_o).max() < 1e-9
    dq, dk, dv = O.stage2_backward(q, k, v, dout, cu_q, cu_k, words, scale, causal)
    assert np.abs(dq - ref_dq).max() < 1e-9 and np.abs(dk - ref_dk).max() < 1e-9 and np.abs(dv - ref_dv).max() < 1e-9
    # rows with no allowed key: zero output, +inf LSE, in the expanded (Hk, T*16) layout
    dead = ~_dead_rows_alive(bits, cu_q, cu_k, causal)
    assert lse.shape == (2, q.shape[0] * 16)
    for h in range(2):
        for t in np.nonzero(dead[h])[0]:
            assert np.all(out[t, 16 * h:16 * h + 16] == 0) and np.all(np.isinf(lse[h, t * 16:(t + 1) * 16]))


def _dead_rows_alive(bits, cu_q, cu_k, causal):
    alive = np.zeros(bits.shape[:2], dtype=bool)
    for b in range(len(cu_q) - 1):
        Sq, Sk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
        for i in range(Sq):
            last = min(Sk - 1, i + Sk - Sq) if causal else Sk - 1
            if last >= 0:
                alive[:, cu_q[b] + i] = bits[:, cu_q[b] + i, :last // 64 + 1].any(-1)
    return alive


@pytest.mark.parametrize("S,k_sel", [(300, 2), (200, 4), (130, 1)])
def test_key_block_backward_is_a_slice_of_the_library_gradients(S, k_sel):
    """stage2_backward_key_block (token-by-token, only the tokens that select the block) against autograd of the
    masked-softmax attention in fp64: every key block and KV head, including blocks no token selects and the ragged
    last block."""
    q, k, v, cu_q, cu_k, words, bits = _random_case(21, [S], [S], k_sel, True)
    scale = 128 ** -0.5
    dout = rng(22).standard_normal(q.shape).astype(np.float32)
    _, _, ref_dk, ref_dv = _torch_stage2(q, k, v, cu_q, cu_k, bits, scale, True, dout)
    for h in range(2):
        for kb in range((S + 63) // 64):
            dk, dv, toks = O.stage2_backward_key_block(q, k, v, dout, words[h], kb, h, scale, dtype=np.float64)
            lo, hi = kb * 64, min(kb * 64 + 64, S)
            assert dk.shape == (hi - lo, 128)
            assert np.abs(dk - ref_dk[lo:hi, h]).max() < 1e-9 and np.abs(dv - ref_dv[lo:hi, h]).max() < 1e-9
            assert all(bits[h, t, kb] and t >= lo for t in toks)


def test_stage2_dense_equals_all_blocks_selected():
    q, k, v, cu_q, cu_k, _, _ = _random_case(13, [90], [150], 1, True)
    full = np.tile(np.arange(3, dtype=np.int32), (2, 90, 1))
    words, _ = O.topk_to_uint64(full, 150, 64)
    a, la = O.stage2_forward(q, k, v, cu_q, cu_k, words, 0.1, True)
    b, lb = O.stage2_forward(q, k, v, cu_q, cu_k, None, 0.1, True)
    assert np.array_equal(a, b) and np.array_equal(la, lb)


def test_stage2_lse_is_log_of_softmax_denominator():
    q, k, v, cu_q, cu_k, words, bits = _random_case(14, [64], [64], 1, False)
    out, lse = O.stage2_forward(q, k, v, cu_q, cu_k, words, 0.2, False)
    t, h, g = 5, 1, 3
    s = 0.2 * (k[:64, h].astype(np.float64) @ q[t, 16 * h + g].astype(np.float64))
    assert abs(lse[h, t * 16 + g] - math.log(np.exp(s).sum())) < 1e-9


def test_stage2_backward_finite_differences():
    q, k, v, cu_q, cu_k, words, _ = _random_case(15, [20], [70], 1, True)
    scale = 0.3
    dout = rng(16).standard_normal(q.shape)
    dq, dk, dv = O.stage2_backward(q, k, v, dout, cu_q, cu_k, words, scale, True)

    def loss(qq, kk, vv):
        return float((O.stage2_forward(qq, kk, vv, cu_q, cu_k, words, scale, True)[0] * dout).sum())
    eps = 1e-5
    for arr, grad, pos in ((q, dq, (7, 3, 5)), (k, dk, (10, 1, 9)), (v, dv, (3, 0, 100)), (k, dk, (69, 0, 0))):
        a = arr.astype(np.float64)
        ap, am = a.copy(), a.copy()
        ap[pos] += eps
        am[pos] -= eps
        args_p = [ap if arr is x else x.astype(np.float64) for x in (q, k, v)]
        args_m = [am if arr is x else x.astype(np.float64) for x in (q, k, v)]
        fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
        assert abs(fd - grad[pos]) < 1e-6 * max(1.0, abs(fd))


def test_decode_is_stage2_with_one_query():
    r = rng(17)
    B, cap = 3, 300
    q = O.bf16_round(r.standard_normal((B, 1, 32, 128)).astype(np.float32))
    kc = O.bf16_round(r.standard_normal((B, cap, 2, 128)).astype(np.float32))
    vc = O.bf16_round(r.standard_normal((B, cap, 2, 128)).astype(np.float32))
    lens = [100, 257, 64]
    idx = np.array([[[[0, 1, -1]], [[1, -1, -1]]], [[[0, 4, 2]], [[3, 4, -1]]], [[[0, -1, -1]], [[0, -1, -1]]]], dtype=np.int32)
    words, _ = O.topk_to_uint64(idx, cap, 64)
    knew = O.bf16_round(r.standard_normal((B, 1, 2, 128)).astype(np.float32))
    vnew = O.bf16_round(r.standard_normal((B, 1, 2, 128)).astype(np.float32))
    kc2, vc2 = kc.copy(), vc.copy()
    out, lse = O.decode_forward(q, kc2, vc2, lens, words, 128 ** -0.5, knew, vnew)
    for b in range(B):
        L = lens[b] + 1
        assert np.array_equal(kc2[b, lens[b]], knew[b, 0]) and np.array_equal(kc2[b, :lens[b]], kc[b, :lens[b]])
        bits = O.uint64_to_bool(words[b], (L + 63) // 64)
        ref = _torch_stage2(q[b], kc2[b, :L], vc2[b, :L], [0, 1], [0, L], bits, 128 ** -0.5, False)
        assert np.abs(out[b] - ref).max() < 1e-9
    assert lse.shape == (B, 32, 1)


# ---------------------------------------------------------------------------------------------------------------
# decode options (rotary, paged cache, cache_batch_idx, left padding)
# ---------------------------------------------------------------------------------------------------------------
def _angles(n_pos, half, seed=0):
    rng = np.random.default_rng(seed)
    theta = rng.uniform(-np.pi, np.pi, size=(n_pos, half))
    return O.bf16_round(np.cos(theta).astype(np.float32)), O.bf16_round(np.sin(theta).astype(np.float32)), theta


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("half", [8, 32, 64])
def test_rotary_is_complex_multiplication(interleaved, half):
    """Each pair (a, b) becomes (a + ib)(cos + i sin) (rotary.h:57-62, 131-133); columns beyond rotary_dim stay."""
    rng = np.random.default_rng(1)
    cos, sin, _ = _angles(5, half)
    x = O.bf16_round(rng.standard_normal((3, 128)).astype(np.float32))
    y = O.rotary_apply(x, cos, sin, 3, interleaved)
    if interleaved:
        za = x[:, 0:2 * half:2] + 1j * x[:, 1:2 * half:2]
        zb = y[:, 0:2 * half:2] + 1j * y[:, 1:2 * half:2]
    else:
        za = x[:, :half] + 1j * x[:, half:2 * half]
        zb = y[:, :half] + 1j * y[:, half:2 * half]
    want = za * (cos[3].astype(np.float64) + 1j * sin[3].astype(np.float64))
    assert np.allclose(zb, want, rtol=2 ** -7, atol=1e-6)                 # one bf16 rounding
    assert np.array_equal(y[:, 2 * half:], x[:, 2 * half:])


def test_rotary_identity_norm_and_angle_addition():
    half = 64
    x = np.random.default_rng(2).standard_normal((4, 128)).astype(np.float32)
    one, zero = np.ones((1, half), np.float32), np.zeros((1, half), np.float32)
    for inter in (True, False):
        assert np.array_equal(O.rotary_apply(O.bf16_round(x), one, zero, 0, inter), O.bf16_round(x))
        # a quarter turn maps (a, b) to (-b, a)
        y = O.rotary_apply(O.bf16_round(x), zero, one, 0, inter)
        xb = O.bf16_round(x)
        if inter:
            assert np.array_equal(y[:, 0::2], -xb[:, 1::2]) and np.array_equal(y[:, 1::2], xb[:, 0::2])
        else:
            assert np.array_equal(y[:, :half], -xb[:, half:]) and np.array_equal(y[:, half:], xb[:, :half])
    # exact (unrounded) angles: norms are preserved and two turns add up, within bf16 rounding of the result
    theta = np.random.default_rng(3).uniform(-3, 3, size=(2, half))
    c, s_ = np.cos(theta).astype(np.float32), np.sin(theta).astype(np.float32)
    y = O.rotary_apply(O.bf16_round(x), c, s_, 0, True)
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(O.bf16_round(x), axis=1), rtol=2e-3)
    c2, s2 = np.cos(theta[:1] + theta[1:]).astype(np.float32), np.sin(theta[:1] + theta[1:]).astype(np.float32)
    twice = O.rotary_apply(O.rotary_apply(O.bf16_round(x), c, s_, 0, True), c, s_, 1, True)
    assert np.allclose(twice, O.rotary_apply(O.bf16_round(x), c2, s2, 0, True), atol=0.05)


def _decode_case(seed, B=3, cap=512, Hk=2):
    rng = np.random.default_rng(seed)
    q = O.bf16_round(rng.standard_normal((B, 1, 16 * Hk, 128)).astype(np.float32))
    kc = O.bf16_round(rng.standard_normal((B, cap, Hk, 128)).astype(np.float32))
    vc = O.bf16_round(rng.standard_normal((B, cap, Hk, 128)).astype(np.float32))
    lens = np.array([200, 333, 448][:B], dtype=np.int32)
    idx = np.stack([np.stack([np.sort(rng.choice(cap // 64, size=4, replace=False)) for _ in range(Hk)]) for _ in range(B)])
    words = O.topk_to_uint64(idx.reshape(B, Hk, 1, 4).astype(np.int32), cap, 64)[0]
    return q, kc, vc, lens, words


def test_decode_ext_reduces_to_plain_decode():
    q, kc, vc, lens, words = _decode_case(4)
    a = O.decode_forward(q, kc.copy(), vc.copy(), lens, words, 128 ** -0.5)
    b = O.decode_forward_ext(q, kc.copy(), vc.copy(), lens, words, 128 ** -0.5)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_decode_ext_relabelling_invariance():
    """Paging, cache_batch_idx and left padding only say where a sequence's rows lie: moving the rows and telling
    the oracle where they went must not change the result."""
    q, kc, vc, lens, words = _decode_case(5)
    base = O.decode_forward_ext(q, kc.copy(), vc.copy(), lens, words, 128 ** -0.5)
    B, cap = kc.shape[:2]
    # cache_batch_idx: shuffle the sequences inside a larger cache
    perm = np.array([4, 0, 2])
    big_k, big_v = np.zeros((6,) + kc.shape[1:], np.float32), np.zeros((6,) + vc.shape[1:], np.float32)
    big_k[perm], big_v[perm] = kc, vc
    got = O.decode_forward_ext(q, big_k, big_v, lens, words, 128 ** -0.5, cache_batch_idx=perm)
    assert np.array_equal(got[0], base[0]) and np.array_equal(got[1], base[1])
    # paged: cut every sequence into pages of 128 rows and scatter them
    page = 128
    n_pages = B * cap // page
    order = np.random.default_rng(6).permutation(n_pages)
    table = order.reshape(B, cap // page).astype(np.int32)
    pk, pv = np.zeros((n_pages, page) + kc.shape[2:], np.float32), np.zeros((n_pages, page) + kc.shape[2:], np.float32)
    pk[table.reshape(-1)] = kc.reshape(n_pages, page, *kc.shape[2:])
    pv[table.reshape(-1)] = vc.reshape(n_pages, page, *vc.shape[2:])
    got = O.decode_forward_ext(q, pk, pv, lens, words, 128 ** -0.5, block_table=table)
    assert np.array_equal(got[0], base[0]) and np.array_equal(got[1], base[1])
    # left padding: shift every sequence right by its pad
    pad = np.array([7, 64, 30], dtype=np.int32)
    sk, sv = np.zeros_like(kc), np.zeros_like(vc)
    for b in range(B):
        sk[b, pad[b]:pad[b] + lens[b]] = kc[b, :lens[b]]
        sv[b, pad[b]:pad[b] + lens[b]] = vc[b, :lens[b]]
    got = O.decode_forward_ext(q, sk, sv, lens + pad, words, 128 ** -0.5, cache_leftpad=pad)
    assert np.array_equal(got[0], base[0]) and np.array_equal(got[1], base[1])


def test_decode_ext_rotary_equals_rotating_by_hand():
    q, kc, vc, lens, words = _decode_case(7)
    rng = np.random.default_rng(8)
    kn = O.bf16_round(rng.standard_normal((3, 2, 2, 128)).astype(np.float32))
    vn = O.bf16_round(rng.standard_normal((3, 2, 2, 128)).astype(np.float32))
    cos, sin, _ = _angles(600, 32, seed=9)
    got = O.decode_forward_ext(q, kc.copy(), vc.copy(), lens, words, 128 ** -0.5, k_new=kn, v_new=vn,
                               rotary_cos=cos, rotary_sin=sin, rotary_interleaved=False)
    q2, kn2 = q.copy(), kn.copy()
    for b in range(3):
        q2[b] = O.rotary_apply(q[b], cos, sin, int(lens[b]), False)
        for t in range(2):
            kn2[b, t] = O.rotary_apply(kn[b, t], cos, sin, int(lens[b]) + t, False)
    want = O.decode_forward(q2, kc.copy(), vc.copy(), lens, words, 128 ** -0.5, k_new=kn2, v_new=vn)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
