"""The operators strung together as a model would (infllmv2_cuda_impl_amd/layer.py): prefill over packed sequences,
and a decode loop whose every step must reproduce what a prefill of the same, one token longer, sequence computes for
its last token — same selected blocks, same attention — through the other set of kernels (Stage 1 with one query
against the compressed-key caches, pooling with cache_len, the split decode kernel, compressed keys appended as windows
complete).  Tolerance of the Stage-2 forward: max-abs <= 2e-2, mean-abs <= 1e-3."""
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


def qkv(seed, T, Hk=2):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(T, h, 128, generator=g).to(torch.bfloat16).cuda()
    return mk(16 * Hk), mk(Hk), mk(Hk)


def test_prefill_matches_oracle_pipeline(ops):
    """Packed prefill through the layer == oracle Stage-2 on the blocks the layer selected."""
    seqs = [700, 1300, 300]
    T = sum(seqs)
    q, k, v = qkv(1, T)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    cu = torch.from_numpy(cu_np).cuda()
    layer = ops.InfLLMv2Attention(topk=8, local_blocks=2, init_blocks=1)
    out = layer(q, k, v, cu, max(seqs))
    idx = ops.select_blocks(q, k, cu, cu, max(seqs), max(seqs), 8, 2, 1,
                            cache_lens=torch.zeros(3, dtype=torch.int32, device="cuda"))
    words = O.topk_to_uint64(idx.cpu().numpy(), max(seqs), 64)[0]
    ref, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_np, cu_np, words, 128 ** -0.5, True)
    err = np.abs(bf16_np(out) - ref)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3


def test_short_sequences_attend_densely(ops):
    q, k, v = qkv(2, 200)
    cu = torch.tensor([0, 200], dtype=torch.int32, device="cuda")
    out = ops.InfLLMv2Attention(topk=2, local_blocks=0, init_blocks=1, dense_len=256)(q, k, v, cu, 200)
    ref, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), [0, 200], [0, 200], None, 128 ** -0.5, True)
    assert np.abs(bf16_np(out) - ref).max() <= 2e-2


@pytest.mark.parametrize("start,steps,topk,local", [(1000, 40, 6, 1), (96, 70, 3, 0), (2048, 20, 16, 2)])
def test_decode_steps_equal_prefill_of_the_longer_sequence(ops, start, steps, topk, local):
    total = start + steps
    q, k, v = qkv(3, total)
    cu = lambda n: torch.tensor([0, n], dtype=torch.int32, device="cuda")
    layer = ops.InfLLMv2Attention(topk=topk, local_blocks=local, init_blocks=1)
    full = layer(q, k, v, cu(total), total)                    # every position computed by the prefill kernels
    cache = ops.SequenceCache.empty(total + 64, 2, 128, "cuda")
    head = layer(q[:start], k[:start], v[:start], cu(start), start, cache=cache)
    assert torch.equal(head, layer(q[:start], k[:start], v[:start], cu(start), start))
    worst = 0.0
    checked = 0
    for t in range(start, total):
        out = layer.decode(q[t][None, None], k[t][None, None], v[t][None, None], cache)
        assert cache.length == t + 1
        L = t + 1
        if L % 16 == 15 or L % 64 == 63:
            continue                                           # the prefill's last token does not see the newest compressed key
        # the prefill of the whole sequence computed token t against keys 0..t, with the selection of token t
        err = (out[0, 0].float() - full[t].float()).abs()
        worst = max(worst, float(err.max()))
        assert float(err.max()) <= 2e-2 and float(err.mean()) <= 1e-3, (t, float(err.max()))
        checked += 1
    assert checked >= steps * 3 // 4
    # the caches hold what a fresh compression of the whole sequence gives
    kf, _ = ops.compress_keys(k, cu(total), total, 32, 16)
    kc, _ = ops.compress_keys(k, cu(total), total, 128, 64)
    assert torch.equal(cache.k_fine[:kf.shape[0]], kf) and torch.equal(cache.k_coarse[:kc.shape[0]], kc)
    assert torch.equal(cache.k[0, :total], k) and torch.equal(cache.v[0, :total], v)


def _forced_words(S_list, positions, local, init, n64, q_rows):
    """Oracle-side mask of the window branch: block kb is set iff kb < init or 0 <= bq - kb <= local."""
    words = np.zeros((2, q_rows, n64), dtype=np.uint64)
    row = 0
    for S, pos in zip(S_list, positions):
        for i in range(S):
            bq = (i + pos) // 64
            for kb in list(range(min(init, bq + 1))) + list(range(max(0, bq - local), bq + 1)):
                words[:, row, kb // 64] |= np.uint64(1) << np.uint64(kb % 64)
            row += 1
    return words


def test_window_and_dense_branches(ops):
    """selection='window': only the first block(s) and the local window, no scoring; selection='dense': everything.
    Prefill over packed sequences and decode steps (single sequence and batched) against the oracle."""
    seqs = [700, 300, 1100]
    T = sum(seqs)
    q, k, v = qkv(8, T)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    cu = torch.from_numpy(cu_np).cuda()
    local, init = 3, 1
    win = ops.InfLLMv2Attention(topk=8, local_blocks=local, init_blocks=init, selection="window")
    out = win(q, k, v, cu, max(seqs))
    words = _forced_words(seqs, [0, 0, 0], local, init, 1, T)
    ref, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_np, cu_np, words, 128 ** -0.5, True)
    err = np.abs(bf16_np(out) - ref)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3
    dense = ops.InfLLMv2Attention(selection="dense")(q, k, v, cu, max(seqs))
    ref_d, _ = O.stage2_forward(bf16_np(q), bf16_np(k), bf16_np(v), cu_np, cu_np, None, 128 ** -0.5, True)
    assert np.abs(bf16_np(dense) - ref_d).max() <= 2e-2
    # decode: the window branch of a step == the prefill's last token of the one-token-longer sequence
    start, steps = 900, 12
    q1, k1, v1 = qkv(9, start + steps)
    one = lambda n: torch.tensor([0, n], dtype=torch.int32, device="cuda")
    full = win(q1, k1, v1, one(start + steps), start + steps)
    cache = ops.SequenceCache.empty(start + steps + 64, 2, 128, "cuda")
    win(q1[:start], k1[:start], v1[:start], one(start), start, cache=cache)
    bcache = ops.BatchCache.empty(2, start + steps + 64, 2, 128, "cuda")
    win.fill_cache(bcache, torch.cat([k1[:start], k1[:start - 100]]), torch.cat([v1[:start], v1[:start - 100]]), [start, start - 100])
    for t in range(start, start + steps):
        o1 = win.decode(q1[t][None, None], k1[t][None, None], v1[t][None, None], cache)
        e = (o1[0, 0].float() - full[t].float()).abs()
        assert float(e.max()) <= 2e-2 and float(e.mean()) <= 1e-3, t
        ob = win.decode_batch(q1[t][None, None].expand(2, 1, 32, 128).contiguous(), k1[t][None, None].expand(2, 1, 2, 128).contiguous(),
                              v1[t][None, None].expand(2, 1, 2, 128).contiguous(), bcache)
        e = (ob[0, 0].float() - full[t].float()).abs()
        assert float(e.max()) <= 2e-2 and float(e.mean()) <= 1e-3, t
