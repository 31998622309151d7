"""GPU parity (bit-exact) of the mask, pooling and top-k kernels against the CPU oracle, called
through the package operators (which call the C ABI).  Case tables follow the reference's tests
(tests/test_topk_to_uint64.py:259-281, tests/test_uint64_to_bool.py:113-121,
tests/test_blockmask.py:104-113, tests/test_cache_lens.py:10-37, tests/test_pooling_varlen.py:541-571)."""
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


def dev():
    return torch.device("cuda:0")


@pytest.mark.parametrize("shape,max_k,bs", [
    ((2, 128, 16), 256, 4), ((8, 512, 32), 1024, 16), ((16, 1024, 64), 2048, 32), ((32, 2048, 128), 4096, 64),
    ((16, 1024, 64), 8192, 16), ((2, 2, 64, 16), 256, 4), ((4, 8, 128, 32), 1024, 16), ((2, 5, 3), 64, 64),
    ((2, 0, 16), 256, 4)])
def test_topk_to_uint64(ops, shape, max_k, bs):
    torch.manual_seed(0)
    k_blocks = (max_k + bs - 1) // bs
    idx = torch.randint(-1, k_blocks, shape, dtype=torch.int32, device=dev())
    words, kb = ops.topk_to_uint64(idx, max_k, bs)
    ref, kb_ref = O.topk_to_uint64(idx.cpu().numpy(), max_k, bs)
    assert kb == kb_ref and words.dtype == torch.int64 and tuple(words.shape) == ref.shape
    assert np.array_equal(words_np(words), ref)


def test_topk_to_uint64_full_size_popcount(ops):
    """BASELINE size (2, 32768, 64) over 512 blocks: popcount of each row == number of distinct indices."""
    torch.manual_seed(1)
    idx = torch.stack([torch.stack([torch.randperm(512, device=dev())[:64] for _ in range(64)]) for _ in range(2)])
    idx = idx.to(torch.int32).repeat(1, 512, 1)                     # (2, 32768, 64)
    words, _ = ops.topk_to_uint64(idx, 32768, 64)
    ref, _ = O.topk_to_uint64(idx.cpu().numpy(), 32768, 64)
    assert np.array_equal(words_np(words), ref)
    bits = ops.uint64_to_bool(words, 512)
    assert bool((bits.sum(-1) == 64).all())


@pytest.mark.parametrize("shape,last", [((100, 1), 64), ((100, 1), 63), ((100, 2), 65), ((100, 2), 128), ((100, 4), 200),
                                        ((2, 3, 4, 2), 100), ((1000, 16), 1000), ((7, 3), 129), ((0, 2), 100)])
def test_uint64_to_bool_and_roundtrip(ops, shape, last):
    g = torch.Generator(device="cpu").manual_seed(2)
    words = torch.randint(-2 ** 63, 2 ** 63 - 1, shape, dtype=torch.int64, generator=g).to(dev())
    b = ops.uint64_to_bool(words, last)
    assert b.dtype == torch.bool and tuple(b.shape) == shape[:-1] + (last,)
    assert np.array_equal(b.cpu().numpy(), O.uint64_to_bool(words_np(words), last))
    back, l2 = ops.blockmask_to_uint64(b)
    assert l2 == last
    assert np.array_equal(words_np(back), O.blockmask_to_uint64(b.cpu().numpy())[0])
    assert torch.equal(ops.uint64_to_bool(back, last), b)


@pytest.mark.parametrize("shape", [(100, 64), (100, 63), (100, 65), (100, 128), (100, 200), (2, 3, 4, 100),
                                   (1000, 1000), (50, 100, 1000)])
def test_blockmask_to_uint64(ops, shape):
    torch.manual_seed(3)
    m = torch.rand(shape, device=dev()) < 0.5
    words, last = ops.blockmask_to_uint64(m)
    assert last == shape[-1]
    assert np.array_equal(words_np(words), O.blockmask_to_uint64(m.cpu().numpy())[0])


@pytest.mark.parametrize("Hk,T,nblk", [(2, 150, 70), (2, 64, 64), (1, 1, 1), (2, 1000, 130), (2, 4096, 64)])
def test_transpose_blockmask(ops, Hk, T, nblk):
    torch.manual_seed(4)
    m = torch.rand((Hk, T, nblk), device=dev()) < 0.25
    fwd, _ = ops.blockmask_to_uint64(m)
    bwd = ops.transpose_blockmask(fwd, nblk)
    assert np.array_equal(words_np(bwd), O.transpose_blockmask(words_np(fwd), nblk))
    # equals the reference's three-step sequence (infllmv2_sparse_attention.py:344-350)
    seq, _ = ops.blockmask_to_uint64(ops.uint64_to_bool(fwd, nblk).transpose(1, 2).contiguous())
    assert torch.equal(seq, bwd)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("q,kl,cache,local,init", [(70, 127, 0, 1, 1), (130, 30, 0, 2, 1), (33, 17, 64, 4, 1),
                                                   (200, 51, 128, 0, 0), (5, 3, 0, 1, 2), (512, 2047, 0, 31, 1),
                                                   (300, 5, 0, 0, 0)])
def test_max_pooling_1d(ops, dtype, q, kl, cache, local, init):
    torch.manual_seed(5)
    x = torch.randn(2, q, kl, device=dev()).to(dtype)
    out = ops.max_pooling_1d(x, cache, local, init)
    ref = O.max_pooling_1d_fast(bf16_np(x), cache, local, init)
    assert out.dtype == dtype and tuple(out.shape) == ref.shape
    assert np.array_equal(bf16_np(out), ref)


def test_max_pooling_1d_strided_view_and_special_values(ops):
    """A padded score buffer (row stride 2048, 2047 valid columns) is pooled in place; NaN, signed zero
    and infinities pick the element the sequential '>' scan of the reference picks."""
    torch.manual_seed(6)
    buf = torch.randn(2, 256, 2048, device=dev()).to(torch.bfloat16)
    buf[0, 3, 40:48] = 0.0
    buf[0, 3, 44] = -0.0
    buf[1, 7, 100] = float("inf")
    buf[1, 9, 203] = float("-inf")
    view = buf[:, :, :2047]
    assert not view.is_contiguous()
    out = ops.max_pooling_1d(view, 0, 1, 1)
    assert torch.equal(out, ops.max_pooling_1d(view.contiguous(), 0, 1, 1))
    assert np.array_equal(bf16_np(out), O.max_pooling_1d_fast(bf16_np(view), 0, 1, 1))


def test_max_pooling_1d_varlen(ops):
    sq, sk, cl = [10, 15, 8], [20, 25, 16], [0, 64, 128]             # tests/test_cache_lens.py:10-37
    cu_q = torch.tensor(np.cumsum([0] + sq), dtype=torch.int32, device=dev())
    cu_k = torch.tensor(np.cumsum([0] + sk), dtype=torch.int32, device=dev())
    cache = torch.tensor(cl, dtype=torch.int32, device=dev())
    torch.manual_seed(7)
    x = torch.randn(2, sum(sq), max(sk), device=dev()).to(torch.float16)
    out = ops.max_pooling_1d_varlen(x, cu_q, cu_k, cache, max(sq), max(sk), 4, 1)
    ref = O.max_pooling_1d_varlen(bf16_np(x), cu_q.cpu().numpy(), cu_k.cpu().numpy(), cl, max(sq), max(sk), 4, 1)
    assert tuple(out.shape) == ref.shape and np.array_equal(bf16_np(out), ref)


def test_max_pooling_1d_varlen_packed_prefill(ops):
    """Four packed sequences, compressed-key lengths (S-32)//16+1, cache_len 0: equals the fixed-length
    operator applied per sequence (tests/test_pooling_varlen.py:535-652 compares the same two paths)."""
    S = [320, 1024, 64, 700]
    Lk = [(s - 32) // 16 + 1 for s in S]
    cu_q = torch.tensor(np.cumsum([0] + S), dtype=torch.int32, device=dev())
    cu_k = torch.tensor(np.cumsum([0] + Lk), dtype=torch.int32, device=dev())
    cache = torch.zeros(4, dtype=torch.int32, device=dev())
    torch.manual_seed(8)
    x = torch.randn(2, sum(S), max(Lk), device=dev()).to(torch.bfloat16)
    out = ops.max_pooling_1d_varlen(x, cu_q, cu_k, cache, max(S), max(Lk), 3, 1)
    ref = O.max_pooling_1d_varlen(bf16_np(x), cu_q.cpu().numpy(), cu_k.cpu().numpy(), [0] * 4, max(S), max(Lk), 3, 1)
    assert np.array_equal(bf16_np(out), ref)
    for b in range(4):
        seg = x[:, int(cu_q[b]):int(cu_q[b + 1]), :Lk[b]].contiguous()
        fixed = ops.max_pooling_1d(seg, 0, 3, 1)
        assert torch.equal(out[:, int(cu_q[b]):int(cu_q[b + 1]), :fixed.shape[2]], fixed)


@pytest.mark.parametrize("rows,n,k", [((2, 100), 100, 16), ((2, 300), 512, 64), ((3, 50), 33, 64), ((2, 64), 2048, 64),
                                      ((1, 10), 4100, 16), ((2, 8), 700, 256), ((2, 5), 64, 64), ((2, 5), 1, 1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_topk_blocks(ops, rows, n, k, dtype):
    torch.manual_seed(9)
    x = torch.randn(rows + (n,), device=dev()).to(dtype)
    x[..., : min(3, n)] = float("inf")
    if n > 60:
        x[..., 50:60] = 0.0                       # exact ties
        x[..., n - 5:] = float("-inf")
    got = ops.topk_blocks(x, k)
    ref = O.topk_blocks(bf16_np(x), k)
    assert got.dtype == torch.int32 and np.array_equal(got.cpu().numpy(), ref)


def test_topk_blocks_many_ties_full_size(ops):
    """Rows of pooled scores as Stage 1 produces them: +inf forced blocks, zeros for blocks in the
    future of the query, few distinct values.  Bit-exact indices and, order-free, the packed mask."""
    torch.manual_seed(10)
    n, k = 512, 64
    x = (torch.randn(2, 4096, n, device=dev()) * 0.05).abs().to(torch.bfloat16)
    x[:, :, 0] = float("inf")
    for t in range(0, 4096, 64):
        b = t // 64
        x[:, t:t + 64, max(0, b - 31):b + 1] = float("inf")
        x[:, t:t + 64, b + 1:] = 0.0
    got = ops.topk_blocks(x, k)
    ref = O.topk_blocks(bf16_np(x), k)
    assert np.array_equal(got.cpu().numpy(), ref)
    w, _ = ops.topk_to_uint64(got, n * 64, 64)
    assert np.array_equal(words_np(w), O.topk_to_uint64(ref, n * 64, 64)[0])


def _postprocess(ref_idx, x_np, by_index, drop):
    """Oracle-side statement of the options of topk_blocks: drop columns whose score is -inf, then (by_index) sort
    the survivors by column; -1 pads the end either way."""
    out = np.full_like(ref_idx, -1)
    flat_i, flat_o = ref_idx.reshape(-1, ref_idx.shape[-1]), out.reshape(-1, ref_idx.shape[-1])
    flat_x = x_np.reshape(-1, x_np.shape[-1])
    for r in range(flat_i.shape[0]):
        keep = [int(c) for c in flat_i[r] if c >= 0 and not (drop and np.isneginf(flat_x[r, c]))]
        if by_index:
            keep.sort()
        flat_o[r, :len(keep)] = keep
    return out


@pytest.mark.parametrize("rows,n,k", [((2, 130), 512, 64), ((3, 40), 100, 16), ((2, 30), 2048, 64), ((2, 9), 700, 256),
                                      ((1, 70), 33, 64), ((2, 33), 4100, 16)])
@pytest.mark.parametrize("by_index,drop", [(False, False), (True, False), (False, True), (True, True)])
def test_topk_select_options_and_fused_mask(ops, rows, n, k, by_index, drop):
    """The fused selection: indices in score or block order, -inf columns optionally never selected, and the packed
    mask written by the same launch == topk_to_uint64 of the indices == the oracle's packing.  Consecutive rows are
    made to differ wildly (the search of a row starts at its neighbour's threshold): scale jumps by orders of
    magnitude, rows of all ties, rows with only a handful of reachable columns."""
    g = torch.Generator(device="cpu").manual_seed(11)
    x = torch.randn(rows + (n,), generator=g)
    R = rows[-1]
    for r in range(R):
        x[:, r] *= float(10.0 ** ((r * 7) % 9 - 4))           # 1e-4 .. 1e4 from one row to the next
        if r % 5 == 1:
            x[:, r] = 0.25                                     # every column ties
        if r % 5 == 2:
            x[:, r, min(7, n - 1):] = float("-inf")            # fewer reachable columns than k
        if r % 5 == 3:
            x[:, r, : min(40, n)] = float("inf")               # forced columns, ties at +inf
            x[:, r, n // 2:] = float("-inf")
        if r % 7 == 4:
            x[:, r] = -x[:, r].abs()                           # all negative
    x = x.to(torch.bfloat16).to(dev())
    idx, mask = ops.topk_blocks(x, k, by_index=by_index, drop_unreachable=drop, return_mask=True)
    x_np = bf16_np(x)
    want = _postprocess(O.topk_blocks(x_np, k), x_np, by_index, drop)
    assert np.array_equal(idx.cpu().numpy(), want)
    n64 = (n + 63) // 64
    assert tuple(mask.shape) == rows + (n64,) and mask.dtype == torch.int64
    assert np.array_equal(words_np(mask), O.topk_to_uint64(want, n * 64, 64)[0])
    again, _ = ops.topk_to_uint64(idx, n * 64, 64)
    assert torch.equal(again, mask)
    # without the mask and with a wider mask row
    assert torch.equal(ops.topk_blocks(x, k, by_index=by_index, drop_unreachable=drop), idx)
    _, wide = ops.topk_blocks(x, k, by_index=by_index, drop_unreachable=drop, return_mask=True, n_uint64_per_row=n64 + 3)
    assert torch.equal(wide[..., :n64], mask) and not bool(wide[..., n64:].any())


def test_topk_select_fp16_drops_fp16_minus_infinity(ops):
    x = torch.randn(2, 20, 200, device=dev()).to(torch.float16)
    x[..., 150:] = float("-inf")
    idx = ops.topk_blocks(x, 180, drop_unreachable=True, by_index=True)
    want = torch.arange(150, device=dev(), dtype=torch.int32).expand(2, 20, 150)
    assert torch.equal(idx[..., :150], want) and bool((idx[..., 150:] == -1).all())


def test_block_mask_argument_equals_topk_idx_argument(ops):
    """Stage 2 fed with the fused launch's mask == Stage 2 fed with the index list (which it packs itself); forward
    and backward, and the decode operator."""
    torch.manual_seed(12)
    S, k_sel = 700, 6
    mk = lambda h: torch.randn(S, h, 128, device=dev()).to(torch.bfloat16)
    q, k, v = mk(32), mk(2), mk(2)
    cu = torch.tensor([0, S], dtype=torch.int32, device=dev())
    idx, mask = ops.select_blocks(q, k, cu, cu, S, S, k_sel, 1, 1, return_mask=True)
    assert torch.equal(idx, ops.select_blocks(q, k, cu, cu, S, S, k_sel, 1, 1))
    outs = []
    for kw in (dict(topk_idx=idx), dict(topk_idx=idx, block_mask=mask), dict(block_mask=mask)):
        qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
        o = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, S, S, causal=True, **kw)
        o.backward(torch.ones_like(o))
        outs.append((o.detach(), qg.grad, kg.grad.float(), vg.grad.float()))
    for o, dq, dk, dv in outs[1:]:
        assert torch.equal(o, outs[0][0]) and torch.equal(dq, outs[0][1])
        assert float((dk - outs[0][2]).abs().max()) <= 2e-2 * float(outs[0][2].abs().max())
        assert float((dv - outs[0][3]).abs().max()) <= 2e-2 * float(outs[0][3].abs().max())
    with pytest.raises(RuntimeError, match="block_mask"):
        ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, S, S, causal=True, block_mask=mask[:, :, :0])
    B, cap = 3, 640
    qd = torch.randn(B, 1, 32, 128, device=dev()).to(torch.bfloat16)
    kc = torch.randn(B, cap, 2, 128, device=dev()).to(torch.bfloat16)
    vc = torch.randn(B, cap, 2, 128, device=dev()).to(torch.bfloat16)
    L = torch.tensor([640, 300, 65], dtype=torch.int32, device=dev())
    pooled = torch.rand(B, 2, 1, cap // 64, device=dev()).to(torch.bfloat16)
    di, dm = ops.topk_blocks(pooled, 4, return_mask=True)
    a = ops.infllmv2_attn_with_kvcache(qd, kc, vc, cache_seqlens=L, topk_idx=di)
    b = ops.infllmv2_attn_with_kvcache(qd, kc, vc, cache_seqlens=L, block_mask=dm)
    assert torch.equal(a, b)
