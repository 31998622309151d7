"""IEEE half (fp16) through every attention entry point, against the CPU oracle on the same fp16-rounded inputs.

The reference switches on the tensors' dtype (csrc/entry.cu:20-29) and its build instantiates bfloat16 only; here both
element types exist.  Tolerances are the bf16 ones (fp16 has three more mantissa bits, so the errors are smaller):
Stage-1 |err| <= 2^-7 |ref| + 2e-3; Stage-2 forward / decode max-abs <= 2e-2, mean-abs <= 1e-3, LSE <= 2e-3; gradients
max-abs <= 2e-2 s, mean-abs <= 1e-3 s with s = max(1, max|ref|).  Compressed keys, pooling, top-k and masks: bit-exact.
Two tests also check that the results carry fp16's precision (errors below what one bf16 rounding of the output would
leave), so a bf16 instantiation run on reinterpreted bits could not pass."""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np, words_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F16 = torch.float16


@pytest.fixture(scope="module")
def ops():
    import infllmv2_cuda_impl_amd as ops
    return ops


def rand(shape, seed, gain=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * gain).to(F16)


def random_selection(seed, Hk, seqs, k_sel):
    g = torch.Generator(device="cpu").manual_seed(seed)
    T = sum(seqs)
    idx = torch.full((Hk, T, k_sel), -1, dtype=torch.int32)
    row = 0
    for s in seqs:
        nb = (s + 63) // 64
        for t in range(row, row + s):
            for h in range(Hk):
                sel = torch.randperm(nb, generator=g)[:k_sel].sort().values
                idx[h, t, :len(sel)] = sel.to(torch.int32)
        row += s
    return idx


def test_compressed_keys_fp16_bit_exact(ops):
    """Mean of fp16 keys over windows 32/16 and 128/64: fp32 sum in window order, divided, rounded once to fp16
    (a plain sequential sum written out here, not the oracle's vectorised mean)."""
    seqs = [700, 130, 31, 1000]
    k = rand((sum(seqs), 2, 128), 1)
    cu = torch.tensor(np.cumsum([0] + seqs), dtype=torch.int32)
    for kernel, stride in ((32, 16), (128, 64)):
        got, cu_c = ops.compress_keys(k.to(DEV), cu.to(DEV), max(seqs), kernel, stride)
        assert got.dtype == F16
        kn = k.float().numpy()
        want = []
        for b, s in enumerate(seqs):
            seq = kn[int(cu[b]):int(cu[b + 1])]
            for j in range(O.compressed_len(s, kernel, stride)):
                acc = np.zeros(seq.shape[1:], dtype=np.float32)
                for i in range(kernel):
                    acc = acc + seq[stride * j + i]
                want.append((acc / np.float32(kernel)).astype(np.float16))
        want = np.stack(want)
        n = int(cu_c[-1])
        assert n == want.shape[0]
        assert np.array_equal(got[:n].cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("seqs,Hk,k_sel,causal", [([300, 1000], 2, 5, True), ([257], 1, 3, True), ([64, 130], 2, 2, False)])
def test_stage2_forward_backward_fp16(ops, seqs, Hk, k_sel, causal):
    T = sum(seqs)
    q, k, v, dout = rand((T, 16 * Hk, 128), 2), rand((T, Hk, 128), 3), rand((T, Hk, 128), 4), rand((T, 16 * Hk, 128), 5)
    idx = random_selection(6, Hk, seqs, k_sel)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    cu = torch.from_numpy(cu_np).to(DEV)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out, lse, _ = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, max(seqs), max(seqs), causal=causal,
                                                topk_idx=idx.to(DEV), return_attn_probs=True)
    assert out.dtype == F16
    out.backward(dout.to(DEV))
    words = O.topk_to_uint64(idx.numpy(), max(seqs), 64)[0]
    qn, kn, vn, dn = [bf16_np(t) for t in (q, k, v, dout)]
    ref_o, ref_lse = O.stage2_forward(qn, kn, vn, cu_np, cu_np, words, 128 ** -0.5, causal)
    err = np.abs(bf16_np(out).astype(np.float64) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    l = lse.cpu().numpy().astype(np.float64)
    fin = np.isfinite(ref_lse)
    assert np.array_equal(np.isinf(l) & (l > 0), ~fin) and np.abs(l[fin] - ref_lse[fin]).max() <= 2e-3
    dq, dk, dv = O.stage2_backward(qn, kn, vn, dn, cu_np, cu_np, words, 128 ** -0.5, causal)
    for name, got, ref in (("dq", qg.grad, dq), ("dk", kg.grad, dk), ("dv", vg.grad, dv)):
        assert got.dtype == F16
        s = max(1.0, float(np.abs(ref).max()))
        e = np.abs(bf16_np(got).astype(np.float64) - ref)
        assert e.max() <= 2e-2 * s and e.mean() <= 1e-3 * s, (name, e.max(), e.mean(), s)
    # fp16 keeps three more mantissa bits than bf16: its output error must be clearly below what bf16 rounding of the
    # output alone would leave, i.e. the fp16 kernels ran, not the bf16 ones on reinterpreted bits
    assert err.mean() < 4e-4


def test_backward_modes_fp16(ops):
    """Deterministic dK/dV in fp16 agrees with the default mode to rounding and is bit-reproducible."""
    seqs = [900]
    T = 900
    q, k, v, dout = rand((T, 32, 128), 7), rand((T, 2, 128), 8), rand((T, 2, 128), 9), rand((T, 32, 128), 10)
    idx = random_selection(11, 2, seqs, 6).to(DEV)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)

    def grads(deterministic=False):
        qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
        out = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, T, T, causal=True, topk_idx=idx, deterministic=deterministic)
        out.backward(dout.to(DEV))
        return [t.grad.float() for t in (qg, kg, vg)]

    base = grads()
    det1, det2 = grads(True), grads(True)
    for a, c, d in zip(base, det1, det2):
        s = max(1.0, float(a.abs().max()))
        assert float((a - c).abs().max()) <= 2e-2 * s
        assert torch.equal(c, d)


def test_stage1_fp16_scores_pooled_and_topk(ops):
    """Stage 1 on fp16 q / compressed keys against the oracle; fused pooling == separate calls bit for bit; top-k and
    mask words bit-exact on the GPU's pooled scores."""
    seqs = [1100, 500]
    T = sum(seqs)
    q, k = rand((T, 32, 128), 12), rand((T, 2, 128), 13)
    cu_np = np.cumsum([0] + seqs).astype(np.int32)
    kf, cu_f = O.compress_keys(bf16_np(k), cu_np, 32, 16, rounding=O.f16_round)
    kc, cu_c = O.compress_keys(bf16_np(k), cu_np, 128, 64, rounding=O.f16_round)
    Lk = max(np.diff(cu_f))
    t = lambda x, dt=None: torch.from_numpy(np.ascontiguousarray(x)).to(DEV) if dt is None else torch.from_numpy(np.ascontiguousarray(x)).to(dt).to(DEV)
    args = (q.to(DEV), t(kf, F16), t(kc, F16), t(cu_np), t(cu_f), t(cu_c), max(seqs), int(Lk))
    score = ops.infllmv2_attn_stage1(*args, causal=True)
    assert score.dtype == F16
    ref = O.stage1_scores(bf16_np(q), kf, kc, cu_np, cu_f, cu_c, int(Lk), 128 ** -0.5, True, round_output=False)
    got = bf16_np(score).astype(np.float64)
    assert (np.abs(got - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3).all()
    # an fp16 result, not a bf16 one: mostly closer to the unrounded reference than bf16 rounding allows
    big = np.abs(ref) > 0.05
    assert np.mean(np.abs(got[big] - ref[big]) <= 2.0 ** -9 * np.abs(ref[big])) > 0.9
    cache_lens = torch.zeros(2, dtype=torch.int32, device=DEV)
    sep = ops.max_pooling_1d_varlen(score, t(cu_np), t(cu_f), cache_lens, max(seqs), int(Lk), 2, 1)
    fused = ops.infllmv2_attn_stage1_pooled(*args, 2, 1, cache_lens=cache_lens, causal=True)
    assert fused.dtype == F16 and torch.equal(sep.view(torch.int16), fused.view(torch.int16))
    idx, mask = ops.topk_blocks(fused, 6, return_mask=True)
    want = O.topk_blocks(bf16_np(fused), 6)
    assert np.array_equal(idx.cpu().numpy(), want)
    assert np.array_equal(words_np(mask), O.topk_to_uint64(want, fused.shape[-1] * 64, 64)[0])
    # select_blocks (compress on the GPU + fused Stage 1 + top-k) picks the same blocks
    idx2 = ops.select_blocks(q.to(DEV), k.to(DEV), t(cu_np), t(cu_np), max(seqs), max(seqs), 6, 2, 1, cache_lens=cache_lens)
    assert torch.equal(idx, idx2)


def test_decode_fp16_with_append_and_rotary(ops):
    B, cap, Hk = 3, 640, 2
    q, kc, vc = rand((B, 1, 32, 128), 14), rand((B, cap, Hk, 128), 15), rand((B, cap, Hk, 128), 16)
    kn, vn = rand((B, 1, Hk, 128), 17), rand((B, 1, Hk, 128), 18)
    lens = np.array([100, 575, 320], dtype=np.int32)
    g = torch.Generator(device="cpu").manual_seed(19)
    nblk = cap // 64
    bits = torch.rand(B, Hk, 1, nblk, generator=g) < 0.5
    bits[..., 0] = True
    words = O.blockmask_to_uint64(bits.numpy())[0]
    theta = torch.arange(cap)[:, None].float() * (10000.0 ** (-torch.arange(32).float() / 32))[None, :]
    cos, sin = torch.cos(theta).to(F16), torch.sin(theta).to(F16)
    idx = torch.full((B, Hk, 1, nblk), -1, dtype=torch.int32)
    for b in range(B):
        for h in range(Hk):
            sel = torch.nonzero(bits[b, h, 0]).flatten().to(torch.int32)
            idx[b, h, 0, :len(sel)] = sel
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    out, lse = ops.infllmv2_attn_with_kvcache(q.to(DEV), kcd, vcd, k=kn.to(DEV), v=vn.to(DEV), rotary_cos=cos.to(DEV),
                                              rotary_sin=sin.to(DEV), cache_seqlens=torch.from_numpy(lens).to(DEV),
                                              topk_idx=idx.to(DEV), return_softmax_lse=True, rotary_interleaved=False)
    assert out.dtype == F16
    kc_np, vc_np = bf16_np(kc).copy(), bf16_np(vc).copy()
    ref_o, ref_lse = O.decode_forward_ext(bf16_np(q), kc_np, vc_np, lens, words, 128 ** -0.5, k_new=bf16_np(kn),
                                          v_new=bf16_np(vn), rotary_cos=bf16_np(cos), rotary_sin=bf16_np(sin),
                                          rotary_interleaved=False, rounding=O.f16_round)
    err = np.abs(bf16_np(out).astype(np.float64) - ref_o)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 2e-3
    # the appended rows, turned by the rotary embedding, are in the cache bit for bit
    for b in range(B):
        assert np.array_equal(bf16_np(kcd[b, lens[b]]), kc_np[b, lens[b]])
        assert np.array_equal(bf16_np(vcd[b, lens[b]]), vc_np[b, lens[b]])


def test_layer_fp16_decode_steps_equal_prefill(ops):
    """The whole call sequence in fp16: prefill, then decode steps (single sequence and batched) that must reproduce
    the prefill of the one-token-longer sequence."""
    start, steps = 700, 24
    total = start + steps
    q, k, v = rand((total, 32, 128), 20).to(DEV), rand((total, 2, 128), 21).to(DEV), rand((total, 2, 128), 22).to(DEV)
    cu = lambda n: torch.tensor([0, n], dtype=torch.int32, device=DEV)
    layer = ops.InfLLMv2Attention(topk=6, local_blocks=1, init_blocks=1)
    full = layer(q, k, v, cu(total), total)
    assert full.dtype == F16
    cache = ops.SequenceCache.empty(total + 64, 2, 128, DEV, dtype=F16)
    layer(q[:start], k[:start], v[:start], cu(start), start, cache=cache)
    bcache = ops.BatchCache.empty(2, total + 64, 2, 128, DEV, dtype=F16)
    layer.fill_cache(bcache, torch.cat([k[:start], k[:start - 50]]), torch.cat([v[:start], v[:start - 50]]), [start, start - 50])
    checked = 0
    for t in range(start, total):
        o1 = layer.decode(q[t][None, None], k[t][None, None], v[t][None, None], cache)
        ob = layer.decode_batch(q[t][None, None].expand(2, 1, 32, 128).contiguous(), k[t][None, None].expand(2, 1, 2, 128).contiguous(),
                                v[t][None, None].expand(2, 1, 2, 128).contiguous(), bcache)
        L = t + 1
        if L % 16 == 15 or L % 64 == 63:
            continue                                           # the prefill's last token does not see the newest compressed key
        for o in (o1[0, 0], ob[0, 0]):
            e = (o.float() - full[t].float()).abs()
            assert float(e.max()) <= 2e-2 and float(e.mean()) <= 1e-3, t
        checked += 1
    assert checked >= steps * 3 // 4


def test_native_module_style_calls_fp16(ops):
    """The pybind-style module (infllm_v2.C) with fp16 tensors: varlen_fwd / varlen_bwd on re-laid-out queries."""
    from infllmv2_cuda_impl_amd import C
    S = 320
    q, k, v, dout = [rand(s, i).to(DEV) for i, s in ((23, (S, 32, 128)), (24, (S, 2, 128)), (25, (S, 2, 128)), (26, (S, 32, 128)))]
    idx = random_selection(27, 2, [S], 3).to(DEV)
    cu = torch.tensor([0, S], dtype=torch.int32, device=DEV)
    out = ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, S, S, causal=True, topk_idx=idx)
    words, _ = ops.topk_to_uint64(idx, S, 64)
    from test_gpu_c_module import expand, collapse
    res = C.varlen_fwd(expand(q, 2), k, v, None, cu * 16, cu, None, None, None, None, S * 16, S, 0.0, 128 ** -0.5, False,
                       True, -1, -1, 0.0, False, None, words)
    back = collapse(res[0], 2)
    assert back.dtype == F16 and torch.equal(back, out)
