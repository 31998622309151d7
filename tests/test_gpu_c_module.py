"""The reference's native module (`infllm_v2.C`: the compiled extension `infllmv2_cuda_impl_amd._C`, and its
pure-Python twin `infllmv2_cuda_impl_amd.C`) called the way the reference's own Python
wrappers call it (infllm_v2/infllmv2_sparse_attention.py:71-130, 174-263, 551-589, max_pooling_1d.py:25-41,
topk_to_uint64.py:60-68): re-laid-out (T*16, Hk, d) queries, cu_seqlens * 16, transposed column mask for
the backward.  Results must equal those of the package operators, which run the same kernels in place."""
import numpy as np
import pytest
import torch

from test_gpu_stage2_fwd import make_case

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["compiled", "python"])
def C(request):
    """Both implementations of the native-module interface: the compiled extension is what `infllm_v2.C` resolves to."""
    if request.param == "compiled":
        from infllm_v2 import C as mod
        import infllmv2_cuda_impl_amd._C as ext
        assert mod.varlen_fwd is ext.varlen_fwd
        return mod
    import infllmv2_cuda_impl_amd.C as mod
    return mod


def expand(x, Hk):           # (T, Hq, d) -> (T*16, Hk, d), as infllmv2_sparse_attention.py:88
    T, Hq, d = x.shape
    return x.reshape(T, Hk, 16, d).transpose(1, 2).reshape(T * 16, Hk, d).contiguous()


def collapse(x, Hk):         # inverse, as infllmv2_sparse_attention.py:130
    T16, _, d = x.shape
    return x.reshape(T16 // 16, 16, Hk, d).transpose(1, 2).reshape(T16 // 16, Hk * 16, d).contiguous()


def test_reference_style_forward_backward_through_C(C):
    import infllm_v2
    dev = torch.device("cuda:0")
    sq = [300, 200]
    q, k, v, cu_q, cu_k, idx = make_case(21, sq, sq, 2, 3, dev)
    stream = torch.cuda.current_stream().cuda_stream
    # topk_to_uint64 through raw pointers (topk_to_uint64.py:56-68)
    k_blocks, n64 = (max(sq) + 63) // 64, 1
    words = torch.zeros((2, q.shape[0], n64), dtype=torch.int64, device=dev)
    C.topk_to_uint64(stream, idx.data_ptr(), words.data_ptr(), 2 * q.shape[0], idx.shape[-1], k_blocks, n64)
    ref_words, _ = infllm_v2.topk_to_uint64(idx, max(sq), 64)
    assert torch.equal(words, ref_words)
    # forward (infllmv2_sparse_attention.py:97-130)
    qe = expand(q, 2)
    out_e, lse, p, rng = C.varlen_fwd(qe, k, v, None, cu_q * 16, cu_k, None, None, None, None, max(sq) * 16, max(sq), 0.0,
                                      128 ** -0.5, False, True, -1, -1, 0.0, False, None, words)
    out_ref, lse_ref, _ = infllm_v2.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_k, max(sq), max(sq), causal=True,
                                                            topk_idx=idx, return_attn_probs=True)
    assert torch.equal(collapse(out_e, 2), out_ref) and torch.equal(lse, lse_ref) and p.numel() == 0
    # backward with the transposed mask (infllmv2_sparse_attention.py:344-350, 217-243)
    col_mask = infllm_v2.blockmask_to_uint64(infllm_v2.uint64_to_bool(words, k_blocks).transpose(1, 2).contiguous())[0]
    dout = torch.randn_like(q)
    dq_e, dk, dv = torch.empty_like(qe), torch.empty_like(k), torch.empty_like(v)
    res = C.varlen_bwd(expand(dout, 2), qe, k, v, out_e, lse, dq_e, dk, dv, cu_q * 16, cu_k, None, max(sq) * 16, max(sq),
                       0.0, 128 ** -0.5, False, True, -1, -1, 0.0, False, col_mask, None, rng)
    assert len(res) == 4
    qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
    infllm_v2.infllmv2_attn_varlen_func(qg, kg, vg, cu_q, cu_k, max(sq), max(sq), causal=True, topk_idx=idx).backward(dout)
    assert torch.equal(collapse(dq_e, 2), qg.grad)
    assert (dk.float() - kg.grad.float()).abs().max() <= 0.07 and (dv.float() - vg.grad.float()).abs().max() <= 0.13  # fp32 atomics order


def test_reference_style_stage1_and_pooling_through_C(C):
    import infllm_v2
    dev = torch.device("cuda:0")
    S = 640
    g = torch.Generator(device="cpu").manual_seed(5)
    q = torch.randn(S, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    kf = torch.randn((S - 32) // 16 + 1, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    kc = torch.randn((S - 128) // 64 + 1, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    mk = lambda n: torch.tensor([0, n], dtype=torch.int32, device=dev)
    Lk = kf.shape[0]
    res = C.varlen_fwd_stage1(expand(q, 2), kf, kc, None, mk(S) * 16, mk(Lk), mk(kc.shape[0]), None, None, None, None,
                              S * 16, Lk, 0.0, 128 ** -0.5, True, True, -1, -1, 0.0, True, None)
    p = res[0]
    assert tuple(p.shape) == (2, S, 128) and float(p[:, :, Lk:].abs().max()) == 0.0
    score = infllm_v2.infllmv2_attn_stage1(q, kf, kc, mk(S), mk(Lk), mk(kc.shape[0]), S, Lk, causal=True)
    assert torch.equal(p[:, :, :Lk], score)
    # max_pooling_1d through raw pointers (max_pooling_1d.py:25-41)
    x = score.contiguous()
    out_len = (S + 63) // 64
    pooled = torch.zeros(2, S, out_len, dtype=x.dtype, device=dev)
    C.max_pooling_1d(torch.cuda.current_stream().cuda_stream, x.data_ptr(), pooled.data_ptr(), True, 2, S, Lk, out_len,
                     0, 5, 4, 1, 64, 1, 1)
    assert torch.equal(pooled, infllm_v2.max_pooling_1d(score, 0, 1, 1))
    # varlen variant with its host read-back of total_q
    pooled_v = torch.zeros_like(pooled)
    zeros = torch.zeros(1, dtype=torch.int32, device=dev)
    cu_q_t, cu_k_t = mk(S), mk(Lk)                          # keep the tensors alive: only raw pointers are passed
    C.max_pooling_1d_varlen(torch.cuda.current_stream().cuda_stream, x.data_ptr(), pooled_v.data_ptr(), cu_q_t.data_ptr(),
                            cu_k_t.data_ptr(), zeros.data_ptr(), True, 1, 2, S, Lk, out_len, 5, 4, 1, 64, 1, 1)
    assert torch.equal(pooled_v, pooled)
    # the reference's own top-k binding: values and positions, row stride = next power of two
    val = torch.zeros(2 * S, 16, dtype=x.dtype, device=dev)
    pos = torch.zeros(2 * S, 16, dtype=torch.int32, device=dev)
    C.topk(torch.cuda.current_stream().cuda_stream, 2 * S, out_len, 10, 1, pooled.data_ptr(), val.data_ptr(), pos.data_ptr())
    ref_idx = infllm_v2.topk_blocks(pooled, 10).reshape(2 * S, 10)
    assert torch.equal(pos[:, :10], ref_idx)
    assert torch.equal(val[:, :10], torch.gather(pooled.reshape(2 * S, out_len), 1, ref_idx.long()))
    with pytest.raises(NotImplementedError):
        C.get_probs()


@pytest.mark.parametrize("causal", [True, False])
def test_fixed_length_fwd_bwd_through_C(C, causal):
    """`C.fwd` / `C.bwd` (mha_fwd / mha_bwd, flash_api.cpp:349-517, 1062-1276): dense attention over a
    (batch, seqlen, heads, d) batch.  Checked against the fp64 oracle per sequence; gradients land in the
    caller's tensors, also when those are not viewable as packed rows."""
    from oracle import infllmv2_oracle as O
    from conftest import bf16_np
    dev = torch.device("cuda:0")
    b, sq, sk, Hk = 3, 70, 130, 2
    g = torch.Generator(device="cpu").manual_seed(31)
    mk = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16).to(dev)
    q, k, v, dout = mk(b, sq, 16 * Hk, 128), mk(b, sk, Hk, 128), mk(b, sk, Hk, 128), mk(b, sq, 16 * Hk, 128)
    out, lse, _, _ = C.fwd(q, k, v, None, None, 0.0, 128 ** -0.5, causal, -1, -1, 0.0, False, None)
    assert out.shape == q.shape and lse.shape == (b, 16 * Hk, sq) and lse.dtype == torch.float32
    dq = torch.empty_like(q)
    dk_wide = torch.zeros(b, sk, Hk, 256, dtype=torch.bfloat16, device=dev)
    dk = dk_wide[..., :128]                                     # last-dim contiguous, rows twice as far apart
    dv_t = torch.empty(sk, b, Hk, 128, dtype=torch.bfloat16, device=dev).transpose(0, 1)    # not packable: copied back
    r = C.bwd(dout, q, k, v, out, lse, dq, dk, dv_t, None, 0.0, 128 ** -0.5, causal, -1, -1, 0.0, False, None, None)
    assert r[0] is dq and r[1] is dk and r[2] is dv_t
    cu_q = np.arange(b + 1, dtype=np.int32) * sq
    cu_k = np.arange(b + 1, dtype=np.int32) * sk
    flat = lambda t: bf16_np(t.reshape(-1, t.shape[2], t.shape[3]))
    ref_o, ref_lse = O.stage2_forward(flat(q), flat(k), flat(v), cu_q, cu_k, None, 128 ** -0.5, causal)
    assert np.abs(bf16_np(out).reshape(ref_o.shape).astype(np.float64) - ref_o).max() <= 2e-2
    got_lse = lse.permute(1, 0, 2).reshape(16 * Hk, b * sq).cpu().numpy()
    ref_heads = ref_lse.reshape(Hk, b * sq, 16).transpose(0, 2, 1).reshape(16 * Hk, b * sq)     # column t*16+g -> row 16h+g
    assert np.abs(got_lse - ref_heads).max() <= 1e-3
    rq, rk, rv = O.stage2_backward(flat(q), flat(k), flat(v), flat(dout), cu_q, cu_k, None, 128 ** -0.5, causal)
    for name, got, ref in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv_t, rv)):
        gnp = bf16_np(got.contiguous()).reshape(ref.shape).astype(np.float64)
        s = max(1.0, float(np.abs(ref).max()))
        err = np.abs(gnp - ref)
        assert err.max() <= 2e-2 * s and err.mean() <= 1e-3 * s, (name, err.max(), err.mean())


def test_decode_through_C(C):
    """`C.fwd_kvcache` (mha_fwd_kvcache, flash_api.cpp:1549-1843) as infllmv2_sparse_attention.py:730-760 calls it: packed
    mask words, new keys appended in place, rotary tables.  Equal to the package operator bit for bit (same kernels)."""
    import infllm_v2
    import test_gpu_decode as D
    dev = torch.device("cuda:0")
    lens = [700, 64, 1000, 333]
    q, kc, vc, kn, vn, L, idx = D.make(8, 4, 1024, lens, 5, new=2)
    cos, sin = D.rotary_tables(9, 1024, 32)
    d = lambda t: t.to(dev)
    words, _ = infllm_v2.topk_to_uint64(d(idx), 1024, 64)
    k1, v1, k2, v2 = d(kc).clone(), d(vc).clone(), d(kc).clone(), d(vc).clone()
    out, lse = C.fwd_kvcache(d(q), k1, v1, d(kn), d(vn), d(L), d(cos), d(sin), None, None, None, None, None, 128 ** -0.5,
                             False, -1, -1, 0.0, True, 3, words)
    ref_out, ref_lse = infllm_v2.infllmv2_attn_with_kvcache(d(q), k2, v2, k=d(kn), v=d(vn), rotary_cos=d(cos),
                                                            rotary_sin=d(sin), cache_seqlens=d(L), topk_idx=d(idx),
                                                            num_splits=3, return_softmax_lse=True, rotary_interleaved=True)
    assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse)
    assert torch.equal(k1, k2) and torch.equal(v1, v2) and not torch.equal(k1, d(kc))
    with pytest.raises(RuntimeError, match="does not support alibi"):
        C.fwd_kvcache(d(q), k1, v1, None, None, d(L), None, None, None, None, None, d(L).float(), None, 128 ** -0.5,
                      False, -1, -1, 0.0, True, 0, words)
