"""Known-answer fixtures of tests/golden (written by tests/golden/make_golden.py from the pinned CPU oracle; the
reference stores no vectors of its own).  CPU: today's oracle still reproduces every stored answer.  GPU: the
HIP path, called through the package, reproduces them — bit for bit where the work is integer or a bf16 copy
(pooling, top-k, masks), within the usual tolerances elsewhere (Stage 1: 2^-7 relative + 2e-3; outputs and
gradients: max-abs 2e-2, mean-abs 1e-3, gradients relative to max(1, max|ref|))."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden as G  # noqa: E402
from oracle import infllmv2_oracle as O  # noqa: E402

PREFILL = ["prefill_two_sequences_hk1.npz", "prefill_one_sequence_hk2.npz"]
DECODE = ["decode_three_sequences_hk1.npz"]


def load(name):
    return np.load(os.path.join(HERE, "golden", name))


def prefill_inputs(z):
    q, k, v, dout, cu = G.prefill_inputs(int(z["seed"][0]), [int(s) for s in z["seqs"]], int(z["params"][0]))
    assert G.crc(q, k, v, dout)[0] == z["input_crc"][0], "numpy's random stream changed: regenerate the fixtures"
    return q, k, v, dout, cu


def decode_inputs(z):
    cap, Hk, topk = [int(x) for x in z["params"]]
    q, kc, vc, idx = G.decode_inputs(int(z["seed"][0]), [int(x) for x in z["cache_seqlens"]], cap, Hk, topk)
    assert G.crc(q, kc, vc, idx)[0] == z["input_crc"][0], "numpy's random stream changed: regenerate the fixtures"
    return q, kc, vc, idx


@pytest.mark.parametrize("name", PREFILL + DECODE)
def test_oracle_reproduces_fixture(name):
    z = load(name)
    fresh = G.CASES[name]()
    assert set(fresh) == set(z.files)
    for key in z.files:
        a, b = z[key], fresh[key]
        assert a.shape == b.shape and a.dtype == b.dtype, key
        if a.dtype.kind == "f":
            assert np.allclose(a.astype(np.float64), b.astype(np.float64), rtol=1e-3, atol=1e-6, equal_nan=True), key
        else:
            assert np.array_equal(a, b), key


def _close(got, ref, max_abs=2e-2, mean_abs=1e-3, relative=False):
    ref = ref.astype(np.float64)
    s = max(1.0, float(np.abs(ref).max())) if relative else 1.0
    err = np.abs(got.astype(np.float64) - ref)
    assert err.max() <= max_abs * s and err.mean() <= mean_abs * s, (err.max(), err.mean(), s)


@pytest.mark.gpu
@pytest.mark.parametrize("name", PREFILL)
def test_hip_path_reproduces_prefill_fixture(name):
    import torch
    import infllmv2_cuda_impl_amd as ops
    from conftest import bf16_np, words_np
    z = load(name)
    q, k, v, dout, cu = prefill_inputs(z)
    Hk, topk, local_blocks, init_blocks = [int(x) for x in z["params"]]
    dev = torch.device("cuda:0")
    t = lambda x: torch.from_numpy(x).to(torch.bfloat16).to(dev)
    ti = lambda x: torch.from_numpy(np.asarray(x, np.int32)).to(dev)
    tq, tk, tv, tdo, tcu = t(q), t(k), t(v), t(dout), ti(cu)
    seqs = [int(s) for s in z["seqs"]]
    # compressed keys
    kf, cu_f = ops.compress_keys(tk, tcu, max(seqs), 32, 16)
    kc, cu_c = ops.compress_keys(tk, tcu, max(seqs), 128, 64)
    nf, nc = int(z["cu_fine"][-1]), int(z["cu_coarse"][-1])
    assert np.array_equal(G.bits(bf16_np(kf[:nf])), z["k_fine"]) and np.array_equal(G.bits(bf16_np(kc[:nc])), z["k_coarse"])
    assert np.array_equal(cu_f.cpu().numpy(), z["cu_fine"]) and np.array_equal(cu_c.cpu().numpy(), z["cu_coarse"])
    # Stage 1
    max_lk = int(np.diff(z["cu_fine"]).max())
    score = ops.infllmv2_attn_stage1(tq, kf, kc, tcu, cu_f, cu_c, max(seqs), max_lk, causal=True)
    ref = G.unbits(z["score"]).astype(np.float64)
    assert np.all(np.abs(bf16_np(score) - ref) <= 2.0 ** -7 * np.abs(ref) + 2e-3)
    # pooling, top-k and the masks are exact functions of their input: feed them the stored tensors
    gscore = torch.from_numpy(G.unbits(z["score"])).to(torch.bfloat16).to(dev)
    cache_lens = torch.zeros(len(seqs), dtype=torch.int32, device=dev)
    pooled = ops.max_pooling_1d_varlen(gscore, tcu, cu_f, cache_lens, max(seqs), max_lk, local_blocks, init_blocks)
    assert np.array_equal(bf16_np(pooled), z["pooled"])
    idx = ops.topk_blocks(pooled, topk)
    assert np.array_equal(idx.cpu().numpy(), z["topk_idx"])
    words, k_blocks = ops.topk_to_uint64(idx, max(seqs), 64)
    assert np.array_equal(words_np(words), z["mask_words"])
    from infllmv2_cuda_impl_amd.masks import transpose_blockmask
    assert np.array_equal(words_np(transpose_blockmask(words, k_blocks)), z["mask_words_transposed"])
    # Stage 2
    qg, kg, vg = [x.clone().requires_grad_(True) for x in (tq, tk, tv)]
    out, lse, _ = ops.infllmv2_attn_varlen_func(qg, kg, vg, tcu, tcu, max(seqs), max(seqs), causal=True,
                                                topk_idx=torch.from_numpy(z["topk_idx"]).to(dev), return_attn_probs=True)
    out.backward(tdo)
    _close(bf16_np(out)[::G.SAMPLE], z["out_sampled"])
    fin = np.isfinite(z["lse"])
    assert np.abs(lse.cpu().numpy()[fin] - z["lse"][fin]).max() <= 2e-3
    _close(bf16_np(qg.grad)[::G.SAMPLE], z["dq_sampled"], relative=True)
    _close(bf16_np(kg.grad), z["dk"], relative=True)
    _close(bf16_np(vg.grad), z["dv"], relative=True)


@pytest.mark.gpu
@pytest.mark.parametrize("name", DECODE)
def test_hip_path_reproduces_decode_fixture(name):
    import torch
    import infllmv2_cuda_impl_amd as ops
    from conftest import bf16_np
    z = load(name)
    q, kc, vc, idx = decode_inputs(z)
    dev = torch.device("cuda:0")
    t = lambda x: torch.from_numpy(x).to(torch.bfloat16).to(dev)
    out, lse = ops.infllmv2_attn_with_kvcache(t(q), t(kc), t(vc), cache_seqlens=torch.from_numpy(z["cache_seqlens"]).to(dev),
                                              topk_idx=torch.from_numpy(idx).to(dev), return_softmax_lse=True)
    _close(bf16_np(out), z["out"])
    assert np.abs(lse.cpu().numpy() - z["lse"]).max() <= 2e-3
