"""The decode entry point that allocates nothing (infllmv2_fwd_kvcache_static) against infllmv2_fwd_kvcache.

Both are called straight through the C ABI (ctypes) on the same inputs; the two run the same kernels with the same
split count, so outputs and LSE must agree bit for bit.  Two calls in a row share the built-in scratch buffer, the
second on a smaller batch with fewer splits, so stale partials of the first call lie next to the second call's.
The oracle checks the result of the existing entry point to the decode tolerance (max-abs 2e-2, mean-abs 1e-3).
"""
import numpy as np
import pytest
import torch

from oracle import infllmv2_oracle as O
from conftest import bf16_np

pytestmark = pytest.mark.gpu


def _case(seed, B, cap, lens, k_sel, Hk=2):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, 1, 16 * Hk, 128, generator=g).to(torch.bfloat16)
    kc = torch.randn(B, cap, Hk, 128, generator=g).to(torch.bfloat16)
    vc = torch.randn(B, cap, Hk, 128, generator=g).to(torch.bfloat16)
    idx = torch.full((B, Hk, 1, k_sel), -1, dtype=torch.int32)
    for b in range(B):
        nb = (lens[b] + 63) // 64
        for h in range(Hk):
            sel = torch.randperm(nb, generator=g)[:k_sel]
            idx[b, h, 0, :len(sel)] = sel.sort().values.to(torch.int32)
    return q, kc, vc, torch.tensor(lens, dtype=torch.int32), idx


def _call(entry, q, kc, vc, lens, mask, splits, workspace, out=None, lse=None):
    from infllmv2_cuda_impl_amd import _lib
    B, _, Hq, d = q.shape
    Hk, cap = kc.shape[2], kc.shape[1]
    if out is None:
        out = torch.empty_like(q)
        lse = torch.empty((B, Hq, 1), dtype=torch.float32, device=q.device)
    s3 = lambda t: _lib.i64_array([t.stride(0), t.stride(1), t.stride(2)])
    two = lambda t: _lib.i64_array([t.stride(0), t.stride(2)])
    zero3 = _lib.i64_array([0, 0, 0])
    stream = torch.cuda.current_stream(q.device).cuda_stream
    head = [stream, q.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, None, lens.data_ptr(), out.data_ptr(),
            lse.data_ptr(), mask.data_ptr()]
    tail = [B, 1, Hq, Hk, d, cap, 0, two(q), s3(kc), s3(vc), zero3, zero3, two(out), mask.shape[-1], splits,
            float(d ** -0.5), None, None, None, 0, 0, None, None, 0, 1]
    if entry == "infllmv2_fwd_kvcache":
        _lib.call(entry, *head, workspace.data_ptr(), workspace.numel(), *tail)
    else:
        _lib.call(entry, *head, *tail)
    return out, lse


@pytest.mark.parametrize("first,second", [
    (dict(B=8, cap=4096, lens=[4096, 4000, 3000, 2048, 1000, 777, 64, 1], k_sel=16, splits=8),
     dict(B=3, cap=1024, lens=[1000, 513, 64], k_sel=6, splits=3)),
])
def test_static_scratch_decode_equals_workspace_decode(first, second):
    import infllmv2_cuda_impl_amd as ops
    from infllmv2_cuda_impl_amd import _lib
    dev = torch.device("cuda:0")
    for call_no, cfg in enumerate((first, second)):
        print(f"[no-alloc] call {call_no}: {cfg}", flush=True)
        q, kc, vc, lens, idx = _case(10 + call_no, cfg["B"], cfg["cap"], cfg["lens"], cfg["k_sel"])
        qd, kcd, vcd, ld = q.to(dev), kc.to(dev), vc.to(dev), lens.to(dev)
        mask, _ = ops.topk_to_uint64(idx.to(dev), cfg["cap"], 64)
        splits = cfg["splits"]
        ws = torch.empty(_lib.lib.infllmv2_fwd_kvcache_workspace_bytes(cfg["B"], 2, splits), dtype=torch.uint8, device=dev)
        out_ws, lse_ws = _call("infllmv2_fwd_kvcache", qd, kcd, vcd, ld, mask, splits, ws)
        out_st, lse_st = _call("infllmv2_fwd_kvcache_static", qd, kcd, vcd, ld, mask, splits, None)
        torch.cuda.synchronize()
        assert torch.equal(out_st, out_ws) and torch.equal(lse_st, lse_ws)
        # The same call again into the outputs that exist by now, with the driver's own count of free device memory
        # (hipMemGetInfo) read before and after: it sees every allocation on the GPU, also one made inside the
        # library behind torch's allocator.  The first call above has resolved the symbol address already.
        out_st.zero_(); lse_st.zero_()
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info(dev)
        _call("infllmv2_fwd_kvcache_static", qd, kcd, vcd, ld, mask, splits, None, out=out_st, lse=lse_st)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(dev)
        assert free_after == free_before, (free_before, free_after)
        assert torch.equal(out_st, out_ws) and torch.equal(lse_st, lse_ws)
        words = O.topk_to_uint64(idx.numpy(), cfg["cap"], 64)[0]
        ro, rl = O.decode_forward(bf16_np(q), bf16_np(kc), bf16_np(vc), lens.numpy(), words, 128 ** -0.5, None, None)
        err = np.abs(bf16_np(out_st) - ro)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())
        l = lse_st.cpu().numpy().astype(np.float64)
        fin = np.isfinite(rl)
        assert np.array_equal(np.isinf(l), ~fin) and np.abs(l[fin] - rl[fin]).max() <= 2e-3


def test_static_scratch_decode_rejects_oversized_requests():
    from infllmv2_cuda_impl_amd import _lib
    dev = torch.device("cuda:0")
    B, Hk, cap, splits = 1024, 2, 64, 64          # 1024 x 2 x 64 x 16 x 129 x 4 bytes of partials: beyond the buffer
    assert _lib.lib.infllmv2_fwd_kvcache_workspace_bytes(B, Hk, splits) > 32 << 20
    q = torch.zeros(B, 1, 32, 128, dtype=torch.bfloat16, device=dev)
    kc = torch.zeros(B, cap, Hk, 128, dtype=torch.bfloat16, device=dev)
    lens = torch.full((B,), cap, dtype=torch.int32, device=dev)
    mask = torch.ones(B, Hk, 1, 1, dtype=torch.int64, device=dev)
    with pytest.raises(RuntimeError, match="built-in buffer"):
        _call("infllmv2_fwd_kvcache_static", q, kc, kc, lens, mask, splits, None)
