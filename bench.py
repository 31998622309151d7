#!/usr/bin/env python3
"""Benchmark of the InfLLM-V2 sparse-attention hot path on one MI355X.

A step is one end-to-end prefill forward of BASELINE config 2: one sequence of 32768 tokens, bf16,
GQA 32 query / 2 KV heads, d = 128, compressed keys kernel 32 / stride 16 (LSE over kernel 128 /
stride 64), block 64, topk = 64 (1 init + 32 local blocks forced), causal:
Stage-1 scores -> max-pool (one fused launch; --unfused-front-end times the two separate calls) -> top-k ->
mask packing -> Stage-2 block-sparse forward.
Inputs (q, k, v and the caller-side compressed keys) are resident in HBM before the timed region.

`value` = Stage-2 algorithmic sparse FLOPs (4*16*64*128 per selected causal block per token and KV head)
divided by the time of the WHOLE step, in TFLOP/s.  The JSON line also carries the per-stage times, the
Stage-2 forward kernel's own roofline figures (HIP events around the kernel alone, K/V images
prepacked), forward + backward, the other BASELINE configurations as extra keys (config 3: four packed sequences
forward + backward; config 4: 131072 tokens per stage; config 5: batched decode, selection and attention), a measured
device-copy bandwidth and the CPU oracle timed per stage on BASELINE config 1.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA peak (vendor figure, no sparsity)
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E peak
FLOPS_PER_BLOCK = 4 * 16 * 64 * 128

# the Stage-2 forward kernel's HBM traffic cannot be read from inside this process (rocprofv3 --pmc counters); it is
# taken from the tracked summary below, which names the sources it was measured on by their hash
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "stage2_fwd_config2_hbm_traffic.md")
FWD_KERNEL_SOURCES = ["stage2_fwd_hybrid.hip", "stage2_fwd.hip", "stage2_fwd.h", "kv_image.h", "block_walker.h", "common.h"]


def fwd_kernel_source_hash() -> str:
    h = hashlib.sha256()
    for name in FWD_KERNEL_SOURCES:
        with open(os.path.join(ROOT, "infllmv2_cuda_impl_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic_bytes(seqlen: int, topk: int):
    """HBM bytes per launch of the Stage-2 forward kernel from the tracked rocprofv3 summary, or None when the summary
    was measured on other kernel sources or another workload."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None
    fields = dict(re.findall(r"^(kernel_source_hash|traffic_bytes_per_launch|seqlen|topk):\s*(\S+)\s*$", text, re.M))
    if fields.get("kernel_source_hash") != fwd_kernel_source_hash():
        return None
    if fields.get("seqlen") != str(seqlen) or fields.get("topk") != str(topk):
        return None
    try:
        return float(fields["traffic_bytes_per_launch"])
    except (KeyError, ValueError):
        return None


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seqlen", type=int, default=32768)
    ap.add_argument("--topk", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--unfused-front-end", action="store_true",
                    help="time the reference's call sequence (Stage-1 scores, then max_pooling_1d) instead of the fused launch")
    ap.add_argument("--no-stages", action="store_true", help="skip the per-stage and kernel-only timings")
    ap.add_argument("--no-shared-selection", action="store_true",
                    help="skip the extra leg with selections shared inside each query block (keeps a profile of the "
                         "Stage-2 kernel to one workload)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip BASELINE configs 3, 4 and 5 (keeps a profile to the default workload)")
    ap.add_argument("--only-config", type=int, default=0, choices=[0, 3, 4, 5],
                    help="run one of the extra configurations alone (for profiling it) and print its record")
    ap.add_argument("--sharing-stats", action="store_true",
                    help="print how many fetches a tile of 8 / 16 / 32 / 64 consecutive tokens could share on the selections "
                         "of BASELINE configs 2, 3 and 4, and exit")
    ap.add_argument("--print-source-hash", action="store_true",
                    help="print the hash of the Stage-2 forward kernel sources (what a traffic summary must name) and exit")
    return ap.parse_args()


def make_inputs(torch, S, dev, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(S, 32, 128, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(S, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    # caller-side compression (mean over [16j, 16j+32) and [64j, 64j+128)), outside the step
    kf = k.unfold(0, 32, 16).float().mean(-1).to(torch.bfloat16).contiguous()
    kc = k.unfold(0, 128, 64).float().mean(-1).to(torch.bfloat16).contiguous()
    mk = lambda n: torch.tensor([0, n], dtype=torch.int32, device=dev)
    return q, k, v, kf, kc, mk(S), mk(kf.shape[0]), mk(kc.shape[0])


_SLEEP_CYCLES_PER_MS = None


def hold_device(torch, ms):
    """Keep the stream busy for about `ms` milliseconds (a spinning kernel), so that the launches enqueued after it are
    all queued by the time the device gets to them: what is timed behind it is device time, not how fast this process
    can issue launches.  No-op when torch has no spin kernel."""
    global _SLEEP_CYCLES_PER_MS
    sleep = getattr(torch.cuda, "_sleep", None)
    if sleep is None:
        return
    if _SLEEP_CYCLES_PER_MS is None:                           # the spin kernel's clock differs between devices: measure it once
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        sleep(1000)
        torch.cuda.synchronize()
        e0.record()
        sleep(200000)
        e1.record()
        torch.cuda.synchronize()
        _SLEEP_CYCLES_PER_MS = 200000 / max(e0.elapsed_time(e1), 1e-3)
    sleep(int(min(ms, 5.0) * min(_SLEEP_CYCLES_PER_MS, 5e6)))   # bounded whatever the calibration read: at most 5 ms of a 5 GHz clock


def event_ms(torch, fn, iters, warmup=2):
    """Device time per call of fn: HIP events around `iters` back-to-back calls.  Calls shorter than 0.2 ms are timed a
    second time queued behind a short spin (this process cannot issue such launches as fast as the device retires
    them, and the events would bracket the host); longer ones are not, because the near-idle spin lets the clocks drop
    and costs them 2-3 %."""
    def timed(hold):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if hold:
            hold_device(torch, 0.5 + 0.1 * iters)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters
    for _ in range(warmup):
        fn()
    ms = timed(False)
    return min(ms, timed(True)) if ms < 0.2 else ms


def selected_causal_blocks(torch, ops, idx, cu_lens, max_len, dev):
    """Number of (token, KV head, block) triples the Stage-2 kernels work on: set bits of the mask at or below each
    token's own block."""
    words, _ = ops.topk_to_uint64(idx, max_len, 64)
    nblk = (max_len + 63) // 64
    bits = ops.uint64_to_bool(words, nblk)
    total = 0
    start = 0
    for n in cu_lens:
        tok = torch.arange(n, device=dev)
        causal_blk = torch.arange(nblk, device=dev)[None, :] <= (tok // 64)[:, None]
        total += int((bits[:, start:start + n] & causal_blk[None]).sum())
        start += n
    return total


def copy_bandwidth(torch, dev):
    """A plain device copy of 1 GiB (read + write = 2 GiB of traffic): the practical ceiling for the HBM-bound kernels."""
    src = torch.ones(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    ms = event_ms(torch, lambda: dst.copy_(src), 10)
    out = {"gbs": 2 * src.numel() / ms / 1e6, "ms": ms, "what": "torch copy_ of 1 GiB, read + write bytes"}
    del dst
    # what a read-only stream gets: a library reduction over 1 GiB (HBM) and over 184 MiB, the size of the decode
    # step's compressed keys, which the last-level cache partly holds between the timed calls
    f32 = src.view(torch.float32)
    for name, t in (("read_only_1gib_gbs", f32), ("read_only_184mib_gbs", f32[:184 << 18])):
        ms_r = event_ms(torch, t.sum, 10)
        out[name] = t.numel() * 4 / ms_r / 1e6
    out["read_only_what"] = "torch sum over fp32, bytes read"
    return out


def sharing_stats(torch, ops, dev):
    """How many fetches of a selected key block a tile of consecutive tokens could share, on the selections the
    benchmark's own inputs produce (BASELINE configs 2, 3 and 4, real Stage-1 scores): per tile size, selected causal
    (token, block) pairs divided by the distinct blocks the tiles touch - over all pairs, and over the pairs that are
    NOT selected by every token of their tile (what the kernels walk per token)."""
    import numpy as np
    out = {}

    def stats(idx, lens, mx):
        words, _ = ops.topk_to_uint64(idx, mx, 64)
        nblk = (mx + 63) // 64
        bits = ops.uint64_to_bool(words, nblk).bool()
        rec = {}
        for tile in (8, 16, 32, 64):
            picks = distinct = own_picks = own_distinct = 0
            start = 0
            for n in lens:
                full = n // tile * tile
                tok = torch.arange(full, device=dev)
                causal_blk = torch.arange(nblk, device=dev)[None, :] <= (tok // 64)[:, None]
                b = (bits[:, start:start + full] & causal_blk[None]).view(bits.shape[0], full // tile, tile, nblk)
                anyb, allb = b.any(2), b.all(2)
                picks += int(b.sum()); distinct += int(anyb.sum())
                own = b & ~allb[:, :, None, :]
                own_picks += int(own.sum()); own_distinct += int(own.any(2).sum())
                start += n
            rec[str(tile)] = {"pairs_per_distinct_block": picks / max(distinct, 1),
                              "own_pairs_per_distinct_own_block": own_picks / max(own_distinct, 1),
                              "own_share_of_pairs": own_picks / max(picks, 1)}
        return rec

    for S, name in ((32768, "config2_32k"), (131072, "config4_128k")):
        g = torch.Generator(device="cuda").manual_seed(0 if S == 32768 else 4)
        q = torch.randn(S, 32, 128, generator=g, device=dev).to(torch.bfloat16)
        k = torch.randn(S, 2, 128, generator=g, device=dev).to(torch.bfloat16)
        cu = torch.tensor([0, S], dtype=torch.int32, device=dev)
        idx = ops.select_blocks(q, k, cu, cu, S, S, 64, 31, 1)
        out[name] = stats(idx, [S], S)
        del q, k, idx
    rng = np.random.default_rng(1)
    lens = [int(64 * x) for x in rng.integers(64, 385, size=4)]
    T, mx = sum(lens), max(lens)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=dev)
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn(T, 32, 128, generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn(T, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    zeros = torch.zeros(4, dtype=torch.int32, device=dev)
    idx = ops.select_blocks(q, k, cu, cu, mx, mx, 64, 31, 1, cache_lens=zeros, max_cache_len=0)
    out["config3_varlen"] = stats(idx, lens, mx)
    out["what"] = ("selected causal (token, KV head, block) pairs per distinct block of a tile of consecutive tokens; "
                   "'own' = pairs whose block is not selected by every token of the tile")
    return out


def config3_bench(torch, ops, dev):
    """BASELINE config 3: four packed sequences, lengths 64*U[64,384] (seeded), forward + backward, topk 64."""
    import numpy as np
    rng = np.random.default_rng(1)
    lens = [int(64 * x) for x in rng.integers(64, 385, size=4)]
    T, mx = sum(lens), max(lens)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=dev)
    g = torch.Generator(device="cuda").manual_seed(3)
    mkt = lambda h: torch.randn(T, h, 128, generator=g, device=dev).to(torch.bfloat16)
    q, k, v, dout = mkt(32), mkt(2), mkt(2), mkt(32)
    zeros = torch.zeros(4, dtype=torch.int32, device=dev)
    sel = lambda: ops.select_blocks(q, k, cu, cu, mx, mx, 64, 31, 1, cache_lens=zeros, max_cache_len=0)
    idx = sel()
    nsel = selected_causal_blocks(torch, ops, idx, lens, mx, dev)
    flops = FLOPS_PER_BLOCK * nsel
    sel_ms = event_ms(torch, sel, 5)
    fwd_ms = event_ms(torch, lambda: ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, mx, mx, causal=True, topk_idx=idx), 5)
    qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]

    def fwd_bwd():
        ops.infllmv2_attn_varlen_func(qg, kg, vg, cu, cu, mx, mx, causal=True, topk_idx=idx).backward(dout)
        qg.grad = kg.grad = vg.grad = None
    fb_ms = event_ms(torch, fwd_bwd, 3)
    return {"workload": f"BASELINE config 3: 4 packed sequences {lens} = {T} tokens, GQA 32q/2kv, d=128, block 64, topk=64, "
                        "causal; selection (compress + fused Stage-1/pool + top-k) timed apart from Stage 2",
            "tokens": T, "selected_causal_blocks_per_token_head": nsel / (2 * T), "selection_ms": sel_ms,
            "stage2_fwd_ms": fwd_ms, "stage2_fwd_tflops": flops / fwd_ms / 1e9,
            "stage2_fwd_frac_peak": flops / fwd_ms / 1e9 / PEAK_BF16_TFLOPS,
            "stage2_fwd_bwd_ms": fb_ms, "stage2_fwd_bwd_tflops": 3.5 * flops / fb_ms / 1e9,
            "stage2_fwd_bwd_frac_peak": 3.5 * flops / fb_ms / 1e9 / PEAK_BF16_TFLOPS}


def config4_bench(torch, ops, dev):
    """BASELINE config 4: one sequence of 131072 tokens, forward, per stage."""
    S, topk = 131072, 64
    g = torch.Generator(device="cuda").manual_seed(4)
    mkt = lambda h: torch.randn(S, h, 128, generator=g, device=dev).to(torch.bfloat16)
    q, k, v = mkt(32), mkt(2), mkt(2)
    cu = torch.tensor([0, S], dtype=torch.int32, device=dev)
    kf, cu_f = ops.compress_keys(k, cu, S, 32, 16)
    kc, cu_c = ops.compress_keys(k, cu, S, 128, 64)
    Lk, nblk = kf.shape[0], S // 64
    s1 = lambda: ops.infllmv2_attn_stage1_pooled(q, kf, kc, cu, cu_f, cu_c, S, Lk, 31, 1, causal=True)
    pooled = s1()
    idx = ops.topk_blocks(pooled, topk)
    nsel = selected_causal_blocks(torch, ops, idx, [S], S, dev)
    flops = FLOPS_PER_BLOCK * nsel
    s1_flops = 2 * 16 * 128 * 2 * sum(max(0, (t + 1) // 16 - 1) + max(0, (t + 1) // 64 - 1) for t in range(S))
    ms = {
        "compress_keys": event_ms(torch, lambda: (ops.compress_keys(k, cu, S, 32, 16), ops.compress_keys(k, cu, S, 128, 64)), 5),
        "stage1_pooled_fused": event_ms(torch, s1, 3),
        "topk_with_mask": event_ms(torch, lambda: ops.topk_blocks(pooled, topk, return_mask=True), 5),
        "stage2_fwd_op": event_ms(torch, lambda: ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, S, S, causal=True, topk_idx=idx), 3),
    }

    def step():
        p = s1()
        i, m = ops.topk_blocks(p, topk, return_mask=True)
        return ops.infllmv2_attn_varlen_func(q, k, v, cu, cu, S, S, causal=True, topk_idx=i, block_mask=m)
    step_ms = event_ms(torch, step, 3, warmup=1)
    n64 = (nblk + 63) // 64
    return {"workload": f"BASELINE config 4: prefill forward, 1 x {S} tokens, GQA 32q/2kv, d=128, block 64, topk={topk}, "
                        "causal; fused Stage-1/pool + top-k with mask words + Stage-2 fwd",
            "selected_causal_blocks_per_token_head": nsel / (2 * S), "stages_ms": ms, "ms_per_step": step_ms,
            "tflops_whole_step": flops / step_ms / 1e9, "stage2_fwd_tflops": flops / ms["stage2_fwd_op"] / 1e9,
            "stage2_fwd_frac_peak": flops / ms["stage2_fwd_op"] / 1e9 / PEAK_BF16_TFLOPS,
            "stage1_tflops": s1_flops / ms["stage1_pooled_fused"] / 1e9,
            "stage1_frac_peak": s1_flops / ms["stage1_pooled_fused"] / 1e9 / PEAK_BF16_TFLOPS,
            "stage1_topk_share_of_fwd": (ms["stage1_pooled_fused"] + ms["topk_with_mask"]) / step_ms,
            "stages_hbm_gbs": {"topk_with_mask": (2 * S * nblk * 2 + 2 * S * topk * 4 + 2 * S * n64 * 8) / ms["topk_with_mask"] / 1e6}}


def decode_bench(torch, ops, dev):
    """BASELINE config 5: batch 64, one query token per sequence, cache lengths 64*U[256,2048], topk 64 (1 init + 32
    local forced): the selection leg (Stage 1 over each sequence's compressed-key caches, pooled at the sequence's
    position, top-k) and the attention leg (mask packing + split decode kernel), each against the HBM roofline."""
    import numpy as np
    rng = np.random.default_rng(1)
    B, topk = 64, 64
    lens = [int(64 * x) for x in rng.integers(256, 2049, size=B)]      # tokens per sequence, the new one included
    cap = max(lens)
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, 1, 32, 128, generator=g, device=dev).to(torch.bfloat16)
    kc = torch.randn(B, cap, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    vc = torch.randn(B, cap, 2, 128, generator=g, device=dev).to(torch.bfloat16)
    L = torch.tensor(lens, dtype=torch.int32, device=dev)
    pos = (L - 1).contiguous()
    fine = torch.empty(B, cap // 16 + 1, 2, 128, dtype=torch.bfloat16, device=dev)
    coarse = torch.empty(B, cap // 64 + 1, 2, 128, dtype=torch.bfloat16, device=dev)
    fl = ops.compress_keys_cache(kc, L, 32, 16, out=fine)
    cl = ops.compress_keys_cache(kc, L, 128, 64, out=coarse)
    s1 = lambda: ops.infllmv2_attn_stage1_kvcache(q, fine, coarse, fl, cl, pos, 31, 1, max_cache_len=cap - 1, causal=False)
    pooled = s1()
    idx = ops.topk_blocks(pooled, topk).unsqueeze(2)
    s1_ms = event_ms(torch, s1, 20)
    topk_ms = event_ms(torch, lambda: ops.topk_blocks(pooled, topk, return_mask=True, by_index=True), 20)
    append = lambda: ops.compress_keys_cache_pair(kc, L, (32, 16, fine), (128, 64, coarse), old_lens=pos, max_new_rows=1)
    append_ms = event_ms(torch, append, 20)
    s2_ms = event_ms(torch, lambda: ops.infllmv2_attn_with_kvcache(q, kc, vc, cache_seqlens=L, topk_idx=idx), 20)
    _, bm = ops.topk_blocks(pooled, topk, return_mask=True, by_index=True)
    bm = bm.unsqueeze(2)
    s2_mask_ms = event_ms(torch, lambda: ops.infllmv2_attn_with_kvcache(q, kc, vc, cache_seqlens=L, block_mask=bm), 20)

    def step():
        p = s1()
        _, m = ops.topk_blocks(p, topk, return_mask=True, by_index=True)
        return ops.infllmv2_attn_with_kvcache(q, kc, vc, cache_seqlens=L, block_mask=m.unsqueeze(2))
    step_ms = event_ms(torch, step, 20)

    # the same step with the append to both compressed-key caches (one launch) in front, once launched call by call and once as one captured
    # HIP graph (a serving loop replays the graph: the gaps between the step's ten small launches disappear)
    def full_step():
        append()
        return step()
    full_ms = event_ms(torch, full_step, 20)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = full_step()
    torch.cuda.synchronize()
    graph_ms = event_ms(torch, graph.replay, 20)
    graph_ok = bool(torch.equal(captured, full_step()))
    s1_bytes = 2 * 128 * 2 * (int(fl.sum()) + int(cl.sum()))           # Hk * (Lk_b + Lc_b) * d * 2 bytes over the batch
    s2_bytes = B * 2 * 64 * 64 * 128 * 2 * 2 + 2 * B * 32 * 128 * 2
    gbs = lambda b, ms: b / ms / 1e6
    return {"workload": "BASELINE config 5: batch 64, seqlen_q 1, cache lengths 64*U[256,2048], topk 64; Stage 1 over "
                        "per-sequence compressed-key caches + pooling + top-k with mask words, then Stage-2 decode (ms: mask packing + decode from an index list)",
            "ms": s2_ms, "algorithmic_bytes": s2_bytes, "hbm_gbs": gbs(s2_bytes, s2_ms),
            "frac_hbm_peak": gbs(s2_bytes, s2_ms) / PEAK_HBM_GBS,
            "ms_with_block_mask": s2_mask_ms, "hbm_gbs_with_block_mask": gbs(s2_bytes, s2_mask_ms),
            "frac_hbm_peak_with_block_mask": gbs(s2_bytes, s2_mask_ms) / PEAK_HBM_GBS,
            "stage1_ms": s1_ms, "stage1_algorithmic_bytes": s1_bytes, "stage1_hbm_gbs": gbs(s1_bytes, s1_ms),
            "stage1_frac_hbm_peak": gbs(s1_bytes, s1_ms) / PEAK_HBM_GBS,
            "topk_ms": topk_ms, "compressed_key_append_ms": append_ms, "step_ms": step_ms,
            "step_with_append_ms": full_ms, "step_with_append_graph_ms": graph_ms, "graph_equals_eager": graph_ok,
            "step_graph_frac_hbm_peak": gbs(s1_bytes + s2_bytes, graph_ms) / PEAK_HBM_GBS,
            "step_hbm_gbs": gbs(s1_bytes + s2_bytes, step_ms),
            "step_frac_hbm_peak": gbs(s1_bytes + s2_bytes, step_ms) / PEAK_HBM_GBS}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(runs: int = 5):
    """The CPU oracle on BASELINE config 1 (2048 tokens, topk 16, block 0 + 2 local blocks forced), per stage and end
    to end: one warm-up run, then the median of `runs` runs."""
    import numpy as np
    from oracle import infllmv2_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = 1
    S, topk = 2048, 16
    r = np.random.default_rng(0)
    q = O.bf16_round(r.standard_normal((S, 32, 128)).astype(np.float32))
    k = O.bf16_round(r.standard_normal((S, 2, 128)).astype(np.float32))
    v = O.bf16_round(r.standard_normal((S, 2, 128)).astype(np.float32))
    cu = np.array([0, S], np.int32)
    kf, cu_f = O.compress_keys(k, cu, 32, 16)
    kc, cu_c = O.compress_keys(k, cu, 128, 64)
    stage_names = ["stage1", "pool", "topk", "pack_mask", "stage2_fwd"]
    samples = {n: [] for n in stage_names + ["total"]}
    flops = 0
    for run in range(runs + 1):
        t = [time.perf_counter()]
        score = O.stage1_scores(q, kf, kc, cu, cu_f, cu_c, int(cu_f[-1]), 128 ** -0.5, True)
        t.append(time.perf_counter())
        pooled = O.max_pooling_1d_fast(score, 0, 1, 1)
        t.append(time.perf_counter())
        idx = O.topk_blocks(pooled, topk)
        t.append(time.perf_counter())
        words, kb = O.topk_to_uint64(idx, S, 64)
        t.append(time.perf_counter())
        O.stage2_forward(q, k, v, cu, cu, words, 128 ** -0.5, True, dtype=np.float32)
        t.append(time.perf_counter())
        if run == 0:                                           # warm-up: also yields the FLOP count
            bits = O.uint64_to_bool(words, kb)
            causal = np.arange(kb)[None, :] <= (np.arange(S) // 64)[:, None]
            flops = FLOPS_PER_BLOCK * int((bits & causal[None]).sum())
            continue
        for i, n in enumerate(stage_names):
            samples[n].append(t[i + 1] - t[i])
        samples["total"].append(t[-1] - t[0])
    med = {n: sorted(x)[len(x) // 2] for n, x in samples.items()}
    return {"value": flops / med["total"] / 1e12, "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
            "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
            "sample": f"BASELINE config 1 (2048 tokens, 32q/2kv, d=128, topk=16, init 1 + 2 local blocks), whole "
                      f"pipeline in the numpy oracle, 1 warm-up + median of {runs} runs = {med['total']:.2f} s",
            "seconds": med["total"], "stage_seconds": {n: med[n] for n in stage_names}, "runs": runs}


def main():
    args = parse_args()
    if args.print_source_hash:
        print(fwd_kernel_source_hash())
        return
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus must be 1 "
              "(the path shards by KV head or query range with no collective in the kernels; no multi-GPU figure is produced)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    import infllmv2_cuda_impl_amd as ops
    from infllmv2_cuda_impl_amd import _lib

    dev = torch.device("cuda:0")
    if args.sharing_stats:
        print(json.dumps(sharing_stats(torch, ops, dev)))
        return
    if args.only_config:
        fn = {3: config3_bench, 4: config4_bench, 5: decode_bench}[args.only_config]
        print(json.dumps(fn(torch, ops, dev)))
        return
    S, topk = args.seqlen, args.topk
    nblk = (S + 63) // 64
    local_blocks, init_blocks = 31, 1
    q, k, v, kf, kc, cu_q, cu_f, cu_c = make_inputs(torch, S, dev)
    Lk = kf.shape[0]

    def step():
        if args.unfused_front_end:      # the reference's own call sequence
            score = ops.infllmv2_attn_stage1(q, kf, kc, cu_q, cu_f, cu_c, S, Lk, causal=True)
            pooled = ops.max_pooling_1d(score, 0, local_blocks, init_blocks)
        else:                           # same pooled tensor, bit for bit, in one launch
            pooled = ops.infllmv2_attn_stage1_pooled(q, kf, kc, cu_q, cu_f, cu_c, S, Lk, local_blocks, init_blocks,
                                                     causal=True)
        idx, mask = ops.topk_blocks(pooled, topk, return_mask=True)      # the selection launch writes the packed mask too
        return ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_q, S, S, causal=True, topk_idx=idx, block_mask=mask), idx

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, idx = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # algorithmic FLOPs from the mask actually selected
    words, _ = ops.topk_to_uint64(idx, S, 64)
    bits = ops.uint64_to_bool(words, nblk)
    causal_blk = torch.arange(nblk, device=dev)[None, :] <= (torch.arange(S, device=dev) // 64)[:, None]
    nsel = int((bits & causal_blk[None]).sum())
    fwd_flops = FLOPS_PER_BLOCK * nsel
    s1_flops = 2 * 16 * 128 * 2 * sum(max(0, (t + 1) // 16 - 1) + max(0, (t + 1) // 64 - 1) for t in range(S))
    baseline_config = "BASELINE config 2" if (S, topk) == (32768, 64) else \
        ("BASELINE config 4" if (S, topk) == (131072, 64) else "not a BASELINE configuration")

    result = {
        "metric": "sparse_attn_fwd_tflops_32k", "value": fwd_flops / ms_per_step / 1e9, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{baseline_config}: prefill forward, 1 x {S} tokens, GQA 32q/2kv, d=128, "
                               f"kernel 32/stride 16 compressed keys, block 64, topk={topk} "
                               f"({init_blocks} init + {local_blocks + 1} local forced), causal; "
                               + ("Stage-1 + pool" if args.unfused_front_end else "fused Stage-1/pool")
                               + " + top-k with mask words + Stage-2 fwd",
                   "seqlen": S, "topk": topk, "selected_causal_blocks_per_token_head": nsel / (2 * S)},
        "stage2_fwd_algorithmic_flops": fwd_flops, "stage1_algorithmic_flops": s1_flops,
        "frac_bf16_mfma_peak_whole_step": fwd_flops / ms_per_step / 1e9 / PEAK_BF16_TFLOPS,
        "peaks": {"bf16_mfma_tflops": PEAK_BF16_TFLOPS, "hbm_gbs": PEAK_HBM_GBS},
    }

    if not args.no_stages:
        score = ops.infllmv2_attn_stage1(q, kf, kc, cu_q, cu_f, cu_c, S, Lk, causal=True)
        pooled = ops.max_pooling_1d(score, 0, local_blocks, init_blocks)
        stages = {
            "stage1": event_ms(torch, lambda: ops.infllmv2_attn_stage1(q, kf, kc, cu_q, cu_f, cu_c, S, Lk, causal=True), 10),
            "pool": event_ms(torch, lambda: ops.max_pooling_1d(score, 0, local_blocks, init_blocks), 10),
            "stage1_pooled_fused": event_ms(torch, lambda: ops.infllmv2_attn_stage1_pooled(
                q, kf, kc, cu_q, cu_f, cu_c, S, Lk, local_blocks, init_blocks, causal=True), 10),
            "topk": event_ms(torch, lambda: ops.topk_blocks(pooled, topk), 10),
            "topk_with_mask": event_ms(torch, lambda: ops.topk_blocks(pooled, topk, return_mask=True), 10),
            "topk_by_index_with_mask": event_ms(torch, lambda: ops.topk_blocks(pooled, topk, return_mask=True, by_index=True), 10),
            "pack_mask": event_ms(torch, lambda: ops.topk_to_uint64(idx, S, 64), 10),
            "stage2_fwd_op": event_ms(torch, lambda: ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_q, S, S, causal=True, topk_idx=idx,
                                                                               block_mask=words), 10),
            "transpose_mask": event_ms(torch, lambda: ops.transpose_blockmask(words, nblk), 10),
        }
        n64 = words.shape[-1]
        stages_gbs = {
            "pool": (2 * S * Lk * 2 + 2 * S * nblk * 2) / stages["pool"] / 1e6,
            "topk": (2 * S * nblk * 2 + 2 * S * topk * 4) / stages["topk"] / 1e6,
            "topk_with_mask": (2 * S * nblk * 2 + 2 * S * topk * 4 + 2 * S * n64 * 8) / stages["topk_with_mask"] / 1e6,
            "topk_by_index_with_mask": (2 * S * nblk * 2 + 2 * S * topk * 4 + 2 * S * n64 * 8) / stages["topk_by_index_with_mask"] / 1e6,
            "pack_mask": (2 * S * topk * 4 + 2 * S * n64 * 8) / stages["pack_mask"] / 1e6,
            "transpose_mask": (2 * 2 * S * n64 * 8) / stages["transpose_mask"] / 1e6,
        }
        result["stages_ms"] = stages
        result["stages_hbm_gbs"] = stages_gbs
        result["stage1_tflops"] = s1_flops / stages["stage1"] / 1e9
        sel_ms = stages["stage1"] + stages["pool"] + stages["topk"]
        result["stage1_pool_topk_share_of_fwd"] = sel_ms / (sel_ms + stages["pack_mask"] + stages["stage2_fwd_op"])
        sel_ms = stages["stage1_pooled_fused"] + stages["topk_with_mask"]
        result["fused_front_end_share_of_fwd"] = sel_ms / (sel_ms + stages["stage2_fwd_op"])
        del score, pooled

        # the dominant kernel alone: K/V images prepacked, mask packed, HIP events on the launch stream
        out_k = torch.empty_like(q)
        lse = torch.empty((2, S * 16), dtype=torch.float32, device=dev)
        ws = torch.empty(_lib.lib.infllmv2_kv_image_bytes(S, 1, 2), dtype=torch.uint8, device=dev)
        qs = _lib.i64_array([q.stride(0), q.stride(1), 16 * q.stride(1)])
        ks = _lib.i64_array([k.stride(0), k.stride(1)])
        ls = _lib.i64_array([16, 1, S * 16])
        stream = torch.cuda.current_stream(dev).cuda_stream

        def kernel_only(prepacked=1):
            _lib.call("infllmv2_varlen_fwd", stream, q.data_ptr(), k.data_ptr(), v.data_ptr(), out_k.data_ptr(),
                      lse.data_ptr(), cu_q.data_ptr(), cu_q.data_ptr(), words.data_ptr(), ws.data_ptr(), ws.numel(),
                      prepacked, 1, S, S, 32, 2, 128, S, S, qs, ks, ks, qs, ls, n64, 128 ** -0.5, 1)
        kernel_only(0)
        k_ms = event_ms(torch, kernel_only, max(10, args.steps))
        achieved = fwd_flops / k_ms / 1e9
        result["roofline"] = {"bound": "mfma", "kernel": "stage2_fwd_hybrid_kernel<causal>", "achieved": achieved,
                              "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                              "traffic": profiled_traffic_bytes(S, topk), "kernel_ms": k_ms,
                              "kernel_source_hash": fwd_kernel_source_hash()}
        if S % 8 == 0:
            # the K/V gather bound reported beside the MFMA one: a block common to the 8 tokens of a workgroup is
            # fetched once per workgroup, every other selected block once per token, 32 KiB each, and a CU's
            # vector-memory return path moves 64 B/clk (256 CUs, 2.4 GHz peak clock)
            sel = (bits & causal_blk[None]).view(2, S // 8, 8, nblk)
            n_common = int(sel.all(dim=2).sum())
            gather_bytes = 32768 * (n_common + int(sel.sum()) - 8 * n_common)
            peak_l1 = 256 * 64 * 2.4e9 / 1e12
            result["roofline"]["gather"] = {"bound": "l1", "bytes": gather_bytes, "achieved": gather_bytes / k_ms / 1e9,
                                            "peak": peak_l1, "unit": "TB/s", "frac": gather_bytes / k_ms / 1e9 / peak_l1}
        if S % 64 == 0 and not args.no_shared_selection:
            # the same operator when neighbouring tokens agree on their blocks (every token of a 64-token query block
            # takes the selection of the block's first token): the i.i.d. scores of the synthetic input are the worst
            # case for the row-parallel kernels, whose shared-block walk this leg shows
            idx_shared = idx.view(2, S // 64, 64, topk)[:, :, :1].expand(2, S // 64, 64, topk).reshape(2, S, topk).contiguous()
            sh_ms = event_ms(torch, lambda: ops.infllmv2_attn_varlen_func(q, k, v, cu_q, cu_q, S, S, causal=True,
                                                                         topk_idx=idx_shared), 10)
            sh_bits = ops.uint64_to_bool(ops.topk_to_uint64(idx_shared, S, 64)[0], nblk) & causal_blk[None]
            sh_flops = FLOPS_PER_BLOCK * int(sh_bits.sum())
            result["stage2_fwd_block_shared_selection"] = {"ms": sh_ms, "tflops": sh_flops / sh_ms / 1e9,
                                                           "frac_peak": sh_flops / sh_ms / 1e9 / PEAK_BF16_TFLOPS}
        qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
        dout = torch.randn_like(q)

        def fwd_bwd():
            o = ops.infllmv2_attn_varlen_func(qg, kg, vg, cu_q, cu_q, S, S, causal=True, topk_idx=idx)
            o.backward(dout)
            qg.grad = kg.grad = vg.grad = None
        fb_ms = event_ms(torch, fwd_bwd, 5)
        result["stage2_fwd_bwd_ms"] = fb_ms
        result["stage2_bwd_ms"] = fb_ms - stages["stage2_fwd_op"]          # the backward alone (incl. its packing and mask transpose)
        result["stage2_fwd_bwd_tflops"] = 3.5 * fwd_flops / fb_ms / 1e9
        result["stage2_fwd_bwd_frac_peak"] = 3.5 * fwd_flops / fb_ms / 1e9 / PEAK_BF16_TFLOPS
        del qg, kg, vg, dout, out_k, lse, ws

    if not args.no_stages and not args.no_other_configs:
        del q, k, v, kf, kc, out, idx, words, bits
        torch.cuda.empty_cache()
        result["config3_varlen_fwd_bwd"] = config3_bench(torch, ops, dev)
        torch.cuda.empty_cache()
        result["config4_prefill_128k"] = config4_bench(torch, ops, dev)
        torch.cuda.empty_cache()
        result["decode_config5"] = decode_bench(torch, ops, dev)
        torch.cuda.empty_cache()
    if not args.no_stages:
        result["device_copy_bandwidth"] = copy_bandwidth(torch, dev)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
