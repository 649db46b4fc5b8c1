#!/usr/bin/env python3
"""Benchmark of the affix-KV reuse hot path on one MI355X.

One "step" = one pass of relocate + RoPE re-rotate + gather over the ragged bf16
batch of 16 LLaDA-8B-shaped requests, all 32 layers (one kernel launch), inputs
resident in HBM.  The same run also measures, each with its own workload, roofline
and CPU baseline on a bounded sample:
  "attention"              the anchor-recompute varlen attention, one layer call (configs[3]);
  "relocate_fp32"          the fp32 single-request configuration, 32 layers (configs[0]);
  "anchor_select_scatter"  one top-k launch + one 28-layer scatter launch, Dream shape (configs[2]);
  "engine"                 full affix recompute vs anchor ratios 0 / 0.1 / 0.2 / 0.3 / 0.5 / 1.0 on random-init
                           LLaDA-8B-shaped weights, 16 requests x 256 generated tokens (configs[4]); its
                           headline value is the ratio-0.2 run.

Prints ONE JSON line.  `python bench.py --gpus 1 --steps K --warmup W`.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, vendor figure

# HBM bytes per launch of the default workloads.  Not measured by this run: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script (raw counters scaled by what they read for the 1 GiB copy of
# --copy-calibration), each taken at the commit named with it; profiles/*.md hold the summaries and their commands.
# A kernel changed after that commit makes its figure stale: tests/test_traffic_constants.py fails when one of
# the listed sources has a commit after it, and the counters have to be taken again.
MEASURED_TRAFFIC = {
    "relocate_32_layers": {"bytes": 18028.3e6, "commit": "b696828",
                           "sources": ["acache_amd/csrc/relocate.hip", "acache_amd/csrc/common.h"]},
    "relocate_fp32": {"bytes": 1879.1e6, "commit": "b696828",
                      "sources": ["acache_amd/csrc/relocate.hip", "acache_amd/csrc/common.h"]},
    "scatter_28_layers": {"bytes": 332.0e6, "commit": "b696828",
                          "sources": ["acache_amd/csrc/scatter.hip", "acache_amd/csrc/common.h"]},
    "attention": {"bytes": 339.4e6, "commit": "b696828",
                  "sources": ["acache_amd/csrc/attn.hip", "acache_amd/csrc/attn_common.h", "acache_amd/csrc/mma.h",
                              "acache_amd/csrc/common.h", "acache_amd/csrc/attn_plan.hip"]},
}
MEASURED_TRAFFIC_BYTES = {name: entry["bytes"] for name, entry in MEASURED_TRAFFIC.items()}
MEASURED_TRAFFIC_COMMIT = ", ".join(f"{name}: {entry['commit']}" for name, entry in MEASURED_TRAFFIC.items())


def _event_times_ms(fn, steps, torch):
    """Average launch duration in ms: one HIP event pair on the current stream around `steps` back-to-back launches
    (the launches queue up behind each other, so host enqueue time is hidden and the figure is device time)."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return [start.elapsed_time(stop) / steps]


def build_relocation_workload(torch, device, layers):
    from acache_amd.synthetic import ragged_relocation_batch
    from acache_amd.rope import rope_table

    w = ragged_relocation_batch(seed=0)
    H, D, BS = 32, 128, 256
    cos, sin = rope_table(1201, D, 5e5)
    gen = torch.Generator(device=device).manual_seed(0)
    shape = (layers, w["num_blocks"], BS, H, D)
    k = torch.empty(shape, dtype=torch.bfloat16, device=device)
    v = torch.empty(shape, dtype=torch.bfloat16, device=device)
    for l in range(layers):  # fill layer by layer to bound the fp32 temporary
        k[l] = torch.randn(shape[1:], generator=gen, device=device).to(torch.bfloat16)
        v[l] = torch.randn(shape[1:], generator=gen, device=device).to(torch.bfloat16)
    T = w["slot_map"].numel()
    out_k = torch.empty(layers, T, H, D, dtype=torch.bfloat16, device=device)
    out_v = torch.empty_like(out_k)
    return dict(w=w, k=k, v=v, cos=cos.to(device), sin=sin.to(device), slot=w["slot_map"].to(device),
                delta=w["delta"].to(device), out_k=out_k, out_v=out_v, T=T, H=H, D=D, layers=layers)


def cpu_relocation_baseline(torch, wl, budget_s=20.0):
    """Reference-style torch CPU path (index_select + x*cos + rot_half(x)*sin) on a quarter of the workload's layers."""
    from oracle import acache_oracle as O

    torch.set_num_threads(os.cpu_count() or 1)
    n_layers = min(8, wl["layers"])
    k1 = wl["k"][0:n_layers].cpu()
    v1 = wl["v"][0:n_layers].cpu()
    slot, delta = wl["slot"].cpu(), wl["delta"].cpu()
    cos, sin = wl["cos"].cpu(), wl["sin"].cpu()
    times = []
    t_begin = time.perf_counter()
    for i in range(7):
        t0 = time.perf_counter()
        O.relocate_rope_gather(k1, v1, slot, delta, cos, sin)
        dt = time.perf_counter() - t0
        if i >= 2:
            times.append(dt)
        if time.perf_counter() - t_begin > budget_s and len(times) >= 1:
            break
    med = statistics.median(times)
    bytes_sample = n_layers * 2 * 2 * wl["T"] * wl["H"] * wl["D"] * 2
    return dict(value=round(bytes_sample / med / 1e9, 3), unit="GB/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{n_layers} of {wl['layers']} layers of the same batch ({wl['T']} rows), median of {len(times)} runs after 2 warm-ups, {med * 1e3:.0f} ms each")


def cpu_attention_baseline(torch, q, kc, vc, w, budget_s=15.0):
    """Reference-style torch CPU path for the attention call: per request, gather K/V through the slot map and run
    ``F.scaled_dot_product_attention`` over all heads (the formulation of nano-vdllm/model_runner.py:385-399), bf16
    inputs up-cast to fp32.  Timed on the whole call (all requests, all heads)."""
    import torch.nn.functional as F

    torch.set_num_threads(os.cpu_count() or 1)
    H, D = q.shape[1], q.shape[2]
    qc, kf, vf = q.cpu(), kc.cpu().view(-1, kc.shape[-2], D), vc.cpu().view(-1, vc.shape[-2], D)
    cu_q, cu_k, slots = w["cu_q"].tolist(), w["cu_k"].tolist(), w["slot_map"].long()
    sample = list(range(len(w["q_lens"])))

    def run():
        for b in sample:
            sl = slots[cu_k[b]:cu_k[b + 1]]
            qb = qc[cu_q[b]:cu_q[b + 1]].float().transpose(0, 1)
            kb = kf[sl].float().transpose(0, 1)
            vb = vf[sl].float().transpose(0, 1)
            F.scaled_dot_product_attention(qb, kb, vb).transpose(0, 1).to(torch.bfloat16)

    times, t_begin = [], time.perf_counter()
    for i in range(7):
        t0 = time.perf_counter()
        run()
        dt = time.perf_counter() - t0
        if i >= 2:
            times.append(dt)
        if time.perf_counter() - t_begin > budget_s and times:
            break
    med = statistics.median(times)
    flops = 4 * H * D * sum(w["q_lens"][b] * w["kv_lens"][b] for b in sample)
    return dict(value=round(flops / med / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{len(sample)} of {len(w['q_lens'])} requests of the same call, all 32 heads, median of {len(times)} runs after 2 warm-ups, {med * 1e3:.0f} ms each")


def attention_bench(torch, device, ops, steps, warmup, cpu_baseline=False):
    """Anchor-recompute bidirectional varlen attention, one layer call: batch 16, 32 heads (MHA), D = 128, bf16."""
    from acache_amd.synthetic import attention_batch

    w = attention_batch(seed=0)
    H = Hkv = 32
    D, BS = 128, 256
    gen = torch.Generator(device=device).manual_seed(0)
    total_q = int(w["cu_q"][-1])
    q = (torch.randn(total_q, H, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    kc = (torch.randn(w["num_blocks"], BS, Hkv, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    vc = (torch.randn(w["num_blocks"], BS, Hkv, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    cu_q, cu_k, slots = w["cu_q"].to(device), w["cu_k"].to(device), w["slot_map"].to(device)

    # the dispatch plan of these lengths, made on the host once as the engine makes it once per forward pass for
    # all of its layers (`--attention-shapes` times the same call with and without a plan)
    t0 = time.perf_counter()
    plan = ops.attention_plan(w["cu_q"], w["cu_k"], H, Hkv, device)
    plan_host_ms = (time.perf_counter() - t0) * 1e3

    def step():
        return ops.acache_attention(q, kc, vc, cu_q, cu_k, slots, plan=plan)

    # A launch takes about 0.1 ms: a region of 20 launches is 2 ms long and carries the idle time in front of its
    # first launch (about 5 us per launch), and after the CPU legs the chip needs about 270 launches (27 ms) to
    # come back to the clocks it holds under load (regions of 200 launches after an idle period measure 100, 95.2,
    # 95.7, 95.6 us per launch).  The leg therefore times at least 200 launches after at least 300 untimed ones
    # and says so in its line.
    attn_warmup, attn_steps = max(warmup, 300), max(steps, 200)
    for _ in range(attn_warmup):
        step()
    torch.cuda.synchronize()
    ms = _event_times_ms(step, attn_steps, torch)
    avg_ms = sum(ms) / len(ms)
    flops = 4 * H * D * sum(a * b for a, b in zip(w["q_lens"], w["kv_lens"]))
    kv_bytes = 2 * sum(w["kv_lens"]) * Hkv * D * 2
    qo_bytes = 2 * total_q * H * D * 2
    tflops = flops / (avg_ms * 1e-3) / 1e12
    extra = {"cpu_baseline": cpu_attention_baseline(torch, q, kc, vc, w)} if cpu_baseline else {}
    # the same kernel on a batch without raggedness (4 requests x 4096 queries x 4096 keys, distinct rows): what its
    # inner loop reaches when every query tile is full and all units are equal (reported, not used in `frac`)
    ub, un = 4, 4096
    uq = (torch.randn(ub * un, H, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    uk = (torch.randn(ub * un // BS, BS, Hkv, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    uv = (torch.randn(ub * un // BS, BS, Hkv, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    ucu = torch.arange(0, (ub + 1) * un, un, dtype=torch.int32, device=device)
    uslots = torch.arange(ub * un, dtype=torch.int32, device=device)
    for _ in range(3):
        ops.acache_attention(uq, uk, uv, ucu, ucu, uslots)
    torch.cuda.synchronize()
    uni_ms = _event_times_ms(lambda: ops.acache_attention(uq, uk, uv, ucu, ucu, uslots), 7, torch)
    uniform_tflops = 4 * H * D * ub * un * un / (statistics.median(uni_ms) * 1e-3) / 1e12
    del uq, uk, uv
    # what the library GEMM reaches on a large square bf16 product on the same box: the practical matrix-core
    # reference next to the nominal peak (reported, not used in `frac`)
    n = 8192
    ga = torch.randn(n, n, device=device).to(torch.bfloat16)
    gb = torch.randn(n, n, device=device).to(torch.bfloat16)
    for _ in range(3):
        torch.matmul(ga, gb)
    torch.cuda.synchronize()
    gemm_ms = _event_times_ms(lambda: torch.matmul(ga, gb), 10, torch)
    gemm_tflops = 2 * n ** 3 / (sum(gemm_ms) / len(gemm_ms) * 1e-3) / 1e12
    del ga, gb
    return {
        **extra,
        "metric": "anchor-recompute attn TFLOP/s", "value": round(tflops, 1), "unit": "TFLOP/s",
        "ms_per_call": round(avg_ms, 4),
        "plan_host_ms": round(plan_host_ms, 3),
        "launches_timed": attn_steps, "warmup_launches": attn_warmup,
        "config": {"workload": "configs[3]: batch 16, 32 heads (MHA), D 128, bf16, q = 20% anchors + 32 per request, "
                               "kv = affix + request + 256 (920-1712), slot map over shared affix slots and shuffled private "
                               "blocks; units dispatched by a host-made plan of the lengths (made once, outside the timed calls)",
                   "total_q": total_q, "total_kv": sum(w["kv_lens"])},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": MEASURED_TRAFFIC_BYTES["attention"],
                     "kernel": "varlen_attn_unit_kernel<bf16,128,plain>", "algorithmic_flops": flops,
                     "algorithmic_bytes": kv_bytes + qo_bytes,
                     "achieved_GBps": round((kv_bytes + qo_bytes) / (avg_ms * 1e-3) / 1e9, 1),
                     "library_gemm_8192_TFLOPs": round(gemm_tflops, 1),
                     "same_kernel_uniform_4x4096x4096_TFLOPs": round(uniform_tflops, 1)},
    }


def _cpu_median_s(fn, runs=7, warm=2, budget_s=15.0):
    times, t_begin = [], time.perf_counter()
    for i in range(runs):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        if i >= warm:
            times.append(dt)
        if time.perf_counter() - t_begin > budget_s and times:
            break
    return statistics.median(times), len(times)


def relocate_fp32_bench(torch, device, ops, steps, warmup, cpu_baseline=True):
    """configs[0]: one request, fp32, 32 layers x 32 KV heads x 128; a 512-token affix cached at positions 0..511
    moved behind 384 request rows (shift +384, theta 5e5), identity block table, packed [896, 32, 128] per layer.
    Reported twice: the whole packed buffer (384 copied + 512 rotated rows) and the affix rows alone."""
    from acache_amd.rope import rope_table
    from oracle import acache_oracle as O

    L, H, D, A, shift, BS, R = 32, 32, 128, 512, 384, 256, 384
    gen = torch.Generator(device=device).manual_seed(0)
    k = torch.randn(L, 4, BS, H, D, generator=gen, device=device)
    v = torch.randn(L, 4, BS, H, D, generator=gen, device=device)
    cos, sin = rope_table(A + shift, D, 5e5)
    cos, sin = cos.to(device), sin.to(device)
    slot = torch.cat([torch.arange(2 * BS, 2 * BS + R), torch.arange(A)]).to(torch.int32).to(device)
    delta = torch.cat([torch.zeros(R), torch.full((A,), shift)]).to(torch.int32).to(device)
    out_k = torch.empty(L, R + A, H, D, device=device)
    out_v = torch.empty_like(out_k)

    def whole():
        ops.relocate_rope_gather(k, v, slot, delta, cos, sin, out_k=out_k, out_v=out_v)

    def affix_only():
        ops.relocate_rope_gather(k, v, slot[R:], delta[R:], cos, sin, out_k=out_k[:, :A], out_v=out_v[:, :A])

    row = H * D * 4
    res = {}
    for name, fn, rows in (("whole_buffer", whole, R + A), ("affix_only", affix_only, A)):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        ms = _event_times_ms(fn, steps, torch)[0]
        nbytes = 2 * 2 * rows * row * L + 8 * rows
        res[name] = {"rows": rows, "ms_per_launch": round(ms, 4), "algorithmic_bytes": nbytes,
                     "GBps": round(nbytes / ms / 1e6, 1)}
    out = {
        "metric": "affix KV relocate+RoPE GB/s, fp32", "unit": "GB/s", "value": res["whole_buffer"]["GBps"],
        "dtype": "f32",
        "config": {"workload": "configs[0]: 1 request, fp32, 32 layers x 32 KV heads x 128, affix 512 rows shifted by +384 "
                               "behind 384 request rows, 256-token blocks, identity block table, packed [896, 32, 128] per layer"},
        "whole_buffer": res["whole_buffer"], "affix_only": res["affix_only"],
        "roofline": {"bound": "hbm", "achieved": res["whole_buffer"]["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(res["whole_buffer"]["GBps"] / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES["relocate_fp32"], "kernel": "relocate_kernel<f32,128>",
                     "avg_launch_ms": res["whole_buffer"]["ms_per_launch"],
                     "algorithmic_bytes": res["whole_buffer"]["algorithmic_bytes"]},
    }
    if cpu_baseline:
        torch.set_num_threads(os.cpu_count() or 1)
        layers = 2
        ck, cv = k[:layers].cpu(), v[:layers].cpu()
        cslot, cdelta, ccos, csin = slot.cpu(), delta.cpu(), cos.cpu(), sin.cpu()
        med, n = _cpu_median_s(lambda: O.relocate_rope_gather(ck, cv, cslot, cdelta, ccos, csin), budget_s=10.0)
        out["cpu_baseline"] = dict(value=round(2 * 2 * (R + A) * row * layers / med / 1e9, 2), unit="GB/s",
                                   cores=torch.get_num_threads(), kind="port",
                                   sample=f"{layers} of {L} layers of the same request (whole buffer), median of {n} runs after 2 warm-ups, {med * 1e3:.0f} ms each")
    return out


def anchor_select_scatter_bench(torch, device, ops, steps, warmup, cpu_baseline=True):
    """configs[2]: Dream shape (28 layers, 4 KV heads, D 128, bf16), batch 16 with infix placement: one top-k launch
    over the ragged influence scores (anchor ratio 0.2, 5 % injected ties) and one launch that scatters the
    recomputed anchor K/V of all 28 layers back into the paged cache."""
    from acache_amd.synthetic import anchor_batch

    w = anchor_batch(seed=0)
    L, Hkv, D, BS = 28, 4, 128, 256
    n_anchor, n_scores = sum(w["K"]), sum(w["A"])
    gen = torch.Generator(device=device).manual_seed(0)
    # the configuration's slot layout: every request owns ceil((K_b + R_b) / 256) blocks drawn from a shuffled
    # pool, and its anchors go to the first K_b private slots through its block table
    nblk_req = [-(-(k + r) // BS) for k, r in zip(w["K"], w["R"])]
    pool = torch.randperm(sum(nblk_req) + 8, generator=torch.Generator().manual_seed(1))
    slot_list, off = [], 0
    for k_b, n_b in zip(w["K"], nblk_req):
        bt = pool[off:off + n_b]
        off += n_b
        pos = torch.arange(k_b)
        slot_list.append(bt[pos // BS] * BS + pos % BS)
    slots = torch.cat(slot_list).to(torch.int32).to(device)
    nblk = int(pool.max()) + 1
    # Several source / destination sets used in turn: one launch reads and writes 332 MB, which the 256 MB
    # last-level cache in front of HBM would otherwise partly hold from the launch before.
    n_sets = 4
    keys = [torch.randn(L, n_anchor, Hkv, D, generator=gen, device=device).to(torch.bfloat16) for _ in range(n_sets)]
    vals = [torch.randn(L, n_anchor, Hkv, D, generator=gen, device=device).to(torch.bfloat16) for _ in range(n_sets)]
    kcs = [torch.zeros(L, nblk, BS, Hkv, D, dtype=torch.bfloat16, device=device) for _ in range(n_sets)]
    vcs = [torch.zeros_like(kcs[0]) for _ in range(n_sets)]
    key, val = keys[0], vals[0]
    turn = [0]
    scores = torch.cat(w["scores"]).to(device)
    cu_a = torch.tensor([0] + np_cumsum(w["A"]), dtype=torch.int32, device=device)
    cu_k = torch.tensor([0] + np_cumsum(w["K"]), dtype=torch.int32, device=device)
    starts = torch.tensor(w["affix_start"], dtype=torch.int32, device=device)

    def scatter():
        i = turn[0] % n_sets
        turn[0] += 1
        ops.kv_scatter_layers(keys[i], vals[i], kcs[i], vcs[i], slots)

    def topk():
        ops.topk_anchors(scores, cu_a, cu_k, n_anchor, offsets=starts)

    timed = {}
    for name, fn in (("scatter", scatter), ("topk", topk)):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        timed[name] = _event_times_ms(fn, steps, torch)[0]
    scatter_bytes = 2 * 2 * n_anchor * Hkv * D * 2 * L + 4 * n_anchor
    topk_bytes = 4 * n_scores + 8 * n_anchor
    gbps = scatter_bytes / timed["scatter"] / 1e6
    out = {
        "metric": "anchor top-k us; anchor K/V scatter GB/s", "unit": "GB/s", "value": round(gbps, 1), "dtype": "bf16",
        "config": {"workload": f"configs[2]: Dream shape (28 layers, 4 KV heads, D 128, bf16), batch 16, infix placement, "
                               f"{n_scores} fp32 influence scores with 5% ties, anchor ratio 0.2 -> {n_anchor} anchors, "
                               f"their K/V rows of all 28 layers scattered into the first K_b private slots of each request "
                               f"(block tables from a shuffled pool of {nblk} blocks); {n_sets} source / cache sets used in turn "
                               f"({n_sets * scatter_bytes / 1e6:.0f} MB touched before a set repeats)"},
        "topk": {"us_per_launch": round(timed["topk"] * 1e3, 2), "algorithmic_bytes": topk_bytes,
                 "GBps": round(topk_bytes / timed["topk"] / 1e6, 2), "kernel": "topk_kernel",
                 "note": "81 KB of input: a latency-bound launch (16 workgroups), not a bandwidth figure"},
        "scatter": {"us_per_launch": round(timed["scatter"] * 1e3, 2), "algorithmic_bytes": scatter_bytes,
                    "GBps": round(gbps, 1), "kernel": "scatter_kernel<bf16>"},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES["scatter_28_layers"],
                     "kernel": "scatter_kernel<bf16>", "avg_launch_ms": round(timed["scatter"], 5),
                     "algorithmic_bytes": scatter_bytes},
    }
    if cpu_baseline:
        torch.set_num_threads(os.cpu_count() or 1)
        cpu_scores = [t.clone() for t in w["scores"]]
        ck, cv = key[0].cpu(), val[0].cpu()
        ckc = torch.zeros(nblk * BS, Hkv, D, dtype=torch.bfloat16)
        cvc = torch.zeros_like(ckc)
        cslots = slots.cpu().long()

        def cpu_topk():   # the reference's formulation: torch.topk + sort per request (model_runner.py:833-843)
            return [torch.topk(sc, k).indices.sort().values + a0 for sc, k, a0 in zip(cpu_scores, w["K"], w["affix_start"])]

        def cpu_scatter():
            ckc.index_copy_(0, cslots, ck)
            cvc.index_copy_(0, cslots, cv)

        t_topk, n1 = _cpu_median_s(cpu_topk, budget_s=5.0)
        t_scatter, n2 = _cpu_median_s(cpu_scatter, budget_s=5.0)
        out["cpu_baseline"] = dict(
            value=round(2 * 2 * n_anchor * Hkv * D * 2 / t_scatter / 1e9, 2), unit="GB/s", cores=torch.get_num_threads(),
            kind="port", topk_us=round(t_topk * 1e6, 1),
            sample=f"scatter: index_copy_ of K and V for 1 of 28 layers ({n_anchor} rows), median of {n2} runs, "
                   f"{t_scatter * 1e6:.0f} us each; top-k: torch.topk + sort per request on the same scores, "
                   f"median of {n1} runs, {t_topk * 1e6:.0f} us")
    return out


def attention_shape_sweep(torch, device, ops, steps):
    """Uniform-shape runs of the same attention kernel (D = 128, bf16, identity slot map): decode-like shapes are
    bound by streaming K/V once, long-query shapes by the matrix core.  LLaDA heads (32, MHA) and Dream heads
    (28 over 4 KV heads).  Median of per-call HIP event pairs."""
    D = 128
    rows = []
    shapes = [(16, 32, 1400, 32, 32), (16, 32, 2800, 32, 32), (64, 32, 1400, 32, 32), (16, 128, 1400, 32, 32),
              (16, 600, 1400, 32, 32), (4, 4096, 4096, 32, 32), (16, 32, 1400, 28, 4), (16, 232, 1400, 28, 4),
              (16, 600, 1400, 28, 4)]
    for B, q, kv, H, Hkv in shapes:
        S = B * kv
        Q = (torch.randn(B * q, H, D, device=device) / D ** 0.5).to(torch.bfloat16)
        K = (torch.randn(S, 1, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        V = (torch.randn(S, 1, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        cu_q = torch.arange(0, (B + 1) * q, q, dtype=torch.int32, device=device)
        cu_k = torch.arange(0, (B + 1) * kv, kv, dtype=torch.int32, device=device)
        slots = torch.arange(S, dtype=torch.int32, device=device)
        for _ in range(3):
            ops.acache_attention(Q, K, V, cu_q, cu_k, slots)
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in pairs:
            a.record()
            ops.acache_attention(Q, K, V, cu_q, cu_k, slots)
            b.record()
        torch.cuda.synchronize()
        ms = statistics.median(a.elapsed_time(b) for a, b in pairs)
        kv_bytes = 2 * S * Hkv * D * 2
        rows.append({"B": B, "q": q, "kv": kv, "H": H, "H_kv": Hkv, "us": round(ms * 1e3, 1),
                     "TFLOPs": round(4 * H * D * B * q * kv / ms / 1e9, 0), "kv_GBps": round(kv_bytes / ms / 1e6, 0)})
    # Decode shapes as the engine issues them: the non-anchor affix rows of every request are the SAME slots (L2 hits
    # after the first request), only the anchors, the request text and the generation window are private rows.
    shared_rows = []
    for B, q, kv, shared, H, Hkv in ((16, 32, 1400, 1000, 32, 32), (16, 32, 1400, 800, 32, 32), (16, 32, 1400, 1000, 28, 4)):
        S = shared + B * (kv - shared)
        Q = (torch.randn(B * q, H, D, device=device) / D ** 0.5).to(torch.bfloat16)
        K = (torch.randn(S, 1, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        V = (torch.randn(S, 1, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        cu_q = torch.arange(0, (B + 1) * q, q, dtype=torch.int32, device=device)
        cu_k = torch.arange(0, (B + 1) * kv, kv, dtype=torch.int32, device=device)
        common = torch.arange(shared, dtype=torch.int32)
        slots = torch.cat([torch.cat([common, torch.arange(shared + b * (kv - shared), shared + (b + 1) * (kv - shared),
                                                           dtype=torch.int32)]) for b in range(B)]).to(device)
        for _ in range(3):
            ops.acache_attention(Q, K, V, cu_q, cu_k, slots)
        ms = _event_times_ms(lambda: ops.acache_attention(Q, K, V, cu_q, cu_k, slots), steps, torch)[0]
        shared_rows.append({"B": B, "q": q, "kv": kv, "shared_kv": shared, "H": H, "H_kv": Hkv, "us": round(ms * 1e3, 1),
                            "distinct_kv_GBps": round(2 * S * Hkv * D * 2 / ms / 1e6, 0),
                            "streamed_kv_GBps": round(2 * B * kv * Hkv * D * 2 / ms / 1e6, 0)})
    # The three relocation modes on one relocated anchor-recompute shape: batch 16, 232 queries and 1 400 keys per
    # request, a shared affix of 1 000 slots placed 50 + 10 b positions into request b (back-to-back launches).
    from acache_amd.rope import rope_table
    B, H, A, R, q_per = 16, 32, 1000, 400, 232
    S = A + B * R + 64
    K = (torch.randn(S, 1, H, D, device=device) / D ** 0.5).to(torch.bfloat16)
    V = torch.randn(S, 1, H, D, device=device).to(torch.bfloat16)
    Q = (torch.randn(B * q_per, H, D, device=device) / D ** 0.5).to(torch.bfloat16)
    cos, sin = (t.to(device) for t in rope_table(2048, D, 5e5))
    shared = torch.arange(A, dtype=torch.int32)
    private = [torch.arange(A + b * R, A + (b + 1) * R, dtype=torch.int32) for b in range(B)]
    start = [50 + 10 * b for b in range(B)]
    in_place = torch.cat([torch.cat([private[b][:start[b]], shared, private[b][start[b]:]]) for b in range(B)]).to(device)
    shared_first = torch.cat([torch.cat([shared, private[b]]) for b in range(B)]).to(device)
    cu_q = torch.arange(0, (B + 1) * q_per, q_per, dtype=torch.int32, device=device)
    cu_k = torch.arange(0, (B + 1) * (A + R), A + R, dtype=torch.int32, device=device)
    shifts = torch.tensor(start, dtype=torch.int32, device=device)
    shared_lens = torch.full((B,), A, dtype=torch.int32, device=device)
    flops = 4 * H * D * B * q_per * (A + R)
    modes = []
    for name, call in (
            ("plain", lambda: ops.acache_attention(Q, K, V, cu_q, cu_k, in_place)),
            ("key_side", lambda: ops.acache_attention(Q, K, V, cu_q, cu_k, in_place, None, A, None, shifts, cos, sin)),
            ("query_side", lambda: ops.acache_attention(Q, K, V, cu_q, cu_k, shared_first, None, A, shared_lens, shifts,
                                                        cos, sin))):
        for _ in range(3):
            call()
        ms = _event_times_ms(call, steps, torch)[0]
        modes.append({"mode": name, "us": round(ms * 1e3, 1), "TFLOPs": round(flops / ms / 1e9, 0)})
    # The benchmark's anchor-recompute batch (configs[3]) with the units ordered inside the kernel (longest request
    # first) and under a host-made dispatch plan; MHA as the benchmark runs it and with 8 KV heads.
    from acache_amd.synthetic import attention_batch
    w = attention_batch(seed=0)
    plan_rows = []
    for H, Hkv in ((32, 32), (32, 8)):
        Q = (torch.randn(int(w["cu_q"][-1]), H, D, device=device) / D ** 0.5).to(torch.bfloat16)
        K = (torch.randn(w["num_blocks"], 256, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        V = (torch.randn(w["num_blocks"], 256, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        cu_q, cu_k, slots = w["cu_q"].to(device), w["cu_k"].to(device), w["slot_map"].to(device)
        plan = ops.attention_plan(w["cu_q"], w["cu_k"], H, Hkv, device)
        row = {"H": H, "H_kv": Hkv}
        for name, p in (("in_kernel_order_us", None), ("planned_us", plan), ("in_kernel_order_again_us", None),
                        ("planned_again_us", plan)):
            call = lambda: ops.acache_attention(Q, K, V, cu_q, cu_k, slots, plan=p)
            for _ in range(50):
                call()
            row[name] = round(_event_times_ms(call, max(steps, 200), torch)[0] * 1e3, 1)
        plan_rows.append(row)
    # The same comparison on other shapes the engine issues: a block refresh of four requests at anchor ratio 0.2
    # (613 queries, 1 413 keys of which 800 are shared affix rows), a uniform batch, a refinement step.
    def ragged_case(name, q_lens, kv_lens, H, Hkv, shared):
        cu = lambda lens: torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
        cu_q, cu_k = cu(q_lens), cu(kv_lens)
        pieces, nxt = [], shared
        for kv in kv_lens:
            pieces += [torch.arange(shared), nxt + torch.arange(kv - shared)]
            nxt += kv - shared
        slots = torch.cat(pieces).to(torch.int32).to(device)
        nb = (nxt + 255) // 256
        Q = (torch.randn(int(cu_q[-1]), H, D, device=device) / D ** 0.5).to(torch.bfloat16)
        K = (torch.randn(nb, 256, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        V = (torch.randn(nb, 256, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
        dq, dk = cu_q.to(device), cu_k.to(device)
        plan = ops.attention_plan(cu_q, cu_k, H, Hkv, device)
        row = {"shape": name, "H": H, "H_kv": Hkv, "units_per_xcd": plan.shape[0] // 8}
        for key, p in (("in_kernel_order_us", None), ("planned_us", plan), ("in_kernel_order_again_us", None),
                       ("planned_again_us", plan)):
            call = lambda: ops.acache_attention(Q, K, V, dq, dk, slots, plan=p)
            for _ in range(30):
                call()
            row[key] = round(_event_times_ms(call, max(steps, 100), torch)[0] * 1e3, 1)
        return row

    other_rows = [
        ragged_case("block refresh, 4 requests, anchor ratio 0.2", [613, 600, 640, 590], [1413, 1400, 1440, 1390], 32, 32, 800),
        ragged_case("block refresh, 4 requests, full recompute", [1413, 1400, 1440, 1390], [1413, 1400, 1440, 1390], 32, 32, 0),
        ragged_case("uniform 16 x 600 x 1400", [600] * 16, [1400] * 16, 32, 32, 0),
        ragged_case("Dream heads, 16 x 232 x 1400", [232] * 16, [1400] * 16, 28, 4, 1000),
        ragged_case("refinement step, 16 x 32 x 1400", [32] * 16, [1400] * 16, 32, 32, 1000),
    ]
    print(json.dumps({"attention_shape_sweep": rows, "decode_shapes_with_shared_affix_rows": shared_rows,
                      "relocation_modes": modes, "anchor_recompute_batch_dispatch_plan": plan_rows,
                      "dispatch_plan_other_shapes": other_rows}))


def kernel_sweep(torch, device, ops, steps):
    """Every other kernel of the path at the shape its config names, plus a plain device copy as the practical HBM
    reference.  Median of per-call HIP event pairs; bytes are the algorithmic ones."""
    from acache_amd.rope import rope_table
    from acache_amd.synthetic import anchor_batch

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in pairs:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return statistics.median(a.elapsed_time(b) for a, b in pairs) * 1e3  # us

    out = []

    def row(name, us, nbytes, note):
        out.append({"kernel": name, "us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1), "bytes": nbytes, "workload": note})

    src = torch.empty(1 << 32, dtype=torch.uint8, device=device).random_(0, 255)
    dst = torch.empty_like(src)
    row("device copy (torch copy_)", timed(lambda: dst.copy_(src)), 2 * (1 << 32), "4 GiB read + 4 GiB written")
    del src, dst
    # the practical matrix-core reference: what the library GEMM reaches on a large square bf16 product
    n = 8192
    a = torch.randn(n, n, device=device).to(torch.bfloat16)
    b = torch.randn(n, n, device=device).to(torch.bfloat16)
    us = timed(lambda: torch.matmul(a, b))
    out.append({"kernel": "library GEMM (torch.matmul, bf16)", "us": round(us, 1), "TFLOPs": round(2 * n ** 3 / us / 1e6, 1),
                "flops": 2 * n ** 3, "workload": "8192 x 8192 x 8192"})
    del a, b

    # configs[2]: Dream shape (28 layers, 4 KV heads, D 128), anchors of 16 requests
    w = anchor_batch(seed=0)
    L, Hkv, D, BS = 28, 4, 128, 256
    n_anchor = sum(w["K"])
    gen = torch.Generator(device=device).manual_seed(0)
    nblk = sum(-(-k // BS) for k in w["K"]) + 2
    key = torch.randn(L, n_anchor, Hkv, D, generator=gen, device=device).to(torch.bfloat16)
    val = torch.randn(L, n_anchor, Hkv, D, generator=gen, device=device).to(torch.bfloat16)
    kc = torch.zeros(L, nblk, BS, Hkv, D, dtype=torch.bfloat16, device=device)
    vc = torch.zeros_like(kc)
    slots = torch.randperm(nblk * BS, device=device)[:n_anchor].to(torch.int32)
    row("scatter_kernel (all layers, one launch)", timed(lambda: ops.kv_scatter_layers(key, val, kc, vc, slots)),
        2 * 2 * n_anchor * Hkv * D * 2 * L, f"configs[2]: {n_anchor} anchor rows x 28 layers x 4 KV heads x 128, bf16")
    scores = torch.cat(w["scores"]).to(device)
    cu_a = torch.tensor([0] + list(np_cumsum(w["A"])), dtype=torch.int32, device=device)
    cu_k = torch.tensor([0] + list(np_cumsum(w["K"])), dtype=torch.int32, device=device)
    starts = torch.tensor(w["affix_start"], dtype=torch.int32, device=device)
    row("topk_kernel (batch of 16, one launch)", timed(lambda: ops.topk_anchors(scores, cu_a, cu_k, n_anchor, offsets=starts)),
        4 * sum(w["A"]) + 8 * n_anchor, f"configs[2]: {sum(w['A'])} fp32 scores, {n_anchor} indices out")
    # the same two steps in the reference's torch formulation on the host cores (one layer of the scatter)
    import time as _time
    cpu_scores = [t.clone() for t in w["scores"]]
    def cpu_topk():
        return [torch.topk(sc, k).indices.sort().values + a0 for sc, k, a0 in zip(cpu_scores, w["K"], w["affix_start"])]
    ck, cv = key[0].cpu(), val[0].cpu()
    ckc = torch.zeros(nblk * BS, Hkv, D, dtype=torch.bfloat16)
    cvc = torch.zeros_like(ckc)
    cslots = slots.cpu().long()
    def cpu_scatter():
        ckc.index_copy_(0, cslots, ck)
        cvc.index_copy_(0, cslots, cv)
    def cpu_timed(fn, n=7):
        fn(); fn()
        ts = []
        for _ in range(n):
            t0 = _time.perf_counter(); fn(); ts.append(_time.perf_counter() - t0)
        return statistics.median(ts) * 1e6
    us_topk, us_scatter = cpu_timed(cpu_topk), cpu_timed(cpu_scatter)
    out.append({"kernel": "cpu baseline: torch.topk + sort per request", "us": round(us_topk, 1), "cores": torch.get_num_threads(),
                "workload": "configs[2], same scores"})
    out.append({"kernel": "cpu baseline: index_copy_ of K and V, one layer", "us": round(us_scatter, 1),
                "GBps": round(2 * 2 * n_anchor * Hkv * D * 2 / us_scatter / 1e3, 2), "cores": torch.get_num_threads(),
                "workload": f"configs[2], one of 28 layers ({n_anchor} rows)"})
    del key, val, kc, vc

    # the steps on either side of attention, LLaDA-8B shape
    H, D = 32, 128
    cos, sin = rope_table(4096, D, 5e5)
    cos, sin = cos.to(device), sin.to(device)
    for n_tok, what in ((512, "refinement step: 16 x 32 tokens"), (21252, "block refresh: all tokens of 16 requests")):
        q = torch.randn(n_tok, H, D, generator=gen, device=device).to(torch.bfloat16)
        k = torch.randn(n_tok, H, D, generator=gen, device=device).to(torch.bfloat16)
        v = torch.randn(n_tok, H, D, generator=gen, device=device).to(torch.bfloat16)
        pos = torch.randint(0, 4096, (n_tok,), generator=gen, device=device)
        kc = torch.zeros(-(-n_tok // 256) + 1, 256, H, D, dtype=torch.bfloat16, device=device)
        vc = torch.zeros_like(kc)
        sl = torch.randperm(kc.shape[0] * 256, device=device)[:n_tok].to(torch.int32)
        row("rope_scatter_kernel", timed(lambda: ops.rope_qk_scatter(q, k, v, pos, cos, sin, kc, vc, sl)),
            n_tok * H * D * 2 * (3 + 4), f"{what}, 32 heads x 128, bf16 (q, k, v read; q, k, K-slot, V-slot written)")
    # anchor-selection probe of one layer: 16 requests x 256 [MASK] queries against 1 000 shared affix keys
    B, M, A = 16, 256, 1000
    qp = (torch.randn(B * M, H, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    kp = (torch.randn(1024, H, D, generator=gen, device=device) / D ** 0.5).to(torch.bfloat16)
    rows_p = torch.arange(B * M, dtype=torch.int32, device=device)
    cu_p = torch.arange(0, (B + 1) * M, M, dtype=torch.int32, device=device)
    sh_p = torch.randint(1, 256, (B,), generator=gen, device=device).to(torch.int32)
    imp = torch.zeros(B, A, dtype=torch.float32, device=device)
    ws = torch.empty(ops.affix_importance_workspace_bytes(B * M, B, H, H, D, A, True), dtype=torch.uint8, device=device)
    us = timed(lambda: ops.affix_importance(imp, qp, kp, rows_p, cu_p, A, M, None, sh_p, cos, sin, 0, ws))
    flops = 2 * 2 * B * M * A * H * D   # the scores are computed twice (row statistics, then column sums)
    out.append({"kernel": "importance kernels (pack + counter-rotate queries, stats, colsum, reduce)", "us": round(us, 1),
                "TFLOPs": round(flops / us / 1e6, 1), "flops": flops,
                "workload": "one layer: 16 requests x 256 mask queries x 1 000 affix keys, 32 heads x 128, bf16, relocated (shifts 1-255)"})
    logits = torch.randn(512, 126464, generator=gen, device=device).to(torch.bfloat16)
    row("confidence_kernel", timed(lambda: ops.argmax_confidence(logits)), 512 * 126464 * 2,
        "512 rows x 126 464 logits, bf16")
    print(json.dumps({"kernel_sweep": out}))


def np_cumsum(values):
    """Inclusive running sums as a list of Python ints."""
    total, acc = 0, []
    for v in values:
        total += int(v)
        acc.append(total)
    return acc


def cpu_engine_baseline(torch, cfg, rows):
    """Reference-style torch CPU formulation of ONE transformer layer (fp32: RMSNorm, q/k/v projections, rotary,
    ``scaled_dot_product_attention`` over each request's keys, output projection, SwiGLU MLP) on the 512 query
    tokens of one refinement step (16 requests x 32 tokens, 1 400 keys each).  Scaled to an engine rate by the
    layer count and by the query tokens the GPU's ratio-0.2 run pushed through the model."""
    import torch.nn.functional as F

    torch.set_num_threads(os.cpu_count() or 1)
    d, h, m = cfg.d_model, cfg.n_heads, cfg.mlp_hidden_size
    hd = d // h
    g = torch.Generator().manual_seed(0)
    w = {n: torch.randn(o, i, generator=g) * 0.02 for n, (o, i) in
         dict(q=(d, d), k=(d, d), v=(d, d), o=(d, d), gate=(m, d), up=(m, d), down=(d, m)).items()}
    B, Lq, Lk = 16, 32, 1400
    x = torch.randn(B, Lq, d, generator=g)
    kc = torch.randn(B, h, Lk, hd, generator=g)
    vc = torch.randn(B, h, Lk, hd, generator=g)
    cos = torch.randn(Lq, hd, generator=g)
    sin = torch.randn(Lq, hd, generator=g)

    def rot(t):
        t1, t2 = t[..., : hd // 2], t[..., hd // 2:]
        return t * cos + torch.cat([-t2, t1], dim=-1) * sin

    def layer():
        y = F.rms_norm(x, (d,))
        q = rot(F.linear(y, w["q"]).view(B, Lq, h, hd).transpose(1, 2))
        k = rot(F.linear(y, w["k"]).view(B, Lq, h, hd).transpose(1, 2))
        v = F.linear(y, w["v"]).view(B, Lq, h, hd).transpose(1, 2)
        kk = torch.cat([kc[:, :, : Lk - Lq], k], dim=2)
        vv = torch.cat([vc[:, :, : Lk - Lq], v], dim=2)
        a = F.scaled_dot_product_attention(q, kk, vv).transpose(1, 2).reshape(B, Lq, d)
        z = x + F.linear(a, w["o"])
        y2 = F.rms_norm(z, (d,))
        return z + F.linear(F.silu(F.linear(y2, w["gate"])) * F.linear(y2, w["up"]), w["down"])

    med, n = _cpu_median_s(layer, runs=5, warm=1, budget_s=15.0)
    acache = next((r for r in rows if r["mode"] == "acache_0.2"), None) or next(r for r in rows if r["mode"].startswith("acache"))
    tokens = acache["timing"].get("cache_forward_tokens", 0) + acache["timing"].get("decode_forward_tokens", 0)
    est = tokens / (B * Lq) * med * cfg.n_layers
    return dict(value=round(acache["generated_tokens"] / est, 2), unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                sample=f"one of {cfg.n_layers} layers on the 512 query tokens of one refinement step, fp32, median of {n} runs, "
                       f"{med * 1e3:.0f} ms; scaled by {cfg.n_layers} layers and the {tokens} query tokens of the GPU's "
                       f"{acache['mode']} run (an extrapolation: the whole run on the host would take ~{est:.0f} s)")


def engine_bench(torch, device, args, ratios=None, cpu_baseline=False):
    """configs[4]: nano-vdllm-style engine step on random-init LLaDA-8B-shaped weights, anchor-ratio sweep
    against full affix recompute.  Returns the result object (``--engine`` prints it as its own JSON line; the
    default run embeds a two-mode version under "engine")."""
    import numpy as np
    from acache_amd import Config, Sequence
    from acache_amd.llada import LLaDAConfig, LLaDAModelLM
    from acache_amd.model_runner import ModelRunner

    torch.manual_seed(0)
    cfg = LLaDAConfig(n_layers=args.engine_layers)
    with torch.device(device):
        model = LLaDAModelLM(cfg)
    model = model.to(torch.bfloat16).eval()
    rng = np.random.default_rng(0)
    vocab = np.array([t for t in range(cfg.vocab_size) if t != cfg.mask_token_id])
    affix = rng.choice(vocab, args.engine_affix).tolist()
    requests = [rng.choice(vocab, int(rng.integers(64, 257))).tolist() for _ in range(args.engine_batch)]
    gen, block = args.engine_gen, 32

    def prompts():
        if args.engine_placement == "prefix":
            return [Sequence(affix + r, gen_length=gen, block_length=block, cache_block_size=256,
                             mask_id=cfg.mask_token_id, prompt_affix_len=len(affix)) for r in requests]
        out = []
        for r in requests:  # infix: request head, affix, request tail
            cut = len(r) // 2
            out.append(Sequence(r[:cut] + affix + r[cut:], gen_length=gen, block_length=block, cache_block_size=256,
                                mask_id=cfg.mask_token_id, prompt_affix_start=cut, prompt_affix_end=cut + len(affix)))
        return out

    def serve(enable, ratio):
        return Config(hf_config=cfg, mask_id=cfg.mask_token_id, recompute_batch_size=4, max_num_seqs=0,
                      gen_length=gen, block_length=block, threshold=0.9, cache_block_size=256,
                      num_kvcache_blocks=args.engine_kv_blocks, temperature=0.0, enable_acache=enable,
                      anchor_ratio=ratio, profile_timing=True, decode_hip_graph=args.engine_graph,
                      anchor_selection_batch_size=args.engine_probe_batch)

    def prompts_of(gen_length):
        nonlocal gen
        keep, gen = gen, gen_length
        try:
            return prompts()
        finally:
            gen = keep

    # untimed warm-up of both loops (one block each) so that library handles, GEMM heuristics and allocator
    # pools exist before the first timed run; otherwise the first mode measured pays for them
    for enable in (False, True):
        warm_cfg = serve(enable, 0.2)
        warm_cfg.gen_length = block
        warm = ModelRunner(model, warm_cfg)
        (warm.generate_with_acache if enable else warm.generate_with_dual_cache)(prompts_of(block))
        del warm
        torch.cuda.empty_cache()
    print("[engine] warm-up done", file=sys.stderr, flush=True)

    rows = []
    ratios = args.engine_ratios if ratios is None else ratios
    for label, enable, ratio in [("full_recompute", False, 0.0)] + [(f"acache_{r}", True, r) for r in ratios]:
        runner = ModelRunner(model, serve(enable, ratio))
        seqs = prompts()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out, nfe = (runner.generate_with_acache if enable else runner.generate_with_dual_cache)(seqs)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tokens = sum(len(o) for o in out)
        timing = {k: round(v, 4) if isinstance(v, float) else v for k, v in runner.last_timing.items()
                  if isinstance(v, (int, float)) and not k.startswith("kv_cache_")}
        rows.append({"mode": label, "anchor_ratio": ratio, "seconds": round(dt, 3), "generated_tokens": tokens,
                     "tokens_per_s": round(tokens / dt, 1), "nfe": int(nfe), "timing": timing})
        print(f"[engine] {label}: {tokens / dt:.1f} tok/s, nfe {nfe}, {dt:.2f} s", file=sys.stderr, flush=True)
        del runner
        torch.cuda.empty_cache()
    base = rows[0]["tokens_per_s"]
    for r in rows:
        r["speedup_vs_full_recompute"] = round(r["tokens_per_s"] / base, 3)
        # matrix-product work of the forwards (projections, MLP, output head on the kept rows), attention excluded
        tok = r["timing"].get("cache_forward_tokens", 0) + r["timing"].get("decode_forward_tokens", 0)
        kept = (r["timing"].get("cache_forward_nfe", 0) + r["timing"].get("decode_forward_nfe", 0)) * block
        per_token = 2 * cfg.n_layers * (4 * cfg.d_model ** 2 + 3 * cfg.d_model * cfg.mlp_hidden_size)
        r["gemm_flops"] = tok * per_token + kept * 2 * cfg.d_model * cfg.vocab_size
        r["query_tokens"] = tok
    # headline: anchor ratio 0.2 when it was run, else the fastest ACache mode
    best = next((r for r in rows[1:] if abs(r["anchor_ratio"] - 0.2) < 1e-9), None) or max(rows[1:], key=lambda r: r["tokens_per_s"])
    tflops = best["gemm_flops"] / best["seconds"] / 1e12
    result = {
        "metric": "engine generated tokens/s vs full affix recompute", "unit": "tokens/s", "value": best["tokens_per_s"],
        "n_gpus": 1, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"configs[4]: LLaDA-8B shape ({cfg.n_layers} layers, d 4096, 32 heads, vocab 126464), random init, "
                               f"batch {args.engine_batch}, shared affix {args.engine_affix} ({args.engine_placement}) + 64-256 request tokens, "
                               f"gen_length {gen}, block_length 32, threshold 0.9 (random weights: ~1 token per step, worst-case NFE)"},
        "full_recompute_tokens_per_s": base, "speedup_vs_full_recompute": best["speedup_vs_full_recompute"],
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "whole engine loop (library GEMMs at M = 512 dominate)",
                     "note": f"matrix-product flops of all forwards of the {best['mode']} run (attention excluded) over its wall time"},
        "results": rows}
    if cpu_baseline:
        result["cpu_baseline"] = cpu_engine_baseline(torch, cfg, rows)
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=32, help="layers of the relocation workload (32 = LLaDA-8B)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-attention", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the configs[0] and configs[2] legs")
    ap.add_argument("--no-engine", action="store_true", help="skip the configs[4] engine leg (about a minute)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run three plain 1 GiB device copies (known traffic, to scale rocprofv3's FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--attention-shapes", action="store_true", help="only run the attention kernel on a few uniform shapes")
    ap.add_argument("--kernels", action="store_true", help="only time the other kernels of the path and a plain device copy")
    ap.add_argument("--engine", action="store_true", help="run the engine-step sweep (configs[4]) instead")
    ap.add_argument("--engine-graph", action="store_true",
                    help="replay the refinement forward from a captured HIP graph (measured: no gain, the loop is GPU-bound)")
    ap.add_argument("--engine-probe-batch", type=int, default=0,
                    help="requests per anchor-selection probe forward (0 = all admitted requests at once, 1 = the reference's choice)")
    ap.add_argument("--engine-layers", type=int, default=32)
    ap.add_argument("--engine-batch", type=int, default=16)
    ap.add_argument("--engine-affix", type=int, default=1000)
    ap.add_argument("--engine-gen", type=int, default=256)
    ap.add_argument("--engine-kv-blocks", type=int, default=160)
    ap.add_argument("--engine-placement", choices=["prefix", "infix"], default="prefix")
    ap.add_argument("--engine-ratios", type=float, nargs="*", default=[0.0, 0.1, 0.2, 0.3, 0.5, 1.0])
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only; --gpus N with N > 1 is not supported "
              "(the path shards by request or by KV head without communication between GPUs)", file=sys.stderr)
        sys.exit(2)

    import torch
    from acache_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.copy_calibration:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_(0, 255)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": "3 x 1 GiB device-to-device copy_", "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return
    if args.attention_shapes:
        attention_shape_sweep(torch, device, ops, args.steps)
        return
    if args.kernels:
        kernel_sweep(torch, device, ops, args.steps)
        return
    if args.engine:
        print(json.dumps(engine_bench(torch, device, args)))
        return

    wl = build_relocation_workload(torch, device, args.layers)

    def step():
        ops.relocate_rope_gather(wl["k"], wl["v"], wl["slot"], wl["delta"], wl["cos"], wl["sin"],
                                 out_k=wl["out_k"], out_v=wl["out_v"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    kernel_ms = _event_times_ms(step, args.steps, torch)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    payload = 2 * 2 * wl["T"] * wl["H"] * wl["D"] * 2 * args.layers   # K,V x read,write x rows x 8 KiB
    index = 8 * wl["T"]                                                # slot + delta, 4 B each
    algo_bytes = payload + index
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    achieved = algo_bytes / (avg_kernel_ms * 1e-3) / 1e9
    value = algo_bytes / (ms_per_step * 1e-3) / 1e9

    result = {
        "metric": "affix KV relocate+RoPE GB/s (% HBM peak); anchor-recompute attn TFLOP/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: ragged batch of 16, LLaDA-8B shape (32 layers x 32 KV heads x 128), bf16, "
                        "affix 600-1200 + request 64-256 rows per request, 256-token blocks from a shuffled pool, "
                        "per-request shifts in [-1200, 1200]; relocate + RoPE + gather into packed varlen layout",
            "layers": args.layers, "rows": wl["T"], "batch": 16, "seed": 0,
        },
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES["relocate_32_layers"] if args.layers == 32 else None,
            "kernel": "relocate_kernel<bf16,128>", "avg_launch_ms": round(avg_kernel_ms, 4),
            "algorithmic_bytes": algo_bytes,
        },
    }

    if not args.no_attention:
        result["attention"] = attention_bench(torch, device, ops, steps=max(args.steps, 20), warmup=args.warmup,
                                              cpu_baseline=not args.no_cpu_baseline)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_relocation_baseline(torch, wl)
    for name in list(wl):   # the 32-layer caches (18 GB): the legs below bring their own inputs
        if torch.is_tensor(wl[name]):
            del wl[name]
    torch.cuda.empty_cache()

    if not args.no_configs:
        result["relocate_fp32"] = relocate_fp32_bench(torch, device, ops, max(args.steps, 20), args.warmup,
                                                      cpu_baseline=not args.no_cpu_baseline)
        result["anchor_select_scatter"] = anchor_select_scatter_bench(torch, device, ops, max(args.steps, 20), args.warmup,
                                                                      cpu_baseline=not args.no_cpu_baseline)
    if not args.no_engine:
        result["engine"] = engine_bench(torch, device, args, cpu_baseline=not args.no_cpu_baseline)
    result["traffic_measured_at_commit"] = MEASURED_TRAFFIC_COMMIT

    print(json.dumps(result))


if __name__ == "__main__":
    main()
