#!/usr/bin/env python3
"""Benchmark of the affix-KV reuse hot path on one MI355X.

One "step" = one pass of relocate + RoPE re-rotate + gather over the ragged bf16
batch of 16 LLaDA-8B-shaped requests, all 32 layers (one kernel launch), inputs
resident in HBM.  The same run also times the anchor-recompute varlen attention
(one layer call, reported under "attention") and the reference-style torch CPU
formulation on a bounded sample (reported under "cpu_baseline").

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


def _event_times_ms(fn, steps, torch):
    """Run fn() `steps` times, each bracketed by HIP events on the current stream."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for s, e in zip(starts, stops):
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return [s.elapsed_time(e) for s, e in zip(starts, stops)]


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
    """Reference-style torch CPU path (index_select + x*cos + rot_half(x)*sin) on ONE layer of the workload."""
    from oracle import acache_oracle as O

    torch.set_num_threads(os.cpu_count() or 1)
    k1 = wl["k"][0:1].cpu()
    v1 = wl["v"][0:1].cpu()
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
    bytes_layer = 2 * 2 * wl["T"] * wl["H"] * wl["D"] * 2
    return dict(value=bytes_layer / med / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                sample=f"1 of {wl['layers']} layers of the same batch ({wl['T']} rows), median of {len(times)} runs after 2 warm-ups, {med * 1e3:.0f} ms each")


def attention_bench(torch, device, ops, steps, warmup):
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

    def step():
        return ops.acache_attention(q, kc, vc, cu_q, cu_k, slots)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ms = _event_times_ms(step, steps, torch)
    avg_ms = sum(ms) / len(ms)
    flops = 4 * H * D * sum(a * b for a, b in zip(w["q_lens"], w["kv_lens"]))
    kv_bytes = 2 * sum(w["kv_lens"]) * Hkv * D * 2
    qo_bytes = 2 * total_q * H * D * 2
    tflops = flops / (avg_ms * 1e-3) / 1e12
    return {
        "metric": "anchor-recompute attn TFLOP/s", "value": round(tflops, 1), "unit": "TFLOP/s",
        "ms_per_call": round(avg_ms, 4), "min_ms": round(min(ms), 4),
        "config": {"workload": "configs[3]: batch 16, 32 heads (MHA), D 128, bf16, q = 20% anchors + 32 per request, "
                               "kv = affix + request + 256 (920-1712), slot map over shared affix slots and shuffled private blocks",
                   "total_q": total_q, "total_kv": sum(w["kv_lens"])},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "varlen_attn_kernel<bf16,128>", "algorithmic_flops": flops,
                     "algorithmic_bytes": kv_bytes + qo_bytes,
                     "achieved_GBps": round((kv_bytes + qo_bytes) / (avg_ms * 1e-3) / 1e9, 1)},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=32, help="layers of the relocation workload (32 = LLaDA-8B)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-attention", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only; --gpus N with N > 1 is not supported "
              "(the path shards by request or KV head without communication, see DESIGN.md)", file=sys.stderr)
        sys.exit(2)

    import torch
    from acache_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

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
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
            "kernel": "relocate_kernel<bf16,128>", "avg_launch_ms": round(avg_kernel_ms, 4),
            "algorithmic_bytes": algo_bytes,
        },
    }

    if not args.no_attention:
        result["attention"] = attention_bench(torch, device, ops, steps=args.steps, warmup=args.warmup)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_relocation_baseline(torch, wl)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
