"""The benchmark's output contract: one JSON line with the agreed keys, a roofline object whose fraction is
achieved / peak, a CPU baseline, and a refusal to run on more than one GPU."""
import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stdout + proc.stderr)


@pytest.mark.gpu
def test_default_line_has_the_contract_keys(device):
    # the relocation leg on 4 of 32 layers and the engine leg on a 2-layer model with 4 short requests: same code
    # paths and keys as the default run, a fraction of its time
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--steps", "3", "--warmup", "1", "--layers", "4",
                           "--engine-layers", "2", "--engine-batch", "4", "--engine-gen", "32", "--engine-affix", "300",
                           "--engine-kv-blocks", "24"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1                                            # exactly one line on stdout
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["vs_baseline"] is None
    assert d["unit"] == "GB/s" and d["higher_is_better"] is True and "workload" in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    c = d["cpu_baseline"]
    assert c["kind"] in ("port", "reference") and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    a = d["attention"]
    assert a["roofline"]["bound"] == "mfma" and a["roofline"]["peak"] == 2500.0 and a["value"] > 0
    assert a["cpu_baseline"]["value"] > 0
    for name, bound in (("relocate_fp32", "hbm"), ("anchor_select_scatter", "hbm"), ("engine", "mfma")):
        leg = d[name]
        assert "workload" in leg["config"] and leg["value"] > 0, name
        assert leg["roofline"]["bound"] == bound and abs(leg["roofline"]["frac"] - leg["roofline"]["achieved"] / leg["roofline"]["peak"]) < 1e-3
        assert leg["cpu_baseline"]["value"] > 0 and leg["cpu_baseline"]["sample"], name
    assert d["relocate_fp32"]["affix_only"]["rows"] == 512 and d["relocate_fp32"]["whole_buffer"]["rows"] == 896
    assert d["anchor_select_scatter"]["topk"]["us_per_launch"] > 0
    # the whole anchor-ratio sweep of the engine configuration, against full affix recompute; headline = ratio 0.2
    rows = d["engine"]["results"]
    assert [r["mode"] for r in rows] == ["full_recompute", "acache_0.0", "acache_0.1", "acache_0.2", "acache_0.3",
                                         "acache_0.5", "acache_1.0"]
    assert all(r["tokens_per_s"] > 0 and r["speedup_vs_full_recompute"] > 0 for r in rows)
    assert d["engine"]["value"] == rows[3]["tokens_per_s"] and d["engine"]["speedup_vs_full_recompute"] > 0
    assert "sets used in turn" in d["anchor_select_scatter"]["config"]["workload"]
