"""The HBM traffic figures that bench.py quotes were measured with rocprofv3 at a named commit.  A source of the
measured kernel that changed after that commit makes the figure stale: this test fails until the counters are taken
again and the commit in bench.py is updated.  Skipped where the history is not available."""
import importlib.util
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def _bench_module():
    spec = importlib.util.spec_from_file_location("bench_for_traffic_test", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _git(*args):
    return subprocess.run(["git", "-C", str(ROOT), *args], capture_output=True, text=True)


def test_traffic_table_is_well_formed():
    table = _bench_module().MEASURED_TRAFFIC
    assert set(table) == {"relocate_32_layers", "relocate_fp32", "scatter_28_layers", "attention"}
    for name, entry in table.items():
        assert entry["bytes"] > 0 and entry["commit"], name
        for src in entry["sources"]:
            assert (ROOT / src).is_file(), f"{name}: {src} does not exist"


def test_measured_kernels_unchanged_since_their_commit():
    if shutil.which("git") is None or _git("rev-parse", "--git-dir").returncode != 0:
        pytest.skip("no git history here")
    stale = []
    for name, entry in _bench_module().MEASURED_TRAFFIC.items():
        if _git("cat-file", "-e", entry["commit"] + "^{commit}").returncode != 0:
            pytest.skip(f"commit {entry['commit']} is not in this clone")
        log = _git("log", "--oneline", f"{entry['commit']}..HEAD", "--", *entry["sources"])
        assert log.returncode == 0, log.stderr
        if log.stdout.strip():
            stale.append(f"{name} (measured at {entry['commit']}): " + "; ".join(log.stdout.strip().splitlines()))
    assert not stale, "traffic figures in bench.py are older than their kernels:\n" + "\n".join(stale)
