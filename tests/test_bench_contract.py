"""bench.py's command-line contract, as far as it can be checked without a GPU."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def run_bench(*args, env=None):
    return subprocess.run([sys.executable, str(ROOT / "bench.py"), *args], capture_output=True, text=True, timeout=300,
                          env=env)


def test_more_than_one_gpu_is_refused_with_a_message():
    """W virtual ranks share one GPU; nothing here uses a second one."""
    for extra in (["--gpus", "2"], ["--gpus", "8", "--steps", "5", "--warmup", "1"]):
        proc = run_bench(*extra)
        assert proc.returncode == 2
        assert "one GPU" in proc.stderr and not proc.stdout.strip()


def test_a_launcher_that_sets_world_size_is_refused_too():
    import os

    env = dict(os.environ, WORLD_SIZE="2", RANK="0", LOCAL_RANK="0")
    proc = run_bench("--gpus", "1", env=env)
    assert proc.returncode == 2 and "one GPU" in proc.stderr


def test_the_committed_traffic_table_is_what_the_bench_line_cites():
    """profiles/traffic.json: every entry names the summary it comes from, that summary exists,
    and the HBM bytes per launch are within 1 % of the algorithmic bytes (no wasted traffic)."""
    table = json.loads((ROOT / "profiles" / "traffic.json").read_text())
    assert table["entries"]
    seen = set()
    for e in table["entries"]:
        assert (ROOT / e["profile"]).exists(), e["profile"]
        key = (e["workload"], e["layout"], e["world_size"], e["kernel"], e.get("unit_shape"))
        assert key not in seen, f"duplicate entry {key}"
        seen.add(key)
        assert 0.99 < e["hbm_bytes_per_launch"] / e["algorithmic_bytes"] < 1.01, key
    assert ("layer", "per-param", 8, "accum", None) in seen
    assert ("model", "per-param", 8, "accum", "embedding") in seen


@pytest.mark.parametrize("flag", ["--help"])
def test_help_lists_the_workloads_and_probes(flag):
    proc = run_bench(flag)
    assert proc.returncode == 0
    for word in ("--workload", "model", "uneven", "--probe", "tiny-items", "--lazy-clear", "--no-graph"):
        assert word in proc.stdout
