"""bench.py's modes as child processes on the device: the JSON line of a short run carries the fields the contract asks
for, and the measurement aids (back-to-back launches, the copy probe) run."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


def run_bench(*args, timeout=300):
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), *args], capture_output=True, text=True, timeout=timeout, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    return json.loads(r.stdout.strip().splitlines()[-1])


def test_short_run_prints_the_contract_line():
    d = run_bench("--workload", "decode_small", "--steps", "5", "--warmup", "2", "--no-configs", "--cpu-seqs", "2")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["unit"] == "tokens/s" and d["vs_baseline"] is None
    assert d["config"]["workload"] == "decode_small" and "model" not in d["config"]
    roof = d["roofline"]
    assert roof["bound"] in ("hbm", "mfma") and roof["peak"] in (8000.0, 2500.0) and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9
    assert d["cpu_baseline"]["kind"] == "port" and d["cpu_baseline"]["cores"] >= 1 and d["cpu_baseline"]["value"] > 0
    assert d["parity"]["ok"]


def test_other_operations_and_cache_dtypes():
    for extra in (("--op", "rpa_v3"), ("--op", "rpa_v3", "--cache-dtype", "fp8"), ("--op", "page_attention"),
                  ("--op", "ragged_decode", "--sinks", "3", "--window", "64")):
        d = run_bench("--workload", "decode_small", "--steps", "3", "--warmup", "1", "--no-configs", "--no-cpu-baseline", *extra)
        assert d["value"] > 0 and d.get("parity", {}).get("ok", True), extra


def test_measurement_aids():
    d = run_bench("--workload", "decode_small", "--sustain", "0.2")
    assert d["launches"] >= 50 and d["ms_per_launch"] > 0
    d = run_bench("--copy-probe", "64", "--steps", "3")
    assert d["copy_probe_bytes_read"] == 64 << 20
