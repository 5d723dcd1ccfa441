"""Every mode of bench.py prints one JSON line with the fields its readers take (short runs: two layers, a dozen steps)."""
import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
pytestmark = pytest.mark.gpu


def run(*flags: str) -> dict:
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), *flags], capture_output=True, text=True, timeout=280, cwd=ROOT)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [line for line in done.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1, done.stdout[-2000:]
    return json.loads(lines[0])


@pytest.mark.parametrize("flags, kernel", [
    (("--config", "2", "--no-cpu", "--layers", "2", "--steps", "12", "--warmup", "2"), "w3_fc1_route_one_kernel"),
    (("--config", "2", "--e4m3", "--layers", "2", "--steps", "12", "--warmup", "2"), "w3_stream_kernel"),
    (("--config", "0", "--no-cpu", "--steps", "12", "--warmup", "2"), "w3_stream_kernel"),
    (("--config", "1", "--no-cpu", "--steps", "12", "--warmup", "2"), "nvfp4_stream_kernel"),
])
def test_decode_modes(flags, kernel):
    line = run(*flags)
    assert line["n_gpus"] == 1 and line["value"] > 0 and line["unit"] == "tokens/s" and line["higher_is_better"] is True
    roof = line["roofline"]
    assert kernel in roof["kernel"] and roof["bound"] == "hbm" and roof["peak"] == 8000.0
    assert 0 < roof["frac"] < 1 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9


def test_routing_mode():
    line = run("--routing", "16", "--steps", "12")
    assert line["by_rows"]["16"]["route_topk_us"] > 0 and line["by_rows"]["16"]["route_budget_us"] > 0


def test_more_than_one_gpu_is_refused():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120, cwd=ROOT)
    assert done.returncode != 0 and "one gpu" in (done.stdout + done.stderr).lower()
