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


def test_config_0_carries_the_cpu_leg_and_its_parity():
    """The reference's own CPU-runnable case: the C oracle's dense product timed beside the GPU's, and the two results
    held against each other (scale-relative 2e-2, norm-relative 4e-3)."""
    line = run("--config", "0", "--steps", "12", "--warmup", "2")
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "tokens/s" and cpu["value"] > 0 and cpu["cores"] >= 1 and "whole calls" in cpu["sample"]
    assert line["parity"]["max_rel_vs_cpu_oracle"] < 2e-2 and line["parity"]["norm_rel_vs_cpu_oracle"] < 4e-3


def test_headline_modes():
    line = run("--no-cpu", "--headline-only", "--layers", "2", "--steps", "24", "--warmup", "4", "--copy-mib", "64")
    assert "w3_fc12_kernel" in line["roofline"]["kernel"] and line["cpu_baseline"] is None and line["m1"]["value"] > 0
    roof = line["roofline"]  # the two yardsticks of the same run: a plain read, and the stream's requests without its arithmetic
    assert roof["achieved"] < roof["skeleton"] < roof["peak_measured"] < roof["peak"]
    assert line["config"]["workload"].startswith("BASELINE config 3") and line["vs_baseline"] is None and line["dtype"] == "bf16"
    line = run("--e4m3", "--headline-only", "--layers", "2", "--steps", "24", "--warmup", "4")
    assert "E4M3" in line["metric"] and line["value"] > 0


def test_prefill_layer_and_its_small_calls():
    line = run("--config", "4", "--no-cpu", "--steps", "10", "--warmup", "2")
    assert line["roofline"]["bound"] == "mfma" and line["roofline"]["peak"] == 2500.0 and 0 < line["roofline"]["frac"] < 1
    assert "tile_kernel<TileNvfp4" in line["roofline"]["kernel"] and line["unit"] == "tokens/s"
    line = run("--config", "4", "--small-rows", "4", "--steps", "8", "--warmup", "2")
    assert line["rows"] == 4 and line["us_per_call"] > 0


def test_routing_mode():
    line = run("--routing", "16", "--steps", "12")
    assert line["by_rows"]["16"]["route_topk_us"] > 0 and line["by_rows"]["16"]["route_budget_us"] > 0


def test_more_than_one_gpu_is_refused():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120, cwd=ROOT)
    assert done.returncode != 0 and "one gpu" in (done.stdout + done.stderr).lower()
