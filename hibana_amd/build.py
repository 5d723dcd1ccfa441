"""Compile the HIP kernels into hibana_amd/libhibana_hip.so (gfx950 only). Run as `python -m hibana_amd.build`."""
from __future__ import annotations

import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
SOURCES = sorted((HERE / "csrc").glob("*.hip"))
LIBRARY = HERE / "libhibana_hip.so"
# packed FP32 instructions are switched off for every kernel in this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
NOISE = "is not a recognized feature for this target"  # the host pass does not know the device feature


def _run(cmd: list[str]) -> str:
    run = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(line for line in (run.stdout + run.stderr).splitlines() if NOISE not in line)
    if run.returncode != 0:
        raise RuntimeError(f"hipcc failed ({run.returncode}):\n{log}")
    return log


def build_library(verbose: bool = False) -> Path:
    """Every source to an object of its own (side by side: they share no device symbols), then one link."""
    with tempfile.TemporaryDirectory(prefix="hibana_build_") as tmp:
        objects = [str(Path(tmp) / (src.stem + ".o")) for src in SOURCES]
        with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
            logs = list(pool.map(lambda pair: _run(["hipcc", *FLAGS, "-c", str(pair[0]), "-o", pair[1]]), zip(SOURCES, objects)))
        logs.append(_run(["hipcc", "--offload-arch=gfx950", "-fPIC", "-shared", *objects, "-o", str(LIBRARY)]))
    log = "\n".join(l for l in logs if l.strip())
    if verbose and log:
        print(log)
    return LIBRARY


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
