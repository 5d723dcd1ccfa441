"""Compile the HIP kernels into hibana_amd/libhibana_hip.so (gfx950 only). Run as `python -m hibana_amd.build`."""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
SOURCES = sorted((HERE / "csrc").glob("*.hip"))
LIBRARY = HERE / "libhibana_hip.so"
# packed FP32 instructions are switched off for every kernel in this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_library(verbose: bool = False) -> Path:
    cmd = ["hipcc", *FLAGS, *map(str, SOURCES), "-o", str(LIBRARY)]
    run = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"  # the host pass does not know the device feature
    log = "\n".join(line for line in (run.stdout + run.stderr).splitlines() if noise not in line)
    if run.returncode != 0:
        raise RuntimeError(f"hipcc failed ({run.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    return LIBRARY


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
