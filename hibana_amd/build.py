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


def build_library(verbose: bool = False, no_debug_hooks: bool = False, output: Path | None = None) -> Path:
    """Every source to an object of its own (side by side: they share no device symbols), then one link.
    `no_debug_hooks`: a serving build (-DHB_NO_DEBUG_HOOKS) that exports none of hb_tune / hb_debug_*; give it an
    `output` of its own - the tests and the benchmark use the default build."""
    target = Path(output) if output else LIBRARY
    flags = FLAGS + (["-DHB_NO_DEBUG_HOOKS"] if no_debug_hooks else [])
    with tempfile.TemporaryDirectory(prefix="hibana_build_") as tmp:
        objects = [str(Path(tmp) / (src.stem + ".o")) for src in SOURCES]
        with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
            logs = list(pool.map(lambda pair: _run(["hipcc", *flags, "-c", str(pair[0]), "-o", pair[1]]), zip(SOURCES, objects)))
        logs.append(_run(["hipcc", "--offload-arch=gfx950", "-fPIC", "-shared", *objects, "-o", str(target)]))
    log = "\n".join(l for l in logs if l.strip())
    if verbose and log:
        print(log)
    return target


def host_symbols(no_debug_hooks: bool) -> set[str]:
    """The hb_* functions the sources define, from a host-only compile (seconds, no device code): what a build with or
    without -DHB_NO_DEBUG_HOOKS would export."""
    flags = ["--offload-arch=gfx950", "-O0", "-std=c++17", "-fPIC", "--cuda-host-only"] + (["-DHB_NO_DEBUG_HOOKS"] if no_debug_hooks else [])
    names: set[str] = set()
    with tempfile.TemporaryDirectory(prefix="hibana_syms_") as tmp:
        for src in SOURCES:
            obj = str(Path(tmp) / (src.stem + ".o"))
            _run(["hipcc", *flags, "-c", str(src), "-o", obj])
            listing = subprocess.run(["nm", "-g", "--defined-only", obj], capture_output=True, text=True, check=True).stdout
            names |= {line.split()[-1] for line in listing.splitlines() if " T hb_" in line}
    return names


if __name__ == "__main__":
    serving = "--no-debug-hooks" in sys.argv[1:]
    print(build_library(verbose=True, no_debug_hooks=serving, output=HERE / "libhibana_hip_serving.so" if serving else None))
    sys.exit(0)
