"""Build libhelix_a2a.so for gfx950 with hipcc.

    python helix-a2a_amd/build.py

Cross-compiles without a GPU. The library is written next to the Python
package (helix_a2a/libhelix_a2a.so) so that it travels with the source tree.
This takes the place of the reference's CUDAExtension build (setup.py:14-43).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
SOURCES = [HERE / "csrc" / "helix_kernels.hip", HERE / "csrc" / "helix_c_api.hip"]
OUTPUT = HERE / "helix_a2a" / "libhelix_a2a.so"

HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    "-Wall",
    "-Wno-unused-command-line-argument",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


TIMELINE_OUTPUT = HERE / "helix_a2a" / "libhelix_a2a_timeline.so"


def build_library(verbose: bool = True, timeline: bool = False) -> Path:
    """The library; with ``timeline`` the measuring variant whose kernels stamp their phases (a file of its own)."""
    output = TIMELINE_OUTPUT if timeline else OUTPUT
    cmd = [find_hipcc(), *HIPCC_FLAGS, *(["-DHELIX_A2A_TIMELINE"] if timeline else []), *map(str, SOURCES), "-o", str(output)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "unknown and unsupported"  # host pass does not know the packed-fp32 feature
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if verbose and log.strip():
        print(log, flush=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}\n{log}")
    return output


PROBE_SOURCE = HERE / "benchmark" / "memory_probe.hip"
PROBE_OUTPUT = HERE / "benchmark" / "libhelix_memory_probe.so"


def build_memory_probe(verbose: bool = True) -> Path:
    """The chunked-copy yardstick of bench.py --probe chunk-copy (measuring equipment, a library of its own)."""
    cmd = [find_hipcc(), *HIPCC_FLAGS, str(PROBE_SOURCE), "-o", str(PROBE_OUTPUT)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}\n{proc.stdout}{proc.stderr}")
    return PROBE_OUTPUT


if __name__ == "__main__":
    if "--probe" in sys.argv[1:]:
        out = build_memory_probe()
    else:
        out = build_library(timeline="--timeline" in sys.argv[1:])
    print(f"built {out}")
    sys.exit(0)
