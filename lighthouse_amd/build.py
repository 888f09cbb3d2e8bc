"""Build liblighthouse_hip.so (gfx950).

Usage: ``python -m lighthouse_amd.build`` or ``lighthouse_amd.build.build_hip()``.
hipcc cross-compiles for gfx950 without a GPU present.  Objects go to ``build/``,
the libraries to ``lighthouse_amd/lib/`` (all git-ignored).
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "lighthouse_amd" / "csrc"
LIB_DIR = ROOT / "lighthouse_amd" / "lib"
LIB_PATH = LIB_DIR / "liblighthouse_hip.so"
PROBE_LIB = LIB_DIR / "liblighthouse_probe.so"  # bench.py's MFMA-rate probe, not part of the product library

HIP_SOURCES = ["runtime.hip", "gemm16.hip", "gemm32.hip", "gemm8.hip", "attention.hip", "rowwise.hip", "api.hip"]

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    # Packed FP32 instructions are kept out of the generated code on purpose.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        sys.stderr.write(proc.stderr)
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}")


def build_hip(verbose: bool = False) -> Path:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_dir = ROOT / "build" / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = obj_dir / (Path(src).stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)
        return str(obj)

    with ThreadPoolExecutor(max_workers=min(8, len(HIP_SOURCES) + 1)) as pool:
        probe = pool.submit(compile_one, "probe.hip")
        objs = list(pool.map(compile_one, HIP_SOURCES))
        probe_obj = probe.result()
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(LIB_PATH)])
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", probe_obj, "-o", str(PROBE_LIB)])
    return LIB_PATH


if __name__ == "__main__":
    print(f"built {build_hip(verbose=True)}")
