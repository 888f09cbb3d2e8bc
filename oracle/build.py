"""Build the C restatement of the reference's loop nests (test infrastructure, like the rest of
this directory): ``python -m oracle.build`` or ``oracle.build.build()``.  The library goes to
``oracle/_build/libcpu_ref.so`` (git-ignored).  Only the tests, ``__graft_entry__`` and
``bench.py``'s CPU baseline call this; nothing under ``lighthouse_amd/`` does."""

from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "_build" / "libcpu_ref.so"


def build(verbose: bool = False) -> Path:
    LIB_PATH.parent.mkdir(parents=True, exist_ok=True)
    cmd = [
        os.environ.get("CC", "gcc"), "-O3", "-march=x86-64-v3", "-ffp-contract=off", "-fopenmp", "-shared", "-fPIC",
        str(HERE / "cpu_ref.c"), "-o", str(LIB_PATH), "-lm",
    ]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        sys.stderr.write(proc.stderr)
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}")
    return LIB_PATH


if __name__ == "__main__":
    print(f"built {build(verbose=True)}")
