"""Tuned-parameter database keyed by problem: what matmul_params.json is to the XeGPU schedule
(lighthouse/schedule/xegpu/matmul_params.json, read by xegpu_parameter_selector.py:26-85), here for
the knobs the HIP kernels expose: workgroup tile and cut along K of the 16-bit GEMM
(LH_GEMM_TILE_* / LH_GEMM_SPLITK_*), query rows per wave and K/V ring depth of the head-dimension-64
attention kernel (LH_ATTN_ROWS_* / LH_ATTN_STAGES_*).  An entry exists only where a measured
setting beat the library's own choice; `ops.gemm` / `ops.attention` ask the active database when the
caller requests nothing.  The packaged database (gfx950_tuned.json, written by tune_gemm.py on an
MI355X) is active by default."""

from __future__ import annotations

import json
import os
from pathlib import Path

DEFAULT_DB_PATH = Path(__file__).resolve().parent / "gfx950_tuned.json"

_DEFAULT = object()
_ACTIVE: "TileDB | None | object" = _DEFAULT


class TileDB:
    def __init__(self, path: str | None = None):
        self.path = path
        self.entries: dict[str, dict] = {}
        if path and os.path.exists(path):
            with open(path) as f:
                self.entries = json.load(f)
            for key, entry in self.entries.items():
                ok = isinstance(entry, dict) and (
                    (key.startswith("attn:") and ("rows_per_wave" in entry or "stages" in entry))
                    or (not key.startswith("attn:") and (len(entry.get("tile") or ()) == 2 or entry.get("split_k"))))
                if not ok:
                    raise ValueError(f"{path}: entry '{key}' names no parameter (tile / split_k, or rows_per_wave / stages)")

    # ---- GEMM -------------------------------------------------------------------------------
    @staticmethod
    def key(dtype: str, M: int, N: int, K: int) -> str:
        return f"{dtype}:{M}x{N}x{K}"

    def lookup_gemm(self, dtype: str, M: int, N: int, K: int):
        """(tile or None, split_k or None) for this problem."""
        entry = self.entries.get(self.key(dtype, M, N, K))
        if not entry:
            return None, None
        tile = entry.get("tile")
        return (tuple(tile) if tile else None), entry.get("split_k")

    def lookup(self, dtype: str, M: int, N: int, K: int) -> tuple[int, int] | None:
        return self.lookup_gemm(dtype, M, N, K)[0]

    def record(self, dtype: str, M: int, N: int, K: int, tile, time_us: float, tflops: float, split_k=None) -> None:
        entry = {"time_us": round(float(time_us), 3), "tflops": round(float(tflops), 2)}
        if tile:
            entry["tile"] = [int(tile[0]), int(tile[1])]
        if split_k:
            entry["split_k"] = int(split_k)
        self.entries[self.key(dtype, M, N, K)] = entry

    # ---- attention --------------------------------------------------------------------------
    @staticmethod
    def attention_key(dtype: str, BH: int, T: int, d: int, causal: bool) -> str:
        return f"attn:{dtype}:{BH}x{T}x{d}:{'causal' if causal else 'full'}"

    def lookup_attention(self, dtype: str, BH: int, T: int, d: int, causal: bool):
        """(rows_per_wave, stages, kv_split), each None where the entry leaves the choice to the
        library, for this problem (BH = batch x heads)."""
        entry = self.entries.get(self.attention_key(dtype, BH, T, d, causal))
        if not entry:
            return None, None, None
        return entry.get("rows_per_wave"), entry.get("stages"), entry.get("kv_split")

    def record_attention(self, dtype: str, BH: int, T: int, d: int, causal: bool, rows_per_wave, stages, time_us: float,
                         tflops: float, kv_split=None) -> None:
        entry = {"time_us": round(float(time_us), 3), "tflops": round(float(tflops), 2)}
        if rows_per_wave:
            entry["rows_per_wave"] = int(rows_per_wave)
        if stages:
            entry["stages"] = int(stages)
        if kv_split:
            entry["kv_split"] = int(kv_split)
        self.entries[self.attention_key(dtype, BH, T, d, causal)] = entry

    def save(self, path: str | None = None) -> str:
        path = path or self.path
        if not path:
            raise ValueError("no file name to save the tile database to")
        with open(path, "w") as f:
            json.dump(self.entries, f, indent=2, sort_keys=True)
            f.write("\n")
        self.path = path
        return path


def use_db(db: "TileDB | str | None") -> "TileDB | None":
    """Make `db` (or the file it names) the database `ops.gemm` / `ops.attention` consult when the
    caller requests nothing; None switches every lookup off (the library's own choices)."""
    global _ACTIVE
    _ACTIVE = TileDB(db) if isinstance(db, str) else db
    return _ACTIVE


def use_default_db() -> "TileDB | None":
    """Back to the packaged database."""
    global _ACTIVE
    _ACTIVE = _DEFAULT
    return active_db()


def active_db() -> "TileDB | None":
    global _ACTIVE
    if _ACTIVE is _DEFAULT:
        _ACTIVE = TileDB(str(DEFAULT_DB_PATH)) if DEFAULT_DB_PATH.is_file() else None
    return _ACTIVE
