"""Tile-parameter database keyed by (dtype, M, N, K): what matmul_params.json is to the XeGPU
schedule (examples/xegpu/matmul.py loads per-shape wg/sg/k tiles from it), here for the one knob
the HIP GEMM exposes, the workgroup tile."""

from __future__ import annotations

import json
import os

_ACTIVE: "TileDB | None" = None


class TileDB:
    def __init__(self, path: str | None = None):
        self.path = path
        self.entries: dict[str, dict] = {}
        if path and os.path.exists(path):
            with open(path) as f:
                self.entries = json.load(f)
            for key, entry in self.entries.items():
                if not (isinstance(entry, dict) and len(entry.get("tile", ())) == 2):
                    raise ValueError(f"{path}: entry '{key}' has no [bm, bn] tile")

    @staticmethod
    def key(dtype: str, M: int, N: int, K: int) -> str:
        return f"{dtype}:{M}x{N}x{K}"

    def lookup(self, dtype: str, M: int, N: int, K: int) -> tuple[int, int] | None:
        entry = self.entries.get(self.key(dtype, M, N, K))
        return tuple(entry["tile"]) if entry else None

    def record(self, dtype: str, M: int, N: int, K: int, tile, time_us: float, tflops: float) -> None:
        self.entries[self.key(dtype, M, N, K)] = {
            "tile": [int(tile[0]), int(tile[1])], "time_us": round(float(time_us), 3), "tflops": round(float(tflops), 2)}

    def save(self, path: str | None = None) -> str:
        path = path or self.path
        if not path:
            raise ValueError("no file name to save the tile database to")
        with open(path, "w") as f:
            json.dump(self.entries, f, indent=2, sort_keys=True)
        self.path = path
        return path


def use_db(db: "TileDB | str | None") -> "TileDB | None":
    """Make `db` (or the file it names) the database `ops.gemm` consults when no tile is given;
    None switches back to the library's own choice."""
    global _ACTIVE
    _ACTIVE = TileDB(db) if isinstance(db, str) else db
    return _ACTIVE


def active_db() -> "TileDB | None":
    return _ACTIVE
