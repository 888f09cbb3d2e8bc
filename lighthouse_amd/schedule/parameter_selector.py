"""Matmul schedule parameters for a problem shape: the tuned database first, the cost model otherwise.

The counterpart of lighthouse/schedule/xegpu/xegpu_parameter_selector.py:26-85 (a per-shape JSON
database, `matmul_params.json` there, with the cost model's best configuration as the fallback) for
the kernels of this target: the answer is a workgroup tile (`wg_m`, `wg_n`) or a cut along K
(`split_k`), as entries of a `ScheduleParameters` list that `with_schedule_parameters` (torch
ingress) and the `kernel:` stage of a descriptor understand."""

from __future__ import annotations

from ..tuning.tile_db import DEFAULT_DB_PATH, TileDB
from ..tuning.tune_gemm import candidate_splits, prefilter
from .parameters import ScheduleParameters


class HipParameterSelector:
    def __init__(self, json_file: str | None = None, dtype: str = "bf16"):
        self.dtype = dtype
        self.db = TileDB(str(json_file if json_file is not None else DEFAULT_DB_PATH))

    def get_parameters_dict(self, shape: tuple[int, int, int], transpose_a: bool = False, transpose_b: bool = False,
                            **kwargs) -> dict:
        """{"layer_kind": "matmul", "m", "n", "k", then "wg_m" + "wg_n" or "split_k", "source"}.
        A database entry wins (untransposed operands only: tuned entries assume them); otherwise the
        cost model's cheapest tile; a shape no tile of the direct kernels takes is an error.  A tile
        request switches the library's own cut along K off, so for a shape the library may cut (too
        few tiles for the compute units, a long K) the cost model names no tile and the library
        chooses ("source": "library")."""
        m, n, k = (int(x) for x in shape)
        dtype = kwargs.get("dtype", self.dtype)
        params = {"layer_kind": "matmul", "m": m, "n": n, "k": k, "transpose_a": bool(transpose_a),
                  "transpose_b": bool(transpose_b)}
        tile, split_k = (None, None) if (transpose_a or transpose_b) else self.db.lookup_gemm(dtype, m, n, k)
        if tile is not None or split_k is not None:
            params["source"] = "database"
        else:
            candidates = prefilter(m, n, k, dtype=dtype)
            if not candidates:
                raise ValueError(f"Cost model did not return any valid configurations for matmul {(m, n, k)}.")
            if dtype != "f32" and candidate_splits(m, n, k):
                tile = None
                params["source"] = "library"
            else:
                tile = candidates[0]
                params["source"] = "cost model"
        if tile is not None:
            params["wg_m"], params["wg_n"] = int(tile[0]), int(tile[1])
        if split_k is not None:
            params["split_k"] = int(split_k)
        return params

    def get_parameters(self, shape: tuple[int, int, int], transpose_a: bool = False, transpose_b: bool = False,
                       **kwargs) -> ScheduleParameters:
        return ScheduleParameters([self.get_parameters_dict(shape, transpose_a, transpose_b, **kwargs)])

    def get_parameters_for_layers(self, param_list: list[dict]) -> ScheduleParameters:
        return ScheduleParameters([self.get_parameters_dict(**params) for params in param_list])
