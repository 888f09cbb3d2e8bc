"""Tile search for the 16-bit GEMM: enumerate the tiles that fit a shape, drop the ones a cost
model already rules out, time the rest in child processes, log every trial and keep the winner.

The structure follows the reference's tuner for the XeGPU matmul: candidate generation and the
roofline pre-filter of examples/xegpu/tune_matmul_costmodel.py, crash- and hang-isolated trials of
examples/xegpu/tune_utils.py:35-85 (`run_with_timeout`), CSV logging of csv_logger.py and the
per-shape JSON parameters.  Usage:

    python -m lighthouse_amd.tuning.tune_gemm --sizes 8192,2304,768 --dtype bf16 --db tiles.json --csv tune.csv
"""

from __future__ import annotations

import argparse
import multiprocessing
import sys

from .csv_logger import CSVLogger
from .tile_db import TileDB

TILES = ((256, 256), (256, 128), (128, 256), (128, 128))
# Relative cost per output element of the smaller tiles (more operand traffic per flop).
_PENALTY = {(256, 256): 1.0, (256, 128): 1.1, (128, 256): 1.1, (128, 128): 1.25}
_CUS = 256


def candidate_tiles(M: int, N: int, K: int) -> list[tuple[int, int]]:
    """Tiles the direct-to-LDS kernel accepts for this shape (K % 64 == 0, tile divides M x N)."""
    if K % 64:
        return []
    return [t for t in TILES if M % t[0] == 0 and N % t[1] == 0]


def estimate_cost(M: int, N: int, K: int, tile: tuple[int, int]) -> float:
    """Rounds of one workgroup per CU x tile area x penalty x (K + a fixed per-round cost worth
    about 320 k of main loop: launch, first loads, output stores)."""
    tiles = (M // tile[0]) * (N // tile[1])
    rounds = -(-tiles // _CUS)
    return rounds * tile[0] * tile[1] * _PENALTY[tile] * (K + 320)


def prefilter(M: int, N: int, K: int, slack: float = 1.35) -> list[tuple[int, int]]:
    """Candidates whose estimated cost is within `slack` of the best estimate, best first."""
    cands = sorted(candidate_tiles(M, N, K), key=lambda t: estimate_cost(M, N, K, t))
    if not cands:
        return []
    best = estimate_cost(M, N, K, cands[0])
    return [t for t in cands if estimate_cost(M, N, K, t) <= slack * best]


def _time_tile(res, M, N, K, dtype, tile, nruns, nwarmup):
    import torch

    from .. import ops

    tdt = {"bf16": torch.bfloat16, "f16": torch.float16}[dtype]
    a = torch.randn(M, K, device="cuda").to(tdt)
    b = torch.randn(K, N, device="cuda").to(tdt)
    out = torch.empty(M, N, device="cuda", dtype=tdt)
    for _ in range(nwarmup):
        ops.gemm(a, b, out=out, tile=tile)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(nruns):
        ops.gemm(a, b, out=out, tile=tile)
    stop.record()
    torch.cuda.synchronize()
    seconds = start.elapsed_time(stop) * 1e-3 / nruns
    res["time"] = seconds
    res["throughput"] = 2.0 * M * N * K / seconds / 1e12


def run_with_timeout(experiment_func, *args, timeout: float = 60.0, **kwargs) -> dict:
    """Run `experiment_func(res, *args)` in a forked child process; a crash, an exception or a
    timeout becomes an `error` string instead of taking the tuner down.  Returns
    {time, throughput, error}.  The parent must not have initialised the GPU (a forked copy of a
    live GPU context is unusable): the tuner's own command line never touches it."""
    if "torch" in sys.modules and sys.modules["torch"].cuda.is_initialized():
        raise RuntimeError("run_with_timeout forks; call it from a process that has not initialised the GPU "
                           "(or use tune_shape(..., isolate=False))")

    def wrapped(res, *a, **kw):
        try:
            experiment_func(res, *a, **kw)
        except Exception as exc:  # noqa: BLE001 - reported, not raised
            res["error"] = str(exc).split("\n")[0]

    ctx = multiprocessing.get_context("fork")
    with ctx.Manager() as manager:
        res = manager.dict({"time": 0.0, "throughput": 0.0, "error": ""})
        proc = ctx.Process(target=wrapped, args=(res, *args), kwargs=kwargs)
        proc.start()
        proc.join(timeout)
        if proc.is_alive():
            proc.kill()
            proc.join()
            return {"time": 0.0, "throughput": 0.0, "error": "TIMEOUT"}
        out = dict(res)
        if proc.exitcode != 0 and not out["error"]:
            out["error"] = f"Execution failed with exit code: {proc.exitcode}"
        return out


def tune_shape(M: int, N: int, K: int, dtype: str = "bf16", db: TileDB | None = None, logger: CSVLogger | None = None,
               nruns: int = 50, nwarmup: int = 20, timeout: float = 60.0, exhaustive: bool = False,
               isolate: bool = True) -> dict | None:
    """Time the (pre-filtered) tiles for one shape; record the fastest in `db`.  Returns its row.
    `isolate=False` times in this process (no protection against a hanging or crashing trial)."""
    cands = candidate_tiles(M, N, K) if exhaustive else prefilter(M, N, K)
    best = None
    # The library's own choice (tile None: its cost model, split K for decode shapes) is timed first;
    # a tile enters the database only if it beats that.
    for tile in [None, *cands] if cands else []:
        if isolate:
            res = run_with_timeout(_time_tile, M, N, K, dtype, tile, nruns, nwarmup, timeout=timeout)
        else:
            res = {"time": 0.0, "throughput": 0.0, "error": ""}
            try:
                _time_tile(res, M, N, K, dtype, tile, nruns, nwarmup)
            except (ValueError, RuntimeError) as exc:
                res["error"] = str(exc).split("\n")[0]
        row = {"dtype": dtype, "M": M, "N": N, "K": K, "tile_m": tile[0] if tile else 0, "tile_n": tile[1] if tile else 0,
               "estimate": round(estimate_cost(M, N, K, tile) / 1e6, 3) if tile else 0.0,
               "time_us": round(res["time"] * 1e6, 3),
               "tflops": round(res["throughput"], 2), "error": res["error"]}
        if logger is not None:
            logger.log(row)
        if not res["error"] and res["time"] > 0 and (best is None or row["time_us"] < best["time_us"]):
            best = row
    if best is not None and db is not None and best["tile_m"]:
        db.record(dtype, M, N, K, (best["tile_m"], best["tile_n"]), best["time_us"], best["tflops"])
    return best


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(description="Tile search for the 16-bit HIP GEMM.")
    ap.add_argument("--sizes", action="append", required=True, help="M,N,K (repeatable)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16"])
    ap.add_argument("--db", default="gemm_tiles.json", help="JSON tile database to update")
    ap.add_argument("--csv", default=None, help="CSV log of every trial")
    ap.add_argument("--nruns", type=int, default=50)
    ap.add_argument("--nwarmup", type=int, default=20)
    ap.add_argument("--timeout", type=float, default=60.0)
    ap.add_argument("--exhaustive", action="store_true", help="skip the cost-model pre-filter")
    args = ap.parse_args(argv)
    db = TileDB(args.db)
    logger = CSVLogger(args.csv)
    for spec in args.sizes:
        try:
            M, N, K = (int(x) for x in spec.split(","))
        except ValueError:
            print(f"Error: --sizes expects M,N,K, got '{spec}'", file=sys.stderr)
            return 1
        best = tune_shape(M, N, K, args.dtype, db, logger, args.nruns, args.nwarmup, args.timeout, args.exhaustive)
        if best is None:
            print(f"{spec}: no tile of the direct kernel fits (or every trial failed)", file=sys.stderr)
    db.save()
    return 0


if __name__ == "__main__":
    sys.exit(main())
