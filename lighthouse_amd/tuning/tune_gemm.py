"""Parameter search for the GEMMs (16-bit: workgroup tile, cut along K; f32: workgroup tile) and the
head-dimension-64 attention kernel (query rows per wave, K/V ring depth, key-range split): enumerate the settings that fit a shape,
drop the ones a cost model already rules out, time the rest in child processes, log every trial
and keep the winner when it beats the library's own choice.

The structure follows the reference's tuner for the XeGPU matmul: candidate generation and the
roofline pre-filter of examples/xegpu/tune_matmul_costmodel.py, crash- and hang-isolated trials of
examples/xegpu/tune_utils.py:35-85 (`run_with_timeout`), CSV logging of csv_logger.py and the
per-shape JSON parameters.  Usage:

    python -m lighthouse_amd.tuning.tune_gemm --sizes 8192,2304,768 --dtype bf16 --db tiles.json --csv tune.csv
    python -m lighthouse_amd.tuning.tune_gemm --sizes 8192,768,768 --dtype f32 --db tiles.json
    python -m lighthouse_amd.tuning.tune_gemm --attention 64,2048,causal --db tiles.json

Without --db the packaged database (gfx950_tuned.json, the one `ops` consults by default) is updated.
"""

from __future__ import annotations

import argparse
import multiprocessing
import sys

from .csv_logger import CSVLogger
from .tile_db import TileDB

TILES = ((256, 256), (256, 128), (128, 256), (128, 128))
TILES_F32 = ((128, 128), (128, 64), (64, 64))
# Cost per flop relative to the largest tile, as the library's own tile choice prices it (16-bit:
# measured one round of 256 tiles each at K = 2048 and 4096; 128 x 128 runs two workgroups per CU).
_PENALTY = {(256, 256): 1.0, (256, 128): 1.19, (128, 256): 1.17, (128, 128): 1.19}
_PENALTY_F32 = {(128, 128): 1.0, (128, 64): 1.08, (64, 64): 1.3}
_CUS = 256


def candidate_tiles(M: int, N: int, K: int, dtype: str = "bf16") -> list[tuple[int, int]]:
    """Tiles the direct-to-LDS kernel accepts for this shape: 16-bit K % 64 == 0 and the tile
    divides M x N; f32 K % 32 == 0 and N % 4 == 0 (edge tiles are clipped)."""
    if dtype == "f32":
        return [] if K % 32 or N % 4 else list(TILES_F32)
    if K % 64:
        return []
    return [t for t in TILES if M % t[0] == 0 and N % t[1] == 0]


def estimate_cost(M: int, N: int, K: int, tile: tuple[int, int], dtype: str = "bf16") -> float:
    """Rounds of resident workgroups x tile area x cost per flop x (K + a fixed per-round cost worth
    about 320 k of main loop: launch, first loads, output stores).  The 16-bit 128 x 128 tile runs
    two workgroups per CU that share its rate: a round is two CUs' worth of tiles at twice the cost.
    For the 16-bit tiles a last round that fills a fraction r of the CUs costs 0.6 + 0.4 r^2 of a
    round (128 x 128: 0.12 + 0.88 r), as in the library's own choice."""
    tiles = -(-M // tile[0]) * -(-N // tile[1])
    if dtype == "f32":
        return -(-tiles // _CUS) * tile[0] * tile[1] * _PENALTY_F32[tile] * (K + 320)
    if tile == (128, 128):
        # short K: prologue and epilogue weigh as much as the main loop and the two co-resident
        # workgroups cover each other's; long K and a lone workgroup per CU: nobody covers its waits
        if tiles <= _CUS:
            return tile[0] * tile[1] * (1.08 if K <= 1536 else 1.30) * (K + 320)
        full, rest = divmod(tiles, 2 * _CUS)
        rounds = full + (0.12 + 0.88 * rest / (2 * _CUS) if rest else 0.0)
        return rounds * 2 * tile[0] * tile[1] * (1.05 if K <= 1536 else _PENALTY[tile]) * (K + 320)
    full, rest = divmod(tiles, _CUS)
    rounds = full + (0.6 + 0.4 * (rest / _CUS) ** 2 if rest else 0.0)
    return rounds * tile[0] * tile[1] * _PENALTY[tile] * (K + 320)


def prefilter(M: int, N: int, K: int, slack: float = 1.35, dtype: str = "bf16") -> list[tuple[int, int]]:
    """Candidates whose estimated cost is within `slack` of the best estimate, best first."""
    cands = sorted(candidate_tiles(M, N, K, dtype), key=lambda t: estimate_cost(M, N, K, t, dtype))
    if not cands:
        return []
    best = estimate_cost(M, N, K, cands[0], dtype)
    return [t for t in cands if estimate_cost(M, N, K, t, dtype) <= slack * best]


SPLITS = (2, 4, 8)


def candidate_splits(M: int, N: int, K: int) -> list[int]:
    """Cuts of K worth timing: the problem's 128 x 128 tiles leave CUs idle and every piece of K is
    a multiple of the k-step, at least 256 long."""
    tiles = -(-M // 128) * -(-N // 128)
    if K % 64 or N % 8 or tiles >= _CUS:
        return []
    return [sp for sp in SPLITS if K % (64 * sp) == 0 and K // sp >= 256 and tiles * sp <= 4 * _CUS]


def candidate_settings(M: int, N: int, K: int, exhaustive: bool = False, dtype: str = "bf16") -> list[tuple]:
    """(tile or None, split_k or None) pairs to time after the library's own choice (None, None);
    f32 inputs have tiles only."""
    tiles = candidate_tiles(M, N, K, dtype) if exhaustive else prefilter(M, N, K, dtype=dtype)
    if dtype == "f32":
        return [(t, None) for t in tiles]
    return [(t, None) for t in tiles] + [(None, sp) for sp in candidate_splits(M, N, K)]


def _time_tile(res, M, N, K, dtype, tile, nruns, nwarmup, split_k=None):
    import torch

    from .. import ops
    from .tile_db import use_db

    use_db(None)  # the baseline trial must be the library's own choice, not an earlier database entry
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype]
    a = torch.randn(M, K, device="cuda").to(tdt)
    b = torch.randn(K, N, device="cuda").to(tdt)
    out = torch.empty(M, N, device="cuda", dtype=tdt)
    for _ in range(nwarmup):
        ops.gemm(a, b, out=out, tile=tile, split_k=split_k)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(nruns):
        ops.gemm(a, b, out=out, tile=tile, split_k=split_k)
    stop.record()
    torch.cuda.synchronize()
    seconds = start.elapsed_time(stop) * 1e-3 / nruns
    res["time"] = seconds
    res["throughput"] = 2.0 * M * N * K / seconds / 1e12


def _time_attention(res, BH, T, d, causal, dtype, rows_per_wave, stages, kv_split, nruns, nwarmup):
    import torch

    from .. import ops
    from .tile_db import use_db

    use_db(None)
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16}[dtype]
    q, k, v = (torch.randn(1, BH, T, d, device="cuda").to(tdt) for _ in range(3))
    out = torch.empty_like(q)
    for _ in range(nwarmup):
        ops.attention(q, k, v, causal=causal, out=out, rows_per_wave=rows_per_wave, stages=stages, kv_split=kv_split)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(nruns):
        ops.attention(q, k, v, causal=causal, out=out, rows_per_wave=rows_per_wave, stages=stages, kv_split=kv_split)
    stop.record()
    torch.cuda.synchronize()
    seconds = start.elapsed_time(stop) * 1e-3 / nruns
    res["time"] = seconds
    res["throughput"] = 4.0 * BH * T * T * d * (0.5 if causal else 1.0) / seconds / 1e12


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


def _trial(fn, args, isolate, timeout):
    if isolate:
        return run_with_timeout(fn, *args, timeout=timeout)
    res = {"time": 0.0, "throughput": 0.0, "error": ""}
    try:
        fn(res, *args)
    except (ValueError, RuntimeError) as exc:
        res["error"] = str(exc).split("\n")[0]
    return res


# A setting enters the database only if it beats the library's own choice by this factor
# (two timings of one kernel in different child processes differ by up to 4 %).
MIN_GAIN = 1.05


def tune_shape(M: int, N: int, K: int, dtype: str = "bf16", db: TileDB | None = None, logger: CSVLogger | None = None,
               nruns: int = 300, nwarmup: int = 200, timeout: float = 60.0, exhaustive: bool = False,
               isolate: bool = True) -> dict | None:
    """Time the (pre-filtered) tiles and K cuts for one shape; record the fastest in `db` if it beats
    the library's own choice.  Returns the fastest row.  `isolate=False` times in this process (no
    protection against a hanging or crashing trial)."""
    cands = candidate_settings(M, N, K, exhaustive, dtype)
    best = base = None
    # The library's own choice (no request: its cost model, its own split-K criterion) is timed first.
    for tile, split_k in [(None, None), *cands] if cands else []:
        res = _trial(_time_tile, (M, N, K, dtype, tile, nruns, nwarmup, split_k), isolate, timeout)
        row = {"dtype": dtype, "M": M, "N": N, "K": K, "tile_m": tile[0] if tile else 0, "tile_n": tile[1] if tile else 0,
               "split_k": split_k or 0,
               "estimate": round(estimate_cost(M, N, K, tile, dtype) / 1e6, 3) if tile else 0.0,
               "time_us": round(res["time"] * 1e6, 3),
               "tflops": round(res["throughput"], 2), "error": res["error"]}
        if logger is not None:
            logger.log(row)
        ok = not res["error"] and res["time"] > 0
        if ok and tile is None and split_k is None:
            base = row
        if ok and (best is None or row["time_us"] < best["time_us"]):
            best = row
    if best is not None and db is not None and (best["tile_m"] or best["split_k"]) and (
            base is None or best["time_us"] * MIN_GAIN <= base["time_us"]):
        db.record(dtype, M, N, K, (best["tile_m"], best["tile_n"]) if best["tile_m"] else None, best["time_us"],
                  best["tflops"], split_k=best["split_k"] or None)
    elif best is not None and db is not None:
        db.entries.pop(db.key(dtype, M, N, K), None)  # an older entry no longer beats the library
    return best


ATTENTION_SETTINGS = ((64, None, 1), (64, None, 2), (32, 3, None), (32, 4, None))


def tune_attention(BH: int, T: int, causal: bool, dtype: str = "bf16", db: TileDB | None = None,
                   logger: CSVLogger | None = None, nruns: int = 300, nwarmup: int = 200, timeout: float = 60.0,
                   isolate: bool = True, d: int = 64) -> dict | None:
    """The same for the head-dimension-64 attention kernel: query rows per wave x K/V ring depth x
    split of the key range between two wave groups."""
    best = base = None
    settings = [s for s in ATTENTION_SETTINGS if s[0] != 64 or T % 64 == 0]
    for rows, stages, split in [(None, None, None), *settings]:
        res = _trial(_time_attention, (BH, T, d, causal, dtype, rows, stages, split, nruns, nwarmup), isolate, timeout)
        row = {"dtype": dtype, "BH": BH, "T": T, "d": d, "causal": int(causal), "rows_per_wave": rows or 0,
               "stages": stages or 0, "kv_split": split or 0, "time_us": round(res["time"] * 1e6, 3),
               "tflops": round(res["throughput"], 2), "error": res["error"]}
        if logger is not None:
            logger.log(row)
        ok = not res["error"] and res["time"] > 0
        if ok and rows is None:
            base = row
        if ok and (best is None or row["time_us"] < best["time_us"]):
            best = row
    if best is not None and db is not None and best["rows_per_wave"] and (
            base is None or best["time_us"] * MIN_GAIN <= base["time_us"]):
        db.record_attention(dtype, BH, T, d, causal, best["rows_per_wave"], best["stages"] or None, best["time_us"],
                            best["tflops"], kv_split=best["kv_split"] or None)
    elif best is not None and db is not None:
        db.entries.pop(db.attention_key(dtype, BH, T, d, causal), None)  # an older entry no longer beats the library
    return best


def main(argv: list[str] | None = None) -> int:
    from .tile_db import DEFAULT_DB_PATH

    ap = argparse.ArgumentParser(description="Parameter search for the HIP GEMMs (16-bit and f32) and the attention kernel.")
    ap.add_argument("--sizes", action="append", default=[], help="GEMM M,N,K (repeatable)")
    ap.add_argument("--attention", action="append", default=[], help="attention BH,T[,causal] (repeatable; head_dim 64)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32"],
                    help="GEMM operand type (f32: tiles 128x128 / 128x64 / 64x64, no cut along K); attention is 16-bit")
    ap.add_argument("--db", default=str(DEFAULT_DB_PATH), help="JSON database to update (default: the packaged one)")
    ap.add_argument("--csv", default=None, help="CSV log of every GEMM trial (attention trials: <name>_attention.csv)")
    ap.add_argument("--nruns", type=int, default=300)
    ap.add_argument("--nwarmup", type=int, default=200, help="untimed launches first (the clocks need ~100 to settle)")
    ap.add_argument("--timeout", type=float, default=60.0)
    ap.add_argument("--exhaustive", action="store_true", help="skip the cost-model pre-filter")
    args = ap.parse_args(argv)
    if not args.sizes and not args.attention:
        print("Error: nothing to tune (give --sizes and / or --attention)", file=sys.stderr)
        return 1
    if args.attention and args.dtype == "f32":
        print("Error: the attention variants exist for 16-bit tensors (--dtype bf16 / f16)", file=sys.stderr)
        return 1
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
            print(f"{spec}: no setting of the direct kernel fits (or every trial failed)", file=sys.stderr)
    alog = CSVLogger(args.csv.replace(".csv", "_attention.csv") if args.csv else None)
    for spec in args.attention:
        parts = spec.split(",")
        try:
            BH, T = int(parts[0]), int(parts[1])
            causal = len(parts) > 2 and parts[2] == "causal"
        except (ValueError, IndexError):
            print(f"Error: --attention expects BH,T[,causal], got '{spec}'", file=sys.stderr)
            return 1
        tune_attention(BH, T, causal, args.dtype, db, alog, args.nruns, args.nwarmup, args.timeout)
    db.save()
    return 0


if __name__ == "__main__":
    sys.exit(main())
