"""Tile search harness: candidates, cost-model pre-filter, isolated trials, CSV log, database."""

import csv
import time

import pytest

from lighthouse_amd.tuning import CSVLogger, TileDB, active_db, candidate_settings, candidate_tiles, estimate_cost, \
    prefilter, run_with_timeout, use_db, use_default_db


def test_candidates_and_prefilter():
    assert candidate_tiles(8192, 768, 768) == [(256, 256), (256, 128), (128, 256), (128, 128)]
    assert candidate_tiles(384, 128, 64) == [(128, 128)]
    assert candidate_tiles(256, 256, 96) == []          # K must be a multiple of 64
    # 4096^3: 256 tiles of 256 x 256 are exactly one round, every smaller tile costs more
    assert prefilter(4096, 4096, 4096)[0] == (256, 256)
    # N = 768: 96 big tiles leave CUs idle; the quarters (384 tiles, three quarters of a round of pairs) are cheapest
    assert prefilter(8192, 768, 768)[0] == (128, 128)
    assert prefilter(8192, 768, 4096)[0] == (128, 128)
    # a partial last round costs less than a full one: 1152 quarter tiles (2.25 rounds of pairs) beat 576 halves
    assert prefilter(8192, 2304, 3072)[0] == (128, 128)
    assert estimate_cost(8192, 2304, 3072, (128, 128)) < 2.5 * estimate_cost(8192, 1024, 3072, (128, 128))
    assert estimate_cost(8192, 768, 768, (256, 256)) > estimate_cost(8192, 768, 768, (256, 128))
    assert all(t in candidate_tiles(8192, 2304, 768) for t in prefilter(8192, 2304, 768))
    # 192 tiles of 256 x 256 in three quarters of a round beat 768 of 128 x 128 in a round and a half of pairs
    assert prefilter(4096, 3072, 4096)[0] == (256, 256)
    # f32: three tiles, edge tiles clipped, no cut along K
    assert candidate_tiles(1000, 1000, 1024, "f32") == [(128, 128), (128, 64), (64, 64)]
    assert candidate_tiles(1024, 1024, 1000, "f32") == [] and candidate_tiles(1024, 1022, 1024, "f32") == []
    assert prefilter(4096, 4096, 4096, dtype="f32")[0] == (128, 128)
    assert prefilter(8192, 768, 768, dtype="f32")[0] == (128, 64)     # 384 wide tiles = 2 rounds, 768 narrow = 3 x 0.54
    assert all(sp is None for _, sp in candidate_settings(16, 8192, 8192, dtype="f32"))


def _ok(res, x):
    res["time"] = 0.5
    res["throughput"] = float(x)


def _boom(res):
    raise RuntimeError("tile does not fit\\nsecond line")


def _hang(res):
    time.sleep(30)


def test_run_with_timeout_isolates_failures():
    assert run_with_timeout(_ok, 3, timeout=20) == {"time": 0.5, "throughput": 3.0, "error": ""}
    assert "tile does not fit" in run_with_timeout(_boom, timeout=20)["error"]
    assert run_with_timeout(_hang, timeout=0.5)["error"] == "TIMEOUT"


def test_csv_logger(tmp_path, capsys):
    path = tmp_path / "log.csv"
    path.write_text("taken\\n")
    logger = CSVLogger(str(path))
    assert logger.filename.endswith("log_1.csv")        # never overwrites an existing log
    logger.log({"M": 1, "tile": "a", "tflops": 2.5})
    logger.log({"M": 2, "tile": "b", "tflops": 3.5})
    with pytest.raises(ValueError):
        logger.log({"M": 3})
    rows = list(csv.DictReader(open(logger.filename)))
    assert rows == [{"M": "1", "tile": "a", "tflops": "2.5"}, {"M": "2", "tile": "b", "tflops": "3.5"}]
    assert capsys.readouterr().out.splitlines()[0] == "M,tile,tflops"


def test_tile_db_round_trip(tmp_path):
    db = TileDB(str(tmp_path / "tiles.json"))
    assert db.lookup("bf16", 8192, 768, 768) is None
    db.record("bf16", 8192, 768, 768, (256, 128), 19.7, 491.0)
    db.save()
    again = TileDB(str(tmp_path / "tiles.json"))
    assert again.lookup("bf16", 8192, 768, 768) == (256, 128)
    assert again.lookup("f16", 8192, 768, 768) is None
    (tmp_path / "bad.json").write_text('{"bf16:1x1x1": {"time_us": 1}}')
    with pytest.raises(ValueError):
        TileDB(str(tmp_path / "bad.json"))
    try:
        assert use_db(again) is again and active_db() is again
        use_db(None)
        assert active_db() is None
    finally:
        use_default_db()


def test_settings_and_database_kinds(tmp_path):
    """Cuts along K are offered where the tiles leave CUs idle; the database keeps tile, cut and the
    attention variant apart and the packaged one loads by default."""
    assert ((None, 8) in candidate_settings(16, 8192, 8192)) and ((None, 2) in candidate_settings(16, 8192, 8192))
    assert all(sp is None for _, sp in candidate_settings(4096, 4096, 4096))      # 1024 tiles: nothing to cut for
    assert all(sp != 8 for _, sp in candidate_settings(128, 1024, 1024))           # K / 8 = 128 is too short a piece
    db = TileDB(str(tmp_path / "t.json"))
    db.record("bf16", 16, 8192, 8192, None, 25.0, 86.0, split_k=8)
    db.record("bf16", 8192, 768, 768, (128, 128), 20.0, 480.0)
    db.record_attention("bf16", 64, 2048, 64, True, 32, 3, 50.0, 690.0)
    db.save()
    again = TileDB(str(tmp_path / "t.json"))
    assert again.lookup_gemm("bf16", 16, 8192, 8192) == (None, 8)
    assert again.lookup_gemm("bf16", 8192, 768, 768) == ((128, 128), None)
    assert again.lookup_gemm("bf16", 1, 1, 1) == (None, None)
    assert again.lookup_attention("bf16", 64, 2048, 64, True) == (32, 3, None)
    assert again.lookup_attention("bf16", 64, 2048, 64, False) == (None, None, None)
    default = use_default_db()
    assert default is None or isinstance(default, TileDB)
    if default is not None:
        for key, entry in default.entries.items():
            assert key.split(":")[0] in ("bf16", "f16", "f32", "attn") and entry["time_us"] > 0
