from .csv_logger import CSVLogger
from .tile_db import TileDB, active_db, use_db, use_default_db
from .tune_gemm import candidate_settings, candidate_tiles, estimate_cost, prefilter, run_with_timeout, tune_attention, \
    tune_shape

__all__ = ["CSVLogger", "TileDB", "active_db", "use_db", "use_default_db", "candidate_settings", "candidate_tiles",
           "estimate_cost", "prefilter", "run_with_timeout", "tune_attention", "tune_shape"]
