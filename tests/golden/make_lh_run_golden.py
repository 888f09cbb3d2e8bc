"""Writes tests/golden/lh_run_pipeline_check.json.

The expected values are the 16 numbers the reference's own known-answer test prints
(test/run/pipeline-check.mlir:16-31 of the Lighthouse tree: lh-run on a 16x64 . 64x32 f32
matmul with inputs `16x64xf32xrnd,64x32xf32x1,16x32xf32x0`, --seed=123); they are data
copied from that test's CHECK lines, not produced by running the reference.
"""

import json
from pathlib import Path

ROW_VALUES = [
    32.873924, 31.594452, 33.101555, 31.069946, 30.436699, 32.59776, 30.10459, 32.242332,
    31.32454, 34.80585, 33.510525, 35.42333, 31.94259, 32.442146, 30.075504, 26.437485,
]

if __name__ == "__main__":
    out = {
        "source": "test/run/pipeline-check.mlir:1,16-31",
        "seed": 123,
        "input_shape": "16x64xf32xrnd,64x32xf32x1,16x32xf32x0",
        "print_tensor": 3,
        "row_values": ROW_VALUES,
    }
    Path(__file__).with_name("lh_run_pipeline_check.json").write_text(json.dumps(out, indent=2) + "\n")
