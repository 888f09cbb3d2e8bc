"""``lh-run`` for the HIP target: run or benchmark a payload function on the GPU.

Same command line as lighthouse/lh_run.py:14-145 (``payload_module --entry-point F
--input-shape SPECS --stage S... [--seed N] [-O n] [--benchmark] [--print-tensor N]
[--print-optimized-module] [--print-mlir-after-all]``), same output lines (``N runs: T seconds``,
``Output: <array>``) and exit codes (1 on FileNotFoundError / OSError / ValueError, 130 on
Ctrl-C).  The payload module is MLIR text of one of the matmul forms this target has a kernel for
(see ingress/mlir_text.py), or, for the payloads the reference builds with its Python generators and
ships no MLIR text of (attention, LayerNorm, softmax, elementwise, the nanoGPT block), the generator
call itself: ``gen:attention{Z=4 H=16 n_ctx=2048 n_head=64 dtype=bf16 causal}`` (see
ingress/payloads.py:generate_payload_module; ``--input-shape`` may then be left out: outputs are
zero-filled, inputs uniform random).  A ``--stage`` that names a pipeline descriptor with a ``kernel:`` stage
(descriptors/gfx950/<pipeline>/<dtype>.yaml) sets that kernel's request flags (every parameter of
such a stage acts; an unknown one is an error); MLIR pass /
transform stages have no counterpart here (the kernels are already lowered) and are skipped with a
note on stderr, so the reference's own RUN lines work unchanged.
"""

from __future__ import annotations

import argparse
import sys
from datetime import datetime

import numpy as np

from . import _lib
from .execution.init import KernelArgumentParser
from .execution.runner import Runner
from .ingress.mlir_text import load_payload_module
from .ingress.payloads import PayloadModule, default_input_shapes, generate_payload_module, is_generated_module
from .pipeline.descriptor import Descriptor, PipelineDescriptor


# Parameters a `kernel:` stage may carry, per payload kind: each one changes what runs (a request
# flag of the C entry point).  Anything else in a stage is an error, so a descriptor cannot
# describe a kernel it does not select.
KERNEL_PARAMETERS = {
    "matmul": {"tile_m", "tile_n", "split_k"},
    "attention": {"q_rows_per_wave", "kv_stages", "kv_split", "scale_f32"},
    "matmul_fp8": set(), "mlp": set(), "layer_norm": set(), "elementwise": set(), "nanogpt_block": set(),
    "gpt_fused": set(),
}


def _apply_matmul(fn, params: dict, notes: list[str]) -> None:
    if not params:
        return
    out_shape = fn.args[fn.arg_order[0] if fn.arg_order else 0].shape
    f32 = fn.attrs.ab_dtype == _lib.F32
    flags = fn.attrs.flags
    if "tile_m" in params or "tile_n" in params:
        tile = (params.get("tile_m"), params.get("tile_n"))
        if tile not in _lib.GEMM_TILES:
            raise ValueError(f"stage 'matmul': unsupported tile {tile[0]}x{tile[1]}; choose from {sorted(_lib.GEMM_TILES)}")
        allowed = _lib.GEMM_TILES_F32 if f32 else _lib.GEMM_TILES_16BIT
        if tile not in allowed:
            notes.append(f"stage 'matmul': tile {tile[0]}x{tile[1]} is not one the {'f32' if f32 else '16-bit'} kernel of "
                         f"@{fn.name} takes ({sorted(allowed)}); the library chooses")
        elif f32 or (out_shape[0] % tile[0] == 0 and out_shape[1] % tile[1] == 0):
            flags = (flags & ~_lib.GEMM_TILE_MASK) | _lib.GEMM_TILES[tile]
        else:
            notes.append(f"stage 'matmul': tile {tile[0]}x{tile[1]} does not apply to @{fn.name} "
                         f"({out_shape[0]}x{out_shape[1]}); the library chooses")
    if "split_k" in params and f32:
        notes.append(f"stage 'matmul': a cut along K applies to 16-bit operands, not to @{fn.name}; the library chooses")
    elif "split_k" in params:
        sp = params["split_k"]
        if sp not in _lib.GEMM_SPLITK:
            raise ValueError(f"stage 'matmul': unsupported split_k {sp}; choose from {sorted(_lib.GEMM_SPLITK)}")
        if sp > 1 and flags & _lib.GEMM_TILE_MASK:
            raise ValueError("stage 'matmul': a cut along K runs on 128x128 tiles and excludes tile_m / tile_n")
        flags = (flags & ~_lib.GEMM_SPLITK_MASK) | _lib.GEMM_SPLITK[sp]
    fn.attrs.flags = flags


def _apply_attention(fn, params: dict, notes: list[str]) -> None:
    rows, stages, split = params.get("q_rows_per_wave", 0), params.get("kv_stages", 0), params.get("kv_split", 0)
    if rows not in _lib.ATTN_ROWS or stages not in _lib.ATTN_STAGES or split not in _lib.ATTN_KSPLIT:
        raise ValueError(f"stage 'attention': q_rows_per_wave must be 32 or 64, kv_stages 3 or 4 and kv_split 1 or 2, "
                         f"got {rows} / {stages} / {split}")
    scale_f32 = params.get("scale_f32", False)
    if scale_f32 not in (True, False):
        raise ValueError(f"stage 'attention': scale_f32 is a flag, got {scale_f32}")
    if not (rows or stages or split or scale_f32):
        return
    if fn.attrs.dtype == _lib.F32 or fn.args[0].shape[-1] != 64:
        notes.append(f"stage 'attention': variant requests apply to 16-bit tensors with head dimension 64, not to "
                     f"@{fn.name}; the library chooses")
        return
    fn.attrs.causal = ((fn.attrs.causal & _lib.ATTN_CAUSAL) | _lib.ATTN_ROWS[rows] | _lib.ATTN_STAGES[stages]
                       | _lib.ATTN_KSPLIT[split] | (_lib.ATTN_SCALE_F32 if scale_f32 else 0))


def apply_stage(module: PayloadModule, stage: str, notes: list[str]) -> None:
    """Apply one ``--stage`` to every function of the module."""
    desc = Descriptor(stage)
    if desc.is_include():
        stages = PipelineDescriptor(desc).get_stages()
    else:
        stages = [desc]
    for st in stages:
        if not st.is_kernel():
            notes.append(f"stage '{st}': MLIR {st.type or 'pass'} stage skipped (the HIP kernels are already lowered)")
            continue
        params = {**st.args, **st.opts}
        if st.basename not in KERNEL_PARAMETERS:
            raise ValueError(f"kernel stage '{st.basename}': no such payload kind; known: {sorted(KERNEL_PARAMETERS)}")
        unknown = sorted(set(params) - KERNEL_PARAMETERS[st.basename])
        if unknown:
            raise ValueError(f"kernel stage '{st.basename}': unknown parameter(s) {unknown}; "
                             f"it takes {sorted(KERNEL_PARAMETERS[st.basename]) or 'none'}")
        matched = False
        for fn in module.functions.values():
            if fn.entry != st.basename:
                continue
            matched = True
            if fn.entry == "matmul":
                _apply_matmul(fn, params, notes)
            elif fn.entry == "attention":
                _apply_attention(fn, params, notes)
        if not matched:
            notes.append(f"stage '{st.basename}': no function of this kind in the module")


def main(argv: list[str] | None = None) -> int:
    try:
        parser = argparse.ArgumentParser(
            prog="lh-run",
            description="Lighthouse runner, HIP target: runs a payload function of an MLIR module on the GPU.")
        parser.add_argument("payload_module", type=str,
                            help="Path to the payload MLIR module, or gen:KIND{key=value ...} for a generated payload.")
        parser.add_argument("--entry-point", type=str, required=True,
                            help="Name of the entrypoint function in the payload MLIR module.")
        parser.add_argument("--input-shape", required=False, default=None,
                            help="Shape of the input tensors in format: DIMS(MxNx...)xTYPE(f16/f32/f64/bf16/i8)"
                                 "xINIT(0/1/rnd/id). For multiple inputs, separate by comma.")
        parser.add_argument("--seed", type=int, default=0, help="Random seed for initializing input tensors.")
        parser.add_argument("--stage", action="append", required=True,
                            help="Pipeline descriptors / stages to apply to the input module.")
        parser.add_argument("-O", type=int, default=3, help="Optimization level (accepted, unused).")
        parser.add_argument("--benchmark", action=argparse.BooleanOptionalAction,
                            help="Whether to run the benchmark. Default is False.")
        parser.add_argument("--print-optimized-module", action=argparse.BooleanOptionalAction,
                            help="Whether to print the module after all stages. Default is False.")
        parser.add_argument("--print-tensor", type=int, default=0, help="Print the Nth tensor. Default is 0 (no print).")
        parser.add_argument("--print-mlir-after-all", action=argparse.BooleanOptionalAction,
                            help="Whether to print the module after every stage. Default is False.")
        args = parser.parse_args(argv)

        np.random.seed(args.seed if args.seed else int(datetime.now().timestamp()))

        if is_generated_module(args.payload_module):
            module = generate_payload_module(args.payload_module, args.entry_point)
            if args.input_shape is None:
                args.input_shape = default_input_shapes(module.lookup(args.entry_point))
        else:
            module = load_payload_module(args.payload_module, [args.entry_point])
        if args.input_shape is None:
            raise ValueError("--input-shape is required for a module read from MLIR text")
        notes: list[str] = []
        for stage in args.stage:
            apply_stage(module, stage, notes)
            if args.print_mlir_after_all:
                print(f"// -----// after stage {stage} //----- //\n{module}")
        for note in notes:
            print(f"lh-run: {note}", file=sys.stderr)
        if args.print_optimized_module:
            print(module)

        buffers = [arg.arg for arg in KernelArgumentParser.parse_all(args.input_shape)]
        runner = Runner(module, opt_level=args.O)
        if args.benchmark:
            time_array = runner.benchmark(host_input_buffers=buffers, payload_function_name=args.entry_point)
            print(f"{len(time_array)} runs: {np.mean(time_array)} seconds")
        else:
            runner.execute(payload_function_name=args.entry_point, host_input_buffers=buffers)

        if args.print_tensor > 0:
            print(f"Output: {buffers[args.print_tensor - 1]}")
        return 0
    except KeyboardInterrupt:
        print("\nInterrupted", file=sys.stderr)
        return 130
    except (FileNotFoundError, OSError, ValueError) as exc:
        print(f"Error: {exc}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
