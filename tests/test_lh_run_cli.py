"""MLIR-text ingress and the lh-run command line (host side; no GPU needed).

Forms covered are those of the reference's fixtures: the named-op module of
test/run/pipeline-check.mlir:8-14 and the linalg.generic chain of test/opt/pipeline-check.mlir:27-46
(re-typed here with other shapes and names, not copied).
"""

import pytest

from lighthouse_amd import _lib
from lighthouse_amd.ingress.mlir_text import parse_payload_module
from lighthouse_amd.lh_run import apply_stage, main

NAMED = """
module {
  func.func @mm(%a: tensor<8x24xf32>, %b: tensor<24x16xf32>, %c: tensor<8x16xf32>) {
    %zero = arith.constant 0.000000e+00 : f32
    %unused = linalg.fill ins(%zero : f32) outs(%c : tensor<8x16xf32>) -> tensor<8x16xf32>
    %r = linalg.matmul ins(%a, %b : tensor<8x24xf32>, tensor<24x16xf32>) outs(%c : tensor<8x16xf32>) -> tensor<8x16xf32>
    return
  }
}
"""

NAMED_ZERO_INIT = NAMED.replace("outs(%c : tensor<8x16xf32>) -> tensor<8x16xf32>\n    return",
                                "outs(%unused : tensor<8x16xf32>) -> tensor<8x16xf32>\n    return")

GENERIC = """
#mk = affine_map<(d0, d1, d2) -> (d0, d2)>
#kn = affine_map<(d0, d1, d2) -> (d2, d1)>
#mn = affine_map<(d0, d1, d2) -> (d0, d1)>
#row = affine_map<(d0, d1) -> (d1)>
#id = affine_map<(d0, d1) -> (d0, d1)>
module {
  func.func @layer(%x: tensor<32x64xbf16>, %w: tensor<64x128xbf16>, %bias: tensor<128xbf16>, %y: tensor<32x128xbf16>) -> tensor<32x128xbf16> {
    %0 = linalg.generic {indexing_maps = [#mk, #kn, #mn], iterator_types = ["parallel", "parallel", "reduction"]} ins(%x, %w : tensor<32x64xbf16>, tensor<64x128xbf16>) outs(%y : tensor<32x128xbf16>) {
    ^bb0(%in: bf16, %in_0: bf16, %out: bf16):
      %5 = arith.mulf %in, %in_0 : bf16
      %6 = arith.addf %5, %out : bf16
      linalg.yield %6 : bf16
    } -> tensor<32x128xbf16>
    %1 = linalg.generic {indexing_maps = [#row, #id], iterator_types = ["parallel", "parallel"]} ins(%bias : tensor<128xbf16>) outs(%0 : tensor<32x128xbf16>) {
    ^bb0(%in: bf16, %out: bf16):
      %5 = arith.addf %in, %out : bf16
      linalg.yield %5 : bf16
    } -> tensor<32x128xbf16>
    %cst = arith.constant 0.000000e+00 : bf16
    %2 = linalg.generic {indexing_maps = [#id], iterator_types = ["parallel", "parallel"]} outs(%1 : tensor<32x128xbf16>) {
    ^bb0(%out: bf16):
      %5 = arith.maximumf %out, %cst : bf16
      linalg.yield %5 : bf16
    } -> tensor<32x128xbf16>
    return %2 : tensor<32x128xbf16>
  }
}
"""


def test_named_matmul_accumulates_into_argument():
    fn = parse_payload_module(NAMED).lookup("mm")
    assert fn.entry == "matmul" and fn.arg_order == [2, 0, 1]
    assert fn.attrs.flags == _lib.GEMM_ACCUMULATE_C
    assert [a.shape for a in fn.args] == [(8, 24), (24, 16), (8, 16)]
    assert [a.writable for a in fn.args] == [False, False, True]
    assert fn.flops == 2 * 8 * 16 * 24


def test_zero_fill_means_no_accumulation():
    fn = parse_payload_module(NAMED_ZERO_INIT).lookup("mm")
    assert fn.attrs.flags == 0 and fn.arg_order == [2, 0, 1]


MEMREF = """
module {
  func.func @mm(%a: memref<8x24xf32>, %b: memref<24x16xf32>, %bias: memref<16xf32>, %c: memref<8x16xf32>) {
    %zero = arith.constant 0.000000e+00 : f32
    linalg.fill ins(%zero : f32) outs(%c : memref<8x16xf32>)
    linalg.matmul ins(%a, %b : memref<8x24xf32>, memref<24x16xf32>) outs(%c : memref<8x16xf32>)
    %bc = memref.alloc() : memref<8x16xf32>
    linalg.broadcast ins(%bias : memref<16xf32>) outs(%bc : memref<8x16xf32>) dimensions = [0]
    linalg.add ins(%c, %bc : memref<8x16xf32>, memref<8x16xf32>) outs(%c : memref<8x16xf32>)
    %zeros = memref.alloc() : memref<8x16xf32>
    linalg.fill ins(%zero : f32) outs(%zeros : memref<8x16xf32>)
    linalg.max ins(%c, %zeros : memref<8x16xf32>, memref<8x16xf32>) outs(%c : memref<8x16xf32>)
    return
  }
}
"""


def test_bufferised_form_follows_program_order():
    """Operations on memrefs have no results: a zero fill of the output buffer BEFORE the matmul
    means the product does not accumulate into what the caller passed; without the fill, or with
    the fill after the matmul's read, it does."""
    fn = parse_payload_module(MEMREF).lookup("mm")
    assert fn.arg_order == [3, 0, 1, 2]
    assert fn.attrs.flags == _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU
    no_fill = MEMREF.replace("    linalg.fill ins(%zero : f32) outs(%c : memref<8x16xf32>)\n", "")
    assert parse_payload_module(no_fill).lookup("mm").attrs.flags == (
        _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU | _lib.GEMM_ACCUMULATE_C)
    plain = """
    func.func @mm(%a: memref<8x24xf32>, %b: memref<24x16xf32>, %c: memref<8x16xf32>) {
      %zero = arith.constant 0.0 : f32
      linalg.fill ins(%zero : f32) outs(%c : memref<8x16xf32>)
      linalg.matmul ins(%a, %b : memref<8x24xf32>, memref<24x16xf32>) outs(%c : memref<8x16xf32>)
      return
    }"""
    assert parse_payload_module(plain).lookup("mm").attrs.flags == 0
    one = plain.replace("arith.constant 0.0", "arith.constant 1.0")
    with pytest.raises(ValueError, match="non-zero fill"):
        parse_payload_module(one)


def test_generic_chain_with_bias_and_relu():
    fn = parse_payload_module(GENERIC, ["layer"]).lookup("layer")
    assert fn.arg_order == [3, 0, 1, 2]
    assert fn.attrs.flags == _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU | _lib.GEMM_ACCUMULATE_C
    assert fn.attrs.ab_dtype == _lib.BF16 and fn.attrs.out_dtype == _lib.BF16


def test_transposed_contraction_maps():
    text = GENERIC.replace("#kn = affine_map<(d0, d1, d2) -> (d2, d1)>", "#kn = affine_map<(d0, d1, d2) -> (d1, d2)>")
    text = text.replace("tensor<64x128xbf16>", "tensor<128x64xbf16>")
    fn = parse_payload_module(text).lookup("layer")
    assert fn.attrs.flags & _lib.GEMM_TRANSPOSE_B and not fn.attrs.flags & _lib.GEMM_TRANSPOSE_A


@pytest.mark.parametrize("text,match", [
    (NAMED.replace("linalg.matmul", "linalg.batch_matmul"), "unsupported operation"),
    (NAMED.replace("tensor<24x16xf32>", "tensor<25x16xf32>"), "inconsistent matmul shapes"),
    (NAMED.replace("@mm", "@other"), "no function named"),
    (NAMED.replace("tensor<8x24xf32>", "tensor<?x24xf32>"), "unsupported argument type"),
])
def test_rejected_modules(text, match):
    with pytest.raises(ValueError, match=match):
        parse_payload_module(text, ["mm"])


def test_stage_application(tmp_path):
    text = GENERIC.replace("32x", "256x").replace("x128", "x384").replace("<128x", "<384x")
    module = parse_payload_module(text)
    notes = []
    apply_stage(module, "canonicalize", notes)                 # an MLIR pass: skipped
    assert "skipped" in notes[0]
    yaml_path = tmp_path / "bf16.yaml"
    yaml_path.write_text('Pipeline:\n  - kernel: "matmul{tile_m=256 tile_n=128}"\n  - pass: cse\n')
    apply_stage(module, str(yaml_path), notes)
    assert module.lookup("layer").attrs.flags & 0x700 == _lib.GEMM_TILES[(256, 128)]
    yaml_path.write_text('Pipeline:\n  - kernel: "matmul{tile_m=256 tile_n=256}"\n')
    apply_stage(module, str(yaml_path), notes)                 # 384 % 256 != 0: left to the library
    assert module.lookup("layer").attrs.flags & 0x700 == _lib.GEMM_TILES[(256, 128)]
    assert "does not apply" in notes[-1]
    # the f32 kernel has tiles of its own (edge tiles clipped: no divisibility rule) and no cut along K
    f32 = parse_payload_module(NAMED)
    yaml_path.write_text('Pipeline:\n  - kernel: "matmul{tile_m=128 tile_n=64}"\n')
    apply_stage(f32, str(yaml_path), notes)
    assert f32.lookup("mm").attrs.flags & 0x700 == _lib.GEMM_TILES[(128, 64)] == 0x500
    apply_stage(module, str(yaml_path), notes)                 # not a tile of the 16-bit kernel
    assert module.lookup("layer").attrs.flags & 0x700 == _lib.GEMM_TILES[(256, 128)] and "16-bit kernel" in notes[-1]
    yaml_path.write_text('Pipeline:\n  - kernel: "matmul{tile_m=256 tile_n=128 split_k=1}"\n')
    apply_stage(f32, str(yaml_path), notes)
    assert f32.lookup("mm").attrs.flags & 0x700 == 0x500 and f32.lookup("mm").attrs.flags & _lib.GEMM_SPLITK_MASK == 0
    assert "f32 kernel" in notes[-2] and "cut along K" in notes[-1]


def test_stage_parameters_all_act_or_fail(tmp_path):
    """Every parameter of a `kernel:` stage sets a request flag; an unknown one is an error, so a
    descriptor cannot carry text that selects nothing."""
    from lighthouse_amd.ingress import generate_gpu_attention_payload
    from lighthouse_amd.pipeline.finder import find_pipeline_file
    from lighthouse_amd.execution.target import TargetInfo

    text = GENERIC.replace("32x", "256x").replace("x128", "x384").replace("<128x", "<384x")
    module = parse_payload_module(text)
    notes = []
    y = tmp_path / "s.yaml"
    y.write_text('Pipeline:\n  - kernel: "matmul{split_k=4}"\n')
    apply_stage(module, str(y), notes)
    assert module.lookup("layer").attrs.flags & _lib.GEMM_SPLITK_MASK == _lib.GEMM_SPLITK[4]
    y.write_text('Pipeline:\n  - kernel: "matmul{split_k=1}"\n')
    apply_stage(module, str(y), notes)
    assert module.lookup("layer").attrs.flags & _lib.GEMM_SPLITK_MASK == _lib.GEMM_SPLITK[1]
    for bad, match in (('matmul{tile_m=256 tile_n=128 wave_m=128}', "unknown parameter"), ('matmul{split_k=3}', "split_k"),
                       ('matmul{tile_m=96 tile_n=128}', "unsupported tile"), ('conv{tile=1}', "no such payload kind"),
                       ('matmul{tile_m=128 tile_n=128 split_k=2}', "excludes"), ('attention{rescale=lazy}', "unknown parameter"),
                       ('layer_norm{rows_per_wg=4}', "unknown parameter")):
        y.write_text(f'Pipeline:\n  - kernel: "{bad}"\n')
        with pytest.raises(ValueError, match=match):
            apply_stage(parse_payload_module(text), str(y), notes)
    att = generate_gpu_attention_payload("payload", 4, 16, 2048, 64, "bf16", causal=True)
    y.write_text('Pipeline:\n  - kernel: "attention{q_rows_per_wave=32 kv_stages=3}"\n')
    apply_stage(att, str(y), notes)
    assert att.lookup("payload").attrs.causal == _lib.ATTN_CAUSAL | _lib.ATTN_ROWS[32] | _lib.ATTN_STAGES[3]
    y.write_text('Pipeline:\n  - kernel: "attention{kv_split=2}"\n')
    apply_stage(att, str(y), notes)
    assert att.lookup("payload").attrs.causal == _lib.ATTN_CAUSAL | _lib.ATTN_KSPLIT[2]
    y.write_text('Pipeline:\n  - kernel: "attention{q_rows_per_wave=48}"\n')
    with pytest.raises(ValueError, match="q_rows_per_wave"):
        apply_stage(att, str(y), notes)
    y.write_text('Pipeline:\n  - kernel: "attention{q_rows_per_wave=64 scale_f32}"\n')
    apply_stage(att, str(y), notes)
    assert att.lookup("payload").attrs.causal == _lib.ATTN_CAUSAL | _lib.ATTN_ROWS[64] | _lib.ATTN_SCALE_F32
    # every packaged descriptor parses and applies: none carries a parameter that does nothing
    target = TargetInfo("gfx950", [])
    for pipeline, dtypes in {"matmul": ["bf16", "f16", "f32", "f8E4M3FN"], "attention": ["bf16", "f16", "f32"],
                             "layer_norm": ["f32", "bf16"], "softmax": ["f32", "bf16"], "element_wise": ["f32", "bf16"],
                             "nanogpt_block": ["f32", "bf16"]}.items():
        for dt in dtypes:
            path = find_pipeline_file(target, pipeline, dt)
            assert path is not None, (pipeline, dt)
            apply_stage(parse_payload_module(text), str(path), [])


def test_cli_error_codes(tmp_path, capsys):
    missing = main([str(tmp_path / "nope.mlir"), "--entry-point", "mm", "--input-shape", "8x24xf32x1", "--stage", "cse"])
    assert missing == 1 and "Error:" in capsys.readouterr().err
    f = tmp_path / "m.mlir"
    f.write_text(NAMED)
    bad_stage = main([str(f), "--entry-point", "mm", "--input-shape", "8x24xf32x1,24x16xf32x1,8x16xf32x0",
                      "--stage", str(tmp_path / "absent.yaml")])
    assert bad_stage == 1
    bad_entry = main([str(f), "--entry-point", "zz", "--input-shape", "8x24xf32x1", "--stage", "cse"])
    assert bad_entry == 1


def test_plain_add_becomes_an_elementwise_payload():
    """`linalg.add` of two arguments into a third (examples/basic/compile_and_run.py:25-31) maps to the
    elementwise sum kernel with the output first; anything else about it is rejected."""
    text = """
func.func @add(%a: memref<16x32xf32>, %b: memref<16x32xf32>, %out: memref<16x32xf32>) {
    linalg.add ins(%a, %b : memref<16x32xf32>, memref<16x32xf32>) outs(%out : memref<16x32xf32>)
    return
}
"""
    fn = parse_payload_module(text).lookup("add")
    assert fn.entry == "elementwise" and fn.arg_order == [2, 0, 1]
    assert fn.attrs.kind == _lib.EW_ADD and [a.writable for a in fn.args] == [False, False, True]
    with pytest.raises(ValueError, match="one shape"):
        parse_payload_module(text.replace("%b: memref<16x32xf32>", "%b: memref<16x64xf32>"))
    with pytest.raises(ValueError, match="2-D"):
        parse_payload_module(text.replace("16x32xf32", "16xf32"))
    with pytest.raises(ValueError, match="distinct"):
        parse_payload_module(text.replace("outs(%out", "outs(%a"))


def test_generated_payload_modules(capsys):
    """`gen:KIND{...}` as lh-run's module: the generator's own keyword names in the descriptor
    grammar; default input shapes follow the payload's argument list (outputs zero, inputs random)."""
    from lighthouse_amd.ingress.payloads import default_input_shapes, generate_payload_module, is_generated_module

    assert is_generated_module("gen:softmax{M=2 N=4 dtype=f32}") and not is_generated_module("payload.mlir")
    fn = generate_payload_module("gen:attention{Z=4 H=16 n_ctx=2048 n_head=64 dtype=bf16 causal}", "attn").lookup("attn")
    assert fn.entry == "attention" and fn.attrs.causal == 1 and fn.args[0].writable
    assert default_input_shapes(fn) == ",".join(["4x16x2048x64xbf16x0"] + ["4x16x2048x64xbf16xrnd"] * 3)
    fn = generate_payload_module("gen:matmul{M=256 N=512 K=128 ab_type=bf16 c_type=f32 result_type=bf16 has_bias has_relu}",
                                 "mm").lookup("mm")
    assert fn.entry == "matmul" and fn.attrs.flags == _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU
    assert default_input_shapes(fn) == "256x512xbf16x0,256x128xbf16xrnd,128x512xbf16xrnd,512xbf16xrnd"
    blk = generate_payload_module("gen:nanogpt_block{B=8 T=1024 C=768 n_head=12 dtype=bf16}", "blk").lookup("blk")
    assert blk.entry == "nanogpt_block" and default_input_shapes(blk).endswith("xi8x0")
    for bad, match in (("gen:conv{M=1}", "no payload generator"), ("gen:softmax{M=32 N=256}", "missing key"),
                       ("gen:softmax{M=32 N=256 dtype=f32 tile=4}", "unknown key")):
        with pytest.raises(ValueError, match=match):
            generate_payload_module(bad, "f")
        assert main([bad, "--entry-point=f", "--stage=cse"]) == 1
        assert "Error:" in capsys.readouterr().err
