"""nanoGPT block parity and the Runner boundary on the GPU."""

import numpy as np
import pytest
import torch

from oracle import lh_oracle as orc
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu


def make_block_params(C, rng, std=0.02, bias_std=0.0):
    def w(*s):
        return (rng.standard_normal(s) * std).astype(np.float32)

    def bvec(n):
        return (rng.standard_normal(n) * bias_std).astype(np.float32)

    return {
        "ln1_g": np.ones(C, np.float32), "ln1_b": np.zeros(C, np.float32),
        "w_qkv": w(C, 3 * C), "b_qkv": bvec(3 * C), "w_o": w(C, C), "b_o": bvec(C),
        "ln2_g": np.ones(C, np.float32), "ln2_b": np.zeros(C, np.float32),
        "w_fc": w(C, 4 * C), "b_fc": bvec(4 * C), "w_proj": w(4 * C, C), "b_proj": bvec(C),
    }


def to_device(params, dtype):
    out = {}
    for k, v in params.items():
        t = torch.from_numpy(v).cuda()
        out[k] = t if k.startswith("ln") else t.to(dtype)
    return out


@pytest.mark.parametrize("mode,dtype,rtol", [("f32", torch.float32, 1e-4), ("bf16", torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("bias_std", [0.0, 0.02])
def test_nanogpt_block_small(mode, dtype, rtol, bias_std):
    from lighthouse_amd import ops

    B, T, C, H = 2, 128, 256, 4
    rng = np.random.default_rng(0xB10C)
    p = make_block_params(C, rng, bias_std=bias_std)
    p["ln1_g"] = rng.uniform(0.5, 1.5, C).astype(np.float32)
    p["ln2_b"] = rng.uniform(-0.1, 0.1, C).astype(np.float32)
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    y = ops.nanogpt_block(torch.from_numpy(x).cuda(), to_device(p, dtype), H)
    ref = orc.nanogpt_block(x, p, H, mode=mode)
    assert_close(y.cpu().numpy(), ref, rtol, f"nanoGPT block {mode}")


@pytest.mark.parametrize("mode,dtype,rtol", [("f32", torch.float32, 1e-4), ("bf16", torch.bfloat16, 2e-2)])
def test_nanogpt_block_benchmark_shape(mode, dtype, rtol):
    """n_embd 768, 12 heads, T 1024 (batch 2 of the 8 for the oracle's sake; the batch entries
    are independent, and the full batch is checked for equality of repeated entries)."""
    from lighthouse_amd import ops

    B, T, C, H = 2, 1024, 768, 12
    rng = np.random.default_rng(0x6E616E6F)
    p = make_block_params(C, rng)
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    dp = to_device(p, dtype)
    y = ops.nanogpt_block(torch.from_numpy(x).cuda(), dp, H)
    ref = orc.nanogpt_block(x, p, H, mode=mode)
    assert_close(y.cpu().numpy(), ref, rtol, f"nanoGPT block {mode} C=768 H=12 T=1024", report=True)
    x8 = torch.from_numpy(x).cuda().repeat(4, 1, 1)
    y8 = ops.nanogpt_block(x8, dp, H)
    # repeated entries of one launch are computed identically; across batch sizes the GEMMs may be
    # cut differently (split K for few tiles), which changes the summation order, not the result
    assert torch.equal(y8[:2], y8[6:]) and torch.equal(y8[2:4], y8[4:6]) and torch.equal(y8[:2], y8[2:4])
    assert_close(y8[:2].cpu().numpy(), ref, rtol, f"nanoGPT block {mode} 768/12/1024, batch of 8")


def test_runner_matmul_golden():
    """lh-run's known-answer test (test/run/pipeline-check.mlir:1,16-31) through the Runner."""
    from lighthouse_amd.execution import KernelArgumentParser, Runner
    from lighthouse_amd.ingress import generate_gpu_matmul_payload
    import json
    from pathlib import Path

    golden = json.loads((Path(__file__).parent / "golden" / "lh_run_pipeline_check.json").read_text())
    np.random.seed(golden["seed"])
    a, b, c = (arg.arg for arg in KernelArgumentParser.parse_all(golden["input_shape"]))
    module = generate_gpu_matmul_payload("main", 16, 32, 64, "f32", "f32")
    runner = Runner(module)
    runner.execute("main", [c, a, b])
    np.testing.assert_allclose(c[:, 0], np.array(golden["row_values"], dtype=np.float32), rtol=2e-6)
    assert (c == c[:, :1]).all()
    times = runner.benchmark([c, a, b])
    assert times.shape == (100,) and (times > 0).all()


def test_runner_memory_managers():
    from lighthouse_amd.execution import GPUMemoryManager, Runner, TorchMemoryManager
    from lighthouse_amd.ingress import generate_gpu_matmul_payload
    from lighthouse_amd.utils.numpy import bf16_to_f32, f32_to_bf16

    M, N, K = 256, 128, 64
    rng = np.random.default_rng(2)
    a = f32_to_bf16(rng.standard_normal((M, K)))
    b = f32_to_bf16(rng.standard_normal((K, N)))
    bias = f32_to_bf16(rng.standard_normal(N))
    c = f32_to_bf16(np.zeros((M, N)))
    module = generate_gpu_matmul_payload("payload", M, N, K, "bf16", "f32", has_bias=True, has_relu=True,
                                         result_type="bf16")
    ref = orc.matmul(bf16_to_f32(a), bf16_to_f32(b), bias=bf16_to_f32(bias), relu=True, result_type="bf16")
    runner = Runner(module, mem_manager_cls=GPUMemoryManager)
    host_out = np.zeros_like(c)
    runner.execute("payload", [c, a, b, bias], Runner.get_gpu_argument_access_callback(host_out))
    assert_close(bf16_to_f32(host_out), ref, 2e-2, "runner GPUMemoryManager")
    times = runner.benchmark([c, a, b, bias], nruns=5, nwarmup=2)
    assert times.shape == (5,) and (times > 0).all()
    # Pass-through manager with torch tensors.
    tr = Runner(module, mem_manager_cls=TorchMemoryManager)
    tens = [torch.from_numpy(np.asarray(t).view(np.int16)).cuda().view(torch.bfloat16) for t in (c, a, b, bias)]
    tr.execute("payload", tens)
    assert_close(tens[0].float().cpu().numpy(), ref, 2e-2, "runner TorchMemoryManager")
    with pytest.raises(ValueError):
        Runner(module, mem_manager_cls=dict).execute("payload", [c, a, b, bias])
    with pytest.raises(ValueError):
        runner.execute("payload", [c, a, b])
    with pytest.raises(ValueError):
        runner.execute("payload", [c, a, b[:, :-1], bias])


def test_runner_attention_and_layer_norm_payloads():
    from lighthouse_amd.execution import GPUMemoryManager, Runner
    from lighthouse_amd.ingress import generate_gpu_attention_payload, generate_gpu_layer_norm_payload

    shape = (1, 2, 128, 64)
    np.random.seed(42)
    q, k, v = (np.random.uniform(-0.5, 0.5, shape).astype(np.float16) for _ in range(3))
    out = np.zeros(shape, np.float16)
    runner = Runner(generate_gpu_attention_payload("payload", *shape, "f16"), mem_manager_cls=GPUMemoryManager)
    runner.execute("payload", [out, q, k, v], Runner.get_gpu_argument_access_callback(out))
    ref = orc.attention(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32))
    assert np.allclose(out.astype(np.float32), ref, rtol=1e-3, atol=1e-3)

    M, N = 64, 768
    x = np.random.uniform(-1, 1, (M, N)).astype(np.float32)
    g = np.random.uniform(0.5, 1.5, N).astype(np.float32)
    b = np.random.uniform(-0.1, 0.1, N).astype(np.float32)
    o = np.zeros((M, N), np.float32)
    Runner(generate_gpu_layer_norm_payload("payload", M, N, "f32")).execute("payload", [o, x, g, b])
    assert np.allclose(o, orc.layer_norm(x, g, b), rtol=1e-3, atol=1e-4)


def test_lh_run_cli_golden(tmp_path, capsys):
    """The command line of test/run/pipeline-check.mlir:1-2 on a module of the same form: seed 123,
    uniform A, all-ones B, zero C; prints buffer 3 and, with --benchmark, '100 runs: T seconds'."""
    import json
    import re
    from pathlib import Path

    from lighthouse_amd.lh_run import main

    golden = json.loads((Path(__file__).parent / "golden" / "lh_run_pipeline_check.json").read_text())
    mlir = tmp_path / "payload.mlir"
    mlir.write_text("""
module {
  func.func @main(%lhs: tensor<16x64xf32>, %rhs: tensor<64x32xf32>, %acc: tensor<16x32xf32>) {
    %r = linalg.matmul ins(%lhs, %rhs : tensor<16x64xf32>, tensor<64x32xf32>) outs(%acc : tensor<16x32xf32>) -> tensor<16x32xf32>
    return
  }
}
""")
    common = [str(mlir), "--entry-point=main", f"--input-shape={golden['input_shape']}", "--stage=canonicalize"]
    assert main(common + ["--print-tensor=3", f"--seed={golden['seed']}"]) == 0
    out = capsys.readouterr().out
    assert out.startswith("Output: [[")
    rows = [[float(v) for v in re.findall(r"[-+]?\d+\.\d+(?:e[-+]?\d+)?", line)] for line in out.splitlines() if "[" in line]
    first_values = np.array([r[0] for r in rows if r], dtype=np.float32)
    np.testing.assert_allclose(first_values, np.array(golden["row_values"], dtype=np.float32), rtol=2e-6)
    assert main(common + ["--benchmark"]) == 0
    assert re.match(r"100 runs: [0-9.e-]+ seconds", capsys.readouterr().out)


def test_basic_example_add_kernel(tmp_path, capsys):
    """The kernel of examples/basic/compile_and_run.py:25-31 (`linalg.add` on three 16x32xf32 buffers)
    through the text front end: the Runner on the example's own inputs (a, b random, out zero;
    checked as there against a + b, :170-176) and the command line."""
    import re

    from lighthouse_amd.execution import GPUMemoryManager, Runner
    from lighthouse_amd.ingress.mlir_text import parse_payload_module
    from lighthouse_amd.lh_run import main

    text = """
func.func @add(%a: memref<16x32xf32>, %b: memref<16x32xf32>, %out: memref<16x32xf32>) {
    linalg.add ins(%a, %b : memref<16x32xf32>, memref<16x32xf32>)
               outs(%out : memref<16x32xf32>)
    return
}
"""
    module = parse_payload_module(text)
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((16, 32)).astype(np.float32), rng.standard_normal((16, 32)).astype(np.float32)
    out = np.zeros((16, 32), dtype=np.float32)
    result = {}

    def read_back(inputs, *, execution_engine, memory_manager):
        memory_manager.copy(inputs[2], out)
        result["done"] = True

    Runner(module, mem_manager_cls=GPUMemoryManager).execute("add", [a, b, out], read_back)
    assert result["done"] and np.array_equal(out, a + b)
    mlir = tmp_path / "add.mlir"
    mlir.write_text(text)
    assert main([str(mlir), "--entry-point=add", "--input-shape=16x32xf32xrnd,16x32xf32x1,16x32xf32x0", "--print-tensor=3",
                 "--seed=7", "--stage=canonicalize"]) == 0
    printed = capsys.readouterr().out
    np.random.seed(7)
    expect = np.random.rand(16, 32).astype(np.float32) + 1.0
    vals = np.array([float(v) for v in re.findall(r"[-+]?\d+\.\d+(?:e[-+]?\d+)?", printed)], dtype=np.float32)
    assert vals.size >= 6 and np.allclose(vals[:3], expect[0, :3], rtol=1e-5)


@pytest.mark.parametrize("ab,res,bias_t", [("f32", "f32", "f32"), ("bf16", "bf16", "bf16"), ("bf16", "f32", "f32")])
@pytest.mark.parametrize("variant", ["plain", "bias_relu", "bias_relu_final_tb", "acc"])
def test_runner_mlp_payload(ab, res, bias_t, variant):
    """generate_gpu_mlp_payload: three layers 192 -> 256 -> 128 -> 64 on a batch of 96 (the argument
    list of gpu_mlp_payload.py:44-48: output, input, weights, biases)."""
    from lighthouse_amd.execution import Runner
    from lighthouse_amd.ingress import generate_gpu_mlp_payload
    from lighthouse_amd.utils.numpy import astype as to_host_array, to_float32

    rng = np.random.default_rng(31)
    sizes = [192, 256, 128, 64]
    batch = 96
    has_bias = variant != "plain" and variant != "acc"
    has_relu = has_bias
    tb = variant.endswith("tb")
    final = "final" in variant
    acc = variant == "acc"
    x = orc.round_to(rng.standard_normal((batch, sizes[0])).astype(np.float32), ab)
    ws = [orc.round_to((rng.standard_normal((i, o)) / np.sqrt(i)).astype(np.float32), ab)
          for i, o in zip(sizes[:-1], sizes[1:])]
    bs = [orc.round_to(rng.standard_normal(o).astype(np.float32), bias_t) for o in sizes[1:]] if has_bias else None
    c0 = orc.round_to(rng.standard_normal((batch, sizes[-1])).astype(np.float32), res)
    module = generate_gpu_mlp_payload("payload", batch, sizes[0], sizes[-1], sizes[1:-1], ab, "f32", bias_t, res,
                                      transpose_b=tb, has_bias=has_bias, has_relu=has_relu, accumulate_c=acc,
                                      relu_on_final_layer=final)
    out = to_host_array((c0 if acc else np.zeros_like(c0)).copy(), res)
    bufs = [out, to_host_array(x, ab)] + [to_host_array(w.T.copy() if tb else w, ab) for w in ws]
    if has_bias:
        bufs += [to_host_array(b, bias_t) for b in bs]
    Runner(module).execute("payload", bufs)
    ref = orc.mlp(x, ws, bs, has_relu=has_relu, relu_on_final_layer=final, accumulate_c=c0 if acc else None,
                  ab_type=ab, result_type=res)
    assert_close(to_float32(out), ref, 1e-4 if ab == "f32" else 2e-2, f"mlp {ab}->{res} {variant}")


@pytest.mark.parametrize("mode,dtype,rtol", [("f32", torch.float32, 1e-4), ("bf16", torch.bfloat16, 2e-2)])
def test_nanogpt_forward_two_layers(mode, dtype, rtol):
    """Two blocks + ln_f + lm_head (the tail of build_gpt_fused_payload, nanoGPT_payload.py:399-407)."""
    from lighthouse_amd import ops

    B, T, C, H, V = 2, 128, 256, 4, 384
    rng = np.random.default_rng(0x6770)
    layers = [make_block_params(C, rng, bias_std=0.02) for _ in range(2)]
    lnf_g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    lnf_b = rng.uniform(-0.1, 0.1, C).astype(np.float32)
    lm_w = (rng.standard_normal((C, V)) * 0.05).astype(np.float32)
    lm_b = (rng.standard_normal(V) * 0.02).astype(np.float32)
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    dev = lambda a, dt=torch.float32: torch.from_numpy(a).cuda().to(dt)  # noqa: E731
    y = ops.nanogpt_forward(dev(x), [to_device(p, dtype) for p in layers], dev(lnf_g), dev(lnf_b), dev(lm_w, dtype),
                            dev(lm_b, dtype), H)
    ref = orc.nanogpt_forward(x, layers, lnf_g, lnf_b, lm_w, lm_b, H, mode=mode)
    assert y.shape == (B, T, V)
    assert_close(y.cpu().numpy(), ref, rtol, f"nanoGPT forward {mode}")


# ---- the reference's own nanoGPT configuration (examples/xegpu/nanoGPT.py:186-188,243-297) -------------


def _ref_layer_weights(C, hidden, sc=0.05, nontrivial=False, rng=None):
    """One layer as the reference's driver draws it (np.random.randn * 0.05 in f16, LayerNorm 1 / 0,
    zero biases, examples/xegpu/nanoGPT.py:243-258); `nontrivial` replaces the constant LayerNorm
    parameters and biases by random ones so that a dropped one would show."""
    r = np.random.randn if rng is None else (lambda *s: rng.standard_normal(s))
    f16 = lambda a: a.astype(np.float16)  # noqa: E731
    w = dict(g1=np.ones(C, np.float32), b1n=np.zeros(C, np.float32), wq=f16(r(C, C) * sc), wk=f16(r(C, C) * sc),
             wv=f16(r(C, C) * sc), wp=f16(r(C, C) * sc), bp=np.zeros(C, np.float32), g2=np.ones(C, np.float32),
             b2n=np.zeros(C, np.float32), w1=f16(r(C, hidden) * sc), bb1=np.zeros(hidden, np.float32),
             w2=f16(r(hidden, C) * sc), bb2=np.zeros(C, np.float32))
    if nontrivial:
        for k in ("g1", "g2"):
            w[k] = (1.0 + 0.3 * r(C)).astype(np.float32)
        for k, n in (("b1n", C), ("b2n", C), ("bp", C), ("bb1", hidden), ("bb2", C)):
            w[k] = (0.1 * r(n)).astype(np.float32)
    return w


_REF_KEYS = ("g1", "b1n", "wq", "wk", "wv", "wp", "bp", "g2", "b2n", "w1", "bb1", "w2", "bb2")


def _ref_to_ops_params(w):
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    return dict(ln1_g=dev(w["g1"]), ln1_b=dev(w["b1n"]), w_q=dev(w["wq"]), w_k=dev(w["wk"]), w_v=dev(w["wv"]),
                w_o=dev(w["wp"]), b_o=dev(w["bp"]), ln2_g=dev(w["g2"]), ln2_b=dev(w["b2n"]), w_fc=dev(w["w1"]),
                b_fc=dev(w["bb1"]), w_proj=dev(w["w2"]), b_proj=dev(w["bb2"]))


def _ref_to_oracle_params(w):
    return dict(ln1_g=w["g1"], ln1_b=w["b1n"], w_q=w["wq"], w_k=w["wk"], w_v=w["wv"], w_o=w["wp"], b_o=w["bp"],
                ln2_g=w["g2"], ln2_b=w["b2n"], w_fc=w["w1"], b_fc=w["bb1"], w_proj=w["w2"], b_proj=w["bb2"])


@pytest.mark.parametrize("causal", [False, True])
def test_reference_block_f16(causal):
    """The reference's block at the reference's shapes (T = C = 256, H = 4, hidden 1024; f16 weights,
    separate q/k/v projections, ReLU, f32 biases) against the reference's own checker restated
    (orc.ref_block_fused) with its pass criterion max|diff| / max|ref| < 5e-2
    (examples/xegpu/nanoGPT.py:298-302), the tighter 2e-2, and against the oracle that has the
    kernels' rounding points."""
    from lighthouse_amd import ops

    T, C, hidden, H = 256, 256, 1024, 4
    rng = np.random.default_rng(0x16F)
    w = _ref_layer_weights(C, hidden, nontrivial=True, rng=rng)
    x = (rng.standard_normal((T, C)) * 0.5).astype(np.float32)
    y = ops.nanogpt_block(torch.from_numpy(x).cuda()[None], _ref_to_ops_params(w), H, causal=causal, activation="relu")
    got = y[0].cpu().numpy()
    ref = orc.ref_block_fused(x, w, H, causal=causal)
    rel = np.abs(got - ref).max() / np.abs(ref).max()
    assert rel < 5e-2 and rel < 2e-2, rel
    assert_close(got, ref, 2e-2, f"reference nanoGPT block f16 causal={causal} vs its numpy checker", report=True)
    mine = orc.nanogpt_block(x[None], _ref_to_oracle_params(w), H, mode="f16", causal=causal, activation="relu",
                             bias_f32=True)[0]
    assert_close(got, mine, 4e-3, f"reference nanoGPT block f16 causal={causal} vs oracle")
    # a dropped bias, LayerNorm parameter or the wrong activation / mask is far outside these bounds
    other = orc.ref_block_fused(x, w, H, causal=not causal)
    assert np.abs(got - other).max() / np.abs(ref).max() > 5e-2


def test_reference_gpt_payload_through_runner():
    """build_gpt_fused_payload's argument list through the Runner, with the inputs the reference's
    driver builds (np.random.seed(0), x = randn * 0.5, weights randn * 0.05 in f16, two layers;
    examples/xegpu/nanoGPT.py:236-291) and its checker (numpy_ref_gpt_fused restated) with its own
    pass criterion rel < 5e-2 (:298-302)."""
    from lighthouse_amd.execution import GPUMemoryManager, Runner
    from lighthouse_amd.ingress import build_gpt_fused_payload

    T, C, hidden, vocab, H, L = 256, 256, 1024, 256, 4, 2
    module = build_gpt_fused_payload("payload", T, C, hidden, vocab, L, H)
    fn = module.lookup("payload")
    np.random.seed(0)
    out = np.zeros((T, vocab), np.float32)
    x = (np.random.randn(T, C) * 0.5).astype(np.float32)
    layers, host = [], [out, x]
    for _ in range(L):
        lw = _ref_layer_weights(C, hidden)
        layers.append(lw)
        host += [lw[k] for k in _REF_KEYS]
    gf_g, gf_b = np.ones(C, np.float32), np.zeros(C, np.float32)
    lmw = (np.random.randn(C, vocab) * 0.05).astype(np.float16)
    lmb = np.zeros(vocab, np.float32)
    host += [gf_g, gf_b, lmw, lmb, np.zeros(fn.args[-1].shape, np.int8)]
    runner = Runner(module, mem_manager_cls=GPUMemoryManager)
    cb = Runner.get_gpu_argument_access_callback(out, arg_index=0)
    runner.execute(host_input_buffers=host, payload_function_name="payload", argument_access_callback=cb)
    ref = orc.ref_gpt_fused(x, layers, gf_g, gf_b, lmw, lmb, H)
    rel = np.abs(out - ref).max() / (np.abs(ref).max() + 1e-6)
    assert rel < 5e-2 and rel < 2e-2, rel
    assert_close(out, ref, 2e-2, "reference nanoGPT (2 layers, f16) through the Runner", report=True)
    times = runner.benchmark(host_input_buffers=host, nruns=3, nwarmup=1)
    assert times.shape == (3,) and (times > 0).all()


def test_nanogpt_small_batch_and_ragged_vocab_use_only_the_workspace():
    """Two rows per launch run the projections cut along K, a 50257-column lm_head runs on padded
    copies: both take their temporaries from the caller's workspace (sized by the library's query),
    and the library's own pool stays empty."""
    from lighthouse_amd import _lib, ops

    ops.release_scratch()
    B, T, C, H, V = 1, 2, 768, 12, 50257
    rng = np.random.default_rng(0x5A11)
    layers = [make_block_params(C, rng, bias_std=0.02)]
    lnf_g, lnf_b = np.ones(C, np.float32), np.zeros(C, np.float32)
    lm_w = (rng.standard_normal((C, V)) * 0.05).astype(np.float32)
    lm_b = (rng.standard_normal(V) * 0.02).astype(np.float32)
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    dev = lambda a, dt=torch.float32: torch.from_numpy(a).cuda().to(dt)  # noqa: E731
    torch.cuda.synchronize()
    before = torch.cuda.mem_get_info()[0]
    y = ops.nanogpt_forward(dev(x), [to_device(p, torch.bfloat16) for p in layers], dev(lnf_g), dev(lnf_b),
                            dev(lm_w, torch.bfloat16), dev(lm_b, torch.bfloat16), H)
    ref = orc.nanogpt_forward(x, layers, lnf_g, lnf_b, lm_w, lm_b, H, mode="bf16")
    assert_close(y.cpu().numpy(), ref, 2e-2, "nanoGPT forward, 2 rows, vocab 50257")
    # the workspace query covers both cases by itself
    need = _lib.load().lh_hip_nanogpt_forward_workspace_bytes(B, T, C, V, _lib.BF16, None)
    fixed = B * T * (C * (2 + 6 + 2 + 4) + 4 * C * 2) + 2 * B * T * C * 4
    assert need > fixed + C * 50264 * 2  # at least the padded lm_head weight on top of the fixed buffers
    del before


def test_generic_form_module_at_the_fixture_size():
    """The linalg.generic chain of test/opt/pipeline-check.mlir:27-46 at that fixture's own shapes
    (256x1024 . 1024x2048, f32): the product accumulates into the passed C, then bias, then
    max(., 0).  The module text is generated here, parsed by the MLIR-text front end and run
    through the Runner; integer-valued operands make the f32 result exact in any summation order."""
    from lighthouse_amd.execution import Runner
    from lighthouse_amd.ingress.mlir_text import parse_payload_module

    M, K, N = 256, 1024, 2048
    t = lambda *dims: "tensor<" + "x".join(str(d) for d in dims) + "xf32>"
    text = f"""
#lhs = affine_map<(i, j, k) -> (i, k)>
#rhs = affine_map<(i, j, k) -> (k, j)>
#acc = affine_map<(i, j, k) -> (i, j)>
#vec = affine_map<(i, j) -> (j)>
#mat = affine_map<(i, j) -> (i, j)>
module {{
  func.func @entry(%a: {t(M, K)}, %b: {t(K, N)}, %bias: {t(N)}, %c: {t(M, N)}) -> {t(M, N)} {{
    %p = linalg.generic {{indexing_maps = [#lhs, #rhs, #acc], iterator_types = ["parallel", "parallel", "reduction"]}} ins(%a, %b : {t(M, K)}, {t(K, N)}) outs(%c : {t(M, N)}) {{
    ^bb0(%x: f32, %y: f32, %o: f32):
      %m = arith.mulf %x, %y : f32
      %s = arith.addf %m, %o : f32
      linalg.yield %s : f32
    }} -> {t(M, N)}
    %q = linalg.generic {{indexing_maps = [#vec, #mat], iterator_types = ["parallel", "parallel"]}} ins(%bias : {t(N)}) outs(%p : {t(M, N)}) {{
    ^bb0(%x: f32, %o: f32):
      %s = arith.addf %x, %o : f32
      linalg.yield %s : f32
    }} -> {t(M, N)}
    %zero = arith.constant 0.000000e+00 : f32
    %r = linalg.generic {{indexing_maps = [#mat], iterator_types = ["parallel", "parallel"]}} outs(%q : {t(M, N)}) {{
    ^bb0(%o: f32):
      %s = arith.maximumf %o, %zero : f32
      linalg.yield %s : f32
    }} -> {t(M, N)}
    return %r : {t(M, N)}
  }}
}}
"""
    module = parse_payload_module(text, ["entry"])
    rng = np.random.default_rng(77)
    a = rng.integers(-3, 4, (M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (K, N)).astype(np.float32)
    bias = rng.integers(-40, 41, N).astype(np.float32)
    c0 = rng.integers(-50, 51, (M, N)).astype(np.float32)
    c = c0.copy()
    Runner(module).execute("entry", [a, b, bias, c])
    want = np.maximum(a.astype(np.float64) @ b.astype(np.float64) + c0 + bias[None, :], 0.0)
    assert (want > 0).any() and (want == 0).any()
    np.testing.assert_array_equal(c, want.astype(np.float32))
    # Real-valued operands: the benchmark's f32 tolerance against the f64 product.
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    c = c0.copy()
    Runner(module).execute("entry", [a, b, bias, c])
    assert_close(c, orc.matmul(a, b, c=c0, bias=bias, relu=True, accumulate_c=True), 1e-4,
                 what="generic-form fixture 256x1024x2048 f32")


def test_lh_run_cli_generated_payloads(capsys):
    """The payloads the reference builds with its generators (no MLIR text of them exists) from the
    command line: `gen:KIND{...}` as the module, every packaged descriptor of the kind as a stage,
    output printed and checked against the oracle on the CLI's own seeded inputs; --benchmark prints
    the reference's line."""
    import re

    from lighthouse_amd.execution import TargetInfo
    from lighthouse_amd.lh_run import main
    from lighthouse_amd.pipeline import find_pipeline_file

    np.set_printoptions(threshold=10_000_000, linewidth=200, precision=8)
    target = TargetInfo("gfx950", [])

    def numbers(text):
        return np.array([float(v) for v in re.findall(r"[-+]?(?:\d+\.\d*|\d+)(?:e[-+]?\d+)?|nan|inf", text.split("Output:", 1)[1])],
                        dtype=np.float64)

    # LayerNorm 64 x 96 f32: out, x, gamma, beta in the payload's order
    stage = str(find_pipeline_file(target, "layer_norm", "f32"))
    spec = "gen:layer_norm{M=64 N=96 dtype=f32}"
    assert main([spec, "--entry-point=payload", "--stage", stage, "--seed=5", "--print-tensor=1"]) == 0
    got = numbers(capsys.readouterr().out).reshape(64, 96)
    np.random.seed(5)
    _ = np.zeros((64, 96))  # (the zero-filled output draws nothing)
    x, g, b = np.random.rand(64, 96).astype(np.float32), np.random.rand(96).astype(np.float32), np.random.rand(96).astype(np.float32)
    assert np.allclose(got, orc.layer_norm(x, g, b), rtol=1e-4, atol=1e-5)
    # attention [1, 2, 128, 64] f32, causal, with explicit input shapes
    stage = str(find_pipeline_file(target, "attention", "f32"))
    shapes = ",".join(["1x2x128x64xf32x0"] + ["1x2x128x64xf32xrnd"] * 3)
    assert main(["gen:attention{Z=1 H=2 n_ctx=128 n_head=64 dtype=f32 causal}", "--entry-point=attn", "--stage", stage,
                 "--input-shape", shapes, "--seed=9", "--print-tensor=1"]) == 0
    got = numbers(capsys.readouterr().out).reshape(1, 2, 128, 64)
    np.random.seed(9)
    q, k, v = (np.random.rand(1, 2, 128, 64).astype(np.float32) for _ in range(3))
    assert np.allclose(got, orc.attention(q, k, v, causal=True), rtol=1e-4, atol=1e-5)
    # softmax, GELU and a bf16 matmul with bias + ReLU run and benchmark
    for spec, pipeline, dt in (("gen:softmax{M=32 N=256 dtype=f32}", "softmax", "f32"),
                               ("gen:elementwise{kind=gelu M=32 N=256 dtype=f32}", "element_wise", "f32"),
                               ("gen:matmul{M=256 N=256 K=128 ab_type=bf16 c_type=f32 result_type=bf16 has_bias has_relu}",
                                "matmul", "bf16"),
                               ("gen:nanogpt_block{B=1 T=128 C=128 n_head=2 dtype=bf16}", "nanogpt_block", "bf16")):
        stage = str(find_pipeline_file(target, pipeline, dt))
        assert main([spec, "--entry-point=f", "--stage", stage, "--seed=3", "--benchmark"]) == 0, spec
        assert re.match(r"100 runs: [0-9.e-]+ seconds", capsys.readouterr().out)
    # errors: unknown kind, unknown / missing keys, and MLIR text still needs --input-shape
    for bad in ("gen:conv{M=1}", "gen:softmax{M=32 N=256}", "gen:softmax{M=32 N=256 dtype=f32 tile=4}"):
        assert main([bad, "--entry-point=f", "--stage=cse"]) == 1
        assert "Error:" in capsys.readouterr().err
