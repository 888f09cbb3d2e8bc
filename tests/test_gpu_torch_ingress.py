"""torch.compile models through the HIP backend, checked against the oracle."""

import numpy as np
import pytest
import torch
import torch.nn as nn

from tests.conftest import assert_close
from oracle import lh_oracle as orc
from tests.test_torch_ingress import Block

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().float().cpu().numpy()


def test_compiled_mlp_f32():
    """Linear+ReLU, Linear: the shape of examples/ingress/torch/compile_model.py's MLP."""
    from lighthouse_amd.ingress.torch import gpu_backend

    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(256, 512), nn.ReLU(), nn.Linear(512, 128)).cuda()
    x = torch.randn(64, 256, device="cuda")
    backend = gpu_backend()
    compiled = torch.compile(model, backend=backend, dynamic=False)
    with torch.no_grad():
        y = compiled(x)
    h = orc.matmul(_np(x), _np(model[0].weight).T, bias=_np(model[0].bias), relu=True)
    ref = orc.matmul(h, _np(model[2].weight).T, bias=_np(model[2].bias))
    assert_close(_np(y), ref, 1e-4, "compiled MLP f32")
    assert backend.last_jit_function.kinds == ["hip.gemm", "hip.gemm"]


def _block_params(m: Block):
    t = lambda w: _np(w).T.copy()  # noqa: E731  Linear stores [out, in]; the oracle takes [in, out]
    return {
        "ln1_g": _np(m.ln_1.weight), "ln1_b": _np(m.ln_1.bias), "w_qkv": t(m.c_attn.weight), "b_qkv": _np(m.c_attn.bias),
        "w_o": t(m.c_proj.weight), "b_o": _np(m.c_proj.bias), "ln2_g": _np(m.ln_2.weight), "ln2_b": _np(m.ln_2.bias),
        "w_fc": t(m.c_fc.weight), "b_fc": _np(m.c_fc.bias), "w_proj": t(m.mlp_proj.weight), "b_proj": _np(m.mlp_proj.bias),
    }


def test_compiled_block_f32():
    from lighthouse_amd.ingress.torch import gpu_backend

    torch.manual_seed(1)
    B, T, C, H = 2, 128, 256, 4
    model = Block(C, H).cuda()
    with torch.no_grad():
        model.ln_1.weight.uniform_(0.5, 1.5)
        model.ln_2.bias.uniform_(-0.1, 0.1)
    x = torch.randn(B, T, C, device="cuda")
    backend = gpu_backend()
    compiled = torch.compile(model, backend=backend, dynamic=False)
    with torch.no_grad():
        y = compiled(x)
    ref = orc.nanogpt_block(_np(x), _block_params(model), H, mode="f32")
    assert_close(_np(y), ref, 1e-4, "compiled nanoGPT block f32")
    assert backend.last_jit_function.kinds.count("hip.gemm") == 4
    # second call reuses the cached transposed weights and gives the same result
    with torch.no_grad():
        assert torch.equal(compiled(x), y)


def test_compiled_block_bf16():
    """A bfloat16 module: every tensor bf16 (residual stream included), statistics and accumulators
    f32.  Reference: the oracle's operators chained with the same rounding points."""
    from lighthouse_amd.ingress.torch import gpu_backend

    torch.manual_seed(2)
    B, T, C, H = 2, 128, 256, 4
    model = Block(C, H).cuda().bfloat16()
    x = torch.randn(B, T, C, device="cuda").bfloat16()
    compiled = torch.compile(model, backend=gpu_backend(), dynamic=False)
    with torch.no_grad():
        y = compiled(x)
    assert y.dtype == torch.bfloat16
    p = _block_params(model)
    r = orc.round_bf16
    x2 = _np(x).reshape(B * T, C)
    ln1 = orc.layer_norm(x2, p["ln1_g"], p["ln1_b"], 1e-5, "bf16")
    qkv = orc.matmul(ln1, p["w_qkv"], bias=p["b_qkv"], result_type="bf16").reshape(B, T, 3, H, C // H)
    q, k, v = (qkv[:, :, i].transpose(0, 2, 1, 3) for i in range(3))
    att = orc.attention(q, k, v, causal=True, result_type="bf16")
    att = att.transpose(0, 2, 1, 3).reshape(B * T, C)
    a = r(x2 + orc.matmul(att, p["w_o"], bias=p["b_o"], result_type="bf16"))
    ln2 = orc.layer_norm(a, p["ln2_g"], p["ln2_b"], 1e-5, "bf16")
    h = orc.matmul(ln2, p["w_fc"], bias=p["b_fc"], gelu=True, result_type="bf16")
    ref = r(a + orc.matmul(h, p["w_proj"], bias=p["b_proj"], result_type="bf16")).reshape(B, T, C)
    assert_close(_np(y), ref, 2e-2, "compiled nanoGPT block bf16")


def test_jit_function_benchmark_protocol():
    from lighthouse_amd.ingress.torch import gpu_backend

    model = nn.Sequential(nn.Linear(128, 128), nn.ReLU()).cuda()
    x = torch.randn(128, 128, device="cuda")
    backend = gpu_backend()
    jit = backend(torch.fx.symbolic_trace(model), [x])
    out = jit(x)
    assert isinstance(out, list) and len(out) == 1 and out[0].shape == (128, 128)
    times = jit.benchmark(x, nruns=5, nwarmup=2)
    assert times.shape == (5,) and times.dtype == np.float64 and (times > 0).all()
    with pytest.raises(ValueError):
        jit(x.cpu())


@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
def test_compiled_matmul_nodes(dtype, rtol):
    """Plain matmul graph nodes (torch.matmul, `@` on a transposed weight view, addmm, a 3-D left
    operand): each runs as one GEMM, transposed views as transpose flags; integer-valued operands make
    the f32 chain exact."""
    from lighthouse_amd.ingress.torch import gpu_backend

    class M(nn.Module):
        def __init__(self, w, b):
            super().__init__()
            self.w, self.b = nn.Parameter(w), nn.Parameter(b)

        def forward(self, x, y):
            h = torch.relu(torch.matmul(x, y))            # [3, 40, 96] @ [96, 64], ReLU fused
            h = h @ self.w.t()                             # w [128, 64] read as its transpose
            return torch.addmm(self.b, h.flatten(0, 1), self.w)   # [120, 128] @ [128, 64] + b

    g = torch.Generator().manual_seed(5)
    ints = lambda *shape: torch.randint(-2, 3, shape, generator=g).float()  # noqa: E731
    x, y, w, b = ints(3, 40, 96), ints(96, 64), ints(128, 64), ints(64)
    model = M(w.clone(), b.clone()).cuda().to(dtype)
    backend = gpu_backend()
    compiled = torch.compile(model, backend=backend, dynamic=False)
    with torch.no_grad():
        out = compiled(x.cuda().to(dtype), y.cuda().to(dtype))
    assert backend.last_jit_function.kinds == ["hip.gemm", "hip.gemm", "hip.gemm"]
    assert out.shape == (120, 64) and out.dtype == dtype
    rt = "f32" if dtype == torch.float32 else "bf16"
    h = orc.matmul(_np(x).reshape(120, 96), _np(y), relu=True, result_type=rt)
    h = orc.matmul(h, _np(w).T, result_type=rt)
    ref = orc.matmul(h, _np(w), bias=_np(b), result_type=rt)
    if dtype == torch.float32:
        np.testing.assert_array_equal(_np(out), ref)
    else:
        assert_close(_np(out), ref, rtol, "compiled matmul nodes bf16")


def test_reference_compile_model_examples():
    """The three flows of the reference's torch-ingress examples at their own shapes and pass criteria:
    a decorated matmul model called with two input shapes, each of which gets its own specialisation
    (examples/ingress/torch/compile_model.py:60-107: [8,16] @ [16,4], then [2,4] @ [4,16], allclose
    rtol = atol = 1e-3), `model.compile(...)` on a Linear(16, 8) with batch 2 (:113-142, rtol = atol =
    1e-2), and the MLP of examples/ingress/torch/MLPModel/model.py (Linear(10, 32), ReLU, Linear(32, 2)
    on a [1, 10] input)."""
    from lighthouse_amd.ingress.torch import gpu_backend

    backend = gpu_backend()

    @torch.compile(dynamic=False, backend=backend)
    class Model(nn.Module):
        def forward(self, a, b):
            return torch.matmul(a, b)

    torch.manual_seed(0)
    model = Model()
    for shape_a, shape_b in (((8, 16), (16, 4)), ((2, 4), (4, 16))):
        a, b = torch.randn(shape_a, device="cuda"), torch.randn(shape_b, device="cuda")
        out = model(a, b)
        assert backend.last_jit_function.kinds == ["hip.gemm"]
        assert out.shape == (shape_a[0], shape_b[1])
        assert torch.allclose(torch.matmul(a.cpu(), b.cpu()), out.cpu(), rtol=0.001, atol=0.001)

    linear = nn.Sequential(nn.Linear(16, 8)).cuda()
    x = torch.randn(2, 16, device="cuda")
    with torch.no_grad():
        out_ref = linear(x)
        linear.compile(dynamic=False, backend=backend)
        out = linear(x)
    assert backend.last_jit_function.kinds == ["hip.gemm"]
    assert torch.allclose(out_ref, out, rtol=0.01, atol=0.01)
    assert_close(_np(out), orc.matmul(_np(x), _np(linear[0].weight).T, bias=_np(linear[0].bias)), 1e-4, "Linear(16, 8)")

    mlp = nn.Sequential(nn.Linear(10, 32), nn.ReLU(), nn.Linear(32, 2)).cuda()
    x = torch.randn(1, 10, device="cuda")
    compiled = torch.compile(mlp, backend=backend, dynamic=False)
    with torch.no_grad():
        out = compiled(x)
    assert backend.last_jit_function.kinds == ["hip.gemm", "hip.gemm"]
    h = orc.matmul(_np(x), _np(mlp[0].weight).T, bias=_np(mlp[0].bias), relu=True)
    assert_close(_np(out), orc.matmul(h, _np(mlp[2].weight).T, bias=_np(mlp[2].bias)), 1e-4, "MLPModel")


def test_reference_torch_matmul_example():
    """examples/xegpu/torch_matmul.py: an f16 matmul model with per-layer schedule parameters handed
    to the backend through `fn_compile`, `model.compile(dynamic=False, backend=...)`, the result
    checked with allclose rtol = atol = 1e-2 (:291-296), then `backend.jit_function.benchmark(a, b,
    nruns, nwarmup)` (:299-305).  Here on 2048^3 with the workgroup tile as the parameter that acts;
    parameters for another problem size are refused when the layer runs."""
    from lighthouse_amd.ingress.torch import gpu_backend, with_schedule_parameters

    class Model(nn.Module):
        def forward(self, A, B):
            return torch.matmul(A, B)

    m = n = k = 2048
    torch.manual_seed(0)
    a = torch.randn(m, k, device="cuda", dtype=torch.float16)
    b = torch.randn(k, n, device="cuda", dtype=torch.float16)
    from lighthouse_amd.schedule import ScheduleParameters

    params = ScheduleParameters([{"layer_kind": "matmul", "m": m, "n": n, "k": k}])
    params[0]["wg_m"], params[0]["wg_n"] = 256, 128      # (as the example's --wg-tile argument does, :237-238)
    backend = gpu_backend(with_schedule_parameters(params), device=torch.device("cuda"))
    model = Model()
    model.compile(dynamic=False, backend=backend)
    out = model(a, b)
    assert backend.jit_function.kinds == ["hip.gemm"]
    rows = [0, 777, m - 1]
    ref = orc.matmul(_np(a[rows]), _np(b), result_type="f16")
    assert torch.allclose(torch.from_numpy(ref).to(torch.float16), out[rows].cpu(), rtol=0.01, atol=0.01)
    assert_close(_np(out[rows]), ref, 2e-2, "torch_matmul example f16 2048^3")
    unrequested = gpu_backend()
    plain = torch.compile(Model(), backend=unrequested, dynamic=False)(a, b)
    assert torch.equal(plain, out)                      # another tile, the same sums in the same order of k
    times = backend.jit_function.benchmark(a, b, nruns=5, nwarmup=2)
    assert times.shape == (5,) and (times > 0).all()
    wrong = gpu_backend(with_schedule_parameters([{"m": 64, "n": 64, "k": 64, "wg_m": 128, "wg_n": 128}]))
    with pytest.raises(ValueError, match="64x64x64"):
        torch.compile(Model(), backend=wrong, dynamic=False)(a, b)
    # parameters chosen for a transposed operand on a layer whose operand is not: refused as well;
    # with the flags the layer has they pass (the selector writes them)
    from lighthouse_amd.schedule import HipParameterSelector

    sel = HipParameterSelector().get_parameters((m, n, k), transpose_a=False, transpose_b=False)
    ok = gpu_backend(with_schedule_parameters(sel), device=torch.device("cuda"))
    assert torch.equal(torch.compile(Model(), backend=ok, dynamic=False)(a, b), out)
    tb = gpu_backend(with_schedule_parameters([{"m": m, "n": n, "k": k, "transpose_b": True}]))
    with pytest.raises(ValueError, match="transpose_b=True"):
        torch.compile(Model(), backend=tb, dynamic=False)(a, b)
