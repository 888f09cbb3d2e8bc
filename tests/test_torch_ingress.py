"""Lowering of FX graphs to HIP kernel plans (no GPU needed: plans are built, not run).

Contract mirrored: lighthouse/ingress/torch/compile.py:154-496 (backend callable, static shapes,
JITFunction) and examples/ingress/torch/compile_model.py:60-140 (how the backend is driven).
"""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from lighthouse_amd.ingress.torch import JITFunction, gpu_backend


class Block(nn.Module):
    """GPT-2 block written the nanoGPT way (fused QKV Linear, SDPA, tanh-GELU MLP)."""

    def __init__(self, C=64, H=4):
        super().__init__()
        self.ln_1, self.ln_2 = nn.LayerNorm(C), nn.LayerNorm(C)
        self.c_attn, self.c_proj = nn.Linear(C, 3 * C), nn.Linear(C, C)
        self.c_fc, self.mlp_proj = nn.Linear(C, 4 * C), nn.Linear(4 * C, C)
        self.H = H

    def forward(self, x):
        B, T, C = x.size()
        q, k, v = self.c_attn(self.ln_1(x)).split(C, dim=2)
        q, k, v = (t.view(B, T, self.H, C // self.H).transpose(1, 2) for t in (q, k, v))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.c_proj(y.transpose(1, 2).contiguous().view(B, T, C))
        return x + self.mlp_proj(F.gelu(self.c_fc(self.ln_2(x)), approximate="tanh"))


def test_mlp_plan_fuses_activations():
    model = nn.Sequential(nn.Linear(8, 16), nn.ReLU(), nn.Linear(16, 4), nn.GELU(approximate="tanh"))
    jit = gpu_backend()(torch.fx.symbolic_trace(model), [torch.randn(2, 8)])
    assert isinstance(jit, JITFunction)
    assert jit.kinds == ["hip.gemm", "hip.gemm"]
    gemms = [s for s in jit.plan if s.kind == "hip.gemm"]
    assert [g.detail["activation"] for g in gemms] == ["relu", "gelu"]
    assert all(g.detail["bias"] for g in gemms)


def test_activation_with_second_user_is_not_fused():
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(8, 8)

        def forward(self, x):
            h = self.fc(x)
            return F.relu(h) + h

    jit = gpu_backend()(torch.fx.symbolic_trace(M()), [torch.randn(2, 8)])
    assert jit.kinds == ["hip.gemm", "hip.relu", "hip.add"]


def test_residual_add_is_fused_only_when_the_residual_exists_before_the_linear():
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc, self.ln = nn.Linear(8, 8), nn.LayerNorm(8)

        def forward(self, x):
            early = self.ln(x)
            a = early + self.fc(x)      # residual computed before the linear: one GEMM
            h = self.fc(a)
            late = self.ln(a)           # computed after the linear it is added to: a separate add
            return h + late

    jit = gpu_backend()(torch.fx.symbolic_trace(M()), [torch.randn(2, 8)])
    assert jit.kinds == ["hip.layer_norm", "hip.gemm", "hip.gemm", "hip.layer_norm", "hip.add"]
    assert [s.detail["residual"] for s in jit.plan if s.kind == "hip.gemm"] == [True, False]


def test_block_plan_through_dynamo():
    backend = gpu_backend()
    compiled = torch.compile(Block(), backend=backend, dynamic=False)
    with pytest.raises(ValueError, match="compiled for cuda"):  # the plan exists; running needs the GPU
        with torch.no_grad():
            compiled(torch.randn(2, 8, 64))
    # both residual adds start the accumulation of the projection GEMM in front of them
    assert backend.last_jit_function.kinds == [
        "hip.layer_norm", "hip.gemm", "hip.attention", "hip.gemm",
        "hip.layer_norm", "hip.gemm", "hip.gemm"]
    gemms = [s for s in backend.last_jit_function.plan if s.kind == "hip.gemm"]
    assert [g.detail["residual"] for g in gemms] == [False, True, False, True]
    assert [g.detail["activation"] for g in gemms] == [None, None, "gelu", None]
    attn = next(s for s in backend.last_jit_function.plan if s.kind == "hip.attention")
    assert attn.detail["causal"] is True


def test_unsupported_compute_node_is_an_error():
    model = nn.Sequential(nn.Linear(8, 16), nn.Sigmoid())
    with pytest.raises(ValueError, match="no HIP kernel"):
        gpu_backend()(torch.fx.symbolic_trace(model), [torch.randn(2, 8)])
    jit = gpu_backend(allow_torch_fallback=True)(torch.fx.symbolic_trace(model), [torch.randn(2, 8)])
    assert jit.kinds == ["hip.gemm", "torch.Sigmoid"]


def test_unsupported_attention_arguments():
    class M(nn.Module):
        def forward(self, q, k, v, m):
            return F.scaled_dot_product_attention(q, k, v, attn_mask=m)

    with pytest.raises(ValueError, match="masks"):
        gpu_backend()(torch.fx.symbolic_trace(M()), [torch.randn(1, 1, 4, 4)] * 4)


def test_fn_compile_hook_and_device_check():
    seen = []

    def fn_compile(plan):
        seen.extend(s.kind for s in plan)
        return plan

    gpu_backend(fn_compile)(torch.fx.symbolic_trace(nn.Linear(4, 4)), [torch.randn(1, 4)])
    assert "hip.gemm" in seen
    with pytest.raises(AssertionError):
        gpu_backend(device="cpu")


def test_argument_resolvers_follow_nested_structures():
    """Arguments are resolved by functions built at lowering time: nodes inside tuples, lists,
    dicts and slices are looked up in the environment, anything else is passed through as it is."""
    from lighthouse_amd.ingress.torch.compile import _Ref, _resolver

    env = {"a": 3, "b": 5}
    a, b = _Ref("a"), _Ref("b")
    assert _resolver(a)(env) == 3
    assert _resolver((a, [b, 7], {"k": a}, slice(a, None, b)))(env) == (3, [5, 7], {"k": 3}, slice(3, None, 5))
    const = (1, [2, 3], {"k": None}, slice(0, 4))
    assert _resolver(const)(env) is const  # no node inside: returned without a walk
    assert _resolver(None)(env) is None


def test_plain_matmul_nodes_become_gemms():
    """torch.matmul / `@` / mm / addmm with a 2-D right operand (the form of the KernelBench level-1
    problems the reference's backend is driven with, tools/kernel-bench:443-452): one GEMM each,
    a following ReLU fused; a batched right operand is refused when the plan runs."""

    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.w = nn.Parameter(torch.randn(16, 8))
            self.b = nn.Parameter(torch.randn(16))

        def forward(self, x, y):
            h = torch.relu(torch.matmul(x, y))   # [4, 8] @ [8, 8]
            h = h @ self.w.t()                   # transposed view of a row-major weight
            h = torch.addmm(self.b, h, torch.mm(self.w, self.w.t()))
            return h.matmul(self.w)

    jit = gpu_backend()(torch.fx.symbolic_trace(M()), [torch.randn(4, 8), torch.randn(8, 8)])
    assert jit.kinds == ["hip.gemm"] * 5
    gemms = [s for s in jit.plan if s.kind == "hip.gemm"]
    assert [g.detail["activation"] for g in gemms] == ["relu", None, None, None, None]
    assert [g.detail["bias"] for g in gemms] == [False, False, False, True, False]

    class Scaled(nn.Module):
        def forward(self, x, y):
            return torch.addmm(x, x, y, beta=0.5)

    with pytest.raises(ValueError, match="addmm"):
        gpu_backend()(torch.fx.symbolic_trace(Scaled()), [torch.randn(4, 4), torch.randn(4, 4)])


def test_schedule_parameters_reach_the_gemm_steps():
    """Per-layer schedule parameters (the dictionaries of the reference's ScheduleParameters) set the
    tile / K-cut request of the graph's GEMMs in order; keys without a counterpart, a wrong count and
    a lone wg_m are errors; `backend.jit_function` raises before the first compilation."""
    from lighthouse_amd.ingress.torch import gpu_backend, with_schedule_parameters
    from lighthouse_amd.ingress.torch.compile import _Lowering

    with pytest.raises(ValueError, match="Compile the torch model first"):
        gpu_backend().jit_function
    model = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 8))
    gm = torch.fx.symbolic_trace(model)
    _, plan, _ = _Lowering(gm, False).lower()
    fn = with_schedule_parameters([{"layer_kind": "matmul", "m": 4, "n": 32, "k": 16, "wg_m": 128, "wg_n": 128},
                                   {"split_k": 2}])
    plan = fn(plan)
    gemms = [st for st in plan if st.kind == "hip.gemm"]
    assert gemms[0].detail["schedule"] == {"tile": (128, 128), "mnk": (4, 32, 16)}
    assert gemms[1].detail["schedule"] == {"split_k": 2}
    with pytest.raises(ValueError, match="no counterpart"):
        with_schedule_parameters([{"wg_m": 256, "wg_n": 256, "sg_m": 32}])
    with pytest.raises(ValueError, match="come together"):
        with_schedule_parameters([{"wg_m": 256}])
    with pytest.raises(ValueError, match="2 matmul layers"):
        with_schedule_parameters([{"wg_m": 256, "wg_n": 256}])(_Lowering(gm, False).lower()[1])
