"""LayerNorm, softmax, GELU and the elementwise kernels on the GPU vs the CPU oracle."""

import numpy as np
import pytest
import torch

from oracle import lh_oracle as orc
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu


def _dev(x, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to("cuda").to(dtype)


def _host(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize("shape", [(64, 768), (8192, 768), (33, 1024), (7, 100), (5, 3072), (3, 5000), (1, 1)])
def test_layer_norm_f32(shape):
    from lighthouse_amd import ops

    # Inputs of the reference workload: examples/xegpu/layer_norm.py:106-114
    np.random.seed(42)
    x = np.random.uniform(-1.0, 1.0, shape).astype(np.float32)
    g = np.random.uniform(0.5, 1.5, shape[1:]).astype(np.float32)
    b = np.random.uniform(-0.1, 0.1, shape[1:]).astype(np.float32)
    out = ops.layer_norm(_dev(x), _dev(g), _dev(b), 1e-5)
    assert_close(_host(out), orc.layer_norm(x, g, b, 1e-5), 1e-4, f"layer_norm {shape}")


@pytest.mark.parametrize("shape", [(100, 50000), (64, 8192), (33, 5001), (7, 1026), (3, 50257), (300, 1280)])
@pytest.mark.parametrize("elt", ["f32", "bf16"])
def test_long_rows_one_workgroup_per_row(shape, elt):
    """Rows that do not stay in a wave's registers: LayerNorm and softmax with one workgroup per row,
    vector accesses when the row length and alignment allow (N % 4 == 0), scalar otherwise."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(shape[0] + shape[1])
    dt = torch.float32 if elt == "f32" else torch.bfloat16
    x = orc.round_to(rng.standard_normal(shape).astype(np.float32) * 2 + 0.5, elt)
    g = rng.uniform(0.5, 1.5, shape[1:]).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, shape[1:]).astype(np.float32)
    out = ops.layer_norm(_dev(x, dt), _dev(g), _dev(b), 1e-5)
    rtol = 1e-4 if elt == "f32" else 2e-2
    assert_close(_host(out), orc.layer_norm(x, g, b, 1e-5, result_type=elt), rtol, f"layer_norm {shape} {elt}")
    sm = _host(ops.softmax(_dev(x, dt)))
    ref = orc.softmax(x, result_type=elt)
    if elt == "f32":
        assert np.allclose(sm.sum(1), 1.0, rtol=1e-5, atol=1e-6)
        assert np.allclose(sm, ref, rtol=1e-4, atol=1e-6)
    else:
        assert_close(sm, ref, 2e-2, f"softmax {shape} bf16")


@pytest.mark.parametrize(
    "shape", [(777, 64), (513, 260), (1030, 384), (300, 640), (257, 896), (129, 1000), (66, 1152), (35, 1284),
              (34, 2560), (9, 3332), (6, 3584), (5, 4092)]
)
@pytest.mark.parametrize("elt", ["f32", "bf16"])
def test_rows_of_whole_vector_groups_stay_in_registers(shape, elt):
    """Row lengths that are multiples of 4 but not of 256 (or an uncommon multiple): one wave per row
    with the tail groups masked. Row counts are not multiples of 4 so the last workgroup is partial."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    dt = torch.float32 if elt == "f32" else torch.bfloat16
    x = orc.round_to(rng.standard_normal(shape).astype(np.float32) * 2 - 0.75, elt)
    g = rng.uniform(0.5, 1.5, shape[1:]).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, shape[1:]).astype(np.float32)
    # The output buffer is one row longer than the result and pre-filled: nothing past the end may change.
    m, n = shape
    buf = torch.full((m + 1, n), 123.0, device="cuda", dtype=dt)
    out = ops.layer_norm(_dev(x, dt), _dev(g), _dev(b), 1e-5, out=buf[:m])
    rtol = 1e-4 if elt == "f32" else 2e-2
    assert_close(_host(out), orc.layer_norm(x, g, b, 1e-5, result_type=elt), rtol, f"layer_norm {shape} {elt}")
    assert torch.all(buf[m] == 123.0)
    buf.fill_(123.0)
    sm = _host(ops.softmax(_dev(x, dt), out=buf[:m]))
    assert torch.all(buf[m] == 123.0)
    ref = orc.softmax(x, result_type=elt)
    if elt == "f32":
        assert np.allclose(sm.sum(1), 1.0, rtol=1e-5, atol=1e-6)
        assert np.allclose(sm, ref, rtol=1e-4, atol=1e-6)
    else:
        assert_close(sm, ref, 2e-2, f"softmax {shape} bf16")


def test_layer_norm_bf16_out_and_in():
    from lighthouse_amd import ops

    rng = np.random.default_rng(1)
    x = rng.standard_normal((512, 768)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 768).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, 768).astype(np.float32)
    out = ops.layer_norm(_dev(x), _dev(g), _dev(b), out_dtype=torch.bfloat16)
    assert_close(_host(out), orc.layer_norm(x, g, b, result_type="bf16"), 2e-2, "ln f32->bf16")
    xb = orc.round_bf16(x)
    out = ops.layer_norm(_dev(xb, torch.bfloat16), _dev(g), _dev(b))
    assert_close(_host(out), orc.layer_norm(xb, g, b, result_type="bf16"), 2e-2, "ln bf16->bf16")


def test_layer_norm_f16_out():
    """f32 rows to f16: the LayerNorm + cast_f16 pair of the reference's block
    (examples/xegpu/nanoGPT_payload.py:305-306)."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(2)
    for M, N in ((256, 256), (100, 768), (33, 1000)):
        x = rng.standard_normal((M, N)).astype(np.float32)
        g = rng.uniform(0.5, 1.5, N).astype(np.float32)
        b = rng.uniform(-0.1, 0.1, N).astype(np.float32)
        out = ops.layer_norm(_dev(x), _dev(g), _dev(b), out_dtype=torch.float16)
        assert out.dtype == torch.float16
        assert_close(_host(out), orc.layer_norm(x, g, b, result_type="f16"), 2e-3, f"ln f32->f16 {M}x{N}")


def test_layer_norm_special_cases():
    from lighthouse_amd import ops

    # Constant rows normalise to beta exactly when the row sum and 1/N are exact (N a power of two).
    n = 1024
    x = torch.full((16, n), 3.25, device="cuda")
    beta = torch.linspace(-1, 1, n, device="cuda")
    assert torch.equal(ops.layer_norm(x, torch.ones(n, device="cuda"), beta), beta.expand(16, n))
    n = 768
    ones, zeros = torch.ones(n, device="cuda"), torch.zeros(n, device="cuda")
    # gamma = 1, beta = 0: zero mean, unit variance rows.
    y = ops.layer_norm(torch.randn(64, n, device="cuda") * 5 + 2, ones, zeros)
    assert y.mean(1).abs().max() < 1e-5
    assert (y.var(1, unbiased=False) - 1).abs().max() < 1e-3


@pytest.mark.parametrize("shape", [(64, 1024), (5, 77), (128, 4096), (33, 768), (16, 8192), (7, 260)])
def test_softmax(shape):
    from lighthouse_amd import ops

    rng = np.random.default_rng(4)
    x = rng.standard_normal(shape).astype(np.float32) * 3
    out = _host(ops.softmax(_dev(x)))
    ref = orc.softmax(x)
    # examples/xegpu/softmax.py:62-66 tolerances
    assert np.allclose(out.sum(1), 1.0, rtol=1e-5, atol=1e-6)
    assert np.allclose(out, ref, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("dtype,elt,rtol", [(torch.float32, "f32", 1e-4), (torch.bfloat16, "bf16", 2e-2)])
def test_gelu(dtype, elt, rtol):
    from lighthouse_amd import ops

    x = orc.round_to(np.linspace(-12, 12, 8192 * 3 + 5, dtype=np.float32), elt)
    out = ops.gelu_tanh(_dev(x, dtype))
    assert_close(_host(out), orc.gelu_tanh(x, elt), rtol, f"gelu {elt}")


def test_gelu_all_bf16_inputs():
    """Every finite bf16 value through the standalone kernel."""
    from lighthouse_amd import ops

    bits = np.arange(65536, dtype=np.uint16)
    x = orc.bf16_bits_to_f32(bits)
    keep = np.isfinite(x)
    xs = x[keep]
    out = ops.gelu_tanh(torch.from_numpy(xs).cuda().to(torch.bfloat16))
    ref = orc.gelu_tanh(xs, "bf16")
    got = _host(out)
    # Below ~1e-12 the oracle's own 1 + tanh(u) cancels in f64 (eps / |1 + tanh u| exceeds the
    # tolerance), so those outputs are compared absolutely.
    ok = np.isclose(got, ref, rtol=2e-2, atol=1e-12)
    assert ok.all(), f"{(~ok).sum()} mismatches, first at x={xs[~ok][0]}"


def test_elementwise_kernels():
    from lighthouse_amd import ops

    rng = np.random.default_rng(6)
    x = rng.standard_normal((300, 257)).astype(np.float32)
    y = rng.standard_normal((300, 257)).astype(np.float32)
    bias = rng.standard_normal(257).astype(np.float32)
    np.testing.assert_array_equal(_host(ops.add(_dev(x), _dev(y))), orc.residual_add(x, y))
    np.testing.assert_array_equal(_host(ops.bias_act(_dev(x), _dev(bias))), orc.bias_act(x, bias))
    np.testing.assert_array_equal(_host(ops.bias_act(_dev(x), _dev(bias), relu=True)), orc.bias_act(x, bias, relu=True))
    x4 = rng.standard_normal((64, 768)).astype(np.float32)
    b4 = rng.standard_normal(768).astype(np.float32)
    np.testing.assert_array_equal(_host(ops.bias_act(_dev(x4), _dev(b4), relu=True)), orc.bias_act(x4, b4, relu=True))


def test_cast_all_patterns():
    """f32 -> bf16 on values around every bf16 rounding boundary, and bf16 -> f32 on all codes."""
    from lighthouse_amd import ops

    bits = np.arange(65536, dtype=np.uint16)
    as_f32 = orc.bf16_bits_to_f32(bits)
    up = ops.cast(torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16), torch.float32)
    got = up.cpu().numpy()
    fin = np.isfinite(as_f32)
    np.testing.assert_array_equal(got[fin], as_f32[fin])
    rng = np.random.default_rng(9)
    u = rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    # Force many exact ties and near-ties.
    u[::4] = (u[::4] & 0xFFFF0000) | 0x8000
    u[1::4] = (u[1::4] & 0xFFFF0000) | 0x7FFF
    x = u.view(np.float32)
    x = x[np.isfinite(x)]
    down = ops.cast(torch.from_numpy(x).cuda(), torch.bfloat16)
    np.testing.assert_array_equal(down.view(torch.int16).cpu().numpy().view(np.uint16), orc.f32_to_bf16_bits(x))
