"""Pins the CPU oracle: every oracle function is checked against something it does not share
code with -- the reference's own golden vector, a library routine (torch on the CPU), a closed
form, or brute force -- chosen so that a dropped term, a wrong sign, index or transposed
operand fails at least one check.  Runs without a GPU."""

import ctypes
import json
import math
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import lh_oracle as orc

ROOT = Path(__file__).resolve().parent.parent
GOLDEN = json.loads((Path(__file__).parent / "golden" / "lh_run_pipeline_check.json").read_text())


@pytest.fixture(scope="module")
def cref():
    path = ROOT / "oracle" / "_build" / "libcpu_ref.so"
    if not path.is_file():
        from oracle import build as oracle_build

        oracle_build.build()
    return ctypes.CDLL(str(path))


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


# ---- lh-run protocol + matmul: the reference's known-answer test -------------------------


def test_lh_run_golden_numpy_oracle():
    """test/run/pipeline-check.mlir:1,16-31: seed 123, `16x64xf32xrnd,64x32xf32x1,16x32xf32x0`."""
    a, b, c = orc.lh_run_inputs(GOLDEN["input_shape"], GOLDEN["seed"])
    out = orc.matmul(a, b, c, accumulate_c=True)
    assert out.shape == (16, 32)
    # The oracle sums in float64 and rounds once; the golden was summed in float32 by the
    # reference's loop nest (64 sequential additions), so the two differ by a few float32 ulps.
    gold = np.array(GOLDEN["row_values"], np.float32)
    assert np.abs(out[:, 0] - gold).max() <= 4 * np.spacing(np.float32(32.0))
    assert (out == out[:, :1]).all()


def test_lh_run_golden_c_oracle(cref):
    a, b, c = orc.lh_run_inputs(GOLDEN["input_shape"], GOLDEN["seed"])
    out = c.copy()
    cref.lhref_matmul_f32(_p(out), _p(a), _p(b), None, ctypes.c_int64(16), ctypes.c_int64(32), ctypes.c_int64(64),
                          ctypes.c_uint32(4), ctypes.c_int(1))
    # Same loop order and float32 accumulation as the reference's lowering: the printed text
    # (numpy's shortest float32 repr, as lh-run prints it) matches digit for digit.
    printed = [np.format_float_positional(np.float32(v), unique=True) for v in out[:, 0]]
    expected = [np.format_float_positional(np.float32(v), unique=True) for v in GOLDEN["row_values"]]
    assert printed == expected
    assert (out == out[:, :1]).all()


def test_lh_run_input_protocol_details():
    a1, = orc.lh_run_inputs("4x4xf32xid", 1)
    np.testing.assert_array_equal(a1, np.eye(4, dtype=np.float32))
    x, y = orc.lh_run_inputs("3x5xf32xrnd,2x2xf64xrnd", 7)
    np.random.seed(7)
    np.testing.assert_array_equal(x, np.random.rand(3, 5).astype(np.float32))
    np.testing.assert_array_equal(y, np.random.rand(2, 2))


# ---- narrow formats ------------------------------------------------------------------------


def test_bf16_rounding_matches_torch_on_boundaries():
    rng = np.random.default_rng(0)
    u = rng.integers(0, 2**32, 1 << 18, dtype=np.uint64).astype(np.uint32)
    u[::4] = (u[::4] & 0xFFFF0000) | 0x8000   # exact ties
    u[1::4] = (u[1::4] & 0xFFFF0000) | 0x7FFF  # just below a tie
    u[2::4] = (u[2::4] & 0xFFFF0000) | 0x8001  # just above a tie
    x = u.view(np.float32)
    x = x[np.isfinite(x)]
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(orc.f32_to_bf16_bits(x), ref)
    bits = np.arange(65536, dtype=np.uint16)
    back = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    got = orc.bf16_bits_to_f32(bits)
    fin = np.isfinite(back)
    np.testing.assert_array_equal(got[fin], back[fin])
    assert np.isnan(orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(np.array([np.nan], np.float32)))).all()


def test_e4m3_table_and_quantisation_match_torch():
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = orc.e4m3_decode_table()
    np.testing.assert_array_equal(np.isnan(got), np.isnan(ref))
    np.testing.assert_array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)])
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(1 << 16).astype(np.float32) * 100,
                        rng.uniform(-448, 448, 1 << 16).astype(np.float32),
                        (got[:127, None] + got[1:128, None]).ravel() / 2])  # all midpoints: ties
    x = x[np.abs(x) <= 448]
    tq = torch.from_numpy(x.astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    oq = orc.e4m3_quant(x.astype(np.float32))
    # +0 / -0 both decode to zero; compare decoded values.
    np.testing.assert_array_equal(got[oq], got[tq])
    # Saturation beyond the largest finite value.
    np.testing.assert_array_equal(got[orc.e4m3_quant(np.array([1e6, -1e6, 449.0], np.float32))], [448, -448, 448])
    q, s = orc.quantize_per_tensor_e4m3(np.array([[1.0, -2.0], [0.5, 4.0]], np.float32))
    assert s == np.float32(4.0 / 448.0) and got[q].max() == 448.0


# ---- matmul payload ------------------------------------------------------------------------


@pytest.mark.parametrize("flags", ["plain", "bias", "bias_relu", "acc", "ta", "tb"])
def test_matmul_against_torch(flags):
    rng = np.random.default_rng(3)
    M, N, K = 37, 29, 53
    a = rng.standard_normal((K, M) if flags == "ta" else (M, K)).astype(np.float32)
    b = rng.standard_normal((N, K) if flags == "tb" else (K, N)).astype(np.float32)
    c = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ta, tb = torch.from_numpy(a).double(), torch.from_numpy(b).double()
    if flags == "ta":
        ta = ta.T
    if flags == "tb":
        tb = tb.T
    ref = ta @ tb
    kw = {}
    if flags in ("bias", "bias_relu"):
        ref = torch.addmm(torch.from_numpy(bias).double(), ta, tb)
        kw["bias"] = bias
    if flags == "bias_relu":
        ref = torch.relu(ref)
        kw["relu"] = True
    if flags == "acc":
        ref = ref + torch.from_numpy(c).double()
        kw.update(c=c, accumulate_c=True)
    out = orc.matmul(a, b, transpose_a=flags == "ta", transpose_b=flags == "tb", **kw)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-6, atol=1e-6)


def test_matmul_rounding_order_bias_convert_relu():
    """Bias is added in f32 BEFORE the conversion, ReLU AFTER it (gpu_mlp_payload.py:142-151):
    1 + 2^-9 survives only if the sum is formed before rounding to bf16."""
    a = np.array([[1.0]], np.float32)
    b = np.array([[1.0]], np.float32)
    bias = np.array([2.0 ** -8], np.float32)
    out = orc.matmul(a, b, bias=bias, result_type="bf16")
    assert out[0, 0] == np.float32(1.0 + 2.0 ** -7) or out[0, 0] == np.float32(1.0)  # RNE tie -> even (1.0)
    assert orc.matmul(a, b, bias=np.array([2.0 ** -7], np.float32), result_type="bf16")[0, 0] == np.float32(1.0078125)
    assert orc.matmul(a, -b, bias=np.array([0.5], np.float32), relu=True, result_type="bf16")[0, 0] == 0.0


def test_matmul_special_cases():
    rng = np.random.default_rng(4)
    a = orc.round_bf16(rng.standard_normal((16, 16)).astype(np.float32))
    np.testing.assert_array_equal(orc.matmul(a, np.eye(16, dtype=np.float32), result_type="bf16"), a)
    ai = rng.integers(-3, 4, (8, 12)).astype(np.float32)
    bi = rng.integers(-3, 4, (12, 5)).astype(np.float32)
    np.testing.assert_array_equal(orc.matmul(ai, bi, result_type="bf16"), ai @ bi)
    ref = orc.matmul_check_reference(np.zeros((8, 5), np.float32), ai, bi, None, accumulate_c=False, has_bias=False,
                                     has_relu=False)
    np.testing.assert_array_equal(ref, ai @ bi)


def test_c_oracle_matmul_matches_numpy_oracle(cref):
    rng = np.random.default_rng(5)
    M, N, K = 24, 40, 64
    a = orc.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    b = orc.round_bf16(rng.standard_normal((K, N)).astype(np.float32))
    bias = orc.round_bf16(rng.standard_normal(N).astype(np.float32))
    ab, bb, biasb = (orc.f32_to_bf16_bits(t) for t in (a, b, bias))
    out = np.zeros((M, N), np.uint16)
    cref.lhref_matmul_bf16(_p(out), _p(ab), _p(bb), _p(biasb), ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K),
                           ctypes.c_uint32(3), ctypes.c_int(2))
    ref = orc.matmul(a, b, bias=bias, relu=True, result_type="bf16")
    np.testing.assert_allclose(orc.bf16_bits_to_f32(out), ref, rtol=2 ** -7, atol=1e-6)
    o32 = np.zeros((M, N), np.float32)
    cref.lhref_matmul_f32(_p(o32), _p(a), _p(b), _p(bias), ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K),
                          ctypes.c_uint32(3), ctypes.c_int(1))
    np.testing.assert_allclose(o32, orc.matmul(a, b, bias=bias, relu=True), rtol=1e-5, atol=1e-5)


def test_fp8_matmul_oracle(cref):
    rng = np.random.default_rng(6)
    M, N, K = 16, 24, 48
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    aq, sa = orc.quantize_per_tensor_e4m3(a)
    bq, sb = orc.quantize_per_tensor_e4m3(b)
    ta = torch.from_numpy(aq).view(torch.float8_e4m3fn).double() * float(sa)
    tb = torch.from_numpy(bq).view(torch.float8_e4m3fn).double() * float(sb)
    ref = (ta @ tb).numpy()
    out = orc.matmul_fp8(aq, bq, sa, sb, result_type="f32")
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-6)
    # Quantisation error is what the 5e-2 tolerance of the benchmark is for.
    assert np.abs(out - a.astype(np.float64) @ b).max() / np.abs(a @ b).max() < 5e-2
    co = np.zeros((M, N), np.uint16)
    cref.lhref_matmul_fp8(_p(co), _p(aq), _p(bq), ctypes.c_float(sa), ctypes.c_float(sb), ctypes.c_int64(M),
                          ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int(1))
    np.testing.assert_allclose(orc.bf16_bits_to_f32(co), orc.matmul_fp8(aq, bq, sa, sb), rtol=2 ** -7, atol=1e-6)


# ---- attention -----------------------------------------------------------------------------


@pytest.mark.parametrize("causal", [False, True])
def test_attention_against_sdpa(causal):
    rng = np.random.default_rng(7)
    q, k, v = (rng.standard_normal((2, 3, 40, 16)).astype(np.float32) for _ in range(3))
    ref = F.scaled_dot_product_attention(*(torch.from_numpy(t).double() for t in (q, k, v)), is_causal=causal).numpy()
    np.testing.assert_allclose(orc.attention(q, k, v, causal=causal), ref, rtol=1e-5, atol=1e-6)
    # A scale other than the default must be honoured (guards a dropped scale).
    ref2 = F.scaled_dot_product_attention(*(torch.from_numpy(t).double() for t in (q, k, v)), is_causal=causal,
                                          scale=0.3).numpy()
    np.testing.assert_allclose(orc.attention(q, k, v, causal=causal, scale=0.3), ref2, rtol=1e-5, atol=1e-6)


def test_attention_closed_forms():
    rng = np.random.default_rng(8)
    q, k, v = (rng.standard_normal((33, 8)).astype(np.float32) for _ in range(3))
    np.testing.assert_allclose(orc.attention(q, np.zeros_like(k), v), np.broadcast_to(v.mean(0), v.shape), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(orc.attention(q, k, np.full_like(v, 2.5)), np.full_like(v, 2.5), rtol=1e-5)
    np.testing.assert_array_equal(orc.attention(q, k, v, causal=True)[0], v[0])
    perm = rng.permutation(33)
    np.testing.assert_allclose(orc.attention(q, k[perm], v[perm]), orc.attention(q, k, v), rtol=1e-5, atol=1e-6)
    # Brute force, causal, scalar loops.
    out = orc.attention(q, k, v, causal=True)
    for i in (1, 17, 32):
        w = np.array([math.exp(float(q[i] @ k[j]) / math.sqrt(8)) for j in range(i + 1)])
        np.testing.assert_allclose(out[i], (w[:, None] * v[: i + 1]).sum(0) / w.sum(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("tile", [8, 16, 64, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_online_softmax_recurrence_is_tile_independent(tile, causal):
    """The tiled recurrence (replace_with_fused_attention.py:366-455) equals the one-shot form
    up to the declared rounding of P, for every tile size."""
    rng = np.random.default_rng(9)
    q, k, v = (orc.round_bf16(rng.standard_normal((128, 32)).astype(np.float32)) for _ in range(3))
    exact = orc.attention(q, k, v, causal=causal)
    got32 = orc.attention_online(q, k, v, tile=tile, causal=causal, elt="f32")
    np.testing.assert_allclose(got32, exact, rtol=2e-5, atol=2e-6)
    got16 = orc.attention_online(q, k, v, tile=tile, causal=causal, elt="bf16")
    assert np.abs(got16 - exact).max() <= 2e-2 * np.abs(exact).max()


def test_c_oracle_attention(cref):
    rng = np.random.default_rng(10)
    BH, T, d = 3, 48, 16
    q, k, v = (rng.standard_normal((BH, T, d)).astype(np.float32) for _ in range(3))
    for causal in (0, 1):
        out = np.zeros_like(q)
        cref.lhref_attention(_p(out), _p(q), _p(k), _p(v), ctypes.c_int64(BH), ctypes.c_int64(T), ctypes.c_int64(d),
                             ctypes.c_float(0.25), ctypes.c_int(causal), ctypes.c_int(0), ctypes.c_int(2))
        np.testing.assert_allclose(out, orc.attention(q, k, v, causal=bool(causal)), rtol=2e-5, atol=2e-6)


# ---- row-wise payloads --------------------------------------------------------------------


def test_layer_norm_against_torch_and_special_cases(cref):
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, (19, 96)).astype(np.float32) * 3 + 1
    g = rng.uniform(0.5, 1.5, 96).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, 96).astype(np.float32)
    ref = F.layer_norm(torch.from_numpy(x).double(), (96,), torch.from_numpy(g).double(), torch.from_numpy(b).double(),
                       1e-5).numpy()
    np.testing.assert_allclose(orc.layer_norm(x, g, b, 1e-5), ref, rtol=1e-6, atol=1e-6)
    # eps matters: a wrong eps shows on low-variance rows.
    xs = (x * 1e-3).astype(np.float32)
    ref = F.layer_norm(torch.from_numpy(xs).double(), (96,), None, None, 1e-2).numpy()
    np.testing.assert_allclose(orc.layer_norm(xs, np.ones(96), np.zeros(96), 1e-2), ref, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(orc.layer_norm(np.full((2, 8), 4.0), np.ones(8), np.arange(8.0)), np.tile(np.arange(8.0), (2, 1)))
    out = np.zeros_like(x)
    cref.lhref_layer_norm_f32(_p(out), _p(x), _p(g), _p(b), ctypes.c_int64(19), ctypes.c_int64(96),
                              ctypes.c_float(1e-5), ctypes.c_int(1))
    np.testing.assert_allclose(out, orc.layer_norm(x, g, b, 1e-5), rtol=1e-4, atol=1e-5)


def test_softmax_gelu_elementwise_against_torch(cref):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((9, 33)).astype(np.float32) * 4
    np.testing.assert_allclose(orc.softmax(x), F.softmax(torch.from_numpy(x).double(), -1).numpy(), rtol=1e-6)
    xs = np.linspace(-9, 9, 4001).astype(np.float32)
    ref = F.gelu(torch.from_numpy(xs).double(), approximate="tanh").numpy()
    np.testing.assert_allclose(orc.gelu_tanh(xs), ref, rtol=1e-6, atol=1e-9)
    assert abs(orc.gelu_tanh(np.array([1.0]))[0] - 0.8411919906082768) < 1e-6  # known value
    out = np.zeros_like(xs)
    cref.lhref_gelu_tanh_f32(_p(out), _p(xs), ctypes.c_int64(xs.size), ctypes.c_int(1))
    np.testing.assert_allclose(out, ref, rtol=2e-5, atol=1e-6)
    so = np.zeros_like(x)
    cref.lhref_softmax_f32(_p(so), _p(x), ctypes.c_int64(9), ctypes.c_int64(33), ctypes.c_int(1))
    np.testing.assert_allclose(so, orc.softmax(x), rtol=1e-5)
    bias = rng.standard_normal(33).astype(np.float32)
    np.testing.assert_array_equal(orc.bias_act(x, bias, relu=True), np.maximum(x + bias, 0))
    np.testing.assert_array_equal(orc.residual_add(x, x), x + x)


# ---- nanoGPT block ---------------------------------------------------------------------------


class _TorchBlock(torch.nn.Module):
    """Independent statement of the benchmark's block (GPT-2 / nanoGPT): pre-LN, fused c_attn,
    causal SDPA, c_proj, MLP with tanh-GELU."""

    def __init__(self, C, H):
        super().__init__()
        self.H = H
        self.ln_1 = torch.nn.LayerNorm(C, eps=1e-5)
        self.c_attn = torch.nn.Linear(C, 3 * C)
        self.c_proj = torch.nn.Linear(C, C)
        self.ln_2 = torch.nn.LayerNorm(C, eps=1e-5)
        self.c_fc = torch.nn.Linear(C, 4 * C)
        self.mlp_proj = torch.nn.Linear(4 * C, C)

    def forward(self, x):
        B, T, C = x.shape
        q, k, v = self.c_attn(self.ln_1(x)).split(C, dim=2)
        q, k, v = (t.view(B, T, self.H, C // self.H).transpose(1, 2) for t in (q, k, v))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).contiguous().view(B, T, C)
        x = x + self.c_proj(y)
        return x + self.mlp_proj(F.gelu(self.c_fc(self.ln_2(x)), approximate="tanh"))


def _block_params(C, rng):
    p = {
        "ln1_g": rng.uniform(0.5, 1.5, C), "ln1_b": rng.uniform(-0.1, 0.1, C),
        "w_qkv": rng.standard_normal((C, 3 * C)) * 0.05, "b_qkv": rng.standard_normal(3 * C) * 0.05,
        "w_o": rng.standard_normal((C, C)) * 0.05, "b_o": rng.standard_normal(C) * 0.05,
        "ln2_g": rng.uniform(0.5, 1.5, C), "ln2_b": rng.uniform(-0.1, 0.1, C),
        "w_fc": rng.standard_normal((C, 4 * C)) * 0.05, "b_fc": rng.standard_normal(4 * C) * 0.05,
        "w_proj": rng.standard_normal((4 * C, C)) * 0.05, "b_proj": rng.standard_normal(C) * 0.05,
    }
    return {k: v.astype(np.float32) for k, v in p.items()}


def test_nanogpt_block_against_torch_module():
    rng = np.random.default_rng(13)
    B, T, C, H = 2, 24, 32, 4
    p = _block_params(C, rng)
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    blk = _TorchBlock(C, H).double()
    _load_block(blk, p)
    with torch.no_grad():
        ref = blk(torch.from_numpy(x).double()).numpy()
    np.testing.assert_allclose(orc.nanogpt_block(x, p, H, mode="f32"), ref, rtol=2e-5, atol=2e-5)
    bf = orc.nanogpt_block(x, p, H, mode="bf16")
    assert np.abs(bf - ref).max() <= 2e-2 * np.abs(ref).max()
    assert np.abs(bf - ref).max() > 0  # the bf16 rounding points are really applied


def _load_block(blk, p):
    t = lambda a: torch.from_numpy(np.asarray(a)).double()
    with torch.no_grad():
        blk.ln_1.weight.copy_(t(p["ln1_g"])); blk.ln_1.bias.copy_(t(p["ln1_b"]))
        blk.c_attn.weight.copy_(t(p["w_qkv"]).T); blk.c_attn.bias.copy_(t(p["b_qkv"]))
        blk.c_proj.weight.copy_(t(p["w_o"]).T); blk.c_proj.bias.copy_(t(p["b_o"]))
        blk.ln_2.weight.copy_(t(p["ln2_g"])); blk.ln_2.bias.copy_(t(p["ln2_b"]))
        blk.c_fc.weight.copy_(t(p["w_fc"]).T); blk.c_fc.bias.copy_(t(p["b_fc"]))
        blk.mlp_proj.weight.copy_(t(p["w_proj"]).T); blk.mlp_proj.bias.copy_(t(p["b_proj"]))


def test_nanogpt_forward_against_torch_stack():
    """n blocks, final LayerNorm, lm_head with bias (examples/xegpu/nanoGPT_payload.py:399-407) against an
    independent float64 torch stack.  The final gamma / beta and the lm_head bias are non-trivial, the
    vocabulary is ragged, and a variant of the torch model with one piece left out must NOT match, so a
    skipped LayerNorm, bias or layer in the oracle cannot pass."""
    rng = np.random.default_rng(29)
    B, T, C, H, V, L = 2, 20, 32, 4, 45, 3
    layers = [_block_params(C, rng) for _ in range(L)]
    lnf_g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    lnf_b = rng.uniform(-0.3, 0.3, C).astype(np.float32)
    lm_w = (rng.standard_normal((C, V)) * 0.1).astype(np.float32)
    lm_b = rng.uniform(-0.5, 0.5, V).astype(np.float32)
    x = rng.standard_normal((B, T, C)).astype(np.float32)

    blocks = [_TorchBlock(C, H).double() for _ in range(L)]
    for blk, p in zip(blocks, layers):
        _load_block(blk, p)
    ln_f = torch.nn.LayerNorm(C, eps=1e-5).double()
    head = torch.nn.Linear(C, V).double()
    with torch.no_grad():
        ln_f.weight.copy_(torch.from_numpy(lnf_g).double()); ln_f.bias.copy_(torch.from_numpy(lnf_b).double())
        head.weight.copy_(torch.from_numpy(lm_w).double().T); head.bias.copy_(torch.from_numpy(lm_b).double())

        def run(skip_ln=False, skip_bias=False, n=L):
            h = torch.from_numpy(x).double()
            for blk in blocks[:n]:
                h = blk(h)
            if not skip_ln:
                h = ln_f(h)
            out = h @ head.weight.T
            return (out if skip_bias else out + head.bias).numpy()

        ref = run()
        wrong = [run(skip_ln=True), run(skip_bias=True), run(n=L - 1)]
    got = orc.nanogpt_forward(x, layers, lnf_g, lnf_b, lm_w, lm_b, H, mode="f32")
    assert got.shape == (B, T, V)
    np.testing.assert_allclose(got, ref, rtol=2e-5, atol=2e-5)
    for w in wrong:
        assert np.abs(got - w).max() > 1e-2
    no_bias = orc.nanogpt_forward(x, layers, lnf_g, lnf_b, lm_w, None, H, mode="f32")
    np.testing.assert_allclose(no_bias, wrong[1], rtol=2e-5, atol=2e-5)
    bf = orc.nanogpt_forward(x, layers, lnf_g, lnf_b, lm_w, lm_b, H, mode="bf16")
    err = np.abs(bf - ref).max()
    assert 0 < err <= 2e-2 * np.abs(ref).max()


class _TorchRefBlock(torch.nn.Module):
    """Independent statement of the reference's own block (examples/xegpu/nanoGPT_payload.py:299-317):
    separate bias-free q/k/v projections, non-causal attention, ReLU MLP."""

    def __init__(self, C, H, hidden, causal=False):
        super().__init__()
        self.H, self.causal = H, causal
        self.ln_1 = torch.nn.LayerNorm(C, eps=1e-5)
        self.q = torch.nn.Linear(C, C, bias=False)
        self.k = torch.nn.Linear(C, C, bias=False)
        self.v = torch.nn.Linear(C, C, bias=False)
        self.proj = torch.nn.Linear(C, C)
        self.ln_2 = torch.nn.LayerNorm(C, eps=1e-5)
        self.fc1 = torch.nn.Linear(C, hidden)
        self.fc2 = torch.nn.Linear(hidden, C)

    def forward(self, x):  # x: [T, C]
        T, C = x.shape
        h = self.ln_1(x)
        q, k, v = (m(h).view(T, self.H, C // self.H).transpose(0, 1) for m in (self.q, self.k, self.v))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=self.causal).transpose(0, 1).reshape(T, C)
        x = x + self.proj(y)
        return x + self.fc2(F.relu(self.fc1(self.ln_2(x))))


def _ref_block_weights(C, hidden, rng, sc=0.05):
    """Weights shaped and typed as the reference's driver makes them (examples/xegpu/nanoGPT.py:243-258),
    with non-trivial LayerNorm parameters and biases so that a dropped one shows."""
    f16 = lambda a: a.astype(np.float16)
    return dict(
        g1=rng.uniform(0.5, 1.5, C).astype(np.float32), b1n=rng.uniform(-0.1, 0.1, C).astype(np.float32),
        wq=f16(rng.standard_normal((C, C)) * sc), wk=f16(rng.standard_normal((C, C)) * sc),
        wv=f16(rng.standard_normal((C, C)) * sc), wp=f16(rng.standard_normal((C, C)) * sc),
        bp=(rng.standard_normal(C) * sc).astype(np.float32),
        g2=rng.uniform(0.5, 1.5, C).astype(np.float32), b2n=rng.uniform(-0.1, 0.1, C).astype(np.float32),
        w1=f16(rng.standard_normal((C, hidden)) * sc), bb1=(rng.standard_normal(hidden) * sc).astype(np.float32),
        w2=f16(rng.standard_normal((hidden, C)) * sc), bb2=(rng.standard_normal(C) * sc).astype(np.float32),
    )


def _load_ref_block(blk, w):
    t = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).double()
    with torch.no_grad():
        blk.ln_1.weight.copy_(t(w["g1"])); blk.ln_1.bias.copy_(t(w["b1n"]))
        blk.q.weight.copy_(t(w["wq"]).T); blk.k.weight.copy_(t(w["wk"]).T); blk.v.weight.copy_(t(w["wv"]).T)
        blk.proj.weight.copy_(t(w["wp"]).T); blk.proj.bias.copy_(t(w["bp"]))
        blk.ln_2.weight.copy_(t(w["g2"])); blk.ln_2.bias.copy_(t(w["b2n"]))
        blk.fc1.weight.copy_(t(w["w1"]).T); blk.fc1.bias.copy_(t(w["bb1"]))
        blk.fc2.weight.copy_(t(w["w2"]).T); blk.fc2.bias.copy_(t(w["bb2"]))


def _ref_to_block_params(w):
    """The reference's weight names -> the parameter names of orc.nanogpt_block (separate projections)."""
    return dict(ln1_g=w["g1"], ln1_b=w["b1n"], w_q=w["wq"], w_k=w["wk"], w_v=w["wv"], w_o=w["wp"], b_o=w["bp"],
                ln2_g=w["g2"], ln2_b=w["b2n"], w_fc=w["w1"], b_fc=w["bb1"], w_proj=w["w2"], b_proj=w["bb2"])


@pytest.mark.parametrize("causal", [False, True])
def test_reference_block_checker_against_torch_module(causal):
    """orc.ref_block_fused (the reference's numpy checker restated, f16 rounding points) and
    orc.nanogpt_block in the reference's configuration (the kernels' rounding points) against the
    float64 torch module: both within f16 rounding of it, neither equal to it, and within the
    reference's own pass criterion max|diff| / max|ref| < 5e-2 (examples/xegpu/nanoGPT.py:298-302)
    of each other by a wide margin."""
    rng = np.random.default_rng(31)
    T, C, hidden, H = 48, 64, 256, 4
    w = _ref_block_weights(C, hidden, rng)
    x = (rng.standard_normal((T, C)) * 0.5).astype(np.float32)
    blk = _TorchRefBlock(C, H, hidden, causal).double()
    _load_ref_block(blk, w)
    with torch.no_grad():
        ref = blk(torch.from_numpy(x).double()).numpy()
    got = orc.ref_block_fused(x, w, H, causal=causal)
    scale = np.abs(ref).max()
    assert 0 < np.abs(got - ref).max() <= 4e-3 * scale
    # f32 "rounding": the restatement is the torch module to float32 accuracy
    np.testing.assert_allclose(orc.ref_block_fused(x, w, H, causal=causal, elt="f32"), ref, rtol=2e-5, atol=2e-5)
    mine = orc.nanogpt_block(x[None], _ref_to_block_params(w), H, mode="f16", causal=causal, activation="relu",
                             bias_f32=True)[0]
    assert 0 < np.abs(mine - ref).max() <= 4e-3 * scale
    assert np.abs(mine - got).max() <= 4e-3 * scale
    exact = orc.nanogpt_block(x[None], _ref_to_block_params(w), H, mode="f32", causal=causal, activation="relu",
                              bias_f32=True)[0]
    np.testing.assert_allclose(exact, ref, rtol=2e-5, atol=2e-5)


def test_reference_gpt_checker_against_torch_stack():
    """orc.ref_gpt_fused (examples/xegpu/nanoGPT.py:128-135) and orc.nanogpt_forward in the reference's
    configuration against two float64 torch blocks + LayerNorm + Linear."""
    rng = np.random.default_rng(37)
    T, C, hidden, H, V, L = 32, 64, 128, 4, 40, 2
    ws = [_ref_block_weights(C, hidden, rng) for _ in range(L)]
    gf_g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    gf_b = rng.uniform(-0.3, 0.3, C).astype(np.float32)
    lmw = (rng.standard_normal((C, V)) * 0.05).astype(np.float16)
    lmb = rng.uniform(-0.5, 0.5, V).astype(np.float32)
    x = (rng.standard_normal((T, C)) * 0.5).astype(np.float32)
    with torch.no_grad():
        h = torch.from_numpy(x).double()
        for w in ws:
            blk = _TorchRefBlock(C, H, hidden).double()
            _load_ref_block(blk, w)
            h = blk(h)
        h = F.layer_norm(h, (C,), torch.from_numpy(gf_g).double(), torch.from_numpy(gf_b).double(), 1e-5)
        ref = (h @ torch.from_numpy(lmw.astype(np.float32)).double() + torch.from_numpy(lmb).double()).numpy()
    scale = np.abs(ref).max()
    got = orc.ref_gpt_fused(x, ws, gf_g, gf_b, lmw, lmb, H)
    assert 0 < np.abs(got - ref).max() <= 4e-3 * scale
    np.testing.assert_allclose(orc.ref_gpt_fused(x, ws, gf_g, gf_b, lmw, lmb, H, elt="f32"), ref, rtol=2e-5, atol=2e-5)
    mine = orc.nanogpt_forward(x[None], [_ref_to_block_params(w) for w in ws], gf_g, gf_b, lmw, lmb, H, mode="f16",
                               causal=False, activation="relu", bias_f32=True)[0]
    assert 0 < np.abs(mine - ref).max() <= 4e-3 * scale


def test_complexity_formulas():
    """examples/xegpu/matmul.py:41-64, fused_attention.py:26-43, layer_norm.py:27-40 at the benchmark sizes."""
    assert orc.matmul_complexity(4096, 4096, 4096, False, False, False, 2, 2) == (137438953472, 67108864, 33554432)
    assert orc.matmul_complexity(1024, 1024, 1024, True, True, False, 4, 4)[0] == 2 * 1024**3 + 2 * 1024**2
    assert orc.fused_attention_complexity(4, 16, 2048, 64, 2) == (68719476736, 50331648, 16777216)
    assert orc.layer_norm_complexity(8192, 768, 4) == (8 * 8192 * 768, (8192 * 768 + 2 * 768) * 4, 8192 * 768 * 4)


def test_mlp_matches_torch_sequential():
    """orc.mlp against a library model: torch Linear / ReLU stack in float64 (weights stored
    [out, in] there, so transpose_b on the oracle side), ReLU on hidden layers only."""
    import torch

    rng = np.random.default_rng(17)
    sizes = [12, 20, 9, 5]
    x = rng.standard_normal((7, sizes[0])).astype(np.float32)
    layers, ws, bs = [], [], []
    for i, o in zip(sizes[:-1], sizes[1:]):
        lin = torch.nn.Linear(i, o, dtype=torch.float64)
        with torch.no_grad():
            lin.weight.copy_(torch.from_numpy(rng.standard_normal((o, i))).float().double())
            lin.bias.copy_(torch.from_numpy(rng.standard_normal(o)).float().double())
        ws.append(lin.weight.detach().numpy().astype(np.float32))
        bs.append(lin.bias.detach().numpy().astype(np.float32))
        layers += [lin, torch.nn.ReLU()]
    model = torch.nn.Sequential(*layers[:-1])
    ref = model(torch.from_numpy(x).double()).detach().numpy()
    got = orc.mlp(x, ws, bs, has_relu=True, transpose_b=True)
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=2e-6)
    with_final = orc.mlp(x, ws, bs, has_relu=True, relu_on_final_layer=True, transpose_b=True)
    np.testing.assert_allclose(with_final, np.maximum(ref, 0), rtol=2e-6, atol=2e-6)
    # only the last layer accumulates into the passed output
    c = rng.standard_normal(ref.shape).astype(np.float32)
    np.testing.assert_allclose(orc.mlp(x, ws, bs, has_relu=True, transpose_b=True, accumulate_c=c), ref + c,
                               rtol=2e-6, atol=2e-6)
