"""Infinities and NaN through the kernels: a special value reaches exactly the outputs that depend on
it, in the form the arithmetic of the reference payloads gives (an f32 accumulator, maximumf for
ReLU, which passes NaN on: lighthouse/ingress/mlir_gen/named.py:28-32), and nothing else changes.
The expected patterns come from numpy in f64 on the same inputs."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

INF, NAN = float("inf"), float("nan")


def _same_specials(got: np.ndarray, ref: np.ndarray, what: str) -> None:
    """NaN where the reference has NaN, the same signed infinity where it has one, finite elsewhere."""
    assert np.array_equal(np.isnan(got), np.isnan(ref)), f"{what}: NaN pattern differs"
    assert np.array_equal(np.isposinf(got), np.isposinf(ref)), f"{what}: +inf pattern differs"
    assert np.array_equal(np.isneginf(got), np.isneginf(ref)), f"{what}: -inf pattern differs"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(256, 256, 128), (1024, 768, 768), (200, 136, 96), (16, 4096, 4096)])
def test_gemm_special_values_reach_their_row_and_column(shape, dtype):
    """+inf in A[r0, k0], NaN in A[r1, k1], -inf in B[k2, c0]: row r0 is +-inf by the sign of B[k0, :]
    (NaN where that is 0), row r1 is NaN, column c0 is -+inf by the sign of A[:, k2]; every other
    element equals the product without the special values (small integers: exact).  With bias and
    ReLU the NaN stays NaN and -inf becomes 0."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-2, 3, (M, K)).astype(np.float64)
    b = rng.integers(-2, 3, (K, N)).astype(np.float64)
    r0, r1, c0 = 3, M - 2, N - 5
    a[r0, 1], a[r1, K - 1], b[K // 2, c0] = INF, NAN, -INF
    with np.errstate(invalid="ignore"):
        ref = a @ b
    da = torch.from_numpy(a).to("cuda").to(dtype)
    db = torch.from_numpy(b).to("cuda").to(dtype)
    out = ops.gemm(da, db, out_dtype=torch.float32).cpu().numpy().astype(np.float64)  # (f32 output: the sums are exact)
    _same_specials(out, ref, f"gemm {shape} {dtype}")
    finite = np.isfinite(ref)
    assert np.array_equal(out[finite], ref[finite]), f"gemm {shape} {dtype}: finite elements changed"
    bias = rng.integers(-4, 5, (N,)).astype(np.float64)
    with np.errstate(invalid="ignore"):
        ref_relu = np.maximum(ref + bias, 0.0)  # numpy's maximum passes NaN on, like arith.maximumf
    out = ops.gemm(da, db, torch.from_numpy(bias).to("cuda").float(), relu=True, out_dtype=torch.float32).cpu().numpy().astype(np.float64)
    _same_specials(out, ref_relu, f"gemm + bias + ReLU {shape} {dtype}")
    finite = np.isfinite(ref_relu)
    assert np.array_equal(out[finite], ref_relu[finite])


def test_fp8_gemm_has_no_special_values_but_saturates_nothing():
    """e4m3fn has no infinity; its NaN code (0x7f / 0xff) in A makes that row NaN, nothing else."""
    from lighthouse_amd import ops

    M = N = K = 256
    rng = np.random.default_rng(5)
    a = torch.from_numpy(rng.integers(-2, 3, (M, K)).astype(np.float32)).to("cuda").to(torch.float8_e4m3fn)
    b = torch.from_numpy(rng.integers(-2, 3, (K, N)).astype(np.float32)).to("cuda").to(torch.float8_e4m3fn)
    a.view(torch.uint8)[7, 9] = 0x7F
    out = ops.gemm_fp8(a, b, 1.0, 1.0).float().cpu().numpy()
    ref = a.float().cpu().numpy().astype(np.float64) @ b.float().cpu().numpy().astype(np.float64)
    assert np.isnan(out[7]).all() and np.isnan(ref[7]).all()
    keep = np.arange(M) != 7
    assert np.array_equal(out[keep].astype(np.float64), ref[keep])


@pytest.mark.parametrize("N", [768, 1000, 5000])
def test_row_kernels_keep_special_values_in_their_row(N):
    """LayerNorm, softmax: a NaN or an infinity spoils its own row only (mean and variance of that
    row are NaN; a +inf in a softmax row gives NaN there: inf - inf).  GELU and the bias / add
    kernels work element by element: gelu(+inf) = +inf, gelu(-inf) = 0 * ... = NaN in the tanh form
    0.5 x (1 + tanh(...)), as numpy computes it."""
    from lighthouse_amd import ops
    from oracle import lh_oracle as orc

    M = 12
    rng = np.random.default_rng(N)
    x = rng.standard_normal((M, N)).astype(np.float32)
    x[2, 5], x[5, N - 1], x[9, N // 2] = NAN, INF, -INF
    g = rng.uniform(0.5, 1.5, N).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, N).astype(np.float32)
    dx = torch.from_numpy(x).cuda()
    clean = [r for r in range(M) if r not in (2, 5, 9)]
    with np.errstate(invalid="ignore", over="ignore"):
        ln_ref = orc.layer_norm(x, g, b, 1e-5)
        sm_ref = orc.softmax(x)
        ge_ref = orc.gelu_tanh(x)
    ln = ops.layer_norm(dx, torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda(), 1e-5).cpu().numpy()
    _same_specials(ln, ln_ref, f"layer_norm N={N}")
    assert np.allclose(ln[clean], ln_ref[clean], rtol=1e-4, atol=1e-5)
    assert np.isnan(ln[[2, 5, 9]]).all()
    sm = ops.softmax(dx).cpu().numpy()
    _same_specials(sm, sm_ref, f"softmax N={N}")
    assert np.allclose(sm[clean], sm_ref[clean], rtol=1e-4, atol=1e-7)
    assert np.isnan(sm[2]).all() and np.isnan(sm[5]).all()
    assert np.isfinite(sm[9]).all() and sm[9, N // 2] == 0.0      # exp(-inf - max) = 0: the row is fine
    ge = ops.gelu_tanh(dx).cpu().numpy()
    _same_specials(ge, ge_ref, f"gelu N={N}")
    assert np.isnan(ge[2, 5]) and ge[5, N - 1] == INF and np.isfinite(np.delete(ge.ravel(), [2 * N + 5, 5 * N + N - 1, 9 * N + N // 2])).all()


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 64), (torch.float32, 64), (torch.bfloat16, 128),
                                     (torch.bfloat16, 80)])
def test_attention_special_values(dtype, d, causal):
    """NaN in one query row spoils that output row; NaN in one value row spoils every output row
    that can see that key (all of them, or the later ones under the causal mask) and only column c
    of them when it sits in V[j, c]; a key row of large finite scores leaves a one-hot softmax, not
    NaN.  Other heads are untouched."""
    from lighthouse_amd import ops

    Z, H, T = 1, 3, 256
    rng = np.random.default_rng(d + causal)
    q, k, v = (torch.from_numpy(rng.standard_normal((Z, H, T, d)).astype(np.float32)).cuda().to(dtype) for _ in range(3))
    ref = ops.attention(q, k, v, causal=causal).float().cpu().numpy()
    assert np.isfinite(ref).all()
    q2, v2 = q.clone(), v.clone()
    q2[0, 1, 17, 3] = NAN
    v2[0, 1, 100, 5] = NAN
    out = ops.attention(q2, k, v2, causal=causal).float().cpu().numpy()
    assert np.array_equal(out[0, 0], ref[0, 0]) and np.array_equal(out[0, 2], ref[0, 2])
    bad = np.isnan(out[0, 1])
    must = np.zeros((T, d), dtype=bool)
    must[17, :] = True                                    # the NaN query row
    must[(100 if causal else 0):, 5] = True               # rows that attend to key 100, column 5
    # Under the causal mask the rows before 100 multiply the NaN by a probability of exactly 0
    # (0 x NaN = NaN, as in the reference's softmax(S + mask) V) unless their kernel skips the key
    # tile altogether: either is accepted there.
    may = must.copy()
    may[:100, 5] = True
    assert (bad[must]).all() and not bad[~may].any()
    # (rows that share a wave with the NaN row may take another softmax offset than without it: equal
    # up to the rounding of P, not bit for bit)
    assert np.allclose(out[0, 1][~may], ref[0, 1][~may], rtol=2e-2, atol=4e-3)
    # one key with a huge score for every query: softmax is one-hot on it (exp of very negative numbers is 0)
    k3 = k.clone()
    k3[0, 0, 0, :] = 0.0
    q3 = q.clone()
    q3[0, 0, :, 0] = 200.0
    k3[0, 0, 0, 0] = 200.0
    out = ops.attention(q3, k3, v, causal=causal).float().cpu().numpy()
    assert np.isfinite(out).all()
    assert np.allclose(out[0, 0], v[0, 0, 0].float().cpu().numpy()[None, :], rtol=2e-2, atol=2e-2)
