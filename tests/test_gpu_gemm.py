"""GEMM parity on the GPU: HIP kernels (through the C ABI) vs the CPU oracle."""

import numpy as np
import pytest
import torch

from oracle import lh_oracle as orc
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu

F32_RTOL = 1e-4   # benchmark definition: f32 within rtol 1e-4
BF16_RTOL = 2e-2  # bf16 within rtol 2e-2 of the f32 reference
FP8_RTOL = 5e-2   # fp8 within rtol 5e-2 of the dequantised f32 reference


def _dev(x, dtype):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to("cuda").to(dtype)


def _host(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize("shape", [(64, 64, 32), (128, 128, 64), (256, 192, 96), (1024, 1024, 1024), (100, 70, 50),
                                   (1, 1, 1), (33, 65, 17),
                                   # 64 x 64 tiles take four k-steps per barrier: K = 5, 7, 9 and 13 steps
                                   (128, 128, 160), (192, 64, 224), (64, 128, 288), (256, 256, 416),
                                   # 128 x 128 tiles, two per workgroup; 128 x 64 tiles, three per workgroup; one
                                   (4096, 2048, 64), (4096, 1536, 96), (2048, 2048, 512)])
@pytest.mark.parametrize("epi", ["none", "bias_relu"])
def test_gemm_f32(shape, epi):
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(0xC0FFEE + M + N + K)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    bias = rng.uniform(-1, 1, (N,)).astype(np.float32)
    has = epi == "bias_relu"
    out = ops.gemm(_dev(a, torch.float32), _dev(b, torch.float32), _dev(bias, torch.float32) if has else None, relu=has)
    ref = orc.matmul(a, b, bias=bias if has else None, relu=has)
    assert_close(_host(out), ref, F32_RTOL, f"f32 gemm {shape} {epi}", report=shape == (1024, 1024, 1024) and epi != "none")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 256, 128), (512, 768, 256), (1024, 1024, 512),
                                   (2048, 2048, 256), (100, 70, 50), (1, 1, 1), (130, 257, 66)])
@pytest.mark.parametrize("epi", ["none", "bias_relu", "bias_gelu", "f32out", "acc"])
def test_gemm_16bit(dtype, shape, epi):
    from lighthouse_amd import ops

    M, N, K = shape
    elt = "bf16" if dtype == torch.bfloat16 else "f16"
    rng = np.random.default_rng(7 + M + 3 * N + 5 * K)
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), elt)
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32), elt)
    bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), elt)
    da, db = _dev(a, dtype), _dev(b, dtype)
    if epi == "none":
        out = ops.gemm(da, db)
        ref = orc.matmul(a, b, result_type=elt)
    elif epi == "bias_relu":
        out = ops.gemm(da, db, _dev(bias, dtype), relu=True)
        ref = orc.matmul(a, b, bias=bias, relu=True, result_type=elt)
    elif epi == "bias_gelu":
        out = ops.gemm(da, db, _dev(bias, dtype), gelu=True)
        ref = orc.matmul(a, b, bias=bias, gelu=True, result_type=elt)
    elif epi == "f32out":
        out = ops.gemm(da, db, out_dtype=torch.float32)
        ref = orc.matmul(a, b, result_type="f32")
    else:
        c = rng.standard_normal((M, N)).astype(np.float32)
        out = _dev(c, torch.float32)
        ops.gemm(da, db, out=out, accumulate_c=True)
        ref = orc.matmul(a, b, c=c, accumulate_c=True, result_type="f32")
    rtol = F32_RTOL if epi in ("f32out", "acc") else BF16_RTOL
    assert_close(_host(out), ref, rtol, f"{elt} gemm {shape} {epi}")


@pytest.mark.parametrize("tile", [(256, 256), (256, 128), (128, 256), (128, 128)])
@pytest.mark.parametrize("K", [64, 128, 192, 448])
@pytest.mark.parametrize("epi", ["none", "bias_gelu", "f32out_acc"])
def test_gemm_16bit_requested_tile(tile, K, epi):
    """Every workgroup tile of the direct-to-LDS kernel, on a grid of 2 x 3 tiles, with K spanning
    the pipeline's prologue-only, one-pair and multi-pair paths."""
    from lighthouse_amd import ops

    M, N = 2 * tile[0], 3 * tile[1]
    rng = np.random.default_rng(K + tile[0] + 7 * tile[1])
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), "bf16")
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32), "bf16")
    da, db = _dev(a, torch.bfloat16), _dev(b, torch.bfloat16)
    if epi == "none":
        out = ops.gemm(da, db, tile=tile)
        ref = orc.matmul(a, b, result_type="bf16")
    elif epi == "bias_gelu":
        bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), "bf16")
        out = ops.gemm(da, db, _dev(bias, torch.bfloat16), gelu=True, tile=tile)
        ref = orc.matmul(a, b, bias=bias, gelu=True, result_type="bf16")
    else:
        c = rng.standard_normal((M, N)).astype(np.float32)
        out = _dev(c, torch.float32)
        ops.gemm(da, db, out=out, accumulate_c=True, tile=tile)
        ref = orc.matmul(a, b, c=c, accumulate_c=True, result_type="f32")
    rtol = F32_RTOL if epi == "f32out_acc" else BF16_RTOL
    assert_close(_host(out), ref, rtol, f"bf16 gemm tile {tile} K={K} {epi}")


@pytest.mark.parametrize("epi", ["bias_relu", "f32out_acc"])
@pytest.mark.parametrize("tile,M,N", [((256, 256), 4608, 4608), ((256, 128), 4608, 2304), ((128, 256), 2304, 4608),
                                      ((128, 128), 3072, 3072), (None, 4600, 4600)])
def test_gemm_16bit_several_tiles_per_workgroup(tile, M, N, epi):
    """More tiles than resident workgroups: a workgroup issues its next tile's first loads before
    the epilogue of the current one (some workgroups get two tiles, others one).  The last case
    is the edge instantiation (M, N not multiples of the tile)."""
    from lighthouse_amd import ops

    K = 128
    rng = np.random.default_rng(M + N)
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), "bf16")
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32), "bf16")
    da, db = _dev(a, torch.bfloat16), _dev(b, torch.bfloat16)
    if epi == "bias_relu":
        bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), "bf16")
        out = ops.gemm(da, db, _dev(bias, torch.bfloat16), relu=True, tile=tile)
        ref = orc.matmul(a, b, bias=bias, relu=True, result_type="bf16")
        rtol = BF16_RTOL
    else:
        c = rng.standard_normal((M, N)).astype(np.float32)
        out = _dev(c, torch.float32)
        ops.gemm(da, db, out=out, accumulate_c=True, tile=tile)
        ref = orc.matmul(a, b, c=c, accumulate_c=True, result_type="f32")
        rtol = F32_RTOL
    assert_close(_host(out), ref, rtol, f"bf16 gemm {M}x{N} tile {tile} {epi}")


@pytest.mark.parametrize("shape", [(1000, 520, 192), (130, 264, 64), (257, 8, 128), (1, 1000, 256), (3000, 776, 320)])
@pytest.mark.parametrize("epi", ["none", "bias_relu", "f32out_acc_bias"])
def test_gemm_16bit_ragged_shapes(shape, epi):
    """M and N that no tile divides (N a multiple of 8, K of 64): the direct kernel's edge
    instantiation; rows and columns past the end must be neither read as bias nor written."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(3 * M + 5 * N + K)
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), "bf16")
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32), "bf16")
    bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), "bf16")
    da, db = _dev(a, torch.bfloat16), _dev(b, torch.bfloat16)
    # output embedded in a larger canvas: everything around it must stay untouched
    pad = 8
    if epi == "f32out_acc_bias":
        c = rng.standard_normal((M, N)).astype(np.float32)
        canvas = torch.full((M + 2, N + 2 * pad), 7.0, device="cuda")
        view = canvas[1:M + 1, pad:pad + N]
        view.copy_(_dev(c, torch.float32))
        ops.gemm(da, db, _dev(bias.astype(np.float32), torch.float32), out=view, accumulate_c=True)
        ref = orc.matmul(a, b, c=c, bias=bias, accumulate_c=True, result_type="f32")
        rtol = F32_RTOL
    else:
        canvas = torch.full((M + 2, N + 2 * pad), 7.0, device="cuda", dtype=torch.bfloat16)
        view = canvas[1:M + 1, pad:pad + N]
        has = epi == "bias_relu"
        ops.gemm(da, db, _dev(bias, torch.bfloat16) if has else None, relu=has, out=view)
        ref = orc.matmul(a, b, bias=bias if has else None, relu=has, result_type="bf16")
        rtol = BF16_RTOL
    assert_close(_host(view), ref, rtol, f"ragged bf16 gemm {shape} {epi}")
    border = canvas.float().clone()
    border[1:M + 1, pad:pad + N] = 7.0
    assert (border == 7.0).all(), "the kernel wrote outside the output matrix"


@pytest.mark.parametrize("shape", [(1000, 520, 192), (130, 264, 64), (257, 4, 128), (1, 1000, 256), (3000, 772, 320),
                                   (4100, 2052, 96)])  # the last: 128-wide tiles, several per workgroup
@pytest.mark.parametrize("epi", ["none", "bias_relu", "acc_bias"])
def test_gemm_f32_ragged_shapes(shape, epi):
    """f32 with M and N that no tile divides (N a multiple of 4, K of 32): the direct kernel's edge
    instantiation; rows and columns past the end must be neither read as bias nor written."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(7 * M + 3 * N + K)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    bias = rng.uniform(-1, 1, (N,)).astype(np.float32)
    pad = 4
    canvas = torch.full((M + 2, N + 2 * pad), 7.0, device="cuda")
    view = canvas[1:M + 1, pad:pad + N]
    da, db = _dev(a, torch.float32), _dev(b, torch.float32)
    if epi == "acc_bias":
        c = rng.standard_normal((M, N)).astype(np.float32)
        view.copy_(_dev(c, torch.float32))
        ops.gemm(da, db, _dev(bias, torch.float32), out=view, accumulate_c=True)
        ref = orc.matmul(a, b, c=c, bias=bias, accumulate_c=True)
    else:
        has = epi == "bias_relu"
        ops.gemm(da, db, _dev(bias, torch.float32) if has else None, relu=has, out=view)
        ref = orc.matmul(a, b, bias=bias if has else None, relu=has)
    assert_close(_host(view), ref, F32_RTOL, f"ragged f32 gemm {shape} {epi}")
    border = canvas.clone()
    border[1:M + 1, pad:pad + N] = 7.0
    assert (border == 7.0).all(), "the kernel wrote outside the output matrix"


def test_gemm_tile_request_errors():
    from lighthouse_amd import ops

    a = torch.zeros(256, 64, device="cuda", dtype=torch.bfloat16)
    b = torch.zeros(64, 384, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.gemm(a, b, tile=(256, 256))  # N = 384 is not a multiple of 256
    with pytest.raises(ValueError):
        ops.gemm(a, b, tile=(64, 64))
    with pytest.raises(ValueError):
        ops.gemm(a.float(), b.float(), tile=(256, 128))  # a tile of the 16-bit kernel
    with pytest.raises(ValueError):
        ops.gemm(a.float(), b.float(), split_k=2)
    with pytest.raises(ValueError, match="K % 32"):
        ops.gemm(torch.zeros(64, 48, device="cuda"), torch.zeros(48, 64, device="cuda"), tile=(64, 64))
    ops.gemm(a, b, tile=(256, 128))
    ops.gemm(a.float(), b.float(), tile=(128, 128))


@pytest.mark.parametrize("tile", [(128, 128), (128, 64), (64, 64)])
@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (8192, 768, 768), (200, 332, 96), (64, 64, 32), (4096, 2304, 256)])
def test_gemm_f32_tile_requests(shape, tile):
    """Each tile of the f32 kernel on request (edge tiles clipped): integer operands make the result
    exact, so every tile must give the bits of the library's own choice, with and without bias +
    ReLU, and nothing outside the output may be written."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-3, 4, (M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (K, N)).astype(np.float32)
    bias = rng.integers(-8, 9, (N,)).astype(np.float32)
    da, db, dbias = _dev(a, torch.float32), _dev(b, torch.float32), _dev(bias, torch.float32)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    out = ops.gemm(da, db, tile=tile)
    assert np.array_equal(_host(out).astype(np.float64), ref), f"f32 gemm {shape} tile {tile}"
    assert torch.equal(out, ops.gemm(da, db))
    canvas = torch.full((M + 2, N + 8), 7.0, device="cuda")
    view = canvas[1:M + 1, 4:4 + N]
    ops.gemm(da, db, dbias, relu=True, out=view, tile=tile)
    assert np.array_equal(_host(view).astype(np.float64), np.maximum(ref + bias, 0.0))
    canvas[1:M + 1, 4:4 + N] = 7.0
    assert (canvas == 7.0).all(), "the kernel wrote outside the output matrix"


@pytest.mark.parametrize("kind", ["bf16_bias_relu", "bf16_f32_acc", "f32", "fp8"])
def test_gemm_row_strided_views(kind):
    """Operands and output that are column ranges of wider buffers (lda, ldb, ldc larger than the
    logical widths): results match the contiguous call and nothing outside the output view changes."""
    from lighthouse_amd import ops

    M, N, K = (2048, 4096, 128) if kind == "fp8" else (512, 768, 256)
    pad = 64
    g = torch.Generator(device="cuda").manual_seed(31)
    if kind == "fp8":
        dt, odt = torch.float8_e4m3fn, torch.bfloat16
    elif kind == "f32":
        dt, odt = torch.float32, torch.float32
    else:
        dt, odt = torch.bfloat16, torch.float32 if kind == "bf16_f32_acc" else torch.bfloat16
    wide_a = torch.randn(M, K + 2 * pad, device="cuda", generator=g).clamp(-4, 4).to(dt)
    wide_b = torch.randn(K, N + 2 * pad, device="cuda", generator=g).clamp(-4, 4).to(dt)
    a, b = wide_a[:, pad:pad + K], wide_b[:, pad:pad + N]
    wide_o = torch.full((M, N + 2 * pad), 7.0, device="cuda").to(odt)
    out = wide_o[:, pad:pad + N]
    assert not a.is_contiguous() and not out.is_contiguous()
    if kind == "fp8":
        ops.gemm_fp8(a, b, 0.5, 0.25, out=out)
        ref = ops.gemm_fp8(a.contiguous(), b.contiguous(), 0.5, 0.25)
    elif kind == "bf16_f32_acc":
        bias = torch.randn(N, device="cuda", generator=g)
        c = torch.randn(M, N, device="cuda", generator=g)
        out.copy_(c)
        ops.gemm(a, b, bias, out=out, accumulate_c=True)
        ref = c.clone()
        ops.gemm(a.contiguous(), b.contiguous(), bias, out=ref, accumulate_c=True)
    else:
        bias = torch.randn(N, device="cuda", generator=g).to(odt)
        ops.gemm(a, b, bias, relu=True, out=out)
        ref = ops.gemm(a.contiguous(), b.contiguous(), bias, relu=True)
    assert torch.equal(out.contiguous(), ref)
    assert torch.all(wide_o[:, :pad].float() == 7.0) and torch.all(wide_o[:, pad + N:].float() == 7.0)


@pytest.mark.parametrize("ta,tb", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(256, 128, 192),   # operands transposed into the library's buffer first
                                   (1000, 776, 512),  # the same with several tiles and an M no tile divides
                                   (100, 72, 64),     # M no multiple of 8: the element-wise transpose
                                   (70, 50, 33)])     # K no multiple of a k-step: the kernels that read in place
def test_gemm_transposed(dtype, ta, tb, shape):
    from lighthouse_amd import ops

    M, N, K = shape
    elt = "bf16" if dtype == torch.bfloat16 else "f32"
    rng = np.random.default_rng(99)
    a = orc.round_to(rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32), elt)
    b = orc.round_to(rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32), elt)
    out = ops.gemm(_dev(a, dtype), _dev(b, dtype), out_dtype=torch.float32, transpose_a=ta, transpose_b=tb)
    ref = orc.matmul(a, b, transpose_a=ta, transpose_b=tb)
    assert_close(_host(out), ref, F32_RTOL, f"transposed gemm {shape} ta={ta} tb={tb} {elt}")


def test_gemm_integer_inputs_exact():
    """Integer inputs in [-3, 3] (examples/xegpu/matmul.py:143-152) are exact in bf16 and f32."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(2)
    a = rng.integers(-3, 4, (512, 256)).astype(np.float32)
    b = rng.integers(-3, 4, (256, 384)).astype(np.float32)
    out = ops.gemm(_dev(a, torch.bfloat16), _dev(b, torch.bfloat16), out_dtype=torch.float32)
    np.testing.assert_array_equal(_host(out), a @ b)


def test_gemm_identity_and_ones():
    """B = I gives C == A bit for bit; B = 1 gives row sums (the lh-run golden's structure)."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(5)
    a = orc.round_bf16(rng.standard_normal((256, 256)).astype(np.float32))
    out = ops.gemm(_dev(a, torch.bfloat16), torch.eye(256, device="cuda", dtype=torch.bfloat16))
    np.testing.assert_array_equal(_host(out), a)
    a32 = rng.uniform(0, 1, (128, 64)).astype(np.float32)
    out = ops.gemm(_dev(a32, torch.float32), torch.ones(64, 128, device="cuda"))
    assert_close(_host(out), np.repeat(a32.astype(np.float64).sum(1, keepdims=True), 128, 1), F32_RTOL, "ones")


def test_gemm_bf16_4096_properties():
    """Benchmark size (4096^3): checked against the oracle on a sampled set of rows/columns and
    through linearity: (A1 + A2) B == A1 B + A2 B when all three are exact in f32 output."""
    from lighthouse_amd import ops

    n = 4096
    g = torch.Generator(device="cuda").manual_seed(1234)
    a = torch.randn(n, n, device="cuda", generator=g).to(torch.bfloat16)
    b = torch.randn(n, n, device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randn(n, device="cuda", generator=g).to(torch.bfloat16)
    out = ops.gemm(a, b)
    out_epi = ops.gemm(a, b, bias, relu=True)
    rows = np.array([0, 1, 255, 256, 1023, 2048, 3071, 4095])
    cols = np.array([0, 31, 32, 63, 64, 2047, 4000, 4095])
    a_h = a[rows].float().cpu().numpy()
    b_h = b[:, cols].float().cpu().numpy()
    ref = orc.matmul(a_h, b_h, result_type="bf16")
    assert_close(_host(out[rows][:, cols]), ref, BF16_RTOL, "bf16 GEMM 4096^3 (sampled)", report=True)
    ref_epi = orc.matmul(a_h, b_h, bias=bias[cols].float().cpu().numpy(), relu=True, result_type="bf16")
    assert_close(_host(out_epi[rows][:, cols]), ref_epi, BF16_RTOL, "bf16 GEMM 4096^3 + bias + ReLU (sampled)",
                 report=True)
    # The same samples far inside the benchmark tolerance: the result is the float64 sum rounded to
    # bf16, up to one more bf16 step where the f32 accumulation error crosses a rounding boundary
    # (|err| <= 2^-7 |ref| + 0.02).  An element is ~N(0, 64^2) here, a lost 16-wide k-slice ~N(0, 4^2).
    for got, want in ((_host(out[rows][:, cols]), ref), (_host(out_epi[rows][:, cols]), ref_epi)):
        assert (np.abs(got - want) <= 2.0**-7 * np.abs(want) + 0.02).all()
    # The WHOLE result of an integer problem at the same size, bit for bit: with |values| <= 3 every
    # product and every partial sum (<= 9 * 4096) is an integer that f32, f64 and bf16-free int64 all
    # hold exactly, so the CPU's f64 product is the only correct answer; any wrong, missing or doubled
    # product in any tile changes an integer.  The bf16 output of the same problem must be that
    # integer rounded once.
    ai = torch.randint(-3, 4, (n, n), device="cuda", generator=g).to(torch.bfloat16)
    bint = torch.randint(-3, 4, (n, n), device="cuda", generator=g).to(torch.bfloat16)
    exact = ops.gemm(ai, bint, out_dtype=torch.float32)
    want = ai.cpu().double() @ bint.cpu().double()
    assert torch.equal(exact.cpu().double(), want)
    assert torch.equal(ops.gemm(ai, bint).cpu(), want.to(torch.bfloat16))
    want_epi = torch.relu(want + bias.cpu().double()).to(torch.bfloat16)
    assert torch.equal(ops.gemm(ai, bint, bias, relu=True).cpu(), want_epi)
    # Small-integer matrices: every partial sum is exact, so linearity must hold bit for bit.
    a1 = torch.randint(-2, 3, (n, n), device="cuda", generator=g).to(torch.bfloat16)
    a2 = torch.randint(-2, 3, (n, n), device="cuda", generator=g).to(torch.bfloat16)
    bi = torch.randint(-2, 3, (n, n), device="cuda", generator=g).to(torch.bfloat16)
    lhs = ops.gemm(a1 + a2, bi, out_dtype=torch.float32)
    rhs = ops.gemm(a1, bi, out_dtype=torch.float32) + ops.gemm(a2, bi, out_dtype=torch.float32)
    assert torch.equal(lhs, rhs)


def test_gemm_errors():
    from lighthouse_amd import ops

    a = torch.zeros(8, 8, device="cuda")
    with pytest.raises(ValueError):
        ops.gemm(a, torch.zeros(8, 8, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        ops.gemm(a.to(torch.float64), a.to(torch.float64))
    with pytest.raises(ValueError):
        ops.gemm(a, a, relu=True, gelu=True)


@pytest.mark.parametrize("shape", [(128, 128, 128), (256, 256, 512), (96, 80, 200), (16, 256, 1024), (5, 128, 256),
                                   # direct-to-LDS kernel: one tile per workgroup (twice), two tiles per workgroup
                                   (2048, 4096, 128), (4096, 2048, 384), (8192, 4096, 128)])
def test_gemm_fp8(shape):
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(11 + M + N + K)
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    aq, sa = orc.quantize_per_tensor_e4m3(a)
    bq, sb = orc.quantize_per_tensor_e4m3(b)
    da = torch.from_numpy(aq).to("cuda").view(torch.float8_e4m3fn)
    db = torch.from_numpy(bq).to("cuda").view(torch.float8_e4m3fn)
    out = ops.gemm_fp8(da, db, float(sa), float(sb))
    ref = orc.matmul_fp8(aq, bq, sa, sb)
    assert_close(_host(out), ref, 5e-2, f"fp8 gemm {shape}")
    # Against the dequantised float reference, as the benchmark defines the tolerance.
    deq = (orc.e4m3_dequant(aq).astype(np.float64) * sa) @ (orc.e4m3_dequant(bq).astype(np.float64) * sb)
    assert_close(_host(out), deq, 5e-2, f"fp8 gemm vs dequantised {shape}")


def test_gemm_fp8_all_codes():
    """Every finite e4m3 code against every other: a 256 x 256 outer-product table (K padded with zeros)."""
    from lighthouse_amd import ops

    table = orc.e4m3_decode_table()
    codes = np.array([c for c in range(256) if np.isfinite(table[c])], dtype=np.uint8)
    n = 256
    a = np.zeros((n, 128), np.uint8)
    b = np.zeros((128, n), np.uint8)
    a[: len(codes), 0] = codes
    b[0, : len(codes)] = codes
    out = ops.gemm_fp8(torch.from_numpy(a).cuda().view(torch.float8_e4m3fn),
                       torch.from_numpy(b).cuda().view(torch.float8_e4m3fn), 1.0, 1.0, out_dtype=torch.float32)
    ref = np.outer(table[a[:, 0]].astype(np.float64), table[b[0, :]].astype(np.float64))
    np.testing.assert_array_equal(_host(out), ref.astype(np.float32))


def test_gemm_fp8_8192_properties():
    """The benchmark's 8192^3 problem (four tiles per persistent workgroup), quantised as the
    benchmark states (seeded N(0,1) f32 matrices, scale = amax / 448 per tensor): sampled rows against
    the oracle; with B the identity the output is exactly the scaled, bf16-rounded A; and the WHOLE
    result of an integer-valued problem of the same size bit for bit."""
    from lighthouse_amd import ops

    n = 8192
    g = torch.Generator(device="cuda").manual_seed(13)

    def quantise(x):
        # the oracle's recipe (quantize_per_tensor_e4m3) on the device: f32 scale = amax / 448, then
        # round to nearest even; a slab of the codes is compared with the oracle's own quantiser
        amax = float(x.abs().max().item())
        scale = np.float32(np.float32(amax) / np.float32(orc.E4M3_MAX))
        q = (x / float(scale)).to(torch.float8_e4m3fn)
        slab = slice(4000, 4064)
        np.testing.assert_array_equal(q.view(torch.uint8)[slab].cpu().numpy(), orc.e4m3_quant(_host(x[slab]) / scale))
        return q, float(scale)

    xa = torch.randn(n, n, device="cuda", generator=g)
    xb = torch.randn(n, n, device="cuda", generator=g)
    a, sa = quantise(xa)
    b, sb = quantise(xb)
    del xa, xb
    out = ops.gemm_fp8(a, b, sa, sb)
    rows = [0, 1, 255, 256, 4095, 4096, 8190, 8191]
    a_codes = a.view(torch.uint8)[rows].cpu().numpy()
    b_codes = b.view(torch.uint8).cpu().numpy()
    ref = orc.matmul_fp8(a_codes, b_codes, sa, sb)
    assert_close(_host(out[rows]), ref, FP8_RTOL, "fp8 GEMM 8192^3, amax/448 scales (sampled rows)", report=True)
    eye = torch.eye(n, device="cuda").to(torch.float8_e4m3fn)
    out_id = ops.gemm_fp8(a, eye, 0.5, 0.25)
    expect = (a.float() * 0.125).to(torch.bfloat16)
    assert torch.equal(out_id, expect)
    del out, out_id, expect, eye
    # Integers -3 .. 3 are e4m3 values and every partial sum (<= 9 * 8192) is exact in f32: the CPU's
    # f32 product is the one correct result, for all 1024 tiles of the launch.
    ai = torch.randint(-3, 4, (n, n), device="cuda", generator=g).float()
    bi = torch.randint(-3, 4, (n, n), device="cuda", generator=g).float()
    got = ops.gemm_fp8(ai.to(torch.float8_e4m3fn), bi.to(torch.float8_e4m3fn), 1.0, 1.0, out_dtype=torch.float32)
    want = ai.cpu() @ bi.cpu()
    assert torch.equal(got.cpu(), want)
    got16 = ops.gemm_fp8(ai.to(torch.float8_e4m3fn), bi.to(torch.float8_e4m3fn), 0.5, 0.25)
    assert torch.equal(got16.cpu(), (want * 0.125).to(torch.bfloat16))


@pytest.mark.parametrize("shape", [(16, 1024, 8192), (7, 384, 4096), (1, 128, 2048), (16, 2048, 384),
                                   (16, 8192, 8192)])  # the last: the benchmark's decode configuration
def test_gemm_fp8_decode_path(shape):
    """M <= 16: split-K streaming kernel plus the reduction kernel; called three times in a row
    (the library's partial-sum buffer is reused) and with an f32 output."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(5 + M + N + K)
    aq, sa = orc.quantize_per_tensor_e4m3(rng.standard_normal((M, K)).astype(np.float32))
    bq, sb = orc.quantize_per_tensor_e4m3(rng.standard_normal((K, N)).astype(np.float32))
    da = torch.from_numpy(aq).to("cuda").view(torch.float8_e4m3fn)
    db = torch.from_numpy(bq).to("cuda").view(torch.float8_e4m3fn)
    ref = orc.matmul_fp8(aq, bq, sa, sb, result_type="bf16")
    first = None
    for _ in range(3):
        out = ops.gemm_fp8(da, db, float(sa), float(sb))
        assert_close(_host(out), ref, FP8_RTOL, f"fp8 decode {shape}", report=shape == (16, 8192, 8192))
        first = out if first is None else first
        assert torch.equal(out, first)
    out32 = ops.gemm_fp8(da, db, float(sa), float(sb), out_dtype=torch.float32)
    assert_close(_host(out32), orc.matmul_fp8(aq, bq, sa, sb, result_type="f32"), FP8_RTOL, f"fp8 decode f32 {shape}")


@pytest.mark.parametrize("shape", [(17, 256, 1024), (32, 1024, 4096), (33, 512, 2048), (48, 256, 384),
                                   (64, 2048, 8192), (64, 8192, 8192), (65, 512, 1024), (100, 1024, 2048),
                                   (128, 8192, 8192),
                                   # few 256 x 256 tiles, long K: split K of the direct kernel
                                   (256, 512, 4096), (512, 256, 8192), (768, 1024, 2048),
                                   # M that no tile divides, N a multiple of 128: the fast kernel's M-edge form
                                   (100, 384, 512), (129, 256, 256), (1000, 1024, 1024),
                                   # K no multiple of 128 / N no multiple of 128: zero-padded copies
                                   (64, 1000, 1000), (300, 520, 777), (16, 8192, 200)])
def test_gemm_fp8_decode_batches_and_ragged_m(shape):
    """16 < M <= 128: the streaming kernel with 2, 4 or 8 row groups (B still read once; rows past M
    repeat the last row and are not stored); other M: tile kernel with clamped rows.  Run twice
    (the partial-sum buffer is reused) with a guard row behind the output."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(11 + M + N + K)
    aq, sa = orc.quantize_per_tensor_e4m3(rng.standard_normal((M, K)).astype(np.float32))
    bq, sb = orc.quantize_per_tensor_e4m3(rng.standard_normal((K, N)).astype(np.float32))
    da = torch.from_numpy(aq).to("cuda").view(torch.float8_e4m3fn)
    db = torch.from_numpy(bq).to("cuda").view(torch.float8_e4m3fn)
    ref = orc.matmul_fp8(aq, bq, sa, sb, result_type="bf16")
    buf = torch.full((M + 1, N), 7.0, device="cuda", dtype=torch.bfloat16)
    for _ in range(2):
        ops.gemm_fp8(da, db, float(sa), float(sb), out=buf[:M])
        assert_close(_host(buf[:M]), ref, FP8_RTOL, f"fp8 gemm {shape}")
        assert bool((buf[M] == 7.0).all()), "a row past M was written"
    out32 = ops.gemm_fp8(da, db, float(sa), float(sb), out_dtype=torch.float32)
    assert_close(_host(out32), orc.matmul_fp8(aq, bq, sa, sb, result_type="f32"), FP8_RTOL, f"fp8 f32 {shape}")


@pytest.mark.parametrize("elt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("shape", [(512, 521, 200), (300, 1000, 1000), (257, 136, 4100), (1024, 4097, 96)])
@pytest.mark.parametrize("epi", ["none", "bias_relu", "acc", "residual"])
def test_gemm_shapes_run_on_padded_copies(shape, elt, epi):
    """K that is no multiple of the k-step, N that is no multiple of the vector width (rows of B
    and of the output not 16-byte aligned): operands are copied into zero-padded library buffers,
    the direct kernels run, the result is copied back.  The output is a view with two guard
    columns, which must stay as they were."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[elt]
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), elt)
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32) * 0.1, elt)
    bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), elt)
    c = orc.round_to(rng.standard_normal((M, N)).astype(np.float32), elt)
    da, db = _dev(a, dt), _dev(b, dt)
    buf = torch.full((M, N + 2), 5.0, device="cuda", dtype=dt)
    out = buf[:, :N]
    if epi == "none":
        ops.gemm(da, db, out=out)
        ref = orc.matmul(a, b, result_type=elt)
    elif epi == "bias_relu":
        ops.gemm(da, db, _dev(bias, dt), relu=True, out=out)
        ref = orc.matmul(a, b, bias=bias, relu=True, result_type=elt)
    elif epi == "acc":
        out.copy_(_dev(c, dt))
        ops.gemm(da, db, out=out, accumulate_c=True)
        ref = orc.matmul(a, b, c=c, accumulate_c=True, result_type=elt)
    else:
        res = torch.full((M, N + 2), 0.0, device="cuda", dtype=dt)
        res[:, :N] = _dev(c, dt)
        ops.gemm(da, db, _dev(bias, dt), out=out, residual=res[:, :N])
        ref = orc.matmul(a, b, c=c, accumulate_c=True, bias=bias, result_type=elt)
    rtol = F32_RTOL if elt == "f32" else BF16_RTOL
    assert_close(_host(out), ref, rtol, f"{elt} gemm {shape} {epi} (padded)")
    assert bool((buf[:, N:] == 5.0).all()), "columns behind the output were written"


@pytest.mark.parametrize("elt", ["bf16", "f16"])
@pytest.mark.parametrize("shape", [(16, 1024, 4096), (1, 520, 2048), (64, 512, 8192), (130, 256, 4096), (256, 1024, 2048)])
@pytest.mark.parametrize("epi", ["none", "bias_gelu", "f32_acc", "residual"])
def test_gemm_16bit_split_k(shape, elt, epi):
    """Few tiles and a long K (decode shapes): the tile list is cut along K, each part writes an
    f32 block, a second kernel adds them and runs the epilogue.  Called twice (the library's
    partial-result buffer is reused)."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + 5 * N + 11 * K)
    dt = {"bf16": torch.bfloat16, "f16": torch.float16}[elt]
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), elt)
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32) * 0.05, elt)
    bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), elt)
    c = rng.standard_normal((M, N)).astype(np.float32)
    da, db = _dev(a, dt), _dev(b, dt)
    for _ in range(2):
        if epi == "none":
            out = ops.gemm(da, db)
            ref, rtol = orc.matmul(a, b, result_type=elt), BF16_RTOL
        elif epi == "bias_gelu":
            out = ops.gemm(da, db, _dev(bias, dt), gelu=True)
            ref, rtol = orc.matmul(a, b, bias=bias, gelu=True, result_type=elt), BF16_RTOL
        elif epi == "f32_acc":
            out = _dev(c, torch.float32)
            ops.gemm(da, db, out=out, accumulate_c=True)
            ref, rtol = orc.matmul(a, b, c=c, accumulate_c=True, result_type="f32"), F32_RTOL
        else:
            cr = orc.round_to(c, elt)
            out = ops.gemm(da, db, _dev(bias, dt), residual=_dev(cr, dt))
            ref, rtol = orc.matmul(a, b, c=cr, accumulate_c=True, bias=bias, result_type=elt), BF16_RTOL
        assert_close(_host(out), ref, rtol, f"{elt} gemm {shape} {epi} (split K)")


@pytest.mark.parametrize("elt", ["bf16", "f32"])
@pytest.mark.parametrize("ta,tb", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("shape", [(300, 521, 200), (512, 1000, 1000)])
def test_gemm_transposed_and_ragged(shape, ta, tb, elt):
    """Transposed operands of a problem whose K / N need padding: the padded copy is where they
    get untransposed."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + N + K + 2 * ta + tb)
    dt = {"bf16": torch.bfloat16, "f32": torch.float32}[elt]
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), elt)
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32) * 0.1, elt)
    bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), elt)
    da = _dev(a.T.copy() if ta else a, dt)
    db = _dev(b.T.copy() if tb else b, dt)
    out = ops.gemm(da, db, _dev(bias, dt), relu=True, transpose_a=ta, transpose_b=tb)
    ref = orc.matmul(a, b, bias=bias, relu=True, result_type=elt)
    assert_close(_host(out), ref, F32_RTOL if elt == "f32" else BF16_RTOL, f"{elt} gemm {shape} ta={ta} tb={tb}")


def test_tile_search_and_database(tmp_path):
    """The tuner times the library's own choice and every fitting tile for a shape, logs the trials,
    records a tile that beats the library's choice, and ops.gemm picks a recorded tile up when the
    database is in use (same results either way)."""
    from lighthouse_amd import ops
    from lighthouse_amd.tuning import CSVLogger, TileDB, tune_shape, use_db

    M, N, K = 1024, 768, 256
    db = TileDB(str(tmp_path / "tiles.json"))
    logger = CSVLogger(str(tmp_path / "trials.csv"), echo_stdout=False)
    best = tune_shape(M, N, K, "bf16", db, logger, nruns=5, nwarmup=2, exhaustive=True, isolate=False)
    rows = (tmp_path / "trials.csv").read_text().strip().splitlines()
    assert len(rows) == 1 + 1 + 4 and best is not None and best["error"] == "" and best["tflops"] > 0
    assert rows[1].split(",")[4:6] == ["0", "0"]  # the first trial is the automatic choice
    if best["tile_m"]:
        assert db.lookup("bf16", M, N, K) == (best["tile_m"], best["tile_n"])
    else:
        assert db.lookup("bf16", M, N, K) is None
        db.record("bf16", M, N, K, (128, 128), 1.0, 1.0)  # (so that the lookup below has something to find)
    a = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    b = torch.randn(K, N, device="cuda").to(torch.bfloat16)
    plain = ops.gemm(a, b)
    try:
        use_db(db)
        tuned = ops.gemm(a, b)
    finally:
        use_db(None)
    assert torch.equal(plain, tuned)  # every tile accumulates k in the same order


@pytest.mark.parametrize("shape", [(512, 768, 768), (8192, 768, 3072), (130, 264, 64), (96, 50, 40)])
@pytest.mark.parametrize("elt,out_elt", [("bf16", "bf16"), ("f16", "f16"), ("bf16", "f32"), ("f32", "f32")])
def test_gemm_residual_input(shape, elt, out_elt):
    """lh_hip_gemm_residual: the accumulation starts from a separate matrix (the x of x + linear(y)),
    which is only read; bias is added as in the in-place form.  Shapes cover the staged epilogues
    of the direct kernels, their edge instantiation and the generic kernel."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N + K)
    dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}
    a = orc.round_to(rng.standard_normal((M, K)).astype(np.float32), elt)
    b = orc.round_to(rng.standard_normal((K, N)).astype(np.float32) * 0.1, elt)
    bias = orc.round_to(rng.standard_normal((N,)).astype(np.float32), out_elt)
    res = orc.round_to(rng.standard_normal((M, N)).astype(np.float32), out_elt)
    d_res = _dev(res, dt[out_elt])
    out = ops.gemm(_dev(a, dt[elt]), _dev(b, dt[elt]), _dev(bias, dt[out_elt]), out_dtype=dt[out_elt], residual=d_res)
    ref = orc.matmul(a, b, c=res, accumulate_c=True, bias=bias, result_type=out_elt)
    rtol = F32_RTOL if elt == "f32" else BF16_RTOL
    assert_close(_host(out), ref, rtol, f"{elt}->{out_elt} gemm {shape} + residual")
    assert np.array_equal(_host(d_res), res), "the residual input was modified"
    assert out.data_ptr() != d_res.data_ptr()


# ---- temporary memory: caller workspaces and the per-stream pool -------------------------------------


@pytest.mark.parametrize("case", ["split_k", "padded", "transposed_a", "transposed_b", "plain"])
def test_gemm_with_caller_workspace(case):
    """lh_hip_gemm_ws: same kernels, temporaries from the caller's buffer; results equal the pooled
    call bit for bit, a short workspace is refused before anything runs.  A transposed A is copied
    into [M, K] (temporary memory); a transposed B with aligned rows is read in place (none)."""
    from lighthouse_amd import ops

    shapes = {"split_k": (16, 2048, 8192), "padded": (300, 520, 776), "transposed_a": (512, 512, 512),
              "transposed_b": (512, 512, 512), "plain": (512, 512, 512)}
    M, N, K = shapes[case]
    ta, tb = case == "transposed_a", case == "transposed_b"
    rng = np.random.default_rng(11)
    a_h = orc.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    a = _dev(a_h.T.copy() if ta else a_h, torch.bfloat16)
    b_h = orc.round_bf16(rng.standard_normal((K, N)).astype(np.float32))
    b = _dev(b_h.T.copy() if tb else b_h, torch.bfloat16)
    bias = _dev(orc.round_bf16(rng.standard_normal(N).astype(np.float32)), torch.bfloat16)
    need = ops.gemm_workspace_bytes(M, N, K, torch.bfloat16, bias=True, relu=True, transpose_a=ta, transpose_b=tb)
    assert (need > 0) == (case not in ("plain", "transposed_b"))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = ops.gemm(a, b, bias, relu=True, transpose_a=ta, transpose_b=tb)
    got = ops.gemm(a, b, bias, relu=True, transpose_a=ta, transpose_b=tb, workspace=ws)
    assert torch.equal(got, want)
    ref = orc.matmul(a_h, b_h, bias=_host(bias), relu=True, result_type="bf16")
    assert_close(_host(got), ref, BF16_RTOL, f"bf16 gemm {case} with a caller workspace")
    if need:
        sentinel = torch.full((M, N), 7.0, device="cuda", dtype=torch.bfloat16)
        with pytest.raises(ValueError, match="workspace too small"):
            ops.gemm(a, b, bias, relu=True, transpose_a=ta, transpose_b=tb, workspace=ws[: need - 256], out=sentinel)
        with pytest.raises(ValueError, match="workspace too small"):
            ops.gemm(a, b, bias, relu=True, transpose_a=ta, transpose_b=tb, workspace=ws[:0], out=sentinel)


@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(4096, 4096, 1024), (8192, 768, 768), (2048, 2304, 768), (512, 1024, 4096), (16, 4096, 8192),
                                   (200, 136, 192), (1000, 520, 320), (64, 8192, 2048)])
def test_gemm_transposed_b_in_place(shape, dtype, elt):
    """B stored [N, K] (the layout of a torch Linear weight): the direct kernels read its panel like
    A's, whole and edge tiles, every tile on request and the launches cut along K.  Integer operands:
    the f32-output result is exact and equals the untransposed call bit for bit; with bias + ReLU and
    16-bit output against the oracle; on a row-strided view of a wider buffer too."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-3, 4, (M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (K, N)).astype(np.float32)
    bias = rng.integers(-8, 9, (N,)).astype(np.float32)
    da, db, dbt = _dev(a, dtype), _dev(b, dtype), _dev(b.T.copy(), dtype)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    out = ops.gemm(da, dbt, transpose_b=True, out_dtype=torch.float32)
    assert np.array_equal(_host(out).astype(np.float64), exact), f"B^T gemm {shape} {elt}"
    assert torch.equal(out, ops.gemm(da, db, out_dtype=torch.float32))
    assert ops.gemm_workspace_bytes(M, N, K, dtype, transpose_b=True) == ops.gemm_workspace_bytes(M, N, K, dtype)
    ref = orc.matmul(a, b, bias=bias, relu=True, result_type=elt)
    got = ops.gemm(da, dbt, _dev(bias, dtype), relu=True, transpose_b=True)
    assert_close(_host(got), ref, BF16_RTOL, f"B^T gemm + bias + ReLU {shape} {elt}")
    wide = torch.zeros(N, K + 64, device="cuda", dtype=dtype)
    wide[:, 8:8 + K] = dbt
    assert torch.equal(ops.gemm(da, wide[:, 8:8 + K], transpose_b=True, out_dtype=torch.float32), out)
    for tile in [(256, 256), (256, 128), (128, 256), (128, 128)]:
        if M % tile[0] == 0 and N % tile[1] == 0:
            assert torch.equal(ops.gemm(da, dbt, transpose_b=True, out_dtype=torch.float32, tile=tile), out), tile
    if K % 256 == 0 and K // 4 >= 128:
        assert torch.equal(ops.gemm(da, dbt, transpose_b=True, out_dtype=torch.float32, split_k=4), out)


def test_gemm_fp8_with_caller_workspace():
    from lighthouse_amd import ops

    rng = np.random.default_rng(12)
    for M, N, K in ((16, 2048, 4096), (64, 1024, 2048), (256, 512, 8192), (512, 512, 512)):
        aq = _dev(rng.integers(0, 256, (M, K), dtype=np.uint8) & 0x77, torch.uint8).view(torch.float8_e4m3fn)
        bq = _dev(rng.integers(0, 256, (K, N), dtype=np.uint8) & 0x77, torch.uint8).view(torch.float8_e4m3fn)
        need = ops.gemm_fp8_workspace_bytes(M, N, K)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = ops.gemm_fp8(aq, bq, 0.5, 0.25)
        got = ops.gemm_fp8(aq, bq, 0.5, 0.25, workspace=ws)
        assert torch.equal(got, want), (M, N, K)
        if need:
            with pytest.raises(ValueError, match="workspace too small"):
                ops.gemm_fp8(aq, bq, 0.5, 0.25, workspace=ws[: need // 2])


def test_split_k_gemms_on_two_streams():
    """Two streams run decode-shaped GEMMs of different shapes (both cut along K, so both use f32
    partial blocks) at the same time, many times over: each stream has its own temporaries, so
    every result equals the one computed alone and matches the oracle."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(13)
    problems = []
    for M, N, K in ((16, 4096, 8192), (32, 1024, 4096)):
        a_h = rng.integers(-3, 4, (M, K)).astype(np.float32)
        b_h = rng.integers(-3, 4, (K, N)).astype(np.float32)
        assert ops.gemm_workspace_bytes(M, N, K, torch.bfloat16, torch.float32) > 0
        problems.append((_dev(a_h, torch.bfloat16), _dev(b_h, torch.bfloat16), a_h @ b_h))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    torch.cuda.synchronize()
    for _ in range(20):
        for i, (a, b, _) in enumerate(problems):
            with torch.cuda.stream(streams[i]):
                outs[i].append(ops.gemm(a, b, out_dtype=torch.float32))
    torch.cuda.synchronize()
    for i, (_, _, want) in enumerate(problems):
        for o in outs[i]:
            np.testing.assert_array_equal(_host(o), want)  # small integers: exact whatever the K cut
    # growing a pool buffer mid-stream leaves the work already enqueued intact
    ops.release_scratch()
    a, b, want = problems[1]
    small = ops.gemm(a, b, out_dtype=torch.float32)
    a2, b2, want2 = problems[0]
    big = ops.gemm(a2, b2, out_dtype=torch.float32)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(_host(small), want)
    np.testing.assert_array_equal(_host(big), want2)
    ops.release_scratch()


@pytest.mark.parametrize("shape,split_k", [((16, 2048, 4096), 2), ((16, 2048, 4096), 8), ((100, 520, 1024), 4),
                                           ((512, 512, 2048), 2), ((256, 256, 512), 1), ((16, 8192, 8192), 1)])
def test_gemm_split_k_request(shape, split_k):
    """LH_GEMM_SPLITK_*: an explicit cut (or its prohibition) computes the same product; small
    integers make every summation order exact."""
    from lighthouse_amd import ops

    M, N, K = shape
    rng = np.random.default_rng(M + N + K + split_k)
    a_h = rng.integers(-3, 4, (M, K)).astype(np.float32)
    b_h = rng.integers(-3, 4, (K, N)).astype(np.float32)
    bias_h = rng.integers(-3, 4, N).astype(np.float32)
    out = ops.gemm(_dev(a_h, torch.bfloat16), _dev(b_h, torch.bfloat16), _dev(bias_h, torch.float32), relu=True,
                   out_dtype=torch.float32, split_k=split_k)
    np.testing.assert_array_equal(_host(out), np.maximum(a_h @ b_h + bias_h, 0))
    a = _dev(orc.round_bf16(rng.standard_normal((M, K)).astype(np.float32)), torch.bfloat16)
    b = _dev(orc.round_bf16(rng.standard_normal((K, N)).astype(np.float32)), torch.bfloat16)
    got = ops.gemm(a, b, split_k=split_k)
    assert_close(_host(got), orc.matmul(_host(a), _host(b), result_type="bf16"), BF16_RTOL, f"bf16 gemm {shape} split_k={split_k}")


def test_gemm_split_k_request_errors():
    from lighthouse_amd import ops

    a = torch.zeros(128, 192, device="cuda", dtype=torch.bfloat16)
    b = torch.zeros(192, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="cut of K"):
        ops.gemm(a, b, split_k=2)                       # 96 is no multiple of the k-step
    with pytest.raises(ValueError, match="excludes a tile"):
        ops.gemm(torch.zeros(128, 256, device="cuda", dtype=torch.bfloat16),
                 torch.zeros(256, 128, device="cuda", dtype=torch.bfloat16), split_k=2, tile=(128, 128))
    with pytest.raises(ValueError, match="16-bit"):
        ops.gemm(torch.zeros(128, 256, device="cuda"), torch.zeros(256, 128, device="cuda"), split_k=2)
    with pytest.raises(ValueError, match="unsupported split_k"):
        ops.gemm(a, b, split_k=3)
