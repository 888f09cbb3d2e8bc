"""Fused attention parity on the GPU vs the CPU oracle."""

import numpy as np
import pytest
import torch

from oracle import lh_oracle as orc
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu


def _dev(x, dtype):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to("cuda").to(dtype)


def _host(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt,rtol", [(torch.bfloat16, "bf16", 2e-2), (torch.float16, "f16", 2e-2),
                                            (torch.float32, "f32", 1e-4)])
@pytest.mark.parametrize("shape", [(1, 1, 128, 64), (2, 3, 256, 64), (1, 2, 512, 64)])
def test_attention_vs_oracle(shape, dtype, elt, rtol, causal):
    from lighthouse_amd import ops

    rng = np.random.default_rng(42 + shape[2] + causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    out = ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal)
    ref = orc.attention(q, k, v, causal=causal)
    assert_close(_host(out), ref, rtol, f"attention {shape} {elt} causal={causal}")


def test_attention_reference_inputs():
    """Inputs of the reference workload (examples/xegpu/fused_attention.py:145-154):
    seed 42, uniform(-0.5, 0.5); checker tolerance rtol = atol = 1e-3 in f16."""
    from lighthouse_amd import ops

    shape = (2, 2, 256, 64)
    np.random.seed(42)
    q, k, v = (np.random.uniform(-0.5, 0.5, shape).astype(np.float16) for _ in range(3))
    out = ops.attention(*(torch.from_numpy(t).cuda() for t in (q, k, v)))
    ref = orc.attention(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32))
    assert np.allclose(_host(out), ref, rtol=1e-3, atol=1e-3)


def test_attention_online_recurrence_matches_kernel_rounding():
    """The kernel follows the tiled recurrence with P rounded to bf16 before P.V: it must agree
    with the oracle's tiled restatement more tightly than with the unrounded one-shot form."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(3)
    q, k, v = (orc.round_bf16(rng.standard_normal((256, 64)).astype(np.float32)) for _ in range(3))
    out = _host(ops.attention(*( _dev(t[None, None], torch.bfloat16) for t in (q, k, v)), causal=True))[0, 0]
    tiled = orc.attention_online(q, k, v, tile=64, causal=True, elt="bf16")
    assert_close(out, tiled, 1e-2, "attention vs tiled oracle")


def test_attention_closed_forms():
    from lighthouse_amd import ops

    rng = np.random.default_rng(8)
    shape = (1, 2, 256, 64)
    q = _dev(rng.standard_normal(shape), torch.bfloat16)
    k = _dev(rng.standard_normal(shape), torch.bfloat16)
    v = _dev(rng.standard_normal(shape), torch.bfloat16)
    # K = 0: uniform weights, O = mean of V over keys.
    o = ops.attention(q, torch.zeros_like(k), v)
    assert_close(_host(o), np.broadcast_to(_host(v).mean(2, keepdims=True), shape), 2e-2, "K=0")
    # Constant V rows: O = that constant.
    vc = torch.full_like(v, 0.75)
    assert torch.equal(ops.attention(q, k, vc), vc)
    # Causal row 0 sees only key 0.
    oc = ops.attention(q, k, v, causal=True)
    assert torch.equal(oc[:, :, 0], v[:, :, 0])
    # Jointly permuting keys and values leaves the non-causal output unchanged (up to summation order).
    perm = torch.randperm(shape[2], device="cuda")
    assert_close(_host(ops.attention(q, k[:, :, perm], v[:, :, perm])), _host(ops.attention(q, k, v)), 2e-2, "perm")


def test_attention_strided_views():
    """(T, H*d) projection buffers viewed as (H, T, d) without a copy
    (examples/xegpu/nanoGPT_payload.py:198-217)."""
    from lighthouse_amd import ops

    B, T, H, d = 2, 256, 3, 64
    rng = np.random.default_rng(21)
    qkv = _dev(rng.standard_normal((B, T, 3 * H * d)), torch.bfloat16)
    q, k, v = (qkv[:, :, i * H * d:(i + 1) * H * d].view(B, T, H, d).permute(0, 2, 1, 3) for i in range(3))
    out_buf = torch.empty(B, T, H * d, device="cuda", dtype=torch.bfloat16)
    out = out_buf.view(B, T, H, d).permute(0, 2, 1, 3)
    ops.attention(q, k, v, causal=True, out=out)
    ref = ops.attention(q.contiguous(), k.contiguous(), v.contiguous(), causal=True)
    assert torch.equal(out.contiguous(), ref)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_benchmark_size(causal):
    """[4,16,2048,64] bf16: every one of the 64 (batch, head) slices against the f64 oracle (the
    launch order permutes (query block, head) ids, so no slice is taken on trust); the largest error
    over all of them is reported."""
    from lighthouse_amd import ops

    g = torch.Generator(device="cuda").manual_seed(77)
    shape = (4, 16, 2048, 64)
    q, k, v = (torch.randn(shape, device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
    out = ops.attention(q, k, v, causal=causal)
    assert torch.isfinite(out.float()).all()
    qh, kh, vh, oh = _host(q), _host(k), _host(v), _host(out)
    worst = (0.0, None)
    for z in range(shape[0]):
        for h in range(shape[1]):
            ref = orc.attention(qh[z, h], kh[z, h], vh[z, h], causal=causal)
            assert_close(oh[z, h], ref, 2e-2, f"attention bf16 [4,16,2048,64] z={z} h={h} causal={causal}")
            e = float(np.abs(oh[z, h] - ref).max() / np.abs(ref).max())
            if e > worst[0]:
                worst = (e, (z, h))
    z, h = worst[1]
    assert_close(oh[z, h], orc.attention(qh[z, h], kh[z, h], vh[z, h], causal=causal), 2e-2,
                 f"attention bf16 [4,16,2048,64] causal={causal}, worst of all 64 slices (z={z} h={h})", report=True)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,shape,rtol", [(torch.bfloat16, (8, 20, 1024, 64), 2e-2), (torch.float32, (3, 8, 1024, 64), 1e-4)])
def test_attention_many_groups(dtype, shape, rtol, causal):
    """More workgroups than two per CU: the 64-rows-per-wave kernel with the heaviest-first causal
    launch order (16-bit), and the 1-D causal grid of the f32 kernel; sampled (batch, head) pairs."""
    from lighthouse_amd import ops

    g = torch.Generator(device="cuda").manual_seed(78)
    q, k, v = (torch.randn(shape, device="cuda", generator=g).to(dtype) for _ in range(3))
    out = ops.attention(q, k, v, causal=causal)
    assert torch.isfinite(out.float()).all()
    for z, h in [(0, 0), (shape[0] - 1, shape[1] - 1), (1, 5)]:
        ref = orc.attention(_host(q[z, h]), _host(k[z, h]), _host(v[z, h]), causal=causal)
        assert_close(_host(out[z, h]), ref, rtol, f"attention {shape} z={z} h={h} causal={causal}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(1, 2, 512, 64), (8, 20, 1024, 64), (1, 2, 512, 128), (2, 3, 1024, 128)])
def test_attention_scores_outgrow_the_offset(shape, dtype, elt, causal):
    """The softmax offset is only raised when a partial row sum of P says so: scores that climb
    from one key tile to the next (by little, by 2^10 and more, and by more than f32 exp can hold)
    must still give the one-shot softmax.  Both row-per-wave variants (few / many groups)."""
    from lighthouse_amd import ops

    Z, H, T, d = shape
    rng = np.random.default_rng(5 + T)
    # score(q, key t) = 0.125 * 64 * 0.25 * ramp[t] + noise = 2 ramp[t] + noise (natural-log units; 2.8 ramp[t]
    # at head_dim 128, whose kernel has the same lazy offset)
    steps = np.array([0, 1, 3, 3.5, 9, 9, 30, 31, 90, 90, 91, 160, 40, 0, 161, 161], dtype=np.float32)
    ramp = np.repeat(steps[: T // 64], 64) if T // 64 <= 16 else np.repeat(steps, T // 16)
    q = 0.5 + 0.05 * rng.standard_normal((Z, H, T, d)).astype(np.float32)
    k = 0.5 * ramp[None, None, :, None] + 0.05 * rng.standard_normal((Z, H, T, d)).astype(np.float32)
    v = rng.standard_normal((Z, H, T, d)).astype(np.float32)
    q, k, v = (orc.round_to(t, elt) for t in (q, k, v))
    out = ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal)
    assert torch.isfinite(out.float()).all()
    for z, h in [(0, 0), (Z - 1, H - 1)]:
        ref = orc.attention(q[z, h], k[z, h], v[z, h], causal=causal)
        assert_close(_host(out[z, h]), ref, 2e-2, f"attention ramp {shape} {elt} z={z} h={h} causal={causal}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(2, 3, 256, 128), (1, 2, 333, 128), (1, 2, 512, 32), (1, 2, 200, 96), (1, 1, 384, 192),
                                   (1, 2, 257, 256), (1, 1, 1, 128), (2, 2, 64, 32)])
def test_attention_other_head_dims_on_the_matrix_cores(shape, dtype, elt, causal):
    """16-bit tensors with head_dim 32, 96, 128, 192 or 256: the matrix-core kernels for head
    dimensions other than 64 (128: key tiles by LDS-DMA, two stages; the others: copied through
    registers), at sequence lengths that are and are not multiples of the 64-key tile and 128-row
    query block; also on head-innermost views ([batch, seq, heads, d] seen as [batch, heads, seq, d])."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    rng = np.random.default_rng(sum(shape) + 2 * causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    ref = orc.attention(q, k, v, causal=causal, result_type=elt)
    out = ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal)
    assert_close(_host(out), ref, 2e-2, f"attention {shape} {elt} causal={causal}")
    # the same problem on strided views
    qs, ks, vs = (_dev(x, dtype).transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    outs = torch.empty((Z, T, H, D), dtype=dtype, device="cuda").transpose(1, 2)
    ops.attention(qs, ks, vs, causal=causal, out=outs)
    assert torch.equal(outs, out)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(1, 2, 200, 8), (2, 2, 130, 24), (1, 3, 257, 40), (1, 2, 64, 56), (2, 1, 300, 72),
                                   (1, 2, 129, 80), (1, 1, 200, 104), (1, 2, 192, 120), (1, 1, 140, 160),
                                   (1, 1, 131, 224), (1, 1, 70, 248)])
def test_attention_padded_head_dims_on_the_matrix_cores(shape, dtype, elt, causal):
    """16-bit tensors whose head dimension is a multiple of 8 without a kernel width of its own run
    on the next wider matrix-core kernel with the columns from head_dim on masked.  The tensors are
    views into wider buffers whose other columns hold NaN (inputs) or a marker (output): the result
    is that of the head dimension itself and nothing outside it is written."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    W = D + 8 * (1 + (T + D) % 3)  # row stride of the buffers
    rng = np.random.default_rng(sum(shape) + 5 * causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    ref = orc.attention(q, k, v, causal=causal, result_type=elt)

    def widened(x):
        buf = torch.full((Z, H, T, W), float("nan"), dtype=dtype, device="cuda")
        buf[..., :D] = _dev(x, dtype)
        return buf[..., :D]

    out_buf = torch.full((Z, H, T, W), 7.0, dtype=dtype, device="cuda")
    out = out_buf[..., :D]
    ops.attention(widened(q), widened(k), widened(v), causal=causal, out=out)
    assert_close(_host(out), ref, 2e-2, f"attention {shape} {elt} causal={causal}")
    assert torch.all(out_buf[..., D:] == 7.0), "columns past head_dim were written"
    # contiguous tensors give the same bits
    out_c = ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal)
    assert torch.equal(out_c, out)


@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(14, 8, 1024, 64), (14, 8, 1000, 64), (15, 4, 2048, 64), (2, 16, 4096, 64), (1, 128, 1000, 64)])
def test_attention_causal_second_block_per_workgroup(shape, dtype, elt):
    """Causal problems with 3.5 to 4 128-row query blocks per compute unit (256 CUs) and sequences from
    1000 keys on: every workgroup is resident at once and a third of them take a second query block.
    Every (batch, head) slice against an f32 evaluation on the GPU, the first and the last one
    against the f64 oracle; the row after the last query survives."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    g = torch.Generator(device="cuda").manual_seed(sum(shape))
    q, k, v = (torch.randn(shape, device="cuda", generator=g).to(dtype) for _ in range(3))
    buf = torch.full((Z, H, T + 1, D), 55.0, device="cuda", dtype=dtype)
    out = ops.attention(q, k, v, causal=True, out=buf[:, :, :T])
    assert bool((buf[:, :, T] == 55.0).all()), "wrote past the last query row"
    mask = torch.ones(T, T, dtype=torch.bool, device="cuda").tril()
    worst = 0.0
    for z in range(Z):
        sc = torch.einsum("hqd,hkd->hqk", q[z].float(), k[z].float()) / D ** 0.5
        ref = torch.einsum("hqk,hkd->hqd", torch.softmax(sc.masked_fill(~mask, float("-inf")), dim=-1), v[z].float())
        err = ((out[z].float() - ref).abs().amax(dim=(1, 2)) / ref.abs().amax(dim=(1, 2))).max().item()
        worst = max(worst, err)
    assert worst <= 2e-2, f"attention {shape} {elt} causal: worst slice max|err|/max|ref| = {worst:.3e}"
    for z, h in [(0, 0), (Z - 1, H - 1)]:
        ref = orc.attention(_host(q[z, h]), _host(k[z, h]), _host(v[z, h]), causal=True, result_type=elt)
        assert_close(_host(out[z, h]), ref, 2e-2, f"attention {shape} {elt} z={z} h={h} causal, second block per workgroup")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 3, 256, 128), (1, 2, 333, 128), (1, 2, 512, 32), (1, 2, 200, 96), (1, 1, 384, 160),
                                   (1, 1, 130, 192), (1, 1, 320, 224), (1, 2, 257, 256), (1, 1, 1, 128), (2, 2, 64, 32),
                                   (8, 2, 384, 96)])
def test_attention_f32_other_head_dims_on_the_matrix_cores(shape, causal):
    """f32 tensors with head_dim 32, 96, ..., 256: the f32 matrix-core kernel for head dimensions
    other than 64 (K and V tiles copied through registers), at sequence lengths that are and are not
    multiples of the 64-key tile and the 128-row query block; also on head-innermost views."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    rng = np.random.default_rng(sum(shape) + 2 * causal)
    q, k, v = (rng.standard_normal(shape).astype(np.float32) for _ in range(3))
    ref = orc.attention(q, k, v, causal=causal, result_type="f32")
    out = ops.attention(_dev(q, torch.float32), _dev(k, torch.float32), _dev(v, torch.float32), causal=causal)
    assert_close(_host(out), ref, 1e-4, f"attention f32 {shape} causal={causal}")
    qs, ks, vs = (_dev(x, torch.float32).transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    outs = torch.empty((Z, T, H, D), dtype=torch.float32, device="cuda").transpose(1, 2)
    ops.attention(qs, ks, vs, causal=causal, out=outs)
    assert torch.equal(outs, out)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 2, 200, 4), (2, 2, 130, 24), (1, 3, 257, 36), (1, 2, 64, 60), (2, 1, 300, 68),
                                   (1, 2, 129, 100), (1, 1, 200, 124), (1, 1, 140, 132), (1, 1, 131, 180),
                                   (1, 1, 150, 200), (1, 1, 70, 252)])
def test_attention_f32_padded_head_dims_on_the_matrix_cores(shape, causal):
    """f32 head dimensions that are multiples of 4 but not of 32 run on the next wider f32
    matrix-core kernel with the columns from head_dim on masked.  The tensors are views into wider
    buffers whose other columns hold NaN (inputs) or a marker (output): the result is that of the
    head dimension itself and nothing outside it is written."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    W = D + 4 * (1 + (T + D) % 3)  # row stride of the buffers
    rng = np.random.default_rng(sum(shape) + 5 * causal)
    q, k, v = (rng.standard_normal(shape).astype(np.float32) for _ in range(3))
    ref = orc.attention(q, k, v, causal=causal, result_type="f32")

    def widened(x):
        buf = torch.full((Z, H, T, W), float("nan"), dtype=torch.float32, device="cuda")
        buf[..., :D] = _dev(x, torch.float32)
        return buf[..., :D]

    out_buf = torch.full((Z, H, T, W), 7.0, dtype=torch.float32, device="cuda")
    out = out_buf[..., :D]
    ops.attention(widened(q), widened(k), widened(v), causal=causal, out=out)
    assert_close(_host(out), ref, 1e-4, f"attention f32 {shape} causal={causal}")
    assert torch.all(out_buf[..., D:] == 7.0), "columns past head_dim were written"
    out_c = ops.attention(_dev(q, torch.float32), _dev(k, torch.float32), _dev(v, torch.float32), causal=causal)
    assert torch.equal(out_c, out)


def test_attention_f32_head_dim_128_runs_at_matrix_core_speed():
    """[2, 8, 1024, 128] f32: 34 GFLOP.  The matrix-core kernel takes well under a millisecond; the
    one-wave-per-row kernel that other f32 head dimensions (not multiples of 4) still use takes
    tens of milliseconds.  The bound sits between the two with a wide margin on either side."""
    from lighthouse_amd import ops

    q, k, v = (torch.randn(2, 8, 1024, 128, device="cuda") for _ in range(3))
    o = torch.empty_like(q)
    for _ in range(3):
        ops.attention(q, k, v, out=o)
    torch.cuda.synchronize()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    beg.record()
    for _ in range(10):
        ops.attention(q, k, v, out=o)
    end.record()
    torch.cuda.synchronize()
    ms = beg.elapsed_time(end) / 10
    assert ms < 3.0, f"f32 head_dim 128 attention took {ms:.2f} ms per call"


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt,rtol", [(torch.bfloat16, "bf16", 2e-2), (torch.float16, "f16", 2e-2),
                                            (torch.float32, "f32", 1e-4)])
@pytest.mark.parametrize("shape", [(1, 2, 100, 1), (2, 1, 77, 3), (1, 1, 130, 7), (1, 2, 200, 33), (1, 3, 257, 64),
                                   (1, 1, 131, 65), (2, 2, 64, 100), (1, 1, 300, 129), (1, 1, 140, 161), (1, 1, 70, 200),
                                   (1, 1, 129, 255), (1, 2, 192, 256)])
def test_attention_any_head_dim_and_alignment(shape, dtype, elt, rtol, causal):
    """Head dimensions that are no multiple of 8 (16-bit) or 4 (f32), and rows that are not 16-byte
    aligned, run on the matrix-core kernels with element loads and stores.  The tensors are views
    that start one element into buffers with an odd row stride; the other columns hold NaN
    (inputs) or a marker (output): the result is that of the head dimension itself, whatever the
    alignment, and nothing outside it is written."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    W = D + 3 + 2 * ((T + D) % 3)  # odd or even row stride, never a multiple of 16 bytes past an aligned start
    rng = np.random.default_rng(sum(shape) + 7 * causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    ref = orc.attention(q, k, v, causal=causal, result_type=elt)

    def shifted(x):
        buf = torch.full((Z, H, T, W), float("nan"), dtype=dtype, device="cuda")
        buf[..., 1:1 + D] = _dev(x, dtype)
        return buf[..., 1:1 + D]

    out_buf = torch.full((Z, H, T, W), 7.0, dtype=dtype, device="cuda")
    out = out_buf[..., 1:1 + D]
    ops.attention(shifted(q), shifted(k), shifted(v), causal=causal, out=out)
    assert_close(_host(out), ref, rtol, f"attention {shape} {elt} causal={causal}")
    assert torch.all(out_buf[..., :1] == 7.0) and torch.all(out_buf[..., 1 + D:] == 7.0), "columns outside the view were written"
    # contiguous tensors (aligned rows when head_dim allows) run the same kernel with wider accesses: the
    # same bits (64 and 128 have streaming kernels of their own, with other rounding points)
    out_c = ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal)
    if D in (64, 128):
        assert_close(_host(out_c), ref, rtol, f"attention {shape} {elt} causal={causal} contiguous")
    else:
        assert torch.equal(out_c, out)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt,rtol", [(torch.bfloat16, "bf16", 2e-2), (torch.float32, "f32", 1e-4)])
@pytest.mark.parametrize("shape", [(1, 2, 100, 40), (2, 1, 77, 64), (1, 1, 130, 128), (1, 3, 64, 64), (1, 1, 1, 8),
                                   (1, 1, 200, 256), (1, 2, 100, 36), (1, 1, 70, 100), (1, 1, 33, 3)])
def test_attention_any_shape(shape, dtype, elt, rtol, causal):
    """Small and odd shapes of every kind: each takes a matrix-core kernel (16-byte accesses where
    rows and head_dim allow them, element accesses otherwise)."""
    from lighthouse_amd import ops

    rng = np.random.default_rng(sum(shape) + causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    out = ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal)
    ref = orc.attention(q, k, v, causal=causal, result_type=elt)
    assert_close(_host(out), ref, rtol, f"generic attention {shape} {elt} causal={causal}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt,rtol", [(torch.bfloat16, "bf16", 2e-2), (torch.float16, "f16", 2e-2),
                                            (torch.float32, "f32", 1e-4)])
@pytest.mark.parametrize("shape", [(1, 2, 65, 64), (2, 3, 1000, 64), (1, 1, 300, 64), (1, 2, 63, 64), (1, 1, 1, 64),
                                   (2, 2, 192, 64), (12, 20, 449, 64)])
def test_attention_ragged_sequence(shape, dtype, elt, rtol, causal):
    """head_dim 64 with a sequence length that is no multiple of the key tile / query block: the
    MFMA kernels mask the partial last key tile and skip rows past the end (the last shape has more
    than two 256-row groups per CU, i.e. the 64-rows-per-wave 16-bit instantiation); nothing past the
    end is written."""
    from lighthouse_amd import ops

    Z, H, T, d = shape
    rng = np.random.default_rng(sum(shape) + 3 * causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    # outputs live in a longer buffer whose tail must stay untouched
    buf = torch.full((Z, H, T + 70, d), 5.0, device="cuda").to(dtype)
    out = buf[:, :, :T]
    ops.attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), causal=causal, out=out)
    assert torch.all(buf[:, :, T:].float() == 5.0)
    for z, h in {(0, 0), (Z - 1, H - 1)}:
        ref = orc.attention(q[z, h], k[z, h], v[z, h], causal=causal, result_type=elt)
        assert_close(_host(out[z, h]), ref, rtol, f"ragged attention {shape} {elt} z={z} h={h} causal={causal}")


def test_attention_errors():
    from lighthouse_amd import ops

    x = torch.zeros(1, 1, 128, 320, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.attention(x, x, x)          # head_dim above 256
    y = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.attention(y, y, y)          # not on the GPU
    z = torch.zeros(1, 1, 64, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.attention(z, z[:, :, :32], z)


@pytest.mark.parametrize("rows,stages", [(64, None), (32, 3), (32, 4), (32, None), (None, 3)])
@pytest.mark.parametrize("causal", [False, True])
def test_attention_variant_requests(rows, stages, causal):
    """LH_ATTN_ROWS_* / LH_ATTN_STAGES_*: every variant of the head-dimension-64 kernel computes the
    same attention (oracle on one head, equality of all heads with the library's own choice up to
    the rounding of a different summation order)."""
    from lighthouse_amd import ops

    shape = (2, 3, 512, 64)
    g = torch.Generator(device="cuda").manual_seed(21)
    q, k, v = (torch.randn(shape, device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
    out = ops.attention(q, k, v, causal=causal, rows_per_wave=rows, stages=stages)
    ref = orc.attention(q[1, 2].float().cpu().numpy(), k[1, 2].float().cpu().numpy(), v[1, 2].float().cpu().numpy(),
                        causal=causal)
    assert_close(out[1, 2].float().cpu().numpy(), orc.round_bf16(ref), 2e-2, f"attention rows={rows} stages={stages} causal={causal}")
    auto = ops.attention(q, k, v, causal=causal)
    assert (out.float() - auto.float()).abs().max() <= 2e-2 * auto.float().abs().max()


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 3, 512, 64), (1, 2, 64, 64), (1, 2, 192, 64), (1, 3, 320, 64), (2, 2, 1088, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_split_key_range(shape, causal, dtype):
    """LH_ATTN_KSPLIT_2: two groups of four waves per workgroup walk the two halves of a query block's
    key tiles and are combined at the end.  Sequence lengths with an odd tile count, a single tile (the
    second group has nothing to do), a last query block that is partly past the end, strided views
    (the [B, T, 3C] projection buffer of a transformer block): every head against the oracle."""
    from lighthouse_amd import ops

    Z, H, T, d = shape
    g = torch.Generator(device="cuda").manual_seed(33)
    qkv = torch.randn(Z, T, 3, H, d, device="cuda", generator=g).to(dtype)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))       # [Z, H, T, d] views, row stride 3 H d
    out = ops.attention(q, k, v, causal=causal, kv_split=2)
    rnd = orc.round_bf16 if dtype == torch.bfloat16 else orc.round_f16
    for z in range(Z):
        for h in range(H):
            ref = orc.attention(*(t[z, h].float().cpu().numpy() for t in (q, k, v)), causal=causal)
            assert_close(out[z, h].float().cpu().numpy(), rnd(ref), 2e-2 if dtype == torch.bfloat16 else 5e-3,
                         f"attention kv_split=2 {shape} causal={causal} head ({z},{h})")
    whole = ops.attention(q, k, v, causal=causal, kv_split=1, rows_per_wave=64)
    assert (out.float() - whole.float()).abs().max() <= (2e-2 if dtype == torch.bfloat16 else 5e-3) * whole.float().abs().max()


def test_attention_variant_request_errors():
    from lighthouse_amd import ops

    q = torch.zeros(1, 2, 256, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="rows_per_wave"):
        ops.attention(q, q, q, rows_per_wave=48)
    with pytest.raises(ValueError, match="4-stage ring only"):
        ops.attention(q, q, q, rows_per_wave=64, stages=3)
    with pytest.raises(ValueError, match="kv_split"):
        ops.attention(q, q, q, kv_split=3)
    with pytest.raises(ValueError, match="split key range"):
        ops.attention(q, q, q, kv_split=2, rows_per_wave=32)
    q100 = torch.zeros(1, 2, 100, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="multiple of 64"):
        ops.attention(q100, q100, q100, rows_per_wave=64)
    q32 = torch.zeros(1, 2, 256, 64, device="cuda")
    with pytest.raises(ValueError, match="16-bit"):
        ops.attention(q32, q32, q32, rows_per_wave=32)
    q128 = torch.zeros(1, 2, 256, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="head_dim 64"):
        ops.attention(q128, q128, q128, rows_per_wave=32)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(1, 1, 4096, 64), (1, 2, 2048, 64), (1, 3, 1024, 64), (2, 2, 512, 64), (1, 1, 8192, 64),
                                   (1, 5, 1088, 64)])
def test_attention_key_range_split_between_workgroups(shape, dtype, elt, causal):
    """Few query blocks with many key tiles: the key range of every block is shared out to several
    workgroups and a second kernel merges their (unnormalised output, offset, row sum).  Against the
    oracle on sampled heads, on strided views with the same bits, and twice in a row (the temporary
    memory is reused)."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    rng = np.random.default_rng(sum(shape) + 3 * causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    dq, dk, dv = (_dev(x, dtype) for x in (q, k, v))
    out = ops.attention(dq, dk, dv, causal=causal)
    for z, h in {(0, 0), (Z - 1, H - 1)}:
        ref = orc.attention(q[z, h], k[z, h], v[z, h], causal=causal, result_type=elt)
        assert_close(_host(out[z, h]), ref, 2e-2, f"split attention {shape} {elt} z={z} h={h} causal={causal}")
    assert torch.equal(ops.attention(dq, dk, dv, causal=causal), out)
    qs, ks, vs = (x.transpose(1, 2).contiguous().transpose(1, 2) for x in (dq, dk, dv))
    outs = torch.empty((Z, T, H, D), dtype=dtype, device="cuda").transpose(1, 2)
    ops.attention(qs, ks, vs, causal=causal, out=outs)
    assert torch.equal(outs, out)
    # one workgroup per query block (an explicit variant request) gives the same result up to the grouping of the sums
    whole = ops.attention(dq, dk, dv, causal=causal, rows_per_wave=64, kv_split=1)
    assert_close(_host(out), _host(whole), 2e-2, f"split vs whole {shape} {elt} causal={causal}")
    # The same call on a caller's workspace of the size the query gives (no pool memory, no allocation):
    # same bits; a requested variant needs no workspace at all; too small a workspace is refused
    # before anything runs.
    need = ops.attention_workspace_bytes(Z, H, T, D, dtype, causal=causal)
    assert ops.attention_workspace_bytes(Z, H, T, D, dtype, causal=causal, kv_split=1) == 0
    ws = torch.empty(need, device="cuda", dtype=torch.uint8)
    free_before = torch.cuda.mem_get_info()[0]
    out_ws = ops.attention(dq, dk, dv, causal=causal, workspace=ws, out=torch.empty_like(out))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before
    assert torch.equal(out_ws, out)
    if need > 0:
        untouched = torch.full_like(out, 3.0)
        with pytest.raises(ValueError, match="workspace too small"):
            ops.attention(dq, dk, dv, causal=causal, workspace=ws[:need - 256], out=untouched)
        torch.cuda.synchronize()
        assert bool((untouched == 3.0).all())


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,elt", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("shape", [(2, 3, 512, 64), (4, 16, 2048, 64), (1, 2, 200, 64), (8, 12, 1024, 64)])
def test_attention_scores_scaled_in_f32(shape, dtype, elt, causal):
    """LH_ATTN_SCALE_F32: Q as stored, scores scaled in f32 (replace_with_fused_attention.py:386) instead of Q
    multiplied by the scale once and rounded again.  Same tolerance; the error against the f64 oracle
    is not larger than the default's (it is about a fifth smaller in bf16 at the benchmark size, whose
    figures are printed); every kernel variant that has the form; the others refuse it."""
    from lighthouse_amd import ops

    Z, H, T, D = shape
    rng = np.random.default_rng(sum(shape) + 5 * causal)
    q, k, v = (orc.round_to(rng.standard_normal(shape).astype(np.float32), elt) for _ in range(3))
    dq, dk, dv = (_dev(x, dtype) for x in (q, k, v))
    default = _host(ops.attention(dq, dk, dv, causal=causal))
    exact = _host(ops.attention(dq, dk, dv, causal=causal, scale_in_f32=True))
    heads = [(0, 0), (Z - 1, H - 1)] if Z * H > 8 else [(z, h) for z in range(Z) for h in range(H)]
    err_default = err_exact = 0.0
    for z, h in heads:
        ref = orc.attention(q[z, h], k[z, h], v[z, h], causal=causal, result_type=elt)
        assert_close(exact[z, h], ref, 2e-2, f"attention scaled in f32 {shape} {elt} z={z} h={h} causal={causal}",
                     report=shape == (4, 16, 2048, 64) and elt == "bf16" and (z, h) == heads[-1])
        rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        err_default = max(err_default, float(np.sqrt(np.mean((default[z, h] - ref) ** 2))) / rms)
        err_exact = max(err_exact, float(np.sqrt(np.mean((exact[z, h] - ref) ** 2))) / rms)
    assert err_exact <= 1.05 * err_default, (err_exact, err_default)
    if shape == (4, 16, 2048, 64) and elt == "bf16":
        print(f"attention bf16 [4,16,2048,64] causal={causal}: rms error / rms reference {err_default:.3e} with Q scaled once, "
              f"{err_exact:.3e} with the scores scaled in f32")
    if T % 64 == 0:
        for rows in (32, 64):
            got = ops.attention(dq, dk, dv, causal=causal, scale_in_f32=True, rows_per_wave=rows)
            ref = orc.attention(q[0, 0], k[0, 0], v[0, 0], causal=causal, result_type=elt)
            assert_close(_host(got[0, 0]), ref, 2e-2, f"attention scaled in f32, {rows} rows per wave")
        with pytest.raises(ValueError, match="LH_ATTN_SCALE_F32"):
            ops.attention(dq, dk, dv, causal=causal, scale_in_f32=True, kv_split=2)
    q32 = torch.zeros(1, 1, 128, 64, device="cuda")
    with pytest.raises(ValueError, match="16-bit"):
        ops.attention(q32, q32, q32, scale_in_f32=True)
