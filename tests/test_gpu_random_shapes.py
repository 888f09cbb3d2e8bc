"""Seeded random problem shapes through every GEMM dispatch path, bit-exact against the CPU oracle.

Operands are small integers (the `randint(-3, 4)` initialisation of examples/xegpu/matmul.py:143-152),
so every product and partial sum is exact in f32 and the result is independent of the summation
order: the oracle's value is the only correct bit pattern, whatever tile, split or padded copy
the library chooses. Row strides, output strides, transposes, bias, ReLU, accumulate and the
separate residual input are drawn at random; the columns between N and the output's row stride
hold a sentinel that must survive.
"""

import random

import numpy as np
import pytest
import torch

from oracle import lh_oracle as orc

pytestmark = pytest.mark.gpu

_DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def _dim(rnd):
    k = rnd.random()
    if k < 0.3:
        return rnd.randint(1, 200)
    if k < 0.5:
        return 64 * rnd.randint(1, 12)
    if k < 0.65:
        return 256 * rnd.randint(1, 5)
    if k < 0.8:
        return rnd.choice([16, 17, 33, 100, 127, 129, 768, 1000, 2304, 4100])
    return rnd.randint(1, 3000)


def _shape(rnd, limit):
    m, n, k = _dim(rnd), _dim(rnd), _dim(rnd)
    if rnd.random() < 0.25:
        m = rnd.choice([1, 8, 16, 24, 48, 64, 100, 128])  # decode batches
    if rnd.random() < 0.25:
        k = rnd.choice([2048, 4096, 8192, 2112])          # long reductions (split along K)
    while m * n * k > limit:
        if k >= 4096 and n > 256:
            n = max(1, n // 2)
        elif m >= n and m >= k:
            m = max(1, m // 2)
        elif n >= k:
            n = max(1, n // 2)
        else:
            k = max(1, k // 2)
    return m, n, k


def _ints(rng, rows, cols, ld, dtype):
    """[rows, cols] integer matrix as a view of a [rows, ld] device buffer (host copy returned too)."""
    host = rng.integers(-3, 4, (rows, cols)).astype(np.float32)
    buf = torch.zeros((rows, ld), device="cuda", dtype=dtype)
    buf[:, :cols] = torch.from_numpy(host).to("cuda").to(dtype)
    return host, buf[:, :cols]


@pytest.mark.parametrize("seed", range(6))
def test_gemm_random_shapes_are_exact(seed):
    from lighthouse_amd import ops

    rnd = random.Random(1000 + seed)
    rng = np.random.default_rng(seed)
    for case in range(40):
        kind = rnd.choice(["f32", "bf16", "bf16", "f16"])
        dt = _DT[kind]
        m, n, k = _shape(rnd, 1 << 27)
        ta, tb = rnd.random() < 0.15, rnd.random() < 0.15
        a_host, a = _ints(rng, *((k, m) if ta else (m, k)), (m if ta else k) + rnd.choice([0, 0, 0, 8, 1]), dt)
        b_host, b = _ints(rng, *((n, k) if tb else (k, n)), (k if tb else n) + rnd.choice([0, 0, 0, 8, 3]), dt)
        out_kind = kind if kind == "f32" else rnd.choice([kind, kind, "f32"])
        odt = _DT[out_kind]
        has_bias, relu, acc = rnd.random() < 0.5, rnd.random() < 0.4, rnd.random() < 0.25
        resid = not acc and rnd.random() < 0.2
        ldc = n + rnd.choice([0, 0, 0, 8, 2])
        bias_host = rng.integers(-3, 4, n).astype(np.float32) if has_bias else None
        bias = torch.from_numpy(bias_host).to("cuda").to(odt) if has_bias else None
        c_host, c_dev = _ints(rng, m, n, ldc, odt)
        buf = torch.full((m, ldc), 77.0, device="cuda", dtype=odt)
        if acc:
            buf[:, :n] = c_dev
        what = (f"seed {seed} case {case}: {kind}->{out_kind} M={m} N={n} K={k} ta={ta} tb={tb} lda={a.stride(0)} "
                f"ldb={b.stride(0)} ldc={ldc} bias={has_bias} relu={relu} acc={acc} resid={resid}")
        ops.gemm(a, b, bias, out=buf[:, :n], relu=relu, accumulate_c=acc, transpose_a=ta, transpose_b=tb,
                 residual=c_dev if resid else None)
        ref = orc.matmul(a_host, b_host, c_host, bias_host, relu=relu, accumulate_c=acc or resid, transpose_a=ta,
                         transpose_b=tb, result_type=out_kind)
        got = buf[:, :n].float().cpu().numpy()
        assert np.array_equal(got, ref), f"{what}: {(got != ref).sum()} elements differ"
        assert ldc == n or bool((buf[:, n:] == 77.0).all()), f"{what}: wrote past column N"
        if resid:
            assert np.array_equal(c_dev.float().cpu().numpy(), c_host), f"{what}: residual input modified"


@pytest.mark.parametrize("seed", range(3))
def test_gemm_fp8_random_shapes_are_exact(seed):
    from lighthouse_amd import ops

    rnd = random.Random(2000 + seed)
    rng = np.random.default_rng(100 + seed)
    for case in range(40):
        m, n, k = _shape(rnd, 1 << 27)
        lda, ldb = k + rnd.choice([0, 0, 16, 3]), n + rnd.choice([0, 0, 16, 5])
        ldc = n + rnd.choice([0, 0, 8, 1])
        a_host = rng.integers(-3, 4, (m, k)).astype(np.float32)
        b_host = rng.integers(-3, 4, (k, n)).astype(np.float32)
        a_codes, b_codes = orc.e4m3_quant(a_host), orc.e4m3_quant(b_host)
        aq = torch.zeros((m, lda), device="cuda", dtype=torch.uint8)
        bq = torch.zeros((k, ldb), device="cuda", dtype=torch.uint8)
        aq[:, :k] = torch.from_numpy(a_codes).to("cuda")
        bq[:, :n] = torch.from_numpy(b_codes).to("cuda")
        sa, sb = rnd.choice([1.0, 0.5, 0.25]), rnd.choice([1.0, 2.0, 0.125])
        out_kind = rnd.choice(["bf16", "bf16", "f32"])
        buf = torch.full((m, ldc), 77.0, device="cuda", dtype=_DT[out_kind])
        what = f"seed {seed} case {case}: fp8->{out_kind} M={m} N={n} K={k} lda={lda} ldb={ldb} ldc={ldc}"
        ops.gemm_fp8(aq[:, :k].view(torch.float8_e4m3fn), bq[:, :n].view(torch.float8_e4m3fn), sa, sb,
                     out=buf[:, :n])
        ref = orc.matmul_fp8(a_codes, b_codes, sa, sb, result_type=out_kind)
        got = buf[:, :n].float().cpu().numpy()
        assert np.array_equal(got, ref), f"{what}: {(got != ref).sum()} elements differ"
        assert ldc == n or bool((buf[:, n:] == 77.0).all()), f"{what}: wrote past column N"


@pytest.mark.parametrize("seed", range(3))
def test_attention_random_shapes_and_layouts(seed):
    """Random [Z,H,T,d] problems (every kernel family: head dimension 64, 128, other multiples of 32,
    of 8 and of 4, anything else), causal or not, in four memory layouts (one of them misaligned, inside
    NaN padding); the row after the last query must survive."""
    from lighthouse_amd import ops
    from tests.conftest import assert_close

    rnd = random.Random(3000 + seed)
    rng = np.random.default_rng(200 + seed)
    for case in range(25):
        kind = rnd.choice(["bf16", "bf16", "f16", "f32"])
        dt = _DT[kind]
        d = rnd.choice([64, 64, 64, 128, 128, 32, 96, 192, 256, 40, 80, 16, 100, 36, 7, 65, 130, 255])
        z, h = rnd.randint(1, 3), rnd.randint(1, 6)
        t = rnd.choice([rnd.randint(1, 300), 64 * rnd.randint(1, 12), 256 * rnd.randint(1, 4), rnd.randint(1, 1100)])
        while z * h * t * t * d > (1 << 28):
            t = max(1, t // 2)
        causal = rnd.random() < 0.5
        layout = rnd.choice(["zhtd", "zthd", "packed", "shifted"])
        what = f"seed {seed} case {case}: {kind} Z={z} H={h} T={t} d={d} causal={causal} {layout}"
        host = orc.round_to(rng.standard_normal((3, z, h, t, d)).astype(np.float32), kind)
        if layout == "zhtd":
            q, k, v = (torch.from_numpy(host[i]).to("cuda").to(dt) for i in range(3))
        elif layout == "zthd":
            q, k, v = (torch.from_numpy(host[i]).to("cuda").to(dt).transpose(1, 2).contiguous().transpose(1, 2)
                       for i in range(3))
        elif layout == "shifted":  # views that start one element into rows of d + 3 elements; NaN around them
            wide = torch.full((3, z, h, t, d + 3), float("nan"), device="cuda", dtype=dt)
            wide[..., 1:1 + d] = torch.from_numpy(host).to("cuda").to(dt)
            q, k, v = (wide[i, ..., 1:1 + d] for i in range(3))
        else:  # one [Z, T, 3, H, d] tensor, as the fused QKV projection of the nanoGPT block leaves it
            packed = torch.from_numpy(host).to("cuda").to(dt).permute(1, 3, 0, 2, 4).contiguous()
            q, k, v = (packed[:, :, i].transpose(1, 2) for i in range(3))
        buf = torch.full((z, h, t + 1, d), 55.0, device="cuda", dtype=dt)
        out = ops.attention(q, k, v, causal=causal, out=buf[:, :, :t])
        ref = orc.attention(host[0], host[1], host[2], causal=causal, result_type=kind)
        assert_close(out.float().cpu().numpy(), ref, 1e-4 if kind == "f32" else 2e-2, what)
        assert bool((buf[:, :, t] == 55.0).all()), f"{what}: wrote past the last query row"


@pytest.mark.parametrize("seed", range(3))
def test_rows_random_lengths(seed):
    """LayerNorm and softmax over random row counts and lengths (every row kernel: register-resident exact
    and masked, one workgroup per row, scalar), with a sentinel row after the result."""
    from lighthouse_amd import ops
    from tests.conftest import assert_close

    rnd = random.Random(4000 + seed)
    rng = np.random.default_rng(300 + seed)
    for case in range(40):
        kind = rnd.choice(["f32", "bf16"])
        m = rnd.choice([1, 3, rnd.randint(1, 600), 1024])
        n = rnd.choice([rnd.randint(1, 600), 4 * rnd.randint(1, 1100), 256 * rnd.randint(1, 20), rnd.randint(1, 20000),
                        4 * rnd.randint(1000, 5000)])
        while m * n > (1 << 21):
            m = max(1, m // 2)
        out_kind = rnd.choice([kind, "bf16" if kind == "f32" else "f32"])
        what = f"seed {seed} case {case}: {kind}->{out_kind} M={m} N={n}"
        x = orc.round_to(rng.standard_normal((m, n)).astype(np.float32) * 2 + 0.5, kind)
        g = rng.uniform(0.5, 1.5, n).astype(np.float32)
        b = rng.uniform(-0.1, 0.1, n).astype(np.float32)
        xd = torch.from_numpy(x).to("cuda").to(_DT[kind])
        buf = torch.full((m + 1, n), 55.0, device="cuda", dtype=_DT[out_kind])
        ops.layer_norm(xd, torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda(), 1e-5, out=buf[:m])
        rtol = 1e-4 if (kind, out_kind) == ("f32", "f32") else 2e-2
        assert_close(buf[:m].float().cpu().numpy(), orc.layer_norm(x, g, b, 1e-5, result_type=out_kind), rtol,
                     "layer_norm " + what)
        assert bool((buf[m] == 55.0).all()), f"layer_norm {what}: wrote past the last row"
        buf = torch.full((m + 1, n), 55.0, device="cuda", dtype=_DT[kind])
        ops.softmax(xd, out=buf[:m])
        assert_close(buf[:m].float().cpu().numpy(), orc.softmax(x, result_type=kind), 1e-4 if kind == "f32" else 2e-2,
                     "softmax " + what)
        assert bool((buf[m] == 55.0).all()), f"softmax {what}: wrote past the last row"
