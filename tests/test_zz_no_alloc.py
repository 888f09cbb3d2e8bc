"""lh_hip_gemm_static: the GEMM entry point that allocates nothing (temporaries in a device array
that is part of the library's image), called through the C ABI and compared bit for bit with
lh_hip_gemm on the same inputs: a decode shape that is cut along K, then a smaller one (the array
keeps the first call's contents), then problems with padded operands and a transposed A (copies in
the array), a transposed B and a plain problem (no temporaries), then one whose temporaries exceed
the array."""

import ctypes

import numpy as np
import pytest
import torch

from lighthouse_amd import _lib

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 << 20


def _call(fn, out, a, b, bias, M, N, K, flags, stream=None):
    return fn(out.data_ptr(), a.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None, M, N, K,
              a.stride(0), b.stride(0), out.stride(0), _lib.BF16, _lib.F32 if out.dtype == torch.float32 else _lib.BF16,
              flags, stream)


def _problem(M, N, K, seed, transpose_b=False, transpose_a=False):
    g = torch.Generator(device="cuda").manual_seed(seed)
    a = torch.randn((K, M) if transpose_a else (M, K), device="cuda", generator=g).to(torch.bfloat16)
    b = torch.randn((N, K) if transpose_b else (K, N), device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16)
    return a, b, bias


def test_static_scratch_gemm_matches_the_pooled_entry_point():
    lib = _lib.load()
    flags = _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU
    # (M, N, K, extra flags): cut along K (4 MiB of partial sums); smaller, cut along K; ragged N and K
    # (padded copies); transposed A (untransposed copy); then no temporaries at all: transposed B (read in
    # place), plain
    cases = [(16, 8192, 8192, 0), (16, 1024, 4096, 0), (300, 520, 776, 0), (512, 512, 512, _lib.GEMM_TRANSPOSE_A),
             (512, 512, 512, _lib.GEMM_TRANSPOSE_B), (512, 512, 512, 0)]
    # The array itself becomes resident on the device when the runtime is first asked for its
    # address; one call up front keeps that out of the memory readings below.
    a, b, bias = _problem(256, 256, 256, 99)
    first = torch.empty(256, 256, device="cuda", dtype=torch.bfloat16)
    _lib.check(_call(lib.lh_hip_gemm_static, first, a, b, bias, 256, 256, 256, flags), "lh_hip_gemm_static")
    torch.cuda.synchronize()
    for i, (M, N, K, extra) in enumerate(cases):
        tb, ta = bool(extra & _lib.GEMM_TRANSPOSE_B), bool(extra & _lib.GEMM_TRANSPOSE_A)
        a, b, bias = _problem(M, N, K, 100 + i, tb, ta)
        need = lib.lh_hip_gemm_workspace_bytes(M, N, K, a.stride(0), b.stride(0), N, _lib.BF16, _lib.BF16, flags | extra)
        assert need <= STATIC_BYTES and (need > 0) == (i < 4)
        want = torch.full((M, N), 3.0, device="cuda", dtype=torch.bfloat16)
        got = torch.full((M, N), 5.0, device="cuda", dtype=torch.bfloat16)
        _lib.check(_call(lib.lh_hip_gemm, want, a, b, bias, M, N, K, flags | extra), "lh_hip_gemm")
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        _lib.check(_call(lib.lh_hip_gemm_static, got, a, b, bias, M, N, K, flags | extra), "lh_hip_gemm_static")
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] >= free_before  # the call took no device memory
        assert torch.equal(got, want), (M, N, K)
        ref = torch.relu((a.float().T if ta else a.float()) @ (b.float().T if tb else b.float()) + bias.float())
        assert (got.float() - ref).abs().max() <= 2e-2 * ref.abs().max()
    # the two decode shapes again in the opposite order, back to back on one stream without a
    # synchronisation in between: the second call's kernels run after the first call's
    (a1, b1, bias1), (a2, b2, bias2) = _problem(16, 1024, 4096, 101), _problem(16, 8192, 8192, 100)
    o1 = torch.empty(16, 1024, device="cuda", dtype=torch.bfloat16)
    o2 = torch.empty(16, 8192, device="cuda", dtype=torch.bfloat16)
    w1, w2 = torch.empty_like(o1), torch.empty_like(o2)
    _lib.check(_call(lib.lh_hip_gemm_static, o1, a1, b1, bias1, 16, 1024, 4096, flags), "static")
    _lib.check(_call(lib.lh_hip_gemm_static, o2, a2, b2, bias2, 16, 8192, 8192, flags), "static")
    _lib.check(_call(lib.lh_hip_gemm, w1, a1, b1, bias1, 16, 1024, 4096, flags), "pooled")
    _lib.check(_call(lib.lh_hip_gemm, w2, a2, b2, bias2, 16, 8192, 8192, flags), "pooled")
    torch.cuda.synchronize()
    assert torch.equal(o1, w1) and torch.equal(o2, w2)


def test_static_scratch_gemm_refuses_what_does_not_fit():
    lib = _lib.load()
    M, N, K = 128, 8192, 8192
    cut8 = _lib.GEMM_SPLITK[8]  # eight f32 blocks of 128 x 8192: 32 MiB (the library's own choice, four, just fits)
    assert lib.lh_hip_gemm_workspace_bytes(M, N, K, K, N, N, _lib.BF16, _lib.BF16, 0) <= STATIC_BYTES
    assert lib.lh_hip_gemm_workspace_bytes(M, N, K, K, N, N, _lib.BF16, _lib.BF16, cut8) > STATIC_BYTES
    a, b, _ = _problem(M, N, K, 7)
    out = torch.full((M, N), 9.0, device="cuda", dtype=torch.bfloat16)
    rc = _call(lib.lh_hip_gemm_static, out, a, b, None, M, N, K, cut8)
    assert rc == _lib.LH_ERR_INVALID
    assert b"static scratch holds" in lib.lh_hip_last_error()
    torch.cuda.synchronize()
    assert bool((out == 9.0).all())  # nothing ran
    with pytest.raises(ValueError):
        _lib.check(rc, "lh_hip_gemm_static")
    # argument validation is the plain entry point's
    assert _call(lib.lh_hip_gemm_static, out, a, b, None, 0, N, K, 0) == _lib.LH_ERR_INVALID


def test_static_scratch_gemm_with_misaligned_operands():
    """Operands that are not 16-byte aligned run on padded copies, which the pointer-less workspace
    query does not count; the entry points that must not allocate compute the need from the actual
    pointers, so the call either matches lh_hip_gemm bit for bit or is refused up front with the
    output untouched, never half way through."""
    lib = _lib.load()
    flags = _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU
    g = torch.Generator(device="cuda").manual_seed(5)

    def shifted(rows, cols, ld):
        # an [rows, cols] matrix with row stride ld whose first element sits 2 bytes past an aligned address
        buf = torch.randn(rows * ld + 8, device="cuda", generator=g).to(torch.bfloat16)
        return buf[1:1 + rows * ld].view(rows, ld)[:, :cols]

    # small: the padded copies fit the array
    M, N, K = 384, 512, 512
    a, b = shifted(M, K, K + 8), shifted(K, N, N + 8)
    bias = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16)
    assert a.data_ptr() % 16 == 2 and b.data_ptr() % 16 == 2
    want = torch.full((M, N), 3.0, device="cuda", dtype=torch.bfloat16)
    got = torch.full((M, N), 5.0, device="cuda", dtype=torch.bfloat16)
    plain = lib.lh_hip_gemm_workspace_bytes(M, N, K, a.stride(0), b.stride(0), N, _lib.BF16, _lib.BF16, flags)
    exact = lib.lh_hip_gemm_workspace_bytes_for(got.data_ptr(), a.data_ptr(), b.data_ptr(), bias.data_ptr(), M, N, K,
                                                a.stride(0), b.stride(0), N, _lib.BF16, _lib.BF16, flags)
    assert plain == 0 and 0 < exact <= STATIC_BYTES
    _lib.check(_call(lib.lh_hip_gemm, want, a, b, bias, M, N, K, flags), "lh_hip_gemm")
    _lib.check(_call(lib.lh_hip_gemm_static, got, a, b, bias, M, N, K, flags), "lh_hip_gemm_static")
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    ref = torch.relu(a.float() @ b.float() + bias.float())
    assert (got.float() - ref).abs().max() <= 2e-2 * ref.abs().max()
    # the workspace entry point with exactly that many bytes, and refused up front with one byte short of a block
    ws = torch.empty(exact, device="cuda", dtype=torch.uint8)
    got2 = torch.full((M, N), 5.0, device="cuda", dtype=torch.bfloat16)
    rc = lib.lh_hip_gemm_ws(got2.data_ptr(), a.data_ptr(), b.data_ptr(), bias.data_ptr(), M, N, K, a.stride(0), b.stride(0),
                            N, _lib.BF16, _lib.BF16, flags, ws.data_ptr(), exact, None)
    _lib.check(rc, "lh_hip_gemm_ws")
    torch.cuda.synchronize()
    assert torch.equal(got2, want)
    got2.fill_(7.0)
    rc = lib.lh_hip_gemm_ws(got2.data_ptr(), a.data_ptr(), b.data_ptr(), bias.data_ptr(), M, N, K, a.stride(0), b.stride(0),
                            N, _lib.BF16, _lib.BF16, flags, ws.data_ptr(), exact - 256, None)
    assert rc == _lib.LH_ERR_INVALID and b"workspace too small" in lib.lh_hip_last_error()
    torch.cuda.synchronize()
    assert bool((got2 == 7.0).all())
    # large, with a transposed and misaligned A: more than the array holds although the aligned query
    # says otherwise; refused before the transpose kernel (or anything else) is enqueued
    M, N, K = 4096, 2048, 2048
    a_t, b = shifted(K, M, M + 8), shifted(K, N, N + 8)
    out = torch.full((M, N), 9.0, device="cuda", dtype=torch.bfloat16)
    fl = _lib.GEMM_TRANSPOSE_A
    aligned_need = lib.lh_hip_gemm_workspace_bytes(M, N, K, a_t.stride(0), b.stride(0), N, _lib.BF16, _lib.BF16, fl)
    exact = lib.lh_hip_gemm_workspace_bytes_for(out.data_ptr(), a_t.data_ptr(), b.data_ptr(), None, M, N, K, a_t.stride(0),
                                                b.stride(0), N, _lib.BF16, _lib.BF16, fl)
    assert exact > STATIC_BYTES >= 0 and exact > aligned_need
    rc = _call(lib.lh_hip_gemm_static, out, a_t, b, None, M, N, K, fl)
    assert rc == _lib.LH_ERR_INVALID and b"static scratch holds" in lib.lh_hip_last_error()
    torch.cuda.synchronize()
    assert bool((out == 9.0).all())  # nothing ran
