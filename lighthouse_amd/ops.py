"""Torch-tensor front end of the C ABI: launches on torch's current stream, no allocation
except outputs the caller did not pass.  Used by the torch ingress path, the benchmark and
the tests; every function goes straight to liblighthouse_hip.so.
"""

from __future__ import annotations

import ctypes
import math

import torch

from . import _lib
from .utils.numpy import lh_dtype


def _stream() -> int:
    """Raw handle of torch's current stream on the current device (the accessor torch's own
    extensions use: no Stream object is built per launch)."""
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def _need_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("expected tensors on the GPU")


def device_info() -> dict:
    info = _lib.DeviceInfo()
    _lib.check(_lib.load().lh_hip_device_info(ctypes.byref(info)), "device_info")
    return {
        "arch": info.arch.decode(), "name": info.name.decode(), "compute_units": info.compute_units,
        "clock_khz": info.clock_khz, "memory_clock_khz": info.memory_clock_khz,
        "memory_bus_bits": info.memory_bus_bits, "lds_bytes_per_cu": info.lds_bytes_per_cu,
        "wavefront_size": info.wavefront_size, "hbm_bytes": info.hbm_bytes,
    }


def gemm(a, b, bias=None, *, out=None, out_dtype=None, relu=False, gelu=False, accumulate_c=False,
         transpose_a=False, transpose_b=False, tile=None, residual=None):
    """out = epilogue(A @ B); see lh_hip_gemm.  `tile=(bm, bn)` requests a workgroup tile;
    `residual` [M, N] is added to A @ B before the epilogue (lh_hip_gemm_residual) and is left intact."""
    _need_cuda(a, b, bias, out, residual)
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("gemm expects 2-D tensors")
    if a.stride(1) != 1 or b.stride(1) != 1:
        raise ValueError("innermost stride must be 1")
    M, K = (a.shape[1], a.shape[0]) if transpose_a else a.shape
    N = b.shape[0] if transpose_b else b.shape[1]
    if out is None:
        if accumulate_c:
            raise ValueError("accumulate_c needs an explicit out tensor")
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    flags = ((_lib.GEMM_HAS_BIAS if bias is not None else 0) | (_lib.GEMM_HAS_RELU if relu else 0)
             | (_lib.GEMM_HAS_GELU if gelu else 0) | (_lib.GEMM_ACCUMULATE_C if accumulate_c else 0)
             | (_lib.GEMM_TRANSPOSE_A if transpose_a else 0) | (_lib.GEMM_TRANSPOSE_B if transpose_b else 0))
    if tile is None and a.dtype in (torch.bfloat16, torch.float16) and not (transpose_a or transpose_b):
        from .tuning.tile_db import active_db  # a tuned tile for this shape, if a database is in use

        db = active_db()
        if db is not None:
            tile = db.lookup("bf16" if a.dtype == torch.bfloat16 else "f16", M, N, K)
    if tile is not None:
        if tuple(tile) not in _lib.GEMM_TILES:
            raise ValueError(f"unsupported tile {tile}; choose from {sorted(_lib.GEMM_TILES)}")
        flags |= _lib.GEMM_TILES[tuple(tile)]
    if bias is not None and bias.dtype != out.dtype:
        raise ValueError("bias must have the output dtype")
    if a.dtype != b.dtype:
        raise ValueError("A and B must have the same dtype")
    if residual is not None:
        if accumulate_c:
            raise ValueError("residual and accumulate_c are exclusive")
        if tuple(residual.shape) != (M, N) or residual.dtype != out.dtype or residual.stride(1) != 1 \
                or residual.stride(0) != out.stride(0):
            raise ValueError("residual must be an [M, N] matrix of the output dtype with the output's row stride")
        _lib.check(_lib.load().lh_hip_gemm_residual(
            out.data_ptr(), residual.data_ptr(), a.data_ptr(), b.data_ptr(),
            bias.data_ptr() if bias is not None else None, M, N, K, a.stride(0), b.stride(0), out.stride(0),
            lh_dtype(a.dtype), lh_dtype(out.dtype), flags, _stream()), "gemm")
        return out
    _lib.check(_lib.load().lh_hip_gemm(
        out.data_ptr(), a.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None,
        M, N, K, a.stride(0), b.stride(0), out.stride(0), lh_dtype(a.dtype), lh_dtype(out.dtype), flags, _stream()),
        "gemm")
    return out


def gemm_fp8(a_q, b_q, scale_a: float, scale_b: float, *, out=None, out_dtype=torch.bfloat16):
    """out = out_dtype((Aq @ Bq)_f32 * scale_a * scale_b); see lh_hip_gemm_fp8."""
    _need_cuda(a_q, b_q, out)
    M, K = a_q.shape
    N = b_q.shape[1]
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a_q.device)
    _lib.check(_lib.load().lh_hip_gemm_fp8(
        out.data_ptr(), a_q.data_ptr(), b_q.data_ptr(), float(scale_a), float(scale_b), M, N, K,
        a_q.stride(0), b_q.stride(0), out.stride(0), lh_dtype(out.dtype), _stream()), "gemm_fp8")
    return out


def _strides3(t) -> _lib.Strides3:
    return _lib.Strides3(t.stride(0), t.stride(1), t.stride(2))


def attention(q, k, v, *, causal=False, scale=None, out=None):
    """Fused attention forward on [Z,H,T,d] tensors (any strides with unit stride along d)."""
    _need_cuda(q, k, v, out)
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("attention expects Q, K, V of equal 4-D shape [Z,H,T,d]")
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    for t in (q, k, v, out):
        if t.stride(3) != 1:
            raise ValueError("innermost stride must be 1")
    Z, H, T, d = q.shape
    _lib.check(_lib.load().lh_hip_attention(
        out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), Z, H, T, d,
        _strides3(out), _strides3(q), _strides3(k), _strides3(v),
        float(scale) if scale is not None else 1.0 / math.sqrt(d), 1 if causal else 0, lh_dtype(q.dtype), _stream()),
        "attention")
    return out


def layer_norm(x, gamma, beta, eps=1e-5, *, out=None, out_dtype=None):
    _need_cuda(x, gamma, beta, out)
    M, N = x.shape
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    if gamma.dtype != torch.float32 or beta.dtype != torch.float32:
        raise ValueError("gamma and beta must be float32")
    if not x.is_contiguous() or not out.is_contiguous():
        raise ValueError("layer_norm expects contiguous tensors")
    _lib.check(_lib.load().lh_hip_layer_norm(
        out.data_ptr(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), M, N, float(eps),
        lh_dtype(x.dtype), lh_dtype(out.dtype), _stream()), "layer_norm")
    return out


def softmax(x, *, out=None):
    _need_cuda(x, out)
    out = torch.empty_like(x) if out is None else out
    M, N = x.shape
    _lib.check(_lib.load().lh_hip_softmax(out.data_ptr(), x.data_ptr(), M, N, lh_dtype(x.dtype), _stream()), "softmax")
    return out


def gelu_tanh(x, *, out=None):
    _need_cuda(x, out)
    out = torch.empty_like(x) if out is None else out
    _lib.check(_lib.load().lh_hip_gelu_tanh(out.data_ptr(), x.data_ptr(), x.numel(), lh_dtype(x.dtype), _stream()),
               "gelu_tanh")
    return out


def bias_act(x, bias, relu=False, *, out=None):
    _need_cuda(x, bias, out)
    out = torch.empty_like(x) if out is None else out
    M, N = x.shape
    _lib.check(_lib.load().lh_hip_bias_act(out.data_ptr(), x.data_ptr(), bias.data_ptr(), M, N, 1 if relu else 0,
                                           lh_dtype(x.dtype), _stream()), "bias_act")
    return out


def add(a, b, *, out=None):
    _need_cuda(a, b, out)
    out = torch.empty_like(a) if out is None else out
    _lib.check(_lib.load().lh_hip_add(out.data_ptr(), a.data_ptr(), b.data_ptr(), a.numel(), lh_dtype(a.dtype),
                                      _stream()), "add")
    return out


def cast(x, dtype, *, out=None):
    _need_cuda(x, out)
    out = torch.empty(x.shape, dtype=dtype, device=x.device) if out is None else out
    _lib.check(_lib.load().lh_hip_cast(out.data_ptr(), x.data_ptr(), x.numel(), lh_dtype(x.dtype), lh_dtype(dtype),
                                       _stream()), "cast")
    return out


BLOCK_PARAM_NAMES = ("ln1_g", "ln1_b", "w_qkv", "b_qkv", "w_o", "b_o", "ln2_g", "ln2_b", "w_fc", "b_fc", "w_proj",
                     "b_proj")


def nanogpt_block_workspace_bytes(B, T, C, dtype) -> int:
    return int(_lib.load().lh_hip_nanogpt_block_workspace_bytes(B, T, C, lh_dtype(dtype)))


def nanogpt_block(x, params: dict, n_head: int, *, eps=1e-5, out=None, workspace=None):
    """One GPT-2 block forward. x: [B,T,C] float32; params: tensors named BLOCK_PARAM_NAMES with
    weights stored [in,out] in float32 or bfloat16 (LayerNorm parameters float32)."""
    _need_cuda(x, out, workspace, *params.values())
    B, T, C = x.shape
    dtype = params["w_qkv"].dtype
    if out is None:
        out = torch.empty_like(x)
    need = nanogpt_block_workspace_bytes(B, T, C, dtype)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    p = _lib.NanoGPTBlockParams(*[params[n].data_ptr() for n in BLOCK_PARAM_NAMES])
    _lib.check(_lib.load().lh_hip_nanogpt_block(
        out.data_ptr(), x.data_ptr(), ctypes.byref(p), B, T, C, n_head, float(eps), lh_dtype(dtype),
        workspace.data_ptr(), workspace.numel(), _stream()), "nanogpt_block")
    return out


def nanogpt_forward(x, layers: list, lnf_g, lnf_b, lm_w, lm_b, n_head: int, *, eps=1e-5, out=None, workspace=None):
    """n blocks + final LayerNorm + lm_head. x: [B,T,C] float32; `layers`: one parameter dict per
    block (see nanogpt_block); lm_w [C, vocab] and lm_b [vocab] in the blocks' dtype. Returns float32
    logits [B,T,vocab]."""
    _need_cuda(x, out, workspace, lnf_g, lnf_b, lm_w, lm_b, *[t for p in layers for t in p.values()])
    B, T, C = x.shape
    vocab = lm_w.shape[1]
    dtype = lm_w.dtype
    if out is None:
        out = torch.empty((B, T, vocab), dtype=torch.float32, device=x.device)
    need = int(_lib.load().lh_hip_nanogpt_forward_workspace_bytes(B, T, C, lh_dtype(dtype)))
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    blocks = (_lib.NanoGPTBlockParams * max(len(layers), 1))(
        *[_lib.NanoGPTBlockParams(*[p[n].data_ptr() for n in BLOCK_PARAM_NAMES]) for p in layers])
    _lib.check(_lib.load().lh_hip_nanogpt_forward(
        out.data_ptr(), x.data_ptr(), blocks, len(layers), lnf_g.data_ptr(), lnf_b.data_ptr(), lm_w.data_ptr(),
        lm_b.data_ptr() if lm_b is not None else None, B, T, C, n_head, vocab, float(eps), lh_dtype(dtype),
        workspace.data_ptr(), workspace.numel(), _stream()), "nanogpt_forward")
    return out


def probe_mfma_rate(dtype, random_operands: bool, iters: int = 20000) -> float:
    """TFLOP/s of a register-only MFMA loop on every SIMD (see lh_hip_probe_mfma_rate)."""
    out = ctypes.c_double(0.0)
    _lib.check(_lib.load().lh_hip_probe_mfma_rate(lh_dtype(dtype), 1 if random_operands else 0, int(iters),
                                                  ctypes.byref(out)), "probe_mfma_rate")
    return out.value
