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


# The C side sees pointers and sizes only, so everything it cannot check is checked here, before
# any device work: a mismatched call must raise, not read or write outside a buffer.
_FLOATS = (torch.float32, torch.bfloat16, torch.float16)


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _tuned_db():
    """The active tuned-parameter database (None when there is none); the import is deferred so that
    loading this module does not read the database file."""
    global _active_db
    if _active_db is None:
        from .tuning.tile_db import active_db

        _active_db = active_db
    return _active_db()


_active_db = None
_DTYPE_NAMES = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}


def _rows_aligned16(*tensors) -> bool:
    """Base address and every stride but the innermost are multiples of 16 bytes."""
    for t in tensors:
        if t is None:
            continue
        per = 16 // t.element_size()
        if t.data_ptr() % 16 or any(s % per for s in t.stride()[:-1]):
            return False
    return True


def _is_matrix(t, rows, cols, what: str) -> None:
    _require(t.dim() == 2 and tuple(t.shape) == (rows, cols), f"{what} must have shape [{rows}, {cols}], got {tuple(t.shape)}")
    _require(t.stride(1) == 1 or cols == 1, f"{what}: innermost stride must be 1")
    _require(t.stride(0) >= cols or rows == 1, f"{what}: rows overlap (stride {t.stride(0)} < {cols} columns)")


def _is_vector(t, n, dtype, what: str) -> None:
    _require(t.dim() == 1 and t.shape[0] == n, f"{what} must have shape [{n}], got {tuple(t.shape)}")
    _require(t.dtype == dtype, f"{what} must be {dtype}, got {t.dtype}")
    _require(t.stride(0) == 1 or n == 1, f"{what} must be contiguous")


def _same_dense(out, x, what: str) -> None:
    _require(tuple(out.shape) == tuple(x.shape) and out.dtype == x.dtype,
             f"{what}: out must have the shape and dtype of the input ({tuple(x.shape)}, {x.dtype})")
    _require(x.is_contiguous() and out.is_contiguous(), f"{what} expects contiguous tensors")


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
         transpose_a=False, transpose_b=False, tile=None, split_k=None, residual=None, workspace=None):
    """out = epilogue(A @ B); see lh_hip_gemm.  `tile=(bm, bn)` requests a workgroup tile and
    `split_k` (1 = never, 2 / 4 / 8) a cut along K for the 16-bit kernels (f32 inputs take the tiles
    128x128, 128x64 and 64x64 and no cut); with neither given the
    tuned-parameter database is asked, then the library's own choice applies;
    `residual` [M, N] is added to A @ B before the epilogue (lh_hip_gemm_residual) and is left intact;
    `workspace` (uint8, see gemm_workspace_bytes) makes the call take its temporary memory from
    there instead of the library's pool (lh_hip_gemm_ws)."""
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("gemm expects 2-D tensors")
    if a.stride(1) != 1 or b.stride(1) != 1:
        raise ValueError("innermost stride must be 1")
    _require(a.dtype in _FLOATS, f"unsupported A/B dtype {a.dtype}")
    if a.dtype != b.dtype:
        raise ValueError("A and B must have the same dtype")
    M, K = (a.shape[1], a.shape[0]) if transpose_a else a.shape
    N = b.shape[0] if transpose_b else b.shape[1]
    _require((b.shape[1] if transpose_b else b.shape[0]) == K,
             f"B has {b.shape[1] if transpose_b else b.shape[0]} rows of K, A has {K}")
    _require(a.stride(0) >= a.shape[1] and b.stride(0) >= b.shape[1], "rows of A or B overlap")
    if out is None:
        if accumulate_c:
            raise ValueError("accumulate_c needs an explicit out tensor")
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    _is_matrix(out, M, N, "out")
    _require(out.dtype in (torch.float32, a.dtype), "out must be float32 or have the A/B dtype")
    if bias is not None:
        if bias.dtype != out.dtype:
            raise ValueError("bias must have the output dtype")
        _is_vector(bias, N, out.dtype, "bias")
    if residual is not None:
        if accumulate_c or workspace is not None:
            raise ValueError("residual excludes accumulate_c and workspace")
        if tuple(residual.shape) != (M, N) or residual.dtype != out.dtype or residual.stride(1) != 1 \
                or residual.stride(0) != out.stride(0):
            raise ValueError("residual must be an [M, N] matrix of the output dtype with the output's row stride")
    if workspace is not None:
        _require(workspace.dtype == torch.uint8 and workspace.dim() == 1 and workspace.is_contiguous(),
                 "workspace must be a contiguous uint8 vector")
    _need_cuda(a, b, bias, out, residual, workspace)
    flags = ((_lib.GEMM_HAS_BIAS if bias is not None else 0) | (_lib.GEMM_HAS_RELU if relu else 0)
             | (_lib.GEMM_HAS_GELU if gelu else 0) | (_lib.GEMM_ACCUMULATE_C if accumulate_c else 0)
             | (_lib.GEMM_TRANSPOSE_A if transpose_a else 0) | (_lib.GEMM_TRANSPOSE_B if transpose_b else 0))
    if tile is None and split_k is None and not transpose_a:  # (a transposed B runs on the same kernels in place)
        db = _tuned_db()  # tuned parameters for this shape, if the database has any
        if db is not None:
            tile, split_k = db.lookup_gemm(_DTYPE_NAMES[a.dtype], M, N, K)
            # (a request needs aligned rows; tuned entries assume them)
            if (tile is not None or split_k is not None) and not _rows_aligned16(a, b, out, bias):
                tile = split_k = None
    if tile is not None:
        allowed = _lib.GEMM_TILES_F32 if a.dtype == torch.float32 else _lib.GEMM_TILES_16BIT
        if tuple(tile) not in allowed:
            raise ValueError(f"unsupported tile {tile} for {_DTYPE_NAMES[a.dtype]} inputs; choose from {sorted(allowed)}")
        flags |= _lib.GEMM_TILES[tuple(tile)]
    if split_k is not None:
        if a.dtype == torch.float32 and split_k != 0:
            raise ValueError("split_k applies to 16-bit inputs")
        if split_k not in _lib.GEMM_SPLITK:
            raise ValueError(f"unsupported split_k {split_k}; choose from {sorted(_lib.GEMM_SPLITK)}")
        flags |= _lib.GEMM_SPLITK[split_k]
    bias_ptr = bias.data_ptr() if bias is not None else None
    if residual is not None:
        _lib.check(_lib.load().lh_hip_gemm_residual(
            out.data_ptr(), residual.data_ptr(), a.data_ptr(), b.data_ptr(), bias_ptr, M, N, K,
            a.stride(0), b.stride(0), out.stride(0), lh_dtype(a.dtype), lh_dtype(out.dtype), flags, _stream()), "gemm")
        return out
    if workspace is not None:
        _lib.check(_lib.load().lh_hip_gemm_ws(
            out.data_ptr(), a.data_ptr(), b.data_ptr(), bias_ptr, M, N, K, a.stride(0), b.stride(0), out.stride(0),
            lh_dtype(a.dtype), lh_dtype(out.dtype), flags, workspace.data_ptr() if workspace.numel() else None,
            workspace.numel(), _stream()), "gemm")
        return out
    _lib.check(_lib.load().lh_hip_gemm(
        out.data_ptr(), a.data_ptr(), b.data_ptr(), bias_ptr,
        M, N, K, a.stride(0), b.stride(0), out.stride(0), lh_dtype(a.dtype), lh_dtype(out.dtype), flags, _stream()),
        "gemm")
    return out


def gemm_workspace_bytes(M, N, K, dtype, out_dtype=None, *, lda=None, ldb=None, ldc=None, bias=False, relu=False,
                         gelu=False, accumulate_c=False, transpose_a=False, transpose_b=False, tile=None, split_k=None,
                         operands=None) -> int:
    """Bytes of temporary memory `gemm(..., workspace=...)` needs for this problem (0 for most).
    `tile` and `split_k` are the requests of the `gemm` call the workspace is for (a requested cut
    along K needs its f32 blocks whatever the library would have chosen itself).  The plain query
    assumes 16-byte aligned operands; `operands=(out, a, b, bias_or_None)` asks for those tensors,
    whose alignment then counts (an unaligned operand runs on a padded copy in the workspace)."""
    flags = ((_lib.GEMM_HAS_BIAS if bias else 0) | (_lib.GEMM_HAS_RELU if relu else 0)
             | (_lib.GEMM_HAS_GELU if gelu else 0) | (_lib.GEMM_ACCUMULATE_C if accumulate_c else 0)
             | (_lib.GEMM_TRANSPOSE_A if transpose_a else 0) | (_lib.GEMM_TRANSPOSE_B if transpose_b else 0))
    if tile is not None:
        if tuple(tile) not in _lib.GEMM_TILES:
            raise ValueError(f"unsupported tile {tile}")
        flags |= _lib.GEMM_TILES[tuple(tile)]
    if split_k is not None:
        if split_k not in _lib.GEMM_SPLITK:
            raise ValueError(f"unsupported split_k {split_k}; choose from {sorted(_lib.GEMM_SPLITK)}")
        flags |= _lib.GEMM_SPLITK[split_k]
    lda = lda or (M if transpose_a else K)
    ldb = ldb or (K if transpose_b else N)
    if operands is not None:
        out, a, b, bias_t = operands
        if (bias_t is not None) != bool(bias):
            raise ValueError("operands and the bias flag disagree")
        return int(_lib.load().lh_hip_gemm_workspace_bytes_for(
            out.data_ptr(), a.data_ptr(), b.data_ptr(), bias_t.data_ptr() if bias_t is not None else None, M, N, K,
            a.stride(0), b.stride(0), out.stride(0), lh_dtype(dtype), lh_dtype(out_dtype or dtype), flags))
    return int(_lib.load().lh_hip_gemm_workspace_bytes(M, N, K, lda, ldb, ldc or N, lh_dtype(dtype),
                                                       lh_dtype(out_dtype or dtype), flags))


def gemm_fp8(a_q, b_q, scale_a: float, scale_b: float, *, out=None, out_dtype=torch.bfloat16, workspace=None):
    """out = out_dtype((Aq @ Bq)_f32 * scale_a * scale_b); see lh_hip_gemm_fp8 (lh_hip_gemm_fp8_ws
    with a `workspace`)."""
    _require(a_q.dim() == 2 and b_q.dim() == 2, "gemm_fp8 expects 2-D tensors")
    _require(a_q.dtype == torch.float8_e4m3fn and b_q.dtype == torch.float8_e4m3fn,
             "gemm_fp8 expects float8_e4m3fn operands")
    M, K = a_q.shape
    N = b_q.shape[1]
    _require(b_q.shape[0] == K, f"B has {b_q.shape[0]} rows, A has {K} columns")
    _require(a_q.stride(1) == 1 and b_q.stride(1) == 1, "innermost stride must be 1")
    _require(a_q.stride(0) >= K and b_q.stride(0) >= N, "rows of A or B overlap")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a_q.device)
    _is_matrix(out, M, N, "out")
    _require(out.dtype in (torch.bfloat16, torch.float32), "out must be bfloat16 or float32")
    _need_cuda(a_q, b_q, out, workspace)
    if workspace is not None:
        _require(workspace.dtype == torch.uint8 and workspace.dim() == 1 and workspace.is_contiguous(),
                 "workspace must be a contiguous uint8 vector")
        _lib.check(_lib.load().lh_hip_gemm_fp8_ws(
            out.data_ptr(), a_q.data_ptr(), b_q.data_ptr(), float(scale_a), float(scale_b), M, N, K,
            a_q.stride(0), b_q.stride(0), out.stride(0), lh_dtype(out.dtype),
            workspace.data_ptr() if workspace.numel() else None, workspace.numel(), _stream()), "gemm_fp8")
        return out
    _lib.check(_lib.load().lh_hip_gemm_fp8(
        out.data_ptr(), a_q.data_ptr(), b_q.data_ptr(), float(scale_a), float(scale_b), M, N, K,
        a_q.stride(0), b_q.stride(0), out.stride(0), lh_dtype(out.dtype), _stream()), "gemm_fp8")
    return out


def gemm_fp8_workspace_bytes(M, N, K, out_dtype=torch.bfloat16, *, lda=None, ldb=None, ldc=None) -> int:
    """Bytes of temporary memory `gemm_fp8(..., workspace=...)` needs; the row strides default to
    those of contiguous operands."""
    return int(_lib.load().lh_hip_gemm_fp8_workspace_bytes(M, N, K, lda or K, ldb or N, ldc or N, lh_dtype(out_dtype)))


def _strides3(t) -> _lib.Strides3:
    return _lib.Strides3(t.stride(0), t.stride(1), t.stride(2))


def attention(q, k, v, *, causal=False, scale=None, out=None, rows_per_wave=None, stages=None, kv_split=None,
              workspace=None, scale_in_f32=False):
    """Fused attention forward on [Z,H,T,d] tensors (any strides with unit stride along d).
    `rows_per_wave` (32 or 64), `stages` (3 or 4, K/V ring of the 32-row kernel) and `kv_split`
    (2: two wave groups per workgroup on halves of the key range, 1: never) request a
    kernel variant for 16-bit tensors with head dimension 64; with none given the
    tuned-parameter database is asked, then the library chooses by shape.
    `workspace` (uint8, see attention_workspace_bytes) makes the call take its temporary memory
    from there instead of the library's pool (lh_hip_attention_ws).
    `scale_in_f32` (16-bit tensors, head dimension 64): Q stays as stored and every score is scaled
    in f32, the reference's rounding points exactly (LH_ATTN_SCALE_F32; about 7 % slower), instead
    of Q multiplied by the scale once and rounded to the element type again."""
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("attention expects Q, K, V of equal 4-D shape [Z,H,T,d]")
    _require(q.dtype in _FLOATS and k.dtype == q.dtype and v.dtype == q.dtype,
             "attention expects Q, K, V of one dtype (float32, bfloat16 or float16)")
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    _require(tuple(out.shape) == tuple(q.shape) and out.dtype == q.dtype, "out must have the shape and dtype of Q")
    for t in (q, k, v, out):
        if t.stride(3) != 1:
            raise ValueError("innermost stride must be 1")
    _need_cuda(q, k, v, out)
    Z, H, T, d = q.shape
    if rows_per_wave is None and stages is None and kv_split is None and d == 64 and q.dtype != torch.float32:
        db = _tuned_db()
        if db is not None:
            rows_per_wave, stages, kv_split = db.lookup_attention("bf16" if q.dtype == torch.bfloat16 else "f16", Z * H, T, d, causal)
            if (rows_per_wave or stages or kv_split) and not _rows_aligned16(q, k, v, out):
                rows_per_wave = stages = kv_split = None
    _require((rows_per_wave or 0) in _lib.ATTN_ROWS and (stages or 0) in _lib.ATTN_STAGES
             and (kv_split or 0) in _lib.ATTN_KSPLIT,
             f"rows_per_wave must be one of {sorted(_lib.ATTN_ROWS)[1:]}, stages one of {sorted(_lib.ATTN_STAGES)[1:]}, "
             f"kv_split one of {sorted(_lib.ATTN_KSPLIT)[1:]}")
    word = ((_lib.ATTN_CAUSAL if causal else 0) | _lib.ATTN_ROWS[rows_per_wave or 0] | _lib.ATTN_STAGES[stages or 0]
            | _lib.ATTN_KSPLIT[kv_split or 0] | (_lib.ATTN_SCALE_F32 if scale_in_f32 else 0))
    if workspace is not None:
        _require(workspace.dtype == torch.uint8 and workspace.dim() == 1 and workspace.is_contiguous(),
                 "workspace must be a contiguous uint8 vector")
        _need_cuda(workspace)
        _lib.check(_lib.load().lh_hip_attention_ws(
            out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), Z, H, T, d,
            _strides3(out), _strides3(q), _strides3(k), _strides3(v),
            float(scale) if scale is not None else 1.0 / math.sqrt(d), word, lh_dtype(q.dtype),
            workspace.data_ptr() if workspace.numel() else None, workspace.numel(), _stream()), "attention")
        return out
    _lib.check(_lib.load().lh_hip_attention(
        out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), Z, H, T, d,
        _strides3(out), _strides3(q), _strides3(k), _strides3(v),
        float(scale) if scale is not None else 1.0 / math.sqrt(d), word, lh_dtype(q.dtype), _stream()),
        "attention")
    return out


def attention_workspace_bytes(Z, H, T, d, dtype, *, causal=False, rows_per_wave=None, stages=None, kv_split=None,
                              scale_in_f32=False) -> int:
    """Bytes of temporary memory `attention(..., workspace=...)` needs for contiguous [Z,H,T,d]
    tensors: the partial results of a key range split between workgroups, which the library
    chooses for 16-bit problems with few query blocks and long sequences; 0 for everything else
    and for every call that requests a kernel variant."""
    word = ((_lib.ATTN_CAUSAL if causal else 0) | _lib.ATTN_ROWS[rows_per_wave or 0] | _lib.ATTN_STAGES[stages or 0]
            | _lib.ATTN_KSPLIT[kv_split or 0] | (_lib.ATTN_SCALE_F32 if scale_in_f32 else 0))
    st = _lib.Strides3(H * T * d, T * d, d)
    return int(_lib.load().lh_hip_attention_workspace_bytes(Z, H, T, d, st, st, st, st, word, lh_dtype(dtype)))


def layer_norm(x, gamma, beta, eps=1e-5, *, out=None, out_dtype=None):
    _require(x.dim() == 2, "layer_norm expects a 2-D input")
    M, N = x.shape
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    if gamma.dtype != torch.float32 or beta.dtype != torch.float32:
        raise ValueError("gamma and beta must be float32")
    _is_vector(gamma, N, torch.float32, "gamma")
    _is_vector(beta, N, torch.float32, "beta")
    _require(tuple(out.shape) == (M, N), f"out must have shape [{M}, {N}]")
    if not x.is_contiguous() or not out.is_contiguous():
        raise ValueError("layer_norm expects contiguous tensors")
    _need_cuda(x, gamma, beta, out)
    _lib.check(_lib.load().lh_hip_layer_norm(
        out.data_ptr(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), M, N, float(eps),
        lh_dtype(x.dtype), lh_dtype(out.dtype), _stream()), "layer_norm")
    return out


def softmax(x, *, out=None):
    _require(x.dim() == 2, "softmax expects a 2-D input")
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device) if out is None else out
    _same_dense(out, x, "softmax")
    _need_cuda(x, out)
    M, N = x.shape
    _lib.check(_lib.load().lh_hip_softmax(out.data_ptr(), x.data_ptr(), M, N, lh_dtype(x.dtype), _stream()), "softmax")
    return out


def gelu_tanh(x, *, out=None):
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device) if out is None else out
    _same_dense(out, x, "gelu_tanh")
    _need_cuda(x, out)
    _lib.check(_lib.load().lh_hip_gelu_tanh(out.data_ptr(), x.data_ptr(), x.numel(), lh_dtype(x.dtype), _stream()),
               "gelu_tanh")
    return out


def bias_act(x, bias, relu=False, *, out=None):
    _require(x.dim() == 2, "bias_act expects a 2-D input")
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device) if out is None else out
    _same_dense(out, x, "bias_act")
    M, N = x.shape
    _is_vector(bias, N, x.dtype, "bias")
    _need_cuda(x, bias, out)
    _lib.check(_lib.load().lh_hip_bias_act(out.data_ptr(), x.data_ptr(), bias.data_ptr(), M, N, 1 if relu else 0,
                                           lh_dtype(x.dtype), _stream()), "bias_act")
    return out


def add(a, b, *, out=None):
    out = torch.empty(a.shape, dtype=a.dtype, device=a.device) if out is None else out
    _same_dense(out, a, "add")
    _same_dense(b, a, "add (second operand)")
    _need_cuda(a, b, out)
    _lib.check(_lib.load().lh_hip_add(out.data_ptr(), a.data_ptr(), b.data_ptr(), a.numel(), lh_dtype(a.dtype),
                                      _stream()), "add")
    return out


def cast(x, dtype, *, out=None):
    out = torch.empty(x.shape, dtype=dtype, device=x.device) if out is None else out
    _require(tuple(out.shape) == tuple(x.shape) and out.dtype == dtype, "cast: out must have the input's shape and the target dtype")
    _require(x.is_contiguous() and out.is_contiguous(), "cast expects contiguous tensors")
    _need_cuda(x, out)
    _lib.check(_lib.load().lh_hip_cast(out.data_ptr(), x.data_ptr(), x.numel(), lh_dtype(x.dtype), lh_dtype(dtype),
                                       _stream()), "cast")
    return out


BLOCK_PARAM_NAMES = ("ln1_g", "ln1_b", "w_qkv", "b_qkv", "w_o", "b_o", "ln2_g", "ln2_b", "w_fc", "b_fc", "w_proj",
                     "b_proj", "w_q", "w_k", "w_v")


def _block_opts(dtype, causal, activation, bias_dtype, hidden):
    acts = {"gelu_tanh": _lib.ACT_GELU_TANH, "relu": _lib.ACT_RELU}
    _require(activation in acts, f"activation must be one of {sorted(acts)}")
    return _lib.NanoGPTBlockOpts(1 if causal else 0, acts[activation], lh_dtype(bias_dtype or dtype), int(hidden))


def _block_params(params: dict, C: int, n_head: int):
    """Validate one block's parameter tensors and pack their pointers.  Returns (struct, dtype,
    bias dtype or None, hidden)."""
    _require(C % n_head == 0, f"C={C} is not a multiple of n_head={n_head}")
    fused = params.get("w_qkv") is not None
    if not fused:
        _require(all(params.get(k) is not None for k in ("w_q", "w_k", "w_v")),
                 "the block needs w_qkv or all of w_q, w_k, w_v")
    dtype = (params["w_qkv"] if fused else params["w_q"]).dtype
    _require(dtype in _FLOATS, f"unsupported weight dtype {dtype}")
    hidden = params["w_fc"].shape[1] if params["w_fc"].dim() == 2 else -1
    want = {"w_qkv": (C, 3 * C), "w_q": (C, C), "w_k": (C, C), "w_v": (C, C), "w_o": (C, C), "w_fc": (C, hidden),
            "w_proj": (hidden, C)}
    for name, shape in want.items():
        t = params.get(name)
        if t is None:
            _require(name in ("w_qkv", "w_q", "w_k", "w_v"), f"missing block parameter {name}")
            continue
        _require(tuple(t.shape) == shape and t.dtype == dtype and t.is_contiguous(),
                 f"{name} must be a contiguous {dtype} tensor of shape {shape}, got {tuple(t.shape)} {t.dtype}")
    for name in ("ln1_g", "ln1_b", "ln2_g", "ln2_b"):
        _is_vector(params[name], C, torch.float32, name)
    bias_dtype = None
    for name, n in (("b_qkv", 3 * C), ("b_o", C), ("b_fc", hidden), ("b_proj", C)):
        t = params.get(name)
        if t is None:
            continue
        bias_dtype = bias_dtype or t.dtype
        _require(t.dtype in (dtype, torch.float32), f"{name} must be float32 or have the weight dtype")
        _is_vector(t, n, bias_dtype, name)
    ptr = lambda n: params[n].data_ptr() if params.get(n) is not None else None  # noqa: E731
    return _lib.NanoGPTBlockParams(*[ptr(n) for n in BLOCK_PARAM_NAMES]), dtype, bias_dtype, hidden


def nanogpt_block_workspace_bytes(B, T, C, dtype, *, causal=True, activation="gelu_tanh", bias_dtype=None,
                                  hidden=0) -> int:
    o = _block_opts(dtype, causal, activation, bias_dtype, hidden)
    return int(_lib.load().lh_hip_nanogpt_block_workspace_bytes(B, T, C, lh_dtype(dtype), ctypes.byref(o)))


def _workspace(workspace, need, device):
    if workspace is None:
        return torch.empty(need, dtype=torch.uint8, device=device)
    _require(workspace.dtype == torch.uint8 and workspace.dim() == 1 and workspace.is_contiguous()
             and workspace.numel() >= need, f"workspace must be a contiguous uint8 vector of at least {need} bytes")
    return workspace


def nanogpt_block(x, params: dict, n_head: int, *, eps=1e-5, out=None, workspace=None, causal=True,
                  activation="gelu_tanh"):
    """One GPT-2 block forward. x: [B,T,C] float32; params: tensors named BLOCK_PARAM_NAMES with
    weights stored [in,out] in float32, bfloat16 or float16 (LayerNorm parameters float32; biases
    float32 or the weight type, or absent).  Either `w_qkv` [C,3C] or `w_q`, `w_k`, `w_v` [C,C] each.
    The defaults are the benchmark's block; `causal=False, activation="relu"` with separate
    projections and float32 biases is the reference's (examples/xegpu/nanoGPT_payload.py:299-317)."""
    _require(x.dim() == 3 and x.dtype == torch.float32 and x.is_contiguous(), "x must be a contiguous float32 [B,T,C] tensor")
    B, T, C = x.shape
    p, dtype, bias_dtype, hidden = _block_params(params, C, n_head)
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _same_dense(out, x, "nanogpt_block")
    o = _block_opts(dtype, causal, activation, bias_dtype, hidden)
    _need_cuda(x, out, workspace, *[t for t in params.values() if t is not None])
    need = int(_lib.load().lh_hip_nanogpt_block_workspace_bytes(B, T, C, lh_dtype(dtype), ctypes.byref(o)))
    workspace = _workspace(workspace, need, x.device)
    _lib.check(_lib.load().lh_hip_nanogpt_block(
        out.data_ptr(), x.data_ptr(), ctypes.byref(p), B, T, C, n_head, float(eps), lh_dtype(dtype), ctypes.byref(o),
        workspace.data_ptr(), workspace.numel(), _stream()), "nanogpt_block")
    return out


def nanogpt_forward(x, layers: list, lnf_g, lnf_b, lm_w, lm_b, n_head: int, *, eps=1e-5, out=None, workspace=None,
                    causal=True, activation="gelu_tanh"):
    """n blocks + final LayerNorm + lm_head. x: [B,T,C] float32; `layers`: one parameter dict per
    block (see nanogpt_block); lm_w [C, vocab] in the blocks' dtype and lm_b [vocab] (or None) in
    their bias dtype. Returns float32 logits [B,T,vocab]."""
    _require(x.dim() == 3 and x.dtype == torch.float32 and x.is_contiguous(), "x must be a contiguous float32 [B,T,C] tensor")
    B, T, C = x.shape
    _require(lm_w.dim() == 2 and lm_w.shape[0] == C and lm_w.is_contiguous(), f"lm_w must be a contiguous [{C}, vocab] matrix")
    vocab = lm_w.shape[1]
    dtype = lm_w.dtype
    packed = [_block_params(p, C, n_head) for p in layers]
    for _, dt, _, _ in packed:
        _require(dt == dtype, "every block must have lm_w's dtype")
    bias_dtype = next((b for _, _, b, _ in packed if b is not None), lm_b.dtype if lm_b is not None else None)
    hidden = packed[0][3] if packed else 0
    _require(all(h == hidden for _, _, _, h in packed), "every block must have the same MLP width")
    _require(all(b in (None, bias_dtype) for _, _, b, _ in packed), "every block must have the same bias dtype")
    _is_vector(lnf_g, C, torch.float32, "lnf_g")
    _is_vector(lnf_b, C, torch.float32, "lnf_b")
    if lm_b is not None:
        _is_vector(lm_b, vocab, bias_dtype, "lm_b")
    if out is None:
        out = torch.empty((B, T, vocab), dtype=torch.float32, device=x.device)
    _require(tuple(out.shape) == (B, T, vocab) and out.dtype == torch.float32 and out.is_contiguous(),
             f"out must be a contiguous float32 [{B}, {T}, {vocab}] tensor")
    o = _block_opts(dtype, causal, activation, bias_dtype, hidden)
    _need_cuda(x, out, workspace, lnf_g, lnf_b, lm_w, lm_b, *[t for p in layers for t in p.values() if t is not None])
    need = int(_lib.load().lh_hip_nanogpt_forward_workspace_bytes(B, T, C, vocab, lh_dtype(dtype), ctypes.byref(o)))
    workspace = _workspace(workspace, need, x.device)
    blocks = (_lib.NanoGPTBlockParams * max(len(layers), 1))(*[p for p, _, _, _ in packed])
    _lib.check(_lib.load().lh_hip_nanogpt_forward(
        out.data_ptr(), x.data_ptr(), blocks, len(layers), lnf_g.data_ptr(), lnf_b.data_ptr(), lm_w.data_ptr(),
        lm_b.data_ptr() if lm_b is not None else None, B, T, C, n_head, vocab, float(eps), lh_dtype(dtype),
        ctypes.byref(o), workspace.data_ptr(), workspace.numel(), _stream()), "nanogpt_forward")
    return out


def release_scratch() -> None:
    """Free the library's pool of temporary buffers on the current device (waits for the device)."""
    _lib.check(_lib.load().lh_hip_release_scratch(), "release_scratch")
