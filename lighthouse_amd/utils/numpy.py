"""Element-type tables and narrow-float host arrays.

Mirrors lighthouse/utils/numpy.py:15-84 (``numpy_to_mlir_type`` / ``mlir_to_numpy_dtype``)
with type NAMES ("f32", "bf16", ...) in place of MLIR type objects, because this runtime
selects hand-written kernels and never builds MLIR.  numpy has no bfloat16 or float8, and
the ml_dtypes package the reference uses is optional here: such host arrays are numpy
arrays of the raw bit patterns (uint16 / uint8) whose dtype carries the element type in
its ``metadata`` field, created and decoded by the helpers below.
"""

from __future__ import annotations

import numpy as np

from .. import _lib

bfloat16 = np.dtype(np.uint16, metadata={"lh_elem": "bf16"})
float8_e4m3fn = np.dtype(np.uint8, metadata={"lh_elem": "f8E4M3FN"})

_NAME_TO_NUMPY = {
    "f64": np.dtype(np.float64),
    "f32": np.dtype(np.float32),
    "f16": np.dtype(np.float16),
    "bf16": bfloat16,
    "f8E4M3FN": float8_e4m3fn,
    "i64": np.dtype(np.int64),
    "i32": np.dtype(np.int32),
    "i16": np.dtype(np.int16),
    "i8": np.dtype(np.int8),
    "i1": np.dtype(np.bool_),
}

_NAME_TO_LH = {
    "f32": _lib.F32, "bf16": _lib.BF16, "f16": _lib.F16, "f8E4M3FN": _lib.F8E4M3, "f64": _lib.F64,
    "i8": _lib.I8, "i16": _lib.I16, "i32": _lib.I32, "i64": _lib.I64,
}


def elem_name(dtype) -> str:
    """Element type name of a numpy dtype, torch dtype or name."""
    if isinstance(dtype, str):
        if dtype not in _NAME_TO_NUMPY:
            raise ValueError(f"Unsupported MLIR type: {dtype}")
        return dtype
    try:
        import torch

        if isinstance(dtype, torch.dtype):
            table = {
                torch.float32: "f32", torch.float64: "f64", torch.float16: "f16", torch.bfloat16: "bf16",
                torch.float8_e4m3fn: "f8E4M3FN", torch.int8: "i8", torch.int16: "i16", torch.int32: "i32",
                torch.int64: "i64", torch.bool: "i1",
            }
            if dtype not in table:
                raise ValueError(f"Unsupported dtype: {dtype}")
            return table[dtype]
    except ImportError:  # pragma: no cover
        pass
    dt = np.dtype(dtype)
    if dt.metadata and "lh_elem" in dt.metadata:
        return dt.metadata["lh_elem"]
    for name, cand in _NAME_TO_NUMPY.items():
        if cand.metadata is None and cand == dt:
            return name
    raise ValueError(f"Unsupported numpy dtype: {dtype}")


def numpy_to_mlir_type(dtype) -> str:
    """numpy dtype -> element type name (lighthouse/utils/numpy.py:15-47)."""
    return elem_name(dtype)


def mlir_to_numpy_dtype(mlir_type: str) -> np.dtype:
    """Element type name -> numpy dtype (lighthouse/utils/numpy.py:50-84)."""
    if mlir_type not in _NAME_TO_NUMPY:
        raise ValueError(f"Unsupported MLIR type: {mlir_type}")
    return _NAME_TO_NUMPY[mlir_type]


_TORCH_LH_CACHE: dict = {}  # torch.dtype -> lh_dtype value (the per-launch path of the torch front end)


def lh_dtype(dtype) -> int:
    """lh_dtype enum value for a numpy dtype / torch dtype / name."""
    hit = _TORCH_LH_CACHE.get(dtype) if type(dtype).__module__ == "torch" else None
    if hit is not None:
        return hit
    value = _lh_dtype_uncached(dtype)
    # numpy dtypes are not cached: the narrow-float dtypes above compare (and hash) equal to the
    # plain uint16 / uint8 they are built on.
    if type(dtype).__module__ == "torch":
        _TORCH_LH_CACHE[dtype] = value
    return value


def _lh_dtype_uncached(dtype) -> int:
    name = elem_name(dtype)
    if name not in _NAME_TO_LH:
        raise ValueError(f"Unsupported element type for the HIP target: {name}")
    return _NAME_TO_LH[name]


def itemsize(dtype) -> int:
    return _NAME_TO_NUMPY[elem_name(dtype)].itemsize


# ---- narrow float conversions on the host ---------------------------------------


def f32_to_bf16(x) -> np.ndarray:
    """float array -> bfloat16 host array (round to nearest even)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        r = np.where(nan, (((u >> 16) & 0x8000) | 0x7FC0).astype(np.uint16), r)
    return r.reshape(x.shape).view(bfloat16)


def bf16_to_f32(x) -> np.ndarray:
    b = np.ascontiguousarray(x).view(np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32).reshape(b.shape)


def astype(x, dtype) -> np.ndarray:
    """``x.astype(dtype)`` that also understands the tagged narrow-float dtypes."""
    name = elem_name(dtype)
    src = elem_name(x.dtype)
    if name == src:
        return np.asarray(x).view(_NAME_TO_NUMPY[name])
    if src == "bf16":
        x = bf16_to_f32(x)
    elif src == "f8E4M3FN":
        import torch

        x = torch.from_numpy(np.ascontiguousarray(x).view(np.uint8)).view(torch.float8_e4m3fn).float().numpy()
    if name == "bf16":
        return f32_to_bf16(np.asarray(x, dtype=np.float32))
    if name == "f8E4M3FN":
        import torch

        t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).clamp(-448.0, 448.0)
        return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy().view(float8_e4m3fn)
    return np.asarray(x).astype(_NAME_TO_NUMPY[name])


def to_float32(x) -> np.ndarray:
    """Any supported host array as float32 values."""
    return astype(x, "f32")
