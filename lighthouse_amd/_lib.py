"""ctypes binding of liblighthouse_hip.so (the C ABI declared in include/lighthouse_hip.h).

The library is the only compute path of this package: if it is missing the import of
any compute entry point raises, there is no CPU fallback.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path

LIB_NAME = "liblighthouse_hip.so"
LIB_PATH = Path(__file__).resolve().parent / "lib" / LIB_NAME

# lh_dtype
F32, BF16, F16, F8E4M3, F64, I8, I16, I32, I64 = range(9)

# LH_GEMM_* flags
GEMM_HAS_BIAS = 1
GEMM_HAS_RELU = 2
GEMM_ACCUMULATE_C = 4
GEMM_TRANSPOSE_A = 8
GEMM_TRANSPOSE_B = 16
GEMM_HAS_GELU = 32
GEMM_TILE_AUTO = 0
GEMM_TILES = {(256, 256): 0x100, (256, 128): 0x200, (128, 256): 0x300, (128, 128): 0x400, (128, 64): 0x500, (64, 64): 0x600}
GEMM_TILES_16BIT = ((256, 256), (256, 128), (128, 256), (128, 128))  # what bf16 / f16 inputs take
GEMM_TILES_F32 = ((128, 128), (128, 64), (64, 64))                   # what f32 inputs take
GEMM_TILE_MASK = 0x700
# LH_GEMM_SPLITK_*: 0 = the library decides, 1 = never cut, 2 / 4 / 8 = cut K that many times
GEMM_SPLITK = {0: 0x0000, 1: 0x0800, 2: 0x1000, 4: 0x1800, 8: 0x2000}
GEMM_SPLITK_MASK = 0x3800
# LH_ATTN_*: bit 0 causal; query rows per wave and K/V ring depth requests (0 = the library decides)
ATTN_CAUSAL = 1
ATTN_ROWS = {0: 0, 32: 0x100, 64: 0x200}
ATTN_STAGES = {0: 0, 3: 0x400, 4: 0x800}
ATTN_KSPLIT = {0: 0, 1: 0x1000, 2: 0x2000}
ATTN_SCALE_F32 = 0x4000  # scores scaled in f32 (the reference's rounding points) instead of Q scaled once

# lh_elementwise_kind
EW_SOFTMAX, EW_GELU, EW_BIAS, EW_ADD, EW_CAST = range(5)

LH_ERR_INVALID = -1
LH_ERR_UNSUPPORTED = -2
LH_ERR_RUNTIME = -3


class Strides3(ctypes.Structure):
    _fields_ = [("z", ctypes.c_int64), ("h", ctypes.c_int64), ("t", ctypes.c_int64)]


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("arch", ctypes.c_char * 64),
        ("name", ctypes.c_char * 128),
        ("compute_units", ctypes.c_int32),
        ("clock_khz", ctypes.c_int32),
        ("memory_clock_khz", ctypes.c_int32),
        ("memory_bus_bits", ctypes.c_int32),
        ("lds_bytes_per_cu", ctypes.c_int32),
        ("wavefront_size", ctypes.c_int32),
        ("hbm_bytes", ctypes.c_int64),
    ]


class NanoGPTBlockParams(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in (
        "ln1_g", "ln1_b", "w_qkv", "b_qkv", "w_o", "b_o", "ln2_g", "ln2_b", "w_fc", "b_fc", "w_proj", "b_proj",
        "w_q", "w_k", "w_v")]


# lh_activation
ACT_GELU_TANH, ACT_RELU = 0, 1


class NanoGPTBlockOpts(ctypes.Structure):
    _fields_ = [("causal", ctypes.c_int32), ("activation", ctypes.c_int32), ("bias_dtype", ctypes.c_int32),
                ("hidden", ctypes.c_int32)]


class MatmulAttrs(ctypes.Structure):
    _fields_ = [("ab_dtype", ctypes.c_int32), ("out_dtype", ctypes.c_int32), ("flags", ctypes.c_uint32)]


class MlpAttrs(ctypes.Structure):
    _fields_ = [("ab_dtype", ctypes.c_int32), ("out_dtype", ctypes.c_int32), ("bias_dtype", ctypes.c_int32),
                ("flags", ctypes.c_uint32), ("nlayers", ctypes.c_int32), ("relu_on_final_layer", ctypes.c_int32)]


class MatmulFp8Attrs(ctypes.Structure):
    _fields_ = [("out_dtype", ctypes.c_int32), ("scale_a", ctypes.c_float), ("scale_b", ctypes.c_float)]


class AttentionAttrs(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("causal", ctypes.c_int32), ("scale", ctypes.c_float)]


class LayerNormAttrs(ctypes.Structure):
    _fields_ = [("x_dtype", ctypes.c_int32), ("out_dtype", ctypes.c_int32), ("eps", ctypes.c_float)]


class ElementwiseAttrs(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("dtype", ctypes.c_int32), ("dst_dtype", ctypes.c_int32),
                ("relu", ctypes.c_int32)]


class NanoGPTBlockAttrs(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("n_head", ctypes.c_int32), ("B", ctypes.c_int32), ("T", ctypes.c_int32),
                ("eps", ctypes.c_float)]


class GptFusedAttrs(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("n_head", ctypes.c_int32), ("n_layer", ctypes.c_int32),
                ("causal", ctypes.c_int32), ("eps", ctypes.c_float)]


_vp, _i64, _i32, _u32, _f32, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_uint32,
                                    ctypes.c_float, ctypes.c_size_t)

# name -> (restype, argtypes); every symbol include/lighthouse_hip.h declares.
PROTOTYPES = {
    "lh_hip_last_error": (ctypes.c_char_p, []),
    "lh_hip_device_info": (_i32, [ctypes.POINTER(DeviceInfo)]),
    "lh_hip_device_count": (_i32, [ctypes.POINTER(_i32)]),
    "lh_hip_alloc": (_i32, [ctypes.POINTER(_vp), _sz]),
    "lh_hip_free": (_i32, [_vp]),
    "lh_hip_memcpy_h2d": (_i32, [_vp, _vp, _sz]),
    "lh_hip_memcpy_d2h": (_i32, [_vp, _vp, _sz]),
    "lh_hip_memcpy_d2d": (_i32, [_vp, _vp, _sz]),
    "lh_hip_memset": (_i32, [_vp, _i32, _sz]),
    "lh_hip_sync": (_i32, [_vp]),
    "lh_hip_release_scratch": (_i32, []),
    "lh_hip_gemm": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _u32, _vp]),
    "lh_hip_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _u32]),
    "lh_hip_gemm_workspace_bytes_for": (_sz, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _u32]),
    "lh_hip_gemm_ws": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _u32, _vp, _sz, _vp]),
    "lh_hip_gemm_static": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _u32, _vp]),
    "lh_hip_gemm_residual": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _u32, _vp]),
    "lh_hip_gemm_fp8": (_i32, [_vp, _vp, _vp, _f32, _f32, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _vp]),
    "lh_hip_gemm_fp8_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _i64, _i32]),
    "lh_hip_gemm_fp8_ws": (_i32, [_vp, _vp, _vp, _f32, _f32, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _vp, _sz, _vp]),
    "lh_hip_attention": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, Strides3, Strides3, Strides3, Strides3,
                                _f32, _i32, _i32, _vp]),
    "lh_hip_attention_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, Strides3, Strides3, Strides3, Strides3, _i32, _i32]),
    "lh_hip_attention_ws": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, Strides3, Strides3, Strides3, Strides3,
                                   _f32, _i32, _i32, _vp, _sz, _vp]),
    "lh_hip_layer_norm": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32, _i32, _vp]),
    "lh_hip_softmax": (_i32, [_vp, _vp, _i64, _i64, _i32, _vp]),
    "lh_hip_gelu_tanh": (_i32, [_vp, _vp, _i64, _i32, _vp]),
    "lh_hip_bias_act": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp]),
    "lh_hip_add": (_i32, [_vp, _vp, _vp, _i64, _i32, _vp]),
    "lh_hip_cast": (_i32, [_vp, _vp, _i64, _i32, _i32, _vp]),
    "lh_hip_nanogpt_block_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32, ctypes.POINTER(NanoGPTBlockOpts)]),
    "lh_hip_nanogpt_block": (_i32, [_vp, _vp, ctypes.POINTER(NanoGPTBlockParams), _i64, _i64, _i64, _i64, _f32, _i32,
                                    ctypes.POINTER(NanoGPTBlockOpts), _vp, _sz, _vp]),
    "lh_hip_nanogpt_forward_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i32, ctypes.POINTER(NanoGPTBlockOpts)]),
    "lh_hip_nanogpt_forward": (_i32, [_vp, _vp, ctypes.POINTER(NanoGPTBlockParams), _i64, _vp, _vp, _vp, _vp, _i64, _i64,
                                      _i64, _i64, _i64, _f32, _i32, ctypes.POINTER(NanoGPTBlockOpts), _vp, _sz, _vp]),
    "lh_hip_payload_matmul": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(MatmulAttrs)]),
    "lh_hip_payload_matmul_fp8": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(MatmulFp8Attrs)]),
    "lh_hip_payload_mlp": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(MlpAttrs)]),
    "lh_hip_payload_attention": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(AttentionAttrs)]),
    "lh_hip_payload_layer_norm": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(LayerNormAttrs)]),
    "lh_hip_payload_elementwise": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(ElementwiseAttrs)]),
    "lh_hip_payload_nanogpt_block": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(NanoGPTBlockAttrs)]),
    "lh_hip_payload_gpt_fused": (_i32, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(GptFusedAttrs)]),
    "lh_hip_payload_benchmark": (_i32, [ctypes.c_char_p, ctypes.POINTER(_vp), _i32, _vp,
                                        ctypes.POINTER(ctypes.c_double), _i64, _i64]),
}

_lib = None


def library_path() -> Path:
    override = os.environ.get("LIGHTHOUSE_HIP_LIBRARY")
    return Path(override) if override else LIB_PATH


def load() -> ctypes.CDLL:
    """Load the shared object once and attach prototypes. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.is_file():
        raise ValueError(
            f"Could not find shared library {path}; build it with `python -m lighthouse_amd.build`"
        )
    lib = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc: int, what: str = "") -> None:
    """Map a C status code to the exception the reference runner raises for that class of error."""
    if rc == 0:
        return
    msg = load().lh_hip_last_error().decode("utf-8", "replace")
    if what:
        msg = f"{what}: {msg}"
    if rc == LH_ERR_RUNTIME:
        raise RuntimeError(msg)
    raise ValueError(msg)
