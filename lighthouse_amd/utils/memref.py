"""Ranked memref descriptors and packed arguments.

Same layout and helpers as the reference: ``to_ctype`` / ``get_packed_arg`` /
``to_packed_args`` follow lighthouse/utils/memref.py:5-44; the descriptor structure
{allocated, aligned, offset, shape[rank], strides[rank]} with strides in ELEMENTS is the
one ``mlir.runtime.np_to_memref`` builds and lighthouse/utils/torch.py:41-66 fills for
torch tensors.  The element type is not part of the descriptor; pointers are stored as
``void*``.
"""

from __future__ import annotations

import ctypes
from collections.abc import Sequence
from functools import lru_cache

import numpy as np


@lru_cache(maxsize=None)
def make_nd_memref_descriptor(rank: int):
    """ctypes structure type of a rank-``rank`` memref descriptor."""
    if rank == 0:

        class MemRefDescriptor0(ctypes.Structure):
            _fields_ = [("allocated", ctypes.c_void_p), ("aligned", ctypes.c_void_p), ("offset", ctypes.c_longlong)]

        return MemRefDescriptor0

    class MemRefDescriptor(ctypes.Structure):
        _fields_ = [
            ("allocated", ctypes.c_void_p),
            ("aligned", ctypes.c_void_p),
            ("offset", ctypes.c_longlong),
            ("shape", ctypes.c_longlong * rank),
            ("strides", ctypes.c_longlong * rank),
        ]

    MemRefDescriptor.__name__ = f"MemRefDescriptor{rank}"
    return MemRefDescriptor


def make_memref(ptr: int, shape: Sequence[int], strides: Sequence[int] | None = None, offset: int = 0):
    """Descriptor for the buffer at address ``ptr``; default strides are row-major contiguous."""
    rank = len(shape)
    desc = make_nd_memref_descriptor(rank)()
    desc.allocated = ptr
    desc.aligned = ptr
    desc.offset = offset
    if rank:
        if strides is None:
            strides, acc = [], 1
            for d in reversed(shape):
                strides.insert(0, acc)
                acc *= int(d)
        desc.shape = (ctypes.c_longlong * rank)(*[int(d) for d in shape])
        desc.strides = (ctypes.c_longlong * rank)(*[int(s) for s in strides])
    return desc


def get_ranked_memref_descriptor(arr: np.ndarray):
    """Descriptor of a numpy array (host memory); numpy byte strides become element strides."""
    if not isinstance(arr, np.ndarray):
        raise ValueError("expected a numpy array")
    item = arr.dtype.itemsize
    return make_memref(arr.ctypes.data, arr.shape, [s // item for s in arr.strides])


def torch_to_memref(t):
    """Descriptor of a torch tensor (lighthouse/utils/torch.py:41-66): data_ptr + element strides."""
    return make_memref(t.data_ptr(), tuple(t.shape), tuple(t.stride()))


def to_ctype(memref_desc):
    """Pointer to pointer to the descriptor: one packed argument (lighthouse/utils/memref.py:5-12)."""
    return ctypes.pointer(ctypes.pointer(memref_desc))


def get_packed_arg(ctypes_args):
    packed_args = (ctypes.c_void_p * len(ctypes_args))()
    for i, a in enumerate(ctypes_args):
        packed_args[i] = ctypes.cast(a, ctypes.c_void_p)
    return packed_args


def to_packed_args(args):
    """Descriptors and/or integers -> packed argument array (lighthouse/utils/memref.py:31-44).

    The returned array keeps the intermediate ctypes objects alive in ``_keepalive``.
    """
    ctype_args = []
    for arg in args:
        if isinstance(arg, int):
            ctype_args.append(ctypes.pointer(ctypes.c_int64(arg)))
        else:
            ctype_args.append(to_ctype(arg))
    packed = get_packed_arg(ctype_args)
    packed._keepalive = (ctype_args, list(args))
    return packed


def memref_shape(desc) -> tuple[int, ...]:
    return tuple(desc.shape) if hasattr(desc, "shape") else ()


def memref_num_elements(desc) -> int:
    n = 1
    for d in memref_shape(desc):
        n *= int(d)
    return n
