"""Torch tensors as memref descriptors and packed arguments, under the names of
lighthouse/utils/torch.py:41-83 (`to_memref`, `to_packed_args`), for callers that hand device
tensors straight to a payload entry point."""

from __future__ import annotations

from . import memref as _memref


def to_memref(input):
    """Descriptor {allocated, aligned, offset, shape, strides} of a tensor; strides in elements,
    any rank including 0."""
    return _memref.torch_to_memref(input)


def to_packed_args(inputs):
    """Tensors (and plain integers) -> the `void*[]` a payload entry point takes."""
    return _memref.to_packed_args([a if isinstance(a, int) else to_memref(a) for a in inputs])
