"""Kernel argument initialisation from ``DIMSxTYPExINIT`` strings.

Grammar, error messages and random protocol are the boundary the reference's command line and its
known-answer run depend on (lighthouse/execution/init.py:12-118: ``rnd`` is ``np.random.rand(*shape)``
drawn in argument order after ``np.random.seed``, then converted to the element type), extended to
the narrow float types of the HIP target.  The initialisers live in one table keyed by ``InitType``.
"""

from __future__ import annotations

from enum import Enum

import numpy as np

from ..utils.numpy import astype, mlir_to_numpy_dtype


class InitType(Enum):
    ZERO = "0"
    ONE = "1"
    RANDOM = "rnd"
    IDENTITY = "id"


def _identity(shape):
    if len(shape) != 2 or shape[0] != shape[1]:
        raise ValueError("Identity initializer only works for square matrices.")
    return np.eye(shape[0], dtype=np.float32)


# f32 (f64 for the uniform draw, as numpy hands it out) contents before the conversion to the element type
_FILL = {
    InitType.ZERO: lambda shape: np.zeros(shape, dtype=np.float32),
    InitType.ONE: lambda shape: np.ones(shape, dtype=np.float32),
    InitType.RANDOM: lambda shape: np.random.rand(*shape),
    InitType.IDENTITY: _identity,
}


class KernelArgument:
    """One host buffer of a payload call: `dims`, `element_type`, `init_type` and the array `arg`."""

    def __init__(self, dims: list[int], element_type, init_type: InitType = InitType.ZERO):
        if not dims or any(not isinstance(d, int) or d <= 0 for d in dims):
            raise ValueError("Dimensions must be a non-empty list of non-zero integers.")
        self.dims, self.element_type, self.init_type = dims, element_type, init_type
        self.arg: np.ndarray = self.initialize(dims, init_type, element_type)

    def initialize(self, shape: list[int], init_type: InitType, element_type) -> np.ndarray:
        fill = _FILL.get(init_type)
        if fill is None:
            raise ValueError(f"Unsupported initializer type: {init_type}")
        return astype(fill(shape), element_type)


class KernelArgumentParser:
    @staticmethod
    def parse(shape_str: str) -> KernelArgument:
        """``16x64xf32xrnd`` -> dims [16, 64], element type f32, uniform [0, 1) contents."""
        fields = shape_str.split("x")
        if len(fields) < 2:
            raise ValueError(f"Invalid element type in shape string: {shape_str}")
        *dim_fields, type_field, init_field = fields
        try:
            element_type = mlir_to_numpy_dtype(type_field)
        except ValueError:
            raise ValueError(f"Invalid element type in shape string: {shape_str}")
        if not all(f.lstrip("+-").isdigit() for f in dim_fields):
            raise ValueError(f"Invalid dims in shape string: {shape_str}")
        if init_field not in InitType._value2member_map_:
            raise ValueError(f"Invalid init type in shape string: {shape_str}")
        return KernelArgument([int(f) for f in dim_fields], element_type, InitType(init_field))

    @staticmethod
    def parse_all(shape_str: str) -> list[KernelArgument]:
        return [KernelArgumentParser.parse(one) for one in shape_str.split(",")]
