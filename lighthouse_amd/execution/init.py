"""Kernel argument initialisation from ``DIMSxTYPExINIT`` strings.

Same grammar, errors and random protocol as lighthouse/execution/init.py:12-118
(``rnd`` is ``np.random.rand(*shape)`` converted to the element type, arguments are
generated in order), extended to the narrow float types of the HIP target.
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


class KernelArgument:
    dims: list[int]
    element_type: np.dtype
    init_type: InitType
    arg: np.ndarray

    def __init__(self, dims: list[int], element_type, init_type: InitType = InitType.ZERO):
        if dims is None or len(dims) == 0 or not all(isinstance(dim, int) and dim > 0 for dim in dims):
            raise ValueError("Dimensions must be a non-empty list of non-zero integers.")
        self.dims = dims
        self.element_type = element_type
        self.init_type = init_type
        self.arg = self.initialize(dims, init_type, element_type)

    def initialize(self, shape: list[int], init_type: InitType, element_type) -> np.ndarray:
        if init_type == InitType.ZERO:
            return astype(np.zeros(shape, dtype=np.float32), element_type)
        elif init_type == InitType.ONE:
            return astype(np.ones(shape, dtype=np.float32), element_type)
        elif init_type == InitType.RANDOM:
            return astype(np.random.rand(*shape), element_type)
        elif init_type == InitType.IDENTITY:
            if len(shape) != 2 or shape[0] != shape[1]:
                raise ValueError("Identity initializer only works for square matrices.")
            return astype(np.eye(shape[0], dtype=np.float32), element_type)
        else:
            raise ValueError(f"Unsupported initializer type: {init_type}")


class KernelArgumentParser:
    @staticmethod
    def parse(shape_str: str) -> KernelArgument:
        parts = shape_str.split("x")
        try:
            element_type = mlir_to_numpy_dtype(parts[-2])
        except (ValueError, IndexError):
            raise ValueError(f"Invalid element type in shape string: {shape_str}")
        try:
            dims = [int(dim) for dim in parts[:-2]]
        except ValueError:
            raise ValueError(f"Invalid dims in shape string: {shape_str}")
        try:
            init_type = InitType(parts[-1])
        except ValueError:
            raise ValueError(f"Invalid init type in shape string: {shape_str}")
        return KernelArgument(dims, element_type, init_type)

    @staticmethod
    def parse_all(shape_str: str) -> list[KernelArgument]:
        return [KernelArgumentParser.parse(s) for s in shape_str.split(",")]
