"""Memory managers of the HIP target.

Class hierarchy and method contracts of lighthouse/execution/memory_manager.py:19-188.
``GPUMemoryManager`` there allocates/copies by invoking JIT'd ``gpu_alloc_*`` helpers;
here the same operations are C ABI calls (lh_hip_alloc / lh_hip_memcpy_* / lh_hip_free).
``TorchMemoryManager`` is the pass-through manager of lighthouse/ingress/torch/compile.py:19-30.
"""

from __future__ import annotations

import abc
import ctypes
from contextlib import contextmanager
from dataclasses import dataclass, field

import numpy as np

from .. import _lib
from ..utils import memref as memref_utils
from ..utils.numpy import elem_name, itemsize


@dataclass
class MemoryManager(abc.ABC):
    """Abstract base class for memory management."""

    execution_engine: object = None

    @abc.abstractmethod
    def alloc(self, name: str | None = None, **kwargs) -> ctypes.Structure: ...

    @abc.abstractmethod
    def get(self, name: str) -> ctypes.Structure: ...

    @abc.abstractmethod
    def deallocate_all(self): ...

    @staticmethod
    def emit_memory_management_funcs(payload_module, **kwargs):
        """Nothing to emit: allocation and copies are library calls, not payload functions."""


@dataclass
class ExternalMemoryManager(MemoryManager, abc.ABC):
    """Pass-through: converts caller-owned buffers to memref descriptors."""

    @abc.abstractmethod
    def get_memrefs(self, inputs): ...

    def alloc(self, name: str | None = None, **kwargs) -> ctypes.Structure:
        raise NotImplementedError("Allocation not supported.")

    def get(self, name: str) -> ctypes.Structure:
        raise NotImplementedError("Lookup not supported.")

    def deallocate_all(self):
        raise NotImplementedError("Deallocation not supported.")


@dataclass
class DeviceMemoryManager(MemoryManager, abc.ABC):
    @abc.abstractmethod
    def copy(self, src, dst): ...

    @abc.abstractmethod
    def clone_host_buffers(self, host_inputs, names=None): ...


@dataclass
class GPUMemoryManager(DeviceMemoryManager):
    """Device buffers owned by the manager (hipMalloc through the C ABI)."""

    allocated_buffers: dict[str, tuple[ctypes.Structure, str]] = field(default_factory=dict)
    buf_counter: int = 0

    def alloc(self, shape: tuple[int, ...], elem_type, name: str | None = None) -> ctypes.Structure:
        if name is None:
            name = f"buffer_{self.buf_counter}"
            self.buf_counter += 1
        assert name not in self.allocated_buffers, f"Buffer with name '{name}' already exists."
        elem = elem_name(elem_type)
        nbytes = int(np.prod(shape, dtype=np.int64)) * itemsize(elem)
        ptr = ctypes.c_void_p()
        _lib.check(_lib.load().lh_hip_alloc(ctypes.byref(ptr), nbytes), "alloc")
        mref = memref_utils.make_memref(ptr.value, shape)
        # The descriptor carries no element type; track it next to the buffer.
        self.allocated_buffers[name] = mref, elem
        return mref

    def get(self, name: str) -> ctypes.Structure:
        assert name in self.allocated_buffers, f"No buffer found with name '{name}'."
        return self.allocated_buffers[name][0]

    def elem_type_of(self, mref: ctypes.Structure) -> str:
        for m, elem in self.allocated_buffers.values():
            if m is mref:
                return elem
        raise ValueError("memref was not allocated by this manager")

    def deallocate_all(self):
        lib = _lib.load()
        errors = []
        for mref, _ in self.allocated_buffers.values():
            rc = lib.lh_hip_free(mref.allocated)
            if rc:
                errors.append(lib.lh_hip_last_error().decode())
        self.allocated_buffers.clear()
        self.buf_counter = 0
        if errors:
            raise RuntimeError("; ".join(errors))

    def copy(self, src, dst):
        """Copy between a host numpy array and a device buffer, or between two device buffers."""
        lib = _lib.load()
        if isinstance(src, np.ndarray) and isinstance(dst, np.ndarray):
            raise ValueError("At least one of src or dst must be a device buffer.")
        if isinstance(src, np.ndarray):
            if not src.flags["C_CONTIGUOUS"]:
                src = np.ascontiguousarray(src)
            if memref_utils.memref_num_elements(dst) != src.size:
                raise ValueError("copy: element count mismatch")
            _lib.check(lib.lh_hip_memcpy_h2d(dst.aligned, src.ctypes.data, src.nbytes), "copy h2d")
        elif isinstance(dst, np.ndarray):
            if not dst.flags["C_CONTIGUOUS"]:
                raise ValueError("copy: destination host array must be contiguous")
            if memref_utils.memref_num_elements(src) != dst.size:
                raise ValueError("copy: element count mismatch")
            _lib.check(lib.lh_hip_memcpy_d2h(dst.ctypes.data, src.aligned, dst.nbytes), "copy d2h")
        else:
            nbytes = memref_utils.memref_num_elements(src) * itemsize(self.elem_type_of(src))
            _lib.check(lib.lh_hip_memcpy_d2d(dst.aligned, src.aligned, nbytes), "copy d2d")

    @contextmanager
    def clone_host_buffers(self, host_inputs: list[np.ndarray], names: list[str] | None = None):
        buffers = []
        try:
            for i, host_arr in enumerate(host_inputs):
                name = names[i] if names is not None else None
                buf = self.alloc(host_arr.shape, host_arr.dtype, name=name)
                self.copy(host_arr, buf)
                buffers.append(buf)
            yield buffers
        finally:
            self.deallocate_all()


@dataclass
class TorchMemoryManager(ExternalMemoryManager):
    """Torch tensors already on the device, passed through as memref descriptors."""

    @contextmanager
    def get_memrefs(self, inputs):
        for t in inputs:
            if not t.is_cuda:
                raise ValueError("TorchMemoryManager expects tensors on the GPU")
        yield [memref_utils.torch_to_memref(t) for t in inputs]
