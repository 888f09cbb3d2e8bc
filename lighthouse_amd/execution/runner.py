"""Runner of the HIP target: executes and benchmarks payload modules on the GPU.

Method signatures, buffer handling and errors follow ``Runner`` in
lighthouse/execution/runner.py:42-330.  Where the reference JIT-compiles the module with
MLIR's ExecutionEngine and looks up a native symbol, this runner resolves each payload
function to an entry point of liblighthouse_hip.so and calls it with the same packed
memref arguments.
"""

from __future__ import annotations

import ctypes
import os
import typing
from collections.abc import Callable
from contextlib import contextmanager
from functools import partial

import numpy as np

from .. import _lib
from ..ingress.payloads import PayloadFunction, PayloadModule
from ..utils.memref import memref_shape, to_packed_args
from ..utils.numpy import elem_name
from .memory_manager import ExternalMemoryManager, GPUMemoryManager, MemoryManager
from .target import TargetInfo


class RunnerCallable(typing.Protocol):
    """Protocol of the argument access callback (lighthouse/execution/runner.py:29-39)."""

    def __call__(self, inputs: list[ctypes.Structure], execution_engine, memory_manager: MemoryManager | None) -> None: ...


class HipEngine:
    """Stands where the reference has an ExecutionEngine: symbol lookup in the HIP library."""

    def __init__(self, module: PayloadModule, shared_libs: list[str]):
        self.module = module
        self.lib = _lib.load()
        self.extra_libs = [ctypes.CDLL(p) for p in shared_libs]

    def lookup(self, function_name: str) -> Callable[[ctypes.Array], None]:
        fn = self.module.lookup(function_name)
        entry = getattr(self.lib, f"lh_hip_payload_{fn.entry}")

        def call(packed_args: ctypes.Array) -> None:
            _lib.check(entry(packed_args, len(packed_args), ctypes.byref(fn.attrs)), function_name)

        return call

    def lookup_benchmark(self, function_name: str):
        fn = self.module.lookup(function_name)

        def call(packed_args: ctypes.Array, time_array: np.ndarray, nruns: int, nwarmup: int) -> None:
            _lib.check(
                self.lib.lh_hip_payload_benchmark(
                    fn.entry.encode(), packed_args, len(packed_args),
                    ctypes.cast(ctypes.byref(fn.attrs), ctypes.c_void_p),
                    time_array.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), nruns, nwarmup,
                ),
                function_name,
            )

        return call


class Runner:
    """Runner class for executing and benchmarking payload modules on the GPU."""

    payload_benchmark_function_name: str = "__benchmark"

    def __init__(
        self,
        module: PayloadModule,
        mem_manager_cls: type | None = None,
        shared_libs: list[str] | None = None,
        opt_level: int = 3,
        target: TargetInfo | None = None,
    ):
        if not isinstance(module, PayloadModule):
            raise ValueError("module must be a PayloadModule")
        self.payload = module
        self.target = target if target else TargetInfo(arch="gfx950")
        self.mem_manager_cls = mem_manager_cls
        if shared_libs is None:
            shared_libs = []
        self.lib_dir = str(_lib.library_path().parent)
        found = self._find_shared_libs(shared_libs)
        self.shared_libs = list(dict.fromkeys(found))
        self.opt_level = opt_level
        self.engine = self._get_engine()
        # Function the benchmark wrapper times; set by get_bench_wrapper_schedule/benchmark.
        self._bench_target: str | None = None

    def _find_shared_libs(self, shared_libs: list[str]) -> list[str]:
        found_libs = []
        for so_file in shared_libs:
            so_path = so_file if os.path.isabs(so_file) else os.path.join(self.lib_dir, so_file)
            if not os.path.isfile(so_path):
                raise ValueError(f"Could not find shared library {so_path}")
            found_libs.append(so_path)
        return found_libs

    def _get_engine(self) -> HipEngine:
        return HipEngine(self.payload, self.shared_libs)

    @contextmanager
    def _numpy_to_device_manager(self, fn: PayloadFunction, inputs: list[np.ndarray]):
        """Host numpy buffers, mutated in place by the reference's CPU path: stage them on the
        device, run, and write every writable argument back."""
        manager = GPUMemoryManager(self.engine)
        with manager.clone_host_buffers(inputs) as device_inputs:
            yield device_inputs
            for idx in fn.outputs:
                manager.copy(device_inputs[idx], inputs[idx])

    def _check_buffers(self, fn: PayloadFunction, buffers: list) -> None:
        if len(buffers) != len(fn.args):
            raise ValueError(f"function '{fn.name}' takes {len(fn.args)} buffers, got {len(buffers)}")
        for i, (spec, buf) in enumerate(zip(fn.args, buffers)):
            if not hasattr(buf, "shape") or not hasattr(buf, "dtype"):
                raise ValueError(f"argument {i} of '{fn.name}' is not an array or tensor: {type(buf).__name__}")
            shape = tuple(buf.shape)
            if shape != tuple(spec.shape):
                raise ValueError(f"argument {i} of '{fn.name}' has shape {shape}, expected {tuple(spec.shape)}")
            elem = elem_name(buf.dtype)
            if elem != spec.elem and not (spec.elem == "i8" and elem in ("i8",)):
                raise ValueError(f"argument {i} of '{fn.name}' has element type {elem}, expected {spec.elem}")

    def _execute_kernel(
        self,
        host_input_buffers: list,
        payload_function_name: str = "",
        argument_access_callback: Callable | None = None,
        nruns: int = 100,
        nwarmup: int = 10,
        benchmark: bool = True,
    ) -> np.ndarray | None:
        if host_input_buffers is None:
            raise ValueError("host_input_buffers must be provided")
        if not payload_function_name:
            names = list(self.payload.functions)
            if len(names) != 1:
                raise ValueError("payload_function_name is required for modules with several functions")
            payload_function_name = names[0]
        fn = self.payload.lookup(payload_function_name)
        self._check_buffers(fn, host_input_buffers)

        if self.mem_manager_cls is None:
            if any(not isinstance(buf, np.ndarray) for buf in host_input_buffers):
                raise ValueError("host_input_buffers must be numpy arrays when no mem_manager_cls is provided")
            mem_manager = None
            allocator = partial(self._numpy_to_device_manager, fn, host_input_buffers)
        elif self.mem_manager_cls is GPUMemoryManager:
            mem_manager = self.mem_manager_cls(self.engine)
            allocator = partial(mem_manager.clone_host_buffers, host_input_buffers)
        elif isinstance(self.mem_manager_cls, type) and issubclass(self.mem_manager_cls, ExternalMemoryManager):
            mem_manager = self.mem_manager_cls(self.engine)
            allocator = partial(mem_manager.get_memrefs, host_input_buffers)
        else:
            raise ValueError(f"Unsupported mem_manager_cls type: {self.mem_manager_cls}")

        with allocator() as inputs:
            for i, (spec, m) in enumerate(zip(fn.args, inputs)):
                if memref_shape(m) != tuple(spec.shape):
                    raise ValueError(f"argument {i}: descriptor shape {memref_shape(m)} != {tuple(spec.shape)}")
            args = to_packed_args(inputs if fn.arg_order is None else [inputs[i] for i in fn.arg_order])
            if benchmark:
                time_array = np.zeros((nruns,), dtype=np.float64)
                self.engine.lookup_benchmark(payload_function_name)(args, time_array, nruns, nwarmup)
            else:
                time_array = None
                self.engine.lookup(payload_function_name)(args)
            if argument_access_callback is not None:
                argument_access_callback(inputs, execution_engine=self.engine, memory_manager=mem_manager)
        return time_array

    def benchmark(
        self,
        host_input_buffers: list,
        argument_access_callback: RunnerCallable = None,
        nruns: int = 100,
        nwarmup: int = 10,
        payload_function_name: str = "",
    ) -> np.ndarray:
        """``nwarmup`` untimed calls, then ``nruns`` timed calls; returns seconds per call."""
        return self._execute_kernel(
            host_input_buffers=host_input_buffers,
            payload_function_name=payload_function_name or (self._bench_target or ""),
            argument_access_callback=argument_access_callback,
            nruns=nruns,
            nwarmup=nwarmup,
            benchmark=True,
        )

    def execute(
        self,
        payload_function_name: str,
        host_input_buffers: list,
        argument_access_callback: RunnerCallable = None,
    ) -> None:
        self._execute_kernel(
            host_input_buffers=host_input_buffers,
            payload_function_name=payload_function_name,
            argument_access_callback=argument_access_callback,
            benchmark=False,
        )

    def dump_object_file(self, file_name: str) -> str:
        """The "object file" of this target is the prebuilt shared library: copy it."""
        if not file_name:
            raise ValueError("non-empty file_name must be provided")
        import shutil

        shutil.copyfile(_lib.library_path(), file_name)
        return file_name

    @staticmethod
    def get_bench_wrapper_schedule(payload_func: str) -> str:
        """The reference returns a transform schedule that wraps ``payload_func`` in a timing
        loop named ``__benchmark``; the HIP library's benchmark entry point takes the function
        by name, so the "schedule" is just that name."""
        return payload_func

    @staticmethod
    def get_gpu_argument_access_callback(host_buffer: np.ndarray, arg_index: int = 0) -> RunnerCallable:
        """Callback that copies a device-resident argument to the host after execution."""

        def argument_access_callback(inputs, *, memory_manager: GPUMemoryManager, **kwargs):
            memory_manager.copy(inputs[arg_index], host_buffer)

        return argument_access_callback

    @staticmethod
    def make_function_callable(module: PayloadModule, func_name: str) -> None:
        """Every payload function of this target is callable; only checks that it exists."""
        module.lookup(func_name)
