"""Target description used to select pipelines and kernels.

The interface and the override rules are those of lighthouse/execution/target.py:13-132, which the
descriptor lookup and its ported behaviour tests depend on: `TargetInfo(arch, features, filter)`
with the host as default, a cached `host()`, nested `override(features=, arch=)` scopes that
snapshot their arguments and apply only where the constructor was given nothing, feature queries
and the vector register table.  One addition: a `gfx*` architecture is an AMD GPU
(`TargetInfo.gpu()` asks the HIP library which one), so that descriptor lookup finds
``descriptors/gfx950/...`` the way the reference finds ``descriptors/xegpu/...``.
"""

from __future__ import annotations

import platform
import subprocess
from contextlib import contextmanager
from dataclasses import dataclass
from typing import NamedTuple


@dataclass(frozen=True)
class RegisterInfo:
    width_bits: int
    count: int


class _Scope(NamedTuple):
    """One active `override`: what a constructor without that argument sees (None: nothing)."""

    arch: str | None
    features: tuple[str, ...] | None


# first matching rule wins: (predicate over the feature list, registers)
_CPU_VECTOR_REGISTERS = (
    (lambda f: "avx512f" in f, RegisterInfo(width_bits=512, count=32)),
    (lambda f: "avx2" in f or "avx" in f, RegisterInfo(width_bits=256, count=16)),
    (lambda f: any(x.startswith("sse") for x in f), RegisterInfo(width_bits=128, count=16)),
)
_GPU_VECTOR_REGISTERS = RegisterInfo(width_bits=64 * 32, count=512)  # one VGPR across a 64-lane wavefront

_GPU_FEATURES = {
    "gfx950": ("mfma", "mfma_bf16", "mfma_fp8_ocp", "mfma_f8f6f4", "lds160k"),
    "gfx942": ("mfma", "mfma_bf16"), "gfx940": ("mfma", "mfma_bf16"), "gfx90a": ("mfma", "mfma_bf16"),
}


def _gpu_features(arch: str) -> list[str]:
    """Feature names usable as descriptor sub-directories for an AMD GPU architecture."""
    return list(_GPU_FEATURES.get(arch, ()))


def _host_cpu_flags() -> list[str]:
    listing = subprocess.run(["lscpu"], capture_output=True, text=True).stdout if _have_lscpu() else ""
    for line in listing.splitlines():
        if line.startswith("Flags:"):
            return line.split()[1:]
    raise RuntimeError("Could not get CPU features from lscpu. Make sure lscpu is installed and available in PATH.")


def _have_lscpu() -> bool:
    import shutil

    return shutil.which("lscpu") is not None


class TargetInfo:
    _cached_host: "TargetInfo | None" = None
    _scopes: list[_Scope] = []

    def __init__(self, arch: str | None = None, features: list[str] | None = None, filter: list[str] | None = None):
        scope = type(self)._scopes[-1] if type(self)._scopes else _Scope(None, None)
        if arch is None:
            arch = scope.arch
        if features is None and scope.features is not None:
            features = list(scope.features)
        self.arch = platform.machine() if arch is None else arch
        if features is None:
            features = _gpu_features(self.arch) if self.is_gpu() else self._get_feature_list()
        self.features = features
        if filter is not None:
            self.features = self.has_features(filter)

    # -- construction ---------------------------------------------------------------------
    @classmethod
    def host(cls) -> "TargetInfo":
        """The machine this runs on; cached, except inside an `override`, where every call builds anew."""
        if cls._scopes:
            return cls()
        if cls._cached_host is None:
            cls._cached_host = cls()
        return cls._cached_host

    @classmethod
    def gpu(cls) -> "TargetInfo":
        """The GPU of the current HIP device; raises RuntimeError when there is none."""
        from ..ops import device_info

        arch = device_info()["arch"].split(":")[0]
        return cls(arch=arch, features=_gpu_features(arch))

    @classmethod
    def reset_host_cache(cls) -> None:
        cls._cached_host = None

    @classmethod
    @contextmanager
    def override(cls, *, features: list[str] | None = None, arch: str | None = None):
        """Within the block a `TargetInfo()` without `arch` / `features` takes these instead of the
        host's; the innermost scope alone counts, and later changes to the caller's list do not."""
        cls._scopes.append(_Scope(arch, None if features is None else tuple(features)))
        cls.reset_host_cache()
        try:
            yield
        finally:
            cls._scopes.pop()
            cls.reset_host_cache()

    # -- queries --------------------------------------------------------------------------
    def _get_feature_list(self) -> list[str]:
        return _host_cpu_flags()

    def has_features(self, filter: list[str]) -> list[str]:
        wanted = set(filter)
        return [f for f in self.features if f in wanted]

    def is_supported(self, hw_extension: str) -> bool:
        prefix = hw_extension.lower()
        return any(f.startswith(prefix) for f in self.features)

    def is_gpu(self) -> bool:
        return self.arch.startswith("gfx")

    def vector_register_info(self) -> RegisterInfo | None:
        if self.is_gpu():
            return _GPU_VECTOR_REGISTERS
        return next((regs for applies, regs in _CPU_VECTOR_REGISTERS if applies(self.features)), None)

    @property
    def vector_register_width_bits(self) -> int | None:
        info = self.vector_register_info()
        return None if info is None else info.width_bits
