"""Target description used to select pipelines and kernels.

Behaviour of lighthouse/execution/target.py:13-132 (constructor defaults, cached host,
nested ``override`` scopes that snapshot their arguments, feature queries) with one
addition: ``TargetInfo.gpu()`` describes the AMD GPU the HIP library sees, arch string
"gfx950" for MI355X, so descriptor lookup finds ``descriptors/gfx950/...`` the way the
reference finds ``descriptors/xegpu/...``.
"""

from __future__ import annotations

import platform
import subprocess
from contextlib import contextmanager
from dataclasses import dataclass


@dataclass(frozen=True)
class RegisterInfo:
    width_bits: int
    count: int


class TargetInfo:
    _cached_host: "TargetInfo | None" = None
    _override_features_stack: list[list[str] | None] = []
    _override_arch_stack: list[str | None] = []

    def __init__(self, arch: str | None = None, features: list[str] | None = None, filter: list[str] | None = None):
        cls = self.__class__
        if arch is None and cls._override_arch_stack:
            arch = cls._override_arch_stack[-1]
        if features is None and cls._override_features_stack:
            override = cls._override_features_stack[-1]
            if override is not None:
                features = list(override)
        self.arch = arch if arch is not None else platform.machine()
        if features is not None:
            self.features = features
        elif self.arch.startswith("gfx"):
            self.features = _gpu_features(self.arch)
        else:
            self.features = self._get_feature_list()
        if filter is not None:
            self.features = self.has_features(filter)

    @classmethod
    def host(cls) -> "TargetInfo":
        if cls._override_features_stack or cls._override_arch_stack:
            return cls()
        if cls._cached_host is None:
            cls._cached_host = cls()
        return cls._cached_host

    @classmethod
    def gpu(cls) -> "TargetInfo":
        """The GPU of the current HIP device; raises RuntimeError when there is none."""
        from ..ops import device_info

        info = device_info()
        arch = info["arch"].split(":")[0]
        return cls(arch=arch, features=_gpu_features(arch))

    @classmethod
    def reset_host_cache(cls) -> None:
        cls._cached_host = None

    @classmethod
    @contextmanager
    def override(cls, *, features: list[str] | None = None, arch: str | None = None):
        cls._override_features_stack.append(None if features is None else list(features))
        cls._override_arch_stack.append(arch)
        cls.reset_host_cache()
        try:
            yield
        finally:
            cls._override_features_stack.pop()
            cls._override_arch_stack.pop()
            cls.reset_host_cache()

    def _get_feature_list(self) -> list[str]:
        flags = subprocess.run("lscpu | grep Flags", capture_output=True, text=True, shell=True).stdout
        if not flags.startswith("Flags:"):
            raise RuntimeError(
                "Could not get CPU features from lscpu. Make sure lscpu is installed and available in PATH."
            )
        return flags.split()[1:]

    def has_features(self, filter: list[str]) -> list[str]:
        return [ext for ext in self.features if ext in filter]

    def is_supported(self, hw_extension: str) -> bool:
        hw_extension = hw_extension.lower()
        return any(feature.startswith(hw_extension) for feature in self.features)

    def is_gpu(self) -> bool:
        return self.arch.startswith("gfx")

    def vector_register_info(self) -> RegisterInfo | None:
        if self.is_gpu():
            return RegisterInfo(width_bits=64 * 32, count=512)  # one VGPR across a 64-lane wavefront
        if "avx512f" in self.features:
            return RegisterInfo(width_bits=512, count=32)
        if "avx2" in self.features or "avx" in self.features:
            return RegisterInfo(width_bits=256, count=16)
        if any(feature.startswith("sse") for feature in self.features):
            return RegisterInfo(width_bits=128, count=16)
        return None

    @property
    def vector_register_width_bits(self) -> int | None:
        info = self.vector_register_info()
        return None if info is None else info.width_bits


def _gpu_features(arch: str) -> list[str]:
    """Feature names usable as descriptor sub-directories for an AMD GPU architecture."""
    if arch == "gfx950":
        return ["mfma", "mfma_bf16", "mfma_fp8_ocp", "mfma_f8f6f4", "lds160k"]
    if arch in ("gfx942", "gfx940", "gfx90a"):
        return ["mfma", "mfma_bf16"]
    return []
