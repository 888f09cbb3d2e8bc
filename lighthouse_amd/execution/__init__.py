from .memory_manager import (
    MemoryManager,
    ExternalMemoryManager,
    DeviceMemoryManager,
    GPUMemoryManager,
    TorchMemoryManager,
)
from .target import TargetInfo
from .init import KernelArgument, KernelArgumentParser, InitType
from .runner import Runner

__all__ = [
    "MemoryManager", "ExternalMemoryManager", "DeviceMemoryManager", "GPUMemoryManager", "TorchMemoryManager",
    "TargetInfo", "KernelArgument", "KernelArgumentParser", "InitType", "Runner",
]
