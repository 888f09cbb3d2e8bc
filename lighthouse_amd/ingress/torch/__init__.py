from .compile import HipBackend, JITFunction, PlanStep, gpu_backend

__all__ = ["HipBackend", "JITFunction", "PlanStep", "gpu_backend"]
