from .compile import HipBackend, JITFunction, PlanStep, gpu_backend, with_schedule_parameters

__all__ = ["HipBackend", "JITFunction", "PlanStep", "gpu_backend", "with_schedule_parameters"]
