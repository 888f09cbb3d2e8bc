from . import finder
from .finder import find_pipeline_file
from .descriptor import Descriptor, PipelineDescriptor, KernelStage, string_to_type

__all__ = ["finder", "find_pipeline_file", "Descriptor", "PipelineDescriptor", "KernelStage", "string_to_type"]
