from .parameter_selector import HipParameterSelector
from .parameters import ScheduleParameters

__all__ = ["HipParameterSelector", "ScheduleParameters"]
