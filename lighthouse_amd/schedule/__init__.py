from .parameters import ScheduleParameters

__all__ = ["ScheduleParameters"]
