from .step import StepEntry, StepRunner, StepError
from .scheduler import Scheduler, Request, Scheduled, SchedulerError
from .device_cache import DeviceCache

__all__ = ["StepEntry", "StepRunner", "StepError", "Scheduler", "Request", "Scheduled", "SchedulerError",
           "DeviceCache"]
