from .step import StepEntry, Stepper
from .scheduler import Engine, Portion, Request
from .trace import Trace, read_events

__all__ = ["StepEntry", "Stepper", "Engine", "Portion", "Request", "Trace", "read_events"]
