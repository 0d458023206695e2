from .step import StepEntry, Stepper

__all__ = ["StepEntry", "Stepper"]
