from .engine import Engine, StepEntry, StepError, StepOutput

__all__ = ["Engine", "StepEntry", "StepError", "StepOutput"]
