from .engine import Engine, StepEntry, StepError, StepOutput
from .scheduler import (ORCA_STRATEGY, SARATHI_STRATEGY, SUPPORTED_SCHEDULING_STRATEGIES,
                        ContinuousBatchScheduler, RequestState)

__all__ = [
    "ContinuousBatchScheduler", "Engine", "GenerationOutput", "LLM", "ORCA_STRATEGY",
    "RequestState", "SARATHI_STRATEGY", "SUPPORTED_SCHEDULING_STRATEGIES", "StepEntry",
    "StepError", "StepOutput", "build_scheduler",
]


def __getattr__(name):
    if name in ("LLM", "GenerationOutput", "build_scheduler"):
        from . import llm
        return getattr(llm, name)
    raise AttributeError(name)
