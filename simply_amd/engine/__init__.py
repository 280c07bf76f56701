from .context import GroupStep, StepContext
from .executor import Executor, StepEntry

__all__ = ["GroupStep", "StepContext", "Executor", "StepEntry"]
