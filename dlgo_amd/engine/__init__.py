from .context import StepContext, Workspace
from .engine import Engine, EngineError, Entry, run_dtype

__all__ = ["StepContext", "Workspace", "Engine", "EngineError", "Entry", "run_dtype"]
