from .engine import Engine, GenerationResult
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler

__all__ = ["Engine", "GenerationResult", "ModelRunner", "StepEntry", "Request", "Scheduler"]
