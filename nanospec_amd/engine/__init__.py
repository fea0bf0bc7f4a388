from .engine import Engine, EngineConfig
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler, Work

__all__ = ["Engine", "EngineConfig", "ModelRunner", "StepEntry", "Request", "Scheduler", "Work"]
