from .engine import Engine
from .scheduler import Scheduler
from .step import ModelRunner, StepEntry

__all__ = ["Engine", "ModelRunner", "Scheduler", "StepEntry"]
