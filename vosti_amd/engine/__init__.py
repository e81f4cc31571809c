from .engine import Engine
from .native import NativeEngine, NativeEngineError
from .scheduler import Scheduler
from .step import ModelRunner, StepEntry

__all__ = ["Engine", "ModelRunner", "NativeEngine", "NativeEngineError", "Scheduler", "StepEntry"]
