from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler, Scheduled
from .sequence import Sequence, State
from .engine import Engine, EngineConfig, RequestOutput

__all__ = ["ModelRunner", "StepEntry", "Scheduler", "Scheduled", "Sequence", "State", "Engine", "EngineConfig",
           "RequestOutput"]
