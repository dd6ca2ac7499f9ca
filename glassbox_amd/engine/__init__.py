from .engine import Engine, EngineError
from .generate import Generator, generate, greedy
from .scheduler import RequestOutput, Scheduler, SchedulerConfig, StepRecord

__all__ = ["Engine", "EngineError", "Generator", "generate", "greedy", "RequestOutput", "Scheduler",
           "SchedulerConfig", "StepRecord"]
