from .batch import StepEntry
from .engine import Engine, StepReport
from .scheduler import Request, Scheduler, Work

__all__ = ["StepEntry", "Engine", "StepReport", "Request", "Scheduler", "Work", "ModelRunner", "parse_dtype"]


def __getattr__(name):
    if name in ("ModelRunner", "parse_dtype"):
        from . import runner
        return getattr(runner, name)
    raise AttributeError(name)
