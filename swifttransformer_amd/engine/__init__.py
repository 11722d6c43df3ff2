from .batch import StepItem, StepContext, pack_batch, BatchError
from .step import ModelRunner, StepEntry
from .scheduler import Scheduler, Request, Scheduled

__all__ = ["StepItem", "StepContext", "pack_batch", "BatchError", "ModelRunner", "StepEntry",
           "Scheduler", "Request", "Scheduled", "Engine"]


def __getattr__(name):
    if name == "Engine":
        from .engine import Engine
        return Engine
    raise AttributeError(name)
