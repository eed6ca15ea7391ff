from .batch import StepEntry, StepContext
from .model import Model
from .runner import ModelRunner, parse_dtype
from .request import Request
from .scheduler import Scheduler, StepPlan
from .engine import Engine, StepOutput, EngineStats

__all__ = ["StepEntry", "StepContext", "Model", "ModelRunner", "parse_dtype", "Request", "Scheduler",
           "StepPlan", "Engine", "StepOutput", "EngineStats"]
