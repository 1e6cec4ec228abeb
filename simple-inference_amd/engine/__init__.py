from .step import StepEntry, StepRunner
from .build import build_model, model_from_folder, model_from_random
from .request import Request, RequestState
from .scheduler import Scheduler
from .engine import Engine

__all__ = ["StepEntry", "StepRunner", "build_model", "model_from_folder", "model_from_random",
           "Request", "RequestState", "Scheduler", "Engine"]
