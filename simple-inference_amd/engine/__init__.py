from .step import StepEntry, StepRunner
from .build import build_model, model_from_folder, model_from_random

__all__ = ["StepEntry", "StepRunner", "build_model", "model_from_folder", "model_from_random"]
