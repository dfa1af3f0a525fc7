from .engine import Engine, Finished, GenerationStats, random_model_tensors
from .model import Model
from .step import OutOfPages, StepContext, StepEntry, StepRunner

__all__ = ["Engine", "Finished", "GenerationStats", "random_model_tensors", "Model", "OutOfPages",
           "StepContext", "StepEntry", "StepRunner"]
