from .engine import Emitted, Engine, Finished, GenerationStats, random_model_tensors
from .model import Model
from .step import OutOfPages, StepContext, StepEntry, StepRunner

__all__ = ["Emitted", "Engine", "Finished", "GenerationStats", "random_model_tensors", "Model", "OutOfPages",
           "StepContext", "StepEntry", "StepRunner"]
