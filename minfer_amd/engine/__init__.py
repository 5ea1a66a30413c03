from .batch import StepContext
from .engine import Engine, StepError
from .loading import load_model, random_model, run_dtype
from .model import DecoderModel, expected_tensors

__all__ = ["StepContext", "Engine", "StepError", "load_model", "random_model", "run_dtype",
           "DecoderModel", "expected_tensors"]
