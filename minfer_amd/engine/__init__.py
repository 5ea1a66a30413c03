from .batch import StepContext
from .decode import DecodeSession
from .engine import Engine, StepError
from .generate import GenerationResult, generate, plan_batches
from .loading import load_model, random_model, run_dtype
from .model import DecoderModel, expected_tensors

__all__ = ["DecodeSession", "GenerationResult", "generate", "plan_batches", "StepContext", "Engine", "StepError", "load_model", "random_model", "run_dtype",
           "DecoderModel", "expected_tensors"]
