"""minfer_amd: a small generation library for one GPU (AMD MI355X, gfx950) with hand-written
HIP kernels, built after what yusiwen/minfer does for its one architecture, the Qwen2 dense
decoder."""
from .config import ConfigError, Qwen2Config
from .registry import config_from_dict, load_config, register_architecture, registered_architectures
from .weights import WeightError, write_random_model
from .engine import DecoderModel, Engine, GenerationResult, StepError, generate, load_model, random_model
from .sampling import Sampler, SamplingParams
from .api import LLM

__version__ = "0.1.0"

__all__ = ["ConfigError", "Qwen2Config", "config_from_dict", "load_config", "register_architecture",
           "registered_architectures", "WeightError", "write_random_model", "DecoderModel", "Engine",
           "StepError", "load_model", "random_model", "GenerationResult", "generate", "Sampler",
           "SamplingParams", "LLM"]
