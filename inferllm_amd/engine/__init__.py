from .engine import Engine, parse_dtype
from .generate import GenerationLoop, GenerationStats
from .model import DecoderModel, expected_tensors
from .step import StepEntry, StepError, StepRunner

__all__ = ["Engine", "parse_dtype", "GenerationLoop", "GenerationStats", "DecoderModel",
           "expected_tensors", "StepEntry", "StepError", "StepRunner"]
