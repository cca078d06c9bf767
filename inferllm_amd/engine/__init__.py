from .engine import Engine, parse_dtype
from .generate import GenerationLoop, GenerationStats, plan_prefill
from .model import DecoderModel, expected_tensors
from .session import Session
from .step import StepEntry, StepError, StepRunner

__all__ = ["Engine", "Session", "parse_dtype", "GenerationLoop", "GenerationStats", "plan_prefill", "DecoderModel",
           "expected_tensors", "StepEntry", "StepError", "StepRunner"]
