"""inferllm_amd: a small, whole LLaMA inference library for one AMD MI355X.

    from inferllm_amd import Engine
    eng = Engine.from_pretrained(model_dir, dtype="bfloat16", max_batch=8)
    out = eng.generate([[1, 5, 9], [1, 7]], max_new_tokens=16)
"""
from . import models  # registers the architectures
from .config import (ConfigError, config_from_dict, load_config, register_architecture,
                     registered_architectures)
from .engine import Engine, Session, StepEntry, StepError
from .sampling import SamplingParams
from .weights import WeightsError, write_random_model

__all__ = ["Engine", "Session", "StepEntry", "StepError", "SamplingParams", "ConfigError", "WeightsError",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures",
           "write_random_model"]
