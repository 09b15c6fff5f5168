from .engine import Engine, parse_dtype
from .generate import GenerationResult, generate, decide, plan_batches
from .model import Model, expected_tensors

__all__ = ["Engine", "parse_dtype", "GenerationResult", "generate", "decide", "plan_batches", "Model",
           "expected_tensors"]
