"""rbitnet_amd: a small, whole Llama-decoder library for one MI355X (gfx950).

    import rbitnet_amd
    engine = rbitnet_amd.Engine.load_path("model_dir", dtype="bfloat16")
    results = engine.generate([[1, 2, 3], [4, 5]], max_tokens=64, temperature=0.8)

The layering follows the reference's bitnet-core (config -> weights -> model -> runtime
-> Engine): `config` (typed configuration and architecture registry), `weights`
(safetensors by name, random weights), `parts` (norm, position, mixer, feed-forward,
block), `cache` (slots, pages, state), `engine` (model, step, generation), `sampling`,
`csrc` (the HIP kernels).  Importing the package needs no GPU; building an Engine does.
"""
from .errors import (CacheError, ConfigError, InferenceError, KernelError, RbitnetError, WeightError)
from .config import LlamaConfig, load_config, register_architecture
from .engine import Engine, GenerationResult
from .weights import write_random_model

__version__ = "0.1.0"

__all__ = ["Engine", "GenerationResult", "LlamaConfig", "load_config", "register_architecture",
           "write_random_model", "RbitnetError", "ConfigError", "WeightError", "CacheError", "InferenceError",
           "KernelError", "__version__"]
