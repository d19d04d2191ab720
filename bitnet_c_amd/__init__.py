"""bitnet.c_amd: a small model library with generation of its own for one AMD Instinct
MI355X (gfx950): a model folder (config.json + safetensors) to generated tokens, for the
Llama-style dense decoder.

    import bitnet_c_amd as bn
    llm = bn.load("/path/to/model", dtype="bfloat16", max_tokens=8192)
    out = llm.generate([[1, 2, 3], [4, 5]], max_new_tokens=16, temperature=0.0)
"""
from .api import LLM, load  # noqa: F401
from .config import LlamaConfig, load_config, register_architecture  # noqa: F401
from .engine import Engine, Request, Result, StepEntry  # noqa: F401
from .sampling import SamplingParams  # noqa: F401
from .weights import WeightError, write_model_folder  # noqa: F401

__all__ = ["LLM", "load", "Engine", "StepEntry", "Request", "Result", "SamplingParams", "LlamaConfig",
           "load_config", "register_architecture", "WeightError", "write_model_folder"]
