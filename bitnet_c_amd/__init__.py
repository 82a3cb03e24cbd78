"""bitnet.c_amd: a small model library with generation of its own for one AMD Instinct
MI355X (gfx950): a model folder (config.json + safetensors) to generated tokens, for the
Llama-style dense decoder, for Sunusun (recurrent and attention layers listed in config.json) and for Sonodra
(windowed and latent attention layers, dense and mixture-of-experts feed-forwards, listed in config.json) and for Fazopel
(linear-attention and sink-attention layers with norms on their outputs, gated experts with a shared expert).

    import bitnet_c_amd as bn
    llm = bn.load("/path/to/model", dtype="bfloat16", max_tokens=8192)
    out = llm.generate([[1, 2, 3], [4, 5]], max_new_tokens=16, temperature=0.0)
"""
from .api import LLM, load  # noqa: F401
from .config import FazopelConfig, LlamaConfig, MutiraxConfig, SonodraConfig, SunusunConfig, load_config, register_architecture  # noqa: F401
from .engine import Engine, Request, Result, StepEntry  # noqa: F401
from .sampling import SamplingParams  # noqa: F401
from .weights import WeightError, write_model_folder  # noqa: F401

__all__ = ["LLM", "load", "Engine", "StepEntry", "Request", "Result", "SamplingParams", "LlamaConfig", "SunusunConfig", "SonodraConfig", "FazopelConfig", "MutiraxConfig",
           "load_config", "register_architecture", "WeightError", "write_model_folder"]
