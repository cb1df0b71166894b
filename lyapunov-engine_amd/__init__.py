"""An inference engine for the Llama decoder on one AMD MI355X (gfx950).

From a model folder (config.json, safetensors) to generated tokens: typed
configuration and registry (``config``), weights by tensor name (``weights``),
layers put together from parts (``parts``, ``models``), a paged cache with block
tables (``cache``), one step function and a scheduler above it (``engine``),
sampling (``sampling``), hand-written HIP kernels (``csrc``, ``kernels``), a
command line (``entrypoints``) and a trace replay (``bin/trace_run``).
"""
from . import config, models, parts  # noqa: F401  (registers the built-in parts and architecture)

__version__ = "0.1.0"


def __getattr__(name):
    # The engine classes load lazily so that configuration and weights can be
    # used without touching the GPU libraries.
    if name in ("LLMEngine", "RequestOutput", "LLM", "generate"):
        from .engine import llm_engine
        return getattr(llm_engine, name)
    if name == "SamplingParams":
        from .sampling.params import SamplingParams
        return SamplingParams
    if name == "EngineConfig":
        from .config.engine_config import EngineConfig
        return EngineConfig
    raise AttributeError(name)
