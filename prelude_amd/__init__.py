"""A small, whole LLM inference engine for one AMD Instinct MI355X (gfx950).

    from prelude_amd import LLM
    llm = LLM("path/to/model")             # config.json + model.safetensors
    outs = llm.generate([[1, 2, 3]], max_tokens=16, temperature=0.0)
"""
__version__ = "0.1.0"


def __getattr__(name):
    # heavy imports (torch, the native libraries) wait until something is used
    if name in ("LLM", "Session", "GenerationResult", "generate"):
        from . import llm
        return getattr(llm, name)
    if name in ("Engine", "StepEntry"):
        from . import engine
        return getattr(engine, name)
    if name == "SamplingParams":
        from .sampling.sampler import SamplingParams
        return SamplingParams
    if name == "EngineConfig":
        from .config import EngineConfig
        return EngineConfig
    raise AttributeError(name)
