"""hfee_amd: a small inference engine for the Llama dense decoder on one MI355X.

    from hfee_amd import LLM, SamplingParams
    llm = LLM("path/to/model_folder", dtype="bfloat16")
    outs = llm.generate([[1, 2, 3]], SamplingParams(temperature=0, num_predict=16))
"""
from . import models as _models  # noqa: F401  (registers the architectures)
from .config import ConfigError, LlamaConfig, register_architecture
from .weights import WeightsError, write_model_folder

__all__ = ["LLM", "SamplingParams", "ConfigError", "WeightsError", "LlamaConfig",
           "register_architecture", "write_model_folder", "replay"]


def __getattr__(name):
    if name in ("LLM", "Output"):
        from . import api
        return getattr(api, name)
    if name == "replay":
        from .trace_replay import replay
        return replay
    if name == "SamplingParams":
        from .sampling import SamplingParams
        return SamplingParams
    raise AttributeError(name)
