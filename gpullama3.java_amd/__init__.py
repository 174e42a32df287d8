"""A Llama 3 engine for one MI355X: configuration, weights, parts, cache, one step
function, generation and sampling, on hand-written HIP kernels for gfx950."""
from .config import (ConfigError, LlamaConfiguration, config_from_dict, load_config, register_architecture,
                     registered_architectures)
from .chat import LlamaChatFormat, Message
from .sampling import SamplingParams, select_sampler
from .weights import WeightsError, write_random_model


def __getattr__(name):
    # the engine needs torch and the device library; configuration and weights do not
    if name in ("Engine", "SequenceState", "CacheFull", "Generated", "Request", "RunMetrics"):
        from . import engine
        return getattr(engine, name)
    if name == "load_model":
        from .entry import load_model
        return load_model
    raise AttributeError(name)


__all__ = ["ConfigError", "LlamaConfiguration", "config_from_dict", "load_config", "register_architecture",
           "registered_architectures", "SamplingParams", "select_sampler", "WeightsError", "write_random_model",
           "Engine", "SequenceState", "CacheFull", "Generated", "Request", "RunMetrics", "load_model", "LlamaChatFormat",
           "Message"]
