"""The programming entry point in the reference's manner.

Reference: ``ModelLoader.loadModel(path, contextLength, loadWeights, useTornadovm)``
returns the model (J/model/loader/ModelLoader.java:107-115), ``Sampler.selectSampler``
the sampler (J/inference/sampler/Sampler.java:56), ``model.generateTokens(...)`` the
tokens (J/model/Model.java:66). Here: ``load_model`` -> ``Engine``,
``select_sampler`` -> ``SamplingParams``, ``Engine.generate_tokens`` / ``Engine.generate``.
"""
from __future__ import annotations


def load_model(model_path, context_length=-1, dtype="bfloat16", device="cuda:0", **kw):
    """``context_length`` < 0 keeps the model's own (J/model/llama/LlamaConfiguration.java:49-64)."""
    from .engine import Engine
    return Engine.from_folder(str(model_path), dtype=dtype, device=device,
                              max_context=None if context_length is None or context_length < 0 else context_length,
                              **kw)
