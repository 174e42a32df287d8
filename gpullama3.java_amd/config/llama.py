"""Typed configuration of the Llama 3 decoder, read from config.json's own keys.

The reference's ``LlamaConfiguration`` holds nine numbers read from GGUF metadata
(J/model/llama/LlamaConfiguration.java:6-39, J/model/loader/LlamaModelLoader.java:33-47)
and fixes in code what a model folder states itself: the head size ``dim/heads``,
the four numbers of the llama3 frequency scaling and whether it is on
(J/model/loader/ModelLoader.java:234-239). Here every one of them is a key.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional

from .registry import ConfigError, _as_ids, register_architecture
from .specs import (AttentionSpec, BlockSpec, GatedFeedForwardSpec, Llama3RopeScaling, ModelSpec,
                    NormSpec, RotarySpec, Run)

_MISSING = object()


def _need(d, key, kind=int):
    v = d.get(key, _MISSING)
    if v is _MISSING or v is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    if kind is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"config.json: '{key}' must be an integer, found {v!r}")
    if kind is int and v <= 0:
        raise ConfigError(f"config.json: '{key}' must be positive, found {v}")
    return v


@dataclass(frozen=True)
class LlamaConfiguration:
    hidden_size: int                 # dim
    intermediate_size: int           # hiddenDim
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int     # contextLength
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[Llama3RopeScaling]
    rope_pairing: str
    tie_word_embeddings: bool
    stop_ids: tuple = ()
    architecture: str = "LlamaForCausalLM"

    # derived, as J/model/llama/LlamaConfiguration.java:27-39
    @property
    def kv_dim(self):
        return self.num_key_value_heads * self.head_dim

    @property
    def kv_mul(self):
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(cls, d):
        hidden = _need(d, "hidden_size")
        heads = _need(d, "num_attention_heads")
        kv_heads = d.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads          # J/model/loader/LlamaModelLoader.java:39-41
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(f"config.json: hidden_size {hidden} is not a multiple of "
                                  f"num_attention_heads {heads} and no 'head_dim' is given")
            head_dim = hidden // heads  # J/model/llama/LlamaConfiguration.java:27-29
        for key, v in (("num_key_value_heads", kv_heads), ("head_dim", head_dim)):
            if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
                raise ConfigError(f"config.json: '{key}' must be a positive integer, found {v!r}")
        if heads % kv_heads:
            raise ConfigError(f"config.json: num_attention_heads {heads} is not a multiple of "
                              f"num_key_value_heads {kv_heads}")
        if head_dim % 2:
            raise ConfigError(f"config.json: head_dim {head_dim} is odd; rotary pairs need an even size")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"config.json: '{key}' is true; this decoder has no bias terms")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act {act!r} is not supported (silu)")
        pairing = d.get("rope_pairing", "half")
        if pairing not in ("half", "adjacent"):
            raise ConfigError(f"config.json: rope_pairing {pairing!r} is not 'half' or 'adjacent'")
        eps = float(d.get("rms_norm_eps", 1e-5))    # default of LlamaModelLoader.java:45
        theta = float(d.get("rope_theta", 10000.0))  # default of LlamaModelLoader.java:46
        if not eps > 0 or not theta > 0:
            raise ConfigError("config.json: rms_norm_eps and rope_theta must be positive")
        return cls(
            hidden_size=hidden,
            intermediate_size=_need(d, "intermediate_size"),
            num_hidden_layers=_need(d, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            vocab_size=_need(d, "vocab_size"),
            max_position_embeddings=_need(d, "max_position_embeddings"),
            rms_norm_eps=eps,
            rope_theta=theta,
            rope_scaling=_rope_scaling(d.get("rope_scaling")),
            rope_pairing=pairing,
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            stop_ids=_as_ids(d.get("eos_token_id")),
        )

    def to_dict(self):
        sc = self.rope_scaling
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None if sc is None else {
                "rope_type": "llama3", "factor": sc.factor, "low_freq_factor": sc.low_freq_factor,
                "high_freq_factor": sc.high_freq_factor,
                "original_max_position_embeddings": sc.original_max_position},
            "rope_pairing": self.rope_pairing,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    def chat_format(self, tokenizer):
        """The dialogue's token protocol of this architecture over ``tokenizer`` (the command line asks
        the configuration for it: another architecture brings its own or none)."""
        from ..chat import LlamaChatFormat
        return LlamaChatFormat(tokenizer)

    def with_stop_ids(self, ids):
        return replace(self, stop_ids=tuple(ids))

    def with_context_length(self, n):
        """A shorter context for a run; negative keeps the model's
        (J/model/llama/LlamaConfiguration.java:49-64)."""
        if n is None or n < 0:
            return self
        return replace(self, max_position_embeddings=min(n, self.max_position_embeddings))

    def model_spec(self):
        """The decoder as data: L equal pre-norm blocks run once each in order
        (J/inference/InferenceCore.java:72-173), final norm, head tied or not
        (J/model/loader/ModelLoader.java:252-253)."""
        rotary = RotarySpec(head_dim=self.head_dim, theta=self.rope_theta, scaling=self.rope_scaling,
                            pairing=self.rope_pairing, max_positions=self.max_position_embeddings)
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(BlockSpec(
                kind="prenorm",
                mixer_norm=NormSpec(dim=self.hidden_size, eps=self.rms_norm_eps,
                                    names={"weight": p + "input_layernorm.weight"}),
                mixer=AttentionSpec(hidden=self.hidden_size, n_heads=self.num_attention_heads,
                                    n_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                                    position=rotary, window=None, scale=None,
                                    names={"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                                           "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"}),
                ffn_norm=NormSpec(dim=self.hidden_size, eps=self.rms_norm_eps,
                                  names={"weight": p + "post_attention_layernorm.weight"}),
                ffn=GatedFeedForwardSpec(hidden=self.hidden_size, intermediate=self.intermediate_size,
                                         activation="silu",
                                         names={"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                                                "down": p + "mlp.down_proj.weight"}),
            ))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden=self.hidden_size,
            layers=tuple(layers),
            run_order=tuple(Run(layer=i) for i in range(self.num_hidden_layers)),
            final_norm=NormSpec(dim=self.hidden_size, eps=self.rms_norm_eps, names={"weight": "model.norm.weight"}),
            max_positions=self.max_position_embeddings,
            tie_embeddings=self.tie_word_embeddings,
            embedding_name="model.embed_tokens.weight",
            head_name=None if self.tie_word_embeddings else "lm_head.weight",
            stop_ids=self.stop_ids,
        )


def _rope_scaling(v):
    if v is None:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: rope_scaling must be null or an object, found {v!r}")
    kind = v.get("rope_type", v.get("type"))
    if kind in (None, "default"):
        return None
    if kind != "llama3":
        raise ConfigError(f"config.json: rope_scaling.rope_type {kind!r} is not supported (llama3)")
    try:
        sc = Llama3RopeScaling(
            factor=float(v["factor"]),
            low_freq_factor=float(v["low_freq_factor"]),
            high_freq_factor=float(v["high_freq_factor"]),
            original_max_position=int(v["original_max_position_embeddings"]))
    except KeyError as e:
        raise ConfigError(f"config.json: rope_scaling lacks {e.args[0]!r}") from None
    if sc.high_freq_factor == sc.low_freq_factor or sc.factor <= 0:
        raise ConfigError("config.json: rope_scaling needs factor > 0 and high_freq_factor != low_freq_factor")
    return sc


register_architecture("LlamaForCausalLM", LlamaConfiguration)
