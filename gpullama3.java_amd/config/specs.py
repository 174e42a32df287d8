"""Descriptions of model parts as plain data.

A model is described without any tensor: a list of block descriptions (each
naming its norm, mixer and feed-forward with every size and constant), the order
in which the blocks run, and the names under which each part's tensors are
stored. The parts of ``parts/`` are built from these and from nothing else, so
no part knows which architecture it serves.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class Llama3RopeScaling:
    """Frequency scaling of long wavelengths (the reference fixes the four numbers in
    code, J/model/loader/ModelLoader.java:235-239; here they come from config.json)."""
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position: int


@dataclass(frozen=True)
class RotarySpec:
    """Rotary position encoding of queries and keys."""
    kind: str = "rotary"
    head_dim: int = 0
    theta: float = 10000.0
    scaling: Optional[Llama3RopeScaling] = None
    pairing: str = "half"        # "half": (j, j + hs/2); "adjacent": (2j, 2j+1)
    max_positions: int = 0


@dataclass(frozen=True)
class NormSpec:
    kind: str = "rmsnorm"
    dim: int = 0
    eps: float = 1e-5
    names: dict = field(default_factory=dict)     # local tensor name -> stored name


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a cache of keys and values. Names ``q_bias``, ``k_bias``,
    ``v_bias`` (together) and ``o_bias`` among ``names`` add biases to the projections."""
    kind: str = "attention"
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    position: Optional[RotarySpec] = None
    window: Optional[int] = None      # None: every earlier key; n: the last n keys
    scale: Optional[float] = None     # None: 1/sqrt(head_dim)
    names: dict = field(default_factory=dict)


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """down(act(gate(x)) * up(x)); ``activation``: "silu" or "gelu_tanh". Names ``gate_bias`` and
    ``up_bias`` (together) and ``down_bias`` among ``names`` add biases to the products."""
    kind: str = "gated"
    hidden: int = 0
    intermediate: int = 0
    activation: str = "silu"
    names: dict = field(default_factory=dict)


@dataclass(frozen=True)
class BlockSpec:
    """One layer: how norm, mixer and feed-forward are arranged is ``kind``."""
    kind: str = "prenorm"             # x += mixer(norm(x)); x += ffn(norm(x))
    mixer_norm: object = None
    mixer: object = None
    ffn_norm: object = None
    ffn: object = None


@dataclass(frozen=True)
class Run:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers``. A layer may be named by several
    entries; each entry then has storage of its own in the cache, unless
    ``reads`` names an earlier entry of the run order, whose keys and values this
    entry reads instead of making its own.
    """
    layer: int
    reads: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    layers: tuple
    run_order: tuple
    final_norm: object                # the norm in front of the head; None: the head reads the rows as they are
    max_positions: int
    tie_embeddings: bool
    embedding_name: str
    head_name: Optional[str]          # None when tied
    stop_ids: tuple = ()
    # what other decoders put around the blocks; the reference's model has none of them
    # (J/inference/InferenceCore.java:69, :175-177):
    embedding_scale: Optional[float] = None       # the embedding row times this
    position_table_name: Optional[str] = None     # a stored [max_positions, hidden] table whose row at the token's position is added to it
    logit_scale: Optional[float] = None           # the logits times this
    head_bias_name: Optional[str] = None          # a stored [vocab] vector added to the logits (before the scale)
    logit_softcap: Optional[float] = None         # the logits become cap * tanh(logits / cap) (after the scale)
