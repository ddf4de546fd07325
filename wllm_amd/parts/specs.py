"""Descriptions of a model as data: which parts each layer is made of, with every
size and constant as a field, and the order in which layers run.

A specification names a part kind (the key of a registry in
`wllm_amd.parts.registry`) and carries that part's parameters and the names of
its tensors in the checkpoint.  No part, and nothing in here, knows which model
it belongs to: an architecture is a function from its configuration to a
`ModelPlan`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class NormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * (weight_offset + w), computed in float32."""
    size: int
    eps: float
    weight: str                    # tensor name
    weight_offset: float = 0.0     # 1.0: the weight is stored as an offset from one
    kind: str = "rms"


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.  kind "rope": rotation of query and key by
    angles position * theta^(-2j/rotary_dim), pairing element j with
    j + rotary_dim/2 ("half") ; kind "none": nothing."""
    kind: str = "rope"
    rotary_dim: int = 0
    theta: float = 10000.0
    pairing: str = "half"


@dataclass(frozen=True)
class MixerSpec:
    """Base of token-mixer specifications; `kind` selects the implementation."""
    kind: str = ""


@dataclass(frozen=True)
class AttentionSpec(MixerSpec):
    """Softmax attention of each query over the earlier keys of its request,
    read from the paged cache.  Query head h uses key/value head
    h // (num_heads // num_kv_heads).  `window` = W limits a query at position p
    to keys p-W+1..p; None is all keys."""
    kind: str = "attention"
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    window: Optional[int] = None
    position: PositionSpec = field(default_factory=PositionSpec)
    q_weight: str = ""
    k_weight: str = ""
    v_weight: str = ""
    o_weight: str = ""
    q_bias: Optional[str] = None
    k_bias: Optional[str] = None
    v_bias: Optional[str] = None


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str = ""


@dataclass(frozen=True)
class GatedMLPSpec(FeedForwardSpec):
    """down(act(gate(x)) * up(x)) without biases; `activation` names the
    nonlinearity ("gelu_tanh")."""
    kind: str = "gated_mlp"
    hidden_size: int = 0
    intermediate_size: int = 0
    activation: str = "gelu_tanh"
    gate_weight: str = ""
    up_weight: str = ""
    down_weight: str = ""


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward with their norms, and how they are
    arranged around the residual stream ("pre_norm": x += mixer(norm(x));
    x += ffn(norm(x)))."""
    mixer: MixerSpec
    feed_forward: FeedForwardSpec
    mixer_norm: NormSpec
    feed_forward_norm: NormSpec
    arrangement: str = "pre_norm"


@dataclass(frozen=True)
class EmbeddingSpec:
    """x = table[id] * scale.  `scale_in_model_dtype`: the factor is rounded to
    the model's dtype before use, as a buffer cast with the model would be."""
    vocab_size: int
    hidden_size: int
    weight: str
    scale: float = 1.0
    scale_in_model_dtype: bool = False


@dataclass(frozen=True)
class HeadSpec:
    """logits = hidden @ W^T; W is the embedding table when `weight` is None.  `tied_checkpoint_name`:
    the name under which a checkpoint of tied weights may still store the head; such a tensor is
    accepted if it equals the table."""
    vocab_size: int
    hidden_size: int
    weight: Optional[str] = None
    tied_checkpoint_name: Optional[str] = None


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `layer` indexes ModelPlan.layers (the same layer may
    be named by several entries: its weights are shared, each run has a cache
    of its own).  `reads_cache_of` = index of an earlier schedule entry whose
    cache this run reads instead of writing one."""
    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    embedding: EmbeddingSpec
    layers: tuple
    schedule: tuple
    final_norm: NormSpec
    head: HeadSpec
    max_positions: int
    # tensor names that may appear in a checkpoint and are ignored
    ignored_tensor_suffixes: tuple = ()

    def __post_init__(self):
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, the plan has {n}")
            if e.reads_cache_of is not None:
                j = e.reads_cache_of
                if not 0 <= j < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {j}, which is not an earlier entry")
                if self.schedule[j].reads_cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {j}, which owns none")
